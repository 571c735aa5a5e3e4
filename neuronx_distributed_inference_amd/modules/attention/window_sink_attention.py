"""Sliding-window GQA softmax attention with rotary positions, per-head
query/key norms, a value-less sink in the softmax and one output gate per head.

Per head, queries and keys are RMS-normed over the head size (one weight
vector of that size shared by all heads), then rotated in the half-split
layout on the first ``rot_dims`` channels (frequencies optionally extended by
parts, see :func:`half_split_inv_freq`). Query ``i`` sees keys ``j`` with
``0 <= i - j < window``. The softmax denominator carries one extra term
``exp(sink)`` that has no value (``sink = 0`` adds exactly one), so a query
can attend to nothing. Each head's output is multiplied by the sigmoid of one
gate number per head. Every one of these (norm, rotation, window, sink,
gate, head sizes) is a constructor parameter and can be switched off.

The module owns the norm weights, the frequency table and the cache access;
the q/k/v/gate projections are the caller's (so they can be one fused GEMM).
Normed and rotated K and V go to the paged cache first, then one kernel
serves prompt portions, single decoded tokens and mixed batches: every query
carries its own position.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.modules.rope import half_split_inv_freq
from neuronx_distributed_inference_amd.ops import seqmix


class RotaryWindowSinkAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, qk_dim: int, v_dim: int,
                 scale: float, eps: float, window: Optional[int] = None,
                 rot: Optional[dict] = None, qk_norm: bool = True,
                 sink: Optional[float] = 0.0):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.qk_dim = qk_dim
        self.v_dim = v_dim
        self.scale = float(scale)
        self.eps = float(eps)
        self.window = None if window is None else int(window)
        f32 = dict(dtype=torch.float32)
        self.qk_norm = bool(qk_norm)
        if qk_norm:
            self.q_norm = nn.Parameter(torch.ones(qk_dim, **f32), requires_grad=False)
            self.k_norm = nn.Parameter(torch.ones(qk_dim, **f32), requires_grad=False)
        self.mscale = 1.0
        if rot:
            dims = int(rot.get("dims", qk_dim))
            assert dims % 2 == 0 and dims <= qk_dim
            inv_freq, self.mscale = half_split_inv_freq(rot["base"], dims, rot.get("scaling"))
            self.register_buffer("inv_freq", inv_freq, persistent=False)
        else:
            self.inv_freq = None
        # the sink's score, the same for every head (None = plain softmax)
        if sink is not None:
            self.register_buffer("sink", torch.full((num_heads,), float(sink), **f32),
                                 persistent=False)
        else:
            self.sink = None

    def kv_shape(self):
        return (self.num_kv_heads, self.qk_dim, self.v_dim)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                kv_mgr, cache_idx: int, step: seqmix.StepLayout,
                gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q (B,S,H*Dk), k (B,S,G*Dk), v (B,S,G*Dv), gate (B,S,H) — column
        slices of a fused projection are fine. Returns (B,S,H*Dv)."""
        B, S = q.shape[0], q.shape[1]
        H, G, D = self.num_heads, self.num_kv_heads, self.qk_dim
        kc, vc = kv_mgr.get_cache(cache_idx)
        qn = seqmix.head_norm_rotate(
            q.unflatten(-1, (H, D)), step, self.q_norm if self.qk_norm else None, self.eps,
            self.inv_freq, self.mscale, out_dtype=q.dtype)
        kn = seqmix.head_norm_rotate(
            k.unflatten(-1, (G, D)), step, self.k_norm if self.qk_norm else None, self.eps,
            self.inv_freq, self.mscale, out_dtype=k.dtype)
        seqmix.paged_kv_write(kc.data, vc.data, kn.view(B * S, -1), v.flatten(0, 1),
                              kv_mgr.slot_mapping, step)
        return seqmix.paged_attention(
            qn, kc.data, vc.data, step, kv_mgr.block_table, self.scale, H,
            window=self.window, sink=self.sink, gate=gate, gate_per_head=True,
            out_dtype=q.dtype)
