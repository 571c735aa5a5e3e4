"""Latent (low-rank KV) attention with an optional softmax sink, sliding
window and output gate.

Each token stores only a normed latent ``c`` (``kv_rank`` channels) and one
rotated key part shared by all heads (``rot_dim`` channels). Per head the
unrotated key is ``W_uk c`` and the value ``W_uv c``; the score is
``(q_plain . k_plain + q_rot . k_rot) * scale``. Rotary positions use the
interleaved pair layout on the first ``rot_dims`` channels of the rotated
part. With ``sink`` the softmax denominator carries one extra term
``exp(sink_h)`` per head: a key without a value, unscaled. With ``window``
query ``i`` sees keys ``i - window < j <= i`` only. A ``gate`` handed to
the call multiplies the concatenated heads by ``sigmoid(gate)`` element by
element.

Steps that continue a sequence (decoded tokens, later prompt portions, mixed
batches) are computed in the *absorbed* form, which never expands the cache:
``q_plain . (W_uk c) = (W_uk^T q_plain) . c``, so the query is mapped into
latent space (one small batched GEMM per step), attention runs as
multi-query attention over cache rows ``[c | k_rot]`` whose values are the
rows' own first ``kv_rank`` channels, and ``W_uv`` is applied to the
attended latent afterwards. One page row per token holds everything; there
is no value cache. A step in which every row starts its sequence (a whole
prompt, ``step.fresh``) has all its keys at hand and takes the *expanded*
form instead: keys and values are materialised per head for the step only
(two GEMMs) and ordinary multi-head attention runs over them, which costs
``dim + rot_dim`` instead of ``kv_rank + rot_dim`` multiply-adds per score.
The cache rows are written either way.

The module owns the latent norm, the two up-projections, the sink and the
cache access; the projections of the layer input (queries and the
down-projection) are the caller's.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.modules.norm import StreamRMSNorm
from neuronx_distributed_inference_amd.modules.rope import interleaved_inv_freq
from neuronx_distributed_inference_amd.ops import seqmix


class LatentSinkAttention(nn.Module):
    def __init__(self, num_heads: int, dim: int, rot_dim: int, v_dim: int, kv_rank: int,
                 scale: float, eps: float, rope_base: float, rot_dims: int,
                 dtype: torch.dtype, sink: bool = True, window: Optional[int] = None):
        super().__init__()
        assert rot_dims <= rot_dim and rot_dims % 2 == 0
        self.num_heads = num_heads
        self.dim = dim
        self.rot_dim = rot_dim
        self.v_dim = v_dim
        self.kv_rank = kv_rank
        self.scale = float(scale)
        self.window = None if window is None else int(window)
        self.row = kv_rank + rot_dim                      # one cache row
        self.latent_norm = StreamRMSNorm(kv_rank, eps=eps, one_plus=False)
        self.register_buffer("inv_freq", interleaved_inv_freq(rope_base, rot_dims),
                             persistent=False)
        # per-head up-projections in checkpoint layout: uk (H, dim, kv_rank),
        # uv (H, v_dim, kv_rank). Flattened they expand the latent; batched,
        # uk maps q_plain into latent space and uv^T the attended latent out
        self.uk = nn.Parameter(torch.zeros(num_heads, dim, kv_rank, dtype=dtype),
                               requires_grad=False)
        self.uv = nn.Parameter(torch.zeros(num_heads, v_dim, kv_rank, dtype=dtype),
                               requires_grad=False)
        self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32),
                                 requires_grad=False) if sink else None

    def kv_shape(self):
        """One key 'head' of kv_rank + rot_dim channels, no value pages."""
        return (1, self.row, 0)

    @torch.no_grad()           # inference only: the batched products write into views
    def forward(self, q: torch.Tensor, dkv: torch.Tensor, kv_mgr, cache_idx: int,
                step: seqmix.StepLayout, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q (B,S,H*(dim+rot_dim)), dkv (B,S,kv_rank+rot_dim), gate
        (B,S,H*v_dim) or None: column slices of a fused projection are fine.
        Returns (B,S,H*v_dim)."""
        B, S = q.shape[0], q.shape[1]
        H, D, R, C = self.num_heads, self.dim, self.rot_dim, self.kv_rank
        T = B * S
        dt = q.dtype
        # cache row [rms_norm(latent) | rotated shared key part], normed, rotated
        # and scattered to the token's page slot in one launch; only the
        # whole-prompt form reads it back as a dense tensor
        kc, _ = kv_mgr.get_cache(cache_idx)
        q4 = q.unflatten(-1, (H, D + R))
        fresh = bool(getattr(step, "fresh", False))
        row = torch.empty(B, S, self.row, dtype=dt, device=q.device) if fresh else None
        seqmix.latent_row_write(dkv, self.latent_norm.weight, self.latent_norm.eps,
                                self.inv_freq, step, kc.data, kv_mgr.slot_mapping, C, row=row)
        if fresh:
            return self._expanded(q4, row, step, gate)
        # query in latent space: [uk_h^T q_plain | rotated q_rot] per head
        qa = torch.empty(B, S, H, self.row, dtype=dt, device=q.device)
        torch.bmm(q4[..., :D].flatten(0, 1).transpose(0, 1), self.uk,
                  out=qa.view(T, H, self.row)[..., :C].transpose(0, 1))
        seqmix.rotate_interleaved(q4[..., D:], step, self.inv_freq, out=qa[..., C:])
        k_cache = kc.data
        lat = seqmix.paged_attention(
            qa.view(B, S, H * self.row), k_cache, k_cache[..., :C], step, kv_mgr.block_table,
            self.scale, H, window=self.window, sink=self.sink, out_dtype=dt)   # (B,S,H*C)
        out = torch.empty(B, S, H * self.v_dim, dtype=dt, device=q.device)
        torch.bmm(lat.view(T, H, C).transpose(0, 1), self.uv.transpose(1, 2),
                  out=out.view(T, H, self.v_dim).transpose(0, 1))
        if gate is not None:
            seqmix.sigmoid_gate_(out, gate)
        return out

    def _expanded(self, q4: torch.Tensor, row: torch.Tensor, step, gate=None) -> torch.Tensor:
        """Whole prompts: per-head keys [W_uk c | k_rot] and values W_uv c of
        this step's tokens, attended in place: the (B, S) token grid is
        addressed as B pages of S tokens."""
        B, S, H = q4.shape[0], q4.shape[1], self.num_heads
        D, R, C, Dv = self.dim, self.rot_dim, self.kv_rank, self.v_dim
        dt = q4.dtype
        c = row[..., :C]
        kx = torch.empty(B, S, H, D + R, dtype=dt, device=q4.device)
        kx[..., :D] = torch.nn.functional.linear(c, self.uk.view(H * D, C)).view(B, S, H, D)
        kx[..., D:] = row[..., C:].unsqueeze(2)
        vx = torch.nn.functional.linear(c, self.uv.view(H * Dv, C)).view(B, S, H, Dv)
        qx = q4.clone(memory_format=torch.contiguous_format)
        seqmix.rotate_interleaved(qx[..., D:], step, self.inv_freq, out=qx[..., D:])
        pages = torch.arange(B, device=q4.device, dtype=torch.int32).view(B, 1)
        return seqmix.paged_attention(
            qx.view(B, S, H * (D + R)), kx, vx, step, pages, self.scale, H,
            window=self.window, sink=self.sink, gate=gate, out_dtype=dt)
