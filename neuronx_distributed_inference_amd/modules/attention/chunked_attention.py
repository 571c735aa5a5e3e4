"""Chunk-local GQA softmax attention with a linear distance penalty and a
learned softmax sink.

A rotation-free attention core. Positions enter in two places: the mask,
which cuts the sequence into blocks of ``chunk`` positions counted from
position 0 (query ``i`` sees key ``j <= i`` only when ``floor(i / chunk) ==
floor(j / chunk)``, wherever a prompt was cut for processing), and the
score, from which ``slope_h * (i - j)`` is taken off. The slopes are a fixed
geometric ladder over the heads, ``slope_h = 2^(-slope_log2 * (h + 1) / H)``.
The softmax denominator carries one extra term ``exp(sink_h)`` per head, a
learned score that stands for no key: nothing is added to the output for it
and neither the scale nor the penalty applies to it. Chunk
size, scale, the ladder's exponent and the presence of the sink are
constructor parameters; key and value heads may have different sizes.

The module owns the sink, the slope table and the cache access; the q/k/v
projections are the caller's (so they can be one fused GEMM). K/V go to the
paged cache first, then one kernel serves prompt portions, single decoded
tokens and mixed batches: every query carries its own position.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.ops import seqmix


def geometric_slopes(num_heads: int, log2_span: float = 8.0) -> torch.Tensor:
    """slope_h = 2^(-log2_span * (h + 1) / H), evaluated in float64."""
    h = torch.arange(1, num_heads + 1, dtype=torch.float64)
    return torch.pow(torch.tensor(2.0, dtype=torch.float64),
                     -float(log2_span) * h / num_heads).float()


class ChunkedSlopeAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, qk_dim: int, v_dim: int,
                 scale: float, chunk: int, slope_log2: float = 8.0, sink: bool = True):
        super().__init__()
        assert num_heads % num_kv_heads == 0 and chunk >= 0
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.qk_dim = qk_dim
        self.v_dim = v_dim
        self.scale = float(scale)
        self.chunk = int(chunk)
        self.register_buffer("slopes", geometric_slopes(num_heads, slope_log2), persistent=False)
        self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32),
                                 requires_grad=False) if sink else None

    def kv_shape(self):
        """(kv_heads, key size, value size) of the pages this layer owns."""
        return (self.num_kv_heads, self.qk_dim, self.v_dim)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kv_mgr,
                cache_idx: int, step: seqmix.StepLayout) -> torch.Tensor:
        """q (B,S,H*Dk), k (B,S,G*Dk), v (B,S,G*Dv) — column slices of a
        fused projection are fine. Returns (B,S,H*Dv)."""
        kc, vc = kv_mgr.get_cache(cache_idx)
        seqmix.paged_kv_write(kc.data, vc.data, k.flatten(0, 1), v.flatten(0, 1),
                              kv_mgr.slot_mapping, step)
        return seqmix.paged_attention(
            q, kc.data, vc.data, step, kv_mgr.block_table, self.scale, self.num_heads,
            chunk=self.chunk, slopes=self.slopes, sink=self.sink, out_dtype=q.dtype)
