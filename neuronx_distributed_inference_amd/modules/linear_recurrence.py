"""Linear-recurrence token mixer cores with matrix state: the gated delta
rule (below), selective state spaces (:class:`StateSpaceDuality`) and
retention (:class:`Retention`).

Gated delta rule.

Per head the state is a (dim x vdim) fp32 matrix ``M`` updated once per token

    M <- diag(d_t) M            d_t = exp(-exp(A_log) * softplus(a_t + dt_bias))
    u  = beta_t (v_t - M^T k_t)                  (delta-rule correction)
    M <- M + k_t u^T
    o_t = M^T q_t                                (reads the fresh write)

with one decay per head AND key channel (``decay_per_channel``) or a single
one per head, unit-norm q/k (q also scaled by dim^-1/2), beta a sigmoid.
q/k/v first pass a short causal convolution and SiLU; the output is
RMS-normalised per head, scaled by a weight shared across heads and
multiplied by a gate (``gate_act``: sigmoid or silu of the gate projection).
``a_t`` and the gate either come through low-rank two-stage projections whose
second stages live here (``decay_rank``/``gate_rank`` > 0) or are handed in
at full size by the caller (ranks 0).

State (``M`` and the convolution tail) is engine state in the cache
manager's :class:`RecurrentStateManager`, keyed by this module's name and
the layer run, so prompts can be cut anywhere and decode continues from
prefill. The first-stage projections of the layer input are the caller's.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.modules.conv import CausalShortConv
from neuronx_distributed_inference_amd.ops import seqmix
from neuronx_distributed_inference_amd.parallel.layers import ColumnParallelLinear


class GatedDeltaRule(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, dim: int, vdim: int,
                 conv_taps: int, decay_rank: int, gate_rank: int, eps: float,
                 dtype: torch.dtype, tp_degree: int = 1,
                 decay_per_channel: bool = True, gate_act: str = "sigmoid"):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        assert (decay_rank > 0) == (gate_rank > 0), "both low-rank or both direct"
        assert gate_act in ("sigmoid", "silu")
        self.decay_per_channel = bool(decay_per_channel)
        self.gate_act = gate_act
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.dim = dim
        self.vdim = vdim
        self.eps = float(eps)
        self.qkv_channels = 2 * num_kv_heads * dim + num_heads * vdim
        self.conv = CausalShortConv(self.qkv_channels, conv_taps, activation="silu")
        # second stages of the two low-rank projections as ONE block-diagonal
        # GEMM: [a_low | g_low] (rank_a + rank_g) -> [a (H*dim) | gate (H*vdim)];
        # the off-diagonal blocks are exact zeros
        self.decay_rank = decay_rank
        self.gate_rank = gate_rank
        self.decay_width = num_heads * (dim if decay_per_channel else 1)
        self.ag2 = None
        if decay_rank > 0:
            self.ag2 = ColumnParallelLinear(decay_rank + gate_rank,
                                            self.decay_width + num_heads * vdim, dtype=dtype,
                                            tp_degree=tp_degree)
        f32 = dict(dtype=torch.float32)
        self.A_log = nn.Parameter(torch.zeros(num_heads, **f32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(self.decay_width, **f32), requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(vdim, **f32), requires_grad=False)

    def state_shapes(self):
        return {"conv": self.conv.state_shape(),
                "mem": (self.num_heads, self.vdim, self.dim)}   # stored transposed

    @staticmethod
    def block_diagonal(a2: torch.Tensor, g2: torch.Tensor) -> torch.Tensor:
        """(H*dim, rank_a), (H*vdim, rank_g) -> the fused second-stage weight."""
        w = torch.zeros(a2.shape[0] + g2.shape[0], a2.shape[1] + g2.shape[1], dtype=a2.dtype)
        w[:a2.shape[0], :a2.shape[1]] = a2
        w[a2.shape[0]:, a2.shape[1]:] = g2
        return w

    def forward(self, qkv: torch.Tensor, beta: torch.Tensor, ag_low: torch.Tensor,
                states, key: str, step: seqmix.StepLayout,
                gate: torch.Tensor = None) -> torch.Tensor:
        """qkv (B,S,q|k|v channels) raw projections, beta (B,S,H) logits.
        With low-rank stages: ag_low (B,S,rank_a+rank_g), the first-stage
        projections [decay | gate]. Without: ag_low is the decay projection
        itself (B,S,decay_width) and ``gate`` (B,S,H*vdim) the gate's.
        `states` is the RecurrentStateManager, `key` this layer run's prefix
        in it."""
        qkv_c = self.conv(qkv, states.get(key + ".conv"), step, out_dtype=torch.float32)
        if self.ag2 is not None:
            ag = self.ag2(ag_low)
            a, gate = torch.split(ag, [self.decay_width, self.num_heads * self.vdim], dim=-1)
        else:
            a = ag_low
        return seqmix.gated_delta_rule(
            qkv_c, beta, a, self.dt_bias, self.A_log, gate, self.norm_weight,
            self.eps, states.get(key + ".mem"), step, self.num_kv_heads, self.dim,
            self.vdim, out_dtype=a.dtype, gate_act=self.gate_act)


class StateSpaceDuality(nn.Module):
    """Selective state-space token mixer core (the scalar-decay, multi-head
    form that is dual to a masked linear attention).

    Per head the state is an (state x vdim) fp32 matrix

        S_t = exp(-exp(A_log) dt_t) S_{t-1} + dt_t B_t x_t^T ,
        y_t = S_t^T C_t + D x_t ,   dt_t = softplus(dt_proj_t + dt_bias)

    with one decay, step size and skip weight ``D`` per head; ``B`` and ``C``
    (``groups`` of them, each shared by heads/groups consecutive heads) and
    ``x`` first pass one short causal convolution with bias and SiLU. The
    output is multiplied by silu(z) and THEN RMS-normed in ``norm_groups``
    equal channel groups and weighted.

    The caller owns the input projection, laid out [z | x | B | C | dt], and
    the output projection. State (``S`` and the convolution tail) lives in the
    cache manager's :class:`RecurrentStateManager`.
    """

    def __init__(self, num_heads: int, vdim: int, state: int, groups: int,
                 conv_taps: int, norm_groups: int, eps: float, conv_bias: bool = True):
        super().__init__()
        assert num_heads % groups == 0 and (num_heads * vdim) % norm_groups == 0
        self.num_heads = num_heads
        self.vdim = vdim
        self.state = state
        self.groups = groups
        self.norm_groups = norm_groups
        self.eps = float(eps)
        self.inner = num_heads * vdim
        self.conv_channels = self.inner + 2 * groups * state
        # [z | x B C | dt] widths of the caller's input projection
        self.splits = [self.inner, self.conv_channels, num_heads]
        self.conv = CausalShortConv(self.conv_channels, conv_taps, activation="silu",
                                    bias=conv_bias)
        f32 = dict(dtype=torch.float32)
        self.A_log = nn.Parameter(torch.zeros(num_heads, **f32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(num_heads, **f32), requires_grad=False)
        self.D = nn.Parameter(torch.ones(num_heads, **f32), requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(self.inner, **f32), requires_grad=False)

    def state_shapes(self):
        return {"conv": self.conv.state_shape(),
                "ssm": (self.num_heads, self.vdim, self.state)}   # stored transposed

    def forward(self, z: torch.Tensor, xbc: torch.Tensor, dt: torch.Tensor,
                states, key: str, step: seqmix.StepLayout) -> torch.Tensor:
        """z (B,S,inner), xbc (B,S,inner + 2*groups*state), dt (B,S,heads):
        raw projections (column slices of one GEMM output are fine). Returns
        (B,S,inner) in z's dtype."""
        GN = self.groups * self.state
        c = self.conv(xbc, states.get(key + ".conv"), step, out_dtype=torch.float32)
        x, Bm, Cm = torch.split(c, [self.inner, GN, GN], dim=-1)
        y = seqmix.decay_scan(Cm, Bm, x, states.get(key + ".ssm"), step, self.state,
                              self.vdim, dt=dt, dt_bias=self.dt_bias, a_log=self.A_log,
                              skip=self.D)
        return seqmix.group_gated_norm(y, z, self.norm_weight, self.eps, self.norm_groups,
                                       gate_first=True, out_dtype=z.dtype)


class Retention(nn.Module):
    """Linear attention with a fixed decay per head and no softmax or
    denominator: per head a (dim x vdim) fp32 state

        S_t = decay_h S_{t-1} + (dim^-1/2 k_t) v_t^T ,   o_t = S_t^T q_t ,

    each head's read-out divided by its root mean square (no weight), then
    multiplied by silu of a gate projection. The caller owns the q/k/v/gate
    and output projections; the state lives in the cache manager's
    :class:`RecurrentStateManager`.
    """

    def __init__(self, num_heads: int, dim: int, vdim: int, decay, eps: float):
        super().__init__()
        assert len(decay) == num_heads
        self.num_heads = num_heads
        self.dim = dim
        self.vdim = vdim
        self.eps = float(eps)
        self.register_buffer("decay", torch.tensor([float(d) for d in decay],
                                                   dtype=torch.float32), persistent=False)

    def state_shapes(self):
        return {"mem": (self.num_heads, self.vdim, self.dim)}      # stored transposed

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor,
                states, key: str, step: seqmix.StepLayout) -> torch.Tensor:
        """q, k (B,S,H*dim), v, gate (B,S,H*vdim). Returns (B,S,H*vdim) in the
        gate's dtype."""
        o = seqmix.decay_scan(q, k, v, states.get(key + ".mem"), step, self.dim, self.vdim,
                              head_decay=self.decay, k_scale=self.dim ** -0.5)
        return seqmix.group_gated_norm(o, gate, None, self.eps, self.num_heads,
                                       gate_first=False, out_dtype=gate.dtype)
