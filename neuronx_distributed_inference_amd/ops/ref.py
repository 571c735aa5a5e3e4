"""Pure-PyTorch reference implementations of every device op.

These are (a) the CPU execution path (the analog of the reference's
`to_cpu()` gloo fallback, `models/application_base.py:556-628`) and (b) the
numerics oracle for the HIP kernels: every GPU test compares the CDNA4
kernel against these run in fp32.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


def rms_norm(
    x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6,
    residual: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """RMSNorm with optional fused residual add.

    Returns (normed, new_residual): when `residual` is given the op computes
    h = x + residual first, returns rmsnorm(h) and h.
    """
    orig_dtype = x.dtype
    xf = x.float()
    if residual is not None:
        xf = xf + residual.float()
        new_residual = xf.to(orig_dtype)
    else:
        new_residual = None
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps)
    out = out * weight.float()
    return out.to(orig_dtype), new_residual


def rope_apply(
    q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rotary embedding, rotate-half convention (HF Llama).

    q,k: (B, H, S, D); cos,sin: (B, S, D) or (S, D) broadcastable.
    """

    def rot_half(t):
        d = t.shape[-1] // 2
        return torch.cat((-t[..., d:], t[..., :d]), dim=-1)

    if cos.dim() == 2:
        cos = cos.unsqueeze(0)
        sin = sin.unsqueeze(0)
    cos = cos.unsqueeze(1)  # (B,1,S,D)
    sin = sin.unsqueeze(1)
    qf, kf = q.float(), k.float()
    cf, sf = cos.float(), sin.float()
    q_out = qf * cf + rot_half(qf) * sf
    k_out = kf * cf + rot_half(kf) * sf
    return q_out.to(q.dtype), k_out.to(k.dtype)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return (torch.nn.functional.silu(gate.float()) * up.float()).to(gate.dtype)


def gelu_tanh_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return (torch.nn.functional.gelu(gate.float(), approximate="tanh") * up.float()).to(gate.dtype)


def kv_cache_update(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    positions: torch.Tensor,
    seq_ids: Optional[torch.Tensor] = None,
) -> None:
    """Scatter-write new K/V rows into a linear (B, Hkv, S, D) cache in place.

    k_new/v_new: (B, Hkv, S_new, D); positions: (B, S_new) target sequence
    positions; seq_ids: (B,) cache-row mapping for continuous batching
    (ref `kv_cache_manager.py:369-586`, `:616`).
    """
    B, Hkv, S_new, D = k_new.shape
    if seq_ids is None:
        seq_ids = torch.arange(B, device=k_new.device)
    max_s = k_cache.shape[2]
    for b in range(B):
        row = int(seq_ids[b])
        if row < 0 or row >= k_cache.shape[0]:
            continue  # garbage row for SPMD-uniform DP writes
        valid = (positions[b] >= 0) & (positions[b] < max_s)
        pos = positions[b][valid].long()
        k_cache[row, :, pos, :] = k_new[b][:, valid].to(k_cache.dtype)
        v_cache[row, :, pos, :] = v_new[b][:, valid].to(v_cache.dtype)


def block_kv_cache_update(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """Paged cache scatter (ref `block_kv_cache_manager.py:268-375`).

    k_cache/v_cache: (num_blocks, block_size, Hkv, D); k_new/v_new:
    (N_tokens, Hkv, D); slot_mapping: (N_tokens,) flat slot index (or -1).
    """
    bs = k_cache.shape[1]
    flat_k = k_cache.view(-1, *k_cache.shape[2:])
    flat_v = v_cache.view(-1, *v_cache.shape[2:])
    valid = slot_mapping >= 0
    slots = slot_mapping[valid].long()
    flat_k[slots] = k_new[valid].to(flat_k.dtype)
    flat_v[slots] = v_new[valid].to(flat_v.dtype)


def sdpa(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    sinks: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Masked attention in fp32: q (B,Hq,Sq,D), k/v (B,Hkv,Skv,D); GQA by
    head repetition; optional learned attention sinks (GPT-OSS,
    ref `modules/attention/sink.py`)."""
    B, Hq, Sq, D = q.shape
    Hkv = k.shape[1]
    if Hkv != Hq:
        rep = Hq // Hkv
        k = k.repeat_interleave(rep, dim=1)
        v = v.repeat_interleave(rep, dim=1)
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    scores = torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale
    if mask is not None:
        if mask.dtype == torch.bool:
            # -inf (not finfo.min): a FULLY-masked row (pad query) must
            # produce zero output, not a uniform average (softmax over a
            # constant-min row is uniform — the kernel/ref divergence the
            # ragged ring test caught)
            scores = scores.masked_fill(~mask, float("-inf"))
        else:
            scores = scores + mask.float()
    if sinks is not None:
        sink_col = sinks.float().view(1, Hq, 1, 1).expand(B, Hq, Sq, 1)
        scores = torch.cat([scores, sink_col], dim=-1)
        probs = torch.softmax(scores, dim=-1)[..., :-1]
    else:
        probs = torch.softmax(scores, dim=-1)
    probs = torch.nan_to_num(probs)  # fully-masked rows -> 0
    out = torch.matmul(probs, v.float())
    return out.to(q.dtype)


def paged_gather_kv(
    k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, max_len: int
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gather per-sequence contiguous (B,Hkv,S,D) K/V from a paged cache via
    `block_table` (B, max_blocks) (ref `block_kv_cache_manager.py:150-182`)."""
    B = block_table.shape[0]
    bs = k_cache.shape[1]
    nblk = (max_len + bs - 1) // bs
    tbl = block_table[:, :nblk].long().clamp(min=0)
    k = k_cache[tbl]  # (B, nblk, bs, Hkv, D)
    v = v_cache[tbl]
    k = k.flatten(1, 2)[:, :max_len].permute(0, 2, 1, 3)
    v = v.flatten(1, 2)[:, :max_len].permute(0, 2, 1, 3)
    return k.contiguous(), v.contiguous()


def topk_topp_sample(
    logits: torch.Tensor,
    top_k: torch.Tensor,
    top_p: torch.Tensor,
    temperature: torch.Tensor,
    rand: torch.Tensor,
    global_topk: int = 256,
) -> torch.Tensor:
    """Per-request top-k -> temperature -> top-p -> inverse-CDF sample
    (ref `modules/generation/sampling.py:285-370`).

    logits: (B, V); top_k/top_p/temperature/rand: (B,). rand in [0,1).
    Returns (B,) sampled token ids. top_k<=0 means greedy.
    """
    B, V = logits.shape
    kcap = min(global_topk, V)
    vals, idxs = logits.float().topk(kcap, dim=-1)  # sorted desc
    out = torch.empty(B, dtype=torch.long, device=logits.device)
    for b in range(B):
        k = int(top_k[b])
        if k == 1:
            out[b] = idxs[b, 0]
            continue
        k = kcap if k <= 0 else min(k, kcap)
        vb = vals[b, :k] / max(float(temperature[b]), 1e-6)
        probs = torch.softmax(vb, dim=-1)
        p = float(top_p[b])
        if p < 1.0:
            csum = probs.cumsum(0)
            keep = (csum - probs) < p  # always keep the first token
            probs = probs * keep
            probs = probs / probs.sum()
        cdf = probs.cumsum(0)
        j = int(torch.searchsorted(cdf, rand[b].float().clamp(max=1 - 1e-7)))
        j = min(j, k - 1)
        out[b] = idxs[b, j]
    return out


# ----------------------------------------------------------------------
# Sequence-mixing ops of the hybrid (windowed attention + linear
# recurrence) models. All take the engine's ragged step layout: (B, S)
# rows whose real tokens sit at columns 0..n-1 with consecutive positions
# p0..p0+n-1; pad columns carry position -1 and pad rows seq_id -1.

def layer_norm(x: torch.Tensor, weight: torch.Tensor, eps: float,
               out_dtype: torch.dtype) -> torch.Tensor:
    """Bias-free LayerNorm with fp32 statistics."""
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    xc = xf - mu
    var = (xc * xc).mean(-1, keepdim=True)
    return (xc * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)


def _row_extent(positions: torch.Tensor):
    valid = positions >= 0
    return valid.sum(-1), positions[:, 0]


def _masked_tail(tail_row: torch.Tensor, p0: int) -> torch.Tensor:
    """Tail rows hold inputs p0-R..p0-1 (oldest first); the ones that lie
    before the sequence start read as zero."""
    R = tail_row.shape[0]
    src = p0 - R + torch.arange(R, device=tail_row.device)
    return tail_row * (src >= 0).view(R, 1).to(tail_row.dtype)


def short_conv(x, w, tail, positions, seq_ids, activation="none",
               residual=False, out_dtype=torch.float32, bias=None):
    """Depthwise causal convolution over time with a carried tail:
    y_t = sum_j w[:, j] * x_{t-(taps-1)+j} (+ bias); the last column of `w`
    multiplies the current token. x (B,S,C); w (C,taps); tail
    (slots, taps-1, C) fp32; bias (C,) or None."""
    B, S, C = x.shape
    taps = w.shape[1]
    R = taps - 1
    xf = x.float()
    wf = w.float()
    y = torch.zeros(B, S, C, dtype=torch.float32, device=x.device)
    n_valid, p0s = _row_extent(positions)
    for b in range(B):
        slot = int(seq_ids[b])
        n = int(n_valid[b])
        if slot < 0 or n == 0:
            continue
        ext = torch.cat([_masked_tail(tail[slot].float(), int(p0s[b])), xf[b, :n]], 0)
        acc = torch.zeros(n, C, dtype=torch.float32, device=x.device)
        for j in range(taps):
            acc = acc + wf[:, j] * ext[j:j + n]
        if bias is not None:
            acc = acc + bias.float()
        y[b, :n] = acc
    if activation == "silu":
        y = torch.nn.functional.silu(y)
    if residual:
        y = y + xf
    return y.to(out_dtype)


def short_conv_commit(x, tail, positions, seq_ids):
    """Advance the carried tail by this step's inputs."""
    B = x.shape[0]
    R = tail.shape[1]
    n_valid, p0s = _row_extent(positions)
    for b in range(B):
        slot = int(seq_ids[b])
        n = int(n_valid[b])
        if slot < 0 or n == 0:
            continue
        ext = torch.cat([_masked_tail(tail[slot].float(), int(p0s[b])),
                         x[b, :n].float()], 0)
        tail[slot] = ext[-R:].to(tail.dtype)


def paged_kv_write(k_cache, v_cache, k_new, v_new, slot_mapping):
    """k_new (N,G,Dk), v_new (N,G,Dv) into (blocks, block, G, D*) caches;
    K and V may have different head sizes."""
    ok = slot_mapping >= 0
    idx = slot_mapping[ok].long()
    kc = k_cache.view(-1, *k_cache.shape[2:])
    kc[idx] = k_new[ok].to(kc.dtype)
    if v_cache is not None:          # caches whose values live inside the key rows
        vc = v_cache.view(-1, *v_cache.shape[2:])
        vc[idx] = v_new[ok].to(vc.dtype)


def paged_attention(q, k_cache, v_cache, positions, block_table, scale,
                    window=None, keep_first=0, r1=None, r2=None, gate=None,
                    softcap=0.0, sink=None, q_temp=None, out_dtype=torch.float32,
                    gate_per_head=False, chunk=0, slopes=None):
    """Softmax attention of ragged queries against a paged cache, every
    option a parameter. Query at position i sees key j <= i when no window
    is given, else when i-j < window or j < keep_first; with ``chunk`` > 0
    also only keys of its own block of ``chunk`` positions (floor(i/chunk)
    = floor(j/chunk), blocks counted from position 0). ``slopes`` (H,)
    takes slope_h * (i-j) off the score. Score, in order:
    q.k * scale * temp(i) with temp(i) = 1 + coef*ln(floor((i+1)/every)+1)
    (``q_temp`` = (coef, every)); minus r1_h*log1p(r2_h*(i-j)) when r1/r2
    are given; then softcap*tanh(score/softcap) when softcap > 0. ``sink``
    (H,) adds exp(sink_h) to the softmax denominator (a key without value).
    ``v_cache`` may be a narrowed view of ``k_cache`` (values stored inside
    the key rows). q (B,S,H,Dk) -> (B,S,H*Dv), optionally times
    sigmoid(gate): gate (B,S,H*Dv), or (B,S,H) with ``gate_per_head`` (one
    number per head)."""
    B, S, H, Dk = q.shape
    G, Dv = v_cache.shape[2], v_cache.shape[3]
    bs = k_cache.shape[1]
    L = int(positions.max()) + 1 if positions.numel() else 0
    out = torch.zeros(B, S, H, Dv, dtype=torch.float32, device=q.device)
    if L > 0:
        nb = (L + bs - 1) // bs
        bt = block_table[:, :nb].long().clamp(min=0)
        k = k_cache[bt].reshape(B, nb * bs, G, Dk)[:, :L].float()
        v = v_cache[bt].reshape(B, nb * bs, G, Dv)[:, :L].float()
        rep = H // G
        k = k.repeat_interleave(rep, dim=2)
        v = v.repeat_interleave(rep, dim=2)
        s = torch.einsum("bshd,blhd->bhsl", q.float(), k) * scale
        i = positions.view(B, 1, S, 1).float()
        j = torch.arange(L, device=q.device).view(1, 1, 1, L).float()
        if q_temp is not None:
            coef, every = q_temp
            s = s * (1.0 + coef * torch.log(torch.floor((i.clamp(min=0) + 1) / every) + 1.0))
        if r1 is not None:
            dist = (i - j).clamp(min=0)
            s = s - r1.float().view(1, H, 1, 1) * torch.log1p(
                r2.float().view(1, H, 1, 1) * dist)
        if slopes is not None:
            s = s - slopes.float().view(1, H, 1, 1) * (i - j).clamp(min=0)
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        vis = j <= i
        if window is not None:
            vis = vis & ((i - j < window) | (j < keep_first))
        if chunk:
            vis = vis & (torch.floor(i / chunk) == torch.floor(j / chunk))
        s = s.masked_fill(~vis, float("-inf"))
        if sink is not None:
            sk = sink.float().view(1, H, 1, 1).expand(B, H, S, 1)
            p = torch.nan_to_num(torch.softmax(torch.cat([s, sk], -1), dim=-1))[..., :L]
        else:
            p = torch.nan_to_num(torch.softmax(s, dim=-1))
        out = torch.einsum("bhsl,blhd->bshd", p, v)
    if gate is not None and gate_per_head:
        out = out.reshape(B, S, H, Dv) * torch.sigmoid(gate.float()).view(B, S, H, 1)
    out = out.reshape(B, S, H * Dv)
    if gate is not None and not gate_per_head:
        out = out * torch.sigmoid(gate.float())
    return out.to(out_dtype)


def window_bias_attention(q, k_cache, v_cache, positions, block_table, r1, r2,
                          scale, window, keep_first, gate=None,
                          out_dtype=torch.float32):
    """Sliding window plus kept first tokens, log-distance score penalty."""
    return paged_attention(q, k_cache, v_cache, positions, block_table, scale,
                           window=window, keep_first=keep_first, r1=r1, r2=r2,
                           gate=gate, out_dtype=out_dtype)


def gated_delta_rule(qkv, beta, a, dt_bias, a_log, gate, norm_w, eps, state,
                     positions, seq_ids, kv_heads, dim, vdim,
                     out_dtype=torch.float32, gate_act="sigmoid"):
    """Delta-rule recurrence with a decay per head and key channel (``a``
    (B,S,H*dim)) or one per head (``a`` (B,S,H), dt_bias (H)), carried state
    (slots, H, vdim, dim) fp32 (stored transposed: a value channel's key
    rows are contiguous). qkv (B,S,2*G*dim + H*vdim) holds the
    convolved+activated q|k|v; beta (B,S,H) and a (B,S,H*dim), gate
    (B,S,H*vdim) are pre-activation projections. Per token and head:
      S <- diag(decay) S ; u = beta (v - S^T k) ; S <- S + k u^T ; o = S^T q
    followed by o / rms(o) * norm_w * act(gate), act = sigmoid or silu."""
    B, S, _ = qkv.shape
    G, D, Dv = kv_heads, dim, vdim
    H = beta.shape[-1]
    rep = H // G
    f = qkv.float()
    q = f[..., :G * D].view(B, S, G, D)
    k = f[..., G * D:2 * G * D].view(B, S, G, D)
    v = f[..., 2 * G * D:].view(B, S, H, Dv)
    q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6) * (D ** -0.5)
    k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q = q.repeat_interleave(rep, dim=2)
    k = k.repeat_interleave(rep, dim=2)
    bt = torch.sigmoid(beta.float())
    dt = torch.nn.functional.softplus(a.float() + dt_bias.float()).view(B, S, H, -1)
    decay = torch.exp(-torch.exp(a_log.float()).view(1, 1, H, 1) * dt).expand(B, S, H, D)
    out = torch.zeros(B, S, H, Dv, dtype=torch.float32, device=qkv.device)
    n_valid, p0s = _row_extent(positions)
    for b in range(B):
        slot = int(seq_ids[b])
        n = int(n_valid[b])
        if slot < 0 or n == 0:
            continue
        St = state[slot].float().transpose(-1, -2) if int(p0s[b]) > 0 else torch.zeros(
            H, D, Dv, dtype=torch.float32, device=qkv.device)
        for t in range(n):
            St = decay[b, t].unsqueeze(-1) * St
            u = bt[b, t].unsqueeze(-1) * (v[b, t] - torch.einsum("hdv,hd->hv", St, k[b, t]))
            St = St + k[b, t].unsqueeze(-1) * u.unsqueeze(1)
            out[b, t] = torch.einsum("hdv,hd->hv", St, q[b, t])
        state[slot] = St.transpose(-1, -2).to(state.dtype)
    out = out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps) * norm_w.float()
    gf = gate.float()
    gf = torch.sigmoid(gf) if gate_act == "sigmoid" else torch.nn.functional.silu(gf)
    out = out.reshape(B, S, H * Dv) * gf
    return out.to(out_dtype)


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(logits.float() / cap)


def rms_norm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float,
                  one_plus: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w  (or * (1 + w)), fp32 statistics."""
    xf = x.float()
    w = weight.float()
    y = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * (1.0 + w if one_plus else w)
    return y.to(out_dtype)


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor,
                       inv_freq: torch.Tensor) -> torch.Tensor:
    """Rotary positions on channel pairs (2i, 2i+1) of the first
    2*len(inv_freq) channels of the last axis, angle p * inv_freq[i] in
    fp32; the other channels pass unchanged. x (B,S,N,C), positions (B,S);
    returns fp32."""
    B, S = positions.shape
    dims = 2 * inv_freq.numel()
    xf = x.float().clone()
    ang = positions.clamp(min=0).float().view(B, S, 1, 1) * inv_freq.float()
    c, sn = torch.cos(ang), torch.sin(ang)
    a, b = xf[..., 0:dims:2].clone(), xf[..., 1:dims:2].clone()
    xf[..., 0:dims:2] = a * c - b * sn
    xf[..., 1:dims:2] = b * c + a * sn
    return xf


def clamped_glu(gate: torch.Tensor, up: torch.Tensor, limit: float,
                alpha: float = 1.702) -> torch.Tensor:
    """min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, +-limit) + 1)."""
    g = gate.float().clamp(max=limit)
    u = up.float().clamp(-limit, limit)
    return g * torch.sigmoid(alpha * g) * (u + 1.0)


def head_norm_rotate(x: torch.Tensor, positions: torch.Tensor, norm_weight, eps: float,
                     inv_freq, mscale: float = 1.0) -> torch.Tensor:
    """Per-head RMS norm (weight (C,) shared by the heads; None = no norm)
    followed by rotary positions in the half-split layout: inside the first
    2*len(inv_freq) channels of every head, channel i pairs with channel
    i + len(inv_freq); angle p * inv_freq[i] in fp32, cos and sin times
    ``mscale``; the other channels pass unchanged (``inv_freq`` None = no
    rotation). x (B,S,N,C), positions (B,S); returns fp32."""
    B, S = positions.shape
    xf = x.float()
    if norm_weight is not None:
        xf = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * norm_weight.float()
    if inv_freq is None or inv_freq.numel() == 0:
        return xf
    half = inv_freq.numel()
    ang = positions.clamp(min=0).float().view(B, S, 1, 1) * inv_freq.float()
    c, sn = torch.cos(ang) * mscale, torch.sin(ang) * mscale
    u, v = xf[..., :half], xf[..., half:2 * half]
    return torch.cat([u * c - v * sn, v * c + u * sn, xf[..., 2 * half:]], dim=-1)


def decay_scan(q, k, v, state, positions, seq_ids, dim: int, vdim: int,
               dt=None, dt_bias=None, a_log=None, head_decay=None,
               k_scale: float = 1.0, skip=None):
    """Linear recurrence with a scalar decay per head and matrix state,
    carried in ``state`` (slots, H, vdim, dim) fp32 (stored transposed):

        S_t = a_t S_{t-1} + k_t (w_t v_t)^T ;  o_t = S_t^T q_t (+ skip_h v_t)

    Two ways to give the decay: ``dt`` (B,S,H) raw step-size projections with
    ``dt_bias`` and ``a_log`` (H,): w_t = softplus(dt + dt_bias), a_t =
    exp(-exp(a_log) w_t) (selective state spaces: k = B, q = C, v = x); or
    ``head_decay`` (H,): a_t = head_decay, w_t = 1 (retention). q, k
    (B,S,G*dim) are shared by H/G consecutive heads, v (B,S,H*vdim); k is
    multiplied by ``k_scale``. Returns fp32 (B,S,H*vdim)."""
    B, S = positions.shape
    D, Dv = dim, vdim
    H = v.shape[-1] // Dv
    G = q.shape[-1] // D
    rep = H // G
    qf = q.float().reshape(B, S, G, D).repeat_interleave(rep, dim=2)
    kf = (k.float() * k_scale).reshape(B, S, G, D).repeat_interleave(rep, dim=2)
    vf = v.float().reshape(B, S, H, Dv)
    if dt is not None:
        w = torch.nn.functional.softplus(dt.float() + dt_bias.float(), threshold=20.0)
        a = torch.exp(-torch.exp(a_log.float()) * w)
    else:
        a = head_decay.float().view(1, 1, H).expand(B, S, H)
        w = torch.ones(B, S, H, dtype=torch.float32, device=v.device)
    out = torch.zeros(B, S, H, Dv, dtype=torch.float32, device=v.device)
    n_valid, p0s = _row_extent(positions)
    for b in range(B):
        slot = int(seq_ids[b])
        n = int(n_valid[b])
        if slot < 0 or n == 0:
            continue
        St = state[slot].float().transpose(-1, -2).clone() if int(p0s[b]) > 0 else torch.zeros(
            H, D, Dv, dtype=torch.float32, device=v.device)
        for t in range(n):
            St = a[b, t].view(H, 1, 1) * St + kf[b, t].unsqueeze(-1) * (
                w[b, t].view(H, 1) * vf[b, t]).unsqueeze(1)
            out[b, t] = torch.einsum("hdv,hd->hv", St, qf[b, t])
        state[slot] = St.transpose(-1, -2).to(state.dtype)
    if skip is not None:
        out = out + skip.float().view(1, 1, H, 1) * vf
    return out.reshape(B, S, H * Dv)


def group_gated_norm(y, gate, weight, eps: float, groups: int, gate_first: bool,
                     out_dtype=torch.float32):
    """RMS norm of (.., C) rows in ``groups`` equal parts (each part by its
    own root mean square), optional weight (C,), and a silu gate applied
    before the norm (``gate_first``) or after it."""
    yf = y.float()
    g = torch.nn.functional.silu(gate.float())
    if gate_first:
        yf = yf * g
    shp = yf.shape
    yg = yf.reshape(*shp[:-1], groups, shp[-1] // groups)
    yf = (yg * torch.rsqrt((yg * yg).mean(-1, keepdim=True) + eps)).reshape(shp)
    if weight is not None:
        yf = yf * weight.float()
    if not gate_first:
        yf = yf * g
    return yf.to(out_dtype)


def group_limited_router(logits, num_experts: int, top_k: int, n_groups: int,
                         keep_groups: int, scale: float, normalize: bool = False,
                         correction=None):
    """Softmax over the first ``num_experts`` columns of fp32 ``logits``
    (T, E + extra); experts form ``n_groups`` groups of neighbours, a group
    scores as its best expert and only experts of the ``keep_groups`` best
    groups compete for the ``top_k`` places. Weights are the chosen experts'
    softmax scores times ``scale`` (divided by their sum first when
    ``normalize``). ``correction`` (E,) is added to the scores for the choice
    only (the weights stay the scores). Extra columns are per-token sigmoid
    gates. Returns
    (dense (T, E + extra) fp32 with zeros at unchosen experts, idx (T, top_k)
    int32, weights (T, top_k) fp32)."""
    T = logits.shape[0]
    E = num_experts
    lf = logits.float()
    s = torch.softmax(lf[:, :E], dim=-1)
    cand = s if correction is None else s + correction.float()
    if n_groups > 1 and keep_groups < n_groups:
        per = E // n_groups
        gs = s.view(T, n_groups, per).max(-1).values
        best = gs.topk(keep_groups, dim=-1).indices
        gmask = torch.zeros_like(gs, dtype=torch.bool).scatter(1, best, True)
        cand = torch.where(gmask.repeat_interleave(per, dim=1), cand,
                           torch.full_like(s, float("-inf")))
    idx = cand.topk(top_k, dim=-1).indices
    w = s.gather(1, idx)
    if normalize:
        w = w / w.sum(-1, keepdim=True)
    w = w * scale
    dense = torch.zeros_like(lf)
    dense[:, :E] = torch.zeros_like(s).scatter(1, idx, w)
    dense[:, E:] = torch.sigmoid(lf[:, E:])
    return dense, idx.to(torch.int32), w


def clamped_glu_scale(hid, gates, expert_ff: int, num_experts: int, limit: float,
                      shared_limit: float, alpha: float, out_dtype):
    """Clamped gated units of stacked experts: ``hid`` (T, 2*C) holds
    [gate | up] pre-activations of C = E*ff + rest columns; column c < E*ff
    belongs to expert c // ff (clamp ``limit``, times the token's routing
    weight ``gates[t, c // ff]``), the remaining columns to an always-on
    shared expert (clamp ``shared_limit``, weight one). ``gates`` (T, >= E)
    fp32; further columns are ignored."""
    T, C2 = hid.shape
    C = C2 // 2
    E = num_experts
    g, u = hid.float()[:, :C], hid.float()[:, C:]
    ne = E * expert_ff
    out = torch.empty(T, C, dtype=torch.float32, device=hid.device)
    if ne:
        cols = torch.arange(ne, device=hid.device) // expert_ff
        out[:, :ne] = clamped_glu(g[:, :ne], u[:, :ne], limit, alpha) * gates.float()[:, cols]
    if C > ne:
        out[:, ne:] = clamped_glu(g[:, ne:], u[:, ne:], shared_limit, alpha)
    return out.to(out_dtype)


def relu2_scale(hid, gates, expert_ff: int, num_experts: int, out_dtype):
    """(T, E*ff + rest) hidden pre-activations -> relu(x)^2 times the token's
    gate of the column's owner: column c < E*ff belongs to expert c // ff,
    the remaining columns (a shared expert) to gate column E; ``gates`` is
    (T, E + 1), or (T, E) when there are no remaining columns, or None for a
    plain relu(x)^2."""
    T, C = hid.shape
    E = num_experts
    hf = torch.relu(hid.float()) ** 2
    if gates is None:
        return hf.to(out_dtype)
    assert C == E * expert_ff or gates.shape[1] == E + 1
    cols = (torch.arange(C, device=hid.device) // expert_ff).clamp(max=E)
    return (hf * gates.float()[:, cols]).to(out_dtype)


def scaled_residual(x, terms):
    """In place on the fp32 stream: x += sum_i f_i(y_i) * w_i with w_i a
    per-channel vector and f_i the identity or an RMS norm over the row
    (``terms``: (y, w, eps or None))."""
    for y, w, eps in terms:
        yf = y.float()
        if eps is not None:
            yf = yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps)
        x.add_(yf * w.float())
    return x
