"""Plain, slow, whole-sequence Kuterax in float64, one function per
mechanism, written from the equations. Shares no code with the package:
it is the yardstick the engine, its cache/state handling and its kernels are
compared with.

A model is ``(cfg, weights)``: ``cfg`` the checkpoint's config dictionary,
``weights`` a dict of tensors under the checkpoint's names. Every function
takes the full token sequence of ONE request; nothing is cached.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def causal_conv(x, taps_w, bias=None):
    """x (T, C), taps_w (C, K): y_t = sum_j w[:, j] x_{t-(K-1)+j} (+ bias),
    zeros before the start."""
    T, C = x.shape
    K = taps_w.shape[1]
    xp = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros(T, C, dtype=x.dtype)
    for j in range(K):
        y = y + taps_w[:, j] * xp[j:j + T]
    return y if bias is None else y + bias


# ------------------------------------------------------------------ rotary
def rotary_table(rot):
    """Per-pair frequencies (dims/2,) and the factor on cos and sin."""
    dims, base = rot["dims"], float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(t):
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(sc["fast"])), 0)
    hi = min(math.ceil(turn_dim(sc["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                         for i in range(dims // 2)], dtype=F64)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half_layout(x, rot):
    """x (T, heads, dim): channel i pairs with channel i + dims/2 inside the
    first ``dims`` channels; token t has position t."""
    T = x.shape[0]
    dims = rot["dims"]
    half = dims // 2
    f, m = rotary_table(rot)
    ang = torch.arange(T, dtype=F64).view(T, 1, 1) * f
    c, s = torch.cos(ang) * m, torch.sin(ang) * m
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# --------------------------------------------------------------- attention
def window_sink_attention(h, weights, pre, mc, eps):
    """GQA softmax attention: biased projections, per-head q/k RMS norm,
    partial rotate-half rotary with scaled frequencies, sliding window, a
    value-less zero-score sink in the denominator, one sigmoid gate per head."""
    T = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]

    def proj(name):
        y = h @ _w(weights, pre + name).T
        if pre + name + ".b" in weights:
            y = y + _w(weights, pre + name + ".b")
        return y

    q = proj("q").view(T, H, D)
    k = proj("k").view(T, G, D)
    v = proj("v").view(T, G, Dv)
    if pre + "q.norm" in weights:
        q = rms(q, eps) * _w(weights, pre + "q.norm")
        k = rms(k, eps) * _w(weights, pre + "k.norm")
    if mc.get("rot"):
        q = rotate_half_layout(q, mc["rot"])
        k = rotate_half_layout(k, mc["rot"])
    size = (mc.get("mask") or {}).get("size")
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    vis = j <= i
    if size is not None:
        vis = vis & (i - j < size)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * mc["scale"]
        e = torch.where(vis, torch.exp(s), torch.zeros_like(s))
        p = e / (1.0 + e.sum(-1, keepdim=True))
        out[:, hd] = p @ v[:, g]
    gate = torch.sigmoid(h @ _w(weights, pre + "g").T)                 # (T, H)
    out = out * gate.unsqueeze(-1)
    return out.reshape(T, H * Dv) @ _w(weights, pre + "o").T


# -------------------------------------------------------- state-space mixer
def ssd_mixer(h, weights, pre, mc, eps):
    """Mamba-2: per head an (N x vdim) state with a scalar data-dependent
    decay; gate before a norm in equal channel groups."""
    T = h.shape[0]
    Hh, P, N, G = mc["heads"], mc["vdim"], mc["state"], mc["groups"]
    inner = Hh * P
    y = h @ _w(weights, pre + "in").T
    z, xbc, dt = torch.split(y, [inner, inner + 2 * G * N, Hh], dim=-1)
    bias = _w(weights, pre + "conv.b") if pre + "conv.b" in weights else None
    xbc = silu(causal_conv(xbc, _w(weights, pre + "conv"), bias))
    x, Bm, Cm = torch.split(xbc, [inner, G * N, G * N], dim=-1)
    x = x.view(T, Hh, P)
    Bm = Bm.view(T, G, N)
    Cm = Cm.view(T, G, N)
    dt = softplus(dt + _w(weights, pre + "dt_bias"))                   # (T, Hh)
    decay = torch.exp(-torch.exp(_w(weights, pre + "A_log")) * dt)     # (T, Hh)
    Dskip = _w(weights, pre + "D")
    out = torch.zeros(T, Hh, P, dtype=F64)
    for hd in range(Hh):
        g = hd // (Hh // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = decay[t, hd] * S + dt[t, hd] * torch.outer(Bm[t, g], x[t, hd])
            out[t, hd] = S.T @ Cm[t, g] + Dskip[hd] * x[t, hd]
    yv = out.reshape(T, inner) * silu(z)
    ng = mc.get("norm_groups", 1)
    yv = rms(yv.view(T, ng, inner // ng), eps).reshape(T, inner) * _w(weights, pre + "norm")
    return yv @ _w(weights, pre + "o").T


def parallel_mixer(h, weights, pre, mc, eps):
    """Half the sum of the two branches, each RMS-normed over the width with
    its own plain weight."""
    left = window_sink_attention(h, weights, pre + "left.", mc["left"], eps)
    right = ssd_mixer(h, weights, pre + "right.", mc["right"], eps)
    return 0.5 * (rms(left, eps) * _w(weights, pre + "left.out")
                  + rms(right, eps) * _w(weights, pre + "right.out"))


# ---------------------------------------------------------------- retention
def retention_mixer(h, weights, pre, mc, eps):
    """Linear attention with one fixed decay per head, no denominator."""
    T = h.shape[0]
    H, D, Dv = mc["heads"], mc["dim"], mc["vdim"]
    q = (h @ _w(weights, pre + "q").T).view(T, H, D)
    k = (h @ _w(weights, pre + "k").T).view(T, H, D) * D ** -0.5
    v = (h @ _w(weights, pre + "v").T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = float(mc["decay"][hd]) * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    out = rms(out, eps).reshape(T, H * Dv) * silu(h @ _w(weights, pre + "g").T)
    return out @ _w(weights, pre + "o").T


# ------------------------------------------------------------- feed-forward
def relu2_expert(h, weights, pre):
    return torch.relu(h @ _w(weights, pre + "up").T) ** 2 @ _w(weights, pre + "down").T


def route(h, weights, pre, rc):
    """(T, E) matrix of expert weights, zero where an expert is not chosen."""
    E, top = rc["experts"], rc["top"]
    s = torch.softmax(h @ _w(weights, pre + "router").T, dim=-1)       # (T, E)
    allowed = torch.ones_like(s, dtype=torch.bool)
    gc = rc.get("groups")
    if gc:
        per = E // gc["count"]
        gscore = s.view(-1, gc["count"], per).max(-1).values
        best = gscore.topk(gc["keep"], dim=-1).indices
        gmask = torch.zeros_like(gscore, dtype=torch.bool).scatter(1, best, True)
        allowed = gmask.repeat_interleave(per, dim=1)
    idx = torch.where(allowed, s, torch.full_like(s, -1.0)).topk(top, dim=-1).indices
    chosen = torch.zeros_like(s, dtype=torch.bool).scatter(1, idx, True)
    return torch.where(chosen, s * rc.get("scale", 1.0), torch.zeros_like(s))


def moe_feed_forward(h, weights, pre, fc):
    wts = route(h, weights, pre, fc["router"])
    out = torch.zeros_like(h)
    for e in range(fc["router"]["experts"]):
        out = out + wts[:, e:e + 1] * relu2_expert(h, weights, pre + f"e{e}.")
    if fc.get("shared"):
        gate = torch.sigmoid(h @ _w(weights, pre + "shared.sg").T)     # (T, 1)
        out = out + gate * relu2_expert(h, weights, pre + "shared.")
    return out


# -------------------------------------------------------------------- model
def run_order(cfg):
    """[(layer index, pass number or None, opens a pass)] in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None, False) for i in range(n)]
    order = [(i, None, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        order += [(i, t, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return order + [(i, None, False) for i in range(lp["stop"], n)]


def forward(cfg, weights, tokens, return_layers=False):
    """tokens (T,) -> logits (T, vocab) [and the stream after every layer run]."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    x = _w(weights, "embed")[tokens] + _w(weights, "pos")[:T]
    x0 = x
    streams = []
    for li, t, opens in run_order(cfg):
        if opens:
            x = torch.cat([x, x0], dim=-1) @ _w(weights, "loop.in").T + _w(weights, "loop.step")[t]
        lc = cfg["layers"][li]
        pre = f"l{li}."
        h = rms(x, eps) * (1.0 + _w(weights, pre + "norm1"))
        if lc["type"] == "parallel":
            mix = parallel_mixer(h, weights, pre + "mix.", lc["mixer"], eps)
        elif lc["type"] == "retention":
            mix = retention_mixer(h, weights, pre + "mix.", lc["mixer"], eps)
        else:
            raise ValueError(lc["type"])
        upd = mix * _w(weights, pre + "ls1")
        if lc.get("mlp"):
            upd = upd + moe_feed_forward(h, weights, pre + "mlp.", lc["mlp"]) * _w(weights, pre + "ls2")
        x = x + upd
        streams.append(x)
    logits = (rms(x, eps) * (1.0 + _w(weights, "final.norm"))) @ _w(weights, "head").T
    if return_layers:
        return logits, torch.stack(streams)
    return logits
