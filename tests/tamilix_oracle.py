"""Plain, slow, whole-sequence Tamilix in float64, one function per
mechanism, written from the equations. Shares no code with the package: it
is the yardstick the engine, its cache handling and its kernels are compared
with.

A model is ``(cfg, weights)``: ``cfg`` the checkpoint's config dictionary,
``weights`` a dict of tensors under the checkpoint's names. Every function
takes the full token sequence of ONE request; nothing is cached.
"""

from __future__ import annotations

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w


def rotate_pairs(x, positions, base, dims):
    """x (T, N, C): channels (2i, 2i+1), i < dims/2, turn by the angle
    p * base^(-2i/dims); the channels from ``dims`` on pass unchanged."""
    out = x.clone()
    p = positions.to(F64).view(-1, 1)
    for i in range(dims // 2):
        a = p * float(base) ** (-2.0 * i / dims)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., 2 * i + 1] = v * torch.cos(a) + u * torch.sin(a)
    return out


def head_slopes(H):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F64)


def chunk_visible(T, size):
    """vis[i, j]: j <= i and both in the same block of ``size`` positions."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    return (j <= i) & (i // size == j // size)


def window_visible(T, size):
    """vis[i, j]: 0 <= i - j < size."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    return (j <= i) & (i - j < size)


def sink_softmax(s, vis, sink=None):
    """Softmax of the rows of s (T, T) over the visible keys; with ``sink``
    the denominator has one more term exp(sink)."""
    s = s.masked_fill(~vis, float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, torch.full_like(m, float(sink)))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(float(sink) - m)
    return e / den


def attention_mixer(h, weights, pre, mc):
    """Chunked GQA without rotation, linear distance penalty, sink. h (T, W)."""
    T = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = (h @ _w(weights, pre + "q").T).view(T, H, D)
    k = (h @ _w(weights, pre + "k").T).view(T, G, D)
    v = (h @ _w(weights, pre + "v").T).view(T, G, Dv)
    vis = chunk_visible(T, mc["mask"]["size"])
    slopes = head_slopes(H)
    sink = _w(weights, pre + "sink")
    dist = (torch.arange(T).view(T, 1) - torch.arange(T).view(1, T)).to(F64)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * mc["scale"] - slopes[hd] * dist
        out[:, hd] = sink_softmax(s, vis, sink[hd]) @ v[:, g]
    return out.reshape(T, H * Dv) @ _w(weights, pre + "o").T


def latent_attend(q, dkv, weights, pre, mc, eps):
    """The attention of the latent mixer from its projections: q (T, H *
    (dim + rot_dim)) after the query up-projection, dkv (T, kv_rank +
    rot_dim) before the latent's norm. Returns the concatenated heads."""
    T = q.shape[0]
    H, D, R, Dv, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    rot = mc["rot"]
    pos = torch.arange(T)
    q = q.view(T, H, D + R)
    c = norm(dkv[:, :C], _w(weights, pre + "dkv.norm"), eps)
    k_rot = rotate_pairs(dkv[:, C:].reshape(T, 1, R), pos, rot["base"], rot["dims"])[:, 0]
    q_rot = rotate_pairs(q[..., D:], pos, rot["base"], rot["dims"])
    k_plain = (c @ _w(weights, pre + "uk").T).view(T, H, D)
    v = (c @ _w(weights, pre + "uv").T).view(T, H, Dv)
    vis = window_visible(T, mc["mask"]["size"])
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :D] @ k_plain[:, hd].T + q_rot[:, hd] @ k_rot.T) * mc["scale"]
        out[:, hd] = sink_softmax(s, vis) @ v[:, hd]
    return out.reshape(T, H * Dv)


def latent_mixer(h, weights, pre, mc, eps):
    """Latent attention: queries through a normed latent, keys and values
    expanded from a normed latent, one rotated key part for all heads, a
    sliding window, an element-wise sigmoid gate. h (T, W)."""
    cq = norm(h @ _w(weights, pre + "dq").T, _w(weights, pre + "dq.norm"), eps)
    q = cq @ _w(weights, pre + "uq").T
    dkv = h @ _w(weights, pre + "dkv").T
    heads = latent_attend(q, dkv, weights, pre, mc, eps)
    gate = torch.sigmoid(h @ _w(weights, pre + "g").T)
    return (heads * gate) @ _w(weights, pre + "o").T


def dense_ff(h, weights, pre):
    u = torch.relu(h @ _w(weights, pre + "up").T)
    return (u * u) @ _w(weights, pre + "down").T


def clamped_expert(h, weights, pre, limit):
    g = torch.clamp(h @ _w(weights, pre + "gate").T, max=limit)
    u = torch.clamp(h @ _w(weights, pre + "up").T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ _w(weights, pre + "down").T


def route(h, weights, pre, top):
    """(chosen (T, top), weight (T, top)): softmax over all router outputs,
    choice by score + correction, weights the scores themselves."""
    s = torch.softmax(h @ _w(weights, pre + "router").T, dim=-1)
    choice = s + _w(weights, pre + "correction")
    idx = torch.topk(choice, top, dim=-1).indices
    return idx, torch.gather(s, 1, idx)


def moe_ff(h, weights, pre, fc):
    rc = fc["router"]
    E, I, top = rc["experts"], rc.get("identity", 0), rc["top"]
    idx, wts = route(h, weights, pre, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(idx[t].tolist(), wts[t]):
            if e >= E:                      # identity expert: the input itself
                assert e < E + I
                out[t] += wt * h[t]
            else:
                out[t] += wt * clamped_expert(h[t:t + 1], weights, pre + f"e{e}.",
                                              fc["expert"]["limit"])[0]
    if fc.get("shared"):
        out = out + clamped_expert(h, weights, pre + "shared.", fc["shared"]["limit"])
    return out


def owner(cfg, i):
    """Index of the layer whose tensors layer i uses."""
    j = cfg["layers"][i].get("weights_of")
    return i if j is None else j


def layer(x, cfg, weights, i):
    lc = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    p = f"l{owner(cfg, i)}."
    h = norm(x, _w(weights, p + "norm1"), eps)
    if lc["type"] == "attention":
        y = attention_mixer(h, weights, p + "mix.", lc["mixer"])
    elif lc["type"] == "latent_attention":
        y = latent_mixer(h, weights, p + "mix.", lc["mixer"], eps)
    else:
        raise ValueError(lc["type"])
    x = x + norm(y, _w(weights, p + "norm1b"), eps)
    fc = lc.get("mlp")
    if fc:
        h = norm(x, _w(weights, p + "norm2"), eps)
        y = dense_ff(h, weights, p + "mlp.") if fc["kind"] == "dense" \
            else moe_ff(h, weights, p + "mlp.", fc)
        x = x + norm(y, _w(weights, p + "norm2b"), eps)
    return x


def forward(cfg, weights, tokens, collect=None):
    """Logits (T, vocab) in float64; ``collect`` (a list) receives the
    stream after every layer."""
    x = _w(weights, "embed")[torch.as_tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i in range(len(cfg["layers"])):
        x = layer(x, cfg, weights, i)
        if collect is not None:
            collect.append(x.clone())
    x = norm(x, _w(weights, "final.norm"), cfg["norm"]["eps"])
    return x @ _w(weights, "head").T

