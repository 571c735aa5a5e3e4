"""Kuterax (one pre-norm feeding a token mixer and a group-routed expert
feed-forward side by side; mixers: windowed sink attention + selective state
space in parallel, or retention) against the plain float64 oracle in
``kuterax_oracle.py``.

Every test builds its own small configuration and weights. The
device-parametrized tests run the torch reference ops on the CPU and the
gfx950 kernels on the GPU (``-m gpu``) through the same engine code.
"""

import copy
import json
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kuterax_oracle as oracle  # noqa: E402

from neuronx_distributed_inference_amd.config import EngineConfig  # noqa: E402
from neuronx_distributed_inference_amd.models.kuterax.modeling_kuterax import (  # noqa: E402
    KuteraxForCausalLM,
    KuteraxInferenceConfig,
)
from neuronx_distributed_inference_amd.modules.attention.window_sink_attention import (  # noqa: E402
    RotaryWindowSinkAttention,
)
from neuronx_distributed_inference_amd.modules.kvcache.block_kv_cache_manager import (  # noqa: E402
    BlockKVCacheManager,
    RecurrentStateManager,
    generate_slot_mapping,
)
from neuronx_distributed_inference_amd.modules.linear_recurrence import (  # noqa: E402
    Retention,
    StateSpaceDuality,
)
from neuronx_distributed_inference_amd.modules.moe import GroupRoutedFeedForward  # noqa: E402
from neuronx_distributed_inference_amd.modules.rope import half_split_inv_freq  # noqa: E402
from neuronx_distributed_inference_amd.ops import seqmix  # noqa: E402
from neuronx_distributed_inference_amd.serving import ServingEngine  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32 = torch.float32
BF16 = torch.bfloat16
F64 = torch.float64
EPS = 1e-5


# ---------------------------------------------------------------- builders
def left_cfg(heads=4, kv_heads=2, dim=8, vdim=6, size=5, scale=0.4, base=100.0, dims=None,
             scaling=None):
    rot = {"base": base, "dims": dims or dim}
    if scaling:
        rot["scaling"] = scaling
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "mask": {"size": size}, "rot": rot}


YARN = {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 0.5}


def right_cfg(heads=4, vdim=6, state=8, groups=2, conv=3, norm_groups=2):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
            "norm_groups": norm_groups}


def ret_cfg(heads=2, dim=8, vdim=4, decay=(0.9, 0.99)):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def moe_cfg(experts=8, top=3, count=4, keep=2, scale=1.5, ff=12, shared=20):
    fc = {"kind": "moe", "expert": {"ff": ff},
          "router": {"experts": experts, "top": top, "scale": scale,
                     "groups": {"count": count, "keep": keep}}}
    if shared:
        fc["shared"] = {"ff": shared}
    return fc


def layer(kind, mixer, mlp="default"):
    return {"type": kind, "mixer": mixer, "mlp": moe_cfg() if mlp == "default" else mlp}


def model_cfg(layers=None, width=16, vocab=37, loop="default", max_positions=128):
    layers = layers or [
        layer("parallel", {"left": left_cfg(scaling=YARN), "right": right_cfg()}),
        layer("retention", ret_cfg()),
        layer("parallel", {"left": left_cfg(size=7, dims=4), "right": right_cfg()}, mlp=None),
        layer("retention", ret_cfg(decay=(0.5, 0.999))),
    ]
    cfg = {"architecture": "Kuterax", "width": width, "vocab": vocab,
           "max_positions": max_positions, "norm": {"eps": EPS}, "layers": layers}
    if loop == "default":
        loop = {"start": 1, "stop": 3, "times": 2}
    if loop:
        cfg["loop"] = loop
    return cfg


def varied_cfg():
    """Other sizes and another order: one KV head, heads == KV heads, one
    group, three norm groups, sizes that are no powers of two, two taps, a
    loop that starts at the first layer and runs three times, a window of one
    token, a router without groups, a single chosen expert, no shared expert,
    rotation on all channels without frequency scaling."""
    return model_cfg(layers=[
        layer("retention", ret_cfg(3, 5, 7, (0.8, 0.95, 1.0)), mlp=moe_cfg(6, 3, 1, 1, 0.7, 10, 0)),
        layer("parallel", {"left": left_cfg(3, 1, 6, 5, size=9, scale=0.6, base=9.0),
                           "right": right_cfg(3, 5, 5, 1, 2, 3)},
              mlp=moe_cfg(9, 1, 3, 1, 2.0, 8, 14)),
        layer("parallel", {"left": left_cfg(3, 3, 10, 4, size=1, scale=0.3, dims=6),
                           "right": right_cfg(6, 4, 3, 3, 4, 1)}, mlp=None),
        layer("retention", ret_cfg(1, 12, 9, (0.97,))),
    ], width=24, vocab=29, loop={"start": 0, "stop": 2, "times": 3})


def make_weights(cfg, seed=0):
    """Checkpoint-named tensors, values exactly representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    Wd = cfg["width"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def uni(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).bfloat16().float()

    def lin(o, i, gain=1.0):
        return rnd(o, i, std=gain / i ** 0.5)

    W["embed"] = rnd(cfg["vocab"], Wd)
    W["pos"] = rnd(cfg["max_positions"], Wd, std=0.5)
    W["head"] = lin(cfg["vocab"], Wd)
    W["final.norm"] = rnd(Wd, std=0.2)
    if cfg.get("loop"):
        W["loop.in"] = lin(Wd, 2 * Wd, 1.4)
        W["loop.step"] = rnd(cfg["loop"]["times"], Wd, std=0.3)
    for i, lc in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = p + "mix."
        mc = lc["mixer"]
        W[p + "norm1"] = rnd(Wd, std=0.2)
        W[p + "ls1"] = (0.7 + rnd(Wd, std=0.2)).bfloat16().float()
        if lc["type"] == "parallel":
            L, R = mc["left"], mc["right"]
            H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
            for n, ch in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                W[m + "left." + n] = lin(ch, Wd, 2.0)
                W[m + "left." + n + ".b"] = rnd(ch, std=0.3)
            W[m + "left.q.norm"] = (1 + rnd(D, std=0.3)).bfloat16().float()
            W[m + "left.k.norm"] = (1 + rnd(D, std=0.3)).bfloat16().float()
            W[m + "left.g"] = lin(H, Wd, 2.0)
            W[m + "left.o"] = lin(Wd, H * Dv)
            W[m + "left.out"] = (1 + rnd(Wd, std=0.2)).bfloat16().float()
            Hr, P, N, Gr = R["heads"], R["vdim"], R["state"], R["groups"]
            inner, ch = Hr * P, Hr * P + 2 * Gr * N
            W[m + "right.in"] = lin(2 * inner + 2 * Gr * N + Hr, Wd, 2.0)
            W[m + "right.conv"] = rnd(ch, R["conv"], std=0.6)
            W[m + "right.conv.b"] = rnd(ch, std=0.3)
            W[m + "right.dt_bias"] = rnd(Hr)
            W[m + "right.A_log"] = uni(Hr, -1.0, 0.5)
            W[m + "right.D"] = rnd(Hr)
            W[m + "right.norm"] = (1 + rnd(inner, std=0.1)).bfloat16().float()
            W[m + "right.o"] = lin(Wd, inner)
            W[m + "right.out"] = (1 + rnd(Wd, std=0.2)).bfloat16().float()
        else:
            H, D, Dv = mc["heads"], mc["dim"], mc["vdim"]
            W[m + "q"] = lin(H * D, Wd, 2.0)
            W[m + "k"] = lin(H * D, Wd, 2.0)
            W[m + "v"] = lin(H * Dv, Wd, 2.0)
            W[m + "g"] = lin(H * Dv, Wd, 2.0)
            W[m + "o"] = lin(Wd, H * Dv)
        fc = lc["mlp"]
        if fc:
            W[p + "ls2"] = (0.7 + rnd(Wd, std=0.2)).bfloat16().float()
            W.update(moe_weights(fc, Wd, p + "mlp.", g))
    return W


def moe_weights(fc, Wd, pre, g):
    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    W = {}
    ff = fc["expert"]["ff"]
    for e in range(fc["router"]["experts"]):
        W[pre + f"e{e}.up"] = rnd(ff, Wd, std=1.5 / Wd ** 0.5)
        W[pre + f"e{e}.down"] = rnd(Wd, ff, std=1.0 / ff ** 0.5)
    # a wide spread of router logits: no near ties between experts
    W[pre + "router"] = rnd(fc["router"]["experts"], Wd, std=6.0 / Wd ** 0.5)
    if fc.get("shared"):
        sf = fc["shared"]["ff"]
        W[pre + "shared.up"] = rnd(sf, Wd, std=1.5 / Wd ** 0.5)
        W[pre + "shared.down"] = rnd(Wd, sf, std=1.0 / sf ** 0.5)
        W[pre + "shared.sg"] = rnd(1, Wd, std=2.0 / Wd ** 0.5)
    return W


def make_engine(cfg, W, device="cpu", dtype="float32", slots=3, page=4, pages=40,
                max_len=96, **engine_kw):
    ec = EngineConfig(batch_size=slots, max_batch_size=slots, kv_cache_batch_size=slots,
                      seq_len=max_len, max_length=max_len, torch_dtype=dtype, tp_degree=1,
                      is_block_kv_layout=True, pa_block_size=page, pa_num_blocks=pages,
                      enable_hip_graphs=False)
    config = KuteraxInferenceConfig(neuron_config=ec, **copy.deepcopy(cfg))
    model = KuteraxForCausalLM(config)
    sd = KuteraxForCausalLM.convert_hf_to_native_state_dict(W, config)
    missing, unexpected = model.model.load_state_dict(sd, strict=False)
    assert not unexpected and all(m.startswith("kv_mgr.") for m in missing), (missing, unexpected)
    model = model.to(device).eval()
    engine_kw.setdefault("capture_decode", False)
    engine_kw.setdefault("async_depth", 1)
    return ServingEngine(model, max_slots=slots, **engine_kw)


def feed(engine, tokens, cuts):
    """One request alone, fed in portions of the given sizes; logits (T, V)."""
    req = engine.admit()
    out, at = [], 0
    for n in cuts:
        lg = engine.forced_step([(req, torch.tensor(tokens[at:at + n]))])
        out.append(lg[0, :n].float().cpu())
        at += n
    assert at == len(tokens)
    engine.release(req)
    return torch.cat(out)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def close(got, want, tol, rtol=0.0):
    """|got - want| <= tol + rtol * |want| everywhere."""
    excess = ((got.double() - want.double()).abs() - rtol * want.double().abs()).max().item()
    assert excess < tol, excess


def step_for(pos, slots, device):
    return seqmix.StepLayout(pos.to(device), torch.as_tensor(slots).to(device))


# ------------------------------------------------------------ single ops
def test_frequency_table_by_parts():
    for rot in ({"base": 100.0, "dims": 8, "scaling": YARN},
                {"base": 5e4, "dims": 32, "scaling": {"factor": 8.0, "original": 64,
                                                      "fast": 16.0, "slow": 2.0}},
                {"base": 9.0, "dims": 6}):
        f, m = half_split_inv_freq(rot["base"], rot["dims"], rot.get("scaling"))
        wf, wm = oracle.rotary_table(rot)
        close(f, wf, 1e-9, rtol=1e-6)
        assert abs(m - wm) < 1e-12
    # the ramp really bends the table: the slowest pair is divided by the factor
    f, _ = half_split_inv_freq(100.0, 8, YARN)
    plain, _ = half_split_inv_freq(100.0, 8)
    assert abs(float(f[-1]) * 3.0 - float(plain[-1])) < 1e-6 and float(f[0]) == float(plain[0])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("C,dims,norm", [(6, 6, True), (10, 4, True), (16, 16, False),
                                        (7, 0, True), (72, 64, True)])
def test_head_norm_rotate_op(device, C, dims, norm):
    torch.manual_seed(2)
    B, S, N = 2, 5, 3
    wide = torch.randn(B, S, N * C + 5)
    x = wide[..., 5:].unflatten(-1, (N, C))             # a strided view, read in place
    pos = torch.tensor([[900, 901, 902, 903, 904], [0, 1, 2, -1, -1]])
    st = step_for(pos, [0, 1], device)
    w = (1 + 0.3 * torch.randn(C)) if norm else None
    rot = {"base": 100.0, "dims": dims, "scaling": YARN} if dims else None
    inv, m = half_split_inv_freq(100.0, dims, YARN) if dims else (None, 1.0)
    got = seqmix.head_norm_rotate(x.to(device), st, None if w is None else w.to(device), EPS,
                                  None if inv is None else inv.to(device), m,
                                  out_dtype=F32).cpu()
    for b in range(B):
        n = int((pos[b] >= 0).sum())
        xs = x[b, :n].double()
        if norm:
            xs = oracle.rms(xs, EPS) * w.double()
        if rot:
            # the oracle counts positions from 0: rotate a longer run and cut
            p0 = int(pos[b, 0])
            full = torch.zeros(p0 + n, N, C, dtype=F64)
            full[p0:] = xs
            xs = oracle.rotate_half_layout(full, rot)[p0:]
        close(got[b, :n].view(n, N, C), xs, 3e-4)       # fp32 angles near position 900


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("groups,gate_first,weighted", [(2, True, True), (3, False, False),
                                                       (1, True, False), (4, False, True)])
def test_group_gated_norm_op(device, groups, gate_first, weighted):
    torch.manual_seed(4)
    C = 24
    y = torch.randn(3, 5, C) * 2
    wide = torch.randn(3, 5, C + 9)
    gate = wide[..., 9:]
    w = (1 + 0.2 * torch.randn(C)) if weighted else None
    g = oracle.silu(gate.double())
    v = y.double() * g if gate_first else y.double()
    v = oracle.rms(v.view(3, 5, groups, C // groups), EPS).reshape(3, 5, C)
    if weighted:
        v = v * w.double()
    if not gate_first:
        v = v * g
    got = seqmix.group_gated_norm(y.to(device), gate.to(device),
                                  None if w is None else w.to(device), EPS, groups, gate_first)
    close(got.cpu(), v, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,count,keep,extra", [(8, 3, 4, 2, 1), (12, 3, 3, 2, 0),
                                                   (6, 3, 1, 1, 1), (9, 1, 3, 1, 0),
                                                   (130, 5, 13, 4, 1)])
def test_group_limited_router_op(device, E, top, count, keep, extra):
    torch.manual_seed(5)
    T, Wd = 33, 12
    h = torch.randn(T, Wd).double()
    Wr = torch.randn(E, Wd).double() * 1.5
    rc = {"experts": E, "top": top, "scale": 1.7, "groups": {"count": count, "keep": keep}}
    want = oracle.route(h, {"p.router": Wr}, "p.", rc)
    logits = torch.cat([h @ Wr.T, torch.randn(T, extra).double()], 1).float()
    dense, idx, wts = seqmix.group_limited_router(logits.to(device), E, top, count, keep, 1.7)
    close(dense[:, :E].cpu(), want, 1e-5)
    if extra:
        close(dense[:, E:].cpu(), torch.sigmoid(logits[:, E:].double()), 1e-6)
    assert sorted(idx[0].tolist()) == sorted(want[0].nonzero().flatten().tolist())
    close(wts.sum(-1).cpu(), want.sum(-1), 1e-5)
    if count > 1 and keep < min(count, top):
        # the group limit matters here: plain top-k would choose otherwise somewhere
        plain = oracle.route(h, {"p.router": Wr}, "p.", {**rc, "groups": None})
        assert bool(((plain > 0) != (want > 0)).any())


@pytest.mark.parametrize("device", DEVICES)
def test_router_rows_that_are_not_numbers(device):
    """Pad tokens carry garbage: such a row must stay inside its own memory
    and leave the other rows alone."""
    torch.manual_seed(5)
    E, T = 10, 9
    logits = torch.randn(T, E + 1) * 3
    clean = seqmix.group_limited_router(logits.to(device), E, 3, 5, 2, 1.0)
    logits[2] = float("nan")
    logits[7, 3] = float("inf")
    dense, idx, wts = seqmix.group_limited_router(logits.to(device), E, 3, 5, 2, 1.0)
    ok = [0, 1, 3, 4, 5, 6, 8]
    assert torch.equal(dense[ok].cpu(), clean[0][ok].cpu())
    assert int(idx.min()) >= 0 and int(idx.max()) < E


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,ff,rest", [(3, 5, 0), (4, 8, 16), (2, 12, 7)])   # scalar / 8-wide
def test_relu2_scale_op(device, E, ff, rest):
    torch.manual_seed(6)
    T = 9
    hid = torch.randn(T, E * ff + rest)
    gates = torch.rand(T, E + (1 if rest else 0))
    gates[gates < 0.4] = 0.0
    cols = (torch.arange(E * ff + rest) // ff).clamp(max=E)
    want = torch.relu(hid.double()) ** 2 * gates.double()[:, cols]
    got = seqmix.relu2_scale(hid.to(device), gates.to(device), ff, E)
    close(got.cpu(), want, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("C", [40, 37, 2304])             # 16-byte / scalar / two vectors a thread
def test_scaled_residual_op(device, C):
    torch.manual_seed(7)
    x = torch.randn(2, 3, C)
    ys = [torch.randn(2, 3, C) * s for s in (3.0, 0.2, 1.0)]
    ws = [torch.randn(C) for _ in range(3)]
    for k, normed in ((1, [False]), (2, [True, True]), (3, [True, False, True])):
        want = x.double().clone()
        for y, w, nm in zip(ys[:k], ws[:k], normed):
            want += (oracle.rms(y.double(), EPS) if nm else y.double()) * w.double()
        s = x.clone().to(device)
        seqmix.scaled_residual(s, [(y.to(device), w.to(device), nm)
                                   for y, w, nm in zip(ys[:k], ws[:k], normed)], EPS)
        close(s.cpu(), want, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("C,taps", [(16, 4), (16, 2), (10, 3)])        # tiled / scalar kernels
def test_short_conv_with_bias(device, C, taps):
    """Whole sequence against portions through the carried tail, with a bias."""
    torch.manual_seed(8)
    T = 21
    x = torch.randn(T, C)
    w, bias = torch.randn(C, taps) * 0.6, torch.randn(C)
    want = oracle.silu(oracle.causal_conv(x.double(), w.double(), bias.double()))
    tail = torch.randn(2, taps - 1, C).to(device)        # stale contents
    got, at = [], 0
    for n in (9, 1, 2, 8, 1):
        pos = torch.arange(at, at + n).view(1, n)
        st = step_for(pos, [1], device)
        xs = x[at:at + n].view(1, n, C).to(device)
        got.append(seqmix.short_conv(xs, w.to(device), tail, st, "silu", bias=bias.to(device))[0])
        seqmix.short_conv_commit(xs, tail, st)
        at += n
    close(torch.cat(got).cpu(), want, 1e-5)


# ------------------------------------------------------------ attention alone
def _attention_alone(device, L, T, spikes=(), page=4, cuts=None, dtype=F32, tol=3e-5, gain=30.0):
    """The attention core on its own paged cache against the oracle. `spikes`:
    (query i, key j) pairs whose score is made to stand out (one dominant
    channel outside the rotated ones in both), so a lost or misplaced key
    shows."""
    torch.manual_seed(3)
    Wd = 12
    H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
    g = torch.Generator().manual_seed(11)
    W = {"p.q": torch.randn(H * D, Wd, generator=g).double() * 0.3,
         "p.k": torch.randn(G * D, Wd, generator=g).double() * 0.3,
         "p.v": torch.randn(G * Dv, Wd, generator=g).double(),
         "p.q.b": torch.randn(H * D, generator=g).double() * 0.2,
         "p.k.b": torch.randn(G * D, generator=g).double() * 0.2,
         "p.v.b": torch.randn(G * Dv, generator=g).double() * 0.2,
         "p.q.norm": (1 + 0.3 * torch.randn(D, generator=g)).double(),
         "p.k.norm": (1 + 0.3 * torch.randn(D, generator=g)).double(),
         "p.g": torch.randn(H, Wd, generator=g).double(),
         "p.o": torch.eye(H * Dv, dtype=F64)}
    h = torch.randn(T, Wd, generator=g).double()
    # spikes enter through two extra input channels per pair
    ex = torch.zeros(T, 2 * len(spikes), dtype=F64)
    for n, (i, j) in enumerate(spikes):
        ex[i, 2 * n] = 1.0
        ex[j, 2 * n + 1] = 1.0
    qcol = torch.zeros(H * D, 2 * len(spikes), dtype=F64)
    kcol = torch.zeros(G * D, 2 * len(spikes), dtype=F64)
    for n in range(len(spikes)):
        qcol[D - 1::D, 2 * n] = gain                   # last channel of every head
        kcol[D - 1::D, 2 * n + 1] = gain
    h = torch.cat([h, ex], 1)
    W["p.q"] = torch.cat([W["p.q"], qcol], 1)
    W["p.k"] = torch.cat([W["p.k"], kcol], 1)
    for n in ("p.v", "p.g"):
        W[n] = torch.cat([W[n], torch.zeros(W[n].shape[0], 2 * len(spikes), dtype=F64)], 1)
    q = h @ W["p.q"].T + W["p.q.b"]
    k = h @ W["p.k"].T + W["p.k.b"]
    v = h @ W["p.v"].T + W["p.v.b"]
    gt = h @ W["p.g"].T
    if dtype != F32:      # both sides see the values the kernel is given
        q, k, v, gt = (t.to(dtype).double() for t in (q, k, v, gt))
        Wq = {"p.q": torch.eye(H * D, dtype=F64), "p.k": torch.eye(G * D, dtype=F64),
              "p.v": torch.eye(G * Dv, dtype=F64), "p.g": torch.eye(H, dtype=F64)}
        Wo = {**W, **Wq}
        for n in ("p.q.b", "p.k.b", "p.v.b"):
            del Wo[n]
        want = _attention_from_projections(q, k, v, gt, Wo, L)
    else:
        want = oracle.window_sink_attention(h, W, "p.", L, EPS)
    att = RotaryWindowSinkAttention(H, G, D, Dv, L["scale"], EPS, window=L["mask"]["size"],
                                    rot=L.get("rot"))
    att.q_norm.data, att.k_norm.data = W["p.q.norm"].float(), W["p.k.norm"].float()
    att = att.to(device)
    nblk = (T + page - 1) // page
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=nblk + 3, block_size=page, dtype=dtype,
                              tp_degree=1, layer_kv_shapes=[(G, D, Dv)]).to(device)
    for t in list(mgr.k_caches) + list(mgr.v_caches):
        t.data.normal_()                                 # stale pages
    perm = torch.randperm(nblk + 3)[:nblk]               # scattered pages
    bt = perm.view(1, nblk).to(device)
    got, at = [], 0
    for n in cuts or [T]:
        pos = torch.arange(at, at + n).view(1, n).to(device)
        mgr.set_step_context(bt, generate_slot_mapping(bt, pos, page))
        st = seqmix.StepLayout(pos, torch.zeros(1, dtype=torch.long, device=device))
        sl = slice(at, at + n)
        fused = torch.cat([q[sl], k[sl], v[sl], gt[sl]], 1).view(1, n, -1).to(device, dtype)
        a, b, c, d = torch.split(fused, [H * D, G * D, G * Dv, H], dim=-1)
        got.append(att(a, b, c, mgr, 0, st, gate=d)[0].float().cpu())
        at += n
    got = torch.cat(got)
    if dtype == F32:
        close(got, want, tol)
    else:
        assert (got.double() - want).std().item() < tol * want.std().item()


def _attention_from_projections(q, k, v, gt, Wo, L):
    """The oracle on given projections: they are fed as the layer input of
    identity weights."""
    H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
    T = q.shape[0]
    out = torch.zeros(T, H * Dv, dtype=F64)
    # run the oracle once per projection set by stacking them as the input
    hq = torch.cat([q, k, v, gt], 1)
    n0, n1, n2 = H * D, H * D + G * D, H * D + G * D + G * Dv
    eye = torch.eye(hq.shape[1], dtype=F64)
    Wp = {**Wo, "p.q": eye[:n0], "p.k": eye[n0:n1], "p.v": eye[n1:n2], "p.g": eye[n2:]}
    out = oracle.window_sink_attention(hq, Wp, "p.", L, EPS)
    return out


@pytest.mark.parametrize("device", DEVICES)
def test_attention_window_edges_in_a_prompt(device):
    """Keys just inside (distance size-1) and just outside (distance size) the
    window, at page borders, and the first tokens, where the sink weighs most."""
    L = left_cfg(4, 2, 8, 6, size=6, dims=4)
    _attention_alone(device, L, 30, spikes=[(9, 4), (10, 4), (13, 8), (14, 8), (21, 16),
                                            (23, 17), (1, 0), (2, 2)])


@pytest.mark.parametrize("device", DEVICES)
def test_attention_window_edges_decoded_and_portions(device):
    L = left_cfg(4, 2, 8, 6, size=6, dims=4)
    spikes = [(9, 4), (10, 4), (13, 8), (14, 8), (21, 16), (23, 17), (1, 0)]
    _attention_alone(device, L, 30, spikes, cuts=[1] * 30)
    _attention_alone(device, L, 30, spikes, cuts=[2, 7, 2, 1, 2, 9, 1, 1, 5])
    _attention_alone(device, L, 30, spikes, cuts=[8] + [1] * 22)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [
    left_cfg(3, 1, 6, 5, size=9, scale=0.6, base=9.0),                 # one KV head, all rotated
    left_cfg(3, 3, 10, 4, size=1, scale=0.3, dims=6),                  # heads == KV heads, window 1
    left_cfg(2, 1, 20, 70, size=40, scale=0.2, dims=8, scaling=YARN),  # wide values
])
def test_attention_other_shapes(device, L):
    _attention_alone(device, L, 23, cuts=[5, 2, 1, 9, 1, 1, 4])
    _attention_alone(device, L, 23)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [None, [300] + [1] * 40])
def test_attention_far_key_among_hundreds(device, cuts):
    """A wide window: one far key dominates a query 330 tokens later, and the
    same key one step beyond the window does not."""
    L = left_cfg(2, 1, 8, 4, size=331, scale=0.4, base=1e4, dims=4)
    _attention_alone(device, L, 340, spikes=[(333, 3), (339, 8)], page=16, cuts=cuts, tol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("L,cuts", [
    (left_cfg(8, 2, 64, 64, size=40, scale=0.12, base=1e4), [70, 2, 1, 1, 26]),
    (left_cfg(4, 4, 32, 48, size=17, scale=0.2, dims=16, scaling=YARN), [100]),
    (left_cfg(6, 1, 128, 128, size=64, scale=0.09, base=5e5), [33, 67]),
])
def test_attention_bf16_matrix_path_gpu(L, cuts):
    _attention_alone("cuda", L, 100, spikes=[(50, 50 - L["mask"]["size"] + 1),
                                             (60, 60 - L["mask"]["size"])],
                     page=16, cuts=cuts, dtype=BF16, tol=0.03, gain=12.0)


# ------------------------------------------------------- recurrent mixers alone
def _ssd_alone(device, R, T, cuts, seed=0, tol=3e-5):
    g = torch.Generator().manual_seed(seed)
    Wd = 10
    Hh, P, N, G = R["heads"], R["vdim"], R["state"], R["groups"]
    inner, ch = Hh * P, Hh * P + 2 * G * N
    W = {"p.in": torch.randn(2 * inner + 2 * G * N + Hh, Wd, generator=g).double() * 0.5,
         "p.conv": torch.randn(ch, R["conv"], generator=g).double() * 0.6,
         "p.conv.b": torch.randn(ch, generator=g).double() * 0.3,
         "p.dt_bias": torch.randn(Hh, generator=g).double(),
         "p.A_log": (torch.rand(Hh, generator=g).double() * 1.5 - 1.0),
         "p.D": torch.randn(Hh, generator=g).double(),
         "p.norm": (1 + 0.1 * torch.randn(inner, generator=g)).double(),
         "p.o": torch.eye(inner, dtype=F64)}
    h = torch.randn(T, Wd, generator=g).double()
    want = oracle.ssd_mixer(h, W, "p.", R, EPS)
    mod = StateSpaceDuality(Hh, P, N, G, R["conv"], R["norm_groups"], EPS)
    mod.conv.weight.data, mod.conv.bias.data = W["p.conv"].float(), W["p.conv.b"].float()
    mod.dt_bias.data, mod.A_log.data = W["p.dt_bias"].float(), W["p.A_log"].float()
    mod.D.data, mod.norm_weight.data = W["p.D"].float(), W["p.norm"].float()
    mod = mod.to(device)
    states = RecurrentStateManager(3)
    for name, shape in mod.state_shapes().items():
        states.register("k." + name, shape)
    states = states.to(device)
    for t in states.tensors.values():
        t.data.normal_()                                  # a reused slot: stale contents
    y = (h @ W["p.in"].T).float()
    got, at = [], 0
    for n in cuts:
        pos = torch.arange(at, at + n).view(1, n)
        st = step_for(pos, [2], device)
        z, xbc, dt = torch.split(y[at:at + n].view(1, n, -1).to(device), mod.splits, dim=-1)
        got.append(mod(z, xbc, dt, states, "k", st)[0].float().cpu())
        at += n
    close(torch.cat(got), want, tol, rtol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R", [right_cfg(), right_cfg(3, 5, 5, 1, 2, 3), right_cfg(6, 4, 3, 3, 4, 1),
                               right_cfg(2, 20, 1, 2, 3, 5), right_cfg(2, 3, 40, 1, 4, 2)])
def test_state_space_portions(device, R):
    _ssd_alone(device, R, 37, [37])
    _ssd_alone(device, R, 37, [1] * 37)
    _ssd_alone(device, R, 37, [2, 5, 2, 1, 17, 2, 2, 6])
    _ssd_alone(device, R, 37, [2] * 18 + [1])


@pytest.mark.parametrize("device", DEVICES)
def test_state_space_long_decode(device):
    _ssd_alone(device, right_cfg(), 120, [3] + [1] * 117)


def _retention_alone(device, R, T, cuts, seed=1, tol=3e-5, dtype=F32):
    g = torch.Generator().manual_seed(seed)
    Wd = 10
    H, D, Dv = R["heads"], R["dim"], R["vdim"]
    W = {"p.q": torch.randn(H * D, Wd, generator=g).double() * 0.5,
         "p.k": torch.randn(H * D, Wd, generator=g).double() * 0.5,
         "p.v": torch.randn(H * Dv, Wd, generator=g).double() * 0.5,
         "p.g": torch.randn(H * Dv, Wd, generator=g).double() * 0.5,
         "p.o": torch.eye(H * Dv, dtype=F64)}
    h = torch.randn(T, Wd, generator=g).double()
    want = oracle.retention_mixer(h, W, "p.", R, EPS)
    mod = Retention(H, D, Dv, R["decay"], EPS).to(device)
    states = RecurrentStateManager(2)
    states.register("k.mem", mod.state_shapes()["mem"])
    states = states.to(device)
    states.get("k.mem").normal_()
    y = torch.cat([h @ W[n].T for n in ("p.q", "p.k", "p.v", "p.g")], 1).float()
    got, at = [], 0
    for n in cuts:
        pos = torch.arange(at, at + n).view(1, n)
        st = step_for(pos, [1], device)
        q, k, v, gt = torch.split(y[at:at + n].view(1, n, -1).to(device),
                                  [H * D, H * D, H * Dv, H * Dv], dim=-1)
        got.append(mod(q, k, v, gt, states, "k", st)[0].float().cpu())
        at += n
    close(torch.cat(got), want, tol, rtol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R", [ret_cfg(), ret_cfg(3, 5, 7, (0.8, 0.95, 1.0)),
                               ret_cfg(1, 12, 9, (0.97,)), ret_cfg(2, 1, 3, (0.5, 0.25)),
                               ret_cfg(1, 70, 18, (0.99,)), ret_cfg(1, 130, 5, (0.9,))])
def test_retention_portions(device, R):
    _retention_alone(device, R, 33, [33])
    _retention_alone(device, R, 33, [1] * 33)
    _retention_alone(device, R, 33, [2, 5, 2, 1, 13, 2, 2, 6])
    _retention_alone(device, R, 33, [2] * 16 + [1])


@pytest.mark.parametrize("device", DEVICES)
def test_retention_remembers_far_tokens(device):
    """A decay close to one keeps the first tokens' writes alive for hundreds
    of steps; a lost state would show at once."""
    _retention_alone(device, ret_cfg(2, 8, 4, (0.9995, 0.5)), 300, [280] + [1] * 20, tol=1e-4)


# ------------------------------------------------------------- feed-forward alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("fc", [moe_cfg(), moe_cfg(6, 3, 1, 1, 0.7, 10, 0),
                                moe_cfg(9, 1, 3, 1, 2.0, 8, 14), moe_cfg(10, 4, 5, 3, 1.0, 16, 8)])
def test_expert_feed_forward(device, fc):
    g = torch.Generator().manual_seed(9)
    Wd, T = 16, 29
    W = moe_weights(fc, Wd, "p.", g)
    h = torch.randn(2, T, Wd, generator=g)
    want = oracle.moe_feed_forward(h.view(-1, Wd).double(), W, "p.", fc).view(2, T, Wd)
    rc = fc["router"]
    E = rc["experts"]
    shared = bool(fc.get("shared"))
    mod = GroupRoutedFeedForward(Wd, E, rc["top"], fc["expert"]["ff"], F32,
                                 n_groups=rc["groups"]["count"], keep_groups=rc["groups"]["keep"],
                                 scale=rc["scale"], shared_ff=fc["shared"]["ff"] if shared else 0)
    mod.router.weight.data = torch.cat([W["p.router"]] + ([W["p.shared.sg"]] if shared else []), 0)
    mod.experts.up.weight.data = torch.cat(
        [W[f"p.e{e}.up"] for e in range(E)] + ([W["p.shared.up"]] if shared else []), 0)
    mod.experts.down.weight.data = torch.cat(
        [W[f"p.e{e}.down"] for e in range(E)] + ([W["p.shared.down"]] if shared else []), 1)
    mod = mod.to(device)
    close(mod(h.to(device)).cpu(), want, 5e-5, rtol=1e-4)


# ------------------------------------------------------------ whole model
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make", [model_cfg, varied_cfg])
def test_prefill_decode_portions_match_oracle(device, make):
    cfg = make()
    W = make_weights(cfg, seed=5)
    toks = tokens_for(cfg, 41, seed=6)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, device)
    close(feed(eng, toks, [41]), want, 3e-4)
    close(feed(eng, toks, [1] * 41), want, 3e-4)          # token by token from the start
    close(feed(eng, toks, [2, 5, 2, 1, 9, 3, 2, 16, 1]), want, 3e-4)
    close(feed(eng, toks, [2] * 20 + [1]), want, 3e-4)
    close(feed(eng, toks, [11] + [1] * 30), want, 3e-4)   # decoding far past every window


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make", [model_cfg, varied_cfg,
                                  lambda: model_cfg(loop=None),
                                  lambda: model_cfg(loop={"start": 3, "stop": 4, "times": 1})])
def test_residual_stream_per_layer_run(device, make):
    """The stream after every layer run; a looped layer counts each time."""
    cfg = make()
    W = make_weights(cfg, seed=7)
    toks = tokens_for(cfg, 9, seed=8)
    _, streams = oracle.forward(cfg, W, toks, return_layers=True)
    eng = make_engine(cfg, W, device)
    dm = eng.model.model
    seen = []
    hooks = [l.register_forward_hook(lambda m, a, out: seen.append(out.detach().clone().cpu()))
             for l in dm.layers]
    feed(eng, toks, [9])
    for hk in hooks:
        hk.remove()
    assert len(seen) == streams.shape[0] == len(oracle.run_order(cfg))
    for r, s in enumerate(seen):
        close(s[0], streams[r], 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reuse(device):
    """Unequal requests side by side (portions beside single tokens, one
    request pausing) equal each request alone; slots and pages are handed
    back and used again with stale contents."""
    cfg = varied_cfg()
    W = make_weights(cfg, seed=9)
    seqs = {n: tokens_for(cfg, L, seed=10 + i)
            for i, (n, L) in enumerate([("a", 30), ("b", 7), ("c", 19), ("d", 26), ("e", 12)])}
    want = {n: oracle.forward(cfg, W, t) for n, t in seqs.items()}
    eng = make_engine(cfg, W, device, slots=3, page=4, pages=18, max_len=32)
    for t in eng.kv_mgr.state.tensors.values():
        t.data.normal_()
    for t in list(eng.kv_mgr.k_caches) + list(eng.kv_mgr.v_caches):
        t.data.normal_()
    plan = [                                   # (name, count) per step
        [("a", 6), ("b", 1), ("c", 2)],
        [("a", 1), ("b", 3), ("c", 9)],
        [("a", 11), ("c", 1)],                 # b pauses
        [("a", 1), ("b", 3), ("c", 7)],        # b, c end
        [("a", 1), ("d", 13), ("e", 2)],       # d, e take the freed slots/pages
        [("a", 10), ("d", 1), ("e", 1)],       # a ends
        [("d", 12), ("e", 9)],
    ]
    live, at, got = {}, {n: 0 for n in seqs}, {n: [] for n in seqs}
    for step in plan:
        parts = []
        for n, c in step:
            if n not in live:
                live[n] = eng.admit()
            parts.append((live[n], torch.tensor(seqs[n][at[n]:at[n] + c])))
        lg = eng.forced_step(parts)
        for i, (n, c) in enumerate(step):
            got[n].append(lg[i, :c].float().cpu())
            at[n] += c
            if at[n] == len(seqs[n]):
                eng.release(live.pop(n))
    assert not live and eng.allocator.available() == 18 and len(eng.free_slots) == 3
    for n in seqs:
        close(torch.cat(got[n]), want[n], 3e-4)


def _oracle_greedy(cfg, W, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(oracle.forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(chunk_size=4), dict(chunk_size=4, mixed_chunking=True)])
def test_greedy_generation_through_scheduler(device, kw):
    """Queue -> slots -> (chunked / mixed) prefill -> batched decode; more
    requests than slots, so slots and pages are recycled."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=11)
    prompts = [tokens_for(cfg, n, seed=20 + n) for n in (9, 5, 14, 6)]
    want = [_oracle_greedy(cfg, W, p, 7) for p in prompts]
    eng = make_engine(cfg, W, device, slots=2, page=4, pages=14, max_len=28, **kw)
    rids = [eng.add_request(torch.tensor(p), max_new_tokens=7) for p in prompts]
    out = eng.run()
    assert [out[r] for r in rids] == want


@pytest.mark.gpu
def test_greedy_generation_captured_decode_gpu():
    """The engine's default GPU configuration: hipGraph-captured decode."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=11)
    prompts = [tokens_for(cfg, n, seed=20 + n) for n in (9, 5, 14, 6)]
    want = [_oracle_greedy(cfg, W, p, 7) for p in prompts]
    eng = make_engine(cfg, W, "cuda", slots=2, page=4, pages=14, max_len=28,
                      capture_decode=True, async_depth=2)
    rids = [eng.add_request(torch.tensor(p), max_new_tokens=7) for p in prompts]
    out = eng.run()
    assert [out[r] for r in rids] == want


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_generate_adapter(device):
    """The plain generate() entry point (no page table passed: the model
    lays its slots out linearly over the page pool)."""
    from neuronx_distributed_inference_amd.utils.hf_adapter import (
        GenerationConfig,
        HuggingFaceGenerationAdapter,
    )

    cfg = model_cfg()
    W = make_weights(cfg, seed=15)
    prompts = [tokens_for(cfg, 8, seed=40), tokens_for(cfg, 8, seed=41)]
    want = [_oracle_greedy(cfg, W, p, 6) for p in prompts]
    eng = make_engine(cfg, W, device, slots=2, page=4, pages=16, max_len=32)
    out = HuggingFaceGenerationAdapter(eng.model).generate(
        torch.tensor(prompts, device=device),
        generation_config=GenerationConfig(max_new_tokens=6))
    assert out[:, 8:].tolist() == want


def bigger_cfg():
    return model_cfg(layers=[
        layer("parallel", {"left": left_cfg(4, 2, 32, 48, size=24, scale=0.15, base=1e4,
                                            dims=16, scaling=YARN),
                           "right": right_cfg(4, 24, 16, 2, 4, 2)},
              mlp=moe_cfg(8, 3, 4, 2, 2.0, 64, 32)),
        layer("retention", ret_cfg(2, 32, 48, (0.95, 0.999)), mlp=moe_cfg(8, 3, 4, 2, 2.0, 64, 32)),
        layer("parallel", {"left": left_cfg(4, 2, 32, 48, size=24, scale=0.15, base=1e4),
                           "right": right_cfg(4, 24, 16, 2, 4, 2)},
              mlp=moe_cfg(8, 3, 4, 2, 2.0, 64, 0)),
    ], width=128, vocab=96, loop={"start": 1, "stop": 3, "times": 2})


@pytest.mark.gpu
def test_bfloat16_serving_precision_gpu():
    """bf16 projections, fp32 stream/scores/state/router: close to the oracle
    and independent of how the prompt is cut, beyond rounding."""
    cfg = bigger_cfg()
    W = make_weights(cfg, seed=12)
    toks = tokens_for(cfg, 80, seed=13)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, "cuda", dtype="bfloat16", page=16, pages=12, max_len=96)
    a = feed(eng, toks, [80])
    b = feed(eng, toks, [7, 30, 2, 1, 1, 39])
    scale = want.std().item()
    assert (a.double() - want).std().item() < 0.08 * scale
    assert (b.double() - want).std().item() < 0.08 * scale
    assert (a - b).double().std().item() < 0.08 * scale


@pytest.mark.gpu
def test_bfloat16_odd_sizes_gpu():
    """Sizes that leave every column slice of the fused projections
    misaligned: the kernels' scalar paths in bf16."""
    cfg = varied_cfg()
    W = make_weights(cfg, seed=12)
    toks = tokens_for(cfg, 41, seed=13)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, "cuda", dtype="bfloat16")
    a = feed(eng, toks, [41])
    b = feed(eng, toks, [2, 5, 2, 1, 9, 3, 2, 16, 1])
    scale = want.std().item()

    def close_rows(x, y):
        """Share of tokens whose logits agree. (This configuration routes
        every token to ONE expert of nine: where two scores nearly tie, bf16
        rounding picks the other one and that token's logits change
        altogether, with the torch reference ops as well.)"""
        return ((x.double() - y.double()).std(-1) < 0.1 * scale).float().mean().item()

    assert close_rows(a, want) >= 0.85 and close_rows(b, want) >= 0.85
    assert close_rows(a, b) >= 0.85


@pytest.mark.gpu
def test_float32_on_the_kernels_at_larger_sizes_gpu():
    cfg = bigger_cfg()
    W = make_weights(cfg, seed=12)
    toks = tokens_for(cfg, 80, seed=13)
    want = oracle.forward(cfg, W, toks)
    torch.backends.cuda.matmul.allow_tf32 = False
    eng = make_engine(cfg, W, "cuda", page=16, pages=12, max_len=96)
    close(feed(eng, toks, [80]), want, 1e-3)
    close(feed(eng, toks, [7, 30, 2, 1, 1, 39]), want, 1e-3)


def test_checkpoint_folder_and_schedule_replay(tmp_path):
    """config.json + model.safetensors on disk -> registry lookup by the
    config's architecture -> schedule replay writes the wanted logits. Sizes
    the file leaves out come from the tensors' shapes."""
    from safetensors.torch import save_file

    from neuronx_distributed_inference_amd import trace_replay
    from neuronx_distributed_inference_amd.registry import model_type_from_config

    cfg = varied_cfg()
    W = make_weights(cfg, seed=14)
    disk = copy.deepcopy(cfg)
    del disk["vocab"], disk["width"], disk["max_positions"]
    for lc in disk["layers"]:
        if lc["mlp"]:
            del lc["mlp"]["expert"]["ff"]
        if lc["type"] == "parallel":
            del lc["mixer"]["right"]["conv"], lc["mixer"]["left"]["vdim"]
        else:
            del lc["mixer"]["dim"], lc["mixer"]["vdim"]
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(disk))
    save_file({k: v.bfloat16() for k, v in W.items()}, str(mdir / "model.safetensors"))
    assert model_type_from_config(str(mdir)) == "kuterax"
    a, b = tokens_for(cfg, 21, 30), tokens_for(cfg, 9, 31)
    lines = [
        {"step": 0, "entries": [{"id": "x", "tokens": a[:8], "want": [0, 7]}], "end": []},
        {"step": 1, "entries": [{"id": "x", "tokens": a[8:20], "want": []},
                                {"id": "y", "tokens": b[:1], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "y", "tokens": b[1:], "want": [7]},
                                {"id": "x", "tokens": a[20:], "want": [0]}], "end": ["x", "y"]},
    ]
    out = tmp_path / "out"
    out.mkdir()
    eng = trace_replay.build_engine(str(mdir), "float32", 128, device=torch.device("cpu"))
    said = []
    trace_replay.replay(eng, [json.dumps(x) for x in lines], str(out), said.append)
    assert said == ["done 0", "done 1", "done 2"]
    wa, wb = oracle.forward(cfg, W, a), oracle.forward(cfg, W, b)
    import numpy as np

    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    g1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1))
    close(g0, wa[[0, 7]], 3e-4)
    close(g1, wb[[0]], 3e-4)
    close(g2, torch.stack([wb[8], wa[20]]), 3e-4)


def test_command_line_generation(tmp_path, capsys):
    """inference_demo --model-type kuterax: checkpoint folder -> compile ->
    load -> greedy generation, the same path as every other family."""
    from safetensors.torch import save_file

    from neuronx_distributed_inference_amd.inference_demo import main

    cfg = model_cfg()
    W = make_weights(cfg, seed=3)
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16() for k, v in W.items()}, str(mdir / "model.safetensors"))
    prompt = tokens_for(cfg, 9, seed=1)
    rc = main(["--model-type", "kuterax", "run", "--model-path", str(mdir),
               "--compiled-model-path", str(tmp_path / "compiled"),
               "--prompt-ids", json.dumps([prompt]), "--max-new-tokens", "6",
               "--torch-dtype", "float32", "--on-cpu", "--seq-len", "32",
               "--max-context-length", "16"])
    assert rc == 0
    printed = [json.loads(l) for l in capsys.readouterr().out.splitlines() if l.startswith("[[")]
    assert printed and printed[-1][0] == prompt + _oracle_greedy(cfg, W, prompt, 6)


def test_config_rejects_what_it_does_not_know():
    cfg = model_cfg()
    bad = copy.deepcopy(cfg)
    bad["layers"][1]["type"] = "window"
    with pytest.raises(ValueError):
        KuteraxInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)
    bad = copy.deepcopy(cfg)
    bad["layers"][0]["mlp"]["kind"] = "dense"
    with pytest.raises(ValueError):
        KuteraxInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)
    bad = copy.deepcopy(cfg)
    bad["layers"][1]["mixer"]["decay"] = [0.5]          # two heads, one decay
    with pytest.raises(ValueError):
        KuteraxInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)
    bad = copy.deepcopy(cfg)
    bad["loop"] = {"start": 2, "stop": 9, "times": 2}
    with pytest.raises(ValueError):
        KuteraxInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)


@pytest.mark.parametrize("device", DEVICES)
def test_state_space_long_prompt_then_decode(device):
    """Long portions take the segmented scan on the GPU (segments side by
    side, joined through their end states)."""
    _ssd_alone(device, right_cfg(2, 20, 12, 1, 4, 2), 340, [300, 2, 37, 1], tol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_decay_scan_unequal_long_rows(device):
    """Rows of unequal length in one step, one continuing from a carried
    state, one starting, one pad row: against the reference op on the CPU."""
    from neuronx_distributed_inference_amd.ops import ref

    torch.manual_seed(21)
    B, S, H, G, D, Dv = 3, 330, 4, 2, 24, 20
    q, k = torch.randn(B, S, G * D) * 0.3, torch.randn(B, S, G * D) * 0.3
    v = torch.randn(B, S, H * Dv)
    dt = torch.randn(B, S, H)
    dt_bias, a_log, skip = torch.randn(H), torch.rand(H) - 1.0, torch.randn(H)
    pos = torch.full((B, S), -1, dtype=torch.long)
    pos[0, :330] = torch.arange(5, 335)          # continues
    pos[1, :77] = torch.arange(0, 77)            # starts, short
    state0 = torch.randn(4, H, Dv, D)
    st_ref = state0.clone()
    want = ref.decay_scan(q, k, v, st_ref, pos, torch.tensor([2, 0, -1]), D, Dv, dt=dt,
                          dt_bias=dt_bias, a_log=a_log, skip=skip)
    st_dev = state0.clone().to(device)
    step = step_for(pos, [2, 0, -1], device)
    got = seqmix.decay_scan(q.to(device), k.to(device), v.to(device), st_dev, step, D, Dv,
                            dt=dt.to(device), dt_bias=dt_bias.to(device),
                            a_log=a_log.to(device), skip=skip.to(device)).cpu()
    close(got[0], want[0], 1e-4, rtol=1e-4)
    close(got[1, :77], want[1, :77], 1e-4, rtol=1e-4)
    close(st_dev.cpu()[[0, 2]], st_ref[[0, 2]], 1e-4, rtol=1e-4)
    assert torch.equal(st_dev.cpu()[[1, 3]], state0[[1, 3]])      # untouched slots


@pytest.mark.parametrize("device", DEVICES)
def test_embed_positions_op(device):
    torch.manual_seed(22)
    emb = torch.randn(2, 4, 10)
    table = torch.randn(7, 10)
    pos = torch.tensor([[3, 4, 5, 6], [0, 1, -1, -1]])
    got = seqmix.embed_positions(emb.to(device), table.to(device), step_for(pos, [0, 1], device))
    want = emb.double() + table.double()[pos.clamp(min=0)]
    close(got.cpu(), want, 1e-6)
