"""Tamilix (sandwich-norm decoder mixing chunk-local slope attention and
windowed gated latent attention, dense and identity-routed expert
feed-forwards, layers that share weights) against the plain float64 oracle in
``tamilix_oracle.py``.

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
import tamilix_oracle as oracle  # noqa: E402

from neuronx_distributed_inference_amd.config import EngineConfig  # noqa: E402
from neuronx_distributed_inference_amd.models.tamilix.modeling_tamilix import (  # noqa: E402
    TamilixForCausalLM,
    TamilixInferenceConfig,
)
from neuronx_distributed_inference_amd.modules.attention.chunked_attention import (  # noqa: E402
    ChunkedSlopeAttention,
    geometric_slopes,
)
from neuronx_distributed_inference_amd.modules.attention.latent_attention import (  # noqa: E402
    LatentSinkAttention,
)
from neuronx_distributed_inference_amd.modules.kvcache.block_kv_cache_manager import (  # noqa: E402
    BlockKVCacheManager,
    generate_slot_mapping,
)
from neuronx_distributed_inference_amd.modules.mlp import SquaredReluMLP  # noqa: E402
from neuronx_distributed_inference_amd.modules.moe import (  # noqa: E402
    FusedGatedExperts,
    IdentityRoutedFeedForward,
)
from neuronx_distributed_inference_amd.ops import seqmix  # noqa: E402
from neuronx_distributed_inference_amd.serving import ServingEngine  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32 = torch.float32
BF16 = torch.bfloat16
EPS = 1e-5


# ---------------------------------------------------------------- builders
def attn_cfg(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.4, chunk=7):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "mask": {"size": chunk}}


def latent_cfg(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=10, q_rank=12, scale=0.3, base=50.0,
               dims=None, window=5):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
            "q_rank": q_rank, "scale": scale, "rot": {"base": base, "dims": dims or rot_dim},
            "mask": {"size": window}}


def dense(ff=24):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, identity=2, top=3, ff=8, limit=0.8, shared_ff=12, shared_limit=0.5):
    fc = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
          "router": {"experts": experts, "identity": identity, "top": top}}
    if shared_ff:
        fc["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return fc


def layer(kind, mixer, mlp, weights_of=None):
    lc = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        lc["weights_of"] = weights_of
    return lc


def model_cfg(layers=None, width=16, vocab=37, scale=3.0):
    layers = layers or [
        layer("attention", attn_cfg(), dense()),
        layer("latent_attention", latent_cfg(), moe()),
        layer("attention", attn_cfg(), moe()),
        layer("latent_attention", latent_cfg(), moe(), weights_of=1),
    ]
    return {"architecture": "Tamilix", "width": width, "vocab": vocab,
            "embedding": {"scale": scale}, "norm": {"eps": EPS}, "layers": layers}


def varied_cfg():
    """Other sizes and another order: a latent layer first, one KV head and
    heads == KV heads, sizes that are no powers of two, a layer without
    feed-forward, a chunk of one position and one longer than any prompt here,
    a window of one, rotation on a part of the rotated channels, no identity
    experts / no shared expert / one chosen expert / one expert, a layer that
    shares an EARLIER and one that shares a LATER layer's weights."""
    la = latent_cfg(2, 6, 8, 10, 12, q_rank=9, scale=0.5, base=9.0, dims=4, window=9)
    at = attn_cfg(3, 1, 6, 5, scale=0.7, chunk=11)
    return model_cfg(layers=[
        layer("latent_attention", la, moe(3, 0, 1, ff=6, limit=2.0, shared_ff=0)),
        layer("attention", dict(at), None, weights_of=4),
        layer("attention", attn_cfg(3, 3, 5, 7, scale=0.2, chunk=1), dense(20)),
        layer("latent_attention", copy.deepcopy(la), moe(3, 0, 1, ff=6, limit=2.0, shared_ff=0),
              weights_of=0),
        layer("attention", at, None),
        layer("latent_attention", latent_cfg(4, 4, 2, 3, 5, q_rank=7, scale=0.9, window=1),
              moe(1, 3, 2, ff=10, limit=0.3, shared_ff=4, shared_limit=3.0)),
        layer("attention", attn_cfg(2, 2, 12, 4, scale=0.3, chunk=500), moe(6, 1, 6, ff=4)),
    ], width=24, vocab=29, scale=0.7)


def make_weights(cfg, seed=0):
    """Checkpoint-named tensors, values exactly representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    Wd = cfg["width"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def lin(o, i, gain=1.0):
        return rnd(o, i, std=gain / i ** 0.5)

    def nw(n):
        return (1 + rnd(n, std=0.3)).bfloat16().float()

    W["embed"] = rnd(cfg["vocab"], Wd)
    W["head"] = lin(cfg["vocab"], Wd)
    W["final.norm"] = nw(Wd)
    for i, lc in enumerate(cfg["layers"]):
        if lc.get("weights_of") is not None:
            continue
        p = "l%d." % i
        m = p + "mix."
        mc = lc["mixer"]
        W[p + "norm1"] = nw(Wd)
        W[p + "norm1b"] = nw(Wd)
        if lc["type"] == "attention":
            H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
            W[m + "q"] = lin(H * D, Wd, 2.0)
            W[m + "k"] = lin(G * D, Wd, 2.0)
            W[m + "v"] = lin(G * Dv, Wd)
            W[m + "sink"] = rnd(H, std=1.5)
            W[m + "o"] = lin(Wd, H * Dv)
        else:
            H, D, R, Dv, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
            Q = mc["q_rank"]
            W[m + "dq"] = lin(Q, Wd, 2.0)
            W[m + "dq.norm"] = nw(Q)
            W[m + "uq"] = lin(H * (D + R), Q, 2.0)
            W[m + "dkv"] = lin(C + R, Wd, 2.0)
            W[m + "dkv.norm"] = nw(C)
            W[m + "uk"] = lin(H * D, C, 2.0)
            W[m + "uv"] = lin(H * Dv, C)
            W[m + "g"] = lin(H * Dv, Wd, 2.0)
            W[m + "o"] = lin(Wd, H * Dv)
        fc = lc["mlp"]
        if not fc:
            continue
        W[p + "norm2"] = nw(Wd)
        W[p + "norm2b"] = nw(Wd)
        f = p + "mlp."
        if fc["kind"] == "dense":
            W[f + "up"] = lin(fc["ff"], Wd, 2.0)
            W[f + "down"] = lin(Wd, fc["ff"])
            continue
        E, I = fc["router"]["experts"], fc["router"]["identity"]
        for e in range(E):
            W[f + f"e{e}.gate"] = lin(fc["expert"]["ff"], Wd, 2.0)
            W[f + f"e{e}.up"] = lin(fc["expert"]["ff"], Wd, 2.0)
            W[f + f"e{e}.down"] = lin(Wd, fc["expert"]["ff"])
        W[f + "router"] = lin(E + I, Wd, 3.0)
        W[f + "correction"] = rnd(E + I, std=0.15)
        if fc.get("shared"):
            W[f + "shared.gate"] = lin(fc["shared"]["ff"], Wd, 2.0)
            W[f + "shared.up"] = lin(fc["shared"]["ff"], Wd, 2.0)
            W[f + "shared.down"] = lin(Wd, fc["shared"]["ff"])
    return W


def make_engine(cfg, W, device="cpu", dtype="float32", slots=3, page=4, pages=40,
                max_len=96, **engine_kw):
    ec = EngineConfig(batch_size=slots, max_batch_size=slots, kv_cache_batch_size=slots,
                      seq_len=max_len, max_length=max_len, torch_dtype=dtype, tp_degree=1,
                      is_block_kv_layout=True, pa_block_size=page, pa_num_blocks=pages,
                      enable_hip_graphs=False)
    config = TamilixInferenceConfig(neuron_config=ec, **copy.deepcopy(cfg))
    model = TamilixForCausalLM(config)
    sd = TamilixForCausalLM.convert_hf_to_native_state_dict(W, config)
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


# ------------------------------------------------------------ ops alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [20, 32, 264])            # scalar / 16-byte kernels / a long row
def test_post_norm_step_with_pass_through_and_next_pre_norm(device, n):
    """stream += norm(y + sum(coef) * extra) * w, and the next sublayer's
    pre-norm of the new stream from the same call."""
    torch.manual_seed(0)
    stream, y, extra = torch.randn(2, 5, n), torch.randn(2, 5, n) * 4, torch.randn(2, 5, n) * 2
    w, w2 = torch.randn(n) * 0.3 + 1, torch.randn(n) * 0.3 + 1
    dense_w = torch.rand(10, 6)                          # the last two columns are the coefficients
    coef = dense_w[:, 4:]
    v = y.double() + coef.double().sum(-1).view(2, 5, 1) * extra.double()
    new = stream.double() + oracle.norm(v, w.double(), EPS)
    s = stream.clone().to(device)
    out = seqmix.add_rms_norm(s, y.to(device), w.to(device), EPS, False, F32,
                              extra=extra.to(device), coef=coef.to(device),
                              next_weight=w2.to(device))
    close(s.cpu(), new, 2e-5)
    close(out.cpu(), oracle.norm(new, w2.double(), EPS), 2e-5)
    assert out.data_ptr() != s.data_ptr()
    # without the extras it is the plain step, the copy the stream itself
    s = stream.clone().to(device)
    cp = seqmix.add_rms_norm(s, y.to(device), w.to(device), EPS, False, F32)
    close(s.cpu(), stream.double() + oracle.norm(y.double(), w.double(), EPS), 2e-5)
    assert cp.data_ptr() == s.data_ptr()
    # a pre-norm only, no pass-through term; and no output at all
    s = stream.clone().to(device)
    out = seqmix.add_rms_norm(s, y.to(device), w.to(device), EPS, False, F32,
                              next_weight=w2.to(device))
    close(out.cpu(), oracle.norm(s.cpu().double(), w2.double(), EPS), 2e-5)
    assert seqmix.add_rms_norm(s, y.to(device), w.to(device), EPS, False, None) is None


@pytest.mark.gpu
def test_post_norm_step_bf16_gpu():
    torch.manual_seed(1)
    stream, w, w2 = torch.randn(7, 96), torch.randn(96) * 0.2 + 1, torch.randn(96) * 0.2 + 1
    y, extra = (torch.randn(7, 96) * 2).bfloat16(), torch.randn(7, 96).bfloat16()
    coef = torch.rand(7, 3)
    v = y.double() + coef.double().sum(-1, keepdim=True) * extra.double()
    new = stream.double() + oracle.norm(v, w.double(), EPS)
    s = stream.clone().cuda()
    out = seqmix.add_rms_norm(s, y.cuda(), w.cuda(), EPS, False, BF16, extra=extra.cuda(),
                              coef=coef.cuda(), next_weight=w2.cuda())
    close(s.cpu(), new, 2e-5)
    assert out.dtype == BF16
    close(out.float().cpu(), oracle.norm(new, w2.double(), EPS), 0.03, rtol=0.01)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top", [(7, 3), (1, 1), (13, 13), (130, 5)])
def test_router_correction_moves_the_choice_not_the_weights(device, E, top):
    torch.manual_seed(2)
    T = 33
    logits = torch.randn(T, E) * 2
    corr = torch.randn(E) * 0.3
    s = torch.softmax(logits.double(), -1)
    want_idx = torch.topk(s + corr.double(), top, dim=-1).indices
    plain_idx = torch.topk(s, top, dim=-1).indices
    dense_w, idx, wts = seqmix.group_limited_router(logits.to(device), E, top,
                                                    correction=corr.to(device))
    assert torch.equal(idx.long().cpu().sort(-1).values, want_idx.sort(-1).values)
    if 1 < top < E:
        assert not torch.equal(want_idx.sort(-1).values, plain_idx.sort(-1).values)
    close(wts.cpu(), torch.gather(s, 1, idx.long().cpu()), 1e-6)
    want_dense = torch.zeros(T, E, dtype=torch.float64).scatter(1, want_idx, s.gather(1, want_idx))
    close(dense_w.cpu(), want_dense, 1e-6)
    # without a correction the op is the plain top-k it was
    _, idx0, _ = seqmix.group_limited_router(logits.to(device), E, top)
    assert torch.equal(idx0.long().cpu().sort(-1).values, plain_idx.sort(-1).values)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,ff,sff", [(3, 5, 7), (4, 8, 16), (2, 16, 0), (0, 8, 24)])
def test_stacked_clamped_experts_activation(device, E, ff, sff):
    torch.manual_seed(3)
    T, C = 9, E * ff + sff
    hid = torch.randn(T, 2 * C) * 2
    gates = torch.rand(T, E + 2) * (torch.rand(T, E + 2) > 0.4)     # zeros = unchosen
    lim, slim = 0.7, 1.9

    def glu(g, u, limit):
        g, u = g.clamp(max=limit), u.clamp(-limit, limit)
        return g * torch.sigmoid(1.702 * g) * (u + 1)

    g, u = hid[:, :C].double(), hid[:, C:].double()
    want = torch.empty(T, C, dtype=torch.float64)
    for e in range(E):
        sl = slice(e * ff, (e + 1) * ff)
        want[:, sl] = glu(g[:, sl], u[:, sl], lim) * gates[:, e:e + 1].double()
    want[:, E * ff:] = glu(g[:, E * ff:], u[:, E * ff:], slim)
    got = seqmix.clamped_glu_scale(hid.to(device), gates.to(device), ff, E, lim, slim)
    close(got.cpu(), want, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("C", [12, 40])
def test_plain_relu_squared_and_sigmoid_gate(device, C):
    torch.manual_seed(4)
    x = torch.randn(6, C) * 2
    close(seqmix.relu2_scale(x.to(device), None, C, 1).cpu(), torch.relu(x.double()) ** 2, 1e-5)
    wide = torch.randn(2, 3, C + 16)
    y = torch.randn(2, 3, C)
    gate = wide[..., 8:8 + C]                            # a column slice, read in place
    got = seqmix.sigmoid_gate_(y.clone().to(device), wide.to(device)[..., 8:8 + C])
    close(got.cpu(), y.double() * torch.sigmoid(gate.double()), 1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,W,E,extra", [(5, 24, 7, 0), (64, 64, 18, 0), (9, 136, 5, 2),
                                         (600, 32, 9, 1)])
def test_router_product_and_selection_in_one_call(device, T, W, E, extra):
    """Few tokens: product and selection in one launch; many: the library
    product first. Both equal the selection on float64 logits."""
    torch.manual_seed(7)
    wide = torch.randn(T, W + 8)
    x = wide[:, 8:]                                      # a column slice, read in place
    w = torch.randn(E + extra, W) * 0.5
    corr = torch.randn(E) * 0.2
    s = torch.softmax(x.double() @ w[:E].double().T, -1)
    want_idx = torch.topk(s + corr.double(), 3 if E > 3 else 1, dim=-1).indices
    top = want_idx.shape[1]
    dense_w, idx, wts = seqmix.route_tokens(wide.to(device)[:, 8:], w.to(device), E, top,
                                            correction=corr.to(device))
    assert torch.equal(idx.long().cpu().sort(-1).values, want_idx.sort(-1).values)
    close(wts.cpu(), torch.gather(s, 1, idx.long().cpu()), 2e-6)
    assert dense_w.shape == (T, E + extra)
    if extra:
        close(dense_w[:, E:].cpu(), torch.sigmoid(x.double() @ w[E:].double().T), 2e-6)


@pytest.mark.gpu
def test_router_one_launch_bf16_input_gpu():
    torch.manual_seed(8)
    x = torch.randn(33, 256).bfloat16()
    w = torch.randn(14, 256) * 0.2
    s = torch.softmax(x.double() @ w.double().T, -1)
    want_idx = torch.topk(s, 4, dim=-1).indices
    _, idx, wts = seqmix.route_tokens(x.cuda(), w.cuda(), 14, 4)
    assert torch.equal(idx.long().cpu().sort(-1).values, want_idx.sort(-1).values)
    close(wts.cpu(), torch.gather(s, 1, idx.long().cpu()), 2e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("C,R,dims", [(10, 4, 4), (12, 8, 4), (64, 32, 32), (5, 2, 2)])
def test_latent_cache_row_in_one_call(device, C, R, dims):
    """Norm, rotation and the scatter into page slots; pad tokens and stale
    pages stay as they are."""
    from neuronx_distributed_inference_amd.modules.rope import interleaved_inv_freq

    torch.manual_seed(9)
    B, S, page, nblk = 2, 5, 4, 6
    wide = torch.randn(B, S, C + R + 3) * 2
    x = wide[..., 3:]
    w = 1 + 0.3 * torch.randn(C)
    pos = torch.tensor([[900, 901, 902, 903, 904], [0, 1, 2, -1, -1]])
    slots = torch.tensor([[17, 18, 19, 4, 5], [9, 10, 11, -1, -1]])
    cache = torch.randn(nblk, page, 1, C + R)
    before = cache.clone()
    st = seqmix.StepLayout(pos.to(device), torch.tensor([0, 1]).to(device))
    inv = interleaved_inv_freq(100.0, dims)
    cd = cache.clone().to(device)
    row = torch.zeros(B, S, C + R, device=device)
    seqmix.latent_row_write(wide.to(device)[..., 3:], w.to(device), EPS, inv.to(device), st, cd,
                            slots.view(-1).to(device), C, row=row)
    flat = cd.cpu().view(-1, C + R)
    for b in range(B):
        for t in range(S):
            if pos[b, t] < 0:
                continue
            want = torch.cat([
                oracle.norm(x[b, t, :C].double(), w.double(), EPS),
                oracle.rotate_pairs(x[b, t, C:].double().view(1, 1, R), pos[b, t:t + 1], 100.0,
                                    dims).view(R)])
            close(flat[slots[b, t]], want, 3e-4)          # fp32 angles near position 900
            close(row[b, t].cpu(), want, 3e-4)
    untouched = torch.ones(nblk * page, dtype=torch.bool)
    untouched[slots[slots >= 0]] = False
    assert torch.equal(flat[untouched], before.view(-1, C + R)[untouched])
    cd2 = cache.clone().to(device)                       # without the dense copy
    seqmix.latent_row_write(wide.to(device)[..., 3:], w.to(device), EPS, inv.to(device), st, cd2,
                            slots.view(-1).to(device), C)
    assert torch.equal(cd2.cpu(), cd.cpu())


def test_slope_ladder():
    for H in (1, 3, 8, 20):
        close(geometric_slopes(H), oracle.head_slopes(H), 1e-7)
    assert abs(float(geometric_slopes(8)[-1]) - 2.0 ** -8) < 1e-9


# ------------------------------------------------------------ chunked attention
def _chunked_alone(device, L, T, spikes=(), page=4, cuts=None, dtype=F32, tol=2e-5, gain=6.0,
                   sink=None):
    """Attention core on its own paged cache. `spikes`: (query i, key j) pairs
    whose score is made to stand out, so a lost or misplaced key shows."""
    torch.manual_seed(3)
    Wd = 12
    H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
    h = torch.randn(T, Wd).double()
    q = h @ (torch.randn(H * D, Wd).double() * 0.3).T
    k = h @ (torch.randn(G * D, Wd).double() * 0.3).T
    v = h @ torch.randn(G * Dv, Wd).double().T
    for i, j in spikes:
        d = torch.zeros(G * D, dtype=torch.float64)
        d[(i + j) % D::D] = 1.0                   # the same channel in every head
        k[j] += gain * d
        q[i] += gain * d.view(G, D)[:1].repeat(H, 1).reshape(-1)
    if dtype != F32:      # both sides see the values the kernel is given
        q, k, v = (t.to(dtype).double() for t in (q, k, v))
    hq = torch.cat([q, k, v], 1)
    o0, o1 = H * D, H * D + G * D
    eye = torch.eye(hq.shape[1], dtype=torch.float64)
    sk = torch.randn(H).double() if sink is None else torch.full((H,), sink).double()
    Wo = {"p.q": eye[:o0], "p.k": eye[o0:o1], "p.v": eye[o1:], "p.sink": sk,
          "p.o": torch.eye(H * Dv, dtype=torch.float64)}
    want = oracle.attention_mixer(hq, Wo, "p.", L)

    att = ChunkedSlopeAttention(H, G, D, Dv, L["scale"], L["mask"]["size"])
    att.sink.data = sk.float()
    att = att.to(device)
    nblk = (T + page - 1) // page
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=nblk + 3, block_size=page, dtype=dtype,
                              tp_degree=1, layer_kv_shapes=[(G, D, Dv)]).to(device)
    mgr.k_caches[0].data.normal_()                      # stale pages
    mgr.v_caches[0].data.normal_()
    perm = torch.randperm(nblk + 3)[:nblk]              # scattered pages
    bt = perm.view(1, nblk).to(device)
    got, at = [], 0
    for n in cuts or [T]:
        pos = torch.arange(at, at + n).view(1, n).to(device)
        mgr.set_step_context(bt, generate_slot_mapping(bt, pos, page))
        st = seqmix.StepLayout(pos, torch.zeros(1, dtype=torch.long, device=device))
        sl = slice(at, at + n)
        y = att(q[sl].view(1, n, -1).to(device, dtype), k[sl].view(1, n, -1).to(device, dtype),
                v[sl].view(1, n, -1).to(device, dtype), mgr, 0, st)
        got.append(y[0].float().cpu())
        at += n
    got = torch.cat(got)
    if dtype == F32:
        close(got, want, tol)
    else:
        assert (got.double() - want).std().item() < tol * want.std().item()
    return got


# chunk 7: blocks start at 0, 7, 14, 21, 28. (20, 14) is the first key of the
# query's block, (20, 13) the last key of the block before (invisible: the
# oracle's answer does not move, the engine's must not either), (27, 21) a
# whole block back, (21, 21) and (28, 28) queries that open a block and see
# only themselves and the sink, (6, 0) the very first token, pages of 4 tokens
# put page borders inside every block
_EDGES = [(20, 14), (20, 13), (27, 21), (26, 20), (21, 21), (28, 28), (6, 0), (13, 7), (14, 7)]


@pytest.mark.parametrize("device", DEVICES)
def test_chunked_attention_prompt(device):
    _chunked_alone(device, attn_cfg(), 31, _EDGES)


@pytest.mark.parametrize("device", DEVICES)
def test_chunked_attention_decoded_and_portions(device):
    L = attn_cfg()
    _chunked_alone(device, L, 31, _EDGES, cuts=[5] + [1] * 26)
    _chunked_alone(device, L, 31, _EDGES, cuts=[1] * 31)
    _chunked_alone(device, L, 31, _EDGES, cuts=[2, 5, 2, 1, 9, 3, 2, 6, 1])     # cuts inside blocks
    _chunked_alone(device, L, 31, _EDGES, cuts=[13, 2, 2, 2, 2, 10], page=8)
    _chunked_alone(device, L, 31, _EDGES, cuts=[14, 7, 7, 3])                   # cuts at block starts


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [attn_cfg(3, 1, 6, 5, chunk=11), attn_cfg(3, 3, 5, 7, chunk=1),
                               attn_cfg(2, 2, 12, 4, chunk=500), attn_cfg(20, 4, 4, 70, chunk=6),
                               attn_cfg(1, 1, 16, 16, chunk=64)])
def test_chunked_attention_other_shapes(device, L):
    _chunked_alone(device, L, 30, [(23, 22), (23, 12), (29, 24)])
    _chunked_alone(device, L, 30, [(23, 22), (23, 12), (29, 24)], cuts=[3, 9, 1, 1, 1, 14, 1])


@pytest.mark.parametrize("device", DEVICES)
def test_chunked_attention_sink_counts_once(device):
    """A dominant sink empties the output, an absent one (-> -inf) leaves a
    plain softmax; a query that opens a block shares its weight with it."""
    L = attn_cfg()
    big = _chunked_alone(device, L, 9, sink=30.0)
    none = _chunked_alone(device, L, 9, sink=-80.0)
    assert big.abs().max() < 1e-6 < none.abs().max()
    _chunked_alone(device, L, 1, sink=0.5)
    _chunked_alone(device, L, 16, cuts=[1] * 16, sink=2.0)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [None, [300] + [1] * 40, [130, 130, 60, 20]])
def test_chunked_attention_far_key_among_hundreds(device, cuts):
    """Blocks of 128: keys a hundred positions back inside the block (where
    the distance penalty is largest), the block's first key, the last key of
    the block before, in a prompt and decoded."""
    L = attn_cfg(4, 2, 8, 8, scale=0.4, chunk=128)
    _chunked_alone(device, L, 340, [(339, 256), (339, 255), (330, 257), (320, 200), (255, 128),
                                    (255, 127), (300, 256), (127, 0), (128, 128)],
                   page=16, cuts=cuts, tol=1e-4, gain=9.0)


@pytest.mark.gpu
@pytest.mark.parametrize("L,cuts", [
    (attn_cfg(8, 4, 64, 64, scale=0.125, chunk=50), None),
    (attn_cfg(8, 4, 64, 64, scale=0.125, chunk=50), [3, 60, 1, 66]),
    (attn_cfg(6, 2, 24, 40, scale=0.2, chunk=64), [100, 29, 1]),          # padded tiles
    (attn_cfg(4, 4, 128, 128, scale=0.09, chunk=33), [64, 66]),
    (attn_cfg(16, 1, 32, 32, scale=0.18, chunk=128), [70, 50] + [1] * 10),
])
def test_chunked_attention_bf16_matrix_path_gpu(L, cuts):
    c = L["mask"]["size"]
    spikes = [(129, (129 // c) * c), (129, (129 // c) * c - 1), (2 * c - 1, c), (c, c - 1)]
    spikes = [(i, j) for i, j in spikes if i < 130]
    _chunked_alone("cuda", L, 130, spikes, cuts=cuts, page=16, dtype=BF16, tol=0.03, gain=3.0)
    _chunked_alone("cuda", L, 130, spikes, cuts=[100] + [1] * 30, page=16, dtype=BF16, tol=0.03,
                   gain=3.0)


@pytest.mark.gpu
@pytest.mark.parametrize("L", [attn_cfg(8, 4, 64, 64, scale=0.125, chunk=256),
                               attn_cfg(16, 4, 128, 128, scale=0.09, chunk=150)])
def test_chunked_attention_bf16_fully_visible_tiles_gpu(L):
    """Blocks much longer than a key tile: most tiles are visible to every
    query row of a workgroup and take the unmasked path, which still has to
    apply the distance penalty."""
    c = L["mask"]["size"]
    spikes = [(329, c), (329, c - 1), (c + 60, c + 3), (c - 1, 0), (min(2 * c - 1, 300), c)]
    _chunked_alone("cuda", L, 330, spikes, page=16, dtype=BF16, tol=0.03, gain=3.0)
    _chunked_alone("cuda", L, 330, spikes, cuts=[200, 100, 29, 1], page=16, dtype=BF16, tol=0.03,
                   gain=3.0)


# ------------------------------------------------------------ latent attention
def _latent_alone(device, L, T, cuts=None, page=4, dtype=F32, tol=3e-5, spikes=(), fresh=False,
                  gated=True):
    torch.manual_seed(5)
    Wd = 14
    H, D, R, Dv, C = L["heads"], L["dim"], L["rot_dim"], L["vdim"], L["kv_rank"]
    Q = L["q_rank"]
    h = torch.randn(T, Wd).double()
    W = {"p.dq": torch.randn(Q, Wd).double() * 0.4, "p.dq.norm": (1 + 0.3 * torch.randn(Q)).double(),
         "p.uq": (torch.randn(H * (D + R), Q) * 0.5).bfloat16().double(),
         "p.dkv": torch.randn(C + R, Wd).double() * 0.6,
         "p.dkv.norm": (1 + 0.3 * torch.randn(C)).double(),
         "p.uk": torch.randn(H * D, C).double().bfloat16().double() * 0.5,
         "p.uv": torch.randn(H * Dv, C).double().bfloat16().double() * 0.5,
         "p.g": torch.randn(H * Dv, Wd).double() * (1.0 if gated else 0.0),
         "p.o": torch.eye(H * Dv, dtype=torch.float64)}
    # the module is handed what its caller's projections produce
    q = oracle.norm(h @ W["p.dq"].T, W["p.dq.norm"], EPS) @ W["p.uq"].T
    dkv = h @ W["p.dkv"].T
    gate = h @ W["p.g"].T
    for i, j in spikes:                       # through the shared rotated part
        dkv[j, C:] *= 5.0
        q.view(T, H, D + R)[i, :, D:] *= 5.0
    if dtype != F32:
        q, dkv, gate = q.to(dtype).double(), dkv.to(dtype).double(), gate.to(dtype).double()
    # the oracle's attention from the same (spiked, rounded) projections
    want = oracle.latent_attend(q.clone(), dkv, W, "p.", L, EPS)
    if gated:
        want = want * torch.sigmoid(gate)

    att = LatentSinkAttention(H, D, R, Dv, C, L["scale"], EPS, L["rot"]["base"],
                              L["rot"]["dims"], dtype, sink=False, window=L["mask"]["size"])
    att.latent_norm.weight.data = W["p.dkv.norm"].float()
    att.uk.data = W["p.uk"].view(H, D, C).to(dtype)
    att.uv.data = W["p.uv"].view(H, Dv, C).to(dtype)
    att = att.to(device)
    nblk = (T + page - 1) // page
    mgr = BlockKVCacheManager(1, 1, 1, num_blocks=nblk + 2, block_size=page, dtype=dtype,
                              tp_degree=1, layer_kv_shapes=[att.kv_shape()]).to(device)
    assert mgr.v_caches[0].numel() == 0                 # one row per token, no value pages
    mgr.k_caches[0].data.normal_()                      # stale pages
    perm = torch.randperm(nblk + 2)[:nblk]
    bt = perm.view(1, nblk).to(device)
    got, at = [], 0
    for n in cuts or [T]:
        pos = torch.arange(at, at + n).view(1, n).to(device)
        mgr.set_step_context(bt, generate_slot_mapping(bt, pos, page))
        st = seqmix.StepLayout(pos, torch.zeros(1, dtype=torch.long, device=device))
        st.fresh = fresh and at == 0          # whole-prompt form for the first portion
        sl = slice(at, at + n)
        y = att(q[sl].view(1, n, -1).to(device, dtype), dkv[sl].view(1, n, -1).to(device, dtype),
                mgr, 0, st, gate=gate[sl].view(1, n, -1).to(device, dtype) if gated else None)
        got.append(y[0].float().cpu())
        at += n
    got = torch.cat(got)
    if dtype == F32:
        close(got, want, tol)
    else:
        assert (got.double() - want).std().item() < tol * want.std().item()
    return got


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [latent_cfg(), latent_cfg(2, 6, 8, 10, 12, base=9.0, dims=4, window=9),
                               latent_cfg(5, 4, 2, 3, 5, window=1),
                               latent_cfg(1, 16, 16, 24, 40, window=100)])
def test_latent_attention_window_and_gate_in_portions(device, L):
    w = L["mask"]["size"]
    # the oldest key the window keeps and the first one it has dropped
    spikes = [(25, max(25 - w + 1, 0)), (25, max(25 - w, 0)), (12, max(12 - w + 1, 0)),
              (w - 1 if w <= 26 else 3, 0)]
    _latent_alone(device, L, 26, spikes=spikes)
    _latent_alone(device, L, 26, spikes=spikes, cuts=[1, 2, 7, 1, 1, 1, 13])
    _latent_alone(device, L, 26, spikes=spikes, cuts=[3] + [1] * 23, page=8)
    _latent_alone(device, L, 26, spikes=spikes, cuts=[2] * 13, gated=False)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("L", [latent_cfg(), latent_cfg(2, 6, 8, 10, 12, base=9.0, dims=4, window=9)])
def test_latent_attention_whole_prompt_form(device, L):
    """A prompt taken in the expanded form, then continued from the cache
    rows it left (absorbed form): both equal the oracle."""
    _latent_alone(device, L, 26, fresh=True)
    _latent_alone(device, L, 26, cuts=[17, 1, 1, 7], fresh=True)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [None, [250] + [1] * 30, [100, 100, 60, 20]])
def test_latent_attention_window_edge_far_into_a_sequence(device, cuts):
    L = latent_cfg(2, 8, 8, 6, 12, scale=0.4, base=10000.0, window=72)
    _latent_alone(device, L, 280, cuts=cuts, page=16, tol=1e-4,
                  spikes=[(279, 208), (279, 207), (270, 199), (270, 198), (260, 192), (100, 29),
                          (100, 28), (71, 0), (72, 0), (72, 1)])


@pytest.mark.gpu
@pytest.mark.parametrize("L,cuts", [
    (latent_cfg(4, 32, 16, 32, 64, scale=0.1, window=40), None),
    (latent_cfg(6, 24, 8, 40, 72, scale=0.1, window=64), [3, 60, 1, 66]),      # 80-wide rows
    (latent_cfg(2, 64, 32, 64, 96, scale=0.08, dims=16, window=33), [64, 66]),
    # wide rows: 32-key tiles, values split over workgroups, also when decoding
    (latent_cfg(8, 32, 32, 48, 224, scale=0.1, window=50), [70, 50] + [1] * 10),
    (latent_cfg(16, 64, 64, 64, 512, scale=0.07, window=90), [100] + [1] * 30),
    (latent_cfg(3, 12, 6, 10, 20, scale=0.2, window=17), [100, 29, 1]),        # vector kernel
])
def test_latent_attention_bf16_matrix_path_gpu(L, cuts):
    w = L["mask"]["size"]
    spikes = [(129, 129 - w + 1), (129, 129 - w), (110, 110 - w + 1), (110, 110 - w)]
    _latent_alone("cuda", L, 130, spikes=spikes, cuts=cuts, page=16, dtype=BF16, tol=0.03)
    _latent_alone("cuda", L, 130, spikes=spikes, cuts=[100] + [1] * 30, page=16, dtype=BF16,
                  tol=0.03, fresh=True)


@pytest.mark.gpu
@pytest.mark.parametrize("L", [latent_cfg(16, 64, 64, 64, 512, scale=0.07, window=300),
                               latent_cfg(20, 32, 32, 48, 224, scale=0.1, window=130),
                               latent_cfg(8, 32, 32, 32, 128, scale=0.1, window=1)])
def test_latent_attention_windowed_decode_key_splits_gpu(L):
    """Single-token steps over a latent cache: the window's keys are split
    over several workgroups whose partial softmaxes are merged; splits that
    fall outside a short window contribute nothing."""
    w = L["mask"]["size"]
    spikes = [(419, 419 - w + 1), (419, max(419 - w, 0)), (405, 405 - w + 1), (405, 405 - w)]
    _latent_alone("cuda", L, 420, spikes=spikes, cuts=[400] + [1] * 20, page=16, dtype=BF16,
                  tol=0.03)


# ------------------------------------------------------------ feed-forwards
def _ff_alone(device, fc, T=19, Wd=16, seed=6):
    cfg = model_cfg(layers=[layer("attention", attn_cfg(), fc)], width=Wd)
    W = make_weights(cfg, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    h = torch.randn(T, Wd, generator=g)
    if fc["kind"] == "dense":
        want = oracle.dense_ff(h.double(), W, "l0.mlp.")
        mod = SquaredReluMLP(Wd, fc["ff"], tp_degree=1, dtype=F32)
        mod.up_proj.weight.data, mod.down_proj.weight.data = W["l0.mlp.up"], W["l0.mlp.down"]
        close(mod.to(device)(h.to(device).view(1, T, Wd))[0].cpu(), want, 2e-5)
        return
    want = oracle.moe_ff(h.double(), W, "l0.mlp.", fc)
    rc, sc = fc["router"], fc.get("shared") or {}
    E = rc["experts"]
    mod = IdentityRoutedFeedForward(Wd, E, rc["identity"], rc["top"], fc["expert"]["ff"],
                                    fc["expert"]["limit"], F32, shared_ff=sc.get("ff", 0),
                                    shared_limit=sc.get("limit", 0.0))
    m = "l0.mlp."
    mod.router.weight.data, mod.router.correction.data = W[m + "router"], W[m + "correction"]
    mod.experts.gate_up.weight.data = FusedGatedExperts.stack_gate_up(
        [W[m + f"e{e}.gate"] for e in range(E)], [W[m + f"e{e}.up"] for e in range(E)],
        W.get(m + "shared.gate"), W.get(m + "shared.up"))
    mod.experts.down.weight.data = FusedGatedExperts.stack_down(
        [W[m + f"e{e}.down"] for e in range(E)], W.get(m + "shared.down"))
    y, coef = mod.to(device)(h.to(device).view(1, T, Wd))
    got = y[0].double().cpu()
    if rc["identity"]:
        idx, _ = oracle.route(h.double(), W, m, rc["top"])
        assert bool((idx >= E).any()) and bool((idx < E).any())      # both kinds are exercised
        assert coef.shape == (T, rc["identity"])
        got = got + coef.double().cpu().sum(-1, keepdim=True) * h.double()
    else:
        assert coef is None
    close(got, want, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("fc", [dense(24), dense(7), moe(), moe(3, 0, 1, ff=6, limit=2.0, shared_ff=0),
                                moe(1, 3, 2, ff=10, limit=0.3, shared_ff=4, shared_limit=3.0),
                                moe(6, 1, 7, ff=4), moe(8, 2, 2, ff=16, shared_ff=24)])
def test_feed_forwards_alone(device, fc):
    _ff_alone(device, fc)


def test_correction_decides_an_expert_in_the_model_configurations():
    """The test weights make the correction matter: for some token the
    corrected choice is not the plain top-k."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=6)
    h = torch.randn(64, cfg["width"]).double()
    s = torch.softmax(h @ W["l1.mlp.router"].double().T, -1)
    a = torch.topk(s, 3, dim=-1).indices.sort(-1).values
    b = torch.topk(s + W["l1.mlp.correction"].double(), 3, dim=-1).indices.sort(-1).values
    assert not torch.equal(a, b)


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
def test_long_decoding_across_many_blocks_and_windows(device):
    cfg = model_cfg()
    W = make_weights(cfg, seed=21)
    toks = tokens_for(cfg, 90, seed=22)
    eng = make_engine(cfg, W, device, pages=30, max_len=96)
    close(feed(eng, toks, [3] + [1] * 87), oracle.forward(cfg, W, toks), 3e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make", [model_cfg, varied_cfg])
def test_residual_stream_per_layer_run(device, make):
    """The stream after every layer run; a layer that shares weights counts
    as a run of its own."""
    cfg = make()
    W = make_weights(cfg, seed=7)
    toks = tokens_for(cfg, 9, seed=8)
    streams = []
    oracle.forward(cfg, W, toks, streams)
    eng = make_engine(cfg, W, device)
    dm = eng.model.model
    assert len(dm.layers) == len(set(dm.config.owners())) < len(cfg["layers"])
    seen = []
    hooks = [l.register_forward_hook(lambda m, a, out: seen.append(out.detach().clone().cpu()))
             for l in dm.layers]
    feed(eng, toks, [9])
    for hk in hooks:
        hk.remove()
    assert len(seen) == len(streams) == len(cfg["layers"])
    for r, s in enumerate(seen):
        close(s[0], streams[r], 1e-4)


def test_sharing_entries_may_chain_and_omit_what_equals_the_owner():
    cfg = model_cfg()
    W = make_weights(cfg, seed=18)
    toks = tokens_for(cfg, 14, seed=19)
    want = oracle.forward(cfg, W, toks)
    short = copy.deepcopy(cfg)
    short["layers"][3] = {"type": "latent_attention", "weights_of": 1}
    short["layers"].append({"weights_of": 3})            # through layer 3 to layer 1
    full = copy.deepcopy(cfg)
    full["layers"].append(copy.deepcopy(full["layers"][3]))
    eng = make_engine(short, W)
    assert eng.model.model._order_slots == [0, 1, 2, 1, 1]
    close(feed(eng, toks, [9, 5]), oracle.forward(full, W, toks), 3e-4)
    assert not torch.allclose(oracle.forward(full, W, toks), want)


def test_shared_weights_keep_their_own_cache():
    """A layer with weights_of has no parameters but pages of its own: the
    two runs of one module see different keys."""
    cfg = model_cfg()
    W = make_weights(cfg, seed=16)
    eng = make_engine(cfg, W)
    dm, mgr = eng.model.model, eng.kv_mgr
    assert len(dm.layers) == 3 and dm._order_slots == [0, 1, 2, 1]
    assert mgr.k_caches[1].data_ptr() != mgr.k_caches[3].data_ptr()
    assert mgr.k_caches[1].shape == mgr.k_caches[3].shape and mgr.v_caches[3].numel() == 0
    toks = tokens_for(cfg, 12, seed=17)
    close(feed(eng, toks, [5, 7]), oracle.forward(cfg, W, toks), 3e-4)
    assert not torch.equal(mgr.k_caches[1], mgr.k_caches[3])


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


@pytest.mark.gpu
def test_bfloat16_serving_precision_gpu():
    """bf16 projections, fp32 stream/scores/norms/router: close to the oracle
    and independent of how the prompt is cut, beyond rounding."""
    cfg = model_cfg(layers=[
        layer("latent_attention", latent_cfg(8, 32, 16, 48, 64, q_rank=96, scale=0.12, window=24),
              moe(6, 2, 3, ff=64, limit=2.0, shared_ff=64, shared_limit=1.5)),
        layer("attention", attn_cfg(4, 2, 32, 64, scale=0.15, chunk=30), dense(256)),
        layer("latent_attention", latent_cfg(8, 32, 16, 48, 64, q_rank=96, scale=0.12, window=24),
              moe(6, 2, 3, ff=64, limit=2.0, shared_ff=64, shared_limit=1.5), weights_of=0),
        layer("attention", attn_cfg(4, 4, 32, 32, scale=0.15, chunk=17), None),
    ], width=128, vocab=96, scale=8.0)
    W = make_weights(cfg, seed=12)
    toks = tokens_for(cfg, 80, seed=13)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, "cuda", dtype="bfloat16", page=16, pages=12, max_len=96)
    a = feed(eng, toks, [80])
    b = feed(eng, toks, [7, 30, 2, 1, 1, 39])
    scale = want.std().item()
    assert (a.double() - want).std().item() < 0.06 * scale
    assert (b.double() - want).std().item() < 0.06 * scale
    assert (a - b).double().std().item() < 0.06 * scale


@pytest.mark.gpu
def test_float32_kernels_at_larger_sizes_gpu():
    cfg = model_cfg(layers=[
        layer("attention", attn_cfg(8, 2, 64, 48, scale=0.12, chunk=40), moe(8, 2, 3, ff=32,
                                                                             shared_ff=48)),
        layer("latent_attention", latent_cfg(4, 48, 16, 40, 96, q_rank=112, scale=0.1, window=50,
                                             base=10000.0), dense(288)),
        layer("attention", attn_cfg(8, 2, 64, 48, scale=0.12, chunk=40),
              moe(8, 2, 3, ff=32, shared_ff=48), weights_of=0),
    ], width=160, vocab=101, scale=3.0)
    W = make_weights(cfg, seed=30)
    toks = tokens_for(cfg, 150, seed=31)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, "cuda", page=16, pages=24, max_len=160, slots=2)
    close(feed(eng, toks, [150]), want, 5e-4)
    close(feed(eng, toks, [100, 7, 2] + [1] * 41), want, 5e-4)


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
    del disk["vocab"], disk["width"]
    for lc in disk["layers"]:
        mc, fc = lc["mixer"], lc["mlp"]
        if lc["type"] == "attention":
            del mc["heads"], mc["dim"], mc["vdim"]
        else:
            del mc["q_rank"], mc["kv_rank"], mc["heads"], mc["vdim"]
        if fc and fc["kind"] == "dense":
            del fc["ff"]
        elif fc:
            del fc["expert"]["ff"], fc["router"]["identity"]
            if fc.get("shared"):
                del fc["shared"]["ff"]
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(disk))
    save_file({k: v.bfloat16() for k, v in W.items()}, str(mdir / "model.safetensors"))
    assert model_type_from_config(str(mdir)) == "tamilix"
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
    """inference_demo --model-type tamilix: checkpoint folder -> compile ->
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
    rc = main(["--model-type", "tamilix", "run", "--model-path", str(mdir),
               "--compiled-model-path", str(tmp_path / "compiled"),
               "--prompt-ids", json.dumps([prompt]), "--max-new-tokens", "6",
               "--torch-dtype", "float32", "--on-cpu", "--seq-len", "32",
               "--max-context-length", "16"])
    assert rc == 0
    printed = [json.loads(l) for l in capsys.readouterr().out.splitlines() if l.startswith("[[")]
    assert printed and printed[-1][0] == prompt + _oracle_greedy(cfg, W, prompt, 6)


def test_config_rejects_what_it_does_not_know():
    cfg = model_cfg()
    for change in (lambda c: c["layers"][1].update(type="window"),
                   lambda c: c["layers"][0]["mlp"].update(kind="experts"),
                   lambda c: c["layers"][3].update(weights_of=3),        # itself
                   lambda c: c["layers"][3].update(weights_of=9),        # no such layer
                   lambda c: c["layers"][3].update(weights_of=0),        # another kind of layer
                   lambda c: c["layers"][1]["mlp"]["router"].update(top=9)):
        bad = copy.deepcopy(cfg)
        change(bad)
        with pytest.raises(ValueError):
            TamilixInferenceConfig(neuron_config=EngineConfig(tp_degree=1), **bad)


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
