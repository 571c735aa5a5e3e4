"""Tamilix for MI355X: a decoder with sandwich norms whose layers each pick
one of two attention mixers and one of two feed-forwards.

Layer: ``x += norm1b(mixer(norm1(x)))`` then, when the layer has a
feed-forward, ``x += norm2b(ff(norm2(x)))``; all four are RMS norms with
plain weights. The stream is the embedding times a constant. A layer entry
with ``weights_of: j`` has no tensors: it runs layer j's modules against a
cache of its own. Mixers, chosen per layer by ``type``:

- ``attention``: :class:`ChunkedSlopeAttention` — GQA without rotation, keys
  visible only inside the query's block of ``mask.size`` positions, a linear
  distance penalty with a fixed ladder of slopes, a learned softmax sink;
- ``latent_attention``: :class:`LatentSinkAttention` (no sink, sliding
  window ``mask.size``) — queries through a normed low-rank latent, keys and
  values expanded per head from a normed low-rank latent, one rotated key
  part shared by all heads (interleaved rotary), the concatenated heads
  times ``sigmoid(W_g h)``.

Feed-forwards, chosen by ``mlp.kind``: ``dense`` — ``W_down relu(W_up h)^2``;
``moe`` — :class:`IdentityRoutedFeedForward`: clamped gated experts behind a
softmax router with a choice-only correction, experts that pass their input
through, and a shared expert. Output: the model's norm, then an untied head.

Engine integration (shared with the other hybrid decoders through
:class:`HybridDecoderModel`): fp32 residual stream, paged KV with per-run
page shapes (a latent layer keeps one row per token and no value pages), one
set of kernels for prompt portions, decoded tokens and mixed batches. Every
projection that reads a sublayer's input is one fused GEMM; a post-norm
residual step is one kernel that also emits the NEXT sublayer's pre-norm
(of this layer's feed-forward, or of the next layer's mixer) from the same
pass over the stream.
"""

from __future__ import annotations

import json
import os
from typing import Dict, List

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.config import InferenceConfig
from neuronx_distributed_inference_amd.models.hybrid_base import HybridDecoderModel
from neuronx_distributed_inference_amd.models.model_base import CausalLMBase
from neuronx_distributed_inference_amd.modules.attention.chunked_attention import (
    ChunkedSlopeAttention,
)
from neuronx_distributed_inference_amd.modules.attention.latent_attention import (
    LatentSinkAttention,
)
from neuronx_distributed_inference_amd.modules.mlp import SquaredReluMLP
from neuronx_distributed_inference_amd.modules.moe import (
    FusedGatedExperts,
    IdentityRoutedFeedForward,
)
from neuronx_distributed_inference_amd.modules.norm import StreamRMSNorm
from neuronx_distributed_inference_amd.parallel.layers import (
    ColumnParallelLinear,
    RowParallelLinear,
)

MIXER_TYPES = ("attention", "latent_attention")
FF_KINDS = ("dense", "moe")
GLU_ALPHA = 1.702          # fixed by the design; the clamp limits are per model
SLOPE_LOG2 = 8.0           # fixed by the design: slope_h = 2^(-8 (h + 1) / H)


class TamilixInferenceConfig(InferenceConfig):
    """Reads the checkpoint's ``config.json`` as is (keys: architecture,
    width, vocab, embedding.scale, layers[], norm.eps) and derives the
    generic attribute names the engine uses."""

    def get_required_attributes(self) -> List[str]:
        return ["width", "vocab", "layers", "norm"]

    def add_derived_config(self):
        if not hasattr(self, "layers"):
            return
        if not getattr(self, "embedding", None):
            self.embedding = {"scale": 1.0}       # a file without the entry scales nothing
        self.hidden_size = self.width
        self.vocab_size = self.vocab
        self.num_hidden_layers = len(self.layers)
        self.tie_word_embeddings = False
        for i, lc in enumerate(self.layers):
            if lc.get("weights_of") is not None:
                oc = self.layers[self._owner(i)]         # what the entry omits is the owner's
                for key in ("type", "mixer", "mlp"):
                    if key not in lc:
                        lc[key] = oc.get(key)
        for i, lc in enumerate(self.layers):
            if lc.get("type") not in MIXER_TYPES:
                raise ValueError(f"unknown Tamilix layer type {lc.get('type')!r}")
            fc = lc.get("mlp")
            if fc and fc.get("kind") not in FF_KINDS:
                raise ValueError(f"unknown Tamilix feed-forward kind {fc.get('kind')!r}")
            if lc.get("weights_of") is not None:
                j = self._owner(i)
                oc = self.layers[j]
                if oc["type"] != lc["type"] or oc["mixer"] != lc["mixer"] or \
                        oc.get("mlp") != lc.get("mlp"):
                    raise ValueError(f"layer {i}: its entry differs from layer {j}'s")
            if fc and fc["kind"] == "moe":
                rc = fc["router"]
                if not 1 <= rc["top"] <= rc["experts"] + rc.get("identity", 0):
                    raise ValueError(f"layer {i}: top exceeds the router's outputs")
        ec = self.neuron_config
        if ec.tp_degree != 1:
            raise ValueError("Tamilix runs with tp_degree=1")
        ec.is_block_kv_layout = True

    def _owner(self, i: int) -> int:
        """Index of the entry whose tensors entry i uses (an entry that names
        a sharing entry uses that one's owner)."""
        seen = {i}
        while self.layers[i].get("weights_of") is not None:
            j = self.layers[i]["weights_of"]
            if not (isinstance(j, int) and 0 <= j < len(self.layers)) or j in seen:
                raise ValueError(f"layer {i}: weights_of must name a layer with tensors")
            seen.add(j)
            i = j
        return i

    def owners(self) -> List[int]:
        """For every layer entry, the index of the entry whose tensors it uses."""
        return [self._owner(i) for i in range(len(self.layers))]

    @classmethod
    def from_hf_config(cls, model_path: str, neuron_config=None, **overrides):
        """Sizes that config.json leaves out are taken from the tensors'
        shapes in the checkpoint header, where a shape determines them."""
        with open(os.path.join(model_path, "config.json")) as f:
            hf = json.load(f)
        hf.update(overrides)
        ckpt = os.path.join(model_path, "model.safetensors")
        if os.path.exists(ckpt):
            from safetensors import safe_open

            with safe_open(ckpt, framework="pt") as st:
                names = set(st.keys())

                def shape(name):
                    return st.get_slice(name).get_shape() if name in names else None

                emb = shape("embed")
                if emb:
                    hf.setdefault("vocab", emb[0])
                    hf.setdefault("width", emb[1])
                for i, lc in enumerate(hf["layers"]):
                    src, seen = i, set()
                    while isinstance(hf["layers"][src].get("weights_of"), int) and \
                            src not in seen and 0 <= hf["layers"][src]["weights_of"] < len(hf["layers"]):
                        seen.add(src)
                        src = hf["layers"][src]["weights_of"]
                    if src != i:
                        for key in ("type", "mixer", "mlp"):
                            if key not in lc:
                                lc[key] = json.loads(json.dumps(hf["layers"][src].get(key)))
                    _fill_from_shapes(lc, lambda n, src=src: shape(f"l{src}.{n}"))
        return cls(neuron_config=neuron_config, **hf)


def _fill_from_shapes(lc: dict, shape):
    mc = lc.setdefault("mixer", {})
    if lc["type"] == "attention":
        if "heads" not in mc and shape("mix.sink"):
            mc["heads"] = shape("mix.sink")[0]
        if "dim" not in mc and "heads" in mc and shape("mix.q"):
            mc["dim"] = shape("mix.q")[0] // mc["heads"]
        if "heads" not in mc and "dim" in mc and shape("mix.q"):
            mc["heads"] = shape("mix.q")[0] // mc["dim"]
        if "kv_heads" not in mc and "dim" in mc and shape("mix.k"):
            mc["kv_heads"] = shape("mix.k")[0] // mc["dim"]
        if "vdim" not in mc and "kv_heads" in mc and shape("mix.v"):
            mc["vdim"] = shape("mix.v")[0] // mc["kv_heads"]
    elif lc["type"] == "latent_attention":
        if "q_rank" not in mc and shape("mix.dq"):
            mc["q_rank"] = shape("mix.dq")[0]
        if "kv_rank" not in mc and shape("mix.dkv.norm"):
            mc["kv_rank"] = shape("mix.dkv.norm")[0]
        if "rot_dim" not in mc and "kv_rank" in mc and shape("mix.dkv"):
            mc["rot_dim"] = shape("mix.dkv")[0] - mc["kv_rank"]
        uq, uk = shape("mix.uq"), shape("mix.uk")
        if "heads" not in mc and uq and uk:
            if "dim" in mc:
                mc["heads"] = uk[0] // mc["dim"]
            elif mc.get("rot_dim"):
                mc["heads"] = (uq[0] - uk[0]) // mc["rot_dim"]
        if "dim" not in mc and "heads" in mc and uk:
            mc["dim"] = uk[0] // mc["heads"]
        if "vdim" not in mc and "heads" in mc and shape("mix.uv"):
            mc["vdim"] = shape("mix.uv")[0] // mc["heads"]
        if isinstance(mc.get("rot"), dict) and "dims" not in mc["rot"] and "rot_dim" in mc:
            mc["rot"]["dims"] = mc["rot_dim"]
    fc = lc.get("mlp")
    if not isinstance(fc, dict):
        return
    if fc.get("kind") == "dense":
        if "ff" not in fc and shape("mlp.up"):
            fc["ff"] = shape("mlp.up")[0]
    elif fc.get("kind") == "moe":
        rc = fc.setdefault("router", {})
        if "experts" not in rc:
            n = 0
            while shape(f"mlp.e{n}.gate"):
                n += 1
            rc["experts"] = n
        if "identity" not in rc and shape("mlp.router"):
            rc["identity"] = shape("mlp.router")[0] - rc["experts"]
        xc = fc.setdefault("expert", {})
        if "ff" not in xc and shape("mlp.e0.gate"):
            xc["ff"] = shape("mlp.e0.gate")[0]
        sc = fc.get("shared")
        if isinstance(sc, dict) and "ff" not in sc and shape("mlp.shared.gate"):
            sc["ff"] = shape("mlp.shared.gate")[0]


# ----------------------------------------------------------------- mixers
class TamilixAttentionMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        self.core = ChunkedSlopeAttention(
            H, G, D, Dv, mc["scale"], chunk=(mc.get("mask") or {}).get("size", 0),
            slope_log2=SLOPE_LOG2, sink=True)
        self.splits = [H * D, G * D, G * Dv]
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.o_proj = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)

    def kv_shape(self):
        return self.core.kv_shape()

    def forward(self, h, kv_mgr, run_idx: int, step):
        q, k, v = torch.split(self.in_proj(h), self.splits, dim=-1)
        return self.o_proj(self.core(q, k, v, kv_mgr, run_idx, step))

    @staticmethod
    def convert(sd, s, d, w, f, out, mc):
        out[d + "in_proj.weight"] = torch.cat([w(s + "q"), w(s + "k"), w(s + "v")], dim=0)
        out[d + "core.sink"] = f(s + "sink")
        out[d + "o_proj.weight"] = w(s + "o")


class TamilixLatentMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        H, D, R, Dv, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
        Q = mc["q_rank"]
        rot = mc.get("rot") or {}
        self.core = LatentSinkAttention(
            H, D, R, Dv, C, mc["scale"], eps, rot.get("base", 10000.0), rot.get("dims", R),
            dtype, sink=False, window=(mc.get("mask") or {}).get("size"))
        # one GEMM for everything that reads the mixer's input: the query
        # latent, the key/value latent with the rotated key part, the gate
        self.splits = [Q, C + R, H * Dv]
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.q_norm = StreamRMSNorm(Q, eps=eps, one_plus=False, out_dtype=dtype)
        self.q_up = ColumnParallelLinear(Q, H * (D + R), dtype=dtype, tp_degree=1)
        self.o_proj = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)

    def kv_shape(self):
        return self.core.kv_shape()

    def forward(self, h, kv_mgr, run_idx: int, step):
        cq, dkv, gate = torch.split(self.in_proj(h), self.splits, dim=-1)
        q = self.q_up(self.q_norm(cq))
        return self.o_proj(self.core(q, dkv, kv_mgr, run_idx, step, gate=gate))

    @staticmethod
    def convert(sd, s, d, w, f, out, mc):
        out[d + "in_proj.weight"] = torch.cat([w(s + "dq"), w(s + "dkv"), w(s + "g")], dim=0)
        out[d + "q_norm.weight"] = f(s + "dq.norm")
        out[d + "q_up.weight"] = w(s + "uq")
        out[d + "core.latent_norm.weight"] = f(s + "dkv.norm")
        uk, uv = w(s + "uk"), w(s + "uv")
        H, C = mc["heads"], uk.shape[1]
        out[d + "core.uk"] = uk.view(H, -1, C).contiguous()                   # (H, dim, C)
        out[d + "core.uv"] = uv.view(H, -1, C).contiguous()                   # (H, vdim, C)
        out[d + "o_proj.weight"] = w(s + "o")


_MIXERS = {"attention": TamilixAttentionMixer, "latent_attention": TamilixLatentMixer}


class TamilixLayer(nn.Module):
    def __init__(self, config: TamilixInferenceConfig, layer_idx: int):
        super().__init__()
        ec = config.neuron_config
        lc = config.layers[layer_idx]
        eps = float(config.norm["eps"])
        W, dt = config.width, ec.torch_dtype
        self.dtype = dt
        self.norm1 = StreamRMSNorm(W, eps=eps, out_dtype=dt)
        self.mixer = _MIXERS[lc["type"]](W, lc["mixer"], eps, dt)
        self.norm1b = StreamRMSNorm(W, eps=eps)
        self.mlp = None
        self.routed = False
        fc = lc.get("mlp")
        if fc:
            self.norm2 = StreamRMSNorm(W, eps=eps, out_dtype=dt)
            self.norm2b = StreamRMSNorm(W, eps=eps)
            if fc["kind"] == "dense":
                self.mlp = SquaredReluMLP(W, fc["ff"], tp_degree=1, dtype=dt)
            else:
                rc, xc, sc = fc["router"], fc["expert"], fc.get("shared") or {}
                self.routed = True
                self.mlp = IdentityRoutedFeedForward(
                    W, rc["experts"], rc.get("identity", 0), rc["top"], xc["ff"], xc["limit"],
                    dt, shared_ff=sc.get("ff", 0), shared_limit=sc.get("limit", 0.0),
                    alpha=GLU_ALPHA, normalize=False, correction=True)

    def kv_shape(self):
        return self.mixer.kv_shape()

    def state_shapes(self) -> Dict[str, tuple]:
        return {}

    def forward(self, x, kv_mgr, run_idx: int):
        step = kv_mgr.step
        # this layer's pre-norm: left by the previous layer's last residual
        # kernel, or computed here for the first layer
        h, step.prenorm = step.prenorm, None
        if h is None:
            h = self.norm1(x)
        after = step.next_norm          # the next layer's norm1 weight (None: last layer)
        y = self.mixer(h, kv_mgr, run_idx, step)
        if self.mlp is None:
            step.prenorm = self.norm1b.add_into(
                x, y, self.dtype if after is not None else None, next_weight=after)
            return x
        h = self.norm1b.add_into(x, y, self.dtype, next_weight=self.norm2.weight)
        if self.routed:
            y, coef = self.mlp(h)
        else:
            y, coef = self.mlp(h), None
        step.prenorm = self.norm2b.add_into(
            x, y, self.dtype if after is not None else None,
            extra=h if coef is not None else None, coef=coef, next_weight=after)
        return x


class TamilixModel(HybridDecoderModel):
    def __init__(self, config):
        self.embed_scale = float(config.embedding["scale"])
        super().__init__(config)

    def build_layers(self, config) -> nn.ModuleList:
        # modules exist for the entries that own tensors; an entry with
        # weights_of runs its owner's module against a cache of its own
        owners = config.owners()
        own = sorted(set(owners))
        self._slot_of = {li: k for k, li in enumerate(own)}
        self._order_slots = [self._slot_of[o] for o in owners]
        return nn.ModuleList(TamilixLayer(config, li) for li in own)

    def run_order(self, config):
        return list(self._order_slots)

    def build_norm(self, config) -> nn.Module:
        return StreamRMSNorm(config.width, eps=config.norm["eps"],
                             out_dtype=config.neuron_config.torch_dtype)

    def begin_step(self, position_ids, seq_ids, block_table):
        block_table = super().begin_step(position_ids, seq_ids, block_table)
        self.kv_mgr.step.prenorm = None
        self.kv_mgr.step.next_norm = None
        return block_table

    def before_layer_run(self, run_idx, h, h_embed):
        h = super().before_layer_run(run_idx, h, h_embed)
        nxt = run_idx + 1
        self.kv_mgr.step.next_norm = self.layers[self._order_slots[nxt]].norm1.weight \
            if nxt < len(self._order_slots) else None
        return h

    def finalize_logits(self, logits):
        return logits.float()


class TamilixForCausalLM(CausalLMBase):
    _model_cls = TamilixModel
    _config_cls = TamilixInferenceConfig

    @staticmethod
    def convert_hf_to_native_state_dict(sd: Dict[str, torch.Tensor], config) -> Dict[str, torch.Tensor]:
        dt = config.neuron_config.torch_dtype
        out: Dict[str, torch.Tensor] = {}

        def w(name):                       # projection weights: engine dtype
            return sd[name].to(dt)

        def f(name):                       # 32-bit parameters
            return sd[name].float()

        out["embed_tokens.weight"] = w("embed")
        out["lm_head.weight"] = w("head")
        out["norm.weight"] = f("final.norm")
        own = sorted(set(config.owners()))
        for k, i in enumerate(own):
            lc = config.layers[i]
            s, d = f"l{i}.", f"layers.{k}."
            out[d + "norm1.weight"] = f(s + "norm1")
            out[d + "norm1b.weight"] = f(s + "norm1b")
            _MIXERS[lc["type"]].convert(sd, s + "mix.", d + "mixer.", w, f, out, lc["mixer"])
            fc = lc.get("mlp")
            if not fc:
                continue
            out[d + "norm2.weight"] = f(s + "norm2")
            out[d + "norm2b.weight"] = f(s + "norm2b")
            m = s + "mlp."
            if fc["kind"] == "dense":
                out[d + "mlp.up_proj.weight"] = w(m + "up")
                out[d + "mlp.down_proj.weight"] = w(m + "down")
                continue
            E = fc["router"]["experts"]
            shared = bool(fc.get("shared"))
            out[d + "mlp.router.weight"] = f(m + "router")
            out[d + "mlp.router.correction"] = f(m + "correction")
            out[d + "mlp.experts.gate_up.weight"] = FusedGatedExperts.stack_gate_up(
                [w(m + f"e{e}.gate") for e in range(E)], [w(m + f"e{e}.up") for e in range(E)],
                w(m + "shared.gate") if shared else None, w(m + "shared.up") if shared else None)
            out[d + "mlp.experts.down.weight"] = FusedGatedExperts.stack_down(
                [w(m + f"e{e}.down") for e in range(E)], w(m + "shared.down") if shared else None)
        return out
