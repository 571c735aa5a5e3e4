"""Kuterax for MI355X: a decoder whose layers run a token mixer and a
mixture-of-experts feed-forward side by side on ONE pre-norm.

Layer: ``h = norm1(x)`` (RMS norm, weight stored around zero), then
``x += ls1 * mixer(h) + ls2 * ff(h)`` with per-channel layer scales. The
stream starts as the token embedding plus a learned position row. Mixers,
chosen per layer by ``type``:

- ``parallel``: two branches on the same input, each RMS-normed over the
  width with its own weight, half their sum. Left:
  :class:`RotaryWindowSinkAttention` (GQA with biased projections, per-head
  q/k norm, partial half-split rotary with by-parts frequency scaling,
  sliding window, a zero-score sink in the softmax, one sigmoid gate per
  head). Right: :class:`StateSpaceDuality` (scalar-decay selective state
  space with a biased short convolution, gate before a grouped norm).
- ``retention``: :class:`Retention` (fixed per-head decay, no softmax).

Feed-forward: :class:`GroupRoutedFeedForward` — relu-squared experts behind
a group-limited softmax router, plus a sigmoid-gated shared expert. A span of
layers may be repeated with shared weights ("loop"); every run has its own
pages and state, and every pass (the first too) opens with ``x <- W_in [x;
x0] + step[t]``, ``x0`` the embedding output. Output: the same one-plus RMS
norm and an untied head.

Engine integration (shared with the other hybrid decoders through
:class:`HybridDecoderModel`): fp32 residual stream, paged KV for the attention
branch, convolution tails and recurrent matrices in the cache manager's
state slots, one set of kernels for prompt portions, decoded tokens and mixed
batches. Everything that reads ``h`` in a mixer is one fused GEMM; all
experts are two GEMMs; the branch norms, the layer scales and the residual
sum are one kernel.
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
from neuronx_distributed_inference_amd.modules.attention.window_sink_attention import (
    RotaryWindowSinkAttention,
)
from neuronx_distributed_inference_amd.modules.linear_recurrence import (
    Retention,
    StateSpaceDuality,
)
from neuronx_distributed_inference_amd.modules.moe import (
    FusedUngatedExperts,
    GroupRoutedFeedForward,
)
from neuronx_distributed_inference_amd.modules.norm import StreamRMSNorm
from neuronx_distributed_inference_amd.ops import seqmix
from neuronx_distributed_inference_amd.parallel.layers import (
    ColumnParallelLinear,
    RowParallelLinear,
)

MIXER_TYPES = ("parallel", "retention")
SINK_SCORE = 0.0           # fixed by the design: the sink adds exp(0) = 1


class KuteraxInferenceConfig(InferenceConfig):
    """Reads the checkpoint's ``config.json`` as is (keys: architecture,
    width, vocab, max_positions, layers[], loop, norm.eps) and derives the
    generic attribute names the engine uses."""

    def get_required_attributes(self) -> List[str]:
        return ["width", "vocab", "layers", "norm"]

    def add_derived_config(self):
        if not hasattr(self, "layers"):
            return
        self.hidden_size = self.width
        self.vocab_size = self.vocab
        self.num_hidden_layers = len(self.layers)
        self.tie_word_embeddings = False
        if not getattr(self, "loop", None):
            self.loop = None
        else:
            lp = self.loop
            if not (0 <= lp["start"] < lp["stop"] <= len(self.layers)) or lp["times"] < 1:
                raise ValueError(f"bad loop {lp!r}")
        for i, lc in enumerate(self.layers):
            if lc.get("type") not in MIXER_TYPES:
                raise ValueError(f"unknown Kuterax layer type {lc.get('type')!r}")
            fc = lc.get("mlp")
            if fc and fc.get("kind", "moe") != "moe":
                raise ValueError(f"unknown Kuterax feed-forward kind {fc.get('kind')!r}")
            if lc["type"] == "retention" and len(lc["mixer"]["decay"]) != lc["mixer"]["heads"]:
                raise ValueError(f"layer {i}: one decay per head is needed")
        ec = self.neuron_config
        if ec.tp_degree != 1:
            raise ValueError("Kuterax runs with tp_degree=1")
        ec.is_block_kv_layout = True

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
                if shape("pos"):
                    hf.setdefault("max_positions", shape("pos")[0])
                for i, lc in enumerate(hf["layers"]):
                    _fill_from_shapes(lc, lambda n, i=i: shape(f"l{i}.{n}"))
        return cls(neuron_config=neuron_config, **hf)

    def run_order(self) -> List[int]:
        """Layer index of every layer run, in execution order."""
        n = len(self.layers)
        lp = self.loop
        if not lp:
            return list(range(n))
        order = list(range(lp["start"]))
        for _ in range(lp["times"]):
            order += list(range(lp["start"], lp["stop"]))
        return order + list(range(lp["stop"], n))

    def pass_starts(self) -> Dict[int, int]:
        """Run index that opens a pass of the loop -> number of the pass."""
        lp = self.loop
        if not lp:
            return {}
        span = lp["stop"] - lp["start"]
        return {lp["start"] + t * span: t for t in range(lp["times"])}


def _fill_from_shapes(lc: dict, shape):
    mc = lc["mixer"]
    if lc["type"] == "parallel":
        rc = mc["right"]
        if "conv" not in rc and shape("mix.right.conv"):
            rc["conv"] = shape("mix.right.conv")[1]
        if "heads" not in rc and shape("mix.right.A_log"):
            rc["heads"] = shape("mix.right.A_log")[0]
        if "vdim" not in rc and "heads" in rc and shape("mix.right.norm"):
            rc["vdim"] = shape("mix.right.norm")[0] // rc["heads"]
        lc_ = mc["left"]
        if "dim" not in lc_ and shape("mix.left.q.norm"):
            lc_["dim"] = shape("mix.left.q.norm")[0]
        if "heads" not in lc_ and shape("mix.left.g"):
            lc_["heads"] = shape("mix.left.g")[0]
        if "kv_heads" not in lc_ and "dim" in lc_ and shape("mix.left.k"):
            lc_["kv_heads"] = shape("mix.left.k")[0] // lc_["dim"]
        if "vdim" not in lc_ and "kv_heads" in lc_ and shape("mix.left.v"):
            lc_["vdim"] = shape("mix.left.v")[0] // lc_["kv_heads"]
    elif lc["type"] == "retention":
        if "heads" not in mc and "decay" in mc:
            mc["heads"] = len(mc["decay"])
        if "dim" not in mc and "heads" in mc and shape("mix.q"):
            mc["dim"] = shape("mix.q")[0] // mc["heads"]
        if "vdim" not in mc and "heads" in mc and shape("mix.v"):
            mc["vdim"] = shape("mix.v")[0] // mc["heads"]
    fc = lc.get("mlp")
    if isinstance(fc, dict):
        if "ff" not in fc.setdefault("expert", {}) and shape("mlp.e0.up"):
            fc["expert"]["ff"] = shape("mlp.e0.up")[0]
        if "experts" not in fc.setdefault("router", {}) and shape("mlp.router"):
            fc["router"]["experts"] = shape("mlp.router")[0]
        if shape("mlp.shared.up") and not fc.get("shared"):
            fc["shared"] = {"ff": shape("mlp.shared.up")[0]}
        elif fc.get("shared") and "ff" not in fc["shared"] and shape("mlp.shared.up"):
            fc["shared"]["ff"] = shape("mlp.shared.up")[0]


# ----------------------------------------------------------------- mixers
class KuteraxParallelMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        lc, rc = mc["left"], mc["right"]
        H, G, D, Dv = lc["heads"], lc["kv_heads"], lc["dim"], lc["vdim"]
        self.left = RotaryWindowSinkAttention(
            H, G, D, Dv, lc["scale"], eps, window=(lc.get("mask") or {}).get("size"),
            rot=lc.get("rot"), qk_norm=True, sink=SINK_SCORE)
        self.right = StateSpaceDuality(
            rc["heads"], rc["vdim"], rc["state"], rc["groups"], rc["conv"],
            rc.get("norm_groups", 1), eps, conv_bias=True)
        # one GEMM for every projection that reads the layer input
        self.splits = [H * D, G * D, G * Dv, H] + self.right.splits
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), bias=True, dtype=dtype,
                                            tp_degree=1)
        self.left_o = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)
        self.right_o = RowParallelLinear(self.right.inner, width, dtype=dtype, tp_degree=1)
        # branch norm weight x layer scale x 1/2, folded once at load time
        f32 = dict(dtype=torch.float32)
        self.left_w = nn.Parameter(torch.ones(width, **f32), requires_grad=False)
        self.right_w = nn.Parameter(torch.ones(width, **f32), requires_grad=False)

    def kv_shape(self):
        return self.left.kv_shape()

    def state_shapes(self):
        return self.right.state_shapes()

    def forward(self, h, kv_mgr, run_idx: int, step):
        lq, lk, lv, lg, z, xbc, dt = torch.split(self.in_proj(h), self.splits, dim=-1)
        left = self.left(lq, lk, lv, kv_mgr, run_idx, step, gate=lg)
        right = self.right(z, xbc, dt, kv_mgr.state, f"run{run_idx}", step)
        return [(self.left_o(left), self.left_w, True),
                (self.right_o(right), self.right_w, True)]

    @staticmethod
    def convert(sd, s, d, w, f, ls1, out):
        L, R = s + "left.", s + "right."
        parts = [L + "q", L + "k", L + "v", L + "g", R + "in"]
        out[d + "in_proj.weight"] = torch.cat([w(n) for n in parts], dim=0)
        out[d + "in_proj.bias"] = torch.cat(
            [w(n + ".b") if n + ".b" in sd else torch.zeros(sd[n].shape[0], dtype=w(n).dtype)
             for n in parts], dim=0)
        out[d + "left.q_norm"] = f(L + "q.norm")
        out[d + "left.k_norm"] = f(L + "k.norm")
        out[d + "left_o.weight"] = w(L + "o")
        out[d + "right_o.weight"] = w(R + "o")
        out[d + "right.conv.weight"] = f(R + "conv")
        out[d + "right.conv.bias"] = f(R + "conv.b") if R + "conv.b" in sd else \
            torch.zeros(sd[R + "conv"].shape[0])
        out[d + "right.A_log"] = f(R + "A_log")
        out[d + "right.dt_bias"] = f(R + "dt_bias")
        out[d + "right.D"] = f(R + "D")
        out[d + "right.norm_weight"] = f(R + "norm")
        out[d + "left_w"] = 0.5 * ls1 * f(L + "out")
        out[d + "right_w"] = 0.5 * ls1 * f(R + "out")


class KuteraxRetentionMixer(nn.Module):
    def __init__(self, width: int, mc: dict, eps: float, dtype: torch.dtype):
        super().__init__()
        H, D, Dv = mc["heads"], mc["dim"], mc["vdim"]
        self.core = Retention(H, D, Dv, mc["decay"], eps)
        self.splits = [H * D, H * D, H * Dv, H * Dv]            # q k v gate
        self.in_proj = ColumnParallelLinear(width, sum(self.splits), dtype=dtype, tp_degree=1)
        self.o_proj = RowParallelLinear(H * Dv, width, dtype=dtype, tp_degree=1)
        self.mix_w = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)

    def kv_shape(self):
        return None

    def state_shapes(self):
        return self.core.state_shapes()

    def forward(self, h, kv_mgr, run_idx: int, step):
        q, k, v, g = torch.split(self.in_proj(h), self.splits, dim=-1)
        y = self.core(q, k, v, g, kv_mgr.state, f"run{run_idx}", step)
        return [(self.o_proj(y), self.mix_w, False)]

    @staticmethod
    def convert(sd, s, d, w, f, ls1, out):
        out[d + "in_proj.weight"] = torch.cat(
            [w(s + "q"), w(s + "k"), w(s + "v"), w(s + "g")], dim=0)
        out[d + "o_proj.weight"] = w(s + "o")
        out[d + "mix_w"] = ls1


_MIXERS = {"parallel": KuteraxParallelMixer, "retention": KuteraxRetentionMixer}


class KuteraxLayer(nn.Module):
    def __init__(self, config: KuteraxInferenceConfig, layer_idx: int):
        super().__init__()
        ec = config.neuron_config
        lc = config.layers[layer_idx]
        self.eps = float(config.norm["eps"])
        W = config.width
        self.dtype = ec.torch_dtype
        self.norm1 = StreamRMSNorm(W, eps=self.eps, one_plus=True, out_dtype=ec.torch_dtype)
        self.mixer = _MIXERS[lc["type"]](W, lc["mixer"], self.eps, ec.torch_dtype)
        self.mlp = None
        fc = lc.get("mlp")
        if fc:
            rc = fc["router"]
            gc = rc.get("groups") or {"count": 1, "keep": 1}
            self.mlp = GroupRoutedFeedForward(
                W, rc["experts"], rc["top"], fc["expert"]["ff"], ec.torch_dtype,
                n_groups=gc["count"], keep_groups=gc["keep"], scale=rc.get("scale", 1.0),
                normalize=False, shared_ff=(fc.get("shared") or {}).get("ff", 0))
            self.ff_w = nn.Parameter(torch.ones(W, dtype=torch.float32), requires_grad=False)

    def kv_shape(self):
        return self.mixer.kv_shape()

    def state_shapes(self) -> Dict[str, tuple]:
        return self.mixer.state_shapes()

    def forward(self, x, kv_mgr, run_idx: int):
        step = kv_mgr.step
        h = self.norm1(x)
        terms = self.mixer(h, kv_mgr, run_idx, step)
        if self.mlp is not None:
            terms.append((self.mlp(h), self.ff_w, False))
        seqmix.scaled_residual(x, terms, self.eps)
        return x


class KuteraxModel(HybridDecoderModel):
    def __init__(self, config):
        super().__init__(config)
        W, dt = config.width, config.neuron_config.torch_dtype
        self.pos_embed = nn.Parameter(torch.zeros(config.max_positions, W, dtype=dt),
                                      requires_grad=False)
        self.loop_in = None
        if config.loop:
            self.loop_in = ColumnParallelLinear(2 * W, W, dtype=dt, tp_degree=1)
            self.loop_step = nn.Parameter(
                torch.zeros(config.loop["times"], W, dtype=torch.float32), requires_grad=False)

    def build_layers(self, config) -> nn.ModuleList:
        return nn.ModuleList(KuteraxLayer(config, i) for i in range(len(config.layers)))

    def build_norm(self, config) -> nn.Module:
        return StreamRMSNorm(config.width, eps=config.norm["eps"], one_plus=True,
                             out_dtype=config.neuron_config.torch_dtype)

    def run_order(self, config):
        self._pass_at = config.pass_starts()
        return config.run_order()

    def prepare_hidden(self, h):
        return seqmix.embed_positions(h, self.pos_embed, self.kv_mgr.step)

    def before_layer_run(self, run_idx, h, h_embed):
        t = self._pass_at.get(run_idx)
        if t is not None:
            # a pass opens: x <- W_in [x; x0] + step[t], x0 the embedding output
            xin = torch.cat([h, h_embed], dim=-1).to(self.dtype)
            return self.loop_in(xin).float() + self.loop_step[t]
        if run_idx == 0 and self._pass_at:
            return h.clone()          # layers update the stream in place; x0 is read later
        return h

    def finalize_logits(self, logits):
        return logits.float()


class KuteraxForCausalLM(CausalLMBase):
    _model_cls = KuteraxModel
    _config_cls = KuteraxInferenceConfig

    @staticmethod
    def convert_hf_to_native_state_dict(sd: Dict[str, torch.Tensor], config) -> Dict[str, torch.Tensor]:
        dt = config.neuron_config.torch_dtype
        out: Dict[str, torch.Tensor] = {}

        def w(name):                       # projection weights: engine dtype
            return sd[name].to(dt)

        def f(name):                       # 32-bit parameters
            return sd[name].float()

        out["embed_tokens.weight"] = w("embed")
        out["pos_embed"] = w("pos")
        out["lm_head.weight"] = w("head")
        out["norm.weight"] = f("final.norm")
        if config.loop:
            out["loop_in.weight"] = w("loop.in")
            out["loop_step"] = f("loop.step")
        for i, lc in enumerate(config.layers):
            s, d = f"l{i}.", f"layers.{i}."
            out[d + "norm1.weight"] = f(s + "norm1")
            ls1 = f(s + "ls1") if s + "ls1" in sd else torch.ones(config.width)
            _MIXERS[lc["type"]].convert(sd, s + "mix.", d + "mixer.", w, f, ls1, out)
            fc = lc.get("mlp")
            if fc:
                E = fc["router"]["experts"]
                m = s + "mlp."
                shared = bool(fc.get("shared"))
                out[d + "mlp.router.weight"] = torch.cat(
                    [f(m + "router")] + ([f(m + "shared.sg")] if shared else []), dim=0)
                out[d + "mlp.experts.up.weight"] = FusedUngatedExperts.stack_up(
                    [w(m + f"e{e}.up") for e in range(E)], w(m + "shared.up") if shared else None)
                out[d + "mlp.experts.down.weight"] = FusedUngatedExperts.stack_down(
                    [w(m + f"e{e}.down") for e in range(E)],
                    w(m + "shared.down") if shared else None)
                out[d + "ff_w"] = f(s + "ls2") if s + "ls2" in sd else torch.ones(config.width)
        return out
