"""Flagship serving benchmark (driver contract).

Measures BASELINE.json's headline metric — output tokens/sec for
Llama-3.1-8B decode (TP=1 on one GPU; TP=N across N GPUs over RCCL/xGMI)
with random-init weights and synthetic data. A "step" is one
token-generation step for the whole batch (one new token per sequence);
prefill at ctx=128 happens before the timed region. Batch is 64 per GPU
(weak scaling).

    python bench.py --gpus N --steps K --warmup W [--model {8b,70b,tiny}]

Under torchrun, reads RANK/LOCAL_RANK/WORLD_SIZE from the env.
"""

from __future__ import annotations

import argparse
import json
import os
import time

import torch
import torch.distributed as dist

MODELS = {
    "tiny": dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                 num_attention_heads=8, num_key_value_heads=4, vocab_size=1024),
    "1b": dict(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16,
               num_attention_heads=32, num_key_value_heads=8, vocab_size=128256,
               head_dim=64),
    "8b": dict(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
               num_attention_heads=32, num_key_value_heads=8, vocab_size=128256),
    "70b": dict(hidden_size=8192, intermediate_size=28672, num_hidden_layers=80,
                num_attention_heads=64, num_key_value_heads=8, vocab_size=128256),
    # Mixtral-8x7B geometry (MoE): dense-bmm expert decode path
    "mixtral": dict(hidden_size=4096, intermediate_size=14336,
                    num_hidden_layers=32, num_attention_heads=32,
                    num_key_value_heads=8, vocab_size=32000,
                    num_local_experts=8, num_experts_per_tok=2),
    # Qwen3-30B-A3B geometry: 128 experts top-8 (fine-grained MoE)
    "qwen3moe": dict(hidden_size=2048, intermediate_size=768,
                     num_hidden_layers=48, num_attention_heads=32,
                     num_key_value_heads=4, head_dim=128, vocab_size=151936,
                     num_local_experts=128, num_experts_per_tok=8),
    # DBRX-132B geometry (BASELINE config 4): 16 experts top-4
    "dbrx": dict(hidden_size=6144, intermediate_size=10752,
                 num_hidden_layers=40, num_attention_heads=48,
                 num_key_value_heads=8, vocab_size=100352,
                 num_local_experts=16, num_experts_per_tok=4),
}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=32)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--model", default="8b", choices=list(MODELS))
    p.add_argument("--batch-per-gpu", type=int, default=256)
    p.add_argument("--ctx", type=int, default=128)
    p.add_argument("--no-graphs", action="store_true")
    p.add_argument("--e2e", action="store_true",
                   help="also run the generate()-level benchmark (p50/p99 + throughput)")
    p.add_argument("--moe-mx4", action="store_true",
                   help="MXFP4 expert weights (4.25 bits) via the grouped v3 kernel")
    p.add_argument("--fp8", action="store_true",
                   help="fp8 (e4m3) weight quantization via hipBLASLt scaled-mm")
    p.add_argument("--spec", action="store_true",
                   help="fused speculative decoding: --model target + 1b draft, spec-len 5")
    p.add_argument("--spec-len", type=int, default=5)
    p.add_argument("--hybrid", action="store_true",
                   help="prefill/decode throughput of the hybrid decoders (Nabelix: windowed "
                        "attention + gated delta rule; Soputar: latent, delta-rule and capped "
                        "attention layers; Kuterax: sink attention + state space in "
                        "parallel, retention, routed experts; Tamilix: chunk-local slope "
                        "attention, windowed gated latent attention, identity-routed "
                        "experts) beside Llama at equal width/depth/ff/vocab")
    p.add_argument("--hybrid-models", default="llama,nabelix,soputar,kuterax,tamilix",
                   help="comma-separated subset of llama,nabelix,soputar,kuterax,tamilix "
                        "for --hybrid")
    p.add_argument("--hybrid-sizes", default="2048,4096",
                   help="comma-separated layer widths for --hybrid")
    p.add_argument("--hybrid-layers", type=int, default=4)
    p.add_argument("--hybrid-prompt", type=int, default=4096)
    return p.parse_args()


HYBRID_SIZES = {
    256: (2, 1, 512),
    # width: heads, kv_heads, ff  (head size 128 everywhere)
    1024: (8, 2, 4096),
    2048: (16, 4, 8192),
    4096: (32, 8, 14336),
}


def run_hybrid_bench(args):
    """Prefill tokens/s (one prompt of --hybrid-prompt tokens) and decode
    tokens/s (--batch-per-gpu sequences at --ctx, hipGraph-captured step) of
    Nabelix and of Llama with the same width, depth, feed-forward size,
    head geometry and vocabulary; random weights, synthetic tokens. Prints
    one JSON line per (model, width)."""
    on_gpu = torch.cuda.is_available()
    device = torch.device("cuda:0" if on_gpu else "cpu")
    from neuronx_distributed_inference_amd.config import (
        EngineConfig, OnDeviceSamplingConfig,
    )
    from neuronx_distributed_inference_amd.models.llama.modeling_llama import (
        LlamaForCausalLM, LlamaInferenceConfig,
    )
    from neuronx_distributed_inference_amd.models.nabelix.modeling_nabelix import (
        NabelixForCausalLM, NabelixInferenceConfig,
    )
    from neuronx_distributed_inference_amd.models.soputar.modeling_soputar import (
        SoputarForCausalLM, SoputarInferenceConfig,
    )
    from neuronx_distributed_inference_amd.models.kuterax.modeling_kuterax import (
        KuteraxForCausalLM, KuteraxInferenceConfig,
    )
    from neuronx_distributed_inference_amd.models.tamilix.modeling_tamilix import (
        TamilixForCausalLM, TamilixInferenceConfig,
    )

    dtype = "bfloat16" if on_gpu else "float32"
    B, ctx, steps, warmup = args.batch_per_gpu, args.ctx, args.steps, args.warmup
    P = args.hybrid_prompt
    L, V = args.hybrid_layers, 32000
    max_len = max(P, ctx + steps + warmup + 8)

    def sync():
        if on_gpu:
            torch.cuda.synchronize()

    def build(kind, width, batch):
        H, G, ff = HYBRID_SIZES[width]
        ec = EngineConfig(
            batch_size=batch, max_batch_size=batch, seq_len=max_len, max_length=max_len,
            max_context_length=P, torch_dtype=dtype, tp_degree=1,
            on_device_sampling_config=OnDeviceSamplingConfig(top_k=1),
            enable_hip_graphs=not args.no_graphs, fused_qkv=True, fused_gate_up=True,
            enable_batch_bucketing=False, pa_block_size=64,
        )
        if kind == "llama":
            cfg = LlamaInferenceConfig(
                neuron_config=ec, hidden_size=width, intermediate_size=ff,
                num_hidden_layers=L, num_attention_heads=H, num_key_value_heads=G,
                head_dim=128, vocab_size=V, max_position_embeddings=max_len * 2,
                rms_norm_eps=1e-5, rope_theta=500000.0, hidden_act="silu",
                tie_word_embeddings=False)
            cls = LlamaForCausalLM
        elif kind == "soputar":
            # the design's layer mix, repeated to depth L: latent attention
            # (512-wide latent + 64 rotated channels), delta rule, capped
            # GQA attention, and a layer that borrows the previous one's KV
            mlp = {"kind": "dense", "ff": ff, "limit": 7.0}
            att = {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                   "softcap": 30.0, "q_temp": {"coef": 0.3, "every": 128}}
            quad = [
                {"type": "latent_attention", "mlp": mlp, "mixer": {
                    "heads": H, "dim": 128, "rot_dim": 64, "vdim": 128,
                    "kv_rank": min(512, width // 4),
                    "scale": 192 ** -0.5, "rot": {"base": 10000.0, "dims": 64}}},
                {"type": "delta", "mlp": mlp, "mixer": {
                    "heads": H, "kv_heads": H, "dim": 128, "vdim": 128, "conv": 4}},
                {"type": "attention", "mlp": mlp, "mixer": dict(att)},
                {"type": "attention", "mlp": mlp, "mixer": dict(att, kv_from=2)},
            ]
            layers = []
            for i in range(L):
                lc = json.loads(json.dumps(quad[i % 4]))
                if "kv_from" in lc["mixer"]:
                    lc["mixer"]["kv_from"] = i - 1
                layers.append(lc)
            cfg = SoputarInferenceConfig(
                neuron_config=ec, architecture="Soputar", width=width, vocab=V,
                layers=layers, norm={"eps": 1e-5}, embedding={"scale": 8.0})
            cls = SoputarForCausalLM
        elif kind == "kuterax":
            # alternating parallel (sink attention + state space) and retention
            # layers; the feed-forward activates ff columns per token: four of
            # sixteen experts of ff/8 plus a shared expert of ff/2
            mlp = {"kind": "moe", "expert": {"ff": ff // 8}, "shared": {"ff": ff // 2},
                   "router": {"experts": 16, "top": 4, "scale": 1.5,
                              "groups": {"count": 4, "keep": 2}}}
            par = {"type": "parallel", "mlp": mlp, "mixer": {
                "left": {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128,
                         "scale": 128 ** -0.5, "mask": {"size": 1024},
                         "rot": {"base": 500000.0, "dims": 64, "scaling": {
                             "factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}},
                "right": {"heads": 2 * H, "vdim": 64, "state": 128, "groups": G, "conv": 4,
                          "norm_groups": G}}}
            ret = {"type": "retention", "mlp": mlp, "mixer": {
                "heads": H, "dim": 128, "vdim": 128,
                "decay": [1.0 - 2.0 ** (-5 - (i % 4)) for i in range(H)]}}
            cfg = KuteraxInferenceConfig(
                neuron_config=ec, architecture="Kuterax", width=width, vocab=V,
                max_positions=max_len, layers=[par if i % 2 == 0 else ret for i in range(L)],
                loop={"start": 0, "stop": L, "times": 1}, norm={"eps": 1e-5})
            cls = KuteraxForCausalLM
        elif kind == "tamilix":
            # the design's layer mix, repeated to depth L: chunk-local slope
            # attention with a dense relu-squared feed-forward, windowed latent
            # attention (512-wide latent + 64 rotated channels, query latent of
            # 3/4 width) with routed experts, attention with routed experts, and
            # a latent layer that runs the second layer's weights again. The
            # routed feed-forward activates at most ff columns per token: four
            # of sixteen experts of ff/8 and two pass-through experts, plus a
            # shared expert of ff/2
            moe = {"kind": "moe", "expert": {"ff": ff // 8, "limit": 7.0},
                   "shared": {"ff": ff // 2, "limit": 7.0},
                   "router": {"experts": 16, "identity": 2, "top": 4}}
            att = {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                   "mask": {"size": 1024}}
            lat = {"heads": H, "dim": 128, "rot_dim": 64, "vdim": 128,
                   "kv_rank": min(512, width // 4), "q_rank": width * 3 // 4,
                   "scale": 192 ** -0.5, "rot": {"base": 10000.0, "dims": 64},
                   "mask": {"size": 1024}}
            quad = [
                {"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": ff}},
                {"type": "latent_attention", "mixer": lat, "mlp": moe},
                {"type": "attention", "mixer": att, "mlp": moe},
                {"type": "latent_attention", "mixer": lat, "mlp": moe, "weights_of": 1},
            ]
            layers = []
            for i in range(L):
                lc = json.loads(json.dumps(quad[i % 4]))
                if "weights_of" in lc:
                    lc["weights_of"] = i - 2
                layers.append(lc)
            cfg = TamilixInferenceConfig(
                neuron_config=ec, architecture="Tamilix", width=width, vocab=V,
                layers=layers, norm={"eps": 1e-5}, embedding={"scale": 8.0})
            cls = TamilixForCausalLM
        else:
            layer = {"type": "parallel", "mlp": {"kind": "dense", "ff": ff}, "mixer": {
                "left": {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128,
                         "scale": 128 ** -0.5, "mask": {"size": 1024, "keep_first": 4}},
                "right": {"heads": H, "kv_heads": H, "dim": 128, "vdim": 128, "conv": 4,
                          "decay_rank": 64, "gate_rank": 64},
                "left_scale": 1.0, "right_scale": 1.0}}
            cfg = NabelixInferenceConfig(
                neuron_config=ec, architecture="Nabelix", width=width, vocab=V,
                layers=[layer] * L, canon={"taps": 4}, norm={"eps": 1e-5},
                loop={"start": 0, "stop": 0, "times": 1}, logit_softcap=30.0)
            cls = NabelixForCausalLM
        torch.manual_seed(1234)
        if on_gpu:
            with torch.device(device):
                m = cls(cfg).eval()
        else:
            m = cls(cfg).eval()
        with torch.no_grad():
            for p in m.parameters():
                if p.dim() >= 2 and p.requires_grad:   # caches/state do not
                    p.normal_(0, 0.02)
        m.reset()
        m.enable_submodels()
        return m

    for width in [int(x) for x in args.hybrid_sizes.split(",")]:
        for kind in [k for k in ("llama", "nabelix", "soputar", "kuterax", "tamilix")
                     if k in args.hybrid_models.split(",")]:
            with torch.inference_mode():
                # ---- prefill: one prompt, three timed repetitions
                m = build(kind, width, 1)
                ids = torch.randint(0, V, (1, P), device=device)
                pos = torch.arange(P, device=device).view(1, P)
                sid = torch.zeros(1, dtype=torch.long, device=device)
                for _ in range(2):
                    m.reset()
                    m(input_ids=ids, position_ids=pos, seq_ids=sid)
                sync()
                t0 = time.perf_counter()
                for _ in range(3):
                    m.kv_cache_populated = False
                    m(input_ids=ids, position_ids=pos, seq_ids=sid)
                sync()
                prefill_s = (time.perf_counter() - t0) / 3
                del m
                # ---- decode: B sequences at ctx
                m = build(kind, width, B)
                if on_gpu and not args.no_graphs:
                    m.warmup()
                ids = torch.randint(0, V, (B, ctx), device=device)
                pos = torch.arange(ctx, device=device).view(1, ctx).expand(B, ctx).contiguous()
                sid = torch.arange(B, device=device)
                tok = m(input_ids=ids, position_ids=pos, seq_ids=sid).tokens.view(-1, 1)
                pos_t = torch.full((B, 1), ctx, device=device, dtype=torch.long)
                for _ in range(warmup):
                    tok = m(input_ids=tok, position_ids=pos_t, seq_ids=sid).tokens.view(-1, 1)
                    pos_t.add_(1)
                sync()
                t0 = time.perf_counter()
                for _ in range(steps):
                    tok = m(input_ids=tok, position_ids=pos_t, seq_ids=sid).tokens.view(-1, 1)
                    pos_t.add_(1)
                sync()
                decode_s = (time.perf_counter() - t0) / steps
                del m
                if on_gpu:
                    torch.cuda.empty_cache()
            print(json.dumps({
                "bench": "hybrid", "model": kind, "width": width, "layers": L,
                "dtype": dtype, "data": "synthetic, random-init",
                "prefill_tokens": P, "prefill_ms": round(prefill_s * 1e3, 3),
                "prefill_tok_s": round(P / prefill_s, 1),
                "decode_batch": B, "decode_ctx": ctx,
                "decode_ms_per_step": round(decode_s * 1e3, 3),
                "decode_tok_s": round(B / decode_s, 1),
            }), flush=True)


def run_spec_bench(args):
    """Fused speculation round benchmark (BASELINE config 5: 8B target +
    1B draft, spec-len 5). Random-init weights make draft/target agreement
    chance-level, so tokens/s here measures the worst-case (~1 token/round);
    round latency is the hardware-meaningful number."""
    import torch

    on_gpu = torch.cuda.is_available()
    device = torch.device("cuda:0" if on_gpu else "cpu")
    from neuronx_distributed_inference_amd.config import (
        EngineConfig, OnDeviceSamplingConfig,
    )
    from neuronx_distributed_inference_amd.models.llama.modeling_llama import (
        LlamaForCausalLM, LlamaInferenceConfig,
    )
    from neuronx_distributed_inference_amd.modules.speculation import (
        FusedSpeculationModel,
    )
    from neuronx_distributed_inference_amd.runtime.graph_engine import GraphRunner

    steps, warmup = args.steps, args.warmup
    B = args.batch_per_gpu
    total_len = args.ctx + (steps + warmup + 2) * (args.spec_len + 1)
    dtype = "bfloat16" if on_gpu else "float32"

    def build(spec_name):
        ec = EngineConfig(
            batch_size=B, max_batch_size=B, seq_len=total_len, max_length=total_len,
            torch_dtype=dtype, tp_degree=1,
            on_device_sampling_config=OnDeviceSamplingConfig(top_k=1),
            fused_qkv=True, fused_gate_up=True,
        )
        cfg = LlamaInferenceConfig(
            neuron_config=ec, max_position_embeddings=total_len * 2,
            rms_norm_eps=1e-5, rope_theta=500000.0, hidden_act="silu",
            tie_word_embeddings=False, **MODELS[spec_name],
        )
        torch.manual_seed(7)
        m = LlamaForCausalLM(cfg).eval()
        if on_gpu:
            m = m.to(device)
        with torch.no_grad():
            for p in m.parameters():
                if p.dim() >= 2:
                    p.normal_(0, 0.02)
        m.reset()
        return m

    target = build(args.model)
    draft = build("1b" if args.model != "tiny" else "tiny")
    fused = FusedSpeculationModel(target.model, draft.model, args.spec_len)

    ids = torch.randint(0, MODELS[args.model]["vocab_size"], (B, args.ctx), device=device)
    seq_ids = torch.arange(B, device=device)
    pos = torch.arange(args.ctx, device=device).view(1, -1).expand(B, -1)
    with torch.inference_mode():
        t_out = target(input_ids=ids, position_ids=pos, seq_ids=seq_ids)
        draft(input_ids=ids, position_ids=pos, seq_ids=seq_ids)
        tok = t_out.tokens.view(B, 1)
        lengths = torch.full((B, 1), args.ctx, device=device, dtype=torch.long)

        runner = fused
        if on_gpu and not args.no_graphs:
            try:
                runner = GraphRunner(fused, (tok, lengths, seq_ids))
            except Exception:  # noqa: BLE001
                import traceback
                traceback.print_exc()
                torch.cuda.synchronize()
                runner = fused

        accepted_total = 0
        def round_(tok, lengths, accepted_total):
            acc, n = runner(tok, lengths, seq_ids)
            lengths = lengths + n.view(B, 1) + 1
            tok = acc.gather(1, n.view(B, 1))
            return tok, lengths, accepted_total + int(n.sum()) + B

        for _ in range(warmup):
            tok, lengths, _ = round_(tok, lengths, 0)
        if on_gpu:
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            tok, lengths, accepted_total = round_(tok, lengths, accepted_total)
        if on_gpu:
            torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0

    print(json.dumps({
        "metric": "output tokens/sec (node), fused speculation 8B+1B spec-5",
        "value": round(accepted_total / elapsed, 2),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(elapsed / steps * 1000.0, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {
            "model": f"llama-3.1-{args.model} + llama-3.2-1b draft",
            "global_batch": B, "ctx": args.ctx, "speculation_length": args.spec_len,
            "parallelism": "tp1", "weights": "random-init",
            "note": "random weights => chance-level acceptance; ms_per_step is one spec round",
        },
    }))


def main():
    args = parse_args()
    if args.spec:
        return run_spec_bench(args)
    if args.hybrid:
        return run_hybrid_bench(args)
    world = int(os.environ.get("WORLD_SIZE", 1))
    rank = int(os.environ.get("RANK", 0))
    local_rank = int(os.environ.get("LOCAL_RANK", 0))
    assert world == args.gpus or world == 1, f"WORLD_SIZE {world} != --gpus {args.gpus}"

    on_gpu = torch.cuda.is_available()
    device = torch.device(f"cuda:{local_rank}" if on_gpu else "cpu")
    if on_gpu:
        torch.cuda.set_device(device)
    if world > 1:
        dist.init_process_group(
            backend="nccl" if on_gpu else "gloo",
            device_id=device if on_gpu else None,
        )

    from neuronx_distributed_inference_amd.config import (
        EngineConfig,
        OnDeviceSamplingConfig,
    )
    from neuronx_distributed_inference_amd.models.llama.modeling_llama import (
        LlamaForCausalLM,
        LlamaInferenceConfig,
    )
    from neuronx_distributed_inference_amd.models.mixtral.modeling_mixtral import (
        MixtralForCausalLM,
        MixtralInferenceConfig,
    )
    from neuronx_distributed_inference_amd.parallel import state as ps

    tp = world
    ps.initialize_model_parallel(tensor_model_parallel_size=tp)

    spec = dict(MODELS[args.model])
    global_batch = args.batch_per_gpu * max(world, 1)
    steps, warmup = args.steps, args.warmup
    total_len = args.ctx + warmup + steps + 8
    dtype = "bfloat16" if on_gpu else "float32"

    ec = EngineConfig(
        batch_size=global_batch, max_batch_size=global_batch,
        seq_len=total_len, max_length=total_len, max_context_length=args.ctx,
        torch_dtype=dtype, tp_degree=tp,
        on_device_sampling_config=OnDeviceSamplingConfig(top_k=1),
        enable_hip_graphs=not args.no_graphs,
        fused_qkv=True, fused_gate_up=True,
        # the bench always decodes at full batch: a single captured graph
        # (the sub-batch ladder is a serving feature; fewer RCCL-in-graph
        # captures = less surface on the multi-GPU scaling runs)
        enable_batch_bucketing=False,
    )
    if args.model in ("mixtral", "dbrx", "qwen3moe"):
        # dbrx geometry is benchmarked through the same stacked-expert MoE
        # module (the DBRX model class differs in norms/clip, same compute
        # shape); random-init synthetic benchmarking per BASELINE
        model_cls, cfg_cls = MixtralForCausalLM, MixtralInferenceConfig
    else:
        model_cls, cfg_cls = LlamaForCausalLM, LlamaInferenceConfig
    cfg = cfg_cls(
        neuron_config=ec, max_position_embeddings=total_len * 2,
        rms_norm_eps=1e-5, rope_theta=500000.0, hidden_act="silu",
        tie_word_embeddings=False, **spec,
    )

    torch.manual_seed(1234)
    if on_gpu:
        # construct directly on the GPU: a 70B bf16 model is 140 GB and must
        # never round-trip host RAM / PCIe
        with torch.device(device):
            model = model_cls(cfg).eval()
    else:
        model = model_cls(cfg).eval()
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.normal_(0, 0.02)
    model.reset()
    if args.moe_mx4:
        from neuronx_distributed_inference_amd.modules.moe import ExpertMLPs

        nm = sum(1 for m in model.model.modules()
                 if isinstance(m, ExpertMLPs) and m.quantize_mx4())
        if rank == 0:
            print(f"# quantized {nm} expert stacks to MXFP4", flush=True)
    if args.fp8:
        from neuronx_distributed_inference_amd.parallel.layers import quantize_model_fp8

        nq = quantize_model_fp8(model.model)
        if rank == 0:
            print(f"# quantized {nq} linears to fp8", flush=True)
    model.enable_submodels()
    if on_gpu and not args.no_graphs:
        with torch.inference_mode():
            model.warmup()  # hipGraph capture for the decode step

    V = spec["vocab_size"]
    ids = torch.randint(0, V, (global_batch, args.ctx), device=device)
    mask = torch.ones_like(ids)
    seq_ids = torch.arange(global_batch, device=device)

    def barrier_sync():
        if world > 1:
            dist.barrier()
        if on_gpu:
            torch.cuda.synchronize()

    with torch.inference_mode():
        # ---- prefill (untimed) ----
        pos = (mask.long().cumsum(-1) - 1).clamp(min=0)
        out = model(input_ids=ids, attention_mask=mask, position_ids=pos, seq_ids=seq_ids)
        next_tok = out.tokens.view(-1, 1)
        cur_len = args.ctx

        # device-resident position counter: no per-step host->device copy
        pos_t = torch.full((global_batch, 1), cur_len, device=device, dtype=torch.long)

        def decode_step(tok):
            o = model(input_ids=tok, attention_mask=None, position_ids=pos_t, seq_ids=seq_ids)
            pos_t.add_(1)
            return o.tokens.view(-1, 1)

        # ---- warmup ----
        for _ in range(warmup):
            next_tok = decode_step(next_tok)

        barrier_sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            next_tok = decode_step(next_tok)
        barrier_sync()
        elapsed = time.perf_counter() - t0

    # max over ranks
    if world > 1:
        t = torch.tensor([elapsed], device=device if on_gpu else "cpu")
        dist.all_reduce(t, op=dist.ReduceOp.MAX)
        elapsed = float(t.item())

    if rank == 0:
        ms_per_step = elapsed / steps * 1000.0
        tokens_per_sec = global_batch * steps / elapsed
        print(json.dumps({
            "metric": "output tokens/sec (node), Llama-3.1-8B decode" if args.model == "8b"
                      else f"output tokens/sec (node), {args.model} decode",
            "value": round(tokens_per_sec, 2),
            "unit": "tokens/s",
            "n_gpus": max(world, 1),
            "steps": steps,
            "warmup": warmup,
            "ms_per_step": round(ms_per_step, 3),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": ("fp8-weights+bf16" if args.fp8 else ("mxfp4-experts+bf16" if args.moe_mx4 else dtype)),
            "data": "synthetic",
            "config": {
                "model": {"8b": "llama-3.1-8b", "70b": "llama-3.1-70b",
                          "tiny": "tiny-llama-2l", "1b": "llama-3.2-1b",
                          "mixtral": "mixtral-8x7b",
                          "qwen3moe": "qwen3-30b-a3b-geometry",
                          "dbrx": "dbrx-132b-geometry"}[args.model],
                "global_batch": global_batch,
                "seq_len": total_len,
                "ctx": args.ctx,
                "parallelism": f"tp{tp}",
                "weights": "random-init",
            },
        }))

    if args.e2e and rank == 0 and world == 1:
        from neuronx_distributed_inference_amd.utils.benchmark import benchmark_sampling
        from neuronx_distributed_inference_amd.utils.hf_adapter import GenerationConfig

        report = benchmark_sampling(
            model, ids, attention_mask=mask, n_runs=3,
            generation_config=GenerationConfig(max_new_tokens=min(steps, 32)),
            report_path=None,
        )
        print(json.dumps({"e2e_report": report}))

    if world > 1:
        dist.destroy_process_group()


if __name__ == "__main__":
    main()
