#!/usr/bin/env python3
"""Flagship serving benchmark: Llama-3-8B decode throughput (output tok/s).

Contract (driver): `python bench.py --gpus N --steps K --warmup W` — for N>1
launched under torch.distributed.run with one rank per GPU. Each rank runs an
independent engine replica (data-parallel serving, the deployment shape of
BASELINE.json config "Llama-3-8B /v1/completions at 1/2/4/8 MI355X"); the
reported value is the WHOLE-JOB aggregate output tok/s.

A "step" = one continuous-batching decode iteration over the full running
batch. Synthetic random prompts, random-init bf16 weights (no network).
TTFT p50 is measured on the prefill wave and reported alongside.
"""

import argparse
import json
import os
import statistics
import time

# hipBLASLt GEMM algo selection via TunableOp: load the committed gfx950
# tuning table (profiles/tunableop_gfx950<ordinal>.csv) when present.
_TUNE_BASE = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                          "profiles", "tunableop_gfx950.csv")
if os.path.exists(_TUNE_BASE.replace(".csv", "0.csv")):
    os.environ.setdefault("PYTORCH_TUNABLEOP_ENABLED", "1")
    os.environ.setdefault("PYTORCH_TUNABLEOP_TUNING", "0")
    os.environ.setdefault("PYTORCH_TUNABLEOP_FILENAME", _TUNE_BASE)


# layer shapes for --hybrid-compare: widths, head counts and feed-forward
# sizes of common 1-3B and 7-8B models; the state-space sublayers use the
# usual 2x inner width, 64-wide heads and 128 states
HYBRID_SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, head_dim=128, ff=8192,
               ssm_heads=64, ssm_vdim=64, state=128, groups=8, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, head_dim=128, ff=14336,
               ssm_heads=128, ssm_vdim=64, state=128, groups=8, vocab=32000),
}


def _hybrid_model_configs(size: dict, layers: int):
    from kserve_amd.engine.config import (
        AttentionMixerSpec,
        GLUSpec,
        HybridLayerSpec,
        HybridModelConfig,
        ModelConfig,
        SSMMixerSpec,
    )

    ssm = SSMMixerSpec(heads=size["ssm_heads"], vdim=size["ssm_vdim"],
                       state=size["state"], groups=size["groups"], conv=4,
                       norm_groups=size["groups"])
    attn = AttentionMixerSpec(heads=size["heads"], kv_heads=size["kv_heads"],
                              dim=size["head_dim"], vdim=size["head_dim"],
                              scale=size["head_dim"] ** -0.5,
                              q_temp_coef=0.1, q_temp_every=1024)
    mlp = GLUSpec(ff=size["ff"], limit=7.0)
    specs = []
    for i in range(layers):
        if i % 2 == 0:
            specs.append(HybridLayerSpec("mamba2", ssm=ssm, mlp=mlp))
        else:
            specs.append(HybridLayerSpec("parallel", attention=attn, ssm=ssm,
                                         mlp=mlp))
    hybrid = HybridModelConfig(vocab_size=size["vocab"],
                               hidden_size=size["width"], layers=specs,
                               model_name="merulorn-bench")
    llama = ModelConfig(vocab_size=size["vocab"], hidden_size=size["width"],
                        intermediate_size=size["ff"], num_layers=layers,
                        num_heads=size["heads"], num_kv_heads=size["kv_heads"],
                        head_dim=size["head_dim"],
                        max_position_embeddings=8192, model_name="llama-bench")
    return hybrid, llama


# layer shapes for --desalix-compare: the widths and heads of HYBRID_SIZES;
# 8 experts of which a token uses 2, each half as wide as the dense
# feed-forward of that size, so a token does the arithmetic of the dense
# layer; attention is local to `chunk` positions
DESALIX_SIZES = {
    "2k": dict(width=2048, heads=16, kv_heads=4, head_dim=128, ff=4096,
               experts=8, top=2, chunk=1024, vocab=32000),
    "4k": dict(width=4096, heads=32, kv_heads=8, head_dim=128, ff=7168,
               experts=8, top=2, chunk=1024, vocab=32000),
}


def _desalix_model_configs(size: dict, runs: int):
    """A Desalix model whose middle layer is run ``runs - 2`` times (so a
    token passes ``runs`` layers) and a llama model of ``runs`` layers with
    the same width and heads and a dense feed-forward as wide as the experts
    one token uses (equal arithmetic per token; full causal attention, whose
    work per query grows with the context while the chunk-local one's does
    not)."""
    from kserve_amd.engine.config import (
        AttentionMixerSpec,
        HybridLayerSpec,
        HybridModelConfig,
        LoopSpec,
        ModelConfig,
        MoESpec,
    )

    attn = AttentionMixerSpec(heads=size["heads"], kv_heads=size["kv_heads"],
                              dim=size["head_dim"], vdim=size["head_dim"],
                              scale=size["head_dim"] ** -0.5,
                              rot_dims=size["head_dim"] // 2, rot_base=500000.0,
                              chunk=size["chunk"])
    mlp = MoESpec(experts=size["experts"], top=size["top"], ff=size["ff"],
                  limit=7.0, shared=None)
    desalix = HybridModelConfig(
        vocab_size=size["vocab"], hidden_size=size["width"],
        layers=[HybridLayerSpec("attention", attention=attn, mlp=mlp)
                for _ in range(3)],
        loop=LoopSpec(start=1, stop=2, times=runs - 2),
        model_name="desalix-bench", architecture="Desalix",
    )
    llama = ModelConfig(vocab_size=size["vocab"], hidden_size=size["width"],
                        intermediate_size=size["top"] * size["ff"],
                        num_layers=runs,
                        num_heads=size["heads"], num_kv_heads=size["kv_heads"],
                        head_dim=size["head_dim"],
                        max_position_embeddings=8192, model_name="llama-bench")
    return desalix, llama


# layer shapes for --voborax-compare: the widths, head counts and experts of
# DESALIX_SIZES; 128 unrotated + 64 rotated query/key coordinates per head,
# a cached row of 192 latent + 64 rotated columns per token and layer
VOBORAX_SIZES = {
    "2k": dict(width=2048, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=192,
               q_rank=768, window=1024, ff=4096, experts=8, top=2, vocab=32000),
    "4k": dict(width=4096, heads=32, dim=128, rot_dim=64, vdim=128, kv_rank=192,
               q_rank=1536, window=1024, ff=7168, experts=8, top=2, vocab=32000),
}


def _voborax_model_configs(size: dict):
    """A four-layer Voborax model (windowed + experts, windowed reading layer
    0's rows + experts, windowed + dense, causal with sink + experts) and the
    Desalix model of equal width, heads, depth and experts that
    --desalix-compare measures."""
    from kserve_amd.engine.config import (
        HybridLayerSpec,
        HybridModelConfig,
        LatentAttentionSpec,
        MLPSpec,
        SoftmaxMoESpec,
    )

    def latent(window, sink, kv_from=None):
        rot = 0 if sink else size["rot_dim"]
        return LatentAttentionSpec(
            heads=size["heads"], dim=size["dim"], vdim=size["vdim"],
            kv_rank=size["kv_rank"] + (size["rot_dim"] - rot),
            q_rank=size["q_rank"], scale=(size["dim"] + rot) ** -0.5,
            rot_dim=rot, rot_dims=rot, rot_base=500000.0, window=window,
            sink=sink, gate=not sink, kv_from=kv_from,
        )

    moe = SoftmaxMoESpec(experts=size["experts"], top=size["top"], ff=size["ff"],
                         identity=1, shared_ff=0)
    # two matrices instead of an expert's three: equal arithmetic per token
    dense = MLPSpec(ff=3 * size["top"] * size["ff"] // 2)
    w = size["window"]
    voborax = HybridModelConfig(
        vocab_size=size["vocab"], hidden_size=size["width"],
        layers=[
            HybridLayerSpec("latent_attention", latent=latent(w, False), mlp=moe),
            HybridLayerSpec("latent_attention", latent=latent(w, False, 0), mlp=moe),
            HybridLayerSpec("latent_attention", latent=latent(w, False), mlp=dense),
            HybridLayerSpec("latent_attention_2", latent=latent(0, True), mlp=moe),
        ],
        model_name="voborax-bench", architecture="Voborax", residual_mult=0.7,
    )
    dsize = dict(DESALIX_SIZES["2k" if size["width"] == 2048 else "4k"])
    desalix, _ = _desalix_model_configs(dsize, runs=4)
    return voborax, desalix


# layer shapes for --laperax-compare: the widths, head counts and head sizes
# of HYBRID_SIZES; value heads of 128 columns over half as many q/k heads in
# the delta layers, a 1024-token window, 8 experts of which a token uses 2
LAPERAX_SIZES = {
    "2k": dict(hybrid="2k", width=2048, heads=16, kv_heads=4, head_dim=128,
               ff=4096, experts=8, top=2, window=1024, vocab=32000),
    "4k": dict(hybrid="4k", width=4096, heads=32, kv_heads=8, head_dim=128,
               ff=7168, experts=8, top=2, window=1024, vocab=32000),
}


def _laperax_model_configs(size: dict):
    """A four-layer Laperax model (delta, retention, windowed attention,
    retention; experts beside every mixer) and the Merulorn model that
    --hybrid-compare measures at the same width."""
    from kserve_amd.engine.config import (
        AttentionMixerSpec,
        DeltaMixerSpec,
        HybridLayerSpec,
        HybridModelConfig,
        RetentionMixerSpec,
        SquaredReluMoESpec,
    )

    H, D = size["heads"], size["head_dim"]
    moe = SquaredReluMoESpec(experts=size["experts"], top=size["top"],
                             ff=size["ff"], scale=2.5)
    delta = DeltaMixerSpec(heads=H, kv_heads=H // 2, dim=D, vdim=D, conv=4)
    ret = RetentionMixerSpec(
        heads=H, dim=D, vdim=D, rot_dims=D, rot_base=1e6,
        decay=[1.0 - 2.0 ** (-5.0 - 6.0 * i / max(H - 1, 1)) for i in range(H)],
    )
    attn = AttentionMixerSpec(heads=H, kv_heads=size["kv_heads"], dim=D, vdim=D,
                              scale=D ** -0.5, rot_dims=D // 2, rot_base=1e4,
                              window=size["window"])
    layers = [
        HybridLayerSpec("delta", delta=delta, mlp=moe),
        HybridLayerSpec("retention", retention=ret, mlp=moe),
        HybridLayerSpec("attention", attention=attn, mlp=moe),
        HybridLayerSpec("retention", retention=ret, mlp=moe),
    ]
    laperax = HybridModelConfig(
        vocab_size=size["vocab"], hidden_size=size["width"], layers=layers,
        model_name="laperax-bench", architecture="Laperax",
        logit_scale=0.5, logit_softcap=30.0,
    )
    merulorn, _ = _hybrid_model_configs(HYBRID_SIZES[size["hybrid"]], layers=4)
    return laperax, merulorn


def _throughput(mcfg, prompt_len, n_prompts, concurrency, steps, warmup, eager):
    """(prefill tok/s, decode tok/s) through the engine's own step()."""
    import torch

    from kserve_amd.engine.config import CacheConfig, EngineConfig, SchedulerConfig
    from kserve_amd.engine.engine import LLMEngine
    from kserve_amd.engine.sampling_params import SamplingParams

    window = 8
    max_len = prompt_len + (steps + warmup + 2) * window + 64
    blocks = (max(n_prompts, concurrency) + 2) * (-(-max_len // 16)) + 64
    cfg = EngineConfig(
        model=mcfg,
        cache=CacheConfig(block_size=16, num_gpu_blocks=blocks),
        scheduler=SchedulerConfig(
            max_num_seqs=max(n_prompts, concurrency),
            max_num_batched_tokens=n_prompts * prompt_len,
            max_model_len=max_len, multi_step=window,
        ),
        device="cuda", seed=7, enforce_eager=eager, eos_token_id=-1,
    )
    engine = LLMEngine(cfg)
    gen = torch.Generator().manual_seed(3)
    sp = SamplingParams(temperature=0.0, max_tokens=max_len, ignore_eos=True)

    def submit(n, tag):
        for i in range(n):
            engine.add_request(
                torch.randint(0, mcfg.vocab_size, (prompt_len,), generator=gen).tolist(),
                sp, request_id=f"{tag}-{i}",
            )

    # prefill: one step takes n_prompts whole prompts; time the second wave
    submit(n_prompts, "warm")
    engine.step()
    for r in list(engine.scheduler.running):
        engine.abort_request(r.request_id)
    submit(n_prompts, "timed")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    engine.step()
    torch.cuda.synchronize()
    prefill = n_prompts * prompt_len / (time.perf_counter() - t0)
    for r in list(engine.scheduler.running):
        engine.abort_request(r.request_id)

    # decode: `concurrency` sequences with prompt_len context each
    submit(concurrency, "dec")
    while engine.scheduler.num_waiting > 0:
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens = 0
    for _ in range(steps):
        tokens += sum(len(o.new_token_ids) for o in engine.step())
    torch.cuda.synchronize()
    decode = tokens / (time.perf_counter() - t0)
    del engine
    torch.cuda.empty_cache()
    return prefill, decode


def hybrid_compare(args):
    """Prefill and decode tok/s of the Merulorn design next to a llama model
    of equal size, both through LLMEngine.step() on one GPU, bf16, random
    weights. Prints one JSON line per (size, model)."""
    import torch

    assert torch.cuda.is_available(), "--hybrid-compare needs a GPU"
    for name in args.hybrid_compare.split(","):
        size = HYBRID_SIZES[name]
        hybrid, llama = _hybrid_model_configs(size, layers=4)
        for label, mcfg in (("hybrid", hybrid), ("llama", llama)):
            if args.hybrid_only and args.hybrid_only != label:
                continue
            prefill, decode = _throughput(
                mcfg, prompt_len=args.prompt_len if args.prompt_len != 512 else 2048,
                n_prompts=8, concurrency=min(args.concurrency, 256),
                steps=args.steps, warmup=args.warmup, eager=args.eager,
            )
            print(json.dumps({
                "bench": "hybrid-compare", "size": name, "model": mcfg.model_name,
                "layers": 4, "width": size["width"],
                "prefill_tok_s": round(prefill, 1),
                "decode_tok_s": round(decode, 1),
                "prefill_batch": "8 x prompt", "decode_concurrency":
                    min(args.concurrency, 256),
                "dtype": "bfloat16", "data": "synthetic, random-init weights",
            }), flush=True)


def desalix_compare(args):
    """Prefill and decode tok/s of the Desalix design next to a llama model of
    equal width, heads, depth and feed-forward arithmetic per token, both
    through LLMEngine.step() on one GPU, bf16, random weights. One JSON line per
    (size, model), each measured in a process of its own and printed as soon
    as it is done."""
    import subprocess
    import sys

    if args.compare_only is None or "," in args.desalix_compare:
        rc = 0
        for name in args.desalix_compare.split(","):
            for label in ("desalix", "llama"):
                if args.compare_only and args.compare_only != label:
                    continue
                cmd = [sys.executable, "-u", os.path.abspath(__file__),
                       "--desalix-compare", name, "--compare-only", label,
                       "--steps", str(args.steps), "--warmup", str(args.warmup),
                       "--concurrency", str(args.concurrency),
                       "--prompt-len", str(args.prompt_len)]
                if args.eager:
                    cmd.append("--eager")
                rc = subprocess.call(cmd)
                if rc != 0:
                    return rc
        return rc

    import torch

    assert torch.cuda.is_available(), "--desalix-compare needs a GPU"
    name, label = args.desalix_compare, args.compare_only
    size = DESALIX_SIZES[name]
    desalix, llama = _desalix_model_configs(size, runs=4)
    mcfg = desalix if label == "desalix" else llama
    prefill, decode = _throughput(
        mcfg, prompt_len=args.prompt_len if args.prompt_len != 512 else 2048,
        n_prompts=8, concurrency=min(args.concurrency, 256),
        steps=args.steps, warmup=args.warmup, eager=args.eager,
    )
    print(json.dumps({
        "bench": "desalix-compare", "size": name, "model": mcfg.model_name,
        "layer_runs": 4, "width": size["width"],
        "experts": size["experts"], "top": size["top"],
        "prefill_tok_s": round(prefill, 1),
        "decode_tok_s": round(decode, 1),
        "prefill_batch": "8 x prompt", "decode_concurrency":
            min(args.concurrency, 256),
        "dtype": "bfloat16", "data": "synthetic, random-init weights",
    }), flush=True)
    return 0


def voborax_compare(args):
    """Prefill and decode tok/s of the Voborax design next to the Desalix
    model of equal width, heads, depth and experts (the closest design the
    engine serves: the same fp32 attention kernel and routed experts), both
    through LLMEngine.step() on one GPU, bf16, random weights. One JSON line
    per (size, model), each measured in a process of its own."""
    import subprocess
    import sys

    if args.compare_only is None or "," in args.voborax_compare:
        rc = 0
        for name in args.voborax_compare.split(","):
            for label in ("voborax", "desalix"):
                if args.compare_only and args.compare_only != label:
                    continue
                cmd = [sys.executable, "-u", os.path.abspath(__file__),
                       "--voborax-compare", name, "--compare-only", label,
                       "--steps", str(args.steps), "--warmup", str(args.warmup),
                       "--concurrency", str(args.concurrency),
                       "--prompt-len", str(args.prompt_len)]
                if args.eager:
                    cmd.append("--eager")
                rc = subprocess.call(cmd)
                if rc != 0:
                    return rc
        return rc

    import torch

    assert torch.cuda.is_available(), "--voborax-compare needs a GPU"
    name, label = args.voborax_compare, args.compare_only
    size = VOBORAX_SIZES[name]
    voborax, desalix = _voborax_model_configs(size)
    mcfg = voborax if label == "voborax" else desalix
    prefill, decode = _throughput(
        mcfg, prompt_len=args.prompt_len if args.prompt_len != 512 else 2048,
        n_prompts=8, concurrency=min(args.concurrency, 256),
        steps=args.steps, warmup=args.warmup, eager=args.eager,
    )
    print(json.dumps({
        "bench": "voborax-compare", "size": name, "model": mcfg.model_name,
        "layers": 4, "width": size["width"],
        "experts": size["experts"], "top": size["top"],
        "prefill_tok_s": round(prefill, 1),
        "decode_tok_s": round(decode, 1),
        "prefill_batch": "8 x prompt", "decode_concurrency":
            min(args.concurrency, 256),
        "dtype": "bfloat16", "data": "synthetic, random-init weights",
    }), flush=True)
    return 0


def laperax_compare(args):
    """Prefill and decode tok/s of the Laperax design next to the Merulorn
    model of equal width and depth (the closest design the engine serves:
    recurrent state per slot beside KV pages, a scan kernel, a short
    convolution), both through LLMEngine.step() on one GPU, bf16, random
    weights. One JSON line per (size, model), each measured in a process of
    its own."""
    import subprocess
    import sys

    if args.compare_only is None or "," in args.laperax_compare:
        rc = 0
        for name in args.laperax_compare.split(","):
            for label in ("laperax", "merulorn"):
                if args.compare_only and args.compare_only != label:
                    continue
                cmd = [sys.executable, "-u", os.path.abspath(__file__),
                       "--laperax-compare", name, "--compare-only", label,
                       "--steps", str(args.steps), "--warmup", str(args.warmup),
                       "--concurrency", str(args.concurrency),
                       "--prompt-len", str(args.prompt_len)]
                if args.eager:
                    cmd.append("--eager")
                rc = subprocess.call(cmd)
                if rc != 0:
                    return rc
        return rc

    import torch

    assert torch.cuda.is_available(), "--laperax-compare needs a GPU"
    name, label = args.laperax_compare, args.compare_only
    size = LAPERAX_SIZES[name]
    laperax, merulorn = _laperax_model_configs(size)
    mcfg = laperax if label == "laperax" else merulorn
    prefill, decode = _throughput(
        mcfg, prompt_len=args.prompt_len if args.prompt_len != 512 else 2048,
        n_prompts=8, concurrency=min(args.concurrency, 256),
        steps=args.steps, warmup=args.warmup, eager=args.eager,
    )
    print(json.dumps({
        "bench": "laperax-compare", "size": name, "model": mcfg.model_name,
        "layers": 4, "width": size["width"],
        "prefill_tok_s": round(prefill, 1),
        "decode_tok_s": round(decode, 1),
        "prefill_batch": "8 x prompt", "decode_concurrency":
            min(args.concurrency, 256),
        "dtype": "bfloat16", "data": "synthetic, random-init weights",
    }), flush=True)
    return 0


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    # defaults sized so a flagless run finishes in minutes AND its KV
    # demand (concurrency * (prompt + 8*(steps+warmup) + 64) tokens) fits
    # the pool with no preemption churn
    parser.add_argument("--steps", type=int, default=16)
    parser.add_argument("--warmup", type=int, default=4)
    parser.add_argument("--concurrency", type=int, default=1536,
                        help="concurrent sequences per GPU")
    parser.add_argument("--prompt-len", type=int, default=512)
    parser.add_argument("--model", type=str, default="llama-3-8b",
                        choices=["llama-3-8b", "llama-3-70b", "mixtral-8x7b",
                                 "mistral-7b", "tiny"])
    parser.add_argument("--tp", type=int, default=1,
                        help="tensor-parallel degree (ranks per engine)")
    parser.add_argument("--kv-blocks", type=int, default=0,
                        help="override KV pool size (0 = derive from HBM)")
    parser.add_argument("--eager", action="store_true",
                        help="disable hipGraph capture")
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--multi-step", dest="multi_step", type=int, default=8,
                        help="decode iterations per hipGraph window")
    parser.add_argument("--kv-cache-dtype", type=str, default="auto",
                        choices=["auto", "fp8"],
                        help="opt-in fp8 E4M3 KV cache (NOT the headline "
                             "config; bf16 compute is unchanged)")
    parser.add_argument("--hybrid-compare", type=str, default=None,
                        metavar="SIZE[,SIZE...]",
                        help="instead of the flagship workload: prefill and "
                             "decode throughput of a Merulorn-design model "
                             "beside a llama model of equal width, heads, "
                             "feed-forward and depth (sizes: "
                             + ", ".join(HYBRID_SIZES) + ")")
    parser.add_argument("--hybrid-only", type=str, default=None,
                        choices=["hybrid", "llama"],
                        help="with --hybrid-compare: run one side only "
                             "(e.g. under a profiler)")
    parser.add_argument("--desalix-compare", type=str, default=None,
                        metavar="SIZE[,SIZE...]",
                        help="instead of the flagship workload: prefill and "
                             "decode throughput of a Desalix-design model "
                             "beside a llama model of equal width, heads, "
                             "depth and arithmetic per token (sizes: "
                             + ", ".join(DESALIX_SIZES) + ")")
    parser.add_argument("--voborax-compare", type=str, default=None,
                        metavar="SIZE[,SIZE...]",
                        help="instead of the flagship workload: prefill and "
                             "decode throughput of a Voborax-design model "
                             "beside the Desalix model of equal width, heads, "
                             "depth and experts (sizes: "
                             + ", ".join(VOBORAX_SIZES) + ")")
    parser.add_argument("--laperax-compare", type=str, default=None,
                        metavar="SIZE[,SIZE...]",
                        help="instead of the flagship workload: prefill and "
                             "decode throughput of a Laperax-design model "
                             "beside the Merulorn model of equal width and "
                             "depth (sizes: " + ", ".join(LAPERAX_SIZES) + ")")
    parser.add_argument("--compare-only", type=str, default=None,
                        choices=["desalix", "llama", "voborax", "laperax",
                                 "merulorn"],
                        help="with --desalix-compare / --voborax-compare / "
                             "--laperax-compare: run one side only (e.g. "
                             "under a profiler)")
    parser.add_argument("--profile-cpu", action="store_true",
                        help="cProfile the timed loop and print hot functions")
    args = parser.parse_args()
    if args.hybrid_compare:
        return hybrid_compare(args)
    if args.desalix_compare:
        return desalix_compare(args)
    if args.voborax_compare:
        return voborax_compare(args)
    if args.laperax_compare:
        return laperax_compare(args)

    import torch

    from kserve_amd.engine.config import (
        CacheConfig,
        EngineConfig,
        ModelConfig,
        SchedulerConfig,
    )
    from kserve_amd.engine.engine import LLMEngine
    from kserve_amd.engine.sampling_params import SamplingParams
    from kserve_amd.parallel import comm

    state = comm.init_distributed(tp_size=args.tp)
    rank, world = state.rank, state.world_size
    use_gpu = torch.cuda.is_available()
    device = state.device if use_gpu else "cpu"

    if args.model == "llama-3-8b":
        mcfg = ModelConfig.llama3_8b()
    elif args.model == "llama-3-70b":
        mcfg = ModelConfig.llama3_70b()
    elif args.model == "mixtral-8x7b":
        mcfg = ModelConfig.mixtral_8x7b()
    elif args.model == "mistral-7b":
        mcfg = ModelConfig.mistral_7b()
    else:
        mcfg = ModelConfig(
            vocab_size=1024, hidden_size=512, intermediate_size=1024,
            num_layers=2, num_heads=4, num_kv_heads=2, head_dim=128,
            max_position_embeddings=2048, model_name="tiny",
        )

    # each timed "step" is one scheduling iteration = up to `multi_step`
    # decode iterations (hipGraph window); budget the KV/model length for it
    window = args.multi_step
    max_model_len = args.prompt_len + (args.steps + args.warmup) * window + 64
    cfg = EngineConfig(
        model=mcfg,
        cache=CacheConfig(
            block_size=16,
            num_gpu_blocks=args.kv_blocks or None,
            gpu_memory_utilization=0.9,
            kv_cache_dtype=args.kv_cache_dtype,
        ),
        scheduler=SchedulerConfig(
            max_num_seqs=args.concurrency,
            max_num_batched_tokens=16384,
            max_model_len=max_model_len,
            multi_step=args.multi_step,
        ),
        device=device,
        seed=1234 + state.dp_rank,
        enforce_eager=args.eager or not use_gpu,
        eos_token_id=-1,
    )

    engine = LLMEngine(cfg)

    gen = torch.Generator().manual_seed(42 + state.dp_rank)
    sp = SamplingParams(
        temperature=args.temperature,
        max_tokens=max_model_len,  # never finishes inside the run
        ignore_eos=True,
    )
    t_submit = time.perf_counter()
    for i in range(args.concurrency):
        prompt = torch.randint(
            0, mcfg.vocab_size, (args.prompt_len,), generator=gen
        ).tolist()
        engine.add_request(prompt, sp, request_id=f"bench-{rank}-{i}")

    # ---- prefill wave (also measures TTFT) ----
    ttfts = []
    while engine.scheduler.num_waiting > 0 or any(
        r.first_token_time is None for r in engine.scheduler.running
    ):
        engine.step()
    for r in engine.scheduler.running:
        ttfts.append(r.first_token_time - t_submit)
    ttft_p50_ms = statistics.median(ttfts) * 1000 if ttfts else None
    prefill_done = time.perf_counter()

    # ---- warmup decode steps ----
    for _ in range(args.warmup):
        engine.step()

    # ---- timed region ----
    comm.barrier()
    if use_gpu:
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens = 0
    prof = None
    if args.profile_cpu:
        import cProfile

        prof = cProfile.Profile()
        prof.enable()
    for _ in range(args.steps):
        outs = engine.step()
        tokens += sum(len(o.new_token_ids) for o in outs)
    if prof is not None:
        prof.disable()
    comm.barrier()
    if use_gpu:
        torch.cuda.synchronize()
    t1 = time.perf_counter()
    elapsed = t1 - t0

    # max elapsed over ranks; sum tokens over ranks
    if world > 1:
        import torch.distributed as dist

        # NCCL/RCCL requires device tensors for collectives
        red_dev = device if use_gpu else "cpu"
        te = torch.tensor([elapsed], dtype=torch.float64, device=red_dev)
        tk = torch.tensor([float(tokens)], dtype=torch.float64, device=red_dev)
        dist.all_reduce(te, op=dist.ReduceOp.MAX)
        dist.all_reduce(tk, op=dist.ReduceOp.SUM)
        elapsed = float(te[0])
        tokens = int(tk[0])

    if prof is not None and rank == 0:
        import pstats
        import sys

        stats = pstats.Stats(prof, stream=sys.stderr)
        stats.sort_stats("cumulative").print_stats(25)

    if rank == 0:
        value = tokens / elapsed
        n_gpus = world if use_gpu else args.gpus
        result = {
            "metric": f"output tok/s, {mcfg.model_name} /v1/completions decode",
            "value": round(value, 1),
            "unit": "tok/s",
            "n_gpus": n_gpus,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(elapsed / args.steps * 1000, 3),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "bfloat16",
            "data": "synthetic random prompts, random-init weights",
            "ttft_p50_ms": round(ttft_p50_ms, 1) if ttft_p50_ms else None,
            "config": {
                "model": mcfg.model_name,
                "global_batch": args.concurrency * (world // args.tp),
                "seq_len": args.prompt_len,
                "parallelism": f"dp{world // args.tp}"
                + (f"xtp{args.tp}" if args.tp > 1 else ""),
                "kv_block_size": 16,
                "hipgraph": not cfg.enforce_eager,
                # headline runs use the bf16 KV default; fp8 KV is an
                # explicit opt-in and must be visible in the record
                "kv_cache_dtype": args.kv_cache_dtype,
            },
        }
        print(json.dumps(result), flush=True)

    comm.destroy_distributed()


if __name__ == "__main__":
    main()
