"""Decode and prefill throughput of the engine at Qwen2-7B size (or, with --size, 72B or 0.5B) with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the engine's own loop: one token of every request through `Engine.step`,
greedy selection on the device, the chosen ids back to the host. Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SIZES = {
    "7b": dict(vocab_size=152064, hidden_size=3584, num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4,
               head_dim=128, intermediate_size=18944, tie_word_embeddings=False),
    "72b": dict(vocab_size=152064, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8,
                head_dim=128, intermediate_size=29568, tie_word_embeddings=False),
    "0.5b": dict(vocab_size=151936, hidden_size=896, num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2,
                 head_dim=64, intermediate_size=4864, tie_word_embeddings=True),
}
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
BF16_PEAK_FLOPS = 2.5e15       # MI355X dense bf16 MFMA, published
FP32_PEAK_FLOPS = 157.3e12


def serve(args, config, full_layers: int, page_size: int) -> int:
    """The reference's continuous-batching workload through the scheduler; prints one JSON line."""
    from microllm_rocm_amd import Engine
    from microllm_rocm_amd.engine.benchmark import serving_throughput
    requests, longest, new_tokens, chunk, budget = args.serve_requests, 2048, 256, 512, 2048
    max_tokens = requests * (-(-(longest + new_tokens) // page_size) + 1) * page_size
    engine = Engine.from_random(config, seed=0, dtype=args.dtype, device="cuda:0", on_device=True, page_size=page_size,
                                max_tokens=max_tokens, max_requests=requests, weight_copies=args.weight_copies,
                                max_portion=chunk, graph_mixed_steps=not args.no_mixed_graphs)
    runs = max(1, min(args.steps, 5))
    warmup = max(1, min(args.warmup, 2))
    result = serving_throughput(engine, requests=requests, prompt_range=(128, longest), new_tokens=new_tokens,
                                prefill_chunk=chunk, max_batched_tokens=budget, runs=runs, warmup=warmup)
    line = {
        "metric": f"continuous batching, generated tok/s, Qwen2-{args.size.upper()} {'bf16' if args.dtype == 'bfloat16' else 'fp32'}",
        "value": round(result["tokens_per_second"], 1), "unit": "tok/s", "n_gpus": 1, "steps": runs, "warmup": warmup,
        "ms_per_step": round(result["ms_per_run"], 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random N(0,0.02) weights, uniform-random token ids and prompt lengths; a step is one whole run of the workload",
        "config": {"model": f"Qwen2-{args.size.upper()} size", "layers": args.layers, "layers_of_full_model": full_layers,
                   "requests": requests, "prompt_lengths": "uniform 128..2048", "new_tokens": new_tokens,
                   "prefill_chunk": chunk, "max_batched_tokens": budget, "kv_block_size": page_size,
                   "weight_copies": engine.weight_copies, "mixed_step_graphs": not args.no_mixed_graphs,
                   "parallelism": "single GPU"},
        "serve": {key: (round(value, 2) if isinstance(value, float) else value) for key, value in result.items()},
    }
    print(json.dumps(line), flush=True)
    return 0


DESIGN_SIZES = {
    # width, query heads, kv heads, head size, feed-forward width, layers; the linear attention beside the softmax
    # attention of a Siditar layer has half as many heads, keys of half the head size and values of the whole
    "1k": dict(width=1024, heads=8, kv_heads=2, head_dim=128, ff=4096, layers=4),
    "2k": dict(width=2048, heads=16, kv_heads=4, head_dim=128, ff=8192, layers=4),
    "4k": dict(width=4096, heads=32, kv_heads=8, head_dim=128, ff=14336, layers=2),
}
DESIGN_VOCAB = 32768


def gupitar_config(size: dict):
    """A Gupitar configuration of the given layer sizes: heads of 96 unrotated and 32 rotated query/key dims and 128
    value dims, cached rows of 192 + 64 elements (the widest the MFMA attention kernels take), windows of 1024, a
    recurrence as wide as the model in blocks of 128 with four taps; the first layer's feed-forward dense, the others
    16 experts of a quarter of the feed-forward width, two a token, and a shared expert of half of it (as many active
    rows a token as the dense one). Layers in turn: attention, recurrence, attention, attention on the rows of the one before."""
    from microllm_rocm_amd.config.gupitar import (DenseMlpConfig, GupitarConfig, GupitarLayerConfig, LatentAttentionConfig, MoeMlpConfig,
                                                  RglruConfig)
    width, ff = size["width"], size["ff"]

    def attention(kv_from=None):
        return LatentAttentionConfig(heads=size["heads"], dim=96, rot_dim=64, vdim=size["head_dim"], q_rank=width // 2, kv_rank=192,
                                     scale=160 ** -0.5, window=1024, rot_base=1e6, rot_dims=64, kv_from=kv_from)

    layers = []
    for index in range(size["layers"]):
        kind = ("attention", "recurrence", "attention", "borrow")[index % 4]
        mlp = DenseMlpConfig(ff) if index == 0 else MoeMlpConfig(experts=16, top=2, expert_ff=ff // 4, shared_ff=ff // 2)
        if kind == "recurrence":
            layers.append(GupitarLayerConfig("rglru", RglruConfig(width=width, blocks=width // 128, conv=4), mlp))
        else:
            layers.append(GupitarLayerConfig("latent_attention", attention(index - 1 if kind == "borrow" else None), mlp))
    return GupitarConfig(vocab=DESIGN_VOCAB, width=width, norm_eps=1e-6, layers=tuple(layers))


def zabozen_config(size: dict):
    """A Zabozen configuration of the given layer sizes: layers in turn a latent attention (heads of 96 unrotated and 64
    rotated query/key dims and 128 value dims, cached rows of 192 + 64 elements, queries straight from the input, a
    gate a head), a gated delta rule (as many value heads as the model has heads over its key/value head count of
    key heads, 128 dims each, four taps), a window attention with slopes (the model's heads and key/value heads of the
    head size, a window of 1024) and one on the keys and values of the layer before; every feed-forward dense."""
    from microllm_rocm_amd.config.zabozen import (DeltaConfig, DenseMlpConfig, LatentAttentionConfig, WindowAttentionConfig,
                                                  ZabozenConfig, ZabozenLayerConfig)
    width, heads, kv_heads, dim = size["width"], size["heads"], size["kv_heads"], size["head_dim"]
    layers = []
    for index in range(size["layers"]):
        kind = ("latent_attention", "delta", "attention", "borrow")[index % 4]
        if kind == "latent_attention":
            mixer = LatentAttentionConfig(heads=heads, dim=96, rot_dim=64, vdim=dim, kv_rank=192, scale=160 ** -0.5, rot_base=1e6, rot_dims=64)
        elif kind == "delta":
            mixer = DeltaConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, conv=4)
        else:
            mixer = WindowAttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, window=1024,
                                          kv_from=index - 1 if kind == "borrow" else None)
        layers.append(ZabozenLayerConfig("attention" if kind == "borrow" else kind, mixer, DenseMlpConfig(size["ff"])))
    return ZabozenConfig(vocab=DESIGN_VOCAB, width=width, norm_eps=1e-6, residual_mult=0.5, layers=tuple(layers), logit_softcap=30.0)


def kalevik_config(size: dict):
    """A Kalevik configuration of the given layer sizes: layers in turn a latent attention (heads of 96 unrotated and 64
    rotated query/key dims and 128 value dims, cached rows of 192 + 64 elements) with a dense feed-forward, and a parallel
    mixer (a softmax attention of the model's heads and key/value heads inside chunks of 8192 positions, which a
    prompt of 2048 tokens and a context of 4096 lie within, so that it reads every key as Qwen2's does, half of every
    head turned; beside it a retention of half as many heads with keys of half the head size, as Siditar's linear
    attention) with 16 experts of a quarter of the feed-forward width, four a token out of the best two of four groups,
    and a shared expert of half of it. Every layer runs once: a looped range is the same layers again."""
    from microllm_rocm_amd.config.kalevik import (ChunkAttentionConfig, DenseMlpConfig, KalevikConfig, KalevikLayerConfig,
                                                  LatentAttentionConfig, MoeMlpConfig, ParallelConfig, RetentionConfig)
    width, heads, kv_heads, dim, ff = size["width"], size["heads"], size["kv_heads"], size["head_dim"], size["ff"]
    latent = LatentAttentionConfig(heads=heads, dim=96, rot_dim=64, vdim=dim, kv_rank=192, scale=160 ** -0.5, rot_base=1e6, rot_dims=64)
    left = ChunkAttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, chunk=8192, rot_base=1e6,
                                rot_dims=dim // 2, rot_factor=2.0)
    right = RetentionConfig(heads=heads // 2, dim=dim // 2, vdim=dim, decay=tuple(1.0 - 0.1 / (1 + head % 6) for head in range(heads // 2)))
    moe = MoeMlpConfig(experts=16, top=4, expert_ff=ff // 4, groups=4, keep_groups=2, shared_ff=ff // 2)
    layers = [KalevikLayerConfig("latent_attention", latent, DenseMlpConfig(ff)) if index % 2 == 0 else
              KalevikLayerConfig("parallel", ParallelConfig(left, right, 0.75, 1.25), moe) for index in range(size["layers"])]
    return KalevikConfig(vocab=DESIGN_VOCAB, width=width, norm_eps=1e-6, layers=tuple(layers), embedding_scale=2.0)


def design_configs(size: dict, design: str = "siditar"):
    """The design's configuration at the given layer sizes and the Qwen2 configuration of equal width, heads, head size,
    feed-forward width, depth and vocabulary."""
    from microllm_rocm_amd import Qwen2Config
    qwen2 = Qwen2Config(vocab_size=DESIGN_VOCAB, hidden_size=size["width"], num_hidden_layers=size["layers"],
                        num_attention_heads=size["heads"], num_key_value_heads=size["kv_heads"], head_dim=size["head_dim"],
                        intermediate_size=size["ff"], max_position_embeddings=32768, rope_theta=1e6, rms_norm_eps=1e-6,
                        tie_word_embeddings=False)
    if design == "gupitar":
        return {"gupitar": gupitar_config(size), "qwen2": qwen2}
    if design == "zabozen":     # beside the design whose layers are most like its own, and beside Qwen2
        return {"zabozen": zabozen_config(size), "gupitar": gupitar_config(size), "qwen2": qwen2}
    if design == "kalevik":     # beside the designs whose layers are most like its own (latents and experts; a parallel mixer)
        return {"kalevik": kalevik_config(size), "gupitar": gupitar_config(size), "siditar": design_configs(size, "siditar")["siditar"],
                "qwen2": qwen2}
    from microllm_rocm_amd.config.siditar import (BiasAttentionConfig, DenseMlpConfig, LinearAttentionConfig,
                                                  ParallelMixerConfig, SiditarConfig, SiditarLayerConfig)
    left = BiasAttentionConfig(heads=size["heads"], kv_heads=size["kv_heads"], dim=size["head_dim"], vdim=size["head_dim"],
                               scale=size["head_dim"] ** -0.5, bias_max=1024, temp_coef=0.5, temp_every=64, bias_rows=32)
    right = LinearAttentionConfig(heads=size["heads"] // 2, dim=size["head_dim"] // 2, vdim=size["head_dim"], tau=16.0, decay_rank=16)
    layer = SiditarLayerConfig("parallel", ParallelMixerConfig(left, right, 1.0, 1.0), DenseMlpConfig(size["ff"], 7.0))
    siditar = SiditarConfig(vocab=DESIGN_VOCAB, width=size["width"], norm_eps=1e-6, layers=(layer,) * size["layers"], streams=2)
    return {"siditar": siditar, "qwen2": qwen2}


def compare_designs(args) -> int:
    """Prefill and decode throughput of the chosen design beside Qwen2 at equal layer sizes; prints one JSON line."""
    import torch
    from microllm_rocm_amd import Engine
    from microllm_rocm_amd.engine.benchmark import decode_throughput, prefill_throughput, step_bytes, step_flops
    page_size, rows = 16, []
    peak_flops = BF16_PEAK_FLOPS if args.dtype == "bfloat16" else FP32_PEAK_FLOPS
    for name in [part for part in args.design_sizes.split(",") if part]:
        size = DESIGN_SIZES[name]
        for design, config in design_configs(size, args.design).items():
            if args.design_only and design != args.design_only:
                continue
            per_request = args.context + args.steps + args.warmup + 2 * page_size
            engine = Engine.from_random(config, seed=0, dtype=args.dtype, device="cuda:0", on_device=True, page_size=page_size,
                                        max_tokens=max(args.batch * per_request, args.prefill_tokens + page_size),
                                        max_requests=max(args.batch, 4))
            row = {"design": design, "size": name, **size}
            if not args.no_prefill:
                prefill = prefill_throughput(engine, args.prefill_tokens, repeats=3)
                flops = step_flops(engine, args.prefill_tokens)
                row["prefill"] = {"tokens": args.prefill_tokens, "tok_per_s": round(prefill["tokens_per_second"], 1),
                                  "ms": round(prefill["ms"], 3), "frac_of_peak": round(flops / (prefill["ms"] * 1e-3) / peak_flops, 4)}
            decode = decode_throughput(engine, args.batch, args.context, args.steps, args.warmup, seed=1)
            moved = step_bytes(engine, args.batch, args.context + args.warmup + args.steps // 2)
            row["decode"] = {"batch": args.batch, "context": args.context, "tok_per_s": round(decode["tokens_per_second"], 1),
                             "ms_per_step": round(decode["ms_per_step"], 4),
                             "frac_of_hbm": round(moved / (decode["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
            rows.append(row)
            del engine
            torch.cuda.empty_cache()
    first = next((row for row in rows if row["design"] == args.design), rows[0])
    others = " and ".join(name.capitalize() for name in design_configs(DESIGN_SIZES["1k"], args.design) if name != args.design)
    line = {"metric": f"decode tok/s of the {args.design.capitalize()} design beside {others} at equal layer sizes", "value": first["decode"]["tok_per_s"],
            "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": first["decode"]["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: random weights, uniform-random token ids, caches filled with random keys and values",
            "config": {"model": f"{args.design.capitalize()} and {others} at sizes {args.design_sizes}", "global_batch": args.batch, "seq_len": args.context,
                       "vocab": DESIGN_VOCAB, "kv_block_size": page_size, "parallelism": "single GPU"},
            "compare": rows}
    print(json.dumps(line), flush=True)
    return 0


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--size", default="7b", choices=sorted(SIZES), help="layer sizes: Qwen2-7B's (the default), 72B's or 0.5B's")
    parser.add_argument("--layers", type=int, default=None, help="fewer than the model has only where memory or time needs it")
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--weight-copies", default="auto", choices=["auto", "both", "packed"],
                        help="packed: one copy of every weight, and this package's own matrix kernels for every product")
    parser.add_argument("--no-library-tuning", action="store_true",
                        help="leave the choice of the library's algorithm for the prompt's large products to its heuristic")
    parser.add_argument("--no-calibration", action="store_true", help="skip measuring what a read-only and an MFMA-only kernel reach")
    parser.add_argument("--serve", action="store_true",
                        help="the continuous-batching workload instead: 64 requests, prompts of 128 to 2048 tokens, 256 new tokens each, "
                             "portions of 512 (--steps whole runs timed after --warmup untimed ones); meant for --size 0.5b")
    parser.add_argument("--serve-requests", type=int, default=64)
    parser.add_argument("--no-mixed-graphs", action="store_true", help="run steps that mix portions and single tokens eagerly")
    parser.add_argument("--no-extras", action="store_true",
                        help="leave out what the default run adds to its line after the main figures: decoding on the 32-bit path "
                             "at batch 8 and the continuous-batching workload at Qwen2-0.5B sizes")
    parser.add_argument("--design", default=None, choices=["siditar", "gupitar", "zabozen", "kalevik"],
                        help="instead of the default workload: prefill and decode throughput of this design beside Qwen2 at equal "
                             "layer sizes (--design-sizes), random weights; --batch, --context, --prefill-tokens, --steps apply")
    parser.add_argument("--design-sizes", default="1k,2k,4k", help="of " + ", ".join(sorted(DESIGN_SIZES)))
    parser.add_argument("--design-only", default=None, choices=["siditar", "gupitar", "zabozen", "kalevik", "qwen2"], help="one of the designs alone (profiles)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2

    import torch
    from microllm_rocm_amd import Engine, Qwen2Config
    from microllm_rocm_amd.engine.benchmark import decode_throughput, prefill_throughput, step_bytes, step_flops

    if args.design:
        return compare_designs(args)
    sizes = dict(SIZES[args.size])
    full_layers = sizes.pop("num_hidden_layers")
    if args.layers is None:
        args.layers = full_layers
    config = Qwen2Config(num_hidden_layers=args.layers, max_position_embeddings=32768, rope_theta=1e6, rms_norm_eps=1e-6, **sizes)
    page_size = 16
    if args.serve:
        return serve(args, config, full_layers, page_size)
    points = sorted({int(b) for b in args.points.split(",") if b} | {args.batch})
    largest = max(points)
    per_request = args.context + args.steps + args.warmup + 2 * page_size
    max_tokens = max(largest * per_request, args.prefill_tokens + page_size)
    engine = Engine.from_random(config, seed=0, dtype=args.dtype, device="cuda:0", on_device=True,
                                page_size=page_size, max_tokens=max_tokens, max_requests=max(largest, 4),
                                weight_copies=args.weight_copies,
                                tune_library=not args.no_library_tuning and not args.no_prefill)
    peak_flops = BF16_PEAK_FLOPS if args.dtype == "bfloat16" else FP32_PEAK_FLOPS

    results = {}
    for batch in points:
        results[batch] = decode_throughput(engine, batch, args.context, args.steps, args.warmup, seed=batch)
    main_result = results[args.batch]
    bytes_step = step_bytes(engine, args.batch, args.context + args.warmup + args.steps // 2)
    achieved = bytes_step / (main_result["ms_per_step"] * 1e-3) / 1e9

    line = {
        "metric": f"decode tok/s (ctx {args.context}) Qwen2-{args.size.upper()} {'bf16' if args.dtype == 'bfloat16' else 'fp32'}",
        "value": round(main_result["tokens_per_second"], 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_result["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random N(0,0.02) weights, uniform-random token ids, caches filled with random keys and values",
        "config": {
            "model": f"Qwen2-{args.size.upper()} size", "layers": args.layers, "layers_of_full_model": full_layers,
            "hidden_size": config.hidden_size, "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "intermediate_size": config.intermediate_size, "vocab_size": config.vocab_size,
            "tie_word_embeddings": config.tie_word_embeddings, "weight_copies": engine.weight_copies,
            "library_tuning": not args.no_library_tuning and not args.no_prefill, "global_batch": args.batch, "seq_len": args.context,
            "kv_block_size": page_size, "prefill_tokens": args.prefill_tokens, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {f"decode_b{batch}": round(results[batch]["tokens_per_second"], 2) for batch in points if batch != args.batch},
    }
    if not args.no_prefill:
        prefill = prefill_throughput(engine, args.prefill_tokens, repeats=3)
        flops = step_flops(engine, args.prefill_tokens)
        line["prefill"] = {"value": round(prefill["tokens_per_second"], 1), "tokens": args.prefill_tokens,
                           "ms": round(prefill["ms"], 3),
                           "frac": round(flops / (prefill["ms"] * 1e-3) / peak_flops, 4),
                           "runs": "best of 3 (value, ms, frac); their mean beside it",
                           "mean_ms": round(prefill["mean_ms"], 3), "mean_value": round(prefill["mean_tokens_per_second"], 1),
                           "mean_frac": round(flops / (prefill["mean_ms"] * 1e-3) / peak_flops, 4), "all_ms": prefill["all_ms"]}
    if not args.no_calibration and args.dtype == "bfloat16":
        # What kernels that do nothing but read memory, or nothing but bfloat16 MFMAs, reach on this GPU: the
        # fractions of these stand beside the fractions of the published peaks.
        from microllm_rocm_amd.ops.kernels import measured_peaks
        measured = measured_peaks()
        line["measured_peaks"] = measured
        line["roofline"]["frac_of_measured"] = round(achieved / measured["hbm_read_GBps"], 4)
        if "prefill" in line:
            line["prefill"]["frac_of_measured"] = round(flops / (prefill["ms"] * 1e-3) / (measured["mfma_bf16_TFLOPs"] * 1e12), 4)
    extras = not args.no_extras and args.size == "7b" and args.dtype == "bfloat16" and args.layers == full_layers
    if extras:
        # Two more figures of the same program on the same GPU, each on an engine of its own after the main one is
        # gone: decoding on the true 32-bit path, and the continuous-batching workload at the smallest model's sizes.
        del engine
        torch.cuda.empty_cache()
        exact = Engine.from_random(config, seed=0, dtype="float32", device="cuda:0", on_device=True, page_size=page_size,
                                   max_tokens=8 * (args.context + 8 + 2 * page_size), max_requests=8)
        fp32 = decode_throughput(exact, 8, args.context, steps=5, warmup=1, seed=8)
        fp32_bytes = step_bytes(exact, 8, args.context + 3)
        line["points"]["fp32_decode_b8"] = round(fp32["tokens_per_second"], 2)
        line["fp32"] = {"config": "the same model and context on the true 32-bit path, batch 8, 5 steps after 1", "dtype": "fp32",
                        "value": round(fp32["tokens_per_second"], 2), "ms_per_step": round(fp32["ms_per_step"], 3),
                        "roofline_frac": round(fp32_bytes / (fp32["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        del exact
        torch.cuda.empty_cache()
        from microllm_rocm_amd.engine.benchmark import serving_throughput
        small_sizes = dict(SIZES["0.5b"])
        small = Qwen2Config(max_position_embeddings=32768, rope_theta=1e6, rms_norm_eps=1e-6, **small_sizes)
        requests, longest, new_tokens, chunk, budget = 64, 2048, 256, 512, 2048
        server = Engine.from_random(small, seed=0, dtype="bfloat16", device="cuda:0", on_device=True, page_size=page_size,
                                    max_tokens=requests * (-(-(longest + new_tokens) // page_size) + 1) * page_size,
                                    max_requests=requests, max_portion=chunk)
        served = serving_throughput(server, requests=requests, prompt_range=(128, longest), new_tokens=new_tokens,
                                    prefill_chunk=chunk, max_batched_tokens=budget, runs=3, warmup=1)
        line["serve"] = {"config": "Qwen2-0.5B size, bf16, 64 requests, prompts uniform 128..2048, 256 new tokens each, "
                                   "portions of 512, 2048 tokens a step, 3 runs after 1",
                         "value": round(served["tokens_per_second"], 1), "unit": "generated tok/s",
                         "ttft_p50_ms": round(served["ttft_p50_ms"], 1), "ttft_p95_ms": round(served["ttft_p95_ms"], 1),
                         "completion_p95_ms": round(served["completion_p95_ms"], 1), "preemptions": served["preemptions"],
                         "scheduler_steps": served["scheduler_steps"]}
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
