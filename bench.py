#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen2 1.5B shape (random bfloat16 weights, synthetic tokens)
on one MI355X, with the achieved fraction of the HBM and matrix-core rooflines.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

Beside the headline (batch 8, context 4,096) `points` holds decode at batch 1 and 64 and, in the default run, two
further sizes, each with its fraction of the HBM peak computed as `roofline` is (weights once + the live requests'
cache, over the step's time): batch 8 at context 32,768, and batch 64 at context 4,096 of the 7B shape (a second
engine, weights drawn on the device).

A step is one decode step of the engine: `Engine.step()` on requests that the engine itself has prefilled to the
context, every request of the batch getting one token from the paged cache, its next token coming back to the
host; the engine launches the next step before this step's tokens have been waited for.  Prints ONE JSON line;
`device_ms_per_step` is the device's own time for a step's kernels beside the wall time `ms_per_step`.
"""
import argparse
import json
import os
import sys
import tempfile
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# The benchmark's model: the Qwen2 1.5B shape (the layout of DeepSeek-R1-Distill-Qwen-1.5B, the checkpoint the
# reference publishes its numbers on: README.md:31-32 of 11Aln0/ginfer)
SHAPE = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=28, hidden_size=1536,
             num_attention_heads=12, num_key_value_heads=2, head_dim=128, intermediate_size=8960, vocab_size=151936,
             rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=131072,
             use_sliding_window=False, sliding_window=4096, max_window_layers=21)
# a larger shape of the same architecture, for looking at the kernels at other sizes (--shape 7b): Qwen2-7B's sizes
SHAPE_7B = dict(SHAPE, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
                vocab_size=152064, rope_theta=1e6, max_position_embeddings=32768, max_window_layers=28)
# Qwen2.5-72B's sizes: 145 GB of bfloat16 weights on the one GPU, drawn on the device (no model folder)
SHAPE_72B = dict(SHAPE, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, num_key_value_heads=8,
                 intermediate_size=29568, vocab_size=152064, rope_theta=1e6, max_position_embeddings=32768,
                 max_window_layers=70)
SHAPES = {"1.5b": ("qwen2-1.5b-shape", SHAPE), "7b": ("qwen2-7b-shape", SHAPE_7B), "72b": ("qwen2.5-72b-shape", SHAPE_72B)}
HBM_PEAK = 8.0e12            # bytes/s, MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense matrix peaks


def model_numbers(cfg, layers):
    H, nh, nkv, hd, I, V = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                            cfg["intermediate_size"], cfg["vocab_size"])
    qkv = (nh + 2 * nkv) * hd
    per_layer_params = qkv * H + qkv + nh * hd * H + 2 * I * H + H * I + 2 * H
    weight_bytes = 2 * (layers * per_layer_params + V * H + H)        # matrices, biases, gains, head; bf16
    kv_bytes_per_token = layers * 2 * nkv * hd * 2
    def prefill_flops(T):
        gemm = 2 * T * layers * (qkv * H + nh * hd * H + 2 * I * H + H * I)
        attn = layers * 4 * hd * nh * T * (T + 1) // 2
        return gemm + attn + 2 * V * H
    return weight_bytes, kv_bytes_per_token, prefill_flops


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (default: all)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096, help="context length the timed decode steps end at")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    ap.add_argument("--long-context", type=int, default=None,
                    help="context of the further decode point at the headline's batch (default: 32768 in the default run "
                         "of the 1.5b shape, else none; 0: none)")
    ap.add_argument("--second-shape", default=None, choices=sorted(SHAPES) + ["none"],
                    help="shape of the further decode point at batch 64, context 4096 (default: 7b in the default run of "
                         "the 1.5b shape, else none)")
    ap.add_argument("--model-dir", default=None, help="a model folder: reused if it holds a model, else written (implies --file-weights)")
    ap.add_argument("--shape", default="1.5b", choices=sorted(SHAPES), help="layer sizes (the headline is 1.5b)")
    ap.add_argument("--no-measured-peaks", action="store_true",
                    help="leave out the box's own copy bandwidth and product rate (the fractions use the published peaks)")
    ap.add_argument("--no-engine-warmup", action="store_true",
                    help="the engine does not run its warm-up steps when it starts (for kernel profiles: fewer calls that "
                         "are not the measurement's)")
    ap.add_argument("--autotune", action="store_true",
                    help="the engine times the plans of its products before it records a step (EngineConfig.autotune)")
    ap.add_argument("--file-weights", action="store_true",
                    help="write the random weights into a model folder and load them from there, instead of drawing them "
                         "on the device (not for 72b: 145 GB)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on ONE GPU; --gpus %d is not supported" % args.gpus)
        sys.exit(2)

    import torch
    from ginfer_amd import Engine, EngineConfig, SamplingParams, config_from_dict, write_random_model

    shape_name, shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    if args.layers is None:
        args.layers = full_layers
    device_weights = args.shape == "72b" or not (args.file_weights or args.model_dir)
    cfg = dict(shape, num_hidden_layers=args.layers)
    weight_bytes, kv_per_token, prefill_flops = model_numbers(cfg, args.layers)
    if args.dtype == "float32":
        weight_bytes, kv_per_token = 2 * weight_bytes, 2 * kv_per_token
    tmp = None
    folder = args.model_dir
    if device_weights:
        folder = None
    elif folder is None or not os.path.isfile(os.path.join(folder, "config.json")):
        if folder is None:
            tmp = tempfile.TemporaryDirectory(prefix="ginfer_bench_")
            folder = tmp.name
        t0 = time.time()
        write_random_model(folder, config_from_dict(cfg), seed=0, dtype=args.dtype)
        sys.stderr.write("[bench] wrote random weights in %.0f s\n" % (time.time() - t0))

    points = sorted({int(p) for p in args.points.split(",") if p} | {args.batch})
    max_b = max(points)
    page = 16
    default_run = args.shape == "1.5b" and args.dtype == "bfloat16" and args.layers == full_layers and args.context == 4096
    long_context = args.long_context if args.long_context is not None else (32768 if default_run else 0)
    second_shape = args.second_shape or ("7b" if default_run and not args.autotune else "none")
    ctx_pages = -(-(args.context + 24) // page)
    pages = max(max_b * ctx_pages, args.batch * -(-(long_context + 24) // page)) + -(-args.prefill_tokens // page) + 8
    longest = max(args.context, args.prefill_tokens, long_context)
    # The engine itself is what is timed: requests are added, the scheduler cuts their prompts into steps and reserves
    # their pages, the runner replays recorded decode steps, the sampler picks, tokens come back to the host every step.
    engine = Engine(EngineConfig(
        model_path=folder, model_config=config_from_dict(cfg) if device_weights else None,
        random_seed=0 if device_weights else None, dtype=args.dtype,
        max_num_batched_tokens=max(2048, longest + max_b), max_num_seqs=max_b,
        max_seq_len=longest + max_b + 24, kvcache_block_size=page, num_kvcache_blocks=pages,
        enable_prefix_caching=False, warmup=not args.no_engine_warmup, autotune=args.autotune))
    g = torch.Generator().manual_seed(0)
    vocab = cfg["vocab_size"]

    def sync():
        torch.cuda.synchronize()

    first_engine = engine

    def finite(engine):
        if not bool(torch.isfinite(engine.last_logits).all()):
            sys.exit("bench.py: the step that was just timed made logits that are not finite")

    # ---- prefill: one prompt of 2,048 tokens through Engine.step, up to its first token on the host
    T = args.prefill_tokens
    times = []
    for i in range(4):
        prompt = torch.randint(0, vocab, (T,), generator=g).tolist()
        engine.add_request(prompt, SamplingParams(max_tokens=1, ignore_eos=True))
        sync()
        t0 = time.perf_counter()
        done = engine.step()
        sync()
        times.append(time.perf_counter() - t0)
        assert len(done) == 1 and len(done[0].token_ids) == 1 and not engine.has_unfinished()
        finite(engine)
    prefill_s = min(times[1:])
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops(T) / prefill_s / peak, 4)}

    # ---- decode: B requests whose prompts the engine prefills, so that the timed steps end at --context
    def decode(B, steps, warmup, context=args.context, engine=None):
        engine = engine or first_engine
        sched = engine.scheduler
        vocab = engine.runner.vocab_size
        # Requests are added one by one, each prompt running whole in one step beside a token for every request added
        # before it (steps are not launched ahead meanwhile, so it is exactly one step); a request added earlier gets a
        # shorter prompt by as many tokens as it decodes until the last one is in: all reach the same length.
        engine.config.pipeline_decode = False
        params = SamplingParams(max_tokens=steps + warmup + B + 16, ignore_eos=True)
        ids = []
        for i in range(B):
            n = context - steps - warmup - (B - 1 - i)
            ids.append(engine.add_request(torch.randint(0, vocab, (n,), generator=g).tolist(), params))
            engine.step()
        assert not sched.waiting and len(sched.running) == B and all(s.decoding and s.remaining == 1 for s in sched.running)
        engine.config.pipeline_decode = True
        ahead = engine.stats["steps_launched_ahead"]
        for _ in range(warmup):
            engine.step()
        sync()
        engine.step_log.clear()
        t0 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        sync()
        dt = (time.perf_counter() - t0) / steps
        finite(engine)
        log = list(engine.step_log)
        assert len(log) == steps and all(p == 0 and d == B for _, _, p, d in log), "a timed step was no decode step of %d" % B
        assert engine.stats["steps_launched_ahead"] - ahead >= steps, "the timed steps were not launched ahead"
        device_ms = 1e3 * sum(d for _, d, _, _ in log) / steps
        # tokens of a request in the cache after the last timed step (the step launched ahead of it included)
        cached = [engine.runner.cache.length(rid) for rid in ids]
        assert max(cached) - min(cached) <= 1 and abs(max(cached) - context) <= 2, cached
        mean_ctx = sum(cached) / float(B) - steps / 2.0
        for rid in ids:
            engine.abort(rid)
        while engine.has_unfinished():
            engine.step()
        return dt, mean_ctx, device_ms

    def measured_peaks():
        """What this box reaches with library routines, beside the published peaks that the fractions are quoted on:
        a device copy of 2 GB (bytes read + bytes written per second) and a bfloat16 product of 8192^3."""
        dev = engine.runner.device
        src = torch.empty(1 << 30, dtype=torch.int16, device=dev)
        dst = torch.empty_like(src)
        a = torch.randn(8192, 8192, device=dev).bfloat16()
        b = torch.randn(8192, 8192, device=dev).bfloat16()
        out = {}
        for name, fn, work in (("copy_GBps", lambda: dst.copy_(src), 2 * src.numel() * 2 / 1e9),
                               ("bf16_product_TFLOPs", lambda: torch.mm(a, b.t()), 2 * 8192 ** 3 / 1e12)):
            for _ in range(3):
                fn()
            sync()
            t0 = time.perf_counter()
            for _ in range(10):
                fn()
            sync()
            out[name] = round(work / ((time.perf_counter() - t0) / 10), 1)
        return out

    def hbm_frac(weights, kv_token, B, mean_ctx, dt):
        return (weights + B * mean_ctx * kv_token) / dt / HBM_PEAK

    results = {}
    for B in points:
        results[B] = decode(B, args.steps, args.warmup)
    dt, mean_ctx, device_ms = results[args.batch]
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / dt / 1e9
    more = {}
    for B in points:
        if B != args.batch:
            more["decode_b%d" % B] = round(B / results[B][0], 1)
            more["decode_b%d_hbm_frac" % B] = round(hbm_frac(weight_bytes, kv_per_token, B, results[B][1], results[B][0]), 4)
    few = min(args.steps, 20), min(args.warmup, 5)
    if long_context:
        d, ctx, _ = decode(args.batch, few[0], few[1], context=long_context)
        more["decode_b%d_ctx%d" % (args.batch, long_context)] = round(args.batch / d, 1)
        more["decode_b%d_ctx%d_hbm_frac" % (args.batch, long_context)] = round(
            hbm_frac(weight_bytes, kv_per_token, args.batch, ctx, d), 4)
    measured = None if args.no_measured_peaks else measured_peaks()
    if second_shape != "none":
        # a second engine at another shape of the same architecture, its weights drawn on the device
        del engine, first_engine
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        name2, shape2 = SHAPES[second_shape]
        w2, kv2, _ = model_numbers(shape2, shape2["num_hidden_layers"])
        B2, C2 = 64, 4096
        engine2 = Engine(EngineConfig(
            model_path=None, model_config=config_from_dict(shape2), random_seed=0, dtype=args.dtype,
            max_num_batched_tokens=C2 + B2, max_num_seqs=B2, max_seq_len=C2 + B2 + 24, kvcache_block_size=page,
            num_kvcache_blocks=B2 * -(-(C2 + 24) // page) + 8, enable_prefix_caching=False, warmup=False))
        d, ctx, _ = decode(B2, few[0], few[1], context=C2, engine=engine2)
        more["decode_b%d_%s" % (B2, second_shape)] = round(B2 / d, 1)
        more["decode_b%d_%s_hbm_frac" % (B2, second_shape)] = round(hbm_frac(w2, kv2, B2, ctx, d), 4)
    out = {
        "metric": "decode tok/s at batch %d (Qwen2 %s shape, context %d)" % (args.batch, args.shape.upper(), args.context),
        "value": round(args.batch / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "device_ms_per_step": round(device_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic tokens, random weights N(0, 0.02)",
        "config": {"model": shape_name, "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single-gpu", "layers": args.layers, "layers_full": full_layers,
                   "hidden_size": cfg["hidden_size"], "num_attention_heads": cfg["num_attention_heads"],
                   "num_key_value_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
                   "kv_page_size": page, "prefill_tokens": T},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 4)},
        "points": more,
    }
    if measured is not None:
        out["measured"] = measured
    print(json.dumps(out))
    if tmp is not None:
        tmp.cleanup()


if __name__ == "__main__":
    main()
