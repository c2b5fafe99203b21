#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen2 1.5B shape (random bfloat16 weights, synthetic tokens)
on one MI355X, with the achieved fraction of the HBM and matrix-core rooflines.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

A step is one decode step of the engine's own step function plus sampling: every request of the batch
gets one token, from the paged cache, and its next token comes back to the host; as in the engine, the next
step is launched before this step's tokens have been waited for.  Prints ONE JSON line.
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
    ap.add_argument("--model-dir", default=None, help="a model folder: reused if it holds a model, else written (implies --file-weights)")
    ap.add_argument("--shape", default="1.5b", choices=sorted(SHAPES), help="layer sizes (the headline is 1.5b)")
    ap.add_argument("--no-measured-peaks", action="store_true",
                    help="leave out the box's own copy bandwidth and product rate (the fractions use the published peaks)")
    ap.add_argument("--file-weights", action="store_true",
                    help="write the random weights into a model folder and load them from there, instead of drawing them "
                         "on the device (not for 72b: 145 GB)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on ONE GPU; --gpus %d is not supported" % args.gpus)
        sys.exit(2)

    import torch
    from ginfer_amd import ModelRunner, StepEntry, config_from_dict, write_random_model
    from ginfer_amd.sampling import Sampler, SamplingParams

    shape_name, shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    if args.layers is None:
        args.layers = full_layers
    device_weights = args.shape == "72b" or not (args.file_weights or args.model_dir)
    cfg = dict(shape, num_hidden_layers=args.layers)
    weight_bytes, kv_per_token, prefill_flops = model_numbers(cfg, args.layers)
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
    ctx_pages = -(-(args.context + 1) // page)
    pages = max_b * ctx_pages + -(-args.prefill_tokens // page) + 8
    runner = ModelRunner(folder, dtype=args.dtype, page_size=page, num_pages=pages, max_requests=max_b + 1,
                         max_model_len=max(args.context, args.prefill_tokens) + 8,
                         config=config_from_dict(cfg) if device_weights else None,
                         random_seed=0 if device_weights else None)
    sampler = Sampler(runner.device)
    g = torch.Generator().manual_seed(0)
    vocab = cfg["vocab_size"]

    def sync():
        torch.cuda.synchronize()

    # ---- prefill: one prompt of 2,048 tokens, the logits of its last place
    T = args.prefill_tokens
    prompt = torch.randint(0, vocab, (T,), generator=g).tolist()
    times = []
    for i in range(4):
        sync()
        t0 = time.perf_counter()
        logits = runner.step([StepEntry("p", prompt, [T - 1])])
        sampler.sample(logits, [SamplingParams()], [0])
        sync()
        times.append(time.perf_counter() - t0)
        runner.release("p")
    prefill_s = min(times[1:])
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops(T) / prefill_s / peak, 4)}

    # ---- decode: B requests whose caches hold a context that ends at --context after the timed steps
    def decode(B, steps, warmup):
        start = args.context - steps - warmup
        for b in range(B):
            runner.cache.admit(("d", b))
            runner.cache.append(("d", b), start)
            runner.cache.commit(("d", b))
        for grp in runner.cache.groups:      # synthetic keys and values stand in for a prefilled context
            grp.tensor.normal_(0.0, 1.0, generator=None)
        tokens = torch.randint(0, vocab, (B,), generator=g).tolist()
        params = [SamplingParams() for _ in range(B)]

        ring = [(torch.empty(B, dtype=torch.int32, pin_memory=True), torch.cuda.Event()) for _ in range(3)]
        at = [0]

        def launch(tokens=None, device_tokens=None):
            """One step handed to the device: model, sampling, and the tokens' copy to the host behind it."""
            ids = tokens if tokens is not None else [0] * B
            logits = runner.step([StepEntry(("d", b), [ids[b]], [0]) for b in range(B)], borrow=True,
                                 device_tokens=device_tokens)
            dev = sampler.sample_on_device(logits, params, [0] * B)
            host, event = ring[at[0] % len(ring)]
            at[0] += 1
            host.copy_(dev, non_blocking=True)
            event.record()
            return dev, host, event

        def run(n, tokens):
            """n steps, as the engine drives them: the next step is launched (its ids taken on the device) before
            this step's tokens, which come to the host every step, have been waited for."""
            if n <= 0:
                return tokens
            cur = launch(tokens=tokens)
            for _ in range(n - 1):
                nxt = launch(device_tokens=cur[0])
                cur[2].synchronize()
                tokens = cur[1].tolist()
                cur = nxt
            cur[2].synchronize()
            return cur[1].tolist()
        tokens = run(warmup, tokens)
        sync()
        t0 = time.perf_counter()
        tokens = run(steps, tokens)
        sync()
        dt = (time.perf_counter() - t0) / steps
        mean_ctx = args.context - steps / 2.0
        for b in range(B):
            runner.release(("d", b))
        return dt, mean_ctx

    def measured_peaks():
        """What this box reaches with library routines, beside the published peaks that the fractions are quoted on:
        a device copy of 2 GB (bytes read + bytes written per second) and a bfloat16 product of 8192^3."""
        src = torch.empty(1 << 30, dtype=torch.int16, device=runner.device)
        dst = torch.empty_like(src)
        a = torch.randn(8192, 8192, device=runner.device).bfloat16()
        b = torch.randn(8192, 8192, device=runner.device).bfloat16()
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

    results = {}
    for B in points:
        results[B] = decode(B, args.steps, args.warmup)
    dt, mean_ctx = results[args.batch]
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / dt / 1e9
    out = {
        "metric": "decode tok/s at batch %d (Qwen2 %s shape, context %d)" % (args.batch, args.shape.upper(), args.context),
        "value": round(args.batch / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
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
        "points": {"decode_b%d" % B: round(B / results[B][0], 1) for B in points if B != args.batch},
    }
    if not args.no_measured_peaks:
        out["measured"] = measured_peaks()
    print(json.dumps(out))
    if tmp is not None:
        tmp.cleanup()


if __name__ == "__main__":
    main()
