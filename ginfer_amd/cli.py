"""Command line of the engine, in the manner of the reference's test_engine binary
(ginfer/test/test_engine.cc:14-111): the model folder comes from --model-path or the MODEL_PATH
environment variable, the engine settings carry the names of its `engine::Config` fields
(ginfer/engine/config.h:8-21) and the sampling settings those of `SamplingParams`
(ginfer/engine/sampling_params.h:5-8).  There is no tokenizer: prompts are token ids.

    python -m ginfer_amd generate  --model-path DIR --prompt-ids 1,2,3 --prompt-ids 4,5 --max-tokens 16
    python -m ginfer_amd benchmark --model-path DIR --num-prompts 256 --prompt-len 512 --max-tokens 128
    python -m ginfer_amd benchmark --random-config C.json --num-prompts 64 --prompt-len-min 128 --prompt-len-max 2048 \
                                   --max-tokens 256 --max-num-batched-tokens 2048 --max-num-seqs 64
    python -m ginfer_amd random-weights --config config.json --seed 0 --out DIR
    python -m ginfer_amd generate  --random-config config.json --prompt-ids 1,2,3      (weights drawn on the device)
"""
import argparse
import json
import os
import random
import sys
import time


def _engine_args(p):
    p.add_argument("--model-path", default=os.environ.get("MODEL_PATH"),
                   help="folder with config.json and model.safetensors (default: $MODEL_PATH)")
    p.add_argument("--random-config", default=None, metavar="CONFIG.json",
                   help="instead of a model folder: a config.json whose weights are drawn on the device")
    p.add_argument("--weights-seed", type=int, default=0, help="seed of the weights drawn for --random-config")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"],
                   help="bfloat16: the serving kernels; float32: everything in true 32-bit")
    p.add_argument("--max-num-batched-tokens", type=int, default=2048, help="token budget of one step")
    p.add_argument("--max-num-seqs", type=int, default=64, help="requests running at a time")
    p.add_argument("--max-seq-len", type=int, default=4096, help="longest sequence (prompt + output)")
    p.add_argument("--gpu-memory-utilization", type=float, default=0.9,
                   help="share of the free device memory that becomes cache pages")
    p.add_argument("--kvcache-block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--num-kvcache-blocks", type=int, default=None, help="cache pages (default: from free memory)")
    p.add_argument("--max-tokens", type=int, default=64, help="output tokens per request")
    p.add_argument("--ignore-eos", action="store_true", help="do not stop at an end-of-sequence token")
    p.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    p.add_argument("--seed", type=int, default=0, help="seed of the sampler's random stream")
    p.add_argument("--no-pipeline-decode", action="store_true",
                   help="read every step's tokens before the next step is launched")
    p.add_argument("--no-graph-mixed-steps", action="store_true",
                   help="steps with prompt portions are launched kernel by kernel, never replayed from a recording")
    p.add_argument("--strict-weights", action="store_true",
                   help="a tensor in the model folder that the model does not read is an error, not a warning")
    p.add_argument("--autotune", action="store_true",
                   help="time the plans of a step's products on this model's weights before the step is recorded, and "
                        "keep the fastest (a second or so per number of rows, once)")
    p.add_argument("--no-prefix-caching", action="store_true",
                   help="requests do not share the cache pages of a common prefix")


def _engine(args):
    from . import Engine, EngineConfig, config_from_dict
    model_config = None
    if args.random_config:
        with open(args.random_config) as f:
            model_config = config_from_dict(json.load(f))
        args.model_path = None
    elif not args.model_path:
        sys.exit("no model: give --model-path, set MODEL_PATH, or give --random-config")
    return Engine(EngineConfig(
        model_path=args.model_path, model_config=model_config,
        random_seed=args.weights_seed if model_config is not None else None, dtype=args.dtype, max_num_batched_tokens=args.max_num_batched_tokens,
        max_num_seqs=args.max_num_seqs, max_seq_len=args.max_seq_len,
        gpu_memory_utilization=args.gpu_memory_utilization, kvcache_block_size=args.kvcache_block_size,
        num_kvcache_blocks=args.num_kvcache_blocks, pipeline_decode=not args.no_pipeline_decode,
        graph_mixed_steps=not args.no_graph_mixed_steps, strict_weights=args.strict_weights, autotune=args.autotune,
        enable_prefix_caching=False if args.no_prefix_caching else None))


def _params(args, n):
    from . import SamplingParams
    return [SamplingParams(max_tokens=args.max_tokens, ignore_eos=args.ignore_eos, temperature=args.temperature,
                           seed=args.seed + i) for i in range(n)]


def _report(engine, outs, wall):
    st = engine.stats
    for o in outs:
        sys.stderr.write("request %d: prompt_tokens=%d output_tokens=%d finish=%s ttft=%.2f ms tpot=%s evictions=%d\n" % (
            o.request_id, len(o.prompt_token_ids), len(o.token_ids), o.finish_reason, (o.ttft or 0) * 1e3,
            "%.3f ms" % (o.tpot * 1e3) if o.tpot else "-", o.evictions))
    pf = st["prefill_tokens"] / st["prefill_time"] if st["prefill_time"] else 0.0
    dc = st["decode_tokens"] / st["decode_time"] if st["decode_time"] else 0.0
    shared = engine.runner.cache.prefix_hit_tokens
    sys.stderr.write("steps=%d (launched ahead: %d) prefill=%.1f tok/s decode=%.1f tok/s wall=%.3f s evictions=%d "
                     "prompt tokens found in the cache=%d\n"
                     % (st["steps"], st["steps_launched_ahead"], pf, dc, wall, engine.scheduler.num_evictions, shared))
    sys.stderr.write("how the steps ran: %s\n" % engine.runner.counts)
    return dict(steps=st["steps"], steps_launched_ahead=st["steps_launched_ahead"], prefill_tok_s=pf, decode_tok_s=dc,
                wall_s=wall, prefix_hit_tokens=shared, ran=dict(engine.runner.counts))


def cmd_generate(args):
    prompts = [[int(t) for t in p.replace(",", " ").split()] for p in args.prompt_ids or []]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            for line in f:
                line = line.strip()
                if line:
                    prompts.append(json.loads(line) if line.startswith("[") else [int(t) for t in line.replace(",", " ").split()])
    if not prompts:
        sys.exit("no prompts: give --prompt-ids 1,2,3 (repeatable) or --prompt-file FILE (one list of ids a line)")
    engine = _engine(args)
    t0 = time.perf_counter()
    outs = engine.generate(prompts, _params(args, len(prompts)))
    _report(engine, outs, time.perf_counter() - t0)
    for o in outs:
        print(json.dumps({"request_id": o.request_id, "token_ids": o.token_ids, "finish_reason": o.finish_reason}))


def cmd_benchmark(args):
    """The reference's EngineTest.Benchmark (ginfer/test/test_engine.cc:57-111): random prompts of one
    length (or of lengths drawn from a range), a warm-up generate, then the timed one.  Reports output and total
    tokens a second, times to the first and per further token, and every step's wall time beside the device's own
    time for it (mean, median, 99th percentile, histogram)."""
    engine = _engine(args)
    rng = random.Random(0)
    vocab = min(engine.runner.vocab_size, 10001)
    lo = args.prompt_len if args.prompt_len_min is None else args.prompt_len_min
    hi = args.prompt_len if args.prompt_len_max is None else args.prompt_len_max
    if not 1 <= lo <= hi:
        sys.exit("prompt lengths must satisfy 1 <= --prompt-len-min <= --prompt-len-max")
    prompts = [[rng.randrange(vocab) for _ in range(rng.randint(lo, hi))] for _ in range(args.num_prompts)]
    args.ignore_eos = True
    # the warm-up has prompts of its own: the timed run finds nothing of its prompts in the cache
    engine.generate([[rng.randrange(vocab) for _ in range(hi)] for _ in range(2)], _params(args, 2))
    for k in engine.stats:
        engine.stats[k] = 0 if isinstance(engine.stats[k], int) else 0.0
    engine.step_log.clear()
    t0 = time.perf_counter()
    if args.request_rate > 0:
        outs = _generate_as_they_arrive(engine, prompts, _params(args, len(prompts)), args.request_rate, rng)
    else:
        outs = engine.generate(prompts, _params(args, len(prompts)))
    wall = time.perf_counter() - t0
    rep = _report(engine, [], wall)
    total = sum(len(o.prompt_token_ids) + len(o.token_ids) for o in outs)
    rep.update(total_tokens=total, total_tok_s=total / wall, output_tok_s=sum(len(o.token_ids) for o in outs) / wall)
    log = engine.step_log
    rep.update(prompt_tokens=sum(len(p) for p in prompts), prompt_len_min=lo, prompt_len_max=hi,
               device_s=round(sum(d for _, d, _, _ in log), 4))
    for name, values in (("ttft_ms", [o.ttft * 1e3 for o in outs if o.ttft is not None]),
                         ("tpot_ms", [o.tpot * 1e3 for o in outs if o.tpot is not None]),
                         ("step_wall_ms", [w * 1e3 for w, _, _, _ in log]),
                         ("step_device_ms", [d * 1e3 for _, d, _, _ in log]),
                         ("decode_step_wall_ms", [w * 1e3 for w, _, p, d in log if p == 0 and d > 0]),
                         ("decode_step_device_ms", [dv * 1e3 for _, dv, p, d in log if p == 0 and d > 0])):
        values.sort()
        if values:
            rep[name] = dict(mean=round(sum(values) / len(values), 3), p50=round(values[len(values) // 2], 3),
                             p99=round(values[min(len(values) - 1, int(len(values) * 0.99))], 3))
    rep["step_wall_ms_histogram"] = _histogram([w * 1e3 for w, _, _, _ in log])
    rep["step_device_ms_histogram"] = _histogram([d * 1e3 for _, d, _, _ in log])
    print(json.dumps(rep))


def _histogram(values_ms):
    """Counts of steps by time, in bins that double: "<0.5", "0.5-1", "1-2", ... ">=256" (milliseconds)."""
    edges = [0.5 * 2 ** k for k in range(10)]
    names = ["<0.5"] + ["%g-%g" % (a, b) for a, b in zip(edges[:-1], edges[1:])] + [">=%g" % edges[-1]]
    counts = [0] * len(names)
    for v in values_ms:
        k = 0
        while k < len(edges) and v >= edges[k]:
            k += 1
        counts[k] += 1
    return {n: c for n, c in zip(names, counts) if c}


def _generate_as_they_arrive(engine, prompts, params, rate, rng):
    """Requests arrive one by one, `rate` a second on average (exponential gaps from the seeded generator), while
    the engine steps: what a request waits for its first token and for every further one then depends on what
    else is running, as in serving."""
    arrivals, t = [], 0.0
    for _ in prompts:
        t += rng.expovariate(rate)
        arrivals.append(t)
    start = time.perf_counter()
    ids, done, nxt = [], {}, 0
    while nxt < len(prompts) or engine.has_unfinished():
        now = time.perf_counter() - start
        while nxt < len(prompts) and arrivals[nxt] <= now:
            ids.append(engine.add_request(prompts[nxt], params[nxt]))
            nxt += 1
        if engine.has_unfinished():
            for out in engine.step():
                done[out.request_id] = out
        else:
            time.sleep(max(0.0, min(arrivals[nxt] - now, 0.001)))
    return [done[i] for i in ids]


def cmd_random_weights(args):
    from . import config_from_dict, write_random_model
    with open(args.config) as f:
        cfg = config_from_dict(json.load(f))
    write_random_model(args.out, cfg, args.seed, args.storage_dtype)
    print(args.out)


def main(argv=None):
    ap = argparse.ArgumentParser(prog="ginfer_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="generate token ids for prompts given as token ids")
    _engine_args(g)
    g.add_argument("--prompt-ids", action="append", help="one prompt as comma-separated token ids (repeatable)")
    g.add_argument("--prompt-file", help="file with one prompt a line (JSON list or comma-separated ids)")
    g.set_defaults(fn=cmd_generate)
    b = sub.add_parser("benchmark", help="throughput with random prompts")
    _engine_args(b)
    b.add_argument("--num-prompts", type=int, default=256)
    b.add_argument("--prompt-len", type=int, default=512)
    b.add_argument("--prompt-len-min", type=int, default=None,
                   help="with --prompt-len-max: prompt lengths drawn uniformly from this range (default: all --prompt-len)")
    b.add_argument("--prompt-len-max", type=int, default=None)
    b.add_argument("--request-rate", type=float, default=0.0,
                   help="requests a second arriving while the engine runs (0: all at once, the reference's benchmark)")
    b.set_defaults(fn=cmd_benchmark, max_num_batched_tokens=16384, max_num_seqs=256, max_tokens=128)
    r = sub.add_parser("random-weights", help="write a model folder with random weights")
    r.add_argument("--config", required=True, help="a config.json of a registered architecture")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True)
    r.add_argument("--storage-dtype", default="bfloat16", choices=["bfloat16", "float32", "float16"])
    r.set_defaults(fn=cmd_random_weights)
    args = ap.parse_args(argv)
    args.fn(args)


if __name__ == "__main__":
    main()
