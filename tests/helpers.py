"""Shared by the tests: tiny configurations, model folders, traces and the comparison with the plain
implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import torch

import plain_model as pm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Three tiny configurations of the architecture that differ in every size and option.
TINY_A = dict(  # groups of 2, head 16, tied head, no window
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=2, hidden_size=64,
    num_attention_heads=4, num_key_value_heads=2, intermediate_size=160, vocab_size=512, rope_theta=10000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=256, use_sliding_window=False,
    sliding_window=4096, max_window_layers=2, eos_token_id=511)
TINY_B = dict(  # one kv head for 6 heads, head 32, separate head, other theta and eps
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=3, hidden_size=192,
    num_attention_heads=6, num_key_value_heads=1, intermediate_size=448, vocab_size=1000, rope_theta=1e6,
    rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=512, use_sliding_window=False,
    eos_token_id=[998, 999])
TINY_C = dict(  # explicit head_dim 48 with nh*hd != hidden, widths no power of two, windows on layers >= 1
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=4, hidden_size=88,
    num_attention_heads=6, num_key_value_heads=3, head_dim=48, intermediate_size=136, vocab_size=777,
    rope_theta=5e5, rms_norm_eps=3e-6, tie_word_embeddings=False, max_position_embeddings=384,
    use_sliding_window=True, sliding_window=40, max_window_layers=1, eos_token_id=5)
# how the checkpoints of this family of models spell the parts' tensor prefixes (the plain implementation reads these names;
# the toy architectures of the tests spell theirs alike)
LAYER_NAMES = dict(mixer="self_attn", feed_forward="mlp", mixer_norm="input_layernorm",
                   feed_forward_norm="post_attention_layernorm")
MODEL_NAMES = dict(embedding="model.embed_tokens", final_norm="model.norm", head="lm_head")
TINY = {"A": (TINY_A, 0, 16), "B": (TINY_B, 1, 8), "C": (TINY_C, 2, 16)}   # config, seed, page size


def make_model_folder(folder, config_dict, seed, dtype="float32", std_scale=1.0):
    from ginfer_amd import config_from_dict, write_random_model
    return write_random_model(str(folder), config_from_dict(config_dict), seed, dtype, std_scale=std_scale)


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def plain_logits(folder, ids, dtype=torch.float64):
    cfg = pm.read_config(folder)
    w = pm.read_weights(folder, dtype)
    return pm.forward(cfg, w, ids).to(torch.float32).numpy()


def rel_err(got, ref):
    """Largest absolute difference over the largest absolute reference value."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), "non-finite values in the result"
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


# tolerances (largest difference over the largest reference value), fixed once: 32-bit differs from the
# 64-bit plain implementation by the rounding of sums of a few hundred terms (measured: under 1e-6);
# bfloat16 rounds every stored activation to 8 bits a few dozen times (measured: under 1e-2; 2e-2 is the
# reference's own tolerance for one bfloat16 attention, python/test/test_op.py:124-154).
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


# ----------------------------------------------------------------------------- traces

def steps_whole(requests):
    """Each request alone and whole, every place wanted."""
    steps = []
    for rid, ids in requests.items():
        steps.append(dict(entries=[dict(id=rid, tokens=ids, want=list(range(len(ids))))], end=[rid]))
    return steps


def steps_last_decoded(requests, last=32):
    """Most of a request in one step, the last `last` tokens one by one."""
    steps = []
    for rid, ids in requests.items():
        n = max(len(ids) - last, 1)
        steps.append(dict(entries=[dict(id=rid, tokens=ids[:n], want=list(range(n)))], end=[]))
        for i in range(n, len(ids)):
            steps.append(dict(entries=[dict(id=rid, tokens=ids[i:i + 1], want=[0])],
                              end=[rid] if i == len(ids) - 1 else []))
        if n == len(ids):
            steps[-1]["end"] = [rid]
    return steps


def cut(n, sizes):
    """Cuts n tokens into portions of the given sizes, cycling."""
    out, i, k = [], 0, 0
    while i < n:
        s = min(sizes[k % len(sizes)], n - i)
        out.append((i, i + s))
        i += s
        k += 1
    return out


def steps_portions(requests, sizes=(7, 2, 33, 3, 16, 2, 64, 5)):
    steps = []
    for rid, ids in requests.items():
        parts = cut(len(ids), sizes)
        for j, (a, b) in enumerate(parts):
            steps.append(dict(entries=[dict(id=rid, tokens=ids[a:b], want=list(range(b - a)))],
                              end=[rid] if j == len(parts) - 1 else []))
    return steps


def steps_mixed(requests, max_live=4, seed=0, prompt_fraction=0.6):
    """Up to max_live requests at a time: each is fed its first part in portions of changing size and
    the rest token by token, so portions of some run beside decoded tokens of others; a request may
    sit a step out; when one ends the next starts and takes over its pages."""
    rng = np.random.RandomState(seed)
    order = list(requests)
    live, done_upto = [], {}
    steps = []
    nxt = 0
    while nxt < len(order) or live:
        while len(live) < max_live and nxt < len(order):
            live.append(order[nxt])
            done_upto[order[nxt]] = 0
            nxt += 1
        entries, end = [], []
        for rid in list(live):
            ids = requests[rid]
            if len(live) > 1 and rng.rand() < 0.15:
                continue                                  # sits this step out
            at = done_upto[rid]
            if at < int(len(ids) * prompt_fraction):
                n = int(rng.choice([2, 3, 5, 8, 13, 21, 34]))
                n = min(n, len(ids) - at)
            else:
                n = 1
            entries.append(dict(id=rid, tokens=ids[at:at + n], want=list(range(n))))
            done_upto[rid] = at + n
            if at + n == len(ids):
                end.append(rid)
                live.remove(rid)
        if entries:
            steps.append(dict(entries=entries, end=end))
    return steps


def max_live_tokens(steps, round_to=64):
    """The most tokens live requests hold at any time, each request's count rounded up."""
    held, best = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        best = max(best, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return best


def run_steps(runner, steps):
    """Drives a ModelRunner directly.  Returns {(request, position): logits row}."""
    from ginfer_amd import StepEntry
    at, out = {}, {}
    for st in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]
        logits = runner.step(entries).cpu().numpy()
        r = 0
        for e in st["entries"]:
            base = at.get(e["id"], 0)
            for w in e["want"]:
                out[(e["id"], base + w)] = logits[r]
                r += 1
            at[e["id"]] = base + len(e["tokens"])
        assert r == logits.shape[0]
        for rid in st["end"]:
            runner.release(rid)
            at.pop(rid, None)
    return out


def run_trace(model_folder, dtype, steps, out_dir, max_tokens, page_size=16, timeout=600, seed=None):
    """Drives bin/trace_run as a user would: a subprocess, steps on stdin one at a time, each sent
    only after the previous `done`.  Returns {(request, position): logits row}.  With a seed the program gets the
    folder's config.json and the seed instead of the folder, and draws the weights itself."""
    model = ["--model", str(model_folder)] if seed is None else \
        ["--config", os.path.join(str(model_folder), "config.json"), "--seed", str(seed)]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run")] + model + [
        "--dtype", dtype, "--out", str(out_dir), "--max-tokens", str(max_tokens), "--page-size", str(page_size)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    at, out = {}, {}
    vocab = pm.read_config(model_folder)["vocab_size"]
    try:
        for i, st in enumerate(steps):
            proc.stdin.write(json.dumps(dict(step=i, entries=st["entries"], end=st["end"])) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            assert line.strip() == "done %d" % i, "trace_run answered %r to step %d" % (line, i)
            wanted = sum(len(e["want"]) for e in st["entries"])
            path = os.path.join(str(out_dir), "%d.f32" % i)
            if wanted:
                a = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
                r = 0
                for e in st["entries"]:
                    base = at.get(e["id"], 0)
                    for w in e["want"]:
                        out[(e["id"], base + w)] = a[r]
                        r += 1
            else:
                assert not os.path.exists(path)
            for e in st["entries"]:
                at[e["id"]] = at.get(e["id"], 0) + len(e["tokens"])
            for rid in st["end"]:
                at.pop(rid, None)
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    return out


def compare_with_plain(got, requests, model_folder, tol, what=""):
    """got: {(request, position): row}.  Every row is compared with the plain implementation run on the
    bare token list; the first wrong place is named."""
    refs = {rid: plain_logits(model_folder, ids) for rid, ids in requests.items()}
    worst = 0.0
    for (rid, p), row in sorted(got.items(), key=lambda kv: (str(kv[0][0]), kv[0][1])):
        scale = np.abs(refs[rid]).max()
        err = float(np.abs(row.astype(np.float64) - refs[rid][p]).max() / scale)
        assert np.isfinite(row).all(), "%s: request %r position %d: non-finite logits" % (what, rid, p)
        assert err <= tol, ("%s: first wrong place is request %r position %d of %d: error %.3g > %.3g"
                            % (what, rid, p, len(requests[rid]), err, tol))
        worst = max(worst, err)
    for rid, ids in requests.items():
        missing = [p for p in range(len(ids)) if (rid, p) not in got]
        assert not missing, "%s: request %r lacks logits at %s" % (what, rid, missing[:8])
    return worst
