"""The sizes that the measurements are quoted on, checked against the plain implementation: the matrix-core
attention kernels at the benchmark's head layouts, prompt lengths and contexts (2,048- and 8,192-token prompts,
single tokens over 4,096, 32,768 and 131,072 keys, 8 and 64 requests side by side), and two layers of the 1.5B shape
with a 2,048-token prompt through the engine's step function, whole, in portions and followed by single tokens.
Shapes as the reference's paged-attention tests build them (python/test/test_page_attn.py:62-181), at other sizes."""
import math

import numpy as np
import pytest
import torch

import helpers as H
import plain_model as pm

pytestmark = pytest.mark.gpu
NAN = float("nan")


def dev():
    return torch.device("cuda:0")


class _Step:
    """The fields of a step that the attention dispatcher reads; `decode_span` as the runner sets it."""

    def __init__(self, seqs, a, span):
        self.num_entries = len(seqs)
        self.host_q_len = [q for q, _ in seqs]
        self.host_q_start = [kv - q for q, kv in seqs]
        self.token_entry, self.positions = a["token_entry"], a["positions"]
        self.extra = {"decode_span": span}


def _rows_to_check(q_len, g):
    """Rows of a portion whose plain result is computed: all of a short one; of a long one its first and last rows,
    the rows around the edges of the kernels' tiles, and some drawn at random."""
    if q_len <= 48:
        return list(range(q_len))
    rows = {0, 1, 2, q_len - 3, q_len - 2, q_len - 1}
    for edge in (16, 32, 64, 256, q_len // 2 // 64 * 64):
        rows.update(r for r in (edge - 1, edge, edge + 1) if 0 <= r < q_len)
    rows.update(torch.randint(0, q_len, (24,), generator=g).tolist())
    return sorted(rows)


def _large_case(seqs, nh, nkv, hd, ps, seed, spike_at):
    """As the kernel tests' paged case, built without a loop over keys: pages in random order, unused slots NaN, bfloat16
    operands.  spike_at(entry, q_len, kv_len) -> key whose score for the entry's LAST query stands out (or None).
    Returns operands on the device and, per entry, (rows of the step, plain rows, whether the last row has a spike)."""
    g = torch.Generator().manual_seed(seed)
    blocks = [-(-kv // ps) for _, kv in seqs]
    num_pages = sum(blocks) + 3
    perm = torch.randperm(num_pages, generator=g)
    width = max(blocks) + 1
    bt = torch.full((len(seqs), width), -1, dtype=torch.int32)
    kp = torch.full((num_pages, nkv, ps, hd), NAN, dtype=torch.bfloat16)
    vp = torch.full((num_pages, nkv, hd, ps), NAN, dtype=torch.bfloat16)
    T = sum(q for q, _ in seqs)
    q = torch.randn((T, nh, hd), generator=g)
    ent, pos, checks = [], [], []
    o = page_at = 0
    for e, (ql, kv) in enumerate(seqs):
        k = torch.randn((kv, nkv, hd), generator=g)
        v = torch.randn((kv, nkv, hd), generator=g)
        c = spike_at(e, ql, kv)
        if c is not None:
            k[c] = 0
            k[c, :, 0] = 40.0
            q[o + ql - 1] = 0
            q[o + ql - 1, :, 0] = math.sqrt(hd)           # score 40 at key c, about N(0, 1) at the others
            v[c] = 7.0
        k, v = k.bfloat16(), v.bfloat16()
        pages = perm[page_at:page_at + blocks[e]]
        page_at += blocks[e]
        bt[e, :blocks[e]] = pages.to(torch.int32)
        pad = blocks[e] * ps - kv
        fill = torch.full((pad, nkv, hd), NAN, dtype=torch.bfloat16)
        kp[pages] = torch.cat([k, fill]).view(blocks[e], ps, nkv, hd).permute(0, 2, 1, 3)
        vp[pages] = torch.cat([v, fill]).view(blocks[e], ps, nkv, hd).permute(0, 2, 3, 1)
        rows = _rows_to_check(ql, g)
        qe = q[o:o + ql].bfloat16()[rows].double()
        ref = pm.attention(qe, k.double(), v.double(), [kv - ql + r for r in rows])
        checks.append(([o + r for r in rows], ref.reshape(len(rows), nh * hd), c is not None))
        ent += [e] * ql
        pos += list(range(kv - ql, kv))
        o += ql
    d = dev()
    a = dict(q=q.bfloat16().reshape(T, nh * hd).to(d), k_pages=kp.to(d), v_pages=vp.to(d), block_table=bt.to(d),
             token_entry=torch.tensor(ent, dtype=torch.int32, device=d), positions=torch.tensor(pos, dtype=torch.int32, device=d))
    return a, checks


def _span(seqs):
    from ginfer_amd.engine.runner import _context_bucket
    return _context_bucket(max(kv for _, kv in seqs))


def _edge_of_the_last_split(seqs, nh, nkv):
    """The key at which the last of a single token's key splits begins, as the dispatcher cuts them for this step."""
    from ginfer_amd.kernels import ops
    n_decode = sum(1 for q, _ in seqs if q == 1)
    if not n_decode:
        return None
    split_keys, _ = ops._decode_splits(dict(decode_span=_span(seqs), n_decode=n_decode), 0, nkv, -(-(nh // nkv) // 16))
    return split_keys


BENCH_HEADS = (12, 2, 128)
CASES = [
    ("prompt of 2,048", BENCH_HEADS, [(2048, 2048)]),
    ("portion of 512 beside 8 single tokens", BENCH_HEADS, [(512, 2048)] + [(1, 4096 - 3 * i) for i in range(8)]),
    ("8 single tokens at 4,096", BENCH_HEADS, [(1, 4096 - i) for i in range(8)]),
    ("64 single tokens at 4,096", BENCH_HEADS, [(1, 4096 - (i % 7)) for i in range(64)]),
    ("one single token at 4,096", BENCH_HEADS, [(1, 4096)]),
    ("single token at 32,768", BENCH_HEADS, [(1, 32768)]),
    ("single token at 131,072", BENCH_HEADS, [(1, 131072)]),
    ("prompt of 8,192", BENCH_HEADS, [(8192, 8192)]),
    ("7B heads, prompt of 2,048", (28, 4, 128), [(2048, 2048)]),
    ("7B heads, 4 single tokens at 4,096", (28, 4, 128), [(1, 4096 - i) for i in range(4)]),
    ("72B heads, prompt of 2,048", (64, 8, 128), [(2048, 2048)]),
    ("72B heads, 4 single tokens at 4,096", (64, 8, 128), [(1, 4096 - i) for i in range(4)]),
]


# a single token with a far key says whether that key is read, one without says how well thousands of keys are summed:
# every third single token of a batch has none, and the steps of one single token run both ways
RUNS = [(what, heads, seqs, True) for what, heads, seqs in CASES]
RUNS += [(what + ", random keys only", heads, seqs, False) for what, heads, seqs in CASES
         if sum(1 for q, _ in seqs if q == 1) in (1, 2)]


@pytest.mark.parametrize("what,heads,seqs,far_keys", RUNS, ids=[r[0] for r in RUNS])
def test_matrix_core_attention_at_the_measured_sizes(what, heads, seqs, far_keys):
    from ginfer_amd.kernels import ops
    nh, nkv, hd = heads
    split_keys = _edge_of_the_last_split(seqs, nh, nkv)

    def spike_at(e, ql, kv):
        if not far_keys:
            return None
        if ql == 1:      # the first key of the last split, or (every other request) the last key of the split before
            if e % 3 == 2:
                return None
            edge = (kv - 1) // split_keys * split_keys
            return max(edge - (e % 2), 0)
        return kv // 2 // 64 * 64 - (e % 2)      # a far key at the edge of a tile of keys
    a, checks = _large_case(seqs, nh, nkv, hd, 16, seed=len(seqs) + nh, spike_at=spike_at)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a, _span(seqs)), nh,
                                   nkv, hd, 1.0 / math.sqrt(hd)).float().cpu()
    assert torch.isfinite(out).all(), what
    for e, (rows, ref, spiked) in enumerate(checks):
        got = out[rows].double()
        if spiked:       # the last row's weight lies on one far key: its value comes out iff the kernel reads that key
            assert (got[-1] - 7.0).abs().max() < 0.1, "%s: entry %d does not find its far key" % (what, e)
            assert (got[-1] - ref[-1]).abs().max() <= 2e-2 * 7
            got, ref = got[:-1], ref[:-1]
        if len(ref):
            err = (got - ref).abs().max().item() / ref.abs().max().item()
            assert err <= 2e-2, "%s: entry %d: error %.3g" % (what, e, err)


def test_a_prompt_of_2048_tokens_through_two_layers_of_the_1_5b_shape(tmp_path):
    """The headline prefill's own path (wide tiles, keys and values shared through LDS, the gate-up product with the
    weights first) and the hand-over to single tokens at a context of 2,048, against the plain model; in 32-bit the
    three cuttings agree to the bit."""
    from ginfer_amd import ModelRunner
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=1536, num_attention_heads=12,
               num_key_value_heads=2, intermediate_size=8960, vocab_size=151936, rope_theta=10000.0, rms_norm_eps=1e-6,
               tie_word_embeddings=False, max_position_embeddings=4096, use_sliding_window=False, sliding_window=4096,
               max_window_layers=21)
    folder = H.make_model_folder(tmp_path / "real", cfg, 4, "float32")
    # With draws of N(0, 0.02) a query weighs its 2,048 keys nearly alike, so the attention's output is a small mean of
    # values, a thirtieth of what the feed-forward adds to the residual stream: a fault in it would hide in the
    # tolerance.  The output projection is made 16 times as large, which puts the two on a par.
    from safetensors.torch import load_file, save_file
    path = str(tmp_path / "real" / "model.safetensors")
    tensors = load_file(path)
    for name in tensors:
        if name.endswith("o_proj.weight"):
            tensors[name] = tensors[name] * 16.0
    save_file(tensors, path)
    del tensors
    P, D = 2048, 32
    ids = H.random_tokens(P + D, 151936, 9)
    rows = list(range(P - 1, P + D))
    pcfg, w = pm.read_config(folder), pm.read_weights(folder, torch.float32)
    ref = pm.forward(pcfg, w, ids, rows=rows).numpy()
    del w
    scale = np.abs(ref).max()
    singles = [dict(entries=[dict(id="r", tokens=[ids[P + i]], want=[0])], end=[]) for i in range(D)]
    cuttings = {
        "whole": [dict(entries=[dict(id="r", tokens=ids[:P], want=[P - 1])], end=[])] + singles,
        "portions of 512": [dict(entries=[dict(id="r", tokens=ids[i:i + 512], want=[511] if i + 512 == P else [])], end=[])
                            for i in range(0, P, 512)] + singles,
        "portions of other sizes": [dict(entries=[dict(id="r", tokens=ids[a:b], want=[b - a - 1] if b == P else [])], end=[])
                                    for a, b in ((0, 1000), (1000, 1002), (1002, 1700), (1700, P))] + singles,
    }
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner(folder, dtype=dtype, page_size=16, num_pages=(P + D) // 16 + 2, max_requests=2)
        first = None
        for what, steps in cuttings.items():
            got = H.run_steps(runner, steps)
            runner.release("r")
            runner.cache.check()
            assert sorted(p for _, p in got) == rows
            for i, p in enumerate(rows):
                row = got[("r", p)]
                assert np.isfinite(row).all()
                err = np.abs(row - ref[i]).max() / scale
                assert err <= (2 * H.TOL[dtype] if dtype == "float32" else H.TOL[dtype]), \
                    "%s, %s: position %d: error %.3g" % (dtype, what, p, err)
            if dtype == "float32":
                if first is None:
                    first = got
                else:
                    for key, row in got.items():
                        assert np.array_equal(row, first[key]), "32-bit: %s differs from whole at position %d" % (what, key[1])
        del runner
        torch.cuda.empty_cache()
