"""Pins the plain implementation by what fixes it beside the reference's text: vectors of the
reference's own tests, special cases that reduce to a library routine, and invariants; each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a mask off by one) fails."""
import math

import numpy as np
import pytest
import torch

import helpers as H
import plain_model as pm

torch.manual_seed(0)
D = torch.float64


def test_rms_norm_is_the_references_test_formula():
    # python/test/test_op.py:25-38: x * g / sqrt(mean(x^2) + eps) on [3, 127, 128], eps 1e-5
    x, g = torch.randn(3, 127, 128, dtype=D), torch.randn(128, dtype=D)
    ref = x * g / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5)
    assert torch.allclose(pm.rms_norm(x, g, 1e-5), ref, rtol=1e-12, atol=1e-12)
    # unit gain gives rows of unit RMS; no mean is subtracted (a constant row stays constant, not zero)
    y = pm.rms_norm(x, torch.ones(128, dtype=D), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(3, 127, dtype=D))
    c = pm.rms_norm(torch.full((1, 8), 3.0, dtype=D), torch.ones(8, dtype=D), 0.0)
    assert torch.allclose(c, torch.ones(1, 8, dtype=D))
    # eps sits inside the square root, added to the mean (not to the sum, not outside the root)
    z = pm.rms_norm(torch.zeros(1, 4, dtype=D) + 1e-3, torch.ones(4, dtype=D), 1e-2)
    assert abs(z[0, 0].item() - 1e-3 / math.sqrt(1e-6 + 1e-2)) < 1e-12


def test_linear_is_the_library_routine():
    x, w, b = torch.randn(5, 7, dtype=D), torch.randn(3, 7, dtype=D), torch.randn(3, dtype=D)
    assert torch.allclose(pm.linear(x, w, b), torch.nn.functional.linear(x, w, b))
    assert torch.allclose(pm.linear(x, w), torch.nn.functional.linear(x, w))


def test_rope_is_the_references_test_formula_and_a_complex_rotation():
    # python/test/test_op.py:187-209: freqs = theta^(-2i/hd), halves x[:half], x[half:], positions 0..T-1
    for T, nh, hd, theta in ((128, 32, 128, 1e4), (64, 12, 64, 1e4), (40, 2, 32, 1e6)):
        x = torch.randn(T, nh, hd, dtype=D)
        half = hd // 2
        freqs = np.array([1.0 / (theta ** (2.0 * i / hd)) for i in range(half)], dtype=np.float32)
        ang = np.outer(np.arange(T, dtype=np.float32), freqs)
        s, c = torch.tensor(np.sin(ang))[:, None, :].to(D), torch.tensor(np.cos(ang))[:, None, :].to(D)
        ref = torch.cat([x[..., :half] * c - x[..., half:] * s, x[..., :half] * s + x[..., half:] * c], -1)
        sin, cos = pm.rope_tables(theta, hd, T)
        got = pm.apply_rope(x, list(range(T)), sin, cos)
        assert torch.allclose(got, ref, atol=2e-4, rtol=0)      # the reference's 32-bit tolerance 1e-4
        # as a complex product (x_j + i x_{j+half}) * exp(i p theta^(-j/half))
        z = torch.complex(x[..., :half], x[..., half:]) * torch.polar(torch.ones_like(s), torch.tensor(ang)[:, None, :].to(D))
        assert torch.allclose(got, torch.cat([z.real, z.imag], -1), atol=2e-4, rtol=0)
    # position 0 is the identity; each pair keeps its norm
    x = torch.randn(3, 2, 16, dtype=D)
    sin, cos = pm.rope_tables(1e4, 16, 50)
    assert torch.equal(pm.apply_rope(x, [0, 0, 0], sin, cos), x)
    y = pm.apply_rope(x, [7, 21, 49], sin, cos)
    assert torch.allclose(y[..., :8] ** 2 + y[..., 8:] ** 2, x[..., :8] ** 2 + x[..., 8:] ** 2)
    # a rotary_dim below the head size leaves the tail alone
    sin8, cos8 = pm.rope_tables(1e4, 8, 50)
    y = pm.apply_rope(x, [7, 21, 49], sin8, cos8)
    assert torch.equal(y[..., 8:], x[..., 8:]) and not torch.equal(y[..., :8], x[..., :8])


def test_rope_scores_depend_on_distance_only():
    """A shift of all positions changes no score: <rope(q, p), rope(k, p')> is a function of p - p'.
    A wrong sign in the pair, or the interleaved pairing (2j, 2j+1) on one side only, breaks this."""
    sin, cos = pm.rope_tables(1e4, 32, 200)
    q, k = torch.randn(1, 1, 32, dtype=D), torch.randn(1, 1, 32, dtype=D)
    def score(pq, pk):
        return (pm.apply_rope(q, [pq], sin, cos) * pm.apply_rope(k, [pk], sin, cos)).sum().item()
    assert abs(score(10, 3) - score(110, 103)) < 1e-3      # tables are 32-bit
    assert abs(score(10, 3) - score(3, 10)) > 1e-3         # but direction matters
    # the first pair rotates fastest: frequency 1 at j = 0 (angle = position)
    x = torch.zeros(1, 1, 32, dtype=D)
    x[0, 0, 0] = 1.0
    y = pm.apply_rope(x, [1], sin, cos)
    assert abs(y[0, 0, 0].item() - math.cos(1.0)) < 1e-6 and abs(y[0, 0, 16].item() - math.sin(1.0)) < 1e-6


def test_attention_reduces_to_the_library_routine():
    sdpa = torch.nn.functional.scaled_dot_product_attention
    # plain attention: one head, no rotation; whole sequence = causal
    for nh, nkv, hd, T in ((1, 1, 16, 9), (4, 4, 32, 33), (12, 12, 64, 127)):
        q, k, v = (torch.randn(T, n, hd, dtype=D) for n in (nh, nkv, nkv))
        ref = sdpa(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1)
        assert torch.allclose(pm.attention(q, k, v, list(range(T))), ref, atol=1e-10)
    # grouped heads: python/test/test_op.py:89-154 repeats K/V and masks with tril(diagonal = kv - q)
    for nh, nkv, hd, ql, kv in ((32, 8, 128, 1, 258), (12, 2, 128, 9, 9), (12, 2, 128, 25, 60), (6, 1, 32, 1, 1)):
        q, k, v = torch.randn(ql, nh, hd, dtype=D), torch.randn(kv, nkv, hd, dtype=D), torch.randn(kv, nkv, hd, dtype=D)
        mask = torch.ones(ql, kv, dtype=torch.bool).tril(diagonal=kv - ql)
        kk, vv = (t.repeat_interleave(nh // nkv, dim=1).transpose(0, 1) for t in (k, v))
        ref = sdpa(q.transpose(0, 1), kk, vv, attn_mask=mask).transpose(0, 1)
        assert torch.allclose(pm.attention(q, k, v, list(range(kv - ql, kv))), ref, atol=1e-10)
    # a single new token equals the last row of the whole computation
    q, k, v = torch.randn(20, 4, 16, dtype=D), torch.randn(20, 2, 16, dtype=D), torch.randn(20, 2, 16, dtype=D)
    whole = pm.attention(q, k, v, list(range(20)))
    assert torch.allclose(pm.attention(q[19:], k, v, [19]), whole[19:])
    # head h reads kv head h // group (not h % nkv): make the kv heads tell themselves apart
    v2 = torch.zeros(5, 2, 16, dtype=D)
    v2[:, 1, :] = 1.0
    out = pm.attention(torch.randn(5, 4, 16, dtype=D), torch.randn(5, 2, 16, dtype=D), v2, list(range(5)))
    assert torch.allclose(out[:, :2], torch.zeros(5, 2, 16, dtype=D)) and torch.allclose(out[:, 2:], torch.ones(5, 2, 16, dtype=D))


def test_attention_window_edges():
    T, w = 30, 7
    q, k, v = torch.randn(T, 2, 16, dtype=D), torch.randn(T, 2, 16, dtype=D), torch.randn(T, 2, 16, dtype=D)
    got = pm.attention(q, k, v, list(range(T)), window=w)
    for t in (0, 5, 6, 7, 29):
        lo = max(0, t - w + 1)                       # the window counts the token itself
        ref = pm.attention(q[t:t + 1], k[lo:t + 1], v[lo:t + 1], [t - lo])
        assert torch.allclose(got[t:t + 1], ref, atol=1e-12)
    assert torch.allclose(pm.attention(q, k, v, list(range(T)), window=T), pm.attention(q, k, v, list(range(T))))
    assert torch.allclose(pm.attention(q, k, v, list(range(T)), window=1), v.repeat_interleave(1, dim=1))


def test_swiglu_is_the_library_routine():
    for shape in ((4, 128, 256), (2, 511, 1024)):
        g, u = torch.randn(*shape, dtype=D) * 3, torch.randn(*shape, dtype=D)
        assert torch.allclose(pm.swiglu(g, u), torch.nn.functional.silu(g) * u, atol=1e-12)
    assert pm.swiglu(torch.zeros(1, dtype=D), torch.ones(1, dtype=D)).item() == 0.0
    assert abs(pm.swiglu(torch.tensor([30.0], dtype=D), torch.tensor([2.0], dtype=D)).item() - 60.0) < 1e-9


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    out = {}
    for name in ("A", "B", "C"):
        cfg, seed, _ = H.TINY[name]
        folder = H.make_model_folder(tmp_path_factory.mktemp("plain" + name), cfg, seed)
        out[name] = (pm.read_config(folder), pm.read_weights(folder), folder)
    return out


def test_model_is_causal_and_deterministic(tiny):
    for name in ("A", "B", "C"):
        cfg, w, _ = tiny[name]
        ids = H.random_tokens(50, cfg["vocab_size"], 1)
        full = pm.forward(cfg, w, ids)
        assert full.shape == (50, cfg["vocab_size"])
        # logits at position t do not depend on the tokens after t
        assert torch.allclose(pm.forward(cfg, w, ids[:20]), full[:20], atol=1e-12)
        other = ids[:20] + H.random_tokens(30, cfg["vocab_size"], 2)
        assert torch.allclose(pm.forward(cfg, w, other)[:20], full[:20], atol=1e-12)
        assert not torch.allclose(pm.forward(cfg, w, other)[20:], full[20:], atol=1e-6)


def test_block_order_by_switching_parts_off(tiny):
    """With the output and down projections zeroed the blocks add nothing: logits = head(norm(embedding)).
    With only the down projections zeroed: x + attn(norm1(x)) per block.  A norm applied to the residual
    itself (post-norm), or a missing residual, fails one of the two."""
    cfg, w, _ = tiny["B"]
    ids = H.random_tokens(12, cfg["vocab_size"], 3)
    w0 = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        w0["model.layers.%d.self_attn.o_proj.weight" % i] = torch.zeros_like(w["model.layers.%d.self_attn.o_proj.weight" % i])
        w0["model.layers.%d.mlp.down_proj.weight" % i] = torch.zeros_like(w["model.layers.%d.mlp.down_proj.weight" % i])
    x = w["model.embed_tokens.weight"][ids]
    ref = pm.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].t()
    assert torch.allclose(pm.forward(cfg, w0, ids), ref, atol=1e-12)
    w1 = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        w1["model.layers.%d.mlp.down_proj.weight" % i] = torch.zeros_like(w["model.layers.%d.mlp.down_proj.weight" % i])
    sin, cos = pm.rope_tables(cfg["rope_theta"], cfg["head_dim"], 12)
    for i in range(cfg["num_hidden_layers"]):
        p = "model.layers.%d" % i
        a, _ = pm.attention_block(pm.rms_norm(x, w[p + ".input_layernorm.weight"], cfg["rms_norm_eps"]), w,
                                  p + ".self_attn", cfg, list(range(12)), sin, cos, None)
        x = x + a
    ref = pm.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].t()
    assert torch.allclose(pm.forward(cfg, w1, ids), ref, atol=1e-12)


def test_tied_and_untied_heads_agree(tiny):
    cfg, w, _ = tiny["B"]
    ids = H.random_tokens(9, cfg["vocab_size"], 4)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    tied = dict(cfg, tie_word_embeddings=True)
    assert torch.equal(pm.forward(cfg, w2, ids), pm.forward(tied, w, ids))
    assert not torch.allclose(pm.forward(cfg, w, ids), pm.forward(tied, w, ids))


def test_window_layers_follow_the_config(tiny):
    cfg, w, _ = tiny["C"]
    assert cfg["windows"] == [None, 40, 40, 40]
    ids = H.random_tokens(90, cfg["vocab_size"], 5)
    full = dict(cfg, windows=[None] * 4)
    a, b = pm.forward(cfg, w, ids), pm.forward(full, w, ids)
    assert torch.allclose(a[:40], b[:40], atol=1e-12)          # inside the window nothing differs
    assert not torch.allclose(a[41:], b[41:], atol=1e-9)


def test_sampling():
    row = torch.tensor([0.1, 2.0, 2.0, -1.0])
    assert pm.argmax_token(row) == 1                           # lowest index among equals
    assert pm.sample_token(row, 0.0, 0.99) == 1
    assert pm.sample_token(row, 1e-4, 0.3) == 1                # temperature -> 0 tends to the argmax
    p = torch.softmax(row.double() / 0.8, 0).numpy()
    c = np.cumsum(p)
    for u in (0.0, 0.01, 0.3, 0.6, 0.95, 0.999999):
        assert pm.sample_token(row, 0.8, u) == int(np.searchsorted(c, u, side="right"))
    counts = np.bincount([pm.sample_token(row, 0.8, (i + 0.5) / 4000) for i in range(4000)], minlength=4)
    assert np.abs(counts / 4000 - p).max() < 1e-3


def test_generate_stops(tiny):
    cfg, w, _ = tiny["A"]
    out = pm.generate(cfg, w, [1, 2, 3], 5, ignore_eos=True)
    assert len(out) == 5
    first = out[0]
    stop = dict(cfg, eos_token_ids=[first])
    assert pm.generate(stop, w, [1, 2, 3], 5) == [first]
