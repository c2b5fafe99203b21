"""Plans chosen by measurement (kernels/autotune.py): every candidate plan of a product gives the product, and a runner
that times its plans before it records a step gives the plain implementation's logits."""
import numpy as np
import pytest
import torch

import helpers as H
import plain_model as pm

pytestmark = pytest.mark.gpu


def _operands(rows, n, k, seed, bias):
    g = torch.Generator().manual_seed(seed)
    d = torch.device("cuda:0")
    x = (torch.randn((rows, k), generator=g) * 0.7).bfloat16()
    w = (torch.randn((n, k), generator=g) * 0.05).bfloat16()
    b = (torch.randn((n,), generator=g) * 0.3).bfloat16() if bias else None
    return x.to(d), w.to(d), (b.to(d) if bias else None), x.double(), w.double(), (b.double() if bias else None)


@pytest.mark.parametrize("rows,n,k", [(8, 520, 1024), (24, 1536, 4480), (40, 776, 1096), (64, 1544, 2304),
                                      (128, 1536, 2048), (200, 3584, 4096)])
def test_every_candidate_plan_gives_the_product(rows, n, k):
    from ginfer_amd.kernels import ops
    from ginfer_amd.parts import linear as L
    tried = set()
    for bias in (False, True):
        for f32 in (False, True):
            for parts_ok in (False, True):
                x, w, b, xd, wd, bd = _operands(rows, n, k, rows + n + k, bias)
                ref = xd @ wd.T + (bd if bias else 0.0)
                skinny_ok = ops.gemm_skinny_supported(x, w)
                key = ("linear", rows, n, k, bias, f32, parts_ok, skinny_ok)
                for plan in L.linear_candidates(key):
                    y = L.run_linear_plan(plan, x, w, b, torch.float32 if f32 else None)
                    parts = plan[-1] if (plan[0] == "library" or plan[2] > 1) and plan[-1] > 1 else 1
                    if parts > 1:
                        assert y.shape == (parts, rows, n) and y.dtype == torch.float32, (plan, y.shape)
                        y = y.double().sum(0)
                    else:
                        assert y.shape == (rows, n) and y.dtype == (torch.float32 if f32 else torch.bfloat16), (plan, y.dtype)
                    err = float((y.double().cpu() - ref).abs().max() / ref.abs().max())
                    # bfloat16 results carry one rounding (2^-9 of the value); 32-bit ones only the order of the sums
                    tol = 1e-5 if (f32 or parts > 1) else 4e-3
                    assert err <= tol, "plan %s of %s: %.3g" % (plan, key, err)
                    tried.add(plan)
    assert ("library", 1) in tried and len(tried) >= 3, tried
    print("plans tried for rows %d, %d x %d: %s" % (rows, n, k, sorted(tried)))


@pytest.mark.parametrize("rows,n,k", [(8, 520, 1024), (40, 776, 1096), (64, 2304, 1536), (256, 1536, 1024)])
def test_every_candidate_plan_of_the_gated_product(rows, n, k):
    from ginfer_amd.kernels import ops
    from ginfer_amd.parts import linear as L
    x, w, _, xd, wd, _ = _operands(rows, 2 * n, k, rows + n, False)
    gate, up = xd @ wd[:n].T, xd @ wd[n:].T
    # the plain statement rounds the products to bfloat16 before the activation only where the kernels do; compare in
    # 64-bit with a tolerance of two roundings
    ref = gate * torch.sigmoid(gate) * up
    key = ("gated", rows, 2 * n, k, ops.gemm_skinny_supported(x, w), L._transposable(x, w))
    plans = L.gated_candidates(key)
    assert len(plans) >= 2
    for plan in plans:
        y = L.run_gated_plan(plan, x, w)
        assert y.shape == (rows, n) and y.dtype == torch.bfloat16
        err = float((y.double().cpu() - ref).abs().max() / ref.abs().max())
        assert err <= 1.2e-2, "plan %s: %.3g" % (plan, err)


def test_a_runner_that_times_its_plans(tmp_path):
    """Two layers of a 7B shape, 40 requests decoding side by side: the runner times the plans of its products when it
    records the step (the rules' plan for this down projection is not the fastest one), and logits stay the plain
    implementation's, in the recorded step's replays and in eager steps of the same size."""
    from ginfer_amd import ModelRunner
    from ginfer_amd.kernels import autotune
    V, live = 1500, 40
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=3584, num_attention_heads=28,
               num_key_value_heads=4, intermediate_size=18944, vocab_size=V, rope_theta=1e6, rms_norm_eps=1e-6,
               tie_word_embeddings=False, max_position_embeddings=512)
    folder = H.make_model_folder(tmp_path / "wide", cfg, 4, "float32")
    prompt, decoded = 18, 6
    reqs = {"r%d" % i: H.random_tokens(prompt + decoded, V, 100 + i) for i in range(live)}
    steps = [dict(entries=[dict(id=rid, tokens=ids[:prompt], want=[prompt - 1])], end=[]) for rid, ids in reqs.items()]
    for k in range(decoded):
        steps.append(dict(entries=[dict(id=rid, tokens=[ids[prompt + k]], want=[0]) for rid, ids in reqs.items()],
                          end=list(reqs) if k == decoded - 1 else []))
    runner = ModelRunner(folder, dtype="bfloat16", page_size=16, num_pages=2 * live, max_requests=live, autotune=True)
    got = H.run_steps(runner, steps)
    runner.cache.check()
    assert runner.counts["autotuned_keys"] >= 3 and runner.counts["replayed_decode"] >= 3, runner.counts
    assert isinstance(runner.plans, autotune.Table)
    keys = [key for key, _, _ in runner.plans.report]
    assert ("linear", 48, 3584, 18944, False, False, True, True) in keys, keys
    for key, plan, times in runner.plans.report:
        print("%s -> %s (%d plans, %.1f to %.1f us)" % (key, plan, len(times), min(times.values()), max(times.values())))
        assert runner.plans[key] == plan and plan in times
    # the plans are the runner's own: a runner built without autotune runs by the rules, whatever this one has measured
    plain = ModelRunner(folder, dtype="bfloat16", page_size=16, num_pages=2 * live, max_requests=live)
    assert plain.plans is None and not autotune.active()
    del plain
    # a second runner that is handed the first one's table finds the plans and times nothing (its first steps already run
    # by them, where the first runner's ran by the rules: the two agree up to rounding only)
    again = ModelRunner(folder, dtype="bfloat16", page_size=16, num_pages=2 * live, max_requests=live, autotune=runner.plans)
    got2 = H.run_steps(again, steps)
    assert again.counts.get("autotuned_keys", 0) == 0 and again.plans is runner.plans
    # the kept plans in recorded steps and launched kernel by kernel: the same bits (prompts run kernel by kernel in both)
    pair = [ModelRunner(folder, dtype="bfloat16", page_size=16, num_pages=2 * live, max_requests=live, autotune=runner.plans,
                        use_graphs=g, graph_mixed_steps=False) for g in (True, False)]
    a, b = (H.run_steps(r, steps) for r in pair)
    assert pair[0].counts["replayed_decode"] >= 3 and pair[1].counts["replayed_decode"] == 0
    for k in a:
        assert np.array_equal(a[k], b[k]), "replayed and launched steps differ at %s" % (k,)
    pcfg, w = pm.read_config(folder), pm.read_weights(folder, torch.float32)
    for rid in list(reqs)[:3] + list(reqs)[-2:]:
        ref = pm.forward(pcfg, w, reqs[rid]).numpy()
        for p in range(prompt - 1, prompt + decoded):
            for g in (got, got2, a):
                err = np.abs(g[(rid, p)] - ref[p]).max() / np.abs(ref).max()
                assert err <= H.TOL["bfloat16"], "request %s position %d: %.3g" % (rid, p, err)
