"""The engine against the plain implementation, on the GPU: every way of cutting and batching, in
32-bit and in bfloat16, at three tiny configurations."""
import numpy as np
import pytest
import torch

import helpers as H
import plain_model as pm

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, seed, _) in H.TINY.items():
        out[name] = H.make_model_folder(tmp_path_factory.mktemp("tiny" + name), cfg, seed, "float32")
    return out


@pytest.fixture(scope="module")
def sharp_folders(tmp_path_factory):
    """The same configurations with every weight drawn three times as wide.  With the usual N(0, 0.02) a tiny model's
    scores are all but equal, its attention is a plain mean of the values, and one wrong or missing key moves a logit
    by less than bfloat16's rounding; with wide draws the softmax has peaks and such a fault shows."""
    out = {}
    for name, (cfg, seed, _) in H.TINY.items():
        out[name] = H.make_model_folder(tmp_path_factory.mktemp("sharp" + name), cfg, seed, "float32", std_scale=3.0)
    return out


def _requests(name, lengths, seed=10):
    vocab = H.TINY[name][0]["vocab_size"]
    return {"r%d" % i: H.random_tokens(n, vocab, seed + i) for i, n in enumerate(lengths)}


def _runner(folder, name, dtype, pages, max_requests=8):
    from ginfer_amd import ModelRunner
    return ModelRunner(folder, dtype=dtype, page_size=H.TINY[name][2], num_pages=pages, max_requests=max_requests)


LENGTHS = {"A": [5, 17, 33, 70, 131], "B": [1, 9, 40, 64, 100, 150], "C": [3, 50, 97, 160]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_long_prompts_whole_in_portions_and_decoded(folders, tmp_path, name, dtype):
    """Prompts of several hundred tokens: whole, they are a step of so many tokens that the 32-bit attention runs its
    kernel for prompt portions (a wavefront per head and 16 tokens); in portions and decoded, the kernel for single
    tokens and small steps.  The same logits as the plain model, and in 32-bit the same bits whatever the cutting; C has
    windows of 40 keys on three of its layers."""
    if name == "A":
        cfg = dict(H.TINY_A, max_position_embeddings=1024)
        folder, lengths, ps = H.make_model_folder(tmp_path / "long_a", cfg, 5, "float32"), [700, 90], 16
    else:
        folder, lengths, ps = folders["C"], [380, 300], H.TINY["C"][2]
    vocab = H.TINY[name][0]["vocab_size"]
    reqs = {"r%d" % i: H.random_tokens(n, vocab, 40 + i) for i, n in enumerate(lengths)}
    from ginfer_amd import ModelRunner
    runner = ModelRunner(folder, dtype=dtype, page_size=ps, num_pages=-(-1024 // ps), max_requests=4)
    results = {}
    for what, steps in (("whole", H.steps_whole(reqs)), ("last 32 decoded", H.steps_last_decoded(reqs)),
                        ("portions", H.steps_portions(reqs, sizes=(130, 2, 33, 300, 16, 7, 64, 5))),
                        ("mixed", H.steps_mixed(reqs, max_live=2, seed=4))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        assert not runner.cache.requests
        H.compare_with_plain(got, reqs, folder, H.TOL[dtype], "%s %s %s" % (name, dtype, what))
        results[what] = got
    if dtype == "float32":
        for what in ("last 32 decoded", "portions", "mixed"):
            for key, row in results[what].items():
                assert np.array_equal(row, results["whole"][key]), "%s: %r differs in bits from whole" % (what, key)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("weights", ["usual", "wide"])
def test_whole_last_decoded_and_portions(folders, sharp_folders, name, dtype, weights):
    folders = folders if weights == "usual" else sharp_folders
    reqs = _requests(name, LENGTHS[name])
    ps = H.TINY[name][2]
    runner = _runner(folders[name], name, dtype, pages=-(-256 // ps))
    results = {}
    for what, steps in (("whole", H.steps_whole(reqs)), ("last 32 decoded", H.steps_last_decoded(reqs)),
                        ("portions", H.steps_portions(reqs))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        assert not runner.cache.requests
        H.compare_with_plain(got, reqs, folders[name], H.TOL[dtype], "%s %s %s" % (name, dtype, what))
        results[what] = got
    if dtype == "float32":
        # in 32-bit every reduction has a fixed order: the cuttings agree to the last bit
        for what in ("last 32 decoded", "portions"):
            for key, row in results["whole"].items():
                assert np.array_equal(row, results[what][key]), "%s: %r differs in bits from whole" % (what, key)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("weights", ["usual", "wide"])
def test_mixed_with_pages_used_again(folders, sharp_folders, name, dtype, weights):
    folders = folders if weights == "usual" else sharp_folders
    lengths = {"A": [40, 75, 110, 33, 90, 61, 130], "B": [9, 100, 64, 31, 150, 77, 18], "C": [60, 97, 140, 45, 120, 80]}
    reqs = _requests(name, lengths[name], seed=40)
    steps = H.steps_mixed(reqs, max_live=4, seed=3)
    assert any(len(s["entries"]) > 1 and any(len(e["tokens"]) == 1 for e in s["entries"])
               and any(len(e["tokens"]) > 1 for e in s["entries"]) for s in steps)
    ps = H.TINY[name][2]
    pages = -(-H.max_live_tokens(steps) // ps)
    assert pages * ps < sum(len(v) for v in reqs.values()), "the pool is not small enough to reuse pages"
    runner = _runner(folders[name], name, dtype, pages=pages)
    got = H.run_steps(runner, steps)
    runner.cache.check()
    H.compare_with_plain(got, reqs, folders[name], H.TOL[dtype], "%s %s mixed" % (name, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_trace_run_program(folders, tmp_path, dtype, name):
    """bin/trace_run as a user runs it: whole, then mixed with few pages, in one process (A: the head shares the
    embedding's table; C: layers with a window beside layers without, so two groups of pages)."""
    reqs = _requests(name, [70, 33, 120, 64, 90], seed=70)
    whole = H.steps_whole(reqs)
    mixed = H.steps_mixed({k + "m": v for k, v in reqs.items()}, max_live=4, seed=5)
    steps = whole + mixed
    got = H.run_trace(folders[name], dtype, steps, tmp_path / "out", H.max_live_tokens(steps), page_size=H.TINY[name][2])
    both = dict(reqs)
    both.update({k + "m": v for k, v in reqs.items()})
    H.compare_with_plain(got, both, folders[name], H.TOL[dtype], "trace_run %s" % dtype)


def test_trace_run_program_from_a_configuration_and_a_seed(tmp_path):
    """bin/trace_run --config CONFIG.json --seed S draws the weights itself, on the device: the logits are those of
    the model folder that the host writes for the same seed, which the plain implementation reads."""
    cfg, seed, page = H.TINY["B"]
    folder = H.make_model_folder(tmp_path / "b", cfg, 11, "float32")
    reqs = _requests("B", [50, 21], seed=71)
    steps = H.steps_portions(reqs, sizes=(9, 2, 30))
    got = H.run_trace(folder, "float32", steps, tmp_path / "out", H.max_live_tokens(steps), page_size=page, seed=11)
    H.compare_with_plain(got, reqs, folder, H.TOL["float32"], "trace_run from a seed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """Three hundred tokens one by one after a short prompt, across many page edges."""
    name = "B"
    reqs = _requests(name, [330], seed=90)
    steps = H.steps_last_decoded(reqs, last=320)
    runner = _runner(folders[name], name, dtype, pages=48)
    got = H.run_steps(runner, steps)
    H.compare_with_plain(got, reqs, folders[name], H.TOL[dtype], "long decoding %s" % dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_first_tokens(folders, name, dtype):
    """The first tokens of a sequence, one at a time from position 0."""
    reqs = _requests(name, [6], seed=95)
    runner = _runner(folders[name], name, dtype, pages=8)
    got = H.run_steps(runner, H.steps_last_decoded(reqs, last=6))
    H.compare_with_plain(got, reqs, folders[name], H.TOL[dtype], "first tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "B"
    folder = folders[name]
    vocab = H.TINY[name][0]["vocab_size"]
    prompts = [H.random_tokens(n, vocab, 200 + n) for n in (1, 9, 40, 64, 100)]
    eng = Engine(EngineConfig(model_path=folder, dtype=dtype, max_num_batched_tokens=24, max_num_seqs=4,
                              max_seq_len=256, kvcache_block_size=8, num_kvcache_blocks=40))
    streamed = {}
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True),
                        on_token=lambda rid, tok: streamed.setdefault(rid, []).append(tok))
    eng.runner.cache.check()
    assert not eng.runner.cache.requests
    for p, o in zip(prompts, outs):
        assert o.prompt_token_ids == p and len(o.token_ids) == 12 and o.finish_reason == "max_tokens"
        assert streamed[o.request_id] == o.token_ids          # every token was handed out as it came, in order
    _greedy_as_plain(folder, prompts, outs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_with_a_tied_head(folders, dtype):
    """The smallest configuration as it is stated for this engine: tied head, prompts of 5, 17 and 33 tokens, 8 greedy
    tokens each, pages of 16, through the entry point."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "A"
    vocab = H.TINY[name][0]["vocab_size"]
    prompts = [H.random_tokens(n, vocab, 300 + n) for n in (5, 17, 33)]
    eng = Engine(EngineConfig(model_path=folders[name], dtype=dtype, max_num_batched_tokens=32, max_num_seqs=4,
                              max_seq_len=128, kvcache_block_size=16, num_kvcache_blocks=16))
    assert eng.runner.model.head.weight.data_ptr() == eng.runner.model.embedding.weight.data_ptr()     # one table
    outs = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    eng.runner.cache.check()
    assert [len(o.token_ids) for o in outs] == [8, 8, 8]
    _greedy_as_plain(folders[name], prompts, outs, dtype)


def _greedy_as_plain(folder, prompts, outs, dtype):
    """Every generated token is the plain implementation's greedy choice given the engine's own prefix, unless the
    plain top two are within rounding of each other."""
    cfg, w = pm.read_config(folder), pm.read_weights(folder)
    for p, o in zip(prompts, outs):
        ids = p + o.token_ids
        logits = pm.forward(cfg, w, ids[:-1])
        for k, tok in enumerate(o.token_ids):
            row = logits[len(p) - 1 + k]
            best = int(torch.argmax(row))
            if tok != best:
                gap = float(row[best] - row[tok]) / float(row.abs().max())
                assert gap <= H.TOL[dtype], "token %d of prompt %d: engine %d, plain %d, gap %.3g" % (k, len(p), tok, best, gap)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_requests_that_share_a_prefix_share_its_pages(folders, sharp_folders, dtype):
    """A request whose first tokens the cache already holds (from a request before it, finished or still running)
    starts behind them.  Its tokens are the plain implementation's, and in 32-bit the same, bit for bit, as
    without sharing; fewer prompt tokens are run."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "B"
    folder = sharp_folders[name]         # wide draws: a page that holds other tokens would change the output
    vocab = H.TINY[name][0]["vocab_size"]
    stem = H.random_tokens(70, vocab, 1200)
    first = [stem[:50], H.random_tokens(23, vocab, 1201)]
    # the whole first prompt again; its beginning with another end; one that leaves the stem inside the first page;
    # the first request's prompt and output as a prompt (a conversation that goes on)
    later = [stem[:50], stem[:41] + H.random_tokens(9, vocab, 1202), stem[:5] + H.random_tokens(30, vocab, 1203), None,
             stem[:64]]
    results = {}
    for share in (True, False):
        eng = Engine(EngineConfig(model_path=folder, dtype=dtype, max_num_batched_tokens=32, max_num_seqs=4,
                                  max_seq_len=256, kvcache_block_size=8, num_kvcache_blocks=60,
                                  enable_prefix_caching=share))
        sp = SamplingParams(max_tokens=10, ignore_eos=True)
        outs = eng.generate(first, sp)
        prompts = [p if p is not None else first[0] + outs[0].token_ids for p in later]
        # the last one arrives while the others run: it finds pages of a request that is still running
        ids = [eng.add_request(p, SamplingParams(max_tokens=10, ignore_eos=True)) for p in prompts[:4]]
        done, steps = {}, 0
        while eng.has_unfinished():
            for o in eng.step():
                done[o.request_id] = o
            steps += 1
            if steps == 3:
                ids.append(eng.add_request(prompts[4], SamplingParams(max_tokens=10, ignore_eos=True)))
        eng.runner.cache.check()
        assert not eng.runner.cache.requests
        outs2 = [done[i] for i in ids]
        _greedy_as_plain(folder, first + prompts, outs + outs2, dtype)
        results[share] = ([o.token_ids for o in outs + outs2], eng.runner.cache.prefix_hit_tokens, eng.stats["prefill_tokens"])
    (shared, hits, ran), (alone, no_hits, ran_alone) = results[True], results[False]
    # pages of 8: 48 of 50, 40 of 41, none of 5, 56 of the 60 of prompt and output, 48 of 64 (what the first holds)
    assert hits == 48 + 40 + 0 + 56 + 48 and no_hits == 0
    assert ran == ran_alone - hits
    if dtype == "float32":
        assert shared == alone
    # a model with a window cannot share: asked for, it is refused; left open, it goes without
    with pytest.raises(ValueError, match="window"):
        Engine(EngineConfig(model_path=folders["C"], dtype=dtype, max_seq_len=128, num_kvcache_blocks=20,
                            enable_prefix_caching=True))
    assert not Engine(EngineConfig(model_path=folders["C"], dtype=dtype, max_seq_len=128,
                                   num_kvcache_blocks=20)).runner.cache.prefix_caching


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_late_request_finds_the_pages_of_a_request_that_is_still_running(sharp_folders, dtype):
    """Full pages are remembered when they are committed (ginfer/engine/block_manager.cc:98-108), so a request that
    shares 48 tokens with one that is still decoding starts behind them: 48 tokens found at the moment it is admitted,
    the same when the first request has finished before, none with sharing off, and the same tokens in all three."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    folder = sharp_folders["B"]
    vocab = H.TINY["B"][0]["vocab_size"]
    first = H.random_tokens(50, vocab, 1300)
    late = first[:48] + H.random_tokens(7, vocab, 1301)
    tokens, found = {}, {}
    for case, (share, first_outputs) in dict(running=(True, 40), finished=(True, 3), alone=(False, 40)).items():
        eng = Engine(EngineConfig(model_path=folder, dtype=dtype, max_num_batched_tokens=64, max_num_seqs=4, max_seq_len=256,
                                  kvcache_block_size=8, num_kvcache_blocks=60, enable_prefix_caching=share))
        a = eng.add_request(first, SamplingParams(max_tokens=first_outputs, ignore_eos=True))
        done = {}
        for _ in range(8):
            if eng.has_unfinished():
                for o in eng.step():
                    done[o.request_id] = o
        assert (a in done) == (case == "finished")
        before = eng.runner.cache.prefix_hit_tokens
        b = eng.add_request(late, SamplingParams(max_tokens=6, ignore_eos=True))
        while b not in done:
            for o in eng.step():
                done[o.request_id] = o
            if case == "running" and "at_admission" not in found and eng.runner.cache.has(b):
                # the first request is still running when the late one has got its pages
                found["at_admission"] = (eng.runner.cache.prefix_hit_tokens - before, eng.runner.cache.has(a))
        found[case] = eng.runner.cache.prefix_hit_tokens - before
        while eng.has_unfinished():
            for o in eng.step():
                done[o.request_id] = o
        eng.runner.cache.check()
        tokens[case] = (done[a].token_ids[:3], done[b].token_ids)
        _greedy_as_plain(folder, [late], [done[b]], dtype)
        del eng
    assert found == dict(at_admission=(48, True), running=48, finished=48, alone=0)
    if dtype == "float32":
        assert tokens["running"] == tokens["finished"] == tokens["alone"]


def test_requests_without_a_seed_draw_from_streams_of_their_own(folders):
    """Two requests with the same prompt and the same sampling settings, no seed named: each draws from the stream of
    its own id, so their tokens differ (and each is what the plain sampler draws with that stream's numbers); with a
    seed named, both give the same tokens."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    from ginfer_amd.sampling import uniform, request_seed
    folder = folders["B"]
    prompt = H.random_tokens(20, 1000, 77)
    eng = Engine(EngineConfig(model_path=folder, dtype="float32", max_num_batched_tokens=64, max_num_seqs=4, max_seq_len=128,
                              kvcache_block_size=8, num_kvcache_blocks=40, enable_prefix_caching=False))
    outs = eng.generate([prompt, prompt], SamplingParams(max_tokens=16, temperature=1.0, ignore_eos=True))
    assert outs[0].token_ids != outs[1].token_ids
    cfg, w = pm.read_config(folder), pm.read_weights(folder)
    for o in outs:
        logits = pm.forward(cfg, w, (prompt + o.token_ids)[:-1])
        for k, tok in enumerate(o.token_ids):
            row, u = logits[len(prompt) - 1 + k], uniform(request_seed(o.request_id), k)
            want = pm.sample_token(row, 1.0, u)
            assert want == tok or _is_a_tie(row, 1.0, u, tok, want)
    same = eng.generate([prompt, prompt], SamplingParams(max_tokens=16, temperature=1.0, ignore_eos=True, seed=3))
    assert same[0].token_ids == same[1].token_ids


def test_temperature_sampling_matches_plain_with_same_uniforms(folders):
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    from ginfer_amd.sampling import uniform
    name = "B"
    folder = folders[name]
    vocab = H.TINY[name][0]["vocab_size"]
    prompts = [H.random_tokens(n, vocab, 300 + n) for n in (1, 9, 40, 64, 100)]
    eng = Engine(EngineConfig(model_path=folder, dtype="float32", max_num_batched_tokens=24, max_num_seqs=5,
                              max_seq_len=256, kvcache_block_size=8, num_kvcache_blocks=60))
    params = [SamplingParams(max_tokens=12, temperature=0.8, seed=7 + i, ignore_eos=True) for i in range(5)]
    outs = eng.generate(prompts, params)
    cfg, w = pm.read_config(folder), pm.read_weights(folder)
    agree = total = 0
    for p, sp, o in zip(prompts, params, outs):
        ids = p + o.token_ids
        logits = pm.forward(cfg, w, ids[:-1])
        for k, tok in enumerate(o.token_ids):
            total += 1
            agree += int(pm.sample_token(logits[len(p) - 1 + k], 0.8, uniform(sp.seed, k)) == tok)
    # the inverse CDF is a step function of the uniform number; only a draw within rounding of a step may differ
    assert agree >= total - 1, "%d of %d sampled tokens agree with the plain sampler" % (agree, total)
    assert len({tuple(o.token_ids) for o in outs}) > 1


@pytest.mark.parametrize("rows", [40, 150])
def test_recorded_decode_steps_of_many_rows(folders, rows):
    """Decode batches of 40 and 150 rows with wide products (several row blocks and four-tile wavefronts in the
    weight-streaming kernel); recorded into a graph and replayed many times, with eager steps between the
    replays, it must give the eager bits every time."""
    from ginfer_amd import ModelRunner, StepEntry
    name = "B"
    vocab = H.TINY[name][0]["vocab_size"]
    cfgd = dict(H.TINY[name][0], vocab_size=4600, intermediate_size=2304)      # wide: the four-tile kernel variants
    import tempfile
    folder = H.make_model_folder(tempfile.mkdtemp(), cfgd, 9, "float32")
    # graph_mixed_steps=False: the prompt portions between the replays run kernel by kernel in both runners
    runners = [ModelRunner(folder, dtype="bfloat16", page_size=8, num_pages=2000, max_requests=rows + 8, use_graphs=g,
                           graph_mixed_steps=False) for g in (True, False)]
    prompts = {i: H.random_tokens(5 + i % 7, 4600, 800 + i) for i in range(rows)}
    stream = H.random_tokens(rows * 30, 4600, 900)
    outs = [[], []]
    for k, r in enumerate(runners):
        r.step([StepEntry(i, p, []) for i, p in prompts.items()])
        for stepno in range(25):
            outs[k].append(r.step([StepEntry(i, [stream[stepno * rows + i]], [0]) for i in prompts]).cpu())
            if stepno % 6 == 2:                  # eager work between replays
                outs[k].append(r.step([StepEntry("x%d" % stepno, H.random_tokens(30, 4600, stepno), [29])]).cpu())
                r.release("x%d" % stepno)
    assert runners[0]._graphs and not runners[1]._graphs
    worst = 0.0
    for n, (a, b) in enumerate(zip(*outs)):
        worst = max(worst, float((a - b).abs().max() / b.abs().max()))
    print("largest relative difference between replayed and eager steps: %.3g" % worst)
    for n, (a, b) in enumerate(zip(*outs)):
        assert torch.equal(a, b), "step %d: a replayed step differs from the eager step (largest difference %.3g)" % (n, worst)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_recorded_decode_steps_equal_eager_ones(folders, name, dtype):
    """Decode steps replayed from a HIP graph give the bits of the same steps launched one kernel at a
    time: many replays, with eager steps (a prompt portion, another batch size) and synchronisations
    between them, each replay checked."""
    from ginfer_amd import ModelRunner, StepEntry
    vocab = H.TINY[name][0]["vocab_size"]
    ps = H.TINY[name][2]
    runners = [ModelRunner(folders[name], dtype=dtype, page_size=ps, num_pages=160, max_requests=8, use_graphs=g,
                           graph_mixed_steps=False) for g in (True, False)]
    prompts = {i: H.random_tokens(n, vocab, 500 + i) for i, n in enumerate((20, 45, 70))}
    late = H.random_tokens(90, vocab, 600)
    stream = H.random_tokens(400, vocab, 601)
    outs = [[], []]
    for k, r in enumerate(runners):
        for i, p in prompts.items():
            r.step([StepEntry(i, p, [])])
        at = 0
        for stepno in range(60):
            batch = [StepEntry(i, [stream[at + i]], [0]) for i in prompts]
            at += 3
            outs[k].append(r.step(batch).cpu())
            if stepno == 20:                       # an eager step between replays: a prompt portion of a newcomer
                outs[k].append(r.step([StepEntry("late", late[:50], [49])]).cpu())
            if stepno == 30:                       # and the newcomer joins the batch beside a portion of itself
                outs[k].append(r.step([StepEntry("late", late[50:], [39])] + [StepEntry(0, [stream[at]], [0])]).cpu())
                r.release(0)
                prompts_now = [1, 2]
                for _ in range(4):                 # another batch size gets a graph of its own
                    outs[k].append(r.step([StepEntry(i, [stream[at + i]], [0]) for i in prompts_now]).cpu())
                    at += 3
                r.step([StepEntry(0, prompts[0] + stream[:31], [])])      # request 0 comes back, on other pages
        r.cache.check()
    assert runners[0]._graphs and not runners[1]._graphs
    assert len(outs[0]) == len(outs[1])
    for n, (a, b) in enumerate(zip(*outs)):
        assert torch.equal(a, b), "step %d: a replayed step differs from the eager step" % n


def test_eviction_and_recomputation_keep_the_tokens(folders):
    """When pages run out the newest request is evicted and later fed again from its first token; in
    32-bit its continuation is the same as with room for everybody."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "B"
    vocab = H.TINY[name][0]["vocab_size"]
    prompts = [H.random_tokens(n, vocab, 700 + n) for n in (30, 41, 52, 25)]
    results = []
    for blocks in (64, 14):                       # 14 pages of 8: two requests of ~80 tokens do not fit beside a third
        eng = Engine(EngineConfig(model_path=folders[name], dtype="float32", max_num_batched_tokens=48, max_num_seqs=4,
                                  max_seq_len=128, kvcache_block_size=8, num_kvcache_blocks=blocks))
        outs = eng.generate(prompts, [SamplingParams(max_tokens=30, ignore_eos=True, temperature=t, seed=5)
                                      for t in (0.0, 0.0, 0.7, 0.7)])
        eng.runner.cache.check()
        assert not eng.runner.cache.requests
        results.append((outs, eng.scheduler.num_evictions))
    (big, ev_big), (small, ev_small) = results
    assert ev_big == 0 and ev_small > 0
    for a, b in zip(big, small):
        assert a.token_ids == b.token_ids and len(a.token_ids) == 30
    assert max(o.evictions for o in small) >= 1


def test_command_line(folders, tmp_path):
    import json
    import subprocess
    import sys
    import os
    name = "A"
    env = dict(os.environ, MODEL_PATH=str(folders[name]))
    cmd = [sys.executable, os.path.join(H.ROOT, "bin", "ginfer"), "generate", "--dtype", "float32", "--prompt-ids", "5,17,3",
           "--prompt-ids", "9 8 7 6", "--max-tokens", "6", "--ignore-eos", "--max-num-seqs", "2", "--max-seq-len", "64",
           "--num-kvcache-blocks", "16"]
    out = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    lines = [json.loads(l) for l in out.stdout.strip().splitlines()]
    cfg, w = pm.read_config(folders[name]), pm.read_weights(folders[name])
    assert [l["token_ids"] for l in lines] == [pm.generate(cfg, w, p, 6, ignore_eos=True) for p in ([5, 17, 3], [9, 8, 7, 6])]
    assert "decode=" in out.stderr and "ttft=" in out.stderr
    # without a folder: the configuration alone, weights drawn on the device; the same seed gives the same tokens
    runs = []
    for _ in range(2):
        cmd = [sys.executable, os.path.join(H.ROOT, "bin", "ginfer"), "generate", "--random-config",
               os.path.join(str(folders[name]), "config.json"), "--weights-seed", "3", "--dtype", "float32", "--prompt-ids", "5,17,3",
               "--max-tokens", "4", "--ignore-eos", "--max-num-seqs", "2", "--max-seq-len", "64", "--num-kvcache-blocks", "16"]
        out = subprocess.run(cmd, env=dict(os.environ, MODEL_PATH=""), capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr
        runs.append(json.loads(out.stdout.strip().splitlines()[0])["token_ids"])
    assert runs[0] == runs[1] and len(runs[0]) == 4
    # the benchmark with requests that arrive while the engine runs
    cmd = [sys.executable, os.path.join(H.ROOT, "bin", "ginfer"), "benchmark", "--random-config",
           os.path.join(str(folders[name]), "config.json"), "--dtype", "bfloat16", "--num-prompts", "12", "--prompt-len", "9",
           "--max-tokens", "5", "--request-rate", "2000", "--max-num-seqs", "4", "--max-num-batched-tokens", "32",
           "--max-seq-len", "64", "--num-kvcache-blocks", "32"]
    out = subprocess.run(cmd, env=dict(os.environ, MODEL_PATH=""), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    rep = json.loads(out.stdout.strip().splitlines()[-1])
    assert rep["total_tokens"] == 12 * (9 + 5) and rep["ttft_ms"]["p50"] > 0 and rep["tpot_ms"]["mean"] > 0
    assert sum(rep["ran"][k] for k in ("launched", "replayed_decode", "replayed_padded")) >= rep["steps"]


def test_real_layer_sizes(tmp_path):
    """Two layers of the 1.5B shape (width 1536, 12 heads in 2 groups of head size 128, feed-forward 8960,
    vocabulary 151,936): the sizes the kernels serve, cut and batched in every way, in both dtypes."""
    from ginfer_amd import ModelRunner
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=1536, num_attention_heads=12,
               num_key_value_heads=2, intermediate_size=8960, vocab_size=151936, rope_theta=10000.0, rms_norm_eps=1e-6,
               tie_word_embeddings=False, max_position_embeddings=4096, use_sliding_window=False, sliding_window=4096,
               max_window_layers=21)
    folder = H.make_model_folder(tmp_path / "real", cfg, 3, "float32")
    reqs = {"a": H.random_tokens(150, 151936, 1), "b": H.random_tokens(70, 151936, 2), "c": H.random_tokens(40, 151936, 3)}
    pcfg, w = pm.read_config(folder), pm.read_weights(folder, torch.float32)
    refs = {rid: pm.forward(pcfg, w, ids).numpy() for rid, ids in reqs.items()}
    del w
    want_last = 34          # logits of the last places only: the vocabulary is wide
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner(folder, dtype=dtype, page_size=16, num_pages=24, max_requests=4)
        for what, steps in (("whole", H.steps_whole(reqs)), ("last 32 decoded", H.steps_last_decoded(reqs)),
                            ("mixed", H.steps_mixed(reqs, max_live=3, seed=2))):
            at = {}
            for st in steps:                # keep only the wanted places that lie near the end of a request
                for e in st["entries"]:
                    base = at.get(e["id"], 0)
                    e["want"] = [i for i in range(len(e["tokens"])) if base + i >= len(reqs[e["id"]]) - want_last]
                    at[e["id"]] = base + len(e["tokens"])
            got = H.run_steps(runner, steps)
            runner.cache.check()
            assert len(got) == 3 * want_last
            for (rid, p), row in got.items():
                ref = refs[rid]
                err = np.abs(row - ref[p]).max() / np.abs(ref).max()
                # the plain run is itself 32-bit here: both sides round, so twice the 32-bit tolerance
                assert err <= (2 * H.TOL[dtype] if dtype == "float32" else H.TOL[dtype]), \
                    "%s %s: request %s position %d: %.3g" % (dtype, what, rid, p, err)
        del runner
        torch.cuda.empty_cache()
    # recorded decode steps at these sizes (40 rows: the wide products go to the BLAS library) against the
    # same steps launched eagerly, several replays with eager steps between them
    from ginfer_amd import StepEntry
    outs = [[], []]
    stream = H.random_tokens(40 * 12, 151936, 77)
    for k, graphs in enumerate((True, False)):
        # only the decode steps are recorded here: a recorded step with a prompt portion has other row counts than the
        # same step launched kernel by kernel, and in bfloat16 the library then rounds differently
        r = ModelRunner(folder, dtype="bfloat16", page_size=16, num_pages=120, max_requests=41, use_graphs=graphs,
                        graph_mixed_steps=False)
        r.step([StepEntry(i, H.random_tokens(3 + i % 9, 151936, 100 + i), []) for i in range(40)])
        for stepno in range(10):
            outs[k].append(r.step([StepEntry(i, [stream[stepno * 40 + i]], [0]) for i in range(40)]).cpu())
            if stepno in (3, 6):
                outs[k].append(r.step([StepEntry("p", H.random_tokens(70, 151936, stepno), [69])]).cpu())
                r.release("p")
        assert bool(r._graphs) == graphs
        del r
        torch.cuda.empty_cache()
    for n, (a, b) in enumerate(zip(*outs)):
        assert torch.equal(a, b), "real sizes, step %d: a replayed step differs from the eager step by %.3g" % (
            n, float((a - b).abs().max() / b.abs().max()))


def test_recorded_shapes_are_bounded(folders, monkeypatch):
    """Every batch size gets a graph of its own; only the most recently used are kept."""
    from ginfer_amd import ModelRunner, StepEntry
    from ginfer_amd.kernels.tuning import TUNING
    monkeypatch.setattr(TUNING, "graph_keep", 3)
    r = ModelRunner(folders["A"], dtype="bfloat16", page_size=16, num_pages=64, max_requests=8)
    ref = ModelRunner(folders["A"], dtype="bfloat16", page_size=16, num_pages=64, max_requests=8, use_graphs=False)
    toks = H.random_tokens(400, 512, 5)
    at = 0
    for n in (1, 2, 3, 4, 5, 2, 1, 6):
        for _ in range(3):
            batch = [StepEntry(i, [toks[at + i]], [0]) for i in range(n)]
            at += n
            assert torch.equal(r.step(batch), ref.step(batch))
        assert len(r._graphs) <= 3
    assert len(r._graphs) == 3 and (6, 256) in r._graphs


@pytest.mark.parametrize("name,seed", [("C", 1), ("A", 2)])
def test_random_workload_through_the_engine(folders, name, seed):
    """A dozen requests of random lengths and sampling settings through scheduler, cache and kernels with a
    pool that forces evictions (and, for C, windows that give pages back): in 32-bit every request's tokens
    are the plain implementation's."""
    import random
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    from ginfer_amd.sampling import uniform
    rng = random.Random(seed)
    cfgd, _, ps = H.TINY[name]
    vocab = cfgd["vocab_size"]
    prompts = [H.random_tokens(rng.randint(1, 60), vocab, 1000 + i) for i in range(12)]
    params = [SamplingParams(max_tokens=rng.randint(1, 20), ignore_eos=True, temperature=rng.choice([0.0, 0.0, 0.9]),
                             seed=rng.randint(0, 99)) for _ in prompts]
    eng = Engine(EngineConfig(model_path=folders[name], dtype="float32", max_num_batched_tokens=40, max_num_seqs=4,
                              max_seq_len=96, kvcache_block_size=ps, num_kvcache_blocks=(96 // ps) * 2 + 1))
    outs = eng.generate(prompts, params)
    eng.runner.cache.check()
    assert not eng.runner.cache.requests
    cfg, w = pm.read_config(folders[name]), pm.read_weights(folders[name])
    for i, (p, sp, o) in enumerate(zip(prompts, params, outs)):
        assert len(o.token_ids) == sp.max_tokens
        logits = pm.forward(cfg, w, (p + o.token_ids)[:-1])
        for k, tok in enumerate(o.token_ids):
            row, u = logits[len(p) - 1 + k], uniform(sp.seed, k)
            want = pm.sample_token(row, sp.temperature, u)
            assert want == tok or _is_a_tie(row, sp.temperature, u, tok, want), \
                "request %d, its token %d: %d, the plain implementation has %d" % (i, k, tok, want)
    assert eng.scheduler.num_evictions > 0, "the pool was meant to be too small"


def _is_a_tie(row, temperature, u, got, want):
    """Whether `got` in place of `want` is a matter of the last bits: the two best logits all but equal for greedy
    sampling, the uniform number all but on the border between the two tokens' shares otherwise."""
    row = row.double()
    if temperature == 0:
        top = torch.topk(row, 2)
        return ({got, want} == set(top.indices.tolist())
                and float(top.values[0] - top.values[1]) < 1e-5 * float(row.abs().max()))
    if abs(got - want) != 1:
        return False
    cdf = torch.cumsum(torch.softmax(row / temperature, 0), 0)
    return abs(u - float(cdf[min(got, want)])) < 1e-6


@pytest.mark.parametrize("name,seed", [("A", 20), ("B", 4), ("B", 23), ("C", 27)])
def test_requests_that_arrive_and_are_aborted_while_others_run(sharp_folders, name, seed):
    """Sixteen requests, some with a common beginning, come in while others run; now and then one is aborted; the
    pool holds little more than one full request, and steps are launched ahead in most runs.  In 32-bit every
    token of every request, the aborted ones' too, is the plain implementation's, a tie in the last bits aside."""
    import random
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    from ginfer_amd.sampling import uniform
    cfgd, _, ps = H.TINY[name]
    vocab = cfgd["vocab_size"]
    rng = random.Random(seed * 7 + 1)
    common = H.random_tokens(rng.randint(8, 40), vocab, 5000 + seed)
    prompts = []
    for i in range(16):
        p = H.random_tokens(rng.randint(1, 50), vocab, 6000 + 100 * seed + i)
        prompts.append((common + p) if rng.random() < 0.4 else p)
    params = [SamplingParams(max_tokens=rng.randint(1, 24), ignore_eos=True, temperature=rng.choice([0.0, 0.0, 0.8]),
                             seed=rng.randint(0, 99)) for _ in prompts]
    eng = Engine(EngineConfig(model_path=sharp_folders[name], dtype="float32",
                              max_num_batched_tokens=rng.choice([24, 48, 200]), max_num_seqs=rng.choice([3, 5, 8]),
                              max_seq_len=128, kvcache_block_size=ps,
                              num_kvcache_blocks=(128 // ps) + rng.choice([1, 3, 8]),
                              pipeline_decode=rng.random() < 0.7))
    pending = list(range(len(prompts)))
    ids, done, aborted = {}, {}, {}
    steps = 0
    while pending or eng.has_unfinished():
        while pending and (rng.random() < 0.5 or not eng.has_unfinished()):
            i = pending.pop(0)
            ids[eng.add_request(prompts[i], params[i])] = i
        for o in eng.step():
            done[o.request_id] = o
        steps += 1
        if rng.random() < 0.03:
            alive = [r for r in ids if r not in done and r not in aborted]
            if alive:
                r = rng.choice(alive)
                out = eng.abort(r)
                if out is not None:
                    aborted[r] = out
        assert steps < 5000
    eng.runner.cache.check()
    assert not eng.runner.cache.requests
    cfg, w = pm.read_config(sharp_folders[name]), pm.read_weights(sharp_folders[name])
    for r, i in ids.items():
        o = done.get(r) or aborted[r]
        if r in done:
            assert len(o.token_ids) == params[i].max_tokens
        if not o.token_ids:
            continue
        logits = pm.forward(cfg, w, (prompts[i] + o.token_ids)[:-1])
        for k, tok in enumerate(o.token_ids):
            row, u = logits[len(prompts[i]) - 1 + k], uniform(params[i].seed, k)
            want = pm.sample_token(row, params[i].temperature, u)
            assert want == tok or _is_a_tie(row, params[i].temperature, u, tok, want), \
                "request %d, its token %d: %d, the plain implementation has %d" % (i, k, tok, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_fit_no_vector_width(tmp_path, dtype):
    """A width of 50, a feed-forward of 100 and a vocabulary of 333: nothing is a multiple of 8, so the
    kernels' scalar paths and the fall-backs of the matrix products run."""
    from ginfer_amd import ModelRunner
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=50, num_attention_heads=3,
               num_key_value_heads=1, head_dim=16, intermediate_size=100, vocab_size=333, rope_theta=1e4,
               rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=128)
    folder = H.make_model_folder(tmp_path / "odd", cfg, 5, "float32")
    reqs = {"a": H.random_tokens(70, 333, 1), "b": H.random_tokens(33, 333, 2), "c": H.random_tokens(9, 333, 3)}
    runner = ModelRunner(folder, dtype=dtype, page_size=16, num_pages=12, max_requests=4)
    for what, steps in (("whole", H.steps_whole(reqs)), ("mixed", H.steps_mixed(reqs, max_live=3, seed=4)),
                        ("last 32 decoded", H.steps_last_decoded(reqs))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        H.compare_with_plain(got, reqs, folder, H.TOL[dtype], "odd sizes %s %s" % (dtype, what))


def _drawn_configuration(seed):
    """A configuration of the architecture drawn at random: every size and option varies."""
    import random
    rng = random.Random(seed)
    nkv = rng.choice([1, 1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 7])
    hd = 16 * rng.randint(1, 6)
    layers = rng.randint(1, 3)
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=layers, hidden_size=rng.randint(17, 130),
               num_attention_heads=nkv * group, num_key_value_heads=nkv, head_dim=hd,
               intermediate_size=rng.randint(16, 200), vocab_size=rng.randint(50, 700),
               rope_theta=rng.choice([1e4, 1e6, 5e5]), rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]),
               tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=rng.choice([96, 128, 512]))
    if rng.random() < 0.5:
        cfg.update(use_sliding_window=True, sliding_window=rng.randint(3, 40), max_window_layers=rng.randint(0, layers))
    return cfg, rng.choice([8, 16, 32])


@pytest.mark.parametrize("head_dim", [2, 8, 12, 24, 36, 40, 100, 200])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_sizes_between_the_steps_of_16(tmp_path, dtype, head_dim):
    """Even head sizes that are no multiple of 16 go to the general attention kernel in both dtypes."""
    from ginfer_amd import ModelRunner
    cfg = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=72, num_attention_heads=4,
               num_key_value_heads=2, head_dim=head_dim, intermediate_size=120, vocab_size=300, rope_theta=1e4,
               rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=128)
    folder = H.make_model_folder(tmp_path / "hd", cfg, 7, "float32")
    reqs = {"a": H.random_tokens(75, 300, 1), "b": H.random_tokens(34, 300, 2)}
    runner = ModelRunner(folder, dtype=dtype, page_size=16, num_pages=10, max_requests=2)
    for what, steps in (("whole", H.steps_whole(reqs)), ("mixed", H.steps_mixed(reqs, max_live=2, seed=1)),
                        ("last 32 decoded", H.steps_last_decoded(reqs))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        H.compare_with_plain(got, reqs, folder, H.TOL[dtype], "head size %d %s %s" % (head_dim, dtype, what))
    if head_dim == 24:
        # as in serving (only an entry's last place wanted), twice over, so that the steps are laid into recorded steps
        # of padded sizes: the general attention kernel meets the padding rows too
        steps = H.steps_mixed(reqs, max_live=2, seed=1) + H.steps_mixed({k + "x": v for k, v in reqs.items()}, max_live=2, seed=1)
        for st in steps:
            for e in st["entries"]:
                e["want"] = [len(e["tokens"]) - 1]
        got = H.run_steps(runner, steps)
        assert any(k[0] == "padded" for k in runner._graphs)
        both = dict(reqs)
        both.update({k + "x": v for k, v in reqs.items()})
        refs = {rid: H.plain_logits(folder, ids) for rid, ids in both.items()}
        for (rid, p), row in got.items():
            err = float(np.abs(row.astype(np.float64) - refs[rid][p]).max() / np.abs(refs[rid]).max())
            assert np.isfinite(row).all() and err <= H.TOL[dtype], "head size 24 %s padded: %s %d: %.3g" % (dtype, rid, p, err)


@pytest.mark.parametrize("seed", list(range(8)))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    """Whole, mixed with so few pages that they are used again, and the last tokens one by one, for configurations
    nobody chose: heads, groups, widths, windows, page sizes."""
    from ginfer_amd import ModelRunner
    cfg, page = _drawn_configuration(seed)
    folder = H.make_model_folder(tmp_path / "drawn", cfg, seed, "float32")
    V = cfg["vocab_size"]
    reqs = {"a": H.random_tokens(90, V, 10 + seed), "b": H.random_tokens(41, V, 20 + seed),
            "c": H.random_tokens(1 + seed, V, 30 + seed), "d": H.random_tokens(64, V, 40 + seed)}
    mixed = H.steps_mixed(reqs, max_live=3, seed=seed)
    pages = -(-H.max_live_tokens(mixed) // page)
    runner = ModelRunner(folder, dtype=dtype, page_size=page, num_pages=pages, max_requests=4)
    for what, steps in (("mixed", mixed), ("whole", H.steps_whole(reqs)), ("last decoded", H.steps_last_decoded(reqs))):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        H.compare_with_plain(got, reqs, folder, H.TOL[dtype], "drawn %d %s %s %s" % (seed, dtype, what, cfg))


@pytest.mark.parametrize("live", [6, 12, 40])
def test_layer_sizes_of_a_7b_model_decoding_together(tmp_path, live):
    """Two layers of a 7B shape (width 3584, 28 heads in 4 groups, feed-forward 18944) with 6, 12 and 40 requests
    decoding side by side: the products' plans for wider matrices (no packed tiles, norms folded up to 16 rows,
    K split in few parts), against the plain implementation."""
    from ginfer_amd import ModelRunner
    V = 1500
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
    runner = ModelRunner(folder, dtype="bfloat16", page_size=16, num_pages=2 * live, max_requests=live)
    got = H.run_steps(runner, steps)
    runner.cache.check()
    pcfg, w = pm.read_config(folder), pm.read_weights(folder, torch.float32)
    for rid in list(reqs)[:3] + list(reqs)[-2:]:
        ref = pm.forward(pcfg, w, reqs[rid]).numpy()
        for p in range(prompt - 1, prompt + decoded):
            err = np.abs(got[(rid, p)] - ref[p]).max() / np.abs(ref).max()
            assert err <= H.TOL["bfloat16"], "request %s position %d: %.3g" % (rid, p, err)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_ahead_change_nothing(folders, dtype):
    """While every running request decodes, the engine launches the next step before it has read the tokens
    of this one.  The tokens are the same as without that, bit for bit: greedy and sampled requests, requests that
    stop on a token nobody had seen when the step after it was launched, requests that reach max_tokens, and
    others arriving while the pipeline runs."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "B"
    vocab = H.TINY[name][0]["vocab_size"]
    prompts = [H.random_tokens(n, vocab, 900 + n) for n in (5, 17, 33, 9, 12, 21, 3, 40)]

    def run(pipeline):
        eng = Engine(EngineConfig(model_path=folders[name], dtype=dtype, max_num_batched_tokens=64, max_num_seqs=5,
                                  max_seq_len=128, kvcache_block_size=8, num_kvcache_blocks=80, pipeline_decode=pipeline,
                                  graph_mixed_steps=False))     # the two runs cut their steps differently: in bfloat16
        #                                                          a padded step rounds otherwise than a step of few rows
        free = eng.generate(prompts[:2], SamplingParams(max_tokens=12, ignore_eos=True))      # to find tokens to stop on
        stops = sorted({o.token_ids[5] for o in free} | {o.token_ids[8] for o in free})
        params = [SamplingParams(max_tokens=m, temperature=t, seed=7, ignore_eos=False, stop_token_ids=stops if st else None)
                  for m, t, st in ((12, 0.0, True), (12, 0.0, True), (25, 0.8, False), (7, 0.0, False), (30, 0.0, True),
                                   (1, 0.0, False), (16, 1.1, True), (20, 0.0, False))]
        ids = [eng.add_request(p, sp) for p, sp in zip(prompts[:5], params[:5])]
        done, steps = {}, 0
        while eng.has_unfinished():
            for o in eng.step():
                done[o.request_id] = o
            steps += 1
            if steps == 6:             # three more arrive while the others decode
                ids += [eng.add_request(p, sp) for p, sp in zip(prompts[5:], params[5:])]
        eng.runner.cache.check()
        assert not eng.runner.cache.requests
        return [(done[i].token_ids, done[i].finish_reason) for i in ids], eng.stats["steps_launched_ahead"]

    with_ahead, n_ahead = run(True)
    without, none_ahead = run(False)
    assert n_ahead > 5 and none_ahead == 0
    assert {r for _, r in with_ahead} >= {"eos", "max_tokens"}
    if dtype == "float32":
        assert with_ahead == without
        return
    # bfloat16: the two runs put other requests side by side in their steps (a step launched ahead admits nobody), and a
    # product of other row counts rounds otherwise, so a draw that lies on the border between two tokens may fall either
    # way and the request goes on differently from there.  Every token of either run must be what the plain
    # implementation draws after the run's own tokens so far, up to the bfloat16 tolerance on the logits (greedy) or
    # on the token's share of the probability (sampled).
    from ginfer_amd.sampling import uniform
    cfg, w = pm.read_config(folders[name]), pm.read_weights(folders[name])
    settings = ((12, 0.0), (12, 0.0), (25, 0.8), (7, 0.0), (30, 0.0), (1, 0.0), (16, 1.1), (20, 0.0))
    for what, run_tokens in (("launched ahead", with_ahead), ("one by one", without)):
        for i, ((toks, reason), (_, temp)) in enumerate(zip(run_tokens, settings)):
            logits = pm.forward(cfg, w, (prompts[i] + toks)[:-1])
            for k, tok in enumerate(toks):
                row = logits[len(prompts[i]) - 1 + k]
                if temp == 0:
                    best = int(torch.argmax(row))
                    assert tok == best or float(row[best] - row[tok]) <= H.TOL[dtype] * float(row.abs().max()), \
                        "%s: request %d token %d: %d, plain %d" % (what, i, k, tok, best)
                else:
                    cdf = torch.cumsum(torch.softmax(row / temp, 0), 0)
                    lo, hi, u = (float(cdf[tok - 1]) if tok else 0.0), float(cdf[tok]), uniform(7, k)
                    assert lo - H.TOL[dtype] <= u <= hi + H.TOL[dtype], \
                        "%s: request %d token %d: %d holds [%.4f, %.4f], the draw is %.4f" % (what, i, k, tok, lo, hi, u)


def test_weights_drawn_on_the_device():
    """A model without a folder: a configuration and a seed, every tensor drawn on the device.  The same seed
    gives the same logits, another seed others; cutting a request changes nothing."""
    from ginfer_amd import ModelRunner, StepEntry, config_from_dict
    cfg = config_from_dict(H.TINY_B)
    ids = H.random_tokens(40, 1000, 5)
    outs = []
    for seed in (3, 3, 4):
        r = ModelRunner(None, dtype="float32", page_size=8, num_pages=16, max_requests=2, config=cfg, random_seed=seed)
        whole = r.step([StepEntry("a", ids, [39])]).cpu()
        r.release("a")
        r.step([StepEntry("a", ids[:17], [])])
        cut = r.step([StepEntry("a", ids[17:], [22])]).cpu()
        assert torch.isfinite(whole).all() and torch.equal(whole, cut)
        outs.append(whole)
        del r
    assert torch.equal(outs[0], outs[1]) and not torch.equal(outs[0], outs[2])
    with pytest.raises(ValueError):
        ModelRunner(None, dtype="float32", config=cfg)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_weights_drawn_on_the_device_are_the_bits_the_host_writes(tmp_path, dtype):
    """One generator for host and device: a model whose weights are drawn on the device holds, tensor by tensor and bit
    for bit, what the model folder written for the same seed holds, so a model that never passed through a file still
    has its plain twin; and the device's draws have the distribution that is claimed for them."""
    from ginfer_amd import ModelRunner, StepEntry, config_from_dict, write_random_model
    from ginfer_amd.kernels import ops
    from safetensors import safe_open
    from scipy import stats
    cfg = config_from_dict(H.TINY_C)
    folder = write_random_model(str(tmp_path / "m"), cfg, 7, dtype)
    drawn = ModelRunner(None, dtype=dtype, page_size=16, num_pages=8, max_requests=2, config=cfg, random_seed=7)
    loaded = ModelRunner(folder, dtype=dtype, page_size=16, num_pages=8, max_requests=2)
    for (name, a), (_, b) in zip(drawn.model._named_parts(), loaded.model._named_parts()):
        tensors = [(k, v) for k, v in vars(a).items() if isinstance(v, torch.Tensor)]
        assert tensors or not a.weight_specs(), name
        for k, v in tensors:
            assert v.dtype == getattr(b, k).dtype and torch.equal(v, getattr(b, k)), "%s.%s differs" % (name, k)
    ids = H.random_tokens(50, 777, 3)
    got = drawn.step([StepEntry("a", ids, [49])]).cpu()
    assert torch.equal(got, loaded.step([StepEntry("a", ids, [49])]).cpu())
    ref = H.plain_logits(folder, ids)[49]
    assert H.rel_err(got[0].numpy(), ref) <= H.TOL[dtype]
    # the draws themselves: a million numbers of one key against the normal distribution, and against the host's
    x = torch.empty(1 << 20, dtype=torch.float32, device=drawn.device)
    ops.random_normal_fill(x, 99, 0.5, 0.02)
    x = x.cpu().double().numpy()
    assert abs(x.mean() - 0.5) < 1e-4 and abs(x.std() - 0.02) < 1e-4
    z = (x - 0.5) / 0.02
    assert stats.kstest(z, "norm").pvalue > 1e-3 and abs((z ** 4).mean() - 3.0) < 0.05 and abs((z ** 3).mean()) < 0.02
    assert np.abs(np.corrcoef(z[:-1], z[1:])[0, 1]) < 5e-3           # neighbours are not correlated


def test_abort_in_the_middle_leaves_the_others_untouched(folders):
    """A request is ended from outside while steps launched ahead are on the device: it keeps what it has, its pages
    go back, and the other requests generate what they generate alone."""
    from ginfer_amd import Engine, EngineConfig, SamplingParams
    name = "A"
    eng = Engine(EngineConfig(model_path=str(folders[name]), dtype="float32", max_num_batched_tokens=32, max_num_seqs=4,
                              max_seq_len=128, kvcache_block_size=16, num_kvcache_blocks=24))
    prompts = [H.random_tokens(n, 512, 60 + n) for n in (9, 21, 14)]
    ids = [eng.add_request(p, SamplingParams(max_tokens=24, ignore_eos=True)) for p in prompts]
    done = {}
    for _ in range(8):
        for o in eng.step():
            done[o.request_id] = o
    out = eng.abort(ids[1])
    assert out is not None and out.finish_reason == "aborted" and 0 < len(out.token_ids) < 24
    assert eng.abort(ids[1]) is None
    while eng.has_unfinished():
        for o in eng.step():
            done[o.request_id] = o
    cfg, w = pm.read_config(folders[name]), pm.read_weights(folders[name])
    for k in (0, 2):
        assert done[ids[k]].token_ids == pm.generate(cfg, w, prompts[k], 24, ignore_eos=True)
    assert out.token_ids == pm.generate(cfg, w, prompts[1], 24, ignore_eos=True)[:len(out.token_ids)]
    eng.runner.cache.check()
    assert not eng.runner.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_recorded_steps_with_prompt_portions(folders, sharp_folders, name, dtype):
    """Steps that hold prompt portions are laid into recorded steps of padded sizes.  In 32-bit they give the bits of
    the same steps launched one kernel at a time (every sum has a fixed order, whatever the number of rows); in
    bfloat16 both agree with the plain implementation.  The cache they leave is the same: the decoding that follows
    agrees too."""
    from ginfer_amd import ModelRunner
    folder = sharp_folders[name]
    cfg, seed, page = H.TINY[name]
    V = cfg["vocab_size"]
    reqs = {"r%d" % i: H.random_tokens(n, V, 300 + i) for i, n in enumerate([70, 45, 90, 33, 58, 77])}
    steps = H.steps_mixed(reqs, max_live=4, seed=11) + H.steps_mixed({k + "x": v for k, v in reqs.items()}, max_live=4, seed=11)
    both = dict(reqs)
    both.update({k + "x": v for k, v in reqs.items()})
    for st in steps:                 # as in serving: at most the last place of an entry is wanted
        for e in st["entries"]:
            e["want"] = [len(e["tokens"]) - 1]
    pages = -(-H.max_live_tokens(steps) // page)
    got = {}
    for mixed in (True, False):
        runner = ModelRunner(folder, dtype=dtype, page_size=page, num_pages=pages, max_requests=8, graph_mixed_steps=mixed)
        got[mixed] = H.run_steps(runner, steps)
        runner.cache.check()
        padded = [k for k in runner._graphs if k[0] == "padded"]
        assert bool(padded) == mixed, "recorded shapes: %s" % list(runner._graphs)
        del runner
    assert got[True].keys() == got[False].keys()
    if dtype == "float32":
        for k in got[True]:
            assert np.array_equal(got[True][k], got[False][k]), "request %s position %d differs in a recorded step" % k
    refs = {rid: H.plain_logits(folder, ids) for rid, ids in both.items()}
    for (rid, p), row in got[True].items():
        err = float(np.abs(row.astype(np.float64) - refs[rid][p]).max() / np.abs(refs[rid]).max())
        assert np.isfinite(row).all() and err <= H.TOL[dtype], "%s %s: request %s position %d: error %.3g" % (name, dtype, rid, p, err)


def test_the_pool_is_planned_from_free_memory_after_the_largest_step(folders, monkeypatch):
    """The pool is sized from what is free once the weights are loaded and the largest step has run (the order of
    ginfer/engine/model_runner.cc:52-70); layers with a window get the pages a window can hold and nearly all of the
    pool keeps all keys; a utilization that leaves the largest step no room is refused."""
    from ginfer_amd import ModelRunner, Engine, EngineConfig, SamplingParams
    from ginfer_amd.cache import CacheManager
    real = torch.cuda.mem_get_info
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a, **k: (64 << 20, real(*a, **k)[1]))     # as if 64 MB were free
    # the largest step's own needs come to more than the 10 % of 64 MB: refused, and the message says what would fit
    with pytest.raises(ValueError, match="gpu_memory_utilization 0.999 leaves"):
        ModelRunner(folders["C"], dtype="bfloat16", page_size=16, max_requests=4, max_model_len=384,
                    max_num_batched_tokens=128, gpu_memory_utilization=0.999)
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a, **k: (1 << 30, real(*a, **k)[1]))      # as if 1 GB were free
    r = ModelRunner(folders["C"], dtype="bfloat16", page_size=16, max_requests=4, max_model_len=384,
                    max_num_batched_tokens=128, gpu_memory_utilization=0.5)
    plan = r.memory_plan
    assert plan["free_bytes"] == 1 << 30 and plan["pool_bytes"] == 1 << 29 and plan["step_peak_bytes"] > 0
    groups = r.cache.groups
    assert [g.pool.num_pages for g in groups] == plan["pages"]
    all_keys = [g for g in groups if g.window is None]
    windowed = [g for g in groups if g.window is not None]
    assert len(all_keys) == 1 and len(windowed) == 1           # layer 0 keeps all keys, layers 1 to 3 a window of 40
    assert windowed[0].pool.num_pages == CacheManager.window_pages(40, 16, 4, 128, 384) \
        == 4 * (CacheManager.window_span_pages(40, 16) + 1) + 128 // 16
    per_page = lambda g: len(g.entries) * 2 * g.spec.num_kv_heads * 16 * g.spec.head_dim * 2
    assert all_keys[0].pool.num_pages * per_page(all_keys[0]) > 0.9 * plan["pool_bytes"]
    assert r.cache.pool_bytes(2) <= plan["pool_bytes"]
    del r
    monkeypatch.undo()
    torch.cuda.empty_cache()
    # through the engine, with pages from free memory: requests longer than the window, tokens as the plain model's
    eng = Engine(EngineConfig(model_path=folders["C"], dtype="float32", max_num_batched_tokens=48, max_num_seqs=3,
                              max_seq_len=200, gpu_memory_utilization=0.05))
    prompts = [H.random_tokens(n, 777, 40 + n) for n in (90, 7, 130)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    _greedy_as_plain(folders["C"], prompts, outs, "float32")
    eng.runner.cache.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.runner.cache.groups)
