"""Each part alone against its plain function, and the generality of the assembly: a toy mixer with
state of its own, a layer named twice, a layer that reads another layer's cache."""
import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import helpers as H
import plain_model as pm

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g) * scale


def close(got, ref, tol):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
    assert err <= tol, "error %.3g > %.3g" % (err, tol)


PART_DTYPES = [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)]


@pytest.mark.parametrize("dtype,tol", PART_DTYPES)
@pytest.mark.parametrize("T", [1, 7, 200, 512, 768])     # 512, 768: the product with the weights first, transposed
def test_swiglu_part(dtype, tol, T):
    from ginfer_amd.parts import lookup
    Hd, I = 88, 136
    part = lookup("feed_forward", "swiglu")(hidden_size=Hd, intermediate_size=I, dtype=dtype, device=dev())
    w = {n: rnd(s.shape, i, 0.1).to(dtype) for i, (n, s) in enumerate(part.weight_specs().items())}
    part.bind_weights({n: t.to(dev()) for n, t in w.items()})
    x = rnd((T, Hd), 9).to(dtype)
    wd = {"p." + n: t.double() for n, t in w.items()}
    ref = pm.feed_forward(x.double(), wd, "p")
    close(part.forward(x.to(dev())), ref, tol)


@pytest.mark.parametrize("dtype,tol", PART_DTYPES)
def test_norm_part(dtype, tol):
    from ginfer_amd.parts import lookup
    part = lookup("norm", "rmsnorm")(size=96, eps=1e-5, dtype=dtype, device=dev())
    g = (1 + rnd((96,), 1, 0.1)).to(dtype)
    part.bind_weights({"weight": g.to(dev())})
    res, delta = rnd((11, 96), 2), rnd((11, 96), 3).to(dtype)
    ref = pm.rms_norm(res.double() + delta.double(), g.double(), 1e-5)
    r = res.to(dev())
    close(part.forward(r, delta.to(dev())), ref, tol)
    close(r, res.double() + delta.double(), 1e-6)


@pytest.mark.parametrize("dtype,tol", PART_DTYPES)
@pytest.mark.parametrize("tied", [True, False])
def test_embedding_and_head_parts(dtype, tol, tied):
    from ginfer_amd.parts import lookup
    V, Hd = 301, 72
    emb = lookup("embedding", "embedding")(vocab_size=V, hidden_size=Hd, dtype=dtype, device=dev())
    head = lookup("head", "lm_head")(vocab_size=V, hidden_size=Hd, tied=tied, dtype=dtype, device=dev())
    E = rnd((V, Hd), 1).to(dtype)
    emb.bind_weights({"weight": E.to(dev())})
    assert (head.weight_specs() == {}) == tied
    Wh = E if tied else rnd((V, Hd), 2).to(dtype)
    if tied:
        head.tie(emb.weight)
        assert head.weight.data_ptr() == emb.weight.data_ptr()       # one device copy
    else:
        head.bind_weights({"weight": Wh.to(dev())})
    ids = torch.tensor([0, 300, 5, 5], dtype=torch.int32)
    assert torch.equal(emb.forward(ids.to(dev())).cpu(), E[ids.long()].float())
    x = rnd((3, Hd), 4).to(dtype)
    logits = head.forward(x.to(dev()))
    assert logits.dtype == torch.float32
    close(logits, x.double() @ Wh.double().t(), 1e-5 if dtype == torch.float32 else 1e-4)


@pytest.mark.parametrize("theta,rd,n", [(1e4, 16, 300), (1e6, 128, 70), (5e5, 96, 33)])
def test_position_part(theta, rd, n):
    """The position encoding alone: its 32-bit tables equal the plain formula's, bit for bit in the angles'
    inputs (position cast to float before the multiply), and a limit cuts them without changing a value."""
    from ginfer_amd.parts import lookup
    part = lookup("position", "rope_neox")(theta=theta, rotary_dim=rd, max_positions=n, device=dev())
    cos, sin = part.tables()
    ref_sin, ref_cos = pm.rope_tables(theta, rd, n)
    assert cos.dtype == torch.float32 and cos.shape == (n, rd // 2) and sin.shape == (n, rd // 2)
    close(cos, ref_cos, 1e-6)
    close(sin, ref_sin, 1e-6)
    assert torch.equal(cos[0].cpu(), torch.ones(rd // 2)) and torch.equal(sin[0].cpu(), torch.zeros(rd // 2))
    part.limit_positions(10)
    cos10, sin10 = part.tables()
    assert cos10.shape == (10, rd // 2) and torch.equal(cos10, cos[:10]) and torch.equal(sin10, sin[:10])
    with pytest.raises(ValueError):
        lookup("position", "rope_neox")(theta=theta, rotary_dim=15, max_positions=n, device=dev())


@pytest.mark.parametrize("dtype,tol", PART_DTYPES)
@pytest.mark.parametrize("window", [None, 12])
def test_attention_part_in_portions(dtype, tol, window):
    """The mixer alone, fed one request in three portions through a hand-made cache view, equals the
    plain attention block on the whole sequence."""
    from ginfer_amd.config import PartSpec
    from ginfer_amd.parts import lookup, KVView, StepContext
    Hd, nh, nkv, hd, ps, T = 80, 4, 2, 32, 8, 45
    pos = lookup("position", "rope_neox")(theta=1e4, rotary_dim=hd, max_positions=64, device=dev())
    part = lookup("mixer", "attention")(hidden_size=Hd, num_heads=nh, num_kv_heads=nkv, head_dim=hd, qkv_bias=True,
                                        out_bias=False, window=window, position=pos, scale=None, dtype=dtype,
                                        device=dev())
    w = {n: rnd(s.shape, i, 0.15).to(dtype) for i, (n, s) in enumerate(part.weight_specs().items())}
    part.bind_weights({n: t.to(dev()) for n, t in w.items()})
    x = rnd((T, Hd), 20).to(dtype)
    cfg = dict(num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd)
    sin, cos = pm.rope_tables(1e4, hd, 64)
    ref, _ = pm.attention_block(x.double(), {"p." + n: t.double() for n, t in w.items()}, "p", cfg, list(range(T)),
                                sin, cos, window)
    pages = 8
    kp = torch.full((pages, nkv, ps, hd), float("nan"), dtype=dtype, device=dev())
    vp = torch.full((pages, nkv, hd, ps), float("nan"), dtype=dtype, device=dev())
    table = [5, 2, 7, 0, 3, 6]
    outs = []
    for a, b in ((0, 20), (20, 22), (22, 45)):
        n = b - a
        p = np.arange(a, b)
        slots = torch.tensor(np.asarray(table)[p // ps] * ps + p % ps, dtype=torch.int64, device=dev())
        view = KVView(kp, vp, torch.tensor([table], dtype=torch.int32, device=dev()), slots, ps, True)
        step = StepContext(token_ids=None, positions=torch.tensor(p, dtype=torch.int32, device=dev()),
                           token_entry=torch.zeros(n, dtype=torch.int32, device=dev()),
                           cu_tokens=torch.tensor([0, n], dtype=torch.int32, device=dev()),
                           q_start=torch.tensor([a], dtype=torch.int32, device=dev()),
                           logit_rows=None, num_tokens=n, num_entries=1, host_q_start=[a], host_q_len=[n],
                           caches=[view], extra={})
        outs.append(part.forward(x[a:b].to(dev()), step, view))
    close(torch.cat(outs), ref, tol)


@pytest.mark.parametrize("T", [1, 5, 16, 17])
def test_block_folds_the_norm_between_mixer_and_feed_forward(T):
    """With few rows the output projection adds itself to the residual and hands the second norm's rows on in
    two factors; the block's result equals the one with the norm as a kernel of its own."""
    from ginfer_amd.kernels import ops
    from ginfer_amd.parts import lookup, KVView, StepContext
    Hd, nh, nkv, hd, I, ps = 96, 3, 1, 32, 136, 8
    dtype = torch.bfloat16
    pos = lookup("position", "rope_neox")(theta=1e4, rotary_dim=hd, max_positions=64, device=dev())
    mixer = lookup("mixer", "attention")(hidden_size=Hd, num_heads=nh, num_kv_heads=nkv, head_dim=hd, qkv_bias=True,
                                         out_bias=False, window=None, position=pos, scale=None, dtype=dtype, device=dev())
    ff = lookup("feed_forward", "swiglu")(hidden_size=Hd, intermediate_size=I, dtype=dtype, device=dev())
    norms = [lookup("norm", "rmsnorm")(size=Hd, eps=1e-5, dtype=dtype, device=dev()) for _ in range(2)]
    for k, part in enumerate([mixer, ff] + norms):
        part.bind_weights({n: ((1 + rnd(sp.shape, 10 * k + i, 0.1)) if n == "weight" and part in norms
                               else rnd(sp.shape, 10 * k + i, 0.15)).to(dtype).to(dev())
                           for i, (n, sp) in enumerate(part.weight_specs().items())})
    block = lookup("arrangement", "prenorm")(dict(mixer=mixer, feed_forward=ff, mixer_norm=norms[0],
                                                  feed_forward_norm=norms[1]))
    assert block.folds
    seen = []
    inner = mixer.forward
    mixer.forward = lambda *a, **k: (seen.append(inner(*a, **k)), seen[-1])[1]
    results = []
    for folds in (True, False):
        block.folds = folds
        kp = torch.zeros((4, nkv, ps, hd), dtype=dtype, device=dev())
        vp = torch.zeros((4, nkv, hd, ps), dtype=dtype, device=dev())
        p = np.arange(T)
        table = [2, 0, 3]
        slots = torch.tensor(np.asarray(table)[p // ps] * ps + p % ps, dtype=torch.int64, device=dev())
        view = KVView(kp, vp, torch.tensor([table], dtype=torch.int32, device=dev()), slots, ps, True)
        step = StepContext(token_ids=None, positions=torch.tensor(p, dtype=torch.int32, device=dev()),
                           token_entry=torch.zeros(T, dtype=torch.int32, device=dev()),
                           cu_tokens=torch.tensor([0, T], dtype=torch.int32, device=dev()),
                           q_start=torch.tensor([0], dtype=torch.int32, device=dev()),
                           logit_rows=None, num_tokens=T, num_entries=1, host_q_start=[0], host_q_len=[T],
                           caches=[view], extra={})
        residual = rnd((T, Hd), 50).to(dev())
        delta = block.forward(residual, rnd((T, Hd), 51, 0.3).to(dtype).to(dev()), step, view)
        if delta.dim() == 3:
            delta = delta.sum(dim=0)
        results.append((residual, delta.float()))
    assert isinstance(seen[0], ops.ScaledRows) == (T <= 16)        # folded up to 16 rows, else the ordinary way
    assert not isinstance(seen[1], ops.ScaledRows)
    # the ordinary way rounds the mixer's output to bfloat16 before the add, the folded one adds the 32-bit sums
    close(results[0][0], results[1][0], 4e-3)
    close(results[0][1], results[1][1], 2e-2)


# ----------------------------------------------------------------------------- generality of the assembly

def _register_toy():
    """A toy architecture defined here, in the test: blocks whose mixer keeps a running sum of its
    inputs per request (state of fixed size, no pages) between blocks with attention, a layer that runs
    twice and a run that reads another run's keys and values."""
    from ginfer_amd.config import register_architecture, PartSpec, LayerSpec, prenorm_layer, ScheduleEntry, ModelSpec
    from ginfer_amd.parts import register_mixer, Part, StateSpec
    from ginfer_amd.weights import WeightSpec

    @register_mixer("toy_running_mean")
    class RunningMean(Part):
        """out[t] = W . mean(x[0..t]) of the request; the state is (sum, count)."""

        def __init__(self, hidden_size, dtype, device, state_pad=0):
            self.H, self.dtype, self.device, self.pad = hidden_size, dtype, device, int(state_pad)

        def cache_spec(self):
            return StateSpec((self.H + 1 + self.pad,), torch.float32)        # the padding only makes the slot large

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.H, self.H))}

        def bind_weights(self, t):
            self.w = t["mix.weight"]

        def forward(self, x, step, cache):
            out = torch.empty_like(x)
            o = 0
            for e in range(step.num_entries):
                n, start = step.host_q_len[e], step.host_q_start[e]
                slot = cache.slots[e]
                if start == 0:
                    cache.state[slot] = 0
                st = cache.state[slot]
                sums = st[:self.H] + torch.cumsum(x[o:o + n].float(), dim=0)
                counts = st[self.H] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                out[o:o + n] = ((sums / counts[:, None]).to(self.dtype) @ self.w.t())
                cache.state[slot, :self.H] = sums[-1]
                cache.state[slot, self.H] = counts[-1]
                o += n
            return out

    @register_architecture("ToyStateLM")
    @dataclass
    class ToyConfig:
        hidden_size: int = 48
        vocab_size: int = 211
        state_pad: int = 0
        architecture = "ToyStateLM"

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"], d.get("state_pad", 0))

        def to_dict(self):
            return dict(architectures=["ToyStateLM"], hidden_size=self.hidden_size, vocab_size=self.vocab_size,
                        state_pad=self.state_pad)

        def model_spec(self):
            Hd = self.hidden_size
            norm = PartSpec("rmsnorm", dict(size=Hd, eps=1e-5))
            pos = PartSpec("rope_neox", dict(theta=1e4, rotary_dim=16, max_positions=256))
            attn = PartSpec("attention", dict(hidden_size=Hd, num_heads=3, num_kv_heads=1, head_dim=16, qkv_bias=True,
                                              out_bias=False, window=None, position=pos, scale=None))
            toy = PartSpec("toy_running_mean", dict(hidden_size=Hd, state_pad=self.state_pad))
            ffn = PartSpec("swiglu", dict(hidden_size=Hd, intermediate_size=80))
            layers = [prenorm_layer("model.layers.%d" % i, m, ffn, norm, norm, names=H.LAYER_NAMES) for i, m in enumerate([attn, toy, attn])]
            # layer 0, the toy layer, layer 2 reading run 0's cache, the toy layer again (a second state)
            schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2, cache_of=0), ScheduleEntry(1)]
            return ModelSpec(hidden_size=Hd, vocab_size=self.vocab_size, layers=layers, schedule=schedule,
                             embedding=PartSpec("embedding", dict(vocab_size=self.vocab_size, hidden_size=Hd)),
                             final_norm=norm, head=PartSpec("lm_head", dict(vocab_size=self.vocab_size, hidden_size=Hd,
                                                                            tied=True)),
                             max_positions=256, eos_token_ids=[0], names=H.MODEL_NAMES)
    return ToyConfig


def _toy_plain(folder, ids):
    """The toy model on a whole sequence, written out plainly in 64-bit."""
    w = pm.read_weights(folder)
    T = len(ids)
    cfg = dict(num_attention_heads=3, num_key_value_heads=1, head_dim=16)
    sin, cos = pm.rope_tables(1e4, 16, T)
    x = pm.embedding(w["model.embed_tokens.weight"], ids)
    kept = {}
    for run, (layer, cache_of) in enumerate([(0, None), (1, None), (2, 0), (1, None)]):
        p = "model.layers.%d" % layer
        n = pm.rms_norm(x, w[p + ".input_layernorm.weight"], 1e-5)
        if layer == 1:
            mean = torch.cumsum(n, dim=0) / torch.arange(1, T + 1, dtype=n.dtype)[:, None]
            a = mean @ w[p + ".self_attn.mix.weight"].t()
        else:
            a, kv = pm.attention_block(n, w, p + ".self_attn", cfg, list(range(T)), sin, cos, None,
                                       kv_from=None if cache_of is None else kept[cache_of])
            kept[run] = kv
        h = x + a
        n = pm.rms_norm(h, w[p + ".post_attention_layernorm.weight"], 1e-5)
        x = h + pm.feed_forward(n, w, p + ".mlp")
    return pm.linear(pm.rms_norm(x, w["model.norm.weight"], 1e-5), w["model.embed_tokens.weight"]).float().numpy()


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    from ginfer_amd import ModelRunner, write_random_model, config_from_folder
    Toy = _register_toy()
    folder = write_random_model(str(tmp_path / "toy"), Toy(), seed=4, dtype="float32")
    assert type(config_from_folder(folder)).__name__ == "ToyConfig"
    reqs = {"a": H.random_tokens(50, 211, 1), "b": H.random_tokens(23, 211, 2), "c": H.random_tokens(37, 211, 3)}
    runner = ModelRunner(folder, dtype="float32", page_size=8, num_pages=16, max_requests=3)
    specs = runner.cache.cache_specs
    assert [type(s).__name__ for s in specs] == ["KVCacheSpec", "StateSpec", "NoneType", "StateSpec"]
    assert len(runner.cache.groups) == 1 and runner.cache.groups[0].entries == [0]
    for steps in (H.steps_whole(reqs), H.steps_portions(reqs, sizes=(5, 2, 11)), H.steps_mixed(reqs, max_live=3, seed=1)):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        for (rid, p), row in got.items():
            ref = _toy_plain(folder, reqs[rid])
            err = np.abs(row - ref[p]).max() / np.abs(ref).max()
            assert err < 1e-4, "request %s position %d: %.3g" % (rid, p, err)


def _register_recordable_toy():
    """The toy running mean again, written so that its forward may be recorded into a HIP graph: it reads everything
    that changes from step to step from the step's device arrays (entries' first rows, their requests' lengths, the state
    slots) and launches the same operations whatever the batch is.  Entries that are padding read and write whatever
    state slot they are given."""
    from ginfer_amd.config import register_architecture, PartSpec, LayerSpec, prenorm_layer, ScheduleEntry, ModelSpec
    from ginfer_amd.parts import register_mixer, Part, StateSpec
    from ginfer_amd.weights import WeightSpec

    @register_mixer("toy_running_mean_recordable")
    class RecordableRunningMean(Part):
        capturable = True

        def __init__(self, hidden_size, dtype, device):
            self.H, self.dtype, self.device = hidden_size, dtype, device

        def cache_spec(self):
            return StateSpec((self.H + 1,), torch.float32)

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.H, self.H))}

        def bind_weights(self, t):
            self.w = t["mix.weight"]

        def forward(self, x, step, cache):
            T, H = x.shape[0], self.H
            ent = step.token_entry.long()
            cu = step.cu_tokens.long()
            fresh = (step.q_start == 0)[:, None]
            before = torch.where(fresh, torch.zeros_like(cache.state[cache.slots]), cache.state[cache.slots])   # [entries, H + 1]
            sums0 = torch.cat([torch.zeros((1, H), dtype=torch.float32, device=x.device), torch.cumsum(x.float(), dim=0)])
            rows = torch.arange(T, device=x.device)
            sums = before[ent, :H] + sums0[rows + 1] - sums0[cu[ent]]
            counts = before[ent, H] + (rows - cu[ent] + 1).float()
            last = torch.clamp(cu[1:] - 1, min=0)            # an entry without tokens (padding) names some row: its slot is the padding's
            after = torch.cat([sums[last], counts[last][:, None]], dim=1)
            cache.state.index_copy_(0, cache.slots, after)
            return ((sums / counts[:, None]).to(self.dtype) @ self.w.t())

    @register_architecture("ToyRecordableStateLM")
    @dataclass
    class ToyRecordableConfig:
        hidden_size: int = 48
        vocab_size: int = 211
        architecture = "ToyRecordableStateLM"

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"])

        def to_dict(self):
            return dict(architectures=["ToyRecordableStateLM"], hidden_size=self.hidden_size, vocab_size=self.vocab_size)

        def model_spec(self):
            Hd = self.hidden_size
            norm = PartSpec("rmsnorm", dict(size=Hd, eps=1e-5))
            pos = PartSpec("rope_neox", dict(theta=1e4, rotary_dim=16, max_positions=256))
            attn = PartSpec("attention", dict(hidden_size=Hd, num_heads=3, num_kv_heads=1, head_dim=16, qkv_bias=True,
                                              out_bias=False, window=None, position=pos, scale=None))
            toy = PartSpec("toy_running_mean_recordable", dict(hidden_size=Hd))
            ffn = PartSpec("swiglu", dict(hidden_size=Hd, intermediate_size=80))
            layers = [prenorm_layer("model.layers.%d" % i, m, ffn, norm, norm, names=H.LAYER_NAMES) for i, m in enumerate([attn, toy, attn])]
            schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2, cache_of=0), ScheduleEntry(1)]
            return ModelSpec(hidden_size=Hd, vocab_size=self.vocab_size, layers=layers, schedule=schedule,
                             embedding=PartSpec("embedding", dict(vocab_size=self.vocab_size, hidden_size=Hd)),
                             final_norm=norm, head=PartSpec("lm_head", dict(vocab_size=self.vocab_size, hidden_size=Hd,
                                                                            tied=True)),
                             max_positions=256, eos_token_ids=[0], names=H.MODEL_NAMES)
    return ToyRecordableConfig


def test_state_of_a_live_request_survives_the_padding_of_recorded_steps(tmp_path):
    """A mixer with state of its own whose forward may be recorded: steps with prompt portions are laid into recorded
    steps of padded sizes, whose padding entries read and write a state slot of their own, never the slot of a live
    request (the first request here holds slot 0 all along).  Same weights and plain statement as the toy above."""
    from ginfer_amd import ModelRunner, write_random_model
    Toy = _register_recordable_toy()
    folder = write_random_model(str(tmp_path / "toy"), Toy(), seed=4, dtype="float32")
    reqs = {"a": H.random_tokens(60, 211, 1), "b": H.random_tokens(23, 211, 2), "c": H.random_tokens(37, 211, 3),
            "d": H.random_tokens(18, 211, 4)}
    runner = ModelRunner(folder, dtype="float32", page_size=8, num_pages=24, max_requests=3)
    assert runner.use_graphs and runner.cache.pad_slot == 3
    assert all(t.shape[0] == 4 for t in runner.cache.state_tensors.values())
    refs = {rid: _toy_plain(folder, ids) for rid, ids in reqs.items()}
    # "a" trickles along two tokens a step (slot 0) while the others come and go in portions: every step is padded
    steps, at = [], {"a": 0}
    others = [("b", (9, 14)), ("c", (20, 17)), ("d", (5, 13))]
    for rid, cuts in others:
        o = 0
        for n in cuts:
            a0 = at["a"]
            # few wanted places: a recorded step returns at most as many rows as it has entries
            steps.append(dict(entries=[dict(id="a", tokens=reqs["a"][a0:a0 + 2], want=[1]),
                                       dict(id=rid, tokens=reqs[rid][o:o + n], want=[0, n - 1])],
                              end=[rid] if o + n == len(reqs[rid]) else []))
            at["a"] += 2
            o += n
    for rounds in range(3):          # shapes seen a second time are recorded, a third time replayed
        got = H.run_steps(runner, steps)
        runner.release("a")
        runner.cache.check()
        for (rid, p), row in got.items():
            ref = refs[rid]
            err = np.abs(row - ref[p]).max() / np.abs(ref).max()
            assert err < 1e-4, "round %d: request %s position %d: %.3g" % (rounds, rid, p, err)
    assert runner.counts["replayed_padded"] > 0, runner.counts


def _register_toy_arrangements():
    """Two arrangements of a block that the package does not have, registered here: one with two more norms (on the
    mixer's and on the feed-forward's output, before each is added to the residual stream), and one with a single norm
    whose rows go to mixer and feed-forward side by side.  A toy architecture uses one of each kind and a usual block
    between them; tensor names are the roles' own where the layer gives none."""
    from ginfer_amd.config import register_architecture, PartSpec, LayerSpec, prenorm_layer, ScheduleEntry, ModelSpec
    from ginfer_amd.parts import register_arrangement
    from ginfer_amd.parts.block import Arrangement, whole

    @register_arrangement("toy_sandwich")
    class Sandwich(Arrangement):
        """h = x + post_mixer_norm(mixer(mixer_norm(x))); x = h + post_feed_forward_norm(feed_forward(feed_forward_norm(h)))"""
        roles = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "post_mixer_norm": "norm",
                 "feed_forward_norm": "norm", "post_feed_forward_norm": "norm"}

        def forward(self, residual, delta, step, cache):
            n = self.mixer_norm.forward(residual, whole(delta, self.mixer_norm))
            a = whole(self.mixer.forward(n, step, cache))
            a = self.post_mixer_norm.forward(a.float().contiguous())          # a norm over a branch: nothing is added
            n = self.feed_forward_norm.forward(residual, a)
            f = whole(self.feed_forward.forward(n))
            return self.post_feed_forward_norm.forward(f.float().contiguous())

    @register_arrangement("toy_parallel")
    class Parallel(Arrangement):
        """n = norm(x); x = x + mixer(n) + feed_forward(n)"""
        roles = {"mixer": "mixer", "feed_forward": "feed_forward", "norm": "norm"}

        def forward(self, residual, delta, step, cache):
            n = self.norm.forward(residual, whole(delta, self.norm))
            a = whole(self.mixer.forward(n, step, cache))
            f = whole(self.feed_forward.forward(n))
            return (a.float() + f.float()).to(n.dtype)

    @register_architecture("ToyArrangedLM")
    @dataclass
    class ToyArrangedConfig:
        hidden_size: int = 56
        vocab_size: int = 157
        architecture = "ToyArrangedLM"

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"])

        def to_dict(self):
            return dict(architectures=["ToyArrangedLM"], hidden_size=self.hidden_size, vocab_size=self.vocab_size)

        def model_spec(self):
            Hd = self.hidden_size
            norm = PartSpec("rmsnorm", dict(size=Hd, eps=1e-5))
            pos = PartSpec("rope_neox", dict(theta=1e4, rotary_dim=16, max_positions=128))
            attn = PartSpec("attention", dict(hidden_size=Hd, num_heads=4, num_kv_heads=2, head_dim=16, qkv_bias=True,
                                              out_bias=False, window=None, position=pos, scale=None))
            ffn = PartSpec("swiglu", dict(hidden_size=Hd, intermediate_size=72))
            layers = [
                LayerSpec("model.layers.0", dict(mixer=attn, feed_forward=ffn, mixer_norm=norm, post_mixer_norm=norm,
                                                 feed_forward_norm=norm, post_feed_forward_norm=norm),
                          arrangement="toy_sandwich", names=dict(mixer="self_attn", feed_forward="mlp")),
                prenorm_layer("model.layers.1", attn, ffn, norm, norm, names=H.LAYER_NAMES),
                LayerSpec("model.layers.2", dict(mixer=attn, feed_forward=ffn, norm=norm), arrangement="toy_parallel",
                          names=dict(mixer="self_attn", feed_forward="mlp", norm="shared_layernorm")),
            ]
            return ModelSpec(hidden_size=Hd, vocab_size=self.vocab_size, layers=layers,
                             schedule=[ScheduleEntry(i) for i in range(3)],
                             embedding=PartSpec("embedding", dict(vocab_size=self.vocab_size, hidden_size=Hd)),
                             final_norm=norm, head=PartSpec("lm_head", dict(vocab_size=self.vocab_size, hidden_size=Hd,
                                                                            tied=False)),
                             max_positions=128, eos_token_ids=[0], names=H.MODEL_NAMES)
    return ToyArrangedConfig


def _toy_arranged_plain(folder, ids):
    w = pm.read_weights(folder)
    T = len(ids)
    cfg = dict(num_attention_heads=4, num_key_value_heads=2, head_dim=16)
    sin, cos = pm.rope_tables(1e4, 16, T)
    pos = list(range(T))
    x = pm.embedding(w["model.embed_tokens.weight"], ids)
    norm = lambda v, name: pm.rms_norm(v, w[name + ".weight"], 1e-5)
    p = "model.layers.0"
    a, _ = pm.attention_block(norm(x, p + ".mixer_norm"), w, p + ".self_attn", cfg, pos, sin, cos, None)
    h = x + norm(a, p + ".post_mixer_norm")
    x = h + norm(pm.feed_forward(norm(h, p + ".feed_forward_norm"), w, p + ".mlp"), p + ".post_feed_forward_norm")
    p = "model.layers.1"
    a, _ = pm.attention_block(norm(x, p + ".input_layernorm"), w, p + ".self_attn", cfg, pos, sin, cos, None)
    h = x + a
    x = h + pm.feed_forward(norm(h, p + ".post_attention_layernorm"), w, p + ".mlp")
    p = "model.layers.2"
    n = norm(x, p + ".shared_layernorm")
    a, _ = pm.attention_block(n, w, p + ".self_attn", cfg, pos, sin, cos, None)
    x = x + a + pm.feed_forward(n, w, p + ".mlp")
    return pm.linear(norm(x, "model.norm"), w["lm_head.weight"]).float().numpy()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_arrangements_with_other_roles_are_registered_built_and_stepped(tmp_path, dtype):
    """A layer is a dictionary of parts by role, and which roles there are is the arrangement's matter: blocks with six
    parts and with three, defined here, are built from the configuration, loaded by their own tensor names and stepped
    whole, in portions and mixed (recorded steps included) against their plain statement."""
    from ginfer_amd import ModelRunner, write_random_model, config_from_folder
    from ginfer_amd.config import LayerSpec, PartSpec
    from ginfer_amd.parts import build_model
    Toy = _register_toy_arrangements()
    folder = write_random_model(str(tmp_path / "arranged"), Toy(), seed=12, dtype="float32", std_scale=4.0)
    assert type(config_from_folder(folder)).__name__ == "ToyArrangedConfig"
    runner = ModelRunner(folder, dtype=dtype, page_size=8, num_pages=24, max_requests=3)
    names = set(runner.model.weight_specs())
    assert {"model.layers.0.post_mixer_norm.weight", "model.layers.0.post_feed_forward_norm.weight",
            "model.layers.2.shared_layernorm.weight", "model.layers.1.input_layernorm.weight"} <= names
    assert "model.layers.2.feed_forward_norm.weight" not in names
    assert [type(b).__name__ for b in runner.model.blocks] == ["Sandwich", "PreNormBlock", "Parallel"]
    reqs = {"a": H.random_tokens(45, 157, 21), "b": H.random_tokens(18, 157, 22), "c": H.random_tokens(31, 157, 23)}
    refs = {rid: _toy_arranged_plain(folder, ids) for rid, ids in reqs.items()}
    for steps in (H.steps_whole(reqs), H.steps_last_decoded(reqs, last=12), H.steps_portions(reqs, sizes=(7, 2, 13)),
                  H.steps_mixed(reqs, max_live=3, seed=2), H.steps_mixed(reqs, max_live=3, seed=2)):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        for (rid, p), row in got.items():
            ref = refs[rid]
            err = np.abs(row - ref[p]).max() / np.abs(ref).max()
            assert err <= (1e-4 if dtype == "float32" else H.TOL[dtype]), "request %s position %d: %.3g" % (rid, p, err)
    # a layer that names other roles than its arrangement has is refused with both lists
    spec = Toy().model_spec()
    spec.layers[2] = LayerSpec("model.layers.2", dict(spec.layers[2].parts, extra_norm=PartSpec("rmsnorm", dict(size=56, eps=1e-5))),
                               arrangement="toy_parallel")
    with pytest.raises(ValueError, match="extra_norm"):
        build_model(spec, torch.float32, dev())


def _register_routed_toy():
    """A second toy architecture defined here, in the test: a feed-forward that routes every token to one of
    three experts (router logits in 32-bit), in one layer only, beside the package's dense one in the other; and
    a position encoding of its own (rotation by a fraction of the position), used by one layer's attention while
    the other keeps the package's.  None of it touches the package's files."""
    from ginfer_amd.config import register_architecture, PartSpec, LayerSpec, prenorm_layer, ScheduleEntry, ModelSpec
    from ginfer_amd.parts import register_feed_forward, register_position, Part
    from ginfer_amd.weights import WeightSpec

    @register_position("toy_slow_rotation")
    class SlowRotation(Part):
        """Rotary tables of the angle (p / slow) * inv_freq: what the attention kernels need is the tables."""
        capturable = True

        def __init__(self, theta, rotary_dim, max_positions, slow, dtype=None, device=None):
            self.theta, self.rotary_dim, self.max_positions, self.slow = float(theta), int(rotary_dim), int(max_positions), float(slow)
            self.device, self._limit, self._tables = device, None, None

        def limit_positions(self, n):
            self._limit, self._tables = min(self.max_positions, int(n)), None

        def tables(self):
            if self._tables is None:
                half = self.rotary_dim // 2
                inv = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float32), torch.arange(half, dtype=torch.float32) / half)
                ang = (torch.arange(self._limit or self.max_positions, dtype=torch.float32) / self.slow)[:, None] * inv[None, :]
                self._tables = (torch.cos(ang).to(self.device).contiguous(), torch.sin(ang).to(self.device).contiguous())
            return self._tables

    @register_feed_forward("toy_one_of_n")
    class OneOfN(Part):
        """y = p_e * W2_e . relu(W1_e . x) for the expert e with the largest router logit, p_e its softmax weight
        (32-bit).  Routing is a function of the token alone."""

        def __init__(self, hidden_size, intermediate_size, num_experts, dtype, device):
            self.H, self.I, self.E, self.dtype, self.device = hidden_size, intermediate_size, num_experts, dtype, device

        def weight_specs(self):
            specs = {"router.weight": WeightSpec((self.E, self.H), keep_32bit=True)}
            for e in range(self.E):
                specs["experts.%d.w1.weight" % e] = WeightSpec((self.I, self.H))
                specs["experts.%d.w2.weight" % e] = WeightSpec((self.H, self.I))
            return specs

        def bind_weights(self, t):
            self.router = t["router.weight"]
            self.w1 = torch.stack([t["experts.%d.w1.weight" % e] for e in range(self.E)])
            self.w2 = torch.stack([t["experts.%d.w2.weight" % e] for e in range(self.E)])

        def forward(self, x):
            logits = x.float() @ self.router.float().t()
            prob, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            hidden = torch.relu(torch.einsum("th,tih->ti", x, self.w1[choice]))
            return (torch.einsum("ti,thi->th", hidden, self.w2[choice]).float() * prob[:, None]).to(x.dtype)

    @register_architecture("ToyRoutedLM")
    @dataclass
    class ToyRoutedConfig:
        hidden_size: int = 40
        vocab_size: int = 173
        architecture = "ToyRoutedLM"

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"])

        def to_dict(self):
            return dict(architectures=["ToyRoutedLM"], hidden_size=self.hidden_size, vocab_size=self.vocab_size)

        def model_spec(self):
            Hd = self.hidden_size
            norm = PartSpec("rmsnorm", dict(size=Hd, eps=1e-6))
            slow = PartSpec("toy_slow_rotation", dict(theta=500.0, rotary_dim=16, max_positions=128, slow=4.0))
            rope = PartSpec("rope_neox", dict(theta=500.0, rotary_dim=16, max_positions=128))

            def attn(pos):
                return PartSpec("attention", dict(hidden_size=Hd, num_heads=2, num_kv_heads=2, head_dim=16, qkv_bias=True,
                                                  out_bias=False, window=None, position=pos, scale=None))
            dense = PartSpec("swiglu", dict(hidden_size=Hd, intermediate_size=56))
            routed = PartSpec("toy_one_of_n", dict(hidden_size=Hd, intermediate_size=24, num_experts=3))
            layers = [prenorm_layer("model.layers.0", attn(slow), routed, norm, norm, names=H.LAYER_NAMES),
                      prenorm_layer("model.layers.1", attn(rope), dense, norm, norm, names=H.LAYER_NAMES)]
            return ModelSpec(hidden_size=Hd, vocab_size=self.vocab_size, layers=layers,
                             schedule=[ScheduleEntry(0), ScheduleEntry(1)],
                             embedding=PartSpec("embedding", dict(vocab_size=self.vocab_size, hidden_size=Hd)),
                             final_norm=norm, head=PartSpec("lm_head", dict(vocab_size=self.vocab_size, hidden_size=Hd,
                                                                            tied=False)),
                             max_positions=128, eos_token_ids=[0], names=H.MODEL_NAMES)
    return ToyRoutedConfig


def _routed_toy_plain(folder, ids):
    w = pm.read_weights(folder)
    T = len(ids)
    cfg = dict(num_attention_heads=2, num_key_value_heads=2, head_dim=16)
    half = 8
    inv = 1.0 / torch.pow(torch.tensor(500.0, dtype=torch.float32), torch.arange(half, dtype=torch.float32) / half)
    slow_ang = (torch.arange(T, dtype=torch.float32) / 4.0)[:, None] * inv[None, :]
    tables = {0: (torch.sin(slow_ang).double(), torch.cos(slow_ang).double()), 1: pm.rope_tables(500.0, 16, T)}
    x = pm.embedding(w["model.embed_tokens.weight"], ids)
    choices = None
    for layer in (0, 1):
        p = "model.layers.%d" % layer
        n = pm.rms_norm(x, w[p + ".input_layernorm.weight"], 1e-6)
        sin, cos = tables[layer]
        a, _ = pm.attention_block(n, w, p + ".self_attn", cfg, list(range(T)), sin, cos, None)
        h = x + a
        n = pm.rms_norm(h, w[p + ".post_attention_layernorm.weight"], 1e-6)
        if layer == 0:
            prob = torch.softmax(n @ w[p + ".mlp.router.weight"].t(), dim=-1)
            choices = prob.argmax(dim=-1)
            out = torch.zeros_like(n)
            for t in range(T):
                e = int(choices[t])
                hid = torch.relu(w[p + ".mlp.experts.%d.w1.weight" % e] @ n[t])
                out[t] = prob[t, e] * (w[p + ".mlp.experts.%d.w2.weight" % e] @ hid)
            x = h + out
        else:
            x = h + pm.feed_forward(n, w, p + ".mlp")
    return pm.linear(pm.rms_norm(x, w["model.norm.weight"], 1e-6), w["lm_head.weight"]).float().numpy(), choices


def test_toy_routed_feed_forward_and_toy_position_encoding(tmp_path):
    """Layers of one model with different feed-forwards and different position encodings, both toys registered
    here: built from the configuration, stepped whole, in portions and mixed, against a plain statement of them."""
    from ginfer_amd import ModelRunner, write_random_model, config_from_folder
    Toy = _register_routed_toy()
    folder = write_random_model(str(tmp_path / "routed"), Toy(), seed=9, dtype="float32")
    assert type(config_from_folder(folder)).__name__ == "ToyRoutedConfig"
    reqs = {"a": H.random_tokens(45, 173, 11), "b": H.random_tokens(18, 173, 12), "c": H.random_tokens(31, 173, 13)}
    runner = ModelRunner(folder, dtype="float32", page_size=8, num_pages=24, max_requests=3)
    assert len(runner.model.position_parts()) == 2                  # one table set per encoding
    assert not runner.use_graphs                                     # the toy says nothing of being recordable
    refs = {rid: _routed_toy_plain(folder, ids) for rid, ids in reqs.items()}
    assert len({int(c) for _, ch in refs.values() for c in ch}) == 3  # every expert is used
    for steps in (H.steps_whole(reqs), H.steps_portions(reqs, sizes=(7, 2, 13)), H.steps_mixed(reqs, max_live=3, seed=2)):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        for (rid, p), row in got.items():
            ref = refs[rid][0]
            err = np.abs(row - ref[p]).max() / np.abs(ref).max()
            assert err < 1e-4, "request %s position %d: %.3g" % (rid, p, err)


def test_schedule_names_a_layer_twice_and_shares_a_cache(tmp_path):
    """The order of layers is data: a Qwen2 folder run with another schedule."""
    from ginfer_amd import ModelRunner, config_from_folder
    from ginfer_amd.config import ScheduleEntry
    folder = H.make_model_folder(tmp_path / "m", H.TINY_B, 1)
    cfg = config_from_folder(folder)
    base_spec = cfg.model_spec

    def spec_with_schedule():
        s = base_spec()
        s.schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1), ScheduleEntry(2, cache_of=0)]
        return s
    cfg.model_spec = spec_with_schedule
    runner = ModelRunner(folder, dtype="float32", page_size=8, num_pages=32, config=cfg)
    assert len(runner.cache.groups[0].entries) == 3           # runs 0, 1, 2 own caches; run 3 reads run 0's
    ids = H.random_tokens(60, 1000, 8)
    pc, w = pm.read_config(folder), pm.read_weights(folder)
    ref = pm.forward(pc, w, ids, schedule=[(0, None), (1, None), (1, None), (2, 0)]).float().numpy()
    for steps in (H.steps_whole({"x": ids}), H.steps_portions({"x": ids}, sizes=(9, 2, 30))):
        got = H.run_steps(runner, steps)
        for (rid, p), row in got.items():
            assert np.abs(row - ref[p]).max() / np.abs(ref).max() < 1e-4


def _register_toy_ends():
    """A third toy architecture defined here: a norm of another kind (mean taken off, gain and bias), an embedding that
    scales the table's rows and adds a learned vector per position, and a head with a bias whose logits are capped
    softly.  The layers between them are the package's own.  None of it touches the package's files."""
    from ginfer_amd.config import register_architecture, PartSpec, prenorm_layer, ScheduleEntry, ModelSpec
    from ginfer_amd.parts import register_norm, register_embedding, register_head, Part
    from ginfer_amd.weights import WeightSpec

    @register_norm("toy_centered_norm")
    class CenteredNorm(Part):
        """y = (h - mean(h)) / sqrt(var(h) + eps) * g + b, h = residual + delta, in 32-bit.  It says nothing of partial
        sums or folding: the block hands it whole rows."""

        def __init__(self, size, eps, dtype, device):
            self.size, self.eps, self.dtype, self.device = int(size), float(eps), dtype, device

        def weight_specs(self):
            return {"weight": WeightSpec((self.size,), init="one_plus_normal", keep_32bit=True),
                    "bias": WeightSpec((self.size,), std=0.1, keep_32bit=True)}

        def bind_weights(self, t):
            self.weight, self.bias = t["weight"], t["bias"]

        def forward(self, residual, delta=None, rows=None):
            if rows is not None:
                h = residual[rows.long()] + (delta[rows.long()].float() if delta is not None else 0.0)
            else:
                if delta is not None:
                    residual += delta.float()
                h = residual
            c = h - h.mean(dim=-1, keepdim=True)
            y = c * torch.rsqrt(c.pow(2).mean(dim=-1, keepdim=True) + self.eps) * self.weight.float() + self.bias.float()
            return y.to(self.dtype)

    @register_embedding("toy_scaled_with_positions")
    class ScaledWithPositions(Part):
        """x[t] = sqrt(H) * E[id[t]] + P[position[t]]: it reads the positions from the step."""

        def __init__(self, vocab_size, hidden_size, max_positions, dtype, device):
            self.V, self.H, self.P, self.dtype, self.device = int(vocab_size), int(hidden_size), int(max_positions), dtype, device

        def weight_specs(self):
            return {"weight": WeightSpec((self.V, self.H)), "positions.weight": WeightSpec((self.P, self.H), std=0.05)}

        def bind_weights(self, t):
            self.weight, self.positions = t["weight"], t["positions.weight"]

        def forward(self, token_ids, step):
            return self.weight[token_ids.long()].float() * math.sqrt(self.H) + self.positions[step.positions.long()].float()

    @register_head("toy_capped_head")
    class CappedHead(Part):
        """logits = cap * tanh((x . W^T + b) / cap), 32-bit."""

        def __init__(self, vocab_size, hidden_size, cap, dtype, device):
            self.V, self.H, self.cap, self.dtype, self.device = int(vocab_size), int(hidden_size), float(cap), dtype, device

        def weight_specs(self):
            return {"weight": WeightSpec((self.V, self.H), std=0.3), "bias": WeightSpec((self.V,), std=0.5, keep_32bit=True)}

        def bind_weights(self, t):
            self.weight, self.bias = t["weight"], t["bias"]

        def forward(self, x):
            z = x.float() @ self.weight.float().t() + self.bias.float()
            return self.cap * torch.tanh(z / self.cap)

    @register_architecture("ToyEndsLM")
    @dataclass
    class ToyEndsConfig:
        hidden_size: int = 48
        vocab_size: int = 211
        architecture = "ToyEndsLM"

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"])

        def to_dict(self):
            return dict(architectures=["ToyEndsLM"], hidden_size=self.hidden_size, vocab_size=self.vocab_size)

        def model_spec(self):
            Hd = self.hidden_size
            norm = PartSpec("toy_centered_norm", dict(size=Hd, eps=1e-5))
            rope = PartSpec("rope_neox", dict(theta=300.0, rotary_dim=16, max_positions=96))
            attn = PartSpec("attention", dict(hidden_size=Hd, num_heads=3, num_kv_heads=1, head_dim=16, qkv_bias=True,
                                              out_bias=False, window=None, position=rope, scale=None))
            dense = PartSpec("swiglu", dict(hidden_size=Hd, intermediate_size=72))
            layers = [prenorm_layer("model.layers.%d" % i, attn, dense, norm, norm, names=H.LAYER_NAMES) for i in range(2)]
            return ModelSpec(hidden_size=Hd, vocab_size=self.vocab_size, layers=layers,
                             schedule=[ScheduleEntry(0), ScheduleEntry(1)],
                             embedding=PartSpec("toy_scaled_with_positions",
                                                dict(vocab_size=self.vocab_size, hidden_size=Hd, max_positions=96)),
                             final_norm=norm,
                             head=PartSpec("toy_capped_head", dict(vocab_size=self.vocab_size, hidden_size=Hd, cap=3.0)),
                             max_positions=96, eos_token_ids=[0], names=H.MODEL_NAMES)
    return ToyEndsConfig


def _toy_ends_plain(folder, ids):
    w = pm.read_weights(folder)
    T, Hd = len(ids), 48
    cfg = dict(num_attention_heads=3, num_key_value_heads=1, head_dim=16)

    def norm(h, prefix):
        c = h - h.mean(dim=-1, keepdim=True)
        return c / torch.sqrt(c.pow(2).mean(dim=-1, keepdim=True) + 1e-5) * w[prefix + ".weight"] + w[prefix + ".bias"]
    sin, cos = pm.rope_tables(300.0, 16, T)
    x = pm.embedding(w["model.embed_tokens.weight"], ids) * math.sqrt(Hd) + w["model.embed_tokens.positions.weight"][:T]
    for layer in (0, 1):
        p = "model.layers.%d" % layer
        a, _ = pm.attention_block(norm(x, p + ".input_layernorm"), w, p + ".self_attn", cfg, list(range(T)), sin, cos, None)
        h = x + a
        x = h + pm.feed_forward(norm(h, p + ".post_attention_layernorm"), w, p + ".mlp")
    z = pm.linear(norm(x, "model.norm"), w["lm_head.weight"]) + w["lm_head.bias"]
    return (3.0 * torch.tanh(z / 3.0)).float().numpy()


def test_toy_norm_embedding_and_head(tmp_path):
    """The ends of a model and its norms as toys registered here: a norm with a mean and a bias (it takes neither
    partial sums nor folding, so the block adds up what the products leave in parts), an embedding that reads the step's
    positions, a head with a bias and a cap; stepped whole, in portions and mixed against their plain statement."""
    from ginfer_amd import ModelRunner, write_random_model, config_from_folder
    Toy = _register_toy_ends()
    folder = write_random_model(str(tmp_path / "ends"), Toy(), seed=21, dtype="float32")
    assert type(config_from_folder(folder)).__name__ == "ToyEndsConfig"
    reqs = {"a": H.random_tokens(50, 211, 31), "b": H.random_tokens(9, 211, 32), "c": H.random_tokens(27, 211, 33)}
    runner = ModelRunner(folder, dtype="float32", page_size=8, num_pages=30, max_requests=3)
    assert not runner.use_graphs
    refs = {rid: _toy_ends_plain(folder, ids) for rid, ids in reqs.items()}
    assert max(np.abs(r).max() for r in refs.values()) > 1.5          # the cap is felt
    for steps in (H.steps_whole(reqs), H.steps_portions(reqs, sizes=(5, 2, 17)), H.steps_mixed(reqs, max_live=3, seed=4)):
        got = H.run_steps(runner, steps)
        runner.cache.check()
        for (rid, p), row in got.items():
            err = np.abs(row - refs[rid][p]).max() / np.abs(refs[rid]).max()
            assert err < 1e-4, "request %s position %d: %.3g" % (rid, p, err)


# ----------------------------------------------------------------------------- caches of other shapes

def _register_toy_caches():
    """Two toys whose caches are not the usual pair of equally wide keys and values under one mixer: attention whose
    values are half as wide as its keys (written in plain torch over the pages it is handed), and a block that has this
    attention and a running mean side by side, pages and a state slot for one run of one layer."""
    from ginfer_amd.config import register_architecture, PartSpec, LayerSpec, prenorm_layer, ScheduleEntry, ModelSpec
    from ginfer_amd.parts import register_mixer, register_arrangement, Part, KVCacheSpec, StateSpec
    from ginfer_amd.parts.block import Arrangement, whole
    from ginfer_amd.weights import WeightSpec

    @register_mixer("toy_narrow_value_attention")
    class NarrowValueAttention(Part):
        """Causal attention without positions: keys of `key_dim`, values of `value_dim` per head, one kv head per head."""

        def __init__(self, hidden_size, num_heads, key_dim, value_dim, dtype, device):
            self.H, self.nh, self.kd, self.vd, self.dtype, self.device = hidden_size, num_heads, key_dim, value_dim, dtype, device

        def cache_spec(self):
            return KVCacheSpec(self.nh, self.kd, None, value_dim=self.vd)

        def weight_specs(self):
            return {"q.weight": WeightSpec((self.nh * self.kd, self.H)), "k.weight": WeightSpec((self.nh * self.kd, self.H)),
                    "v.weight": WeightSpec((self.nh * self.vd, self.H)), "o.weight": WeightSpec((self.H, self.nh * self.vd))}

        def bind_weights(self, t):
            self.w = {n.split(".")[0]: v for n, v in t.items()}

        def forward(self, x, step, cache):
            nh, kd, vd, ps = self.nh, self.kd, self.vd, cache.page_size
            assert tuple(cache.k_pages.shape[1:]) == (nh, ps, kd) and tuple(cache.v_pages.shape[1:]) == (nh, vd, ps)
            xf = x.float()
            q = (xf @ self.w["q"].float().t()).view(-1, nh, kd)
            k = (xf @ self.w["k"].float().t()).view(-1, nh, kd)
            v = (xf @ self.w["v"].float().t()).view(-1, nh, vd)
            page, off = cache.slot_mapping // ps, cache.slot_mapping % ps
            cache.k_pages[page, :, off, :] = k.to(cache.k_pages.dtype)
            cache.v_pages[page, :, :, off] = v.to(cache.v_pages.dtype)
            out = torch.empty((x.shape[0], nh * vd), dtype=torch.float32, device=x.device)
            o = 0
            for e in range(step.num_entries):
                n, start = step.host_q_len[e], step.host_q_start[e]
                total = start + n
                pages = cache.block_table[e, :-(-total // ps)].long()
                keys = cache.k_pages[pages].float().permute(1, 0, 2, 3).reshape(nh, -1, kd)[:, :total]          # [nh, total, kd]
                vals = cache.v_pages[pages].float().permute(1, 0, 3, 2).reshape(nh, -1, vd)[:, :total]          # [nh, total, vd]
                s = torch.einsum("thd,hkd->htk", q[o:o + n], keys) / kd ** 0.5
                seen = torch.arange(total, device=x.device)[None, :] <= (start + torch.arange(n, device=x.device))[:, None]
                p = torch.softmax(s.masked_fill(~seen[None], float("-inf")), dim=-1)
                out[o:o + n] = torch.einsum("htk,hkd->thd", p, vals).reshape(n, nh * vd)
                o += n
            return (out @ self.w["o"].float().t()).to(self.dtype)

    @register_arrangement("toy_attention_beside_a_mean")
    class AttentionBesideMean(Arrangement):
        """h = x + attention(norm(x)) + running_mean(norm(x)); x' = h + feed_forward(norm2(h)).  One run keeps pages for
        the attention and a state slot for the mean: the list of both is its cache."""
        roles = {"mixer": "mixer", "mean": "mixer", "feed_forward": "feed_forward", "norm": "norm", "feed_forward_norm": "norm"}

        def cache_spec(self):
            return [self.mixer.cache_spec(), self.mean.cache_spec()]

        def forward(self, residual, delta, step, cache):
            pages, slot = cache
            n = self.norm.forward(residual, whole(delta, self.norm))
            a = self.mixer.forward(n, step, pages) + self.mean.forward(n, step, slot)
            return self.feed_forward.forward(self.feed_forward_norm.forward(residual, a))

    @register_architecture("ToyCachesLM")
    @dataclass
    class ToyCachesConfig:
        hidden_size: int = 40
        vocab_size: int = 173
        architecture = "ToyCachesLM"

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"])

        def to_dict(self):
            return dict(architectures=["ToyCachesLM"], hidden_size=self.hidden_size, vocab_size=self.vocab_size)

        def model_spec(self):
            Hd = self.hidden_size
            norm = PartSpec("rmsnorm", dict(size=Hd, eps=1e-5))
            narrow = PartSpec("toy_narrow_value_attention", dict(hidden_size=Hd, num_heads=2, key_dim=16, value_dim=8))
            mean = PartSpec("toy_running_mean", dict(hidden_size=Hd))
            ffn = PartSpec("swiglu", dict(hidden_size=Hd, intermediate_size=56))
            layers = [
                prenorm_layer("model.layers.0", narrow, ffn, norm, norm, names=H.LAYER_NAMES),
                LayerSpec("model.layers.1", dict(mixer=narrow, mean=mean, feed_forward=ffn, norm=norm, feed_forward_norm=norm),
                          arrangement="toy_attention_beside_a_mean",
                          names=dict(mixer="self_attn", mean="mean", feed_forward="mlp", norm="input_layernorm",
                                     feed_forward_norm="post_attention_layernorm")),
            ]
            return ModelSpec(hidden_size=Hd, vocab_size=self.vocab_size, layers=layers,
                             schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)],
                             embedding=PartSpec("embedding", dict(vocab_size=self.vocab_size, hidden_size=Hd)),
                             final_norm=norm, head=PartSpec("lm_head", dict(vocab_size=self.vocab_size, hidden_size=Hd,
                                                                            tied=False)),
                             max_positions=160, eos_token_ids=[0], names=H.MODEL_NAMES)
    return ToyCachesConfig


def _toy_caches_plain(folder, ids):
    """The model of `_register_toy_caches` on a whole sequence, written out plainly in 64-bit."""
    w = pm.read_weights(folder)
    T = len(ids)
    x = pm.embedding(w["model.embed_tokens.weight"], ids)

    def narrow_attention(n, p):
        q = pm.linear(n, w[p + ".q.weight"]).view(T, 2, 16)
        k = pm.linear(n, w[p + ".k.weight"]).view(T, 2, 16)
        v = pm.linear(n, w[p + ".v.weight"]).view(T, 2, 8)
        s = torch.einsum("thd,khd->htk", q, k) / 4.0
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1)[None], float("-inf"))
        return pm.linear(torch.einsum("htk,khd->thd", torch.softmax(s, dim=-1), v).reshape(T, 16), w[p + ".o.weight"])

    for layer in (0, 1, 0):
        p = "model.layers.%d" % layer
        n = pm.rms_norm(x, w[p + ".input_layernorm.weight"], 1e-5)
        a = narrow_attention(n, p + ".self_attn")
        if layer == 1:
            mean = torch.cumsum(n, dim=0) / torch.arange(1, T + 1, dtype=n.dtype)[:, None]
            a = a + mean @ w[p + ".mean.mix.weight"].t()
        h = x + a
        x = h + pm.feed_forward(pm.rms_norm(h, w[p + ".post_attention_layernorm.weight"], 1e-5), w, p + ".mlp")
    return pm.linear(pm.rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"]).float().numpy()


def test_toy_caches_of_other_shapes_are_built_and_stepped(tmp_path):
    """Values half as wide as keys, and a block that keeps pages and a state slot side by side: registered here, built
    and stepped whole, in portions and mixed, against their plain statement.  Layer 0 runs twice (two caches of its
    own); the runs of the narrow attention share one group of pages, whose pages hold 2 x 16 + 2 x 8 elements a token."""
    from ginfer_amd import ModelRunner, write_random_model
    _register_toy()                       # the running mean
    Toy = _register_toy_caches()
    folder = write_random_model(str(tmp_path / "toy"), Toy(), seed=9, dtype="float32")
    reqs = {"a": H.random_tokens(45, 173, 1), "b": H.random_tokens(19, 173, 2), "c": H.random_tokens(33, 173, 3),
            "d": H.random_tokens(27, 173, 4)}
    runner = ModelRunner(folder, dtype="float32", page_size=8, num_pages=14, max_requests=3)
    cache = runner.cache
    assert [type(s).__name__ if not isinstance(s, list) else [type(c).__name__ for c in s] for s in cache.cache_specs] \
        == ["KVCacheSpec", ["KVCacheSpec", "StateSpec"], "KVCacheSpec"]
    assert len(cache.groups) == 1 and cache.groups[0].units == [(0, 0), (1, 0), (2, 0)] and cache.state_units == [(1, 1)]
    assert cache.groups[0].tensors["k"].shape == (3, 14, 8 * 32) and cache.groups[0].tensors["v"].shape == (3, 14, 8 * 16)
    assert cache.pool_bytes(4) == 14 * 3 * 48 * 8 * 4
    assert not runner.use_graphs          # the toys say nothing of recording
    refs = {rid: _toy_caches_plain(folder, ids) for rid, ids in reqs.items()}
    for steps in (H.steps_whole(reqs), H.steps_portions(reqs, sizes=(5, 2, 11, 3)), H.steps_mixed(reqs, max_live=3, seed=2)):
        got = H.run_steps(runner, steps)
        cache.check()
        assert got
        for (rid, p), row in got.items():
            err = np.abs(row - refs[rid][p]).max() / np.abs(refs[rid]).max()
            assert err < 1e-4, "request %s position %d: %.3g" % (rid, p, err)


def test_the_pool_is_planned_around_the_state_of_a_stateful_model(tmp_path, monkeypatch):
    """Per-request state enters the memory plan before the pool of pages is sized: a toy whose state slots are large
    (a quarter of a gigabyte each, two runs of the layer, a slot per request and one more) is planned as if 3 GB were
    free, and generates to the end through the engine."""
    from ginfer_amd import ModelRunner, Engine, EngineConfig, SamplingParams, write_random_model
    from ginfer_amd.cache import CacheManager
    Toy = _register_toy()
    pad = (1 << 26) - 49
    folder = write_random_model(str(tmp_path / "toy"), Toy(state_pad=pad), seed=4, dtype="float32")
    real = torch.cuda.mem_get_info
    torch.cuda.empty_cache()
    if real()[0] < (6 << 30):
        pytest.skip("needs 6 GB of free device memory")
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a, **k: (3 << 30, real(*a, **k)[1]))     # as if 3 GB were free
    r = ModelRunner(folder, dtype="float32", page_size=8, max_requests=3, max_num_batched_tokens=32, gpu_memory_utilization=0.5)
    plan = r.memory_plan
    state = 2 * 4 * (1 << 26) * 4                            # two runs, four slots, 2^26 floats
    assert plan["state_bytes"] == state == CacheManager.state_bytes(r.cache.cache_specs, 3)
    assert plan["pool_bytes"] == ((3 << 30) - state) // 2    # half of what the state leaves, not of all that is free
    assert r.cache.pool_bytes(4) <= plan["pool_bytes"]
    assert plan["step_room_bytes"] >= plan["step_peak_bytes"] > 0
    assert 0 <= plan["graph_budget_bytes"] <= (3 << 30) - state - plan["pool_bytes"] - plan["step_room_bytes"]
    assert sum(t.numel() * t.element_size() for t in r.cache.state_tensors.values()) == state
    del r
    torch.cuda.empty_cache()
    # a utilisation that would have fitted without the state is refused, and the message names the state
    with pytest.raises(ValueError, match="per-request state"):
        monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a, **k: (state + (32 << 20), real(*a, **k)[1]))
        ModelRunner(folder, dtype="float32", page_size=8, max_requests=3, max_num_batched_tokens=32, gpu_memory_utilization=0.5)
    torch.cuda.empty_cache()
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a, **k: (3 << 30, real(*a, **k)[1]))
    eng = Engine(EngineConfig(model_path=folder, dtype="float32", max_num_batched_tokens=32, max_num_seqs=3, max_seq_len=120,
                              kvcache_block_size=8, gpu_memory_utilization=0.5))
    prompts = [H.random_tokens(n, 211, 60 + n) for n in (40, 7, 61, 23)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10, ignore_eos=True))
    eng.runner.cache.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.runner.cache.groups)
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 10
        ids = p + o.token_ids
        logits = _toy_plain(folder, ids[:-1])
        for k, tok in enumerate(o.token_ids):
            row = logits[len(p) - 1 + k]
            best = int(np.argmax(row))
            assert tok == best or float(row[best] - row[tok]) <= 1e-4 * float(np.abs(row).max()), (len(p), k, tok, best)
