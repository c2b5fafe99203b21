import json
import os
import struct

import numpy as np
import pytest
import torch

import helpers as H
from ginfer_amd import config_from_dict, write_random_model
from ginfer_amd.parts import build_model
from ginfer_amd.weights import (SafetensorsFile, SafetensorsError, WeightError, WeightSpec, write_safetensors,
                                open_model_files, check_against)
from ginfer_amd.weights.loader import target_dtype


def test_reader_and_writer_agree_with_the_safetensors_package(tmp_path):
    from safetensors.torch import save_file, load_file
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).view(2, 3),
               "d": torch.randn(2, 2, 2).to(torch.float16), "e": torch.empty(0, 4)}
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    f = SafetensorsFile(str(tmp_path / "theirs.safetensors"))
    assert sorted(f.names()) == sorted(tensors)
    for n, t in tensors.items():
        assert f.info(n) == (t.dtype, tuple(t.shape))
        assert torch.equal(f.tensor(n), t)
    write_safetensors(str(tmp_path / "ours.safetensors"), tensors, metadata={"format": "pt"})
    back = load_file(str(tmp_path / "ours.safetensors"))
    for n, t in tensors.items():
        assert torch.equal(back[n], t)


def test_broken_files_are_refused(tmp_path):
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    def with_header(h, data=b""):
        blob = json.dumps(h).encode()
        p.write_bytes(struct.pack("<Q", len(blob)) + blob + data)
    with_header({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="size mismatch"):
        SafetensorsFile(str(p))
    with_header({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="outside the file"):
        SafetensorsFile(str(p))
    with_header({"t": {"dtype": "Q4", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFile(str(p))
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        open_model_files(str(tmp_path / "nowhere"))


def test_expected_names_are_the_checkpoints(tmp_path):
    """ginfer/model/qwen2.cc:34-46 and ginfer/model/loader/model_loader.cc:54-122."""
    for d, tied in ((H.TINY_A, True), (H.TINY_B, False)):
        model = build_model(config_from_dict(d).model_spec(), torch.float32, None)
        names = set(model.weight_specs())
        L = d["num_hidden_layers"]
        per_layer = ["self_attn.q_proj.weight", "self_attn.q_proj.bias", "self_attn.k_proj.weight", "self_attn.k_proj.bias",
                     "self_attn.v_proj.weight", "self_attn.v_proj.bias", "self_attn.o_proj.weight", "mlp.gate_proj.weight",
                     "mlp.up_proj.weight", "mlp.down_proj.weight", "input_layernorm.weight", "post_attention_layernorm.weight"]
        want = {"model.embed_tokens.weight", "model.norm.weight"} | {"model.layers.%d.%s" % (i, n) for i in range(L) for n in per_layer}
        if not tied:
            want.add("lm_head.weight")
        assert names == want


def test_one_error_lists_missing_unexpected_and_wrong(tmp_path):
    cfg = config_from_dict(H.TINY_A)
    folder = write_random_model(str(tmp_path / "m"), cfg, 0, "float32")
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    del tensors["model.norm.weight"]
    del tensors["model.layers.1.mlp.up_proj.weight"]
    tensors["lm_head.weight"] = torch.zeros(512, 64)                                  # tied: carried, never read
    tensors["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(64)                 # not expected
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 65)           # wrong shape
    tensors["model.layers.0.self_attn.k_proj.bias"] = torch.zeros(32, dtype=torch.int32)   # wrong kind
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    model = build_model(cfg.model_spec(), torch.float32, None)
    files = open_model_files(folder)
    with pytest.raises(WeightError) as e:
        check_against(model.weight_specs(), {n: fl.info(n) for n, fl in files.items()}, folder,
                      unread=model.unread_weights())
    msg = str(e.value)
    assert "model.norm.weight" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "missing tensors (2)" in msg
    assert model.unread_weights() == ["lm_head.weight"]
    assert "unexpected tensors (1): model.layers.0.self_attn.o_proj.bias" in msg
    untied = build_model(config_from_dict(H.TINY_B).model_spec(), torch.float32, None)
    assert untied.unread_weights() == []
    assert "q_proj.weight: expected shape [64, 64], found [64, 65]" in msg
    assert "k_proj.bias: expected a floating tensor" in msg
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]


def test_tensors_that_the_model_does_not_read_are_a_warning_or_an_error_when_strict(tmp_path, capsys):
    """A checkpoint may carry tensors the model never reads (the reference looks tensors up by name and never sees the
    others, ginfer/model/loader/safetensor_loader.cc:44-81): by themselves they are named in a warning; under
    `strict` they are the error."""
    cfg = config_from_dict(H.TINY_A)
    folder = write_random_model(str(tmp_path / "m"), cfg, 0, "float32")
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    model = build_model(cfg.model_spec(), torch.float32, None)
    available = {n: fl.info(n) for n, fl in open_model_files(folder).items()}
    assert check_against(model.weight_specs(), available, folder, unread=model.unread_weights()) == \
        ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert "does not read: model.layers.0.self_attn.rotary_emb.inv_freq" in capsys.readouterr().err
    with pytest.raises(WeightError, match=r"unexpected tensors \(1\): model.layers.0.self_attn.rotary_emb.inv_freq"):
        check_against(model.weight_specs(), available, folder, unread=model.unread_weights(), strict=True)


def test_dtype_rules():
    f32, bf16 = torch.float32, torch.bfloat16
    assert target_dtype(WeightSpec((2,)), f32, bf16) == bf16            # kept in bfloat16
    assert target_dtype(WeightSpec((2,)), bf16, f32) == f32             # the 32-bit path widens
    assert target_dtype(WeightSpec((2,), kind="int"), torch.int64, bf16) == torch.int32
    assert target_dtype(WeightSpec((2,), keep_32bit=True), f32, bf16) == f32   # stored in 32-bit, stays so
    assert target_dtype(WeightSpec((2,), keep_32bit=True), bf16, bf16) == bf16


def test_random_weights_mode(tmp_path):
    cfg = config_from_dict(H.TINY_B)
    a = write_random_model(str(tmp_path / "a"), cfg, 1, "float32")
    b = write_random_model(str(tmp_path / "b"), cfg, 1, "float32")
    c = write_random_model(str(tmp_path / "c"), cfg, 2, "bfloat16")
    fa, fb, fc = (SafetensorsFile(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    assert sorted(fa.names()) == sorted(fc.names())
    for n in fa.names():
        assert torch.equal(fa.tensor(n), fb.tensor(n))                  # same seed, same bytes
        assert fc.info(n)[0] == torch.bfloat16
    w = fa.tensor("model.layers.0.mlp.gate_proj.weight")
    assert abs(w.std().item() - 0.02) < 2e-3 and abs(w.mean().item()) < 1e-3
    g = fa.tensor("model.layers.0.input_layernorm.weight")
    assert abs(g.mean().item() - 1.0) < 0.01 and 0.01 < g.std().item() < 0.03
    assert not torch.equal(fa.tensor("model.norm.weight"), fc.tensor("model.norm.weight").float())
    with open(os.path.join(c, "config.json")) as fh:
        d = json.load(fh)
    assert d["torch_dtype"] == "bfloat16" and d["architectures"] == ["Qwen2ForCausalLM"]
    assert config_from_dict(d).num_key_value_heads == 1


def test_the_host_generator_is_a_function_of_seed_name_and_index():
    """Counter-based: a tensor's draws depend on the seed and its name alone, any stretch of it can be drawn by
    itself, and the numbers are normal (mean, spread, tails, no correlation between neighbours)."""
    import numpy as np
    from scipy import stats
    from ginfer_amd.weights.random_init import draw
    spec = WeightSpec((1 << 18,))
    a = draw(spec, 5, "t.weight", torch.float32)
    assert torch.equal(a, draw(spec, 5, "t.weight", torch.float32))
    assert not torch.equal(a, draw(spec, 6, "t.weight", torch.float32)) and not torch.equal(a, draw(spec, 5, "u.weight", torch.float32))
    assert torch.equal(draw(WeightSpec((1000,)), 5, "t.weight", torch.float32), a[:1000])      # a prefix is the same numbers
    assert torch.equal(draw(spec, 5, "t.weight", torch.bfloat16), a.to(torch.bfloat16))        # one rounding
    z = a.double().numpy() / 0.02
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1) < 0.01 and abs((z ** 4).mean() - 3) < 0.1
    assert stats.kstest(z, "norm").pvalue > 1e-3 and np.abs(z).max() < 6.0
    assert abs(np.corrcoef(z[:-1], z[1:])[0, 1]) < 0.01
    g = draw(WeightSpec((4096,), init="one_plus_normal"), 5, "g.weight", torch.float32)
    assert abs(g.mean().item() - 1) < 2e-3 and abs(g.std().item() - 0.02) < 2e-3


def test_sharded_folder(tmp_path):
    cfg = config_from_dict(H.TINY_A)
    folder = write_random_model(str(tmp_path / "m"), cfg, 0, "float32")
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    names = f.names()
    half = len(names) // 2
    parts = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    for fn, ns in parts.items():
        write_safetensors(os.path.join(folder, fn), {n: f.tensor(n).clone() for n in ns})
    index = {"weight_map": {n: fn for fn, ns in parts.items() for n in ns}}
    os.remove(os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as fh:
        json.dump(index, fh)
    files = open_model_files(folder)
    assert sorted(files) == sorted(names)
    assert files[names[0]].path.endswith("00001-of-00002.safetensors")
