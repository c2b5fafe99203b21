import json

import pytest

import helpers as H
from ginfer_amd.config import (ConfigError, config_from_dict, config_from_folder, registered_architectures,
                               Qwen2Config)


def test_required_keys_and_defaults():
    d = dict(H.TINY_B)
    for k in ("rms_norm_eps", "rope_theta", "tie_word_embeddings", "eos_token_id", "use_sliding_window"):
        d.pop(k, None)
    c = config_from_dict(d)
    assert isinstance(c, Qwen2Config)
    # the reference's defaults: ginfer/model/loader/model_loader.cc:45-51, 100-105
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0 and c.tie_word_embeddings is False
    assert c.eos_token_ids == [d["vocab_size"] - 1] and c.head_dim == 192 // 6
    for k in ("num_hidden_layers", "vocab_size", "max_position_embeddings", "num_attention_heads",
              "num_key_value_heads", "hidden_size", "intermediate_size"):
        bad = dict(H.TINY_B)
        del bad[k]
        with pytest.raises(ConfigError, match=k):
            config_from_dict(bad)


def test_registry_key_and_errors(tmp_path):
    assert "Qwen2ForCausalLM" in registered_architectures()
    d = dict(H.TINY_A)
    del d["architectures"]
    assert isinstance(config_from_dict(d), Qwen2Config)        # model_type is the reference's key
    with pytest.raises(ConfigError, match="NoSuchLM.*registered.*Qwen2ForCausalLM"):
        config_from_dict(dict(H.TINY_A, architectures=["NoSuchLM"], model_type="nosuch"))
    with pytest.raises(ConfigError, match="no config.json"):
        config_from_folder(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        config_from_folder(str(tmp_path))


def test_values_are_checked():
    for change, pat in ((dict(num_key_value_heads=3), "multiple"), (dict(head_dim=15), "even"),
                        (dict(rope_scaling={"type": "yarn"}), "rope_scaling"), (dict(hidden_act="gelu"), "hidden_act"),
                        (dict(num_hidden_layers=0), "num_hidden_layers"), (dict(vocab_size="x"), "vocab_size"),
                        (dict(use_sliding_window=True, sliding_window=None), "sliding_window"),
                        (dict(torch_dtype="int8"), "torch_dtype"), (dict(hidden_size=65), "head_dim")):
        with pytest.raises(ConfigError, match=pat):
            config_from_dict(dict(H.TINY_A, **change))


def test_no_size_stands_in_code():
    """Every size of the model comes from config.json: the spec of each configuration carries its own
    numbers through to the parts."""
    for name, (d, _, _) in H.TINY.items():
        c = config_from_dict(d)
        spec = c.model_spec()
        assert len(spec.layers) == d["num_hidden_layers"] == len(spec.schedule)
        hd = d.get("head_dim") or d["hidden_size"] // d["num_attention_heads"]
        for i, layer in enumerate(spec.layers):
            m, f = layer.parts["mixer"].params, layer.parts["feed_forward"].params
            assert (m["num_heads"], m["num_kv_heads"], m["head_dim"]) == (d["num_attention_heads"], d["num_key_value_heads"], hd)
            assert m["position"].params["theta"] == d["rope_theta"] and m["position"].params["rotary_dim"] == hd
            assert f["intermediate_size"] == d["intermediate_size"] and layer.parts["mixer_norm"].params["eps"] == d["rms_norm_eps"]
            assert m["qkv_bias"] is True and m["out_bias"] is False     # ginfer/model/qwen2.cc:15-17
        assert spec.head.params["tied"] == d["tie_word_embeddings"] and spec.vocab_size == d["vocab_size"]
    c = config_from_dict(H.TINY_C)
    assert [l.parts["mixer"].params["window"] for l in c.model_spec().layers] == [None, 40, 40, 40]
    assert [l.parts["mixer"].params["window"] for l in config_from_dict(H.TINY_A).model_spec().layers] == [None, None]
    assert config_from_dict(H.TINY_B).eos_token_ids == [998, 999]


def test_round_trip_through_a_folder(tmp_path):
    c = config_from_dict(H.TINY_C)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    assert config_from_folder(str(tmp_path)) == c


def test_schedule_is_validated():
    from ginfer_amd.config import ScheduleEntry
    spec = config_from_dict(H.TINY_B).model_spec()
    spec.schedule = [ScheduleEntry(0), ScheduleEntry(5)]
    with pytest.raises(ValueError, match="layer 5"):
        spec.validate()
    spec.schedule = [ScheduleEntry(0, cache_of=0)]
    with pytest.raises(ValueError, match="does not run before"):
        spec.validate()
    spec.schedule = [ScheduleEntry(0), ScheduleEntry(1, cache_of=0), ScheduleEntry(2, cache_of=1)]
    with pytest.raises(ValueError, match="owns none"):
        spec.validate()


def test_partial_sums_are_added_up_for_norms_that_do_not_take_them():
    import torch
    from ginfer_amd.parts.block import whole

    class Plain:
        dtype = torch.bfloat16

    class Taking(Plain):
        accepts_partial_sums = True
    parts = torch.randn(4, 3, 8)
    out = whole(parts, Plain())
    assert out.shape == (3, 8) and out.dtype == torch.bfloat16
    assert torch.allclose(out.float(), parts.sum(0), atol=2e-2)
    assert whole(parts, Taking()) is parts
    x = torch.randn(3, 8)
    assert whole(x, Plain()) is x and whole(None, Plain()) is None


def test_header_declares_every_entry_point_as_it_is_defined():
    """ginfer_amd/csrc/ginfer_amd.h repeats the parameter lists of the `extern "C"` definitions in the sources."""
    import glob
    import os
    import re
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ginfer_amd", "csrc")

    def squeeze(text):
        return re.sub(r"\s+", " ", text.replace("struct ", "")).strip()
    defined = {}
    for path in glob.glob(os.path.join(csrc, "*.hip")):
        src = open(path).read()
        for m in re.finditer(r'extern "C"\s+([\w \*]+?)\s*\b(ga_\w+)\s*\(([^)]*)\)\s*\{', src):
            defined[m.group(2)] = (squeeze(m.group(1)), squeeze(m.group(3)))
    header = open(os.path.join(csrc, "ginfer_amd.h")).read()
    header = re.sub(r"//[^\n]*", "", header)
    declared = {}
    for m in re.finditer(r'([\w \*]+?)\s*\b(ga_\w+)\s*\(([^)]*)\)\s*;', header):
        declared[m.group(2)] = (squeeze(m.group(1)), squeeze(m.group(3)))
    assert defined and set(defined) == set(declared), (sorted(set(defined) ^ set(declared)))
    for name in defined:
        assert defined[name] == declared[name], "%s: defined %s, declared %s" % (name, defined[name], declared[name])


def test_dispatch_thresholds_live_in_one_table():
    import os
    """Every threshold that chooses between two ways of doing the same work is a field of kernels/tuning.py; values can
    be set for the process or from the environment, unknown names are refused."""
    import json
    import subprocess
    import sys
    from ginfer_amd.kernels.tuning import Tuning, TUNING
    t = Tuning()
    t.update({"library_from_rows": 32, "padded_rows_times_weights": 2e12})
    assert t.library_from_rows == 32 and t.padded_rows_times_weights == 2e12 and TUNING.library_from_rows == 16
    with pytest.raises(KeyError, match="no tuning value"):
        t.update({"library_from_row": 1})
    out = subprocess.run([sys.executable, "-c", "from ginfer_amd.kernels.tuning import TUNING; print(TUNING.decode_max_splits)"],
                         env=dict(os.environ, GINFER_AMD_TUNING=json.dumps({"decode_max_splits": 64})), capture_output=True,
                         text=True, cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert out.stdout.strip() == "64", out.stderr
