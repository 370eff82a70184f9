"""The typed configuration and the registry."""
import json

import pytest

from litinfer_amd.config import (ConfigError, Qwen2Config, load_config, lookup, qwen2_model_spec,
                                 register_architecture, registered_architectures)
from tiny_configs import TINY_A, TINY_B, TINY_C


def test_reads_every_size_from_config_json():
    c = Qwen2Config.from_dict(TINY_B)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads) == (3, 96, 3, 1)
    assert (c.head_dim, c.intermediate_size, c.vocab_size) == (32, 224, 320)
    assert (c.rope_theta, c.rms_norm_eps, c.max_position_embeddings) == (1e6, 1e-5, 256)
    assert c.tie_word_embeddings is False and c.eos_token_ids == (7, 9)
    assert [c.window_of_layer(l) for l in range(3)] == [0, 32, 32]


def test_defaults_follow_the_reference_reader():
    # python/llaisys/models/qwen2.py:269-282: kv heads default to heads, head_dim to hidden // heads,
    # eps to 1e-6, theta to 10000
    raw = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 1, "hidden_size": 32,
           "num_attention_heads": 4, "intermediate_size": 48, "vocab_size": 11,
           "max_position_embeddings": 16}
    c = Qwen2Config.from_dict(raw)
    assert c.num_key_value_heads == 4 and c.head_dim == 8
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0
    assert c.eos_token_ids == () and not c.use_sliding_window
    assert [c.window_of_layer(0)] == [0]


def test_config_round_trips():
    for raw in (TINY_A, TINY_B, TINY_C):
        c = Qwen2Config.from_dict(raw)
        assert Qwen2Config.from_dict(c.to_dict()) == c


@pytest.mark.parametrize("patch,word", [
    ({"num_hidden_layers": None}, "num_hidden_layers"), ({"hidden_size": 0}, "hidden_size"),
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"),
    ({"hidden_act": "gelu"}, "hidden_act"), ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"rope_theta": 0}, "rope_theta"), ({"rms_norm_eps": -1.0}, "rms_norm_eps"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window")])
def test_bad_values_are_refused_with_the_key_named(patch, word):
    raw = dict(TINY_A)
    raw.update(patch)
    with pytest.raises(ConfigError, match=word):
        Qwen2Config.from_dict(raw)


def test_spec_is_data_layer_by_layer():
    spec = qwen2_model_spec(Qwen2Config.from_dict(TINY_B))
    assert len(spec.layers) == 3 and [e.layer for e in spec.order] == [0, 1, 2]
    assert [l.parts["mixer"].args["window"] for l in spec.layers] == [0, 32, 32]
    assert spec.layers[1].parts["mixer"].prefix == "model.layers.1.self_attn."
    assert spec.head.args["tied_to"] is None
    assert qwen2_model_spec(Qwen2Config.from_dict(TINY_A)).head.args["tied_to"] == "model.embed_tokens.weight"


def test_registry(tmp_path):
    assert "Qwen2ForCausalLM" in registered_architectures()
    assert lookup("qwen2") is lookup("Qwen2ForCausalLM")
    with pytest.raises(KeyError, match="registered: .*Qwen2ForCausalLM"):
        lookup("NoSuchModel")
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    arch, cfg, spec = load_config(tmp_path)
    assert arch.name == "Qwen2ForCausalLM" and cfg.hidden_size == 64 and spec.vocab_size == 256
    with pytest.raises(FileNotFoundError, match="Config file not found"):
        load_config(tmp_path / "nowhere")
    raw = dict(TINY_A, architectures=["Other"])
    (tmp_path / "config.json").write_text(json.dumps(raw))
    with pytest.raises(KeyError, match="unknown architecture 'Other'"):
        load_config(tmp_path)


def test_order_must_read_an_earlier_owning_entry():
    from dataclasses import replace
    from litinfer_amd.config import ExecEntry
    spec = qwen2_model_spec(Qwen2Config.from_dict(TINY_A))
    replace(spec, order=(ExecEntry(0), ExecEntry(1), ExecEntry(0, cache_from=0))).validate()
    for bad in ((ExecEntry(0, cache_from=0),), (ExecEntry(0), ExecEntry(1, 0), ExecEntry(1, 1)), (ExecEntry(5),)):
        with pytest.raises(ValueError):
            replace(spec, order=bad).validate()


def test_the_references_environment_switches(tmp_path, monkeypatch, capsys, cpu_ops):
    """LLAISYS_NUM_BLOCKS sizes the pool, LLAISYS_TRACE prints a line per step
    (src/llaisys/models/qwen2.cpp:19, :121), LLAISYS_PROFILE's table lists the
    operators by phase (src/utils/profiler.cpp:48-110)."""
    import io
    import helpers
    from tiny_configs import TINY_A
    from litinfer_amd.engine import Engine, StepEntry
    from litinfer_amd.utils import OpProfiler
    d = helpers.make_model(tmp_path, TINY_A, 0)
    monkeypatch.setenv("LLAISYS_NUM_BLOCKS", "7")
    monkeypatch.setenv("LLAISYS_TRACE", "1")
    eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=16, max_seqs=2)
    assert eng.cache.groups[0].pool.capacity == 7
    eng.step([StepEntry("a", [1, 2, 3], [2])])
    assert "step 0: 1 requests, 3 tokens, 1 rows of logits" in capsys.readouterr().err
    monkeypatch.setenv("LLAISYS_NUM_BLOCKS", "many")
    with pytest.raises(ValueError, match="LLAISYS_NUM_BLOCKS"):
        Engine.from_dir(d, dtype="float32", device="cpu", page_size=16, max_seqs=2)
    prof = OpProfiler(False)
    prof.phase = "prefill"
    prof.timed("linear", lambda: None, lambda: None)
    prof.phase = "decode"
    prof.timed("linear", lambda: None, lambda: None)
    prof.timed("linear", lambda: None, lambda: None)
    out = io.StringIO()
    prof.report(out)
    lines = out.getvalue().splitlines()
    assert any(l.startswith("decode") and " 2 " in l for l in lines) and any(l.startswith("prefill") for l in lines)
