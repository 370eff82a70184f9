"""The safetensors reader and writer, the loader's one error, random weights."""
import json
import struct

import numpy as np
import pytest
import torch

import plain_impl
from litinfer_amd.config import Qwen2Config, qwen2_model_spec
from litinfer_amd.engine import expected_params_of_spec
from litinfer_amd.weights import (CheckpointFolder, ParamSpec, SafetensorsFile, WeightError, check_entries,
                                  stored_precision, write_random_model, write_safetensors)
from tiny_configs import TINY_A, TINY_B


def test_safetensors_round_trip_and_own_reader_agrees(tmp_path):
    g = torch.Generator().manual_seed(0)
    tensors = [("a", torch.randn(3, 5, generator=g)), ("b.c", torch.randn(7, generator=g).to(torch.bfloat16)),
               ("t", torch.arange(6, dtype=torch.int64).reshape(2, 3))]
    write_safetensors(tmp_path / "x.safetensors", tensors, metadata={"k": "v"})
    f = SafetensorsFile(tmp_path / "x.safetensors")
    assert f.entries == {"a": ("F32", (3, 5)), "b.c": ("BF16", (7,)), "t": ("I64", (2, 3))}
    for n, t in tensors:
        assert torch.equal(f.tensor(n), t)
    other = plain_impl.read_safetensors(tmp_path / "x.safetensors", np.float64)     # the tests' own reader
    assert np.array_equal(other["b.c"], tensors[1][1].double().numpy())
    from safetensors import safe_open                                               # and the format's library
    with safe_open(str(tmp_path / "x.safetensors"), "pt") as sf:
        assert torch.equal(sf.get_tensor("b.c"), tensors[1][1])


def test_offsets_are_checked(tmp_path):
    header = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}).encode()
    (tmp_path / "bad.safetensors").write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 16)
    with pytest.raises(ValueError, match="data_offsets"):
        SafetensorsFile(tmp_path / "bad.safetensors")


def test_stored_precision():
    assert stored_precision(torch.zeros(2, dtype=torch.bfloat16), False).dtype is torch.bfloat16
    assert stored_precision(torch.zeros(2, dtype=torch.float32), False).dtype is torch.float32
    assert stored_precision(torch.zeros(2, dtype=torch.float16), False).dtype is torch.float32
    assert stored_precision(torch.zeros(2, dtype=torch.int64), True).dtype is torch.int32


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    expected = {"a": ParamSpec((2, 3)), "b": ParamSpec((4,)), "bias": ParamSpec((4,), required=False),
                "c": ParamSpec((5,))}
    found = {"a": ("F32", (3, 2)), "zzz": ("F32", (1,)), "c": ("I32", (5,)),
             "x.rotary_emb.inv_freq": ("F32", (8,))}
    with pytest.raises(WeightError) as e:
        check_entries(expected, found, lambda n: n.endswith("rotary_emb.inv_freq"))
    err = e.value
    assert err.missing == ["b"] and err.unexpected == ["zzz"]
    assert err.wrong_shape == [("a", (2, 3), (3, 2))] and err.wrong_dtype[0][0] == "c"
    msg = str(err)
    for word in ("missing tensors (1)", "- b", "unexpected tensors (1)", "- zzz", "wrong shapes (1)",
                 "a: expected [2, 3], found [3, 2]"):
        assert word in msg


def test_expected_tensor_names_are_the_checkpoints():
    names = expected_params_of_spec(qwen2_model_spec(Qwen2Config.from_dict(TINY_B)))
    assert names["model.embed_tokens.weight"].shape == (320, 96)
    assert names["lm_head.weight"].shape == (320, 96) and names["model.norm.weight"].shape == (96,)
    assert not names["lm_head.weight"].required          # absent: tied to the table, as in the reference
    p = "model.layers.2."
    assert names[p + "self_attn.q_proj.weight"].shape == (96, 96)
    assert names[p + "self_attn.k_proj.weight"].shape == (32, 96)
    assert names[p + "self_attn.v_proj.bias"].shape == (32,) and not names[p + "self_attn.v_proj.bias"].required
    assert names[p + "self_attn.o_proj.weight"].shape == (96, 96)
    assert names[p + "mlp.gate_proj.weight"].shape == (224, 96)
    assert names[p + "mlp.down_proj.weight"].shape == (96, 224)
    assert names[p + "post_attention_layernorm.weight"].shape == (96,)
    assert len(names) == 3 + 3 * 12
    tied = expected_params_of_spec(qwen2_model_spec(Qwen2Config.from_dict(TINY_A)))
    assert "lm_head.weight" not in tied


def test_random_model_folder_is_seeded_and_distributed_as_said(tmp_path):
    a = write_random_model(tmp_path / "a", TINY_B, seed=3, dtype=torch.float32)
    b = write_random_model(tmp_path / "b", TINY_B, seed=3, dtype=torch.float32)
    c = write_random_model(tmp_path / "c", TINY_B, seed=4, dtype=torch.float32)
    fa, fb, fc = (CheckpointFolder(x) for x in (a, b, c))
    name = "model.layers.1.mlp.up_proj.weight"
    assert torch.equal(fa.tensor(name), fb.tensor(name)) and not torch.equal(fa.tensor(name), fc.tensor(name))
    w = fa.tensor(name)
    assert abs(float(w.mean())) < 2e-3 and abs(float(w.std()) - 0.02) < 2e-3
    n = fa.tensor("model.layers.0.input_layernorm.weight")
    assert abs(float(n.mean()) - 1.0) < 1e-2 and float(n.std()) < 0.04
    assert abs(float(fa.tensor("model.layers.0.self_attn.q_proj.bias").mean())) < 2e-2
    assert json.loads((a / "config.json").read_text())["num_hidden_layers"] == 3
    assert SafetensorsFile(write_random_model(tmp_path / "d", TINY_B, 3, torch.bfloat16) /
                           "model.safetensors").entries[name][0] == "BF16"


def _load(folder, cpu_ops, **kw):
    from litinfer_amd.engine import Engine
    return Engine.from_dir(folder, dtype="float32", device="cpu", max_tokens=64, max_seqs=2, **kw)


def _rewrite(folder, change):
    f = SafetensorsFile(folder / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.entries}
    f.close()
    change(tensors)
    write_safetensors(folder / "model.safetensors", tensors.items())
    return tensors


def test_loader_raises_one_error_for_a_broken_folder(tmp_path, cpu_ops):
    d = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype=torch.float32)
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.entries}
    f.close()
    del tensors["model.layers.1.mlp.down_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    tensors["model.layers.9.mlp.up_proj.weight"] = torch.zeros(2, 2)
    write_safetensors(d / "model.safetensors", tensors.items())
    with pytest.raises(WeightError) as e:
        _load(d, cpu_ops, strict_weights=True)
    assert e.value.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.9.mlp.up_proj.weight"]
    assert e.value.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (16, 64))]
    # without the strict switch an unknown tensor is no fault (python/llaisys/models/qwen2.py:152-194
    # lets unknown names fall through); what is missing or misshapen still is, in the same one error
    with pytest.raises(WeightError) as e:
        _load(d, cpu_ops)
    assert e.value.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == []
    assert e.value.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (16, 64))]


def test_unknown_tensors_are_counted_and_reported_in_one_line(tmp_path, cpu_ops, capsys):
    d = write_random_model(tmp_path / "m", TINY_B, seed=1, dtype=torch.float32)

    def change(t):
        t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)      # holds no weights: not even counted
        t["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
        t["some.other.tensor"] = torch.zeros(3)
    _rewrite(d, change)
    eng = _load(d, cpu_ops)
    assert eng.unused_weights == ["model.layers.7.mlp.up_proj.weight", "some.other.tensor"]
    err = capsys.readouterr().err
    lines = [l for l in err.splitlines() if "not used" in l]
    assert len(lines) == 1 and "2 stored tensor(s)" in lines[0] and "some.other.tensor" in lines[0]


def test_the_references_other_names_for_three_tensors_are_taken(tmp_path, cpu_ops):
    """transformer.wte.weight, model.lm_head.weight and transformer.ln_f.weight
    (python/llaisys/models/qwen2.py:139-149)."""
    d = write_random_model(tmp_path / "m", TINY_B, seed=1, dtype=torch.float32)
    want_norm = _load(d, cpu_ops).model.final_norm.weight.clone()      # (on the CPU a tensor may be the file's mapping)

    def change(t):
        t["transformer.wte.weight"] = t.pop("model.embed_tokens.weight")
        t["model.lm_head.weight"] = t.pop("lm_head.weight")
        t["transformer.ln_f.weight"] = t.pop("model.norm.weight")
    stored = _rewrite(d, change)
    eng = _load(d, cpu_ops, strict_weights=True)
    assert eng.unused_weights == []
    assert torch.equal(eng.model.embedding.table, stored["transformer.wte.weight"])
    assert torch.equal(eng.model.head.proj.weight, stored["model.lm_head.weight"])
    assert torch.equal(eng.model.final_norm.weight, want_norm)
    # a tensor stored under its own name wins; the alias beside it is one tensor too many
    _rewrite(d, lambda t: t.__setitem__("model.norm.weight", torch.ones(96)))
    eng = _load(d, cpu_ops)
    assert torch.equal(eng.model.final_norm.weight, torch.ones(96))
    assert eng.unused_weights == ["transformer.ln_f.weight"]


def test_head_matrix_stray_when_tied_and_absent_when_untied(tmp_path, cpu_ops, capsys):
    # tie_word_embeddings = true: a stored lm_head.weight is not used
    d = write_random_model(tmp_path / "a", TINY_A, seed=0, dtype=torch.float32)
    _rewrite(d, lambda t: t.__setitem__("lm_head.weight", torch.zeros(256, 64)))
    eng = _load(d, cpu_ops)
    assert eng.unused_weights == ["lm_head.weight"]
    assert eng.model.head.proj.weight.data_ptr() == eng.model.embedding.table.data_ptr()
    with pytest.raises(WeightError) as e:
        _load(d, cpu_ops, strict_weights=True)
    assert e.value.unexpected == ["lm_head.weight"]
    # untied, but no lm_head.weight stored: the table is used, with a note
    # (python/llaisys/models/qwen2.py:196-199)
    d = write_random_model(tmp_path / "b", TINY_B, seed=1, dtype=torch.float32)
    _rewrite(d, lambda t: t.pop("lm_head.weight"))
    capsys.readouterr()
    eng = _load(d, cpu_ops)
    assert eng.model.head.proj.weight.data_ptr() == eng.model.embedding.table.data_ptr()
    assert "lm_head.weight is not stored" in capsys.readouterr().err


def test_biases_are_optional_and_tied_head_shares_the_table(tmp_path, cpu_ops):
    d = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype=torch.float32)
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.entries if not n.endswith("bias")}
    f.close()
    write_safetensors(d / "model.safetensors", tensors.items())
    eng = _load(d, cpu_ops)
    assert eng.model.layers[0].mixer.qkv.bias is None
    assert eng.model.head.proj.weight.data_ptr() == eng.model.embedding.table.data_ptr()
