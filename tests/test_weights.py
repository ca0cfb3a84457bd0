"""The safetensors container, loading by tensor name with one clear error, random weights."""

import json
import struct

import pytest
import numpy as np
import torch

import helpers
from from_scratch_inference_engine_amd.models import build_model_spec, parse_config
from from_scratch_inference_engine_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError,
                                                       load_weights, write_random_model, write_safetensors)
from from_scratch_inference_engine_amd.weights.loader import check_against, fill_parts


def _raw_file(path, header: dict, data: bytes, header_len=None):
    text = json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(text) if header_len is None else header_len) + text + data)
    return path


def test_reads_the_reference_fixture(tmp_path):
    # tests/cpp/test_safetensors.cpp:26-39: F32 [2,2] and BF16 [2] (0x3F80 -> 1, 0x4000 -> 2)
    data = struct.pack("<4f", 1.0, 2.0, 3.0, 4.0) + struct.pack("<2H", 0x3F80, 0x4000)
    f = SafetensorsFile(_raw_file(tmp_path / "m.safetensors", {
        "__metadata__": {"format": "pt"},
        "a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 16]},
        "b": {"dtype": "BF16", "shape": [2], "data_offsets": [16, 20]}}, data))
    assert f.get("a").tolist() == [[1.0, 2.0], [3.0, 4.0]] and f.dtype("a") == torch.float32
    assert f.get("b").float().tolist() == [1.0, 2.0] and f.dtype("b") == torch.bfloat16
    assert "a" in f and "c" not in f
    with pytest.raises(SafetensorsError, match="missing tensor 'c'"):
        f.get("c")


@pytest.mark.parametrize("header, data, header_len, message", [
    (None, b"\x01\x02", None, "smaller than"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}}, b"\0" * 4, 10 ** 9, "exceeds"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, b"\0" * 4, None, "byte count"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 8]}}, b"\0" * 4, None, "out of range"),
    ({"a": {"dtype": "Q4", "shape": [1], "data_offsets": [0, 4]}}, b"\0" * 4, None, "unsupported dtype"),
    ({"a": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 4]}}, b"\0" * 4, None, "negative"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]},
      "b": {"dtype": "F32", "shape": [1], "data_offsets": [2, 6]}}, b"\0" * 8, None, "overlapping"),
    ({"a": {"dtype": "F32", "shape": [1]}}, b"\0" * 4, None, "malformed"),
])
def test_malformed_files_are_refused(tmp_path, header, data, header_len, message):
    p = tmp_path / "bad.safetensors"
    if header is None:
        p.write_bytes(data)
    else:
        _raw_file(p, header, data, header_len)
    with pytest.raises(SafetensorsError, match=message):
        SafetensorsFile(p)


def test_duplicate_names_and_bad_json(tmp_path):
    text = b'{"a":{"dtype":"F32","shape":[1],"data_offsets":[0,4]},"a":{"dtype":"F32","shape":[1],"data_offsets":[4,8]}}'
    p = tmp_path / "dup.safetensors"
    p.write_bytes(struct.pack("<Q", len(text)) + text + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="duplicate"):
        SafetensorsFile(p)
    p.write_bytes(struct.pack("<Q", 5) + b"{nope" + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="invalid header JSON"):
        SafetensorsFile(p)


def test_round_trip_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file

    g = torch.Generator().manual_seed(0)
    tensors = {"w": torch.randn(3, 5, generator=g).bfloat16(), "v": torch.randn(7, generator=g),
               "i": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    write_safetensors(tmp_path / "ours.safetensors", tensors)
    theirs = load_file(str(tmp_path / "ours.safetensors"))
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    ours = SafetensorsFile(tmp_path / "theirs.safetensors")
    for k, t in tensors.items():
        assert torch.equal(theirs[k], t) and torch.equal(ours.get(k), t) and ours.dtype(k) == t.dtype


def _spec(cfg):
    return build_model_spec(parse_config(cfg))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = helpers.TINY_B
    tensors = helpers.random_tensors(cfg, 0)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(32, dtype=torch.bfloat16)
    tensors["model.layers.2.self_attn.k_proj.bias"] = torch.zeros(64, dtype=torch.bfloat16)
    tensors["model.embed_tokens.weight"] = torch.zeros(509, 191, dtype=torch.bfloat16)
    d = helpers.make_model_dir(tmp_path / "m", cfg, 0, tensors=tensors)
    with pytest.raises(WeightsError) as err:
        load_weights(d / "model.safetensors", _spec(cfg).bindings, torch.bfloat16, "cpu")
    e = err.value
    assert e.missing == ["lm_head.weight", "model.layers.1.mlp.up_proj.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.q_norm.weight"]
    assert [w[0] for w in e.wrong_shape] == ["model.embed_tokens.weight", "model.layers.2.self_attn.k_proj.bias"]
    text = str(e)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "expected [509, 192], found [509, 191]",
                  "model.layers.1.mlp.up_proj.weight  expected shape [320, 192]"):
        assert piece in text


def test_a_weight_stored_in_a_dtype_it_cannot_mean_is_refused(tmp_path):
    """An integer, boolean or 64-bit tensor under a weight's name is a wrong file, not a value to
    cast: the reference's container accepts F32, F16 and BF16 only (include/engine/dtype.hpp:68-79,
    tests/cpp/test_safetensors.cpp:100).  The refusal comes with the other problems, in one error,
    and before any parameter is set."""
    cfg = helpers.TINY_A
    tensors = helpers.random_tensors(cfg, 2)
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.ones(64, 64, dtype=torch.int32)
    tensors["model.layers.1.input_layernorm.weight"] = torch.ones(64, dtype=torch.bool)
    tensors["model.layers.1.mlp.down_proj.weight"] = torch.zeros(64, 176, dtype=torch.float64)
    tensors["model.layers.1.self_attn.v_proj.bias"] = torch.zeros(32, dtype=torch.float16)  # fine
    del tensors["model.norm.weight"]
    d = helpers.make_model_dir(tmp_path / "m", cfg, 2, tensors=tensors)
    spec = _spec(cfg)
    with pytest.raises(WeightsError) as err:
        load_weights(d, spec.bindings, torch.bfloat16, "cpu", spec.ignore_unexpected)
    e = err.value
    assert e.missing == ["model.norm.weight"]
    assert [(n, str(t)) for n, _, t in e.wrong_dtype] == [
        ("model.layers.0.self_attn.q_proj.weight", "torch.int32"),
        ("model.layers.1.input_layernorm.weight", "torch.bool"),
        ("model.layers.1.mlp.down_proj.weight", "torch.float64")]
    for piece in ("wrong dtypes (3)", "q_proj.weight  stored as int32", "input_layernorm.weight  stored as bool",
                  "missing tensors (1)"):
        assert piece in str(e), piece
    assert all(getattr(p, a, None) is None for p in spec.all_parts() for a in p.param_decls()), "nothing was set"
    # the same file with those three as they should be loads
    good = helpers.random_tensors(cfg, 2)
    good["model.layers.1.self_attn.v_proj.bias"] = torch.zeros(32, dtype=torch.float16)
    load_weights(helpers.make_model_dir(tmp_path / "g", cfg, 2, tensors=good), spec.bindings, torch.bfloat16, "cpu",
                 spec.ignore_unexpected)
    # and a caller that fills parts without the check meets the same refusal, tensor by tensor
    with pytest.raises(WeightsError, match="q_proj.weight must hold 32- or 16-bit floating point, found int32"):
        fill_parts(_spec(cfg).bindings, lambda n: tensors.get(n, good[n]), torch.bfloat16, "cpu")


def test_a_checkpoint_in_several_files_is_read_through_its_index(tmp_path):
    """Large checkpoints come as several safetensors files and model.safetensors.index.json; the
    folder loads to the same parameters as the single file, and an index that does not fit its
    files is refused."""
    import json

    from from_scratch_inference_engine_amd.weights import write_safetensors

    cfg = helpers.TINY_A
    tensors = helpers.random_tensors(cfg, 5, torch.float32)
    single = helpers.make_model_dir(tmp_path / "single", cfg, 5, tensors=tensors)
    sharded = tmp_path / "sharded"
    sharded.mkdir()
    (sharded / "config.json").write_text((single / "config.json").read_text())
    names = sorted(tensors)
    parts = {"model-00001-of-00002.safetensors": names[0::2], "model-00002-of-00002.safetensors": names[1::2]}
    for fname, held in parts.items():
        write_safetensors(sharded / fname, {n: tensors[n] for n in held})
    index = {"metadata": {"total_size": 0}, "weight_map": {n: f for f, held in parts.items() for n in held}}
    (sharded / "model.safetensors.index.json").write_text(json.dumps(index))
    a, b = _spec(cfg), _spec(cfg)
    load_weights(single, a.bindings, torch.float32, "cpu")
    load_weights(sharded, b.bindings, torch.float32, "cpu")
    for pa, pb in zip(a.all_parts(), b.all_parts()):
        for attr in pa.param_decls():
            assert torch.equal(getattr(pa, attr), getattr(pb, attr)), attr
    # a tensor missing from the index is reported like any missing tensor
    del index["weight_map"][names[0]]
    (sharded / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(WeightsError, match="holds tensors the index does not send there"):
        load_weights(sharded, _spec(cfg).bindings, torch.float32, "cpu")
    index["weight_map"][names[0]] = "model-00002-of-00002.safetensors"
    (sharded / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(WeightsError, match="which does not hold it"):
        load_weights(sharded, _spec(cfg).bindings, torch.float32, "cpu")
    index["weight_map"][names[0]] = "../elsewhere.safetensors"
    (sharded / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(WeightsError, match="must lie in the model folder"):
        load_weights(sharded, _spec(cfg).bindings, torch.float32, "cpu")
    with pytest.raises(WeightsError, match="neither model.safetensors nor"):
        load_weights(tmp_path, _spec(cfg).bindings, torch.float32, "cpu")


def test_storage_kinds_and_fusion(tmp_path):
    """Matrices take the compute dtype, vectors stay float32 whatever the file stores, q/k/v
    are concatenated in that order, gate/up are interleaved row by row, a tied head shares the
    embedding's memory."""
    cfg = helpers.TINY_A
    tensors = helpers.random_tensors(cfg, 3, torch.float32)
    d = helpers.make_model_dir(tmp_path / "m", cfg, 3, tensors=tensors)
    for dtype in (torch.bfloat16, torch.float32):
        spec = _spec(cfg)
        load_weights(d / "model.safetensors", spec.bindings, dtype, "cpu")
        mixer, ffn = spec.layers[1].mixer, spec.layers[1].ffn
        p = "model.layers.1."
        want = torch.cat([tensors[p + f"self_attn.{n}_proj.weight"] for n in "qkv"]).to(dtype)
        assert mixer.qkv_weight.dtype == dtype and torch.equal(mixer.qkv_weight, want)
        assert mixer.qkv_bias.dtype == torch.float32
        assert torch.equal(mixer.qkv_bias, torch.cat([tensors[p + f"self_attn.{n}_proj.bias"] for n in "qkv"]))
        gate, up = tensors[p + "mlp.gate_proj.weight"].to(dtype), tensors[p + "mlp.up_proj.weight"].to(dtype)
        assert torch.equal(ffn.gate_up_weight[0::2], gate) and torch.equal(ffn.gate_up_weight[1::2], up)  # interleaved
        assert spec.layers[0].mixer_norm.weight.dtype == torch.float32
        assert torch.equal(spec.final_norm.weight, tensors["model.norm.weight"])
        assert spec.lm_head.weight.data_ptr() == spec.embedding.weight.data_ptr()


def test_tied_checkpoint_may_carry_a_head_and_int_tables():
    cfg = helpers.TINY_A
    spec = _spec(cfg)
    found = {n: s for n, s in helpers.expected_tensor_shapes(cfg).items()}
    found["lm_head.weight"] = (256, 64)
    check_against(spec.bindings, found, spec.ignore_unexpected)  # no error
    with pytest.raises(WeightsError, match="unexpected"):
        check_against(spec.bindings, found)
    # integer tables are kept as int32, and a float tensor in their place is refused
    from from_scratch_inference_engine_amd.weights import ParamBinding, TensorSpec

    class Holder:
        table = None
    b = [ParamBinding(Holder, "table", [TensorSpec("t", (4,), "int")], "int_table")]
    fill_parts(b, lambda n: torch.arange(4, dtype=torch.int64), torch.bfloat16, "cpu")
    assert Holder.table.dtype == torch.int32 and Holder.table.tolist() == [0, 1, 2, 3]
    with pytest.raises(WeightsError, match="integers"):
        fill_parts(b, lambda n: torch.zeros(4), torch.bfloat16, "cpu")


def test_random_model_folder(tmp_path):
    cfg = parse_config(helpers.TINY_B)
    a = write_random_model(cfg, 11, tmp_path / "a")
    b = write_random_model(cfg, 11, tmp_path / "b")
    c = write_random_model(cfg, 12, tmp_path / "c", torch.float32)
    fa, fb, fc = (SafetensorsFile(x / "model.safetensors") for x in (a, b, c))
    assert sorted(fa.names()) == sorted(helpers.expected_tensor_shapes(helpers.TINY_B))
    for n in fa.names():
        assert fa.shape(n) == helpers.expected_tensor_shapes(helpers.TINY_B)[n]
        assert torch.equal(fa.get(n), fb.get(n)) and fa.dtype(n) == torch.bfloat16 and fc.dtype(n) == torch.float32
    assert not torch.equal(fa.get("lm_head.weight").float(), fc.get("lm_head.weight"))
    w = fc.get("model.layers.0.mlp.down_proj.weight")
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    assert abs(fc.get("model.norm.weight").mean().item() - 1.0) < 0.01
    assert parse_config(json.loads((a / "config.json").read_text())) == cfg
    # the written folder loads without complaint
    load_weights(a / "model.safetensors", _spec(helpers.TINY_B).bindings, torch.bfloat16, "cpu")


def test_random_values_are_a_function_of_seed_name_and_index():
    """The counter-based generator on the host: an element does not depend on how many elements
    are made with it or on other tensors; the values are close to normal with the stated
    deviation; integer tables are 15-bit ids."""
    from from_scratch_inference_engine_amd.weights import random_init as r
    from from_scratch_inference_engine_amd.weights.loader import TensorSpec

    key = r.stream_key(7, "model.layers.3.mlp.up_proj.weight")
    whole = r.host_values(key, (1 << 20) + 77, "weight")       # more than one chunk of the host loop
    assert np.array_equal(r.host_values(key, 1000, "weight"), whole[:1000])
    assert np.array_equal(r.host_values(key, 50, "norm"), whole[:50] + np.float32(1.0))
    assert not np.array_equal(r.host_values(r.stream_key(8, "model.layers.3.mlp.up_proj.weight"), 1000, "weight"), whole[:1000])
    assert not np.array_equal(r.host_values(r.stream_key(7, "model.layers.3.mlp.gate_proj.weight"), 1000, "weight"), whole[:1000])
    z = whole.astype(np.float64) / 0.02
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3 and abs((z ** 4).mean() - 3.0) < 0.2 and np.abs(z).max() < 4.9
    assert abs((np.abs(z) < 1.0).mean() - 0.68) < 0.01  # (the sum of eight uniform fields: 0.677 where a normal has 0.683)
    ids = r.host_values(key, 4096, "int")
    assert ids.dtype == np.int32 and ids.min() >= 0 and ids.max() < 1 << 15 and len(set(ids.tolist())) > 3500
    # element 0 written out by hand
    def output(number):
        x = (key + (number + 1) * 0x9E3779B97F4A7C15) & ((1 << 64) - 1)
        x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & ((1 << 64) - 1)
        x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & ((1 << 64) - 1)
        return x ^ (x >> 31)
    total = sum((w >> s) & 0xFFFF for w in (output(0), output(1)) for s in (0, 16, 32, 48))
    assert whole[0] == np.float32(total - 262140) * np.float32(1.8688124e-05) * np.float32(0.02)
    t = r.random_tensor(TensorSpec("model.layers.3.mlp.up_proj.weight", (10, 100)), 7, torch.bfloat16)
    assert t.dtype == torch.bfloat16 and torch.equal(t, torch.from_numpy(whole[:1000]).reshape(10, 100).to(torch.bfloat16))
