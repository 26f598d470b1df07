"""Host side of the loader, no GPU needed: the SafeTensors reader against the scenarios of
spec/sharded_safetensors_spec.cr, the reference's tiny-llama data file read with the
`safetensors` package, and files written here in every float type; config.json parsing and the
llama3 RoPE frequencies against transformers' values for the published Llama-3 parameters."""
import json
import os
import struct

import numpy as np
import pytest

import shainet_amd as sa
import tinyllama
from oracle import oracle as orc


def write_safetensors(path, tensors, metadata=None):
    """tensors: name -> (dtype string, shape, raw little-endian bytes)."""
    header, blob = {}, b""
    if metadata:
        header["__metadata__"] = metadata
    for name, (dtype, shape, raw) in tensors.items():
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + blob)


def f32(vals):
    return ("F32", [len(vals)], np.asarray(vals, "<f4").tobytes())


def test_sharded_file_routes_each_tensor_to_its_shard(tmp_path):
    # spec/sharded_safetensors_spec.cr:38-77
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", {"a": f32([1.0, 2.0, 3.0])})
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", {"b": f32([4.0, 5.0])})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({
        "metadata": {"total_size": 20},
        "weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}))
    sf = sa.SafeTensors(str(tmp_path))
    assert sf.has_tensor("a") and sf.has_tensor("b") and not sf.has_tensor("missing")
    assert sorted(sf.tensor_names()) == ["a", "b"]
    np.testing.assert_array_equal(sf.read_f32("a"), [1.0, 2.0, 3.0])
    np.testing.assert_array_equal(sf.read_f32("b"), [4.0, 5.0])
    ma = sf.read_matrix("a")
    assert ma.shape == (1, 3) and ma[0, 2] == 3.0
    with pytest.raises(sa.ArgumentError, match="not found"):
        sf.read_f32("missing")
    sf.close()


def test_open_selects_single_file_then_index_then_fails(tmp_path):
    # spec/sharded_safetensors_spec.cr:80 ff. (HFLoader.open_safetensors)
    single = tmp_path / "single"
    single.mkdir()
    write_safetensors(single / "model.safetensors", {"w": f32([7.0])}, metadata={"format": "pt"})
    sf = sa.SafeTensors(str(single))
    assert sf.tensor_names() == ["w"] and sf.read_f32("w")[0] == 7.0
    assert sa.SafeTensors(str(single / "model.safetensors")).has_tensor("w")   # a file path works too
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(sa.ArgumentError, match="No model.safetensors"):
        sa.SafeTensors(str(empty))
    bad = tmp_path / "bad.safetensors"
    bad.write_bytes(struct.pack("<Q", 200_000_000) + b"{}")
    with pytest.raises(sa.ArgumentError, match="header too large"):
        sa.SafeTensors(str(bad))


def test_float_types_convert_as_the_reference_does(tmp_path):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(300) * 3).astype(np.float32)
    half = x.astype(np.float16)
    bf16_bits = (x.view(np.uint32) >> 16).astype("<u2")           # truncation: any bit pattern will do
    f64 = rng.standard_normal(50) * 1e3
    special = np.array([0x0000, 0x8000, 0x7C00, 0xFC00, 0x7E00, 0x3C00, 0x0001, 0x03FF, 0x8200], "<u2")
    write_safetensors(tmp_path / "t.safetensors", {
        "f32": ("F32", [20, 15], x.tobytes()), "f16": ("F16", [300], half.tobytes()),
        "bf16": ("BF16", [300], bf16_bits.tobytes()), "f64": ("F64", [50], f64.astype("<f8").tobytes()),
        "f16_special": ("F16", [9], special.tobytes()), "i32": ("I32", [2], np.array([1, 2], "<i4").tobytes())})
    sf = sa.SafeTensors(str(tmp_path / "t.safetensors"))
    assert sf.info("f32") == ("F32", [20, 15], 1200)
    np.testing.assert_array_equal(sf.read_matrix("f32"), x.reshape(20, 15))
    np.testing.assert_array_equal(sf.read_f32("f16"), half.astype(np.float32))       # normal halves are exact
    np.testing.assert_array_equal(sf.read_f32("bf16"), (bf16_bits.astype(np.uint32) << 16).view(np.float32))
    np.testing.assert_array_equal(sf.read_f32("f64"), f64.astype(np.float32))
    got = sf.read_f32("f16_special")
    assert got[0] == 0 and np.signbit(got[1]) and got[1] == 0 and got[2] == np.inf and got[3] == -np.inf
    assert np.isnan(got[4]) and got[5] == 1.0
    # subnormal halves: the reference writes exponent 127 + e (safetensors.cr:199-208); kept bit for bit
    assert got[6] == np.float32(2.0 ** -11) and got[7] == np.float32(2.0 ** -2 * (1 + 0x3FE / 1024))
    assert got[8] == -np.float32(2.0 ** -2)
    with pytest.raises(sa.ArgumentError, match="Unsupported dtype"):
        sf.read_f32("i32")


def test_tiny_llama_file_reads_like_the_safetensors_package():
    from safetensors.numpy import load_file

    want = load_file(os.path.join(tinyllama.DIR, "model.safetensors"))
    sf = sa.SafeTensors(tinyllama.DIR)
    assert sorted(sf.tensor_names()) == sorted(want)
    for name, arr in want.items():
        dtype, shape, nbytes = sf.info(name)
        assert shape == list(arr.shape) and nbytes == arr.nbytes
        np.testing.assert_array_equal(sf.read_f32(name), arr.astype(np.float32).reshape(-1))


def _write_config(d, **kw):
    cfg = {"model_type": "llama", "vocab_size": 100, "hidden_size": 64, "num_attention_heads": 4,
           "num_hidden_layers": 2, "intermediate_size": 128, "rms_norm_eps": 1e-5}
    cfg.update(kw)
    (d / "config.json").write_text(json.dumps(cfg))


def test_config_defaults_follow_load_llama_config(tmp_path):
    c = sa.HFLoader.load_llama_config(tinyllama.DIR)
    assert (c["model_type"], c["vocab_size"], c["hidden_size"], c["num_attention_heads"], c["num_hidden_layers"],
            c["intermediate_size"], c["num_key_value_heads"]) == ("llama", 32000, 16, 4, 2, 64, 4)
    assert c["rms_norm_eps"] == 1e-6 and c["rope_theta"] == 10000.0 and c["tie_word_embeddings"] == 0
    assert c["head_dim"] == 0 and c["rope_llama3"] == 0 and sa.HFLoader.compute_rope_freqs(c) is None
    _write_config(tmp_path)                                       # nothing optional given
    c = sa.HFLoader.load_llama_config(str(tmp_path))
    assert c["rope_theta"] == 10000.0 and c["num_key_value_heads"] == 4 and c["tie_word_embeddings"] == 0
    _write_config(tmp_path, rope_parameters={"rope_theta": 1e6}, num_key_value_heads=2, tie_word_embeddings=True,
                  head_dim=32, rope_scaling=None, model_type="qwen3")
    c = sa.HFLoader.load_llama_config(str(tmp_path))
    got = (c["rope_theta"], c["num_key_value_heads"], c["tie_word_embeddings"], c["head_dim"], c["model_type"])
    assert got == (1e6, 2, 1, 32, "qwen3")
    (tmp_path / "config.json").write_text(json.dumps({"vocab_size": 1}))
    with pytest.raises(sa.ArgumentError, match="No model_type"):
        sa.HFLoader.load_llama_config(str(tmp_path))
    with pytest.raises(sa.ArgumentError, match="config.json not found"):
        sa.HFLoader.load_llama_config(str(tmp_path / "nowhere"))


@pytest.mark.parametrize("key", ["llama32_1b", "llama31_8b"])
def test_llama3_rope_freqs_match_transformers(tmp_path, golden_dir, key):
    d = np.load(os.path.join(golden_dir, "hf_rope_llama3_freqs.npz"))
    meta = json.loads(str(d[key + "_params"]))
    meta["theta"] = meta["rope_theta"]
    hd = meta["head_dim"]
    _write_config(tmp_path, hidden_size=hd * 4, rope_theta=meta["theta"], rope_scaling={
        "rope_type": "llama3", "factor": meta["factor"], "low_freq_factor": meta["low_freq_factor"],
        "high_freq_factor": meta["high_freq_factor"],
        "original_max_position_embeddings": meta["original_max_position_embeddings"]})
    c = sa.HFLoader.load_llama_config(str(tmp_path))
    got = sa.HFLoader.compute_rope_freqs(c)
    np.testing.assert_allclose(got, d[key], rtol=2e-6)
    # and bit for bit what the oracle's restatement of compute_rope_freqs gives
    np.testing.assert_array_equal(got, orc.llama3_rope_freqs(meta["theta"], hd, meta["factor"], meta["low_freq_factor"],
                                                             meta["high_freq_factor"],
                                                             meta["original_max_position_embeddings"]))
