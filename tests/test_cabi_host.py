"""CPU-side checks of the product library: it loads, exports every symbol the header
declares, and its host-side argument checks fire without a GPU (no compute calls here)."""
import ctypes as C
import os
import re

import pytest

import shainet_amd
from shainet_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "shainet_hip_attn.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(shainet_amd.library_path()):
        shainet_amd.build_library(force=False)
    return hip.lib()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(\w+)\s*\([^;{]*\)\s*;", text)))


def test_header_and_binding_agree(lib):
    names = declared_functions()
    assert "kv_cache_append_f32" in names and "attention_kv_f32" in names and "shainet_attn_forward" in names
    assert sorted(names) == hip.exported_symbols(), set(names) ^ set(hip.exported_symbols())


def test_every_declared_symbol_is_exported(lib):
    raw = C.CDLL(shainet_amd.library_path())
    for name in declared_functions():
        assert getattr(raw, name) is not None, name


def test_reference_entry_points_keep_the_reference_signature():
    # src/shainet/native/cuda_kernels.cu:713-715 and 808-811
    text = re.sub(r"\s+", " ", open(HEADER).read())
    assert ("void kv_cache_append_f32(const float *staging, float *kc, float *vc, int new_tokens, int start_pos, "
            "int num_kv_heads, int head_dim, int capacity);") in text
    assert ("void attention_kv_f32(const float *q, const float *kc, const float *vc, float *out, float *ws, "
            "int new_tokens, int start_pos, int num_heads, int heads_per_kv, int head_dim, int capacity, "
            "float scale);") in text


def test_argument_errors_without_a_gpu(lib):
    h = C.c_void_p()
    # num_heads % num_kv_heads (llama_block.cr:80)
    assert lib.shainet_attn_create(C.byref(h), 8, 3, 64, 1e4, None, None, -1, None, -1, 1e-6, 16) == 1
    assert b"divisible" in lib.shainet_hip_last_error()
    # head_dim must be positive (llama_block.cr:84)
    assert lib.shainet_attn_create(C.byref(h), 8, 8, 0, 1e4, None, None, -1, None, -1, 1e-6, 16) == 1
    # qk-norm weight size (llama_block.cr:618)
    w = (C.c_float * 4)(1, 1, 1, 1)
    assert lib.shainet_attn_create(C.byref(h), 2, 2, 8, 1e4, None, w, 4, w, 4, 1e-6, 16) == 1
    assert b"qk_norm weight size" in lib.shainet_hip_last_error()
    assert not h.value
    # null handles are rejected, destroy of null is a no-op
    assert lib.shainet_attn_sync(None) == 1
    assert lib.shainet_attn_destroy(None) == 0
    assert lib.shainet_kv_cache_destroy(None) == 0
    assert lib.shainet_kv_cache_len(None, 0) == -1


def test_no_cpu_fallback(lib, monkeypatch):
    """Without a gfx950 device the context cannot be created and says why."""
    if lib.shainet_hip_available():
        pytest.skip("a GPU is present")
    assert not shainet_amd.HIP.fully_available()
    with pytest.raises(shainet_amd.HipError, match="no gfx950 device"):
        shainet_amd.AttnContext(8, 8, 64)
    monkeypatch.setenv("SHAINET_DISABLE_HIP", "1")
    assert not shainet_amd.HIP.available()


def test_product_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "shainet_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h", "Makefile")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
