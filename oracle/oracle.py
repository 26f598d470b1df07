"""ctypes front end of the CPU checker (oracle/shainet_attn_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  The product package never imports it.
"""
import ctypes as C
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libshainet_attn_oracle.so")

_f32p = C.POINTER(C.c_float)


def build(force=False):
    src = os.path.join(_HERE, "shainet_attn_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.orc_last_error.restype = C.c_char_p
        L.orc_block_new.restype = C.c_void_p
        L.orc_block_new.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_double, C.c_double]
        L.orc_block_free.argtypes = [C.c_void_p]
        L.orc_block_set_rope.argtypes = [C.c_void_p, C.c_double, _f32p]
        L.orc_block_set_qk_norm.argtypes = [C.c_void_p, _f32p, C.c_int, _f32p, C.c_int]
        L.orc_block_set_bias.argtypes = [C.c_void_p, _f32p, C.c_int, _f32p, C.c_int, _f32p, C.c_int]
        L.orc_block_set_weights.argtypes = [C.c_void_p, _f32p, _f32p, _f32p, _f32p]
        L.orc_block_clear_cache.argtypes = [C.c_void_p]
        L.orc_block_cache_len.argtypes = [C.c_void_p]
        L.orc_block_cache_len.restype = C.c_int
        L.orc_block_k_cache.argtypes = [C.c_void_p, C.c_int]
        L.orc_block_k_cache.restype = _f32p
        L.orc_block_v_cache.argtypes = [C.c_void_p, C.c_int]
        L.orc_block_v_cache.restype = _f32p
        L.orc_block_fill_cache.argtypes = [C.c_void_p, _f32p, _f32p, C.c_int]
        L.orc_inv_freq.argtypes = [C.c_void_p, _f32p]
        L.orc_rotate_q.argtypes = [C.c_void_p, _f32p, _f32p, C.c_int, C.c_int]
        L.orc_rotate_q.restype = None
        L.orc_scale.argtypes = [C.c_void_p]
        L.orc_scale.restype = C.c_float
        L.orc_head_rmsnorm.argtypes = [C.c_void_p, _f32p, C.c_int, C.c_int, _f32p, C.c_int]
        L.orc_head_rmsnorm.restype = C.c_int
        L.orc_block_prepare_append.argtypes = [C.c_void_p, _f32p, _f32p, _f32p, C.c_int, C.POINTER(C.c_int)]
        L.orc_block_prepare_append.restype = C.c_int
        L.orc_attention_heads_cpu.argtypes = [C.c_void_p, _f32p, _f32p, C.c_int, C.c_int, C.c_int,
                                              C.c_float, C.c_int, C.c_int]
        L.orc_attention_heads_cpu.restype = None
        L.orc_block_attention_cached_qkv.argtypes = [C.c_void_p, _f32p, _f32p, _f32p, C.c_int, _f32p]
        L.orc_block_attention_cached_qkv.restype = C.c_int
        L.orc_block_attention_cached.argtypes = [C.c_void_p, _f32p, C.c_int, _f32p]
        L.orc_block_attention_cached.restype = C.c_int
        L.orc_block_attention_full_qkv.argtypes = [C.c_void_p, _f32p, _f32p, _f32p, C.c_int, _f32p]
        L.orc_block_attention_full_qkv.restype = C.c_int
        L.orc_block_attention_full.argtypes = [C.c_void_p, _f32p, C.c_int, _f32p]
        L.orc_block_attention_full.restype = C.c_int
        L.orc_block_forward.argtypes = [C.c_void_p, _f32p, C.c_int, _f32p, _f32p, C.c_double, _f32p, _f32p,
                                        _f32p, C.c_int, C.c_int, _f32p]
        L.orc_block_forward.restype = C.c_int
        L.orc_matmul.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
        L.orc_rmsnorm.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_double]
        L.orc_swiglu.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
        L.orc_rope_apply.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_double]
        L.orc_llama3_rope_freqs.argtypes = [C.c_double, C.c_int, C.c_double, C.c_double, C.c_double,
                                            C.c_double, _f32p]
        _i32p = C.POINTER(C.c_int)
        L.orc_embed.argtypes = [_f32p, C.c_int, _i32p, C.c_int, C.c_int, _f32p]
        L.orc_embed.restype = C.c_int
        L.orc_logits_last.argtypes = [_f32p, C.c_int, C.c_int, _f32p, C.c_double, _f32p, C.c_int, _f32p, _f32p]
        L.orc_logits_last.restype = None
        L.orc_greedy.argtypes = [_f32p, C.c_int]
        L.orc_greedy.restype = C.c_int
        L.orc_repetition_penalty.argtypes = [_f32p, C.c_int, _i32p, C.c_int, C.c_int, C.c_double]
        L.orc_repetition_penalty.restype = None
        L.orc_topk.argtypes = [_f32p, C.c_int, C.c_int, C.c_double, _i32p, C.POINTER(C.c_double)]
        L.orc_topk.restype = C.c_int
        L.orc_sample.argtypes = [_f32p, C.c_int, C.c_int, C.c_double, C.c_double]
        L.orc_sample.restype = C.c_int
        _lib = L
    return _lib


class ArgumentError(ValueError):
    """What the reference raises as ArgumentError."""


def _p(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _check(rc):
    if rc == 1:
        raise ArgumentError(lib().orc_last_error().decode())
    if rc:
        raise RuntimeError(lib().orc_last_error().decode())


class Block:
    """The attention-relevant state of a reference LlamaBlock (llama_block.cr:7-108)."""

    def __init__(self, d_model, num_heads, num_kv_heads=None, head_dim=None, eps=1e-6, rope_theta=10000.0):
        num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        self._h = lib().orc_block_new(d_model, num_heads, num_kv_heads, head_dim or 0, eps, rope_theta)
        if not self._h:
            raise ArgumentError(lib().orc_last_error().decode())
        self.d_model, self.num_heads, self.num_kv_heads = d_model, num_heads, num_kv_heads
        self.head_dim = head_dim or d_model // num_heads
        self.q_dim, self.kv_dim = num_heads * self.head_dim, num_kv_heads * self.head_dim
        self._keep = {}

    def __del__(self):
        if getattr(self, "_h", None):
            lib().orc_block_free(self._h)
            self._h = None

    def set_rope(self, theta, freqs=None):
        f = _f32(freqs)
        lib().orc_block_set_rope(self._h, theta, _p(f))

    def set_qk_norm(self, q_norm, k_norm):
        q, k = _f32(q_norm), _f32(k_norm)
        lib().orc_block_set_qk_norm(self._h, _p(q), -1 if q is None else q.size, _p(k), -1 if k is None else k.size)

    def set_bias(self, b_q, b_k, b_v):
        a = [_f32(b_q), _f32(b_k), _f32(b_v)]
        args = []
        for x in a:
            args += [_p(x), -1 if x is None else x.size]
        lib().orc_block_set_bias(self._h, *args)

    def set_weights(self, w_q, w_k, w_v, w_o):
        ws = [_f32(w) for w in (w_q, w_k, w_v, w_o)]
        assert ws[0].shape == (self.d_model, self.q_dim) and ws[3].shape == (self.q_dim, self.d_model)
        assert ws[1].shape == (self.d_model, self.kv_dim) and ws[2].shape == (self.d_model, self.kv_dim)
        lib().orc_block_set_weights(self._h, *[_p(w) for w in ws])

    def clear_cache(self):
        lib().orc_block_clear_cache(self._h)

    @property
    def cache_len(self):
        return lib().orc_block_cache_len(self._h)

    def k_cache(self, kv_h):
        n = self.cache_len * self.head_dim
        return np.ctypeslib.as_array(lib().orc_block_k_cache(self._h, kv_h), (n,)).reshape(-1, self.head_dim).copy()

    def v_cache(self, kv_h):
        n = self.cache_len * self.head_dim
        return np.ctypeslib.as_array(lib().orc_block_v_cache(self._h, kv_h), (n,)).reshape(-1, self.head_dim).copy()

    def fill_cache(self, k_rows, v_rows):
        """k_rows, v_rows: [num_kv_heads, n, head_dim]; K already rotated."""
        k, v = _f32(k_rows), _f32(v_rows)
        assert k.shape == v.shape and k.shape[0] == self.num_kv_heads and k.shape[2] == self.head_dim
        lib().orc_block_fill_cache(self._h, _p(k), _p(v), k.shape[1])

    def inv_freq(self):
        out = np.empty(self.head_dim // 2, np.float32)
        lib().orc_inv_freq(self._h, _p(out))
        return out

    def scale(self):
        return lib().orc_scale(self._h)

    def attention_cached_qkv(self, q, k, v, threads=1, keep_q_rot=False):
        """llama_block.cr:256-296 on projected rows; returns output [T, q_dim].

        threads > 1 runs disjoint query-head ranges concurrently; every head's
        arithmetic is unchanged.  keep_q_rot stores the rotated query rows
        (llama_block.cr:332-344) in self.last_q_rot."""
        q, k, v = (np.array(a, dtype=np.float32, order="C") for a in (q, k, v))
        T = q.shape[0]
        assert q.shape == (T, self.q_dim) and k.shape == (T, self.kv_dim) and v.shape == (T, self.kv_dim)
        out = np.empty((T, self.q_dim), np.float32)
        if threads <= 1 and not keep_q_rot:
            _check(lib().orc_block_attention_cached_qkv(self._h, _p(q), _p(k), _p(v), T, _p(out)))
            return out
        start = C.c_int(0)
        _check(lib().orc_block_prepare_append(self._h, _p(q), _p(k), _p(v), T, C.byref(start)))
        if keep_q_rot:
            self.last_q_rot = np.empty_like(q)
            lib().orc_rotate_q(self._h, _p(q), _p(self.last_q_rot), T, start.value)
        total, scale, H = self.cache_len, self.scale(), self.num_heads
        threads = max(1, threads)
        threads = min(threads, H)
        bounds = [H * i // threads for i in range(threads + 1)]

        def run(i):
            lib().orc_attention_heads_cpu(self._h, _p(q), _p(out), T, start.value, total, scale,
                                          bounds[i], bounds[i + 1])

        with ThreadPoolExecutor(threads) as ex:
            list(ex.map(run, range(threads)))
        return out

    def attention_cached(self, x):
        x = _f32(x)
        out = np.empty((x.shape[0], self.d_model), np.float32)
        _check(lib().orc_block_attention_cached(self._h, _p(x), x.shape[0], _p(out)))
        return out

    def attention_full_qkv(self, q, k, v):
        q, k, v = (np.array(a, dtype=np.float32, order="C") for a in (q, k, v))
        out = np.empty((q.shape[0], self.q_dim), np.float32)
        _check(lib().orc_block_attention_full_qkv(self._h, _p(q), _p(k), _p(v), q.shape[0], _p(out)))
        return out

    def attention_full(self, x):
        x = _f32(x)
        out = np.empty((x.shape[0], self.d_model), np.float32)
        _check(lib().orc_block_attention_full(self._h, _p(x), x.shape[0], _p(out)))
        return out

    def head_rmsnorm(self, m, nheads, w):
        m = np.array(m, dtype=np.float32, order="C")
        w = _f32(w)
        _check(lib().orc_head_rmsnorm(self._h, _p(m), m.shape[0], nheads, _p(w), w.size))
        return m

    def forward(self, x, norm1, norm2, norm_eps, gate_w, up_w, down_w, cached):
        x = _f32(x)
        a = [_f32(t) for t in (norm1, norm2, gate_w, up_w, down_w)]
        out = np.empty_like(x)
        _check(lib().orc_block_forward(self._h, _p(x), x.shape[0], _p(a[0]), _p(a[1]), norm_eps, _p(a[2]),
                                       _p(a[3]), _p(a[4]), a[2].shape[1], 1 if cached else 0, _p(out)))
        return out


def matmul(a, b):
    a, b = _f32(a), _f32(b)
    c = np.empty((a.shape[0], b.shape[1]), np.float32)
    lib().orc_matmul(_p(a), _p(b), _p(c), a.shape[0], a.shape[1], b.shape[1])
    return c


def rmsnorm(x, gamma, eps):
    x, g = _f32(x), _f32(gamma)
    out = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(g), _p(out), x.shape[0], x.shape[1], eps)
    return out


def rope_apply(x, start_pos=0, theta=10000.0):
    x = _f32(x)
    out = np.zeros_like(x)
    lib().orc_rope_apply(_p(x), _p(out), x.shape[0], x.shape[1], start_pos, theta)
    return out


def llama3_rope_freqs(theta, head_dim, factor, low_freq_factor, high_freq_factor, old_ctx):
    out = np.empty(head_dim // 2, np.float32)
    lib().orc_llama3_rope_freqs(theta, head_dim, factor, low_freq_factor, high_freq_factor, old_ctx, _p(out))
    return out


def _i32(a):
    return np.ascontiguousarray(a, np.int32).reshape(-1)


def embed(table, ids):
    """EmbeddingLayer#embed_cpu."""
    table, ids = _f32(table), _i32(ids)
    out = np.empty((ids.size, table.shape[1]), np.float32)
    _check(lib().orc_embed(_p(table), table.shape[0], ids.ctypes.data_as(C.POINTER(C.c_int)), ids.size,
                           table.shape[1], _p(out)))
    return out


def logits_last(h, final_gamma, eps, lm_head, bias=None):
    """Final norm (None = the network has none), last row x lm_head [d, vocab], + bias."""
    h, w = _f32(h), _f32(lm_head)
    g = _f32(final_gamma) if final_gamma is not None else None
    b = _f32(bias) if bias is not None else None
    out = np.empty(w.shape[1], np.float32)
    lib().orc_logits_last(_p(h), h.shape[0], h.shape[1], _p(g) if g is not None else None, eps, _p(w), w.shape[1],
                          _p(b) if b is not None else None, _p(out))
    return out


def greedy(logits):
    """Sampler.greedy over one logits row."""
    x = _f32(logits).reshape(-1)
    return lib().orc_greedy(_p(x), x.size)


def repetition_penalty(logits, recent_ids, penalty, window=None):
    """Sampler#apply_repetition_penalty!; returns the penalised copy."""
    x = _f32(logits).reshape(-1).copy()
    ids = _i32(recent_ids)
    lib().orc_repetition_penalty(_p(x), x.size, ids.ctypes.data_as(C.POINTER(C.c_int)), ids.size,
                                 -1 if window is None else window, penalty)
    return x


def topk(logits, k, temperature=1.0):
    """The selection loop of Sampler#sample: (ids, value / temperature), descending."""
    x = _f32(logits).reshape(-1)
    ids = np.empty(k, np.int32)
    vals = np.empty(k, np.float64)
    n = lib().orc_topk(_p(x), x.size, k, temperature, ids.ctypes.data_as(C.POINTER(C.c_int)),
                       vals.ctypes.data_as(C.POINTER(C.c_double)))
    return ids[:n], vals[:n]


def sample(logits, k, temperature, r):
    """Sampler#sample with the uniform draw `r` handed in."""
    x = _f32(logits).reshape(-1)
    return lib().orc_sample(_p(x), x.size, k, temperature, r)
