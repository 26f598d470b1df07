"""ctypes binding of libshainet_hip_kernels.so.

`HIP` plays the role SHAInet::CUDA plays in the reference for this path
(src/shainet/cuda.cr:778-891): availability probes and the two kernel entry
points with the reference's names; `AttnContext` / `KVCache` wrap the fused
batched entry points.  There is no CPU fallback: a missing library or a missing
GPU raises.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
# SHAINET_HIP_LIB: load another build of the library (kernel experiments)
_SO = os.environ.get("SHAINET_HIP_LIB") or os.path.join(_HERE, "lib", "libshainet_hip_kernels.so")

MEM_HOST, MEM_DEVICE = 0, 1
MAX_BATCH = 64

_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int)


class HipError(RuntimeError):
    pass


class ArgumentError(ValueError):
    """What the Crystal layer raises as ArgumentError."""


def library_path():
    return _SO


def build_library(force=True):
    """Compile the HIP library for gfx950 (cross-compiles without a GPU)."""
    cmd = ["make", "-C", _CSRC, "-j8"] + (["-B"] if force else [])
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise HipError("building libshainet_hip_kernels.so failed:\n" + proc.stdout[-4000:])
    return _SO


_lib = None

_SIGNATURES = {
    "shainet_hip_last_error": (C.c_char_p, []),
    "shainet_hip_available": (C.c_int, []),
    "kv_cache_append_f32": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "attention_kv_f32": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]),
    "shainet_attn_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int, C.c_double, _f32p, _f32p,
                                      C.c_int, _f32p, C.c_int, C.c_double, C.c_int]),
    "shainet_attn_set_bias": (C.c_int, [C.c_void_p, _f32p, C.c_int, _f32p, C.c_int, _f32p, C.c_int]),
    "shainet_attn_destroy": (C.c_int, [C.c_void_p]),
    "shainet_attn_sync": (C.c_int, [C.c_void_p]),
    "shainet_attn_stream": (C.c_void_p, [C.c_void_p]),
    "shainet_attn_set_stream": (C.c_int, [C.c_void_p, C.c_void_p]),
    "shainet_attn_inv_freq": (C.c_int, [C.c_void_p, _f32p]),
    "shainet_kv_cache_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_void_p, C.c_int, C.c_int]),
    "shainet_kv_cache_destroy": (C.c_int, [C.c_void_p]),
    "shainet_kv_cache_clear": (C.c_int, [C.c_void_p, C.c_int]),
    "shainet_kv_cache_truncate": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "shainet_kv_cache_len": (C.c_int, [C.c_void_p, C.c_int]),
    "shainet_kv_cache_capacity": (C.c_int, [C.c_void_p]),
    "shainet_kv_cache_reserve": (C.c_int, [C.c_void_p, C.c_int]),
    "shainet_kv_cache_k": (C.c_void_p, [C.c_void_p]),
    "shainet_kv_cache_v": (C.c_void_p, [C.c_void_p]),
    "shainet_kv_cache_fill": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]),
    "shainet_kv_cache_read": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p]),
    "shainet_attn_forward": (C.c_int, [C.c_void_p, C.c_void_p, _i32p, _i32p, C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.c_int]),
    "shainet_attn_forward_noalloc": (C.c_int, [C.c_void_p, C.c_void_p, _i32p, _i32p, C.c_int, C.c_void_p, C.c_void_p,
                                               C.c_void_p, C.c_void_p]),
    "shainet_kv_cache_lengths_to_device": (C.c_int, [C.c_void_p]),
    "shainet_kv_cache_lengths_from_device": (C.c_int, [C.c_void_p]),
    "shainet_attn_decode_step": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                           C.c_void_p]),
    "shainet_attn_last_q_rot": (C.c_int, [C.c_void_p, _f32p, C.c_int]),
    "shainet_attn_describe_plan": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, _i32p, _i32p, _i32p]),
    "shainet_rope_apply": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_double, C.c_int]),
    "shainet_llama_attn_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int, C.c_int, C.c_double,
                                            C.c_double]),
    "shainet_llama_attn_destroy": (C.c_int, [C.c_void_p]),
    "shainet_llama_attn_set_rope": (C.c_int, [C.c_void_p, C.c_double, _f32p]),
    "shainet_llama_attn_set_qk_norm": (C.c_int, [C.c_void_p, _f32p, C.c_int, _f32p, C.c_int]),
    "shainet_llama_attn_set_bias": (C.c_int, [C.c_void_p, _f32p, C.c_int, _f32p, C.c_int, _f32p, C.c_int]),
    "shainet_llama_attn_set_weights": (C.c_int, [C.c_void_p, _f32p, _f32p, _f32p, _f32p]),
    "shainet_llama_attn_clear_cache": (C.c_int, [C.c_void_p]),
    "shainet_llama_attn_cache_len": (C.c_int, [C.c_void_p]),
    "shainet_llama_attn_forward_cached": (C.c_int, [C.c_void_p, _f32p, C.c_int, _f32p]),
    "shainet_llama_attn_forward_full": (C.c_int, [C.c_void_p, _f32p, C.c_int, _f32p]),
    "shainet_llama_block_forward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int]),
    "shainet_llama_block_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int, C.c_double,
                                             C.c_double, C.c_int, C.c_int]),
    "shainet_llama_block_destroy": (C.c_int, [C.c_void_p]),
    "shainet_llama_block_attn": (C.c_void_p, [C.c_void_p]),
    "shainet_llama_block_set_norms": (C.c_int, [C.c_void_p, _f32p, _f32p]),
    "shainet_llama_block_set_ffn": (C.c_int, [C.c_void_p, _f32p, _f32p, _f32p]),
    "shainet_llama_block_clear_cache": (C.c_int, [C.c_void_p]),
    "shainet_llama_block_cache_len": (C.c_int, [C.c_void_p]),
    "shainet_llama_block_forward_cached": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int]),
    "shainet_safetensors_open": (C.c_int, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "shainet_safetensors_close": (C.c_int, [C.c_void_p]),
    "shainet_safetensors_count": (C.c_int, [C.c_void_p]),
    "shainet_safetensors_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "shainet_safetensors_has": (C.c_int, [C.c_void_p, C.c_char_p]),
    "shainet_safetensors_info": (C.c_int, [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_longlong),
                                           C.POINTER(C.c_int), C.POINTER(C.c_longlong)]),
    "shainet_safetensors_read_f32": (C.c_int, [C.c_void_p, C.c_char_p, _f32p, C.c_longlong]),
    "shainet_hf_read_llama_config": (C.c_int, [C.c_char_p, C.c_void_p]),
    "shainet_hf_rope_freqs": (C.c_int, [C.c_void_p, _f32p, C.c_int]),
    "shainet_hf_load_llama": (C.c_int, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "shainet_llama_model_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                             C.c_int, C.c_int, C.c_double, C.c_double]),
    "shainet_llama_model_destroy": (C.c_int, [C.c_void_p]),
    "shainet_llama_model_layers": (C.c_int, [C.c_void_p]),
    "shainet_llama_model_block": (C.c_void_p, [C.c_void_p, C.c_int]),
    "shainet_llama_model_set_embedding": (C.c_int, [C.c_void_p, _f32p]),
    "shainet_llama_model_set_final_norm": (C.c_int, [C.c_void_p, _f32p]),
    "shainet_llama_model_set_lm_head": (C.c_int, [C.c_void_p, _f32p, _f32p]),
    "shainet_llama_model_clear_cache": (C.c_int, [C.c_void_p]),
    "shainet_llama_model_cache_len": (C.c_int, [C.c_void_p]),
    "shainet_llama_model_run": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.c_int, _f32p]),
    "shainet_llama_model_run_full": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.c_int, _f32p]),
    "shainet_llama_model_sync": (C.c_int, [C.c_void_p]),
    "shainet_llama_model_set_decode_mode": (C.c_int, [C.c_void_p, C.c_int]),
    "shainet_llama_model_decode_mode_in_use": (C.c_int, [C.c_void_p]),
    "shainet_llama_model_step_trace": (C.c_int, [C.c_void_p, C.POINTER(C.c_longlong), C.c_int, C.POINTER(C.c_int),
                                                 C.POINTER(C.c_int)]),
    "shainet_llama_model_read_logits": (C.c_int, [C.c_void_p, _f32p]),
    "shainet_llama_model_write_logits": (C.c_int, [C.c_void_p, _f32p]),
    "shainet_llama_model_greedy": (C.c_int, [C.c_void_p, C.POINTER(C.c_int)]),
    "shainet_llama_model_generate_greedy": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int,
                                                      C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "shainet_llama_model_repetition_penalty": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_double]),
    "shainet_llama_model_topk": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), _f32p, C.POINTER(C.c_int)]),
    "shainet_llama_model_sample": (C.c_int, [C.c_void_p, C.c_int, C.c_double, C.c_double, C.POINTER(C.c_int)]),
    "shainet_hip_matmul_f32": (C.c_int, [C.c_void_p, C.c_longlong, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                         C.c_int, C.c_void_p]),
    "shainet_hip_stream_copy_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_longlong, C.c_int, C.c_void_p]),
    "shainet_hip_stream_read_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_longlong, C.c_int, C.c_void_p]),
    "shainet_hip_mfma_f32_loop": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_longlong), C.c_void_p]),
    "shainet_hip_launch_latency": (C.c_int, [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float), C.c_void_p]),
    "shainet_attn_profile": (C.c_int, [C.c_void_p, C.c_int]),
    "shainet_attn_profile_read": (C.c_int, [C.c_void_p, C.POINTER(C.c_double), _i32p]),
    "shainet_attn_profile_samples": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, _i32p]),
}


def exported_symbols():
    """Every symbol include/shainet_hip_attn.h declares."""
    return sorted(_SIGNATURES)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise HipError(f"{_SO} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                           "(there is no CPU fallback)")
        # A process may hold only one HIP runtime.  PyTorch ships its own copy under the
        # same soname; when torch is installed it must be loaded first so that this
        # library binds to that copy instead of bringing in a second one.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(_SO)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _check(rc):
    if rc == 0:
        return
    msg = lib().shainet_hip_last_error().decode()
    if rc == 1:
        raise ArgumentError(msg)
    raise HipError(f"status {rc}: {msg}")


def _ptr(x):
    """Device or host address of a torch tensor / numpy array / int."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    return x.ctypes.data


def _f32_arr(a):
    import numpy as np

    if a is None:
        return None, None, -1
    arr = np.ascontiguousarray(a, dtype=np.float32)
    return arr, arr.ctypes.data_as(_f32p), arr.size


class HIP:
    """Counterpart of SHAInet::CUDA for the attention path."""

    @staticmethod
    def kernels_available():
        # cuda.cr:111-122: can the kernel library be opened?
        try:
            lib()
            return True
        except (HipError, OSError):
            return False

    @staticmethod
    def available():
        if os.environ.get("SHAINET_DISABLE_HIP"):  # cuda.cr:64 (SHAINET_DISABLE_CUDA)
            return False
        return HIP.kernels_available() and bool(lib().shainet_hip_available())

    @staticmethod
    def fully_available():
        return HIP.available() and HIP.kernels_available()  # cuda.cr:778-780

    @staticmethod
    def kv_cache_append_f32(staging, kc, vc, new_tokens, start_pos, num_kv_heads, head_dim, capacity):
        lib().kv_cache_append_f32(_ptr(staging), _ptr(kc), _ptr(vc), new_tokens, start_pos, num_kv_heads, head_dim,
                                  capacity)

    @staticmethod
    def attention_kv_f32(q, kc, vc, out, ws, new_tokens, start_pos, num_heads, heads_per_kv, head_dim, capacity,
                         scale):
        lib().attention_kv_f32(_ptr(q), _ptr(kc), _ptr(vc), _ptr(out), _ptr(ws), new_tokens, start_pos, num_heads,
                               heads_per_kv, head_dim, capacity, scale)


class RoPE:
    """SHAInet::RoPE (src/shainet/transformer/rope.cr) on the device."""

    @staticmethod
    def apply(x, start_pos=0, theta=10000.0):
        """RoPE.apply(x, start_pos, theta): x is [seq_len, head_dim]; numpy in -> numpy out
        (synchronous), a CUDA torch tensor in -> torch tensor out (default stream)."""
        import numpy as np

        if hasattr(x, "is_cuda") and x.is_cuda:
            import torch

            if x.dim() != 2 or x.dtype != torch.float32 or not x.is_contiguous():
                raise ArgumentError("x must be a contiguous float32 [seq_len, head_dim] tensor")
            out = torch.empty_like(x)
            _check(lib().shainet_rope_apply(x.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], start_pos, theta,
                                            MEM_DEVICE))
            return out
        x = np.ascontiguousarray(x, np.float32)
        if x.ndim != 2:
            raise ArgumentError("x must be [seq_len, head_dim]")
        out = np.empty_like(x)
        _check(lib().shainet_rope_apply(x.ctypes.data, out.ctypes.data, x.shape[0], x.shape[1], start_pos, theta,
                                        MEM_HOST))
        return out


PLAN_FIELDS = ("path", "head_dim", "key_chunks", "groups", "turns", "workgroups", "units", "wgs_per_cu")
PATH_DECODE, PATH_PREFILL, PATH_GENERIC = 0, 1, 2


def describe_plan(num_heads, num_kv_heads, head_dim, start_pos, new_tokens):
    """What the attention step of a forward call with these sequences launches (a dict over
    PLAN_FIELDS); nothing is launched and no device is needed."""
    n = len(new_tokens)
    sp, nt = (C.c_int * n)(*start_pos), (C.c_int * n)(*new_tokens)
    plan = (C.c_int * 8)()
    _check(lib().shainet_attn_describe_plan(num_heads, num_kv_heads, head_dim, n, sp, nt, plan))
    d = dict(zip(PLAN_FIELDS, (int(v) for v in plan)))
    d["padded"] = d["head_dim"] != head_dim   # the tiles are laid out for a larger head_dim than the data's
    return d


def matmul(x, w, res=None, out=None, stream=None):
    """y = x @ w (+ res) on torch CUDA float32 tensors: x [T, K] (rows may be strided), w [K, N]."""
    import torch

    assert x.is_cuda and w.is_cuda and x.dtype == w.dtype == torch.float32 and w.is_contiguous()
    assert x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[0] and x.stride(1) == 1
    T, K = x.shape
    N = w.shape[1]
    if out is None:
        out = torch.empty((T, N), device=x.device, dtype=torch.float32)
    assert out.is_contiguous() and tuple(out.shape) == (T, N)
    if res is not None:
        assert res.is_contiguous() and tuple(res.shape) == (T, N)
    _check(lib().shainet_hip_matmul_f32(x.data_ptr(), x.stride(0), w.data_ptr(), _ptr(res), out.data_ptr(), T, K, N,
                                        stream))
    return out


def stream_copy(src, dst, workgroups=4096, stream=None):
    """Plain copy kernel over two torch CUDA float tensors of equal size (n % 4 == 0)."""
    _check(lib().shainet_hip_stream_copy_f32(_ptr(src), _ptr(dst), src.numel(), workgroups, stream))


def stream_read(src, sink, workgroups=4096, stream=None):
    """Plain read kernel; sink is a float tensor of at least `workgroups` elements."""
    _check(lib().shainet_hip_stream_read_f32(_ptr(src), _ptr(sink), src.numel(), workgroups, stream))


def mfma_f32_loop(sink, iters, workgroups=256, stream=None):
    """Loop of nothing but fp32 MFMAs; sink holds at least workgroups * 512 floats.  Returns the flops of the launch."""
    flops = C.c_longlong(0)
    _check(lib().shainet_hip_mfma_f32_loop(_ptr(sink), iters, workgroups, C.byref(flops), stream))
    return flops.value


def launch_latency(chain=1, reps=200, workgroups=256, stream=None):
    """Microseconds from the first clock reading of the first of `chain` empty kernels to the last
    reading of the last one (median of `reps` chains)."""
    us = C.c_float(0)
    _check(lib().shainet_hip_launch_latency(chain, reps, workgroups, C.byref(us), stream))
    return us.value


class AttnContext:
    """Attention parameters of one LlamaBlock (llama_block.cr:10-28, 73-108)."""

    def __init__(self, num_heads, num_kv_heads, head_dim, rope_theta=10000.0, rope_freqs=None, q_norm=None,
                 k_norm=None, eps=1e-6, max_positions=1024):
        self._h = C.c_void_p()
        _, fp, _ = self._keep_f = _f32_arr(rope_freqs)
        _, qp, qn = self._keep_q = _f32_arr(q_norm)
        _, kp, kn = self._keep_k = _f32_arr(k_norm)
        _check(lib().shainet_attn_create(C.byref(self._h), num_heads, num_kv_heads, head_dim, rope_theta, fp, qp, qn,
                                         kp, kn, eps, max_positions))
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.q_dim, self.kv_dim = num_heads * head_dim, num_kv_heads * head_dim

    def close(self):
        if getattr(self, "_h", None):
            lib().shainet_attn_destroy(self._h)
            self._h = None

    __del__ = close

    def set_bias(self, b_q, b_k, b_v):
        a = [_f32_arr(b) for b in (b_q, b_k, b_v)]
        _check(lib().shainet_attn_set_bias(self._h, a[0][1], a[0][2], a[1][1], a[1][2], a[2][1], a[2][2]))

    def sync(self):
        _check(lib().shainet_attn_sync(self._h))

    @property
    def stream(self):
        return lib().shainet_attn_stream(self._h)

    def set_stream(self, stream_ptr):
        _check(lib().shainet_attn_set_stream(self._h, stream_ptr))

    def profile(self, enable):
        _check(lib().shainet_attn_profile(self._h, 1 if enable else 0))

    def profile_read(self):
        """(summed attention-kernel milliseconds, launches) since the last read."""
        ms, n = C.c_double(0), C.c_int(0)
        _check(lib().shainet_attn_profile_read(self._h, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def profile_samples(self, capacity=4096):
        """Attention-kernel milliseconds of each launch since the last read (numpy float32)."""
        import numpy as np

        out = np.zeros(capacity, np.float32)
        n = C.c_int(0)
        _check(lib().shainet_attn_profile_samples(self._h, out.ctypes.data, capacity, C.byref(n)))
        return out[:min(n.value, capacity)]

    def inv_freq(self):
        import numpy as np

        out = np.empty(self.head_dim // 2, np.float32)
        _check(lib().shainet_attn_inv_freq(self._h, out.ctypes.data_as(_f32p)))
        return out

    def last_q_rot(self, rows):
        import numpy as np

        out = np.empty((rows, self.q_dim), np.float32)
        _check(lib().shainet_attn_last_q_rot(self._h, out.ctypes.data_as(_f32p), rows))
        return out

    def forward(self, cache, q, k, v, new_tokens, seq_ids=None, out=None):
        """llama_block.cr:256-296 for len(new_tokens) sequences.  numpy inputs run the
        synchronous host-pointer mode and return numpy; torch CUDA tensors run the
        asynchronous device-pointer mode on the context's stream."""
        import numpy as np

        n = len(new_tokens)
        nt = (C.c_int * n)(*new_tokens)
        ids = (C.c_int * n)(*seq_ids) if seq_ids is not None else None
        rows = sum(new_tokens)
        if isinstance(q, np.ndarray):
            q, k, v = (np.ascontiguousarray(a, np.float32) for a in (q, k, v))
            assert q.shape == (rows, self.q_dim) and k.shape == (rows, self.kv_dim) and v.shape == k.shape
            out = np.empty((rows, self.q_dim), np.float32)
            mem = MEM_HOST
        else:
            assert q.is_cuda and q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
            assert tuple(q.shape) == (rows, self.q_dim) and tuple(k.shape) == (rows, self.kv_dim)
            if out is None:
                import torch

                out = torch.empty_like(q)
            mem = MEM_DEVICE
        _check(lib().shainet_attn_forward(self._h, cache._h, ids, nt, n, _ptr(q), _ptr(k), _ptr(v), _ptr(out), mem))
        return out


    def forward_noalloc(self, cache, q, k, v, new_tokens, seq_ids=None, out=None):
        """shainet_attn_forward_noalloc: decode calls on torch CUDA tensors, with every buffer the
        kernels need beyond inputs and outputs taken from the library's static device array."""
        n = len(new_tokens)
        nt = (C.c_int * n)(*new_tokens)
        ids = (C.c_int * n)(*seq_ids) if seq_ids is not None else None
        rows = sum(new_tokens)
        assert q.is_cuda and q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        assert tuple(q.shape) == (rows, self.q_dim) and tuple(k.shape) == (rows, self.kv_dim)
        assert tuple(v.shape) == tuple(k.shape)
        if out is None:
            import torch

            out = torch.empty_like(q)
        _check(lib().shainet_attn_forward_noalloc(self._h, cache._h, ids, nt, n, _ptr(q), _ptr(k), _ptr(v), _ptr(out)))
        return out

    def decode_step(self, cache, q, k, v, out):
        """shainet_attn_decode_step: one new row for each of the first q.shape[0] sequences of
        `cache`, the cached lengths read and advanced on the device (after
        `cache.lengths_to_device()`); launches that depend on nothing but the shapes, so the call
        can be recorded into a graph on the context's stream and replayed."""
        n = q.shape[0]
        assert q.is_cuda and q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and out.is_contiguous()
        assert tuple(q.shape) == (n, self.q_dim) and tuple(k.shape) == (n, self.kv_dim)
        assert tuple(v.shape) == tuple(k.shape) and tuple(out.shape) == tuple(q.shape)
        _check(lib().shainet_attn_decode_step(self._h, cache._h, n, _ptr(q), _ptr(k), _ptr(v), _ptr(out)))
        return out

    def prepared(self, cache, q, k, v, new_tokens, out, seq_ids=None):
        """A zero-argument callable that repeats this device-pointer forward call with nothing but
        the C call in it (tight decode loops, benchmarks): the argument checks of `forward` run
        once, here.  The tensors must stay alive and in place while the callable is used."""
        n = len(new_tokens)
        nt = (C.c_int * n)(*new_tokens)
        ids = (C.c_int * n)(*seq_ids) if seq_ids is not None else None
        rows = sum(new_tokens)
        assert q.is_cuda and q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and out.is_contiguous()
        assert tuple(q.shape) == (rows, self.q_dim) and tuple(k.shape) == (rows, self.kv_dim)
        assert tuple(v.shape) == tuple(k.shape) and tuple(out.shape) == tuple(q.shape)
        fn, h, ch = lib().shainet_attn_forward, self._h, cache._h
        qp, kp, vp, op = (C.c_void_p(t.data_ptr()) for t in (q, k, v, out))

        def call():
            rc = fn(h, ch, ids, nt, n, qp, kp, vp, op, MEM_DEVICE)
            if rc:
                _check(rc)

        return call


class KVCache:
    """Device-resident fp32 KV cache: [batch][num_kv_heads][capacity][head_dim] for K and V."""

    def __init__(self, ctx, batch, capacity):
        self.ctx = ctx
        self._h = C.c_void_p()
        _check(lib().shainet_kv_cache_create(C.byref(self._h), ctx._h, batch, capacity))
        self.batch = batch

    def close(self):
        if getattr(self, "_h", None) and getattr(self.ctx, "_h", None):
            lib().shainet_kv_cache_destroy(self._h)
        self._h = None

    __del__ = close

    def clear(self, seq=-1):
        _check(lib().shainet_kv_cache_clear(self._h, seq))

    def truncate(self, seq, length):
        _check(lib().shainet_kv_cache_truncate(self._h, seq, length))

    def len(self, seq=0):
        return lib().shainet_kv_cache_len(self._h, seq)

    def lengths_to_device(self):
        """Before `AttnContext.decode_step`: the host's lengths go to the device."""
        _check(lib().shainet_kv_cache_lengths_to_device(self._h))

    def lengths_from_device(self):
        """After the last `decode_step` (or replay of one): waits, and takes the device's lengths back."""
        _check(lib().shainet_kv_cache_lengths_from_device(self._h))

    @property
    def capacity(self):
        return lib().shainet_kv_cache_capacity(self._h)

    def reserve(self, capacity):
        _check(lib().shainet_kv_cache_reserve(self._h, capacity))

    @property
    def k_ptr(self):
        return lib().shainet_kv_cache_k(self._h)

    @property
    def v_ptr(self):
        return lib().shainet_kv_cache_v(self._h)

    def fill(self, seq, k_rows, v_rows):
        """k_rows, v_rows: [num_kv_heads, n, head_dim], K already rotated."""
        import numpy as np

        if isinstance(k_rows, np.ndarray):
            k_rows, v_rows = (np.ascontiguousarray(a, np.float32) for a in (k_rows, v_rows))
            mem = MEM_HOST
        else:
            assert k_rows.is_cuda and k_rows.is_contiguous() and v_rows.is_contiguous()
            mem = MEM_DEVICE
        assert tuple(k_rows.shape) == tuple(v_rows.shape) and k_rows.shape[0] == self.ctx.num_kv_heads
        assert k_rows.shape[2] == self.ctx.head_dim
        _check(lib().shainet_kv_cache_fill(self._h, seq, _ptr(k_rows), _ptr(v_rows), k_rows.shape[1], mem))

    def read(self, seq, kv_head, pos0, n):
        import numpy as np

        k = np.empty((n, self.ctx.head_dim), np.float32)
        v = np.empty((n, self.ctx.head_dim), np.float32)
        _check(lib().shainet_kv_cache_read(self._h, seq, kv_head, pos0, n, k.ctypes.data_as(_f32p),
                                           v.ctypes.data_as(_f32p)))
        return k, v


class LlamaBlock:
    """The reference's LlamaBlock (llama_block.cr:6-130, 189-196, 246-299) on the device: same
    constructor arguments and checks, same settable properties, `clear_cache`,
    `attention_cached(x)` = attention_cached_cpu(x) and, when `ff_hidden` is given,
    `forward_cached(x)` with the two RMSNorms, the residual adds and the dense SwiGLU
    feed-forward.  Matrices are numpy float32, weights in the reference's [in, out] layout."""

    def __init__(self, d_model, num_heads, ff_hidden=None, eps=1e-6, rope_theta=10000.0, num_kv_heads=None,
                 head_dim=None, _borrowed=None):
        num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        self._h = C.c_void_p()
        self._block = None
        self._owns = _borrowed is None
        if _borrowed is not None:  # a block owned by a LlamaModel
            self._block = C.c_void_p(_borrowed)
            self._h = C.c_void_p(lib().shainet_llama_block_attn(self._block))
        elif ff_hidden is None:
            _check(lib().shainet_llama_attn_create(C.byref(self._h), d_model, num_heads, num_kv_heads, head_dim or 0,
                                                   eps, rope_theta))
        else:
            self._block = C.c_void_p()
            _check(lib().shainet_llama_block_create(C.byref(self._block), d_model, num_heads, ff_hidden, eps,
                                                    rope_theta, num_kv_heads, head_dim or 0))
            self._h = C.c_void_p(lib().shainet_llama_block_attn(self._block))
        self.d_model, self.num_heads, self.num_kv_heads, self.ff_hidden = d_model, num_heads, num_kv_heads, ff_hidden
        self.head_dim = head_dim or d_model // num_heads
        self.q_dim, self.kv_dim = num_heads * self.head_dim, num_kv_heads * self.head_dim
        self._rope_theta, self._rope_freqs = rope_theta, None

    def close(self):
        if getattr(self, "_h", None) and lib is not None:
            if self._owns:
                if self._block is not None:
                    lib().shainet_llama_block_destroy(self._block)
                else:
                    lib().shainet_llama_attn_destroy(self._h)
            self._h = None
            self._block = None

    __del__ = close

    def set_weights(self, w_q, w_k, w_v, w_o):
        import numpy as np

        ws = [np.ascontiguousarray(w, np.float32) for w in (w_q, w_k, w_v, w_o)]
        shapes = [(self.d_model, self.q_dim), (self.d_model, self.kv_dim), (self.d_model, self.kv_dim),
                  (self.q_dim, self.d_model)]
        for w, sh in zip(ws, shapes):
            if w.shape != sh:
                raise ArgumentError(f"weight shape {w.shape} != {sh}")
        _check(lib().shainet_llama_attn_set_weights(self._h, *[w.ctypes.data_as(_f32p) for w in ws]))

    def set_rope(self, rope_theta, rope_freqs=None):
        _, fp, _ = keep = _f32_arr(rope_freqs)
        self._rope_theta, self._rope_freqs = rope_theta, keep[0]
        _check(lib().shainet_llama_attn_set_rope(self._h, rope_theta, fp))

    def set_qk_norm(self, q_norm, k_norm):
        a, b = _f32_arr(q_norm), _f32_arr(k_norm)
        _check(lib().shainet_llama_attn_set_qk_norm(self._h, a[1], a[2], b[1], b[2]))

    def set_bias(self, b_q, b_k, b_v):
        a = [_f32_arr(b) for b in (b_q, b_k, b_v)]
        _check(lib().shainet_llama_attn_set_bias(self._h, a[0][1], a[0][2], a[1][1], a[1][2], a[2][1], a[2][2]))

    def _need_block(self):
        if self._block is None:
            raise ArgumentError("this LlamaBlock was built without ff_hidden: attention only")

    def set_norms(self, norm1_gamma, norm2_gamma):
        """gamma of @norm1 / @norm2 ([d_model] each; None = ones)."""
        self._need_block()
        a, b = _f32_arr(norm1_gamma), _f32_arr(norm2_gamma)
        for arr in (a, b):
            if arr[0] is not None and arr[2] != self.d_model:
                raise ArgumentError(f"norm gamma must have {self.d_model} entries")
        _check(lib().shainet_llama_block_set_norms(self._block, a[1], b[1]))

    def set_ffn(self, gate_proj, up_proj, down_proj):
        import numpy as np

        self._need_block()
        ws = [np.ascontiguousarray(w, np.float32) for w in (gate_proj, up_proj, down_proj)]
        shapes = [(self.d_model, self.ff_hidden), (self.d_model, self.ff_hidden), (self.ff_hidden, self.d_model)]
        for w, sh in zip(ws, shapes):
            if w.shape != sh:
                raise ArgumentError(f"weight shape {w.shape} != {sh}")
        _check(lib().shainet_llama_block_set_ffn(self._block, *[w.ctypes.data_as(_f32p) for w in ws]))

    def clear_cache(self):
        _check(lib().shainet_llama_attn_clear_cache(self._h))

    @property
    def cache_len(self):
        return lib().shainet_llama_attn_cache_len(self._h)

    def attention_cached(self, x):
        import numpy as np

        x = np.ascontiguousarray(x, np.float32)
        if x.ndim != 2 or x.shape[1] != self.d_model:
            raise ArgumentError(f"x must be [T, {self.d_model}]")
        out = np.empty_like(x)
        _check(lib().shainet_llama_attn_forward_cached(self._h, x.ctypes.data_as(_f32p), x.shape[0],
                                                       out.ctypes.data_as(_f32p)))
        return out

    def attention_full(self, x):
        """attention_full_cpu(x): the no-cache path; the cache is left as it is."""
        import numpy as np

        x = np.ascontiguousarray(x, np.float32)
        if x.ndim != 2 or x.shape[1] != self.d_model:
            raise ArgumentError(f"x must be [T, {self.d_model}]")
        out = np.empty_like(x)
        _check(lib().shainet_llama_attn_forward_full(self._h, x.ctypes.data_as(_f32p), x.shape[0],
                                                     out.ctypes.data_as(_f32p)))
        return out

    def forward(self, x):
        """LlamaBlock#forward: the whole sequence without the cache."""
        return self.forward_cached(x, _fn="shainet_llama_block_forward")

    def forward_cached(self, x, out=None, _fn="shainet_llama_block_forward_cached"):
        """LlamaBlock#forward_cached.  numpy in -> numpy out (copies, synchronous); a CUDA torch
        tensor in -> torch tensor out (device pointers, asynchronous on the block's stream)."""
        import numpy as np

        self._need_block()
        call = getattr(lib(), _fn)
        if hasattr(x, "is_cuda") and x.is_cuda:
            import torch

            if x.dim() != 2 or x.shape[1] != self.d_model or x.dtype != torch.float32 or not x.is_contiguous():
                raise ArgumentError(f"x must be a contiguous float32 [T, {self.d_model}] tensor")
            out = torch.empty_like(x) if out is None else out
            _check(call(self._block, x.data_ptr(), x.shape[0], out.data_ptr(), MEM_DEVICE))
            return out
        x = np.ascontiguousarray(x, np.float32)
        if x.ndim != 2 or x.shape[1] != self.d_model:
            raise ArgumentError(f"x must be [T, {self.d_model}]")
        out = np.empty_like(x)
        _check(call(self._block, x.ctypes.data, x.shape[0], out.ctypes.data, MEM_HOST))
        return out


class LlamaModel:
    """Network#run with use_kv_cache for a LLaMA-family network (network_run.cr:185-226) on the
    device: embedding -> blocks -> final norm -> lm_head (+ bias), logits kept on the device for
    `Sampler`."""

    def __init__(self, vocab, d_model, n_layers, num_heads, ff_hidden, eps=1e-6, rope_theta=10000.0,
                 num_kv_heads=None, head_dim=None, _loaded=None):
        num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        self._h = C.c_void_p()
        if _loaded is not None:  # a handle HFLoader.load_llama built
            self._h = _loaded
        else:
            _check(lib().shainet_llama_model_create(C.byref(self._h), vocab, d_model, n_layers, num_heads,
                                                    num_kv_heads, head_dim or 0, ff_hidden, eps, rope_theta))
        self.vocab, self.d_model, self.n_layers = vocab, d_model, n_layers
        self.blocks = [LlamaBlock(d_model, num_heads, ff_hidden, eps, rope_theta, num_kv_heads, head_dim,
                                  _borrowed=lib().shainet_llama_model_block(self._h, i)) for i in range(n_layers)]

    def close(self):
        if getattr(self, "_h", None) and lib is not None:
            for b in self.blocks:
                b.close()
            lib().shainet_llama_model_destroy(self._h)
            self._h = None

    __del__ = close

    def set_embedding(self, table):
        import numpy as np

        t = np.ascontiguousarray(table, np.float32)
        if t.shape != (self.vocab, self.d_model):
            raise ArgumentError(f"embedding shape {t.shape} != {(self.vocab, self.d_model)}")
        _check(lib().shainet_llama_model_set_embedding(self._h, t.ctypes.data_as(_f32p)))

    def set_final_norm(self, gamma):
        a = _f32_arr(gamma)
        if a[0] is not None and a[2] != self.d_model:
            raise ArgumentError(f"norm gamma must have {self.d_model} entries")
        _check(lib().shainet_llama_model_set_final_norm(self._h, a[1]))

    def set_lm_head(self, weights, bias=None):
        import numpy as np

        w = np.ascontiguousarray(weights, np.float32)
        if w.shape != (self.d_model, self.vocab):
            raise ArgumentError(f"lm_head shape {w.shape} != {(self.d_model, self.vocab)}")
        b = _f32_arr(bias)
        if b[0] is not None and b[2] != self.vocab:
            raise ArgumentError(f"lm_head bias must have {self.vocab} entries")
        _check(lib().shainet_llama_model_set_lm_head(self._h, w.ctypes.data_as(_f32p), b[1]))

    def clear_cache(self):
        _check(lib().shainet_llama_model_clear_cache(self._h))

    @property
    def cache_len(self):
        return lib().shainet_llama_model_cache_len(self._h)

    def run(self, tokens, want_logits=True):
        """Appends `tokens` to the caches; returns the logits row [vocab] of the last token
        (numpy), or None with want_logits=False (they stay on the device for the Sampler)."""
        import numpy as np

        ids = np.ascontiguousarray(tokens, np.int32).reshape(-1)
        logits = np.empty(self.vocab, np.float32) if want_logits else None
        _check(lib().shainet_llama_model_run(self._h, ids.ctypes.data_as(C.POINTER(C.c_int)), ids.size,
                                             logits.ctypes.data_as(_f32p) if want_logits else None))
        return logits

    def run_full(self, tokens, want_logits=True):
        """Network#run with use_kv_cache off: the rows attend among themselves from position 0,
        the caches are not touched; returns the last row's logits like `run`."""
        import numpy as np

        ids = np.ascontiguousarray(tokens, np.int32).reshape(-1)
        logits = np.empty(self.vocab, np.float32) if want_logits else None
        _check(lib().shainet_llama_model_run_full(self._h, ids.ctypes.data_as(C.POINTER(C.c_int)), ids.size,
                                                  logits.ctypes.data_as(_f32p) if want_logits else None))
        return logits

    def sync(self):
        _check(lib().shainet_llama_model_sync(self._h))

    DECODE_AUTO, DECODE_PER_PRODUCT, DECODE_PERSISTENT = 0, 1, 2

    def set_decode_mode(self, mode):
        """How a run of one token walks the blocks: one launch per product (DECODE_AUTO, the
        default), or the whole stack in a single launch (DECODE_PERSISTENT)."""
        _check(lib().shainet_llama_model_set_decode_mode(self._h, mode))

    @property
    def decode_mode_in_use(self):
        return lib().shainet_llama_model_decode_mode_in_use(self._h)

    def step_trace(self):
        """Clock readings (100 MHz) of the last single-launch step, [workgroups, 1 + 24 * layers];
        needs SHAINET_HIP_STEP_TRACE in the environment before the model's first step."""
        import numpy as np

        wgs, per = C.c_int(), C.c_int()
        lib().shainet_llama_model_step_trace(self._h, None, 0, C.byref(wgs), C.byref(per))
        out = np.zeros((max(wgs.value, 1), max(per.value, 1)), np.int64)
        _check(lib().shainet_llama_model_step_trace(self._h, out.ctypes.data_as(C.POINTER(C.c_longlong)), out.size,
                                                    C.byref(wgs), C.byref(per)))
        return out

    def generate_greedy(self, max_tokens, stop_ids=()):
        """The greedy generation loop on the device, from the logits of the last `run`: returns
        the generated ids (without the stop id that ended it, if any)."""
        import numpy as np

        out = np.empty(max(max_tokens, 1), np.int32)
        stop = np.ascontiguousarray(list(stop_ids), np.int32)
        n = C.c_int()
        _check(lib().shainet_llama_model_generate_greedy(
            self._h, max_tokens, stop.ctypes.data_as(C.POINTER(C.c_int)) if stop.size else None, stop.size,
            out.ctypes.data_as(C.POINTER(C.c_int)), C.byref(n)))
        return [int(t) for t in out[:n.value]]

    def logits(self):
        import numpy as np

        out = np.empty(self.vocab, np.float32)
        _check(lib().shainet_llama_model_read_logits(self._h, out.ctypes.data_as(_f32p)))
        return out

    def set_logits(self, row):
        """Replace the device logits row (e.g. to sample from a row computed elsewhere)."""
        import numpy as np

        r = np.ascontiguousarray(row, np.float32).reshape(-1)
        if r.size != self.vocab:
            raise ArgumentError(f"logits row must have {self.vocab} entries")
        _check(lib().shainet_llama_model_write_logits(self._h, r.ctypes.data_as(_f32p)))


class Sampler:
    """text/sampler.cr over the device logits of a LlamaModel's last run: greedy, repetition
    penalty and the top-k selection run on the device; the temperature softmax over the k
    survivors and the inverse-CDF draw (sampler.cr:118-150) run here in fp64 with `rng`
    (anything with a `random()` method returning a float in [0, 1))."""

    def __init__(self, temperature=1.0, top_k=40, repetition_penalty=1.0, rng=None):
        import random

        if top_k < 1:
            raise ArgumentError("top_k must be >= 1")
        if not temperature > 0.0:
            raise ArgumentError("temperature must be > 0")
        self.temperature, self.top_k, self.repetition_penalty = temperature, top_k, repetition_penalty
        self.rng = rng if rng is not None else random.Random()

    @staticmethod
    def greedy(model):
        tok = C.c_int()
        _check(lib().shainet_llama_model_greedy(model._h, C.byref(tok)))
        return tok.value

    def apply_repetition_penalty(self, model, recent_ids, window=None):
        import numpy as np

        ids = np.ascontiguousarray(recent_ids, np.int32).reshape(-1)
        if window is not None:
            ids = np.ascontiguousarray(ids[max(0, ids.size - window):])
        _check(lib().shainet_llama_model_repetition_penalty(model._h, ids.ctypes.data_as(C.POINTER(C.c_int)),
                                                            ids.size, self.repetition_penalty))

    def top_candidates(self, model):
        import numpy as np

        k = self.top_k
        ids = np.empty(k, np.int32)
        vals = np.empty(k, np.float32)
        n = C.c_int()
        _check(lib().shainet_llama_model_topk(model._h, k, ids.ctypes.data_as(C.POINTER(C.c_int)),
                                              vals.ctypes.data_as(_f32p), C.byref(n)))
        return ids[:n.value], vals[:n.value]

    def sample_on_device(self, model, r=None):
        """Sampler#sample with every step on the device; r: the uniform draw (default: one from `rng`)."""
        tok = C.c_int()
        r = self.rng.random() if r is None else r
        _check(lib().shainet_llama_model_sample(model._h, self.top_k, self.temperature, r, C.byref(tok)))
        return tok.value

    def sample(self, model):
        import math

        ids, vals = self.top_candidates(model)
        if len(ids) == 0:
            return 0  # all-NaN row (sampler.cr:114)
        v = [float(x) / self.temperature for x in vals]
        e = [math.exp(x - v[0]) for x in v]  # descending order: element 0 is the max
        inv = 1.0 / sum(e)
        r = self.rng.random()
        cumulative = 0.0
        best = int(ids[-1])
        for i, ex in enumerate(e):
            cumulative += ex * inv
            if r <= cumulative:
                best = int(ids[i])
                break
        return best


class SafeTensors:
    """SHAInet::SafeTensors::File / ShardedFile (safetensors.cr): a .safetensors file, or a model
    directory with model.safetensors or model.safetensors.index.json.  Host only."""

    def __init__(self, path):
        self._h = C.c_void_p()
        _check(lib().shainet_safetensors_open(os.fsencode(path), C.byref(self._h)))

    def close(self):
        if getattr(self, "_h", None) and lib is not None:
            lib().shainet_safetensors_close(self._h)
            self._h = None

    __del__ = close

    def tensor_names(self):
        L = lib()
        return [L.shainet_safetensors_name(self._h, i).decode() for i in range(L.shainet_safetensors_count(self._h))]

    def has_tensor(self, name):
        return bool(lib().shainet_safetensors_has(self._h, name.encode()))

    def info(self, name):
        dt = C.create_string_buffer(8)
        shape = (C.c_longlong * 8)()
        nd, nb = C.c_int(), C.c_longlong()
        _check(lib().shainet_safetensors_info(self._h, name.encode(), dt, shape, C.byref(nd), C.byref(nb)))
        return dt.value.decode(), [int(shape[i]) for i in range(nd.value)], int(nb.value)

    def read_f32(self, name):
        import numpy as np

        dtype, shape, nbytes = self.info(name)
        size = {"F16": 2, "BF16": 2, "F32": 4, "F64": 8}.get(dtype, 1)
        out = np.empty(nbytes // size, np.float32)
        _check(lib().shainet_safetensors_read_f32(self._h, name.encode(), out.ctypes.data_as(_f32p), out.size))
        return out

    def read_matrix(self, name):
        """read_matrix (safetensors.cr:161-187): 1-D tensors come back as one row."""
        _, shape, _ = self.info(name)
        if len(shape) > 2:
            raise ArgumentError(f"Cannot read tensor '{name}' with {len(shape)}D shape as matrix")
        rows = 1 if len(shape) < 2 else shape[0]
        return self.read_f32(name).reshape(rows, -1)


class _HFLlamaConfig(C.Structure):
    _fields_ = [("model_type", C.c_char * 32), ("vocab_size", C.c_int), ("hidden_size", C.c_int),
                ("num_attention_heads", C.c_int), ("num_hidden_layers", C.c_int), ("intermediate_size", C.c_int),
                ("num_key_value_heads", C.c_int), ("head_dim", C.c_int), ("tie_word_embeddings", C.c_int),
                ("num_experts", C.c_int), ("rms_norm_eps", C.c_double), ("rope_theta", C.c_double),
                ("rope_llama3", C.c_int), ("rope_factor", C.c_double), ("rope_low_freq_factor", C.c_double),
                ("rope_high_freq_factor", C.c_double), ("rope_original_max_position_embeddings", C.c_int)]


class HFLoader:
    """HFLoader (hf_loader.cr) for LLaMA-family models: config.json, llama3 RoPE frequencies and
    load_llama onto the device."""

    @staticmethod
    def load_llama_config(model_dir):
        cfg = _HFLlamaConfig()
        _check(lib().shainet_hf_read_llama_config(os.fsencode(model_dir), C.byref(cfg)))
        d = {name: getattr(cfg, name) for name, _ in _HFLlamaConfig._fields_}
        d["model_type"] = d["model_type"].decode()
        d["_struct"] = cfg
        return d

    @staticmethod
    def compute_rope_freqs(config):
        """Array of head_dim/2 inverse frequencies, or None when the config has no llama3 scaling."""
        import numpy as np

        cfg = config["_struct"]
        hd = cfg.head_dim or cfg.hidden_size // max(cfg.num_attention_heads, 1)
        out = np.empty(max(hd // 2, 1), np.float32)
        n = lib().shainet_hf_rope_freqs(C.byref(cfg), out.ctypes.data_as(_f32p), hd // 2)
        if n < 0:
            _check(-n)
        return out[:n] if n > 0 else None

    @staticmethod
    def load_llama(model_dir):
        cfg = HFLoader.load_llama_config(model_dir)
        h = C.c_void_p()
        _check(lib().shainet_hf_load_llama(os.fsencode(model_dir), C.byref(h)))
        return LlamaModel(cfg["vocab_size"], cfg["hidden_size"], cfg["num_hidden_layers"], cfg["num_attention_heads"],
                          cfg["intermediate_size"], cfg["rms_norm_eps"], cfg["rope_theta"],
                          cfg["num_key_value_heads"], cfg["head_dim"] or None, _loaded=h)
