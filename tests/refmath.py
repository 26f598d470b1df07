"""Independent fp64 formulations used to pin the oracle and the HIP path.

Nothing here follows the reference's loops: RoPE is a complex multiplication,
softmax attention is a dense masked matrix expression, RMSNorm is its closed form.
"""
import numpy as np


def inv_freq_closed_form(theta, hd):
    i = np.arange(hd // 2, dtype=np.float64)
    return theta ** (-2.0 * i / hd)


def rope_complex(x, positions, inv_freq):
    """x [..., T, hd] fp64; half-split pairing (i, i+hd/2) as one complex number."""
    x = np.asarray(x, np.float64)
    half = x.shape[-1] // 2
    z = x[..., :half] + 1j * x[..., half:2 * half]
    ang = np.asarray(positions, np.float64)[:, None] * np.asarray(inv_freq, np.float64)[None, :]
    z = z * np.exp(1j * ang)
    out = x.copy()
    out[..., :half] = z.real
    out[..., half:2 * half] = z.imag
    return out


def head_rmsnorm(x, nheads, hd, w, eps):
    x = np.asarray(x, np.float64).reshape(x.shape[0], nheads, hd)
    y = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * np.asarray(w, np.float64)
    return y.reshape(y.shape[0], nheads * hd)


def attention_f64(q, k, v, H, KV, hd, start_pos, inv_freq, k_cache=None, v_cache=None,
                  q_norm=None, k_norm=None, eps=1e-6, bias=(None, None, None)):
    """Dense fp64 causal GQA attention of T new rows on top of an optional cache.

    q [T,H*hd], k,v [T,KV*hd] (projection outputs); k_cache (already rotated) and
    v_cache are [KV, S, hd].  Returns (out [T,H*hd], k_rot [KV,T,hd], v [KV,T,hd])."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    T = q.shape[0]
    if bias[0] is not None:
        q, k, v = q + bias[0], k + bias[1], v + bias[2]
    if q_norm is not None:
        q = head_rmsnorm(q, H, hd, q_norm, eps)
        k = head_rmsnorm(k, KV, hd, k_norm, eps)
    pos = start_pos + np.arange(T)
    qh = rope_complex(q.reshape(T, H, hd).transpose(1, 0, 2), pos, inv_freq)
    kh = rope_complex(k.reshape(T, KV, hd).transpose(1, 0, 2), pos, inv_freq)
    vh = v.reshape(T, KV, hd).transpose(1, 0, 2)
    if k_cache is not None and start_pos > 0:
        K = np.concatenate([np.asarray(k_cache, np.float64)[:, :start_pos], kh], 1)
        V = np.concatenate([np.asarray(v_cache, np.float64)[:, :start_pos], vh], 1)
    else:
        K, V = kh, vh
    g = H // KV
    L = start_pos + T
    mask = np.arange(L)[None, :] <= (start_pos + np.arange(T))[:, None]
    out = np.empty((T, H, hd))
    for h in range(H):
        s = qh[h] @ K[h // g].T / np.sqrt(hd)
        s = np.where(mask, s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        out[:, h] = p @ V[h // g]
    return out.reshape(T, H * hd), kh, vh


def assert_close(got, want, atol=1e-4, rtol=1e-3, what=""):
    """The parity bar: max-abs <= atol or relative <= rtol, elementwise."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    err = np.abs(got - want)
    bad = err > atol + rtol * np.abs(want)
    assert not bad.any(), f"{what}: max abs err {err.max():.3e}, {bad.sum()} of {bad.size} outside tolerance"
    return err.max()
