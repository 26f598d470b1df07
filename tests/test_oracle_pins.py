"""Pins the CPU oracle before it is trusted as the parity checker.

Every check is one that a plausible restatement mistake (dropped term, wrong
sign, wrong pairing, transposed operand, wrong head mapping) fails:
reference-held known answers, fixtures from an independent implementation
(transformers), closed forms, brute force in fp64 with a different formulation,
and invariants of the cache.
"""
import json
import os

import numpy as np
import pytest

import refmath as rm
from oracle import oracle as orc


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- RoPE.apply
def test_rope_identity_at_position_zero():
    # spec/rope_kv_cache_spec.cr:5-10
    m = np.arange(1, 9, dtype=np.float32)[None]
    out = orc.rope_apply(m, 0, 10000.0)
    assert np.abs(out - m).max() < 1e-5


def test_rope_half_split_known_answer():
    # spec/rope_kv_cache_spec.cr:12-26: hd=4, pos 1, x=(1,0,0,0) -> out[0]=cos 1, out[2]=sin 1
    m = np.array([[1.0, 0.0, 0.0, 0.0]], np.float32)
    out = orc.rope_apply(m, 1, 10000.0)
    assert abs(out[0, 0] - np.cos(1.0)) < 1e-4
    assert abs(out[0, 2] - np.sin(1.0)) < 1e-4
    assert out[0, 1] == 0.0 and out[0, 3] == 0.0


def test_rope_apply_matches_complex_rotation_and_odd_dim_passthrough():
    x = rng(0).standard_normal((5, 9)).astype(np.float32)
    out = orc.rope_apply(x, 3, 10000.0)
    want = rm.rope_complex(x[:, :8].astype(np.float64), 3 + np.arange(5), 10000.0 ** (-2.0 * np.arange(4) / 9))
    assert np.abs(out[:, :8] - want).max() < 1e-6
    assert (out[:, 8] == x[:, 8]).all()


# ---------------------------------------------------------------- inv_freq
@pytest.mark.parametrize("theta,hd", [(10000.0, 64), (500000.0, 64), (1e6, 128), (10000.0, 4)])
def test_inv_freq_closed_form(theta, hd):
    b = orc.Block(hd * 2, 2, 2, hd, rope_theta=theta)
    got = b.inv_freq()
    want = rm.inv_freq_closed_form(theta, hd)
    assert got.dtype == np.float32
    assert (got == want.astype(np.float32)).all()  # fp64 formula rounded once
    assert got[0] == 1.0


def test_rope_freqs_override_inv_freq():
    b = orc.Block(16, 2, 2, 8)
    f = np.array([0.5, 0.25, 0.125, 0.0625], np.float32)
    b.set_rope(123.0, f)
    assert (b.inv_freq() == f).all()


def test_llama3_rope_scaling_matches_transformers(golden_dir):
    d = np.load(os.path.join(golden_dir, "hf_rope_llama3_freqs.npz"))
    for name in ("llama32_1b", "llama31_8b"):
        p = json.loads(str(d[name + "_params"]))
        got = orc.llama3_rope_freqs(p["rope_theta"], p["head_dim"], p["factor"], p["low_freq_factor"],
                                    p["high_freq_factor"], p["original_max_position_embeddings"])
        want = d[name]
        np.testing.assert_allclose(got, want, rtol=2e-6)
        # the three regimes are all present: untouched, scaled by 1/factor, smoothed
        base = rm.inv_freq_closed_form(p["rope_theta"], p["head_dim"])
        ratio = got / base
        assert np.isclose(ratio, 1.0, rtol=1e-6).any()
        assert np.isclose(ratio, 1.0 / p["factor"], rtol=1e-6).any()
        assert ((ratio > 1.0 / p["factor"] * 1.01) & (ratio < 0.99)).any()


# ---------------------------------------------------------------- QK-norm
def test_head_rmsnorm_closed_form_and_unit_rms():
    hd, nh = 16, 3
    b = orc.Block(hd * nh, nh, nh, hd, eps=1e-6)
    x = (rng(1).standard_normal((4, nh * hd)) * 3).astype(np.float32)
    w = (1 + 0.1 * rng(2).standard_normal(hd)).astype(np.float32)
    got = b.head_rmsnorm(x, nh, w)
    want = rm.head_rmsnorm(x, nh, hd, w, 1e-6)
    assert np.abs(got - want).max() < 2e-6 * np.abs(want).max()
    ones = b.head_rmsnorm(x, nh, np.ones(hd, np.float32)).reshape(4, nh, hd).astype(np.float64)
    assert np.abs(np.sqrt((ones ** 2).mean(-1)) - 1).max() < 1e-5


def test_head_rmsnorm_weight_size_mismatch_is_argument_error():
    b = orc.Block(32, 2, 2, 16)
    with pytest.raises(orc.ArgumentError):
        b.head_rmsnorm(np.zeros((1, 32), np.float32), 2, np.ones(8, np.float32))


def test_eps_of_constructor_is_the_qk_norm_eps():
    # llama_block.cr:92: a large eps must change the result
    x = np.full((1, 8), 1e-3, np.float32)
    a = orc.Block(8, 1, 1, 8, eps=1e-6).head_rmsnorm(x, 1, np.ones(8, np.float32))
    c = orc.Block(8, 1, 1, 8, eps=1.0).head_rmsnorm(x, 1, np.ones(8, np.float32))
    assert np.abs(a - 1).max() < 0.5 and np.abs(c - 1e-3).max() < 1e-5


# ---------------------------------------------------------------- constructor checks
def test_constructor_argument_errors():
    with pytest.raises(orc.ArgumentError):
        orc.Block(64, 8, 3)  # heads % kv_heads
    with pytest.raises(orc.ArgumentError):
        orc.Block(64, 7, 7)  # d_model % heads with default head_dim
    with pytest.raises(orc.ArgumentError):
        orc.Block(64, 8, 0)
    b = orc.Block(2048, 32, 4, 128)  # Qwen3 style explicit head_dim
    assert b.q_dim == 4096 and b.kv_dim == 512


# ---------------------------------------------------------------- bias
def _rand_block(seed, d=32, H=4, KV=2, hd=None, theta=10000.0, eps=1e-6):
    r = rng(seed)
    b = orc.Block(d, H, KV, hd, eps=eps, rope_theta=theta)
    ws = [r.uniform(-0.1, 0.1, s).astype(np.float32)
          for s in ((d, b.q_dim), (d, b.kv_dim), (d, b.kv_dim), (b.q_dim, d))]
    b.set_weights(*ws)
    return b, ws, r


def test_nil_bias_equals_zero_bias_and_nonzero_bias_moves_output():
    # spec/llama_qkv_bias_spec.cr:8-72
    a, ws, r = _rand_block(3, d=8, H=2, KV=2)
    b, _, _ = _rand_block(3, d=8, H=2, KV=2)
    c, _, _ = _rand_block(3, d=8, H=2, KV=2)
    b.set_bias(np.zeros(8), np.zeros(8), np.zeros(8))
    c.set_bias(0.3 * np.arange(1, 9), 0.2 * np.arange(1, 9), 0.5 * np.arange(1, 9))
    x = ((np.arange(8) - 4) * 0.05).astype(np.float32)[None]
    oa, ob, oc = a.attention_cached(x), b.attention_cached(x), c.attention_cached(x)
    assert np.abs(oa - ob).max() <= 1e-6
    assert np.abs(oc - oa).sum() > 0.01


def test_bias_size_mismatch_is_argument_error():
    b, _, _ = _rand_block(4, d=8, H=2, KV=2)
    b.set_bias(np.zeros(7), np.zeros(8), np.zeros(8))
    with pytest.raises(orc.ArgumentError):
        b.attention_cached(np.zeros((1, 8), np.float32))


# ---------------------------------------------------------------- cache invariants
def test_cache_append_invariants_and_positions():
    H, KV, hd = 4, 2, 8
    b = orc.Block(H * hd, H, KV, hd, rope_theta=500000.0)
    r = rng(5)
    lens, total = [3, 1, 5, 1], 0
    ks, vs = [], []
    for T in lens:
        q = r.standard_normal((T, H * hd)).astype(np.float32)
        k = r.standard_normal((T, KV * hd)).astype(np.float32)
        v = r.standard_normal((T, KV * hd)).astype(np.float32)
        b.attention_cached_qkv(q, k, v)
        total += T
        assert b.cache_len == total
        ks.append(k)
        vs.append(v)
    k_all, v_all = np.concatenate(ks), np.concatenate(vs)
    invf = rm.inv_freq_closed_form(500000.0, hd)
    for c in range(KV):
        kc, vc = b.k_cache(c), b.v_cache(c)
        assert kc.shape == (total, hd)
        # V rows are stored un-rotated, bit for bit, row index == position
        assert (vc == v_all[:, c * hd:(c + 1) * hd]).all()
        # K row p is the row rotated by position p (complex formulation, fp64)
        want = rm.rope_complex(k_all[:, c * hd:(c + 1) * hd], np.arange(total), invf)
        assert np.abs(kc - want).max() < 1e-6
        # position 0 is the identity rotation, exactly
        assert (kc[0] == k_all[0, c * hd:(c + 1) * hd]).all()
        # a rotation keeps each pair's norm
        n0 = np.hypot(k_all[:, c * hd:c * hd + hd // 2], k_all[:, c * hd + hd // 2:(c + 1) * hd])
        n1 = np.hypot(kc[:, :hd // 2], kc[:, hd // 2:])
        assert np.abs(n0 - n1).max() < 1e-6


def test_chunking_invariance_and_clear_rerun_bit_identical():
    H, KV, hd, T = 4, 2, 8, 11
    r = rng(6)
    q = r.standard_normal((T, H * hd)).astype(np.float32)
    k = r.standard_normal((T, KV * hd)).astype(np.float32)
    v = r.standard_normal((T, KV * hd)).astype(np.float32)
    b = orc.Block(H * hd, H, KV, hd)
    whole = b.attention_cached_qkv(q, k, v)
    kc_whole = b.k_cache(1)
    for chunks in ([4, 7], [1] * T, [10, 1]):
        b.clear_cache()
        assert b.cache_len == 0
        outs, o = [], 0
        for n in chunks:
            outs.append(b.attention_cached_qkv(q[o:o + n], k[o:o + n], v[o:o + n]))
            o += n
        assert (np.concatenate(outs) == whole).all()  # the oracle is order-stable: bit-identical
        assert (b.k_cache(1) == kc_whole).all()


def test_threaded_heads_bit_identical_to_single_thread():
    H, KV, hd, T = 8, 2, 16, 9
    r = rng(7)
    q = r.standard_normal((T, H * hd)).astype(np.float32)
    k = r.standard_normal((T, KV * hd)).astype(np.float32)
    v = r.standard_normal((T, KV * hd)).astype(np.float32)
    a, b = orc.Block(H * hd, H, KV, hd), orc.Block(H * hd, H, KV, hd)
    assert (a.attention_cached_qkv(q, k, v, threads=1) == b.attention_cached_qkv(q, k, v, threads=4)).all()


def test_fill_cache_is_equivalent_to_appending():
    H, KV, hd, S = 4, 2, 8, 6
    r = rng(8)
    b = orc.Block(H * hd, H, KV, hd)
    q, k, v = (r.standard_normal((S, n * hd)).astype(np.float32) for n in (H, KV, KV))
    b.attention_cached_qkv(q, k, v)
    kc = np.stack([b.k_cache(c) for c in range(KV)])
    vc = np.stack([b.v_cache(c) for c in range(KV)])
    q1, k1, v1 = (r.standard_normal((1, n * hd)).astype(np.float32) for n in (H, KV, KV))
    want = b.attention_cached_qkv(q1, k1, v1)
    c = orc.Block(H * hd, H, KV, hd)
    c.fill_cache(kc, vc)
    assert c.cache_len == S
    assert (c.attention_cached_qkv(q1, k1, v1) == want).all()


# ---------------------------------------------------------------- attention vs brute force
@pytest.mark.parametrize("H,KV,hd,S,T,theta,norm", [
    (4, 4, 8, 0, 5, 10000.0, False),
    (8, 4, 16, 7, 1, 500000.0, False),   # g=2 decode
    (8, 2, 16, 5, 3, 1e6, True),         # g=4, QK-norm, chunked prefill
    (8, 1, 32, 33, 2, 1e6, True),        # g=8 (MQA-like)
    (32, 8, 64, 40, 1, 500000.0, False), # Llama-3.2-1B head geometry
])
def test_cached_attention_matches_fp64_brute_force(H, KV, hd, S, T, theta, norm):
    r = rng(100 + H + S)
    b = orc.Block(H * hd if not norm else 64, H, KV, hd, eps=1e-6, rope_theta=theta)
    qn = kn = None
    if norm:
        qn = (1 + 0.1 * r.standard_normal(hd)).astype(np.float32)
        kn = (1 + 0.1 * r.standard_normal(hd)).astype(np.float32)
        b.set_qk_norm(qn, kn)
    invf = rm.inv_freq_closed_form(theta, hd)
    kc = vc = None
    if S:
        q0, k0, v0 = (r.standard_normal((S, n * hd)).astype(np.float32) for n in (H, KV, KV))
        b.attention_cached_qkv(q0, k0, v0)
        _, kc, vc = rm.attention_f64(q0, k0, v0, H, KV, hd, 0, invf, q_norm=qn, k_norm=kn)
    q, k, v = (r.standard_normal((T, n * hd)).astype(np.float32) for n in (H, KV, KV))
    got = b.attention_cached_qkv(q, k, v)
    want, _, _ = rm.attention_f64(q, k, v, H, KV, hd, S, invf, kc, vc, q_norm=qn, k_norm=kn)
    assert np.abs(got - want).max() < 2e-5


def test_attention_closed_form_special_cases():
    H, KV, hd = 4, 2, 8
    r = rng(9)
    # L = 1 -> out = V[0] for every head of the group
    b = orc.Block(H * hd, H, KV, hd)
    q, k, v = (r.standard_normal((1, n * hd)).astype(np.float32) for n in (H, KV, KV))
    out = b.attention_cached_qkv(q, k, v).reshape(H, hd)
    for h in range(H):
        assert np.abs(out[h] - v.reshape(KV, hd)[h // 2]).max() < 1e-6
    # identical (rotated) K rows -> uniform weights -> out = mean of visible V rows
    b = orc.Block(H * hd, H, KV, hd)
    S = 9
    vrows = r.standard_normal((KV, S, hd)).astype(np.float32)
    krows = np.broadcast_to(r.standard_normal((KV, 1, hd)).astype(np.float32), (KV, S, hd)).copy()
    b.fill_cache(krows, vrows)
    q1 = r.standard_normal((1, H * hd)).astype(np.float32)
    k1 = np.zeros((1, KV * hd), np.float32)
    # new K row differs, so make its score hugely negative by using a zero query for check of the mean
    out = b.attention_cached_qkv(np.zeros_like(q1), k1, np.zeros((1, KV * hd), np.float32)).reshape(H, hd)
    want = np.concatenate([vrows, np.zeros((KV, 1, hd), np.float32)], 1).mean(1)
    for h in range(H):
        assert np.abs(out[h] - want[h // 2]).max() < 1e-6
    # one dominant score -> out -> that V row
    b = orc.Block(H * hd, H, KV, hd)
    krows = r.standard_normal((KV, S, hd)).astype(np.float32) * 0.01
    krows[:, 4] = 0
    krows[:, 4, 0] = 100.0  # RoPE at pos S leaves the query's own pairing; use query aligned with dim 0
    b.fill_cache(krows, vrows)
    q1 = np.zeros((1, H * hd), np.float32)
    # choose q so that after rotation by pos S it equals 50*e0: rotate e0 by -S
    invf = rm.inv_freq_closed_form(10000.0, hd)
    e0 = np.zeros((1, hd))
    e0[0, 0] = 50.0
    qpre = rm.rope_complex(e0, [-S], invf)[0]
    q1[:] = np.tile(qpre, H)
    out = b.attention_cached_qkv(q1, np.zeros((1, KV * hd), np.float32), vrows[:, 0].reshape(1, -1)).reshape(H, hd)
    for h in range(H):
        assert np.abs(out[h] - vrows[h // 2, 4]).max() < 1e-5


def test_gqa_mapping_equal_queries_in_a_group_give_equal_outputs():
    H, KV, hd, S = 8, 2, 8, 6
    r = rng(10)
    b = orc.Block(H * hd, H, KV, hd)
    b.fill_cache(r.standard_normal((KV, S, hd)), r.standard_normal((KV, S, hd)))
    qh = r.standard_normal((KV, hd)).astype(np.float32)
    q = np.repeat(qh, H // KV, axis=0).reshape(1, -1)  # heads 0-3 share q[0], heads 4-7 share q[1]
    out = b.attention_cached_qkv(q, r.standard_normal((1, KV * hd)), r.standard_normal((1, KV * hd))).reshape(H, hd)
    assert (out[0] == out[1]).all() and (out[0] == out[3]).all() and (out[4] == out[7]).all()
    assert np.abs(out[0] - out[4]).max() > 1e-3


def test_causality_future_rows_never_change_earlier_outputs():
    H, KV, hd, T = 4, 2, 8, 6
    r = rng(11)
    q, k, v = (r.standard_normal((T, n * hd)).astype(np.float32) for n in (H, KV, KV))
    a = orc.Block(H * hd, H, KV, hd).attention_cached_qkv(q, k, v)
    k2, v2 = k.copy(), v.copy()
    k2[4:] += 5.0
    v2[4:] -= 3.0
    c = orc.Block(H * hd, H, KV, hd).attention_cached_qkv(q, k2, v2)
    assert (a[:4] == c[:4]).all() and np.abs(a[4:] - c[4:]).max() > 1e-3


def test_matches_torch_sdpa():
    import torch

    H, KV, hd, T = 8, 2, 16, 10
    r = rng(12)
    q, k, v = (r.standard_normal((T, n * hd)).astype(np.float32) for n in (H, KV, KV))
    b = orc.Block(H * hd, H, KV, hd, rope_theta=1e6)
    got = b.attention_cached_qkv(q, k, v)
    invf = rm.inv_freq_closed_form(1e6, hd)
    qr = torch.tensor(rm.rope_complex(q.reshape(T, H, hd).transpose(1, 0, 2), np.arange(T), invf))
    kr = torch.tensor(rm.rope_complex(k.reshape(T, KV, hd).transpose(1, 0, 2), np.arange(T), invf))
    vr = torch.tensor(v.reshape(T, KV, hd).transpose(1, 0, 2).astype(np.float64))
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    o = torch.nn.functional.scaled_dot_product_attention(
        qr[None], kr.repeat_interleave(H // KV, 0)[None], vr.repeat_interleave(H // KV, 0)[None], attn_mask=mask)
    want = o[0].permute(1, 0, 2).reshape(T, H * hd).numpy()
    assert np.abs(got - want).max() < 2e-5


# ---------------------------------------------------------------- fixtures from transformers
def _block_from_fixture(d):
    m = json.loads(str(d["meta"]))
    b = orc.Block(m["d_model"], m["num_heads"], m["num_kv_heads"], m["head_dim"], eps=m["eps"],
                  rope_theta=m["rope_theta"])
    b.set_weights(d["w_q"], d["w_k"], d["w_v"], d["w_o"])
    if "b_q" in d:
        b.set_bias(d["b_q"], d["b_k"], d["b_v"])
    if "q_norm" in d:
        b.set_qk_norm(d["q_norm"], d["k_norm"])
    rs = m.get("rope_scaling")
    if rs and rs.get("rope_type") == "llama3":
        b.set_rope(m["rope_theta"], orc.llama3_rope_freqs(
            rs["rope_theta"], m["head_dim"], rs["factor"], rs["low_freq_factor"], rs["high_freq_factor"],
            rs["original_max_position_embeddings"]))
    return b, m


@pytest.mark.parametrize("name", ["hf_llama_attn", "hf_llama3_scaled_attn", "hf_qwen2_attn", "hf_qwen3_attn"])
def test_attention_layer_matches_transformers(golden_dir, name):
    d = np.load(os.path.join(golden_dir, name + ".npz"))
    b, m = _block_from_fixture(d)
    np.testing.assert_allclose(b.inv_freq(), d["inv_freq"], rtol=2e-6)
    x, want = d["x"], d["expected"]
    # whole sequence through the cached path at once (prefill)
    got = b.attention_cached(x)
    assert np.abs(got - want).max() < 2e-5 * max(1.0, np.abs(want).max())
    # prefill T-1 then decode 1: last row again
    b.clear_cache()
    b.attention_cached(x[:-1])
    last = b.attention_cached(x[-1:])
    assert np.abs(last[0] - want[-1]).max() < 2e-5 * max(1.0, np.abs(want).max())
    # the no-cache path (attention_full_cpu)
    full = b.attention_full(x)
    assert np.abs(full - want).max() < 2e-5 * max(1.0, np.abs(want).max())


def test_tiny_llama_cached_equals_full_and_matches_transformers(golden_dir):
    # the scenario of spec/rope_kv_cache_spec.cr:29-59 on the reference's own fixture weights
    d = np.load(os.path.join(golden_dir, "tiny_llama_hidden.npz"))
    m = json.loads(str(d["meta"]))
    blocks = [orc.Block(m["d_model"], m["num_heads"], m["num_kv_heads"], None, eps=m["eps"],
                        rope_theta=m["rope_theta"]) for _ in range(2)]
    for li, b in enumerate(blocks):
        b.set_weights(d[f"l{li}_w_q"], d[f"l{li}_w_k"], d[f"l{li}_w_v"], d[f"l{li}_w_o"])

    def run(x, cached):
        for li, b in enumerate(blocks):
            x = b.forward(x, d[f"l{li}_norm1"], d[f"l{li}_norm2"], m["eps"], d[f"l{li}_gate"], d[f"l{li}_up"],
                          d[f"l{li}_down"], cached)
            yield x

    emb = d["embed"]
    full = list(run(emb, False))
    for li in range(2):
        assert np.abs(full[li] - d[f"hidden_after_{li}"]).max() < 1e-5
    list(run(emb[:3], True))
    inc = list(run(emb[3:], True))[-1]
    assert np.abs(inc[0] - full[-1][3]).max() < 1e-3   # the reference's own tolerance
    assert np.abs(inc[0] - d["hidden_after_1"][3]).max() < 1e-5


def test_matmul_rmsnorm_closed_forms():
    r = rng(13)
    a, b = r.standard_normal((5, 33)).astype(np.float32), r.standard_normal((33, 7)).astype(np.float32)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    assert np.abs(orc.matmul(a, b) - want).max() <= 1e-6
    x, g = r.standard_normal((3, 16)).astype(np.float32), r.standard_normal(16).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-5) * g
    assert np.abs(orc.rmsnorm(x, g, 1e-5) - want).max() < 1e-6
