"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X.

Bar (fp32): |gpu - oracle| <= 1e-4 + 1e-3*|oracle| elementwise; rotated Q rows and
cache contents (RoPE positions, cache indexing) bit-identical.
"""
import os

import numpy as np
import pytest

import prefill_cases as pc
import refmath as rm
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-4, 1e-3


@pytest.fixture(scope="module")
def hip():
    import shainet_amd as sa

    assert sa.HIP.fully_available(), "no gfx950 device or libshainet_hip_kernels.so missing"
    return sa


def make_pair(hip, H, KV, hd, theta=10000.0, norm=False, bias=False, freqs=None, batch=1, capacity=512, seed=0,
              eps=1e-6):
    r = np.random.default_rng(seed)
    qn = kn = None
    if norm:
        qn = (1 + 0.02 * r.standard_normal(hd)).astype(np.float32)
        kn = (1 + 0.02 * r.standard_normal(hd)).astype(np.float32)
    ctx = hip.AttnContext(H, KV, hd, rope_theta=theta, rope_freqs=freqs, q_norm=qn, k_norm=kn, eps=eps)
    cache = hip.KVCache(ctx, batch, capacity)
    blocks = []
    for _ in range(batch):
        b = orc.Block(H * hd, H, KV, hd, eps=eps, rope_theta=theta)
        if freqs is not None:
            b.set_rope(theta, freqs)
        if norm:
            b.set_qk_norm(qn, kn)
        blocks.append(b)
    if bias:
        bq, bk, bv = (0.3 * r.standard_normal(n * hd).astype(np.float32) for n in (H, KV, KV))
        ctx.set_bias(bq, bk, bv)
        for b in blocks:
            b.set_bias(bq, bk, bv)
    return ctx, cache, blocks, r


def rows(r, T, H, KV, hd):
    return tuple(r.standard_normal((T, n * hd)).astype(np.float32) for n in (H, KV, KV))


def check_step(ctx, cache, blocks, r, new_tokens, seq_ids=None, threads=8, what=""):
    """One forward call on both sides; returns the max abs error."""
    H, KV, hd = ctx.num_heads, ctx.num_kv_heads, ctx.head_dim
    ids = list(range(len(new_tokens))) if seq_ids is None else seq_ids
    parts = [rows(r, T, H, KV, hd) for T in new_tokens]
    q, k, v = (np.concatenate([p[i] for p in parts]) for i in range(3))
    got = ctx.forward(cache, q, k, v, new_tokens, seq_ids)
    want = np.concatenate([blocks[s].attention_cached_qkv(*p, threads=threads) for s, p in zip(ids, parts)])
    err = rm.assert_close(got, want, ATOL, RTOL, what)
    for s in ids:
        assert cache.len(s) == blocks[s].cache_len
    return err


def check_cache_bits(cache, blocks, seqs=None):
    for s in (range(len(blocks)) if seqs is None else seqs):
        n = blocks[s].cache_len
        for c in range(blocks[s].num_kv_heads):
            k, v = cache.read(s, c, 0, n)
            assert np.array_equal(k.view(np.uint32), blocks[s].k_cache(c).view(np.uint32)), "K cache bits differ"
            assert np.array_equal(v.view(np.uint32), blocks[s].v_cache(c).view(np.uint32)), "V cache bits differ"


# ------------------------------------------------------------------ the reference's own scenarios
def test_reference_gqa_prefill_then_decode(hip):
    # spec/llama_attention_gpu_spec.cr:16-66: d=64, 8 heads, 4 kv heads (g=2), prefill 6 + 3 decodes
    ctx, cache, blocks, r = make_pair(hip, 8, 4, 8, seed=42)
    for T in (6, 1, 1, 1):
        check_step(ctx, cache, blocks, r, [T])
    check_cache_bits(cache, blocks)


def test_reference_growth_and_clear(hip):
    # spec/llama_attention_gpu_spec.cr:68-104: d=32, 4 heads, 2 kv heads, 290 + 10 rows across the
    # initial capacity 256; a rerun after clear must give the same results (no stale rows leak)
    ctx, cache, blocks, r0 = make_pair(hip, 4, 2, 8, seed=7, capacity=256)
    H, KV, hd = 4, 2, 8
    steps = [rows(r0, T, H, KV, hd) for T in [200, 56] + [1] * 4]
    grow_at = 2
    outs = []
    for run in range(2):
        cache.clear()
        blocks[0].clear_cache()
        res = []
        for i, p in enumerate(steps + [rows(np.random.default_rng(99), 34, H, KV, hd)]):
            if cache.len(0) + p[0].shape[0] > cache.capacity:
                with pytest.raises(hip.HipError):
                    ctx.forward(cache, *p, [p[0].shape[0]])
                assert i >= grow_at
                cache.reserve(2 * cache.capacity)
            got = ctx.forward(cache, *p, [p[0].shape[0]])
            want = blocks[0].attention_cached_qkv(*p)
            rm.assert_close(got, want, ATOL, RTOL, f"run {run} step {i}")
            res.append(got)
        outs.append(res)
        assert cache.len(0) == 294 and cache.capacity == 512
        check_cache_bits(cache, blocks)
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


def test_bias_nil_equals_zero_and_size_check(hip):
    # spec/llama_qkv_bias_spec.cr:8-72
    H, KV, hd = 2, 2, 4
    a = hip.AttnContext(H, KV, hd)
    b = hip.AttnContext(H, KV, hd)
    b.set_bias(np.zeros(8), np.zeros(8), np.zeros(8))
    c = hip.AttnContext(H, KV, hd)
    c.set_bias(0.3 * np.arange(1, 9), 0.2 * np.arange(1, 9), 0.5 * np.arange(1, 9))
    q, k, v = rows(np.random.default_rng(1), 1, H, KV, hd)
    outs = [x.forward(hip.KVCache(x, 1, 8), q, k, v, [1]) for x in (a, b, c)]
    assert np.array_equal(outs[0], outs[1])
    assert np.abs(outs[2] - outs[0]).sum() > 0.01
    with pytest.raises(hip.ArgumentError):
        a.set_bias(np.zeros(7), np.zeros(8), np.zeros(8))
    with pytest.raises(hip.ArgumentError):
        hip.AttnContext(8, 3, 4)
    with pytest.raises(hip.ArgumentError):
        hip.AttnContext(2, 2, 4, q_norm=np.ones(3), k_norm=np.ones(4))


# ------------------------------------------------------------------ exactness of RoPE positions and cache indexing
@pytest.mark.parametrize("H,KV,hd,theta,norm,bias", [
    (32, 8, 64, 500000.0, False, False),
    (32, 8, 128, 1e6, True, False),
    (8, 2, 16, 1e6, True, True),
    (4, 4, 7, 10000.0, False, True),  # odd head_dim: the last slot of rotated rows is 0
])
def test_rotated_q_and_cache_are_bit_identical(hip, H, KV, hd, theta, norm, bias):
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, theta, norm, bias, capacity=64, seed=3)
    b = blocks[0]
    for T in (5, 1, 9):
        q, k, v = rows(r, T, H, KV, hd)
        ctx.forward(cache, q, k, v, [T])
        b.attention_cached_qkv(q, k, v, keep_q_rot=True)
        got_q = ctx.last_q_rot(T)
        assert np.array_equal(got_q.view(np.uint32), b.last_q_rot.view(np.uint32)), "rotated Q bits differ"
    check_cache_bits(cache, blocks)
    # the rotation really depends on the position: same row, two positions, different K
    k0, _ = cache.read(0, 0, 0, 15)
    assert k0.shape == (15, hd) and not np.array_equal(k0[1], k0[2])


@pytest.mark.parametrize("H,KV,hd,norm,bias", [
    (32, 8, 64, False, True), (8, 2, 128, False, False), (8, 4, 8, False, True), (4, 1, 256, False, True),
    (32, 8, 128, True, False), (8, 2, 64, True, True), (8, 4, 16, True, True), (6, 3, 30, True, False),
])
def test_many_rows_take_the_bulk_prep_kernels_same_bits(hip, H, KV, hd, norm, bias):
    # from 8192 head rows on: without QK-norm a kernel with 16-byte accesses, with QK-norm one that
    # walks each row's sum of squares in LDS.  Ragged batch, bias, start positions above zero;
    # rotated Q and both caches bit for bit
    per_token = H + 2 * KV
    T0 = 8192 // per_token + 3
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 500000.0, norm, bias, batch=3, capacity=T0 + 64, seed=hd)
    for new in ([T0 // 2 + 3, 5, T0 // 2 + 1], [1, T0, 7]):
        parts = [rows(r, T, H, KV, hd) for T in new]
        q, k, v = (np.concatenate([p[i] for p in parts]) for i in range(3))
        ctx.forward(cache, q, k, v, new)
        want_q = []
        for s, pt in enumerate(parts):
            blocks[s].attention_cached_qkv(*pt, keep_q_rot=True, threads=16)
            want_q.append(blocks[s].last_q_rot)
        got_q = ctx.last_q_rot(sum(new))
        assert np.array_equal(got_q.view(np.uint32), np.concatenate(want_q).view(np.uint32)), "rotated Q bits differ"
    check_cache_bits(cache, blocks)


# ------------------------------------------------------------------ decode (split-K kernel)
def test_config1_llama1b_decode_on_prefilled_cache(hip):
    # Llama-3.2-1B head geometry, cache pre-filled to 512 positions, one new row
    H, KV, hd, S = 32, 8, 64, 512
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 500000.0, capacity=1024, seed=11)
    kf, vf = (r.standard_normal((KV, S, hd)).astype(np.float32) for _ in range(2))
    cache.fill(0, kf, vf)
    blocks[0].fill_cache(kf, vf)
    for _ in range(3):
        check_step(ctx, cache, blocks, r, [1])
    check_cache_bits(cache, blocks)


@pytest.mark.parametrize("S", [1024, 4096, 16384])
def test_config2_decode_steps_appending(hip, S):
    H, KV, hd = 32, 8, 64
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 500000.0, capacity=S + 256, seed=S)
    kf, vf = (r.standard_normal((KV, S, hd)).astype(np.float32) for _ in range(2))
    cache.fill(0, kf, vf)
    blocks[0].fill_cache(kf, vf)
    steps = 128  # BASELINE.json configs[1]: 128 consecutive decode steps at each context length
    worst = max(check_step(ctx, cache, blocks, r, [1], what=f"S={S} step {i}") for i in range(steps))
    assert cache.len(0) == S + steps
    assert worst < 1e-4


def test_decode_every_length_around_tile_and_chunk_edges(hip):
    H, KV, hd = 8, 2, 128
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=True, capacity=300, seed=5)
    for i in range(270):  # lengths 1..270 cross 16-key tiles, 64-key wave strides and chunk edges
        check_step(ctx, cache, blocks, r, [1], threads=1, what=f"len {i + 1}")


@pytest.mark.parametrize("g,hd", [(1, 64), (2, 128), (8, 128), (16, 64),
                                  # head dimensions between the tile layouts (64, 128, 256 wide): padded tiles
                                  (4, 96), (2, 256), (8, 32), (1, 8), (3, 80), (4, 200), (2, 132)])
def test_decode_group_sizes(hip, g, hd):
    KV = 2
    ctx, cache, blocks, r = make_pair(hip, KV * g, KV, hd, 1e6, capacity=1500, seed=g)
    kf, vf = (r.standard_normal((KV, 1100, hd)).astype(np.float32) for _ in range(2))
    cache.fill(0, kf, vf)
    blocks[0].fill_cache(kf, vf)
    for _ in range(2):
        check_step(ctx, cache, blocks, r, [1])


@pytest.mark.parametrize("H,KV,hd,norm", [(32, 1, 64, False), (64, 2, 128, True), (48, 2, 64, False)])
def test_more_than_16_query_heads_per_kv_head(hip, H, KV, hd, norm):
    """llama_block.cr:80 allows any divisor.  32 (or 24) query heads per kv head do not fit the 16
    columns of the split-K decode kernel: such calls take the MFMA kernel (virtual rows = new rows x
    heads of the group, key chunks + combine on a long cached prefix), also for one new row."""
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=norm, capacity=1400, seed=H + hd)
    kf, vf = (r.standard_normal((KV, 1100, hd)).astype(np.float32) for _ in range(2))
    cache.fill(0, kf, vf)
    blocks[0].fill_cache(kf, vf)
    assert hip.describe_plan(H, KV, hd, [1100], [1])["path"] == hip.hip.PATH_PREFILL
    for T in (1, 1, 40, 1, 3):
        check_step(ctx, cache, blocks, r, [T], what=f"{H // KV} heads per kv head, {T} new rows")
    check_cache_bits(cache, blocks)
    # from an empty cache too
    cache.clear()
    blocks[0].clear_cache()
    for T in (1, 17, 1):
        check_step(ctx, cache, blocks, r, [T])


@pytest.mark.parametrize("seed", range(10))
def test_decode_random_ragged_batches(hip, seed):
    """Spans, segments and merges of the decode split over many shapes: a few to 64 sequences of
    unrelated lengths (1 to 900 cached rows, so pairs of one tile next to pairs of fifty), every
    group size, both head dims; twice per shape, the second call on the grown caches, and a
    third on a shuffled subset."""
    r0 = np.random.default_rng(1000 + seed)
    hd = int(r0.choice([64, 128]))
    KV = int(r0.choice([1, 2, 4, 8]))
    g = int(r0.choice([1, 2, 4, 8]))
    B = int(r0.choice([1, 2, 5, 16, 33, 64]))
    top = int(r0.choice([20, 200, 900]))
    lens = [int(x) for x in r0.integers(1, top + 1, B)]
    ctx, cache, blocks, r = make_pair(hip, KV * g, KV, hd, 1e6, norm=bool(seed & 1), batch=B, capacity=top + 8,
                                      seed=seed)
    for s_, L in enumerate(lens):
        kf, vf = (r.standard_normal((KV, L, hd)).astype(np.float32) for _ in range(2))
        cache.fill(s_, kf, vf)
        blocks[s_].fill_cache(kf, vf)
    what = f"hd {hd} KV {KV} g {g} B {B} lens up to {top}"
    for i in range(2):
        assert check_step(ctx, cache, blocks, r, [1] * B, what=f"{what}, call {i}") < 1e-4
    some = [int(x) for x in r0.permutation(B)[: max(1, B // 2)]]
    check_step(ctx, cache, blocks, r, [1] * len(some), seq_ids=some, what=f"{what}, subset")


@pytest.mark.parametrize("KV,g,hd,B,rows_new,top", [
    (8, 4, 128, 16, [4] * 16, 900),                 # rows x group = 16 columns, all in use
    (8, 4, 128, 16, [1, 2, 3, 4] * 4, 900),         # every row count side by side
    (2, 8, 64, 5, [2, 1, 2, 2, 1], 700),
    (4, 1, 64, 3, [16, 9, 1], 400),                 # one head per group: up to 16 rows
    (2, 16, 128, 2, [1, 1], 300),
    (8, 4, 64, 4, [4, 4, 4, 4], 0),                 # from empty caches: later rows see more keys than earlier ones have
    (8, 2, 128, 1, [7], 5000),
    (8, 4, 128, 16, [8, 5, 7, 1] * 4, 900),         # more rows than one tile has columns: two entries each
    (2, 8, 64, 3, [4, 3, 1], 600),
    (4, 1, 64, 2, [32, 17], 300),
    (4, 4, 96, 6, [1, 4, 2, 8, 3, 1], 700),         # a head dimension the tiles are padded for (Phi-3-mini's)
    (2, 2, 256, 3, [5, 1, 16], 500),                # Gemma's
    (4, 2, 24, 2, [3, 1], 100),
])
def test_few_new_rows_take_the_decode_split(hip, KV, g, hd, B, rows_new, top):
    """A few new rows per sequence (rows x heads of a group <= 16) go through the split-K decode
    kernel as further columns of its tiles: each row sees the keys up to its own position."""
    r0 = np.random.default_rng(hd + B + top)
    ctx, cache, blocks, r = make_pair(hip, KV * g, KV, hd, 1e6, norm=True, batch=B, capacity=top + 64, seed=top)
    for s_ in range(B):
        L = int(r0.integers(1, top + 1)) if top else 0
        if L:
            kf, vf = (r.standard_normal((KV, L, hd)).astype(np.float32) for _ in range(2))
            cache.fill(s_, kf, vf)
            blocks[s_].fill_cache(kf, vf)
    for i in range(3):
        assert check_step(ctx, cache, blocks, r, rows_new, what=f"call {i}") < 1e-4
    check_cache_bits(cache, blocks)


def test_partials_that_never_arrive_are_reported(hip, monkeypatch):
    """Failure handling of the decode split, forced from the host: with the test switch the
    workgroups mark their partials complete in a place nobody looks at and the merging
    workgroups stop polling after 2000 looks, so every kernel still ends by itself; the call
    that waits for the stream must report it.  A context made without the switch is unaffected,
    and the give-up is reported by the context whose kernel gave up, not by whichever context
    waits first."""
    import torch

    import shainet_amd as sa

    H, KV, hd = 8, 2, 64
    monkeypatch.setenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS", "1")
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, capacity=3000, seed=3)
    monkeypatch.delenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS")
    kf, vf = (r.standard_normal((KV, 2500, hd)).astype(np.float32) for _ in range(2))
    cache.fill(0, kf, vf)  # 157 tiles per pair: every pair is spread over many workgroups
    q, k, v = rows(r, 1, H, KV, hd)
    with pytest.raises(sa.hip.HipError, match="gave up waiting"):
        ctx.forward(cache, q, k, v, [1])
    ctx2, cache2, blocks2, r2 = make_pair(hip, H, KV, hd, 1e6, capacity=3000, seed=3)
    cache2.fill(0, kf, vf)
    blocks2[0].fill_cache(kf, vf)
    check_step(ctx2, cache2, blocks2, r2, [1])
    # asynchronous calls on both contexts; the healthy one waits first and must come back clean
    dev = [torch.from_numpy(a).cuda() for a in rows(r, 1, H, KV, hd)]
    torch.cuda.synchronize()
    ctx.forward(cache, *dev, [1])
    good = ctx2.forward(cache2, *dev, [1])
    ctx2.sync()
    assert torch.isfinite(good).all()
    with pytest.raises(sa.hip.HipError, match="gave up waiting"):
        ctx.sync()
    ctx.sync()  # reported once


def test_config3_qwen3_8b_batch16_varlen_decode(hip):
    import torch

    H, KV, hd, B = 32, 8, 128, 16
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=True, batch=B, capacity=8192 + 8, seed=33)
    lens = r.integers(2048, 8193, B)
    gen = torch.Generator(device="cuda").manual_seed(33)
    for s in range(B):
        kf = torch.randn((KV, int(lens[s]), hd), generator=gen, device="cuda")
        vf = torch.randn((KV, int(lens[s]), hd), generator=gen, device="cuda")
        torch.cuda.synchronize()
        cache.fill(s, kf, vf)
        blocks[s].fill_cache(kf.cpu().numpy(), vf.cpu().numpy())
    for i in range(2):
        err = check_step(ctx, cache, blocks, r, [1] * B, what=f"step {i}")
        assert err < 1e-4
    # a subset of the sequences, in another order
    check_step(ctx, cache, blocks, r, [1] * 3, seq_ids=[7, 2, 11])


def test_config5b_long_context_batch4_decode(hip):
    import torch

    H, KV, hd, B, S = 32, 4, 128, 4, 32768
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=True, batch=B, capacity=S + 8, seed=55)
    gen = torch.Generator(device="cuda").manual_seed(55)
    for s in range(B):
        kf = torch.randn((KV, S, hd), generator=gen, device="cuda")
        vf = torch.randn((KV, S, hd), generator=gen, device="cuda")
        torch.cuda.synchronize()
        cache.fill(s, kf, vf)
        blocks[s].fill_cache(kf.cpu().numpy(), vf.cpu().numpy())
    assert check_step(ctx, cache, blocks, r, [1] * B) < 1e-4


# ------------------------------------------------------------------ prefill (MFMA kernel)
@pytest.mark.parametrize("H,KV,hd,S,T,norm", [
    (8, 2, 64, 0, 1, False),      # T*g < one tile
    (8, 2, 64, 0, 33, False),
    (8, 2, 128, 17, 70, True),    # chunked prefill on a cached prefix, partial last block
    (6, 2, 64, 5, 45, False),     # g = 3: virtual rows straddle rows unevenly
    (4, 4, 128, 0, 130, True),    # g = 1
    (16, 1, 64, 40, 9, False),    # g = 16
    # head dimensions below the tile layouts' 64 and 128: padded tiles
    (8, 2, 96, 17, 70, True),
    (6, 2, 32, 5, 45, False),
    (4, 4, 80, 0, 130, True),
    (8, 4, 8, 3, 40, False),
    (4, 1, 100, 0, 200, False),   # several row blocks per kv head
])
def test_prefill_small_shapes(hip, H, KV, hd, S, T, norm):
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=norm, capacity=256, seed=T)
    if S:
        check_step(ctx, cache, blocks, r, [S])
    check_step(ctx, cache, blocks, r, [T])
    check_step(ctx, cache, blocks, r, [2])
    check_cache_bits(cache, blocks)


@pytest.mark.parametrize("ns", [2, 3, 5])
def test_prefill_key_splits(hip, ns, monkeypatch):
    # key range of every row block cut into ns chunks merged by a second kernel; with S = 0 the later
    # chunks start past the last visible key of the early rows (their partial stays at -inf)
    monkeypatch.setenv("SHAINET_HIP_PREFILL_SPLITS", str(ns))
    for H, KV, hd, S, T, norm in [(8, 2, 64, 0, 70, False), (8, 1, 128, 100, 37, True), (6, 2, 64, 300, 130, False),
                                  (8, 2, 96, 200, 40, True), (4, 2, 24, 0, 150, False)]:
        ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=norm, capacity=512, seed=ns + T)
        if S:
            check_step(ctx, cache, blocks, r, [S])
        check_step(ctx, cache, blocks, r, [T], what=f"ns={ns} hd={hd} S={S} T={T}")
        check_step(ctx, cache, blocks, r, [3])


def test_prefill_then_decode_equals_one_prefill(hip):
    # chunking invariance: T rows at once == in chunks == row by row (to fp32 round-off)
    H, KV, hd, T = 8, 2, 64, 97
    q, k, v = rows(np.random.default_rng(8), T, H, KV, hd)
    outs = []
    for chunks in ([T], [40, 57], [96, 1], [1] * T):
        ctx = hip.AttnContext(H, KV, hd, rope_theta=500000.0)
        cache = hip.KVCache(ctx, 1, 128)
        o, res = 0, []
        for n in chunks:
            res.append(ctx.forward(cache, q[o:o + n], k[o:o + n], v[o:o + n], [n]))
            o += n
        outs.append(np.concatenate(res))
    for o in outs[1:]:
        assert np.abs(o - outs[0]).max() < 2e-5


@pytest.mark.parametrize("name,H,KV,hd,norm,S,T,inst", pc.CASES, ids=[c[0] for c in pc.CASES])
def test_prefill_full_size_every_instantiation(hip, name, H, KV, hd, norm, S, T, inst, monkeypatch):
    """Every instantiation of the MFMA prefill kernels that the planner can pick, each on a shape
    for which the planner picks it by itself (no tuning variable set), all rows against the
    oracle.  The table holds BASELINE.json configs[3] (2048 and 8192 rows into an empty cache)
    and configs[4](a) (512 rows on 16384 cached positions, Qwen3-30B-A3B geometry) at full size."""
    for var in ("SHAINET_HIP_PREFILL_SPLITS", "SHAINET_HIP_PREFILL_GROUPS", "SHAINET_HIP_PREFILL_WGS_PER_CU",
                "SHAINET_HIP_PREFILL_NO_TURNS"):
        monkeypatch.delenv(var, raising=False)
    plan = hip.describe_plan(H, KV, hd, [S], [T])
    assert plan["path"] == hip.hip.PATH_PREFILL and pc.instantiation(plan) == inst, plan
    theta = 1e6 if hd == 128 else 500000.0
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, theta, norm=norm, capacity=S + T + 8, seed=S + T + hd)
    if S:
        kf, vf = (r.standard_normal((KV, S, hd), dtype=np.float32) for _ in range(2))
        cache.fill(0, kf, vf)
        blocks[0].fill_cache(kf, vf)
    assert check_step(ctx, cache, blocks, r, [T], threads=16, what=name) < 1e-4
    check_step(ctx, cache, blocks, r, [1], threads=16, what=name + ", then one row")
    cache.close()
    ctx.close()


def test_batched_prefill_mixed_lengths(hip):
    H, KV, hd = 8, 2, 64
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, batch=4, capacity=400, seed=9)
    check_step(ctx, cache, blocks, r, [100, 1, 37, 260])
    check_step(ctx, cache, blocks, r, [1, 1, 1, 1])          # decode kernel, unequal lengths
    check_step(ctx, cache, blocks, r, [5, 64], seq_ids=[2, 0])
    check_cache_bits(cache, blocks)


def test_maximum_batch_ragged_and_call_errors(hip):
    # 64 sequences (the limit per call): fresh, short and longer ones in one call, a prefill call with
    # mixed row counts (1 row included), then a decode call; then what a call must refuse
    H, KV, hd, B = 8, 2, 64, 64
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=True, bias=True, batch=B, capacity=96, seed=64)
    first = [int(x) for x in r.integers(1, 40, B)]
    first[0], first[1], first[63] = 1, 39, 1
    check_step(ctx, cache, blocks, r, first, threads=16, what="64 sequences, 1..39 rows each")
    check_step(ctx, cache, blocks, r, [1] * B, threads=16, what="64 sequences, decode")
    some = [5, 17, 40, 63, 0]
    check_step(ctx, cache, blocks, r, [1, 3, 1, 2, 1], seq_ids=some, what="five of them, out of order")
    check_cache_bits(cache, blocks)
    q, k, v = rows(r, 2, H, KV, hd)
    for bad_ids, bad_new in (([3, 3], [1, 1]), ([64, 0], [1, 1]), ([-1, 0], [1, 1]), ([0, 1], [1, 0])):
        before = [cache.len(s) for s in range(B)]
        n = sum(bad_new)
        with pytest.raises(hip.ArgumentError):
            ctx.forward(cache, q[:n], k[:n], v[:n], bad_new, bad_ids)
        assert [cache.len(s) for s in range(B)] == before, "a refused call changed a length"
    with pytest.raises(hip.HipError):  # capacity: nothing appended
        qq, kk, vv = rows(r, 96, H, KV, hd)
        ctx.forward(cache, qq, kk, vv, [96], [7])
    assert cache.len(7) == blocks[7].cache_len


def test_cache_slot_beyond_four_gib(hip):
    # the last slot of a large cache starts 4.3 GB into each tensor: offsets must not be 32-bit
    H, KV, hd, cap = 32, 8, 128, 131072
    r = np.random.default_rng(5)
    qn, kn = ((1 + 0.02 * r.standard_normal(hd)).astype(np.float32) for _ in range(2))
    ctx = hip.AttnContext(H, KV, hd, rope_theta=1e6, q_norm=qn, k_norm=kn, eps=1e-6)
    cache = hip.KVCache(ctx, 9, cap)
    blk = orc.Block(H * hd, H, KV, hd, eps=1e-6, rope_theta=1e6)
    blk.set_qk_norm(qn, kn)
    for T in (300, 1, 1):  # prefill kernel, then the split-K decode kernel
        q, k, v = rows(r, T, H, KV, hd)
        got = ctx.forward(cache, q, k, v, [T], [8])
        rm.assert_close(got, blk.attention_cached_qkv(q, k, v, threads=16), ATOL, RTOL, f"T={T} in slot 8")
    for c in (0, KV - 1):
        kd, vd = cache.read(8, c, 0, 302)
        assert np.array_equal(kd, blk.k_cache(c)) and np.array_equal(vd, blk.v_cache(c))
    assert cache.len(8) == 302 and cache.len(0) == 0
    cache.close()
    ctx.close()


def test_decode_context_131072(hip):
    # one sequence of 131 072 cached positions (65 536 tiles over the 8 kv heads), one new row
    H, KV, hd, S = 32, 8, 128, 131072
    ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=True, capacity=S + 8, seed=13)
    kf, vf = (r.standard_normal((KV, S, hd), dtype=np.float32) for _ in range(2))
    cache.fill(0, kf, vf)
    blocks[0].fill_cache(kf, vf)
    assert check_step(ctx, cache, blocks, r, [1], threads=16) < 1e-4
    assert cache.len(0) == S + 1


# ------------------------------------------------------------------ properties at full size
def test_full_size_properties_prefill_8192(hip):
    """T = 8192 (Llama-1B geometry), on top of the comparison of all rows with the oracle in
    test_prefill_full_size_every_instantiation: (a) rows around tile and block edges against the
    oracle run on just those rows, from the device's own cache contents, (b) causality, (c) GQA
    sharing."""
    import torch

    H, KV, hd, T = 32, 8, 64, 8192
    ctx = hip.AttnContext(H, KV, hd, rope_theta=500000.0)
    cache = hip.KVCache(ctx, 1, T)
    gen = torch.Generator(device="cuda").manual_seed(4)
    q = torch.randn((T, H * hd), generator=gen, device="cuda")
    k = torch.randn((T, KV * hd), generator=gen, device="cuda")
    v = torch.randn((T, KV * hd), generator=gen, device="cuda")
    q.view(T, KV, 4, hd)[:, :, 1] = q.view(T, KV, 4, hd)[:, :, 0]  # heads 4c and 4c+1 share a query
    torch.cuda.synchronize()
    out = ctx.forward(cache, q, k, v, [T])
    ctx.sync()
    o = out.cpu().numpy().reshape(T, H, hd)
    assert np.isfinite(o).all()
    assert np.array_equal(o[:, 0::4], o[:, 1::4])            # equal queries of a group -> equal outputs
    assert np.abs(o[0] - v[0].cpu().numpy().reshape(KV, 1, hd).repeat(4, 1).reshape(H, hd)).max() < 1e-6
    # oracle on sampled rows: fill its cache with the GPU's cache (bit-identical by the tests above)
    b = orc.Block(H * hd, H, KV, hd, rope_theta=500000.0)
    qh, kh, vh = q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()
    for pos in (1, 31, 32, 33, 127, 128, 4095, 4096, 8191):
        kc = np.stack([cache.read(0, c, 0, pos)[0] for c in range(KV)])
        vc = np.stack([cache.read(0, c, 0, pos)[1] for c in range(KV)])
        b.fill_cache(kc, vc)
        want = b.attention_cached_qkv(qh[pos:pos + 1], kh[pos:pos + 1], vh[pos:pos + 1], threads=8)
        rm.assert_close(o[pos].reshape(1, -1), want, ATOL, RTOL, f"row {pos}")
    # causality: changing rows >= 5000 leaves outputs of rows < 5000 bit-identical
    k2, v2 = k.clone(), v.clone()
    k2[5000:] += 1.0
    v2[5000:] -= 1.0
    cache.clear()
    torch.cuda.synchronize()
    out2 = ctx.forward(cache, q, k2, v2, [T])
    ctx.sync()
    assert torch.equal(out2[:5000], out[:5000]) and not torch.equal(out2[5000:], out[5000:])


# ------------------------------------------------------------------ RoPE.apply (rope.cr:7-33)
def test_rope_apply_reference_known_answers(hip):
    # spec/rope_kv_cache_spec.cr:5-26
    m = np.arange(1, 9, dtype=np.float32).reshape(1, 8)
    assert np.abs(hip.RoPE.apply(m, 0, 10000.0) - m).max() < 1e-5
    m = np.array([[1.0, 0.0, 0.0, 0.0]], np.float32)
    out = hip.RoPE.apply(m, 1, 10000.0)
    assert abs(out[0, 0] - np.cos(1.0)) < 1e-4 and abs(out[0, 2] - np.sin(1.0)) < 1e-4


@pytest.mark.parametrize("T,hd,start,theta", [(1, 8, 0, 1e4), (33, 64, 5, 1e4), (700, 128, 32000, 1e6), (9, 7, 3, 5e5),
                                              (4, 1, 2, 1e4), (50, 33, 100, 1e4)])
def test_rope_apply_matches_oracle(hip, T, hd, start, theta):
    """Against orc_rope_apply.  Both sides compute in fp64 and round once; the device's fp64 pow, cos
    and sin may differ from the host libm's in the last bit of a double, which can move a result
    across an fp32 rounding boundary: at most one unit in the last place, and rarely."""
    import torch

    r = np.random.default_rng(T + hd)
    x = r.standard_normal((T, hd)).astype(np.float32)
    want = orc.rope_apply(x, start, theta)
    got = hip.RoPE.apply(x, start, theta)
    ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
    assert ulp.max() <= 1 and (ulp > 0).mean() < 1e-3, (ulp.max(), (ulp > 0).mean())
    if hd & 1:
        assert np.array_equal(got[:, hd - 1], x[:, hd - 1])  # the odd trailing column is copied through
    dev = hip.RoPE.apply(torch.from_numpy(x).cuda(), start, theta)
    torch.cuda.synchronize()
    assert np.array_equal(dev.cpu().numpy(), got)
    # rotation: every pair keeps its norm
    h = hd // 2
    n0 = x[:, :h].astype(np.float64) ** 2 + x[:, h:2 * h].astype(np.float64) ** 2
    n1 = got[:, :h].astype(np.float64) ** 2 + got[:, h:2 * h].astype(np.float64) ** 2
    if h:
        assert np.abs(n1 - n0).max() <= 1e-5 * max(1.0, n0.max())


# ------------------------------------------------------------------ entry points with the reference's names
@pytest.mark.parametrize("H,g,hd,S,T", [(8, 2, 8, 0, 6), (8, 2, 8, 6, 1), (32, 4, 64, 300, 1), (32, 4, 64, 0, 200),
                                        (32, 8, 128, 100, 40)])
def test_reference_named_entry_points(hip, H, g, hd, S, T):
    import torch

    KV, cap = H // g, 512
    r = np.random.default_rng(H + S + T)
    b = orc.Block(H * hd, H, KV, hd)
    if S:
        b.attention_cached_qkv(*rows(r, S, H, KV, hd))
    q, k, v = rows(r, T, H, KV, hd)
    kc = torch.zeros((KV, cap, hd), device="cuda")
    vc = torch.zeros((KV, cap, hd), device="cuda")
    for c in range(KV):
        kc[c, :S] = torch.from_numpy(b.k_cache(c)) if S else kc[c, :S]
        vc[c, :S] = torch.from_numpy(b.v_cache(c)) if S else vc[c, :S]
    want = b.attention_cached_qkv(q, k, v)
    # host side of attention_heads_gpu (llama_block.cr:432-467): staging = K tails, V tails, rotated Q
    k_new = np.stack([b.k_cache(c)[S:] for c in range(KV)])
    v_new = np.stack([b.v_cache(c)[S:] for c in range(KV)])
    invf = b.inv_freq()
    ang = (np.arange(S, S + T, dtype=np.float32)[:, None] * invf[None]).astype(np.float32)
    cs, sn = np.cos(ang).astype(np.float32)[:, None], np.sin(ang).astype(np.float32)[:, None]
    qh = q.reshape(T, H, hd)
    x0, x1 = qh[..., :hd // 2], qh[..., hd // 2:]
    q_rot = np.concatenate([x0 * cs - x1 * sn, x1 * cs + x0 * sn], -1).reshape(T, H * hd).astype(np.float32)
    staging = torch.from_numpy(np.concatenate([k_new.ravel(), v_new.ravel(), q_rot.ravel()])).cuda()
    out = torch.empty((T, H * hd), device="cuda")
    torch.cuda.synchronize()
    hip.HIP.kv_cache_append_f32(staging, kc, vc, T, S, KV, hd, cap)
    hip.HIP.attention_kv_f32(staging[2 * k_new.size:], kc, vc, out, None, T, S, H, g, hd, cap, b.scale())
    torch.cuda.synchronize()
    rm.assert_close(out.cpu().numpy(), want, ATOL, RTOL)
    assert torch.equal(kc[:, S:S + T].cpu(), torch.from_numpy(k_new))


def test_reference_named_attention_reports_a_given_up_wait(hip):
    """attention_kv_f32 returns nothing and is asynchronous: what an earlier call's kernel reported is
    printed by the next call, as the reference prints the launch error of every call
    (cuda_kernels.cu:821-824).  Forced from the host in a child process (the switch is read when
    the handle-less context is made): marks go where nobody looks, polling ends after 2000 looks."""
    import subprocess
    import sys

    code = """
import numpy as np, torch, shainet_amd as sa
H, g, hd, S, cap = 8, 2, 64, 2500, 3000
KV = H // g
kc = torch.randn((KV, cap, hd), device="cuda"); vc = torch.randn((KV, cap, hd), device="cuda")
q = torch.randn((1, H * hd), device="cuda"); out = torch.empty_like(q)
torch.cuda.synchronize()
for i in range(2):
    sa.HIP.attention_kv_f32(q, kc, vc, out, None, 1, S, H, g, hd, cap, 0.125)
    torch.cuda.synchronize()
print("done")
"""
    env = dict(os.environ, SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS="1", PYTHONPATH=ROOT)
    done = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and "done" in done.stdout, done.stderr[-2000:]
    assert "HIP Error in attention_kv_f32 (an earlier call)" in done.stderr and "gave up waiting" in done.stderr, done.stderr[-2000:]
    env.pop("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS")
    done = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and "HIP Error" not in done.stderr, done.stderr[-2000:]


def test_device_pointer_mode_matches_host_pointer_mode(hip):
    import torch

    H, KV, hd = 32, 8, 128
    r = np.random.default_rng(2)
    parts = [rows(r, T, H, KV, hd) for T in (300, 1, 1)]
    res = []
    for dev in (False, True):
        ctx = hip.AttnContext(H, KV, hd, rope_theta=1e6)
        cache = hip.KVCache(ctx, 1, 512)
        outs = []
        for p in parts:
            if dev:
                t = [torch.from_numpy(a).cuda() for a in p]
                torch.cuda.synchronize()
                o = ctx.forward(cache, *t, [p[0].shape[0]])
                ctx.sync()
                outs.append(o.cpu().numpy())
            else:
                outs.append(ctx.forward(cache, *p, [p[0].shape[0]]))
        res.append(np.concatenate(outs))
    assert np.array_equal(res[0], res[1])


def test_two_contexts_decode_at_the_same_time(hip):
    """Two contexts, each on its own stream, take decode calls in turn without waiting for each
    other: their kernels share the chip, and each launch's merging workgroups wait only for
    workgroups of their own launch."""
    import torch

    H, KV, hd, steps = 16, 4, 128, 12
    sides = []
    for seed, L in ((11, 3000), (12, 1700)):
        ctx, cache, blocks, r = make_pair(hip, H, KV, hd, 1e6, norm=True, capacity=L + steps + 8, seed=seed)
        kf, vf = (r.standard_normal((KV, L, hd)).astype(np.float32) for _ in range(2))
        cache.fill(0, kf, vf)
        blocks[0].fill_cache(kf, vf)
        rows_ = [rows(r, 1, H, KV, hd) for _ in range(steps)]
        dev = [[torch.from_numpy(a).cuda() for a in p] for p in rows_]
        sides.append((ctx, cache, blocks[0], rows_, dev, []))
    torch.cuda.synchronize()
    for i in range(steps):
        for ctx, cache, _, _, dev, outs in sides:
            outs.append(ctx.forward(cache, *dev[i], [1]))  # device pointers: asynchronous
    for ctx, cache, blk, rows_, _, outs in sides:
        ctx.sync()
        for i in range(steps):
            want = blk.attention_cached_qkv(*rows_[i], threads=4)
            rm.assert_close(outs[i].cpu().numpy(), want, ATOL, RTOL, f"step {i}")


# ------------------------------------------------------------------ the layer, projections included
def _layer_pair(hip, d, H, KV, hd, theta, seed, norm=False, bias=False, wscale=0.02):
    r = np.random.default_rng(seed)
    blk = hip.LlamaBlock(d, H, eps=1e-6, rope_theta=theta, num_kv_heads=KV, head_dim=hd)
    ob = orc.Block(d, H, KV, hd, eps=1e-6, rope_theta=theta)
    hd_ = blk.head_dim
    ws = [(wscale * r.standard_normal(s)).astype(np.float32)
          for s in ((d, H * hd_), (d, KV * hd_), (d, KV * hd_), (H * hd_, d))]
    blk.set_weights(*ws)
    ob.set_weights(*ws)
    if norm:
        qn, kn = ((1 + 0.02 * r.standard_normal(hd_)).astype(np.float32) for _ in range(2))
        blk.set_qk_norm(qn, kn)
        ob.set_qk_norm(qn, kn)
    if bias:
        bs = [0.3 * r.standard_normal(n * hd_).astype(np.float32) for n in (H, KV, KV)]
        blk.set_bias(*bs)
        ob.set_bias(*bs)
    return blk, ob, r


def test_config1_llama1b_attention_layer_with_projections(hip):
    # BASELINE configs[0]: hidden 2048, 32 Q / 8 KV heads, head_dim 64, theta 5e5, weights ~N(0, 0.02),
    # x ~N(0,1); cache brought to 512 positions, then one new row at a time.  The oracle's projections
    # accumulate in fp64 (SimpleMatrix#*), the device's in fp32.
    blk, ob, r = _layer_pair(hip, 2048, 32, 8, None, 500000.0, seed=1)
    x = r.standard_normal((512, 2048)).astype(np.float32)
    rm.assert_close(blk.attention_cached(x), ob.attention_cached(x), ATOL, RTOL, "prefill 512")
    for i in range(3):
        x = r.standard_normal((1, 2048)).astype(np.float32)
        rm.assert_close(blk.attention_cached(x), ob.attention_cached(x), ATOL, RTOL, f"decode {i}")
    assert blk.cache_len == ob.cache_len == 515


@pytest.mark.parametrize("d,H,KV,hd,norm,bias,Ts", [
    (64, 8, 4, None, False, False, [6, 1, 1, 1]),     # spec/llama_attention_gpu_spec.cr:16-66
    (32, 4, 2, None, False, False, [290] + [1] * 10),  # :68-104, crosses the initial capacity of 256
    (128, 8, 2, 64, True, True, [20, 3, 1, 17]),       # explicit head_dim (q_dim != d_model), QK-norm, biases
    (256, 8, 8, 128, True, False, [33, 1]),
])
def test_layer_matches_oracle(hip, d, H, KV, hd, norm, bias, Ts):
    blk, ob, r = _layer_pair(hip, d, H, KV, hd, 1e6, seed=d + H, norm=norm, bias=bias, wscale=0.1)
    xs = [r.uniform(-1, 1, (T, d)).astype(np.float32) for T in Ts]
    first = []
    for x in xs:
        got = blk.attention_cached(x)
        rm.assert_close(got, ob.attention_cached(x), ATOL, RTOL)
        first.append(got)
    # rerun after clear: identical results, no stale rows (spec/llama_attention_gpu_spec.cr:90-103)
    blk.clear_cache()
    assert blk.cache_len == 0
    for x, want in zip(xs, first):
        assert np.array_equal(blk.attention_cached(x), want)


def test_layer_argument_errors(hip):
    with pytest.raises(hip.ArgumentError):
        hip.LlamaBlock(64, 8, num_kv_heads=3)
    with pytest.raises(hip.ArgumentError):
        hip.LlamaBlock(64, 7)
    blk, ob, r = _layer_pair(hip, 32, 4, 2, None, 1e4, seed=5)
    blk.set_bias(np.zeros(31), np.zeros(16), np.zeros(16))  # llama_block.cr:587 raises at forward time
    with pytest.raises(hip.ArgumentError):
        blk.attention_cached(np.zeros((1, 32), np.float32))
    blk.set_bias(None, None, None)
    blk.set_qk_norm(np.ones(7), np.ones(8))                 # llama_block.cr:618
    with pytest.raises(hip.ArgumentError):
        blk.attention_cached(np.zeros((1, 32), np.float32))


def test_c_abi_from_plain_c(hip):
    # tests/cabi_smoke.c, compiled by __graft_entry__.build(): the fused entry points called from C,
    # checked against closed forms (one key: out == V; two keys: a two-way softmax in double)
    import subprocess

    here = os.path.dirname(os.path.abspath(__file__))
    exe = os.path.join(here, "cabi_smoke")
    if not os.path.exists(exe):  # normally built by __graft_entry__.build(); a fraction of a second with gcc
        lib_dir = os.path.dirname(hip.library_path())
        subprocess.run(["gcc", "-O1", "-Wall", "-o", exe, os.path.join(here, "cabi_smoke.c"), "-L" + lib_dir,
                        "-lshainet_hip_kernels", "-lm", "-Wl,-rpath,$ORIGIN/../shainet_amd/lib"], check=True)
    done = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0 and "cabi_smoke ok" in done.stdout, done.stdout + done.stderr


def test_yardstick_kernels_do_the_work_they_count(hip):
    # the plain copy / read kernels and the MFMA loop that bench.py compares the attention kernels
    # with: a yardstick that skipped part of its work would flatter every roofline fraction
    import torch

    from shainet_amd import hip as yard

    n = 1 << 20
    a = torch.arange(n, device="cuda", dtype=torch.float32) % 7.0
    b = torch.zeros_like(a)
    yard.stream_copy(a, b, 64)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    sink = torch.zeros(64, device="cuda")
    yard.stream_read(a, sink, 64)
    torch.cuda.synchronize()
    assert float(sink.sum()) == float(a.double().sum())  # small integers: exact in any order

    # every lane's 64 accumulator registers hold sum_k A[m][k] B[k][n] per MFMA with A[m][k] =
    # 0.5 + 1e-6 * (32 k + m) and B = 0.25; a lane's registers cover 16 values of m (both lane halves
    # together all 32), and each accumulator takes 4 MFMAs per round
    iters, wgs = 3, 2
    sink = torch.zeros(wgs * 512, device="cuda")
    flops = yard.mfma_f32_loop(sink, iters, wgs)
    torch.cuda.synchronize()
    assert flops == wgs * 8 * iters * 16 * 2 * 32 * 32 * 2
    got = sink.cpu().numpy().astype(np.float64).reshape(wgs, 8, 64)
    lane_a = lambda wave, lane: 0.5 + 1e-6 * np.float32(64 * wave + lane).astype(np.float64)  # noqa: E731
    for wave in range(8):
        for lane in (0, 5, 31, 32, 63):
            half = lane // 32
            ms = [8 * (r // 4) + 4 * half + r % 4 for r in range(16)]
            per_mfma = [0.25 * (lane_a(wave, m) + lane_a(wave, m + 32)) for m in ms]
            want = 4 * (4 * iters) * sum(per_mfma)
            assert abs(got[0, wave, lane] - want) < 1e-4 * want, (wave, lane, got[0, wave, lane], want)
    assert np.array_equal(got[0], got[1])


@pytest.mark.parametrize("splits", [0, 3])
@pytest.mark.parametrize("H,KV,hd", [(8, 2, 64), (4, 1, 128)])
def test_prefill_scores_far_from_unit_scale(hip, H, KV, hd, splits, monkeypatch):
    # The MFMA prefill kernels keep a reference value per row that moves only when a score exceeds it
    # by 2^8, and take scores relative to it straight from the accumulator: score sequences that climb
    # or fall by more than that from tile to tile, jump between +-hundreds, or have a huge spread must
    # come out as the oracle's running-maximum softmax does.  Scores are steered through the last
    # rotation pair, which RoPE (theta 1e6) turns by less than 1e-3 rad over these positions.
    if splits:
        monkeypatch.setenv("SHAINET_HIP_PREFILL_SPLITS", str(splits))
    S, T = 70, 200
    L = S + T
    pos = np.arange(L, dtype=np.float64)
    shapes = {
        "climbing": 3.0 * pos,                                 # every tile's maximum is 96 above the last one's
        "falling": -3.0 * pos,                                 # the first key dominates; later ones underflow
        "sawtooth": 400.0 * ((pos // 32) % 2) - 200.0,         # whole tiles at -200 and +200 in turn
        "late_spike": np.where(pos == L - 40, 500.0, -500.0),  # one key 1000 above all others
    }
    r = np.random.default_rng(hd + splits)
    for name, target in shapes.items():
        ctx, cache, blocks, _ = make_pair(hip, H, KV, hd, 1e6, capacity=512, seed=3)
        d = hd - 1                                   # second half of the last rotation pair
        k = np.zeros((L, KV * hd), np.float32)
        q = np.zeros((L, H * hd), np.float32)
        v = r.standard_normal((L, KV * hd)).astype(np.float32)
        k[:, d::hd] = (target / 16.0)[:, None]
        q[:, d::hd] = 16.0 * np.sqrt(hd)             # score = q k / sqrt(hd) = target
        q += 0.01 * r.standard_normal(q.shape).astype(np.float32)
        k += 0.01 * r.standard_normal(k.shape).astype(np.float32)
        for lo, hi in ((0, S), (S, L)):
            got = ctx.forward(cache, q[lo:hi], k[lo:hi], v[lo:hi], [hi - lo])
            want = blocks[0].attention_cached_qkv(q[lo:hi], k[lo:hi], v[lo:hi], threads=8)
            assert np.isfinite(got).all(), name
            rm.assert_close(got, want, ATOL, RTOL, f"{name} hd={hd} rows {lo}..{hi}")


@pytest.mark.parametrize("seed", range(10))
def test_prefill_random_shapes(hip, seed, monkeypatch):
    """The MFMA prefill kernels over unrelated shapes: both head dims, every group size, one to four
    sequences with different cached and new lengths in one call (row blocks of one wavefront next to
    full ones, diagonals at every offset inside a tile), QK-norm and bias on odd seeds, the key range
    cut into 1 to 4 chunks; two calls, the second on the grown caches."""
    r0 = np.random.default_rng(2000 + seed)
    hd = int(r0.choice([64, 128]))
    KV = int(r0.choice([1, 2, 4]))
    g = int(r0.choice([1, 2, 3, 4, 8]))
    B = int(r0.choice([1, 2, 4]))
    splits = int(r0.choice([0, 0, 2, 3, 4]))
    if splits:
        monkeypatch.setenv("SHAINET_HIP_PREFILL_SPLITS", str(splits))
    cached = [int(x) for x in r0.integers(0, 400, B)]
    first = [int(x) for x in r0.integers(17, 260, B)]
    second = [int(x) for x in r0.integers(17, 120, B)]
    ctx, cache, blocks, r = make_pair(hip, KV * g, KV, hd, 1e6, norm=bool(seed & 1), bias=bool(seed & 1), batch=B,
                                      capacity=800, seed=seed)
    for s_, L in enumerate(cached):
        if L:
            kf, vf = (r.standard_normal((KV, L, hd)).astype(np.float32) for _ in range(2))
            cache.fill(s_, kf, vf)
            blocks[s_].fill_cache(kf, vf)
    what = f"hd {hd} KV {KV} g {g} B {B} splits {splits} cached {cached}"
    assert check_step(ctx, cache, blocks, r, first, what=f"{what} new {first}") < 1e-4
    assert check_step(ctx, cache, blocks, r, second, what=f"{what} then {second}") < 1e-4
    check_cache_bits(cache, blocks)
