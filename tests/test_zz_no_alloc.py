"""The entry point that allocates nothing (shainet_attn_forward_noalloc) against
shainet_attn_forward, through the C ABI: same inputs into two contexts with identical caches, the
outputs and the caches must be bit-identical (the same kernels run with the same plan; only where
their scratch memory lives differs).  Two calls in a row on the shared static array, the second
with a smaller input, then a third on another context; and what the entry point must refuse."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import shainet_amd as sa

    assert sa.HIP.fully_available(), "no gfx950 device or libshainet_hip_kernels.so missing"
    return sa


def _pair(hip, H, KV, hd, lens, cap, seed):
    """Two contexts with the same parameters and the same cache contents."""
    import torch

    r = np.random.default_rng(seed)
    qn, kn = ((1 + 0.02 * r.standard_normal(hd)).astype(np.float32) for _ in range(2))
    gen = torch.Generator(device="cuda").manual_seed(seed)
    fills = [(torch.randn((KV, L, hd), generator=gen, device="cuda"), torch.randn((KV, L, hd), generator=gen, device="cuda"))
             for L in lens]
    torch.cuda.synchronize()
    sides = []
    for _ in range(2):
        ctx = hip.AttnContext(H, KV, hd, rope_theta=1e6, q_norm=qn, k_norm=kn, eps=1e-6, max_positions=cap)
        cache = hip.KVCache(ctx, len(lens), cap)
        for s, (kf, vf) in enumerate(fills):
            cache.fill(s, kf, vf)
        sides.append((ctx, cache))
    return sides, gen


def _rows(torch, gen, n, H, KV, hd):
    q = torch.randn((n, H * hd), generator=gen, device="cuda")
    k = torch.randn((n, KV * hd), generator=gen, device="cuda")
    v = torch.randn((n, KV * hd), generator=gen, device="cuda")
    torch.cuda.synchronize()
    return q, k, v


def _same_caches(a, b, n_seqs, KV):
    for s in range(n_seqs):
        assert a.len(s) == b.len(s)
        for c in (0, KV - 1):
            ka, va = a.read(s, c, 0, a.len(s))
            kb, vb = b.read(s, c, 0, b.len(s))
            assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32))
            assert np.array_equal(va.view(np.uint32), vb.view(np.uint32))


def test_noalloc_matches_forward_two_calls_second_smaller(hip):
    import torch

    from oracle import oracle as orc

    H, KV, hd = 32, 8, 128
    lens = [int(x) for x in np.random.default_rng(7).integers(300, 3000, 16)]
    (ref, alt), gen = _pair(hip, H, KV, hd, lens, 3100, seed=21)
    # call 1: all 16 sequences, one new row each; call 2: a smaller input, five sequences out of order,
    # with two rows for one of them; call 3: all again (the static array now holds call 2's leftovers)
    calls = [(list(range(16)), [1] * 16), ([9, 2, 15, 0, 4], [1, 2, 1, 1, 1]), (list(range(16)), [1] * 16)]
    outs = []
    for ids, nt in calls:
        q, k, v = _rows(torch, gen, sum(nt), H, KV, hd)
        want = ref[0].forward(ref[1], q, k, v, nt, ids)
        got = alt[0].forward_noalloc(alt[1], q, k, v, nt, ids)
        ref[0].sync()
        alt[0].sync()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), f"ids {ids}: max abs diff {(got - want).abs().max().item():.3e}"
        outs.append((q, k, v, got))
    _same_caches(ref[1], alt[1], 16, KV)
    # and against the oracle for one sequence of the last call (the bar of the parity tests)
    s = 3
    blk = orc.Block(H * hd, H, KV, hd, eps=1e-6, rope_theta=1e6)
    n = alt[1].len(s)
    kv = [alt[1].read(s, c, 0, n - 1) for c in range(KV)]
    blk.set_qk_norm(*_norms(21, hd))
    blk.fill_cache(np.stack([x[0] for x in kv]), np.stack([x[1] for x in kv]))
    q, k, v, got = outs[-1]
    want = blk.attention_cached_qkv(q[s:s + 1].cpu().numpy(), k[s:s + 1].cpu().numpy(), v[s:s + 1].cpu().numpy(), threads=4)
    g = got[s:s + 1].cpu().numpy()
    assert np.all(np.abs(g - want) <= 1e-4 + 1e-3 * np.abs(want)), np.abs(g - want).max()


def test_noalloc_allocates_no_device_memory(hip):
    """Free device memory as the runtime reports it is the same before and after a run of calls
    (contexts, caches and inputs are made first; another cache made afterwards shows that the probe
    sees what the library allocates)."""
    import torch

    H, KV, hd = 32, 8, 128
    (ref, alt), gen = _pair(hip, H, KV, hd, [2900] * 8, 3000, seed=4)
    rows = [_rows(torch, gen, 8, H, KV, hd) for _ in range(6)]
    outs = [torch.empty_like(rows[0][0]) for _ in range(6)]
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for (q, k, v), out in zip(rows, outs):
        alt[0].forward_noalloc(alt[1], q, k, v, [1] * 8, out=out)
    alt[0].sync()
    assert torch.cuda.mem_get_info()[0] == free0
    wants = [ref[0].forward(ref[1], q, k, v, [1] * 8) for q, k, v in rows]
    ref[0].sync()
    extra = hip.KVCache(ref[0], 8, 3000)              # 196 MB from hipMalloc
    assert torch.cuda.mem_get_info()[0] < free0
    del extra
    for want, out in zip(wants, outs):
        assert torch.equal(want, out)


def _norms(seed, hd):
    r = np.random.default_rng(seed)
    return tuple((1 + 0.02 * r.standard_normal(hd)).astype(np.float32) for _ in range(2))


def test_noalloc_other_geometry_shares_the_array(hip):
    # head_dim 64, one long sequence (every pair spread over many workgroups: partials and flags in use),
    # right after the calls above left their contents in the array
    import torch

    H, KV, hd = 32, 8, 64
    (ref, alt), gen = _pair(hip, H, KV, hd, [16000], 16100, seed=5)
    for i in range(3):
        q, k, v = _rows(torch, gen, 1, H, KV, hd)
        want = ref[0].forward(ref[1], q, k, v, [1])
        got = alt[0].forward_noalloc(alt[1], q, k, v, [1])
        ref[0].sync()
        alt[0].sync()
        assert torch.equal(got, want), f"step {i}"
    _same_caches(ref[1], alt[1], 1, KV)


def test_noalloc_refuses_what_it_cannot_hold(hip):
    import torch

    H, KV, hd = 32, 8, 128
    (ref, alt), gen = _pair(hip, H, KV, hd, [100, 50], 4096, seed=9)
    ctx, cache = alt
    # a prefill-sized call is not a decode call
    q, k, v = _rows(torch, gen, 40, H, KV, hd)
    with pytest.raises(hip.ArgumentError, match="decode calls only"):
        ctx.forward_noalloc(cache, q, k, v, [40], [0])
    assert cache.len(0) == 100
    # positions beyond the cos/sin table: the table of this context covers 2048 positions (it was
    # grown to the next power of two by the fill below, which may allocate; this call may not)
    small = hip.AttnContext(H, KV, hd, rope_theta=1e6, max_positions=64)
    c2 = hip.KVCache(small, 1, 4096)
    kf = torch.randn((KV, 2047, hd), generator=gen, device="cuda")
    torch.cuda.synchronize()
    c2.fill(0, kf, kf)
    q, k, v = _rows(torch, gen, 1, H, KV, hd)
    small.forward_noalloc(c2, q, k, v, [1])  # position 2047: the last one the table holds
    small.sync()
    assert c2.len(0) == 2048
    with pytest.raises(hip.HipError, match="cos/sin table"):
        small.forward_noalloc(c2, q, k, v, [1])
    assert c2.len(0) == 2048
    # more rotated-query floats than the array's 2 MiB share: 64 sequences x 2 rows x 32 heads x 128 = 524288
    # fits exactly; with 48 heads it does not
    wide = hip.AttnContext(48, 8, hd, rope_theta=1e6, max_positions=256)
    c3 = hip.KVCache(wide, 64, 64)
    q, k, v = _rows(torch, gen, 128, 48, 8, hd)
    with pytest.raises(hip.HipError, match="static scratch"):
        wide.forward_noalloc(c3, q, k, v, [2] * 64)
    assert c3.len(0) == 0
