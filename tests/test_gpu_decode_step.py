"""Decode steps that read and advance the cached lengths on the device (shainet_attn_decode_step)
against shainet_attn_forward with one new row per sequence, through the C ABI: same inputs into two
contexts with identical caches; outputs and caches must be bit-identical (the same kernels with the
same split of the keys; only who computes the split differs).  Run eagerly, and recorded once into
a graph and replayed, with eager work and waits between the replays, every replay checked."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import shainet_amd as sa

    assert sa.HIP.fully_available(), "no gfx950 device or libshainet_hip_kernels.so missing"
    return sa


def _norms(seed, hd):
    r = np.random.default_rng(seed)
    return tuple((1 + 0.02 * r.standard_normal(hd)).astype(np.float32) for _ in range(2))


def _pair(hip, H, KV, hd, lens, cap, seed, qk_norm=True, bias=False):
    import torch

    qn, kn = _norms(seed, hd) if qk_norm else (None, None)
    r = np.random.default_rng(seed + 1)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    fills = [(torch.randn((KV, L, hd), generator=gen, device="cuda"), torch.randn((KV, L, hd), generator=gen, device="cuda"))
             for L in lens]
    biases = [(0.1 * r.standard_normal(n)).astype(np.float32) for n in (H * hd, KV * hd, KV * hd)] if bias else None
    torch.cuda.synchronize()
    sides = []
    for _ in range(2):
        ctx = hip.AttnContext(H, KV, hd, rope_theta=1e6, q_norm=qn, k_norm=kn, eps=1e-6, max_positions=cap)
        if biases:
            ctx.set_bias(*biases)
        cache = hip.KVCache(ctx, len(lens), cap)
        for s, (kf, vf) in enumerate(fills):
            if kf.shape[1]:
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
        assert a.len(s) == b.len(s), (s, a.len(s), b.len(s))
        for c in (0, KV - 1):
            ka, va = a.read(s, c, 0, a.len(s))
            kb, vb = b.read(s, c, 0, b.len(s))
            assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32))
            assert np.array_equal(va.view(np.uint32), vb.view(np.uint32))


CASES = [
    # H, KV, hd, cached lengths, qk_norm, bias
    (32, 8, 128, [4095], False, False),                       # batch 1 of the decode workloads
    (32, 8, 128, [0, 1, 15, 16, 17, 300, 2999, 31], True, False),  # empty and tile-edge lengths
    (32, 8, 64, [16000], True, False),                        # one pair over many workgroups
    (14, 2, 64, [700, 5, 90], False, True),                   # Qwen2.5-0.5B heads: g = 7, biases
    (8, 8, 128, [int(x) for x in np.random.default_rng(3).integers(1, 1500, 64)], False, False),  # 64 sequences, g = 1
    (32, 2, 128, [513, 64], True, False),                     # g = 16
    (32, 8, 96, [700, 33, 1], True, True),                    # head_dim 96: tiles padded to 128
    (8, 4, 44, [300, 2000], False, False),                    # head_dim 44: tiles padded to 64
    (8, 2, 8, [40], False, False),                            # head_dim 8: tiles padded to 64
]


@pytest.mark.parametrize("H,KV,hd,lens,qk_norm,bias", CASES)
def test_eager_steps_match_forward(hip, H, KV, hd, lens, qk_norm, bias):
    import torch

    n = len(lens)
    steps = 5
    (ref, alt), gen = _pair(hip, H, KV, hd, lens, max(lens) + steps + 3, seed=11, qk_norm=qk_norm, bias=bias)
    alt[1].lengths_to_device()
    for i in range(steps):
        q, k, v = _rows(torch, gen, n, H, KV, hd)
        want = ref[0].forward(ref[1], q, k, v, [1] * n)
        got = alt[0].decode_step(alt[1], q, k, v, torch.empty_like(q))
        ref[0].sync()
        alt[0].sync()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), f"step {i}: max abs diff {(got - want).abs().max().item():.3e}"
    alt[1].lengths_from_device()
    _same_caches(ref[1], alt[1], n, KV)
    # back to the host-planned entry point on the same cache, and to steps again
    q, k, v = _rows(torch, gen, n, H, KV, hd)
    want = ref[0].forward(ref[1], q, k, v, [1] * n)
    got = alt[0].forward(alt[1], q, k, v, [1] * n)
    ref[0].sync()
    alt[0].sync()
    assert torch.equal(got, want)
    alt[1].lengths_to_device()
    q, k, v = _rows(torch, gen, n, H, KV, hd)
    want = ref[0].forward(ref[1], q, k, v, [1] * n)
    got = alt[0].decode_step(alt[1], q, k, v, torch.empty_like(q))
    ref[0].sync()
    alt[1].lengths_from_device()
    assert torch.equal(got, want)
    _same_caches(ref[1], alt[1], n, KV)


def test_first_sequences_only(hip):
    # a step over the first 3 of 8 sequences leaves the others alone
    import torch

    H, KV, hd = 32, 8, 128
    lens = [100, 2000, 37, 5, 5, 5, 5, 5]
    (ref, alt), gen = _pair(hip, H, KV, hd, lens, 2100, seed=4)
    alt[1].lengths_to_device()
    for i in range(3):
        q, k, v = _rows(torch, gen, 3, H, KV, hd)
        want = ref[0].forward(ref[1], q, k, v, [1] * 3)
        got = alt[0].decode_step(alt[1], q, k, v, torch.empty_like(q))
        ref[0].sync()
        alt[0].sync()
        assert torch.equal(got, want), f"step {i}"
    alt[1].lengths_from_device()
    assert [alt[1].len(s) for s in range(8)] == [103, 2003, 40, 5, 5, 5, 5, 5]
    _same_caches(ref[1], alt[1], 8, KV)


@pytest.mark.parametrize("H,KV,hd,lens", [(32, 8, 128, [4090]), (32, 8, 128, [900, 14, 3000, 16]), (32, 8, 64, [33] * 16)])
def test_recorded_step_replays(hip, H, KV, hd, lens):
    """One step recorded into a graph on the context's stream; every replay is one more decode
    step.  Between the replays: new inputs copied into the recorded buffers, unrelated eager
    kernels, waits.  Every replay is compared with the eager entry point on a twin cache."""
    import torch

    n = len(lens)
    replays = 7
    (ref, alt), gen = _pair(hip, H, KV, hd, lens, max(lens) + replays + 4, seed=31)
    side = torch.cuda.Stream()
    alt[0].set_stream(side.cuda_stream)
    alt[1].lengths_to_device()
    qb, kb, vb = _rows(torch, gen, n, H, KV, hd)
    ob = torch.empty_like(qb)
    # an eager step first (also what a warm-up before recording would do) ...
    want = ref[0].forward(ref[1], qb, kb, vb, [1] * n)
    alt[0].decode_step(alt[1], qb, kb, vb, ob)
    ref[0].sync()
    alt[0].sync()
    assert torch.equal(ob, want)
    # ... then the recording: nothing runs, nothing is appended
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        alt[0].decode_step(alt[1], qb, kb, vb, ob)
    torch.cuda.synchronize()
    busy = torch.randn((1024, 1024), device="cuda")
    for i in range(replays):
        q, k, v = _rows(torch, gen, n, H, KV, hd)
        want = ref[0].forward(ref[1], q, k, v, [1] * n)
        ref[0].sync()
        with torch.cuda.stream(side):
            qb.copy_(q)
            kb.copy_(k)
            vb.copy_(v)
            ob.zero_()
            busy = torch.tanh(busy @ busy * 1e-3)  # eager work of the program's own
            graph.replay()
        if i % 2 == 0:
            torch.cuda.synchronize()
        else:
            side.synchronize()
        assert torch.isfinite(ob).all()
        assert torch.equal(ob, want), f"replay {i}: max abs diff {(ob - want).abs().max().item():.3e}"
    alt[1].lengths_from_device()
    assert [alt[1].len(s) for s in range(n)] == [L + 1 + replays for L in lens]
    _same_caches(ref[1], alt[1], n, KV)
    del graph


def test_step_at_capacity_appends_nothing_and_reports(hip):
    import torch

    H, KV, hd = 32, 8, 128
    lens, cap = [10, 18], 20
    (ref, alt), gen = _pair(hip, H, KV, hd, lens, cap, seed=8)
    ctx, cache = alt
    cache.lengths_to_device()
    outs = []
    for i in range(4):  # the third step would take sequence 1 to 21 rows
        q, k, v = _rows(torch, gen, 2, H, KV, hd)
        out = torch.full_like(q, 7.0)
        ctx.decode_step(cache, q, k, v, out)
        outs.append(out)
    with pytest.raises(hip.HipError, match="capacity"):
        cache.lengths_from_device()
    assert torch.all(outs[2] == 7.0) and torch.all(outs[3] == 7.0) and not torch.any(outs[1] == 7.0)
    assert [cache.len(0), cache.len(1)] == [12, 20]
    # the error is reported once; the cache goes on after a truncate
    cache.truncate(1, 5)
    cache.lengths_to_device()
    q, k, v = _rows(torch, gen, 2, H, KV, hd)
    ctx.decode_step(cache, q, k, v, torch.empty_like(q))
    cache.lengths_from_device()
    assert [cache.len(0), cache.len(1)] == [13, 6]


def test_step_refuses_what_it_cannot_do(hip):
    import torch

    H, KV, hd = 32, 8, 128
    (ref, alt), gen = _pair(hip, H, KV, hd, [10], 64, seed=2)
    ctx, cache = alt
    q, k, v = _rows(torch, gen, 1, H, KV, hd)
    with pytest.raises(hip.ArgumentError, match="lengths_to_device"):
        ctx.decode_step(cache, q, k, v, torch.empty_like(q))
    with pytest.raises(hip.ArgumentError, match="lengths_to_device"):
        cache.lengths_from_device()
    cache.lengths_to_device()
    # between the two copies the device's lengths are the ones that count: whatever reads or writes the
    # host's copy is refused (it would drop or overwrite the rows the steps append)
    for refused in (lambda: cache.reserve(128), lambda: cache.truncate(0, 5), lambda: cache.clear(),
                    lambda: cache.fill(0, np.zeros((KV, 3, hd), np.float32), np.zeros((KV, 3, hd), np.float32)),
                    lambda: ctx.forward(cache, q, k, v, [1]), lambda: cache.lengths_to_device()):
        with pytest.raises(hip.ArgumentError, match="lengths_from_device"):
            refused()
    assert cache.len(0) == -1
    ctx.decode_step(cache, q, k, v, torch.empty_like(q))
    cache.lengths_from_device()
    assert cache.len(0) == 11
    cache.reserve(128)
    with pytest.raises(hip.ArgumentError, match="lengths_to_device"):   # the lengths are back on the host
        ctx.decode_step(cache, q, k, v, torch.empty_like(q))
    q2, k2, v2 = _rows(torch, gen, 2, H, KV, hd)
    cache.lengths_to_device()
    with pytest.raises(hip.ArgumentError, match="n_seqs"):
        ctx.decode_step(cache, q2, k2, v2, torch.empty_like(q2))
    for odd_hd in (6, 256):   # not a multiple of 4; above 128
        odd = hip.AttnContext(4, 4, odd_hd, rope_theta=1e4, max_positions=64)
        with pytest.raises(hip.ArgumentError, match="head_dim"):
            hip.KVCache(odd, 1, 64).lengths_to_device()
