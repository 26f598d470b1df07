"""The decode step that runs a whole stack of blocks as one launch (LlamaModel decode mode
PERSISTENT) against the CPU oracle, the transformers fixture and the launch-per-product path,
through the C ABI, on a real MI355X.  Same bar as the other model tests: logits within
1e-4 + 1e-3*|oracle|; the two paths of the library agree far closer than that (they differ in
summation order only), and greedy ids are the same."""
import os

import numpy as np
import pytest

import refmath as rm
import tinyllama
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-4, 1e-3


@pytest.fixture(scope="module")
def hip():
    import shainet_amd as sa

    assert sa.HIP.fully_available(), "no gfx950 device or libshainet_hip_kernels.so missing"
    return sa


def tiny_model(hip):
    w = tinyllama.load()
    c = w["cfg"]
    m = hip.LlamaModel(c["vocab_size"], c["hidden_size"], c["num_hidden_layers"], c["num_attention_heads"],
                       c["intermediate_size"], eps=c["rms_norm_eps"], rope_theta=c["rope_theta"],
                       num_kv_heads=c["num_key_value_heads"])
    m.set_embedding(w["embed"])
    m.set_final_norm(w["final_norm"])
    m.set_lm_head(w["lm_head"])
    for b, lw in zip(m.blocks, w["layers"]):
        b.set_weights(lw["w_q"], lw["w_k"], lw["w_v"], lw["w_o"])
        b.set_norms(lw["norm1"], lw["norm2"])
        b.set_ffn(lw["gate"], lw["up"], lw["down"])
    return m, w


def random_model(hip, V, d, L, H, KV, hd, ff, seed, qknorm=False, bias=False, scale=0.05):
    r = np.random.default_rng(seed)
    m = hip.LlamaModel(V, d, L, H, ff, eps=1e-5, rope_theta=5e5, num_kv_heads=KV, head_dim=hd)
    m.set_embedding(r.standard_normal((V, d), dtype=np.float32))
    m.set_lm_head(scale * r.standard_normal((d, V), dtype=np.float32))
    m.set_final_norm((1 + 0.1 * r.standard_normal(d)).astype(np.float32))
    for b in m.blocks:
        ws = [(scale * r.standard_normal(sh, dtype=np.float32)) for sh in
              ((d, H * hd), (d, KV * hd), (d, KV * hd), (H * hd, d), (d, ff), (d, ff), (ff, d))]
        b.set_weights(*ws[:4])
        b.set_ffn(*ws[4:])
        b.set_norms((1 + 0.1 * r.standard_normal(d)).astype(np.float32),
                    (1 + 0.1 * r.standard_normal(d)).astype(np.float32))
        if qknorm:
            b.set_qk_norm((1 + 0.1 * r.standard_normal(hd)).astype(np.float32),
                          (1 + 0.1 * r.standard_normal(hd)).astype(np.float32))
        if bias:
            b.set_bias(*(0.1 * r.standard_normal(n * hd).astype(np.float32) for n in (H, KV, KV)))
    return m


def test_tiny_llama_single_launch_steps_match_transformers_and_oracle(hip, golden_dir):
    d = np.load(os.path.join(golden_dir, "tiny_llama_logits.npz"))
    m, w = tiny_model(hip)
    assert m.decode_mode_in_use == m.DECODE_PER_PRODUCT          # the default
    m.set_decode_mode(m.DECODE_PERSISTENT)
    assert m.decode_mode_in_use == m.DECODE_PERSISTENT
    om = tinyllama.OracleModel(w, orc)
    m.run(d["tokens_t3"])                                        # three rows: the prefill path
    om.run(d["tokens_t3"])
    got4 = m.run(d["tokens_t4"][3:])                             # one row: the single launch
    assert np.abs(got4 - d["logits_t4"]).max() < 1e-5
    rm.assert_close(got4, om.run(d["tokens_t4"][3:]), ATOL, RTOL, "decode logits")
    assert m.cache_len == 4
    # token by token from an empty cache: position 0 has no cached key at all
    m.clear_cache()
    om.clear_cache()
    for t in d["tokens_t4"]:
        got = m.run([int(t)])
        want = om.run([int(t)])
    assert np.abs(got - d["logits_t4"]).max() < 1e-5
    rm.assert_close(got, want, ATOL, RTOL, "logits after four single-row runs")
    # greedy generation on the device: the ids of the oracle's loop
    ol = want
    ids = m.generate_greedy(12)
    for i in ids:
        assert i == orc.greedy(ol)
        ol = om.run([i])
    assert m.cache_len == 4 + 12


@pytest.mark.parametrize("V,d,L,H,KV,hd,ff,prompt,steps,kw", [
    (1000, 256, 3, 8, 2, 32, 512, 20, 12, {}),                                  # 4 query heads per kv head
    (1000, 512, 2, 8, 4, 64, 1024, 250, 10, {"qknorm": True, "bias": True}),    # grows the 256-row cache on the way
    (500, 1024, 2, 8, 1, 128, 2048, 0, 6, {"qknorm": True}),                    # 8 per kv head, from an empty cache
    (300, 128, 2, 8, 8, 16, 384, 700, 5, {}),                                   # several key chunks per kv head
    (400, 96, 2, 6, 3, 16, 200, 33, 7, {"bias": True}),                         # widths that no tile divides
])
def test_single_launch_steps_equal_the_launch_per_product_path(hip, V, d, L, H, KV, hd, ff, prompt, steps, kw):
    m = random_model(hip, V, d, L, H, KV, hd, ff, 5, **kw)
    r = np.random.default_rng(1)
    first = list(r.integers(0, V, prompt))
    toks = list(r.integers(0, V, steps))
    rows = {}
    for mode in (m.DECODE_PER_PRODUCT, m.DECODE_PERSISTENT):
        m.set_decode_mode(mode)
        assert m.decode_mode_in_use == mode
        m.clear_cache()
        out = [m.run(first)] if prompt else []
        out += [m.run([t]) for t in toks]
        assert m.cache_len == prompt + steps
        rows[mode] = np.stack(out)
    a, b = rows[m.DECODE_PER_PRODUCT], rows[m.DECODE_PERSISTENT]
    assert np.isfinite(b).all()
    assert np.abs(a - b).max() <= 2e-5 * max(1.0, np.abs(a).max()), np.abs(a - b).max()
    np.testing.assert_array_equal(a.argmax(1), b.argmax(1))
    # the caches the two paths leave are interchangeable: continue one with the other
    m.set_decode_mode(m.DECODE_PER_PRODUCT)
    mixed = m.run([toks[0]])
    m.set_decode_mode(m.DECODE_PERSISTENT)
    m.clear_cache()
    if prompt:
        m.run(first)
    for t in toks:
        m.run([t])
    again = m.run([toks[0]])
    assert np.abs(mixed - again).max() <= 2e-5 * max(1.0, np.abs(mixed).max())
    m.close()


def test_single_launch_step_refuses_a_geometry_it_does_not_fit(hip):
    m = random_model(hip, 50, 96, 1, 6, 6, 24, 64, 2)            # head_dim 24 is no power of two
    m.run([1, 2, 3])
    m.set_decode_mode(m.DECODE_PERSISTENT)
    assert m.decode_mode_in_use == m.DECODE_PER_PRODUCT
    with pytest.raises(hip.ArgumentError, match="does not fit"):
        m.run([4])
    m.set_decode_mode(m.DECODE_AUTO)
    assert np.isfinite(m.run([4])).all()
    with pytest.raises(hip.ArgumentError):
        m.set_decode_mode(7)
    m.close()


def test_workgroups_that_never_arrive_at_the_barrier_are_reported(hip, monkeypatch):
    """Failure handling of the single launch, forced from the host: with the test switch the
    workgroups count their arrivals at a barrier in a place nobody polls and stop polling after
    200 looks, so the kernel still ends by itself; the call that waits for the model's stream
    must report it."""
    m = random_model(hip, 200, 128, 2, 4, 2, 32, 256, 9)
    m.set_decode_mode(m.DECODE_PERSISTENT)
    m.run([5, 6, 7])
    monkeypatch.setenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS", "1")
    try:
        with pytest.raises(hip.hip.HipError, match="gave up waiting"):
            m.run([8])                                           # the first single-row run plans the step: reads the switch
    finally:
        monkeypatch.delenv("SHAINET_HIP_TEST_LOSE_PARTIAL_MARKS")
    m.close()
    # a model made afterwards is unaffected
    m2 = random_model(hip, 200, 128, 2, 4, 2, 32, 256, 9)
    m2.set_decode_mode(m2.DECODE_PERSISTENT)
    m2.run([5, 6, 7])
    assert np.isfinite(m2.run([8])).all()
    m2.close()
