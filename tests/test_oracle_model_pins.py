"""Pins of the oracle's restatement of what follows the last block: embedding lookup, final
norm + lm_head, and text/sampler.cr.  Known answers are those of spec/sampler_spec.cr; the
rest is brute force in numpy and the end-to-end logits of the reference's tiny-llama data
fixture computed by transformers (tests/golden/make_golden.py)."""
import os

import numpy as np
import pytest

import oracle.oracle as orc
import tinyllama

NAN, INF = float("nan"), float("inf")


# ---- spec/sampler_spec.cr -------------------------------------------------------------------
def test_greedy_known_answers():
    assert orc.greedy([0.1, 3.2, -1.0, 2.9]) == 1                       # "picks the argmax"
    assert orc.greedy([NAN, INF, 0.5, -INF]) == 2                        # "never selects NaN/Inf"
    assert orc.greedy([1.0, 0.0, 0.0]) == 0 and orc.greedy([0.0, 0.0, 5.0]) == 2  # "requested row"
    assert orc.greedy([NAN, INF, -INF]) == 0                             # best_id starts at 0
    assert orc.greedy([2.0, 7.0, 7.0, 1.0]) == 1                         # strict >: first of equals


def test_sample_top1_is_greedy_and_nan_never_selected():
    row = [0.3, 1.7, 1.69, -0.4, 0.9]
    for r in np.linspace(0, 1, 11):
        assert orc.sample(row, 1, 0.7, float(r)) == orc.greedy(row)     # "top_k = 1 is equivalent to greedy"
    row = [NAN, 2.0, NAN, 1.5, NAN]
    picks = {orc.sample(row, 5, 1.0, float(r)) for r in np.linspace(0, 1, 201)}
    assert picks == {1, 3}                                                # "never selects a NaN logit"
    assert orc.sample([NAN, NAN], 3, 1.0, 0.5) == 0                      # all-NaN row


def test_sample_only_from_the_top_k_set():
    vals = [10.0 - j if j < 5 else -50.0 for j in range(100)]
    picks = {orc.sample(vals, 5, 1.0, float(r)) for r in np.linspace(0, 1, 301)}
    assert picks <= set(range(5)) and 0 in picks


def test_repetition_penalty_known_answers():
    np.testing.assert_array_equal(orc.repetition_penalty([2.0, -2.0, 0.0, 4.0], [0, 1, 3], 2.0), [1.0, -4.0, 0.0, 2.0])
    np.testing.assert_array_equal(orc.repetition_penalty([2.0, -2.0], [0, 1], 1.0), [2.0, -2.0])
    np.testing.assert_array_equal(orc.repetition_penalty([4.0, 4.0, 4.0], [0, 1, 2], 2.0, window=1), [4.0, 4.0, 2.0])
    # an id that repeats is penalised once per occurrence; ids outside the row are skipped
    np.testing.assert_array_equal(orc.repetition_penalty([8.0, -1.0], [0, 0, 7, -3, 1], 2.0), [2.0, -2.0])


# ---- brute force ----------------------------------------------------------------------------
def _brute_topk(row, k):
    row = np.asarray(row, np.float32)
    idx = [i for i in range(row.size) if not np.isnan(row[i])]
    idx.sort(key=lambda i: (-float(row[i]), i))  # descending value, ascending index among equals
    return idx[:k]


@pytest.mark.parametrize("seed", range(6))
def test_topk_matches_a_sort(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 400))
    row = rng.standard_normal(n).astype(np.float32)
    row[rng.integers(0, n, n // 3)] = row[rng.integers(0, n, n // 3)]      # ties
    row[rng.integers(0, n, n // 10)] = np.nan
    if seed % 2:
        row[rng.integers(0, n, 2)] = np.inf
        row[rng.integers(0, n, 2)] = -np.inf
        row[rng.integers(0, n, 3)] = 0.0
        row[rng.integers(0, n, 3)] = -0.0
    for k in (1, 5, 40, n + 3):
        ids, vals = orc.topk(row, k, 0.7)
        want = _brute_topk(row, k)
        assert list(ids) == want
        np.testing.assert_array_equal(vals, row[want].astype(np.float64) / 0.7)


def test_sample_follows_the_temperature_softmax():
    rng = np.random.default_rng(3)
    row = rng.standard_normal(50).astype(np.float32) * 2
    k, t, n = 6, 0.8, 20000
    top = _brute_topk(row, k)
    p = np.exp(row[top].astype(np.float64) / t)
    p /= p.sum()
    counts = np.zeros(50)
    for i in range(n):
        counts[orc.sample(row, k, t, (i + 0.5) / n)] += 1
    assert counts.sum() == n and set(np.nonzero(counts)[0]) == set(top)
    np.testing.assert_allclose(counts[top] / n, p, atol=2.0 / n)


# ---- embedding, final norm, lm_head ----------------------------------------------------------
def test_embed_is_a_row_gather_and_checks_ids():
    rng = np.random.default_rng(0)
    table = rng.standard_normal((11, 5)).astype(np.float32)
    ids = [3, 0, 10, 3]
    np.testing.assert_array_equal(orc.embed(table, ids), table[ids])
    with pytest.raises(orc.ArgumentError):
        orc.embed(table, [11])
    with pytest.raises(orc.ArgumentError):
        orc.embed(table, [-1])


def test_logits_last_closed_form():
    rng = np.random.default_rng(1)
    h = rng.standard_normal((3, 8)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(8)).astype(np.float32)
    w = rng.standard_normal((8, 13)).astype(np.float32)
    b = rng.standard_normal(13).astype(np.float32)
    h64 = h.astype(np.float64)
    normed = (h64 / np.sqrt((h64 ** 2).mean(1, keepdims=True) + 1e-5) * g).astype(np.float32)
    want = (normed[-1].astype(np.float64) @ w.astype(np.float64)).astype(np.float32)
    np.testing.assert_allclose(orc.logits_last(h, g, 1e-5, w), want, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(orc.logits_last(h, g, 1e-5, w, b), (want.astype(np.float64) + b).astype(np.float32),
                               rtol=1e-6, atol=1e-6)
    # no final norm: the raw last row
    want_raw = (h64[-1] @ w.astype(np.float64)).astype(np.float32)
    np.testing.assert_allclose(orc.logits_last(h, None, 1e-5, w), want_raw, rtol=1e-6, atol=1e-6)


def test_tiny_llama_logits_match_transformers(golden_dir):
    d = np.load(os.path.join(golden_dir, "tiny_llama_logits.npz"))
    m = tinyllama.OracleModel(tinyllama.load(), orc)
    got3 = m.run(d["tokens_t3"])                       # prefill of three tokens
    assert np.abs(got3 - d["logits_t3"]).max() < 2e-6
    got4 = m.run(d["tokens_t4"][3:])                   # one decode step on top of the cache
    assert np.abs(got4 - d["logits_t4"]).max() < 2e-6
    assert orc.greedy(got4) == int(np.argmax(d["logits_t4"]))
