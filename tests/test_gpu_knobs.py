"""The alternative code paths behind the library's tuning variables give the same results: a part of
the GPU parity tests (ragged decode batches, a few new rows, prefill shapes and key splits, whole
blocks) runs again in a child process per setting.  One child at a time."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
SUBSET = ("decode_random_ragged or few_new_rows or prefill_random_shapes or prefill_small_shapes or prefill_key_splits "
          "or every_small_row_count or block_forward_cached_matches or decode_every_length or two_contexts "
          "or single_row_products")

SETTINGS = [
    {"SHAINET_HIP_DECODE_NO_ROTATE": "1"},                      # every workgroup walks its segments from their first tile
    {"SHAINET_HIP_DECODE_WGS": "512"},                          # two workgroups per compute unit
    {"SHAINET_HIP_DECODE_WGS": "37", "SHAINET_HIP_GEMV_WGS": "256"},
    # more workgroups than the chip holds at once: merging workgroups wait for partials of workgroups that start late
    {"SHAINET_HIP_DECODE_WGS": "2048", "SHAINET_HIP_GEMV_WGS": "8192"},
    {"SHAINET_HIP_DECODE_SHARES": "0"},
    {"SHAINET_HIP_DECODE_SHARES": "1200,800,1100,900,1000,1000,700,1300"},
    {"SHAINET_HIP_PREFILL_GROUPS": "1", "SHAINET_HIP_PREFILL_NO_TURNS": "1"},
    {"SHAINET_HIP_PREFILL_GROUPS": "2", "SHAINET_HIP_PREFILL_WGS_PER_CU": "2"},
    {"SHAINET_HIP_NO_FUSED_PREP": "1"},                         # q | k | v product without the prep epilogue
    {"SHAINET_HIP_NO_TRANSPOSED_WEIGHTS": "1"},                 # one-row products over the [in, out] matrices only
    # ... over the transposed ones, several outputs per wavefront; more rows read ahead beside the attention
    {"SHAINET_HIP_GEMVT_WAVES": "300", "SHAINET_HIP_READ_AHEAD_WGS": "700"},
]
# the model with rows of 8192 (its oracle takes 20 s) runs again only where the setting is about its products
WIDE_TOO = ("SHAINET_HIP_GEMVT_WAVES",)


@pytest.mark.parametrize("setting", SETTINGS, ids=[",".join(f"{k[12:]}={v}" for k, v in s.items()) for s in SETTINGS])
def test_parity_subset_with_tuning_variable(setting):
    env = dict(os.environ)
    env.update(setting)
    cmd = [sys.executable, "-u", "-m", "pytest", os.path.join(HERE, "test_gpu_parity.py"), os.path.join(HERE, "test_gpu_model.py"),
           "-x", "-q", "-m", "gpu", "-k", SUBSET if any(k in setting for k in WIDE_TOO) else f"({SUBSET}) and not 8192",
           "--timeout", "120", "--timeout-method", "thread", "-p", "no:cacheprovider"]
    done = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=600)
    tail = (done.stdout + done.stderr)[-3000:]
    assert done.returncode == 0, tail
    assert " passed" in done.stdout and " failed" not in done.stdout, tail
