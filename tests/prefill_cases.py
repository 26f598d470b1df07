"""The prefill launches whose parity the GPU suite checks at full size, each with the kernel
instantiation the library's own planner picks for it: (head_dim, key chunks merged by the
combine kernel?, wavefront groups, row blocks a workgroup takes in turn), and `+ (True,)` for the
instantiations that run a smaller head_dim in padded tiles.

tests/test_gpu_parity.py runs every case against the oracle on all rows with no tuning
variable set and asserts that the planner's choice is the instantiation named here;
tests/test_prefill_plan_coverage.py (no GPU) asserts that the table still matches the planner
and that every shape of the benchmark configurations, and every instantiation the planner can
reach over a sweep of shapes, is named here."""

# name, H, KV, head_dim, QK-norm, cached positions, new rows, (head_dim, split, groups, turns)
CASES = [
    ("llama1b_prefill_t2048", 32, 8, 64, False, 0, 2048, (64, False, 2, 2)),
    ("llama1b_prefill_t3072", 32, 8, 64, False, 0, 3072, (64, False, 2, 3)),
    ("llama1b_prefill_t8192", 32, 8, 64, False, 0, 8192, (64, False, 1, 0)),
    ("llama1b_prefill_t2560", 32, 8, 64, False, 0, 2560, (64, False, 2, 0)),
    ("llama1b_prefill_t1024", 32, 8, 64, False, 0, 1024, (64, True, 2, 0)),
    ("llama1b_chunked_prefill_t512_on_16384", 32, 8, 64, False, 16384, 512, (64, True, 1, 0)),
    ("qwen3_30b_chunked_prefill_t512_on_16384", 32, 4, 128, True, 16384, 512, (128, True, 1, 0)),
    ("qwen3_30b_chunked_prefill_t512_on_4096", 32, 4, 128, True, 4096, 512, (128, True, 2, 0)),
    ("qwen3_8b_prefill_t2048", 32, 8, 128, True, 0, 2048, (128, False, 2, 2)),
    ("qwen3_8b_prefill_t3072", 32, 8, 128, True, 0, 3072, (128, False, 2, 3)),
    ("qwen3_8b_prefill_t2560", 32, 8, 128, True, 0, 2560, (128, False, 2, 0)),
    ("qwen3_8b_prefill_t4096", 32, 8, 128, True, 0, 4096, (128, False, 1, 0)),
    # head dims below the tile layouts (padded tiles): Phi-3-mini's heads at the bench's size, and smaller ones
    ("phi3_hd96_prefill_t2048", 32, 32, 96, False, 0, 2048, (128, False, 2, 2, True)),
    ("hd96_chunked_prefill_t256_on_8192", 16, 4, 96, True, 8192, 256, (128, True, 2, 0, True)),
    ("hd48_prefill_t8192", 16, 8, 48, False, 0, 8192, (64, False, 1, 0, True)),
    ("hd32_prefill_t1024", 32, 8, 32, True, 0, 1024, (64, True, 2, 0, True)),
]

# The prefill shapes of the benchmark configurations (BASELINE.json configs[3] and configs[4](a)):
# (H, KV, head_dim, cached positions, new rows).
BASELINE_PREFILL_SHAPES = [
    (32, 8, 64, 0, 2048),
    (32, 8, 64, 0, 8192),
    (32, 4, 128, 16384, 512),
]


def instantiation(plan):
    """The kernel instantiation of a plan dict from shainet_amd.describe_plan."""
    inst = (plan["head_dim"], plan["key_chunks"] > 1, plan["groups"], plan["turns"])
    return inst + (True,) if plan.get("padded") else inst
