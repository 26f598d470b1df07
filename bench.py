#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A "step" is one layer-step of the hot path over one batch of synthetic rows:
bias/QK-norm/RoPE/append of the new rows plus causal GQA attention over the
device cache, through the C ABI with inputs already resident in HBM.

Headline workload (BASELINE.json configs[2], the one the decode target is quoted
on): Qwen3-8B-shaped decode, 32 Q / 8 KV heads, head_dim 128, QK-norm, theta 1e6,
fp32, batch 16 with cached lengths drawn uniform in [2048, 8192].  The other
configurations are timed as well and reported under "workloads".

Prints ONE JSON line.  `value` is microseconds per layer-step of the headline
workload (whole step: the prep kernel and the split-K decode kernel); `roofline` prices the
split-K decode kernel against HBM, `roofline_prefill` the MFMA prefill kernel
against the fp32 matrix peak; `cpu_baseline` times the CPU oracle (a C
restatement of the reference's single-threaded Crystal path) on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
FP32_MFMA_PEAK_TFLOPS = 157.3
MIN_WARMUP_S = 0.06         # every workload is warmed up for at least this long (and --warmup steps)

# The seeded cached lengths of the headline workload: 16 draws from U[2048, 8192]
def headline_lengths():
    import numpy as np

    return [int(x) for x in np.random.default_rng(2024).integers(2048, 8193, 16)]


# name, H, KV, head_dim, rope theta, QK-norm, cached length per sequence (None = the headline's), new rows per sequence
HEADLINE = ("qwen3_8b_decode_b16_ctx2048-8192", 32, 8, 128, 1e6, True, None, 1)
HEADLINE_MIN_SAMPLES = 100  # event-timed launches of the headline kernel, whatever --steps is
DECODE_WORKLOADS = [
    ("llama1b_decode_b1_ctx1024", 32, 8, 64, 5e5, False, [1024], 1),
    ("llama1b_decode_b1_ctx4096", 32, 8, 64, 5e5, False, [4096], 1),
    ("llama1b_decode_b1_ctx16384", 32, 8, 64, 5e5, False, [16384], 1),
    ("qwen3_30b_decode_b4_ctx32768", 32, 4, 128, 1e6, True, [32768] * 4, 1),
    # the headline shape with every sequence near the top of its length range (1.07 GB per step)
    ("qwen3_8b_decode_b16_ctx8192", 32, 8, 128, 1e6, True, [7936] * 16, 1),
    # not a BASELINE configuration: four new rows per sequence on the headline's caches (they go
    # through the split-K decode kernel as further columns of its tiles: the same bytes, HBM bound)
    ("qwen3_8b_decode_b16_4rows_ctx2048-8192", 32, 8, 128, 1e6, True, None, 4),
    # not BASELINE configurations: head dims between the decode kernel's tile layouts (64, 128 and
    # 256 wide; llama_block.cr:80-89 accepts any head_dim), which run in tiles padded to the next
    # layout, alone and as a batch (Phi-3-mini's heads: 32 of 96, no grouping), and 32 query heads
    # per kv head (more columns than the decode kernel's tile: the MFMA prefill kernel serves it)
    ("hd96_decode_b1_ctx4096", 32, 8, 96, 5e5, False, [4096], 1),
    ("hd256_decode_b1_ctx4096", 16, 4, 256, 5e5, False, [4096], 1),
    ("phi3_hd96_decode_b16_ctx4096", 32, 32, 96, 1e4, False, [4096] * 16, 1),
    ("gemma_hd256_decode_b16_ctx4096", 16, 8, 256, 1e4, False, [4096] * 16, 1),
    ("mqa_g32_hd128_decode_b1_ctx4096", 32, 1, 128, 5e5, False, [4096], 1),
]
# name, H, KV, head_dim, rope theta, QK-norm, cached length per sequence, new rows per sequence
PREFILL_WORKLOADS = [
    ("llama1b_prefill_t2048", 32, 8, 64, 5e5, False, [0], 2048),
    ("llama1b_prefill_t8192", 32, 8, 64, 5e5, False, [0], 8192),
    ("qwen3_30b_chunked_prefill_t512_on_16384", 32, 4, 128, 1e6, True, [16384], 512),
    # not a BASELINE configuration: the headline model's shape (QK-norm, head_dim 128) from an empty cache
    ("qwen3_8b_prefill_t2048", 32, 8, 128, 1e6, True, [0], 2048),
    # not a BASELINE configuration: Phi-3-mini's heads (32 of head_dim 96, no grouping) in tiles padded to 128
    ("phi3_hd96_prefill_t2048", 32, 32, 96, 1e4, False, [0], 2048),
]


def decode_bytes(KV, hd, visible):
    """Algorithmic bytes of one decode layer-step: K and V rows read once per kv head."""
    return sum(2 * KV * hd * 4 * L for L in visible)


def prefill_flops(H, hd, S, T):
    """Unmasked pairs only, 2 FLOP per MAC, QK^T and PV."""
    return 4 * hd * H * (T * S + T * (T + 1) // 2)


class Workload:
    def __init__(self, sa, torch, name, H, KV, hd, theta, norm, lens, T, seed):
        self.sa, self.torch, self.name = sa, torch, name
        self.H, self.KV, self.hd, self.T, self.lens = H, KV, hd, T, list(lens)
        self.B = len(self.lens)
        self.gen = torch.Generator(device="cuda").manual_seed(seed)
        qn = kn = None
        if norm:
            qn = (1 + 0.02 * torch.randn(hd, generator=self.gen, device="cuda")).cpu().numpy()
            kn = (1 + 0.02 * torch.randn(hd, generator=self.gen, device="cuda")).cpu().numpy()
        self.qn, self.kn, self.theta = qn, kn, theta
        self.ctx = sa.AttnContext(H, KV, hd, rope_theta=theta, q_norm=qn, k_norm=kn, eps=1e-6,
                                  max_positions=max(self.lens) + 4096)
        self.cache = None

    def alloc(self, extra_rows):
        torch = self.torch
        self.cache = self.sa.KVCache(self.ctx, self.B, max(self.lens) + extra_rows)
        for s, L in enumerate(self.lens):
            if L:
                k = torch.randn((self.KV, L, self.hd), generator=self.gen, device="cuda")
                v = torch.randn((self.KV, L, self.hd), generator=self.gen, device="cuda")
                torch.cuda.synchronize()
                self.cache.fill(s, k, v)
        torch.cuda.synchronize()

    def rows(self, n_steps):
        torch = self.torch
        R = self.B * self.T
        q = torch.randn((n_steps, R, self.H * self.hd), generator=self.gen, device="cuda")
        k = torch.randn((n_steps, R, self.KV * self.hd), generator=self.gen, device="cuda")
        v = torch.randn((n_steps, R, self.KV * self.hd), generator=self.gen, device="cuda")
        out = torch.empty((R, self.H * self.hd), device="cuda")
        torch.cuda.synchronize()
        return q, k, v, out

    def run_decode(self, steps, warmup, min_samples=0):
        """Consecutive decode steps (self.T new rows per sequence) appending to the cache; the kernel is
        then timed with events over max(steps, min_samples) further steps."""
        torch, ctx, T = self.torch, self.ctx, self.T
        prof_steps = max(steps, min_samples)
        self.alloc(T * (steps + prof_steps) + 1)
        q, k, v, out = self.rows(min(2 * steps, 64))
        nt = [T] * self.B
        n = q.shape[0]
        # the timed loop holds nothing but the C call: the row sets are bound beforehand
        calls = [ctx.prepared(self.cache, q[i], k[i], v[i], nt, out) for i in range(n)]

        def step(i):
            calls[i % n]()

        # Warm-up: at least `warmup` steps and at least MIN_WARMUP_S of them, in runs of `steps`
        # steps after each of which the caches are cut back to their starting lengths (the timed
        # steps then see exactly the lengths of the workload's name).  A handful of 0.1 ms
        # launches after an idle stretch run on a device that has not reached the clocks and power
        # state it then holds: measured that way, the same kernel is 3 to 15 % slower.
        t_w, n_w = time.perf_counter(), 0
        while n_w < warmup or time.perf_counter() - t_w < MIN_WARMUP_S:
            for i in range(steps):
                step(i)
            n_w += steps
            ctx.sync()
            for s, L in enumerate(self.lens):
                self.cache.truncate(s, L)
        warm_ms = (time.perf_counter() - t_w) * 1e3
        # what a call costs the host: a few calls into an empty queue, not waited for
        n_host = min(16, steps)
        t0 = time.perf_counter()
        for i in range(n_host):
            step(i)
        host_us = (time.perf_counter() - t0) / n_host * 1e6
        ctx.sync()
        for s, L in enumerate(self.lens):
            self.cache.truncate(s, L)
        t0 = time.perf_counter()
        for i in range(steps):
            step(i)
        ctx.sync()
        wall = time.perf_counter() - t0
        # second pass with HIP events around the split-K kernel only
        ctx.profile(True)
        for i in range(prof_steps):
            step(steps + i)
        samples = ctx.profile_samples(prof_steps + 8)
        k_ms, launches = float(samples.sum()), len(samples)
        ctx.profile(False)
        vis_wall = [[L + T * (i + 1) for L in self.lens] for i in range(steps)]
        vis_prof = [[L + T * (steps + i + 1) for L in self.lens] for i in range(prof_steps)]
        b_wall = sum(decode_bytes(self.KV, self.hd, v_) for v_ in vis_wall) / steps
        b_prof = sum(decode_bytes(self.KV, self.hd, v_) for v_ in vis_prof) / prof_steps
        us = wall / steps * 1e6
        kus = k_ms / max(launches, 1) * 1e3
        import numpy as np

        pct = [float(x) * 1e3 for x in np.percentile(samples, (10, 50, 90))] if launches else [0.0] * 3
        return {"workload": self.name, "us_per_step": us, "kernel_us": kus, "kernel_us_p10": pct[0],
                "kernel_us_p50": pct[1], "kernel_us_p90": pct[2], "launches": launches,
                "warmup_launches": n_w, "warmup_ms": warm_ms, "host_us_per_call": host_us,
                "bytes_per_step": b_wall, "step_gbps": b_wall / us / 1e3, "kernel_gbps": b_prof / kus / 1e3,
                "kernel_bytes": b_prof, "frac_of_hbm_peak": b_prof / kus / 1e3 / HBM_PEAK_GBPS}

    def run_prefill(self, steps, warmup):
        """T new rows on top of S cached ones; the cache is truncated back between steps."""
        torch, ctx = self.torch, self.ctx
        self.alloc(self.T + 1)
        q, k, v, out = self.rows(1)
        nt = [self.T] * self.B

        def step():
            for s, L in enumerate(self.lens):
                self.cache.truncate(s, L)
            ctx.forward(self.cache, q[0], k[0], v[0], nt, out=out)

        # at least `warmup` launches and at least 60 ms of them: the device reaches the clock it
        # then holds only after some tens of milliseconds of matrix work (the first launches of
        # T = 2048 take 183 us, later ones 165 us)
        t_w, n_w = time.perf_counter(), 0
        while n_w < warmup or time.perf_counter() - t_w < MIN_WARMUP_S:
            step()
            n_w += 1
            if n_w % 4 == 0:
                ctx.sync()
        ctx.sync()
        warm_ms = (time.perf_counter() - t_w) * 1e3
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        ctx.sync()
        wall = time.perf_counter() - t0
        ctx.profile(True)
        for _ in range(steps):
            step()
        k_ms, launches = ctx.profile_read()
        ctx.profile(False)
        fl = sum(prefill_flops(self.H, self.hd, L, self.T) for L in self.lens)
        us = wall / steps * 1e6
        kus = k_ms / max(launches, 1) * 1e3
        return {"workload": self.name, "us_per_step": us, "kernel_us": kus, "launches": launches,
                "warmup_launches": n_w, "warmup_ms": warm_ms, "flops": fl,
                "step_tflops": fl / us / 1e6, "kernel_tflops": fl / kus / 1e6,
                "frac_of_mfma_peak": fl / kus / 1e6 / FP32_MFMA_PEAK_TFLOPS}

    def close(self):
        if self.cache is not None:
            self.cache.close()
        self.ctx.close()
        self.torch.cuda.empty_cache()


def cpu_baseline(w, reps):
    """The oracle (C restatement of the reference's scalar CPU path), one thread, on one
    decode layer-step of the headline workload: same shapes, same cache contents."""
    import numpy as np

    from oracle import oracle as orc

    blocks = []
    for s in range(w.B):
        b = orc.Block(w.H * w.hd, w.H, w.KV, w.hd, eps=1e-6, rope_theta=w.theta)
        if w.qn is not None:
            b.set_qk_norm(w.qn, w.kn)
        n = w.cache.len(s)
        kv = [w.cache.read(s, c, 0, n) for c in range(w.KV)]
        b.fill_cache(np.stack([x[0] for x in kv]), np.stack([x[1] for x in kv]))
        blocks.append(b)
    r = np.random.default_rng(0)
    times = []
    for _ in range(reps):
        rows = [tuple(r.standard_normal((1, n_ * w.hd)).astype(np.float32) for n_ in (w.H, w.KV, w.KV))
                for _ in blocks]
        t0 = time.perf_counter()
        for b, (q, k, v) in zip(blocks, rows):
            b.attention_cached_qkv(q, k, v, threads=1)
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2] * 1e6


def cpu_baseline_prefill(reps=3):
    """The oracle, one thread, on a bounded part of the 2048-row causal prefill of the Llama-3.2-1B
    shape: its last 256 rows on top of the 1792 rows before them, extrapolated to the whole prefill
    by the multiply-adds of the head loop (the scalar path's time is proportional to them)."""
    import numpy as np

    from oracle import oracle as orc

    H, KV, hd, T, n_rows = 32, 8, 64, 2048, 256
    r = np.random.default_rng(4)
    b = orc.Block(H * hd, H, KV, hd, rope_theta=5e5)
    b.fill_cache(r.standard_normal((KV, T - n_rows, hd)).astype(np.float32),
                 r.standard_normal((KV, T - n_rows, hd)).astype(np.float32))
    q, k, v = (r.standard_normal((n_rows, n_ * hd)).astype(np.float32) for n_ in (H, KV, KV))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        b.attention_cached_qkv(q, k, v, threads=1)
        times.append(time.perf_counter() - t0)
        b.clear_cache()
        b.fill_cache(r.standard_normal((KV, T - n_rows, hd)).astype(np.float32),
                     r.standard_normal((KV, T - n_rows, hd)).astype(np.float32))
    times.sort()
    whole = T * (T + 1) // 2
    part = whole - (T - n_rows) * (T - n_rows + 1) // 2
    return {"value": round(times[len(times) // 2] * 1e6 * whole / part, 1), "unit": "us/prefill", "cores": 1,
            "kind": "port", "workload": "llama1b_prefill_t2048",
            "sample": "the last %d of the 2048 rows (%.1f %% of the head loop's multiply-adds), median of %d, "
                      "scaled to the whole prefill; C restatement of the reference's single-threaded Crystal "
                      "path" % (n_rows, 100.0 * part / whole, reps)}


def recorded_step(sa, torch, steps):
    """Batch-1 decode at 4096 cached positions (Llama-3.2-1B shape) three ways, wall time per step of a
    loop that is not waited for until its end: the host-planned call, shainet_attn_decode_step called
    eagerly, and one such step recorded into a graph on the context's stream and replayed."""
    H, KV, hd, L = 32, 8, 64, 4096
    w = Workload(sa, torch, "llama1b_decode_b1_ctx4096_recorded_step", H, KV, hd, 5e5, False, [L], 1, 9)
    n_warm = 200
    w.alloc(4 * (steps + n_warm) + 8)
    q, k, v, out = w.rows(1)
    ctx, cache = w.ctx, w.cache
    side = torch.cuda.Stream()
    ctx.set_stream(side.cuda_stream)
    res = {"workload": w.name}

    def timed(fn, sync):
        for _ in range(n_warm):
            fn()
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        sync()
        return (time.perf_counter() - t0) / steps * 1e6

    res["host_planned_us_per_step"] = timed(ctx.prepared(cache, q[0], k[0], v[0], [1], out), ctx.sync)
    cache.truncate(0, L)
    cache.lengths_to_device()
    res["eager_step_us_per_step"] = timed(lambda: ctx.decode_step(cache, q[0], k[0], v[0], out), ctx.sync)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ctx.decode_step(cache, q[0], k[0], v[0], out)
    with torch.cuda.stream(side):
        res["replayed_graph_us_per_step"] = timed(graph.replay, side.synchronize)
    cache.lengths_from_device()
    res["cached_positions_at_end"] = cache.len(0)
    del graph
    w.close()
    return res


def layer_decode(sa, np, steps):
    """BASELINE configs[0] on the device: one Llama-3.2-1B-shaped attention layer (hidden 2048, 32 Q /
    8 KV heads, head_dim 64), projections included, 512 cached positions, one new row per call, host
    pointers in and out (so the time includes the PCIe copies and the synchronisation)."""
    r = np.random.default_rng(1)
    d, H, KV, hd = 2048, 32, 8, 64
    blk = sa.LlamaBlock(d, H, rope_theta=5e5, num_kv_heads=KV)
    blk.set_weights(*[(0.02 * r.standard_normal(sh)).astype(np.float32)
                      for sh in ((d, H * hd), (d, KV * hd), (d, KV * hd), (H * hd, d))])
    blk.attention_cached(r.standard_normal((512, d)).astype(np.float32))
    xs = [r.standard_normal((1, d)).astype(np.float32) for _ in range(8)]
    for x in xs[:4]:
        blk.attention_cached(x)
    t0 = time.perf_counter()
    for i in range(steps):
        blk.attention_cached(xs[i % 8])
    us = (time.perf_counter() - t0) / steps * 1e6
    blk.close()
    return {"workload": "llama1b_layer_decode_ctx512", "us_per_step": us, "host_pointers": True,
            "weight_bytes_per_step": 4 * (2 * d * H * hd + 2 * d * KV * hd)}


def model_decode(sa, np, steps, ctx_len=512):
    """Greedy decode of a Llama-3.2-1B-shaped model (16 blocks, hidden 2048, 32 Q / 8 KV heads,
    head_dim 64, ff 8192, vocab 128256, fp32, seeded random weights) with everything on the device:
    token id in, next token id out.  A token reads every weight once, so the yardstick is weight
    bytes per token over HBM bandwidth."""
    r = np.random.default_rng(11)
    V, d, L, H, KV, hd, ff = 128256, 2048, 16, 32, 8, 64, 8192
    m = sa.LlamaModel(V, d, L, H, ff, eps=1e-5, rope_theta=5e5, num_kv_heads=KV)
    table = (0.02 * r.standard_normal((V, d), dtype=np.float32))
    m.set_embedding(table)
    m.set_lm_head(table.reshape(d, V))  # same seeded values read as [d, vocab]
    m.set_final_norm(np.ones(d, np.float32))
    del table
    # one block's worth of seeded weights, uploaded into every block (timing does not depend on the values)
    ws = [(0.02 * r.standard_normal(sh, dtype=np.float32)) for sh in
          ((d, H * hd), (d, KV * hd), (d, KV * hd), (H * hd, d), (d, ff), (d, ff), (ff, d))]
    gammas = [(1 + 0.1 * r.standard_normal(d)).astype(np.float32) for _ in range(2)]
    for b in m.blocks:
        b.set_weights(*ws[:4])
        b.set_ffn(*ws[4:])
        b.set_norms(*gammas)  # (a Llama block has both norm weights)
    del ws
    weight_bytes = 4 * (L * (2 * d * H * hd + 2 * d * KV * hd + 3 * d * ff) + d * V)
    # prefill of the context: more than 16 rows go through the library's own MFMA product and the MFMA attention kernel
    prompt = list(r.integers(0, V, ctx_len))
    m.run(prompt, want_logits=False)
    m.sync()
    pf = []
    for _ in range(3):
        m.clear_cache()
        t0 = time.perf_counter()
        m.run(prompt, want_logits=False)
        m.sync()
        pf.append(time.perf_counter() - t0)
    prefill_s = sorted(pf)[1]
    tok = sa.Sampler.greedy(m)
    for _ in range(5):
        m.run([tok], want_logits=False)
        tok = sa.Sampler.greedy(m)
    m.run([tok], want_logits=False)
    m.generate_greedy(16)
    t0 = time.perf_counter()
    n = len(m.generate_greedy(steps))
    dt = (time.perf_counter() - t0) / max(n, 1)
    # the same steps as one launch per token (the opt-in decode mode), from the same cached context
    m.set_decode_mode(m.DECODE_PERSISTENT)
    m.clear_cache()
    m.run(prompt, want_logits=False)
    m.generate_greedy(16)
    t0 = time.perf_counter()
    n1 = len(m.generate_greedy(steps))
    dt1 = (time.perf_counter() - t0) / max(n1, 1)
    m.close()
    return {"workload": "llama1b_model_greedy_decode_ctx%d" % ctx_len, "us_per_token": dt * 1e6,
            "us_per_token_single_launch_step": dt1 * 1e6,
            "tokens_per_s": 1.0 / dt, "weight_bytes_per_token": weight_bytes,
            "weight_gbps": weight_bytes / dt / 1e9, "frac_of_hbm_peak": weight_bytes / dt / 1e9 / HBM_PEAK_GBPS,
            "prefill_tokens": ctx_len, "prefill_ms": prefill_s * 1e3, "prefill_tokens_per_s": ctx_len / prefill_s,
            "prefill_tflops": 2.0 * (weight_bytes / 4 - d * V) * ctx_len / prefill_s / 1e12}


# The kernels the two roofline objects of the bench line price, and the workloads they are priced on.
ROOFLINE_KERNELS = {
    "roofline": ("decode_splitk_kernel<128, 4, false, false, false>", "qwen3_8b_decode_b16_ctx2048-8192"),
    "roofline_prefill": ("prefill_turns_kernel<64, 2, false>", "llama1b_prefill_t2048"),
}


def profile_file(kernel, workload):
    """Name of the rocprofv3 summary under profiles/ that covers a kernel on a workload."""
    import re

    return re.sub(r"[^A-Za-z0-9]+", "_", kernel).strip("_") + "_" + workload + ".md"


def load_traffic(kernel, workload, bytes_per_launch=None):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), kept as a
    committed summary; None until measured.  The decode launches of the counter runs are the first
    few steps, those timed here come later and see longer caches: the measured bytes are scaled by
    the ratio of the algorithmic bytes of the two sets of launches."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            t = json.load(f).get(kernel, {}).get(workload)
    except (OSError, ValueError):
        return None
    if isinstance(t, dict):
        if not bytes_per_launch:
            return t["bytes"]
        return int(t["bytes"] * (bytes_per_launch / t["algorithmic_bytes_of_those_launches"]))
    return t


def yardsticks(torch, reps=5):
    """What the device sustains on this box under the simplest possible load of each kind: a
    plain coalesced read of 1 GiB (HBM) and a loop of nothing but fp32 MFMAs (matrix cores at
    the clock the device holds under that load).  Reported next to the published peaks."""
    from shainet_amd import hip

    stream = torch.cuda.current_stream().cuda_stream
    n = 256 * 1024 * 1024
    a = torch.empty(n, device="cuda").normal_()
    sink = torch.zeros(256 * 512, device="cuda")
    out = {}
    flops = [0]

    def mfma():
        flops[0] = hip.mfma_f32_loop(sink, 4096, 256, stream)

    for key, fn, amount in (("stream_read_gbps", lambda: hip.stream_read(a, sink, 768, stream), lambda: 4 * n / 1e3),
                            ("mfma_f32_loop_tflops", mfma, lambda: flops[0] / 1e6)):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out[key] = round(amount() / (e0.elapsed_time(e1) / reps * 1e3), 1)
    del a
    # what a launch costs with no work in it, by the kernels' own clocks: one empty kernel of 256
    # workgroups, and two of them one after the other on one stream (one kernel boundary: the floor
    # under a step that is a prep kernel followed by an attention kernel)
    out["launch_us"] = round(hip.launch_latency(1, 200, 256, stream), 2)
    out["launch_pair_us"] = round(hip.launch_latency(2, 200, 256, stream), 2)
    out["launch_chain8_us"] = round(hip.launch_latency(8, 100, 256, stream), 2)
    return out


def calibrate(torch, sa, reps):
    """Plain copy and read kernels over 1 GiB: the bandwidth a perfectly coalesced stream
    reaches here, and (under rocprofv3 --pmc) what FETCH_SIZE / WRITE_SIZE read per byte."""
    from shainet_amd import hip

    n = 256 * 1024 * 1024
    a = torch.randn(n, device="cuda")
    b = torch.empty_like(a)
    sink = torch.zeros(8192, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    res = {"bytes_per_launch": {"copy_f32x4_kernel": {"read": 4 * n, "write": 4 * n},
                                "read_f32x4_kernel": {"read": 4 * n, "write": 4 * 768}}}
    for name, fn, moved in (("copy_f32x4_kernel", lambda: hip.stream_copy(a, b, 4096, stream), 8 * n),
                            ("read_f32x4_kernel", lambda: hip.stream_read(a, sink, 768, stream), 4 * n)):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        res[name + "_gbps"] = round(moved / (e0.elapsed_time(e1) / reps) / 1e6, 1)
    print(json.dumps({"calibration": res}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", default="", help="comma-separated workload names (default: all)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibrate", action="store_true",
                    help="run only the plain copy/read kernels of known size (counter and bandwidth yardstick)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is built and measured on one GPU only (sequences, kv heads and context "
              "slices shard without communication inside attention); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import shainet_amd as sa

    if not sa.HIP.fully_available():
        print("bench.py: no gfx950 device or libshainet_hip_kernels.so missing (no CPU fallback)", file=sys.stderr)
        sys.exit(1)

    if args.calibrate:
        calibrate(torch, sa, 10)
        return

    K, W = args.steps, args.warmup
    only = set(filter(None, args.only.split(",")))
    lens3 = headline_lengths()
    results = {}

    def want(name):
        return not only or name in only

    # headline: configs[2]
    name, H, KV, hd, th, norm, _, T1 = HEADLINE
    head = Workload(sa, torch, name, H, KV, hd, th, norm, lens3, T1, 3)
    results[head.name] = head.run_decode(K, W, HEADLINE_MIN_SAMPLES)
    cpu = None
    if not args.no_cpu:
        cpu_us = cpu_baseline(head, 21)
        cpu = {"value": cpu_us, "unit": "us/layer-step", "cores": 1, "kind": "port",
               "sample": "one decode layer-step of the headline workload (16 sequences, same cache), "
                         "median of 21, C restatement of the reference's single-threaded Crystal path",
               "host_cores_visible": os.cpu_count()}
    head.close()

    for name, H, KV, hd, th, norm, lens, T in DECODE_WORKLOADS:
        if want(name):
            lens = lens3 if lens is None else lens
            w = Workload(sa, torch, name, H, KV, hd, th, norm, lens, T, 5)
            results[name] = w.run_decode(K if len(lens) < 16 else max(20, K // 2), W)
            w.close()
    fewer = {"llama1b_prefill_t2048": K, "llama1b_prefill_t8192": max(5, K // 20),
             "qwen3_30b_chunked_prefill_t512_on_16384": max(5, K // 10), "qwen3_8b_prefill_t2048": max(5, K // 2),
             "phi3_hd96_prefill_t2048": max(5, K // 4)}
    for name, H, KV, hd, th, norm, lens, T in PREFILL_WORKLOADS:
        if want(name):
            w = Workload(sa, torch, name, H, KV, hd, th, norm, lens3 if lens is None else lens, T, 7)
            results[name] = w.run_prefill(fewer[name], max(2, W // 4))
            w.close()

    if want("llama1b_layer_decode_ctx512"):
        results["llama1b_layer_decode_ctx512"] = layer_decode(sa, np, max(20, K // 4))

    if want("llama1b_model_greedy_decode_ctx512"):
        results["llama1b_model_greedy_decode_ctx512"] = model_decode(sa, np, max(20, K // 4))

    if want("llama1b_decode_b1_ctx4096_recorded_step"):
        results["llama1b_decode_b1_ctx4096_recorded_step"] = recorded_step(sa, torch, max(100, K))

    h = results[head.name]
    line = {
        "metric": "decode attn us/layer-step (achieved HBM GB/s and prefill TFLOP/s alongside)",
        "value": round(h["us_per_step"], 3),
        "unit": "us/layer-step",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(h["us_per_step"] / 1e3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": head.name, "num_heads": 32, "num_kv_heads": 8, "head_dim": 128, "qk_norm": True,
                   "rope_theta": 1e6, "batch": 16, "cached_lengths": lens3, "new_rows_per_sequence": 1},
        "hbm_gbps": round(h["step_gbps"], 1),
        "roofline": {"bound": "hbm", "kernel": ROOFLINE_KERNELS["roofline"][0], "achieved": round(h["kernel_gbps"], 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(h["kernel_gbps"] / HBM_PEAK_GBPS, 4),
                     "kernel_us": round(h["kernel_us"], 2), "kernel_samples": h["launches"],
                     "kernel_us_p10_p50_p90": [round(h["kernel_us_p10"], 2),
                                                                                      round(h["kernel_us_p50"], 2),
                                                                                      round(h["kernel_us_p90"], 2)],
                     "bytes_per_launch": int(h["kernel_bytes"]),
                     "warmup_ms": round(h["warmup_ms"], 1), "warmup_launches": h["warmup_launches"],
                     "profile": "profiles/" + profile_file(*ROOFLINE_KERNELS["roofline"]),
                     "traffic": load_traffic(ROOFLINE_KERNELS["roofline"][0], head.name, h["kernel_bytes"])},
        "cpu_baseline": cpu,
        "workloads": {k_: {kk: (round(vv, 3) if isinstance(vv, float) else vv) for kk, vv in r.items()
                           if kk != "workload"} for k_, r in results.items()},
    }
    p = results.get("llama1b_prefill_t2048")
    if p:
        line["prefill_tflops"] = round(p["step_tflops"], 2)
        line["roofline_prefill"] = {"bound": "mfma", "kernel": ROOFLINE_KERNELS["roofline_prefill"][0],
                                    "workload": p["workload"],
                                    "achieved": round(p["kernel_tflops"], 2), "peak": FP32_MFMA_PEAK_TFLOPS,
                                    "unit": "TFLOP/s", "frac": round(p["kernel_tflops"] / FP32_MFMA_PEAK_TFLOPS, 4),
                                    "kernel_us": round(p["kernel_us"], 2), "flops_per_launch": p["flops"],
                                    "warmup_ms": round(p["warmup_ms"], 1), "warmup_launches": p["warmup_launches"],
                                    "profile": "profiles/" + profile_file(*ROOFLINE_KERNELS["roofline_prefill"]),
                                    "traffic": load_traffic(ROOFLINE_KERNELS["roofline_prefill"][0], p["workload"])}
    if p and not args.no_cpu:
        line["cpu_baseline_prefill"] = cpu_baseline_prefill()
    yard = yardsticks(torch)
    line["yardsticks"] = yard
    # every HBM-bound figure also as a fraction of what a plain read of 1 GiB reaches on this box
    for r in list(line["workloads"].values()) + [line["roofline"]]:
        f = r.get("frac_of_hbm_peak", r.get("frac") if r is line["roofline"] else None)
        if f is not None:
            r["frac_of_stream_yardstick"] = round(f * HBM_PEAK_GBPS / yard["stream_read_gbps"], 4)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
