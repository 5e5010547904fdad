#!/usr/bin/env python3
"""Headline benchmark: shared-prefix decode attention, tokens/s/layer, on one MI355X.

Workload = BASELINE config 2: fp16, 32 heads x 128, batch 64 decode queries that
share one 4096-token prefix, per-request suffix lengths U[16,512], K/V in a flat
1M-slot token pool at randomly permuted slots, seed 1.  One step = one pass of
the hot path (prefix phase on MFMA + suffix phase + LSE merge) for one layer.
Steps rotate over several layers' KV sets (distinct slots of the same pool), as a
model's layers do, so the KV of a step is not cache-resident from the previous
step; the single-set (cache-warm) rate is reported beside it.

Prints ONE JSON line (see the keys at the bottom).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16

# HBM traffic per launch of this workload's kernels and the matrix-pipe counters of the prefix kernel come from
# rocprofv3 --pmc passes over this file (the commands stand at the top of each profiles/*.txt); their figures are
# kept in profiles/counters.json together with the commit they were taken at, and are read from there -- nothing
# is typed in.
COUNTERS_JSON = os.path.join(ROOT, "profiles", "counters.json")


def measured_counters():
    try:
        with open(COUNTERS_JSON) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


class HipEvents:
    """hipEvent_t handles through the HIP runtime torch already loaded."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def create(self, n):
        evs = (ctypes.c_void_p * n)()
        for i in range(n):
            e = ctypes.c_void_p()
            assert self.hip.hipEventCreate(ctypes.byref(e)) == 0
            evs[i] = e
        return evs

    def elapsed_ms(self, a, b):
        """None when the pair was never recorded (the call did not launch that kernel)."""
        out = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(out), a, b)
        if rc != 0:
            self.hip.hipGetLastError()  # the failed query must not surface in a later, unrelated call
            return None
        return out.value

    def destroy(self, evs):
        for e in evs:
            self.hip.hipEventDestroy(e)


def cpu_baseline(case, sample_reqs: int, budget_s: float = 12.0):
    """The oracle's one-shot decode attention (gather by slot + softmax attention, the
    reference's token-granular algorithm) timed on the host cores: passes over the sampled
    requests are repeated until about ``budget_s`` seconds of CPU work are done."""
    import torch

    from oracle.ref_ops import ref_decode_attention

    host_cores = os.cpu_count() or 1
    cores = min(host_cores, 16)  # the GPU box's CPU share for one GPU
    torch.set_num_threads(cores)
    lists = case.full_lists()[:sample_reqs]
    q = case.q[:sample_reqs]
    ref_decode_attention(q[:1], case.k_rows, case.v_rows, lists[:1])  # warm-up
    times = []
    t_begin = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_begin < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        ref_decode_attention(q, case.k_rows, case.v_rows, lists)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    return {
        "value": sample_reqs / t,
        "unit": "tokens/s/layer",
        "cores": cores,
        "host_cores": host_cores,
        "kind": "port",
        "sample": f"{sample_reqs} of {case.num_reqs} requests of the same workload (fp32 math on fp16-rounded inputs), "
                  f"median of {len(times)} passes ({time.perf_counter() - t_begin:.1f} s of host work)",
    }


def _time_gpu(torch, fn, iters=20, warmup=3, inner=10):
    """Median over `iters` samples of the time per call when `inner` calls are queued back to back between two
    events (the queue stays full, so host launch latency is not in the figure); also p10 and p90."""
    for _ in range(warmup):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ts = []
    for _ in range(iters):
        a.record()
        for _ in range(inner):
            fn()
        b.record()
        b.synchronize()
        ts.append(a.elapsed_time(b) * 1e-3 / inner)
    ts.sort()
    return ts[len(ts) // 2]


class _Rotor:
    def __init__(self, n):
        self.n, self.i = n, 0

    def next(self):
        self.i = (self.i + 1) % self.n
        return self.i


def extras(torch, dev):
    """The other configurations' kernels, each against its own roofline (median launch time, torch events
    on the launch stream).  Data is synthetic of the configured shapes; parity for these shapes is in tests/."""
    from parrotserve_amd import kernels, synth

    out = {}
    H, D = 32, 128
    # --- config 3: token move, 65,536 random rows of 8 KB inside a 4M-slot pool (one tensor) ---------------
    pool = 1 << 22
    kc = torch.empty((pool, H, D), dtype=torch.float16, device=dev)
    kc.normal_()
    src, dst = synth.config3_move()
    src, dst = src.to(dev), dst.to(dev)
    t = _time_gpu(torch, lambda: kernels.discontinuous_move_tokens(kc, kc, src, dst))
    nbytes = 2 * src.numel() * H * D * 2
    out["c3_token_move"] = {"rows": src.numel(), "row_bytes": H * D * 2, "us": t * 1e6, "GB/s": nbytes / t / 1e9,
                            "frac_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": nbytes}
    # the same kernel as a plain copy of as many rows in order (what a read + write stream of this size reaches on
    # this device: the ceiling a move of scattered rows can approach)
    ident = torch.arange(src.numel(), device=dev)
    half = pool // 2
    t_copy = _time_gpu(torch, lambda: kernels.discontinuous_move_tokens(kc[:half], kc[half:], ident, ident))
    out["c3_token_move"]["same_rows_in_order_us"] = t_copy * 1e6
    out["c3_token_move"]["same_rows_in_order_frac_hbm"] = nbytes / t_copy / 1e9 / HBM_PEAK_GBS
    # one side scattered, the other in order: which side of a scattered move costs what
    t_sr = _time_gpu(torch, lambda: kernels.discontinuous_move_tokens(kc, kc[half:], src, ident))
    t_dr = _time_gpu(torch, lambda: kernels.discontinuous_move_tokens(kc[:half], kc, ident, dst))
    out["c3_token_move"]["scattered_reads_ordered_writes_us"] = t_sr * 1e6
    out["c3_token_move"]["ordered_reads_scattered_writes_us"] = t_dr * 1e6
    # --- the same 65,536 rows gathered out of the block-structured layouts (block 16, x 8) of a 4M-slot cache:
    # whole blocks in random order (a context that owns its blocks) and fully random slots -----------------------
    bs, x = 16, 8
    gen = torch.Generator().manual_seed(3)
    blocks = torch.randperm(pool // bs, generator=gen)[: src.numel() // bs]
    runs = (blocks[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1).to(dev)
    dest = torch.empty((src.numel(), H, D), dtype=torch.float16, device=dev)
    rows = torch.arange(src.numel(), device=dev)
    for name, cache, fn in (("k", kc.view(pool // bs, H, D // x, bs, x), kernels.move_tokens_from_blocked_k_cache),
                            ("v", kc.view(pool // bs, H, D, bs), kernels.move_tokens_from_blocked_v_cache)):
        for pat, slots in (("block_runs", runs), ("random_slots", src)):
            t = _time_gpu(torch, lambda: fn(cache, dest, slots, rows))
            out[f"c3_blocked_{name}_gather_{pat}"] = {"rows": src.numel(), "us": t * 1e6, "GB/s": nbytes / t / 1e9,
                                                      "frac_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS,
                                                      "algorithmic_bytes": nbytes}
    del dest
    # --- config 3: ragged non-shared decode, B 256, ctx log-uniform[128, 8192] ------------------------------
    vc = torch.empty_like(kc)
    vc.normal_()
    case = synth.config3(batch=256, pool_slots=pool)
    lens = [l.numel() for l in case.suffix_lists]
    tabs = kernels.DecodeTables.build([], [], case.pool_lists(case.suffix_lists), dev)
    q = case.q.to(dev)
    o = torch.empty_like(q)
    t = _time_gpu(torch, lambda: kernels.decode_attention(q, kc, vc, tabs, out=o), iters=10)
    nbytes = 2 * sum(lens) * H * D * 2
    out["c3_ragged_decode"] = {"batch": 256, "sum_ctx": sum(lens), "ms": t * 1e3, "GB/s": nbytes / t / 1e9,
                               "frac_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": nbytes,
                               "tokens/s/layer": 256 / t}
    del kc, vc, tabs
    # --- config 4: RoPE + append + prefill with parent context, bf16 40x128 ---------------------------------
    c4 = synth.config4()
    T, H4, _ = c4.q.shape
    kc4, vc4 = synth.pool_to_device(c4.k_rows, c4.v_rows, c4.used_slots, c4.pool_slots, dev)
    cache = kernels_cos_sin(torch, int(c4.positions.max()) + 1, D, c4.theta, torch.bfloat16, dev)
    # RoPE and append rotate over 4 projections' outputs (4 x 289 MB) so that their inputs come from HBM,
    # not from the 256 MB memory-side cache
    qkvs = [torch.randn((T, 3 * H4 * D), device=dev, dtype=torch.bfloat16) for _ in range(4)]
    rot = _Rotor(len(qkvs))
    q4, k4, v4 = qkvs[0].chunk(3, dim=-1)
    pos = c4.positions.to(dev)

    def rope_step():
        qi, ki, _ = qkvs[rot.next()].chunk(3, dim=-1)
        kernels.vllm_rotary_emb(pos, qi, ki, cache, D)

    t_rope = _time_gpu(torch, rope_step)
    rope_bytes = 2 * T * 2 * H4 * D * 2 + T * D * 2
    # the same kernel on q and k rows that lie side by side without the v third between them, and the library's
    # element-wise in-place kernel over the same bytes: what an in-place pass of this size reaches on this device
    qks = [torch.randn((T, 2 * H4 * D), device=dev, dtype=torch.bfloat16) for _ in range(6)]
    rot2 = _Rotor(len(qks))

    def rope_dense_step():
        qi, ki = qks[rot2.next()].chunk(2, dim=-1)
        kernels.vllm_rotary_emb(pos, qi, ki, cache, D)

    t_rope_dense = _time_gpu(torch, rope_dense_step)
    t_rmw = _time_gpu(torch, lambda: qks[rot2.next()].mul_(1.0001))
    del qks
    new_slots = torch.cat([c4.used_slots[n] for n in c4.new_lists]).to(torch.int32).to(dev)
    k3, v3 = k4.view(T, H4, D), v4.view(T, H4, D)

    def append_step():
        _, ki, vi = qkvs[rot.next()].chunk(3, dim=-1)
        kernels.vllm_reshape_and_cache(ki.view(T, H4, D), vi.view(T, H4, D), kc4, vc4, new_slots)

    t_app = _time_gpu(torch, append_step)

    def fused_step():
        qi, ki, vi = qkvs[rot.next()].chunk(3, dim=-1)
        kernels.rope_and_cache(pos, qi, ki, vi, cache, D, kc4, vc4, new_slots)

    t_fused = _time_gpu(torch, fused_step)

    def fused_cache_only_step():  # the layer's form: attention reads K from the cache, k is not written back
        qi, ki, vi = qkvs[rot.next()].chunk(3, dim=-1)
        kernels.rope_and_cache(pos, qi, ki, vi, cache, D, kc4, vc4, new_slots, key_in_place=False)

    t_fused_co = _time_gpu(torch, fused_cache_only_step)
    ctx = [c4.used_slots[torch.cat([p, n])].tolist() for p, n in zip(c4.parent_lists, c4.new_lists)]
    ptab = kernels.PrefillTables.build(c4.q_lens, ctx, dev)
    qc = q4.reshape(T, H4, D).contiguous()
    o4 = torch.empty_like(qc)
    t_pre = _time_gpu(torch, lambda: kernels.prefill_attention(qc, kc4, vc4, ptab, out=o4), iters=10)
    par = c4.parent_lists[0].numel()
    flops = 4 * H4 * D * sum(n * par + n * (n + 1) // 2 for n in c4.q_lens)
    out["c4_rope"] = {"tokens": T, "us": t_rope * 1e6, "GB/s": rope_bytes / t_rope / 1e9,
                      "frac_hbm": rope_bytes / t_rope / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": rope_bytes,
                      "q_k_rows_without_v_between_us": t_rope_dense * 1e6,
                      "q_k_rows_without_v_between_frac_hbm": rope_bytes / t_rope_dense / 1e9 / HBM_PEAK_GBS,
                      "torch_mul_in_place_same_bytes_us": t_rmw * 1e6}
    app_bytes = 2 * 2 * T * H4 * D * 2
    out["c4_kv_append"] = {"tokens": T, "us": t_app * 1e6, "GB/s": app_bytes / t_app / 1e9,
                           "frac_hbm": app_bytes / t_app / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": app_bytes}
    fused_bytes = rope_bytes + 3 * T * H4 * D * 2  # + v read, K and V rows written to their slots
    out["c4_rope_append_fused"] = {"tokens": T, "us": t_fused * 1e6, "GB/s": fused_bytes / t_fused / 1e9,
                                   "frac_hbm": fused_bytes / t_fused / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": fused_bytes,
                                   "unfused_us": (t_rope + t_app) * 1e6}
    co_bytes = fused_bytes - T * H4 * D * 2
    out["c4_rope_append_fused_k_to_cache_only"] = {
        "tokens": T, "us": t_fused_co * 1e6, "GB/s": co_bytes / t_fused_co / 1e9,
        "frac_hbm": co_bytes / t_fused_co / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": co_bytes,
        "unfused_us": (t_rope + t_app) * 1e6}
    out["c4_prefill"] = {"tokens": T, "chunks": len(c4.q_lens), "ms": t_pre * 1e3, "flops": flops,
                         "TFLOP/s": flops / t_pre / 1e12, "frac_mfma_peak": flops / t_pre / 1e12 / MFMA_F16_PEAK_TFLOPS,
                         "tokens/s/layer": T / t_pre}
    # Where the distance between the chunk figure and the matrix peak lies: the tile loop alone, measured as the
    # time one 1024-query chunk (160 workgroups, all resident at once, K/V warm in the last-level cache) gains
    # when its parent grows by 4096 tokens = 64 steps of 64 tokens for every workgroup.
    n1, pool1 = 1024, kc4.shape[0]
    g1 = torch.Generator().manual_seed(11)
    q1 = torch.randn((n1, H4, D), device=dev, dtype=torch.bfloat16)
    o1 = torch.empty_like(q1)
    ts = {}
    for par1 in (2048, 6144):
        slots1 = torch.randperm(pool1, generator=g1)[: par1 + n1].tolist()
        tab1 = kernels.PrefillTables.build([n1], [slots1], dev)
        ts[par1] = _time_gpu(torch, lambda: kernels.prefill_attention(q1, kc4, vc4, tab1, out=o1), iters=10)
    step_s = (ts[6144] - ts[2048]) / 64
    step_flops = 4 * 256 * 64 * D  # one 256-query workgroup, one head, one step
    out["c4_prefill"]["tile_loop"] = {
        "what": "one 1024-query chunk, parent 2048 -> 6144 tokens: time gained / 64 steps",
        "us_per_64_token_step": step_s * 1e6,
        "frac_mfma_peak_if_every_cu_ran_the_loop":
            step_flops * torch.cuda.get_device_properties(dev).multi_processor_count / step_s / 1e12 / MFMA_F16_PEAK_TFLOPS,
        "us_parent_2048": ts[2048] * 1e6, "us_parent_6144": ts[6144] * 1e6}
    del kc4, vc4, qkvs
    # --- config 5: full LLaMA-13B decoder layer, 4 prefix groups x 32 branches, prefix 6000 ------------------
    out["c5_layer"] = config5_layer(torch, dev)
    out["c2_iteration_tables"] = iteration_tables_cost(torch, dev)
    out["prefix_length_sweep"] = prefix_length_sweep(torch, dev)
    out["prefix_regimes"] = prefix_regimes(torch, dev)
    out["bench_kernel_shape"] = bench_kernel_shape(torch, dev)
    out["e2e_decode_13b"] = e2e_decode(torch, dev)
    out["e2e_decode_13b_fused_ops"] = e2e_decode(torch, dev, fused_ops=True)
    # --- RMSNorm at a bandwidth-sized row count (LLaMA-13B hidden) -----------------------------------------
    xs = [torch.randn((8192, 5120), device=dev, dtype=torch.float16) for _ in range(8)]  # 8 x 84 MB, rotated
    w = torch.ones(5120, device=dev, dtype=torch.float16)
    rot = _Rotor(len(xs))
    t = _time_gpu(torch, lambda: kernels.vllm_rms_norm(xs[rot.next()], w, 1e-6))
    nbytes = 2 * xs[0].numel() * 2 + 5120 * 2
    out["rms_norm_8192x5120"] = {"us": t * 1e6, "GB/s": nbytes / t / 1e9, "frac_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS,
                                 "algorithmic_bytes": nbytes}
    out["sampler_64x32000"] = sampler_cost(torch, dev)
    out["c2_shape_head_size_64"] = head_size_64_step(torch, dev)
    out["c2_shape_grouped_kv_heads_32_over_8"] = grouped_kv_heads_step(torch, dev)
    return out


TIMELINE_MARKS = ["kernel entry", "prefix slot window in LDS", "prefix ring requested, query loaded",
                  None, "prefix step 0 (tile landed, workgroup barrier passed)", "prefix step 1",
                  "prefix step 2", "prefix step 3", "prefix main loop done", "token groups folded",
                  None, "kernel exit"]


def _mark_table(rel, marks):
    out = {}
    for i, name in enumerate(marks):
        c = rel[:, i]
        c = c[~__import__("numpy").isnan(c)]
        if name is None or c.size == 0:
            continue
        out[name] = {k: round(float(v), 2) for k, v in
                     zip(("min", "p10", "p50", "p90", "max"), __import__("numpy").percentile(c, [0, 10, 50, 90, 100]))}
    return out


def fused_timeline(torch, lib, step, prefix_wgs, launches=8):
    """Per-wave timestamps at the marks of the fused prefix + suffix kernel (profiling variant of the library), in
    microseconds from the first wave's entry; the median over the launches of every wave's time, then its spread
    over the waves of each kind of workgroup: workgroups [0, prefix_wgs) run prefix units only, the others suffix
    pieces only.  The marks cost a store each: the instrumented kernel runs about 2 us longer.  The shader clock
    between the first prefix step and the end of the prefix loop comes from the same marks."""
    import numpy as np

    for i in range(16):
        step(i)
    torch.cuda.synchronize()
    runs, mhz = [], []
    for i in range(launches):
        lib.ph_timeline_clear()
        torch.cuda.synchronize()
        step(i)
        torch.cuda.synchronize()
        buf = np.zeros(4096 * 12, dtype=np.uint64)
        assert lib.ph_timeline_read(buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes) == 0
        clk = np.zeros(4096 * 12, dtype=np.uint64)
        assert lib.ph_timeline_read_clocks(clk.ctypes.data_as(ctypes.c_void_p), clk.nbytes) == 0
        t = buf.reshape(4096, 12).astype(np.float64)
        c = clk.reshape(4096, 12).astype(np.float64)
        n = int((t[:, 0] > 0).sum())
        ok = (t[:n, 4] > 0) & (t[:n, 8] > t[:n, 4])
        if ok.any():
            mhz.append(float(np.median((c[:n][ok, 8] - c[:n][ok, 4]) / ((t[:n][ok, 8] - t[:n][ok, 4]) / 100.0))))
        t = t[:n]
        runs.append(np.where(t > 0, (t - t[:, 0].min()) / 100.0, np.nan))
    rel = np.nanmedian(np.stack(runs), axis=0)
    out = {"waves": int(rel.shape[0]), "unit": "us from the first wave's entry", "prefix_workgroups": int(prefix_wgs),
           "suffix_workgroups": int(rel.shape[0] // 8 - prefix_wgs)}
    if prefix_wgs > 0:
        out["prefix_marks"] = _mark_table(rel[: prefix_wgs * 8], TIMELINE_MARKS)
        out["suffix_marks"] = _mark_table(rel[prefix_wgs * 8:], TIMELINE_MARKS)
    else:
        out["marks"] = _mark_table(rel, TIMELINE_MARKS)
    if mhz:
        out["shader_clock_mhz_during_prefix_loop"] = round(float(np.median(mhz)), 0)
    wg = rel.reshape(-1, 8, 12)
    out["exit_by_xcd_p50"] = [round(float(np.nanmedian(wg[x::8, :, 11].max(1))), 2) for x in range(8)]
    return out


PREFILL_TIMELINE_MARKS = ["kernel entry", "slot window in LDS", "ring requested, q loaded", None,
                          "step 0 (tile landed, workgroup barrier passed)", "step 1", "step 2", "step 3",
                          "tile loop done", None, None, "kernel exit"]


def prefill_timeline(torch, lib, dev, launches=6):
    """The same marks in the prefill kernel: one 256-query chunk over a 2048-token parent, 40 heads = 40 workgroups
    that all start at once, so a workgroup's prologue (entry to step 0) and epilogue (loop done to exit) can be
    read off beside its tile loop."""
    import numpy as np
    from parrotserve_amd import kernels

    H, D, pool, n, par = 40, 128, 1 << 15, 256, 2048
    kc = torch.randn((pool, H, D), device=dev, dtype=torch.bfloat16)
    vc = torch.randn_like(kc)
    slots = torch.randperm(pool, generator=torch.Generator().manual_seed(7))[: par + n].tolist()
    q = torch.randn((n, H, D), device=dev, dtype=torch.bfloat16)
    o = torch.empty_like(q)
    tab = kernels.PrefillTables.build([n], [slots], dev)
    for _ in range(5):
        kernels.prefill_attention(q, kc, vc, tab, out=o)
    torch.cuda.synchronize()
    runs, mhz = [], []
    for _ in range(launches):
        lib.ph_timeline_clear()
        torch.cuda.synchronize()
        kernels.prefill_attention(q, kc, vc, tab, out=o)
        torch.cuda.synchronize()
        buf = np.zeros(4096 * 12, dtype=np.uint64)
        clk = np.zeros(4096 * 12, dtype=np.uint64)
        assert lib.ph_timeline_read(buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes) == 0
        assert lib.ph_timeline_read_clocks(clk.ctypes.data_as(ctypes.c_void_p), clk.nbytes) == 0
        t = buf.reshape(4096, 12).astype(np.float64)[: H * 8]
        c = clk.reshape(4096, 12).astype(np.float64)[: H * 8]
        ok = (t[:, 7] > 0) & (t[:, 8] > t[:, 7])
        if ok.any():
            mhz.append(float(np.median((c[ok, 8] - c[ok, 7]) / ((t[ok, 8] - t[ok, 7]) / 100.0))))
        runs.append(np.where(t > 0, (t - t[:, 0][t[:, 0] > 0].min()) / 100.0, np.nan))
    rel = np.nanmedian(np.stack(runs), axis=0)
    out = {"waves": int(rel.shape[0]), "steps": (par + n) // 64, "unit": "us from the first wave's entry", "marks": {}}
    if mhz:
        out["shader_clock_mhz_during_tile_loop"] = round(float(np.median(mhz)), 0)
    for i, name in enumerate(PREFILL_TIMELINE_MARKS):
        c = rel[:, i]
        c = c[~np.isnan(c)]
        if name is None or c.size == 0:
            continue
        out["marks"][name] = {k: round(float(v), 2) for k, v in
                              zip(("min", "p10", "p50", "p90", "max"), np.percentile(c, [0, 10, 50, 90, 100]))}
    return out


def prefix_timeline(torch, lib, dev, launches=6):
    """The prefix kernel where the matrix pipe is the bound (one group of 1024 requests over 8192 tokens, 32 x 128
    fp16: 256 workgroups of 256 queries x 4096 tokens each, the same tile loop as the prefill's): time per 64-token
    step of a workgroup and the shader clock the compute units hold while every one of them runs the loop, from the
    marks at the fourth step and at the end of the loop.  (The prefill timeline gives the same for 40 workgroups on
    256 compute units.)"""
    import numpy as np

    from parrotserve_amd import kernels

    B, H, D, P = 1024, 32, 128, 8192
    g = torch.Generator(device=dev).manual_seed(11)
    kc = torch.randn((2 * P, H, D), generator=g, device=dev, dtype=torch.float16)
    vc = torch.randn((2 * P, H, D), generator=g, device=dev, dtype=torch.float16)
    perm = torch.randperm(2 * P, generator=torch.Generator().manual_seed(11))
    q = torch.randn((B, H, D), generator=g, device=dev, dtype=torch.float16)
    o = torch.empty_like(q)
    tabs = [kernels.DecodeTables.build([perm[i * P:(i + 1) * P].tolist()], [0, B], [[] for _ in range(B)], dev,
                                       num_heads=H, head_dim=D) for i in range(2)]
    for i in range(4):
        kernels.decode_attention(q, kc, vc, tabs[i % 2], out=o)
    torch.cuda.synchronize()
    loop_us, mhz, wgs, first = [], [], 0, []
    for i in range(launches):
        lib.ph_timeline_clear()
        torch.cuda.synchronize()
        kernels.decode_attention(q, kc, vc, tabs[i % 2], out=o)
        torch.cuda.synchronize()
        buf = np.zeros(4096 * 12, dtype=np.uint64)
        clk = np.zeros(4096 * 12, dtype=np.uint64)
        assert lib.ph_timeline_read(buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes) == 0
        assert lib.ph_timeline_read_clocks(clk.ctypes.data_as(ctypes.c_void_p), clk.nbytes) == 0
        t = buf.reshape(4096, 12).astype(np.float64)
        c = clk.reshape(4096, 12).astype(np.float64)
        ok = (t[:, 7] > 0) & (t[:, 8] > t[:, 7])
        wgs = int(ok.sum()) // 8
        us = (t[ok, 8] - t[ok, 7]) / 100.0
        mhz.append(float(np.median((c[ok, 8] - c[ok, 7]) / us)))
        loop_us.append(float(np.median(us)))
        first.append(float(np.median((t[ok, 4] - t[ok, 1].min()) / 100.0)))
    steps = P // 2 // 64  # two splits of 4096 tokens, 64-token steps
    return {"batch": B, "prefix_len": P, "workgroups": wgs, "steps_per_workgroup": steps,
            "first_step_us_after_first_window": round(float(np.median(first)), 2),
            "us_per_step": round(float(np.median(loop_us)) / (steps - 4), 3),
            "shader_clock_mhz_during_tile_loop": round(float(np.median(mhz)), 0)}


def head_size_64_step(torch, dev):
    """Config 2's batch with 64-wide heads (32 x 64, the OPT-1.3B shape): the prefix phase runs on head pairs through
    the 128-wide matrix-core kernel, the suffix phase and the merge at the native width.  Warm (one KV set)."""
    from parrotserve_amd import kernels, synth

    g = torch.Generator().manual_seed(1)
    B, P, H, D = 64, 4096, 32, 64
    s = torch.randint(16, 513, (B,), generator=g).tolist()
    case = synth.make_decode_case("d64", 1, torch.float16, 1, B, P, s, H, D, 1 << 20)
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    tables = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                        case.pool_lists(case.suffix_lists), dev, num_heads=H, head_dim=D)
    q = case.q.to(dev)
    o = torch.empty_like(q)
    t = _time_gpu(torch, lambda: kernels.decode_attention(q, kc, vc, tables, out=o))
    nbytes = 2 * (P + sum(s)) * H * D * 2
    res = {"batch": B, "prefix": P, "sum_suffix": sum(s), "heads": H, "head_dim": D, "us": t * 1e6,
           "GB/s": nbytes / t / 1e9, "frac_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": nbytes,
           "tokens/s/layer": B / t}
    del kc, vc
    # config 4's chunks (16 x U[64,1024] new tokens over 2048-token parents, bf16) at 40 x 64: every head runs as one
    # half of a head pair on the 128-wide prefill kernel
    c4 = synth.config4()
    p4 = synth.make_prefill_case("C4-64", 3, torch.bfloat16, c4.q_lens, 2048, 40, 64, 1 << 18)
    kc4, vc4 = synth.pool_to_device(p4.k_rows, p4.v_rows, p4.used_slots, p4.pool_slots, dev)
    ctx = [p4.used_slots[torch.cat([a, b])].tolist() for a, b in zip(p4.parent_lists, p4.new_lists)]
    tab = kernels.PrefillTables.build(p4.q_lens, ctx, dev)
    q4 = p4.q.to(dev)
    o4 = torch.empty_like(q4)
    tp = _time_gpu(torch, lambda: kernels.prefill_attention(q4, kc4, vc4, tab, out=o4), iters=10, inner=5)
    flops = 4 * 40 * 64 * sum(n * 2048 + n * (n + 1) // 2 for n in p4.q_lens)
    res["prefill_c4_chunks_40x64"] = {"tokens": int(sum(p4.q_lens)), "ms": tp * 1e3, "flops": flops,
                                      "TFLOP/s": flops / tp / 1e12}
    return res


def grouped_kv_heads_step(torch, dev):
    """Config 2's batch with grouped KV heads (32 query heads over 8 KV heads, head_mapping h // 4 -- the
    argument of csrc/attention/attention_post_kernels.cu:79,101 that the reference's own models leave at the
    identity): the decode step through ``ph_decode_attention_gqa`` over K/V sets that rotate out of the caches."""
    from parrotserve_amd import kernels

    B, P, H, HKV, D, pool = 64, 4096, 32, 8, 128, 1 << 20
    g = torch.Generator().manual_seed(1)
    lens = torch.randint(16, 513, (B,), generator=g).tolist()
    need = P + sum(lens)
    nbytes = 2 * need * HKV * D * 2
    nsets = 8
    kc = torch.randn((pool, HKV, D), device=dev, dtype=torch.float16)
    vc = torch.randn_like(kc)
    perm = torch.randperm(pool, generator=g)
    tabs = []
    for i in range(nsets):
        sl = perm[i * need:(i + 1) * need].tolist()
        pos, suf = P, []
        for n in lens:
            suf.append(sl[pos:pos + n])
            pos += n
        tabs.append(kernels.DecodeTables.build([sl[:P]], [0, B], suf, dev, num_heads=H, head_dim=D, kv_group=H // HKV))
    q = torch.randn((B, H, D), device=dev, dtype=torch.float16)
    o = torch.empty_like(q)
    hm = (torch.arange(H, dtype=torch.int32) // (H // HKV)).to(dev)
    rot = _Rotor(nsets)
    t = _time_gpu(torch, lambda: kernels.decode_attention(q, kc, vc, tabs[rot.next()], out=o, head_mapping=hm,
                                                          kv_group=H // HKV))
    return {"batch": B, "prefix": P, "sum_suffix": sum(lens), "heads": H, "kv_heads": HKV, "kv_sets": nsets,
            "us": t * 1e6, "GB/s": nbytes / t / 1e9, "frac_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS,
            "algorithmic_bytes": nbytes, "tokens/s/layer": B / t}


def sampler_cost(torch, dev):
    """Temperature + top-p + draw for a batch of 64 rows of 32,000 fp16 logits (everything in Sampler.forward after
    the logits GEMM): the one-launch kernel, and beside it the reference's own sequence of library calls
    (models/sampler.py:33-64: div, sort, softmax, cumsum, mask, argsort, gather, softmax, multinomial) timed on the
    same GPU with the same inputs."""
    from parrotserve_amd import kernels

    B, V = 64, 32000
    g = torch.Generator(device=dev).manual_seed(1)
    logits = (torch.randn((B, V), device=dev, generator=g) * 4).half()
    temp = torch.full((B,), 0.8, device=dev)
    top_p = torch.full((B,), 0.9, device=dev)
    u = torch.rand(B, device=dev, generator=g)

    def library_sequence(filtered):
        x = logits.clone()
        x.div_(temp.unsqueeze(-1))
        if filtered:
            sorted_logits, idx = x.sort(dim=-1, descending=True)
            probs = sorted_logits.softmax(dim=-1)
            mask = (probs.cumsum(dim=-1) - probs) > top_p.unsqueeze(-1)
            sorted_logits[mask] = -float("inf")
            x = torch.gather(sorted_logits, dim=-1, index=torch.argsort(idx, dim=-1))
        return torch.multinomial(torch.softmax(x, dim=-1, dtype=torch.float), num_samples=1, replacement=True)

    res = {"rows": B, "vocab": V, "dtype": "f16"}
    res["kernel_top_p_us"] = _time_gpu(torch, lambda: kernels.sample_top_p(logits, temp, top_p, u)) * 1e6
    res["kernel_plain_draw_us"] = _time_gpu(torch, lambda: kernels.sample_top_p(logits, temp, None, u)) * 1e6
    res["library_sequence_top_p_us"] = _time_gpu(torch, lambda: library_sequence(True), iters=10, inner=3) * 1e6
    res["library_sequence_plain_draw_us"] = _time_gpu(torch, lambda: library_sequence(False), iters=10, inner=3) * 1e6
    return res


def prefix_length_sweep(torch, dev):
    """Fixed cost and steady state of the prefix + suffix launch: batch 64, 32 heads, ten-token suffixes, the shared
    prefix swept from 512 to 32K tokens; a line through the two longest points gives the streaming rate, its
    intercept the part of a launch that does not scale with the prefix (the chain of dependent steps)."""
    from parrotserve_amd import _lib, kernels, synth

    lib = _lib.load()
    ev = HipEvents()
    B, H, D = 64, 32, 128
    res = {"batch": B, "heads": H, "suffix_len": "U[5,14]", "launch_us": {}}
    pts = []
    for P in (512, 2048, 8192, 16384, 32768):
        g = torch.Generator().manual_seed(1)
        lens = torch.randint(5, 15, (B,), generator=g).tolist()
        case = synth.make_decode_case("sweep", 1, torch.float16, 1, B, P, lens, H, D, 1 << 18)
        kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
        tabs = kernels.DecodeTables.build(case.pool_lists(case.prefix_lists), case.group_req_cu,
                                          case.pool_lists(case.suffix_lists), dev, num_heads=H, head_dim=D)
        q = case.q.to(dev)
        o = torch.empty_like(q)
        for _ in range(5):
            kernels.decode_attention(q, kc, vc, tabs, out=o)
        sets = [ev.create(6) for _ in range(30)]
        for s6 in sets:
            kernels.decode_attention(q, kc, vc, tabs, out=o, events6=s6)
        torch.cuda.synchronize()
        t = sorted(ev.elapsed_ms(s6[2], s6[3]) for s6 in sets)[15] * 1e3
        for s6 in sets:
            ev.destroy(s6)
        res["launch_us"][str(P)] = t
        pts.append((2 * P * H * D * 2 / 1e6, t))
        del kc, vc, tabs
    (x0, y0), (x1, y1) = pts[-2], pts[-1]
    slope = (y1 - y0) / (x1 - x0)  # microseconds per MB of K/V
    res["steady_state_GB/s"] = 1e3 / slope
    res["fixed_us"] = y1 - slope * x1
    return res


def _event_time_us(torch, ev, call, which, launches=24, warm=4):
    """Median dispatch time (start / stop events attached to the launch) of kernel `which` (0 prefix, 1 suffix or
    fused, 2 merge) of `call(i, events6)` over `launches` calls."""
    for i in range(warm):
        call(i, None)
    sets = [ev.create(6) for _ in range(launches)]
    for i, s6 in enumerate(sets):
        call(i, s6)
    torch.cuda.synchronize()
    ts = [ev.elapsed_ms(s6[2 * which], s6[2 * which + 1]) for s6 in sets]
    for s6 in sets:
        ev.destroy(s6)
    if any(t is None for t in ts):
        return None
    return sorted(ts)[len(ts) // 2] * 1e3


def prefix_regimes(torch, dev):
    """The prefix phase (matrix-core kernel alone: empty suffixes) from the bandwidth-bound to the matrix-bound regime:
    one group of B requests over a P-token prefix, 32 x 128 fp16.  The contraction has B FLOP per K/V byte, so its
    ceiling is min(matrix peak, B x HBM peak); cold = the launches rotate over K/V sets that do not fit the
    memory-side cache together, warm = one set re-read."""
    from parrotserve_amd import kernels

    ev = HipEvents()
    H, D, pool = 32, 128, 1 << 16
    g = torch.Generator(device=dev).manual_seed(11)
    kc = torch.randn((pool, H, D), generator=g, device=dev, dtype=torch.float16)
    vc = torch.randn((pool, H, D), generator=g, device=dev, dtype=torch.float16)
    perm = torch.randperm(pool, generator=torch.Generator().manual_seed(11))
    res = {"heads": H, "head_dim": D, "dtype": "f16", "points": []}
    for P in (4096, 8192):
        nsets = pool // P
        for B in (64, 128, 256, 512, 1024):
            q = torch.randn((B, H, D), generator=g, device=dev, dtype=torch.float16)
            o = torch.empty_like(q)
            tabs = [kernels.DecodeTables.build([perm[i * P:(i + 1) * P].tolist()], [0, B], [[] for _ in range(B)], dev,
                                               num_heads=H, head_dim=D) for i in range(nsets)]
            flops = 4 * B * H * P * D
            kv = 2 * P * H * D * 2
            bound = min(MFMA_F16_PEAK_TFLOPS, B * HBM_PEAK_GBS / 1e3)
            pt = {"batch": B, "prefix_len": P, "flops": flops, "kv_bytes": kv, "bound_tflops": bound}
            for label, pick in (("cold", lambda i: tabs[i % nsets]), ("warm", lambda i: tabs[0])):
                t = _event_time_us(torch, ev, lambda i, e6: kernels.decode_attention(q, kc, vc, pick(i), out=o,
                                                                                     events6=e6), 0)
                if t is None:
                    continue
                tf = flops / t / 1e6
                pt[label] = {"us": t, "tflops": tf, "frac_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS,
                             "frac_of_min_mfma_hbm_bound": tf / bound, "kv_GB/s": kv / t / 1e3}
            res["points"].append(pt)
            del tabs
    return res


def bench_kernel_shape(torch, dev):
    """The one shape the reference's own kernel benchmark runs (benchmark/bench_kernel.py:11-83): batch 64 sharing an
    8192-token prefix, 40 x 128 heads, ten to twenty diverged tokens per request.  The launch that runs the prefix and
    suffix phases against the HBM roofline (K/V of the prefix once, of every suffix once), and the merge beside it."""
    from parrotserve_amd import kernels, synth

    ev = HipEvents()
    B, P, H, D = 64, 8192, 40, 128
    g = torch.Generator().manual_seed(1)
    lens = torch.randint(10, 21, (B,), generator=g).tolist()
    nsets = 4
    case = synth.make_decode_case("bk", 1, torch.float16, 1, B, P, lens, H, D, 1 << 16)
    n_used = case.k_rows.shape[0]
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    perm = torch.randperm(case.pool_slots, generator=torch.Generator().manual_seed(2))
    dgen = torch.Generator(device=dev).manual_seed(2)
    tabs = []
    for i in range(nsets):  # K/V sets at other slots of the pool, device-generated rows
        used = perm[i * n_used:(i + 1) * n_used]
        idx = used.to(dev)
        kc[idx] = torch.randn((n_used, H, D), generator=dgen, device=dev, dtype=torch.float16)
        vc[idx] = torch.randn((n_used, H, D), generator=dgen, device=dev, dtype=torch.float16)
        tabs.append(kernels.DecodeTables.build([used[p].tolist() for p in case.prefix_lists], case.group_req_cu,
                                               [used[x].tolist() for x in case.suffix_lists], dev, num_heads=H,
                                               head_dim=D))
    q = case.q.to(dev)
    o = torch.empty_like(q)
    call = lambda i, e6: kernels.decode_attention(q, kc, vc, tabs[i % nsets], out=o, events6=e6)
    t_k = _event_time_us(torch, ev, call, 1)
    t_m = _event_time_us(torch, ev, call, 2)
    t_step = _time_gpu(torch, lambda: call(0, None), iters=10)
    nbytes = 2 * (P + sum(lens)) * H * D * 2
    return {"batch": B, "prefix_len": P, "heads": H, "sum_suffix_len": sum(lens), "kv_sets": nsets,
            "step_us_one_set": t_step * 1e6, "merge_us": t_m,
            "roofline": {"kernel": "decode_fused_kernel (prefix + suffix phases)", "bound": "hbm",
                         "algorithmic_bytes": nbytes, "avg_launch_us": t_k,
                         "achieved": None if t_k is None else nbytes / t_k / 1e3, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": None if t_k is None else nbytes / t_k / 1e3 / HBM_PEAK_GBS}}


def iteration_tables_cost(torch, dev):
    """Host time per decode iteration of producing the device index tables (slot tables, lengths, suffix plan)
    for config 2's batch, 64 Generate jobs forked from one 4096-token parent, own contexts U[16,512]: rebuilt
    from the context trees every iteration as the reference does (attn_func.py:462-599), against patched in
    place by the table cache (one appended slot per request)."""
    from parrotserve_amd.attn_func import BuiltinConfig, HipGroupedPrefixAttn
    from parrotserve_amd.context import BlockContext, RecyclePool
    from parrotserve_amd.iter_state import IterationState
    from parrotserve_amd.primitive_job import Generate
    from parrotserve_amd.table_cache import DecodeTableCache

    class Cfg:
        num_attention_heads, hidden_size = 32, 4096

    class Inc(HipGroupedPrefixAttn):
        table_cache = DecodeTableCache()

    class Fresh(HipGroupedPrefixAttn):
        incremental = False

    gen = torch.Generator().manual_seed(1)
    lens = torch.randint(16, 513, (64,), generator=gen).tolist()
    res = {"jobs": 64}
    for label, cls in (("full_rebuild_us", Fresh), ("incremental_us", Inc)):
        pool = RecyclePool(pool_size=1 << 20)
        parent = BlockContext(0, None, pool, 1)
        parent.allocate(4096)
        jobs = []
        for b, n in enumerate(lens):
            c = BlockContext(1 + b, parent, pool, 1)
            c.allocate(n)
            j = Generate(0, b, c.context_id, parent.context_id, sampling_config=None)
            j.context = c
            jobs.append(j)
        cfg = BuiltinConfig(num_kv_cache_blocks=1 << 20, attn_func=cls, dtype=torch.float16, device=dev)
        ts = []
        for it in range(24):
            for j in jobs:
                j.context.allocate(1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            IterationState(jobs, Cfg, cfg)
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        ts = sorted(ts[4:])
        res[label] = ts[len(ts) // 2] * 1e6
        res["sum_context"] = sum(j.context.get_context_len() for j in jobs)
    res["speedup"] = res["full_rebuild_us"] / res["incremental_us"]
    return res


def e2e_decode(torch, dev, fused_ops=False):
    """The reference's decode experiment (benchmark/bench_kernel.py:11-86) end to end on the engine loop: LLaMA-13B
    shape (vicuna-13b-v1.3: 40 layers, hidden 5120, 40x128, FFN 13824, vocab 32000) with random weights, batch 64,
    one shared 8192-token Fill, 64 forked Fills of 10 tokens, then 10 Generate iterations."""
    from parrotserve_amd import mem
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.primitive_job import Fill, Generate
    from parrotserve_amd.runner import BuiltinRunner, LlamaConfig, SamplingConfig

    B, shared_len, diverged_len, output_len = 64, 8192, 10, 10
    mc = LlamaConfig(vocab_size=32000, hidden_size=5120, intermediate_size=13824, num_hidden_layers=40,
                     num_attention_heads=40, rms_norm_eps=1e-6, max_position_embeddings=16384, fused_ops=fused_ops)
    cfg = BuiltinConfig(num_kv_cache_blocks=16384, attn_func="hip_shared_prefix", dtype=torch.float16, device=dev)
    cfg.attn_func.table_cache.clear()
    runner = BuiltinRunner(mc, cfg)
    sc = SamplingConfig(max_gen_length=output_len, ignore_tokenizer_eos=True)
    t_fill = runner.run_iter([Fill(0, 0, 0, -1, token_ids=[100] * shared_len)])
    t_div = runner.run_iter([Fill(0, 0, i + 1, 0, token_ids=[100] * diverged_len) for i in range(B)])
    gens = [Generate(0, 0, i + 1, 0, sampling_config=sc) for i in range(B)]
    its = [runner.run_iter(gens) for _ in range(output_len - 1)]
    e2e = sorted(t[0] for t in its[1:])
    model = sorted(t[1] for t in its[1:])
    res = {"model": "LLaMA-13B shape, random weights", "fused_ops": fused_ops, "batch": B, "shared_len": shared_len, "diverged_len": diverged_len,
           "shared_fill_ms": t_fill[1] / 1e6, "diverged_fills_ms": t_div[1] / 1e6,
           "decode_iter_ms": e2e[len(e2e) // 2] / 1e6, "decode_model_ms": model[len(model) // 2] / 1e6,
           "decode_tokens/s": B / (e2e[len(e2e) // 2] / 1e9)}
    del runner
    mem.Model_Cache = None
    cfg.attn_func.table_cache.clear()
    torch.cuda.empty_cache()
    return res


def config5_layer(torch, dev):
    """RMSNorm -> QKV -> RoPE -> append -> grouped shared-prefix attention -> O-proj -> RMSNorm -> MLP, fp16,
    hidden 5120, 40x128, FFN 13824, weights N(0, 0.02); GEMMs are library GEMMs (nn.Linear)."""
    from parrotserve_amd import kernels, mem, synth
    from parrotserve_amd.attn_func import BuiltinConfig
    from parrotserve_amd.llama_layer import LlamaDecoderLayer

    case = synth.config5()
    dec = case.decode
    B, H, D, hidden = dec.num_reqs, 40, 128, 5120
    store = mem.init_model_cache_storage(1, dec.pool_slots, H, D, torch.float16, dev, max_seq_len=8192,
                                         rope_theta=case.theta)
    kc, vc = synth.pool_to_device(dec.k_rows, dec.v_rows, dec.used_slots, dec.pool_slots, dev)
    store.k_cache[0].copy_(kc)
    store.v_cache[0].copy_(vc)
    del kc, vc
    cfg = BuiltinConfig(num_kv_cache_blocks=dec.pool_slots, attn_func="hip_shared_prefix", dtype=torch.float16,
                        device=dev)

    class _State:  # the iteration state the plug-in builds from the jobs' context trees, here from the case's lists
        pass

    st = _State()
    st.num_fill_tokens = []
    st.generation_sampling_config = [None] * B
    st.num_total_fill_tokens = 0
    st.num_generation_jobs = B
    st.slot_mapping = case.new_slots.to(torch.int32).to(dev)
    st.fill_tables = None
    st.fill_decode_tables = None
    st.decode_perm = None
    st.decode_tables = kernels.DecodeTables.build(dec.pool_lists(dec.prefix_lists), dec.group_req_cu,
                                                  dec.pool_lists(dec.suffix_lists), dev, num_heads=H, head_dim=D)
    layer = LlamaDecoderLayer(hidden, H, 13824, case.eps, 0, cfg.attn_func).half().to(dev)
    w = case.weights
    with torch.no_grad():
        layer.self_attn.qkv_proj.weight.copy_(w["qkv_proj"])
        layer.self_attn.o_proj.weight.copy_(w["o_proj"])
        layer.mlp.gate_proj.weight.copy_(w["gate_proj"])
        layer.mlp.up_proj.weight.copy_(w["up_proj"])
        layer.mlp.down_proj.weight.copy_(w["down_proj"])
    x = case.x.to(dev)
    pos = case.positions.to(dev)
    q = torch.randn((B, H, D), device=dev, dtype=torch.float16)
    o = torch.empty_like(q)
    with torch.inference_mode():
        t_layer = _time_gpu(torch, lambda: layer(x, pos, st), iters=20)
        t_attn = _time_gpu(torch, lambda: kernels.decode_attention(q, store.k_cache[0], store.v_cache[0],
                                                                   st.decode_tables, out=o), iters=20)
    sum_s = sum(l.numel() for l in dec.suffix_lists)
    P = dec.prefix_lists[0].numel()
    kv_bytes = 2 * (len(dec.prefix_lists) * P + sum_s) * H * D * 2
    res = {"batch": B, "groups": len(dec.prefix_lists), "prefix_len": P, "sum_suffix_len": sum_s,
           "layer_ms": t_layer * 1e3, "attention_us": t_attn * 1e6, "attention_kv_bytes": kv_bytes,
           "attention_GB/s": kv_bytes / t_attn / 1e9, "attention_frac_hbm": kv_bytes / t_attn / 1e9 / HBM_PEAK_GBS,
           "tokens/s/layer": B / t_layer}
    mem.Model_Cache = None
    return res


def kernels_cos_sin(torch, n, d, theta, dtype, dev):
    from parrotserve_amd.mem import make_cos_sin_cache

    return make_cos_sin_cache(n, d, theta, dtype, dev)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="distinct KV sets the steps rotate over")
    ap.add_argument("--cpu-sample", type=int, default=64, help="requests of the batch the CPU baseline runs")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations' kernel rooflines")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the move kernel as a plain 1 GiB copy (known traffic, to scale the profiler's "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    ap.add_argument("--e2e-only", action="store_true",
                    help="only run the 13B-shape decode experiment (fused per-layer ops) and exit (for a kernel trace "
                         "of a whole engine iteration)")
    ap.add_argument("--sampler-only", action="store_true",
                    help="only time the token sampler (kernel and the reference's library-call sequence) and exit")
    ap.add_argument("--timeline", action="store_true",
                    help="only record where the waves of the fused decode kernel spend their time (needs the "
                         "profiling variant of the library, built beside the product one) and exit")
    ap.add_argument("--prefix-regimes-only", action="store_true",
                    help="only run the prefix phase over batch sizes from the bandwidth-bound to the matrix-bound "
                         "regime, and the reference benchmark's shape, and exit")
    ap.add_argument("--prefix-point-only", action="store_true",
                    help="only run the prefix phase of one group of 256 requests over 8192 tokens (32 x 128 fp16, empty "
                         "suffixes) a few times (for profiler counter passes on the 256-query tile) and exit")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only run config 4's prefill kernel a few times (for profiler counter passes) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU; --gpus must be 1 "
              "(no collectives or sharding are part of it).", file=sys.stderr)
        sys.exit(2)

    import torch

    from parrotserve_amd import _lib, kernels, synth

    if args.timeline:  # before the first load(): this run binds the profiling variant of the library
        from parrotserve_amd import build as _build

        if not os.path.exists(_build.TIMELINE_LIB_PATH):  # the profiling variant is only built when asked for
            _build.build(verbose=False, timeline=True)
        _lib.LIB_PATH = _build.TIMELINE_LIB_PATH
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    lib = _lib.load()

    if args.sampler_only:
        print(json.dumps({"sampler_64x32000": sampler_cost(torch, dev)}))
        return
    if args.e2e_only:
        print(json.dumps({"e2e_decode_13b_fused_ops": e2e_decode(torch, dev, fused_ops=True)}))
        return

    if args.prefix_regimes_only:
        print(json.dumps({"prefix_regimes": prefix_regimes(torch, dev),
                          "bench_kernel_shape": bench_kernel_shape(torch, dev)}))
        return

    if args.prefix_point_only:
        B, H, D, P = 256, 32, 128, 8192
        g = torch.Generator(device=dev).manual_seed(11)
        kc = torch.randn((4 * P, H, D), generator=g, device=dev, dtype=torch.float16)
        vc = torch.randn((4 * P, H, D), generator=g, device=dev, dtype=torch.float16)
        perm = torch.randperm(4 * P, generator=torch.Generator().manual_seed(11))
        q = torch.randn((B, H, D), generator=g, device=dev, dtype=torch.float16)
        o = torch.empty_like(q)
        tabs = [kernels.DecodeTables.build([perm[i * P:(i + 1) * P].tolist()], [0, B], [[] for _ in range(B)], dev,
                                           num_heads=H, head_dim=D) for i in range(4)]
        rot = _Rotor(4)
        t = _time_gpu(torch, lambda: kernels.decode_attention(q, kc, vc, tabs[rot.next()], out=o), iters=3, warmup=1,
                      inner=4)
        flops = 4 * B * H * P * D
        print(json.dumps({"prefix_point_only": {"batch": B, "prefix_len": P, "us_with_merge": t * 1e6, "flops": flops}}))
        return

    if args.prefill_only:
        # config 4's prefill with parent context alone, a few launches (for counter collection on that kernel)
        c4 = synth.config4()
        T, H4, D4 = c4.q.shape
        kc4, vc4 = synth.pool_to_device(c4.k_rows, c4.v_rows, c4.used_slots, c4.pool_slots, dev)
        ctx = [c4.used_slots[torch.cat([p, n])].tolist() for p, n in zip(c4.parent_lists, c4.new_lists)]
        ptab = kernels.PrefillTables.build(c4.q_lens, ctx, dev)
        qc = c4.q.to(dev)
        o4 = torch.empty_like(qc)
        t_pre = _time_gpu(torch, lambda: kernels.prefill_attention(qc, kc4, vc4, ptab, out=o4), iters=3, warmup=1, inner=4)
        par = c4.parent_lists[0].numel()
        flops = 4 * H4 * D4 * sum(n * par + n * (n + 1) // 2 for n in c4.q_lens)
        print(json.dumps({"c4_prefill_only": {"tokens": T, "ms": t_pre * 1e3, "flops": flops,
                                              "TFLOP/s": flops / t_pre / 1e12}}))
        return

    if args.copy_calibration:
        rows = 131072  # x 8 KiB = 1 GiB read + 1 GiB written per launch
        src = torch.randn(rows, 32, 128, device=dev, dtype=torch.float16)
        dst = torch.empty_like(src)
        idx = torch.arange(rows, device=dev)
        for _ in range(6):
            kernels.discontinuous_move_tokens(src, dst, idx, idx)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"launches": 6, "bytes_read": rows * 8192, "bytes_written": rows * 8192}}))
        return

    case = synth.config2()
    B, H, D = case.q.shape
    P = case.prefix_lists[0].numel()
    sum_s = int(sum(l.numel() for l in case.suffix_lists))
    n_used = case.k_rows.shape[0]
    NL = max(1, args.layers)

    # layer 0 = the seeded CPU case; layers 1.. use other slots of the same pool with device-generated N(0,1) rows
    kc, vc = synth.pool_to_device(case.k_rows, case.v_rows, case.used_slots, case.pool_slots, dev)
    gen = torch.Generator().manual_seed(1)
    perm = torch.randperm(case.pool_slots, generator=gen)  # same first draw as synth.config2 -> perm[:n_used] == used_slots
    assert torch.equal(perm[:n_used], case.used_slots)
    dgen = torch.Generator(device=dev).manual_seed(1)
    tables, qs = [], []
    for l in range(NL):
        used = perm[l * n_used : (l + 1) * n_used]
        if l > 0:
            idx = used.to(dev)
            kc[idx] = torch.randn((n_used, H, D), generator=dgen, device=dev, dtype=torch.float16)
            vc[idx] = torch.randn((n_used, H, D), generator=dgen, device=dev, dtype=torch.float16)
        pre = [used[p].tolist() for p in case.prefix_lists]
        suf = [used[s].tolist() for s in case.suffix_lists]
        tables.append(kernels.DecodeTables.build(pre, case.group_req_cu, suf, dev))
        qs.append(case.q.to(dev) if l == 0 else torch.randn((B, H, D), generator=dgen, device=dev, dtype=torch.float16))
    out = torch.empty((B, H, D), dtype=torch.float16, device=dev)

    def step(i, events6=None):
        l = i % NL
        kernels.decode_attention(qs[l], kc, vc, tables[l], out=out, events6=events6)

    def timed(fn, steps, warmup):
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    if args.timeline:
        hgroups = (H + 3) // 4  # four 128-wide heads per wave
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        prefix_wgs = cus - (int(tables[0].plan.num_lanes) * hgroups + 7) // 8  # what the plan's lane count leaves
        print(json.dumps({"fused_kernel_timeline": fused_timeline(torch, lib, step, max(0, prefix_wgs)),
                          "prefill_kernel_timeline": prefill_timeline(torch, lib, dev),
                          "prefix_kernel_timeline": prefix_timeline(torch, lib, dev)}))
        return

    t_step = timed(step, args.steps, args.warmup)
    t_warm = timed(lambda i: kernels.decode_attention(qs[0], kc, vc, tables[0], out=out), args.steps, args.warmup)

    # spread of single steps inside the same rotation (an event between steps; the events themselves cost the
    # stream about a microsecond per step, so these sit a little above ms_per_step)
    n_pc = min(args.steps, 400)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(n_pc + 1)]
    marks[0].record()
    for i in range(n_pc):
        step(i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(n_pc))
    pct = {k: per_step[min(n_pc - 1, int(q * n_pc))] for k, q in (("p10", 0.1), ("p50", 0.5), ("p90", 0.9))}

    # per-kernel durations inside the same rotation: each kernel's own dispatch begin/end (start/stop events
    # attached to its launch on the launch stream), the quantity a kernel trace reports
    ev = HipEvents()
    n_ev = min(args.steps, 200)
    sets = [ev.create(6) for _ in range(n_ev)]
    for i in range(n_ev):
        step(i, sets[i])
    torch.cuda.synchronize()
    ph = [[ev.elapsed_ms(s[2 * k], s[2 * k + 1]) for s in sets] for k in range(3)]
    for s in sets:
        ev.destroy(s)
    # the prefix pair stays unrecorded when the library runs the prefix and suffix phases in one launch
    fused = all(x is None for x in ph[0])
    _, t_suffix, t_merge = (None if any(v is None for v in x) else sum(x) / len(x) * 1e-3 for x in ph)

    e = 2  # bytes per fp16 element
    suffix_bytes = 2 * sum_s * H * D * e
    prefix_bytes = 2 * P * H * D * e
    prefix_flops = 4 * B * H * P * D
    counters = measured_counters()
    if fused:
        # one kernel streams the prefix K/V (through the matrix cores) and every request's suffix K/V
        kernel_name = "decode_fused_kernel (prefix + suffix phases)"
        kernel_bytes = prefix_bytes + suffix_bytes
        traffic = counters.get("hbm_traffic_bytes", {}).get("decode_fused_kernel")
    else:
        kernel_name = "decode_items_kernel (suffix phase)"
        kernel_bytes = suffix_bytes
        traffic = counters.get("hbm_traffic_bytes", {}).get("decode_items_kernel")
    kernel_gbs = kernel_bytes / t_suffix / 1e9

    result = {
        "metric": "shared-prefix decode attn tokens/s/layer",
        "value": B / t_step,
        "unit": "tokens/s/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": t_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE config 2: fp16 32x128, batch 64 sharing one 4096-token prefix, suffix U[16,512], "
                        "1M-slot pool, seed 1; steps rotate over %d layers' KV sets" % NL,
            "batch": B, "prefix_len": P, "sum_suffix_len": sum_s, "heads": H, "head_dim": D, "kv_sets": NL,
        },
        "roofline": {
            "kernel": kernel_name,
            "bound": "hbm",
            "achieved": kernel_gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": kernel_gbs / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_measured_at_commit": counters.get("commit") if traffic is not None else None,
            "algorithmic_bytes": kernel_bytes,
            "avg_launch_us": t_suffix * 1e6,
        },
        "merge_us": t_merge * 1e6,
        "step_us_percentiles": pct,
        "warm_single_kv_set": {"value": B / t_warm, "ms_per_step": t_warm * 1e3},
    }
    def kernel_time(tabs_of, which, launches=64, warm=8):
        """Average dispatch time (start/stop events attached to the launch) of kernel `which` (0 prefix, 1 suffix)
        over `launches` calls; tabs_of(i) picks the tables and query of call i."""
        for i in range(warm):
            t, q = tabs_of(i)
            kernels.decode_attention(q, kc, vc, t, out=out)
        sets = [ev.create(6) for _ in range(launches)]
        for i, s6 in enumerate(sets):
            t, q = tabs_of(i)
            kernels.decode_attention(q, kc, vc, t, out=out, events6=s6)
        torch.cuda.synchronize()
        ts = [ev.elapsed_ms(s6[2 * which], s6[2 * which + 1]) for s6 in sets]
        for s6 in sets:
            ev.destroy(s6)
        return None if any(v is None for v in ts) else sum(ts) / len(ts) * 1e-3

    # The two phases on their own, each against the roofline that bounds it.
    # Prefix phase: the same batch with empty suffixes (prefix kernel, then merge).  It is a dense contraction with
    # exactly B FLOP per K/V byte, so from HBM its ceiling is min(MFMA peak, B x HBM peak) = 0.51 PFLOP/s at B = 64
    # (20 % of the matrix peak): "cold" rotates over the KV sets as the step does and is measured against that bound;
    # "warm" re-reads one 67 MB set, which stays in the 256 MB memory-side cache, and is measured against the
    # matrix peak itself (the figure the reference quotes for its kernel, shared_flash_decoding.py:407-416).
    ptabs = [kernels.DecodeTables.build([perm[l * n_used:(l + 1) * n_used][p].tolist() for p in case.prefix_lists],
                                        case.group_req_cu, [[] for _ in range(B)], dev) for l in range(NL)]
    prefix_bound_tflops = min(MFMA_F16_PEAK_TFLOPS, B * HBM_PEAK_GBS / 1e3)  # AI = B FLOP per KV byte
    phase = {"kernel": "prefix_mfma8_kernel (run on its own: the batch with empty suffixes)",
             "flops": prefix_flops, "kv_bytes": prefix_bytes}
    for label, pick in (("cold", lambda i: (ptabs[i % NL], qs[i % NL])), ("warm", lambda i: (ptabs[0], qs[0]))):
        tp = kernel_time(pick, 0)
        if tp is None:
            continue
        tf = prefix_flops / tp / 1e12
        phase[label] = {"avg_launch_us": tp * 1e6, "tflops": tf, "frac_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS,
                        "frac_of_min_mfma_hbm_bound": tf / prefix_bound_tflops, "kv_gbs": prefix_bytes / tp / 1e9}
    if "cold" in phase:
        # matrix-pipe utilisation of the kernel from the profiler's counters (profiles/counters.json):
        # SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE per XCD x SIMDs)
        pc = counters.get("prefix_mfma8_kernel", {})
        phase["mfma_pipe_utilisation_from_counters"] = pc.get("mfma_pipe_utilisation")
        phase["mfma_pipe_utilisation_by_trace_duration"] = pc.get("mfma_pipe_utilisation_by_trace_duration")
        phase["counters_measured_at_commit"] = counters.get("commit")
        result["prefix_phase"] = phase
    del ptabs
    # Suffix phase: the same requests without the shared prefix (P = 0) through decode_items_kernel, against HBM.
    stabs = [kernels.DecodeTables.build([], [], [perm[l * n_used:(l + 1) * n_used][sx].tolist()
                                                 for sx in case.suffix_lists], dev) for l in range(NL)]
    ts_ = kernel_time(lambda i: (stabs[i % NL], qs[i % NL]), 1)
    if ts_ is not None:
        result["suffix_phase"] = {
            "kernel": "decode_items_kernel (run on its own: the batch without its shared prefix)",
            "avg_launch_us": ts_ * 1e6, "algorithmic_bytes": suffix_bytes, "GB/s": suffix_bytes / ts_ / 1e9,
            "frac_hbm": suffix_bytes / ts_ / 1e9 / HBM_PEAK_GBS,
            "traffic": counters.get("hbm_traffic_bytes", {}).get("decode_items_kernel"),
        }
    del stabs
    # the same step through the reference-named op unchanged model code calls (flash_paged_attention with the
    # reference's argument list): eight "layers" of one iteration share the length tensor, so layers 2..8 reuse the
    # tables and suffix plan layer 1 built
    suf0 = [perm[:n_used][sx].tolist() for sx in case.suffix_lists]
    width = max(len(x) for x in suf0)
    ptable = torch.tensor([x + [0] * (width - len(x)) for x in suf0], dtype=torch.int32, device=dev)
    flash0 = perm[:n_used][case.prefix_lists[0]].to(torch.int32).to(dev)
    hm = torch.arange(H, dtype=torch.int32, device=dev)
    lens_host = torch.tensor([len(x) for x in suf0], dtype=torch.int32)

    def iteration_of_8_layers():
        plens = lens_host.to(dev)  # a fresh length tensor per iteration, as the reference builds it
        for _ in range(8):
            kernels.flash_paged_attention(qs[0], kc, vc, hm, P, flash0, plens, ptable)

    t_named = _time_gpu(torch, iteration_of_8_layers, iters=10, inner=4) / 8
    result["reference_named_op"] = {"op": "flash_paged_attention", "layers_per_iteration": 8,
                                    "us_per_call": t_named * 1e6,
                                    "note": "one KV set (cache-warm); includes the per-iteration upload of the lengths "
                                            "and one plan build per iteration"}
    if not args.no_extras:
        del kc, vc, tables, qs
        torch.cuda.empty_cache()
        result["extras"] = extras(torch, dev)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(case, min(args.cpu_sample, B))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
