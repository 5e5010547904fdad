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

# HBM traffic of one suffix-kernel launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (profiles/decode_partial_c2_pmc.txt); None until measured.
SUFFIX_TRAFFIC_BYTES = None


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

    def elapsed_ms(self, a, b) -> float:
        out = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(out), a, b)
        assert rc == 0, f"hipEventElapsedTime rc={rc}"
        return out.value

    def destroy(self, evs):
        for e in evs:
            self.hip.hipEventDestroy(e)


def cpu_baseline(case, sample_reqs: int):
    """The oracle's one-shot decode attention (gather by slot + softmax attention, the
    reference's token-granular algorithm) timed on the host cores for a bounded sample."""
    import torch

    from oracle.ref_ops import ref_decode_attention

    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    lists = case.full_lists()[:sample_reqs]
    q = case.q[:sample_reqs]
    ref_decode_attention(q[:1], case.k_rows, case.v_rows, lists[:1])  # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        ref_decode_attention(q, case.k_rows, case.v_rows, lists)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[1]
    return {
        "value": sample_reqs / t,
        "unit": "tokens/s/layer",
        "cores": cores,
        "kind": "port",
        "sample": f"{sample_reqs} of {case.num_reqs} requests of the same workload (fp32 math on fp16-rounded inputs), median of 3",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="distinct KV sets the steps rotate over")
    ap.add_argument("--cpu-sample", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU; --gpus must be 1 "
              "(no collectives or sharding are part of it).", file=sys.stderr)
        sys.exit(2)

    import torch

    from parrotserve_amd import _lib, kernels, synth

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    lib = _lib.load()

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

    def step(i):
        l = i % NL
        kernels.decode_attention(qs[l], kc, vc, tables[l], out=out)

    def timed(fn, steps, warmup):
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    t_step = timed(step, args.steps, args.warmup)
    t_warm = timed(lambda i: kernels.decode_attention(qs[0], kc, vc, tables[0], out=out), args.steps, args.warmup)

    # per-kernel durations inside the same rotation, HIP events on the launch stream
    ev = HipEvents()
    n_ev = min(args.steps, 200)
    sets = [ev.create(4) for _ in range(n_ev)]
    for i in range(n_ev):
        lib.ph_arm_phase_events(sets[i])
        step(i)
    torch.cuda.synchronize()
    ph = [[ev.elapsed_ms(s[k], s[k + 1]) for s in sets] for k in range(3)]
    for s in sets:
        ev.destroy(s)
    t_prefix, t_suffix, t_merge = (sum(x) / len(x) * 1e-3 for x in ph)

    e = 2  # bytes per fp16 element
    suffix_bytes = 2 * sum_s * H * D * e
    prefix_bytes = 2 * P * H * D * e
    prefix_flops = 4 * B * H * P * D
    suffix_gbs = suffix_bytes / t_suffix / 1e9
    prefix_tflops = prefix_flops / t_prefix / 1e12
    prefix_bound_tflops = min(MFMA_F16_PEAK_TFLOPS, B * HBM_PEAK_GBS / 1e3)  # AI = B FLOP per KV byte

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
            "kernel": "decode_partial_kernel (suffix phase)",
            "bound": "hbm",
            "achieved": suffix_gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": suffix_gbs / HBM_PEAK_GBS,
            "traffic": SUFFIX_TRAFFIC_BYTES,
            "algorithmic_bytes": suffix_bytes,
            "avg_launch_us": t_suffix * 1e6,
        },
        "prefix_phase": {
            "kernel": "prefix_mfma_kernel",
            "avg_launch_us": t_prefix * 1e6,
            "tflops": prefix_tflops,
            "frac_mfma_peak": prefix_tflops / MFMA_F16_PEAK_TFLOPS,
            "frac_of_min_mfma_hbm_bound": prefix_tflops / prefix_bound_tflops,
            "kv_gbs": prefix_bytes / t_prefix / 1e9,
        },
        "merge_us": t_merge * 1e6,
        "warm_single_kv_set": {"value": B / t_warm, "ms_per_step": t_warm * 1e3},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(case, min(args.cpu_sample, B))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
