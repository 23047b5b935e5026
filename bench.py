#!/usr/bin/env python
"""bench.py -- attention hot path of libcwick_hip.so on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs 1,2,3,4,5] [--no-cpu]

One JSON line on stdout.  `value` is the headline of BASELINE.json's metric: decode
attention microseconds per token at 32K context (configs[2]: MLA absorbed-latent decode,
128 heads, 32768 x 576 FP8-E4M3 latent), measured as wall time over exactly K steps with
every operand already resident in HBM.  The same line carries the HBM GB/s of that step,
the 8K causal GQA prefill TFLOP/s (configs[1]) and one entry per other configuration
under "configs", each with its kernel times (HIP events on the launch stream, inside
the library) and roofline fraction, and the CPU baseline: the oracle's restatement of
the reference algorithm timed on this host's cores.

A step = one pass of the hot path over one batch of synthetic input (one decode token,
one prefill chunk, one batch of 8 DSA queries).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0      # dense bf16 / fp16 MFMA, published
FP32_VALU_PEAK_TFLOPS = 157.3  # fp32 vector, published

METRIC = "decode attn µs/token + HBM GB/s @32K ctx; prefill attn TFLOP/s @8K (1 GPU)"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def dev(x):
    """numpy -> HBM (torch is only the allocator here)."""
    import torch
    if x.dtype == np.uint16:
        return torch.from_numpy(x.view(np.int16)).cuda()
    return torch.from_numpy(x).cuda()


class Timer:
    """Wall time of K back-to-back steps with device syncs on both sides, then the same K
    steps again with the library's phase timers on (HIP events around each kernel)."""

    def __init__(self, hip, torch, steps, warmup):
        self.hip, self.torch, self.steps, self.warmup = hip, torch, steps, warmup

    def run(self, step):
        torch, hip = self.torch, self.hip
        for _ in range(self.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(self.steps):
            step()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / self.steps
        hip.prof_reset()
        hip.prof_enable(True)
        for _ in range(self.steps):
            step()
        torch.cuda.synchronize()
        hip.prof_enable(False)
        kern = {k: {"avg_us": 1e3 * ms / n, "launches": n}
                for k, (ms, n) in hip.prof_read().items() if n}
        return wall, kern


def roofline(bound, alg, seconds, peak, unit, traffic=None):
    """alg: algorithmic bytes (hbm) or flops (mfma/valu) of ONE launch of the kernel."""
    ach = alg / seconds / (1e9 if unit == "GB/s" else 1e12)
    return {"bound": bound, "achieved": round(ach, 2), "peak": peak, "unit": unit,
            "frac": round(ach / peak, 4), "traffic": traffic}


# ---------------------------------------------------------------- the five configurations
def bench_cfg1(hip, synth, T, stream):
    import torch
    c = synth.cfg1_gqa_decode()
    k, v, q = dev(c["k"]), dev(c["v"]), dev(c["q"])
    out = torch.empty((c["nh"], c["hd"]), dtype=torch.float32, device="cuda")

    def step():
        hip.gqa_decode_dev(k, v, c["n_keys"], c["nkv"], c["hd"], q, c["nh"], c["scale"], out, stream)
    wall, kern = T.run(step)
    alg = 2 * 4096 * 4 * 256 * 2 + 8192 + 16384
    t = kern["gqa_decode_split_kernel"]["avg_us"] * 1e-6
    return {"workload": "cfg1 GQA decode 16q/4kv/hd256, 4096 keys bf16", "us_per_step": wall * 1e6,
            "kernels": kern, "alg_bytes": alg, "flops": 4 * 16 * 4096 * 256,
            "roofline": roofline("hbm", alg, t, HBM_PEAK_GBS, "GB/s"),
            "wall_GBps": alg / wall / 1e9}, (c, out)


def bench_cfg2(hip, synth, T, stream):
    import torch
    c = synth.cfg2_gqa_prefill()
    k, v, q = dev(c["k"]), dev(c["v"]), dev(c["q"])
    out = torch.empty((c["n"], c["nh"], c["hd"]), dtype=torch.float32, device="cuda")

    def step():
        hip.gqa_prefill_dev(k, v, 0, c["n"], c["nkv"], c["hd"], q, c["nh"], c["scale"], out, stream)
    wall, kern = T.run(step)
    n = c["n"]
    flops = 4 * c["nh"] * c["hd"] * n * (n + 1) // 2          # causal count
    t = kern["gqa_prefill_kernel"]["avg_us"] * 1e-6
    return {"workload": "cfg2 GQA causal prefill 8192 tokens 16q/4kv/hd256 bf16",
            "us_per_step": wall * 1e6, "kernels": kern, "flops": flops,
            "roofline": roofline("mfma", flops, t, BF16_PEAK_TFLOPS, "TFLOP/s"),
            "wall_TFLOPs": flops / wall / 1e12}, (c, out)


def bench_cfg3(hip, synth, T, stream):
    import torch
    c = synth.cfg3_mla_decode()
    rows, scales, q = dev(c["rows"]), dev(c["scales"]), dev(c["q"])
    out = torch.empty((c["nh"], 512), dtype=torch.float32, device="cuda")

    def step():
        hip.mla_decode_dev(rows, scales, 0, 0, c["n_keys"], 1, None, c["n_keys"], q, c["nh"],
                           c["scale"], out, stream)
    wall, kern = T.run(step)
    alg = 32768 * (576 + 20) + 128 * 576 * 2 + 128 * 512 * 4
    flops = 2 * 128 * 32768 * (576 + 512)
    t = kern["mla_roles_kernel"]["avg_us"] * 1e-6
    # HBM bytes of one launch of mla_roles_kernel at this geometry (64 key slices): FETCH_SIZE and
    # WRITE_SIZE of rocprofv3 --pmc, each scaled by what a 256 MiB copy reads on the same counter
    # (profiles/mla_decode_cfg3_pmc_traffic.txt): 21.00 MB read + 8.91 MB of split-K partials written
    traffic = 20512 * 1024 + 8704 * 1024
    return {"workload": "cfg3 MLA absorbed-latent decode, 128 heads, 32768 x 576 FP8-E4M3 latent "
                        "+ 5 fp32 block scales/token, bf16 q",
            "us_per_step": wall * 1e6, "kernels": kern, "alg_bytes": alg, "flops": flops,
            "roofline": roofline("hbm", alg, t, HBM_PEAK_GBS, "GB/s", traffic),
            "roofline_mfma": roofline("mfma", flops, t, BF16_PEAK_TFLOPS, "TFLOP/s"),
            "wall_GBps": alg / wall / 1e9}, (c, out)


def bench_cfg4(hip, synth, T, stream):
    import torch
    c = synth.cfg4_mla_prefill()
    rows, scales, q = dev(c["rows"]), dev(c["scales"]), dev(c["q"])
    out = torch.empty((c["n"], c["nh"], 512), dtype=torch.float32, device="cuda")

    def step():
        hip.mla_prefill_chunk_dev(rows, scales, c["pos0"], c["n"], q, c["nh"], c["scale"], out, stream)
    wall, kern = T.run(step)
    keys = c["n"] * c["pos0"] + c["n"] * (c["n"] + 1) // 2
    flops = 2 * c["nh"] * (576 + 512) * keys
    t = kern["mla_roles_kernel"]["avg_us"] * 1e-6
    return {"workload": "cfg4 MLA chunked prefill, 4096 queries appended to 28672 FP8 latent rows",
            "us_per_step": wall * 1e6, "kernels": kern, "flops": flops,
            "roofline": roofline("mfma", flops, t, BF16_PEAK_TFLOPS, "TFLOP/s"),
            "wall_TFLOPs": flops / wall / 1e12}, (c, out)


def bench_cfg5(hip, synth, T, stream):
    import torch
    c = synth.cfg5_dsa()
    B, N, K = c["batch"], c["n_keys"], c["topk"]
    ik, iks = dev(c["ikeys"]), dev(c["ikscale"])
    rows, scales = dev(c["rows"]), dev(c["scales"])
    qi, w, q = dev(c["q_idx"]), dev(c["w"]), dev(c["q"])
    sc = torch.empty((B, N), dtype=torch.float32, device="cuda")
    sel = torch.empty((B, K), dtype=torch.int32, device="cuda")
    out = torch.empty((B, c["nh"], 512), dtype=torch.float32, device="cuda")

    def step():
        hip.dsa_decode_dev(ik, iks, N * 128, N, rows, scales, N * 576, N * 5, B, N, qi, w, c["ih"],
                           K, q, c["nh"], c["scale"], sc, sel, out, stream)
    wall, kern = T.run(step)
    idx_bytes = B * N * 132
    idx_flops = B * 2 * c["ih"] * N * 128
    t_idx = kern["indexer kernels"]["avg_us"] * 1e-6
    t_mla = kern["mla_roles_kernel"]["avg_us"] * 1e-6
    mla_flops = B * 2 * 128 * K * 1088
    return {"workload": "cfg5 DSA decode, 8 independent queries (own caches): indexer 64x128 over "
                        "65536 FP8 keys -> exact top-2048 -> sparse MLA",
            "us_per_step": wall * 1e6, "us_per_query": wall * 1e6 / B, "kernels": kern,
            # the indexer phase of the fused call: approximate scores on the matrix cores (one pass
            # over the key bytes), the select on them, exact rescoring of the keys in the band
            "roofline": roofline("hbm", idx_bytes, t_idx, HBM_PEAK_GBS, "GB/s"),
            "roofline_indexer_mfma": roofline("mfma", idx_flops, t_idx, BF16_PEAK_TFLOPS, "TFLOP/s"),
            "roofline_sparse_mla_mfma": roofline("mfma", mla_flops, t_mla, BF16_PEAK_TFLOPS, "TFLOP/s"),
            "alg_bytes_indexer": idx_bytes}, (c, (out, sel))


# ---------------------------------------------------------------- CPU baseline (oracle, "port")
def cpu_baseline_cfg3(c, budget_s):
    """The oracle's restatement of src/attention.c:749-811 over BASELINE's FP8 storage, all
    host cores, bounded to about `budget_s` seconds of work."""
    from oracle import orc
    threads = min(orc.max_threads(), int(os.environ.get("CWICK_CPU_THREADS", "1000")))
    reps, t_total = 0, 0.0
    best = 1e30
    while (t_total < budget_s and reps < 30) or reps < 2:
        t0 = orc.now_ns()
        orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=threads)
        dt = (orc.now_ns() - t0) * 1e-9
        t_total += dt
        best = min(best, dt)
        reps += 1
    med = t_total / reps
    return {"value": round(med * 1e6, 1), "unit": "us/token", "cores": threads, "kind": "port",
            "sample": "%d full decodes of the same 32768-key workload (mean; best %.0f us), "
                      "position-sliced scores, head-sliced softmax, %d accumulation slices, "
                      "gcc -O2 -fopenmp, nproc=%d" % (reps, best * 1e6, threads, os.cpu_count()),
            "GBps": round((32768 * 596 + 147456 + 262144) / med / 1e9, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--configs", default="1,2,3,5",
                    help="which configurations to time besides the headline (cfg4 takes ~1 min)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run three plain 256 MiB device copies (a kernel of known HBM traffic, "
                         "to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters by)")
    a = ap.parse_args()
    if a.gpus != 1:
        log("bench.py: this build shows one GPU's share of the path; --gpus %d is not run "
            "(no collectives are part of it). Use --gpus 1." % a.gpus)
        return 2

    import torch
    from cwick_amd import hip, synth
    hip.lib()
    if not hip.ready():
        log("bench.py: libcwick_hip.so could not bring the GPU up: " + hip.last_error())
        return 1
    log("[device]", hip.device_info())
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    wanted = {int(x) for x in a.configs.split(",") if x} | {3}

    if a.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    results = {}
    # headline first: exactly K steps of cfg3
    T = Timer(hip, torch, a.steps, a.warmup)
    r3, (c3, _) = bench_cfg3(hip, synth, T, stream)
    results["cfg3"] = r3
    log("[cfg3] %.2f us/token wall, kernel %s" % (r3["us_per_step"], json.dumps(r3["kernels"])))
    cpu = None
    if not a.no_cpu:
        cpu = cpu_baseline_cfg3(c3, a.cpu_seconds)
        log("[cpu ] %.0f us/token on %d threads" % (cpu["value"], cpu["cores"]))
    del c3
    side = {1: (bench_cfg1, a.steps), 2: (bench_cfg2, max(3, a.steps // 20)),
            4: (bench_cfg4, max(2, a.steps // 100)), 5: (bench_cfg5, max(3, a.steps // 10))}
    for i in sorted(wanted - {3}):
        fn, k = side[i]
        Ti = Timer(hip, torch, k, max(1, min(a.warmup, k)))
        r, _ = fn(hip, synth, Ti, stream)
        r["steps"] = k
        results["cfg%d" % i] = r
        log("[cfg%d] %.2f us/step wall, kernels %s" % (i, r["us_per_step"], json.dumps(r["kernels"])))
        torch.cuda.empty_cache()

    line = {
        "metric": METRIC,
        "value": round(r3["us_per_step"], 3),
        "unit": "us/token",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(r3["us_per_step"] * 1e-3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8-e4m3 latent, bf16 q; bf16/fp16 MFMA, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": r3["workload"], "kernel_timing": "HIP events inside the library, "
                   "on the launch stream, second pass of the same K steps"},
        "decode_hbm_GBps_wall": round(r3["wall_GBps"], 1),
        "prefill_TFLOPs_8k": round(results["cfg2"]["wall_TFLOPs"], 1) if "cfg2" in results else None,
        "roofline": r3["roofline"],
        "roofline_mfma": r3["roofline_mfma"],
        "cpu_baseline": cpu,
        "configs": results,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
