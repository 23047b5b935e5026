#!/usr/bin/env python
"""bench.py -- attention hot path of libcwick_hip.so on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs 1,2,3,4,5] [--no-cold] [--no-cpu] [--no-check]

One JSON line on stdout.  `value` is the headline of BASELINE.json's metric: decode
attention microseconds per token at 32K context (configs[2]: MLA absorbed-latent decode,
128 heads, 32768 x 576 FP8-E4M3 latent), measured as wall time over exactly K steps with
every operand already resident in HBM.  The same line carries the HBM GB/s of that step,
the 8K causal GQA prefill TFLOP/s (configs[1]) and one entry per other configuration
under "configs", each with
  * its kernel times (start / stop events bound to each kernel's dispatch, inside the library)
    and roofline fraction against the published peak and against the ceiling measured in this
    run (a 128-bit grid-stride read, a loop of nothing but matrix instructions),
  * for the decode configurations a "cold" run beside the hot one: every step reads another
    copy of the caches (at least 16 copies, more than the 256 MB on-package cache in total), so
    the bytes come from HBM as they do when a layer loop walks through its layers,
  * "checked": sampled rows of the output the timed kernel left, compared with the CPU
    oracle after the timing,
  * "cpu_baseline": the oracle's restatement of the reference algorithm timed on this
    host's cores on a stated sub-sample of the same workload.

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
FP8_PEAK_TFLOPS = 5000.0       # dense fp8 MFMA, published

METRIC = "decode attn µs/token + HBM GB/s @32K ctx; prefill attn TFLOP/s @8K (1 GPU)"
ATOL, RTOL = 2e-3, 1e-2
CEIL = {}                      # measured ceilings of this run: hbm_GBps, bf16_TFLOPs, fp8_TFLOPs


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def dev(x):
    """numpy -> HBM (torch is only the allocator here)."""
    import torch
    if x.dtype == np.uint16:
        return torch.from_numpy(x.view(np.int16)).cuda()
    return torch.from_numpy(x).cuda()


def close(got, ref):
    d = float(np.abs(got - ref).max())
    m = float(np.abs(ref).max())
    return bool(np.isfinite(got).all() and d <= ATOL and d <= RTOL * m), d


class Timer:
    """Wall time of exactly K back-to-back steps with device syncs on both sides (host clock);
    then the same K steps again, each bracketed by a pair of events on the launch stream
    (per-step minimum, median and maximum) with the library's phase timers on.  step(i) gets the
    index of the step, so that a cold run can walk through its copies of the caches."""

    def __init__(self, hip, torch, steps, warmup):
        self.hip, self.torch, self.steps, self.warmup = hip, torch, steps, warmup

    def run(self, step):
        torch, hip = self.torch, self.hip
        for i in range(self.warmup):
            step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(self.steps):
            step(self.warmup + i)
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / self.steps
        hip.prof_reset()
        hip.prof_enable(True)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range(self.steps)]
        for i, (a, b) in enumerate(ev):
            a.record()
            step(self.warmup + self.steps + i)
            b.record()
        torch.cuda.synchronize()
        hip.prof_enable(False)
        per = sorted(a.elapsed_time(b) * 1e3 for a, b in ev)
        kern = {k: {"avg_us": round(1e3 * ms / n, 3), "launches": n}
                for k, (ms, n) in hip.prof_read().items() if n}
        spread = {"min": round(per[0], 2), "median": round(per[len(per) // 2], 2), "max": round(per[-1], 2),
                  "n": len(per)}
        return wall, kern, spread


COLD_BYTES = 320 << 20         # a cold run walks through copies of the caches adding up to at least this much


def n_copies(bytes_per_step):
    """Copies of a step's cache a cold run cycles through: at least 16, and more than the 256 MB
    of on-package cache in total, so that every step's rows come from HBM as a layer loop's do."""
    return max(16, -(-COLD_BYTES // int(bytes_per_step)) + 1)


def roofline(bound, alg, seconds, peak, unit, traffic=None, measured=None, note=None):
    """alg: algorithmic bytes (hbm) or flops (mfma) of ONE launch of the kernel."""
    ach = alg / seconds / (1e9 if unit == "GB/s" else 1e12)
    r = {"bound": bound, "achieved": round(ach, 2), "peak": peak, "unit": unit,
         "frac": round(ach / peak, 4), "traffic": traffic}
    if measured:
        r["measured_ceiling"] = round(measured, 1)
        r["frac_of_measured"] = round(ach / measured, 4)
    if note:
        r["peak_note"] = note
    return r


def cpu_threads(orc):
    return min(orc.max_threads(), int(os.environ.get("CWICK_CPU_THREADS", "1000")))


def timed(orc, fn, budget_s, min_reps=1, max_reps=30):
    reps, total, best = 0, 0.0, 1e30
    while (total < budget_s and reps < max_reps) or reps < min_reps:
        t0 = orc.now_ns()
        fn()
        dt = (orc.now_ns() - t0) * 1e-9
        total += dt
        best = min(best, dt)
        reps += 1
    return total / reps, best, reps


# ---------------------------------------------------------------- the five configurations
def bench_cfg1(hip, synth, orc, T, stream, a):
    import torch
    c = synth.cfg1_gqa_decode()
    k, v, q = dev(c["k"]), dev(c["v"]), dev(c["q"])
    out = torch.empty((c["nh"], c["hd"]), dtype=torch.float32, device="cuda")
    alg = 2 * 4096 * 4 * 256 * 2 + 8192 + 16384

    def run(ks, vs):
        def step(i):
            j = i % len(ks)
            hip.gqa_decode_dev(ks[j], vs[j], c["n_keys"], c["nkv"], c["hd"], q, c["nh"], c["scale"], out, stream)
        wall, kern, spread = T.run(step)
        t = kern["gqa_decode_split_kernel"]["avg_us"] * 1e-6
        tm = kern["splitk_merge_wide_kernel<gqa>"]["avg_us"] * 1e-6
        n_splits = 64
        part = n_splits * c["nh"] * (c["hd"] + 2) * 4
        return {"us_per_step": wall * 1e6, "step_us": spread, "kernels": kern,
                "roofline": roofline("hbm", alg, t, HBM_PEAK_GBS, "GB/s", measured=CEIL.get("hbm_GBps")),
                "roofline_merge": roofline("hbm", part + c["nh"] * c["hd"] * 4, tm, HBM_PEAK_GBS, "GB/s",
                                           note="the merge kernel's own bytes: %d slices of partials read, "
                                                "the output written" % n_splits),
                "roofline_token": roofline("hbm", alg, wall, HBM_PEAK_GBS, "GB/s",
                                           note="algorithmic bytes over the wall time of a whole token"),
                "wall_GBps": alg / wall / 1e9}
    r = {"workload": "cfg1 GQA decode 16q/4kv/hd256, 4096 keys bf16", "alg_bytes": alg, "flops": 4 * 16 * 4096 * 256}
    r.update(run([k], [v]))
    if not a.no_cold:
        nc = n_copies(k.numel() * 4)
        r["cold"] = run([k] + [k.clone() for _ in range(nc - 1)], [v] + [v.clone() for _ in range(nc - 1)])
        r["cold"]["copies"] = nc
        hip.gqa_decode_dev(k, v, c["n_keys"], c["nkv"], c["hd"], q, c["nh"], c["scale"], out, stream)
    if orc:
        ref = orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"], nthreads=0)
        r["checked"], r["check_maxabs"] = close(out.cpu().numpy(), ref)
        r["check"] = "the whole output against the oracle's decode"
        if not a.no_cpu:
            th = cpu_threads(orc)
            mean, best, reps = timed(orc, lambda: orc.gqa_decode(c["q"], c["k"], c["v"], c["scale"], 16, th), 1.0, 5)
            r["cpu_baseline"] = {"value": round(mean * 1e6, 1), "unit": "us/token", "cores": th, "kind": "port",
                                 "sample": "%d full decodes (mean; best %.0f us), position-sliced scores, "
                                           "16 accumulation slices (src/q35_model.c:1656-1701)" % (reps, best * 1e6)}
    return r


def bench_cfg2(hip, synth, orc, T, stream, a):
    import torch
    c = synth.cfg2_gqa_prefill()
    k, v, q = dev(c["k"]), dev(c["v"]), dev(c["q"])
    out = torch.empty((c["n"], c["nh"], c["hd"]), dtype=torch.float32, device="cuda")

    def step(i):
        hip.gqa_prefill_dev(k, v, 0, c["n"], c["nkv"], c["hd"], q, c["nh"], c["scale"], out, stream)
    wall, kern, spread = T.run(step)
    n = c["n"]
    flops = 4 * c["nh"] * c["hd"] * n * (n + 1) // 2          # causal count
    t = kern["gqa_prefill_kernel"]["avg_us"] * 1e-6
    r = {"workload": "cfg2 GQA causal prefill 8192 tokens 16q/4kv/hd256 bf16",
         "us_per_step": wall * 1e6, "step_us": spread, "kernels": kern, "flops": flops,
         "roofline": roofline("mfma", flops, t, BF16_PEAK_TFLOPS, "TFLOP/s", measured=CEIL.get("bf16_TFLOPs")),
         "roofline_median_launch": roofline("mfma", flops, spread["median"] * 1e-6, BF16_PEAK_TFLOPS, "TFLOP/s",
                                            measured=CEIL.get("bf16_TFLOPs")),
         "wall_TFLOPs": flops / wall / 1e12}
    if orc:
        rows = [0, 63, 64, 1023, 1024, 4097, 8128, 8191]
        got = out[rows].cpu().numpy()
        ok, worst = True, 0.0
        for i, t_ in enumerate(rows):
            ref = orc.gqa_decode(c["q"][t_], c["k"][:t_ + 1], c["v"][:t_ + 1], c["scale"], nthreads=0)
            o, d = close(got[i], ref)
            ok, worst = ok and o, max(worst, d)
        r["checked"], r["check_maxabs"] = ok, worst
        r["check"] = "rows %s of the timed output against the oracle's decode at that position" % rows
        if not a.no_cpu:
            th = cpu_threads(orc)
            tiles = [15, 47, 63]
            t0 = orc.now_ns()
            for tl in tiles:
                orc.gqa_prefill(c["q"], c["k"], c["v"], 0, c["scale"], tiles=(tl, tl + 1, 1), nthreads=th)
            dt = (orc.now_ns() - t0) * 1e-9
            fl = sum(4 * c["nh"] * c["hd"] * sum(range(128 * tl + 1, 128 * tl + 129)) for tl in tiles)
            r["cpu_baseline"] = {"value": round(fl / dt / 1e12, 4), "unit": "TFLOP/s (causal count)", "cores": th,
                                 "kind": "port",
                                 "sample": "query tiles %s of 64 (128 queries x 16 heads each, %.2f s): "
                                           "src/q35_model.c:1713-1746 per (head, tile) with its naive GEMM; "
                                           "the whole prefill would take about %.0f s at this rate"
                                           % (tiles, dt, flops / (fl / dt))}
    return r


def bench_cfg3(hip, synth, orc, T, stream, a):
    import torch
    c = synth.cfg3_mla_decode()
    rows, scales, q = dev(c["rows"]), dev(c["scales"]), dev(c["q"])
    out = torch.empty((c["nh"], 512), dtype=torch.float32, device="cuda")
    alg = 32768 * (576 + 20) + 128 * 576 * 2 + 128 * 512 * 4
    flops = 2 * 128 * 32768 * (576 + 512)
    traffic = profile_traffic("hot_kernels_pmc_traffic.txt")

    def run(rs, ss):
        def step(i):
            j = i % len(rs)
            hip.mla_decode_dev(rs[j], ss[j], 0, 0, c["n_keys"], 1, None, c["n_keys"], q, c["nh"],
                               c["scale"], out, stream)
        wall, kern, spread = T.run(step)
        t = kern["mla_roles_kernel"]["avg_us"] * 1e-6
        tm = kern["mla_merge_frag16_kernel"]["avg_us"] * 1e-6
        part = 64 * 128 * (512 * 2 + 4 * 16) + 128 * 512 * 4          # 64 slices of 16-bit partials + their scales, the output
        return {"us_per_step": wall * 1e6, "step_us": spread, "kernels": kern,
                "roofline": roofline("hbm", alg, t, HBM_PEAK_GBS, "GB/s", traffic, measured=CEIL.get("hbm_GBps")),
                "roofline_mfma": roofline(
                    "mfma", flops, t, BF16_PEAK_TFLOPS, "TFLOP/s", measured=CEIL.get("bf16_TFLOPs"),
                    note="algorithmic flops 2*128*32768*(576+512), each counted once, against the dense bf16/fp16 "
                         "peak: the value product runs on the fp16 matrix core; the score product runs on the "
                         "FP8 matrix core (published peak %.0f) with Q as two E4M3 terms, i.e. twice the "
                         "algorithmic score flops at twice the rate" % FP8_PEAK_TFLOPS),
                "roofline_merge": roofline("hbm", part, tm, HBM_PEAK_GBS, "GB/s",
                                           note="the merge kernel's own bytes: the split-K partials read, the output written"),
                "roofline_token": roofline("hbm", alg, wall, HBM_PEAK_GBS, "GB/s", measured=CEIL.get("hbm_GBps"),
                                           note="algorithmic bytes over the wall time of a whole token (both kernels "
                                                "and the dispatch between them)"),
                "wall_GBps": alg / wall / 1e9}
    r = {"workload": "cfg3 MLA absorbed-latent decode, 128 heads, 32768 x 576 FP8-E4M3 latent "
                     "+ 5 fp32 block scales/token, bf16 q", "alg_bytes": alg, "flops": flops}
    r.update(run([rows], [scales]))
    if not a.no_cold:
        nc = n_copies(rows.numel() + scales.numel() * 4)
        r["cold"] = run([rows] + [rows.clone() for _ in range(nc - 1)], [scales] + [scales.clone() for _ in range(nc - 1)])
        r["cold"]["copies"] = nc
    if orc:
        ref = orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"], nthreads=0)
        r["checked"], r["check_maxabs"] = close(out.cpu().numpy(), ref)
        r["check"] = "the whole output against the oracle's decode"
    return r, c


def profile_traffic(name):
    """HBM bytes per launch of the dominant kernel as the committed rocprofv3 --pmc summary states
    them (a line `traffic_bytes: N`), or None when the summary does not carry the line."""
    try:
        for line in open(os.path.join(ROOT, "profiles", name)):
            if line.startswith("traffic_bytes:"):
                return int(line.split(":")[1].split()[0])
    except OSError:
        pass
    return None


def bench_cfg4(hip, synth, orc, T, stream, a):
    import torch
    # the cache comes from the host generator; the 604 MB of queries are drawn on the device
    # (seeded N(0,1), rounded to bf16 with round-to-nearest-even) and only the sampled rows are
    # copied back for the check
    n, pos0, nh = 4096, 28672, 128
    g = synth.rng(synth.SEED0 + 4)
    rows_h, scales_h = synth.latent_cache(g, pos0 + n)
    rows, scales = dev(rows_h), dev(scales_h)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(synth.SEED0 + 4)
    q = torch.randn((n, nh, 576), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    out = torch.empty((n, nh, 512), dtype=torch.float32, device="cuda")
    scale = float(1.0 / np.sqrt(192.0))

    def step(i):
        hip.mla_prefill_chunk_dev(rows, scales, pos0, n, q.data_ptr(), nh, scale, out, stream)
    wall, kern, spread = T.run(step)
    keys = n * pos0 + n * (n + 1) // 2
    flops = 2 * nh * (576 + 512) * keys
    kname = "mla_prefill64_kernel" if "mla_prefill64_kernel" in kern else "mla_roles_kernel"
    t = kern[kname]["avg_us"] * 1e-6
    r = {"workload": "cfg4 MLA chunked prefill, 4096 queries appended to 28672 FP8 latent rows",
         "us_per_step": wall * 1e6, "step_us": spread, "kernels": kern, "flops": flops,
         "roofline": roofline("mfma", flops, t, BF16_PEAK_TFLOPS, "TFLOP/s", measured=CEIL.get("bf16_TFLOPs")),
         "wall_TFLOPs": flops / wall / 1e12}
    if orc:
        qs = [0, 63, 64, 2048, 4095]
        ok, worst = True, 0.0
        th = cpu_threads(orc)
        cpu_t, cpu_fl = 0.0, 0
        for t_ in qs:
            qh = q[t_].view(torch.int16).cpu().numpy().view(np.uint16)
            t0 = orc.now_ns()
            ref = orc.mla_decode(qh, rows_h, scales_h, scale, nlist=pos0 + t_ + 1, nthreads=th)
            cpu_t += (orc.now_ns() - t0) * 1e-9
            cpu_fl += 2 * nh * 1088 * (pos0 + t_ + 1)
            o, d = close(out[t_].cpu().numpy(), ref)
            ok, worst = ok and o, max(worst, d)
        r["checked"], r["check_maxabs"] = ok, worst
        r["check"] = "queries %s of the timed output against the oracle's decode at that position" % qs
        if not a.no_cpu:
            r["cpu_baseline"] = {"value": round(cpu_fl / cpu_t / 1e12, 4), "unit": "TFLOP/s", "cores": th,
                                 "kind": "port",
                                 "sample": "%d of the 4096 queries (%.2f s): the per-token loop of "
                                           "src/attention.c:1010-1019; the whole chunk would take about %.0f s "
                                           "at this rate" % (len(qs), cpu_t, flops / (cpu_fl / cpu_t))}
    return r


def bench_cfg5(hip, synth, orc, T, stream, a, shared=False):
    import torch
    c = synth.cfg5_dsa(shared=shared)
    B, N, K = c["batch"], c["n_keys"], c["topk"]
    ik, iks = dev(c["ikeys"]), dev(c["ikscale"])
    rows, scales = dev(c["rows"]), dev(c["scales"])
    qi, w, q = dev(c["q_idx"]), dev(c["w"]), dev(c["q"])
    sc = torch.empty((B, N), dtype=torch.float32, device="cuda")
    sel = torch.empty((B, K), dtype=torch.int32, device="cuda")
    out = torch.empty((B, c["nh"], 512), dtype=torch.float32, device="cuda")
    st = 0 if shared else 1

    idx_bytes = (1 if shared else B) * N * 132
    idx_flops = B * 2 * c["ih"] * N * 128
    mla_flops = B * 2 * 128 * K * 1088

    def run(sets):
        def step(i):
            ik_, iks_, rows_, scales_ = sets[i % len(sets)]
            hip.dsa_decode_dev(ik_, iks_, st * N * 128, st * N, rows_, scales_, st * N * 576, st * N * 5, B, N, qi, w,
                               c["ih"], K, q, c["nh"], c["scale"], sc, sel, out, stream)
        wall, kern, spread = T.run(step)
        t_idx = kern["indexer kernels"]["avg_us"] * 1e-6
        t_apx = kern["indexer_approx_kernel"]["avg_us"] * 1e-6
        t_mla = kern["mla_roles_kernel"]["avg_us"] * 1e-6
        return {"us_per_step": wall * 1e6, "us_per_query": wall * 1e6 / B, "step_us": spread, "kernels": kern,
                # the approximate scoring kernel: one pass over the key bytes
                "roofline": roofline("hbm", idx_bytes, t_apx, HBM_PEAK_GBS, "GB/s", measured=CEIL.get("hbm_GBps")),
                # the whole indexer phase of the fused call: approximate scores, the select on them,
                # exact rescoring of the keys in the band (several launches, dispatch latency included)
                "roofline_indexer_phase": roofline("hbm", idx_bytes, t_idx, HBM_PEAK_GBS, "GB/s"),
                "roofline_indexer_mfma": roofline("mfma", idx_flops, t_apx, BF16_PEAK_TFLOPS, "TFLOP/s"),
                "roofline_sparse_mla_mfma": roofline("mfma", mla_flops, t_mla, BF16_PEAK_TFLOPS, "TFLOP/s"),
                "roofline_step": roofline("hbm", idx_bytes + B * K * 596, wall, HBM_PEAK_GBS, "GB/s",
                                          note="key bytes and gathered latent rows over the wall time of a whole batch")}
    r = {"workload": "cfg5 DSA decode, 8 independent queries (%s): indexer 64x128 over 65536 FP8 keys -> "
                     "exact top-2048 -> sparse MLA" % ("one shared context" if shared else "own caches"),
         "alg_bytes_indexer": idx_bytes}
    r.update(run([(ik, iks, rows, scales)]))
    if not a.no_cold and not shared:
        nc = max(4, -(-COLD_BYTES // idx_bytes) + 1)
        sets = [(ik, iks, rows, scales)] + [(ik.clone(), iks.clone(), rows.clone(), scales.clone())
                                            for _ in range(nc - 1)]
        r["cold"] = run(sets)
        r["cold"]["copies"] = nc
        del sets
        hip.dsa_decode_dev(ik, iks, st * N * 128, st * N, rows, scales, st * N * 576, st * N * 5, B, N, qi, w,
                           c["ih"], K, q, c["nh"], c["scale"], sc, sel, out, stream)
    if orc:
        got_sel, got = sel.cpu().numpy(), out.cpu().numpy()
        ok, worst, th = True, 0.0, cpu_threads(orc)
        cpu_t = 0.0
        for b in (0, B - 1):
            cb = 0 if shared else b
            t0 = orc.now_ns()
            s_ = orc.indexer_scores(c["q_idx"][b], c["w"][b], c["ikeys"][cb], c["ikscale"][cb], nthreads=th)
            rsel = orc.topk_contract(s_, K)
            ref = orc.mla_decode(c["q"][b], c["rows"][cb], c["scales"][cb], c["scale"], sel=rsel, nthreads=th)
            cpu_t += (orc.now_ns() - t0) * 1e-9
            o, d = close(got[b], ref)
            ok = ok and o and bool(np.array_equal(got_sel[b], rsel))
            worst = max(worst, d)
        r["checked"], r["check_maxabs"] = ok, worst
        r["check"] = "queries 0 and %d: selected indices bit for bit, outputs against the oracle" % (B - 1)
        if not a.no_cpu:
            r["cpu_baseline"] = {"value": round(cpu_t / 2 * 1e6, 1), "unit": "us/query", "cores": th, "kind": "port",
                                 "sample": "2 of the 8 queries: indexer scores (src/attention.c:573-582), "
                                           "contract top-k, sparse decode (src/attention.c:749-811)"}
    return r


# ---------------------------------------------------------------- CPU baseline (oracle, "port")
def bench_cfg6(hip, synth, orc, T, stream, a):
    """Not one of the five configurations the metric names: the block-sparse GQA decode
    (src/mm_model.c:1962-2047 with its block selection, :1733-1780) at the reference's geometry,
    timed so that the kernels of that path have a committed command to profile."""
    import torch
    n, nh, nkv, hd, ih, idim, bs, keep = 65536, 64, 4, 128, 4, 128, 128, 16
    g = synth.rng(synth.SEED0 + 6)
    c = synth.cfg1_gqa_decode(n, nh, nkv, hd, seed=synth.SEED0 + 6)
    keys_h = synth.normal_bf16(g, (n, idim))
    iq_h = g.standard_normal((1, ih, idim)).astype(np.float32)
    k, v, q, keys, iq = dev(c["k"]), dev(c["v"]), dev(c["q"]), dev(keys_h), dev(iq_h)
    max_sel = (keep + 1) * bs
    sc = torch.empty((1, n), dtype=torch.float32, device="cuda")
    sel = torch.empty((1, max_sel), dtype=torch.int32, device="cuda")
    out = torch.empty((nh, hd), dtype=torch.float32, device="cuda")

    def step(i):
        hip.mm_select_dev(keys, iq, 1, n, ih, idim, bs, keep, sc, n, None, sel, max_sel, None, stream)
        hip.gqa_decode_sel_dev(k, v, n, nkv, hd, sel, max_sel, q, nh, c["scale"], out, stream)
    wall, kern, spread = T.run(step)
    # the selection reads every index key once; the attention reads the listed K and V rows
    alg_sel = n * idim * 2 + n * 4
    alg_att = 2 * max_sel * nkv * hd * 2
    ms = kern["mm select kernels"]
    t_sel = ms["avg_us"] * ms["launches"] / T.steps * 1e-6             # two timed sections per call
    r = {"workload": "block-sparse GQA decode 64q/4kv/hd128: 4x128 index scores over 65536 bf16 keys -> 16 of 512 "
                     "blocks + the newest -> attention over 2176 positions (outside BASELINE's five configurations)",
         "us_per_step": wall * 1e6, "step_us": spread, "kernels": kern,
         "alg_bytes_select": alg_sel, "alg_bytes_attention": alg_att,
         "roofline": roofline("hbm", alg_sel, t_sel, HBM_PEAK_GBS, "GB/s", measured=CEIL.get("hbm_GBps"))}
    if orc:
        _, rpos = orc.mm_select_blocks(orc.mm_index_scores(iq_h[0], keys_h), n, bs, keep, max_sel)
        got_sel = sel.cpu().numpy()[0]
        same = bool(np.array_equal(got_sel[:rpos.size], rpos) and (got_sel[rpos.size:] == -1).all())
        ref = orc.gqa_decode(c["q"], c["k"][rpos], c["v"][rpos], c["scale"], nthreads=0)
        ok, d = close(out.cpu().numpy(), ref)
        r["checked"], r["check_maxabs"] = bool(same and ok), d
        r["check"] = "the position list bit for bit, the output against the oracle's decode over the listed rows"
        if not a.no_cpu:
            th = cpu_threads(orc)

            def cpu_step():
                s_ = orc.mm_index_scores(iq_h[0], keys_h)
                _, pos = orc.mm_select_blocks(s_, n, bs, keep, max_sel)
                orc.gqa_decode(c["q"], c["k"][pos], c["v"][pos], c["scale"], 16, th)
            mean, best, reps = timed(orc, cpu_step, 2.0, 2)
            r["cpu_baseline"] = {"value": round(mean * 1e6, 1), "unit": "us/token", "cores": th, "kind": "port",
                                 "sample": "%d full steps (mean; best %.0f us): serial index scores on one thread "
                                           "(src/mm_model.c:1764-1780), block selection, attention over the listed rows"
                                           % (reps, best * 1e6)}
    return r


def cpu_baseline_cfg3(orc, c, budget_s):
    """The oracle's restatement of src/attention.c:749-811 over BASELINE's FP8 storage, all
    host cores, bounded to about `budget_s` seconds of work."""
    threads = cpu_threads(orc)
    mean, best, reps = timed(orc, lambda: orc.mla_decode(c["q"], c["rows"], c["scales"], c["scale"],
                                                         nthreads=threads), budget_s, 2)
    return {"value": round(mean * 1e6, 1), "unit": "us/token", "cores": threads, "kind": "port",
            "sample": "%d full decodes of the same 32768-key workload (mean; best %.0f us), "
                      "position-sliced scores, head-sliced softmax, %d accumulation slices, "
                      "gcc -O2 -fopenmp, nproc=%d" % (reps, best * 1e6, threads, os.cpu_count()),
            "GBps": round((32768 * 596 + 147456 + 262144) / mean / 1e9, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--configs", default="1,2,3,4,5",
                    help="which configurations to time besides the headline (3 always runs); 6 is the "
                         "block-sparse GQA decode, which the metric does not name")
    ap.add_argument("--no-cold", action="store_true",
                    help="skip the cold runs of the decode configurations (every step reads another copy of the "
                         "caches, more than the 256 MB on-package cache in total)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--no-check", action="store_true", help="skip the output checks (and the CPU baselines)")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the read and matrix-core probes")
    ap.add_argument("--cpu-seconds", type=float, default=6.0)
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
    orc = None
    if not a.no_check:
        from oracle import orc as _orc       # the checker and the reported CPU baseline, never the timed path
        orc = _orc
        orc.lib()
    else:
        a.no_cpu = True
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

    if not a.no_ceilings:
        CEIL["hbm_GBps"] = hip.probe_hbm_read(4 << 30, 5)
        CEIL["bf16_TFLOPs"] = hip.probe_mfma(0, 3)
        CEIL["fp8_TFLOPs"] = hip.probe_mfma(1, 3)
        log("[ceilings] read %.0f GB/s, bf16 MFMA %.0f TFLOP/s, fp8 MFMA %.0f TFLOP/s" %
            (CEIL["hbm_GBps"], CEIL["bf16_TFLOPs"], CEIL["fp8_TFLOPs"]))

    results = {}
    # headline first: exactly K steps of cfg3
    T = Timer(hip, torch, a.steps, a.warmup)
    r3, c3 = bench_cfg3(hip, synth, orc, T, stream, a)
    results["cfg3"] = r3
    log("[cfg3] %.2f us/token wall, kernel %s, checked %s" % (r3["us_per_step"], json.dumps(r3["kernels"]),
                                                              r3.get("checked")))
    cpu = None
    if not a.no_cpu:
        cpu = cpu_baseline_cfg3(orc, c3, a.cpu_seconds)
        r3["cpu_baseline"] = cpu
        log("[cpu ] %.0f us/token on %d threads" % (cpu["value"], cpu["cores"]))
    del c3
    # enough steps that the fixed cost of the two device syncs around the timed region (0.1 to 1 ms
    # on this stack, whatever is enqueued) stays below a per cent of the region
    side = {1: (bench_cfg1, max(200, a.steps)), 2: (bench_cfg2, max(50, a.steps // 4)),
            4: (bench_cfg4, max(3, a.steps // 50)), 5: (bench_cfg5, max(100, a.steps // 2)),
            6: (bench_cfg6, max(100, a.steps // 2))}
    for i in sorted(wanted - {3}):
        fn, k = side[i]
        Ti = Timer(hip, torch, k, max(1, min(a.warmup, k // 2)))
        r = fn(hip, synth, orc, Ti, stream, a)
        r["steps"] = k
        results["cfg%d" % i] = r
        log("[cfg%d] %.2f us/step wall, kernels %s, checked %s" % (i, r["us_per_step"], json.dumps(r["kernels"]),
                                                                   r.get("checked")))
        torch.cuda.empty_cache()
        if i == 5:
            r = bench_cfg5(hip, synth, orc, Ti, stream, a, shared=True)
            r["steps"] = k
            results["cfg5_shared_context"] = r
            log("[cfg5 shared] %.2f us/step wall, checked %s" % (r["us_per_step"], r.get("checked")))
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
        "dtype": "fp8-e4m3 latent, bf16 q; scores on the FP8 MFMA (Q as two E4M3 terms), values on the "
                 "fp16 MFMA, f32 accumulate (cfg1/cfg2: bf16 MFMA, f32 accumulate)",
        "data": "synthetic",
        "config": {"workload": r3["workload"],
                   "timing": "value: host clock over exactly K back-to-back steps between two device syncs, every "
                             "step reading the same cache (it stays in the 256 MB on-package cache); value_cold: the "
                             "same with every step reading another copy of the cache, as a layer loop does"},
        "kernel_us_source": "start and stop events bound to each kernel's own dispatch (hipExtLaunchKernel) on the "
                            "launch stream, second pass of the same K steps: the kernel's duration as rocprofv3 "
                            "--kernel-trace reports it, without the dispatch latency around it",
        "value_cold": round(r3["cold"]["us_per_step"], 3) if "cold" in r3 else None,
        "decode_hbm_GBps_wall": round(r3["wall_GBps"], 1),
        "decode_hbm_GBps_wall_cold": round(r3["cold"]["wall_GBps"], 1) if "cold" in r3 else None,
        "roofline_cold": r3["cold"]["roofline"] if "cold" in r3 else None,
        "prefill_TFLOPs_8k": round(results["cfg2"]["wall_TFLOPs"], 1) if "cfg2" in results else None,
        "checked": all(r.get("checked", False) for r in results.values()) if orc else None,
        "measured_ceilings": {k: round(v, 1) for k, v in CEIL.items()} or None,
        "roofline": r3["roofline"],
        "traffic_source": "profiles/hot_kernels_pmc_traffic.txt (rocprofv3 FETCH_SIZE + WRITE_SIZE of the same "
                          "command, scaled by a 256 MiB copy; not measured in this run)",
        "roofline_mfma": r3["roofline_mfma"],
        "cpu_baseline": cpu,
        "configs": results,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
