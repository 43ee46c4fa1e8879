#!/usr/bin/env python3
"""Benchmark of the fused-dequant hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--reps R] [--extras none|quick|full] [--out FILE]
    python bench.py --probe floor|c1|decode|prefill|quantize|w4a4|attention

The LAST line of stdout is the graded record: one JSON object of under 1.5 KB
(metric, value, ms_per_step, config, roofline, cpu_baseline and a dozen summary
scalars).  The detailed records come before it, one JSON line per section
({"section": ...}, each a few KB), and --out FILE writes everything as one
document.  The headline workload is the W4A16 symmetric gs=128,
M=1, N=K=4096 fused GEMM; one "step" is one call of w4_gemm on it.  After W
untimed warm-up steps the benchmark times R repetitions of exactly K steps each
(HIP events on the launch stream around a C launch loop, no interpreter between
launches); `ms_per_step` is the median repetition, every repetition is kept in
the `headline` section (`cold_reps_ms`).  `value` is the achieved HBM rate: algorithmic
bytes (packed codes + scales + x + c = 8 667 136 B) divided by that time, with
the weights rotated through enough distinct copies that no step finds its
matrix in the 256 MB last-level cache ("cold").

Every timed case first passes its gate at bench size on data quantized by the
CPU oracle from the distribution its config names: the dequant hook (w_out /
k_out / v_out) equals the oracle's bytes, the unhooked call is within rel L2
2e-3 of the hooked one (attention: the same bytes), and sampled outputs of both
are within rel L2 1e-3 of the FP64 oracle.  The same figure with one hot copy, the measured streaming
read and copy rates, the launch floor, the other configs of the scope table
and the CPU oracle's times for the same operations are the section lines.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
FINAL_LINE_MAX = 1536  # bytes: the graded record must survive a harness that keeps a short tail of stdout
MFMA_F16_PEAK_TFLOPS = 2500.0
PREWARM_LAUNCHES = 2000
TOL = 1e-3
CROSS_TOL = 2e-3  # between two gated GEMM paths (the reference's fused-vs-two-pass bound, tests/test_gpu.cu:184-193)
# HBM bytes one launch of the headline kernel moves, from two rocprofv3 --pmc runs
# of `python3 bench.py --probe c1` (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch
# of simt_rows4_kernel), each scaled by what the same counter reads for the 1 GiB
# stream_copy kernel of this file's yardstick (1 048 576 KiB each way); the
# figures and the commands are in profiles/simt_rows4_w4sym_gs128_m1_n4096_k4096.md.
HEADLINE_FETCH_KIB, HEADLINE_WRITE_KIB = 4290.5, 8.0
COPY_FETCH_FACTOR, COPY_WRITE_FACTOR = 2.0, 1.0
HEADLINE_TRAFFIC_BYTES = int((HEADLINE_FETCH_KIB * COPY_FETCH_FACTOR +
                              HEADLINE_WRITE_KIB * COPY_WRITE_FACTOR) * 1024)


def _pkg():
    import w4amd
    return w4amd.package()


def cpu_info():
    """Model name and core count of the host (the CPU legs run on one core of it)."""
    model, cores = "unknown", os.cpu_count() or 0
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = cores
    return {"model": model, "logical_cpus": cores, "usable_cpus": usable}


def _events_ms(torch, fn, steps, warmup):
    """Mean ms per call of fn(i) over `steps` back-to-back launches (HIP events
    on the launch stream, after `warmup` untimed calls)."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(steps):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


# After an idle gap (host-side checks, allocations) the device's clock governor takes
# 10 - 15 ms of continuous work to settle: measured on the W4 flash-decode kernel, calls
# 1.5 - 12 ms after the gap run 59 -> 68 - 74 us and then return to 59 us, where they stay
# for seconds of back-to-back calls; the decode-batch GEMMs show 8.9 -> 8.3 us.  Every
# timed region is therefore preceded by SETTLE_MS of the same calls, untimed, on top of
# the warm-up steps, so that the numbers are the steady state a serving loop sees.
SETTLE_MS = 60.0


def _settle(torch, run, ms_per_call):
    """`run(n)` issues n untimed calls; issue SETTLE_MS worth of them."""
    n = int(min(max(SETTLE_MS / max(ms_per_call, 1e-4), 1), 200000))
    run(n)
    torch.cuda.synchronize()


def _reps_ms(torch, fn, steps, warmup, reps=5):
    """(median, sorted raw list) of `reps` repetitions of _events_ms."""
    def run(n):
        for i in range(n):
            fn(i)
    _settle(torch, run, _events_ms(torch, fn, max(2, min(steps, 5)), warmup))
    raw = [_events_ms(torch, fn, steps, 2) for r in range(reps)]
    return sorted(raw)[reps // 2], raw


def _median_events_ms(torch, fn, steps, warmup, reps=5):
    return _reps_ms(torch, fn, steps, warmup, reps)[0]


class Bench:
    def __init__(self, steps, warmup, reps):
        import numpy as np
        import torch
        self.np, self.torch = np, torch
        self.capi = _pkg().capi
        self.capi.load()
        self.steps, self.warmup, self.reps = steps, warmup, reps
        self.stream = torch.cuda.current_stream().cuda_stream
        y = C.CDLL(os.path.join(ROOT, "w4a16-dequant-gemm_amd", "lib", "libw4bench.so"))
        vp, sz, ci = C.c_void_p, C.c_size_t, C.c_int
        y.w4bench_read.argtypes = [vp, sz, vp, ci, vp]
        y.w4bench_copy.argtypes = [vp, vp, sz, ci, vp]
        y.w4bench_gemm_loop.argtypes = [vp, vp, ci, vp, vp, ci, ci, vp]
        y.w4bench_w4a4_loop.argtypes = [vp, vp, ci, vp, vp, ci, vp]
        y.w4bench_probe_loop.argtypes = [ci, vp, ci, sz, ci, vp, ci, vp]
        y.w4bench_gemm_graph.argtypes = [vp, vp, ci, vp, vp, ci, ci, ci, ci, vp]
        y.w4bench_c1_timeline.argtypes = [vp, vp, vp, vp, ci, vp, vp]
        self.yard = y

    # -- timing of the GEMM entry points ----------------------------------------
    def loop_reps(self, entry, views, x_ptr, c_ptr, M, steps, warmup, reps):
        """ms per call over `steps` launches issued by a C loop, rotating through
        `views`; HIP events on the launch stream; returns the raw repetitions."""
        torch = self.torch
        fn = C.cast(getattr(self.capi.load(), entry), C.c_void_p)
        arr = (C.c_void_p * len(views))(*[C.addressof(v) for v in views])

        def run(n):
            rc = self.yard.w4bench_gemm_loop(fn, arr, len(views), x_ptr, c_ptr, M, n, self.stream)
            if rc:
                raise RuntimeError("gemm loop failed: %d" % rc)
        def timed(n):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            run(n)
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n
        run(warmup)
        torch.cuda.synchronize()
        _settle(torch, run, timed(max(2, min(steps, 20))))
        return [timed(steps) for _ in range(reps)]

    def loop_ms(self, entry, views, x_ptr, c_ptr, M, steps, warmup, reps=5):
        raw = self.loop_reps(entry, views, x_ptr, c_ptr, M, steps, warmup, reps)
        return sorted(raw)[len(raw) // 2]

    def gemm_us(self, fn, views, x, c, M):
        """(median us, raw us list) per call, rotating through `views`."""
        raw = self.loop_reps(fn, views, x.data_ptr(), c.data_ptr(), M, self.steps, self.warmup, 5)
        return sorted(raw)[2] * 1e3, [r * 1e3 for r in raw]

    def w4a4_us(self, views, M, N, K, reps=5, a8=False):
        """us per w4_gemm_mx_w4a4 (a8: w4_gemm_mx_w4a8) call over rotating weight copies."""
        torch = self.torch
        if a8:
            xq = torch.randint(0, 0x78, (M * K,), dtype=torch.uint8, device="cuda")
            xs = torch.randint(118, 123, (M * (K // 32),), dtype=torch.uint8, device="cuda")
            xv = (self.capi.act_mx8_view(M, K, K // 32, xq.data_ptr(), xs.data_ptr()), (xq, xs))
        else:
            xv = self.rand_mx(M, K, 1)[0]
        c = torch.empty(M * N, dtype=torch.float16, device="cuda")
        fn = C.cast(self.capi.load().w4_gemm_mx_w4a8 if a8 else self.capi.load().w4_gemm_mx_w4a4,
                    C.c_void_p)
        arr = (C.c_void_p * len(views))(*[C.addressof(v[0]) for v in views])

        def run(n):
            rc = self.yard.w4bench_w4a4_loop(fn, arr, len(views), C.addressof(xv[0]), c.data_ptr(), n,
                                             self.stream)
            if rc:
                raise RuntimeError("w4a4 loop failed: %d" % rc)
        def timed(n):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            run(n)
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n
        run(self.warmup)
        torch.cuda.synchronize()
        _settle(torch, run, timed(max(2, min(self.steps, 10))))
        out = [timed(self.steps) * 1e3 for _ in range(reps)]
        return sorted(out)[len(out) // 2]

    # -- yardsticks ---------------------------------------------------------
    def bandwidth(self):
        torch = self.torch
        n = 1 << 30
        src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")

        def rd(i):
            assert self.yard.w4bench_read(src.data_ptr(), n, sink.data_ptr(), 2048, self.stream) == 0

        def cp(i):
            assert self.yard.w4bench_copy(src.data_ptr(), dst.data_ptr(), n, 4096, self.stream) == 0
        rd_ms, rd_raw = _reps_ms(torch, rd, 10, 3, 7)
        cp_ms, cp_raw = _reps_ms(torch, cp, 10, 3, 7)
        return {"read_GBs": n / rd_ms * 1e-6, "copy_GBs": 2 * n / cp_ms * 1e-6,
                "read_reps_ms": rd_raw, "copy_reps_ms": cp_raw, "bytes": n,
                "kernels": "stream_read / stream_copy: one contiguous chunk per workgroup, 8 dwordx4 in flight per lane"}

    # -- launch floor ---------------------------------------------------------
    def launch_floor(self, srcs_c1, bytes_c1, srcs_c2, bytes_c2):
        """Launch-to-launch us of a kernel that does nothing and of one that only reads
        the weight matrix (grid and access pattern of the decode-shape vector kernel),
        on C1's matrix (8 MiB, 256 workgroups) and C2's (21.5 MiB, 688 workgroups)."""
        torch = self.torch
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        out = {}
        for name, kind, srcs, nbytes, blocks in (("empty_256wg", 0, srcs_c1, 0, 256), ("empty_688wg", 0, srcs_c1, 0, 688),
                                                 ("read_c1_8MiB", 1, srcs_c1, bytes_c1, 0),
                                                 ("read_c2_21MiB", 1, srcs_c2, bytes_c2, 0)):
            if kind == 1 and not srcs:
                continue
            arr = (C.c_void_p * max(1, len(srcs)))(*[t.data_ptr() for t in srcs]) if srcs else (C.c_void_p * 1)()

            def run(n):
                rc = self.yard.w4bench_probe_loop(kind, arr, max(1, len(srcs)), nbytes, blocks, sink.data_ptr(), n,
                                                  self.stream)
                if rc:
                    raise RuntimeError("probe loop failed: %d" % rc)
            run(50)
            torch.cuda.synchronize()
            _settle(torch, run, 0.003)
            raw = []
            for _ in range(7):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                run(200)
                b.record()
                torch.cuda.synchronize()
                raw.append(a.elapsed_time(b) / 200 * 1e3)
            out[name + "_us"] = sorted(raw)[3]
            out[name + "_reps_us"] = raw
        return out

    def c1_timeline(self, dp_list, x_d, c_d, N):
        """Time stamps from inside the waves of the headline kernel (its time-stamped
        instantiation in libw4bench.so), one cold launch after ten ordinary ones: percentiles
        over the N / 4 waves, in ns since the first wave started."""
        np, torch = self.np, self.torch
        from devutil import ptr
        slots = self.yard.w4bench_c1_timeline_slots()
        nw = N // 4
        stamps = torch.zeros(nw * slots, dtype=torch.int64, device="cuda")
        runs = []
        for rep in range(3):
            for i in range(10):
                d = dp_list[i % len(dp_list)]
                self.capi.gemm(d.view, ptr(x_d), ptr(c_d), 1, self.stream, 0)
            d = dp_list[(11 + rep) % len(dp_list)]
            rc = self.yard.w4bench_c1_timeline(ptr(d.q), ptr(d.s), ptr(x_d), ptr(c_d), N, stamps.data_ptr(),
                                               self.stream)
            if rc:
                raise RuntimeError("timeline probe failed: %d" % rc)
            torch.cuda.synchronize()
            t = stamps.cpu().numpy().reshape(nw, slots).astype(np.int64)
            t0 = t[:, 0].min()
            ns = (t[:, :14] - t0) * 10
            names = ["wave_start", "requests_issued", "activations_landed", "group_params_read"] + \
                    ["run%d_landed" % i for i in range(8)] + ["arithmetic_done", "reduced"]
            pct = {n: {"p10": int(np.percentile(ns[:, j], 10)), "p50": int(np.percentile(ns[:, j], 50)),
                       "p90": int(np.percentile(ns[:, j], 90)), "max": int(ns[:, j].max())}
                   for j, n in enumerate(names)}
            die = t[:, slots - 1]
            per_die = {int(x): {"wave_start_p50": int(np.median(ns[die == x, 0])),
                                "first_weights_p50": int(np.median(ns[die == x, 4])),
                                "reduced_p50": int(np.median(ns[die == x, 13])),
                                "reduced_max": int(ns[die == x, 13].max())} for x in np.unique(die)}
            runs.append({"percentiles_ns": pct, "per_compute_die_ns": per_die})
        return {"waves": nw, "tick_ns": 10, "launches": runs}

    # -- synthetic packed weights on device (timing-only cases) --------------------
    def rand_mx(self, N, K, copies=1):
        torch, capi = self.torch, self.capi
        B, wk = (K + 31) // 32, (K + 7) // 8
        out = []
        for _ in range(copies):
            q = torch.randint(-2**31, 2**31 - 1, (N * wk,), dtype=torch.int32, device="cuda")
            s = torch.randint(118, 123, (N * B,), dtype=torch.uint8, device="cuda")
            out.append((capi.packed_mx_view(N, K, B, q.data_ptr(), s.data_ptr()), (q, s)))
        return out


def w4_bytes(N, K, gs, sym, M):
    G = (K + gs - 1) // gs
    b = N * ((K + 7) // 8) * 4 + N * G * 2 + 2 * M * K + 2 * M * N
    if not sym:
        b += N * ((G + 7) // 8) * 4
    return b


def mx_bytes(N, K, M):
    return N * ((K + 7) // 8) * 4 + N * ((K + 31) // 32) + 2 * M * K + 2 * M * N


# The configs' data distributions (10 % one-sided groups; 1 % outliers at 20 sigma) are
# orc.one_sided_group_weights and orc.outlier_weights, shared with the test suite.


def quant_rel_l2(np, w, w16):
    d = w16.view(np.float16).astype(np.float64) - w
    return float(np.sqrt(np.sum(d * d) / np.sum(w * w)))


class Gate:
    """Bench-size correctness gate of one packed matrix: hook bytes against the oracle's
    dequant (bit-exact), unhooked output within CROSS_TOL of the hooked output, sampled rows of
    both within TOL of the FP64 oracle."""

    def __init__(self, b, mx, p, w_ref, N, K):
        self.b, self.mx, self.p, self.w_ref, self.N, self.K = b, mx, p, w_ref, N, K
        np = b.np
        self.rows = np.sort(np.random.default_rng(N * 31 + K).choice(N, size=min(N, 192), replace=False))
        self.w_rows = np.ascontiguousarray(w_ref.reshape(N, K)[self.rows])
        from devutil import to_dev
        self.w_ref_d = to_dev(w_ref)  # the oracle's dequantized matrix, compared on the device
        self.results = []

    def check(self, entry, view, x_host, x_d, M, label):
        import orc
        from devutil import bits, halves, ptr
        np, capi = self.b.np, self.b.capi
        N, K = self.N, self.K
        fn = getattr(capi, entry)
        c_h, w_d = halves(M * N, 0x7E00), halves(N * K, 0x7E00)
        fn(view, ptr(x_d), ptr(c_h), M, self.b.stream, ptr(w_d))
        hook_ok = bool(self.b.torch.equal(w_d, self.w_ref_d))
        del w_d
        c_u = halves(M * N, 0x7E00)
        fn(view, ptr(x_d), ptr(c_u), M, self.b.stream, 0)
        got_h, got_u = bits(c_h), bits(c_u)
        fh, fu = got_h.view(np.float16).astype(np.float64), got_u.view(np.float16).astype(np.float64)
        cross = float(np.sqrt(np.sum((fu - fh) ** 2) / max(np.sum(fh * fh), 1e-300)))
        ms = min(M, 16)  # activation rows sampled for the FP64 oracle
        xs = np.ascontiguousarray(x_host.reshape(M, K)[:ms])
        ref = orc.gemm_oracle(xs, ms, K, self.w_rows, len(self.rows))
        got = got_u.view(np.float16).reshape(M, N)[:ms][:, self.rows]
        rel = orc.rel_l2(got, ref)
        got_hk = got_h.view(np.float16).reshape(M, N)[:ms][:, self.rows]
        rel_h = orc.rel_l2(got_hk, ref)
        ok = hook_ok and cross <= CROSS_TOL and rel <= TOL and rel_h <= TOL
        self.results.append({"case": label, "hook_bitwise": hook_ok, "unhooked_vs_hooked_rel_l2": cross,
                             "rel_l2_sampled": rel, "rel_l2_sampled_hooked": rel_h, "ok": ok})
        if not ok:
            raise RuntimeError("bench-size gate failed: %s" % json.dumps(self.results[-1]))
        return ok


def headline(b, args):
    """C1 on the GPU: real quantized weights (hook checked against the oracle at
    bench size), cold-rotated and warm timings, CPU legs."""
    import orc
    np, torch, capi = b.np, b.torch, b.capi
    from devutil import DevPacked, ptr, to_dev
    N = K = 4096
    gs, M = 128, 1
    w = orc.normal_weights(N * K, 0xB46E) * 0.02
    t0 = time.perf_counter()
    p = orc.quantize(w, N, K, gs, True)
    t_quant = time.perf_counter() - t0
    t0 = time.perf_counter()
    w_ref = orc.dequant_all(p)
    t_deq = time.perf_counter() - t0
    x = orc.normal_activations(M * K, 0xB46F)
    t0 = time.perf_counter()
    orc.gemm_oracle(x, M, K, w_ref, N)
    t_gemm = time.perf_counter() - t0
    # bounded CPU sample: repeat dequant_all + gemm_oracle (the CPU equivalent of
    # one fused call) a few more times and keep the median
    cpu = [t_deq + t_gemm]
    for _ in range(4):
        t0 = time.perf_counter()
        orc.gemm_oracle(x, M, K, orc.dequant_all(p), N)
        cpu.append(time.perf_counter() - t0)
    cpu_s = sorted(cpu)[len(cpu) // 2]
    # the MXFP4 leg on the same matrix (quantize_mx + dequant_all_mx), once
    t0 = time.perf_counter()
    pm = orc.quantize_mx(w, N, K)
    t_qmx = time.perf_counter() - t0
    t0 = time.perf_counter()
    orc.dequant_all_mx(pm)
    t_dmx = time.perf_counter() - t0
    del pm

    dp = DevPacked(p)
    x_d = to_dev(x)
    gate = Gate(b, False, p, w_ref, N, K)
    gate.check("gemm", dp.view, x, x_d, M, "c1 w4 sym gs128 M=1")
    from devutil import halves
    c_d = halves(M * N, 0x7E00)

    nbytes = w4_bytes(N, K, gs, True, M)
    copies = max(2, int(400e6 // nbytes) + 1)  # ~400 MB of distinct weights
    dps = [dp] + [DevPacked(p) for _ in range(copies - 1)]
    vlist = [d.view for d in dps]
    # bring the clocks up before the timed region: the first few hundred launches after idle run
    # ~20 % slower.  Untimed, same kernel and workload as the timed steps.
    b.loop_reps("w4_gemm", vlist, ptr(x_d), ptr(c_d), M, PREWARM_LAUNCHES, 0, 1)
    # the timed region: W warm-up launches, then `reps` repetitions of exactly K steps
    cold = b.loop_reps("w4_gemm", vlist, ptr(x_d), ptr(c_d), M, args.steps, args.warmup, args.reps)
    more = {}
    if args.extras != "none":
        warm = b.loop_reps("w4_gemm", vlist[:1], ptr(x_d), ptr(c_d), M, args.steps, args.warmup, 5)
        more["warm_reps_ms"] = warm
        more["warm_ms"] = sorted(warm)[2]
    res = {
        "N": N, "K": K, "gs": gs, "M": M, "bytes": nbytes, "copies": copies,
        "cold_ms": sorted(cold)[len(cold) // 2], "cold_reps_ms": cold, **more,
        "gate": gate.results,
        "cpu": {"quantize_s": t_quant, "dequant_all_s": t_deq, "gemm_oracle_s": t_gemm,
                "fused_equiv_s": cpu_s, "quantize_mx_s": t_qmx, "dequant_all_mx_s": t_dmx},
    }
    return res, dps, x_d, c_d


def extras_floor(b, dps, x_d, c_d, with_c2=True):
    """Launch floor (empty / read-only kernels) and the in-kernel timeline of the headline."""
    torch = b.torch
    srcs_c1 = [d.q for d in dps]
    srcs_c2, bytes_c2 = [], 11008 * 512 * 4
    if with_c2:
        for _ in range(19):  # 19 x 21.5 MiB > 400 MB
            srcs_c2.append(torch.randint(-2**31, 2**31 - 1, (bytes_c2 // 4,), dtype=torch.int32, device="cuda"))
    out = {"launch_floor": b.launch_floor(srcs_c1, 4096 * 512 * 4, srcs_c2, bytes_c2)}
    del srcs_c2
    torch.cuda.empty_cache()
    out["c1_timeline"] = b.c1_timeline(dps, x_d, c_d, 4096)
    # the headline's launches replayed from a HIP graph (200 kernel nodes, one graph launch per
    # repetition): what is left of the launch-to-launch interval when the host issues nothing
    from devutil import ptr
    fn = C.cast(b.capi.load().w4_gemm, C.c_void_p)
    arr = (C.c_void_p * len(dps))(*[C.addressof(d.view) for d in dps])
    ms = (C.c_float * 9)()
    rc = b.yard.w4bench_gemm_graph(fn, arr, len(dps), ptr(x_d), ptr(c_d), 1, 200, 40, 9, ms)
    if rc:
        raise RuntimeError("graph replay failed: %d" % rc)
    reps = [m / 200 * 1e3 for m in ms]
    out["launch_floor"]["headline_graph_replay_us"] = sorted(reps)[4]
    out["launch_floor"]["headline_graph_replay_reps_us"] = reps
    return out


def extras_gemm(b, full):
    """Configs 2-4: per-M timings of both kernels (crossover), MXFP4, prefill; every case gated."""
    import orc
    from devutil import DevPacked, DevPackedMx, halves, ptr, to_dev
    np, capi, torch = b.np, b.capi, b.torch
    out = {}
    # C2: asymmetric N=11008; K=4096 with gs 32 / 48 / 128, K=4104 with gs 8
    rows, gates = [], []
    shapes = [(11008, 4096, 128), (11008, 4096, 32), (11008, 4096, 48), (11008, 4104, 8)]
    for si, (N, K, gs) in enumerate(shapes):
        w = orc.one_sided_group_weights(N, K, gs, 0xC2C2 + si)
        p = orc.quantize(w, N, K, gs, False)
        w_ref = orc.dequant_all(p)
        qerr = quant_rel_l2(np, w, w_ref)
        del w
        copies = max(2, int(400e6 // w4_bytes(N, K, gs, False, 1)) + 1)
        dps = [DevPacked(p) for _ in range(copies)]
        views = [d.view for d in dps]
        gate = Gate(b, False, p, w_ref, N, K)
        for M in (1, 2, 4, 8, 9, 16, 64):
            x = orc.normal_activations(M * K, 0xC2C2 + 100 * si + M)
            x_d, c_d = to_dev(x), halves(M * N, 0x7E00)
            gate.check("gemm_fused", dps[0].view, x, x_d, M, "c2 gs%d K%d simt M=%d" % (gs, K, M))
            gate.check("gemm_mma", dps[0].view, x, x_d, M, "c2 gs%d K%d mfma M=%d" % (gs, K, M))
            nb = w4_bytes(N, K, gs, False, M)
            # the vector kernel re-reads the weights per 4 activation rows: its time past the
            # crossover is recorded at M = 8 and 16 only (it is 0.2 ms per call at M = 64)
            us_s, raw_s = b.gemm_us("w4_gemm_fused", views, x_d, c_d, M) if M <= 16 else (None, None)
            us_m, raw_m = b.gemm_us("w4_gemm_mma", views, x_d, c_d, M)
            best = min(u for u in (us_s, us_m) if u)
            rows.append({"N": N, "K": K, "gs": gs, "M": M, "bytes": nb, "simt_us": us_s, "mfma_us": us_m,
                         "simt_reps_us": raw_s, "mfma_reps_us": raw_m,
                         "best_GBs": nb / best * 1e-3, "frac_of_hbm_peak": nb / best * 1e-3 / HBM_PEAK_GBS,
                         "winner": "simt" if us_s is not None and us_s <= us_m else "mfma",
                         "dispatcher": "simt" if M < capi.load().w4_dispatch_mma_min_m_for_gs(N, K, gs) else "mfma"})
        gates.append({"N": N, "K": K, "gs": gs, "quant_rel_l2": qerr, "cases": gate.results})
        del dps, views, gate, w_ref, p
        torch.cuda.empty_cache()
    out["c2_w4_asym"] = rows
    out["c2_gates"] = gates
    # C3: MXFP4 N=14336 K=4096, 1 % outliers; format error against W4 gs=128 on the same W
    rows = []
    N, K = 14336, 4096
    w = orc.outlier_weights(N, K, 0xE40F)
    t0 = time.perf_counter()
    p = orc.quantize_mx(w, N, K)
    t_qmx = time.perf_counter() - t0
    t0 = time.perf_counter()
    w_ref = orc.dequant_all_mx(p)
    t_dmx = time.perf_counter() - t0
    fmt = {"mxfp4_rel_l2": quant_rel_l2(np, w, w_ref),
           "w4_sym_gs128_rel_l2": quant_rel_l2(np, w, orc.dequant_all(orc.quantize(w, N, K, 128, True))),
           "cpu_quantize_mx_s": t_qmx, "cpu_dequant_all_mx_s": t_dmx}
    del w
    dps = [DevPackedMx(p) for _ in range(max(2, int(400e6 // mx_bytes(N, K, 1)) + 1))]
    views = [d.view for d in dps]
    gate = Gate(b, True, p, w_ref, N, K)
    for M in (1, 16, 128):
        x = orc.normal_activations(M * K, 0xE40F + M)
        x_d, c_d = to_dev(x), halves(M * N, 0x7E00)
        if M <= 16:
            gate.check("gemm_fused_mx", dps[0].view, x, x_d, M, "c3 mx simt M=%d" % M)
        gate.check("gemm_mma_mx", dps[0].view, x, x_d, M, "c3 mx mfma M=%d" % M)
        nb = mx_bytes(N, K, M)
        us_s, raw_s = b.gemm_us("w4_gemm_fused_mx", views, x_d, c_d, M) if M <= 16 else (None, None)
        us_m, raw_m = b.gemm_us("w4_gemm_mma_mx", views, x_d, c_d, M)
        best = min(u for u in (us_s, us_m) if u)
        rows.append({"N": N, "K": K, "M": M, "bytes": nb, "simt_us": us_s, "mfma_us": us_m,
                     "simt_reps_us": raw_s, "mfma_reps_us": raw_m,
                     "best_GBs": nb / best * 1e-3, "frac_of_hbm_peak": nb / best * 1e-3 / HBM_PEAK_GBS,
                     "mfma_TFLOPs": 2.0 * M * N * K / us_m * 1e-6})
    out["c3_mxfp4"] = rows
    out["c3_format"] = fmt
    out["c3_gates"] = gate.results
    del dps, views, gate, w_ref, p
    torch.cuda.empty_cache()
    # C4: prefill M=2048, N=K=4096 + two-pass baseline (dequant + hipBLASLt), C1's weights
    N = K = 4096
    M = 2048
    p = orc.quantize(orc.normal_weights(N * K, 0xB46E) * 0.02, N, K, 128, True)
    w_ref = orc.dequant_all(p)
    dp = DevPacked(p)
    xh = orc.normal_activations(M * K, 0xC4C4)
    x = to_dev(xh)
    gate = Gate(b, False, p, w_ref, N, K)
    gate.check("gemm", dp.view, xh, x, M, "c4 w4 sym gs128 M=2048")
    c = torch.empty(M * N, dtype=torch.float16, device="cuda")
    w16 = torch.empty(N * K, dtype=torch.float16, device="cuda")
    st = b.stream
    steps = max(5, b.steps // 10)
    fused_ms, fused_raw = _reps_ms(torch, lambda i: capi.gemm(dp.view, x.data_ptr(), c.data_ptr(), M, st, 0),
                                   steps, 3, 9)

    def two_pass(i):
        capi.dequant(dp.view, w16.data_ptr(), st)
        capi.gemm_fp16(w16.data_ptr(), x.data_ptr(), c.data_ptr(), M, N, K, st)
    two_ms, two_raw = _reps_ms(torch, two_pass, steps, 3, 9)
    blas_ms = _median_events_ms(torch, lambda i: capi.gemm_fp16(w16.data_ptr(), x.data_ptr(), c.data_ptr(),
                                                                M, N, K, st), steps, 3)
    flop = 2.0 * M * N * K
    out["c4_prefill"] = {"M": M, "N": N, "K": K, "flop": flop, "fused_ms": fused_ms, "fused_reps_ms": fused_raw,
                         "fused_TFLOPs": flop / fused_ms * 1e-9, "two_pass_ms": two_ms, "two_pass_reps_ms": two_raw,
                         "two_pass_TFLOPs": flop / two_ms * 1e-9, "hipblaslt_only_TFLOPs": flop / blas_ms * 1e-9,
                         "frac_of_mfma_peak": flop / fused_ms * 1e-9 / MFMA_F16_PEAK_TFLOPS,
                         "gate": gate.results}
    # the same weights at other M: fused against two-pass (dequant + hipBLASLt)
    rows = []
    for M2 in (256, 512, 1024, 4096, 8192) if full else (256, 1024, 4096):
        x2 = torch.randn(M2 * K, device="cuda").to(torch.float16)
        c2 = torch.empty(M2 * N, dtype=torch.float16, device="cuda")
        ms = _median_events_ms(torch, lambda i: capi.gemm(dp.view, x2.data_ptr(), c2.data_ptr(), M2, st, 0),
                               steps, 3)

        def two(i):
            capi.dequant(dp.view, w16.data_ptr(), st)
            capi.gemm_fp16(w16.data_ptr(), x2.data_ptr(), c2.data_ptr(), M2, N, K, st)
        ms2 = _median_events_ms(torch, two, steps, 3)
        rows.append({"weights": "w4_sym_gs128", "M": M2, "fused_us": ms * 1e3, "two_pass_us": ms2 * 1e3,
                     "fused_TFLOPs": 2.0 * M2 * N * K / ms * 1e-9})
    out["c4_prefill_other_M"] = rows
    if True:
        # the down-projection side of the MLP shapes (long K) through the dispatcher: timing
        # only, on random codes (the parity tests hold these shapes against the oracle)
        rows = []
        # (8192 x 8192: more 16-row tiles than compute units, where from 17 activation rows on two
        # tiles share a workgroup's activations)
        for (N2, K2) in ((4096, 11008), (4096, 14336), (8192, 8192)):
            vs = [v[0] for v in rand_w4_views(b, N2, K2, 128, True, 10 if N2 == 4096 else 6)]
            for M2 in (1, 2, 4, 8, 16, 32, 64) if full else (1, 4, 16, 64):
                x2 = torch.randn(M2 * K2, device="cuda").to(torch.float16)
                c2 = torch.empty(M2 * N2, dtype=torch.float16, device="cuda")
                us, raw = b.gemm_us("w4_gemm", vs, x2, c2, M2)
                nb = w4_bytes(N2, K2, 128, True, M2)
                rows.append({"N": N2, "K": K2, "gs": 128, "M": M2, "us": us, "reps_us": raw, "bytes": nb,
                             "GBs": nb / us * 1e-3,
                             "dispatcher": "simt" if M2 < capi.load().w4_dispatch_mma_min_m_for(N2, K2) else "mfma"})
            del vs
            torch.cuda.empty_cache()
        out["long_k_w4_sym_gs128"] = rows
    return out


def _slab_cache(b, kind, NS, S, D, gs, seed):
    """NS sample slabs of K/V ~ N(0,1) quantized by the oracle (kind: 'w4' | 'f8'), their
    dequantized halves and the timing of the CPU leg."""
    import orc
    k = orc.normal_weights(NS * S * D, seed)
    v = orc.normal_weights(NS * S * D, seed + 1)
    t0 = time.perf_counter()
    c = orc.quantize_cache(k, v, NS, S, D, gs, True) if kind == "w4" else orc.quantize_cache_f8(k, v, NS, S, D, gs)
    tq = time.perf_counter() - t0
    if kind == "w4":
        kd, vd = orc.dequant_cache(c, False), orc.dequant_cache(c, True)
    else:
        kd, vd = orc.dequant_cache_f8(c, False), orc.dequant_cache_f8(c, True)
    return c, kd, vd, tq


def extras_attention(b, full):
    """Config 5: B=8, Hq=32, Hkv=8, D=128, S=32768, one query token per sequence.  The cache of
    (sequence s, kv-head h) is sample slab h % 4 of four slabs quantized by the CPU oracle, so
    hooks and outputs are checked at bench size against four slabs' worth of oracle work; every
    format is timed over two distinct device copies of its cache (more than 512 MB in all)."""
    import orc
    from devutil import to_dev
    np, capi, torch = b.np, b.capi, b.torch
    Bq, Hq, Hkv, D, S = 8, 32, 8, 128, 32768
    NS = 4
    group, H = Hq // Hkv, Bq * Hkv
    st = b.stream
    slab_of = np.array([(i % Hkv) % NS for i in range(H)])
    qh = orc.normal_activations(H * group * D, 0xA77E)
    q = to_dev(qh)
    res = {"B": Bq, "Hq": Hq, "Hkv": Hkv, "D": D, "S": S, "sample_slabs": NS, "cache_copies": 2}
    steps = max(5, b.steps // 20)
    cpu = {}

    def rep(t):  # (NS, ...) host array -> (H, ...) device tensor following slab_of
        d = to_dev(np.ascontiguousarray(t))
        return d.view(NS, -1)[torch.from_numpy(slab_of).to("cuda")].contiguous().view(-1)

    def out_ok(o, kd, vd):
        """sampled (slab, query head) outputs against the FP64 oracle"""
        got = o.cpu().numpy().view(np.float16).reshape(H * group, D)
        worst = 0.0
        for i in (0, 21, 42, 63):  # slabs of four different sequences and sample slabs
            sl = slab_of[i]
            qs = qh.reshape(H, group * D)[i]
            ref = orc.attention_f16(qs, kd[sl:sl + 1], vd[sl:sl + 1], 1, group, S, D)
            worst = max(worst, orc.rel_l2(got[i * group:(i + 1) * group], ref))
        return worst

    def hooks_equal(ko, want):
        return bool(torch.equal(ko.view(H, -1), want.view(NS, -1)[torch.from_numpy(slab_of).to("cuda")]))

    # ---- W4 gs=32 symmetric, and the FP16 cache made of its dequantized values ----
    gs, G, wd = 32, 4, D // 8
    c4, kd, vd, tq = _slab_cache(b, "w4", NS, S, D, gs, 0xA77E + 1)
    t0 = time.perf_counter()
    orc.attention_f16(qh.reshape(H, group * D)[0], kd[0:1], vd[0:1], 1, group, S, D)
    cpu["attention_reference_4heads_1slab_s"] = time.perf_counter() - t0
    cpu["quantize_cache_w4_4slabs_s"] = tq
    kd_d, vd_d = to_dev(kd), to_dev(vd)
    copies = []
    for _ in range(2):
        t = [rep(c4.q_k.reshape(NS, -1)), rep(c4.s_k.reshape(NS, -1)), rep(c4.q_v.reshape(NS, -1)),
             rep(c4.s_v.reshape(NS, -1))]
        copies.append((capi.kv_view(H, S, D, gs, G, True, t[0].data_ptr(), t[1].data_ptr(), 0, t[2].data_ptr(),
                                    t[3].data_ptr(), 0), t))
    o = torch.empty(H * group * D, dtype=torch.int16, device="cuda")
    ko = torch.empty(H * S * D, dtype=torch.int16, device="cuda")
    vo = torch.empty(H * S * D, dtype=torch.int16, device="cuda")
    capi.attention_w4_flash(copies[0][0], q.data_ptr(), o.data_ptr(), st, ko.data_ptr(), vo.data_ptr(), group=group)
    hook_ok = hooks_equal(ko, kd_d) and hooks_equal(vo, vd_d)
    del ko, vo
    o2 = torch.empty_like(o)
    capi.attention_w4_flash(copies[1][0], q.data_ptr(), o2.data_ptr(), st, group=group)
    gate = {"hooks_bitwise": hook_ok, "unhooked_equals_hooked": bool(torch.equal(o, o2)),
            "rel_l2_sampled": out_ok(o2, kd, vd)}
    if not (gate["hooks_bitwise"] and gate["unhooked_equals_hooked"] and gate["rel_l2_sampled"] <= TOL):
        raise RuntimeError("bench-size gate failed (w4 flash): %s" % json.dumps(gate))
    o_w4 = o2.clone()
    ms, raw = _reps_ms(torch, lambda i: capi.attention_w4_flash(copies[i % 2][0], q.data_ptr(), o.data_ptr(), st,
                                                                group=group), steps, 2)
    nb = 2 * (H * S * wd * 4 + H * S * G * 2)
    res["w4_gs32"] = {"ms": ms, "reps_ms": raw, "bytes": nb, "GBs": nb / ms * 1e-6,
                      "frac_of_hbm_peak": nb / ms * 1e-6 / HBM_PEAK_GBS, "gate": gate}
    # the entry point that allocates nothing, same workload
    ms, raw = _reps_ms(torch, lambda i: capi.attention_w4_flash_noalloc(copies[i % 2][0], q.data_ptr(), o.data_ptr(),
                                                                        st, group=group), steps, 2)
    res["w4_gs32_noalloc_entry"] = {"ms": ms, "reps_ms": raw, "equals_allocating_entry": bool(torch.equal(o, o_w4))}

    # ---- paged W4, page 16: sequences 0-3 share their first 8192 tokens ----
    page, prefix = 16, 8192
    lp, pp = S // page, prefix // page
    npages = pp + 4 * (lp - pp) + 4 * lp
    rows = npages * page
    pools = []
    t_idx = torch.arange(S, device="cuda")
    for cp in range(2):
        perm = torch.randperm(npages, device="cuda", dtype=torch.int32)
        tables = torch.empty((Bq, lp), dtype=torch.int32, device="cuda")
        nxt = pp
        for s in range(Bq):
            if s < 4:
                tables[s, :pp] = perm[:pp]
                tables[s, pp:] = perm[nxt:nxt + lp - pp]
                nxt += lp - pp
            else:
                tables[s] = perm[nxt:nxt + lp]
                nxt += lp
        pool = {}
        for name, width, src in (("q_k", wd, c4.q_k), ("s_k", G, c4.s_k), ("q_v", wd, c4.q_v), ("s_v", G, c4.s_v)):
            src_d = to_dev(src).view(NS, S, width)
            pl = torch.zeros((Hkv, rows, width), dtype=src_d.dtype, device="cuda")
            for s in range(Bq):
                phys = tables[s].long()[t_idx // page] * page + t_idx % page
                for h in range(Hkv):
                    pl[h, phys] = src_d[h % NS]  # sequences that share a page write it the same rows
            pool[name] = pl
        view = capi.kv_view(Hkv, S, D, gs, G, True, pool["q_k"].data_ptr(), pool["s_k"].data_ptr(), 0,
                            pool["q_v"].data_ptr(), pool["s_v"].data_ptr(), 0)
        pools.append((view, tables, pool))
    op = torch.empty_like(o)
    capi.attention_w4_flash_paged_batched(pools[0][0], pools[0][1].data_ptr(), Bq, lp, page, npages, group,
                                          q.data_ptr(), op.data_ptr(), st)
    same = bool(torch.equal(op, o_w4))
    if not same:
        raise RuntimeError("bench-size gate failed: paged output differs from the contiguous output")
    ms, raw = _reps_ms(torch, lambda i: capi.attention_w4_flash_paged_batched(
        pools[i % 2][0], pools[i % 2][1].data_ptr(), Bq, lp, page, npages, group, q.data_ptr(), op.data_ptr(), st),
        steps, 2)
    uniq = 2 * Hkv * rows * (wd * 4 + G * 2)
    res["paged_w4_page16"] = {"ms": ms, "reps_ms": raw, "bytes_logical": nb, "bytes_unique": uniq,
                              "GBs_logical": nb / ms * 1e-6, "GBs_unique": uniq / ms * 1e-6,
                              "frac_of_hbm_peak_unique": uniq / ms * 1e-6 / HBM_PEAK_GBS,
                              "vs_contiguous": res["w4_gs32"]["ms"] / ms,
                              "gate": {"output_equals_contiguous_bytes": same}}
    del pools, copies, pool
    torch.cuda.empty_cache()

    # ---- FP16 cache (the dequantized W4 values): two copies of 1 GiB ----
    k16 = [kd_d.view(NS, -1)[torch.from_numpy(slab_of).to("cuda")].contiguous() for _ in range(2)]
    v16 = [vd_d.view(NS, -1)[torch.from_numpy(slab_of).to("cuda")].contiguous() for _ in range(2)]
    capi.attention_fp16_flash(q.data_ptr(), k16[0].data_ptr(), v16[0].data_ptr(), o.data_ptr(), H, S, D, st, group=group)
    gate = {"rel_l2_sampled": out_ok(o, kd, vd)}
    if gate["rel_l2_sampled"] > TOL:
        raise RuntimeError("bench-size gate failed (fp16 flash): %s" % json.dumps(gate))
    ms, raw = _reps_ms(torch, lambda i: capi.attention_fp16_flash(
        q.data_ptr(), k16[i % 2].data_ptr(), v16[i % 2].data_ptr(), o.data_ptr(), H, S, D, st, group=group), steps, 2)
    nb16 = 2 * H * S * D * 2
    res["fp16"] = {"ms": ms, "reps_ms": raw, "bytes": nb16, "GBs": nb16 / ms * 1e-6,
                   "frac_of_hbm_peak": nb16 / ms * 1e-6 / HBM_PEAK_GBS, "gate": gate}
    del k16, v16, kd_d, vd_d
    torch.cuda.empty_cache()

    # ---- FP8 E4M3: per-(row, group=128) scales and one scale per slab ----
    c8, kd8, vd8, tq8 = _slab_cache(b, "f8", NS, S, D, 128, 0xA77E + 9)
    cpu["quantize_cache_f8_4slabs_s"] = tq8
    kd8_d, vd8_d = to_dev(kd8), to_dev(vd8)
    f8 = []
    for _ in range(2):
        t = [rep(c8.q_k.reshape(NS, -1)), rep(c8.s_k.reshape(NS, -1)), rep(c8.q_v.reshape(NS, -1)),
             rep(c8.s_v.reshape(NS, -1))]
        f8.append((capi.kv_f8_view(H, S, D, 128, 1, *[x.data_ptr() for x in t]), t))
    ko = torch.empty(H * S * D, dtype=torch.int16, device="cuda")
    vo = torch.empty(H * S * D, dtype=torch.int16, device="cuda")
    capi.attention_f8_flash(f8[0][0], q.data_ptr(), o.data_ptr(), st, ko.data_ptr(), vo.data_ptr(), group=group)
    hook_ok = hooks_equal(ko, kd8_d) and hooks_equal(vo, vd8_d)
    capi.attention_f8_flash(f8[1][0], q.data_ptr(), o2.data_ptr(), st, group=group)
    gate = {"hooks_bitwise": hook_ok, "unhooked_equals_hooked": bool(torch.equal(o, o2)),
            "rel_l2_sampled": out_ok(o2, kd8, vd8)}
    if not (gate["hooks_bitwise"] and gate["unhooked_equals_hooked"] and gate["rel_l2_sampled"] <= TOL):
        raise RuntimeError("bench-size gate failed (f8 flash): %s" % json.dumps(gate))
    ms, raw = _reps_ms(torch, lambda i: capi.attention_f8_flash(f8[i % 2][0], q.data_ptr(), o.data_ptr(), st,
                                                                group=group), steps, 2)
    nb8 = 2 * H * S * D + 2 * H * S * 2
    res["fp8_row_scale"] = {"ms": ms, "reps_ms": raw, "bytes": nb8, "GBs": nb8 / ms * 1e-6,
                            "frac_of_hbm_peak": nb8 / ms * 1e-6 / HBM_PEAK_GBS, "gate": gate}
    # one scale per slab ("per-head scale"): the same codes under one FP16 scale per (sequence, kv-head);
    # oracle = the reference arithmetic with that scale in every (row, group) slot
    slab_scales = np.array([0x2000 + 37 * i for i in range(NS)], np.uint16)  # ~0.0078 ... 0.0085
    c8b = orc.KVCacheF8()
    c8b.__dict__.update(c8.__dict__)
    c8b.s_k = np.repeat(slab_scales, S)
    c8b.s_v = np.repeat(slab_scales[::-1].copy(), S)
    kdb, vdb = orc.dequant_cache_f8(c8b, False), orc.dequant_cache_f8(c8b, True)
    f8s = []
    for cp in range(2):
        sk = to_dev(slab_scales)[torch.from_numpy(slab_of).to("cuda")].contiguous()
        sv = to_dev(slab_scales[::-1].copy())[torch.from_numpy(slab_of).to("cuda")].contiguous()
        f8s.append((capi.kv_f8_view(H, S, D, 128, 1, f8[cp][1][0].data_ptr(), sk.data_ptr(), f8[cp][1][2].data_ptr(),
                                    sv.data_ptr()), (sk, sv)))
    capi.attention_f8_flash(f8s[0][0], q.data_ptr(), o.data_ptr(), st, ko.data_ptr(), vo.data_ptr(), group=group,
                            scale_mode=1)
    hook_ok = hooks_equal(ko, to_dev(kdb)) and hooks_equal(vo, to_dev(vdb))
    del ko, vo
    gate = {"hooks_bitwise": hook_ok, "rel_l2_sampled": out_ok(o, kdb, vdb)}
    if not (gate["hooks_bitwise"] and gate["rel_l2_sampled"] <= TOL):
        raise RuntimeError("bench-size gate failed (f8 slab scale): %s" % json.dumps(gate))
    ms, raw = _reps_ms(torch, lambda i: capi.attention_f8_flash(f8s[i % 2][0], q.data_ptr(), o.data_ptr(), st,
                                                                group=group, scale_mode=1), steps, 2)
    nb8s = 2 * H * S * D
    res["fp8_head_scale"] = {"ms": ms, "reps_ms": raw, "bytes": nb8s, "GBs": nb8s / ms * 1e-6,
                             "frac_of_hbm_peak": nb8s / ms * 1e-6 / HBM_PEAK_GBS, "gate": gate}
    res["cpu"] = cpu
    out = {"c5_flash_decode": res}
    if full:
        out["attention_sweep_w4_gs128"] = attention_sweep(b)
    return out


def attention_sweep(b):
    """The shapes of the reference's attention benchmark (bench_attention.cu: H in {32, 8}, S from
    512 to 32768, D = 128, gs = 128, one query token): W4 flash decode on random codes, rotating
    through enough cache copies to stay cold.  Timing only (the parity tests hold the kernels)."""
    torch, capi, st = b.torch, b.capi, b.stream
    D, gs = 128, 128
    G, wd = D // gs, D // 8
    rows = []
    for H in (32, 8):
        for S in (512, 2048, 4096, 8192, 32768):
            nb = 2 * (H * S * wd * 4 + H * S * G * 2)
            ncopy = min(64, max(2, int(600e6 // nb) + 1))
            views, keep = [], []
            for _ in range(ncopy):
                t = [torch.randint(-2**31, 2**31 - 1, (H * S * wd,), dtype=torch.int32, device="cuda"),
                     (torch.rand(H * S * G, device="cuda") * 0.2 + 0.1).to(torch.float16),
                     torch.randint(-2**31, 2**31 - 1, (H * S * wd,), dtype=torch.int32, device="cuda"),
                     (torch.rand(H * S * G, device="cuda") * 0.2 + 0.1).to(torch.float16)]
                keep.append(t)
                views.append(capi.kv_view(H, S, D, gs, G, True, t[0].data_ptr(), t[1].data_ptr(), 0,
                                          t[2].data_ptr(), t[3].data_ptr(), 0))
            q = torch.randn(H * D, device="cuda").to(torch.float16)
            o = torch.empty(H * D, dtype=torch.int16, device="cuda")
            ms, raw = _reps_ms(torch, lambda i: capi.attention_w4_flash(views[i % ncopy], q.data_ptr(),
                                                                        o.data_ptr(), st, group=1), 50, 2)
            rows.append({"H": H, "S": S, "us": ms * 1e3, "reps_us": [r * 1e3 for r in raw], "bytes": nb,
                         "GBs": nb / ms * 1e-6})
            del views, keep
            torch.cuda.empty_cache()
    return rows


def extras_w4a4(b, full):
    """Both operands MXFP4 on the scaled matrix cores (separately gated W4A4 entry)."""
    torch = b.torch
    rows = []
    for (N, K) in ((4096, 4096), (14336, 4096)):
        views = b.rand_mx(N, K, max(2, int(400e6 // mx_bytes(N, K, 1)) + 1))
        for M in ((1, 16, 64, 256, 2048) if not full else (1, 8, 16, 32, 64, 128, 256, 512, 2048, 8192)):
            nb = mx_bytes(N, K, 0) + M * (K // 2 + K // 32) + 2 * M * N
            us = b.w4a4_us(views, M, N, K)
            rows.append({"N": N, "K": K, "M": M, "bytes": nb, "us": us, "GBs": nb / us * 1e-3,
                         "TFLOPs": 2.0 * M * N * K / us * 1e-6})
            if M <= 256 or M == 2048:  # E4M3 activations
                us8 = b.w4a4_us(views, M, N, K, a8=True)
                rows[-1].update({"a8_us": us8, "a8_TFLOPs": 2.0 * M * N * K / us8 * 1e-6})
        del views
        torch.cuda.empty_cache()
    # the activation quantizers that feed it (FP16 -> MXFP4 / MXFP8), K = 4096
    capi, st = b.capi, b.stream
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    act = []
    K = 4096
    for M in (16, 2048):
        x = torch.randn(M * K, device="cuda").to(torch.float16)
        q4 = torch.empty(M * K // 8, dtype=torch.int32, device="cuda")
        q8 = torch.empty(M * K, dtype=torch.uint8, device="cuda")
        sc = torch.empty(M * K // 32, dtype=torch.uint8, device="cuda")
        v4 = capi.packed_mx_view(M, K, K // 32, q4.data_ptr(), sc.data_ptr())
        v8 = capi.act_mx8_view(M, K, K // 32, q8.data_ptr(), sc.data_ptr())
        ms4 = _median_events_ms(torch, lambda i: capi.quantize_mx_f16(v4, x.data_ptr(), status.data_ptr(), st), 50, 5)
        ms8 = _median_events_ms(torch, lambda i: capi.quantize_mx8_f16(v8, x.data_ptr(), status.data_ptr(), st), 50, 5)
        act.append({"M": M, "K": K, "fp4_us": ms4 * 1e3, "fp8_us": ms8 * 1e3})
    return {"w4a4_mxfp4": rows, "w4a4_activation_quantizers": act}


def extras_quantize(b, full):
    """Device-side quantizers (memory-bound streams): bytes read + written per call over the
    call's duration.  Sources: FP64 weights (as the host quantizers take them), FP16 K/V rows."""
    capi, torch = b.capi, b.torch
    st = b.stream
    steps = max(5, b.steps // 20)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    res = {}
    N = K = 4096
    gs, G = 128, 32
    w = torch.randn(N * K, device="cuda", dtype=torch.float64)
    q = torch.empty(N * K // 8, dtype=torch.int32, device="cuda")
    sc = torch.empty(N * G, dtype=torch.int16, device="cuda")
    z = torch.empty(N * G // 8, dtype=torch.int32, device="cuda")
    for sym in (True, False):
        view = capi.packed_view(N, K, gs, G, sym, q.data_ptr(), sc.data_ptr(), 0 if sym else z.data_ptr())
        ms = _median_events_ms(torch, lambda i: capi.quantize(view, w.data_ptr(), status.data_ptr(), st),
                               steps, 2)
        nb = N * K * 8 + w4_bytes(N, K, gs, sym, 0)
        res["w4_%s_f64_4096x4096" % ("sym" if sym else "asym")] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    B = K // 32
    sb = torch.empty(N * B, dtype=torch.uint8, device="cuda")
    view = capi.packed_mx_view(N, K, B, q.data_ptr(), sb.data_ptr())
    ms = _median_events_ms(torch, lambda i: capi.quantize_mx(view, w.data_ptr(), status.data_ptr(), st),
                           steps, 2)
    nb = N * K * 8 + mx_bytes(N, K, 0)
    res["mx_f64_4096x4096"] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    del w
    # KV rows from FP16: a whole prefill (64 slabs x 4096 rows) and one appended row per slab
    D, gs, G = 128, 32, 4
    for H, S in ((64, 4096), (64, 1)):
        rows = H * S
        k16 = torch.randn(rows * D, device="cuda", dtype=torch.float16)
        v16 = torch.randn(rows * D, device="cuda", dtype=torch.float16)
        qk = torch.empty(rows * D // 8, dtype=torch.int32, device="cuda")
        qv = torch.empty_like(qk)
        sk = torch.empty(rows * G, dtype=torch.int16, device="cuda")
        sv = torch.empty_like(sk)
        view = capi.kv_view(H, S, D, gs, G, True, qk.data_ptr(), sk.data_ptr(), 0, qv.data_ptr(),
                            sv.data_ptr(), 0)
        ms = _median_events_ms(torch, lambda i: capi.quantize_cache(
            view, k16.data_ptr(), v16.data_ptr(), status.data_ptr(), True, st), steps, 2)
        nb = 2 * rows * (D * 2 + D // 2 + G * 2)
        res["kv_w4_f16_%dx%d" % (H, S)] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
        bk = torch.empty(rows * D, dtype=torch.uint8, device="cuda")
        bv = torch.empty_like(bk)
        view8 = capi.kv_f8_view(H, S, D, gs, G, bk.data_ptr(), sk.data_ptr(), bv.data_ptr(), sv.data_ptr())
        ms = _median_events_ms(torch, lambda i: capi.quantize_cache_f8(
            view8, k16.data_ptr(), v16.data_ptr(), status.data_ptr(), True, st), steps, 2)
        nb = 2 * rows * (D * 2 + D + G * 2)
        res["kv_f8_f16_%dx%d" % (H, S)] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    return {"quantize": res}


def rand_w4_views(b, N, K, gs, sym, copies):
    """Random packed codes with N(0,0.02)-like scales made on the device: the counter
    probes only (the timed benchmark cases use oracle-quantized data)."""
    torch, capi = b.torch, b.capi
    G = (K + gs - 1) // gs
    wk, wg = (K + 7) // 8, (G + 7) // 8
    out = []
    for _ in range(copies):
        q = torch.randint(-2**31, 2**31 - 1, (N * wk,), dtype=torch.int32, device="cuda")
        s = (torch.rand(N * G, device="cuda") * 0.008 + 0.004).to(torch.float16)
        z = None if sym else torch.randint(-2**31, 2**31 - 1, (N * wg,), dtype=torch.int32, device="cuda")
        v = capi.packed_view(N, K, gs, G, sym, q.data_ptr(), s.data_ptr(), 0 if z is None else z.data_ptr())
        out.append((v, (q, s, z)))
    return out


def probe(b, which, args):
    """Short fixed workloads for counter runs under a profiler (no yardsticks)."""
    capi, torch = b.capi, b.torch
    out = {"probe": which}
    if which == "floor":  # launch floor and in-kernel timeline of the headline kernel
        h, dps, x_d, c_d = headline(b, argparse.Namespace(steps=200, warmup=20, reps=3, extras="none"))
        out["headline_cold_us"] = h["cold_ms"] * 1e3
        out.update(extras_floor(b, dps, x_d, c_d))
    elif which == "c1":  # the headline alone: W + K cold launches of the decode-shape kernel
        h, dps, x_d, c_d = headline(b, argparse.Namespace(steps=args.steps, warmup=args.warmup, reps=1, extras="none"))
        # one pass of the copy yardstick, so that a counter run of this command also holds
        # the reading of a kernel whose traffic is known (1 GiB each way)
        n = 1 << 30
        src = torch.empty(n, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        b.yard.w4bench_copy(src.data_ptr(), dst.data_ptr(), n, 4096, b.stream)
        torch.cuda.synchronize()
        out["headline_cold_us"] = h["cold_ms"] * 1e3
    elif which == "decode":  # C2 shape, symmetric: vector kernel at M=1, matrix-core kernels at M=8 and 16
        N, K = 11008, 4096
        views = [v[0] for v in rand_w4_views(b, N, K, 128, True, 18)]
        for M, fn in ((1, "w4_gemm_fused"), (8, "w4_gemm_mma"), (16, "w4_gemm_mma")):
            x = torch.randn(M * K, device="cuda").to(torch.float16)
            c = torch.empty(M * N, dtype=torch.float16, device="cuda")
            out["%s_M%d_us" % (fn, M)] = b.gemm_us(fn, views, x, c, M)[0]
    elif which == "longk":  # down-projection shapes: K-split vector kernel at M=1, pipelined matrix-core kernel at M=4 and 16
        for (N, K) in ((4096, 11008), (4096, 14336)):
            views = [v[0] for v in rand_w4_views(b, N, K, 128, True, 12)]
            for M in (1, 4, 16):
                x = torch.randn(M * K, device="cuda").to(torch.float16)
                c = torch.empty(M * N, dtype=torch.float16, device="cuda")
                out["w4_gemm_K%d_M%d_us" % (K, M)] = b.gemm_us("w4_gemm", views, x, c, M)[0]
            del views
            torch.cuda.empty_cache()
        # more 16-row tiles than compute units: from 13 activation rows on two tiles share a workgroup's activations
        views = [v[0] for v in rand_w4_views(b, 8192, 8192, 128, True, 6)]
        for M in (16, 64):
            x = torch.randn(M * 8192, device="cuda").to(torch.float16)
            c = torch.empty(M * 8192, dtype=torch.float16, device="cuda")
            out["w4_gemm_N8192_K8192_M%d_us" % M] = b.gemm_us("w4_gemm", views, x, c, M)[0]
        del views
        torch.cuda.empty_cache()
    elif which == "attention":  # C5 flash decode over FP16 / W4 / paged W4 / FP8 caches
        b.steps = 200
        out.update(extras_attention(b, False))
    elif which == "quantize":  # the device-side quantizers, 20 calls of each workload
        b.steps, b.warmup = 200, 2
        out.update(extras_quantize(b, False))
    elif which == "w4a4":  # both operands MXFP4: skinny kernel at M=1/16/64, tile kernel at M=2048
        N = K = 4096
        views = b.rand_mx(N, K, 46)
        for M in (1, 16, 64, 2048):
            b.steps, b.warmup = (20, 3) if M > 64 else (100, 10)
            out["w4a4_M%d_us" % M] = b.w4a4_us(views, M, N, K, reps=1)
    else:  # prefill: the fused tile kernels and the plain FP16 library GEMM, 20 calls each at M = 2048 and 4096
        N = K = 4096
        views = rand_w4_views(b, N, K, 128, True, 1)
        w16 = torch.empty(N * K, dtype=torch.float16, device="cuda")
        capi.dequant(views[0][0], w16.data_ptr(), b.stream)
        for M in (2048, 4096):
            x = torch.randn(M * K, device="cuda").to(torch.float16)
            c = torch.empty(M * N, dtype=torch.float16, device="cuda")
            for _ in range(20):
                capi.gemm(views[0][0], x.data_ptr(), c.data_ptr(), M, b.stream, 0)
                capi.gemm_fp16(w16.data_ptr(), x.data_ptr(), c.data_ptr(), M, N, K, b.stream)
            torch.cuda.synchronize()
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--reps", type=int, default=9, help="repetitions of the K timed steps (median reported)")
    ap.add_argument("--extras", choices=["none", "quick", "full"], default="quick")
    ap.add_argument("--out", default=None, help="also write the full record (graded line + every section) to this file")
    ap.add_argument("--probe", choices=["floor", "c1", "decode", "longk", "prefill", "quantize", "w4a4", "attention"],
                    default=None, help="run only a short fixed workload (for counter collection) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus N with N > 1 is not supported "
              "(the path shards over N or (batch, kv-head) with no exchange)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    b = Bench(args.steps, args.warmup, max(1, args.reps))
    if args.probe:
        if args.probe not in ("c1",):
            b.steps, b.warmup = 30, 5
        probe(b, args.probe, args)
        return
    t_start = time.perf_counter()
    h, dps, x_d, c_d = headline(b, args)
    bw = b.bandwidth()
    cold_gbs = h["bytes"] / h["cold_ms"] * 1e-6
    extra = {"headline": h, "yardstick": bw,
             "cold_frac_of_measured_read": cold_gbs / bw["read_GBs"],
             "cold_frac_of_measured_copy": cold_gbs / bw["copy_GBs"],
             "cold_us": h["cold_ms"] * 1e3, "device": torch.cuda.get_device_name(0), "host_cpu": cpu_info()}
    if "warm_ms" in h:
        extra["warm_us"] = h["warm_ms"] * 1e3
        extra["warm_GBs"] = h["bytes"] / h["warm_ms"] * 1e-6
    if args.extras != "none":
        extra.update(extras_floor(b, dps, x_d, c_d))
    del dps
    torch.cuda.empty_cache()
    if args.extras != "none":
        extra.update(extras_gemm(b, args.extras == "full"))
        extra.update(extras_attention(b, args.extras == "full"))
        extra.update(extras_quantize(b, args.extras == "full"))
        extra.update(extras_w4a4(b, args.extras == "full"))
    extra["bench_wall_s"] = time.perf_counter() - t_start
    cpu = h["cpu"]
    host = extra["host_cpu"]
    legs = {"c1_quantize_s": cpu["quantize_s"], "c1_dequant_all_s": cpu["dequant_all_s"],
            "c1_gemm_oracle_M1_s": cpu["gemm_oracle_s"], "c1_quantize_mx_s": cpu["quantize_mx_s"],
            "c1_dequant_all_mx_s": cpu["dequant_all_mx_s"]}
    if "c5_flash_decode" in extra:
        legs.update({"c5_" + k: v for k, v in extra["c5_flash_decode"]["cpu"].items()})
    line = {
        "metric": "M=1 W4 GEMM us + achieved HBM GB/s (% of peak); M=2048 MFMA TFLOP/s",
        "value": _r(cold_gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": _r(h["cold_ms"], 7), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "C1: W4A16 sym gs=128 fused GEMM M=1 N=K=4096, cold weights (%d HBM copies), "
                               "median of %d x %d steps" % (h["copies"], len(h["cold_reps_ms"]), args.steps),
                   "entry": "w4_gemm", "bytes_per_step": h["bytes"]},
        "roofline": {"bound": "hbm", "achieved": _r(cold_gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": _r(cold_gbs / HBM_PEAK_GBS, 4), "traffic": HEADLINE_TRAFFIC_BYTES},
        "cpu_baseline": {"value": _r(h["bytes"] / cpu["fused_equiv_s"] * 1e-9, 5), "unit": "GB/s",
                         "cores": 1, "kind": "port",
                         "sample": "oracle dequant_all+gemm_oracle, same 4096x4096 matrix, 1 thread of %d, "
                                   "median of 5 (%.3f s)" % (host["usable_cpus"], cpu["fused_equiv_s"])},
        "summary": _summary_or_error(extra, cold_gbs),
    }
    emit(line, extra, legs, args.out)


def _r(v, n):
    return round(float(v), n)


def _summary_or_error(extra, cold_gbs):
    try:  # the summary is a convenience: a section that changed shape must not cost the graded record
        return summarize(extra, cold_gbs)
    except Exception as e:  # noqa: BLE001
        return {"error": "%s: %s" % (type(e).__name__, e)}


def summarize(extra, cold_gbs):
    """At most a dozen scalars for the graded line: yardsticks, C4, the worst C2 / C3 cases, C5 per format."""
    s = {"c1_us": _r(extra["cold_us"], 3),
         "copy_GBs": _r(extra["yardstick"]["copy_GBs"], 0),
         "c1_frac_of_copy": _r(extra["cold_frac_of_measured_copy"], 3)}
    if "launch_floor" in extra:
        s["read_only_c1_us"] = _r(extra["launch_floor"]["read_c1_8MiB_us"], 3)
    if "c4_prefill" in extra:
        c4 = extra["c4_prefill"]
        s["c4_TFLOPs"] = _r(c4["fused_TFLOPs"], 1)
        s["c4_frac_mfma"] = _r(c4["frac_of_mfma_peak"], 3)
        s["c4_two_pass_TFLOPs"] = _r(c4["two_pass_TFLOPs"], 1)
        s["c4_hipblaslt_TFLOPs"] = _r(c4["hipblaslt_only_TFLOPs"], 1)
        for r in extra.get("c4_prefill_other_M", []):
            if r["M"] == 4096:  # where the 256 x 256 tiles take over: fused against dequant + library GEMM
                s["c4_M4096_fused_two_pass_us"] = [_r(r["fused_us"], 1), _r(r["two_pass_us"], 1)]
        c2 = [r for r in extra.get("c2_w4_asym", []) if r["gs"] == 128 and r["M"] == 8]
        if c2:
            s["c2_gs128_M8_us"] = _r(min(v for v in (c2[0].get("simt_us"), c2[0].get("mfma_us")) if v), 2)
    for key, name in (("c2_w4_asym", "c2"), ("c3_mxfp4", "c3")):
        rows = extra.get(key)
        if rows:
            w = min(rows, key=lambda r: r["frac_of_hbm_peak"])
            b = max(rows, key=lambda r: r["frac_of_hbm_peak"])
            s[name + "_worst_frac_hbm"] = _r(w["frac_of_hbm_peak"], 3)
            s[name + "_worst_case"] = "N%d K%d M%d" % (w["N"], w["K"], w["M"]) + (" gs%d" % w["gs"] if "gs" in w else "")
            s[name + "_best_frac_hbm"] = _r(b["frac_of_hbm_peak"], 3)
    c5 = extra.get("c5_flash_decode")
    if c5:
        s["c5_frac_hbm"] = {k: _r(c5[k].get("frac_of_hbm_peak", c5[k].get("frac_of_hbm_peak_unique")), 3) for k in
                            ("fp16", "w4_gs32", "paged_w4_page16", "fp8_row_scale", "fp8_head_scale") if k in c5}
    s["wall_s"] = _r(extra["bench_wall_s"], 1)
    return s


def section_lines(extra, legs):
    """The detailed records as one JSON line per section, each small enough to survive a log tail."""
    scalars = {k: v for k, v in extra.items() if not isinstance(v, (dict, list))}
    lines = [{"section": "run", **scalars, "host_cpu": extra.get("host_cpu")},
             {"section": "cpu_baseline_legs_s", **legs}]
    for k, v in extra.items():
        if k == "host_cpu" or not isinstance(v, (dict, list)):
            continue
        if isinstance(v, list) and len(json.dumps(v)) > 5000:  # long sweeps: a few rows per line
            step = max(1, len(v) * 4000 // len(json.dumps(v)))
            for i in range(0, len(v), step):
                lines.append({"section": k, "part": i // step, "rows": v[i:i + step]})
        elif k == "c1_timeline":
            lines.append({"section": k, "waves": v.get("waves"), "tick_ns": v.get("tick_ns"),
                          "launches": v.get("launches", [])[:1]})
        else:
            lines.append({"section": k, "data": v})
    return lines


def emit(line, extra, legs, out_path):
    """Sections first, the graded record last and short: a harness that keeps only the end of stdout
    still gets metric, value, roofline and cpu_baseline whole."""
    for rec in section_lines(extra, legs):
        print(json.dumps(rec))
    if out_path:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(out_path)), exist_ok=True)
            with open(out_path, "w") as f:
                json.dump({**line, "cpu_baseline_legs_s": legs, "extra": extra}, f)
        except OSError as e:
            print("bench.py: could not write %s: %s" % (out_path, e), file=sys.stderr)
    final = json.dumps(line)
    assert len(final) < FINAL_LINE_MAX, "graded line grew to %d bytes" % len(final)
    sys.stdout.flush()
    print(final, flush=True)


if __name__ == "__main__":
    main()
