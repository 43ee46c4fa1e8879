#!/usr/bin/env python3
"""Benchmark of the fused-dequant hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extras none|quick|full]

Prints ONE JSON line.  The headline workload is the W4A16 symmetric gs=128,
M=1, N=K=4096 fused GEMM; one "step" is one call of w4_gemm on it.  `value` is
the achieved HBM rate: algorithmic bytes (packed codes + scales + x + c =
8 667 136 B) divided by the mean launch-to-launch time over the K timed steps,
with the weights rotated through enough distinct copies that no step finds its
matrix in the 256 MB last-level cache ("cold").  The same figure with one hot
copy, the measured streaming-read and copy rates, the other configs of the
scope table and the CPU oracle's time for the same operation ride along.
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
PREWARM_LAUNCHES = 2000
# HBM bytes one launch of the headline kernel moves, from rocprofv3 --pmc runs of
# `python3 bench.py --extras none --steps 50 --warmup 5`: FETCH_SIZE 4281.0 and
# WRITE_SIZE 16.0 per dispatch, scaled by what the same counters read for the
# 1 GiB stream_copy kernel of this file's yardstick (FETCH_SIZE 524298 and
# WRITE_SIZE 1048591 for 1048576 KiB each way, i.e. factors 2.0 and 1.0):
# 8562 KiB fetched + 16 KiB written, against 8 667 136 algorithmic bytes.
HEADLINE_TRAFFIC_BYTES = int((4281.0 * 2.0 + 16.0 * 1.0) * 1024)


def _pkg():
    import w4amd
    return w4amd.package()


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


def _median_events_ms(torch, fn, steps, warmup, reps=5):
    return sorted(_events_ms(torch, fn, steps, warmup if r == 0 else 2) for r in range(reps))[reps // 2]


class Bench:
    def __init__(self, steps, warmup):
        import numpy as np
        import torch
        self.np, self.torch = np, torch
        self.capi = _pkg().capi
        self.capi.load()
        self.steps, self.warmup = steps, warmup
        self.stream = torch.cuda.current_stream().cuda_stream
        self.yard = C.CDLL(os.path.join(ROOT, "w4a16-dequant-gemm_amd", "lib", "libw4bench.so"))
        self.yard.w4bench_read.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_void_p]
        self.yard.w4bench_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        self.yard.w4bench_gemm_loop.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                                C.c_int, C.c_int, C.c_void_p]

    def w4a4_us(self, views, M, N, K, reps=5, a8=False):
        """us per w4_gemm_mx_w4a4 (a8: w4_gemm_mx_w4a8) call over rotating weight copies (C
        loop, HIP events)."""
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
        self.yard.w4bench_w4a4_loop.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                                C.c_int, C.c_void_p]

        def run(n):
            rc = self.yard.w4bench_w4a4_loop(fn, arr, len(views), C.addressof(xv[0]), c.data_ptr(), n,
                                             self.stream)
            if rc:
                raise RuntimeError("w4a4 loop failed: %d" % rc)
        run(self.warmup)
        torch.cuda.synchronize()
        out = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            run(self.steps)
            b.record()
            torch.cuda.synchronize()
            out.append(a.elapsed_time(b) / self.steps * 1e3)
        return sorted(out)[len(out) // 2]

    def loop_ms(self, entry, views, x_ptr, c_ptr, M, steps, warmup, reps=5):
        """Mean ms per call over `steps` launches issued by a C loop (no
        interpreter between launches), HIP events on the launch stream; median of reps."""
        torch = self.torch
        fn = C.cast(getattr(self.capi.load(), entry), C.c_void_p)
        arr = (C.c_void_p * len(views))(*[C.addressof(v) for v in views])

        def run(n):
            rc = self.yard.w4bench_gemm_loop(fn, arr, len(views), x_ptr, c_ptr, M, n, self.stream)
            if rc:
                raise RuntimeError("gemm loop failed: %d" % rc)
        run(warmup)
        torch.cuda.synchronize()
        out = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            run(steps)
            b.record()
            torch.cuda.synchronize()
            out.append(a.elapsed_time(b) / steps)
        return sorted(out)[len(out) // 2]

    # -- yardsticks ---------------------------------------------------------
    def bandwidth(self):
        torch = self.torch
        n = 1 << 30
        src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        rd = _median_events_ms(torch, lambda i: self.yard.w4bench_read(
            src.data_ptr(), n, sink.data_ptr(), 256 * 16, self.stream), 10, 3)
        cp = _median_events_ms(torch, lambda i: self.yard.w4bench_copy(
            src.data_ptr(), dst.data_ptr(), n, 256 * 16, self.stream), 10, 3)
        return {"read_GBs": n / rd * 1e-6, "copy_GBs": 2 * n / cp * 1e-6}

    # -- synthetic packed weights on device -----------------------------------
    def rand_w4(self, N, K, gs, sym, copies=1):
        """Random packed codes with N(0,0.02)-like FP16 scales, generated on the
        device (timing only; parity is the test suite's job)."""
        torch, capi = self.torch, self.capi
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

    def rand_mx(self, N, K, copies=1):
        torch, capi = self.torch, self.capi
        B, wk = (K + 31) // 32, (K + 7) // 8
        out = []
        for _ in range(copies):
            q = torch.randint(-2**31, 2**31 - 1, (N * wk,), dtype=torch.int32, device="cuda")
            s = torch.randint(118, 123, (N * B,), dtype=torch.uint8, device="cuda")
            out.append((capi.packed_mx_view(N, K, B, q.data_ptr(), s.data_ptr()), (q, s)))
        return out

    def gemm_us(self, fn, views, M, N, K):
        """us per call, rotating through `views` (one view = cache-warm)."""
        torch = self.torch
        x = torch.randn(M * K, device="cuda").to(torch.float16)
        c = torch.empty(M * N, dtype=torch.float16, device="cuda")
        ms = self.loop_ms(fn, [v[0] for v in views], x.data_ptr(), c.data_ptr(), M, self.steps, self.warmup)
        return ms * 1e3


def w4_bytes(N, K, gs, sym, M):
    G = (K + gs - 1) // gs
    b = N * ((K + 7) // 8) * 4 + N * G * 2 + 2 * M * K + 2 * M * N
    if not sym:
        b += N * ((G + 7) // 8) * 4
    return b


def mx_bytes(N, K, M):
    return N * ((K + 7) // 8) * 4 + N * ((K + 31) // 32) + 2 * M * K + 2 * M * N


def headline(b, args):
    """C1 on the GPU: real quantized weights (hook checked against the oracle at
    bench size), cold-rotated and warm timings."""
    import orc
    np, torch, capi = b.np, b.torch, b.capi
    from devutil import DevPacked, bits, halves, ptr, to_dev
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
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    t_gemm = time.perf_counter() - t0
    # bounded CPU sample: repeat dequant_all + gemm_oracle (the CPU equivalent of
    # one fused call) a few more times and keep the median
    cpu = [t_deq + t_gemm]
    for _ in range(4):
        t0 = time.perf_counter()
        orc.gemm_oracle(x, M, K, orc.dequant_all(p), N)
        cpu.append(time.perf_counter() - t0)
    cpu_s = sorted(cpu)[len(cpu) // 2]

    dp = DevPacked(p)
    x_d, c_d, w_d = to_dev(x), halves(M * N, 0x7E00), halves(N * K, 0x7E00)
    capi.gemm(dp.view, ptr(x_d), ptr(c_d), M, b.stream, ptr(w_d))
    hook_ok = bool(np.array_equal(bits(w_d), w_ref))
    rel = orc.rel_l2(bits(c_d).view(np.float16), ref)
    del w_d

    nbytes = w4_bytes(N, K, gs, True, M)
    copies = max(2, int(400e6 // nbytes) + 1)  # ~400 MB of distinct weights
    views = [(dp.view, dp)]
    for _ in range(copies - 1):
        d2 = DevPacked(p)
        views.append((d2.view, d2))
    vlist = [v[0] for v in views]
    # the K timed steps: one C launch loop bracketed by HIP events on the launch
    # stream.  With --extras none the pre-warm + W + K launches (all the same
    # cold-rotated workload) are the only ones of the headline kernel in the
    # process, so a profiler's per-kernel average covers exactly this workload.
    # bring the clocks up before the timed region: the first few hundred launches after idle run
    # ~20 % slower.  Untimed, same kernel and workload as the timed steps.
    b.loop_ms("w4_gemm", vlist, ptr(x_d), ptr(c_d), M, PREWARM_LAUNCHES, 0, reps=1)
    cold_ms = b.loop_ms("w4_gemm", vlist, ptr(x_d), ptr(c_d), M, args.steps, args.warmup, reps=1)
    more = {}
    if args.extras != "none":
        more["cold_median5_ms"] = b.loop_ms("w4_gemm", vlist, ptr(x_d), ptr(c_d), M, args.steps, 2)
        more["warm_ms"] = b.loop_ms("w4_gemm", vlist[:1], ptr(x_d), ptr(c_d), M, args.steps, args.warmup)
    return {
        "N": N, "K": K, "gs": gs, "M": M, "bytes": nbytes, "copies": copies,
        "cold_ms": cold_ms, **more, "hook_bitwise": hook_ok, "rel_l2_vs_oracle": rel,
        "cpu": {"quantize_s": t_quant, "dequant_all_s": t_deq, "gemm_oracle_s": t_gemm,
                "fused_equiv_s": cpu_s},
    }


def extras_gemm(b, full):
    """Configs 2-4: per-M timings of both kernels (crossover), MXFP4, prefill."""
    capi, torch = b.capi, b.torch
    out = {}
    # C2: asymmetric N=11008, K=4096
    rows = []
    shapes = [(11008, 4096, 128)] + ([(11008, 4096, 32), (11008, 4096, 48), (11008, 4104, 8)] if full else [])
    for (N, K, gs) in shapes:
        copies = max(2, int(400e6 // w4_bytes(N, K, gs, False, 1)) + 1)
        views = b.rand_w4(N, K, gs, False, copies)
        for M in (1, 2, 4, 8, 9, 16, 64):
            nb = w4_bytes(N, K, gs, False, M)
            us_s = b.gemm_us("w4_gemm_fused", views, M, N, K)
            us_m = b.gemm_us("w4_gemm_mma", views, M, N, K)
            rows.append({"N": N, "K": K, "gs": gs, "M": M, "bytes": nb, "simt_us": us_s, "mfma_us": us_m,
                         "simt_GBs": nb / us_s * 1e-3, "mfma_GBs": nb / us_m * 1e-3,
                         "winner": "simt" if us_s <= us_m else "mfma"})
        del views
        torch.cuda.empty_cache()
    out["c2_w4_asym"] = rows
    # C3: MXFP4 N=14336 K=4096
    rows = []
    N, K = 14336, 4096
    views = b.rand_mx(N, K, max(2, int(400e6 // mx_bytes(N, K, 1)) + 1))
    for M in (1, 16, 128):
        nb = mx_bytes(N, K, M)
        us_s = b.gemm_us("w4_gemm_fused_mx", views, M, N, K) if M <= 16 else None
        us_m = b.gemm_us("w4_gemm_mma_mx", views, M, N, K)
        rows.append({"N": N, "K": K, "M": M, "bytes": nb, "simt_us": us_s, "mfma_us": us_m,
                     "best_GBs": nb / min(u for u in (us_s, us_m) if u) * 1e-3,
                     "mfma_TFLOPs": 2.0 * M * N * K / us_m * 1e-6})
    del views
    torch.cuda.empty_cache()
    out["c3_mxfp4"] = rows
    # C4: prefill M=2048, N=K=4096 + two-pass baseline (dequant + hipBLASLt)
    N = K = 4096
    M = 2048
    views = b.rand_w4(N, K, 128, True, 1)
    x = torch.randn(M * K, device="cuda").to(torch.float16)
    c = torch.empty(M * N, dtype=torch.float16, device="cuda")
    w16 = torch.empty(N * K, dtype=torch.float16, device="cuda")
    st = b.stream
    steps = max(5, b.steps // 10)
    fused_ms = _median_events_ms(torch, lambda i: capi.gemm(views[0][0], x.data_ptr(), c.data_ptr(), M, st, 0),
                                 steps, 3)

    def two_pass(i):
        capi.dequant(views[0][0], w16.data_ptr(), st)
        capi.gemm_fp16(w16.data_ptr(), x.data_ptr(), c.data_ptr(), M, N, K, st)
    two_ms = _median_events_ms(torch, two_pass, steps, 3)
    blas_ms = _median_events_ms(torch, lambda i: capi.gemm_fp16(w16.data_ptr(), x.data_ptr(), c.data_ptr(),
                                                                M, N, K, st), steps, 3)
    flop = 2.0 * M * N * K
    out["c4_prefill"] = {"M": M, "N": N, "K": K, "flop": flop, "fused_ms": fused_ms,
                         "fused_TFLOPs": flop / fused_ms * 1e-9, "two_pass_ms": two_ms,
                         "two_pass_TFLOPs": flop / two_ms * 1e-9, "hipblaslt_only_TFLOPs": flop / blas_ms * 1e-9,
                         "frac_of_mfma_peak": flop / fused_ms * 1e-9 / MFMA_F16_PEAK_TFLOPS}
    # the same kernel on the other formats it takes, and on a thin and a large grid
    rows = []
    del views
    fmts = [("w4_asym_gs128", lambda: b.rand_w4(N, K, 128, False, 1), capi.gemm),
            ("w4_sym_gs32", lambda: b.rand_w4(N, K, 32, True, 1), capi.gemm),
            ("mxfp4", lambda: b.rand_mx(N, K, 1), capi.gemm_mx)]
    for name, make, fn in fmts:
        v = make()
        ms = _median_events_ms(torch, lambda i: fn(v[0][0], x.data_ptr(), c.data_ptr(), M, st, 0), steps, 3)
        rows.append({"weights": name, "M": M, "us": ms * 1e3, "TFLOPs": flop / ms * 1e-9})
        del v
    v = b.rand_w4(N, K, 128, True, 1)
    for M2 in (256, 4096) if full else (256,):
        x2 = torch.randn(M2 * K, device="cuda").to(torch.float16)
        c2 = torch.empty(M2 * N, dtype=torch.float16, device="cuda")
        ms = _median_events_ms(torch, lambda i: capi.gemm(v[0][0], x2.data_ptr(), c2.data_ptr(), M2, st, 0),
                               steps, 3)
        rows.append({"weights": "w4_sym_gs128", "M": M2, "us": ms * 1e3, "TFLOPs": 2.0 * M2 * N * K / ms * 1e-9})
    out["c4_prefill_other"] = rows
    return out


def extras_attention(b, full):
    """Config 5: B=8, Hq=32, Hkv=8, D=128, S=32768, one query token per sequence."""
    capi, torch = b.capi, b.torch
    Bq, Hq, Hkv, D, S = 8, 32, 8, 128, 32768
    if not full:
        S = 32768
    group, H = Hq // Hkv, Bq * Hkv
    st = b.stream
    q = torch.randn(H * group * D, device="cuda").to(torch.float16)
    o = torch.empty(H * group * D, dtype=torch.float16, device="cuda")
    res = {"B": Bq, "Hq": Hq, "Hkv": Hkv, "D": D, "S": S}
    steps = max(5, b.steps // 20)
    # FP16 cache
    k16 = torch.randn(H * S * D, device="cuda", dtype=torch.float16)
    v16 = torch.randn(H * S * D, device="cuda", dtype=torch.float16)
    ms = _median_events_ms(torch, lambda i: capi.attention_fp16_flash(
        q.data_ptr(), k16.data_ptr(), v16.data_ptr(), o.data_ptr(), H, S, D, st, group=group), steps, 2)
    nb = 2 * H * S * D * 2
    res["fp16"] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    del k16, v16
    torch.cuda.empty_cache()
    # W4 gs=32 symmetric
    gs, G, wd = 32, 4, D // 8
    qk = torch.randint(-2**31, 2**31 - 1, (H * S * wd,), dtype=torch.int32, device="cuda")
    qv = torch.randint(-2**31, 2**31 - 1, (H * S * wd,), dtype=torch.int32, device="cuda")
    sk = (torch.rand(H * S * G, device="cuda") * 0.2 + 0.2).to(torch.float16)
    sv = (torch.rand(H * S * G, device="cuda") * 0.2 + 0.2).to(torch.float16)
    view = capi.kv_view(H, S, D, gs, G, True, qk.data_ptr(), sk.data_ptr(), 0, qv.data_ptr(), sv.data_ptr(), 0)
    ms = _median_events_ms(torch, lambda i: capi.attention_w4_flash(view, q.data_ptr(), o.data_ptr(), st,
                                                                    group=group), steps, 2)
    nb = 2 * (H * S * wd * 4 + H * S * G * 2)
    res["w4_gs32"] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    # paged W4, page 16: sequences 0-3 share their first 8192 tokens
    page, prefix = 16, 8192
    lp, pp = S // page, prefix // page
    npages = pp + 4 * (lp - pp) + 4 * lp
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
    rows = npages * page
    pqk = torch.randint(-2**31, 2**31 - 1, (Hkv * rows * wd,), dtype=torch.int32, device="cuda")
    pqv = torch.randint(-2**31, 2**31 - 1, (Hkv * rows * wd,), dtype=torch.int32, device="cuda")
    psk = (torch.rand(Hkv * rows * G, device="cuda") * 0.2 + 0.2).to(torch.float16)
    psv = (torch.rand(Hkv * rows * G, device="cuda") * 0.2 + 0.2).to(torch.float16)
    pview = capi.kv_view(Hkv, S, D, gs, G, True, pqk.data_ptr(), psk.data_ptr(), 0, pqv.data_ptr(),
                         psv.data_ptr(), 0)
    ms = _median_events_ms(torch, lambda i: capi.attention_w4_flash_paged_batched(
        pview, tables.data_ptr(), Bq, lp, page, npages, group, q.data_ptr(), o.data_ptr(), st), steps, 2)
    uniq = 2 * Hkv * rows * (wd * 4 + G * 2)
    res["paged_w4_page16"] = {"ms": ms, "bytes_logical": nb, "bytes_unique": uniq, "GBs_logical": nb / ms * 1e-6,
                              "vs_contiguous": res["w4_gs32"]["ms"] / ms}
    del qk, qv, sk, sv, pqk, pqv, psk, psv
    torch.cuda.empty_cache()
    # FP8 E4M3: per-(row, group=128) scales and per-slab scale
    k8 = torch.randint(0, 0x7E, (H * S * D,), dtype=torch.uint8, device="cuda")
    v8 = torch.randint(0, 0x7E, (H * S * D,), dtype=torch.uint8, device="cuda")
    s8k = (torch.rand(H * S, device="cuda") * 0.005 + 0.005).to(torch.float16)
    s8v = (torch.rand(H * S, device="cuda") * 0.005 + 0.005).to(torch.float16)
    v8w = capi.kv_f8_view(H, S, D, 128, 1, k8.data_ptr(), s8k.data_ptr(), v8.data_ptr(), s8v.data_ptr())
    ms = _median_events_ms(torch, lambda i: capi.attention_f8_flash(v8w, q.data_ptr(), o.data_ptr(), st,
                                                                    group=group), steps, 2)
    nb = 2 * H * S * D + 2 * H * S * 2
    res["fp8_row_scale"] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    ms = _median_events_ms(torch, lambda i: capi.attention_f8_flash(v8w, q.data_ptr(), o.data_ptr(), st,
                                                                    group=group, scale_mode=1), steps, 2)
    nb = 2 * H * S * D
    res["fp8_head_scale"] = {"ms": ms, "bytes": nb, "GBs": nb / ms * 1e-6}
    return {"c5_flash_decode": res}


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


def probe(b, which):
    """Short fixed workloads for counter runs under a profiler (no headline, no yardsticks)."""
    capi, torch = b.capi, b.torch
    out = {"probe": which}
    if which == "decode":  # C2 shape, symmetric: vector kernel at M=1, matrix-core kernels at M=8 and 16
        N, K = 11008, 4096
        views = b.rand_w4(N, K, 128, True, 18)
        for M, fn in ((1, "w4_gemm_fused"), (8, "w4_gemm_mma"), (16, "w4_gemm_mma")):
            out["%s_M%d_us" % (fn, M)] = b.gemm_us(fn, views, M, N, K)
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
    else:  # prefill: the fused tile kernel and the plain FP16 library GEMM, 20 calls each
        N = K = 4096
        M = 2048
        views = b.rand_w4(N, K, 128, True, 1)
        x = torch.randn(M * K, device="cuda").to(torch.float16)
        c = torch.empty(M * N, dtype=torch.float16, device="cuda")
        w16 = torch.empty(N * K, dtype=torch.float16, device="cuda")
        capi.dequant(views[0][0], w16.data_ptr(), b.stream)
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
    ap.add_argument("--extras", choices=["none", "quick", "full"], default="quick")
    ap.add_argument("--probe", choices=["decode", "prefill", "quantize", "w4a4", "attention"], default=None,
                    help="run only a short fixed workload (for counter collection) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus N with N > 1 is not supported "
              "(the path shards over N or (batch, kv-head) with no exchange)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    b = Bench(args.steps, args.warmup)
    if args.probe:
        b.steps, b.warmup = 30, 5
        probe(b, args.probe)
        return
    h = headline(b, args)
    bw = b.bandwidth()
    cold_gbs = h["bytes"] / h["cold_ms"] * 1e-6
    extra = {"headline": h, "yardstick": bw,
             "cold_frac_of_measured_read": cold_gbs / bw["read_GBs"],
             "cold_frac_of_measured_copy": cold_gbs / bw["copy_GBs"],
             "cold_us": h["cold_ms"] * 1e3, "device": torch.cuda.get_device_name(0)}
    if "warm_ms" in h:
        extra["warm_us"] = h["warm_ms"] * 1e3
        extra["warm_GBs"] = h["bytes"] / h["warm_ms"] * 1e-6
    if args.extras != "none":
        extra.update(extras_gemm(b, args.extras == "full"))
        extra.update(extras_attention(b, args.extras == "full"))
        extra.update(extras_quantize(b, args.extras == "full"))
        extra.update(extras_w4a4(b, args.extras == "full"))
    cpu = h["cpu"]
    line = {
        "metric": "M=1 W4 GEMM us + achieved HBM GB/s (% of peak); M=2048 MFMA TFLOP/s",
        "value": cold_gbs, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": h["cold_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "W4A16 symmetric gs=128 fused GEMM, M=1, N=4096, K=4096 (north_star target "
                               "shape; weights rotated through %d HBM copies)" % h["copies"],
                   "entry": "w4_gemm", "bytes_per_step": h["bytes"]},
        "roofline": {"bound": "hbm", "achieved": cold_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": cold_gbs / HBM_PEAK_GBS, "traffic": HEADLINE_TRAFFIC_BYTES},
        "cpu_baseline": {"value": h["bytes"] / cpu["fused_equiv_s"] * 1e-9, "unit": "GB/s",
                         "cores": 1, "kind": "port",
                         "sample": "oracle dequant_all + gemm_oracle on the same 4096x4096 matrix, median of 5 "
                                   "(%.3f s); quantize %.3f s" % (cpu["fused_equiv_s"], cpu["quantize_s"])},
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
