"""GPU parity gates for the device-side quantizers, through the C ABI.

The kernels must write the bytes the host quantizers write (pack.hpp:64-130,
mx.hpp:71-119, kvcache.hpp:60-108, kvfp8.hpp:70-128; the oracle restates them
and is pinned against the reference's hand vectors by the CPU suite).  Every
comparison here is bit-exact.  Data-dependent failures the host reports by
throwing arrive in the status word: bit 0 non-finite input, bit 1 scale out of
range.
"""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DEV, ptr, to_dev

pytestmark = pytest.mark.gpu


def _status():
    return torch.full((1,), -1, dtype=torch.int32, device=DEV)


def _host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def _dev_quantize(w, N, K, gs, sym):
    c = w4amd.capi()
    G = (K + gs - 1) // gs
    # poisoned outputs: the kernels own every word they are responsible for
    q = torch.full((N * orc.words(K),), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    s = torch.full((N * G,), 0x7E00, dtype=torch.int16, device=DEV)
    z = None if sym else torch.full((N * orc.words(G),), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    st = _status()
    wd = to_dev(np.ascontiguousarray(w, np.float64))
    c.quantize(c.packed_view(N, K, gs, G, sym, ptr(q), ptr(s), ptr(z)), ptr(wd), ptr(st))
    return (_host(q).view(np.uint32), _host(s).view(np.uint16),
            None if sym else _host(z).view(np.uint32), int(_host(st)[0]))


def _check_w4(w, N, K, gs, sym):
    ref = orc.quantize(w, N, K, gs, sym)
    q, s, z, st = _dev_quantize(w, N, K, gs, sym)
    assert st == 0
    assert np.array_equal(s, ref.scales), "scales"
    if not sym:
        assert np.array_equal(z, ref.zeros), "zero-points"
    assert np.array_equal(q, ref.q), "codes"


W4_SHAPES = [(3, 64, 32), (5, 200, 64), (2, 4096, 128), (7, 100, 24), (1, 8, 8), (4, 77, 16),
             (3, 1001, 128), (2, 5000, 4096), (2, 2200, 2048), (9, 130, 136), (16, 333, 8),
             (2, 11008, 128), (1, 1, 8), (300, 48, 48),
             # full power-of-two groups (the lane-exchange kernel), with and without whole
             # zero-point words per workgroup
             (5, 1024, 32), (3, 512, 64), (2, 2048, 256), (2, 4096, 512), (70, 64, 8), (3, 1536, 512)]


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(W4_SHAPES)))
def test_quantize_w4_matches_host(i, sym):
    N, K, gs = W4_SHAPES[i]
    gen = [orc.normal_weights, orc.laplace_weights, orc.uniform_weights][i % 3]
    w = gen(N * K, 0xA11CE + i)
    _check_w4(w, N, K, gs, sym)


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
def test_quantize_w4_special_groups(sym):
    """Ties of the code rounding, the two-step FP64 -> FP32 -> FP16 scale rounding,
    all-zero and single-value groups, signed zeros, FP16-subnormal scales, one-sided
    groups (zero-point clamped to the code range)."""
    gs, rows = 16, []
    rows.append([7.0, -7.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5, 6.5, -6.5, 0.0, -0.0, 4.5, 5.5])
    rows.append([0.0] * 16)
    rows.append([-0.0] * 16)
    rows.append([0.0] * 15 + [3.0])
    step = 1.0 + 2.0 ** -11 + 2.0 ** -30  # rounds to 1.0 in two steps, 1 + 2^-10 in one
    rows.append([7.0 * step] + [step * t for t in (0.5, 1.5, -2.5, 3.4999, -6.5)] + [0.1] * 10)
    rows.append([15.0 * step, 0.0] + [step * (t + 0.5) for t in range(14)])
    rows.append([1e-6 * t for t in range(-8, 8)])          # subnormal FP16 scale
    rows.append([3e-7 * t for t in range(16)])
    rows.append([5.0 + 0.01 * t for t in range(16)])        # all positive
    rows.append([-5.0 - 0.01 * t for t in range(16)])       # all negative
    rows.append([60000.0 * 7 / 7.5] * 8 + [-1.0] * 8)       # large but representable scale
    w = np.array(rows, np.float64)
    _check_w4(w.ravel(), w.shape[0], gs, gs, sym)
    _check_w4(w.ravel(), 1, w.size, gs, sym)


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
def test_quantize_w4_status_word(sym):
    N, K, gs = 4, 64, 32
    base = orc.normal_weights(N * K, 99)
    for bad, bit, text in [(np.nan, 1, "non-finite"), (np.inf, 1, "non-finite"),
                           (-np.inf, 1, "non-finite"), (1e7, 2, "FP16 range"),
                           (1e-9, 2, "FP16 range")]:
        w = base.copy()
        if bit == 2 and bad < 1:
            w[gs:2 * gs] = 0.0
        w[gs + 3] = bad
        with pytest.raises(ValueError, match=text):
            orc.quantize(w, N, K, gs, sym)
        assert _dev_quantize(w, N, K, gs, sym)[3] & bit
    # the call clears a stale status
    assert _dev_quantize(base, N, K, gs, sym)[3] == 0


def test_quantize_w4_headline_shape():
    N = K = 4096
    w = orc.normal_weights(N * K, 7)
    _check_w4(w, N, K, 128, True)
    _check_w4(w, N, K, 128, False)


# ---- MXFP4 -------------------------------------------------------------------
def _dev_quantize_mx(w, N, K):
    c = w4amd.capi()
    B = (K + 31) // 32
    q = torch.full((N * orc.words(K),), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    s = torch.full((N * B,), 0x5A, dtype=torch.uint8, device=DEV)
    st = _status()
    wd = to_dev(np.ascontiguousarray(w, np.float64))
    c.quantize_mx(c.packed_mx_view(N, K, B, ptr(q), ptr(s)), ptr(wd), ptr(st))
    return _host(q).view(np.uint32), _host(s), int(_host(st)[0])


def _check_mx(w, N, K):
    ref = orc.quantize_mx(w, N, K)
    q, s, st = _dev_quantize_mx(w, N, K)
    assert st == 0
    assert np.array_equal(s, ref.scales), "E8M0 bytes"
    assert np.array_equal(q, ref.q), "codes"


MX_SHAPES = [(3, 64), (5, 200), (2, 4096), (7, 100), (1, 8), (4, 77), (3, 1001), (1, 1),
             (2, 14336), (33, 31), (6, 33)]


@pytest.mark.parametrize("i", range(len(MX_SHAPES)))
def test_quantize_mx_matches_host(i):
    N, K = MX_SHAPES[i]
    gen = [orc.normal_weights, orc.laplace_weights, orc.uniform_weights][i % 3]
    _check_mx(gen(N * K, 0xB0B + i), N, K)


def test_quantize_mx_scale_boundaries_and_ties():
    """Block maxima on, just above and just below 6 * 2^e for many e; values on the
    midpoints between E2M1 magnitudes (the lower one wins); signed zeros; blocks whose
    exponent clamps at -127; the largest representable scale."""
    rows = []
    for e in list(range(-130, -120)) + list(range(-20, 21)) + list(range(118, 128)):
        top = 6.0 * 2.0 ** e
        for amax in (top, np.nextafter(top, np.inf), np.nextafter(top, 0.0), 0.75 * top,
                     np.nextafter(0.5 * top, np.inf)):
            if amax > 6.0 * 2.0 ** 127:
                continue  # the host rejects it (covered by the status-word test)
            unit = 2.0 ** max(e, -127) if amax <= top else 2.0 ** max(e + 1, -127)
            mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -1.25, -5.0, 0.0, -0.0]
            row = [amax, -amax] + [m * unit for m in mids]
            row += [np.nextafter(m * unit, np.inf) for m in mids[:7]]
            row += [np.nextafter(m * unit, 0.0) for m in mids[:7]]
            row = [x for x in row if abs(x) <= amax][:32]
            rows.append(row + [0.0] * (32 - len(row)))
    rows.append([0.0] * 32)
    rows.append([-0.0] * 32)
    rows.append([1e-45] * 32)
    w = np.array(rows, np.float64)
    _check_mx(w.ravel(), w.shape[0], 32)
    _check_mx(w.ravel(), 1, w.size)


def test_quantize_mx_status_word():
    N, K = 3, 96
    base = orc.normal_weights(N * K, 5)
    for bad, bit, text in [(np.nan, 1, "non-finite"), (-np.inf, 1, "non-finite"),
                           (6.0 * 2.0 ** 127 * 1.01, 2, "E8M0 range")]:
        w = base.copy()
        w[40] = bad
        with pytest.raises(ValueError, match=text):
            orc.quantize_mx(w, N, K)
        assert _dev_quantize_mx(w, N, K)[2] & bit
    assert _dev_quantize_mx(base, N, K)[2] == 0


# ---- KV caches ---------------------------------------------------------------
KV_SHAPES = [(2, 7, 64, 8), (4, 128, 128, 32), (1, 300, 96, 32), (3, 65, 40, 8), (2, 33, 128, 128),
             (1, 1, 8, 8), (2, 50, 100, 24), (8, 512, 128, 64)]


def _sources(H, S, D, seed, f16):
    k = orc.normal_weights(H * S * D, seed)
    v = orc.laplace_weights(H * S * D, seed + 1) * 20.0
    if f16:
        k16, v16 = k.astype(np.float16), v.astype(np.float16)
        return k16.astype(np.float64), v16.astype(np.float64), to_dev(k16), to_dev(v16)
    return k, v, to_dev(k), to_dev(v)


@pytest.mark.parametrize("f16", [False, True], ids=["f64src", "f16src"])
@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(KV_SHAPES)))
def test_quantize_cache_matches_host(i, sym, f16):
    H, S, D, gs = KV_SHAPES[i]
    c = w4amd.capi()
    k, v, kd, vd = _sources(H, S, D, 0xCAFE + i, f16)
    ref = orc.quantize_cache(k, v, H, S, D, gs, sym)
    rows, G = H * S, ref.G
    mk32 = lambda n: torch.full((n,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    mk16 = lambda n: torch.full((n,), 0x7E00, dtype=torch.int16, device=DEV)
    qk, qv, sk, sv = mk32(rows * orc.words(D)), mk32(rows * orc.words(D)), mk16(rows * G), mk16(rows * G)
    zk = None if sym else mk32(rows * orc.words(G))
    zv = None if sym else mk32(rows * orc.words(G))
    st = _status()
    view = c.kv_view(H, S, D, gs, G, sym, ptr(qk), ptr(sk), ptr(zk), ptr(qv), ptr(sv), ptr(zv))
    c.quantize_cache(view, ptr(kd), ptr(vd), ptr(st), src_f16=f16)
    assert int(_host(st)[0]) == 0
    for name, dev, want in [("s_k", sk, ref.s_k), ("s_v", sv, ref.s_v), ("q_k", qk, ref.q_k),
                            ("q_v", qv, ref.q_v), ("z_k", zk, ref.z_k), ("z_v", zv, ref.z_v)]:
        if want is not None:
            assert np.array_equal(_host(dev).view(want.dtype), want), name


@pytest.mark.parametrize("f16", [False, True], ids=["f64src", "f16src"])
@pytest.mark.parametrize("i", range(len(KV_SHAPES)))
def test_quantize_cache_f8_matches_host(i, f16):
    H, S, D, gs = KV_SHAPES[i]
    c = w4amd.capi()
    k, v, kd, vd = _sources(H, S, D, 0xF8F8 + i, f16)
    if not f16:
        # exercise the encoder's subnormal codes, ties and zeros inside a group
        k[:8] = [448.0, 2.0 ** -9 * 448, 1.5 * 2.0 ** -9 * 448, 0.0, -0.0, 17.0 * 2, 19.0 * 2, -447.9]
        kd = to_dev(k)
    ref = orc.quantize_cache_f8(k, v, H, S, D, gs)
    rows, G = H * S, ref.G
    qk = torch.full((rows * D,), 0x5A, dtype=torch.uint8, device=DEV)
    qv = torch.full((rows * D,), 0x5A, dtype=torch.uint8, device=DEV)
    sk = torch.full((rows * G,), 0x7E00, dtype=torch.int16, device=DEV)
    sv = torch.full((rows * G,), 0x7E00, dtype=torch.int16, device=DEV)
    st = _status()
    view = c.kv_f8_view(H, S, D, gs, G, ptr(qk), ptr(sk), ptr(qv), ptr(sv))
    c.quantize_cache_f8(view, ptr(kd), ptr(vd), ptr(st), src_f16=f16)
    assert int(_host(st)[0]) == 0
    assert np.array_equal(_host(sk).view(np.uint16), ref.s_k)
    assert np.array_equal(_host(sv).view(np.uint16), ref.s_v)
    assert np.array_equal(_host(qk), ref.q_k)
    assert np.array_equal(_host(qv), ref.q_v)


@pytest.mark.parametrize("f8", [False, True], ids=["w4", "f8"])
def test_quantize_cache_f16_sources_on_rounding_ties(f8):
    """FP16 sources divide in FP32 on the device; the host divides in FP64.  Rows built to
    put quotients exactly on, and one FP16 ulp either side of, the code-rounding ties, for
    scales of many magnitudes (FP16-subnormal ones included), must give the host's bytes."""
    c = w4amd.capi()
    rng = np.random.default_rng(12345)
    D = gs = 16
    rows = []
    for _ in range(6000):
        s = np.float16(rng.uniform(1, 2) * 2.0 ** rng.integers(-24, 12))
        with np.errstate(over="ignore"):
            top = np.float16((448.0 if f8 else 7.0) * float(s))
        if not np.isfinite(top) or float(top) == 0.0:
            continue
        ks = rng.integers(-7, 7, 14) + 0.5
        vals = (ks * float(s)).astype(np.float16)
        nudge = rng.integers(-1, 2, 14)
        vals = (vals.view(np.int16) + nudge.astype(np.int16)).view(np.float16)
        vals[~np.isfinite(vals) | (np.abs(vals) > np.abs(top))] = 0
        rows.append(np.concatenate([[top, -top if rng.integers(2) else np.float16(0)], vals]))
    k16 = np.array(rows, np.float16)
    v16 = k16[::-1].copy()
    H, S = 1, k16.shape[0]
    k, v = k16.astype(np.float64).ravel(), v16.astype(np.float64).ravel()
    kd, vd, st = to_dev(k16.ravel()), to_dev(v16.ravel()), _status()
    sk = torch.zeros(S, dtype=torch.int16, device=DEV)
    sv = torch.zeros(S, dtype=torch.int16, device=DEV)
    if f8:
        ref = orc.quantize_cache_f8(k, v, H, S, D, gs)
        qk = torch.zeros(S * D, dtype=torch.uint8, device=DEV)
        qv = torch.zeros(S * D, dtype=torch.uint8, device=DEV)
        c.quantize_cache_f8(c.kv_f8_view(H, S, D, gs, 1, ptr(qk), ptr(sk), ptr(qv), ptr(sv)),
                            ptr(kd), ptr(vd), ptr(st), src_f16=True)
    else:
        for sym in (True, False):
            ref = orc.quantize_cache(k, v, H, S, D, gs, sym)
            qk = torch.zeros(S * 2, dtype=torch.int32, device=DEV)
            qv = torch.zeros(S * 2, dtype=torch.int32, device=DEV)
            zk = None if sym else torch.zeros(S, dtype=torch.int32, device=DEV)
            zv = None if sym else torch.zeros(S, dtype=torch.int32, device=DEV)
            c.quantize_cache(c.kv_view(H, S, D, gs, 1, sym, ptr(qk), ptr(sk), ptr(zk), ptr(qv),
                                       ptr(sv), ptr(zv)), ptr(kd), ptr(vd), ptr(st), src_f16=True)
            assert np.array_equal(_host(qk).view(np.uint32), ref.q_k), sym
            assert np.array_equal(_host(qv).view(np.uint32), ref.q_v), sym
            if not sym:
                assert np.array_equal(_host(zk).view(np.uint32), ref.z_k)
    assert int(_host(st)[0]) == 0
    assert np.array_equal(_host(sk).view(np.uint16), ref.s_k)
    assert np.array_equal(_host(qk).view(ref.q_k.dtype), ref.q_k)
    assert np.array_equal(_host(qv).view(ref.q_v.dtype), ref.q_v)


def test_quantize_cache_f8_f16_sources_on_e4m3_midpoints():
    """FP16 sources whose quotients v / s sit exactly on, and one FP16 ulp either side of, the
    midpoints of the E4M3 grid (normal and subnormal), for scales with short significands so
    that midpoint times scale is an FP16 number: the device rounds v * (1 / s) and must give
    the bytes of the host's division, ties to the even code included."""
    c = w4amd.capi()
    rng = np.random.default_rng(777)
    D = gs = 16
    rows = []
    for _ in range(8000):
        s = np.float16((1 + rng.integers(0, 16) / 16.0) * 2.0 ** rng.integers(-20, 6))
        with np.errstate(over="ignore"):
            top = np.float16(448.0 * float(s))
        if not np.isfinite(top) or float(top) == 0.0:
            continue
        e = rng.integers(-6, 9, 14)
        k = rng.integers(8, 16, 14)
        mids = (k + 0.5) * 2.0 ** (e - 3)
        sub = rng.integers(0, 4, 14) == 0
        mids[sub] = (rng.integers(0, 8, int(sub.sum())) + 0.5) * 2.0 ** -9
        sgn = rng.integers(0, 2, 14) * 2 - 1
        with np.errstate(over="ignore"):
            vals = (sgn * mids * float(s)).astype(np.float16)
        nudge = rng.integers(-1, 2, 14)
        vals = (vals.view(np.int16) + nudge.astype(np.int16)).view(np.float16)
        vals[~np.isfinite(vals) | (np.abs(vals) > np.abs(top))] = 0
        rows.append(np.concatenate([[top, np.float16(0)], vals]))
    k16 = np.array(rows, np.float16)
    v16 = k16[::-1].copy()
    H, S = 1, k16.shape[0]
    k, v = k16.astype(np.float64).ravel(), v16.astype(np.float64).ravel()
    # the rows are what they are meant to be: a fair share of exact midpoints
    q = np.abs(k16[:, 2:].astype(np.float64) / k16[:, :1].astype(np.float64) * 448.0)
    steps = q / 2.0 ** (np.floor(np.log2(np.maximum(q, 2.0 ** -6))) - 3)
    assert np.mean(np.abs(steps - np.floor(steps) - 0.5) == 0) > 0.2
    kd, vd, st = to_dev(k16.ravel()), to_dev(v16.ravel()), _status()
    sk = torch.zeros(S, dtype=torch.int16, device=DEV)
    sv = torch.zeros(S, dtype=torch.int16, device=DEV)
    ref = orc.quantize_cache_f8(k, v, H, S, D, gs)
    qk = torch.zeros(S * D, dtype=torch.uint8, device=DEV)
    qv = torch.zeros(S * D, dtype=torch.uint8, device=DEV)
    c.quantize_cache_f8(c.kv_f8_view(H, S, D, gs, 1, ptr(qk), ptr(sk), ptr(qv), ptr(sv)),
                        ptr(kd), ptr(vd), ptr(st), src_f16=True)
    assert int(_host(st)[0]) == 0
    assert np.array_equal(_host(sk).view(np.uint16), ref.s_k)
    assert np.array_equal(_host(qk), ref.q_k)
    assert np.array_equal(_host(qv), ref.q_v)


def test_quantize_cache_f16_sources_every_group_maximum():
    """Every finite FP16 magnitude as the maximum of a group: the scales of FP16 sources
    (an FP32 division on the device, FP64 -> FP32 -> FP16 on the host) agree for all of them."""
    c = w4amd.capi()
    mags = np.arange(0x0000, 0x7C00, dtype=np.uint16).view(np.float16)
    D = gs = 8
    k16 = np.zeros((mags.size, D), np.float16)
    k16[:, 3] = mags
    v16 = -k16
    v16[:, 5] = (mags.astype(np.float32) * 0.37).astype(np.float16)
    H, S = 1, mags.size
    k, v = k16.astype(np.float64).ravel(), v16.astype(np.float64).ravel()
    kd, vd = to_dev(k16.ravel()), to_dev(v16.ravel())
    # scales beyond FP16 (amax / 7 underflowing to zero) are the host's range error
    ok = np.ones(S, bool)
    for f8 in (False, True):
        div = 448.0 if f8 else 7.0
        ok &= (mags.astype(np.float64) / div).astype(np.float32).astype(np.float16) > 0
    ok[0] = True  # the all-zero group
    sel = np.nonzero(ok)[0]
    k, v = k.reshape(S, D)[sel].ravel(), v.reshape(S, D)[sel].ravel()
    kd, vd = to_dev(k16[sel].ravel()), to_dev(v16[sel].ravel())
    S = sel.size
    st = _status()
    sk = torch.zeros(S, dtype=torch.int16, device=DEV)
    sv = torch.zeros(S, dtype=torch.int16, device=DEV)
    for sym in (True, False):
        ref = orc.quantize_cache(k, v, H, S, D, gs, sym)
        qk = torch.zeros(S, dtype=torch.int32, device=DEV)
        qv = torch.zeros(S, dtype=torch.int32, device=DEV)
        zk = None if sym else torch.zeros(S, dtype=torch.int32, device=DEV)
        zv = None if sym else torch.zeros(S, dtype=torch.int32, device=DEV)
        c.quantize_cache(c.kv_view(H, S, D, gs, 1, sym, ptr(qk), ptr(sk), ptr(zk), ptr(qv), ptr(sv),
                                   ptr(zv)), ptr(kd), ptr(vd), ptr(st), src_f16=True)
        assert int(_host(st)[0]) == 0
        assert np.array_equal(_host(sk).view(np.uint16), ref.s_k)
        assert np.array_equal(_host(sv).view(np.uint16), ref.s_v)
        assert np.array_equal(_host(qk).view(np.uint32), ref.q_k)
        assert np.array_equal(_host(qv).view(np.uint32), ref.q_v)
    ref = orc.quantize_cache_f8(k, v, H, S, D, gs)
    bk = torch.zeros(S * D, dtype=torch.uint8, device=DEV)
    bv = torch.zeros(S * D, dtype=torch.uint8, device=DEV)
    c.quantize_cache_f8(c.kv_f8_view(H, S, D, gs, 1, ptr(bk), ptr(sk), ptr(bv), ptr(sv)), ptr(kd),
                        ptr(vd), ptr(st), src_f16=True)
    assert int(_host(st)[0]) == 0
    assert np.array_equal(_host(sk).view(np.uint16), ref.s_k)
    assert np.array_equal(_host(sv).view(np.uint16), ref.s_v)
    assert np.array_equal(_host(bk), ref.q_k)
    assert np.array_equal(_host(bv), ref.q_v)


def test_quantize_cache_status_word():
    c = w4amd.capi()
    H, S, D, gs = 2, 9, 64, 32
    k = orc.normal_weights(H * S * D, 1)
    v = orc.normal_weights(H * S * D, 2)
    v[100] = np.inf
    G = D // gs
    rows = H * S
    q = [torch.zeros(rows * orc.words(D), dtype=torch.int32, device=DEV) for _ in range(2)]
    s = [torch.zeros(rows * G, dtype=torch.int16, device=DEV) for _ in range(2)]
    st = _status()
    view = c.kv_view(H, S, D, gs, G, True, ptr(q[0]), ptr(s[0]), 0, ptr(q[1]), ptr(s[1]), 0)
    c.quantize_cache(view, ptr(to_dev(k)), ptr(to_dev(v)), ptr(st))
    assert int(_host(st)[0]) & 1  # an infinite input also drives its group's scale out of range
    b = [torch.zeros(rows * D, dtype=torch.uint8, device=DEV) for _ in range(2)]
    v[100] = 1e9  # amax / 448 overflows FP16
    view8 = c.kv_f8_view(H, S, D, gs, G, ptr(b[0]), ptr(s[0]), ptr(b[1]), ptr(s[1]))
    c.quantize_cache_f8(view8, ptr(to_dev(k)), ptr(to_dev(v)), ptr(st))
    assert int(_host(st)[0]) == 2
    with pytest.raises(ValueError, match="FP16 range"):
        orc.quantize_cache_f8(k, v, H, S, D, gs)
