"""The reference's host gates (tests/test_oracle.cpp) applied to the C oracle.

Same configs and seeds as the reference suite: per-element quantizer bounds,
hand pins, degenerate inputs, the invalid_argument list, KV slab layout, the
attention pins, FP8 bounds and the paged scatter.
"""
import numpy as np
import pytest

import orc

CFGS = [(1, 64, 64, 8), (8, 128, 96, 16), (16, 256, 100, 32), (4, 96, 72, 48),
        (2, 32, 128, 64), (3, 40, 256, 128), (5, 72, 40, 8)]
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


def nibbles(q, rows, K):
    """(rows, K) codes out of rows*words(K) packed words, low nibble first."""
    w = q.reshape(rows, -1)
    sh = (4 * np.arange(8, dtype=np.uint32))[None, None, :]
    return ((w[:, :, None] >> sh) & 0xF).reshape(rows, -1)[:, :K].astype(np.int64)


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("i", range(len(CFGS)))
def test_w4_per_element_bounds(i, sym):
    # test_oracle.cpp:23-61
    _, N, K, gs = CFGS[i]
    w = orc.normal_weights(N * K, 0x44A1 ^ (i * 977 + (0 if sym else 1)))
    p = orc.quantize(w, N, K, gs, sym)
    wd = f16(orc.dequant_all(p)).reshape(N, K)
    sf = np.repeat(f16(p.scales).reshape(N, p.G), gs, axis=1)[:, :K]
    q = nibbles(p.q, N, K)
    tol = np.where((q == 0) | (q == 15), 1.1, 0.52) * sf + 1e-12
    assert np.all(np.abs(wd - w.reshape(N, K)) <= tol)
    if sym:
        assert q.min() >= 1  # symmetric codes live in [1, 15]


def test_w4_rounding_ties_go_away_from_zero():
    """pack.hpp:113-121 rounds the zero-point and every code with std::lround, which
    sends halves away from zero.  Codes derived by hand on groups whose stored scale
    is exactly 1.0, so every quotient is the value itself; round-half-to-even would
    give 8, 8, 10, 6, 10, 6, 14 on the symmetric ties and zero-point 2 below."""
    # symmetric: amax = 7 -> scale 7/7 = 1.0, code = lround(w) + 8
    w = np.array([7.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 6.5])
    p = orc.quantize(w, 1, 8, 8, True)
    assert p.scales[0] == 0x3C00
    assert nibbles(p.q, 1, 8)[0].tolist() == [15, 9, 7, 10, 6, 11, 5, 15]
    # asymmetric: lo = -2.5, hi = 12.5 -> scale 15/15 = 1.0, z = lround(2.5) = 3,
    # code = clamp(lround(w) + 3): -2.5 -> -3 + 3 = 0, 12.5 -> 13 + 3 = 16 -> 15
    w = np.array([-2.5, 12.5, 0.5, -0.5, 1.5, 3.5, -1.5, 4.5])
    p = orc.quantize(w, 1, 8, 8, False)
    assert p.scales[0] == 0x3C00 and int(p.zeros[0] & 0xF) == 3
    assert nibbles(p.q, 1, 8)[0].tolist() == [0, 15, 4, 2, 5, 7, 1, 8]
    # a one-sided group: the range is widened to bracket zero (lo = 0, hi = 7.5 ->
    # scale 0.5, z = 0), codes lround(w / 0.5): 0.25 -> lround(0.5) = 1, 1.25 -> 3
    w = np.array([7.5, 0.25, 1.25, 2.0, 0.75, 3.25, 0.0, 5.0])
    p = orc.quantize(w, 1, 8, 8, False)
    assert p.scales[0] == 0x3800 and int(p.zeros[0] & 0xF) == 0
    assert nibbles(p.q, 1, 8)[0].tolist() == [15, 1, 3, 4, 2, 7, 0, 10]


def test_gemm_oracle_hand_pin():
    # test_oracle.cpp:63-78
    x = np.array([1, 2], np.float16).view(np.uint16)
    w = np.array([3, 4, 5, 6], np.float16).view(np.uint16)
    c = orc.gemm_oracle(x, 1, 2, w, 2)
    assert c[0, 0] == 11.0 and c[0, 1] == 17.0


def test_gemm_oracle_is_xwT():
    rng = np.random.default_rng(5)
    M, N, K = 5, 7, 33
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = rng.standard_normal((N, K)).astype(np.float16)
    c = orc.gemm_oracle(x.view(np.uint16), M, K, w.view(np.uint16), N)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.allclose(c, want, rtol=1e-13, atol=1e-13)
    assert not np.allclose(c, (w.astype(np.float64) @ x.astype(np.float64).T).T + 1e-3)


@pytest.mark.parametrize("sym", [True, False])
def test_all_zero_groups(sym):
    # test_oracle.cpp:80-94 and pack.hpp:102-104: scale 1.0, codes = zero-point
    p = orc.quantize(np.zeros(64 * 64), 64, 64, 32, sym)
    assert np.all(f16(orc.dequant_all(p)) == 0.0)
    assert np.all(f16(p.scales) == 1.0)
    assert np.all(nibbles(p.q, 64, 64) == (8 if sym else 0))


def test_w4_throw_contracts():
    # test_oracle.cpp:96-148
    ok = np.full(64 * 64, 0.5)
    for args in ((0, 64, 8), (64, 64, 0), (64, 64, 7), (64, 64, 9)):
        with pytest.raises(orc.OracleInvalid):
            orc.quantize(ok, args[0], args[1], args[2], True)
    with pytest.raises(orc.OracleInvalid):
        orc.quantize(np.zeros(10), 64, 64, 8, True)
    for sym in (True, False):
        bad = ok.copy()
        bad[3] = np.nan
        with pytest.raises(orc.OracleInvalid):
            orc.quantize(bad, 64, 64, 8, sym)
        bad[3] = 1e300
        with pytest.raises(orc.OracleInvalid):
            orc.quantize(bad, 64, 64, 8, sym)
        with pytest.raises(orc.OracleInvalid):
            orc.quantize(np.full(64 * 64, 1e-12), 64, 64, 8, sym)
    p = orc.quantize(ok, 64, 64, 8, True)
    p.gs = 7
    with pytest.raises(orc.OracleInvalid):
        orc.dequant_all(p)
    p = orc.quantize(ok, 64, 64, 8, True)
    p.q = p.q[:3].copy()
    with pytest.raises(orc.OracleInvalid):
        orc.dequant_all(p)
    with pytest.raises(orc.OracleInvalid):
        orc.gemm_oracle(np.zeros(3, np.uint16), 2, 2, np.zeros(4, np.uint16), 1)


MXCFGS = [(64, 64), (128, 96), (256, 100), (96, 72), (32, 33), (40, 256), (72, 40)]


@pytest.mark.parametrize("i", range(len(MXCFGS)))
def test_mx_bounds_and_no_saturation(i):
    # test_oracle.cpp:155-211
    N, K = MXCFGS[i]
    w = orc.normal_weights(N * K, 0x9E4F ^ (i * 977)).reshape(N, K)
    p = orc.quantize_mx(w, N, K)
    wd = f16(orc.dequant_all_mx(p)).reshape(N, K)
    s = np.repeat(2.0 ** (p.scales.reshape(N, p.B).astype(np.int64) - 127), 32, axis=1)[:, :K]
    idx = nibbles(p.q, N, K) & 7
    left = np.where(idx > 0, E2M1[idx] - E2M1[np.maximum(idx - 1, 0)], 0.5)
    right = np.where(idx < 7, E2M1[np.minimum(idx + 1, 7)] - E2M1[idx], left)
    tol = 0.5 * np.maximum(left, right) * s + 1e-12
    err = np.abs(wd - w)
    assert np.all(err <= tol)
    amax = np.array([[np.abs(w[n, b * 32:(b + 1) * 32]).max() for b in range(p.B)] for n in range(N)])
    sb = 2.0 ** (p.scales.reshape(N, p.B).astype(np.int64) - 127)
    assert np.all(amax <= 6.0 * sb * (1 + 1e-12))
    # and the scale is the smallest power of two that avoids saturation
    assert np.all(amax > 3.0 * sb)


def test_mx_hand_pins():
    # test_oracle.cpp:213-263
    p = orc.quantize_mx(np.full(64, 3.0), 2, 32)
    assert p.scales[0] == 126 and p.scales[1] == 126
    wd = f16(orc.dequant_all_mx(p))
    assert wd[0] == 3.0 and wd[63] == 3.0
    assert nibbles(p.q, 2, 32)[0, 0] == 7
    p = orc.quantize_mx(np.full(32, -2.0), 1, 32)
    assert f16(orc.dequant_all_mx(p))[0] == -2.0 and nibbles(p.q, 1, 32)[0, 0] & 8
    p = orc.quantize_mx(np.zeros(64 * 64), 64, 64)
    assert np.all(f16(orc.dequant_all_mx(p)) == 0.0) and np.all(p.scales == 127)
    # ties go to the lower magnitude index: 2.5 sits between 2 (idx 4) and 3 (idx 5)
    w = np.zeros(32)
    w[0], w[1] = 6.0, 2.5
    p = orc.quantize_mx(w, 1, 32)
    assert p.scales[0] == 127 and nibbles(p.q, 1, 32)[0, 1] == 4


def test_mx_throw_contracts():
    # test_oracle.cpp:265-301
    ok = np.full(64 * 64, 0.5)
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_mx(ok, 0, 64)
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_mx(np.zeros(10), 64, 64)
    bad = ok.copy()
    bad[3] = np.nan
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_mx(bad, 64, 64)
    bad[3] = 1e300
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_mx(bad, 64, 64)
    p = orc.quantize_mx(ok, 64, 64)
    p.q = p.q[:3].copy()
    with pytest.raises(orc.OracleInvalid):
        orc.dequant_all_mx(p)


@pytest.mark.parametrize("sym", [True, False])
def test_kv_slab_layout(sym):
    # test_oracle.cpp:313-331: the cache is H independent PackedW slabs
    H, S, D, gs = 3, 5, 24, 8
    k = orc.normal_weights(H * S * D, 0xC1)
    v = orc.normal_weights(H * S * D, 0xC2)
    c = orc.quantize_cache(k, v, H, S, D, gs, sym)
    kd = orc.dequant_cache(c, False)
    for h in range(H):
        ki = orc.dequant_all(orc.quantize(k[h * S * D:(h + 1) * S * D], S, D, gs, sym))
        assert np.array_equal(ki, kd[h].ravel())


def test_attention_zero_keys_is_mean_of_v():
    # test_oracle.cpp:333-357
    H, S, D = 1, 2, 8
    v = np.concatenate([np.full(D, 1.0), np.full(D, 3.0)])
    c = orc.quantize_cache(np.zeros(H * S * D), v, H, S, D, 8, True)
    vd = f16(orc.dequant_cache(c, True)).reshape(S, D)
    q = np.full(H * D, 1.0, np.float16).view(np.uint16)
    out = orc.attention_reference(q, c)
    assert np.array_equal(out[0], 0.5 * vd[0] + 0.5 * vd[1])


def test_attention_softmax_stability():
    # test_oracle.cpp:359-379: scores ~3e4 stay finite through max subtraction
    H, S, D = 1, 2, 8
    c = orc.quantize_cache(np.full(H * S * D, 100.0), np.full(H * S * D, 0.5), H, S, D, 8, True)
    q = np.full(H * D, 100.0, np.float16).view(np.uint16)
    out = orc.attention_reference(q, c)
    assert np.isfinite(out[0, 0]) and out[0, 0] == f16(orc.dequant_cache(c, True)).ravel()[0]


def test_attention_matches_numpy_softmax_and_gqa():
    rng = np.random.default_rng(11)
    H, S, D, R = 2, 37, 24, 3
    k = rng.standard_normal((H, S, D)).astype(np.float16)
    v = rng.standard_normal((H, S, D)).astype(np.float16)
    q = rng.standard_normal((H * R, D)).astype(np.float16)
    out = orc.attention_f16(q.view(np.uint16), k.view(np.uint16), v.view(np.uint16), H, R, S, D)
    for hq in range(H * R):
        kk, vv = k[hq // R].astype(np.float64), v[hq // R].astype(np.float64)
        s = kk @ q[hq].astype(np.float64) / np.sqrt(D)
        pr = np.exp(s - s.max())
        pr /= pr.sum()
        assert np.allclose(out[hq], pr @ vv, rtol=1e-12, atol=1e-14)
    # grouped heads equal the reference run on a replicated cache
    rep = orc.attention_f16(q.view(np.uint16), np.repeat(k, R, 0).view(np.uint16),
                            np.repeat(v, R, 0).view(np.uint16), H * R, 1, S, D)
    assert np.array_equal(out, rep)


def test_kv_throw_contracts():
    # test_oracle.cpp:381-428 (gs = 0 must throw, not divide)
    ok = np.full(4 * 8, 0.5)
    for (H, gs) in ((0, 8), (1, 7), (1, 0)):
        with pytest.raises(orc.OracleInvalid):
            orc.quantize_cache(ok, ok, H, 4, 8, gs, True)
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_cache(np.zeros(10), ok, 1, 4, 8, 8, True)


FCFGS = [(64, 64), (7, 96), (16, 100), (5, 40), (3, 72)]


@pytest.mark.parametrize("i", range(len(FCFGS)))
def test_f8_bounds_and_no_saturation(i):
    # test_oracle.cpp:436-508
    S, D = FCFGS[i]
    seed = 0x8F1D ^ (i * 977)
    k = orc.normal_weights(S * D, seed)
    v = orc.normal_weights(S * D, seed + 1)
    c = orc.quantize_cache_f8(k, v, 1, S, D, 32)
    wd = f16(orc.dequant_cache_f8(c, False)).reshape(S, D)
    tab = np.array([orc.lib().orc_decode_f8_e4m3(b) for b in range(0x7F)])
    sf = np.repeat(f16(c.s_k).reshape(S, c.G), 32, axis=1)[:, :D]
    mag = np.abs(np.array([orc.lib().orc_decode_f8_e4m3(int(b)) for b in c.q_k])).reshape(S, D)
    pos = np.searchsorted(tab, mag)
    prev_m = np.where(pos > 0, tab[np.maximum(pos - 1, 0)], 0.0)
    next_m = np.where(pos < len(tab) - 1, tab[np.minimum(pos + 1, len(tab) - 1)], mag + (mag - prev_m))
    tol = (0.5 * np.maximum(mag - prev_m, next_m - mag) + mag * 4.9e-4) * sf + 1e-12
    assert np.all(np.abs(wd - k.reshape(S, D)) <= tol)
    amax = np.array([[np.abs(k.reshape(S, D)[t, g * 32:(g + 1) * 32]).max() for g in range(c.G)] for t in range(S)])
    assert np.all(amax <= 448.0 * f16(c.s_k).reshape(S, c.G) * (1 + 1e-3))


def test_f8_hand_pins_and_throws():
    # test_oracle.cpp:510-605
    w = np.full(64, 1.0)
    c = orc.quantize_cache_f8(w, w, 1, 8, 8, 8)
    assert c.q_k[0] == 0x7E and f16(orc.dequant_cache_f8(c, False)).ravel()[0] == 1.0
    w = np.full(64, -2.0)
    c = orc.quantize_cache_f8(w, w, 1, 8, 8, 8)
    assert c.q_v[0] & 0x80 and f16(orc.dequant_cache_f8(c, True)).ravel()[0] == -2.0
    z = np.zeros(4 * 16)
    c = orc.quantize_cache_f8(z, z, 1, 4, 16, 8)
    assert np.all(f16(orc.dequant_cache_f8(c, False)) == 0.0) and np.all(f16(c.s_k) == 1.0)
    ok = np.full(4 * 8, 0.5)
    for (H, gs) in ((0, 8), (1, 0), (1, 7)):
        with pytest.raises(orc.OracleInvalid):
            orc.quantize_cache_f8(ok, ok, H, 4, 8, gs)
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_cache_f8(np.zeros(10), ok, 1, 4, 8, 8)
    bad = ok.copy()
    bad[3] = np.nan
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_cache_f8(bad, ok, 1, 4, 8, 8)
    bad[3] = 1e300
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_cache_f8(bad, ok, 1, 4, 8, 8)
    with pytest.raises(orc.OracleInvalid):
        orc.quantize_cache_f8(np.full(4 * 8, 1e-8), ok, 1, 4, 8, 8)


def test_paged_scatter_resolves_to_contiguous_rows():
    # test_oracle.cpp:612-675
    H, S, D, gs, page = 2, 37, 24, 8, 16
    k = orc.normal_weights(H * S * D, 0x7A11)
    v = orc.normal_weights(H * S * D, 0x7A12)
    c = orc.quantize_cache(k, v, H, S, D, gs, True)
    bt = np.array([2, 0, 1], np.int32)
    wd = orc.words(D)
    pq = orc.paged_scatter(c.q_k, H, S, page, bt, wd).reshape(H, 3 * page, wd)
    ps = orc.paged_scatter(c.s_v, H, S, page, bt, c.G).reshape(H, 3 * page, c.G)
    for h in range(H):
        for t in range(S):
            row = bt[t // page] * page + t % page
            assert np.array_equal(pq[h, row], c.q_k.reshape(H, S, wd)[h, t])
            assert np.array_equal(ps[h, row], c.s_v.reshape(H, S, c.G)[h, t])
    assert np.all(pq[:, 1 * page + 5:2 * page] == 0)  # tail of the ragged last page
    for badbt, pg in (([2, 0, 1], 0), ([0, 1], 16), ([0, 1, 1], 16), ([0, 1, 9], 16)):
        with pytest.raises(orc.OracleInvalid):
            orc.paged_scatter(c.q_k, H, S, pg, np.array(badbt, np.int32), wd)


def test_mx8_activation_format_closed_forms():
    """MXFP8 activations (an additive format, no reference counterpart): the block
    exponent is the smallest e with amax <= 448 * 2^e, representable values round-trip
    exactly, the per-element error is at most half an E4M3 step of the scaled value."""
    rows = []
    for e in range(-20, 20):
        top = 448.0 * 2.0 ** e
        for amax in (top, np.nextafter(top, np.inf), np.nextafter(top, 0.0)):
            rows.append([amax, -amax] + [amax * t / 30.0 for t in range(30)])
    x = np.array(rows)
    M, K = x.shape
    p = orc.quantize_mx8(x, M, K)
    amax = np.abs(x).max(axis=1)
    e = p.scales.astype(np.int64) - 127
    assert np.all(amax <= 448.0 * 2.0 ** e) and np.all(amax > 448.0 * 2.0 ** (e - 1))
    d = orc.dequant_mx8(p)
    step = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(x) / 2.0 ** e[:, None], 1e-300))) - 3), 2.0 ** -9)
    assert np.all(np.abs(d - x) <= 0.5 * step * 2.0 ** e[:, None] * (1 + 1e-9))
    p2 = orc.quantize_mx8(d, M, K)
    assert np.array_equal(orc.dequant_mx8(p2), d)
    assert np.array_equal(orc.quantize_mx8(np.zeros(32), 1, 32).scales, [127])
    with pytest.raises(ValueError, match="non-finite"):
        orc.quantize_mx8(np.full(32, np.nan), 1, 32)
    with pytest.raises(ValueError, match="E8M0 range"):
        orc.quantize_mx8(np.full(32, 1e300), 1, 32)
    # gemm_f64 against numpy
    a, b = orc.normal_weights(5 * 64, 1).reshape(5, 64), orc.normal_weights(7 * 64, 2).reshape(7, 64)
    assert np.allclose(orc.gemm_f64(a, 5, 64, b, 7), a @ b.T, rtol=1e-13, atol=1e-13)
