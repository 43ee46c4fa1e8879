"""GPU gates for the W4A4 path: both operands packed MXFP4, scaled matrix cores.

Separate from the W4A16 gates (the activations are quantized too, so the result is
a different number): the activation quantizer must write the host quantize_mx bytes
(mx.hpp:71-119) for the FP16 activations widened to FP64, and the GEMM must be within
rel L2 1e-3 of the FP64 product of the two dequantized operands (dequant_all_mx,
mx.hpp:131-140, and gemm_oracle, pack.hpp:150-170).  Where every partial sum is
exactly representable the result must match bit for bit.
"""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DEV, DevPackedMx, bits, halves, ptr, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3

SHAPES = [(1, 64, 512), (16, 256, 4096), (5, 100, 1000), (3, 48, 100), (33, 80, 640),
          (64, 128, 1024), (100, 64, 512), (17, 1024, 2048), (2, 33, 31), (48, 16, 96),
          (1, 16, 8), (200, 200, 200),
          # a few hundred rows on the skinny kernel's grid.y walk
          (128, 256, 512), (96, 64, 128), (200, 300, 1024), (300, 520, 384), (129, 257, 256),
          # many rows of X on the skinny kernel's grid.y walk (too few tiles for the tiled kernel)
          (384, 256, 512), (500, 300, 1024), (385, 520, 256),
          # K % 256 == 0 and at least 64 tiles of 256 x 128: the LDS-tiled kernel, ragged on both
          # sides, 2 to 5 stages of 256 k
          (900, 2100, 512), (1030, 2050, 768), (1024, 2048, 1280)]


def _quantize_x_on_device(x16, M, K):
    c = w4amd.capi()
    B = (K + 31) // 32
    q = torch.full((M * orc.words(K),), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    s = torch.full((M * B,), 0x5A, dtype=torch.uint8, device=DEV)
    st = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    xd = to_dev(x16)
    view = c.packed_mx_view(M, K, B, ptr(q), ptr(s))
    c.quantize_mx_f16(view, ptr(xd), ptr(st))
    torch.cuda.synchronize()
    assert int(st.item()) == 0
    return view, q, s


@pytest.mark.parametrize("i", range(len(SHAPES)))
def test_w4a4_matches_fp64_product(i):
    M, N, K = SHAPES[i]
    c = w4amd.capi()
    w = orc.normal_weights(N * K, 0x4A4 + i)
    x16 = orc.normal_activations(M * K, 0x4A5 + i)  # FP16 bit patterns
    xf = x16.view(np.float16).astype(np.float64)
    wq, xq = orc.quantize_mx(w, N, K), orc.quantize_mx(xf, M, K)
    ref = orc.gemm_oracle(orc.dequant_all_mx(xq), M, K, orc.dequant_all_mx(wq), N)
    # activations quantized on the device: the host's bytes
    xview, xq_d, xs_d = _quantize_x_on_device(x16, M, K)
    assert np.array_equal(xq_d.cpu().numpy().view(np.uint32), xq.q)
    assert np.array_equal(xs_d.cpu().numpy(), xq.scales)
    dw = DevPackedMx(wq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a4(dw.view, xview, ptr(out))
    got = bits(out).view(np.float16).astype(np.float64).reshape(M, N)
    assert orc.rel_l2(got, ref) <= TOL
    # codes past K in the last word of a row are ignored
    if K % 8:
        junk = np.uint32(0xFFFFFFFF) << np.uint32(4 * (K % 8))
        wq.q.reshape(N, -1)[:, -1] |= junk
        xq.q.reshape(M, -1)[:, -1] |= junk
        dw2, dx2 = DevPackedMx(wq), DevPackedMx(xq)
        out2 = halves(M * N, 0x7E00)
        c.gemm_mx_w4a4(dw2.view, dx2.view, ptr(out2))
        assert np.array_equal(bits(out2), bits(out))


E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6])


def _decode(p, rows):
    """E2M1 table times 2^(byte - 127), in FP64 (no FP16 rounding of the operands)."""
    K = p.K
    codes = (p.q.reshape(rows, -1)[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF
    vals = E2M1[codes.reshape(rows, -1)[:, :K]]
    scale = np.ldexp(1.0, p.scales.reshape(rows, -1).astype(np.int64) - 127)
    return vals * np.repeat(scale, 32, axis=1)[:, :K]


@pytest.mark.parametrize("M,N,K", [(16, 64, 512), (7, 40, 1536), (20, 24, 200)])
def test_w4a4_exact_when_sums_are_representable(M, N, K):
    """Codes in {0, +-0.5, +-1} with unit scales: every partial sum is a multiple of 0.25
    below 2048, exact in FP32 and FP16, so the output bits are determined."""
    c = w4amd.capi()
    rng = np.random.default_rng(K)
    pick = np.array([0, 1, 2, 9, 10], np.uint32)
    def pack(rows):
        codes = pick[rng.integers(0, 5, (rows, orc.words(K) * 8))]
        codes[:, K:] = 0
        q = (codes.reshape(rows, -1, 8) << (4 * np.arange(8, dtype=np.uint32))).sum(axis=2)
        return orc.PackedWm(rows, K, q.astype(np.uint32).ravel(),
                            np.full(rows * ((K + 31) // 32), 127, np.uint8))
    wq, xq = pack(N), pack(M)
    ref = _decode(xq, M) @ _decode(wq, N).T
    assert np.abs(ref).max() < 2048
    dw, dx = DevPackedMx(wq), DevPackedMx(xq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a4(dw.view, dx.view, ptr(out))
    assert np.array_equal(bits(out).view(np.float16).reshape(M, N), ref.astype(np.float16))


def test_w4a4_block_scales_far_from_fp16():
    """Weight scales around 2^+20 against activation scales around 2^-20: neither operand
    is representable in FP16, the products are; the instruction applies the scales exactly."""
    M, N, K = 12, 48, 1024
    c = w4amd.capi()
    rng = np.random.default_rng(3)
    wq = orc.quantize_mx(orc.normal_weights(N * K, 11), N, K)
    xq = orc.quantize_mx(orc.normal_weights(M * K, 12), M, K)
    wq.scales = (wq.scales.astype(np.int64) + rng.integers(15, 25, wq.scales.shape)).astype(np.uint8)
    xq.scales = (xq.scales.astype(np.int64) - rng.integers(15, 25, xq.scales.shape)).astype(np.uint8)
    ref = _decode(xq, M) @ _decode(wq, N).T
    dw, dx = DevPackedMx(wq), DevPackedMx(xq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a4(dw.view, dx.view, ptr(out))
    got = bits(out).view(np.float16).astype(np.float64).reshape(M, N)
    assert np.isfinite(got).all()
    assert orc.rel_l2(got, ref) <= TOL


def test_w4a4_decode_shapes_of_the_benchmarks():
    c = w4amd.capi()
    for (M, N, K) in [(1, 4096, 4096), (16, 14336, 4096), (64, 4096, 4096)]:
        w = orc.normal_weights(N * K, N + M)
        x16 = orc.normal_activations(M * K, K + M)
        wq = orc.quantize_mx(w, N, K)
        xq = orc.quantize_mx(x16.view(np.float16).astype(np.float64), M, K)
        ref = orc.gemm_oracle(orc.dequant_all_mx(xq), M, K, orc.dequant_all_mx(wq), N)
        dw, dx = DevPackedMx(wq), DevPackedMx(xq)
        out = halves(M * N, 0x7E00)
        c.gemm_mx_w4a4(dw.view, dx.view, ptr(out))
        got = bits(out).view(np.float16).astype(np.float64).reshape(M, N)
        assert orc.rel_l2(got, ref) <= TOL, (M, N, K)


def test_w4a4_prefill_shape_sampled_rows():
    """M = 2048, N = K = 4096: every output element of 96 sampled activation rows against
    the FP64 product (the full FP64 product is 3.4e10 multiply-adds)."""
    M, N, K = 2048, 4096, 4096
    c = w4amd.capi()
    wq = orc.quantize_mx(orc.normal_weights(N * K, 21), N, K)
    x16 = orc.normal_activations(M * K, 22)
    xq = orc.quantize_mx(x16.view(np.float16).astype(np.float64), M, K)
    dw, dx = DevPackedMx(wq), DevPackedMx(xq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a4(dw.view, dx.view, ptr(out))
    got = bits(out).view(np.float16).astype(np.float64).reshape(M, N)
    rows = np.unique(np.concatenate([np.arange(0, 16), np.arange(M - 16, M),
                                     np.random.default_rng(5).integers(0, M, 64)]))
    ref = _decode(xq, M)[rows] @ _decode(wq, N).T
    assert orc.rel_l2(got[rows], ref) <= TOL
    assert np.isfinite(got).all()


# ---- W4A8: MXFP4 weights against MXFP8 (E4M3, block-scaled) activations ---------------
W4A8_SHAPES = [(1, 64, 512), (16, 256, 4096), (5, 100, 992), (33, 80, 640), (64, 128, 1024),
               (100, 64, 512), (2, 33, 32), (48, 16, 96), (300, 520, 384),
               # at least 64 tiles and K % 256 == 0: the LDS-tiled kernel with 8-bit X
               (900, 2100, 512), (1030, 2050, 768), (1024, 2048, 1280)]


class _DevXm8:
    def __init__(self, p):
        c = w4amd.capi()
        self.q, self.s = to_dev(p.q), to_dev(p.scales)
        self.view = c.act_mx8_view(p.M, p.K, p.B, ptr(self.q), ptr(self.s))


@pytest.mark.parametrize("i", range(len(W4A8_SHAPES)))
def test_w4a8_matches_fp64_product(i):
    """Activations quantized on the device carry the host quantizer's bytes
    (include/w4/mxact.hpp, restated in the oracle); the product is within rel L2 1e-3 of
    the FP64 product of the two dequantized operands."""
    M, N, K = W4A8_SHAPES[i]
    c = w4amd.capi()
    w = orc.normal_weights(N * K, 0x8A8 + i)
    x16 = orc.normal_activations(M * K, 0x8A9 + i)
    xf = x16.view(np.float16).astype(np.float64)
    xf[::7] *= 37.0  # spread the block maxima (still FP16 values after the cast below)
    x16 = xf.astype(np.float16)
    xf = x16.astype(np.float64)
    wq, xq = orc.quantize_mx(w, N, K), orc.quantize_mx8(xf, M, K)
    wd = orc.dequant_all_mx(wq).view(np.float16).astype(np.float64)
    ref = orc.gemm_f64(orc.dequant_mx8(xq), M, K, wd, N)
    B = (K + 31) // 32
    q = torch.full((M * K,), 0x5A, dtype=torch.uint8, device=DEV)
    s = torch.full((M * B,), 0x5A, dtype=torch.uint8, device=DEV)
    st = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    xd = to_dev(x16)
    xview = c.act_mx8_view(M, K, B, ptr(q), ptr(s))
    c.quantize_mx8_f16(xview, ptr(xd), ptr(st))
    torch.cuda.synchronize()
    assert int(st.item()) == 0
    assert np.array_equal(s.cpu().numpy(), xq.scales)
    assert np.array_equal(q.cpu().numpy(), xq.q)
    dw = DevPackedMx(wq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a8(dw.view, xview, ptr(out))
    got = bits(out).view(np.float16).astype(np.float64).reshape(M, N)
    assert orc.rel_l2(got, ref) <= TOL


def test_w4a8_exact_when_sums_are_representable():
    """Small integer activations (exact in E4M3) against weight codes in {0, +-0.5, +-1}:
    every partial sum is a multiple of 0.5 below 2048, so the output bits are determined."""
    M, N, K = 9, 40, 768
    c = w4amd.capi()
    rng = np.random.default_rng(8)
    pick = np.array([0, 1, 2, 9, 10], np.uint32)
    codes = pick[rng.integers(0, 5, (N, K))]
    wq = orc.PackedWm(N, K, (codes.reshape(N, -1, 8) << (4 * np.arange(8, dtype=np.uint32))).sum(axis=2)
                      .astype(np.uint32).ravel(), np.full(N * (K // 32), 127, np.uint8))
    xv = rng.integers(-3, 4, (M, K)).astype(np.float64)
    xq = orc.quantize_mx8(xv, M, K)
    assert np.array_equal(orc.dequant_mx8(xq), xv)
    ref = xv @ _decode(wq, N).T
    assert np.abs(ref).max() < 2048
    dw, dx = DevPackedMx(wq), _DevXm8(xq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a8(dw.view, dx.view, ptr(out))
    assert np.array_equal(bits(out).view(np.float16).reshape(M, N), ref.astype(np.float16))


def test_w4a8_quantizer_boundaries_and_status():
    """Block maxima on and beside 448 * 2^e, FP16 subnormals, zeros; non-finite input lands
    in the status word."""
    c = w4amd.capi()
    rows = []
    for e in range(-22, 8):
        top = np.float16(448.0 * 2.0 ** e) if e <= 7 else None
        for amax in (top, np.nextafter(top, np.float16(np.inf)), np.nextafter(top, np.float16(0))):
            if not np.isfinite(amax):
                continue
            row = np.zeros(32, np.float16)
            row[0], row[1] = amax, -amax
            row[2:18] = (np.arange(16) / 16.0 * float(amax)).astype(np.float16)
            row[18] = np.float16(6e-8)
            row[19] = np.float16(-0.0)
            rows.append(row)
    x16 = np.array(rows, np.float16)
    M, K = x16.shape
    ref = orc.quantize_mx8(x16.astype(np.float64), M, K)
    q = torch.zeros(M * K, dtype=torch.uint8, device=DEV)
    s = torch.zeros(M, dtype=torch.uint8, device=DEV)
    st = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    xd = to_dev(x16.ravel())
    view = c.act_mx8_view(M, K, 1, ptr(q), ptr(s))
    c.quantize_mx8_f16(view, ptr(xd), ptr(st))
    torch.cuda.synchronize()
    assert int(st.item()) == 0
    assert np.array_equal(s.cpu().numpy(), ref.scales)
    assert np.array_equal(q.cpu().numpy(), ref.q)
    x16[3, 5] = np.float16(np.inf)
    c.quantize_mx8_f16(view, ptr(to_dev(x16.ravel())), ptr(st))
    torch.cuda.synchronize()
    assert int(st.item()) & 1


def test_w4a8_prefill_shape_sampled_rows():
    M, N, K = 2048, 4096, 4096
    c = w4amd.capi()
    wq = orc.quantize_mx(orc.normal_weights(N * K, 23), N, K)
    x16 = orc.normal_activations(M * K, 24)
    xq = orc.quantize_mx8(x16.view(np.float16).astype(np.float64), M, K)
    dw, dx = DevPackedMx(wq), _DevXm8(xq)
    out = halves(M * N, 0x7E00)
    c.gemm_mx_w4a8(dw.view, dx.view, ptr(out))
    got = bits(out).view(np.float16).astype(np.float64).reshape(M, N)
    rows = np.unique(np.concatenate([np.arange(0, 16), np.arange(M - 16, M),
                                     np.random.default_rng(6).integers(0, M, 64)]))
    ref = orc.dequant_mx8(xq)[rows] @ _decode(wq, N).T
    assert orc.rel_l2(got[rows], ref) <= TOL
    assert np.isfinite(got).all()


def test_w4a4_activation_quantizer_ties_and_boundaries():
    """FP16 activations on the midpoints between E2M1 magnitudes (and one FP16 ulp either
    side), block maxima on and beside 6 * 2^e, FP16 subnormals, signed zeros: the device
    quantizer (FP32 arithmetic for FP16 sources) writes the host quantizer's bytes."""
    c = w4amd.capi()
    rows = []
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    for e in range(-24, 13):
        top = np.float16(6.0 * 2.0 ** e)
        if not np.isfinite(top) or top == 0:
            continue
        for amax in (top, np.nextafter(top, np.float16(np.inf)), np.nextafter(top, np.float16(0))):
            if not np.isfinite(amax):
                continue
            unit = 2.0 ** e if amax <= top else 2.0 ** (e + 1)
            m = (mids * unit).astype(np.float16)
            row = np.concatenate([[amax, -amax], m, np.nextafter(m, np.float16(np.inf)),
                                  np.nextafter(m, np.float16(0)), -m, [np.float16(0), np.float16(-0.0)]])
            row = row[np.abs(row.astype(np.float64)) <= float(amax)][:32]
            rows.append(np.concatenate([row, np.zeros(32 - row.size, np.float16)]))
    x16 = np.array(rows, np.float16)
    M, K = x16.shape
    ref = orc.quantize_mx(x16.astype(np.float64), M, K)
    _, q, s = _quantize_x_on_device(x16.ravel(), M, K)
    assert np.array_equal(s.cpu().numpy(), ref.scales)
    assert np.array_equal(q.cpu().numpy().view(np.uint32), ref.q)
