"""GPU parity gates for the packed-weight GEMM path, through the C ABI.

Mirrors the reference device suite (tests/test_gpu.cu:54-498): for every config
and sign mode the materialising dequant and the w_out hooks of both fused
kernels must equal the oracle's dequant_all bit for bit, the GEMM outputs must
be within rel L2 1e-3 of the FP64 oracle, the two kernels within 2e-3 of each
other, and the dispatcher must reproduce its callee's bytes.
"""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DevPacked, DevPackedMx, bits, cross_gate, f64, halves, ptr, to_dev

pytestmark = pytest.mark.gpu

CFGS = [(1, 64, 64, 8), (8, 128, 96, 16), (16, 256, 100, 32), (4, 96, 72, 48),
        (2, 32, 128, 64), (3, 40, 256, 128), (5, 72, 40, 8), (17, 64, 128, 16),
        (33, 48, 104, 24), (20, 32, 100, 8), (65, 96, 100, 16),
        # shapes that take the aligned dwordx4 paths
        (1, 512, 4096, 128), (7, 96, 2048, 32), (9, 80, 1024, 64), (64, 64, 512, 128),
        # shapes of the unrolled decode kernel (K = 2048, 4096, 8192; whole workgroups of rows)
        # shapes of the large-M matrix-core kernel (ragged M and N tiles, gs % 32 != 0)
        (300, 200, 512, 128), (96, 136, 256, 48), (257, 128, 192, 64),
        # odd and even numbers of k-steps, ragged M and N tiles
        (130, 260, 384, 32), (128, 256, 256, 64), (200, 300, 1024, 128), (97, 72, 128, 96),
        (2, 64, 2048, 64), (1, 128, 8192, 128), (4, 72, 4096, 32), (3, 40, 6144, 128), (8, 16, 2048, 128),
        # group sizes that are no multiple of 32 (a lane's 32-k slice spans several groups) on the
        # unrolled and streaming kernels
        (1, 64, 2048, 8), (2, 16, 4096, 48), (3, 24, 2048, 24), (12, 48, 2048, 40), (20, 64, 2048, 48),
        (40, 32, 1024, 8),
        # K % 8 == 0 but K % 32 != 0: whole words, rows of packed words not 16-byte aligned
        (9, 64, 4104, 8), (40, 48, 1032, 24), (3, 32, 520, 8), (100, 40, 264, 16),
        # one activation row, long or odd K: the vector kernel that splits K over the waves
        (1, 64, 11008, 128), (1, 32, 2080, 32), (1, 16, 14336, 64), (1, 24, 5120, 48), (1, 8, 16384, 8),
        (2, 16, 11008, 128), (4, 8, 5120, 32), (3, 24, 14336, 64), (4, 16, 8192, 128),
        # the large-M kernel with direct-to-LDS loads (gs % 128 == 0, at least 64 tiles of 128 x 256):
        # ragged tiles, 4 / 3 / 10 / 2 stages, groups of two stages; then an odd number of scales,
        # which it leaves to the register-staged kernel
        (1030, 2050, 512, 128), (2048, 1024, 384, 128), (1024, 2048, 1280, 256), (1000, 2304, 256, 128),
        (1025, 2049, 384, 128),
        # the same kernel with two and four groups per 128-k stage
        (1030, 2050, 512, 64), (1024, 2048, 384, 32), (2048, 1030, 256, 32), (900, 2304, 640, 64),
        # a thin grid of its tiles (2 x 8, 1 x 9)
        (130, 2000, 256, 128), (100, 2100, 384, 32),
        # M <= 16 with more 16-row tiles than compute units: two, three and four tiles per
        # workgroup share one copy of the activations (the last workgroups have fewer)
        (16, 4128, 2048, 128), (7, 8208, 4096, 64), (9, 12304, 2048, 32), (12, 4144, 4096, 96),
        (1, 8192, 2048, 128),
        # the same with two and four 16-row tiles of activations (17 <= M <= 64), which pass
        # through the wave's LDS region in phases
        (17, 4128, 4096, 128), (32, 8208, 2048, 64), (33, 4144, 4096, 32), (64, 12304, 2048, 128),
        (50, 4128, 2048, 96),
        # more than four tiles per compute unit: four per workgroup, more workgroups than units
        (8, 16416, 2048, 128),
        # 65 <= M <= 256: two or three passes of that kernel over the weights (grid.y) while that is
        # the cheaper way (four passes at N = 2048 are not: the tile kernel takes that one)
        (65, 4128, 2048, 128), (128, 2048, 4096, 64), (100, 96, 2048, 32), (250, 2048, 4096, 128),
        (130, 512, 4096, 128),
        # long K (8, 11 and 14 chunks of 128 per wave; the last waves own fewer when K / 128 is no
        # multiple of 8: 86 chunks at K = 11008, 57 at K = 7296, 81 at K = 10368)
        (16, 256, 11008, 128), (64, 512, 14336, 64), (5, 128, 8192, 32), (33, 96, 7296, 128),
        (100, 64, 10368, 96),
        # four rows per wave with a group lookup per packed word (group sizes that are no power of
        # two, or below 32)
        (1, 64, 4096, 48), (4, 32, 2048, 8), (2, 48, 4096, 96), (3, 16, 2048, 24),
        # the small tiles of the large-M kernel with two sets of waves on an odd number of stages
        # (9 and 15: the second set's last stage does not exist)
        (130, 256, 1152, 128), (200, 384, 1920, 64),
        # an even number of chunks per wave that is not all there: the last waves' whole-line
        # pairs are clamped to the row's last pair (58 and 106 chunks for 8 x 8 and 8 x 14 slots)
        (16, 64, 7424, 128), (40, 48, 13568, 64),
        # ... with the requests pipelined chunk by chunk (M <= 32): odd and even chunk counts, ragged last waves
        (17, 64, 10368, 96), (32, 32, 14336, 32), (9, 48, 7296, 64), (12, 32, 11264, 128), (3, 16, 13440, 64),
        (3, 32, 5120, 128), (8, 16, 6144, 64), (12, 16, 7168, 32), (16, 32, 9216, 128), (24, 16, 10240, 64),
        (5, 16, 12288, 128), (13, 16, 15360, 32), (4, 32, 16384, 128), (3, 16, 4224, 32), (20, 16, 4352, 64),
        # ... four row tiles (M <= 64): units of one row tile in the ring
        (33, 32, 11008, 128), (64, 16, 14336, 32), (50, 32, 8192, 64), (47, 16, 5120, 128), (64, 16, 16384, 128),
        # more workgroups of four tiles than compute units: two chunks of activations per phase
        (6, 16448, 4096, 64),
        # ... and K <= 4096 on grids of at most one tile per compute unit
        (6, 2064, 4096, 128), (8, 4096, 2048, 32), (7, 32, 3072, 64), (20, 48, 2560, 32), (32, 16, 1536, 128),
        (3, 16, 1152, 32),
        # four rows per wave (N % 16 == 0, K = 2048 / 4096 / 8192, gs 32 ... 256): one to four
        # activation rows, one to eight scale loads per lane
        (3, 32, 4096, 32), (4, 48, 2048, 64), (2, 32, 8192, 32), (1, 16, 4096, 256), (4, 16, 4096, 128),
        (1, 4096, 4096, 128), (2, 11008, 4096, 128), (1, 64, 2048, 32),
        # M <= 64 with group parameters through LDS: odd group sizes, ragged K, one and two
        # tiles per workgroup, one / two / four activation row tiles, 2 .. 5 chunks per wave
        (9, 4128, 4096, 48), (50, 4128, 4104, 8), (16, 8208, 2048, 24), (64, 4112, 3072, 48),
        (30, 64, 5000, 40), (8, 32, 1160, 8), (33, 48, 2568, 16)]
TOL, CROSS = 1e-3, 2e-3  # rel L2 vs the FP64 oracle; between two gated paths
# five to eight tiles per workgroup in one round (fused gate / up projections, a 32000-row
# head), one and two activation row tiles: (M, N, K, gs, symmetric)
WIDE = [(9, 22016, 4096, 128, True), (16, 28672, 4096, 32, False), (7, 32000, 4096, 64, True),
        (24, 20480, 4096, 128, False), (32, 28672, 4096, 64, True)]


def _run(fn, view, x_d, M, N, K, hook=True):
    c_d = halves(M * N, 0x7E00)
    w_d = halves(N * K, 0x7E00) if hook else None
    fn(view, ptr(x_d), ptr(c_d), M, 0, ptr(w_d))
    return bits(c_d), (bits(w_d) if hook else None)


@pytest.mark.parametrize("i", range(len(WIDE)))
def test_w4_wide_grids(i):
    """The matrix-core entry on grids of more than four tiles per compute unit: oracle gate,
    hook bytes, hooked against unhooked output (cross gate)."""
    c = w4amd.capi()
    M, N, K, gs, sym = WIDE[i]
    seed = 0x51DE ^ (i * 977)
    p = orc.quantize(orc.normal_weights(N * K, seed), N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, seed + 1)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    dp, x_d = DevPacked(p), to_dev(x)
    cm, wm = _run(c.gemm_mma, dp.view, x_d, M, N, K)
    assert np.array_equal(wm, w_ref), "mma w_out bitwise"
    assert orc.rel_l2(cm.view(np.float16), ref) <= TOL
    cm2, _ = _run(c.gemm_mma, dp.view, x_d, M, N, K, hook=False)
    cross_gate(cm, cm2, ref, "gemm_mma")


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(CFGS)))
def test_w4_gemm_gates(i, sym):
    c = w4amd.capi()
    M, N, K, gs = CFGS[i]
    seed = 0x44A1 ^ (i * 977 + (0 if sym else 1))
    p = orc.quantize(orc.normal_weights(N * K, seed), N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, seed + 1)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    dp, x_d = DevPacked(p), to_dev(x)

    w_d = halves(N * K, 0x7E00)
    c.dequant(dp.view, ptr(w_d))
    assert np.array_equal(bits(w_d), w_ref), "dequant bitwise"

    cf, wf = _run(c.gemm_fused, dp.view, x_d, M, N, K)
    assert np.array_equal(wf, w_ref), "fused w_out bitwise"
    assert orc.rel_l2(cf.view(np.float16), ref) <= TOL
    cm, wm = _run(c.gemm_mma, dp.view, x_d, M, N, K)
    assert np.array_equal(wm, w_ref), "mma w_out bitwise"
    assert orc.rel_l2(cm.view(np.float16), ref) <= TOL
    den = np.sqrt(np.sum(ref ** 2))
    cross = np.sqrt(np.sum((cf.view(np.float16).astype(np.float64) -
                            cm.view(np.float16).astype(np.float64)) ** 2)) / den
    assert cross <= CROSS
    # without the hook: GEMM results under the same gates (only the hook is bit-exact by contract)
    cf2, _ = _run(c.gemm_fused, dp.view, x_d, M, N, K, hook=False)
    cm2, _ = _run(c.gemm_mma, dp.view, x_d, M, N, K, hook=False)
    cross_gate(cf, cf2, ref, "gemm_fused")
    cross_gate(cm, cm2, ref, "gemm_mma")
    # dispatcher: same bytes as the callee it selects at the same hook flag, hook intact
    cd, wd = _run(c.gemm, dp.view, x_d, M, N, K)
    use_mma = M >= c.load().w4_dispatch_mma_min_m_for_gs(N, K, gs)
    assert np.array_equal(cd, cm if use_mma else cf) and np.array_equal(wd, w_ref)
    cd2, _ = _run(c.gemm, dp.view, x_d, M, N, K, hook=False)
    assert np.array_equal(cd2, cm2 if use_mma else cf2)
    # two-pass baseline: dequant + plain FP16 GEMM
    c2 = halves(M * N, 0x7E00)
    c.gemm_fp16(ptr(w_d), ptr(x_d), ptr(c2), M, N, K)
    assert orc.rel_l2(f64(c2), ref) <= TOL


@pytest.mark.parametrize("i", range(len(CFGS)))
def test_mx_gemm_gates(i):
    c = w4amd.capi()
    M, N, K, _ = CFGS[i]
    seed = 0x1E4A ^ (i * 977)
    p = orc.quantize_mx(orc.normal_weights(N * K, seed), N, K)
    w_ref = orc.dequant_all_mx(p)
    x = orc.normal_activations(M * K, seed + 1)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    dp, x_d = DevPackedMx(p), to_dev(x)

    w_d = halves(N * K, 0x7E00)
    c.dequant_mx(dp.view, ptr(w_d))
    assert np.array_equal(bits(w_d), w_ref), "mx dequant bitwise"
    cf, wf = _run(c.gemm_fused_mx, dp.view, x_d, M, N, K)
    assert np.array_equal(wf, w_ref), "mx fused w_out bitwise"
    assert orc.rel_l2(cf.view(np.float16), ref) <= TOL
    cm, wm = _run(c.gemm_mma_mx, dp.view, x_d, M, N, K)
    assert np.array_equal(wm, w_ref), "mx mma w_out bitwise"
    assert orc.rel_l2(cm.view(np.float16), ref) <= TOL
    cd, wd = _run(c.gemm_mx, dp.view, x_d, M, N, K)
    want = cf if M < c.load().w4_dispatch_mma_min_m_for_mx(N, K) else cm
    assert np.array_equal(cd, want) and np.array_equal(wd, w_ref)


# The benchmark configs' own data and shapes at a reduced N: asymmetric weights with one
# (row, group) in ten one-sided, K = 4096 with gs 32 / 48 / 128 and K = 4104 with gs 8,
# M swept over the crossover; MXFP4 with one element in a hundred at 20 sigma, K = 4096
# and the ragged K = 72 / 100, M = 1 / 16 / 128.
C2_SHAPES = [(4096, 32), (4096, 48), (4096, 128), (4104, 8)]


@pytest.mark.parametrize("M", [1, 2, 4, 8, 9, 16, 64])
@pytest.mark.parametrize("ks", range(len(C2_SHAPES)))
def test_w4_asym_one_sided_groups_crossover_sweep(ks, M):
    c = w4amd.capi()
    K, gs = C2_SHAPES[ks]
    N = 352  # 11008 / 32 rounded to whole 16-row tiles
    seed = 0xC2C2 + ks
    w = orc.one_sided_group_weights(N, K, gs, seed)
    p = orc.quantize(w, N, K, gs, False)
    assert p.zeros is not None and (orc_nibbles(p.zeros, N, p.G) == 0).any(), "no one-sided group"
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, seed + 100 + M)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    dp, x_d = DevPacked(p), to_dev(x)
    for fn in (c.gemm_fused, c.gemm_mma, c.gemm):
        cf, wf = _run(fn, dp.view, x_d, M, N, K)
        assert np.array_equal(wf, w_ref), "w_out bitwise"
        assert orc.rel_l2(cf.view(np.float16), ref) <= TOL
        cf2, _ = _run(fn, dp.view, x_d, M, N, K, hook=False)
        cross_gate(cf, cf2, ref, fn.__name__)


def orc_nibbles(words_, rows, n):
    w = words_.reshape(rows, -1)
    sh = (4 * np.arange(8, dtype=np.uint32))[None, None, :]
    return ((w[:, :, None] >> sh) & 0xF).reshape(rows, -1)[:, :n]


@pytest.mark.parametrize("M", [1, 16, 128])
@pytest.mark.parametrize("K", [4096, 72, 100])
def test_mx_outlier_weights(K, M):
    c = w4amd.capi()
    N = 448  # 14336 / 32
    seed = 0xE40F + K
    w = orc.outlier_weights(N, K, seed)
    p = orc.quantize_mx(w, N, K)
    w_ref = orc.dequant_all_mx(p)
    # the no-saturation scale rule holds with the outliers in: no element clips at 6 * 2^e
    err = np.abs(w_ref.view(np.float16).astype(np.float64) - w)
    assert err.max() <= 0.5 * 20 * 0.02, "an outlier was clipped"
    x = orc.normal_activations(M * K, seed + M)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    dp, x_d = DevPackedMx(p), to_dev(x)
    w_d = halves(N * K, 0x7E00)
    c.dequant_mx(dp.view, ptr(w_d))
    assert np.array_equal(bits(w_d), w_ref), "mx dequant bitwise"
    for fn in ((c.gemm_fused_mx, c.gemm_mma_mx, c.gemm_mx) if M <= 16 else (c.gemm_mma_mx, c.gemm_mx)):
        cf, wf = _run(fn, dp.view, x_d, M, N, K)
        assert np.array_equal(wf, w_ref), "w_out bitwise"
        assert orc.rel_l2(cf.view(np.float16), ref) <= TOL
        cf2, _ = _run(fn, dp.view, x_d, M, N, K, hook=False)
        assert np.array_equal(cf, cf2)
    # format error against W4 gs = 128 on the same matrix (needs K a multiple of 8 only)
    if K == 4096:
        w4 = orc.dequant_all(orc.quantize(w, N, K, 128, True))
        e_mx = np.sqrt(np.sum((w_ref.view(np.float16).astype(np.float64) - w) ** 2) / np.sum(w * w))
        e_w4 = np.sqrt(np.sum((w4.view(np.float16).astype(np.float64) - w) ** 2) / np.sum(w * w))
        assert e_mx < e_w4, "per-32 block scales should beat per-128 group scales on outliers"


def test_w4_dequant_exhaustive_scales():
    """Every FP16 scale x every code x every zero-point: the device dequant step
    equals RNE_half(float(s) * (q - z)) bit for bit (NaN scales excluded)."""
    c = w4amd.capi()
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    fin = allh[~np.isnan(allh.view(np.float16))]
    N = fin.size
    # row n: scale fin[n]; 16 groups of 16 codes; group g has zero-point g, codes 0..15
    K, gs = 16 * 16, 16
    q = np.zeros((N, K // 8), np.uint32)
    for k in range(K):
        q[:, k // 8] |= np.uint32(k % 16) << np.uint32(4 * (k % 8))
    zeros = np.zeros((N, 2), np.uint32)
    for g in range(16):
        zeros[:, g // 8] |= np.uint32(g) << np.uint32(4 * (g % 8))
    scales = np.repeat(fin[:, None], 16, axis=1)
    p = orc.PackedW(N, K, gs, False, q.ravel(), np.ascontiguousarray(scales).ravel(), zeros.ravel())
    want = orc.dequant_all(p)
    dp = DevPacked(p)
    w_d = halves(N * K, 0x7E00)
    c.dequant(dp.view, ptr(w_d))
    assert np.array_equal(bits(w_d), want)
    x_d = halves(K, 0x3C00)
    c_d, w2 = halves(N), halves(N * K, 0x7E00)
    c.gemm_fused(dp.view, ptr(x_d), ptr(c_d), 1, 0, ptr(w2))
    assert np.array_equal(bits(w2), want)
    c.gemm_mma(dp.view, ptr(x_d), ptr(c_d), 1, 0, ptr(w2.fill_(0x7E00)))
    assert np.array_equal(bits(w2), want)


def test_mx_dequant_exhaustive():
    """All 255 valid scale bytes x 16 codes."""
    c = w4amd.capi()
    N, K = 255, 32
    q = np.zeros((N, 4), np.uint32)
    for k in range(K):
        q[:, k // 8] |= np.uint32(k % 16) << np.uint32(4 * (k % 8))
    p = orc.PackedWm(N, K, q.ravel(), np.arange(255, dtype=np.uint8))
    want = orc.dequant_all_mx(p)
    dp = DevPackedMx(p)
    w_d = halves(N * K, 0x7E00)
    c.dequant_mx(dp.view, ptr(w_d))
    assert np.array_equal(bits(w_d), want)
    x_d, c_d, w2 = halves(K, 0), halves(N), halves(N * K, 0x7E00)
    c.gemm_fused_mx(dp.view, ptr(x_d), ptr(c_d), 1, 0, ptr(w2))
    assert np.array_equal(bits(w2), want)
    c.gemm_mma_mx(dp.view, ptr(x_d), ptr(c_d), 1, 0, ptr(w2.fill_(0x7E00)))
    assert np.array_equal(bits(w2), want)


@pytest.mark.parametrize("shape", [(1024, 4096, 128, True), (1024, 4096, 128, False), (512, 11008, 128, True),
                                   (512, 4096, 48, False), (512, 8192, 32, True)])
def test_unhooked_kernels_with_one_signed_and_offset_activations(shape):
    """The unhooked arithmetic of the vector kernels (M <= 2 here) and of the gs = 128 decode-batch
    kernel (M = 8, 24) subtracts a bias sum that grows with the sum of the activations; activations
    of one sign, with a large mean or a large magnitude are where that cancellation would show.
    Held to the same 5e-4 against the FP64 oracle as everywhere else."""
    c = w4amd.capi()
    N, K, gs, sym = shape
    p = orc.quantize(orc.normal_weights(N * K, 0x0FF5E7) * 0.02, N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    dp = DevPacked(p)
    rng = np.random.default_rng(5)
    for M in (1, 2, 8, 24):
        for name, x64 in (("abs", np.abs(rng.standard_normal(M * K))), ("mean3", 3 + rng.standard_normal(M * K)),
                          ("mean30", 30 + rng.standard_normal(M * K)),
                          ("large", 1000 * np.abs(rng.standard_normal(M * K))), ("ones", np.ones(M * K))):
            x = np.asarray(x64, np.float16).view(np.uint16)
            ref = orc.gemm_oracle(x, M, K, w_ref, N)
            x_d = to_dev(x)
            ch, _ = _run(c.gemm, dp.view, x_d, M, N, K)
            cu, _ = _run(c.gemm, dp.view, x_d, M, N, K, hook=False)
            cross_gate(ch, cu, ref, name)
