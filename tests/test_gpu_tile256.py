"""The 256 x 256-tile prefill kernel (unhooked calls whose grid of 128 x 256 tiles would take
two rounds or more; mma.cuh:234-260 is the reference's dispatch for these shapes).

It adds the products of a result in the same k order as the 128 x 256 kernel, which serves the
hooked call of the same shape, so the two outputs are compared byte for byte; the hooked call's
dequantized weights are compared with the oracle's on the device, and sampled rows of the
output with the FP64 oracle (<= 1e-3, the reference's gate, tests/test_gpu.cu:184-193)."""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DevPacked, DevPackedMx, bits, halves, ptr, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _check(fn, view, w_ref, x, M, N, K, seed):
    x_d, w_ref_d = to_dev(x), to_dev(w_ref)
    c_h, c_u, w_d = halves(M * N, 0x7E00), halves(M * N, 0x7E00), halves(N * K, 0x7E00)
    fn(view, ptr(x_d), ptr(c_h), M, 0, ptr(w_d))
    fn(view, ptr(x_d), ptr(c_u), M, 0, 0)
    assert torch.equal(w_d, w_ref_d), "w_out bitwise"
    assert torch.equal(c_h, c_u), "256 x 256 tiles add in the order of the hooked kernel"
    rng = np.random.default_rng(seed)
    # the corners of the grid and a sample of its inside
    ms = np.unique(np.concatenate([[0, 255, 256, M - 1], rng.choice(M, size=12, replace=False)]))
    ns = np.unique(np.concatenate([[0, 63, 64, 255, 256, N - 1], rng.choice(N, size=min(N, 90), replace=False)]))
    ref = orc.gemm_oracle(np.ascontiguousarray(x.reshape(M, K)[ms]), len(ms), K,
                          np.ascontiguousarray(w_ref.reshape(N, K)[ns]), len(ns))
    got = np.ascontiguousarray(bits(c_u).reshape(M, N)[ms][:, ns]).view(np.float16)
    assert orc.rel_l2(got, ref) <= TOL


# N x M chosen so that 256 x 256 tiles cover in one round what 128 x 256 tiles cover in two
SHAPES = [
    (4096, 4096, 256),   # whole tiles
    (3900, 4072, 256),   # ragged rows of X, a ragged last tile of W rows
    (3850, 4090, 128),   # N not a multiple of 8: element stores; two stages only
    (4096, 4096, 384),   # six stages
    (12200, 1280, 128),  # five tiles along N: the plain order of tiles over the XCDs
]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("gs,sym", [(128, True), (64, False), (32, True), (32, False), (0, False)])
def test_w4_tile256(M, N, K, gs, sym):
    if gs == 0:
        gs = K  # one group per row
    if K % gs:
        pytest.skip("group size does not divide K")
    if K % 128:
        pytest.skip("the tile kernels take K in multiples of 128")
    c = w4amd.capi()
    seed = M + N + K + gs + sym
    w = orc.normal_weights(N * K, seed) * 0.02
    if not sym:
        w = w + 0.01  # off-centre groups: zero-points away from 8
    p = orc.quantize(w, N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, seed + 1)
    dp = DevPacked(p)
    for fn in (c.gemm_mma, c.gemm):
        _check(fn, dp.view, w_ref, x, M, N, K, seed)


@pytest.mark.parametrize("M,N,K", SHAPES[:3])
def test_mxfp4_tile256(M, N, K):
    c = w4amd.capi()
    seed = M + N + K
    p = orc.quantize_mx(orc.outlier_weights(N, K, seed), N, K)
    w_ref = orc.dequant_all_mx(p)
    x = orc.normal_activations(M * K, seed + 1)
    dp = DevPackedMx(p)
    for fn in (c.gemm_mma_mx, c.gemm_mx):
        _check(fn, dp.view, w_ref, x, M, N, K, seed)


def test_c4_prefill_m4096():
    """C4's matrix at M = 4096 (two rounds of the smaller tiles): hooked == unhooked bytes,
    sampled rows against the oracle."""
    c = w4amd.capi()
    M, N, K, gs = 4096, 4096, 4096, 128
    p = orc.quantize(orc.normal_weights(N * K, 0xC4) * 0.02, N, K, gs, True)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, 0xC4 + 2)
    _check(c.gemm, DevPacked(p).view, w_ref, x, M, N, K, 4)
