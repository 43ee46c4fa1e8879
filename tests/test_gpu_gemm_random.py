"""Randomly drawn GEMM shapes through every entry point: long and ragged K, group sizes with and
without a multiple of 32, widths that are no multiple of 16, 1 to 64 activation rows, W4 with and
without zero-points and MXFP4.  Per case: the fused hook is the host dequantization byte for
byte, hooked and unhooked outputs agree within the cross gate, every kernel is within 1e-3 (rel L2)
of the FP64 oracle, and the dispatcher returns one of its callees' bytes, with and without the
hook.  The draw is fixed (seeded)."""
import numpy as np
import pytest

import orc
import w4amd
from devutil import DevPacked, DevPackedMx, bits, cross_gate, halves, ptr, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _draw(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        mx = rng.integers(0, 3) == 0
        K = 128 * int(rng.integers(9, 129)) if rng.integers(0, 4) else 8 * int(rng.integers(130, 640))
        gs = int(rng.choice([32, 64, 128, 96, 256, 8, 16, 24, 48]))
        if mx:
            K = (K // 32) * 32
        N = 16 * int(rng.integers(1, 7)) if rng.integers(0, 5) else int(rng.integers(1, 100))
        out.append((bool(mx), int(rng.integers(1, 65)), N, K, gs, bool(rng.integers(0, 2)),
                    int(rng.integers(1, 1 << 30))))
    return out


CASES = _draw(48, 0x5EED)


def _run(fn, view, x_d, M, N, K, hook):
    c_d = halves(M * N, 0x7E00)
    w_d = halves(N * K, 0x7E00) if hook else None
    fn(view, ptr(x_d), ptr(c_d), M, 0, ptr(w_d))
    return bits(c_d).copy(), (bits(w_d).copy() if hook else None)


@pytest.mark.parametrize("i", range(len(CASES)))
def test_random_shape(i):
    c = w4amd.capi()
    mx, M, N, K, gs, sym, seed = CASES[i]
    w = orc.normal_weights(N * K, seed)
    x = orc.normal_activations(M * K, seed + 1)
    if mx:
        p = orc.quantize_mx(w, N, K)
        w_ref, dp = orc.dequant_all_mx(p), DevPackedMx(p)
        fns = (c.gemm_fused_mx, c.gemm_mma_mx, c.gemm_mx)
    else:
        p = orc.quantize(w, N, K, gs, sym)
        w_ref, dp = orc.dequant_all(p), DevPacked(p)
        fns = (c.gemm_fused, c.gemm_mma, c.gemm)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    x_d = to_dev(x)
    outs, plains = [], []
    for fn in fns:
        hooked, w_out = _run(fn, dp.view, x_d, M, N, K, True)
        plain, _ = _run(fn, dp.view, x_d, M, N, K, False)
        assert np.array_equal(w_out, w_ref), (fn.__name__, "hook bitwise")
        cross_gate(hooked, plain, ref, fn.__name__)
        assert orc.rel_l2(hooked.view(np.float16), ref) <= TOL, fn.__name__
        outs.append(hooked)
        plains.append(plain)
    assert np.array_equal(outs[2], outs[0]) or np.array_equal(outs[2], outs[1]), "dispatcher == a callee"
    assert np.array_equal(plains[2], plains[0]) or np.array_equal(plains[2], plains[1]), "dispatcher == a callee, no hook"
