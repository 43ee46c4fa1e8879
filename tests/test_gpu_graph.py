"""The entry points that allocate nothing can be captured into a HIP graph: GEMM
calls (vector kernel, resident-activation kernel, large-M tile kernel with two
sets of waves) and the flash-decode entry with the built-in scratch are captured
on first use, replayed several times with eager work and synchronisations in
between, and every replay is compared, byte for byte, with the eager call on the
same inputs.  The inputs change between replays (in place), so a replay that did
not run, or ran on stale operands, would show.
"""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DevKV, DevPacked, bits, halves, ptr, to_dev

pytestmark = pytest.mark.gpu

# (M, N, K, gs, symmetric): decode shape, decode batch, thin grid of small tiles, long K (two row tiles:
# the pipelined kernel asks for its 128 KB of LDS on first use, inside the capture)
GEMMS = [(1, 256, 4096, 128, True), (8, 4128, 2048, 64, False), (100, 256, 2048, 128, True),
         (24, 64, 11008, 128, False)]


@pytest.mark.parametrize("i", range(len(GEMMS)))
def test_gemm_replays_equal_eager_calls(i):
    c = w4amd.capi()
    M, N, K, gs, sym = GEMMS[i]
    seed = 0x6A4F ^ (i * 977)
    p = orc.quantize(orc.normal_weights(N * K, seed), N, K, gs, sym)
    dp = DevPacked(p)
    x_d = to_dev(orc.normal_activations(M * K, seed + 1))
    out_g = halves(M * N, 0x7E00)
    out_e = halves(M * N, 0x7E00)
    g = torch.cuda.CUDAGraph()
    print(f"graph case M={M} N={N} K={K} gs={gs} sym={sym}", flush=True)
    with torch.cuda.graph(g):
        c.gemm(dp.view, ptr(x_d), ptr(out_g), M, torch.cuda.current_stream().cuda_stream, 0)
    for rep in range(3):
        x_new = to_dev(orc.normal_activations(M * K, seed + 10 + rep))
        x_d.copy_(x_new)                       # eager work between the replays
        out_g.fill_(0x7E00)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        c.gemm(dp.view, ptr(x_d), ptr(out_e), M, 0, 0)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out_g), bits(out_e)), f"replay {rep} differs from the eager call"


# matrix-core flash kernel (D = 128) and the vector flash kernel (D = 96, zero-points)
@pytest.mark.parametrize("shape", [(4, 3000, 128, 32, 4, True), (3, 1500, 96, 32, 2, False)],
                         ids=["matrix_core_kernel", "vector_kernel"])
def test_flash_noalloc_replays_equal_eager_calls(shape):
    c = w4amd.capi()
    H, S, D, gs, group, sym = shape
    seed = 0x6A50 + D
    c4 = orc.quantize_cache(orc.normal_weights(H * S * D, seed), orc.normal_weights(H * S * D, seed + 1),
                            H, S, D, gs, sym)
    dk = DevKV(c4)
    q_d = to_dev(orc.normal_activations(H * group * D, seed + 2))
    out_g = halves(H * group * D, 0x7E00)
    out_e = halves(H * group * D, 0x7E00)
    g = torch.cuda.CUDAGraph()
    print("graph case flash noalloc", flush=True)
    with torch.cuda.graph(g):
        c.attention_w4_flash_noalloc(dk.view, ptr(q_d), ptr(out_g),
                                     torch.cuda.current_stream().cuda_stream, 0, 0, group=group)
    for rep in range(3):
        q_d.copy_(to_dev(orc.normal_activations(H * group * D, seed + 10 + rep)))
        out_g.fill_(0x7E00)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        c.attention_w4_flash(dk.view, ptr(q_d), ptr(out_e), group=group)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out_g), bits(out_e)), f"replay {rep} differs from the eager call"
