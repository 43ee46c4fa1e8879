"""Every benchmark configuration at its stated size, as parity tests (the reference's GPU suite
does the same for its own bench shapes, tests/test_gpu.cu:783-924, 1258-1294).

Oracle work is bounded by sampling: weights / caches are quantized by the CPU oracle (for the
attention cases four sample slabs that the 64 slabs repeat), hooks are compared with the oracle's
dequantization on the device, byte for byte and in full, and outputs are checked against the FP64
oracle on sampled rows / heads."""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DevKV, DevPacked, DevPackedMx, bits, cross_gate, halves, ptr, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _sampled_gemm_check(fn, view, w_ref, x, M, N, K, rows_m, n_rows=128, seed=7, hook=True):
    """Run `fn` hooked and unhooked; hook bytes on the device, outputs on `rows_m` x sampled n."""
    x_d = to_dev(x)
    w_ref_d = to_dev(w_ref)
    c_h, c_u = halves(M * N, 0x7E00), halves(M * N, 0x7E00)
    if hook:
        w_d = halves(N * K, 0x7E00)
        fn(view, ptr(x_d), ptr(c_h), M, 0, ptr(w_d))
        assert torch.equal(w_d, w_ref_d), "w_out bitwise"
        del w_d
    fn(view, ptr(x_d), ptr(c_u), M, 0, 0)
    ns = np.sort(np.random.default_rng(seed).choice(N, size=min(N, n_rows), replace=False))
    w_rows = np.ascontiguousarray(w_ref.reshape(N, K)[ns])
    xs = np.ascontiguousarray(x.reshape(M, K)[rows_m])
    ref = orc.gemm_oracle(xs, len(rows_m), K, w_rows, len(ns))
    got_u = bits(c_u).reshape(M, N)[rows_m][:, ns]
    if hook:
        got_h = bits(c_h).reshape(M, N)[rows_m][:, ns]
        assert orc.rel_l2(np.ascontiguousarray(got_h).view(np.float16), ref) <= TOL
        cross_gate(np.ascontiguousarray(got_h), np.ascontiguousarray(got_u), ref, fn.__name__)
    else:
        assert orc.rel_l2(np.ascontiguousarray(got_u).view(np.float16), ref) <= TOL


def test_c4_prefill_m2048_n4096_k4096():
    """W4A16 symmetric gs = 128, M = 2048: hook memcmp on the device, 16 sampled activation rows
    x 128 sampled weight rows against gemm_oracle, fused and two-pass outputs within 2e-3."""
    c = w4amd.capi()
    M, N, K, gs = 2048, 4096, 4096, 128
    p = orc.quantize(orc.normal_weights(N * K, 0xC4) * 0.02, N, K, gs, True)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, 0xC4 + 1)
    dp = DevPacked(p)
    rows_m = np.sort(np.random.default_rng(4).choice(M, size=16, replace=False))
    for fn in (c.gemm_mma, c.gemm):
        _sampled_gemm_check(fn, dp.view, w_ref, x, M, N, K, rows_m)
    # two-pass baseline on the same data: dequant + plain FP16 GEMM, within 2e-3 of the fused output
    x_d, w16 = to_dev(x), halves(N * K, 0x7E00)
    c.dequant(dp.view, ptr(w16))
    c2, c1 = halves(M * N, 0x7E00), halves(M * N, 0x7E00)
    c.gemm_fp16(ptr(w16), ptr(x_d), ptr(c2), M, N, K)
    c.gemm(dp.view, ptr(x_d), ptr(c1), M, 0, 0)
    a = c1.view(torch.float16).double()
    b = c2.view(torch.float16).double()
    assert float(((a - b).norm() / b.norm()).item()) <= 2e-3


@pytest.mark.parametrize("gs,K", [(128, 4096), (32, 4096), (48, 4096), (8, 4104)])
def test_c2_asym_one_sided_groups_n11008(gs, K):
    """C2 at its width: 10 % one-sided groups, zero-points, M over the crossover sweep."""
    c = w4amd.capi()
    N = 11008
    w = orc.one_sided_group_weights(N, K, gs, 0xC2 + gs)
    p = orc.quantize(w, N, K, gs, False)
    w_ref = orc.dequant_all(p)
    dp = DevPacked(p)
    for M in (1, 4, 9, 64):
        x = orc.normal_activations(M * K, 0xC2 + M)
        rows_m = np.arange(M) if M <= 9 else np.array([0, 17, 40, 63])
        _sampled_gemm_check(c.gemm, dp.view, w_ref, x, M, N, K, rows_m, n_rows=96, hook=(M in (1, 64)))


def test_c3_mxfp4_outliers_n14336():
    """C3 at its width: 1 % outliers at 20 sigma, M = 1 / 16 / 128."""
    c = w4amd.capi()
    N, K = 14336, 4096
    w = orc.outlier_weights(N, K, 0xC3)
    p = orc.quantize_mx(w, N, K)
    w_ref = orc.dequant_all_mx(p)
    dp = DevPackedMx(p)
    for M in (1, 16, 128):
        x = orc.normal_activations(M * K, 0xC3 + M)
        rows_m = np.arange(M) if M <= 16 else np.array([0, 31, 64, 127])
        _sampled_gemm_check(c.gemm_mx, dp.view, w_ref, x, M, N, K, rows_m, n_rows=96, hook=(M != 16))


@pytest.mark.parametrize("K,sym,Ms", [(8192, True, (13, 24, 64)), (8192, False, (32, 64)), (11008, False, (24,)),
                                      (13824, True, (32,))])
def test_long_k_two_tiles_per_workgroup(K, sym, Ms):
    """Long K on a grid of more 16-row tiles than compute units (N = 4128: 258) with more than 16
    activation rows: two tiles share a workgroup's activations.  Hook bytes on the device, sampled
    outputs against the oracle, hooked against unhooked within the cross gate."""
    c = w4amd.capi()
    N, gs = 4128, 128
    p = orc.quantize(orc.normal_weights(N * K, 0x10C + K) * 0.02 + (0.0 if sym else 0.01), N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    dp = DevPacked(p)
    for M in Ms:
        x = orc.normal_activations(M * K, 0x10C + M)
        rows_m = np.array([0, M // 3, M - 1])
        for fn in (c.gemm_mma, c.gemm):
            _sampled_gemm_check(fn, dp.view, w_ref, x, M, N, K, rows_m, n_rows=96)


def test_long_k_two_tiles_per_workgroup_mxfp4():
    c = w4amd.capi()
    N, K = 4128, 8192
    p = orc.quantize_mx(orc.outlier_weights(N, K, 0x10D), N, K)
    w_ref = orc.dequant_all_mx(p)
    dp = DevPackedMx(p)
    for M in (24, 64):
        x = orc.normal_activations(M * K, 0x10D + M)
        _sampled_gemm_check(c.gemm_mx, dp.view, w_ref, x, M, N, K, np.array([0, M // 2, M - 1]), n_rows=96)


# ---- C5: batch 8, 8 kv heads, 4 query heads per kv head, D = 128, S = 32768 -------------------
B5, HKV, GROUP, D5, S5, NS5 = 8, 8, 4, 128, 32768, 4
H5 = B5 * HKV
SAMPLED = (0, 9, 18, 27, 63)  # slabs of five sequences, all four sample slabs


def _slab_index():
    return torch.arange(H5, device="cuda") % NS5


def _rep(a):
    return to_dev(np.ascontiguousarray(a).reshape(NS5, -1))[_slab_index()].contiguous()


def _check_heads(out, q, kd, vd):
    got = bits(out).view(np.float16).reshape(H5, GROUP, D5)
    for i in SAMPLED:
        ref = orc.attention_f16(q.reshape(H5, GROUP * D5)[i], kd[i % NS5:i % NS5 + 1], vd[i % NS5:i % NS5 + 1],
                                1, GROUP, S5, D5)
        assert orc.rel_l2(got[i], ref) <= TOL, i


def test_c5_fp16_cache_full_size():
    c = w4amd.capi()
    kd = orc.normal_activations(NS5 * S5 * D5, 0xF16).reshape(NS5, -1)
    vd = orc.normal_activations(NS5 * S5 * D5, 0xF17).reshape(NS5, -1)
    q = orc.normal_activations(H5 * GROUP * D5, 0xF18)
    k_d, v_d = _rep(kd), _rep(vd)
    out = halves(H5 * GROUP * D5, 0x7E00)
    c.attention_fp16_flash(ptr(to_dev(q)), ptr(k_d), ptr(v_d), ptr(out), H5, S5, D5, group=GROUP)
    _check_heads(out, q, kd, vd)


@pytest.mark.parametrize("scale_mode", [0, 1], ids=["row_scales", "slab_scale"])
def test_c5_fp8_cache_full_size(scale_mode):
    """FP8 E4M3 cache, one FP16 scale per (row, group of 128) and one per slab ("per head")."""
    c = w4amd.capi()
    c8 = orc.quantize_cache_f8(orc.normal_weights(NS5 * S5 * D5, 0xF8), orc.normal_weights(NS5 * S5 * D5, 0xF9),
                               NS5, S5, D5, 128)
    q = orc.normal_activations(H5 * GROUP * D5, 0xFA)
    if scale_mode == 1:
        slab_scales = np.array([0x2000 + 37 * i for i in range(NS5)], np.uint16)  # ~ 0.0078 .. 0.0085
        c8.s_k = np.repeat(slab_scales, S5)                 # the oracle sees the slab's scale in every row
        c8.s_v = np.repeat(slab_scales[::-1].copy(), S5)
        s_k, s_v = to_dev(slab_scales)[_slab_index()].contiguous(), to_dev(slab_scales[::-1].copy())[_slab_index()].contiguous()
    else:
        s_k, s_v = _rep(c8.s_k), _rep(c8.s_v)
    kd, vd = orc.dequant_cache_f8(c8, False), orc.dequant_cache_f8(c8, True)
    q_k, q_v = _rep(c8.q_k), _rep(c8.q_v)
    view = c.kv_f8_view(H5, S5, D5, 128, 1, ptr(q_k), ptr(s_k), ptr(q_v), ptr(s_v))
    out, out2 = halves(H5 * GROUP * D5, 0x7E00), halves(H5 * GROUP * D5, 0x7E00)
    ko, vo = halves(H5 * S5 * D5, 0x7E00), halves(H5 * S5 * D5, 0x7E00)
    c.attention_f8_flash(view, ptr(to_dev(q)), ptr(out), 0, ptr(ko), ptr(vo), group=GROUP, scale_mode=scale_mode)
    idx = _slab_index()
    assert torch.equal(ko.view(H5, -1), to_dev(kd).view(NS5, -1)[idx]), "k_out bitwise"
    assert torch.equal(vo.view(H5, -1), to_dev(vd).view(NS5, -1)[idx]), "v_out bitwise"
    del ko, vo
    c.attention_f8_flash(view, ptr(to_dev(q)), ptr(out2), group=GROUP, scale_mode=scale_mode)
    assert torch.equal(out, out2), "hooked and unhooked bytes differ"
    _check_heads(out2, q, kd.reshape(NS5, -1), vd.reshape(NS5, -1))


def test_c5_paged_w4_page16_shared_prefix_full_size():
    """Paged W4, page 16: sequences 0-3 share their first 8192 tokens (512 pages), every sequence
    has a block table of its own over one pool per kv head.  Output bytes equal the contiguous
    kernel's on the same caches; sampled heads against the FP64 oracle."""
    c = w4amd.capi()
    gs, page, prefix = 32, 16, 8192
    c4 = orc.quantize_cache(orc.normal_weights(NS5 * S5 * D5, 0x9A6E), orc.normal_weights(NS5 * S5 * D5, 0x9A6F),
                            NS5, S5, D5, gs, True)
    kd, vd = orc.dequant_cache(c4, False), orc.dequant_cache(c4, True)
    q = orc.normal_activations(H5 * GROUP * D5, 0x9A70)
    G, wd = c4.G, orc.words(D5)
    lp, pp = S5 // page, prefix // page
    npages = pp + 4 * (lp - pp) + 4 * lp
    rows = npages * page
    gen = torch.Generator(device="cuda").manual_seed(16)
    perm = torch.randperm(npages, device="cuda", generator=gen).to(torch.int32)
    tables = torch.empty((B5, lp), dtype=torch.int32, device="cuda")
    nxt = pp
    for s in range(B5):
        if s < 4:
            tables[s, :pp] = perm[:pp]
            tables[s, pp:] = perm[nxt:nxt + lp - pp]
            nxt += lp - pp
        else:
            tables[s] = perm[nxt:nxt + lp]
            nxt += lp
    assert nxt == npages
    t_idx = torch.arange(S5, device="cuda")
    pool = {}
    for name, width, src in (("q_k", wd, c4.q_k), ("s_k", G, c4.s_k), ("q_v", wd, c4.q_v), ("s_v", G, c4.s_v)):
        src_d = to_dev(src).view(NS5, S5, width)
        pl = torch.zeros((HKV, rows, width), dtype=src_d.dtype, device="cuda")
        for s in range(B5):
            phys = tables[s].long()[t_idx // page] * page + t_idx % page
            for h in range(HKV):
                pl[h, phys] = src_d[h % NS5]  # the cache of (sequence, kv head h) is sample slab h % 4
        pool[name] = pl
    view = c.kv_view(HKV, S5, D5, gs, G, True, ptr(pool["q_k"]), ptr(pool["s_k"]), 0, ptr(pool["q_v"]),
                     ptr(pool["s_v"]), 0)
    q_d = to_dev(q)
    out_p = halves(H5 * GROUP * D5, 0x7E00)
    c.attention_w4_flash_paged_batched(view, ptr(tables), B5, lp, page, npages, GROUP, ptr(q_d), ptr(out_p))
    # contiguous caches of the same 64 (sequence, kv head) slabs: slab (s, h) holds sample h % 4
    idx = (torch.arange(H5, device="cuda") % HKV) % NS5

    def rep(a):
        return to_dev(np.ascontiguousarray(a).reshape(NS5, -1))[idx].contiguous()
    t = [rep(c4.q_k), rep(c4.s_k), rep(c4.q_v), rep(c4.s_v)]
    cview = c.kv_view(H5, S5, D5, gs, G, True, ptr(t[0]), ptr(t[1]), 0, ptr(t[2]), ptr(t[3]), 0)
    out_c = halves(H5 * GROUP * D5, 0x7E00)
    c.attention_w4_flash(cview, ptr(q_d), ptr(out_c), group=GROUP)
    assert torch.equal(out_p, out_c), "paged batch == contiguous, bytewise"
    got = bits(out_p).view(np.float16).reshape(H5, GROUP, D5)
    for i in SAMPLED:
        sl = (i % HKV) % NS5
        ref = orc.attention_f16(q.reshape(H5, GROUP * D5)[i], kd[sl:sl + 1], vd[sl:sl + 1], 1, GROUP, S5, D5)
        assert orc.rel_l2(got[i], ref) <= TOL, i
