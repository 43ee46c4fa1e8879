"""GPU gates for base pointers that are not 16-byte aligned, and for arrays that
end exactly where their allocation's payload ends.

The reference takes any pointer a kernel can dereference; this library picks
its wide-load kernels from the alignment of the bases it is given and falls
back to narrower loads otherwise.  A fresh torch allocation is always 256-byte
aligned, so these cases carve every operand out of a larger buffer at a byte
offset of 2, 4 or 8 (4 or 8 for 32-bit words) and apply the same gates as the
aligned suites: hooks equal the oracle's dequant bit for bit, outputs within
rel L2 1e-3 of the FP64 oracle.

The tail cases put the scales and zero-points of a ragged-K matrix (K % 32 != 0,
group size no multiple of 32) directly in front of Inf / NaN bit patterns: a
kernel that reads a group past its row's last one picks those up and turns the
last column into NaN.
"""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DEV, bits, cross_gate, f64, ptr

pytestmark = pytest.mark.gpu
TOL = 1e-3


class Carved:
    """`a`'s bytes at byte offset `off` of a device buffer, poison before and after."""

    def __init__(self, a, off, tail=None):
        a = np.ascontiguousarray(a)
        raw = a.view(np.uint8).ravel()
        pad = 64
        host = np.full(off + raw.size + pad, 0x7E, np.uint8)
        host[off:off + raw.size] = raw
        if tail is not None:
            t = np.resize(np.asarray(tail).view(np.uint8), pad)
            host[off + raw.size:] = t
        self.buf = torch.from_numpy(host).to(DEV)
        self.off, self.n, self.dtype, self.tail = off, raw.size, a.dtype, tail is not None
        self.ptr = self.buf.data_ptr() + off

    def get(self):
        torch.cuda.synchronize()
        return self.buf.cpu().numpy()[self.off:self.off + self.n].copy().view(self.dtype)

    def guards_intact(self):
        torch.cuda.synchronize()
        h = self.buf.cpu().numpy()
        return bool(np.all(h[:self.off] == 0x7E)) and (self.tail or bool(np.all(h[self.off + self.n:] == 0x7E)))


def out_buf(n_halves, off):
    return Carved(np.full(n_halves, 0x7E00, np.uint16), off)


# (M, N, K, gs): one shape per kernel family that chooses by alignment
GEMM = [(1, 64, 4096, 128), (2, 40, 2048, 32), (4, 72, 4096, 32), (1, 64, 11008, 128), (3, 32, 520, 8),
        (8, 64, 2048, 128), (16, 256, 4096, 64), (9, 64, 4104, 8), (40, 48, 1032, 24), (33, 96, 2048, 32),
        (64, 64, 512, 128), (130, 260, 384, 32), (300, 520, 512, 128)]
# byte offsets of (q, scales, zeros, x, c, w_out)
OFFS = [(4, 0, 0, 0, 0, 0), (8, 2, 4, 0, 0, 0), (0, 0, 0, 2, 0, 0), (0, 0, 0, 8, 2, 0), (0, 0, 0, 0, 4, 2),
        (4, 2, 4, 2, 2, 2), (8, 8, 8, 8, 8, 8), (0, 2, 0, 4, 8, 4)]


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(GEMM)))
def test_w4_gemm_unaligned_bases(i, sym):
    c = w4amd.capi()
    M, N, K, gs = GEMM[i]
    seed = 0x0FF5 ^ (i * 977 + (0 if sym else 1))
    p = orc.quantize(orc.normal_weights(N * K, seed), N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, seed + 1)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    for oq, os_, oz, ox, oc, ow in OFFS:
        q_d, s_d = Carved(p.q, oq), Carved(p.scales, os_)
        z_d = None if sym else Carved(p.zeros, oz)
        view = c.packed_view(N, K, gs, p.G, sym, q_d.ptr, s_d.ptr, 0 if sym else z_d.ptr)
        x_d = Carved(x, ox)
        print(f"unaligned gemm M={M} N={N} K={K} gs={gs} sym={sym} offs={(oq, os_, oz, ox, oc, ow)}", flush=True)
        for fn in (c.gemm_fused, c.gemm_mma, c.gemm):
            c_d, w_d = out_buf(M * N, oc), out_buf(N * K, ow)
            fn(view, x_d.ptr, c_d.ptr, M, 0, w_d.ptr)
            assert np.array_equal(w_d.get(), w_ref), "w_out bitwise"
            assert orc.rel_l2(c_d.get().view(np.float16), ref) <= TOL
            assert c_d.guards_intact() and w_d.guards_intact(), "wrote outside c / w_out"
            c2 = out_buf(M * N, oc)
            fn(view, x_d.ptr, c2.ptr, M, 0, 0)
            cross_gate(c_d.get(), c2.get(), ref, fn.__name__)
            assert c2.guards_intact()
        w_d = out_buf(N * K, ow)
        c.dequant(view, w_d.ptr)
        assert np.array_equal(w_d.get(), w_ref) and w_d.guards_intact()


@pytest.mark.parametrize("i", range(len(GEMM)))
def test_mx_gemm_unaligned_bases(i):
    c = w4amd.capi()
    M, N, K, _ = GEMM[i]
    seed = 0x0FF6 ^ (i * 977)
    p = orc.quantize_mx(orc.normal_weights(N * K, seed), N, K)
    w_ref = orc.dequant_all_mx(p)
    x = orc.normal_activations(M * K, seed + 1)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    for oq, os_, _, ox, oc, ow in OFFS:
        q_d, s_d = Carved(p.q, oq), Carved(p.scales, os_ // 2)  # scale bytes at offsets 0, 1, 4
        view = c.packed_mx_view(N, K, p.B, q_d.ptr, s_d.ptr)
        x_d = Carved(x, ox)
        print(f"unaligned mx gemm M={M} N={N} K={K} offs={(oq, os_, ox, oc, ow)}", flush=True)
        for fn in (c.gemm_fused_mx, c.gemm_mma_mx, c.gemm_mx):
            c_d, w_d = out_buf(M * N, oc), out_buf(N * K, ow)
            fn(view, x_d.ptr, c_d.ptr, M, 0, w_d.ptr)
            assert np.array_equal(w_d.get(), w_ref), "w_out bitwise"
            assert orc.rel_l2(c_d.get().view(np.float16), ref) <= TOL
            assert c_d.guards_intact() and w_d.guards_intact()
            c2 = out_buf(M * N, oc)
            fn(view, x_d.ptr, c2.ptr, M, 0, 0)
            if ow % 16 == 0:
                assert np.array_equal(c2.get(), c_d.get())
            assert orc.rel_l2(c2.get().view(np.float16), ref) <= TOL and c2.guards_intact()
        w_d = out_buf(N * K, ow)
        c.dequant_mx(view, w_d.ptr)
        assert np.array_equal(w_d.get(), w_ref) and w_d.guards_intact()


INF_NAN = np.array([0x7C00, 0x7E00, 0xFC00, 0x7FFF], np.uint16)
TAIL = [(9, 64, 4104, 8), (40, 48, 1032, 24), (3, 32, 520, 8), (16, 64, 4104, 8), (64, 48, 1032, 24),
        (5, 16, 264, 16), (12, 32, 2056, 40)]


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(TAIL)))
def test_ragged_k_reads_no_group_past_the_last(i, sym):
    c = w4amd.capi()
    M, N, K, gs = TAIL[i]
    seed = 0x7A11 ^ (i * 977 + (0 if sym else 1))
    p = orc.quantize(orc.normal_weights(N * K, seed), N, K, gs, sym)
    w_ref = orc.dequant_all(p)
    x = orc.normal_activations(M * K, seed + 1)
    ref = orc.gemm_oracle(x, M, K, w_ref, N)
    s_d = Carved(p.scales, 0, tail=INF_NAN)
    z_d = None if sym else Carved(p.zeros, 0, tail=np.array([0xFFFFFFFF], np.uint32))
    q_d = Carved(p.q, 0, tail=np.array([0xFFFFFFFF], np.uint32))
    x_d = Carved(x, 0, tail=INF_NAN)
    view = c.packed_view(N, K, gs, p.G, sym, q_d.ptr, s_d.ptr, 0 if sym else z_d.ptr)
    print(f"tail case M={M} N={N} K={K} gs={gs} sym={sym}", flush=True)
    for fn in (c.gemm_fused, c.gemm_mma):
        for hook in (True, False):
            c_d = out_buf(M * N, 0)
            w_d = out_buf(N * K, 0) if hook else None
            fn(view, x_d.ptr, c_d.ptr, M, 0, w_d.ptr if hook else 0)
            got = c_d.get().view(np.float16).astype(np.float64)
            assert np.all(np.isfinite(got)), "a scale or activation past the arrays reached the output"
            assert orc.rel_l2(got, ref) <= TOL
            if hook:
                assert np.array_equal(w_d.get(), w_ref)


# ---- attention ---------------------------------------------------------------------
ATT = [(2, 300, 128, 32), (1, 777, 64, 16), (2, 130, 96, 32), (3, 65, 40, 8)]
# byte offsets of (q_k / q_v, s_k / s_v, z_k / z_v, q, out, k_out / v_out)
AOFFS = [(4, 0, 0, 0, 0, 0), (8, 2, 4, 2, 2, 2), (0, 0, 0, 8, 4, 8), (0, 2, 0, 0, 0, 0)]


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(ATT)))
def test_w4_flash_unaligned_bases(i, sym):
    c = w4amd.capi()
    H, S, D, gs = ATT[i]
    group = 2
    seed = 0x0FA7 ^ (i * 977 + (0 if sym else 1))
    c4 = orc.quantize_cache(orc.normal_weights(H * S * D, seed), orc.normal_weights(H * S * D, seed + 1),
                            H, S, D, gs, sym)
    q = orc.normal_activations(H * group * D, seed + 2)
    kd, vd = orc.dequant_cache(c4, False), orc.dequant_cache(c4, True)
    ref = orc.attention_f16(q, kd, vd, H, group, S, D)
    npages, page = (S + 15) // 16, 16
    bt = np.random.default_rng(seed).permutation(npages).astype(np.int32)
    for oq, os_, oz, oqq, oo, oh in AOFFS:
        t = [Carved(c4.q_k, oq), Carved(c4.s_k, os_), None if sym else Carved(c4.z_k, oz),
             Carved(c4.q_v, oq), Carved(c4.s_v, os_), None if sym else Carved(c4.z_v, oz)]
        view = c.kv_view(H, S, D, gs, c4.G, sym, *[0 if a is None else a.ptr for a in t])
        q_d = Carved(q, oqq)
        print(f"unaligned w4 flash H={H} S={S} D={D} gs={gs} sym={sym} offs={(oq, os_, oz, oqq, oo, oh)}", flush=True)
        out, ko, vo = out_buf(H * group * D, oo), out_buf(H * S * D, oh), out_buf(H * S * D, oh)
        c.attention_w4_flash(view, q_d.ptr, out.ptr, 0, ko.ptr, vo.ptr, group=group)
        assert np.array_equal(ko.get(), kd.ravel()) and np.array_equal(vo.get(), vd.ravel())
        assert orc.rel_l2(out.get().view(np.float16), ref) <= TOL
        assert out.guards_intact() and ko.guards_intact() and vo.guards_intact()
        out2 = out_buf(H * group * D, oo)
        c.attention_w4_flash(view, q_d.ptr, out2.ptr, group=group)
        if oh % 16 == 0:
            assert np.array_equal(out2.get(), out.get())
        assert orc.rel_l2(out2.get().view(np.float16), ref) <= TOL
        # FP16 flash over the dequantized cache at the same offsets
        k16, v16, o16 = Carved(kd, oq), Carved(vd, oh), out_buf(H * group * D, oo)
        c.attention_fp16_flash(q_d.ptr, k16.ptr, v16.ptr, o16.ptr, H, S, D, group=group)
        assert orc.rel_l2(o16.get().view(np.float16), ref) <= TOL and o16.guards_intact()
        # paged pool at the same offsets: one query head per slab (the reference's entry point)
        wd, wg = orc.words(D), orc.words(c4.G)
        pt = [Carved(orc.paged_scatter(c4.q_k, H, S, page, bt, wd), oq),
              Carved(orc.paged_scatter(c4.s_k, H, S, page, bt, c4.G), os_),
              None if sym else Carved(orc.paged_scatter(c4.z_k, H, S, page, bt, wg), oz),
              Carved(orc.paged_scatter(c4.q_v, H, S, page, bt, wd), oq),
              Carved(orc.paged_scatter(c4.s_v, H, S, page, bt, c4.G), os_),
              None if sym else Carved(orc.paged_scatter(c4.z_v, H, S, page, bt, wg), oz)]
        pview = c.kv_view(H, S, D, gs, c4.G, sym, *[0 if a is None else a.ptr for a in pt])
        q1 = q.reshape(H, group, D)[:, 0].copy()
        q1_d, bt_d = Carved(q1, oqq), Carved(bt, 0)
        o_c, o_p = out_buf(H * D, oo), out_buf(H * D, oo)
        c.attention_w4_flash(view, q1_d.ptr, o_c.ptr)
        c.attention_w4_flash_paged(pview, bt_d.ptr, page, npages, q1_d.ptr, o_p.ptr)
        assert np.array_equal(o_p.get(), o_c.get()), "paged output == contiguous output, bytewise"
        ko, vo, o_h = out_buf(H * S * D, oh), out_buf(H * S * D, oh), out_buf(H * D, oo)
        c.attention_w4_flash_paged(pview, bt_d.ptr, page, npages, q1_d.ptr, o_h.ptr, 0, ko.ptr, vo.ptr)
        assert np.array_equal(ko.get(), kd.ravel()) and np.array_equal(vo.get(), vd.ravel())
        assert orc.rel_l2(o_h.get().view(np.float16), orc.attention_f16(q1, kd, vd, H, 1, S, D)) <= TOL


@pytest.mark.parametrize("i", range(len(ATT)))
def test_f8_flash_unaligned_bases(i):
    c = w4amd.capi()
    H, S, D, gs = ATT[i]
    seed = 0x0FB8 ^ (i * 977)
    c8 = orc.quantize_cache_f8(orc.normal_weights(H * S * D, seed), orc.normal_weights(H * S * D, seed + 1),
                               H, S, D, gs)
    q = orc.normal_activations(H * D, seed + 2)
    kd, vd = orc.dequant_cache_f8(c8, False), orc.dequant_cache_f8(c8, True)
    ref = orc.attention_f16(q, kd, vd, H, 1, S, D)
    for oq, os_, _, oqq, oo, oh in AOFFS:   # cache bases must stay 4-byte aligned (kvflash.cuh:579-582)
        t = [Carved(c8.q_k, oq), Carved(c8.s_k, os_), Carved(c8.q_v, oq), Carved(c8.s_v, os_)]
        view = c.kv_f8_view(H, S, D, gs, c8.G, *[a.ptr for a in t])
        q_d = Carved(q, oqq)
        print(f"unaligned f8 flash H={H} S={S} D={D} gs={gs} offs={(oq, os_, oqq, oo, oh)}", flush=True)
        out, ko, vo = out_buf(H * D, oo), out_buf(H * S * D, oh), out_buf(H * S * D, oh)
        c.attention_f8_flash(view, q_d.ptr, out.ptr, 0, ko.ptr, vo.ptr)
        assert np.array_equal(ko.get(), kd.ravel()) and np.array_equal(vo.get(), vd.ravel())
        assert orc.rel_l2(out.get().view(np.float16), ref) <= TOL
        assert out.guards_intact() and ko.guards_intact() and vo.guards_intact()
        k16 = out_buf(H * S * D, oh)
        c.dequant_f8(t[0].ptr, t[1].ptr, k16.ptr, H * S, D, gs)
        assert np.array_equal(k16.get(), kd.ravel()) and k16.guards_intact()
