"""GPU parity gates for split-S flash-decode attention, through the C ABI.

Follows the reference device suite (tests/test_gpu.cu:506-1467): k_out/v_out
hooks equal the oracle's per-head dequant bit for bit, outputs are within rel
L2 1e-3 of the FP64 softmax(QK^T/sqrt(D))V over the dequantized cache, the FP16
flash path over the dequantized cache is within 2e-3 of the W4 path, and the
paged kernel reproduces the contiguous kernel's bytes.
"""
import numpy as np
import pytest
import torch

import orc
import w4amd
from devutil import DevKV, DevKVF8, bits, f64, halves, ptr, to_dev

pytestmark = pytest.mark.gpu
TOL, CROSS = 1e-3, 2e-3

ATT = [(1, 1, 64, 32), (2, 7, 64, 8), (4, 128, 128, 128), (2, 300, 96, 32), (3, 65, 40, 8),
       (1, 4096, 64, 64),
       # head dimension 128 takes the matrix-core kernel: one position, ragged tiles, gs 32 / 64,
       # and gs = 8 (D = 128 on the general kernel)
       (2, 1, 128, 32), (3, 33, 128, 32), (2, 129, 128, 64), (1, 777, 128, 32), (1, 300, 128, 8),
       # head dimension 64 on the matrix-core kernel (gs a multiple of 16)
       (2, 100, 64, 16), (1, 1, 64, 64), (3, 257, 64, 32),
       # either side of the longest cache that one split per slab serves (its kernel writes the
       # output itself, no merge launch)
       (2, 512, 128, 32), (2, 513, 128, 32), (1, 512, 64, 16), (2, 400, 128, 64)]
BIG = [(2, 5000, 64, 32), (1, 9000, 128, 64)]
# more slabs than workgroups wanted: one split per slab, 9 to 11 tiles per wave
LONG_SPLITS = [(520, 1300, 128, 32), (600, 1100, 64, 32)]


def _w4_case(H, S, D, gs, sym, seed, group=1):
    k = orc.normal_weights(H * S * D, seed)
    v = orc.normal_weights(H * S * D, seed + 1)
    q = orc.normal_activations(H * group * D, seed + 2)
    c4 = orc.quantize_cache(k, v, H, S, D, gs, sym)
    return c4, q


def _check_w4(c4, q, group=1):
    c = w4amd.capi()
    H, S, D = c4.H, c4.S, c4.D
    kd, vd = orc.dequant_cache(c4, False), orc.dequant_cache(c4, True)
    ref = orc.attention_f16(q, kd, vd, H, group, S, D)
    dk, q_d = DevKV(c4), to_dev(q)
    out = halves(H * group * D, 0x7E00)
    ko, vo = halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_w4_flash(dk.view, ptr(q_d), ptr(out), 0, ptr(ko), ptr(vo), group=group)
    assert np.array_equal(bits(ko), kd.ravel()), "k_out bitwise"
    assert np.array_equal(bits(vo), vd.ravel()), "v_out bitwise"
    o_w4 = bits(out).copy()
    assert orc.rel_l2(o_w4.view(np.float16), ref) <= TOL
    # no hooks: same bytes
    out2 = halves(H * group * D, 0x7E00)
    c.attention_w4_flash(dk.view, ptr(q_d), ptr(out2), group=group)
    assert np.array_equal(bits(out2), o_w4)
    # FP16 flash over the dequantized cache: oracle gate + cross gate
    k16, v16, o16 = to_dev(kd), to_dev(vd), halves(H * group * D, 0x7E00)
    c.attention_fp16_flash(ptr(q_d), ptr(k16), ptr(v16), ptr(o16), H, S, D, group=group)
    assert orc.rel_l2(f64(o16), ref) <= TOL
    den = np.sqrt(np.sum(ref ** 2))
    cross = np.sqrt(np.sum((f64(o16) - o_w4.view(np.float16).astype(np.float64)) ** 2)) / den
    assert cross <= CROSS
    return o_w4, dk, q_d, kd, vd, ref


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(ATT)))
def test_w4_flash(i, sym):
    H, S, D, gs = ATT[i]
    c4, q = _w4_case(H, S, D, gs, sym, 0x77B5 ^ (i * 977 + (0 if sym else 1)))
    _check_w4(c4, q)


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(BIG)))
def test_w4_flash_long(i, sym):
    H, S, D, gs = BIG[i]
    c4, q = _w4_case(H, S, D, gs, sym, 0x51D0 ^ (i * 977 + (0 if sym else 1)))
    _check_w4(c4, q)


def test_w4_flash_many_slabs():
    """More (sequence, kv-head) slabs than a 16-bit grid dimension holds."""
    c4, q = _w4_case(70000, 3, 8, 8, True, 0x70000)
    _check_w4(c4, q)


@pytest.mark.parametrize("group", [2, 3, 4, 7, 16, 17, 40])
def test_w4_flash_grouped_query(group):
    """Query heads sharing one slab; more than 16 heads take several passes."""
    c4, q = _w4_case(3 if group < 16 else 2, 700, 128, 32, group % 2 == 0, 0x6A11 + group, group)
    _check_w4(c4, q, group)


@pytest.mark.parametrize("group", [3, 5])
def test_w4_flash_grouped_query_general_kernel(group):
    c4, q = _w4_case(2, 333, 96, 32, True, 0x6B22 + group, group)
    _check_w4(c4, q, group)


@pytest.mark.parametrize("group", [4, 17])
def test_w4_flash_grouped_query_head_dim_64(group):
    c4, q = _w4_case(2, 400, 64, 32, group == 4, 0x6C33 + group, group)
    _check_w4(c4, q, group)


F8 = [(1, 1, 64, 32), (2, 7, 64, 8), (4, 128, 128, 128), (2, 300, 96, 32), (3, 65, 40, 8),
      (1, 9000, 128, 64), (2, 1, 128, 32), (2, 100, 128, 32), (1, 300, 128, 16), (2, 200, 64, 16),
      (1, 2500, 64, 64), (2, 512, 128, 32), (2, 513, 128, 32)]


@pytest.mark.parametrize("i", range(len(F8)))
def test_f8_flash(i):
    H, S, D, gs = F8[i]
    seed = 0xF80A ^ (i * 977)
    k = orc.normal_weights(H * S * D, seed)
    v = orc.normal_weights(H * S * D, seed + 1)
    q = orc.normal_activations(H * D, seed + 2)
    _check_f8(H, S, D, gs, k, v, q)


def test_f8_flash_long_splits():
    """Splits of 6 and more tiles per wave: the loop that only sees whole tiles."""
    H, S, D, gs = LONG_SPLITS[0]
    rng = np.random.default_rng(0xF81B)
    k, v = rng.standard_normal(H * S * D), rng.standard_normal(H * S * D)
    _check_f8(H, S, D, gs, k, v, orc.normal_activations(H * D, 0xF81C))


def _check_f8(H, S, D, gs, k, v, q):
    c = w4amd.capi()
    c8 = orc.quantize_cache_f8(k, v, H, S, D, gs)
    kd, vd = orc.dequant_cache_f8(c8, False), orc.dequant_cache_f8(c8, True)
    ref = orc.attention_f16(q, kd, vd, H, 1, S, D)
    d8, q_d = DevKVF8(c8), to_dev(q)
    out, ko, vo = halves(H * D, 0x7E00), halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_f8_flash(d8.view, ptr(q_d), ptr(out), 0, ptr(ko), ptr(vo))
    assert np.array_equal(bits(ko), kd.ravel()) and np.array_equal(bits(vo), vd.ravel())
    assert orc.rel_l2(f64(out), ref) <= TOL
    # device two-pass: dequant_f8 per side, then FP16 flash
    k16, v16, o16 = halves(H * S * D), halves(H * S * D), halves(H * D)
    c.dequant_f8(ptr(d8.t[0]), ptr(d8.t[1]), ptr(k16), H * S, D, gs)
    c.dequant_f8(ptr(d8.t[2]), ptr(d8.t[3]), ptr(v16), H * S, D, gs)
    assert np.array_equal(bits(k16), kd.ravel()) and np.array_equal(bits(v16), vd.ravel())
    c.attention_fp16_flash(ptr(q_d), ptr(k16), ptr(v16), ptr(o16), H, S, D)
    den = np.sqrt(np.sum(ref ** 2))
    assert np.sqrt(np.sum((f64(o16) - f64(out)) ** 2)) / den <= CROSS


def test_f8_every_code_and_slab_scale():
    """All 256 byte codes under several scales (hooks bit-exact), then the
    per-slab scale mode against the reference arithmetic on a broadcast scale."""
    c = w4amd.capi()
    H, S, D, gs = 2, 64, 32, 32
    c8 = orc.KVCacheF8()
    c8.H, c8.S, c8.D, c8.gs, c8.G = H, S, D, gs, 1
    codes = (np.arange(H * S * D) % 256).astype(np.uint8)
    c8.q_k, c8.q_v = codes, codes[::-1].copy()
    sc = np.array([0x3C00, 0x0001, 0x03FF, 0x5BFF, 0x7BFF, 0x2E66, 0x8400, 0x1400], np.uint16)
    c8.s_k = np.resize(sc, H * S)
    c8.s_v = np.resize(sc[::-1], H * S)
    kd, vd = orc.dequant_cache_f8(c8, False), orc.dequant_cache_f8(c8, True)
    d8 = DevKVF8(c8)
    q_d = to_dev(np.zeros(H * D, np.uint16))
    out, ko, vo = halves(H * D), halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_f8_flash(d8.view, ptr(q_d), ptr(out), 0, ptr(ko), ptr(vo))
    assert np.array_equal(bits(ko), kd.ravel()) and np.array_equal(bits(vo), vd.ravel())
    # per-slab scale: one FP16 scale per slab == the same value in every slot
    rng = np.random.default_rng(2)
    kk = rng.standard_normal(H * S * D)
    c8 = orc.quantize_cache_f8(kk, kk[::-1].copy(), H, S, D, gs)
    slab_k = np.array([0x2000, 0x2400], np.uint16)
    slab_v = np.array([0x2200, 0x1C00], np.uint16)
    c8b = orc.KVCacheF8()
    c8b.__dict__.update(c8.__dict__)
    c8b.s_k, c8b.s_v = np.repeat(slab_k, S), np.repeat(slab_v, S)
    q = orc.normal_activations(H * 2 * D, 77)
    ref = orc.attention_reference_f8(q, c8b, heads_per_slab=2)
    d8 = DevKVF8(c8, slab_k, slab_v)
    out = halves(H * 2 * D, 0x7E00)
    ko, vo = halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_f8_flash(d8.view, ptr(to_dev(q)), ptr(out), 0, ptr(ko), ptr(vo), group=2, scale_mode=1)
    assert np.array_equal(bits(ko), orc.dequant_cache_f8(c8b, False).ravel())
    assert orc.rel_l2(f64(out), ref) <= TOL


@pytest.mark.parametrize("nan_codes", ["none", "first_tile", "all"])
def test_f8_every_code_matrix_core_kernel(nan_codes):
    """Every byte code under odd scales through the D = 128 matrix-core kernel, hooks
    bit-exact.  The closed-form decode reads the NaN codes 0x7F / 0xFF as +-480
    (kvfp8.hpp:41-50); none / some / all of the tiles hold such a code, so a decode
    that treats those tiles differently is covered on both sides."""
    c = w4amd.capi()
    H, S, D, gs = 2, 160, 128, 32
    G = D // gs
    c8 = orc.KVCacheF8()
    c8.H, c8.S, c8.D, c8.gs, c8.G = H, S, D, gs, G
    codes = (np.arange(H * S * D) % 256).astype(np.uint8)
    pos = (np.arange(H * S * D) // D) % S
    special = (codes & 0x7F) == 0x7F
    if nan_codes == "none":
        codes[special] -= 1
    elif nan_codes == "first_tile":
        codes[special & (pos >= 32)] -= 1
    c8.q_k, c8.q_v = codes, codes[::-1].copy()
    sc = np.array([0x3C00, 0x0001, 0x03FF, 0x5BFF, 0x7BFF, 0x2E66, 0x8400, 0x1400, 0x3555], np.uint16)
    c8.s_k = np.resize(sc, H * S * G)
    c8.s_v = np.resize(sc[::-1], H * S * G)
    kd, vd = orc.dequant_cache_f8(c8, False), orc.dequant_cache_f8(c8, True)
    d8 = DevKVF8(c8)
    q_d = to_dev(np.zeros(H * D, np.uint16))
    out, ko, vo = halves(H * D), halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_f8_flash(d8.view, ptr(q_d), ptr(out), 0, ptr(ko), ptr(vo))
    assert np.array_equal(bits(ko), kd.ravel()) and np.array_equal(bits(vo), vd.ravel())


def test_f8_slab_scale_head_dim_128():
    c = w4amd.capi()
    H, S, D, gs, group = 2, 500, 128, 128, 4
    rng = np.random.default_rng(5)
    kk = rng.standard_normal(H * S * D)
    c8 = orc.quantize_cache_f8(kk, kk[::-1].copy(), H, S, D, gs)
    slab_k = np.array([0x2000, 0x2400], np.uint16)
    slab_v = np.array([0x2200, 0x1C00], np.uint16)
    c8b = orc.KVCacheF8()
    c8b.__dict__.update(c8.__dict__)
    c8b.s_k, c8b.s_v = np.repeat(slab_k, S * c8.G), np.repeat(slab_v, S * c8.G)
    q = orc.normal_activations(H * group * D, 78)
    ref = orc.attention_reference_f8(q, c8b, heads_per_slab=group)
    d8 = DevKVF8(c8, slab_k, slab_v)
    out = halves(H * group * D, 0x7E00)
    ko, vo = halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_f8_flash(d8.view, ptr(to_dev(q)), ptr(out), 0, ptr(ko), ptr(vo), group=group, scale_mode=1)
    assert np.array_equal(bits(ko), orc.dequant_cache_f8(c8b, False).ravel())
    assert np.array_equal(bits(vo), orc.dequant_cache_f8(c8b, True).ravel())
    assert orc.rel_l2(f64(out), ref) <= TOL
    out2 = halves(H * group * D, 0x7E00)
    c.attention_f8_flash(d8.view, ptr(to_dev(q)), ptr(out2), group=group, scale_mode=1)
    assert np.array_equal(bits(out2), bits(out))


PAGED = [(2, 300, 96, 32, 16), (2, 520, 64, 32, 16), (1, 1000, 128, 64, 64), (3, 65, 40, 8, 32),
         (1, 5000, 64, 32, 256),
         # matrix-core kernel: page 16, a page size that is no multiple of 16, one-row pages
         (2, 700, 128, 32, 16), (1, 530, 128, 32, 24), (1, 100, 128, 128, 1), (2, 2000, 128, 32, 256),
         (2, 300, 64, 16, 40), (1, 900, 64, 32, 48)]


def _paged_pool(c4, page, bt):
    """Device copy of the cache scattered into a pool by `bt` (kvpaged.hpp:72-134)."""
    c = w4amd.capi()
    H, S, D, G = c4.H, c4.S, c4.D, c4.G
    wd, wg = orc.words(D), orc.words(G)
    t = [to_dev(orc.paged_scatter(c4.q_k, H, S, page, bt, wd)),
         to_dev(orc.paged_scatter(c4.s_k, H, S, page, bt, G)),
         None if c4.symmetric else to_dev(orc.paged_scatter(c4.z_k, H, S, page, bt, wg)),
         to_dev(orc.paged_scatter(c4.q_v, H, S, page, bt, wd)),
         to_dev(orc.paged_scatter(c4.s_v, H, S, page, bt, G)),
         None if c4.symmetric else to_dev(orc.paged_scatter(c4.z_v, H, S, page, bt, wg))]
    view = c.kv_view(H, S, D, c4.gs, G, c4.symmetric, *[ptr(x) for x in t])
    return t, view


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(PAGED)))
def test_paged_equals_contiguous(i, sym):
    c = w4amd.capi()
    H, S, D, gs, page = PAGED[i]
    seed = 0x9A6E ^ (i * 977 + (0 if sym else 1))
    c4, q = _w4_case(H, S, D, gs, sym, seed)
    o_w4, dk, q_d, kd, vd, ref = _check_w4(c4, q)
    npages = (S + page - 1) // page
    bt = np.random.default_rng(seed ^ 0x5ED).permutation(npages).astype(np.int32)
    keep, view = _paged_pool(c4, page, bt)
    bt_d = to_dev(bt)
    out, ko, vo = halves(H * D, 0x7E00), halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_w4_flash_paged(view, ptr(bt_d), page, npages, ptr(q_d), ptr(out), 0, ptr(ko), ptr(vo))
    assert np.array_equal(bits(out), o_w4), "paged output == contiguous output, bytewise"
    assert np.array_equal(bits(ko), kd.ravel()) and np.array_equal(bits(vo), vd.ravel())


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
@pytest.mark.parametrize("i", range(len(LONG_SPLITS)))
def test_w4_flash_long_splits(i, sym):
    """So many slabs that each gets one or two splits: a wave walks 6 and more tiles,
    which takes the loop that only sees whole tiles (its look-ahead of the page
    table included), then the loop for the cut tiles at the end."""
    c = w4amd.capi()
    H, S, D, gs = LONG_SPLITS[i]
    seed = 0x10E6 ^ (i * 977 + (0 if sym else 1))
    rng = np.random.default_rng(seed)
    k, v = rng.standard_normal(H * S * D), rng.standard_normal(H * S * D)
    c4 = orc.quantize_cache(k, v, H, S, D, gs, sym)
    q = orc.normal_activations(H * D, seed + 2)
    o_w4, dk, q_d, kd, vd, ref = _check_w4(c4, q)
    for page in (16, 48):
        npages = (S + page - 1) // page
        bt = np.random.default_rng(seed ^ page).permutation(npages).astype(np.int32)
        keep, view = _paged_pool(c4, page, bt)
        bt_d = to_dev(bt)
        out = halves(H * D, 0x7E00)
        c.attention_w4_flash_paged(view, ptr(bt_d), page, npages, ptr(q_d), ptr(out))
        assert np.array_equal(bits(out), o_w4), "paged output == contiguous output, bytewise"


@pytest.mark.parametrize("D", [64, 128])
def test_paged_batched_prefix_sharing(D):
    """Four sequences over one pool; the first three share their leading pages.
    Each sequence's output equals the contiguous kernel run on its logical cache."""
    c = w4amd.capi()
    Hkv, gs, page, group = 2, 32, 16, 2
    S, prefix = 520, 208                     # 13 shared pages
    nseq = 4
    lp = (S + page - 1) // page
    pp = prefix // page
    rng = np.random.default_rng(0xCAFE)
    # logical caches: sequences 0..2 share the prefix rows, sequence 3 is independent
    base_k = orc.normal_weights(Hkv * S * D, 0xBEEF).reshape(Hkv, S, D)
    base_v = orc.normal_weights(Hkv * S * D, 0xBEE0).reshape(Hkv, S, D)
    caches = []
    for s in range(nseq):
        k = orc.normal_weights(Hkv * S * D, 0x1000 + s).reshape(Hkv, S, D)
        v = orc.normal_weights(Hkv * S * D, 0x2000 + s).reshape(Hkv, S, D)
        if s < 3:
            k[:, :prefix], v[:, :prefix] = base_k[:, :prefix], base_v[:, :prefix]
        caches.append(orc.quantize_cache(k, v, Hkv, S, D, gs, True))
    # pool: shared prefix pages once, then each sequence's own pages, shuffled placement
    npages = pp + 3 * (lp - pp) + lp
    phys = rng.permutation(npages).astype(np.int32)
    tables = np.zeros((nseq, lp), np.int32)
    nxt = pp
    for s in range(nseq):
        for i in range(lp):
            if s < 3 and i < pp:
                tables[s, i] = phys[i]
            else:
                tables[s, i] = phys[nxt]
                nxt += 1
    assert nxt == npages
    wd, G = orc.words(D), caches[0].G
    pool = {n: np.zeros((Hkv, npages * page, w), dt) for n, w, dt in
            (("q_k", wd, np.uint32), ("q_v", wd, np.uint32), ("s_k", G, np.uint16), ("s_v", G, np.uint16))}
    for s, c4 in enumerate(caches):
        for n in pool:
            src = getattr(c4, n).reshape(Hkv, S, -1)
            for t in range(S):
                pool[n][:, tables[s, t // page] * page + t % page] = src[:, t]
    dev = {n: to_dev(a.ravel()) for n, a in pool.items()}
    view = c.kv_view(Hkv, S, D, gs, G, True, ptr(dev["q_k"]), ptr(dev["s_k"]), 0, ptr(dev["q_v"]),
                     ptr(dev["s_v"]), 0)
    q = orc.normal_activations(nseq * Hkv * group * D, 0xFEED)
    q_d, bt_d = to_dev(q), to_dev(tables.ravel())
    out = halves(nseq * Hkv * group * D, 0x7E00)
    c.attention_w4_flash_paged_batched(view, ptr(bt_d), nseq, lp, page, npages, group, ptr(q_d), ptr(out))
    got = bits(out).reshape(nseq, Hkv * group * D)
    qs = q.reshape(nseq, Hkv * group * D)
    for s, c4 in enumerate(caches):
        ref = orc.attention_reference(qs[s], c4, heads_per_slab=group)
        assert orc.rel_l2(got[s].view(np.float16), ref) <= TOL
        dk = DevKV(c4)
        o = halves(Hkv * group * D, 0x7E00)
        c.attention_w4_flash(dk.view, ptr(to_dev(qs[s])), ptr(o), group=group)
        assert np.array_equal(bits(o), got[s]), "paged batch == contiguous, bytewise"


@pytest.mark.parametrize("sym", [True, False], ids=["sym", "asym"])
def test_w4_flash_batch_plan_of_64_slabs_by_32768_positions(sym):
    """The split plan of the batch-8, 8-kv-head decode step: 64 slabs of 32768 positions give
    8 splits per slab and 32 tiles of 32 positions per wave, with 4 query heads per slab.
    The 64 slabs are 4 oracle-quantized sample slabs repeated (slab i holds sample i % 4), so
    hooks and outputs are checked against four slabs' worth of oracle work; everything is
    compared on the device."""
    c = w4amd.capi()
    H, NS, S, D, gs, group = 64, 4, 32768, 128, 32, 4
    seed = 0xB8B8 + (0 if sym else 1)
    c4 = orc.quantize_cache(orc.normal_weights(NS * S * D, seed), orc.normal_weights(NS * S * D, seed + 1),
                            NS, S, D, gs, sym)
    kd, vd = orc.dequant_cache(c4, False), orc.dequant_cache(c4, True)
    q = orc.normal_activations(H * group * D, seed + 2)
    idx = torch.arange(H, device="cuda") % NS

    def rep(a):
        return to_dev(np.ascontiguousarray(a).reshape(NS, -1))[idx].contiguous()
    t = [rep(c4.q_k), rep(c4.s_k), None if sym else rep(c4.z_k), rep(c4.q_v), rep(c4.s_v),
         None if sym else rep(c4.z_v)]
    view = c.kv_view(H, S, D, gs, c4.G, sym, *[ptr(a) for a in t])
    q_d = to_dev(q)
    out, out2 = halves(H * group * D, 0x7E00), halves(H * group * D, 0x7E00)
    ko, vo = halves(H * S * D, 0x7E00), halves(H * S * D, 0x7E00)
    c.attention_w4_flash(view, ptr(q_d), ptr(out), 0, ptr(ko), ptr(vo), group=group)
    assert torch.equal(ko.view(H, -1), to_dev(kd).view(NS, -1)[idx]), "k_out bitwise"
    assert torch.equal(vo.view(H, -1), to_dev(vd).view(NS, -1)[idx]), "v_out bitwise"
    del ko, vo
    c.attention_w4_flash(view, ptr(q_d), ptr(out2), group=group)
    assert torch.equal(out, out2), "hooked and unhooked bytes differ"
    got = bits(out2).view(np.float16).reshape(H, group, D)
    for i in (0, 9, 18, 27, 63):  # slabs of five different sequences, all four samples
        ref = orc.attention_f16(q.reshape(H, group * D)[i], kd[i % NS:i % NS + 1], vd[i % NS:i % NS + 1],
                                1, group, S, D)
        assert orc.rel_l2(got[i], ref) <= TOL
