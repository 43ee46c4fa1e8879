"""ctypes view of the CPU oracle (oracle/libw4oracle.so) for the tests.

The oracle is the checker: tests, the smoke check and the benchmark's CPU
baseline load it; the shipped library never does.  Halves travel as numpy
uint16 bit patterns (``.view(np.float16)`` gives the values).
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(ROOT, "oracle", "libw4oracle.so")

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
        L = C.CDLL(_SO)
        L.orc_last_error.restype = C.c_char_p
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_dequant_one.restype = C.c_uint16
        L.orc_dequant_one.argtypes = [C.c_uint16, C.c_int, C.c_int]
        L.orc_dequant_one_mx.restype = C.c_uint16
        L.orc_dequant_one_mx.argtypes = [C.c_uint8, C.c_int]
        L.orc_decode_f8_e4m3.restype = C.c_float
        L.orc_decode_f8_e4m3.argtypes = [C.c_uint8]
        L.orc_dequant_one_f8.restype = C.c_uint16
        L.orc_dequant_one_f8.argtypes = [C.c_uint16, C.c_uint8]
        L.orc_f32_to_e4m3_satfinite.restype = C.c_uint8
        L.orc_f32_to_e4m3_satfinite.argtypes = [C.c_float]
        L.orc_rel_l2_f16_vs_f64.restype = C.c_double
        L.orc_max_abs_f16_vs_f64.restype = C.c_double
        _lib = L
    return _lib


class OracleInvalid(ValueError):
    """Raised where the reference throws std::invalid_argument."""


def _chk(rc):
    if rc != 0:
        raise OracleInvalid(lib().orc_last_error().decode())


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _sz(n):
    return C.c_size_t(int(n))


def words(n):
    return (n + 7) // 8


def set_threads(n):
    lib().orc_set_threads(C.c_int(n))


# ---- generators ----------------------------------------------------------
def mt_stream(seed, n):
    out = np.empty(n, np.uint64)
    lib().orc_mt19937_64_stream(C.c_uint64(seed), _p(out), _sz(n))
    return out


def normal_weights(n, seed):
    out = np.empty(n, np.float64)
    lib().orc_normal_weights(_p(out), _sz(n), C.c_uint64(seed))
    return out


def normal_activations(n, seed):
    out = np.empty(n, np.uint16)
    lib().orc_normal_activations(_p(out), _sz(n), C.c_uint64(seed))
    return out


def laplace_weights(n, seed):
    out = np.empty(n, np.float64)
    lib().orc_laplace_weights(_p(out), _sz(n), C.c_uint64(seed))
    return out


def uniform_weights(n, seed):
    out = np.empty(n, np.float64)
    lib().orc_uniform_weights(_p(out), _sz(n), C.c_uint64(seed))
    return out


def uniform_int_stream(seed, rng, n):
    out = np.empty(n, np.uint64)
    lib().orc_uniform_int_stream(C.c_uint64(seed), C.c_uint64(rng), _p(out), _sz(n))
    return out


# ---- the benchmark configs' weight distributions ----------------------------
def one_sided_group_weights(N, K, gs, seed, sigma=0.02, fraction=0.10):
    """sigma * N(0,1); `fraction` of the (row, group)s made one-sided (all positive)."""
    w = (normal_weights(N * K, seed) * sigma).reshape(N, K)
    G = (K + gs - 1) // gs
    one_sided = np.random.default_rng(seed ^ 0x51DE).random((N, G)) < fraction
    mask = one_sided[:, np.arange(K) // gs]
    w[mask] = np.abs(w[mask])
    return w.ravel()


def outlier_weights(N, K, seed, sigma=0.02, fraction=0.01, at=20.0):
    """sigma * N(0,1); `fraction` of the elements replaced by an outlier of +-`at` sigma."""
    w = normal_weights(N * K, seed) * sigma
    rng = np.random.default_rng(seed ^ 0x0071)
    idx = rng.random(N * K) < fraction
    w[idx] = np.where(rng.random(int(idx.sum())) < 0.5, -1.0, 1.0) * (at * sigma)
    return w


# ---- W4 --------------------------------------------------------------------
class PackedW:
    def __init__(self, N, K, gs, symmetric, q, scales, zeros):
        self.N, self.K, self.gs = N, K, gs
        self.G = (K + gs - 1) // gs if gs > 0 else 0
        self.symmetric = bool(symmetric)
        self.q, self.scales, self.zeros = q, scales, zeros


def quantize(w, N, K, gs, symmetric):
    w = np.ascontiguousarray(w, np.float64).ravel()
    okdims = N >= 1 and K >= 1 and gs >= 8 and gs % 8 == 0
    G = (K + gs - 1) // gs if okdims else 1
    q = np.zeros(max(1, N) * words(max(1, K)), np.uint32)
    s = np.zeros(max(1, N) * G, np.uint16)
    z = None if symmetric else np.zeros(max(1, N) * words(G), np.uint32)
    _chk(lib().orc_quantize(_p(w), _sz(w.size), N, K, gs, int(bool(symmetric)),
                            _p(q), _p(s), _p(z)))
    return PackedW(N, K, gs, symmetric, q, s, z)


def dequant_all(p):
    out = np.empty(max(1, p.N * p.K), np.uint16)
    z = p.zeros
    _chk(lib().orc_dequant_all(p.N, p.K, p.gs, p.G, int(p.symmetric), _p(p.q),
                               _sz(p.q.size), _p(p.scales), _sz(p.scales.size),
                               _p(z), _sz(0 if z is None else z.size), _p(out)))
    return out


def gemm_oracle(x, M, K, w, N):
    x = np.ascontiguousarray(x, np.uint16).ravel()
    w = np.ascontiguousarray(w, np.uint16).ravel()
    c = np.empty(max(1, M * N), np.float64)
    _chk(lib().orc_gemm_oracle(_p(x), _sz(x.size), M, K, _p(w), _sz(w.size), N,
                               _p(c)))
    return c.reshape(M, N)


# ---- MXFP4 -----------------------------------------------------------------
class PackedWm:
    def __init__(self, N, K, q, scales):
        self.N, self.K, self.B = N, K, (K + 31) // 32
        self.q, self.scales = q, scales


def quantize_mx(w, N, K):
    w = np.ascontiguousarray(w, np.float64).ravel()
    q = np.zeros(max(1, N) * words(max(1, K)), np.uint32)
    s = np.zeros(max(1, N) * ((max(1, K) + 31) // 32), np.uint8)
    _chk(lib().orc_quantize_mx(_p(w), _sz(w.size), N, K, _p(q), _p(s)))
    return PackedWm(N, K, q, s)


def dequant_all_mx(p):
    out = np.empty(max(1, p.N * p.K), np.uint16)
    _chk(lib().orc_dequant_all_mx(p.N, p.K, p.B, _p(p.q), _sz(p.q.size),
                                  _p(p.scales), _sz(p.scales.size), _p(out)))
    return out


# ---- MXFP8 activations (additive format) -------------------------------------
class PackedXm8:
    def __init__(self, M, K, q, scales):
        self.M, self.K, self.B = M, K, (K + 31) // 32
        self.q, self.scales = q, scales


def quantize_mx8(x, M, K):
    x = np.ascontiguousarray(x, np.float64).ravel()
    q = np.zeros(max(1, M) * max(1, K), np.uint8)
    s = np.zeros(max(1, M) * ((max(1, K) + 31) // 32), np.uint8)
    _chk(lib().orc_quantize_mx8(_p(x), _sz(x.size), M, K, _p(q), _p(s)))
    return PackedXm8(M, K, q, s)


def dequant_mx8(p):
    out = np.empty(p.M * p.K, np.float64)
    _chk(lib().orc_dequant_mx8(p.M, p.K, _p(p.q), _p(p.scales), _p(out)))
    return out.reshape(p.M, p.K)


def gemm_f64(x, M, K, w, N):
    x = np.ascontiguousarray(x, np.float64).ravel()
    w = np.ascontiguousarray(w, np.float64).ravel()
    assert x.size == M * K and w.size == N * K
    c = np.empty(M * N, np.float64)
    _chk(lib().orc_gemm_f64(_p(x), M, K, _p(w), N, _p(c)))
    return c.reshape(M, N)


# ---- KV caches -------------------------------------------------------------
class KVCacheW4:
    pass


def quantize_cache(k, v, H, S, D, gs, symmetric):
    k = np.ascontiguousarray(k, np.float64).ravel()
    v = np.ascontiguousarray(v, np.float64).ravel()
    ok = H >= 1 and S >= 1 and D >= 1 and gs >= 8 and gs % 8 == 0
    G = (D + gs - 1) // gs if ok else 1
    n = max(1, H) * max(1, S)
    c = KVCacheW4()
    c.H, c.S, c.D, c.gs, c.G, c.symmetric = H, S, D, gs, G, bool(symmetric)
    c.q_k = np.zeros(n * words(max(1, D)), np.uint32)
    c.q_v = np.zeros_like(c.q_k)
    c.s_k = np.zeros(n * G, np.uint16)
    c.s_v = np.zeros_like(c.s_k)
    c.z_k = None if symmetric else np.zeros(n * words(G), np.uint32)
    c.z_v = None if symmetric else np.zeros(n * words(G), np.uint32)
    _chk(lib().orc_quantize_cache(_p(k), _sz(k.size), _p(v), _sz(v.size), H, S, D,
                                  gs, int(bool(symmetric)), _p(c.q_k), _p(c.s_k),
                                  _p(c.z_k), _p(c.q_v), _p(c.s_v), _p(c.z_v)))
    return c


def dequant_cache(c, vside):
    """All H slabs of one side as (H, S, D) half bits (dequant_head per head)."""
    q = c.q_v if vside else c.q_k
    s = c.s_v if vside else c.s_k
    z = c.z_v if vside else c.z_k
    p = PackedW(c.H * c.S, c.D, c.gs, c.symmetric, q, s, z)
    return dequant_all(p).reshape(c.H, c.S, c.D)


def attention_f16(q, k16, v16, H, heads_per_slab, S, D):
    q = np.ascontiguousarray(q, np.uint16).ravel()
    k16 = np.ascontiguousarray(k16, np.uint16).ravel()
    v16 = np.ascontiguousarray(v16, np.uint16).ravel()
    assert q.size == H * heads_per_slab * D and k16.size == H * S * D == v16.size
    out = np.empty(H * heads_per_slab * D, np.float64)
    _chk(lib().orc_attention_f16(_p(q), _p(k16), _p(v16), H, heads_per_slab, S, D,
                                 _p(out)))
    return out.reshape(H * heads_per_slab, D)


def attention_reference(q, c, heads_per_slab=1):
    return attention_f16(q, dequant_cache(c, False), dequant_cache(c, True), c.H,
                         heads_per_slab, c.S, c.D)


class KVCacheF8:
    pass


def quantize_cache_f8(k, v, H, S, D, gs):
    k = np.ascontiguousarray(k, np.float64).ravel()
    v = np.ascontiguousarray(v, np.float64).ravel()
    ok = H >= 1 and S >= 1 and D >= 1 and gs >= 8 and gs % 8 == 0
    G = (D + gs - 1) // gs if ok else 1
    n = max(1, H) * max(1, S)
    c = KVCacheF8()
    c.H, c.S, c.D, c.gs, c.G = H, S, D, gs, G
    c.q_k = np.zeros(n * max(1, D), np.uint8)
    c.q_v = np.zeros_like(c.q_k)
    c.s_k = np.zeros(n * G, np.uint16)
    c.s_v = np.zeros_like(c.s_k)
    _chk(lib().orc_quantize_cache_f8(_p(k), _sz(k.size), _p(v), _sz(v.size), H, S,
                                     D, gs, _p(c.q_k), _p(c.s_k), _p(c.q_v),
                                     _p(c.s_v)))
    return c


def dequant_cache_f8(c, vside):
    q = c.q_v if vside else c.q_k
    s = c.s_v if vside else c.s_k
    out = np.empty(c.H * c.S * c.D, np.uint16)
    _chk(lib().orc_dequant_f8(_p(q), _p(s), c.H * c.S, c.D, c.gs, _p(out)))
    return out.reshape(c.H, c.S, c.D)


def attention_reference_f8(q, c, heads_per_slab=1):
    return attention_f16(q, dequant_cache_f8(c, False), dequant_cache_f8(c, True),
                         c.H, heads_per_slab, c.S, c.D)


def paged_scatter(src, H, S, page, bt, row_elems):
    """Pool copy of an (H*S*row_elems) array: logical page i -> physical bt[i]."""
    src = np.ascontiguousarray(src)
    bt = np.ascontiguousarray(bt, np.int32)
    dst = np.zeros(H * max(1, bt.size) * max(1, page) * row_elems, src.dtype)
    _chk(lib().orc_paged_scatter(_p(src), _p(dst), H, S, page, _p(bt), int(bt.size),
                                 _sz(row_elems), _sz(src.dtype.itemsize)))
    return dst


def rel_l2_f16_vs_f64(a, b):
    a = np.ascontiguousarray(a, np.float64).ravel()
    b = np.ascontiguousarray(b, np.uint16).ravel()
    return lib().orc_rel_l2_f16_vs_f64(_p(a), _p(b), _sz(a.size))


def max_abs_f16_vs_f64(a, b):
    a = np.ascontiguousarray(a, np.float64).ravel()
    b = np.ascontiguousarray(b, np.uint16).ravel()
    return lib().orc_max_abs_f16_vs_f64(_p(a), _p(b), _sz(a.size))


def rel_l2(dev, ref):
    """sqrt(sum((dev-ref)^2)/sum(ref^2)) -- the device-vs-oracle gate metric
    (reference tests/test_gpu.cu:145-151)."""
    dev = np.asarray(dev, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    den = float(np.sum(ref * ref))
    return float(np.sqrt(np.sum((dev - ref) ** 2) / (den if den > 0 else 1.0)))
