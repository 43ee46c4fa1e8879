"""ctypes view of libw4amd.so.  Arguments are raw device addresses (ints, e.g.
``tensor.data_ptr()``); 0 stands for a null pointer.  Errors map like the C++
wrappers: W4_EINVAL -> ValueError (std::invalid_argument), W4_ERUNTIME ->
RuntimeError.  There is no fallback: a missing library raises at load()."""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# W4AMD_LIB points at another build of the same library (kernel tuning builds)
LIB_PATH = os.environ.get("W4AMD_LIB") or os.path.join(_PKG, "lib", "libw4amd.so")

W4_OK, W4_EINVAL, W4_ERUNTIME = 0, 1, 2

vp = C.c_void_p


class PackedView(C.Structure):
    _fields_ = [("N", C.c_int), ("K", C.c_int), ("gs", C.c_int), ("G", C.c_int),
                ("symmetric", C.c_int), ("q", vp), ("scales", vp), ("zeros", vp)]


class PackedMxView(C.Structure):
    _fields_ = [("N", C.c_int), ("K", C.c_int), ("B", C.c_int), ("q", vp), ("scales", vp)]


class ActMx8View(C.Structure):
    _fields_ = [("M", C.c_int), ("K", C.c_int), ("B", C.c_int), ("q", vp), ("scales", vp)]


class KVView(C.Structure):
    _fields_ = [("H", C.c_int), ("S", C.c_int), ("D", C.c_int), ("gs", C.c_int), ("G", C.c_int),
                ("symmetric", C.c_int), ("q_k", vp), ("s_k", vp), ("z_k", vp), ("q_v", vp),
                ("s_v", vp), ("z_v", vp)]


class KVF8View(C.Structure):
    _fields_ = [("H", C.c_int), ("S", C.c_int), ("D", C.c_int), ("gs", C.c_int), ("G", C.c_int),
                ("q_k", vp), ("s_k", vp), ("q_v", vp), ("s_v", vp)]


# every symbol include/w4_abi.h declares, with its argument types
SIGNATURES = {
    "w4_last_error": ([], C.c_char_p),
    "w4_dispatch_mma_min_m": ([], C.c_int),
    "w4_dispatch_mma_min_m_for": ([C.c_int, C.c_int], C.c_int),
    "w4_dispatch_mma_min_m_for_gs": ([C.c_int, C.c_int, C.c_int], C.c_int),
    "w4_dispatch_mma_min_m_for_mx": ([C.c_int, C.c_int], C.c_int),
    "w4_dequant": ([C.POINTER(PackedView), vp, vp], C.c_int),
    "w4_gemm_fused": ([C.POINTER(PackedView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_gemm_mma": ([C.POINTER(PackedView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_gemm": ([C.POINTER(PackedView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_dequant_mx": ([C.POINTER(PackedMxView), vp, vp], C.c_int),
    "w4_gemm_fused_mx": ([C.POINTER(PackedMxView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_gemm_mma_mx": ([C.POINTER(PackedMxView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_gemm_mx": ([C.POINTER(PackedMxView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_gemm_fp16": ([vp, vp, vp, C.c_int, C.c_int, C.c_int, vp], C.c_int),
    "w4_attention_w4_flash": ([C.POINTER(KVView), vp, vp, vp, vp, vp], C.c_int),
    "w4_attention_fp16_flash": ([vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp], C.c_int),
    "w4_attention_f8_flash": ([C.POINTER(KVF8View), vp, vp, vp, vp, vp], C.c_int),
    "w4_attention_w4_flash_paged": ([C.POINTER(KVView), vp, C.c_int, C.c_int, vp, vp, vp, vp, vp], C.c_int),
    "w4_dequant_f8": ([vp, vp, vp, C.c_int, C.c_int, C.c_int, vp], C.c_int),
    "w4_attention_w4_flash_gqa": ([C.POINTER(KVView), C.c_int, vp, vp, vp, vp, vp], C.c_int),
    "w4_attention_w4_flash_gqa_noalloc": ([C.POINTER(KVView), C.c_int, vp, vp, vp, vp, vp], C.c_int),
    "w4_attention_fp16_flash_gqa": ([vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp], C.c_int),
    "w4_attention_f8_flash_gqa": ([C.POINTER(KVF8View), C.c_int, C.c_int, vp, vp, vp, vp, vp], C.c_int),
    "w4_attention_w4_flash_paged_batched": ([C.POINTER(KVView), vp, C.c_int, C.c_int, C.c_int, C.c_int,
                                             C.c_int, vp, vp, vp], C.c_int),
    "w4_quantize": ([C.POINTER(PackedView), vp, vp, vp], C.c_int),
    "w4_quantize_mx": ([C.POINTER(PackedMxView), vp, vp, vp], C.c_int),
    "w4_quantize_mx_f16": ([C.POINTER(PackedMxView), vp, vp, vp], C.c_int),
    "w4_gemm_mx_w4a4": ([C.POINTER(PackedMxView), C.POINTER(PackedMxView), vp, vp], C.c_int),
    "w4_quantize_mx8_f16": ([C.POINTER(ActMx8View), vp, vp, vp], C.c_int),
    "w4_gemm_mx_w4a8": ([C.POINTER(PackedMxView), C.POINTER(ActMx8View), vp, vp], C.c_int),
    "w4_quantize_cache": ([C.POINTER(KVView), vp, vp, C.c_int, vp, vp], C.c_int),
    "w4_quantize_cache_f8": ([C.POINTER(KVF8View), vp, vp, C.c_int, vp, vp], C.c_int),
}

_lib = None


def load():
    """dlopen the shipped library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run __graft_entry__.build() first")
        L = C.CDLL(LIB_PATH)
        for name, (args, res) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes, fn.restype = args, res
        _lib = L
    return _lib


def check(rc):
    if rc == W4_OK:
        return
    msg = load().w4_last_error().decode()
    if rc == W4_EINVAL:
        raise ValueError(msg)
    raise RuntimeError(msg)


def packed_view(N, K, gs, G, symmetric, q, scales, zeros=0):
    return PackedView(N, K, gs, G, int(bool(symmetric)), q or None, scales or None, zeros or None)


def packed_mx_view(N, K, B, q, scales):
    return PackedMxView(N, K, B, q or None, scales or None)


def kv_view(H, S, D, gs, G, symmetric, q_k, s_k, z_k, q_v, s_v, z_v):
    return KVView(H, S, D, gs, G, int(bool(symmetric)), q_k or None, s_k or None, z_k or None,
                  q_v or None, s_v or None, z_v or None)


def kv_f8_view(H, S, D, gs, G, q_k, s_k, q_v, s_v):
    return KVF8View(H, S, D, gs, G, q_k or None, s_k or None, q_v or None, s_v or None)


def _n(p):
    return p or None


def dequant(view, w, stream=0):
    check(load().w4_dequant(C.byref(view), _n(w), _n(stream)))


def gemm_fused(view, x, c, M, stream=0, w_out=0):
    check(load().w4_gemm_fused(C.byref(view), _n(x), _n(c), M, _n(stream), _n(w_out)))


def gemm_mma(view, x, c, M, stream=0, w_out=0):
    check(load().w4_gemm_mma(C.byref(view), _n(x), _n(c), M, _n(stream), _n(w_out)))


def gemm(view, x, c, M, stream=0, w_out=0):
    check(load().w4_gemm(C.byref(view), _n(x), _n(c), M, _n(stream), _n(w_out)))


def dequant_mx(view, w, stream=0):
    check(load().w4_dequant_mx(C.byref(view), _n(w), _n(stream)))


def gemm_fused_mx(view, x, c, M, stream=0, w_out=0):
    check(load().w4_gemm_fused_mx(C.byref(view), _n(x), _n(c), M, _n(stream), _n(w_out)))


def gemm_mma_mx(view, x, c, M, stream=0, w_out=0):
    check(load().w4_gemm_mma_mx(C.byref(view), _n(x), _n(c), M, _n(stream), _n(w_out)))


def gemm_mx(view, x, c, M, stream=0, w_out=0):
    check(load().w4_gemm_mx(C.byref(view), _n(x), _n(c), M, _n(stream), _n(w_out)))


def gemm_fp16(w, x, c, M, N, K, stream=0):
    check(load().w4_gemm_fp16(_n(w), _n(x), _n(c), M, N, K, _n(stream)))


def attention_w4_flash(view, q, out, stream=0, k_out=0, v_out=0, group=1):
    check(load().w4_attention_w4_flash_gqa(C.byref(view), group, _n(q), _n(out), _n(stream),
                                           _n(k_out), _n(v_out)))


def attention_w4_flash_noalloc(view, q, out, stream=0, k_out=0, v_out=0, group=1):
    """attention_w4_flash with the split-S partials in the library's built-in device
    array: no device allocation; rejects calls whose partials do not fit."""
    check(load().w4_attention_w4_flash_gqa_noalloc(C.byref(view), group, _n(q), _n(out),
                                                   _n(stream), _n(k_out), _n(v_out)))


def attention_fp16_flash(q, k16, v16, out, H, S, D, stream=0, group=1):
    check(load().w4_attention_fp16_flash_gqa(_n(q), _n(k16), _n(v16), _n(out), H, group, S, D,
                                             _n(stream)))


def attention_f8_flash(view, q, out, stream=0, k_out=0, v_out=0, group=1, scale_mode=0):
    check(load().w4_attention_f8_flash_gqa(C.byref(view), group, scale_mode, _n(q), _n(out),
                                           _n(stream), _n(k_out), _n(v_out)))


def attention_w4_flash_paged(view, bt, page, npages, q, out, stream=0, k_out=0, v_out=0):
    check(load().w4_attention_w4_flash_paged(C.byref(view), _n(bt), page, npages, _n(q), _n(out),
                                             _n(stream), _n(k_out), _n(v_out)))


def attention_w4_flash_paged_batched(view, bt, nseq, bt_stride, page, npages, group, q, out,
                                     stream=0):
    check(load().w4_attention_w4_flash_paged_batched(C.byref(view), _n(bt), nseq, bt_stride, page,
                                                     npages, group, _n(q), _n(out), _n(stream)))


def dequant_f8(q, s, w, S, D, gs, stream=0):
    check(load().w4_dequant_f8(_n(q), _n(s), _n(w), S, D, gs, _n(stream)))


# Device-side quantizers: the view's arrays are outputs; `status` is a device int
# (bit 0 non-finite input, bit 1 scale out of range), cleared by the call.
def quantize(view, w, status, stream=0):
    check(load().w4_quantize(C.byref(view), _n(w), _n(status), _n(stream)))


def quantize_mx(view, w, status, stream=0):
    check(load().w4_quantize_mx(C.byref(view), _n(w), _n(status), _n(stream)))


def quantize_cache(view, k, v, status, src_f16=False, stream=0):
    check(load().w4_quantize_cache(C.byref(view), _n(k), _n(v), int(src_f16), _n(status),
                                   _n(stream)))


def quantize_cache_f8(view, k, v, status, src_f16=False, stream=0):
    check(load().w4_quantize_cache_f8(C.byref(view), _n(k), _n(v), int(src_f16), _n(status),
                                      _n(stream)))


def quantize_mx_f16(view, x, status, stream=0):
    check(load().w4_quantize_mx_f16(C.byref(view), _n(x), _n(status), _n(stream)))


def gemm_mx_w4a4(w_view, x_view, c, stream=0):
    """Both operands packed MXFP4 (x_view.N = M); scaled matrix cores."""
    check(load().w4_gemm_mx_w4a4(C.byref(w_view), C.byref(x_view), _n(c), _n(stream)))


def act_mx8_view(M, K, B, q, scales):
    return ActMx8View(M, K, B, q or None, scales or None)


def quantize_mx8_f16(view, x, status, stream=0):
    check(load().w4_quantize_mx8_f16(C.byref(view), _n(x), _n(status), _n(stream)))


def gemm_mx_w4a8(w_view, x_view, c, stream=0):
    """MXFP4 weights against MXFP8 activations (x_view.M rows); scaled matrix cores."""
    check(load().w4_gemm_mx_w4a8(C.byref(w_view), C.byref(x_view), _n(c), _n(stream)))
