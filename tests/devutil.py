"""torch-side plumbing for the GPU tests: device buffers and views for the C ABI.
torch only allocates and copies; every computation under test runs in
libw4amd.so."""
import numpy as np
import torch

import w4amd

DEV = "cuda:0"


def to_dev(a):
    """numpy array -> device tensor with the same bytes (uint16/uint32 as int16/int32)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(DEV)
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def halves(n, fill=None):
    t = torch.empty(int(n), dtype=torch.int16, device=DEV)
    if fill is not None:
        t.fill_(fill)
    return t


def bits(t):
    """device int16 tensor -> numpy uint16 bit patterns."""
    torch.cuda.synchronize()
    return t.cpu().numpy().view(np.uint16)


def f64(t):
    return bits(t).view(np.float16).astype(np.float64)


# An output computed with the w_out hook and one computed without it are both GEMM
# results: each within 1e-3 of the FP64 oracle, and within 2e-3 of each other (the
# bound the reference puts between its fused and its two-pass outputs,
# tests/test_gpu.cu:184-193).  Only the hook's own bytes are bit-exact by contract, so
# an unhooked kernel is free to apply scales and zero-points per group in FP32.  The
# unhooked result is held to half the oracle tolerance so that margin remains.
CROSS_TOL = 2e-3
UNHOOKED_TOL = 5e-4


def cross_gate(hooked, plain, ref, what=""):
    """hooked / plain: uint16 bit patterns of the two outputs; ref: FP64 oracle."""
    h = hooked.view(np.float16).astype(np.float64).ravel()
    u = plain.view(np.float16).astype(np.float64).ravel()
    r = np.asarray(ref, dtype=np.float64).ravel()
    den = float(np.sqrt(np.sum(r * r))) or 1.0
    rel_u = float(np.sqrt(np.sum((u - r) ** 2))) / den
    rel_x = float(np.sqrt(np.sum((u - h) ** 2))) / den
    assert rel_u <= UNHOOKED_TOL, (what, "unhooked vs oracle", rel_u)
    assert rel_x <= CROSS_TOL, (what, "unhooked vs hooked", rel_x)


def ptr(t):
    return 0 if t is None else t.data_ptr()


class DevPacked:
    """Device copy of an oracle PackedW plus its C-ABI view."""

    def __init__(self, p):
        c = w4amd.capi()
        self.q, self.s = to_dev(p.q), to_dev(p.scales)
        self.z = None if p.zeros is None else to_dev(p.zeros)
        self.view = c.packed_view(p.N, p.K, p.gs, p.G, p.symmetric, ptr(self.q), ptr(self.s), ptr(self.z))


class DevPackedMx:
    def __init__(self, p):
        c = w4amd.capi()
        self.q, self.s = to_dev(p.q), to_dev(p.scales)
        self.view = c.packed_mx_view(p.N, p.K, p.B, ptr(self.q), ptr(self.s))


class DevKV:
    def __init__(self, c4):
        c = w4amd.capi()
        self.t = [to_dev(c4.q_k), to_dev(c4.s_k), None if c4.z_k is None else to_dev(c4.z_k),
                  to_dev(c4.q_v), to_dev(c4.s_v), None if c4.z_v is None else to_dev(c4.z_v)]
        self.view = c.kv_view(c4.H, c4.S, c4.D, c4.gs, c4.G, c4.symmetric, *[ptr(t) for t in self.t])


class DevKVF8:
    def __init__(self, c8, s_k=None, s_v=None):
        c = w4amd.capi()
        self.t = [to_dev(c8.q_k), to_dev(c8.s_k if s_k is None else s_k), to_dev(c8.q_v),
                  to_dev(c8.s_v if s_v is None else s_v)]
        self.view = c.kv_f8_view(c8.H, c8.S, c8.D, c8.gs, c8.G, *[ptr(t) for t in self.t])
