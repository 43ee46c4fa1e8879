"""Builds libw4amd.so (the gfx950 kernels + C ABI) in-tree with hipcc.

    python w4a16-dequant-gemm_amd/build.py            # build if sources changed
    python w4a16-dequant-gemm_amd/build.py --force
"""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "lib", "libw4amd.so")
BENCH_LIB = os.path.join(PKG, "lib", "libw4bench.so")
SOURCES = ["abi.hip", "dequant.hip", "gemm_simt.hip", "gemm_mfma.hip", "flash.hip", "flash_mfma.hip", "quantize.hip", "gemm_mxnative.hip", "gemm_tile_dma.hip", "gemm_tile256.hip", "gemm_decode_resident.hip", "gemm_decode_general.hip", "gemm_decode_longk.hip",
           "baseline.hip"]
HEADERS = ["dq.cuh", "kernels.h", "simt_rows4.cuh", "bench_kernels.hip", os.path.join("..", "..", "include", "w4_abi.h")]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 VALU forms stay off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the leading kernel arguments arrive in SGPRs with the wave instead of through a
    # scalar load from the kernarg segment: 0.25 us off every launch at decode sizes
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-function",
    # the direct-to-LDS loads name M0 in their clobber list on purpose
    "-Wno-inline-asm",
]

# Per-file additions.  The flash-decode kernel rescales its accumulators with
# vector-ALU multiplies between matrix instructions: with the accumulators in
# the AGPR half of the register file the compiler copies all 36 of them across
# every loop edge, so keep its MFMA results in ordinary VGPRs.
EXTRA_FLAGS = {"flash_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _stale():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, f) for f in SOURCES + HEADERS] + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    if not force and not _stale():
        return LIB
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    objs, procs = [], []
    os.makedirs(os.path.join(PKG, "lib", "obj"), exist_ok=True)
    hdr_t = max(os.path.getmtime(os.path.join(CSRC, h)) for h in HEADERS if not h.endswith(".hip"))
    hdr_t = max(hdr_t, os.path.getmtime(os.path.abspath(__file__)))
    for src in SOURCES:
        obj = os.path.join(PKG, "lib", "obj", src.replace(".hip", ".o"))
        objs.append(obj)
        if (not force and os.path.exists(obj)
                and os.path.getmtime(obj) > max(hdr_t, os.path.getmtime(os.path.join(CSRC, src)))):
            continue  # this object is newer than its source and every shared header
        cmd = ["hipcc", *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stderr=subprocess.PIPE, text=True)))
    for src, p in procs:
        _, err = p.communicate()
        err = "\n".join(l for l in err.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs,
                           "-lhipblaslt"])
    # bandwidth yardsticks used only by bench.py
    bench_src = os.path.join(CSRC, "bench_kernels.hip")
    if (force or not os.path.exists(BENCH_LIB)
            or os.path.getmtime(BENCH_LIB) < max(hdr_t, os.path.getmtime(bench_src))):
        subprocess.check_call(["hipcc", *[f for f in FLAGS if not f.startswith("-W")], "-shared",
                               bench_src, "-o", BENCH_LIB], stderr=subprocess.DEVNULL)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
