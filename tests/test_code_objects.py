"""What the compiler says about every kernel of the built library (the metadata notes of
its code objects; nothing is disassembled).

No kernel may use scratch memory: an instantiation that spills registers runs several
times slower than the next smaller one that fits (a scale pick that the compiler put in
scratch cost 1.8 us of a 10.5 us call once), so the launchers cap what they ask for at
what fits and do not compile the rest -- this test is what keeps the two in step.  The
vector GEMM kernel that writes registers with hand-placed loads and waits must not have
any of them parked in the AGPR half of the register file either: the compiler does not
know when such a register lands, and a copy made before the wait copies stale bits."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "w4a16-dequant-gemm_amd"))
import codeobj  # noqa: E402

LIB = codeobj.default_lib()


@pytest.fixture(scope="module")
def kernels():
    assert os.path.exists(LIB), "libw4amd.so is not built (python __graft_entry__.py)"
    ks = codeobj.kernels(LIB)
    assert len(ks) > 100, "the code objects of the library were not found"
    return ks


def _demangle(names):
    try:
        out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True).stdout
        return out.split("\n")[:len(names)]
    except OSError:
        return names


def test_every_kernel_is_gfx950(kernels):
    assert {k["target"].split("-")[-1] for k in kernels} == {"gfx950"}


def test_no_kernel_uses_scratch_memory(kernels):
    # (.vgpr_spill_count also counts registers the compiler parks in AGPRs, which costs a
    # copy and no memory traffic; what is policed here is the per-lane scratch segment)
    bad = [k for k in kernels if k.get(".private_segment_fixed_size", 0)]
    names = _demangle([k[".name"] for k in bad])
    assert not bad, "kernels with scratch memory:\n" + "\n".join(
        "%5d B, %d spilled VGPRs: %s" % (k[".private_segment_fixed_size"], k.get(".vgpr_spill_count", 0), n)
        for k, n in zip(bad, names))


def test_asm_loaded_registers_are_never_parked(kernels):
    rows4 = [k for k in kernels if "simt_rows4_kernel" in k[".name"]]
    assert rows4, "the four-rows vector kernel is missing from the library"
    bad = [k for k in rows4 if k.get(".agpr_count", 0)]
    assert not bad, "\n".join(_demangle([k[".name"] for k in bad]))


def test_wave64_and_workgroup_sizes(kernels):
    for k in kernels:
        assert k[".wavefront_size"] == 64
        assert k[".max_flat_workgroup_size"] <= 1024
        assert k.get(".group_segment_fixed_size", 0) <= 160 * 1024
