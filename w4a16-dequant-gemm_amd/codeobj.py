"""Kernel metadata of a built library, read from the code objects inside it.

hipcc puts one clang offload bundle per translation unit into the `.hip_fatbin`
section of the shared library; each bundle carries the gfx950 ELF, whose NT_AMDGPU_METADATA
note is a msgpack map with one record per kernel (register counts, spill counts, the
per-lane scratch size `.private_segment_fixed_size`, LDS size).  Nothing is disassembled:
this reads the notes the compiler wrote.

    python w4a16-dequant-gemm_amd/codeobj.py [lib.so]      # table of kernels that use scratch / AGPR copies
"""
import os
import struct
import sys

_MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def _elf_sections(buf):
    """(name, type, offset, size) of every section of an ELF64 little-endian image."""
    assert buf[:4] == b"\x7fELF" and buf[4] == 2 and buf[5] == 1, "not an ELF64 LE image"
    shoff, = struct.unpack_from("<Q", buf, 0x28)
    shentsize, shnum, shstrndx = struct.unpack_from("<HHH", buf, 0x3A)
    secs = []
    for i in range(shnum):
        name, typ, _flags, _addr, off, size = struct.unpack_from("<IIQQQQ", buf, shoff + i * shentsize)
        secs.append([name, typ, off, size])
    stroff, strsize = secs[shstrndx][2], secs[shstrndx][3]
    strtab = buf[stroff:stroff + strsize]
    out = []
    for name, typ, off, size in secs:
        end = strtab.index(b"\0", name)
        out.append((strtab[name:end].decode(), typ, off, size))
    return out


def _notes(buf, off, size):
    p, end = off, off + size
    while p + 12 <= end:
        namesz, descsz, typ = struct.unpack_from("<III", buf, p)
        p += 12
        name = buf[p:p + namesz].rstrip(b"\0")
        p += (namesz + 3) & ~3
        desc = buf[p:p + descsz]
        p += (descsz + 3) & ~3
        yield name, typ, desc


def device_images(lib_path):
    """The gfx950 ELF images bundled into the library, one per translation unit."""
    with open(lib_path, "rb") as f:
        so = f.read()
    fat = [s for s in _elf_sections(so) if s[0] == ".hip_fatbin"]
    assert fat, "%s has no .hip_fatbin section" % lib_path
    _, _, off, size = fat[0]
    blob = so[off:off + size]
    images, at = [], blob.find(_MAGIC)
    while at >= 0:
        n, = struct.unpack_from("<Q", blob, at + len(_MAGIC))
        p = at + len(_MAGIC) + 8
        for _ in range(n):
            eoff, esize, tlen = struct.unpack_from("<QQQ", blob, p)
            triple = blob[p + 24:p + 24 + tlen].decode()
            p += 24 + tlen
            if "amdgcn" in triple and esize:
                images.append((triple, blob[at + eoff:at + eoff + esize]))
        at = blob.find(_MAGIC, at + len(_MAGIC))
    return images


def kernels(lib_path):
    """One dict per kernel of the library: the compiler's metadata record."""
    import msgpack
    out = []
    for triple, img in device_images(lib_path):
        for name, typ, off, size in _elf_sections(img):
            if typ != 7:  # SHT_NOTE
                continue
            for nname, ntyp, desc in _notes(img, off, size):
                if nname == b"AMDGPU" and ntyp == 32:
                    meta = msgpack.unpackb(desc, raw=False, strict_map_key=False)
                    for k in meta.get("amdhsa.kernels", []):
                        k = dict(k)
                        k["target"] = triple
                        out.append(k)
    return out


def default_lib():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libw4amd.so")


if __name__ == "__main__":
    import subprocess
    ks = kernels(sys.argv[1] if len(sys.argv) > 1 else default_lib())
    names = [k[".name"] for k in ks]
    try:
        dem = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True).stdout.split("\n")
    except OSError:
        dem = names
    print("%d kernels" % len(ks))
    for k, d in zip(ks, dem):
        if k.get(".private_segment_fixed_size", 0) or k.get(".vgpr_spill_count", 0) or k.get(".sgpr_spill_count", 0):
            print("scratch %5d  vgpr %3d agpr %3d spills v%d s%d  %s" % (
                k.get(".private_segment_fixed_size", 0), k.get(".vgpr_count", 0), k.get(".agpr_count", 0),
                k.get(".vgpr_spill_count", 0), k.get(".sgpr_spill_count", 0), d[:150]))
