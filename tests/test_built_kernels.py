"""What the compiler made of the kernels, read from the metadata of the built libraries (the note that every
code object carries: registers, LDS and stack bytes a kernel).  A kernel whose lambda was left as a function of
its own calls it through the stack, and everything the lambda captures then lives in scratch memory: the float
instances of the fused decode attention once took 75 us a launch that way instead of 13, with every test green.
So: no kernel may need a stack whose size is only known at run time (that is what a call leaves), and beyond a
few words (a small object the compiler keeps in memory: the products' kernels have up to 48 bytes) only the
kernels listed here may use scratch memory (true register spills, known and measured)."""

from __future__ import annotations

import pathlib
import struct

import pytest

LIB_DIR = pathlib.Path(__file__).resolve().parent.parent / "lockstep_amd" / "_lib"
# kernels that are known to spill (256 registers a lane are not enough for them), by a part of their name
SMALL = 64                                              # bytes a lane that need no entry here
MAY_SPILL = ("attention_wide_kernelIfLi8E",)          # float, row blocks of 128: 288 bytes a lane at head size 128
MAY_SPILL_AT_HEAD_256 = ("attention_",)               # every float instance at a head size of 256, and some bfloat16


def code_object_notes(blob: bytes):
    """The AMDGPU metadata notes (msgpack) of every code object bundled in a library."""
    import msgpack

    at = 0
    while True:
        at = blob.find(b"\x7fELF", at)
        if at < 0:
            return
        # a 64-bit little-endian ELF: section headers give the notes
        shoff, = struct.unpack_from("<Q", blob, at + 0x28)
        shentsize, shnum = struct.unpack_from("<HH", blob, at + 0x3A)
        machine, = struct.unpack_from("<H", blob, at + 0x12)
        if machine == 224 and shoff and shnum:                 # EM_AMDGPU
            for i in range(shnum):
                base = at + shoff + i * shentsize
                if base + 64 > len(blob):
                    break
                sh_type, = struct.unpack_from("<I", blob, base + 4)
                offset, size = struct.unpack_from("<QQ", blob, base + 0x18)
                if sh_type != 7:                               # SHT_NOTE
                    continue
                pos, end = at + offset, at + offset + size
                while pos + 12 <= end:
                    namesz, descsz, ntype = struct.unpack_from("<III", blob, pos)
                    name = blob[pos + 12: pos + 12 + namesz]
                    desc_at = pos + 12 + (namesz + 3) // 4 * 4
                    if name.startswith(b"AMDGPU") and ntype == 32:
                        yield msgpack.unpackb(blob[desc_at: desc_at + descsz], raw=False, strict_map_key=False)
                    pos = desc_at + (descsz + 3) // 4 * 4
        at += 4


def kernels_of(path: pathlib.Path):
    for note in code_object_notes(path.read_bytes()):
        for kernel in note.get("amdhsa.kernels", []):
            yield kernel


LIBS = sorted(LIB_DIR.glob("liblockstep_*.so")) if LIB_DIR.is_dir() else []


@pytest.mark.skipif(not LIBS, reason="no library has been built in the tree")
def test_no_kernel_calls_a_function_and_only_known_ones_spill():
    seen = 0
    for lib in LIBS:
        head_256 = "attention256" in lib.name
        for kernel in kernels_of(lib):
            seen += 1
            name = kernel[".name"]
            assert not kernel.get(".uses_dynamic_stack", False), f"{lib.name}: {name} calls a function"
            scratch = kernel.get(".private_segment_fixed_size", 0)
            allowed = MAY_SPILL + (MAY_SPILL_AT_HEAD_256 if head_256 else ())
            if scratch > SMALL and not any(part in name for part in allowed):
                pytest.fail(f"{lib.name}: {name} uses {scratch} bytes of scratch memory a lane")
    assert seen > 100, "the libraries' metadata was not found"
