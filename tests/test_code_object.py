"""CPU-only checks of the gfx950 code objects inside the built library: the kernels of the single-token decode step
must not use a private segment.  A kernel with one starts 1.5-2 us later per launch on this hardware (the segment is
set up before the first wave runs), which is a fifth of a 7 us matvec; the compiler creates one silently for register
spills and for small arrays it decides to index in memory (a select chain over a lane-dependent index did).
Nor may the streaming matvec access memory with flat instructions: the compiler cannot wait for a flat load by count,
so the wait for the activation row also waits for every weight copy requested before it (pointers rebuilt from the
integer argument block were flat until they were marked global)."""
import os
import re
import shutil
import subprocess

import pytest

from candle_amd import _lib

LLVM = "/opt/rocm/llvm/bin"
BUNDLER = os.path.join(LLVM, "clang-offload-bundler")
READELF = os.path.join(LLVM, "llvm-readelf")
MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


OBJDUMP = os.path.join(LLVM, "llvm-objdump")


def kernel_private_segments(so_path, tmp, objects=None):
    """{kernel symbol: private_segment_fixed_size} over every gfx950 code object bundled into the library; `objects`, when
    given, receives {kernel symbol: path of the code object that holds it}."""
    fat = os.path.join(tmp, "fat.bin")
    subprocess.run(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", so_path, fat], check=True)
    data = open(fat, "rb").read()
    starts = [m.start() for m in re.finditer(re.escape(MAGIC), data)]
    out = {}
    for i, a in enumerate(starts):
        b = starts[i + 1] if i + 1 < len(starts) else len(data)
        piece, co = os.path.join(tmp, f"bundle{i}.bin"), os.path.join(tmp, f"dev{i}.co")
        open(piece, "wb").write(data[a:b])
        r = subprocess.run([BUNDLER, "--unbundle", "--type=o", f"--input={piece}", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950",
                            f"--output={co}"], capture_output=True, text=True)
        if r.returncode or not os.path.exists(co) or os.path.getsize(co) == 0:
            continue
        notes = subprocess.run([READELF, "--notes", co], capture_output=True, text=True, check=True).stdout
        size = None
        for line in notes.splitlines():
            m = re.match(r"\s*\.private_segment_fixed_size:\s*(\d+)", line)
            if m:
                size = int(m.group(1))
            m = re.match(r"\s*\.symbol:\s*(\S+)", line)      # the last key of a kernel's record
            if m and size is not None:
                out[m.group(1)] = size
                if objects is not None:
                    objects[m.group(1)] = co
                size = None
    return out


@pytest.mark.skipif(not (os.path.exists(BUNDLER) and os.path.exists(READELF) and shutil.which("objcopy")),
                    reason="needs objcopy and ROCm's llvm tools")
def test_decode_step_kernels_have_no_private_segment(tmp_path):
    segs = kernel_private_segments(_lib.LIB_PATH, str(tmp_path))
    assert len(segs) > 500, "kernel metadata not found in the library"

    def hot(sym):
        # one-row and two-row streaming matvecs (eight waves), the two-tensor launch with eight waves, and the
        # single-token attention kernel on 64-key splits
        if "10qms_kernel" in sym or "13qms_kernel_dw" in sym or "16qms_rows2_kernel" in sym:
            return True
        if re.search(r"11qms2_kernelILi\d+ELi\d+ELi8E", sym):
            return True
        return bool(re.search(r"18attn_decode_kernelILi\d+ELi\d+ELi8ELi64E", sym))

    hot_syms = [s for s in segs if hot(s)]
    assert len(hot_syms) > 50, hot_syms[:5]
    bad = {s: v for s, v in segs.items() if hot(s) and v}
    assert not bad, f"decode kernels with a private segment: {bad}"


@pytest.mark.skipif(not (os.path.exists(BUNDLER) and os.path.exists(READELF) and os.path.exists(OBJDUMP) and shutil.which("objcopy")),
                    reason="needs objcopy and ROCm's llvm tools")
def test_streaming_matvec_has_no_flat_memory_instructions(tmp_path):
    objects = {}
    kernel_private_segments(_lib.LIB_PATH, str(tmp_path), objects)
    # the one-row streaming kernels of the 8B-shape decode step: Q4_K rows of 4096 (two spans per wave) and Q6_K rows of
    # 14336 (seven), every prologue / epilogue pair
    syms = [s for s in objects if re.search(r"13qms_kernel_dwILi12ELi2ELi16E|13qms_kernel_dwILi14ELi7ELi64E", s)]
    assert len(syms) >= 8, syms
    co = objects[syms[0]]
    assert all(objects[s] == co for s in syms)
    names = ",".join(s[:-3] if s.endswith(".kd") else s for s in syms)
    text = subprocess.run([OBJDUMP, "-d", f"--disassemble-symbols={names}", co], capture_output=True, text=True, check=True).stdout
    assert text.count("s_endpgm") >= len(syms), "kernels not found in the disassembly"
    flat = [line.strip() for line in text.splitlines() if re.search(r"\bflat_(load|store|atomic)", line)]
    assert not flat, flat[:5]
