"""CPU-only checks of the gfx950 code objects inside the built library: the kernels of the single-token decode step
must not use a private segment.  A kernel with one starts 1.5-2 us later per launch on this hardware (the segment is
set up before the first wave runs), which is a fifth of a 7 us matvec; the compiler creates one silently for register
spills and for small arrays it decides to index in memory (a select chain over a lane-dependent index did)."""
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


def kernel_private_segments(so_path, tmp):
    """{kernel symbol: private_segment_fixed_size} over every gfx950 code object bundled into the library."""
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
