"""Builds libcandle_hip_quant.so (gfx950) in-tree with hipcc.

    python -m candle_amd.build            # compile what changed, link
    python -m candle_amd.build --force    # recompile everything

hipcc cross-compiles for gfx950 without a GPU present.  Flags:
  -ffp-contract=off   the quantizers and the dequantizer must round exactly like the scalar CPU code
                      (kernels that want an FMA call fmaf explicitly);
  -packed-fp32-ops    disabled: hipcc must not form packed-f32 instructions from scalar float code;
  -amdgpu-kernarg-preload-count=14   the first fourteen dwords of scalar kernel arguments are placed in SGPRs at wave
                      launch (kernels keep an entry that loads them for firmware without the feature).
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "libcandle_hip_quant.so")

LIB_BENCH = os.path.join(HERE, "libcq_bench.so")

SOURCES = ["cq_api.hip", "cq_dequant.hip", "cq_actquant.hip", "cq_matvec.hip", "cq_matmul.hip", "cq_moe.hip", "cq_quantize.hip", "cq_nn.hip", "cq_layer.hip", "cq_matvec_batch.hip"]
# the benchmark's plain-read yardstick kernel: a library of its own, not part of the C ABI
BENCH_SOURCES = ["cq_bench.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def _headers_mtime() -> float:
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    inc = os.path.join(os.path.dirname(HERE), "include")
    hs += [os.path.join(inc, f) for f in os.listdir(inc) if f.endswith(".h")]
    return max(os.path.getmtime(h) for h in hs)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), _headers_mtime()):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES + BENCH_SOURCES))
    for lib, lobjs in ((LIB, objs[:len(SOURCES)]), (LIB_BENCH, objs[len(SOURCES):])):
        if force or not os.path.exists(lib) or any(os.path.getmtime(o) > os.path.getmtime(lib) for o in lobjs):
            r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *lobjs], capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
