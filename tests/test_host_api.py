"""CPU-only checks of the host layer: the C-ABI library loads and exports every declared symbol,
argument validation returns the documented codes before anything touches a GPU, and the Python
mirror of candle's API keeps candle's sizes and error behaviour."""
import os
import re

import pytest

import oracle
from candle_amd import _lib
from candle_amd.quantized import GgmlDType, check_shape

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    inc = os.path.join(ROOT, "include")
    text = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 15
    for name in names:
        assert hasattr(L, name), f"{name} declared under include/ but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes signatures out of sync with the header"


def test_dtype_sizes_match_reference_and_oracle():
    # mod.rs:386-421 and the size asserts of k_quants.rs:83-190
    want = {GgmlDType.Q4_0: (32, 18), GgmlDType.Q4_1: (32, 20), GgmlDType.Q5_0: (32, 22), GgmlDType.Q5_1: (32, 24),
            GgmlDType.Q8_0: (32, 34), GgmlDType.Q8_1: (32, 36), GgmlDType.Q2K: (256, 84), GgmlDType.Q3K: (256, 110),
            GgmlDType.Q4K: (256, 144), GgmlDType.Q5K: (256, 176), GgmlDType.Q6K: (256, 210), GgmlDType.Q8K: (256, 292),
            GgmlDType.F32: (1, 4), GgmlDType.F16: (1, 2), GgmlDType.BF16: (1, 2)}
    L = _lib.lib()
    for dt, (bs, ts) in want.items():
        assert (dt.block_size(), dt.type_size()) == (bs, ts)
        assert (L.cq_block_size(int(dt)), L.cq_type_size(int(dt))) == (bs, ts)
    for dt in (oracle.Q4_0, oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q8K):
        assert oracle.block_size(dt) == L.cq_block_size(dt) and oracle.type_size(dt) == L.cq_type_size(dt)
    assert GgmlDType.from_u32(12) is GgmlDType.Q4K and GgmlDType.Q6K.to_u32() == 14 and GgmlDType.BF16.to_u32() == 30
    with pytest.raises(ValueError):
        GgmlDType.from_u32(4)
    # BASELINE shapes (bytes of a [14336 x 4096] Q4_K tensor etc.)
    assert L.cq_storage_bytes(12, 14336 * 4096) == 33030144
    assert L.cq_storage_bytes(14, 4096 * 14336) == 48168960
    assert L.cq_storage_bytes(8, 4096 * 4096) == 17825792
    assert L.cq_storage_bytes(12, 100) == -1


def test_check_shape_errors():
    # mod.rs:518-530
    check_shape((4, 256), 256)
    with pytest.raises(ValueError, match="scalar tensor cannot be quantized"):
        check_shape((), 32)
    with pytest.raises(ValueError, match="divisible by block size"):
        check_shape((4, 100), 32)


def test_argument_validation_codes_without_gpu():
    L = _lib.lib()
    Q4K, Q8_1, Q8K = 12, 9, 15
    OK, DTYPE, SHAPE, ALIGN, NULL, WS, RANGE = 0, -1, -2, -3, -4, -5, -6
    # scratch sizes: K-quants: qs + d + bsums sections, each rounded up to 256 bytes
    assert L.cq_act_scratch_bytes(Q4K, 4096, 1) == 4096 + 256 + 512
    assert L.cq_act_scratch_bytes(8, 4096, 2) == 8192 + 2048
    assert L.cq_act_scratch_bytes(Q4K, 100, 1) == -1
    assert L.cq_quantize_act(Q4K, None, 0, None, 4096, 0, None) == OK          # zero rows: nothing to do
    assert L.cq_quantize_act(Q4K, None, 0, None, 4096, 1, None) == NULL
    assert L.cq_quantize_act(Q4K, 16, 0, 256, 4000, 1, None) == SHAPE
    assert L.cq_quantize_act(Q4K, 8, 0, 256, 4096, 1, None) == ALIGN           # x must be 16-byte aligned
    assert L.cq_quantize_act(Q4K, 16, 12, 256, 4096, 1, None) == DTYPE         # activations must be f32/f16/bf16
    assert L.cq_matvec(Q8_1, 16, 256, 16, 0, 256, 4, 1, 4, None) == DTYPE      # Q8_1 is an activation format
    assert L.cq_matvec(Q8K, 16, 256, 16, 0, 256, 4, 1, 4, None) == DTYPE       # Q8K is not a matmul weight type
    assert L.cq_matvec(Q4K, 16, 256, 16, 0, 256, 4, 9, 4, None) == RANGE       # more than CQ_MATVEC_MAX_ROWS
    assert L.cq_matvec(Q4K, 16, 256, 16, 0, 256, 4, 1, 3, None) == SHAPE       # stride_dst < n
    assert L.cq_matvec(Q4K, 8, 256, 16, 0, 256, 4, 1, 4, None) == ALIGN        # Q4_K weights: 16-byte aligned
    assert L.cq_matvec(Q4K, None, 256, 16, 0, 256, 4, 1, 4, None) == NULL
    assert L.cq_matvec(Q4K, None, None, None, 0, 256, 0, 1, 0, None) == OK     # n == 0
    assert L.cq_qmatmul_workspace_bytes(Q4K, 1, 4096, 14336) == 4096 + 256 + 512
    assert L.cq_qmatmul_forward(Q4K, 16, 16, 0, 16, 0, 1, 4096, 8, 256, 10, None) == WS
    assert L.cq_indexed_moe_workspace_bytes(Q4K, 8, 16, 256, 2, 4, 3) == -1    # input_dim1 must be topk or 1
    assert L.cq_indexed_moe_workspace_bytes(6, 8, 16, 256, 2, 4, 4) == -1      # Q5_0 is a matmul weight format, not an expert format
    assert L.cq_moe_gemm_gguf(6, 16, 16, 4, 4, None, 4, 8, 4, 8, 16, 256, 0, 256, 1 << 20, None) == DTYPE
    assert L.cq_moe_gemm_workspace_bytes(Q4K, 8, 4, 6, 16, 256, 0) == -1       # size_m not a multiple of topk
    assert L.cq_moe_gemm_gguf(Q4K, 16, 16, 4, 4, None, 4, 8, 4, 8, 16, 256, 0, 256, 0, None) == WS
    assert _lib.status_string(SHAPE).startswith("invalid shape")
    assert _lib.status_string(OK) == "ok"


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.lib()


# ---------------------------------------------------------------------------- the workspace guard (no GPU: allocation and stream stubbed)
class _CpuWorkspace:
    """candle_amd.quantized._workspace with the three GPU-facing hooks replaced: CPU allocations, a settable stream key and capture flag."""

    def __new__(cls, stream, nbytes, capturing=False):
        import torch
        from candle_amd import quantized as q

        class G(q._workspace):
            def _key(self):
                return (0, stream)

            def _alloc(self, n):
                return torch.empty(n, dtype=torch.uint8)

            def _capturing(self):
                return capturing

        return G(torch.device("cpu"), nbytes)


def test_workspace_guard_holds_the_lock_until_the_block_ends():
    import threading
    import time
    events = []
    inside = threading.Event()
    release = threading.Event()

    def first():
        with _CpuWorkspace(stream=101, nbytes=1000) as ws:
            events.append(("first in", ws.data_ptr()))
            inside.set()
            release.wait(5)
            time.sleep(0.05)
            events.append(("first out", ws.data_ptr()))

    def second(stream, tag):
        inside.wait(5)
        with _CpuWorkspace(stream=stream, nbytes=5 << 20) as ws:      # larger: would replace the first thread's buffer
            events.append((tag, ws.data_ptr()))

    t1 = threading.Thread(target=first)
    t2 = threading.Thread(target=second, args=(101, "same stream"))
    t3 = threading.Thread(target=second, args=(202, "other stream"))
    t1.start(); t2.start(); t3.start()
    t3.join(5)                     # another stream's buffer is independent: not blocked by the first thread
    assert not t3.is_alive() and [e[0] for e in events] == ["first in", "other stream"]
    time.sleep(0.1)
    assert t2.is_alive()           # the same stream's second call waits for the first call's enqueue to end
    release.set()
    t1.join(5); t2.join(5)
    assert [e[0] for e in events] == ["first in", "other stream", "first out", "same stream"]
    ptrs = dict(events)
    assert ptrs["same stream"] != ptrs["first in"] and ptrs["other stream"] != ptrs["first in"]


def test_workspace_guard_keeps_outgrown_buffers_and_refuses_to_grow_under_capture():
    from candle_amd import quantized as q
    with _CpuWorkspace(stream=303, nbytes=10) as a:
        pa, na = a.data_ptr(), a.numel()
    assert na >= 1 << 20
    with _CpuWorkspace(stream=303, nbytes=100) as b:
        assert b.data_ptr() == pa                     # no growth: the same buffer
    with _CpuWorkspace(stream=303, nbytes=na + 1) as c:
        assert c.numel() >= 2 * na                    # geometric growth bounds what the retired buffers add up to
    slot = q._workspaces[(0, 303)]
    assert [t.data_ptr() for t in slot.retired] == [pa]      # still alive: a captured graph may replay into it
    with pytest.raises(RuntimeError, match="captured"):
        with _CpuWorkspace(stream=303, nbytes=c.numel() + 1, capturing=True):
            pass
    assert not slot.lock.locked()                     # a refused call leaves the stream's lock free
    with _CpuWorkspace(stream=303, nbytes=1000, capturing=True) as d:
        assert d.data_ptr() == c.data_ptr()           # a call that fits may be captured


def test_rust_ffi_declarations_match_the_headers():
    """rust/candle-hip-quant/src/ffi.rs is generated from the two headers; the generator's check mode fails when it is stale.
    Every ffi:: call of the crate's lib.rs names a declared entry point."""
    import subprocess
    import sys
    crate = os.path.join(ROOT, "rust", "candle-hip-quant")
    r = subprocess.run([sys.executable, os.path.join(crate, "gen_ffi.py"), "--check"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    declared = set(re.findall(r"pub fn (cq_\w+)", open(os.path.join(crate, "src", "ffi.rs")).read()))
    assert declared == set(_lib.SIGNATURES)
    used = set(re.findall(r"ffi::(cq_\w+)", open(os.path.join(crate, "src", "lib.rs")).read()))
    assert used and used <= declared
