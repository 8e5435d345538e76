"""cq_qmatmul_forward_static (the entry point that allocates nothing) against cq_qmatmul_forward, through the C ABI.

Both entry points run the same kernels, so the outputs must be equal bit for bit.  Every case makes two calls in a row
on the shared static workspace, the second with a smaller input, each checked against a call of the existing entry
point with a caller-owned workspace; the row counts are chosen so that the workspace is really used (quantized
activation scratch of the 3..8-row matvec, K-split planes and the f32 staging of the matrix-core path).
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from candle_amd import _lib
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

CQ = {"q4k": (12, oracle.Q4K), "q6k": (14, oracle.Q6K), "q8_0": (8, oracle.Q8_0)}
TORCH_DT = {0: torch.float32, 1: torch.float16}


def _vp(t):
    return ctypes.c_void_p(t.data_ptr())


def _forward_pair(L, code, w_dev, x_dev, m, k, n, dst_code):
    """(static result, reference-entry-point result) for one call shape, both synchronized."""
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    got = torch.full((m, n), float("nan"), dtype=TORCH_DT[dst_code], device="cuda:0")
    want = torch.full((m, n), float("nan"), dtype=TORCH_DT[dst_code], device="cuda:0")
    _lib.check("cq_qmatmul_forward_static", L.cq_qmatmul_forward_static(code, _vp(w_dev), _vp(x_dev), 0, _vp(got), dst_code, m, k, n, stream))
    nbytes = L.cq_qmatmul_workspace_bytes(code, m, k, n)
    assert 0 < nbytes <= L.cq_static_workspace_bytes()
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(code, _vp(w_dev), _vp(x_dev), 0, _vp(want), dst_code, m, k, n, _vp(ws), nbytes, stream))
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


@pytest.mark.parametrize("fmt,n,k,m1,m2,dst_code", [
    ("q4k", 512, 1024, 8, 3, 0),        # activation scratch + matvec, then fewer rows
    ("q4k", 384, 2048, 96, 24, 0),      # matrix cores with K-split planes, then a smaller call
    ("q6k", 256, 1024, 40, 12, 1),      # f16 output: f32 staging in the workspace
    ("q8_0", 320, 512, 64, 5, 0),       # matrix cores, then the matvec path on the same memory
])
def test_static_workspace_equals_caller_workspace(fmt, n, k, m1, m2, dst_code):
    print(f"case {fmt} n={n} k={k} m={m1},{m2} dst={dst_code}", flush=True)
    L = _lib.lib()
    code, odt = CQ[fmt]
    w = normal(11, (n, k), 0.02)
    blocks = oracle.from_float(odt, w.reshape(-1))
    w_dev = torch.from_numpy(np.frombuffer(blocks, dtype=np.uint8).copy()).to("cuda:0")
    for seed, m in ((1, m1), (2, m2)):
        x = normal(seed, (m, k))
        x_dev = torch.from_numpy(x).to("cuda:0")
        got, want = _forward_pair(L, code, w_dev, x_dev, m, k, n, dst_code)
        assert not np.isnan(got).any()
        assert np.array_equal(got.view(np.uint16 if dst_code else np.uint32), want.view(np.uint16 if dst_code else np.uint32))
        ref = oracle.matmul(odt, x, blocks, n)
        assert rel_l2(got.astype(np.float64), ref) <= (1e-3 if dst_code == 0 else 2e-3)


def test_static_workspace_rejects_oversized_calls():
    L = _lib.lib()
    cap = L.cq_static_workspace_bytes()
    assert cap == 32 << 20
    m, k, n = 4096, 14336, 4096
    assert L.cq_qmatmul_workspace_bytes(12, m, k, n) > cap
    # the size check comes before any pointer is looked at: nothing is enqueued
    dummy = torch.zeros(64, dtype=torch.uint8, device="cuda:0")
    rc = L.cq_qmatmul_forward_static(12, _vp(dummy), _vp(dummy), 0, _vp(dummy), 0, m, k, n, None)
    assert rc == -6 and "exceeds" in _lib.status_string(rc)


def test_static_workspace_under_graph_capture():
    """The entry point is meant for callers under stream capture: after cq_static_workspace_bytes() has been called eagerly on
    the device (the one-time address lookup), a captured call replays bit-equal to the eager result, several times, with eager
    work between the replays."""
    L = _lib.lib()
    code, odt = CQ["q4k"]
    n, k, m = 512, 1024, 5
    blocks = oracle.from_float(odt, normal(21, (n, k), 0.02).reshape(-1))
    w_dev = torch.from_numpy(np.frombuffer(blocks, dtype=np.uint8).copy()).to("cuda:0")
    x_dev = torch.from_numpy(normal(22, (m, k))).to("cuda:0")
    assert L.cq_static_workspace_bytes() == 32 << 20            # eager, before any capture
    eager, want = _forward_pair(L, code, w_dev, x_dev, m, k, n, 0)
    assert np.array_equal(eager.view(np.uint32), want.view(np.uint32))
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check("cq_qmatmul_forward_static", L.cq_qmatmul_forward_static(code, _vp(w_dev), _vp(x_dev), 0, _vp(out), 0, m, k, n, s))
    torch.cuda.synchronize()
    for rep in range(3):
        out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32)), rep
        # eager work on the shared workspace between the replays
        other, _ = _forward_pair(L, code, w_dev, torch.from_numpy(normal(30 + rep, (m, k))).to("cuda:0"), m, k, n, 0)
        assert not np.isnan(other).any()
