"""Weights that end exactly where their buffer's payload ends: QMatMul::forward through the C ABI must depend on the
bytes of [w, w + size) only.

Q4_0 / Q5_0 / Q8_0 blocks are 18 / 22 / 34 bytes, so every other block starts on an odd halfword and a tensor with an
odd block count has a size of 2 (mod 4).  The tensor is placed inside a larger device buffer at a base that is 0 or 2
(mod 4), between two canary regions, and the same call is made with the canaries holding 0x00 and then 0xFF bytes (as
f16 scale bits 0xFFFF is a NaN, as quants it is the largest value): the outputs must be equal bit for bit, equal to the
result with the tensor in a buffer of its own, and within the matmul bar of the CPU oracle.  Row counts cover the
single-row kernel, the 2..8-row kernel, its 8-rows-per-pass loop and the matrix-core kernels.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from candle_amd import _lib
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

FORMATS = {"q4_0": (2, oracle.Q4_0, 18), "q4_1": (3, oracle.Q4_1, 20), "q5_0": (6, oracle.Q5_0, 22), "q5_1": (7, oracle.Q5_1, 24),
           "q8_0": (8, oracle.Q8_0, 34)}
CANARY = 4096


def _forward(L, code, w_ptr, x_dev, m, k, n):
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    nbytes = L.cq_qmatmul_workspace_bytes(code, m, k, n)
    ws = torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device="cuda:0")
    _lib.check("cq_qmatmul_forward", L.cq_qmatmul_forward(code, ctypes.c_void_p(w_ptr), ctypes.c_void_p(x_dev.data_ptr()), 0,
                                                            ctypes.c_void_p(out.data_ptr()), 0, m, k, n, ctypes.c_void_p(ws.data_ptr()), nbytes, stream))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("fmt", list(FORMATS))
@pytest.mark.parametrize("base_mod4", [0, 2])
@pytest.mark.parametrize("n,k", [(67, 32 * 9), (1, 32), (129, 32 * 65)])
def test_result_depends_on_tensor_bytes_only(fmt, base_mod4, n, k):
    print(f"case {fmt} base%4={base_mod4} n={n} k={k}", flush=True)
    L = _lib.lib()
    code, odt, bb = FORMATS[fmt]
    blocks = oracle.from_float(odt, normal(5, (n, k), 0.02).reshape(-1))
    raw = np.frombuffer(blocks, dtype=np.uint8)
    assert raw.size == n * (k // 32) * bb and (n * (k // 32)) % 2 == 1      # odd block count: the 18/22/34-byte formats end on a halfword
    own = torch.from_numpy(raw.copy()).to("cuda:0")
    buf = torch.empty(CANARY + base_mod4 + raw.size + CANARY, dtype=torch.uint8, device="cuda:0")
    assert buf.data_ptr() % 256 == 0
    w_ptr = buf.data_ptr() + CANARY + base_mod4
    for m in (1, 3, 8, 19, 40):
        x = normal(20 + m, (m, k))
        x_dev = torch.from_numpy(x).to("cuda:0")
        outs = []
        for fill in (0x00, 0xFF):
            buf.fill_(fill)
            buf[CANARY + base_mod4: CANARY + base_mod4 + raw.size] = own
            outs.append(_forward(L, code, w_ptr, x_dev, m, k, n))
        assert not np.isnan(outs[0]).any() and not np.isnan(outs[1]).any(), m
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), m
        if base_mod4 == 0:
            alone = _forward(L, code, own.data_ptr(), x_dev, m, k, n)
            assert np.array_equal(outs[0].view(np.uint32), alone.view(np.uint32)), m
        assert rel_l2(outs[0], oracle.matmul(odt, x, blocks, n)) <= 1e-5, m


@pytest.mark.parametrize("n,k", [(65, 256), (67, 768), (203, 1792), (64, 256), (129, 4096)])
def test_q6k_tensor_of_2_mod_4_bytes_on_the_streaming_kernel(n, k):
    """Q6_K super-blocks are 210 bytes: a tensor with an odd block count has a size of 2 (mod 4), and its last bytes are
    the f16 scale of the last block.  One and two f32 rows take the streaming kernel, whose buffer descriptor ends inside
    the dword that holds that scale: the last row must come out right and nothing beyond the tensor may be used."""
    print(f"case q6k n={n} k={k}", flush=True)
    L = _lib.lib()
    blocks = oracle.from_float(oracle.Q6K, normal(6, (n, k), 0.02).reshape(-1))
    raw = np.frombuffer(blocks, dtype=np.uint8)
    assert raw.size == n * (k // 256) * 210
    own = torch.from_numpy(raw.copy()).to("cuda:0")
    buf = torch.empty(CANARY + raw.size + CANARY, dtype=torch.uint8, device="cuda:0")
    w_ptr = buf.data_ptr() + CANARY                      # 16-byte aligned: the streaming kernel takes it
    for m in (1, 2):
        x = normal(40 + m, (m, k))
        x_dev = torch.from_numpy(x).to("cuda:0")
        outs = []
        for fill in (0x00, 0xFF):
            buf.fill_(fill)
            buf[CANARY: CANARY + raw.size] = own
            outs.append(_forward(L, 14, w_ptr, x_dev, m, k, n))
        assert not np.isnan(outs[0]).any() and not np.isnan(outs[1]).any(), m
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), m
        assert rel_l2(outs[0], oracle.matmul(oracle.Q6K, x, blocks, n)) <= 1e-5, m
        assert rel_l2(outs[0][:, -1], oracle.matmul(oracle.Q6K, x, blocks, n)[:, -1]) <= 1e-5, m     # the row whose scale ends the tensor
