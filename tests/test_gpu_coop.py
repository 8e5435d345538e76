"""Cooperative decode launches (cq_nn_decode_*): several dependent single-row matvecs as one launch whose phases meet at a
barrier across the launch's workgroups.  Each must reproduce the chain of calls it replaces bit for bit (same kernels bodies,
same step -> wave assignment), launch after launch on one set of sync words, and leave the error word clear."""
import numpy as np
import pytest
import torch

import oracle
from candle_amd import _lib
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

ERR_WORD = 1056          # CQ_NN_COOP_ERR_WORD


def L():
    return _lib.lib()


def ok(rc):
    assert rc == 0, _lib.status_string(rc)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def sync_words():
    return torch.zeros(L().cq_nn_coop_sync_bytes() // 4, dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("hidden,ffn,d13,d2", [(4096, 14336, oracle.Q4K, oracle.Q6K), (4096, 14336, oracle.Q4K, oracle.Q4K),
                                              (512, 768, oracle.Q4K, oracle.Q6K), (256, 4096, oracle.Q4K, oracle.Q6K),
                                              (2048, 8192, oracle.Q4K, oracle.Q4K), (1024, 512, oracle.Q4K, oracle.Q6K)])
def test_decode_mlp_equals_the_chain_of_calls(hidden, ffn, d13, d2):
    lib = L()
    w13 = dev(oracle.from_float(d13, normal(1, (2 * ffn, hidden), 0.05).reshape(-1)))
    w2 = dev(oracle.from_float(d2, normal(2, (hidden, ffn), 0.05).reshape(-1)))
    w3_ptr = w13.data_ptr() + w13.numel() // 2
    norm_w = dev(1.0 + 0.1 * normal(3, (hidden,)))
    x0 = normal(4, (1, hidden))
    part0 = np.zeros(256, dtype=np.float32)
    part0[:4] = (x0.reshape(4, -1).astype(np.float64) ** 2).sum(axis=1).astype(np.float32)
    sync = sync_words()
    # the chain of calls and the cooperative launch, each feeding its own output back in, 40 times over
    xa, pa, ha = dev(x0), dev(part0), torch.empty(ffn, device="cuda")
    xb, pb, hb = dev(x0), dev(part0), torch.empty(ffn, device="cuda")
    for it in range(40):
        ok(lib.cq_nn_qmatmul_norm_swiglu(d13, w13.data_ptr(), w3_ptr, xa.data_ptr(), pa.data_ptr(), norm_w.data_ptr(), 1e-5, ha.data_ptr(), hidden,
                                         ffn, None))
        ok(lib.cq_nn_qmatmul_residual(d2, w2.data_ptr(), ha.data_ptr(), None, xa.data_ptr(), pa.data_ptr(), ffn, hidden, None))
        ok(lib.cq_nn_decode_mlp(d13, w13.data_ptr(), w3_ptr, d2, w2.data_ptr(), xb.data_ptr(), pb.data_ptr(), norm_w.data_ptr(), 1e-5, hb.data_ptr(),
                                hidden, ffn, sync.data_ptr(), None))
        if it in (0, 1, 39):
            torch.cuda.synchronize()
            assert int(sync[ERR_WORD]) == 0
            assert np.array_equal(ha.cpu().numpy(), hb.cpu().numpy()), it
            assert np.array_equal(xa.cpu().numpy(), xb.cpu().numpy()), it
            assert np.array_equal(pa.cpu().numpy(), pb.cpu().numpy()), it
    # and the first step against the CPU ops
    xn = (x0 / np.sqrt((x0.astype(np.float64) ** 2).mean() + 1e-5).astype(np.float32) * norm_w.cpu().numpy()).astype(np.float32)
    blocks13 = w13.cpu().numpy()
    g = oracle.matmul_fast(d13, xn, blocks13[:blocks13.size // 2], ffn, 8)
    u = oracle.matmul_fast(d13, xn, blocks13[blocks13.size // 2:], ffn, 8)
    h = (g / (1.0 + np.exp(-g)) * u).astype(np.float32)
    want = x0 + oracle.matmul_fast(d2, h, w2.cpu().numpy(), hidden, 8)
    xc, pc, hc = dev(x0), dev(part0), torch.empty(ffn, device="cuda")
    ok(lib.cq_nn_decode_mlp(d13, w13.data_ptr(), w3_ptr, d2, w2.data_ptr(), xc.data_ptr(), pc.data_ptr(), norm_w.data_ptr(), 1e-5, hc.data_ptr(),
                            hidden, ffn, sync.data_ptr(), None))
    assert rel_l2(xc.cpu().numpy(), want) <= 1e-4


def test_decode_mlp_argument_errors():
    lib = L()
    s = sync_words()
    assert lib.cq_nn_decode_mlp(12, 256, 256, 14, 256, 256, 256, 256, 1e-5, 256, 4096, 14336, None, None) == -4          # no sync words
    assert lib.cq_nn_decode_mlp(12, 256, 256, 14, 256, 256, 256, 256, 1e-5, 256, 4000, 14336, s.data_ptr(), None) == -2   # hidden % 256
    assert lib.cq_nn_decode_mlp(8, 256, 256, 8, 256, 256, 256, 256, 1e-5, 256, 4096, 14336, s.data_ptr(), None) == -6     # Q8_0: no cooperative kernel
    assert lib.cq_nn_decode_mlp(12, 256, 256, 14, 256, 256, 256, 256, 1e-5, 256, 8192, 14336, s.data_ptr(), None) == -6   # w1 rows longer than a wave step
