"""GPU parity of QMatMul::forward for Q4_1, Q5_0, Q5_1, Q2_K, Q3_K weights against the CPU oracle: candle's CPU path
quantizes their activations to Q8_1 / Q8_0 / Q8_1 / Q8_K / Q8_K (k_quants.rs:317,418,524,822,1055).  The GPU quantizes to
the same int8 values and every kernel sums the same integers (matvec kernels; beyond 8 rows the f16 matrix cores with
exact small-integer operands for Q2_K / Q3_K and one int8 MFMA per block for Q4_1 / Q5_0 / Q5_1), so the bar is the same
as for the other K-quants: relative L2 <= 1e-3 by contract, <= 2e-6 observed (f32 summation order only).
"""
import numpy as np
import pytest
import torch

import oracle
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-3
TIGHT = 2e-6
WDTYPES = [oracle.Q4_1, oracle.Q5_0, oracle.Q5_1, oracle.Q2K, oracle.Q3K]
NAMES = {oracle.Q4_1: "q4_1", oracle.Q5_0: "q5_0", oracle.Q5_1: "q5_1", oracle.Q2K: "q2k", oracle.Q3K: "q3k"}


def make_weight(dtype, n, k, seed):
    import candle_amd as ca
    w = normal(seed, (n, k), 0.02)
    blocks = oracle.from_float(dtype, w.reshape(-1))
    qt = ca.QTensor.new(ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype)), (n, k))
    return blocks, ca.QMatMul.from_qtensor(qt)


def forward(qmm, x):
    y = qmm.forward(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_kat_seeded_matmul_q2k_q3k_on_gpu():
    # quantized_tests.rs:1331-1380: m,k,n = 11,512,21, StdRng inputs, weights quantized by the (pinned) CPU quantizer
    import candle_amd as ca
    from tests import stdrng
    from tests.test_oracle_kat import round3
    m, k, n = 11, 512, 21
    lhs, rhs = stdrng.get_random_tensors(m, k, n)
    for dtype, want in ((oracle.Q2K, [0.887, 0.428, 0.219, 1.669]), (oracle.Q3K, [1.001, 1.425, -0.311, 1.493])):
        blocks = oracle.from_float(dtype, rhs.reshape(-1))
        qt = ca.QTensor.new(ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype)), (n, k))
        mm = forward(ca.QMatMul.from_qtensor(qt), lhs).reshape(-1)
        got = round3([mm[0], mm[m * n // 3], mm[m * n * 2 // 3], mm[m * n - 1]])
        assert got.tolist() == [float(np.float32(v)) for v in want], NAMES[dtype]


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 5, 6, 7, 8])
def test_matvec_vs_oracle(dtype, batch):
    n, k = 203, 4096            # ragged n; one wave step per row for the K-quants, two for the 32-element formats
    blocks, qmm = make_weight(dtype, n, k, seed=31 + dtype)
    x = normal(41 + batch, (batch, k), 1.0)
    err = rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, n))
    assert err <= TOL and err <= TIGHT, f"rel-L2 {err}"


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k", [256, 768, 2048, 14336])
@pytest.mark.parametrize("batch", [1, 2, 5])
def test_matvec_k_sweep(dtype, k, batch):
    n = 64
    blocks, qmm = make_weight(dtype, n, k, seed=51)
    x = normal(52, (batch, k), 1.0)
    assert rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, n)) <= TIGHT


@pytest.mark.parametrize("dtype", [oracle.Q4_1, oracle.Q5_0, oracle.Q5_1], ids=lambda d: NAMES[d])
def test_k_not_multiple_of_256(dtype):
    blocks, qmm = make_weight(dtype, 70, 32 * 9, seed=53)
    x = normal(54, (3, 32 * 9), 1.0)
    assert rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, 70)) <= TIGHT


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("m", [9, 16, 33, 128])
def test_more_than_eight_rows(dtype, m):
    # Q2_K / Q3_K: f16 matrix cores; Q4_1 / Q5_0 / Q5_1: int8 matrix cores when k is a multiple of 256
    n, k = 96, 1024
    blocks, qmm = make_weight(dtype, n, k, seed=61 + dtype)
    x = normal(62 + m, (m, k), 1.0)
    err = rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, n))
    assert err <= TOL and err <= TIGHT, f"rel-L2 {err}"


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("tdt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 4, 12])
def test_half_activations_keep_dtype(dtype, tdt, m):
    blocks, qmm = make_weight(dtype, 40, 512, seed=75)
    x = torch.from_numpy(normal(76, (m, 512), 1.0)).to(tdt)
    y = qmm.forward(x.cuda())
    torch.cuda.synchronize()
    assert y.dtype == tdt
    want = torch.from_numpy(oracle.matmul(dtype, x.float().numpy(), blocks, 40)).to(tdt)
    assert rel_l2(y.float().cpu().numpy(), want.float().numpy()) <= (2e-3 if tdt == torch.float16 else 1e-2)


@pytest.mark.parametrize("dtype,n,k", [(oracle.Q4_1, 14336, 4096), (oracle.Q5_0, 4096, 14336), (oracle.Q5_1, 14336, 4096),
                                       (oracle.Q2K, 4096, 14336), (oracle.Q3K, 14336, 4096), (oracle.Q3K, 4096, 14336)],
                         ids=lambda v: NAMES.get(v, str(v)))
@pytest.mark.parametrize("batch", [1, 8])
def test_full_size_vs_oracle(dtype, n, k, batch):
    # the 8B decoder's FFN shapes, every output value against the scalar oracle
    blocks, qmm = make_weight(dtype, n, k, seed=81)
    x = normal(82 + batch, (batch, k), 1.0)
    err = rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, n))
    assert err <= TOL and err <= TIGHT, err


def test_bit_patterns_random_blocks():
    # random block bytes put every bit of qs / qh / hmask / scales in play (quantized normal data rarely sets the top scale bits)
    import candle_amd as ca
    from tests.test_oracle_kat import random_weight_blocks
    rng = np.random.default_rng(7)
    n, k = 130, 2048
    for dtype in WDTYPES:
        blocks = random_weight_blocks(dtype, n * k // oracle.block_size(dtype), rng)
        qt = ca.QTensor.new(ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype)), (n, k))
        x = normal(90 + dtype, (2, k), 1.0)
        got = forward(ca.QMatMul.from_qtensor(qt), x)
        want = oracle.matmul(dtype, x, blocks, n)
        assert rel_l2(got, want) <= TIGHT, NAMES[dtype]


@pytest.mark.parametrize("dtype", [oracle.Q2K, oracle.Q3K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("m,n,k", [(128, 128, 256), (130, 200, 512), (257, 129, 2048), (64, 384, 4096), (20, 260, 1024), (512, 96, 8192)])
def test_prefill_tiles_ragged(dtype, m, n, k):
    # 128 x 64 and 32 x 128 tiles with ragged edges, one super-block rows, split-K shapes (few tiles, long k)
    blocks, qmm = make_weight(dtype, n, k, seed=71)
    x = normal(72, (m, k), 1.0)
    err = rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, n))
    assert err <= TIGHT, err


@pytest.mark.parametrize("dtype", [oracle.Q2K, oracle.Q3K], ids=lambda d: NAMES[d])
def test_prefill_random_blocks(dtype):
    # every bit of qs / hmask / scales in play on the matrix-core path (scales up to 63, mins up to 15)
    import candle_amd as ca
    from tests.test_oracle_kat import random_weight_blocks
    rng = np.random.default_rng(8)
    n, k, m = 130, 1024, 70
    blocks = random_weight_blocks(dtype, n * k // 256, rng)
    qt = ca.QTensor.new(ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype)), (n, k))
    x = normal(91, (m, k), 1.0)
    assert rel_l2(forward(ca.QMatMul.from_qtensor(qt), x), oracle.matmul(dtype, x, blocks, n)) <= TIGHT


@pytest.mark.parametrize("dtype", [oracle.Q4_1, oracle.Q5_0, oracle.Q5_1], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("m,n,k", [(128, 128, 256), (130, 200, 512), (257, 129, 2048), (64, 384, 4096), (20, 260, 1024), (512, 96, 8192)])
def test_int8_matrix_core_tiles_ragged(dtype, m, n, k):
    """Tile edges of the int8 matrix-core kernel: rows and columns that do not fill the block tile, the 32-row tile (20 rows),
    one and many stages, split-K; every row on its own as well."""
    blocks, qmm = make_weight(dtype, n, k, seed=261 + dtype)
    x = normal(262 + m, (m, k), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul(dtype, x, blocks, n)
    assert rel_l2(got, want) <= TIGHT
    assert max(rel_l2(got[r], want[r]) for r in range(m)) <= 4 * TIGHT


@pytest.mark.parametrize("dtype,n,k", [(oracle.Q4_1, 14336, 4096), (oracle.Q5_0, 4096, 14336), (oracle.Q5_1, 14336, 4096)], ids=lambda v: NAMES.get(v, str(v)))
@pytest.mark.parametrize("m", [128, 512])
def test_int8_matrix_core_full_size(dtype, n, k, m):
    """The FFN shapes at prefill row counts: three weight rows x all activation rows and the last activation row x 64 weight
    rows against the scalar oracle."""
    import candle_amd as ca
    w = torch.from_numpy(normal(281, (n, k), 0.02)).cuda()
    qt = ca.QTensor.quantize(w, ca.GgmlDType(dtype))
    x = normal(282 + m, (m, k), 1.0)
    got = forward(ca.QMatMul.from_qtensor(qt), x)
    blocks = np.frombuffer(qt.data(), dtype=np.uint8)
    rb = (k // 32) * oracle.type_size(dtype)
    for rows, xs in (([0, n // 2 + 1, n - 1], slice(0, m)), (list(range(0, n, n // 64)), slice(m - 1, m))):
        sub = np.concatenate([blocks[r * rb:(r + 1) * rb] for r in rows])
        assert rel_l2(got[xs][:, rows], oracle.matmul(dtype, x[xs], sub, len(rows))) <= TIGHT
