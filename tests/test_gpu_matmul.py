"""GPU parity for QMatMul::forward (decode matvec and prefill matmul) against the CPU oracle.

Tolerance: relative L2 error <= 1e-3 against candle's CPU QMatMul::forward on the same seeded inputs
(the north-star bar).  Because the activations are quantized bit-identically to the CPU path, the
observed error is f32 summation order only, so the tests also assert the much tighter 2e-6.
"""
import numpy as np
import pytest
import torch

import oracle
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-3          # north-star tolerance
TIGHT = 2e-6        # what bit-identical activation quantization actually delivers
WDTYPES = [oracle.Q4_0, oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K]
NAMES = {oracle.Q4_0: "q4_0", oracle.Q8_0: "q8_0", oracle.Q4K: "q4k", oracle.Q5K: "q5k", oracle.Q6K: "q6k"}


def make_weight(dtype, n, k, seed):
    """Weights ~N(0, 0.02) quantized by the CPU oracle; returns (host block bytes, device QMatMul)."""
    import candle_amd as ca
    w = normal(seed, (n, k), 0.02)
    blocks = oracle.from_float(dtype, w.reshape(-1))
    st = ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype))
    qt = ca.QTensor.new(st, (n, k))
    return blocks, ca.QMatMul.from_qtensor(qt)


def forward(qmm, x: np.ndarray) -> np.ndarray:
    y = qmm.forward(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    return y.cpu().numpy()


# ---------------------------------------------------------------------------- reference KATs on the GPU
def test_kat_q4_0_matmul_on_gpu():
    # quantized_tests.rs:92-107,139-146 (the CPU goldens: activations are quantized the CPU way)
    import candle_amd as ca
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32).reshape(n, k)
    qt = ca.QTensor.quantize(torch.from_numpy(rhs).cuda(), ca.GgmlDType.Q4_0)
    res = forward(ca.QMatMul.from_qtensor(qt), lhs)
    want = [[85120.0, 214562.0, 345455.0, 474748.0], [213475.0, 604465.0, 1000686.0, 1388317.0],
            [341876.0, 994283.0, 1655709.0, 2301518.0]]
    assert np.round(res).tolist() == want


def test_kat_seeded_matmul_on_gpu():
    # quantized_tests.rs:1383-1459: m,k,n = 11,512,21, StdRng inputs, spot values to 3 decimals
    import candle_amd as ca
    from tests import stdrng
    from tests.test_oracle_kat import round3
    m, k, n = 11, 512, 21
    lhs, rhs = stdrng.get_random_tensors(m, k, n)
    for dtype, want in ((ca.GgmlDType.Q4K, [1.094, 1.442, -0.196, 1.587]), (ca.GgmlDType.Q5K, [1.161, 1.498, -0.175, 1.739]),
                        (ca.GgmlDType.Q6K, [1.293, 1.497, -0.159, 1.737])):
        qt = ca.QTensor.quantize(torch.from_numpy(rhs).cuda(), dtype)
        mm = forward(ca.QMatMul.from_qtensor(qt), lhs).reshape(-1)
        got = round3([mm[0], mm[m * n // 3], mm[m * n * 2 // 3], mm[m * n - 1]])
        assert got.tolist() == [float(np.float32(v)) for v in want], dtype.name


# ---------------------------------------------------------------------------- decode matvec vs oracle
@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 5, 6, 7, 8])
def test_matvec_vs_oracle(dtype, batch):
    n, k = 203, 4096            # ragged n: exercises the row tail of the last workgroup
    blocks, qmm = make_weight(dtype, n, k, seed=31 + dtype)
    x = normal(41 + batch, (batch, k), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul(dtype, x, blocks, n)
    err = rel_l2(got, want)
    assert err <= TOL and err <= TIGHT, f"rel-L2 {err}"


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k", [256, 768, 2048, 14336])
def test_matvec_k_sweep(dtype, k):
    n = 64
    blocks, qmm = make_weight(dtype, n, k, seed=51)
    x = normal(52, (2, k), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul(dtype, x, blocks, n)
    assert rel_l2(got, want) <= TIGHT


@pytest.mark.parametrize("wdt", [oracle.Q4K, oracle.Q5K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k", [256, 768, 2560, 4096, 6144, 8192, 11008, 14336])
@pytest.mark.parametrize("n,batch", [(203, 3), (203, 16), (5, 4), (16, 11), (17, 13), (1024, 9)])
def test_q4k_batched_rows_vs_oracle(wdt, k, n, batch):
    """3 .. 16 rows of Q4_K or Q5_K take the batched matrix-core matvec (16 weight rows per block, K split over the waves in
    1 .. 7 super-block columns each): ragged n, fewer rows than a block, every column count, idle waves (k = 256, 768)."""
    blocks, qmm = make_weight(wdt, n, k, seed=131)
    x = normal(132 + batch, (batch, k), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul_fast(wdt, x, blocks, n, 8)
    err = rel_l2(got, want)
    assert err <= TOL and err <= TIGHT, f"rel-L2 {err}"
    # row by row as well: a wrong batch column would hide in the norm of 16 rows
    for r in range(batch):
        assert rel_l2(got[r], want[r]) <= TIGHT, r


@pytest.mark.parametrize("wdt", [oracle.Q4K, oracle.Q5K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k", [256, 2048, 3072, 4096, 5120, 6144])     # 3072, 5120: some waves hold one column fewer than others
@pytest.mark.parametrize("rows", [3, 4, 5, 6, 8])
def test_q4k_batched_rows_quantized_inside_the_kernel(wdt, k, rows):
    """Few f32 rows are quantized by the waves of the matvec kernel itself (up to 16 spans per wave), more rows by a kernel
    of their own: a row gives the same bits either way, and both agree with the oracle.  The rows hold what the two
    quantizers treat differently inside: a largest value that is negative, a tie between +max and -max, an all-zero span."""
    n = 203
    blocks, qmm = make_weight(wdt, n, k, seed=171)
    x = normal(172 + rows, (rows, k), 1.0)
    x[0, :256] = 0.0
    x[1, 5] = -9.0
    x[2, 7] = 6.0
    x[2, 9] = -6.0
    x[rows - 1, k - 3] = -7.5
    big = np.concatenate([x, normal(173, (16 - rows, k), 1.0)])
    got = forward(qmm, x)
    ref = forward(qmm, big)[:rows]
    assert np.array_equal(got, ref)
    want = oracle.matmul_fast(wdt, x, blocks, n, 8)
    for r in range(rows):
        assert rel_l2(got[r], want[r]) <= TIGHT, r


@pytest.mark.parametrize("wdt", [oracle.Q4K, oracle.Q5K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k", [256, 768, 2048, 4096])
@pytest.mark.parametrize("n,rows", [(203, 17), (203, 32), (96, 33), (50, 47), (130, 64)])
def test_q4k_rows_in_sets_of_16_vs_oracle(wdt, k, n, rows):
    """17 .. 64 f32 rows of Q4_K or Q5_K (rows of up to 4096 elements) run as sets of 16 rows, two sets per pass over the weights: a
    partly filled second set, a second pass with one set and with two, ragged n, one to eight waves per row block."""
    blocks, qmm = make_weight(wdt, n, k, seed=181)
    x = normal(182 + rows, (rows, k), 1.0)
    x[0, :256] = 0.0
    x[rows - 1, k - 3] = -7.5
    got = forward(qmm, x)
    want = oracle.matmul_fast(wdt, x, blocks, n, 8)
    err = rel_l2(got, want)
    assert err <= TOL and err <= TIGHT, f"rel-L2 {err}"
    for r in range(rows):
        assert rel_l2(got[r], want[r]) <= TIGHT, r


def test_cfg1_q8_0_4096x4096():
    # BASELINE configs[0]: Q8_0 weight [4096 x 4096], activation 1 x 4096
    blocks, qmm = make_weight(oracle.Q8_0, 4096, 4096, seed=1)
    x = normal(2, (1, 4096), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul(oracle.Q8_0, x, blocks, 4096)
    err = rel_l2(got, want)
    assert err <= TOL and err <= TIGHT, err


def test_q8k_weights_rejected():
    # the GPU matmul of the reference skips Q8K weights as well (quantized_tests.rs:24-29)
    import candle_amd as ca
    w = torch.zeros((4, 256), device="cuda")
    qt = ca.QTensor.quantize(w, ca.GgmlDType.Q8K)
    with pytest.raises(NotImplementedError):
        ca.QMatMul.from_qtensor(qt).forward(torch.zeros((1, 256), device="cuda"))


# ---------------------------------------------------------------------------- prefill matmul vs oracle
@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("m", [9, 16, 33, 128])
def test_matmul_vs_oracle(dtype, m):
    n, k = 96, 1024
    blocks, qmm = make_weight(dtype, n, k, seed=61 + dtype)
    x = normal(62 + m, (m, k), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul(dtype, x, blocks, n)
    err = rel_l2(got, want)
    assert err <= TOL and err <= prefill_bound(dtype), f"rel-L2 {err}"


def prefill_bound(dtype):
    """More than 8 rows run on the matrix cores, every format with the integer sums of the CPU path: K-quant operands
    are exact integers (f16 cores; Q6_K as an f16 head plus an exact remainder term; Q4_K on the int8 cores), Q4_0 / Q8_0
    blocks are one int8 MFMA each, scaled in f32 per block like the CPU loop."""
    return TIGHT


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("m,n,k", [(128, 128, 256), (130, 200, 512), (257, 129, 2048), (64, 384, 4096)])
def test_prefill_tiles_ragged(dtype, m, n, k):
    # tile edges: rows and columns that do not fill the 128 x 128 block tile, one and many super-blocks
    blocks, qmm = make_weight(dtype, n, k, seed=161 + dtype)
    x = normal(162 + m, (m, k), 1.0)
    got = forward(qmm, x)
    want = oracle.matmul(dtype, x, blocks, n)
    err = rel_l2(got, want)
    assert err <= TOL and err <= prefill_bound(dtype), f"rel-L2 {err}"
    # every row on its own as well: a wrong row/column mapping can hide in an aggregate norm
    worst = max(rel_l2(got[r], want[r]) for r in range(m))
    assert worst <= 4 * prefill_bound(dtype), worst


@pytest.mark.parametrize("dtype", [oracle.Q4_0, oracle.Q8_0], ids=lambda d: NAMES[d])
def test_prefill_k_not_multiple_of_256(dtype):
    blocks, qmm = make_weight(dtype, 48, 32 * 9, seed=171)
    x = normal(172, (20, 32 * 9), 1.0)
    assert rel_l2(forward(qmm, x), oracle.matmul(dtype, x, blocks, 48)) <= TIGHT


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k", [6144, 8192, 14336, 16384])
@pytest.mark.parametrize("n", [67, 203, 1031])
def test_long_rows_ragged_on_the_streaming_kernel(dtype, k, n):
    """One and two f32 rows of 24 / 32 / 56 / 64 super-blocks: the long-row launches of the streaming kernel (three to eight
    activation spans per wave) with fewer steps than waves, steps that are not
    whole cache lines (Q6_K rows of 24 or 56 blocks) and a last step that ends inside the tensor's last row."""
    blocks, qmm = make_weight(dtype, n, k, seed=500 + dtype)
    for batch in (1, 2):
        x = normal(600 + batch, (batch, k), 1.0)
        got = forward(qmm, x)
        err = rel_l2(got, oracle.matmul(dtype, x, blocks, n))
        assert err <= TOL and err <= TIGHT, f"batch {batch}: rel-L2 {err}"
        assert np.array_equal(got, forward(qmm, x))          # and the same bits on a second call


def test_batching_invariance_on_gpu():
    # quantized_tests.rs:224-259: stacking the same rows must not change their results
    blocks, qmm = make_weight(oracle.Q4K, 24, 512, seed=71)
    x = normal(72, (2, 512), 1.0)
    y2 = forward(qmm, x)
    y4 = forward(qmm, np.concatenate([x, x]))
    y12 = forward(qmm, np.concatenate([x] * 6))
    assert np.array_equal(y4[2:], y4[:2])
    assert np.array_equal(y12[10:], y12[:2])
    assert rel_l2(y4[:2], y2) <= TIGHT and rel_l2(y12[:2], y2) <= TIGHT


def test_rank3_input_and_shape_errors():
    import candle_amd as ca
    blocks, qmm = make_weight(oracle.Q4K, 16, 256, seed=73)
    x = normal(74, (2, 3, 256), 1.0)
    y = forward(qmm, x)
    assert y.shape == (2, 3, 16)
    want = oracle.matmul(oracle.Q4K, x.reshape(6, 256), blocks, 16).reshape(2, 3, 16)
    assert rel_l2(y, want) <= TIGHT
    with pytest.raises(ValueError):     # mod.rs:915-917
        qmm.forward(torch.zeros(256, device="cuda"))
    with pytest.raises(ValueError):     # mod.rs:920-922
        qmm.forward(torch.zeros((2, 128), device="cuda"))
    with pytest.raises(ValueError):     # mod.rs:909-911
        qmm.forward(torch.zeros((256, 2), device="cuda").t())


@pytest.mark.parametrize("wdt", [oracle.Q4K, oracle.Q5K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("rows,k", [(3, 512), (5, 8192), (2, 512), (12, 2048), (16, 3072), (9, 5120)])   # 3072, 5120: columns that do not fill the waves evenly
@pytest.mark.parametrize("tdt", [torch.float16, torch.bfloat16])
def test_half_activations_keep_dtype(tdt, rows, k, wdt):
    # CPU f16 path: widen, quantize, dot, round the result to f16 (k_quants.rs:2652-2686); the GPU keeps the input dtype
    # (two rows: the streaming kernel; 3 .. 16 rows: the batched matrix-core kernel, rows of 8192 elements in column chunks)
    blocks, qmm = make_weight(wdt, 40, k, seed=75)
    x = torch.from_numpy(normal(76, (rows, k), 1.0)).to(tdt)
    y = qmm.forward(x.cuda())
    torch.cuda.synchronize()
    assert y.dtype == tdt
    want = torch.from_numpy(oracle.matmul(wdt, x.float().numpy(), blocks, 40)).to(tdt)
    # identical up to one rounding step of the output type
    assert rel_l2(y.float().cpu().numpy(), want.float().numpy()) <= (2e-3 if tdt == torch.float16 else 1e-2)


# ---------------------------------------------------------------------------- full BASELINE sizes: size-independent property
@pytest.mark.parametrize("dtype,n,k", [(oracle.Q4K, 14336, 4096), (oracle.Q4K, 4096, 14336), (oracle.Q6K, 4096, 14336),
                                       (oracle.Q5K, 14336, 4096), (oracle.Q4_0, 14336, 4096), (oracle.Q8_0, 4096, 4096)],
                         ids=lambda v: NAMES.get(v, str(v)))
@pytest.mark.parametrize("batch", [1, 2, 4, 8, 16, 128])
def test_full_size_equals_dot_of_dequantized(dtype, n, k, batch):
    """The quantized dot equals the dot of the two dequantized operands (up to f32 summation error):
    y = dequant(W) @ dequant(x^) in f64.  dequant(W) is the bit-exact GPU dequantizer checked
    elsewhere; x^ is the CPU oracle's quantization of the same seeded activations."""
    import candle_amd as ca
    w = torch.from_numpy(normal(81, (n, k), 0.02)).cuda()
    qt = ca.QTensor.quantize(w, ca.GgmlDType(dtype))
    qmm = ca.QMatMul.from_qtensor(qt)
    x = normal(82 + batch, (batch, k), 1.0)
    got = forward(qmm, x)
    adt = oracle.vec_dot_type(dtype)
    xq = np.stack([oracle.to_float(adt, oracle.from_float(adt, x[r]), k) for r in range(batch)])
    wd = qt.dequantize().double()
    want = (torch.from_numpy(xq).cuda().double() @ wd.t()).cpu().numpy()
    err = rel_l2(got, want)
    assert err <= TOL and err <= (5e-6 if batch <= 8 else max(5e-6, prefill_bound(dtype))), err
    # spot-check a few rows against the scalar oracle itself
    rows = [0, n // 2, n - 1]
    blocks = np.frombuffer(qt.data(), dtype=np.uint8)
    rb = (k // oracle.block_size(dtype)) * oracle.type_size(dtype)
    sub = np.concatenate([blocks[r * rb:(r + 1) * rb] for r in rows])
    want_rows = oracle.matmul(dtype, x, sub, len(rows))
    assert rel_l2(got[:, rows], want_rows) <= (TIGHT if batch <= 8 else prefill_bound(dtype))


_FULL = {}


def _full_size_weight(dtype, n, k):
    """One quantized [n, k] weight per (format, shape), shared by the row counts below: (QTensor, dequantized f64 weight on the GPU)."""
    import candle_amd as ca
    key = (dtype, n, k)
    if key not in _FULL:
        _FULL.clear()                       # one weight at a time: 14336 x 4096 doubles are 470 MB
        w = torch.from_numpy(normal(81, (n, k), 0.02)).cuda()
        qt = ca.QTensor.quantize(w, ca.GgmlDType(dtype))
        _FULL[key] = (qt, qt.dequantize().double())
    return _FULL[key]


@pytest.mark.parametrize("dtype,n,k", [(oracle.Q6K, 4096, 14336), (oracle.Q5K, 14336, 4096), (oracle.Q4_0, 4096, 14336), (oracle.Q4_0, 14336, 4096),
                                       (oracle.Q4K, 14336, 4096), (oracle.Q4K, 4096, 14336), (oracle.Q8_0, 14336, 4096)],
                         ids=lambda v: NAMES.get(v, str(v)))
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_full_size_prefill_rows(dtype, n, k, m):
    """The prefill shapes at 128, 512 and 2048 activation rows: every output against the f64 dot of the dequantized
    operands, three weight rows x all activation rows against the scalar oracle, and the last activation row (the ragged
    end of the last row tile) against the oracle on 64 evenly spaced weight rows."""
    import candle_amd as ca
    qt, wd = _full_size_weight(dtype, n, k)
    qmm = ca.QMatMul.from_qtensor(qt)
    x = normal(182 + m, (m, k), 1.0)
    got = forward(qmm, x)
    adt = oracle.vec_dot_type(dtype)
    xq = oracle.to_float(adt, oracle.from_float(adt, x.reshape(-1)), m * k).reshape(m, k)
    want = (torch.from_numpy(xq).cuda().double() @ wd.t()).cpu().numpy()
    bound = max(5e-6, prefill_bound(dtype))
    err = rel_l2(got, want)
    assert err <= TOL and err <= bound, err
    worst = max(rel_l2(got[r], want[r]) for r in range(0, m, 37))
    assert worst <= 4 * bound, worst
    blocks = np.frombuffer(qt.data(), dtype=np.uint8)
    rb = (k // oracle.block_size(dtype)) * oracle.type_size(dtype)
    rows = [0, n // 2 + 1, n - 1]
    sub = np.concatenate([blocks[r * rb:(r + 1) * rb] for r in rows])
    assert rel_l2(got[:, rows], oracle.matmul(dtype, x, sub, len(rows))) <= prefill_bound(dtype)
    rows = list(range(0, n, n // 64))
    sub = np.concatenate([blocks[r * rb:(r + 1) * rb] for r in rows])
    assert rel_l2(got[-1:, rows], oracle.matmul(dtype, x[-1:], sub, len(rows))) <= prefill_bound(dtype)
