"""GPU parity, bit-exact: dequantize, weight quantize and activation quantize against the CPU oracle.

All calls go through the C ABI (ctypes) via candle_amd.  The bar is bitwise equality: dequantized
floats must match GgmlType::to_float, quantized bytes must match GgmlType::from_float.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from tests.util import bits_equal_or_both_nan, normal

pytestmark = pytest.mark.gpu

DTYPES = [oracle.Q4_0, oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q8K]
# the remaining block formats of GgmlDType
STORAGE_DTYPES = [oracle.Q4_1, oracle.Q5_0, oracle.Q5_1, oracle.Q8_1, oracle.Q2K, oracle.Q3K]
NAMES = {oracle.Q4_0: "q4_0", oracle.Q8_0: "q8_0", oracle.Q4K: "q4k", oracle.Q5K: "q5k", oracle.Q6K: "q6k", oracle.Q8K: "q8k",
         oracle.Q4_1: "q4_1", oracle.Q5_0: "q5_0", oracle.Q5_1: "q5_1", oracle.Q8_1: "q8_1", oracle.Q2K: "q2k", oracle.Q3K: "q3k"}


def _candle():
    import candle_amd
    return candle_amd


def gpu_dequant(dtype, blocks: np.ndarray, n_elems: int, f16=False) -> np.ndarray:
    ca = _candle()
    st = ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype))
    out = st.dequantize(n_elems, f16=f16)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def gpu_quantize(dtype, x: np.ndarray) -> np.ndarray:
    ca = _candle()
    qt = ca.QTensor.quantize(torch.from_numpy(x).cuda(), ca.GgmlDType(dtype))
    torch.cuda.synchronize()
    return np.frombuffer(qt.data(), dtype=np.uint8)


# ------------------------------------------------------------------------------- dequantize
@pytest.mark.parametrize("dtype", DTYPES + STORAGE_DTYPES, ids=lambda d: NAMES[d])
def test_dequantize_random_bytes_bit_exact(dtype):
    # every byte pattern is a valid block, including NaN / Inf / subnormal f16 scales
    rng = np.random.Generator(np.random.PCG64(100 + dtype))
    nblk = 4099  # odd count: exercises the grid tail
    blocks = rng.integers(0, 256, size=nblk * oracle.type_size(dtype), dtype=np.uint8)
    n = nblk * oracle.block_size(dtype)
    want = oracle.to_float(dtype, blocks, n)
    got = gpu_dequant(dtype, blocks, n)
    assert bits_equal_or_both_nan(got, want)


@pytest.mark.parametrize("dtype", DTYPES + STORAGE_DTYPES, ids=lambda d: NAMES[d])
def test_dequantize_quantized_gaussian_bit_exact_and_f16(dtype):
    x = normal(7, 256 * 1024, 0.02)
    blocks = oracle.from_float(dtype, x)
    want = oracle.to_float(dtype, blocks, x.size)
    got = gpu_dequant(dtype, blocks, x.size)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # INV-2 (quantized_tests.rs:351-357): dequantize_f16 == to_f16(dequantize)
    got16 = gpu_dequant(dtype, blocks, x.size, f16=True)
    assert np.array_equal(got16.view(np.uint16), want.astype(np.float16).view(np.uint16))


def test_dequantize_empty_and_errors():
    ca = _candle()
    from candle_amd import _lib
    L = _lib.lib()
    assert L.cq_dequantize(int(ca.GgmlDType.Q4K), None, None, 0, 0, None) == 0          # empty is ok
    assert L.cq_dequantize(int(ca.GgmlDType.Q4K), None, None, 100, 0, None) == -2        # not a block multiple
    assert L.cq_dequantize(int(ca.GgmlDType.F16), None, None, 256, 0, None) == -1        # not a block format
    assert L.cq_quantize(int(ca.GgmlDType.F16), None, None, 256, None) == -1             # not a block format
    assert L.cq_dequantize(int(ca.GgmlDType.Q4K), None, None, 256, 0, None) == -4        # NULL


def test_kat_q4_0_roundtrip_on_gpu():
    # quantized_tests.rs:345-374 run on the device: quantize 0..127, dequantize, spot-check against the oracle
    src = np.arange(128, dtype=np.float32)
    blocks = gpu_quantize(oracle.Q4_0, src)
    assert np.array_equal(blocks, oracle.from_float(oracle.Q4_0, src))
    got = gpu_dequant(oracle.Q4_0, blocks, 128)
    assert got[2] == 3.875 and got[30] == 31.0 and got[64] == 59.375 and got[127] == 127.0
    assert np.signbit(got[0])


# ------------------------------------------------------------------------------- weight quantize
def _quant_inputs():
    yield "gauss_0.02", normal(11, 256 * 257, 0.02)
    yield "gauss_1", normal(12, 256 * 64, 1.0)
    yield "ramp", ((np.arange(4096, dtype=np.float32) - 2048) * np.float32(0.5 / 2048)).astype(np.float32)
    yield "cos", (np.float32(0.1) + np.float32(2.0) * np.cos(np.arange(4096, dtype=np.float32)).astype(np.float32)).astype(np.float32)
    z = normal(13, 256 * 8, 0.5)
    z[:256] = 0.0            # all-zero super-block
    z[256:512] = 1.25        # constant block
    z[512:544] = 0.0         # zero sub-block inside a live block
    z[768] = 1e30            # huge outlier
    z[1024:1280] = -np.abs(z[1024:1280])   # all negative
    yield "edge", z


@pytest.mark.parametrize("dtype", DTYPES + STORAGE_DTYPES, ids=lambda d: NAMES[d])
def test_quantize_bytes_match_cpu_from_float(dtype):
    for name, x in _quant_inputs():
        want = oracle.from_float(dtype, x)
        got = gpu_quantize(dtype, x)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, f"{NAMES[dtype]} {name}: {bad.size} bytes differ, first at {bad[:5]} (block {bad[0] // oracle.type_size(dtype)})"


# ------------------------------------------------------------------------------- activation quantize
def gpu_quantize_act(w_dtype, x: np.ndarray):
    from candle_amd import _lib
    L = _lib.lib()
    rows, k = x.shape
    xs = torch.from_numpy(x).cuda()
    nbytes = L.cq_act_scratch_bytes(w_dtype, k, rows)
    assert nbytes > 0
    scratch = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    _lib.check("cq_quantize_act", L.cq_quantize_act(w_dtype, xs.data_ptr(), 0, scratch.data_ptr(), k, rows, None))
    torch.cuda.synchronize()
    return scratch.cpu().numpy()


def _align256(v):
    return (v + 255) & ~255


def _act_inputs(k):
    x = normal(21, (5, k), 1.0)
    x[1, :256] = 0.0                                   # all-zero block -> d = 0
    x[2, 0] = 9.0; x[2, 100] = -9.0                    # exact +/- tie: the first one (positive) wins
    x[3, 5] = -7.5; x[3, 200] = 7.5                    # tie, the negative one first
    x[4, :64] = np.float32(0.5) * np.arange(64, dtype=np.float32) / np.float32(63)   # .5 rounding ties
    x[4, 255] = 127.0 * 0.5
    return x


@pytest.mark.parametrize("k", [256, 4096, 768])
def test_act_quant_q8k_bit_exact(k):
    x = _act_inputs(k)
    rows = x.shape[0]
    raw = gpu_quantize_act(oracle.Q4K, x)
    d_off = _align256(rows * k)
    bs_off = d_off + _align256(rows * (k // 256) * 4)
    qs = raw[: rows * k].view(np.int8).reshape(rows, k)
    d = raw[d_off: d_off + rows * (k // 256) * 4].view(np.float32).reshape(rows, k // 256)
    bs = raw[bs_off: bs_off + rows * (k // 16) * 2].view(np.int16).reshape(rows, k // 16)
    for r in range(rows):
        blk = oracle.from_float(oracle.Q8K, x[r]).reshape(k // 256, 292)
        want_d = blk[:, :4].copy().view(np.float32).reshape(-1)
        want_qs = blk[:, 4:260].copy().view(np.int8).reshape(-1)
        want_bs = blk[:, 260:].copy().view(np.int16).reshape(-1)
        assert np.array_equal(d[r].view(np.uint32), want_d.view(np.uint32)), f"row {r} d"
        assert np.array_equal(qs[r], want_qs), f"row {r} qs"
        assert np.array_equal(bs[r], want_bs), f"row {r} bsums"


@pytest.mark.parametrize("k", [32, 64, 4096])
def test_act_quant_q8_0_bit_exact(k):
    x = normal(22, (3, k), 1.0)
    x[1, :32] = 0.0
    x[2, :8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.0, -127.0]   # d = 1 -> exact .5 ties, round half away
    rows = x.shape[0]
    raw = gpu_quantize_act(oracle.Q8_0, x)
    d_off = _align256(rows * k)
    qs = raw[: rows * k].view(np.int8).reshape(rows, k)
    ds = raw[d_off: d_off + rows * (k // 32) * 8].view(np.uint32).reshape(rows, k // 32, 2)
    for r in range(rows):
        blk = oracle.from_float(oracle.Q8_0, x[r]).reshape(k // 32, 34)
        want_d16 = blk[:, :2].copy().view(np.uint16).reshape(-1)
        want_qs = blk[:, 2:].copy().view(np.int8)
        assert np.array_equal(qs[r], want_qs.reshape(-1)), f"row {r} qs"
        got_d = ds[r, :, 0].copy().view(np.float32)
        assert np.array_equal(got_d.astype(np.float16).view(np.uint16), want_d16) and np.array_equal(
            got_d, want_d16.view(np.float16).astype(np.float32)), f"row {r} d"
        assert np.array_equal(ds[r, :, 1].astype(np.int32), want_qs.astype(np.int32).sum(axis=1)), f"row {r} sums"


def test_act_quant_f16_bf16_inputs_widen_first():
    # k_quants.rs:2652-2686: f16 activations are converted to f32, then quantized
    from candle_amd import _lib
    L = _lib.lib()
    k = 1024
    x32 = normal(23, (2, k), 1.0)
    for tdt, cq in ((torch.float16, 1), (torch.bfloat16, 30)):
        xt = torch.from_numpy(x32).to(tdt).cuda()
        widened = xt.float().cpu().numpy()
        nbytes = L.cq_act_scratch_bytes(oracle.Q4K, k, 2)
        scratch = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        _lib.check("cq_quantize_act", L.cq_quantize_act(oracle.Q4K, xt.data_ptr(), cq, scratch.data_ptr(), k, 2, None))
        torch.cuda.synchronize()
        raw = scratch.cpu().numpy()
        qs = raw[: 2 * k].view(np.int8).reshape(2, k)
        for r in range(2):
            blk = oracle.from_float(oracle.Q8K, widened[r]).reshape(k // 256, 292)
            assert np.array_equal(qs[r], blk[:, 4:260].copy().view(np.int8).reshape(-1))


# ------------------------------------------------------------------------------- QTensor::embedding
def embedding_weight():
    # quantized_tests.rs:265-273
    i = np.arange(8 * 256, dtype=np.float32)
    return (np.sin(i * np.float32(0.003)) * np.float32(0.5) + np.cos(i * np.float32(0.007)) * np.float32(0.25)).astype(np.float32).reshape(8, 256)


@pytest.mark.parametrize("dtype", DTYPES + STORAGE_DTYPES, ids=lambda d: NAMES[d])
def test_quantized_embedding_equals_dequantize_then_index_select(dtype):
    """quantized_tests.rs:287-322 (tolerance 1e-6 there; the rows are bit-identical here), then a larger table with
    repeated and boundary ids."""
    ca = _candle()
    w = embedding_weight()
    blocks = oracle.from_float(dtype, w.reshape(-1))
    q = ca.QTensor.new(ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype)), (8, 256))
    ids = torch.tensor([[3, 1], [3, 7]], dtype=torch.int32)
    got = q.embedding(ids)
    want = oracle.to_float(dtype, blocks, w.size).reshape(8, 256)[[3, 1, 3, 7]].reshape(2, 2, 256)
    assert got.shape == (2, 2, 256) and np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(got, q.dequantize().index_select(0, ids.reshape(-1).cuda().long()).reshape(2, 2, 256))
    rows, hidden = 1000, 768
    big = normal(9, rows * hidden, 0.05)
    bb = oracle.from_float(dtype, big)
    qb = ca.QTensor.new(ca.QStorage.from_data(bb, "cuda", ca.GgmlDType(dtype)), (rows, hidden))
    idb = np.array([0, 999, 5, 5, 512, 0, 998], dtype=np.int64)
    gotb = qb.embedding(torch.from_numpy(idb)).cpu().numpy()
    wantb = oracle.to_float(dtype, bb, big.size).reshape(rows, hidden)[idb]
    assert np.array_equal(gotb.view(np.uint32), wantb.view(np.uint32))
    with pytest.raises(ValueError):
        qb.embedding(torch.tensor([1000]))


def test_embedding_of_plain_arrays_and_launch_rules():
    ca = _candle()
    from candle_amd import _lib
    w = embedding_weight()
    for dt, arr in ((ca.GgmlDType.F32, w), (ca.GgmlDType.F16, w.astype(np.float16))):
        q = ca.QTensor.new(ca.QStorage.from_data(arr.tobytes(), "cuda", dt), (8, 256))
        got = q.embedding(torch.tensor([7, 0])).cpu().numpy()
        assert np.array_equal(got, arr[[7, 0]].astype(np.float32))
    L = _lib.lib()
    blocks = torch.zeros(8 * 144, dtype=torch.uint8, device="cuda")
    ids = torch.tensor([2, 9], dtype=torch.int32, device="cuda")
    out = torch.full((2, 256), 5.0, device="cuda")
    # the launch itself cannot fail on an id: such a row is zeros
    assert L.cq_embedding(12, blocks.data_ptr(), ids.data_ptr(), out.data_ptr(), 2, 8, 256, None) == 0
    torch.cuda.synchronize()
    assert torch.all(out[1] == 0.0)
    assert L.cq_embedding(12, blocks.data_ptr(), ids.data_ptr(), out.data_ptr(), 2, 8, 100, None) == -2
    assert L.cq_embedding(1, blocks.data_ptr(), ids.data_ptr(), out.data_ptr(), 2, 8, 256, None) == -1
