"""Pins the CPU oracle against the known-answer vectors held by the reference's own tests.

Every expected value below is copied (as data) from candle-core/tests/quantized_tests.rs; the line
ranges are cited next to each case.  The inputs are regenerated here by the closed-form recipes the
reference uses (aranges, `get_test_vector2`, `create_ggml_like_vector`, seeded StdRng).
"""
import numpy as np
import pytest

import oracle
from tests import stdrng


def round3(v):
    # quantized_tests.rs:492-498 round_vector: (1000 * x).round() / 1000 in f32, half away from zero
    v = np.asarray(v, dtype=np.float32)
    t = v * np.float32(1000.0)
    r = np.where(t >= 0, np.floor(t + np.float32(0.5)), np.ceil(t - np.float32(0.5))).astype(np.float32)
    return (r / np.float32(1000.0)).astype(np.float32)


def get_test_vector2(bound, size):
    # quantized_tests.rs:476-488
    v = np.arange(size, dtype=np.float32)
    return ((v - np.float32(size / 2.0)) * np.float32(bound) / np.float32(size / 2.0)).astype(np.float32)


def ggml_like_vector(offset):
    # quantized_tests.rs:513-517: 0.1 + 2.0 * cos(i + offset), computed in f32
    i = np.arange(32 * 128, dtype=np.float32) + np.float32(offset)
    return (np.float32(0.1) + np.float32(2.0) * np.cos(i).astype(np.float32)).astype(np.float32)


# ---------------------------------------------------------------- f16 conversion
def test_f16_roundtrip_all_bit_patterns():
    # to_f32 is exact and from_f32 is its inverse on every non-NaN half
    hs = np.arange(1 << 16, dtype=np.uint16)
    np_vals = hs.view(np.float16).astype(np.float32)
    for h in range(0, 1 << 16, 7):
        f = oracle.f16_to_f32(h)
        if np.isnan(np_vals[h]):
            assert np.isnan(f)
            continue
        assert np.float32(f) == np_vals[h] and np.signbit(f) == np.signbit(np_vals[h])
        assert oracle.f32_to_f16(f) == h


def test_f32_to_f16_matches_ieee_rne():
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(0.02),
        rng.standard_normal(2000).astype(np.float32) * np.float32(1e-6),   # subnormal halves
        rng.standard_normal(2000).astype(np.float32) * np.float32(3e4),    # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -26], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- KAT-1 / KAT-2 : Q4_0 matmul
def test_kat_q4_0_matmul_arange():
    # quantized_tests.rs:92-107
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32)
    rhs_t = oracle.from_float(oracle.Q4_0, rhs)
    dst = oracle.matmul(oracle.Q4_0, lhs, rhs_t, n)
    want = [85120.0, 214562.0, 345455.0, 474748.0, 213475.0, 604465.0, 1000686.0, 1388317.0,
            341876.0, 994283.0, 1655709.0, 2301518.0]
    assert np.round(dst.reshape(-1)).tolist() == want


def test_kat_q4_0_matmul_negative():
    # quantized_tests.rs:152-172
    m, k, n = 3, 64, 4
    lhs = (np.arange(m * k, dtype=np.float32) - np.float32(m * k / 2.0)).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32) - np.float32(k * n) / np.float32(3.0)
    rhs_t = oracle.from_float(oracle.Q4_0, rhs)
    dst = oracle.matmul(oracle.Q4_0, lhs, rhs_t, n)
    want = [243524.0, -19596.0, -285051.0, -549815.0, 23777.0, 21651.0, 19398.0, 18367.0,
            -196472.0, 63012.0, 324585.0, 587902.0]
    assert np.round(dst.reshape(-1)).tolist() == want


# ---------------------------------------------------------------- KAT-3 : Q4_0 quantize -> dequantize
def test_kat_q4_0_roundtrip_arange128():
    # quantized_tests.rs:345-374 (all 128 values, exact)
    src = np.arange(128, dtype=np.float32)
    dst = oracle.to_float(oracle.Q4_0, oracle.from_float(oracle.Q4_0, src))
    want = [
        -0.0, -0.0, 3.875, 3.875, 3.875, 3.875, 7.75, 7.75, 7.75, 7.75, 11.625, 11.625, 11.625,
        11.625, 15.5, 15.5, 15.5, 15.5, 19.375, 19.375, 19.375, 19.375, 23.25, 23.25, 23.25,
        23.25, 27.125, 27.125, 27.125, 27.125, 31.0, 31.0, 31.5, 31.5, 31.5, 31.5, 39.375,
        39.375, 39.375, 39.375, 39.375, 39.375, 39.375, 39.375, 47.25, 47.25, 47.25, 47.25,
        47.25, 47.25, 47.25, 47.25, 55.125, 55.125, 55.125, 55.125, 55.125, 55.125, 55.125,
        55.125, 63.0, 63.0, 63.0, 63.0, 59.375, 59.375, 71.25, 71.25, 71.25, 71.25, 71.25,
        71.25, 71.25, 71.25, 71.25, 71.25, 71.25, 71.25, 83.125, 83.125, 83.125, 83.125,
        83.125, 83.125, 83.125, 83.125, 83.125, 83.125, 83.125, 83.125, 95.0, 95.0, 95.0, 95.0,
        95.0, 95.0, 95.25, 95.25, 95.25, 95.25, 95.25, 95.25, 95.25, 95.25, 111.125, 111.125,
        111.125, 111.125, 111.125, 111.125, 111.125, 111.125, 111.125, 111.125, 111.125,
        111.125, 111.125, 111.125, 111.125, 111.125, 127.0, 127.0, 127.0, 127.0, 127.0, 127.0,
        127.0, 127.0,
    ]
    assert dst.tolist() == want
    # the reference prints -0.0 for the first two entries: the sign bit must match as well
    assert np.signbit(dst[0]) and np.signbit(dst[1])


# ---------------------------------------------------------------- KAT-9..12 : K-quant spot values + bounds
KQUANT_CASES = [
    # dtype, spot values at [0,128,256,512,800,1023], tol(bound .5), tol(bound 128)   (source lines)
    (oracle.Q4K, [-0.5, -0.373, -0.25, 0.0, 0.288, 0.498], 0.017, 4.5),    # :855-890
    (oracle.Q5K, [-0.5, -0.373, -0.25, 0.0, 0.279, 0.499], 0.009, 2.5),    # :896-937
    (oracle.Q6K, [-0.497, -0.372, -0.25, -0.0, 0.284, 0.5], 0.008, 2.0),   # :943-984
    (oracle.Q8K, [-0.5, -0.374, -0.25, -0.0, 0.283, 0.499], 0.008, 0.6),   # :990-1031
]


@pytest.mark.parametrize("dtype,spots,tol_small,tol_big", KQUANT_CASES)
def test_kat_kquant_test_vector2(dtype, spots, tol_small, tol_big):
    src = get_test_vector2(0.5, 1024)
    assert [src[0], src[128], src[256], src[512], src[800], src[1023]] == [-0.5, -0.375, -0.25, 0.0, 0.28125, np.float32(0.49902344)]
    dst = oracle.to_float(dtype, oracle.from_float(dtype, src))
    assert np.all(np.abs(dst - src) < tol_small)
    got = round3(dst)[[0, 128, 256, 512, 800, 1023]]
    assert got.tolist() == [float(np.float32(s)) for s in spots]
    big = get_test_vector2(128.0, 1024)
    dst_big = oracle.to_float(dtype, oracle.from_float(dtype, big))
    assert np.all(np.abs(dst_big - big) < tol_big)


# ---------------------------------------------------------------- KAT-4..6 : Q4_1, Q5_0, Q5_1 on 0..127
Q4_1_WANT = [v for base in (0.0, 32.0, 64.0, 96.0) for v in
             ([base, base] + [x for q in (2.066, 4.133, 6.199, 8.266, 10.332, 12.398, 14.465, 16.531, 18.598, 20.664, 22.73, 24.797,
                                          26.863, 28.93, 30.996) for x in (base + q, base + q)])]      # quantized_tests.rs:392-406
Q5_0_WANT = [-0.0, 1.938, 1.938, 3.875, 3.875, 5.813, 5.813, 7.75, 7.75, 9.688, 9.688, 11.625,
             11.625, 13.563, 13.563, 15.5, 15.5, 17.438, 17.438, 19.375, 19.375, 21.313, 21.313,
             23.25, 23.25, 25.188, 25.188, 27.125, 27.125, 29.063, 29.063, 31.0, 31.5, 31.5, 35.438,
             35.438, 35.438, 35.438, 39.375, 39.375, 39.375, 39.375, 43.313, 43.313, 43.313, 43.313,
             47.25, 47.25, 47.25, 47.25, 51.188, 51.188, 51.188, 51.188, 55.125, 55.125, 55.125,
             55.125, 59.063, 59.063, 59.063, 59.063, 63.0, 63.0, 65.313, 65.313, 65.313, 65.313,
             65.313, 71.25, 71.25, 71.25, 71.25, 71.25, 71.25, 77.188, 77.188, 77.188, 77.188,
             77.188, 77.188, 83.125, 83.125, 83.125, 83.125, 83.125, 83.125, 89.063, 89.063, 89.063,
             89.063, 89.063, 89.063, 95.0, 95.0, 95.0, 95.25, 95.25, 95.25, 95.25, 103.188, 103.188,
             103.188, 103.188, 103.188, 103.188, 103.188, 103.188, 111.125, 111.125, 111.125,
             111.125, 111.125, 111.125, 111.125, 111.125, 119.063, 119.063, 119.063, 119.063,
             119.063, 119.063, 119.063, 119.063, 127.0, 127.0, 127.0, 127.0]                            # :425-438


def test_kat_q4_1_q5_0_q5_1_roundtrip_arange128():
    src = np.arange(128, dtype=np.float32)
    got = round3(oracle.to_float(oracle.Q4_1, oracle.from_float(oracle.Q4_1, src)))
    assert got.tolist() == [float(round3([v])[0]) for v in Q4_1_WANT]
    got = round3(oracle.to_float(oracle.Q5_0, oracle.from_float(oracle.Q5_0, src)))
    assert got.tolist() == [float(np.float32(v)) for v in Q5_0_WANT]
    got = round3(oracle.to_float(oracle.Q5_1, oracle.from_float(oracle.Q5_1, src)))             # :458-470: exact
    assert got.tolist() == src.tolist()


# ---------------------------------------------------------------- KAT-7..8 : Q2K, Q3K spot values + bounds
@pytest.mark.parametrize("dtype,spots,tol_small,tol_big", [
    (oracle.Q2K, [-0.499, -0.366, -0.249, 0.0, 0.295, 0.492], 0.1, 6.0),       # :751-797
    (oracle.Q3K, [-0.493, -0.37, -0.243, -0.0, 0.292, 0.492], 0.03, 3.5),      # :799-844
])
def test_kat_q2k_q3k_test_vector2(dtype, spots, tol_small, tol_big):
    src = get_test_vector2(0.5, 1024)
    dst = oracle.to_float(dtype, oracle.from_float(dtype, src))
    assert np.all(np.abs(dst - src) < tol_small)
    got = round3(dst)[[0, 128, 256, 512, 800, 1023]]
    assert got.tolist() == [float(np.float32(s)) for s in spots]
    big = get_test_vector2(128.0, 1024)
    dst_big = oracle.to_float(dtype, oracle.from_float(dtype, big))
    assert np.all(np.abs(dst_big - big) < tol_big)


@pytest.mark.parametrize("dtype,ceiling", [(oracle.Q4_1, 0.002), (oracle.Q5_0, 0.002), (oracle.Q5_1, 0.002), (oracle.Q8_1, 0.002),
                                           (oracle.Q2K, 0.0075), (oracle.Q3K, 0.004)])
def test_bound_quantization_rmse_remaining_formats(dtype, ceiling):
    # quantized_tests.rs:12-17,531-552 with the 2-bit / 3-bit ceilings of :14-15
    src = ggml_like_vector(0.0)
    dst = oracle.to_float(dtype, oracle.from_float(dtype, src))
    err = np.sqrt(np.sum((src - dst).astype(np.float32) ** 2, dtype=np.float32)) / np.float32(src.size)
    assert err <= ceiling


def test_q8_1_closed_form():
    """No vector in the reference: Q8_1 is the Q8_0 quantizer (same d, same int8 values in the same order) plus
    s = f16(f16(sum) * d) (k_quants.rs:770-799)."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(32 * 40) * 3).astype(np.float32)
    b1 = oracle.from_float(oracle.Q8_1, x).reshape(-1, 36)
    b0 = oracle.from_float(oracle.Q8_0, x).reshape(-1, 34)
    assert np.array_equal(b1[:, :2], b0[:, :2]) and np.array_equal(b1[:, 4:], b0[:, 2:])
    d = b1[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    sums = b1[:, 4:].copy().view(np.int8).astype(np.int32).sum(axis=1)
    want_s = (sums.astype(np.float32).astype(np.float16).astype(np.float32) * d).astype(np.float16)
    assert np.array_equal(b1[:, 2:4].copy().view(np.float16).reshape(-1), want_s)
    assert np.array_equal(oracle.to_float(oracle.Q8_1, b1.reshape(-1)), oracle.to_float(oracle.Q8_0, b0.reshape(-1)))


# ---------------------------------------------------------------- BOUND-1 : ggml quantization RMSE ceiling
@pytest.mark.parametrize("dtype", [oracle.Q4_0, oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q8K])
def test_bound_quantization_rmse(dtype):
    # quantized_tests.rs:12-17,511-552: sqrt(sum((a-b)^2)) / len <= 0.002
    src = ggml_like_vector(0.0)
    dst = oracle.to_float(dtype, oracle.from_float(dtype, src))
    err = np.sqrt(np.sum((src - dst).astype(np.float32) ** 2, dtype=np.float32)) / np.float32(src.size)
    assert err <= 0.002


# ---------------------------------------------------------------- BOUND-2 : dot-product error vs ggml ceilings
GGML_DOT_ERR = {oracle.Q4_0: 0.001143, oracle.Q8_0: 0.000092, oracle.Q4K: 0.002425, oracle.Q5K: 0.000740,
                oracle.Q6K: 0.000952, oracle.Q8K: 0.00065,   # quantized_tests.rs:1101-1122
                oracle.Q2K: 0.004086, oracle.Q3K: 0.017, oracle.Q4_1: 0.008, oracle.Q5_0: 0.001353, oracle.Q5_1: 0.00149}


@pytest.mark.parametrize("dtype", list(GGML_DOT_ERR))
def test_bound_dot_product_error(dtype):
    # quantized_tests.rs:1126-1191
    cases = [(ggml_like_vector(0.0), ggml_like_vector(1.0), 1.0)]
    ramp = (np.arange(4096, dtype=np.float32) / np.float32(4096.0)).astype(np.float32)
    cases.append((ramp, ramp, 2.0))
    for a, b, err_m in cases:
        n = a.size
        aq = oracle.from_float(dtype, a)
        bq = oracle.from_float(oracle.vec_dot_type(dtype), b)
        res = oracle.vec_dot(dtype, n, aq, bq)
        res_mm = float(oracle.matmul(dtype, b.reshape(1, n), aq, 1)[0, 0])
        assert abs(res_mm - res) / n <= 1e-6                       # matmul(1,len,1) == vec_dot
        ref = float(np.sum(a * b, dtype=np.float32))
        for r in (res, res_mm):
            err = abs(r - ref) / n
            assert np.isfinite(err) and err <= 0.02
            assert err - 1e-5 <= GGML_DOT_ERR[dtype] * err_m


# ---------------------------------------------------------------- KAT-13..18 : seeded random matmuls
def test_stdrng_restatement_pinned_by_f32_goldens():
    # quantized_tests.rs:1383-1392: the un-quantized product of the seeded draws
    m, k, n = 11, 512, 21
    lhs, rhs = stdrng.get_random_tensors(m, k, n)
    assert lhs.min() >= -0.5 and lhs.max() < 0.5
    mm = (lhs.astype(np.float64) @ rhs.astype(np.float64).T).astype(np.float32).reshape(-1)
    got = round3([mm[0], mm[m * n // 3], mm[m * n * 2 // 3], mm[m * n - 1]])
    assert got.tolist() == [float(np.float32(v)) for v in (1.262, 1.513, -0.208, 1.702)]


SEEDED_MATMUL = [
    (oracle.Q4K, [1.094, 1.442, -0.196, 1.587]),   # quantized_tests.rs:1383-1407
    (oracle.Q5K, [1.161, 1.498, -0.175, 1.739]),   # :1409-1434
    (oracle.Q6K, [1.293, 1.497, -0.159, 1.737]),   # :1436-1459
    (oracle.Q8K, [1.241, 1.52, -0.2, 1.7]),        # :1461-1483
    (oracle.Q2K, [0.887, 0.428, 0.219, 1.669]),    # :1331-1354
    (oracle.Q3K, [1.001, 1.425, -0.311, 1.493]),   # :1357-1380
]


@pytest.mark.parametrize("dtype,want", SEEDED_MATMUL)
def test_kat_seeded_matmul(dtype, want):
    m, k, n = 11, 512, 21
    lhs, rhs = stdrng.get_random_tensors(m, k, n)
    w = oracle.from_float(dtype, rhs.reshape(-1))
    mm = oracle.matmul(dtype, lhs, w, n).reshape(-1)
    got = round3([mm[0], mm[m * n // 3], mm[m * n * 2 // 3], mm[m * n - 1]])
    assert got.tolist() == [float(np.float32(v)) for v in want]


# ---------------------------------------------------------------- test_matmul (1,3,4,256) mean relative error
@pytest.mark.parametrize("dtype", [oracle.Q4_0, oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q8K,
                                   oracle.Q4_1, oracle.Q5_0, oracle.Q5_1, oracle.Q2K, oracle.Q3K])
def test_matmul_relative_error_ramp(dtype):
    # quantized_tests.rs:19-54 with (b,m,n,k) = (1,3,4,256): mean |mm - res| / |mm| <= 0.02
    m, n, k = 3, 4, 256
    lhs = (np.arange(m * k, dtype=np.float32) / np.float32(m * k)).reshape(m, k)
    rhs = (np.arange(k * n, dtype=np.float32) / np.float32(n * k)).reshape(k, n)
    mm = lhs @ rhs
    w = oracle.from_float(dtype, np.ascontiguousarray(rhs.T).reshape(-1))
    res = oracle.matmul(dtype, lhs, w, n)
    err = float(np.sum(np.abs(mm - res) / np.abs(mm))) / (m * n)
    assert err <= 0.02


# ---------------------------------------------------------------- INV-1 : batching invariance
@pytest.mark.parametrize("dtype", [oracle.Q4_0, oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K,
                                   oracle.Q4_1, oracle.Q5_0, oracle.Q5_1, oracle.Q2K, oracle.Q3K])
def test_batching_invariance(dtype):
    # quantized_tests.rs:224-259: the same rows give bit-identical outputs at any batch size on the CPU
    lhs, rhs = stdrng.get_random_tensors(2, 256, 6)
    w = oracle.from_float(dtype, rhs.reshape(-1))
    mm = oracle.matmul(dtype, lhs, w, 6)
    mm6 = oracle.matmul(dtype, np.concatenate([lhs, lhs, lhs]), w, 6)
    for i in range(3):
        assert np.array_equal(mm6[2 * i:2 * i + 2].view(np.uint32), mm.view(np.uint32))


# ---------------------------------------------------------------- vec_dot of Q4_1, Q5_0, Q5_1, Q2_K, Q3_K
# byte offsets of the f16 fields (d, m / dmin) inside a block, k_quants.rs:86-147
F16_FIELDS = {oracle.Q4_1: (0, 2), oracle.Q5_0: (0,), oracle.Q5_1: (0, 2), oracle.Q2K: (80, 82), oracle.Q3K: (108,),
              oracle.Q4_0: (0,), oracle.Q8_0: (0,), oracle.Q4K: (0, 2), oracle.Q5K: (0, 2), oracle.Q6K: (208,)}


def random_weight_blocks(dtype, nblocks, rng):
    """Random block bytes (every bit of qs / qh / hmask / scales in play) with finite f16 scale fields."""
    ts = oracle.type_size(dtype)
    b = rng.integers(0, 256, size=(nblocks, ts), dtype=np.uint8)
    for off in F16_FIELDS[dtype]:
        h = rng.uniform(-2.0, 2.0, size=nblocks).astype(np.float16).view(np.uint16)
        b[:, off] = (h & 0xff).astype(np.uint8)
        b[:, off + 1] = (h >> 8).astype(np.uint8)
    return b.reshape(-1)


def exact_activations(n, rng):
    """Activations every CPU quantizer represents exactly: x = 2^e * q with integer |q| <= 60 and one 127 per 32-element
    block (so d = amax / 127 = 2^e, q is recovered unchanged, |sum q| <= 2048 and the Q8_1 field s = d * sum is exact)."""
    q = rng.integers(-60, 61, size=n).astype(np.float32)
    q[np.arange(0, n, 32) + rng.integers(0, 32, size=n // 32)] = 127.0
    return (q * np.float32(2.0 ** -5)).astype(np.float32)


@pytest.mark.parametrize("dtype", list(F16_FIELDS))
def test_vec_dot_is_the_dot_product_of_the_dequantized_operands(dtype):
    # With exactly representable activations vec_dot(w, q(a)) is, in real arithmetic, sum(to_float(w) * to_float(q(a))):
    # the pinned to_float functions fix every index, shift, mask, offset and scale of the integer part; what is left is
    # f32 rounding of the block sums.  A wrong nibble / high-bit / sub-block pairing changes the value by O(1).
    rng = np.random.default_rng(1234 + dtype)
    n = 1024
    vdt = oracle.vec_dot_type(dtype)
    for _ in range(8):
        w = random_weight_blocks(dtype, n // oracle.block_size(dtype), rng)
        a = exact_activations(n, rng)
        aq = oracle.from_float(vdt, a)
        assert np.array_equal(oracle.to_float(vdt, aq), a)
        wf = oracle.to_float(dtype, w).astype(np.float64)
        want = float(np.sum(wf * a.astype(np.float64)))
        scale = float(np.sum(np.abs(wf * a.astype(np.float64))))
        got = oracle.vec_dot(dtype, n, w, aq)
        assert abs(got - want) <= 2e-6 * scale
        assert abs(float(oracle.matmul(dtype, a.reshape(1, n), w, 1)[0, 0]) - got) <= 1e-6 * scale
