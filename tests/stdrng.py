"""Restatement of the random generator behind candle's seeded matmul tests.

candle-core/tests/quantized_tests.rs:1208-1228 draws its inputs from rand 0.9
`StdRng::seed_from_u64(314159265358979)` followed by `rng.random::<f32>() - 0.5`.  The `rand` crate
is not vendored in the reference tree, so its published algorithm is restated here:

  * `seed_from_u64` expands the u64 with PCG32 (multiplier 6364136223846793005, increment
    11634580027462260723, XSH-RR output) into 8 little-endian key words;
  * `StdRng` is ChaCha with 12 rounds, 64-bit block counter starting at 0 in words 12-13, stream id 0
    in words 14-15; output words are consumed in order, block after block;
  * `random::<f32>()` keeps the top 24 bits of one u32: (x >> 8) * 2**-24.

The restatement is pinned by the reference's own f32 golden values for the un-quantized matmul of
these draws (quantized_tests.rs:1392), checked in tests/test_oracle_kat.py.
"""
import numpy as np

_MASK64 = (1 << 64) - 1


def _pcg32_seed_words(state: int) -> list[int]:
    words = []
    for _ in range(8):
        state = (state * 6364136223846793005 + 11634580027462260723) & _MASK64
        xorshifted = (((state >> 18) ^ state) >> 27) & 0xFFFFFFFF
        rot = state >> 59
        words.append(((xorshifted >> rot) | (xorshifted << ((32 - rot) & 31))) & 0xFFFFFFFF)
    return words


def _rotl(x: np.ndarray, r: int) -> np.ndarray:
    return (x << np.uint32(r)) | (x >> np.uint32(32 - r))


def _quarter(s, a, b, c, d):
    s[a] += s[b]; s[d] = _rotl(s[d] ^ s[a], 16)
    s[c] += s[d]; s[b] = _rotl(s[b] ^ s[c], 12)
    s[a] += s[b]; s[d] = _rotl(s[d] ^ s[a], 8)
    s[c] += s[d]; s[b] = _rotl(s[b] ^ s[c], 7)


def chacha12_words(seed_u64: int, n_words: int) -> np.ndarray:
    """First n_words u32 outputs of StdRng::seed_from_u64(seed_u64)."""
    key = _pcg32_seed_words(seed_u64)
    n_blocks = (n_words + 15) // 16
    ctr = np.arange(n_blocks, dtype=np.uint64)
    init = [np.full(n_blocks, c, dtype=np.uint32) for c in (0x61707865, 0x3320646E, 0x79622D32, 0x6B206574)]
    init += [np.full(n_blocks, w, dtype=np.uint32) for w in key]
    init += [(ctr & np.uint64(0xFFFFFFFF)).astype(np.uint32), (ctr >> np.uint64(32)).astype(np.uint32)]
    init += [np.zeros(n_blocks, dtype=np.uint32), np.zeros(n_blocks, dtype=np.uint32)]
    s = [w.copy() for w in init]
    with np.errstate(over="ignore"):
        for _ in range(6):  # 12 rounds = 6 double rounds
            _quarter(s, 0, 4, 8, 12); _quarter(s, 1, 5, 9, 13); _quarter(s, 2, 6, 10, 14); _quarter(s, 3, 7, 11, 15)
            _quarter(s, 0, 5, 10, 15); _quarter(s, 1, 6, 11, 12); _quarter(s, 2, 7, 8, 13); _quarter(s, 3, 4, 9, 14)
        out = np.stack([s[i] + init[i] for i in range(16)], axis=1)  # [block, word]
    return out.reshape(-1)[:n_words]


def random_f32(seed_u64: int, count: int) -> np.ndarray:
    """`count` successive `rng.random::<f32>()` draws as float32 in [0, 1)."""
    w = chacha12_words(seed_u64, count)
    return ((w >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)).astype(np.float32)


def get_random_tensors(m: int, k: int, n: int):
    """quantized_tests.rs:1208-1228: lhs [m,k] is drawn before rhs [n,k], each value `random() - 0.5`."""
    draws = random_f32(314159265358979, (m + n) * k) - np.float32(0.5)
    lhs = draws[: m * k].reshape(m, k).astype(np.float32)
    rhs = draws[m * k:].reshape(n, k).astype(np.float32)
    return lhs, rhs
