"""GPU parity for the expert-grouped quantized matmul: QTensor::indexed_moe_forward and
candle_nn::moe::moe_gemm_gguf, against the CPU oracle's per-pair composition of k_quants::matmul.
The reference has no tests for these kernels and no CPU implementation (mod.rs:776-782); the
oracle functions are pinned by brute force in tests/test_oracle_moe.py.
"""
import numpy as np
import pytest
import torch

import oracle
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

TOL = 1e-3
TIGHT = 2e-6
WDTYPES = [oracle.Q8_0, oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q4_0, oracle.Q2K, oracle.Q3K]
NAMES = {oracle.Q4_0: "q4_0", oracle.Q8_0: "q8_0", oracle.Q4K: "q4k", oracle.Q5K: "q5k", oracle.Q6K: "q6k", oracle.Q2K: "q2k", oracle.Q3K: "q3k"}


def make_experts(dtype, E, n, k, seed):
    import candle_amd as ca
    w = normal(seed, (E, n, k), 0.02)
    blocks = oracle.from_float(dtype, w.reshape(-1))
    qt = ca.QTensor.new(ca.QStorage.from_data(blocks, "cuda", ca.GgmlDType(dtype)), (E, n, k))
    return blocks, qt


def route(tokens, E, topk, seed):
    """Router of fused_moe.rs:222-260 on random logits: top-k ids + renormalised softmax weights,
    then the flattened expert list sorted ascending with the matching token-slot permutation."""
    rng = np.random.Generator(np.random.PCG64(seed))
    logits = rng.standard_normal((tokens, E)).astype(np.float32)
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    ids = np.argsort(-p, axis=1, kind="stable")[:, :topk].astype(np.uint32)
    w = np.take_along_axis(p, ids.astype(np.int64), axis=1)
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    flat = ids.reshape(-1).astype(np.int32)
    order = np.argsort(flat, kind="stable").astype(np.int32)
    return ids, w, flat[order], order


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("input_dim1_is_one", [True, False])
def test_indexed_moe_forward(dtype, input_dim1_is_one):
    E, n, k, batch, topk = 8, 48, 512, 5, 3
    blocks, qt = make_experts(dtype, E, n, k, seed=5)
    ids, _, _, _ = route(batch, E, topk, seed=6)
    x = normal(7, (batch, 1 if input_dim1_is_one else topk, k), 1.0)
    out = qt.indexed_moe_forward(torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda())
    torch.cuda.synchronize()
    want = oracle.indexed_moe_forward(dtype, blocks, (E, n, k), x, ids)
    assert out.shape == (batch, topk, n)
    err = rel_l2(out.cpu().numpy(), want)
    assert err <= TOL and err <= TIGHT, err


@pytest.mark.parametrize("dtype", WDTYPES, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("tokens", [1, 16, 40, 100, 300])  # <= 256 pairs: a fused matvec per pair; beyond: grouped by expert, 8 pairs per
                                                           # pass (Q4_0 / Q8_0) or expert tiles of 32 / 128 rows through the MFMA kernel (K-quants)
@pytest.mark.parametrize("is_prefill", [False, True])
def test_moe_gemm_gguf_gate_and_down(dtype, tokens, is_prefill):
    """The two call shapes of FusedMoeGGUF::forward (fused_moe.rs:263-294): gate/up without
    topk_weights on [tokens, k], down with topk_weights on [tokens*topk, k]."""
    import candle_amd as ca
    E, n, k, topk = 16, 64, 256, 4
    blocks, qt = make_experts(dtype, E, n, k, seed=15)
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=16 + tokens)
    sti = torch.from_numpy(sorted_token_ids).cuda()
    eid = torch.from_numpy(expert_ids).cuda()

    x = normal(17, (tokens, k), 1.0)
    got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, None, sti, eid, topk, is_prefill)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(dtype, x, blocks, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    assert got.shape == (tokens * topk, n)
    err = rel_l2(got.cpu().numpy(), want)
    assert err <= TOL and err <= TIGHT, err

    x2 = normal(18, (tokens * topk, k), 1.0)
    twf = tw.reshape(-1)
    got2 = ca.moe_gemm_gguf(torch.from_numpy(x2).cuda(), qt, torch.from_numpy(twf).cuda(), sti, eid, topk, is_prefill)
    torch.cuda.synchronize()
    want2 = oracle.moe_gemm_gguf(dtype, x2, blocks, (E, n, k), sorted_token_ids, expert_ids, twf, topk)
    err2 = rel_l2(got2.cpu().numpy(), want2)
    assert err2 <= TOL and err2 <= TIGHT, err2


@pytest.mark.parametrize("wdt", [oracle.Q4K, oracle.Q5K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k,n", [(256, 64), (512, 40), (768, 203), (1024, 130), (1792, 50), (2048, 96), (2304, 33), (4096, 72)])
@pytest.mark.parametrize("with_weights", [False, True])
def test_moe_gemm_gguf_experts_as_batched_matvecs(wdt, k, n, with_weights):
    """Q4_K or Q5_K experts hit by at most 64 pairs on average run as batched matvecs over their own pairs (sets of 16, two sets per pass
    over the weights).  Expert loads on every edge: none, one pair, 15 / 16 / 17, 31 / 32 / 33 (a second pass), 47 .. 49, 65 (a
    third pass); rows of 1 .. 16 super-blocks (one to eight waves per row block, columns without a wave's second column), ragged
    n, several workgroups per expert."""
    import candle_amd as ca
    counts = [0, 1, 15, 16, 17, 31, 32, 33, 47, 48, 49, 65, 0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 13]
    E, topk = len(counts), 2
    n_pairs = sum(counts)
    assert n_pairs % topk == 0 and 257 <= n_pairs <= 64 * E
    tokens = n_pairs // topk
    blocks, qt = make_experts(wdt, E, n, k, seed=91)
    rng = np.random.Generator(np.random.PCG64(92))
    expert_ids = np.repeat(np.arange(E, dtype=np.int32), counts)
    sorted_token_ids = rng.permutation(n_pairs).astype(np.int32)
    sti, eid = torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda()
    if with_weights:
        x = normal(93, (n_pairs, k), 1.0)
        tw = rng.uniform(0.1, 1.0, n_pairs).astype(np.float32)
        got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, torch.from_numpy(tw).cuda(), sti, eid, topk, True)
    else:
        x = normal(94, (tokens, k), 1.0)
        tw = None
        got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, None, sti, eid, topk, True)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(wdt, x, blocks, (E, n, k), sorted_token_ids, expert_ids, tw, topk)
    got = got.cpu().numpy()
    assert got.shape == (n_pairs, n)
    err = rel_l2(got, want)
    assert err <= TOL and err <= TIGHT, err
    # pair by pair as well: a pair in the wrong slot of its set would hide in the norm of hundreds of rows
    for p in range(n_pairs):
        assert rel_l2(got[p], want[p]) <= 1e-5, (p, int(expert_ids[np.where(sorted_token_ids == p)[0][0]]))


@pytest.mark.parametrize("dtype", [oracle.Q4K, oracle.Q5K, oracle.Q6K, oracle.Q2K, oracle.Q3K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("E,n", [(64, 160), (8, 160)])      # 1200 pairs: about 19 rows per expert (32-row tiles of the MFMA
                                                            # kernel, 128 weight rows wide) or 150 (128-row tiles); n is ragged
def test_moe_gemm_gguf_mfma_tile_sizes(dtype, E, n):
    import candle_amd as ca
    k, topk, tokens = 512, 4, 300
    blocks, qt = make_experts(dtype, E, n, k, seed=65)
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=66)
    sti, eid = torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda()
    x2 = normal(67, (tokens * topk, k), 1.0)
    twf = tw.reshape(-1)
    got = ca.moe_gemm_gguf(torch.from_numpy(x2).cuda(), qt, torch.from_numpy(twf).cuda(), sti, eid, topk, True)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(dtype, x2, blocks, (E, n, k), sorted_token_ids, expert_ids, twf, topk)
    err = rel_l2(got.cpu().numpy(), want)
    assert err <= TIGHT, err


@pytest.mark.parametrize("wdt", [oracle.Q4K, oracle.Q5K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k,n", [(2048, 96), (768, 203)])
def test_moe_gemm_gguf_one_expert_draws_most_pairs(wdt, k, n):
    """A router far from balanced: one expert with 300 of 432 pairs (ten passes over its weights, of which nine are shared out
    among the workgroups of the launch as they finish), two with 40, the rest with none or a few."""
    import candle_amd as ca
    counts = [300, 40, 40, 0, 0, 7, 0, 1, 0, 12, 0, 0, 0, 3, 0, 29]
    E, topk = len(counts), 2
    n_pairs = sum(counts)
    assert n_pairs % topk == 0 and 257 <= n_pairs <= 64 * E
    blocks, qt = make_experts(wdt, E, n, k, seed=95)
    rng = np.random.Generator(np.random.PCG64(96))
    expert_ids = np.repeat(np.arange(E, dtype=np.int32), counts)
    sorted_token_ids = rng.permutation(n_pairs).astype(np.int32)
    x = normal(97, (n_pairs, k), 1.0)
    tw = rng.uniform(0.1, 1.0, n_pairs).astype(np.float32)
    got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, torch.from_numpy(tw).cuda(), torch.from_numpy(sorted_token_ids).cuda(),
                           torch.from_numpy(expert_ids).cuda(), topk, True)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(wdt, x, blocks, (E, n, k), sorted_token_ids, expert_ids, tw, topk)
    got = got.cpu().numpy()
    for p in range(n_pairs):
        assert rel_l2(got[p], want[p]) <= 1e-5, p
    # a second call on the same workspace draws from counters that the grouping pass has set back to zero
    got2 = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, torch.from_numpy(tw).cuda(), torch.from_numpy(sorted_token_ids).cuda(),
                            torch.from_numpy(expert_ids).cuda(), topk, True).cpu().numpy()
    assert np.array_equal(got, got2)


def test_moe_gemm_gguf_q4k_rows_too_long_for_the_batched_form():
    """Q4_K experts with rows of more than 16 super-blocks do not run as batched matvecs: 25 pairs per expert go through the
    32-row tiles of the Q4_K matrix-core kernel."""
    import candle_amd as ca
    E, n, k, topk, tokens = 16, 96, 4352, 4, 100
    blocks, qt = make_experts(oracle.Q4K, E, n, k, seed=75)
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=76)
    sti, eid = torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda()
    x2 = normal(77, (tokens * topk, k), 1.0)
    twf = tw.reshape(-1)
    got = ca.moe_gemm_gguf(torch.from_numpy(x2).cuda(), qt, torch.from_numpy(twf).cuda(), sti, eid, topk, True)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(oracle.Q4K, x2, blocks, (E, n, k), sorted_token_ids, expert_ids, twf, topk)
    err = rel_l2(got.cpu().numpy(), want)
    assert err <= TIGHT, err


@pytest.mark.parametrize("dtype", [oracle.Q4K, oracle.Q6K, oracle.Q8_0], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("tokens", [10, 300])               # 40 pairs: two plain calls; 1200 pairs: one grouping for both (K-quants)
def test_moe_gemm_gguf_pair_equals_two_calls(dtype, tokens):
    """cq_moe_gemm_gguf_pair (gate and up of an expert MLP in one call) gives what two cq_moe_gemm_gguf calls give."""
    import candle_amd as ca
    from candle_amd import _lib
    lib = _lib.lib()
    E, n, k, topk = 16, 96, 512, 4
    blocks_a, qa = make_experts(dtype, E, n, k, seed=75)
    blocks_b, qb = make_experts(dtype, E, n, k, seed=76)
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=77)
    sti, eid = torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda()
    x = torch.from_numpy(normal(78, (tokens, k), 1.0)).cuda()
    pairs = tokens * topk
    wsb = lib.cq_moe_gemm_workspace_bytes(int(dtype), E, topk, pairs, n, k, 0)
    ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device="cuda")
    out_a, out_b = torch.full((pairs, n), 7.0, device="cuda"), torch.full((pairs, n), 7.0, device="cuda")
    _lib.check("pair", lib.cq_moe_gemm_gguf_pair(int(dtype), x.data_ptr(), qa.device_ptr(), qb.device_ptr(), sti.data_ptr(), eid.data_ptr(),
                                                 out_a.data_ptr(), out_b.data_ptr(), E, topk, pairs, n, k, 1, ws.data_ptr(), wsb, None))
    one_a = ca.moe_gemm_gguf(x, qa, None, sti, eid, topk, True)
    one_b = ca.moe_gemm_gguf(x, qb, None, sti, eid, topk, True)
    torch.cuda.synchronize()
    assert np.array_equal(out_a.cpu().numpy(), one_a.cpu().numpy()) and np.array_equal(out_b.cpu().numpy(), one_b.cpu().numpy())
    want_b = oracle.moe_gemm_gguf(dtype, x.cpu().numpy(), blocks_b, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    assert rel_l2(out_b.cpu().numpy(), want_b) <= TIGHT
    assert lib.cq_moe_gemm_gguf_pair(int(dtype), x.data_ptr(), qa.device_ptr(), qb.device_ptr(), sti.data_ptr(), eid.data_ptr(),
                                     out_a.data_ptr(), out_b.data_ptr(), E, topk, pairs, n, k, 1, ws.data_ptr(), 16, None) == -5


@pytest.mark.parametrize("batch", [4, 120, 400])            # 12 pairs (per-pair kernels), 360 (grouped matvec), 1200 (MFMA tiles)
def test_indexed_moe_forward_out_of_range_id_gives_zero_row(batch):
    import candle_amd as ca
    E, n, k, topk = 8, 48, 512, 3
    blocks, qt = make_experts(oracle.Q4K, E, n, k, seed=55)
    ids, _, _, _ = route(batch, E, topk, seed=56)
    ids = ids.astype(np.int64)
    ids[1, 2] = E + 3                                        # not an expert
    x = normal(57, (batch, 1, k), 1.0)
    out = qt.indexed_moe_forward(torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda())
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(got[1, 2] == 0.0)
    good = ids.copy()
    good[1, 2] = 0
    want = oracle.indexed_moe_forward(oracle.Q4K, blocks, (E, n, k), x, good.astype(np.uint32))
    mask = np.ones((batch, topk), dtype=bool)
    mask[1, 2] = False
    assert rel_l2(got[mask], want[mask]) <= TIGHT


def test_moe_gemm_is_invariant_to_pair_order():
    # the reference sorts with an unstable sort (candle-core/src/sort.rs:282-297): any order of the pairs
    # inside an expert segment, and indeed any permutation of the pair list, must give the same output
    import candle_amd as ca
    E, n, k, topk, tokens = 16, 64, 256, 4, 24
    blocks, qt = make_experts(oracle.Q4K, E, n, k, seed=25)
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=26)
    x = torch.from_numpy(normal(27, (tokens, k), 1.0)).cuda()
    base = ca.moe_gemm_gguf(x, qt, None, torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda(), topk, False)
    perm = np.random.Generator(np.random.PCG64(28)).permutation(expert_ids.size)
    shuf = ca.moe_gemm_gguf(x, qt, None, torch.from_numpy(sorted_token_ids[perm].copy()).cuda(),
                            torch.from_numpy(expert_ids[perm].copy()).cuda(), topk, False)
    torch.cuda.synchronize()
    assert torch.equal(base, shuf)


def test_moe_gemm_skips_invalid_experts():
    import candle_amd as ca
    E, n, k, topk, tokens = 4, 32, 256, 2, 3
    blocks, qt = make_experts(oracle.Q4K, E, n, k, seed=35)
    expert_ids = np.array([0, 1, -1, 2, 7, 3], dtype=np.int32)     # -1 and 7 are outside [0, E)
    sorted_token_ids = np.arange(6, dtype=np.int32)
    x = normal(36, (tokens, k), 1.0)
    out = torch.full((6, n), 123.0, device="cuda")
    from candle_amd import _lib
    L = _lib.lib()
    xs = torch.from_numpy(x).cuda()
    sti = torch.from_numpy(sorted_token_ids).cuda()
    eid = torch.from_numpy(expert_ids).cuda()
    need = L.cq_moe_gemm_workspace_bytes(int(ca.GgmlDType.Q4K), E, topk, 6, n, k, 0)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    _lib.check("cq_moe_gemm_gguf", L.cq_moe_gemm_gguf(int(ca.GgmlDType.Q4K), xs.data_ptr(), qt.device_ptr(), sti.data_ptr(), eid.data_ptr(),
                                                      None, out.data_ptr(), E, topk, 6, n, k, 0, ws.data_ptr(), need, None))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(got[2] == 123.0) and np.all(got[4] == 123.0)          # skipped rows untouched (moe_gguf.cu:91)
    want = oracle.moe_gemm_gguf(oracle.Q4K, x, blocks, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    keep = [0, 1, 3, 5]
    assert rel_l2(got[keep], want[keep]) <= TIGHT


def test_moe_qwen3_shape_single_token():
    # BASELINE configs[4] shape: 128 experts, top-8, hidden 2048, expert FFN 768, Q4_K; one token
    import candle_amd as ca
    E, topk = 128, 8
    for (n, k) in ((768, 2048), (2048, 768)):
        w = torch.from_numpy(normal(45, (E, n, k), 0.02)).cuda()
        qt = ca.QTensor.quantize(w, ca.GgmlDType.Q4K)
        blocks = np.frombuffer(qt.data(), dtype=np.uint8)
        ids, tw, expert_ids, sorted_token_ids = route(1, E, topk, seed=46)
        x = normal(47, (1, k), 1.0)
        got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, None, torch.from_numpy(sorted_token_ids).cuda(),
                               torch.from_numpy(expert_ids).cuda(), topk, False)
        torch.cuda.synchronize()
        want = oracle.moe_gemm_gguf(oracle.Q4K, x, blocks, (E, n, k), sorted_token_ids, expert_ids, None, topk)
        err = rel_l2(got.cpu().numpy(), want)
        assert err <= TOL and err <= TIGHT, err


_QWEN3_EXPERTS = {}


@pytest.mark.parametrize("n,k", [(768, 2048), (2048, 768)])
@pytest.mark.parametrize("tokens", [16, 256])
@pytest.mark.parametrize("is_prefill", [False, True])
def test_moe_qwen3_shape_token_batches(n, k, tokens, is_prefill):
    """128 experts, top-8, Q4_K, 16 and 256 tokens: the gate/up call shape (one activation row per token, no weights) and
    the down call shape (one row per pair, scaled by the routing weights) against the oracle, every pair row on its own."""
    import candle_amd as ca
    E, topk = 128, 8
    if (n, k) not in _QWEN3_EXPERTS:
        gen = torch.Generator(device="cuda")
        gen.manual_seed(145)
        qt = ca.QTensor.quantize(torch.randn((E, n, k), generator=gen, device="cuda") * 0.02, ca.GgmlDType.Q4K)
        _QWEN3_EXPERTS[(n, k)] = (qt, np.frombuffer(qt.data(), dtype=np.uint8))
    qt, blocks = _QWEN3_EXPERTS[(n, k)]
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=146 + tokens)
    sti, eid = torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda()
    x = normal(147, (tokens, k), 1.0)
    got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, None, sti, eid, topk, is_prefill)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(oracle.Q4K, x, blocks, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    got = got.cpu().numpy()
    assert got.shape == want.shape == (tokens * topk, n)
    assert rel_l2(got, want) <= TIGHT
    assert max(rel_l2(got[r], want[r]) for r in range(tokens * topk)) <= 4 * TIGHT
    xp = normal(148, (tokens * topk, k), 1.0)
    twf = tw.reshape(-1)
    got = ca.moe_gemm_gguf(torch.from_numpy(xp).cuda(), qt, torch.from_numpy(twf).cuda(), sti, eid, topk, is_prefill)
    torch.cuda.synchronize()
    want = oracle.moe_gemm_gguf(oracle.Q4K, xp, blocks, (E, n, k), sorted_token_ids, expert_ids, twf, topk)
    got = got.cpu().numpy()
    assert rel_l2(got, want) <= TIGHT
    assert max(rel_l2(got[r], want[r]) for r in range(tokens * topk)) <= 4 * TIGHT


@pytest.mark.parametrize("dtype", [oracle.Q8_0, oracle.Q4_0], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("tokens,E,topk", [(300, 16, 4), (330, 128, 8), (1100, 8, 2)])
def test_grouped_matrix_core_tiles_of_the_32_element_formats(dtype, tokens, E, topk):
    """Hundreds of pairs on Q8_0 / Q4_0 experts: the expert-sorted rows go through the int8 matrix-core kernel of the format
    in tiles of one expert (32-row tiles while an expert sees few rows, 128-row tiles beyond), both call shapes, every
    pair row held to the bound on its own; candle's prefill MoE takes these formats on the tensor cores as well
    (candle-nn/src/moe.rs:208-221)."""
    import candle_amd as ca
    n, k = 203, 512
    blocks, qt = make_experts(dtype, E, n, k, seed=160)
    ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=161 + tokens)
    sti, eid = torch.from_numpy(sorted_token_ids).cuda(), torch.from_numpy(expert_ids).cuda()
    x = normal(162, (tokens, k), 1.0)
    got = ca.moe_gemm_gguf(torch.from_numpy(x).cuda(), qt, None, sti, eid, topk, True).cpu().numpy()
    want = oracle.moe_gemm_gguf(dtype, x, blocks, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    assert got.shape == want.shape == (tokens * topk, n)
    assert rel_l2(got, want) <= TIGHT
    assert max(rel_l2(got[r], want[r]) for r in range(tokens * topk)) <= 4 * TIGHT
    xp = normal(163, (tokens * topk, k), 1.0)
    twf = tw.reshape(-1)
    got = ca.moe_gemm_gguf(torch.from_numpy(xp).cuda(), qt, torch.from_numpy(twf).cuda(), sti, eid, topk, True).cpu().numpy()
    want = oracle.moe_gemm_gguf(dtype, xp, blocks, (E, n, k), sorted_token_ids, expert_ids, twf, topk)
    assert rel_l2(got, want) <= TIGHT
    assert max(rel_l2(got[r], want[r]) for r in range(tokens * topk)) <= 4 * TIGHT


@pytest.mark.parametrize("dtype", [oracle.Q4K, oracle.Q6K, oracle.Q8_0, oracle.Q3K], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("n,k", [(5, 256), (1, 768), (77, 1024), (130, 2048), (9, 4096)])
def test_short_expert_rows_ragged(dtype, n, k):
    """Rows of at most 32 units take several weight rows per wave step (2 or 4); n is not a multiple of either, a single
    row, and a row length (4096) that stays on the one-row-per-step kernel for K-quants."""
    E, batch, topk = 3, 3, 2
    blocks, qt = make_experts(dtype, E, n, k, seed=95)
    ids = np.array([[0, 2], [1, 1], [2, 0]], dtype=np.uint32)
    x = normal(96, (batch, topk, k), 1.0)
    out = qt.indexed_moe_forward(torch.from_numpy(x).cuda(), torch.from_numpy(ids.astype(np.int32)).cuda())
    torch.cuda.synchronize()
    want = oracle.indexed_moe_forward(dtype, blocks, (E, n, k), x, ids)
    err = rel_l2(out.cpu().numpy(), want)
    assert err <= TIGHT, err


@pytest.mark.parametrize("tokens", [40, 48, 49, 64])
def test_more_than_256_pairs_on_short_rows(tokens):
    """128 experts, top-8, 768- and 2048-element rows: up to 384 pairs (3 per expert) every pair is still its own matvec
    block, beyond that the grouped matrix-core path takes over; both give the oracle's values."""
    import candle_amd as ca
    E, topk = 128, 8
    for n, k in ((96, 2048), (160, 768)):
        blocks, qt = make_experts(oracle.Q4K, E, n, k, seed=97)
        ids, tw, expert_ids, sorted_token_ids = route(tokens, E, topk, seed=98 + tokens)
        x2 = normal(99, (tokens * topk, k), 1.0)
        twf = tw.reshape(-1)
        got = ca.moe_gemm_gguf(torch.from_numpy(x2).cuda(), qt, torch.from_numpy(twf).cuda(), torch.from_numpy(sorted_token_ids).cuda(),
                               torch.from_numpy(expert_ids).cuda(), topk, False)
        torch.cuda.synchronize()
        want = oracle.moe_gemm_gguf(oracle.Q4K, x2, blocks, (E, n, k), sorted_token_ids, expert_ids, twf, topk)
        assert rel_l2(got.cpu().numpy(), want) <= TIGHT
    from candle_amd import _lib
    L = _lib.lib()
    assert L.cq_moe_direct_pairs(oracle.Q4K, E, tokens * topk, 2048) == (1 if tokens * topk <= 384 else 0)
    assert L.cq_moe_direct_pairs(oracle.Q4K, E, tokens * topk, 4096) == 0
    assert L.cq_moe_direct_pairs(oracle.Q4K, 8, 256, 4096) == 1
