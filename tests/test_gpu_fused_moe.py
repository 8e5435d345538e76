"""GPU parity of candle_amd.fused_moe.FusedMoeGGUF (the mirror of candle-transformers/src/fused_moe.rs:163-303)
against its CPU restatement, and of the routing kernels on their own.

Tolerance: relative L2 <= 1e-3 on the layer output (the bar of the quantized matmul path; the three grouped matmuls
are integer-exact like the CPU, the differences come from the f32 router dot products, exp and summation order).
The routing itself must pick the same experts: the test data has no two probabilities within float rounding of each
other at the top-k boundary."""
import numpy as np
import pytest
import torch

import oracle
from oracle import fused_moe_oracle as fm
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu


def L():
    from candle_amd import _lib
    return _lib.lib()


@pytest.mark.parametrize("tokens,E,hidden,topk,norm", [(1, 128, 2048, 8, True), (7, 16, 256, 4, False), (300, 64, 512, 6, True), (3, 5, 64, 5, True),
                                                            (9, 256, 128, 8, True), (5, 300, 128, 8, True), (2, 1000, 64, 60, False),   # > 256 experts: the LDS kernel
                                                            (256, 128, 2048, 8, True), (130, 40, 256, 4, True), (517, 100, 768, 8, False)])  # token tiles in LDS
def test_route_kernel(tokens, E, hidden, topk, norm):
    x, router = normal(1, (tokens, hidden), 1.0), normal(2, (E, hidden), 0.1)
    xd, rd = torch.from_numpy(x).cuda(), torch.from_numpy(router).cuda()
    ids = torch.empty((tokens, topk), dtype=torch.int32, device="cuda")
    w = torch.empty((tokens, topk), dtype=torch.float32, device="cuda")
    lg = torch.empty((tokens, E), dtype=torch.float32, device="cuda")
    assert L().cq_nn_moe_route(xd.data_ptr(), rd.data_ptr(), ids.data_ptr(), w.data_ptr(), lg.data_ptr(), tokens, hidden, E, topk, 1 if norm else 0,
                               None) == 0
    assert np.allclose(lg.cpu().numpy(), x.astype(np.float64) @ router.astype(np.float64).T, rtol=1e-4, atol=1e-5)
    want_ids, want_w = fm.route(x, router, topk, norm)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), want_ids)
    assert np.allclose(w.cpu().numpy(), want_w, rtol=2e-5, atol=1e-8)
    if tokens >= 128:
        # the logits do not depend on how many tokens a call holds (the kernels differ, the order of a lane's additions does not)
        few = torch.empty((5, E), dtype=torch.float32, device="cuda")
        assert L().cq_nn_moe_route(xd.data_ptr() + 4 * 3 * hidden, rd.data_ptr(), ids.data_ptr(), w.data_ptr(), few.data_ptr(), 5, hidden, E, topk,
                                   1 if norm else 0, None) == 0
        assert np.array_equal(few.cpu().numpy(), lg.cpu().numpy()[3:8])


def test_route_kernel_ties_take_the_lower_expert():
    E, hidden, topk = 8, 8, 3
    router = np.zeros((E, hidden), dtype=np.float32)
    router[np.arange(E), np.arange(E)] = 1.0
    x = np.array([[1.0, 3.0, 3.0, -2.0, 3.0, 0.0, 1.0, 1.0], [0.0] * 8], dtype=np.float32)
    ids = torch.empty((2, topk), dtype=torch.int32, device="cuda")
    w = torch.empty((2, topk), dtype=torch.float32, device="cuda")
    xd, rd = torch.from_numpy(x).cuda(), torch.from_numpy(router).cuda()
    lg = torch.empty((2, E), dtype=torch.float32, device="cuda")
    assert L().cq_nn_moe_route(xd.data_ptr(), rd.data_ptr(), ids.data_ptr(), w.data_ptr(), lg.data_ptr(), 2, hidden, E, topk, 0, None) == 0
    assert ids.cpu().tolist() == [[1, 2, 4], [0, 1, 2]]
    want_ids, want_w = fm.route(x, router, topk, False)
    assert want_ids.tolist() == [[1, 2, 4], [0, 1, 2]] and np.allclose(w.cpu().numpy(), want_w, rtol=1e-6)


@pytest.mark.parametrize("n_pairs,E", [(8, 128), (2048, 128), (5000, 7), (1, 1)])
def test_sort_kernel(n_pairs, E):
    rng = np.random.default_rng(3)
    ids = rng.integers(0, E, size=n_pairs).astype(np.uint32)
    if n_pairs > 100:
        ids[17] = E + 5                                    # an id no expert has: sorted behind every valid one
    d = torch.from_numpy(ids.view(np.int32)).cuda()
    e = torch.empty(n_pairs, dtype=torch.int32, device="cuda")
    s = torch.empty(n_pairs, dtype=torch.int32, device="cuda")
    assert L().cq_nn_moe_sort(d.data_ptr(), e.data_ptr(), s.data_ptr(), n_pairs, E, None) == 0
    eh, sh = e.cpu().numpy(), s.cpu().numpy()
    want_e, _ = fm.sort_pairs(ids)
    assert np.array_equal(eh, want_e)                                               # ascending expert ids
    assert np.array_equal(np.sort(sh), np.arange(n_pairs))                          # a permutation of the pairs
    assert np.array_equal(ids[sh].astype(np.int32), eh)                             # each pair under its own expert


def test_sum_kernel():
    tokens, topk, dim = 9, 8, 2048
    y = normal(4, (tokens * topk, dim), 1.0)
    out = torch.empty((tokens, dim), device="cuda")
    yd = torch.from_numpy(y).cuda()
    assert L().cq_nn_moe_sum(yd.data_ptr(), out.data_ptr(), tokens, topk, dim, None) == 0
    acc = y.reshape(tokens, topk, dim)[:, 0].copy()
    for j in range(1, topk):
        acc = acc + y.reshape(tokens, topk, dim)[:, j]
    assert np.array_equal(out.cpu().numpy(), acc)


@pytest.mark.parametrize("dtype,k", [(oracle.Q4K, 2048), (oracle.Q6K, 512), (oracle.Q8_0, 1024)])
@pytest.mark.parametrize("tokens", [1, 5, 32])
def test_gate_up_swiglu_in_one_launch(dtype, k, tokens):
    """cq_moe_gemm_gguf_swiglu == moe_gemm_gguf(gate), moe_gemm_gguf(up), up * silu(gate) of the oracle."""
    from oracle.llama_oracle import silu
    E, n, topk = 16, 384, 4
    pairs = tokens * topk
    gate_b = oracle.from_float(dtype, normal(70, E * n * k, 0.05))
    up_b = oracle.from_float(dtype, normal(71, E * n * k, 0.05))
    x = normal(72, (tokens, k), 1.0)
    rng = np.random.default_rng(73)
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(tokens)]).astype(np.uint32)
    expert_ids, sorted_token_ids = fm.sort_pairs(ids)
    g = oracle.moe_gemm_gguf(dtype, x, gate_b, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    u = oracle.moe_gemm_gguf(dtype, x, up_b, (E, n, k), sorted_token_ids, expert_ids, None, topk)
    want = (u * silu(g)).astype(np.float32)
    both = torch.from_numpy(np.concatenate([up_b, gate_b])).cuda()          # up in front of gate: a negative distance
    out = torch.full((pairs, n), 7.0, device="cuda")
    xd = torch.from_numpy(x).cuda()
    ed, sd = torch.from_numpy(expert_ids).cuda(), torch.from_numpy(sorted_token_ids).cuda()
    assert L().cq_moe_gemm_gguf_swiglu(dtype, xd.data_ptr(), both.data_ptr() + up_b.size, both.data_ptr(), sd.data_ptr(), ed.data_ptr(),
                                       out.data_ptr(), E, topk, pairs, n, k, None) == 0
    assert rel_l2(out.cpu().numpy(), want) <= 1e-5
    # more pairs than the fused launch takes, or rows of more than one wave step: the caller falls back
    assert L().cq_moe_gemm_gguf_swiglu(dtype, xd.data_ptr(), both.data_ptr(), both.data_ptr(), sd.data_ptr(), ed.data_ptr(), out.data_ptr(),
                                       E, topk, 260, n, k, None) == -6
    assert L().cq_moe_gemm_gguf_swiglu(dtype, xd.data_ptr(), both.data_ptr(), both.data_ptr(), sd.data_ptr(), ed.data_ptr(), out.data_ptr(),
                                       E, topk, pairs, n, 8192, None) == -6


def build_layer(dtype, E, hidden, inter, topk, norm, seed):
    from candle_amd.fused_moe import FusedMoeGGUF
    from candle_amd.quantized import GgmlDType, QStorage, QTensor
    router = normal(seed, (E, hidden), 0.1)
    blocks = [oracle.from_float(dtype, normal(seed + 1 + i, E * inter * hidden, 0.05)) for i in range(3)]
    dev = torch.device("cuda:0")
    shapes = [(E, inter, hidden), (E, inter, hidden), (E, hidden, inter)]
    qts = [QTensor.new(QStorage.from_data(b.tobytes(), dev, GgmlDType(dtype)), sh) for b, sh in zip(blocks, shapes)]
    layer = FusedMoeGGUF(torch.from_numpy(router).cuda(), qts[0], qts[1], qts[2], norm, topk)
    ref = fm.FusedMoeOracle(dtype, router, blocks[0], blocks[1], blocks[2], E, hidden, inter, topk, norm)
    return layer, ref


@pytest.mark.parametrize("dtype", [oracle.Q4K, oracle.Q6K, oracle.Q8_0])
@pytest.mark.parametrize("batch,seq,is_prefill", [(1, 1, False), (2, 3, False), (1, 40, True), (1, 200, True), (1, 300, True)])
def test_fused_moe_layer(dtype, batch, seq, is_prefill):
    E, hidden, inter, topk = 16, 512, 256, 4
    layer, ref = build_layer(dtype, E, hidden, inter, topk, True, seed=20)
    x = normal(30, (batch, seq, hidden), 1.0)
    got = layer.forward(torch.from_numpy(x).cuda(), is_prefill).cpu().numpy()
    want = ref.forward(x)
    assert got.shape == want.shape == (batch, seq, hidden)
    assert rel_l2(got, want) <= 1e-3


def test_fused_moe_layer_qwen3_shape_decode_and_graph_replay():
    """The Qwen3-30B-A3B expert shape (128 experts, top-8, 2048 -> 768 -> 2048) for one token, eager and replayed from a
    HIP graph; f16 input keeps its dtype."""
    E, hidden, inter, topk = 128, 2048, 768, 8
    layer, ref = build_layer(oracle.Q4K, E, hidden, inter, topk, True, seed=40)
    x = normal(50, (1, 1, hidden), 1.0)
    xd = torch.from_numpy(x).cuda()
    want = ref.forward(x)
    eager = layer.forward(xd, False)
    assert rel_l2(eager.cpu().numpy(), want) <= 1e-3
    out = torch.empty((1, hidden), device="cuda")
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        layer.forward(xd, False, out=out)
        st.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            layer.forward(xd, False, out=out)
        for _ in range(3):
            out.zero_()
            g.replay()
            st.synchronize()
            assert np.array_equal(out.cpu().numpy().reshape(1, 1, hidden), eager.cpu().numpy())
    xh = xd.to(torch.float16)
    yh = layer.forward(xh, False)
    assert yh.dtype == torch.float16
    want_h = ref.forward(xh.float().cpu().numpy())
    assert rel_l2(yh.float().cpu().numpy(), want_h) <= 2e-3          # + the f16 rounding of the output


_QWEN3 = {}


def _qwen3_layer():
    """One Qwen3-30B-A3B-shape layer (128 experts, top-8, 2048 -> 768 -> 2048, Q4_K), shared by the token counts below.  The
    expert weights are drawn and quantized on the GPU (bit-exact quantizer, tests/test_gpu_dequant_quant.py); the oracle
    reads the same block bytes."""
    if not _QWEN3:
        from candle_amd.fused_moe import FusedMoeGGUF
        from candle_amd.quantized import GgmlDType, QTensor
        E, hidden, inter, topk = 128, 2048, 768, 8
        gen = torch.Generator(device="cuda")
        gen.manual_seed(60)
        router = normal(61, (E, hidden), 0.1)
        shapes = [(E, inter, hidden), (E, inter, hidden), (E, hidden, inter)]
        qts = [QTensor.quantize(torch.randn(sh, generator=gen, device="cuda") * 0.05, GgmlDType.Q4K) for sh in shapes]
        blocks = [np.frombuffer(q.data(), dtype=np.uint8) for q in qts]
        layer = FusedMoeGGUF(torch.from_numpy(router).cuda(), qts[0], qts[1], qts[2], True, topk)
        _QWEN3["v"] = (layer, fm.FusedMoeOracle(oracle.Q4K, router, blocks[0], blocks[1], blocks[2], E, hidden, inter, topk, True))
    return _QWEN3["v"]


@pytest.mark.parametrize("tokens,is_prefill", [(16, False), (16, True), (40, True), (256, True), (256, False), (600, True)])
def test_fused_moe_layer_qwen3_shape_token_batches(tokens, is_prefill):
    """16 to 600 tokens through the Qwen3-30B-A3B-shape layer: 128 (token, expert) pairs on the per-pair kernels; 320, 2048 and
    4800 pairs with every expert as a batched matvec over its own pairs (2.5, 16 and 37.5 pairs per expert on average: one
    sparse set, two sets, a second pass over the weights), against the CPU restatement of FusedMoeGGUF::forward."""
    layer, ref = _qwen3_layer()
    x = normal(70 + tokens, (1, tokens, 2048), 1.0)
    got = layer.forward(torch.from_numpy(x).cuda(), is_prefill).cpu().numpy()
    want = ref.forward(x)
    assert got.shape == want.shape == (1, tokens, 2048)
    assert rel_l2(got, want) <= 1e-3
    # Row by row: the matmuls agree with the CPU to 2e-6 on the same quantized rows (tests/test_gpu_moe.py), and so does the typical
    # row here.  A few rows in hundreds lie further off: gate and up differ from the CPU's in the last bit, so one value of
    # silu(gate) * up now and then falls on the other side of a rounding boundary of the int8 quantizer of the down projection, a
    # step of 1 / 127 of the row's largest value on one of 768 products.
    errs = np.array([rel_l2(got[0, r], want[0, r]) for r in range(tokens)])
    assert np.median(errs) <= 5e-6, float(np.median(errs))
    assert errs.max() <= 5e-3, float(errs.max())


@pytest.mark.parametrize("dtype", [oracle.Q4K, oracle.Q6K, oracle.Q5K])
@pytest.mark.parametrize("tokens,E,topk", [(70, 16, 4), (300, 16, 4), (1000, 8, 2)])
def test_down_projection_on_the_grouping_of_gate_and_up(dtype, tokens, E, topk):
    """Hundreds of pairs: the down projection run on the grouping the gate / up call left in the workspace, with
    up * silu(gate) inside its activation quantizer, gives the bits of silu_mul + a moe_gemm_gguf call of its own."""
    hidden, inter = 512, 256
    layer, ref = build_layer(dtype, E, hidden, inter, topk, True, seed=120)
    x = normal(121 + tokens, (1, tokens, hidden), 1.0)
    xd = torch.from_numpy(x).cuda()
    layer.share_grouping = False
    layer.sort_pairs = True                    # the reference's sequence: sort, three grouped matmuls, silu_mul between them
    apart = layer.forward(xd, True).cpu().numpy()
    layer.share_grouping = True
    layer.sort_pairs = False
    shared = layer.forward(xd, True).cpu().numpy()
    assert np.array_equal(shared, apart)
    assert rel_l2(shared, ref.forward(x)) <= 1e-3


def test_down_after_pair_refuses_what_it_cannot_reuse():
    lib = L()
    p = 256          # an aligned non-null address: the calls below return before anything is enqueued
    big = 1 << 40
    # 16 pairs: the gate / up call ran every pair as a matvec of its own, there is no grouping to reuse
    assert lib.cq_moe_gemm_gguf_down_after_pair(12, p, p, p, p, p, 128, 8, 16, 2048, 768, 2048, p, big, None) == -6
    # Q8_0 experts: whether they were grouped for the matrix cores depended on the other call's weight addresses
    assert lib.cq_moe_gemm_gguf_down_after_pair(8, p, p, p, p, p, 128, 8, 2048, 2048, 768, 2048, p, big, None) == -6
    # this call's rows (k = 4096) would not fit in front of the tables of a call with k = 256
    assert lib.cq_moe_gemm_gguf_down_after_pair(12, p, p, p, p, p, 128, 8, 2048, 2048, 4096, 256, p, big, None) == -6
    assert lib.cq_moe_gemm_gguf_down_after_pair(12, p, p, p, p, p, 128, 8, 2048, 2048, 768, 2048, p, 1024, None) == -5   # CQ_ERR_WORKSPACE
    assert lib.cq_moe_gemm_gguf_down_after_pair(12, None, p, p, p, p, 128, 8, 2048, 2048, 768, 2048, p, big, None) == -4
    # Q4_K experts that would run as batched matvecs must be 16-byte aligned in the gate / up call (the down call tells from the
    # shape alone how that call grouped its pairs): CQ_ERR_ALIGN, nothing enqueued
    assert lib.cq_moe_gemm_gguf_pair(12, p, p + 8, p, p, p, p, p, 128, 8, 2048, 768, 2048, 1, p, big, None) == -3
    assert lib.cq_moe_gemm_gguf_pair(12, p, p, p + 8, p, p, p, p, 128, 8, 2048, 768, 2048, 1, p, big, None) == -3


def test_fused_moe_argument_errors():
    from candle_amd.fused_moe import FusedMoeGGUF
    layer, _ = build_layer(oracle.Q4K, 4, 256, 512, 2, True, seed=60)
    with pytest.raises(ValueError):
        layer.forward(torch.zeros((2, 256), device="cuda"), False)
    with pytest.raises(ValueError):
        layer.forward(torch.zeros((1, 2, 128), device="cuda"), False)
    with pytest.raises(ValueError):
        FusedMoeGGUF(layer.gate, layer.gate_experts, layer.up_experts, layer.down_experts, True, 5)
    with pytest.raises(ValueError):
        FusedMoeGGUF(layer.gate, layer.gate_experts, layer.up_experts, layer.gate_experts, True, 2)
    lib = L()
    assert lib.cq_nn_moe_route(256, 256, 256, 256, 256, 1, 6, 4, 2, 1, None) == -2          # hidden % 4
    assert lib.cq_nn_moe_route(256, 256, 256, 256, 256, 1, 8, 4, 5, 1, None) == -2          # topk > experts
    assert lib.cq_nn_moe_route(256, 256, 256, 256, 256, 1, 8, 2000, 2, 1, None) == -6
    assert lib.cq_nn_moe_route(256, 256, 256, 256, None, 1, 8, 4, 2, 1, None) == -4
    assert lib.cq_nn_moe_sort(None, 256, 256, 4, 8, None) == -4
    assert lib.cq_nn_moe_sum(256, 256, 1, 2, 6, None) == -2
