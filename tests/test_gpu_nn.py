"""GPU parity of the f32 decoder glue (include/candle_hip_nn.h) against the numpy restatement of candle's CPU ops.

Tolerances: these are f32 ops whose only difference from the CPU path is summation order and the
device exp/sqrt/division, so each result is checked to 1e-5 relative L2 (far inside the 1e-3 bar of the matmul path)."""
import math

import numpy as np
import pytest
import torch

from oracle import llama_oracle as lo
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-5


def L():
    from candle_amd import _lib
    return _lib.lib()


_ALIVE = []


def dev(a, dtype=None):
    """Host array -> device tensor that stays alive until the end of the test (the C ABI takes raw pointers)."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    t = (t if dtype is None else t.to(dtype)).cuda()
    _ALIVE.append(t)
    return t


@pytest.fixture(autouse=True)
def _release_device_tensors():
    yield
    torch.cuda.synchronize()
    _ALIVE.clear()


def ok(status):
    assert status == 0, status


def test_embedding_rows_and_out_of_range():
    table = normal(1, (50, 64), 1.0)
    ids = np.array([0, 49, 7, 7, 50, -1], dtype=np.int32)
    out = torch.full((6, 64), 9.0, device="cuda")
    ok(L().cq_nn_embedding(dev(table).data_ptr(), dev(ids).data_ptr(), out.data_ptr(), 6, 64, 50, None, None))
    got = out.cpu().numpy()
    assert np.array_equal(got[:4], table[[0, 49, 7, 7]])
    assert np.all(got[4:] == 0.0)


@pytest.mark.parametrize("dim", [64, 256, 4096, 5120, 14336])
@pytest.mark.parametrize("with_delta", [False, True])
def test_rms_norm(dim, with_delta):
    rows = 3
    x, d, w = normal(2, (rows, dim), 1.0), normal(3, (rows, dim), 0.5), normal(4, (dim,), 1.0)
    xs = dev(x)
    ds = dev(d)
    out = torch.empty((rows, dim), device="cuda")
    ok(L().cq_nn_rms_norm(xs.data_ptr(), ds.data_ptr() if with_delta else None, dev(w).data_ptr(), xs.data_ptr() if with_delta else None,
                          out.data_ptr(), rows, dim, 1e-5, None))
    torch.cuda.synchronize()
    s = (x + d).astype(np.float32) if with_delta else x
    assert rel_l2(out.cpu().numpy(), lo.rms_norm(s, w, 1e-5)) <= TOL
    assert np.array_equal(xs.cpu().numpy(), s)          # the residual stream was updated in place (or left alone)


def test_rms_norm_kat_on_gpu():
    # candle-nn/tests/ops.rs:55-66 needs dim % 4 == 0 here: pad the 3-wide rows with a zero and rescale the mean
    data = np.array([[3.0, 1.0, 4.0, 0.0], [1.0, 5.0, 9.0, 0.0]], dtype=np.float32)
    alpha = np.array([1.0, 2.0, 3.0, 0.0], dtype=np.float32)
    out = torch.empty((2, 4), device="cuda")
    # mean over 4 instead of 3 elements: eps' = eps * 4/3 and a factor sqrt(3/4) on the result give the reference's numbers
    ok(L().cq_nn_rms_norm(dev(data).data_ptr(), None, dev(alpha).data_ptr(), None, out.data_ptr(), 2, 4, 1e-5 * 3 / 4, None))
    got = out.cpu().numpy()[:, :3] * math.sqrt(3.0 / 4.0)
    assert (np.round(got.astype(np.float64) * 1e4) / 1e4).tolist() == [[1.019, 0.6794, 4.0762], [0.1674, 1.6744, 4.521]]


@pytest.mark.parametrize("rows,pos", [(1, 0), (1, 37), (5, 3)])
def test_rope_i_and_cache_append(rows, pos):
    H, KV, D, ctx = 4, 2, 64, 48
    cos, sin = lo.precomput_freqs_cis(D, 10000.0, ctx)
    q, k, v = normal(5, (rows, H * D), 1.0), normal(6, (rows, KV * D), 1.0), normal(7, (rows, KV * D), 1.0)
    qd, kc, vc = dev(q), torch.zeros((KV, ctx, D), device="cuda"), torch.zeros((KV, ctx, D), device="cuda")
    posd = torch.tensor([pos], dtype=torch.int32, device="cuda")
    # half of the position from the host argument, half from device memory
    ok(L().cq_nn_rope_i_kv(qd.data_ptr(), dev(k).data_ptr(), dev(v).data_ptr(), kc.data_ptr(), vc.data_ptr(), dev(cos).data_ptr(),
                           dev(sin).data_ptr(), posd.data_ptr(), 0, rows, H, KV, D, ctx, H * D, KV * D, KV * D, None))
    torch.cuda.synchronize()
    c, s = cos[pos:pos + rows], sin[pos:pos + rows]
    want_q = lo.rope_i(q.reshape(rows, H, D).transpose(1, 0, 2)[None], c, s)[0].transpose(1, 0, 2).reshape(rows, H * D)
    want_k = lo.rope_i(k.reshape(rows, KV, D).transpose(1, 0, 2)[None], c, s)[0]         # [KV, rows, D]
    assert np.allclose(qd.cpu().numpy(), want_q, rtol=1e-6, atol=1e-6)
    assert np.allclose(kc.cpu().numpy()[:, pos:pos + rows], want_k, rtol=1e-6, atol=1e-6)
    assert np.array_equal(vc.cpu().numpy()[:, pos:pos + rows], v.reshape(rows, KV, D).transpose(1, 0, 2))
    untouched = np.ones(ctx, dtype=bool)
    untouched[pos:pos + rows] = False
    assert np.all(kc.cpu().numpy()[:, untouched] == 0.0) and np.all(vc.cpu().numpy()[:, untouched] == 0.0)


def attention_oracle(q, kc, vc, pos, H, KV, D):
    rows = q.shape[0]
    out = np.empty((rows, H * D), dtype=np.float32)
    scale = np.float32(1.0 / math.sqrt(D))
    for r in range(rows):
        kv_len = pos + r + 1
        for h in range(H):
            kvh = h // (H // KV)
            att = (kc[kvh, :kv_len] @ q[r, h * D:(h + 1) * D]).astype(np.float32) * scale
            p = lo.softmax_last_dim(att)
            out[r, h * D:(h + 1) * D] = p @ vc[kvh, :kv_len]
    return out


@pytest.mark.parametrize("H,KV,D", [(4, 2, 64), (8, 1, 128), (4, 4, 128), (8, 2, 128), (4, 2, 128)])
@pytest.mark.parametrize("rows,pos,ctx", [(1, 0, 32), (1, 199, 256), (1, 600, 1024), (7, 250, 512), (3, 0, 16),
                                          (16, 0, 64), (37, 100, 512), (130, 0, 256), (21, 250, 300), (70, 100, 512), (64, 0, 64), (66, 900, 1024)])
def test_attention(H, KV, D, rows, pos, ctx):
    q = normal(8, (rows, H * D), 1.0)
    kc, vc = normal(9, (KV, ctx, D), 1.0), normal(10, (KV, ctx, D), 1.0)
    out = torch.empty((rows, H * D), device="cuda")
    lib = L()
    for max_kv in sorted({pos + rows, ctx}):              # exact bound and a looser one (empty trailing splits)
        wsb = lib.cq_nn_attention_workspace_bytes(rows, H, D, max_kv)
        ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
        ok(lib.cq_nn_attention(dev(q).data_ptr(), H * D, dev(kc).data_ptr(), dev(vc).data_ptr(), out.data_ptr(), None, pos, rows, H, KV, D,
                               ctx, max_kv, float(np.float32(1.0 / math.sqrt(D))), ws.data_ptr(), wsb, None))
        torch.cuda.synchronize()
        assert rel_l2(out.cpu().numpy(), attention_oracle(q, kc, vc, pos, H, KV, D)) <= TOL


@pytest.mark.parametrize("H,KV,D", [(4, 2, 64), (8, 1, 128), (4, 4, 128), (32, 8, 128)])
def test_attention_rows_share_keys_with_position_on_device(H, KV, D):
    """16 rows and more go several to a workgroup; the position may come from device memory (a captured graph)."""
    rows, pos, ctx = 19, 120, 384
    q = normal(14, (rows, H * D), 1.0)
    kc, vc = normal(15, (KV, ctx, D), 1.0), normal(16, (KV, ctx, D), 1.0)
    out = torch.full((rows + 1, H * D), 7.0, device="cuda")
    pos_dev = torch.tensor([pos], dtype=torch.int32, device="cuda")
    lib = L()
    wsb = lib.cq_nn_attention_workspace_bytes(rows, H, D, ctx)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
    ok(lib.cq_nn_attention(dev(q).data_ptr(), H * D, dev(kc).data_ptr(), dev(vc).data_ptr(), out.data_ptr(), pos_dev.data_ptr(), 0, rows, H, KV, D,
                           ctx, ctx, float(np.float32(1.0 / math.sqrt(D))), ws.data_ptr(), wsb, None))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert rel_l2(got[:rows], attention_oracle(q, kc, vc, pos, H, KV, D)) <= TOL
    assert np.all(got[rows] == 7.0)                       # the padding rows of the last workgroup write nothing


def test_attention_single_key_returns_value():
    H, KV, D, ctx = 4, 2, 64, 8
    q, kc, vc = normal(11, (1, H * D), 5.0), normal(12, (KV, ctx, D), 1.0), normal(13, (KV, ctx, D), 1.0)
    out = torch.empty((1, H * D), device="cuda")
    ok(L().cq_nn_attention(dev(q).data_ptr(), H * D, dev(kc).data_ptr(), dev(vc).data_ptr(), out.data_ptr(), None, 0, 1, H, KV, D, ctx, 1,
                           0.125, None, 0, None))
    got = out.cpu().numpy().reshape(H, D)
    for h in range(H):
        assert np.array_equal(got[h], vc[h // 2, 0])


@pytest.mark.parametrize("H,KV,D", [(4, 2, 64), (8, 1, 128), (32, 8, 128)])
@pytest.mark.parametrize("pos,ctx,max_kv", [(0, 16, 1), (5, 64, 64), (127, 256, 200), (128, 256, 256), (300, 1024, 301), (600, 1024, 1024),
                                            (700, 2048, 2048), (1500, 2048, 2048), (1100, 4096, 4096)])
def test_attention_decode_fused_step(H, KV, D, pos, ctx, max_kv):
    """rope + cache append + attention over 64- or 128-key splits with the in-kernel merge == the CPU ops; called twice in a
    row on fresh caches."""
    lib = L()
    cos, sin = lo.precomput_freqs_cis(D, 500000.0, ctx)
    q, k, v = normal(30, (1, H * D), 1.0), normal(31, (1, KV * D), 1.0), normal(32, (1, KV * D), 1.0)
    kc0, vc0 = normal(33, (KV, ctx, D), 1.0), normal(34, (KV, ctx, D), 1.0)
    kc0[:, pos:], vc0[:, pos:] = np.nan, np.nan          # nothing at or beyond the new position may reach the result (key rows there are read, and masked)
    wsb = lib.cq_nn_attention_decode_workspace_bytes(H, D, max_kv)
    # 64-key splits while at most 32 of them cover max_kv, else 128-key splits; more than 32 splits: not available
    want_splits = (max_kv + 63) // 64 if (max_kv + 63) // 64 <= 32 else (max_kv + 127) // 128
    assert lib.cq_nn_attention_decode_splits(max_kv) == want_splits
    assert lib.cq_nn_attention_decode_splits(2048) == 32 and lib.cq_nn_attention_decode_splits(2049) == 17
    assert lib.cq_nn_attention_decode_splits(4096) == 32 and lib.cq_nn_attention_decode_splits(4097) == -1
    ws = torch.full((wsb,), 0xff, dtype=torch.uint8, device="cuda")
    ws[:256] = 0                                         # the arrival counters of the in-kernel merge start at zero
    posd = torch.tensor([pos], dtype=torch.int32, device="cuda")
    c, s = cos[pos:pos + 1], sin[pos:pos + 1]
    want_q = lo.rope_i(q.reshape(1, H, D).transpose(1, 0, 2)[None], c, s)[0].transpose(1, 0, 2).reshape(1, H * D)
    want_k = lo.rope_i(k.reshape(1, KV, D).transpose(1, 0, 2)[None], c, s)[0]
    kc_ref, vc_ref = kc0.copy(), vc0.copy()
    kc_ref[:, pos:pos + 1], vc_ref[:, pos:pos + 1] = want_k, v.reshape(1, KV, D).transpose(1, 0, 2)
    want = attention_oracle(want_q, kc_ref, vc_ref, pos, H, KV, D)
    for attempt in range(2):
        kc, vc, out = dev(kc0), dev(vc0), torch.zeros((1, H * D), device="cuda")
        # second attempt: the launch also carries read-only workgroups over a 5 MB range (ragged: not a multiple of the stride)
        pf = torch.zeros(5 * 1024 * 1024 + 48, dtype=torch.uint8, device="cuda") if attempt else None
        ok(lib.cq_nn_attention_decode(dev(q).data_ptr(), dev(k).data_ptr(), dev(v).data_ptr(), kc.data_ptr(), vc.data_ptr(), dev(cos).data_ptr(),
                                      dev(sin).data_ptr(), out.data_ptr(), posd.data_ptr(), 0, H, KV, D, ctx, max_kv,
                                      float(np.float32(1.0 / math.sqrt(D))), ws.data_ptr(), wsb, pf.data_ptr() if attempt else None,
                                      pf.numel() // 16 * 16 if attempt else 0, 9216 if attempt and KV == 8 else 0, None))
        torch.cuda.synchronize()
        assert rel_l2(out.cpu().numpy(), want) <= TOL, attempt
        assert np.allclose(kc.cpu().numpy()[:, pos], want_k[:, 0], rtol=1e-6, atol=1e-6)
        assert np.array_equal(vc.cpu().numpy()[:, pos], vc_ref[:, pos])
        assert np.array_equal(kc.cpu().numpy()[:, :pos], kc0[:, :pos])


def _attention_decode_case(lib, ws, wsb, H, KV, D, pos, ctx, max_kv, seed):
    """One fused decode-attention call on a given workspace against the CPU ops."""
    cos, sin = lo.precomput_freqs_cis(D, 500000.0, ctx)
    q, k, v = normal(seed, (1, H * D), 1.0), normal(seed + 1, (1, KV * D), 1.0), normal(seed + 2, (1, KV * D), 1.0)
    kc0, vc0 = normal(seed + 3, (KV, ctx, D), 1.0), normal(seed + 4, (KV, ctx, D), 1.0)
    kc0[:, pos:], vc0[:, pos:] = np.nan, np.nan
    c, s = cos[pos:pos + 1], sin[pos:pos + 1]
    want_q = lo.rope_i(q.reshape(1, H, D).transpose(1, 0, 2)[None], c, s)[0].transpose(1, 0, 2).reshape(1, H * D)
    want_k = lo.rope_i(k.reshape(1, KV, D).transpose(1, 0, 2)[None], c, s)[0]
    kc_ref, vc_ref = kc0.copy(), vc0.copy()
    kc_ref[:, pos:pos + 1], vc_ref[:, pos:pos + 1] = want_k, v.reshape(1, KV, D).transpose(1, 0, 2)
    want = attention_oracle(want_q, kc_ref, vc_ref, pos, H, KV, D)
    kc, vc, out = dev(kc0), dev(vc0), torch.zeros((1, H * D), device="cuda")
    posd = torch.tensor([pos], dtype=torch.int32, device="cuda")
    ok(lib.cq_nn_attention_decode(dev(q).data_ptr(), dev(k).data_ptr(), dev(v).data_ptr(), kc.data_ptr(), vc.data_ptr(), dev(cos).data_ptr(),
                                  dev(sin).data_ptr(), out.data_ptr(), posd.data_ptr(), 0, H, KV, D, ctx, max_kv,
                                  float(np.float32(1.0 / math.sqrt(D))), ws.data_ptr(), wsb, None, 0, 0, None))
    torch.cuda.synchronize()
    assert rel_l2(out.cpu().numpy(), want) <= TOL, (pos, max_kv)
    assert np.array_equal(vc.cpu().numpy()[:, pos], vc_ref[:, pos])


def test_attention_decode_one_workspace_across_split_counts():
    """One partials buffer, sized for the longest context, serves calls whose split count rises and falls: the arrival
    counters sit in front of the records, where no call's records reach them."""
    lib = L()
    H, KV, D, ctx = 32, 8, 128, 4096
    wsb = lib.cq_nn_attention_decode_workspace_bytes(H, D, ctx)
    ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
    # 16 splits of 64 keys, 9 of 128, one split, 32 splits, and back
    for i, (pos, max_kv) in enumerate([(1000, 1024), (1024, 1025), (40, 64), (3000, 4096), (63, 64), (64, 65), (1023, 1024), (3000, 3001)]):
        _attention_decode_case(lib, ws, wsb, H, KV, D, pos, ctx, max_kv, 300 + 10 * i)
        assert int(ws[:256].to(torch.int32).sum()) == 0           # every call leaves its counters at zero


def test_attention_decode_result_does_not_depend_on_the_layout_length():
    """With the merge inside the kernel only the splits that hold keys take part, and up to 2048 keys all splits are 64 keys long:
    a step laid out for 704, 768, 1024 or 2048 keys gives the same bits at position 700 (a server may capture one step for its
    whole context), the splits beyond the position leave their (poisoned) records alone, and the counters end at zero."""
    lib = L()
    H, KV, D, ctx, pos = 32, 8, 128, 2048, 700
    cos, sin = lo.precomput_freqs_cis(D, 500000.0, ctx)
    q, k, v = dev(normal(80, (1, H * D), 1.0)), dev(normal(81, (1, KV * D), 1.0)), dev(normal(82, (1, KV * D), 1.0))
    kc0, vc0 = normal(83, (KV, ctx, D), 1.0), normal(84, (KV, ctx, D), 1.0)
    cd, sd = dev(cos), dev(sin)
    posd = torch.tensor([pos], dtype=torch.int32, device="cuda")
    outs = []
    for max_kv in (704, 768, 1024, 2048):
        wsb = lib.cq_nn_attention_decode_workspace_bytes(H, D, max_kv)
        ws = torch.zeros(wsb // 4, dtype=torch.float32, device="cuda")
        ws[64:] = float("nan")
        kc, vc, out = dev(kc0), dev(vc0), torch.zeros((1, H * D), device="cuda")
        ok(lib.cq_nn_attention_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(), cd.data_ptr(), sd.data_ptr(),
                                      out.data_ptr(), posd.data_ptr(), 0, H, KV, D, ctx, max_kv, float(np.float32(1.0 / math.sqrt(D))),
                                      ws.data_ptr(), wsb, None, 0, 0, None))
        torch.cuda.synchronize()
        assert int(ws[:64].view(torch.int32).abs().sum()) == 0
        splits = lib.cq_nn_attention_decode_splits(max_kv)
        rec = ws[64:].view(H, splits, D + 4)
        assert not torch.isnan(rec[:, :11]).any() and torch.isnan(rec[:, 11:]).all()      # 701 keys: 11 splits of 64
        outs.append(out.cpu().numpy())
    assert not np.isnan(outs[0]).any()
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])


@pytest.mark.parametrize("H,KV,D", [(4, 2, 64), (32, 8, 128)])
def test_attention_decode_beyond_2048_keys(H, KV, D):
    """MAX_SEQ_LEN of quantized_llama.rs:27 is 4096: position 3000 of a 4096-key context, 32 splits of 128 keys."""
    lib = L()
    wsb = lib.cq_nn_attention_decode_workspace_bytes(H, D, 4096)
    ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
    assert lib.cq_nn_attention_decode_splits(4096) == 32
    _attention_decode_case(lib, ws, wsb, H, KV, D, 3000, 4096, 4096, 500)
    _attention_decode_case(lib, ws, wsb, H, KV, D, 4095, 4096, 4096, 510)


@pytest.mark.parametrize("pos,max_kv", [(760, 768), (1000, 1024), (700, 2048), (2040, 2048)],
                         ids=["12-splits", "16-splits", "11-of-32-splits", "32-splits"])
def test_attention_decode_in_kernel_merge_soak(pos, max_kv):
    """The in-kernel merge reads the partials of workgroups on other XCDs after one relaxed device-scope counter increment,
    with no fence.  20 000 launches at the 8B head shape, the records poisoned with NaN before each: every launch must
    reproduce, bit for bit, the merged output that the first launch produced (which is checked against the CPU ops, and whose
    arithmetic test_attention_merge_as_matvec_prologue ties to the merge across a kernel boundary).  A partial read before it
    was visible would come out as NaN."""
    lib = L()
    H, KV, D, ctx = 32, 8, 128, 2048
    cos, sin = lo.precomput_freqs_cis(D, 500000.0, ctx)
    q, k, v = normal(70, (1, H * D), 1.0), normal(71, (1, KV * D), 1.0), normal(72, (1, KV * D), 1.0)
    kc0, vc0 = normal(73, (KV, ctx, D), 1.0), normal(74, (KV, ctx, D), 1.0)
    c, s = cos[pos:pos + 1], sin[pos:pos + 1]
    want_q = lo.rope_i(q.reshape(1, H, D).transpose(1, 0, 2)[None], c, s)[0].transpose(1, 0, 2).reshape(1, H * D)
    kc_ref, vc_ref = kc0.copy(), vc0.copy()
    kc_ref[:, pos:pos + 1] = lo.rope_i(k.reshape(1, KV, D).transpose(1, 0, 2)[None], c, s)[0]
    vc_ref[:, pos:pos + 1] = v.reshape(1, KV, D).transpose(1, 0, 2)
    want = attention_oracle(want_q, kc_ref, vc_ref, pos, H, KV, D)
    wsb = lib.cq_nn_attention_decode_workspace_bytes(H, D, max_kv)
    assert lib.cq_nn_attention_decode_splits(max_kv) == (12 if max_kv == 768 else 16 if max_kv == 1024 else 32)
    ws = torch.zeros(wsb // 4, dtype=torch.float32, device="cuda")
    records = ws[64:]                                     # behind the 256 bytes of counters
    kc, vc, out = dev(kc0), dev(vc0), torch.zeros((1, H * D), device="cuda")
    qd, kd, vd, cd, sd = dev(q), dev(k), dev(v), dev(cos), dev(sin)
    posd = torch.tensor([pos], dtype=torch.int32, device="cuda")
    scale = float(np.float32(1.0 / math.sqrt(D)))

    def launch():
        ok(lib.cq_nn_attention_decode(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), kc.data_ptr(), vc.data_ptr(), cd.data_ptr(), sd.data_ptr(),
                                      out.data_ptr(), posd.data_ptr(), 0, H, KV, D, ctx, max_kv, scale, ws.data_ptr(), wsb, None, 0, 0, None))

    launch()
    torch.cuda.synchronize()
    assert rel_l2(out.cpu().numpy(), want) <= TOL
    first = out.clone().view(torch.int32)
    bad = torch.zeros((), dtype=torch.int64, device="cuda")
    for i in range(20000):
        records.fill_(float("nan"))
        out.fill_(float("nan"))
        launch()
        bad += (out.view(torch.int32) != first).sum()
        if i % 2000 == 1999:
            assert int(bad) == 0, i                       # stop at the first block of launches with a mismatch
    assert int(ws[:64].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("dtype", [12, 14, 2])
@pytest.mark.parametrize("pos,max_kv", [(3, 128), (700, 701), (700, 1024)])
def test_attention_merge_as_matvec_prologue(dtype, pos, max_kv):
    """attention partials merged inside the attention_wo matvec == merge kernel followed by the plain fused matvec, bit for bit."""
    import oracle
    lib = L()
    H, KV, D, ctx, hidden = (32, 8, 128, 2048, 512) if dtype != 2 else (16, 4, 128, 2048, 512)
    k = H * D
    cos, sin = lo.precomput_freqs_cis(D, 500000.0, ctx)
    q, kn, vn = normal(40, (1, k), 1.0), normal(41, (1, KV * D), 1.0), normal(42, (1, KV * D), 1.0)
    kc, vc = dev(normal(43, (KV, ctx, D), 1.0)), dev(normal(44, (KV, ctx, D), 1.0))
    w = dev(oracle.from_float(dtype, normal(45, (hidden, k), 0.05).reshape(-1)))
    wsb = lib.cq_nn_attention_decode_workspace_bytes(H, D, max_kv)
    ws = torch.zeros(wsb, dtype=torch.uint8, device="cuda")
    att = torch.empty((1, k), device="cuda")
    args = (dev(q).data_ptr(), dev(kn).data_ptr(), dev(vn).data_ptr(), kc.data_ptr(), vc.data_ptr(), dev(cos).data_ptr(), dev(sin).data_ptr())
    tail = (None, pos, H, KV, D, ctx, max_kv, float(np.float32(1.0 / math.sqrt(D))), ws.data_ptr(), wsb, None, 0, 0, None)
    ok(lib.cq_nn_attention_decode(*args, att.data_ptr(), *tail))
    res0 = normal(46, (1, hidden), 1.0)
    r1, r2 = dev(res0), dev(res0)
    p1, p2 = torch.empty(256, device="cuda"), torch.empty(256, device="cuda")
    ok(lib.cq_nn_qmatmul_residual(dtype, w.data_ptr(), att.data_ptr(), None, r1.data_ptr(), p1.data_ptr(), k, hidden, None))
    ok(lib.cq_nn_attention_decode(*args, None, *tail))
    ok(lib.cq_nn_qmatmul_residual_attn(dtype, w.data_ptr(), ws.data_ptr() + 256, lib.cq_nn_attention_decode_splits(max_kv), D, r2.data_ptr(),
                                       p2.data_ptr(), k, hidden, None))
    torch.cuda.synchronize()
    assert np.array_equal(r1.cpu().numpy(), r2.cpu().numpy()) and np.array_equal(p1.cpu().numpy(), p2.cpu().numpy())
    assert not np.array_equal(r1.cpu().numpy(), res0)
    assert lib.cq_nn_qmatmul_residual_attn(12, w.data_ptr(), ws.data_ptr(), 17, D, r2.data_ptr(), p2.data_ptr(), k, hidden, None) == -6
    assert lib.cq_nn_qmatmul_residual_attn(12, w.data_ptr(), ws.data_ptr(), 2, D, r2.data_ptr(), p2.data_ptr(), 8192, hidden, None) == -6


def test_silu_mul_strided_views():
    rows, dim = 3, 1024
    gu = normal(14, (rows, 2 * dim), 2.0)
    g = dev(gu)
    out = torch.empty((rows, dim), device="cuda")
    ok(L().cq_nn_silu_mul(g.data_ptr(), g.data_ptr() + 4 * dim, out.data_ptr(), rows, dim, 2 * dim, 2 * dim, None))
    want = lo.silu(gu[:, :dim]) * gu[:, dim:]
    assert rel_l2(out.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("dtype", [12, 14, 13, 2, 8])
@pytest.mark.parametrize("m,k,n", [(3, 512, 96), (8, 1024, 200), (40, 2048, 130), (130, 768, 64), (5, 8192, 70)])
def test_silu_mul_folded_into_the_quantizer_of_a_matmul(dtype, m, k, n):
    """feed_forward_w2 over several rows: equal to cq_nn_silu_mul + cq_qmatmul_forward (same arithmetic, bit for bit), and to
    the CPU sequence within what the device's expf may move through the quantizer."""
    import oracle
    lib = L()
    gu = normal(70, (m, 2 * k), 1.5)
    w = oracle.from_float(dtype, normal(71, (n, k), 0.03).reshape(-1))
    g, wd = dev(gu), dev(w)
    wsb = lib.cq_qmatmul_workspace_bytes(dtype, m, k, n)
    ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device="cuda")
    fused = torch.empty((m, n), device="cuda")
    ok(lib.cq_nn_qmatmul_swiglu_rows(dtype, wd.data_ptr(), g.data_ptr(), g.data_ptr() + 4 * k, 2 * k, 2 * k, fused.data_ptr(), m, k, n,
                                     ws.data_ptr(), wsb, None))
    h = torch.empty((m, k), device="cuda")
    two = torch.empty((m, n), device="cuda")
    ok(lib.cq_nn_silu_mul(g.data_ptr(), g.data_ptr() + 4 * k, h.data_ptr(), m, k, 2 * k, 2 * k, None))
    ok(lib.cq_qmatmul_forward(dtype, wd.data_ptr(), h.data_ptr(), 0, two.data_ptr(), 0, m, k, n, ws.data_ptr(), wsb, None))
    torch.cuda.synchronize()
    assert np.array_equal(fused.cpu().numpy(), two.cpu().numpy())
    hh = (lo.silu(gu[:, :k]) * gu[:, k:]).astype(np.float32)
    assert rel_l2(fused.cpu().numpy(), oracle.matmul_fast(dtype, hh, w, n, 8)) <= 1e-4


def test_silu_mul_folded_argument_errors():
    lib = L()
    assert lib.cq_nn_qmatmul_swiglu_rows(8, 256, 256, 256, 96, 96, 256, 4, 96, 64, 256, 1 << 20, None) == -6      # k % 256
    assert lib.cq_nn_qmatmul_swiglu_rows(12, 256, 256, 256, 256, 510, 256, 4, 512, 64, 256, 1 << 20, None) == -2  # stride < k
    assert lib.cq_nn_qmatmul_swiglu_rows(12, 256, 256, 256, 512, 512, 256, 4, 512, 64, 256, 16, None) == -5       # workspace


def test_argmax_first_of_ties_and_bookkeeping():
    n = 128256
    logits = normal(15, (n,), 1.0)
    logits[[777, 90000]] = 50.0                      # a tie: the lower index wins
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    hist = torch.full((8,), -1, dtype=torch.int32, device="cuda")
    cnt = torch.tensor([2], dtype=torch.int32, device="cuda")
    pos = torch.tensor([41], dtype=torch.int32, device="cuda")
    ok(L().cq_nn_argmax(dev(logits).data_ptr(), n, tok.data_ptr(), hist.data_ptr(), cnt.data_ptr(), pos.data_ptr(), None, None))
    assert tok.item() == 777 and hist.cpu().tolist() == [-1, -1, 777, -1, -1, -1, -1, -1] and cnt.item() == 3 and pos.item() == 42
    logits[5] = 60.0
    ok(L().cq_nn_argmax(dev(logits).data_ptr(), n, tok.data_ptr(), None, None, None, None, None))
    assert tok.item() == 5 == int(np.argmax(logits))
    # the many-workgroup variant (workspace given): same answers, same tie rule, same bookkeeping
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")
    logits[5] = 0.0
    ok(L().cq_nn_argmax(dev(logits).data_ptr(), n, tok.data_ptr(), hist.data_ptr(), cnt.data_ptr(), pos.data_ptr(), ws.data_ptr(), None))
    assert tok.item() == 777 and hist.cpu().tolist()[3] == 777 and cnt.item() == 4 and pos.item() == 43
    for trial, where in enumerate([0, n - 1, 1001, 64127, 64128]):
        lg = normal(50 + trial, (n,), 1.0)
        lg[where] = 99.0
        ok(L().cq_nn_argmax(dev(lg).data_ptr(), n, tok.data_ptr(), None, None, None, ws.data_ptr(), None))
        assert tok.item() == where
    lg = np.full((n,), -np.inf, dtype=np.float32)      # all -inf: index 0, like numpy
    ok(L().cq_nn_argmax(dev(lg).data_ptr(), n, tok.data_ptr(), None, None, None, ws.data_ptr(), None))
    assert tok.item() == 0


@pytest.mark.parametrize("n,dim", [(128256, 4096), (9000, 64)])
def test_argmax_embed_equals_argmax_then_embedding(n, dim):
    """The arg-max that also looks up the chosen token's embedding row: token, bookkeeping, row and partial sums of squares
    equal cq_nn_argmax followed by cq_nn_embedding, bit for bit; an out-of-range vocabulary gives a zero row."""
    table = normal(31, (n, dim), 1.0) if dim == 64 else None
    tab = dev(table) if table is not None else torch.randn((n, dim), device="cuda", generator=torch.Generator(device="cuda").manual_seed(5))
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")
    for trial, where in enumerate([0, n - 1, 4242]):
        lg = normal(70 + trial, (n,), 1.0)
        lg[where] = 77.0
        if where == 4242:
            lg[8000] = 77.0                                  # a tie: the lower index wins
        lgd = dev(lg)
        tok = [torch.zeros(1, dtype=torch.int32, device="cuda") for _ in range(2)]
        hist = [torch.full((4,), -1, dtype=torch.int32, device="cuda") for _ in range(2)]
        cnt = [torch.tensor([1], dtype=torch.int32, device="cuda") for _ in range(2)]
        pos = [torch.tensor([9], dtype=torch.int32, device="cuda") for _ in range(2)]
        row = [torch.full((dim,), 3.0, device="cuda") for _ in range(2)]
        part = [torch.full((256,), 5.0, device="cuda") for _ in range(2)]
        ok(L().cq_nn_argmax(lgd.data_ptr(), n, tok[0].data_ptr(), hist[0].data_ptr(), cnt[0].data_ptr(), pos[0].data_ptr(), ws.data_ptr(), None))
        ok(L().cq_nn_embedding(tab.data_ptr(), tok[0].data_ptr(), row[0].data_ptr(), 1, dim, n, part[0].data_ptr(), None))
        ok(L().cq_nn_argmax_embed(lgd.data_ptr(), n, tok[1].data_ptr(), hist[1].data_ptr(), cnt[1].data_ptr(), pos[1].data_ptr(), ws.data_ptr(),
                                  tab.data_ptr(), row[1].data_ptr(), dim, n, part[1].data_ptr(), None))
        torch.cuda.synchronize()
        assert tok[0].item() == tok[1].item() == where
        for a, b in ((hist[0], hist[1]), (cnt[0], cnt[1]), (pos[0], pos[1])):
            assert torch.equal(a, b)
        assert torch.equal(row[0].view(torch.int32), row[1].view(torch.int32)) and torch.equal(row[1], tab[where])
        assert torch.equal(part[0].view(torch.int32), part[1].view(torch.int32))
    # a table smaller than the logits row: tokens beyond it give a zero row, as cq_nn_embedding does
    lg = normal(99, (n,), 1.0)
    lg[n - 1] = 88.0
    t1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    r1 = torch.full((dim,), 3.0, device="cuda")
    ok(L().cq_nn_argmax_embed(dev(lg).data_ptr(), n, t1.data_ptr(), None, None, None, ws.data_ptr(), tab.data_ptr(), r1.data_ptr(), dim, n - 1, None, None))
    assert t1.item() == n - 1 and bool((r1 == 0).all())
    assert L().cq_nn_argmax_embed(dev(lg).data_ptr(), n, t1.data_ptr(), None, None, None, None, tab.data_ptr(), r1.data_ptr(), dim, n, None, None) == -4      # CQ_ERR_NULL: the workspace is required


FUSE_DTYPES = [2, 8, 12, 13, 14]      # Q4_0, Q8_0, Q4_K, Q5_K, Q6_K


@pytest.mark.parametrize("dtype", FUSE_DTYPES)
@pytest.mark.parametrize("n,k", [(203, 4096), (64, 256), (1024, 14336), (5000, 1024)])
def test_fused_norm_matvec_and_residual_chain(dtype, n, k):
    """embedding -> (rms_norm + matvec) and (matvec + residual add) -> (rms_norm + matvec) against the unfused
    CPU sequence: rms_norm, quantized matmul, add.  Single row, like a decode step."""
    import oracle
    lib = L()
    table = normal(20, (7, k), 1.0)
    nw = (1.0 + 0.1 * normal(21, (k,), 1.0)).astype(np.float32)
    w1 = oracle.from_float(dtype, normal(22, (n, k), 0.05).reshape(-1))
    w1d = dev(w1)
    ids = dev(np.array([3], dtype=np.int32))
    x = torch.empty((1, k), device="cuda")
    part = torch.full((256,), 7.0, device="cuda")
    ok(lib.cq_nn_embedding(dev(table).data_ptr(), ids.data_ptr(), x.data_ptr(), 1, k, 7, part.data_ptr(), None))
    p = part.cpu().numpy()
    assert np.isclose(p.sum(), float((table[3].astype(np.float64) ** 2).sum()), rtol=1e-5) and np.all(p[1:] == 0.0)
    y = torch.empty((1, n), device="cuda")
    ok(lib.cq_nn_qmatmul_norm(dtype, w1d.data_ptr(), x.data_ptr(), part.data_ptr(), dev(nw).data_ptr(), 1e-5, y.data_ptr(), k, n, None))
    xn = lo.rms_norm(table[3:4], nw, 1e-5)
    want = oracle.matmul(dtype, xn, w1, n)
    assert rel_l2(y.cpu().numpy(), want) <= 1e-3
    # second stage: residual[k] += W2[k x n] . y   (n must be a whole number of blocks for W2)
    if n % 256 == 0:
        w2 = oracle.from_float(dtype, normal(23, (k, n), 0.05).reshape(-1))
        res0 = table[3:4].copy()
        res = dev(res0)
        part2 = torch.full((256,), 9.0, device="cuda")
        ok(lib.cq_nn_qmatmul_residual(dtype, dev(w2).data_ptr(), y.data_ptr(), None, res.data_ptr(), part2.data_ptr(), n, k, None))
        want_res = res0 + oracle.matmul(dtype, y.cpu().numpy(), w2, k)
        got_res = res.cpu().numpy()
        assert rel_l2(got_res, want_res) <= 1e-5
        assert np.isclose(part2.cpu().numpy().astype(np.float64).sum(), float((got_res.astype(np.float64) ** 2).sum()), rtol=1e-5)
        # and the partial sums drive the next fused norm
        y2 = torch.empty((1, n), device="cuda")
        ok(lib.cq_nn_qmatmul_norm(dtype, w1d.data_ptr(), res.data_ptr(), part2.data_ptr(), dev(nw).data_ptr(), 1e-5, y2.data_ptr(), k, n, None))
        want2 = oracle.matmul(dtype, lo.rms_norm(got_res, nw, 1e-5), w1, n)
        assert rel_l2(y2.cpu().numpy(), want2) <= 1e-3


@pytest.mark.parametrize("dtype", [12, 14, 8])
def test_fused_silu_mul_matvec_residual(dtype):
    import oracle
    k, n = 14336, 4096
    gu = normal(24, (1, 2 * k), 1.5)
    w = oracle.from_float(dtype, normal(25, (n, k), 0.02).reshape(-1))
    res0 = normal(26, (1, n), 1.0)
    g, res = dev(gu), dev(res0)
    part = torch.empty((256,), device="cuda")
    ok(L().cq_nn_qmatmul_residual(dtype, dev(w).data_ptr(), g.data_ptr(), g.data_ptr() + 4 * k, res.data_ptr(), part.data_ptr(), k, n, None))
    h = (lo.silu(gu[:, :k]) * gu[:, k:]).astype(np.float32)
    want = res0 + oracle.matmul_fast(dtype, h, w, n, 8)
    # expf on the device differs from the host's by an ulp here and there; the quantizer can turn that into a
    # one-step difference of a single int8 value
    assert rel_l2(res.cpu().numpy(), want) <= 1e-4


@pytest.mark.parametrize("dtype", FUSE_DTYPES)
@pytest.mark.parametrize("ffn,k", [(14336, 4096), (300, 512), (33, 2048)])
def test_fused_norm_swiglu_matvec(dtype, ffn, k):
    import oracle
    lib = L()
    x = normal(60, (1, k), 1.0)
    nw = (1.0 + 0.1 * normal(61, (k,), 1.0)).astype(np.float32)
    w1 = oracle.from_float(dtype, normal(62, (ffn, k), 0.03).reshape(-1))
    w3 = oracle.from_float(dtype, normal(63, (ffn, k), 0.03).reshape(-1))
    part = np.zeros(256, dtype=np.float32)
    part[:5] = (x.astype(np.float64) ** 2).sum() / 5.0
    h = torch.empty((1, ffn), device="cuda")
    both = dev(np.concatenate([w1, w3]))                       # adjacent, as the decoder stores them
    if dtype in (2, 8) and k > 2048:                           # longer than one wave step for 32-element blocks
        assert lib.cq_nn_qmatmul_norm_swiglu(dtype, both.data_ptr(), both.data_ptr() + w1.size, dev(x).data_ptr(), dev(part).data_ptr(),
                                             dev(nw).data_ptr(), 1e-5, h.data_ptr(), k, ffn, None) == -6
        return
    ok(lib.cq_nn_qmatmul_norm_swiglu(dtype, both.data_ptr(), both.data_ptr() + w1.size, dev(x).data_ptr(), dev(part).data_ptr(),
                                     dev(nw).data_ptr(), 1e-5, h.data_ptr(), k, ffn, None))
    xn = lo.rms_norm(x, nw, 1e-5)
    want = lo.silu(oracle.matmul_fast(dtype, xn, w1, ffn, 8)) * oracle.matmul_fast(dtype, xn, w3, ffn, 8)
    assert rel_l2(h.cpu().numpy(), want) <= 1e-4
    # w3 anywhere else in memory, in front of w1 included
    sep3, sep1 = dev(w3), dev(w1)
    h2 = torch.empty((1, ffn), device="cuda")
    ok(lib.cq_nn_qmatmul_norm_swiglu(dtype, sep1.data_ptr(), sep3.data_ptr(), dev(x).data_ptr(), dev(part).data_ptr(), dev(nw).data_ptr(), 1e-5,
                                     h2.data_ptr(), k, ffn, None))
    assert np.array_equal(h2.cpu().numpy(), h.cpu().numpy())
    assert lib.cq_nn_qmatmul_norm_swiglu(dtype, sep1.data_ptr(), sep3.data_ptr(), 16, 16, 16, 1e-5, 16, 8192, ffn, None) == -6


@pytest.mark.parametrize("dta,dtb", [(12, 14), (14, 12), (13, 13), (12, 12)])
@pytest.mark.parametrize("na,nb,k", [(5120, 1024, 4096), (96, 4000, 1024), (64, 64, 14336)])
def test_fused_norm_pair_matvec(dta, dtb, na, nb, k):
    import oracle
    lib = L()
    x = normal(70, (1, k), 1.0)
    nw = (1.0 + 0.1 * normal(71, (k,), 1.0)).astype(np.float32)
    wa = oracle.from_float(dta, normal(72, (na, k), 0.03).reshape(-1))
    wb = oracle.from_float(dtb, normal(73, (nb, k), 0.03).reshape(-1))
    part = np.zeros(256, dtype=np.float32)
    part[0] = (x.astype(np.float64) ** 2).sum()
    ya, yb = torch.empty((1, na), device="cuda"), torch.empty((1, nb), device="cuda")
    ok(lib.cq_nn_qmatmul_norm_pair(dta, dev(wa).data_ptr(), na, ya.data_ptr(), dtb, dev(wb).data_ptr(), nb, yb.data_ptr(), dev(x).data_ptr(),
                                   dev(part).data_ptr(), dev(nw).data_ptr(), 1e-5, k, None))
    # the single-tensor entry point gives the same bits
    za, zb = torch.empty((1, na), device="cuda"), torch.empty((1, nb), device="cuda")
    ok(lib.cq_nn_qmatmul_norm(dta, dev(wa).data_ptr(), dev(x).data_ptr(), dev(part).data_ptr(), dev(nw).data_ptr(), 1e-5, za.data_ptr(), k, na, None))
    ok(lib.cq_nn_qmatmul_norm(dtb, dev(wb).data_ptr(), dev(x).data_ptr(), dev(part).data_ptr(), dev(nw).data_ptr(), 1e-5, zb.data_ptr(), k, nb, None))
    assert np.array_equal(ya.cpu().numpy(), za.cpu().numpy()) and np.array_equal(yb.cpu().numpy(), zb.cpu().numpy())
    xn = lo.rms_norm(x, nw, 1e-5)
    assert rel_l2(ya.cpu().numpy(), oracle.matmul_fast(dta, xn, wa, na, 8)) <= 1e-3
    assert rel_l2(yb.cpu().numpy(), oracle.matmul_fast(dtb, xn, wb, nb, 8)) <= 1e-3
    assert lib.cq_nn_qmatmul_norm_pair(8, dev(wa).data_ptr(), na, ya.data_ptr(), dtb, dev(wb).data_ptr(), nb, yb.data_ptr(), dev(x).data_ptr(),
                                       dev(part).data_ptr(), dev(nw).data_ptr(), 1e-5, k, None) == -1


def split_planes(dtype, k):
    """The fewest equal slices of whole blocks (2..4) that are at most one wave step long: 64 units of 64 elements for
    K-quants, of 32 elements for Q4_0 / Q8_0."""
    blk, unit = (256, 64) if dtype in (12, 13, 14) else (32, 32)
    if k % blk:
        return 0
    for p in range(2, 5):
        if (k // blk) % p == 0 and (k // p) // unit <= 64:
            return p
    return 0


@pytest.mark.parametrize("dtype,k", [(14, 14336), (12, 14336), (14, 4096), (12, 8192), (13, 16384), (2, 4096), (8, 6144)])
@pytest.mark.parametrize("n,with_up", [(4096, False), (300, True)])
def test_split_matvec_planes_and_merge_consumers(dtype, k, n, with_up):
    """feed_forward_w2 split along K: the planes add up to the unsplit matvec (each K-slice quantized exactly like the
    CPU, so a plane equals the CPU matmul over that slice), and the rms_norm consumers that add the planes back
    equal rms_norm + matmul over the merged row."""
    import oracle
    lib = L()
    S = split_planes(dtype, k)
    assert S >= 2 and lib.cq_nn_qmatmul_split_planes(dtype, k) == S
    x = normal(80, (1, k), 1.0)
    up = normal(81, (1, k), 1.0)
    w = oracle.from_float(dtype, normal(82, (n, k), 0.02).reshape(-1))
    planes = torch.full((S, n), 5.0, device="cuda")
    ok(lib.cq_nn_qmatmul_split(dtype, dev(w).data_ptr(), dev(x).data_ptr(), dev(up).data_ptr() if with_up else None, planes.data_ptr(), k, n, None))
    h = (lo.silu(x) * up).astype(np.float32) if with_up else x
    got = planes.cpu().numpy()
    want_total = oracle.matmul_fast(dtype, h, w, n, 8)
    acc = np.zeros((1, n), dtype=np.float32)
    for s_ in range(S):
        acc = acc + got[s_:s_ + 1]
    assert rel_l2(acc, want_total) <= (1e-4 if with_up else 1e-5)
    # one plane on its own: the matmul over that K-slice
    sl = k // S
    blk_bytes, blk_elems = {2: (18, 32), 8: (34, 32), 12: (144, 256), 13: (176, 256), 14: (210, 256)}[dtype]
    rows_b = np.asarray(w).view(np.uint8).reshape(n, k // blk_elems * blk_bytes)
    w_slice = np.ascontiguousarray(rows_b[:, sl // blk_elems * blk_bytes:2 * sl // blk_elems * blk_bytes]).reshape(-1)
    want1 = oracle.matmul_fast(dtype, np.ascontiguousarray(h[:, sl:2 * sl]), w_slice, n, 8)
    assert rel_l2(got[1:2], want1) <= (1e-4 if with_up else 1e-5)

    # consumers: hidden row r (length n, must be whole blocks) + planes -> rms_norm -> matvec
    if n % 256 or S > 4:
        return
    r0 = normal(83, (1, n), 1.0)
    nw = (1.0 + 0.1 * normal(84, (n,), 1.0)).astype(np.float32)
    merged_want = r0.copy()
    for s_ in range(S):
        merged_want = merged_want + got[s_:s_ + 1]
    xn = lo.rms_norm(merged_want, nw, 1e-5)
    na, nb = 1536, 512
    wa = oracle.from_float(12, normal(85, (na, n), 0.03).reshape(-1))
    wb = oracle.from_float(14, normal(86, (nb, n), 0.03).reshape(-1))
    ya, yb = torch.empty((1, na), device="cuda"), torch.empty((1, nb), device="cuda")
    rd = dev(r0)
    ok(lib.cq_nn_qmatmul_norm_pair_merge(12, dev(wa).data_ptr(), na, ya.data_ptr(), 14, dev(wb).data_ptr(), nb, yb.data_ptr(), rd.data_ptr(),
                                         planes.data_ptr(), S, dev(nw).data_ptr(), 1e-5, n, None))
    assert rel_l2(ya.cpu().numpy(), oracle.matmul_fast(12, xn, wa, na, 8)) <= 1e-3
    assert rel_l2(yb.cpu().numpy(), oracle.matmul_fast(14, xn, wb, nb, 8)) <= 1e-3
    assert np.array_equal(rd.cpu().numpy(), r0)                               # the residual row itself is only read
    # single-tensor consumer (the output head); a short tensor still gets one wave per span
    for dt_c, n_c in ((14, 2000), (12, 40)):
        wc = oracle.from_float(dt_c, normal(87, (n_c, n), 0.03).reshape(-1))
        yc = torch.empty((1, n_c), device="cuda")
        ok(lib.cq_nn_qmatmul_norm_merge(dt_c, dev(wc).data_ptr(), rd.data_ptr(), planes.data_ptr(), S, dev(nw).data_ptr(), 1e-5, yc.data_ptr(),
                                        n, n_c, None))
        assert rel_l2(yc.cpu().numpy(), oracle.matmul_fast(dt_c, xn, wc, n_c, 8)) <= 1e-3
    # the residual add that folds the planes into the row: row = merged + W . y, and its sum of squares
    for up_too in (False, True):
        kk = 512
        y = normal(88, (1, kk), 1.0)
        u = normal(89, (1, kk), 1.0)
        wr = oracle.from_float(12, normal(90, (n, kk), 0.05).reshape(-1))
        res = dev(r0)
        part = torch.empty((256,), device="cuda")
        ok(lib.cq_nn_qmatmul_residual_merge(12, dev(wr).data_ptr(), dev(y).data_ptr(), dev(u).data_ptr() if up_too else None, res.data_ptr(),
                                            part.data_ptr(), planes.data_ptr(), S, kk, n, None))
        act = (lo.silu(y) * u).astype(np.float32) if up_too else y
        want_res = merged_want + oracle.matmul_fast(12, act, wr, n, 8)
        got_res = res.cpu().numpy()
        assert rel_l2(got_res, want_res) <= (1e-4 if up_too else 1e-5)
        assert np.isclose(part.cpu().numpy().astype(np.float64).sum(), float((got_res.astype(np.float64) ** 2).sum()), rtol=1e-5)


@pytest.mark.parametrize("dtype", [12, 14, 2])
def test_attention_merge_prologue_with_planes(dtype):
    """attention_wo fed from the attention partials, folding two pending planes into the residual row."""
    import oracle
    lib = L()
    D, max_kv, k, n = 128, 512, 1024, 1024
    splits = lib.cq_nn_attention_decode_splits(max_kv)
    rec = D + 4
    rng = np.random.default_rng(91)
    Hn = k // D
    partials = np.zeros((Hn, splits, rec), dtype=np.float32)
    partials[:, :, :D] = rng.standard_normal((Hn, splits, D)).astype(np.float32)
    partials[:, :, D] = rng.standard_normal((Hn, splits)).astype(np.float32)           # m
    partials[:, :, D + 1] = rng.uniform(0.5, 2.0, (Hn, splits)).astype(np.float32)     # l
    m = partials[:, :, D].max(axis=1, keepdims=True)
    wgt = np.exp(partials[:, :, D] - m)
    att = ((wgt[:, :, None] * partials[:, :, :D]).sum(axis=1) / (wgt * partials[:, :, D + 1]).sum(axis=1, keepdims=True)).reshape(1, k)
    w = oracle.from_float(dtype, normal(92, (n, k), 0.05).reshape(-1))
    r0 = normal(93, (1, n), 1.0)
    pl = normal(94, (2, n), 0.5)
    res, part = dev(r0), torch.empty((256,), device="cuda")
    ok(lib.cq_nn_qmatmul_residual_attn_merge(dtype, dev(w).data_ptr(), dev(partials).data_ptr(), splits, D, res.data_ptr(), part.data_ptr(),
                                             dev(pl).data_ptr(), 2, k, n, None))
    want = ((r0 + pl[0:1]) + pl[1:2]) + oracle.matmul_fast(dtype, att.astype(np.float32), w, n, 8)
    assert rel_l2(res.cpu().numpy(), want) <= 1e-4
    # and without planes it is the plain call
    res2, res3 = dev(r0), dev(r0)
    ok(lib.cq_nn_qmatmul_residual_attn_merge(dtype, dev(w).data_ptr(), dev(partials).data_ptr(), splits, D, res2.data_ptr(), part.data_ptr(),
                                             None, 0, k, n, None))
    ok(lib.cq_nn_qmatmul_residual_attn(dtype, dev(w).data_ptr(), dev(partials).data_ptr(), splits, D, res3.data_ptr(), part.data_ptr(), k, n, None))
    assert np.array_equal(res2.cpu().numpy(), res3.cpu().numpy())


def test_split_matvec_availability():
    lib = L()
    assert lib.cq_nn_qmatmul_split_planes(12, 14336) == 4 and lib.cq_nn_qmatmul_split_planes(14, 14336) == 4
    assert lib.cq_nn_qmatmul_split_planes(8, 14336) == 0          # would need 7 planes: more than a consumer adds
    assert lib.cq_nn_qmatmul_split_planes(14, 256) == 0           # a single block: nothing to split
    assert lib.cq_nn_qmatmul_split_planes(12, 256 * 17) == 0      # 17 blocks: no equal split into 2..4 slices
    assert lib.cq_nn_qmatmul_split_planes(12, 256 * 1024) == 0    # slices longer than a wave step even in 4 planes
    assert lib.cq_nn_qmatmul_split_planes(15, 4096) == 0
    assert lib.cq_nn_qmatmul_split(12, 256, 256, None, 256, 256 * 17, 64, None) == -6
    assert lib.cq_nn_qmatmul_norm_merge(12, 256, 256, 256, 2, 256, 1e-5, 256, 8192, 64, None) == -6
    assert lib.cq_nn_qmatmul_norm_merge(12, 256, 256, 256, 5, 256, 1e-5, 256, 4096, 64, None) == -6


def test_argument_validation():
    lib = L()
    assert lib.cq_nn_rms_norm(16, None, 16, None, 16, 1, 6, 1e-5, None) == -2          # dim % 4
    assert lib.cq_nn_rms_norm(None, None, 16, None, 16, 1, 8, 1e-5, None) == -4
    assert lib.cq_nn_attention(16, 384, 16, 16, 16, None, 0, 1, 4, 2, 96, 8, 1, 0.1, None, 0, None) == -6   # head_dim 96
    assert lib.cq_nn_attention(16, 256, 16, 16, 16, None, 0, 1, 4, 3, 64, 8, 1, 0.1, None, 0, None) == -2   # heads not divisible
    assert lib.cq_nn_attention(16, 256, 16, 16, 16, None, 0, 1, 4, 2, 64, 1024, 600, 0.1, None, 0, None) == -5   # splits need a workspace
    assert lib.cq_nn_silu_mul(16, 16, 16, 1, 8, 4, 8, None) == -2
    assert lib.cq_nn_rope_i_kv(16, 16, 16, 16, 16, 16, 16, None, 7, 2, 4, 2, 64, 8, 256, 128, 128, None) == -6   # pos + rows > ctx
