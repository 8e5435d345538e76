"""GGUF files on the GPU: tensors written from device QTensors come back as the same blocks in HBM, and a decoder
loaded from a file (ModelWeights.from_gguf, quantized_llama.rs:367-540) computes what the same weights handed over
directly compute — bit for bit, since the loader uploads the file's blocks as they are.  The reference holds no GGUF
files (its model tests download them); the file here is written by this build's writer, whose layout the CPU tests pin
against the reference's reader tests."""
import io

import numpy as np
import pytest
import torch

import oracle
from oracle import llama_oracle as lo
from tests.util import normal, rel_l2

pytestmark = pytest.mark.gpu

NAMES = {"attention_wq": "attn_q", "attention_wk": "attn_k", "attention_wv": "attn_v", "attention_wo": "attn_output",
         "feed_forward_w1": "ffn_gate", "feed_forward_w2": "ffn_down", "feed_forward_w3": "ffn_up"}


def test_qtensors_round_trip_through_a_file():
    from candle_amd import GgmlDType, QTensor, gguf_file as gf
    x = torch.from_numpy(normal(5, (6, 512), 1.0)).cuda()
    qs = [("a.q4k", QTensor.quantize(x, GgmlDType.Q4K)), ("b.q6k", QTensor.quantize(x, GgmlDType.Q6K)),
          ("c.q8_0", QTensor.quantize(x[:, :96].contiguous(), GgmlDType.Q8_0)), ("d.q4_0", QTensor.quantize(x.reshape(2, 3, 512), GgmlDType.Q4_0))]
    f = io.BytesIO()
    gf.write(f, [("general.name", gf.Value.String("round trip"))], qs)
    f.seek(0)
    ct = gf.Content.read(f)
    assert ct.metadata["general.name"].to_string() == "round trip"
    for name, q in qs:
        back = ct.tensor(f, name, "cuda:0")
        assert back.shape() == q.shape() and back.dtype() == q.dtype() and back.data() == q.data()
        assert torch.equal(back.dequantize(), q.dequantize())
    # plain arrays of a file: f32 and f16 tensors
    from candle_amd.quantized import QStorage
    v = normal(6, (8,), 1.0)
    f2 = io.BytesIO()
    gf.write(f2, [], [("n.f32", QTensor.new(QStorage.from_data(v.tobytes(), "cuda:0", GgmlDType.F32), (8,))),
                      ("n.f16", QTensor.new(QStorage.from_data(v.astype(np.float16).tobytes(), "cuda:0", GgmlDType.F16), (8,)))])
    f2.seek(0)
    ct2 = gf.Content.read(f2)
    assert np.array_equal(ct2.tensor(f2, "n.f32", "cuda:0").dequantize().cpu().numpy(), v)
    assert np.array_equal(ct2.tensor(f2, "n.f16", "cuda:0").dequantize().cpu().numpy(), v.astype(np.float16).astype(np.float32))


class Blocks:
    """Host blocks with the four accessors the writer uses."""

    def __init__(self, dtype, shape, data):
        self._d, self._s, self._b = dtype, tuple(shape), bytes(data)

    def shape(self): return self._s
    def dtype(self): return self._d
    def storage_size_in_bytes(self): return len(self._b)
    def data(self): return self._b


@pytest.mark.parametrize("tied", [False, True], ids=["output-tensor", "tied-embeddings"])
def test_decoder_from_a_gguf_file_equals_decoder_from_blocks(tied):
    from candle_amd import GgmlDType, gguf_file as gf
    from candle_amd.quantized_llama import Config, ModelWeights
    cfg = Config(n_layer=2, hidden=256, n_head=4, n_kv_head=2, head_dim=64, ffn=512, vocab=320, rope_theta=10000.0,
                 rms_eps=float(np.float32(1e-6)), ctx=64)       # the file holds the epsilon as an f32
    mix = {"attention_wq": oracle.Q4K, "attention_wk": oracle.Q4K, "attention_wv": oracle.Q6K, "attention_wo": oracle.Q4K,
           "feed_forward_w1": oracle.Q4K, "feed_forward_w3": oracle.Q4K, "feed_forward_w2": oracle.Q6K, "output": oracle.Q6K}
    t = lo.random_tensors(cfg, seed=31, dtypes=mix, weight_scale=0.05)
    # a file mixes formats per layer (Q4_K_M keeps attn_v / ffn_down in Q6_K for some layers only)
    other = lo.random_tensors(cfg, seed=32, dtypes=dict(mix, attention_wv=oracle.Q4K, feed_forward_w2=oracle.Q4K), weight_scale=0.05)
    for role in ("attention_wv", "feed_forward_w2"):
        t[f"blk.1.{role}"] = other[f"blk.1.{role}"]
    emb = np.asarray(t["tok_embeddings"], dtype=np.float32)
    if tied:
        # the token embedding doubles as the output head: stored quantized, dequantized for the lookup
        emb_blocks = oracle.from_float(oracle.Q6K, emb.reshape(-1))
        t["output"] = (oracle.Q6K, emb_blocks.tobytes())
        t["tok_embeddings"] = oracle.to_float(oracle.Q6K, emb_blocks, emb.size).reshape(emb.shape)
        emb_tensor = Blocks(GgmlDType.Q6K, emb.shape, emb_blocks.tobytes())
    else:
        emb_tensor = Blocks(GgmlDType.F32, emb.shape, emb.tobytes())
    shapes = {"attention_wq": (256, 256), "attention_wk": (128, 256), "attention_wv": (128, 256), "attention_wo": (256, 256),
              "feed_forward_w1": (512, 256), "feed_forward_w3": (512, 256), "feed_forward_w2": (256, 512)}
    tensors = [("token_embd.weight", emb_tensor), ("output_norm.weight", Blocks(GgmlDType.F32, (256,), np.asarray(t["norm"], np.float32).tobytes()))]
    if not tied:
        tensors.append(("output.weight", Blocks(GgmlDType(t["output"][0]), (320, 256), bytes(t["output"][1]))))
    for i in range(cfg.n_layer):
        for mine, theirs in NAMES.items():
            dt, blocks = t[f"blk.{i}.{mine}"]
            tensors.append((f"blk.{i}.{theirs}.weight", Blocks(GgmlDType(dt), shapes[mine], bytes(blocks))))
        tensors.append((f"blk.{i}.attn_norm.weight", Blocks(GgmlDType.F32, (256,), np.asarray(t[f"blk.{i}.attention_norm"], np.float32).tobytes())))
        tensors.append((f"blk.{i}.ffn_norm.weight", Blocks(GgmlDType.F32, (256,), np.asarray(t[f"blk.{i}.ffn_norm"], np.float32).tobytes())))
    md = [("general.architecture", gf.Value.String("llama")), ("llama.attention.head_count", gf.Value.U32(4)),
          ("llama.attention.head_count_kv", gf.Value.U32(2)), ("llama.block_count", gf.Value.U32(2)),
          ("llama.embedding_length", gf.Value.U32(256)), ("llama.rope.dimension_count", gf.Value.U32(64)),
          ("llama.attention.layer_norm_rms_epsilon", gf.Value.F32(1e-6)), ("llama.rope.freq_base", gf.Value.F32(10000.0))]
    f = io.BytesIO()
    gf.write(f, md, tensors)
    f.seek(0)
    ct = gf.Content.read(f)
    loaded = ModelWeights.from_gguf(ct, f, "cuda:0", ctx=64)
    direct = ModelWeights.from_blocks(cfg, t)
    assert loaded.cfg == cfg
    rng = np.random.default_rng(33)
    prompt = rng.integers(0, cfg.vocab, size=12).tolist()
    a = loaded.forward(torch.tensor([prompt], dtype=torch.int32), 0).cpu().numpy()
    b = direct.forward(torch.tensor([prompt], dtype=torch.int32), 0).cpu().numpy()
    assert np.array_equal(a, b)
    ref = lo.LlamaOracle(cfg, t)
    assert rel_l2(a, ref.forward(prompt, 0)) <= 1e-3
    tok = int(np.argmax(a))
    a1 = loaded.forward(torch.tensor([[tok]], dtype=torch.int32), 12).cpu().numpy()
    b1 = direct.forward(torch.tensor([[tok]], dtype=torch.int32), 12).cpu().numpy()
    assert np.array_equal(a1, b1)
    assert rel_l2(a1, ref.forward([tok], 12)) <= 1e-3


def test_from_gguf_reports_what_is_missing_or_unsupported():
    from candle_amd import gguf_file as gf
    from candle_amd.quantized_llama import ModelWeights
    f = io.BytesIO()
    gf.write(f, [("llama.attention.head_count", gf.Value.U32(4))], [])
    f.seek(0)
    with pytest.raises(gf.GgufError) as e:
        ModelWeights.from_gguf(gf.Content.read(f), f)
    assert "cannot find llama.attention.head_count_kv in metadata" in str(e.value)
    md = [("general.architecture", gf.Value.String("qwen2")), ("llama.attention.head_count", gf.Value.U32(4)),
          ("llama.attention.head_count_kv", gf.Value.U32(2)), ("llama.block_count", gf.Value.U32(1)), ("llama.embedding_length", gf.Value.U32(256)),
          ("llama.rope.dimension_count", gf.Value.U32(64)), ("llama.attention.layer_norm_rms_epsilon", gf.Value.F32(1e-6))]
    f = io.BytesIO()
    gf.write(f, md, [])
    f.seek(0)
    with pytest.raises(NotImplementedError):
        ModelWeights.from_gguf(gf.Content.read(f), f)
