"""On-disk formats (CPU): the kquant safetensors checkpoint (config.json layout of the reference's converter,
docs/integration.md:73-95) and the GGUF reader against files written here and against hand-packed bytes."""
import json
import os
import struct

import numpy as np
import pytest
import torch

import oracle_lib as O
from kq import checkpoint, gguf


def _wire(codec, rows, K, seed):
    wpb, bpb = O.geometry(codec)
    return torch.from_numpy(O.synth_wire(codec, rows * (K // wpb), seed).reshape(rows, K // wpb * bpb).copy())


def test_checkpoint_round_trip_and_layout(tmp_path):
    tensors = {
        "model.layers.0.q_proj.weight": _wire("q4_k", 64, 512, 1),
        "model.layers.0.q_proj.bias": torch.randn(64),
        "model.layers.0.experts.up.weight": _wire("q6_k", 3 * 32, 256, 2).reshape(3, 32, -1),
        "model.embed.weight": _wire("q8_0", 100, 64, 3),
        "model.norm.weight": torch.randn(512).to(torch.bfloat16),
    }
    per = {"model.layers.0.q_proj": "q4_k", "model.layers.0.experts.up": "q6_k", "model.embed": "q8_0"}
    d = str(tmp_path / "ckpt")
    checkpoint.save(d, tensors, per, config={"model_type": "toy", "hidden_size": 512})
    cfg = json.load(open(os.path.join(d, "config.json")))
    assert cfg["quantization"] == {"mode": "kquant", "per_tensor": per} == cfg["quantization_config"]
    assert cfg["model_type"] == "toy"
    ck = checkpoint.load(d)
    assert ck.per_tensor == per
    for k, v in tensors.items():
        assert torch.equal(ck.tensors[k], v), k
    for p in per:  # placeholder scales are written even when the caller leaves them out
        s = ck.tensors[p + ".scales"]
        assert s.dtype == torch.uint8 and tuple(s.shape) == (1,)
    # sharded
    d2 = str(tmp_path / "sharded")
    checkpoint.save(d2, tensors, per, max_shard_bytes=20000)
    names = sorted(os.listdir(d2))
    assert "model.safetensors.index.json" in names and sum(n.endswith(".safetensors") for n in names) > 1
    idx = json.load(open(os.path.join(d2, "model.safetensors.index.json")))
    assert set(idx["weight_map"]) == set(ck.tensors)
    ck2 = checkpoint.load(d2)
    assert all(torch.equal(ck2.tensors[k], ck.tensors[k]) for k in ck.tensors)


def test_checkpoint_validation(tmp_path):
    with pytest.raises(ValueError):
        checkpoint.save(str(tmp_path / "a"), {"x.weight": torch.zeros(4, 100, dtype=torch.uint8)}, {"x": "q4_k"})
    with pytest.raises(ValueError):
        checkpoint.save(str(tmp_path / "b"), {"x.weight": torch.zeros(4, 144)}, {"x": "q4_k"})
    with pytest.raises(ValueError):
        checkpoint.save(str(tmp_path / "c"), {}, {"x": "q4_k"})
    os.makedirs(tmp_path / "d")
    json.dump({"model_type": "toy"}, open(tmp_path / "d" / "config.json", "w"))
    with pytest.raises(ValueError):
        checkpoint.load(str(tmp_path / "d"))


def test_quantize_state_and_install_swaps_leaves():
    class Toy(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = torch.nn.Embedding(50, 256)
            self.proj = torch.nn.Linear(256, 96, bias=True)
            self.norm = torch.nn.LayerNorm(96)

    torch.manual_seed(0)
    m = Toy()
    state = {k: v.detach().clone() for k, v in m.state_dict().items()}
    tensors, per = checkpoint.quantize_state(state, {"proj": "q4_k", "embed": "q8_0"})
    assert tensors["proj.weight"].dtype == torch.uint8 and tuple(tensors["proj.weight"].shape) == (96, 144)
    assert tuple(tensors["embed.weight"].shape) == (50, 272) and torch.equal(tensors["norm.weight"], state["norm.weight"])
    m2 = checkpoint.install(Toy(), checkpoint.Checkpoint({}, per, tensors))
    from kq import nn as kqnn
    assert isinstance(m2.proj, kqnn.KQuantLinear) and isinstance(m2.embed, kqnn.KQuantEmbedding)
    assert torch.equal(m2.proj.weight, tensors["proj.weight"]) and torch.equal(m2.proj.bias, state["proj.bias"])
    assert torch.equal(m2.norm.weight, state["norm.weight"])
    # decoded weights are the float ones up to the codec's error
    w = O.dequantize(tensors["proj.weight"].numpy(), "q4_k")
    assert np.linalg.norm(w - state["proj.weight"].numpy()) / np.linalg.norm(state["proj.weight"].numpy()) < 0.12
    with pytest.raises(ValueError):
        checkpoint.install(Toy(), checkpoint.Checkpoint({}, {"nope": "q4_k"}, {"nope.weight": tensors["proj.weight"]}))


def test_gguf_round_trip(tmp_path):
    tensors = {
        "blk.0.attn_q.weight": _wire("q4_k", 32, 512, 4),
        "blk.0.ffn_gate_exps.weight": _wire("iq4_xs", 2 * 16, 256, 5).reshape(2, 16, -1),
        "token_embd.weight": _wire("q8_0", 10, 64, 6),
        "blk.0.ffn_up_exps.weight": _wire("mxfp4", 2 * 8, 64, 7).reshape(2, 8, -1),     # ggml type 39
        "blk.0.ffn_down_exps.weight": _wire("nvfp4", 2 * 8, 128, 8).reshape(2, 8, -1),  # ggml type 40
        "blk.0.attn_norm.weight": torch.randn(512),
        "blk.0.bias_bf16": torch.randn(4, 6).to(torch.bfloat16),
    }
    codecs = {"blk.0.attn_q.weight": "q4_k", "blk.0.ffn_gate_exps.weight": "iq4_xs", "token_embd.weight": "q8_0",
              "blk.0.ffn_up_exps.weight": "mxfp4", "blk.0.ffn_down_exps.weight": "nvfp4"}
    meta = {"general.architecture": "llama", "llama.block_count": 1, "llama.rope.freq_base": 10000.0,
            "tokenizer.ggml.tokens": ["a", "b", "c"], "llama.flag": True, "some.ints": [1, -2, 3]}
    path = str(tmp_path / "toy.gguf")
    gguf.save_gguf(path, tensors, codecs, meta)
    g = gguf.load_gguf(path)
    for k, v in tensors.items():
        assert torch.equal(g.arrays[k], v), k
    assert g.codecs == list(codecs.items())
    assert g.tensor_shapes["blk.0.attn_q.weight"] == (512, 32)            # logical dims, innermost first
    assert g.tensor_shapes["blk.0.ffn_gate_exps.weight"] == (256, 16, 2)
    assert g.tensor_shapes["blk.0.bias_bf16"] == (6, 4)
    assert g.tensor_shapes["blk.0.ffn_up_exps.weight"] == (64, 8, 2)
    assert g.tensor_shapes["blk.0.ffn_down_exps.weight"] == (128, 8, 2)
    assert tuple(g.arrays["blk.0.attn_q.scales"].shape) == (1,)
    assert g.metadata["general.architecture"] == "llama" and g.metadata["llama.block_count"] == 1
    assert g.metadata["tokenizer.ggml.tokens"] == ["a", "b", "c"] and g.metadata["llama.flag"] is True
    assert g.metadata["some.ints"] == [1, -2, 3] and abs(g.metadata["llama.rope.freq_base"] - 10000.0) < 1e-3


def test_gguf_hand_packed_bytes(tmp_path):
    """A file assembled byte by byte from the format description: one q4_0 tensor [K=32, N=2] and a u32 key."""
    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b
    blocks = bytes(range(36))  # 2 rows x one 18-byte block
    head = b"GGUF" + struct.pack("<IQQ", 3, 1, 1) + s("answer") + struct.pack("<II", 4, 42)
    head += s("w.weight") + struct.pack("<IQQ", 2, 32, 2) + struct.pack("<IQ", 2, 0)
    pad = (-len(head)) % 32
    path = str(tmp_path / "hand.gguf")
    open(path, "wb").write(head + b"\0" * pad + blocks)
    g = gguf.load_gguf(path)
    assert g.metadata == {"answer": 42} and g.codecs == [("w.weight", "q4_0")]
    assert g.arrays["w.weight"].dtype == torch.uint8 and tuple(g.arrays["w.weight"].shape) == (2, 18)
    assert bytes(g.arrays["w.weight"].numpy().tobytes()) == blocks
    open(path, "wb").write(b"GGML" + head[4:])
    with pytest.raises(ValueError):
        gguf.load_gguf(path)
    open(path, "wb").write(head + b"\0" * pad + blocks[:20])
    with pytest.raises(ValueError):
        gguf.load_gguf(path)


def test_gguf_hand_packed_fp4_types(tmp_path):
    """ggml tensor types 39 (mxfp4: 32 weights in 17 bytes) and 40 (nvfp4: 64 weights in 36 bytes), the ids the
    reference's reader maps (src/kquant_gguf.cpp:246-252), in a file assembled byte by byte."""
    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b
    assert O.geometry("mxfp4") == (32, 17) and O.geometry("nvfp4") == (64, 36)
    mx = bytes(range(34))           # [K=32, N=2]: 2 rows x one 17-byte block
    nv = bytes(range(100, 172))     # [K=64, N=2]: 2 rows x one 36-byte block
    head = b"GGUF" + struct.pack("<IQQ", 3, 2, 0)
    head += s("a.weight") + struct.pack("<IQQ", 2, 32, 2) + struct.pack("<IQ", 39, 0)
    head += s("b.weight") + struct.pack("<IQQ", 2, 64, 2) + struct.pack("<IQ", 40, 64)
    pad = (-len(head)) % 32
    path = str(tmp_path / "fp4.gguf")
    open(path, "wb").write(head + b"\0" * pad + mx + b"\0" * 30 + nv)
    g = gguf.load_gguf(path)
    assert g.codecs == [("a.weight", "mxfp4"), ("b.weight", "nvfp4")]
    assert tuple(g.arrays["a.weight"].shape) == (2, 17) and bytes(g.arrays["a.weight"].numpy().tobytes()) == mx
    assert tuple(g.arrays["b.weight"].shape) == (2, 36) and bytes(g.arrays["b.weight"].numpy().tobytes()) == nv
