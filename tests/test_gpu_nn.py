"""GPU parity of the module layer (kq.nn) against the CPU oracle: the call conventions of the
reference's mlx_kquant/nn.py -- transpose=True, expert ids as rhs_indices, bias added after the op,
embedding = gather wire rows then decode -- as its tests/test_nn.py expects them (forward == decode +
plain matmul)."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import bits_to_dev, dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def knn():
    import kq.nn as _nn
    return _nn


def _wire(codec, rows, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, rows * (K // wpb), seed).reshape(rows, K // wpb * bpb)


def _rel(got_f32, want_f32):
    g, w = np.asarray(got_f32, np.float64), np.asarray(want_f32, np.float64)
    return float(np.linalg.norm(g - w) / (np.linalg.norm(w) + 1e-30))


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "q8_0", "iq4_xs"])
@pytest.mark.parametrize("bias", [False, True])
def test_linear(knn, codec, bias):
    N, K = 264, 512
    wire = _wire(codec, N, K, seed=71)
    layer = knn.KQuantLinear(K, N, bias, codec, device="cuda:0")
    assert layer.mode == "kquant" and layer.kquant_type == codec and layer.biases is None
    assert tuple(layer.weight.shape) == (N, wire.shape[1]) and layer.weight.dtype == torch.uint8
    b = np.random.default_rng(72).standard_normal(N).astype(np.float32)
    layer.load_wire(wire_to_dev(wire), torch.from_numpy(b).cuda() if bias else None)
    for shape in ((1, K), (2, 3, K), (40, K)):
        xb, xt = make_x(shape, "bfloat16", seed=73)
        y = layer(xt)
        want = O.bits_to_f32(O.qmm(xb.reshape(-1, K), wire, codec, True, "bfloat16"), "bfloat16").reshape(*shape[:-1], N)
        assert tuple(y.shape) == (*shape[:-1], N)
        if bias and codec == "q8_0" and shape == (1, K):
            # fused decode path: x.W^T in f32 + the bias rounded to bf16, one rounding of the sum
            assert y.dtype == torch.bfloat16
            f32 = O.qmm(O.bits_to_f32(xb, "bfloat16").reshape(1, K), wire, codec, True, "float32")
            bb = O.bits_to_f32(O.f32_to_bits(b, "bfloat16"), "bfloat16")
            assert rel_l2(dev_to_bits(y), O.f32_to_bits(f32 + bb, "bfloat16"), "bfloat16") <= TOL
        elif bias:
            assert y.dtype == torch.float32  # bf16 + f32 bias promotes, as in the reference
            assert _rel(y.cpu().numpy(), want + b) <= TOL
        else:
            assert y.dtype == torch.bfloat16
            assert _rel(y.float().cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "q5_0", "iq3_s"])
def test_embedding(knn, codec):
    V, D = 300, 512
    wire = _wire(codec, V, D, seed=74)
    emb = knn.KQuantEmbedding(V, D, codec, device="cuda:0").load_wire(wire_to_dev(wire))
    ids = np.random.default_rng(75).integers(0, V, (3, 7))
    out = emb(torch.from_numpy(ids).cuda())
    assert tuple(out.shape) == (3, 7, D) and out.dtype == torch.bfloat16
    # decode to float16 (the op's default), then cast to the compute dtype: bit-exact
    f16 = O.bits_to_f32(O.dequantize(wire[ids.reshape(-1)], codec, "float16"), "float16")
    want = O.f32_to_bits(f16, "bfloat16").reshape(3, 7, D)
    assert np.array_equal(dev_to_bits(out), want)
    # tied lm_head
    xb, xt = make_x((2, D), "bfloat16", seed=76)
    y = emb.as_linear(xt)
    assert rel_l2(dev_to_bits(y), O.qmm(xb, wire, codec, True, "bfloat16"), "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q2_k", "mxfp4"])
@pytest.mark.parametrize("bias", [False, True])
def test_switch_linear(knn, codec, bias):
    """mlx-lm SwitchGLU shapes: x [T, 1, 1, K] with indices [T, R] (decode / unsorted), and the sorted
    prefill layout x [B, 1, K] with indices [B] ascending."""
    E, N, K, T, R = 6, 136, 512 if codec != "mxfp4" else 288, 9, 3
    wpb, bpb = O.geometry(codec)
    wire = O.synth_wire(codec, E * N * (K // wpb), 77).reshape(E, N, K // wpb * bpb)
    layer = knn.KQuantSwitchLinear(E, N, K, bias, codec, device="cuda:0")
    b = np.random.default_rng(78).standard_normal((E, N)).astype(np.float32)
    layer.load_wire(wire_to_dev(wire), torch.from_numpy(b).cuda() if bias else None)
    rng = np.random.default_rng(79)
    idx = rng.integers(0, E, (T, R))
    xb, xt = make_x((T, 1, 1, K), "bfloat16", seed=80)
    y = layer(xt, torch.from_numpy(idx).cuda())
    assert tuple(y.shape) == (T, R, 1, N)
    lhs = np.repeat(np.arange(T), R)
    want = O.bits_to_f32(O.gather_qmm(xb.reshape(T, 1, K), wire, codec, lhs, idx.reshape(-1), True, "bfloat16"),
                         "bfloat16").reshape(T, R, 1, N)
    if bias:
        want = want + b[idx][:, :, None, :]
    assert _rel(y.float().cpu().numpy(), want) <= TOL
    # sorted prefill layout
    B = 70
    sidx = np.sort(rng.integers(0, E, B))
    xb, xt = make_x((B, 1, K), "bfloat16", seed=81)
    y = layer(xt, torch.from_numpy(sidx).cuda(), sorted_indices=True)
    assert tuple(y.shape) == (B, 1, N)
    want = O.bits_to_f32(O.gather_qmm(xb, wire, codec, np.arange(B), sidx, True, "bfloat16"), "bfloat16")
    if bias:
        want = want + b[sidx][:, None, :]
    assert _rel(y.float().cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q8_0"])
def test_multi_linear(knn, codec):
    H, OUT, IN, B, L = 4, 64, 512, 2, 5
    wpb, bpb = O.geometry(codec)
    wire = O.synth_wire(codec, H * OUT * (IN // wpb), 82).reshape(H, OUT, IN // wpb * bpb)
    layer = knn.KQuantMultiLinear(IN, OUT, H, codec, device="cuda:0").load_wire(wire_to_dev(wire))
    # transpose=True: per-head activations [B, H, L, IN] -> [B, H, L, OUT]
    xb, xt = make_x((B, H, L, IN), "float16", seed=83)
    y = layer(xt)
    assert tuple(y.shape) == (B, H, L, OUT)
    want = O.gather_qmm(xb.reshape(B * H, L, IN), wire, codec, np.arange(B * H), np.tile(np.arange(H), B), True,
                        "float16")
    assert rel_l2(dev_to_bits(y).reshape(B * H, L, OUT), want, "float16") <= TOL
    y2 = layer(xt)  # memoized index arrays
    assert torch.equal(y, y2)
    # transpose=False: a head-shared activation [B, 1, L, OUT] @ W[h] ([OUT, IN]) -> [B, H, L, IN]
    xb, xt = make_x((B, 1, L, OUT), "float16", seed=84)
    y = layer(xt, transpose=False)
    assert tuple(y.shape) == (B, H, L, IN)
    want = O.gather_qmm(xb.reshape(B, L, OUT), wire, codec, np.repeat(np.arange(B), H), np.tile(np.arange(H), B),
                        False, "float16")
    assert rel_l2(dev_to_bits(y).reshape(B * H, L, IN), want, "float16") <= TOL
    with pytest.raises(ValueError):
        layer(torch.zeros((B, 3, L, IN), dtype=torch.float16, device="cuda:0"))


def test_checkpoint_and_gguf_feed_the_kernels(knn, tmp_path):
    """float model -> kq.quantize -> checkpoint on disk -> load -> install on the GPU: the swapped layers compute
    x @ decode(wire).T (oracle parity), and the same wire bytes travel through a GGUF file unchanged."""
    from kq import checkpoint, gguf

    class Toy(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = torch.nn.Embedding(64, 256)
            self.up = torch.nn.Linear(256, 128, bias=False)
            self.down = torch.nn.Linear(128 * 2, 256, bias=True)

        def forward(self, ids):
            h = self.up(self.embed(ids))
            return self.down(torch.cat([h, h], dim=-1))

    torch.manual_seed(1)
    ref = Toy()
    state = {k: v.detach().clone() for k, v in ref.state_dict().items()}
    tensors, per = checkpoint.quantize_state(state, {"embed": "q8_0", "up": "q4_k", "down": "q6_k"})
    d = str(tmp_path / "toy")
    checkpoint.save(d, tensors, per, config={"model_type": "toy"})
    model = checkpoint.install(Toy(), checkpoint.load(d), device="cuda:0")
    assert isinstance(model.up, knn.KQuantLinear) and model.up.weight.is_cuda
    ids = torch.tensor([[1, 5, 9], [63, 0, 2]], device="cuda:0")
    y = model(ids)
    assert tuple(y.shape) == (2, 3, 256)
    # layer by layer against the oracle on the same wire bytes
    e = model.embed(ids)
    want_e = O.f32_to_bits(O.bits_to_f32(O.dequantize(tensors["embed.weight"].numpy()[ids.cpu().numpy().reshape(-1)], "q8_0",
                                                      "float16"), "float16"), "bfloat16").reshape(2, 3, 256)
    assert np.array_equal(dev_to_bits(e), want_e)
    h = model.up(e)
    want_h = O.qmm(dev_to_bits(e).reshape(6, 256), tensors["up.weight"].numpy(), "q4_k", True, "bfloat16")
    assert rel_l2(dev_to_bits(h).reshape(6, 128), want_h, "bfloat16") <= TOL
    # and close to the float model within the codecs' error
    y_ref = ref(ids.cpu()).detach().numpy()
    assert _rel(y.float().cpu().numpy(), y_ref) < 0.15
    # the same bytes through a GGUF file
    path = str(tmp_path / "toy.gguf")
    gguf.save_gguf(path, {"up.weight": tensors["up.weight"], "down.weight": tensors["down.weight"]},
                   {"up.weight": "q4_k", "down.weight": "q6_k"}, {"general.architecture": "toy"})
    g = gguf.load_gguf(path, device="cuda:0")
    layer = knn.KQuantLinear(256, 128, False, dict(g.codecs)["up.weight"], device="cuda:0").load_wire(g.arrays["up.weight"])
    assert torch.equal(layer(e), h)
