"""GPU parity: gradients with respect to the activations through kq.quantized_matmul and kq.gather_qmm (the frozen
quantized base of a LoRA-style setup), against dy @ dequant(W) computed from the CPU oracle's decode; the cases of
the reference's tests/test_vjp.py."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import wire_to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _wire(codec, rows, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, rows * (K // wpb), seed).reshape(rows, K // wpb * bpb)


def _rel(a, b):
    return np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-12)


@pytest.mark.parametrize("codec", ["q8_0", "q4_k", "iq4_xs"])
@pytest.mark.parametrize("M", [1, 5, 40])
def test_matmul_vjp_matches_oracle(kq, codec, M):
    N, K = 96, 512
    wire = _wire(codec, N, K, seed=3)
    wd = O.dequantize(wire, codec).reshape(N, K).astype(np.float64)
    rng = np.random.default_rng(4)
    x = torch.from_numpy((rng.standard_normal((M, K)) * 0.1).astype(np.float32)).cuda().to(torch.float16).requires_grad_()
    cot = (rng.standard_normal((M, N)) * 0.1).astype(np.float32)
    y = kq.quantized_matmul(x, wire_to_dev(wire), None, codec)
    (y.float() * torch.from_numpy(cot).cuda()).sum().backward()
    want = cot.astype(np.float16).astype(np.float64) @ wd  # the cotangent reaches the op in y's dtype
    assert x.grad is not None and x.grad.dtype == torch.float16 and tuple(x.grad.shape) == (M, K)
    assert _rel(x.grad.float().cpu().numpy().astype(np.float64), want) < 3e-3
    # the other orientation: y = x @ W has d/dx = dy @ W.T
    x2 = torch.from_numpy((rng.standard_normal((M, N)) * 0.1).astype(np.float32)).cuda().to(torch.float16).requires_grad_()
    cot2 = (rng.standard_normal((M, K)) * 0.1).astype(np.float32)
    y2 = kq.quantized_matmul(x2, wire_to_dev(wire), None, codec, transpose=False)
    (y2.float() * torch.from_numpy(cot2).cuda()).sum().backward()
    want2 = cot2.astype(np.float16).astype(np.float64) @ wd.T
    assert _rel(x2.grad.float().cpu().numpy().astype(np.float64), want2) < 3e-3


def test_dense_frozen_layer_trains_upstream_param(kq):
    """A trainable matrix in front of a frozen quantized layer: the loss falls, the gradient is finite and not zero,
    the wire bytes do not change."""
    N, K, H = 64, 256, 32
    torch.manual_seed(0)
    w_dev, _ = kq.quantize((torch.randn(N, K) * 0.1).cuda(), "q8_0")
    before = w_dev.clone()
    a = (torch.randn(H, K, device="cuda") * 0.05).requires_grad_()
    inp = torch.randn(16, H, device="cuda")
    target = torch.randn(16, N, device="cuda") * 0.1
    losses = []
    for _ in range(8):
        y = kq.quantized_matmul((inp @ a).to(torch.float16), w_dev, None, "q8_0")
        loss = ((y.float() - target) ** 2).mean()
        loss.backward()
        assert torch.isfinite(a.grad).all() and a.grad.abs().max() > 0
        with torch.no_grad():
            a -= 0.2 * a.grad
            a.grad = None
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0]
    assert torch.equal(w_dev, before)


def test_moe_gather_vjp_scatter_add(kq):
    """gather_qmm with a non-identity lhs selection (rows of x picked twice and never): the gradient of a picked row
    is the sum over its entries, an unpicked row gets zero."""
    E, N, K, M = 3, 48, 256, 2
    wpb, bpb = O.geometry("q8_0")
    wire = O.synth_wire("q8_0", E * N * (K // wpb), 6).reshape(E, N, K // wpb * bpb)
    wd = O.dequantize(wire, "q8_0").reshape(E, N, K).astype(np.float64)
    rng = np.random.default_rng(7)
    x = torch.from_numpy((rng.standard_normal((4, M, K)) * 0.1).astype(np.float32)).cuda().to(torch.float16).requires_grad_()
    lhs = np.array([2, 0, 2, 3, 0])
    rhs = np.array([1, 0, 2, 1, 1])
    cot = (rng.standard_normal((5, M, N)) * 0.1).astype(np.float32)
    y = kq.gather_qmm(x, wire_to_dev(wire), None, "q8_0", lhs_indices=torch.from_numpy(lhs).cuda(),
                      rhs_indices=torch.from_numpy(rhs).cuda())
    assert tuple(y.shape) == (5, M, N)
    (y.float() * torch.from_numpy(cot).cuda()).sum().backward()
    want = np.zeros((4, M, K))
    c16 = cot.astype(np.float16).astype(np.float64)
    for i in range(5):
        want[lhs[i]] += c16[i] @ wd[rhs[i]]
    got = x.grad.float().cpu().numpy().astype(np.float64)
    assert not got[1].any()
    assert _rel(got, want) < 3e-3
    # sorted rhs-only call (the MoE layer's convention)
    x3 = torch.from_numpy((rng.standard_normal((6, 1, K)) * 0.1).astype(np.float32)).cuda().to(torch.bfloat16).requires_grad_()
    rhs3 = np.array([0, 0, 1, 1, 2, 2])
    y3 = kq.gather_qmm(x3, wire_to_dev(wire), None, "q8_0", rhs_indices=torch.from_numpy(rhs3).cuda(), sorted_indices=True)
    y3.float().sum().backward()
    want3 = np.stack([wd[e].sum(0) for e in rhs3])[:, None, :]
    assert _rel(x3.grad.float().cpu().numpy().astype(np.float64), want3) < 1e-2  # bf16 rounding of the gradient


def test_no_grad_path_is_unchanged(kq):
    wire = _wire("q4_k", 32, 256, seed=8)
    x = torch.randn(3, 256, device="cuda", dtype=torch.float16, requires_grad=True)
    with torch.no_grad():
        y = kq.quantized_matmul(x, wire_to_dev(wire), None, "q4_k")
    assert not y.requires_grad
    assert torch.equal(y, kq.quantized_matmul(x.detach(), wire_to_dev(wire), None, "q4_k"))
