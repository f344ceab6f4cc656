"""Argument checks of the packed-layout mxfp4 ops run before anything touches a device
(check_expert_stack, reference src/kquant_moe_glu.cpp:802-841)."""
import pytest
import torch

import kq


def _stack(E=2, N=16, K=64, wdt=torch.int32):
    return (torch.zeros((E, N, K // 8), dtype=wdt), torch.zeros((E, N, K // 32), dtype=torch.uint8),
            torch.zeros((E, N), dtype=torch.float32))


def test_packed_stack_validation():
    w, s, b = _stack()
    x = torch.zeros((3, 64), dtype=torch.float16)
    idx = torch.zeros((3, 2), dtype=torch.int32)
    with pytest.raises(ValueError):  # byte codes instead of 32-bit words
        kq.moe_glu_gather(x, w.to(torch.uint8), s, b, w, s, b, idx)
    with pytest.raises(ValueError):  # scales not uint8
        kq.moe_glu_gather(x, w, s.to(torch.int32), b, w, s, b, idx)
    with pytest.raises(ValueError):  # K mismatch
        kq.moe_glu_gather(torch.zeros((3, 96), dtype=torch.float16), w, s, b, w, s, b, idx)
    with pytest.raises(ValueError):  # bias shape
        kq.moe_glu_gather(x, w, s, b[:, :8], w, s, b, idx)
    with pytest.raises(ValueError):  # N not a multiple of 8
        w2, s2, b2 = _stack(N=12)
        kq.moe_glu_gather(x, w2, s2, b2, w2, s2, b2, idx)
    with pytest.raises(ValueError):  # x not [T, K]
        kq.moe_glu_gather(x[None], w, s, b, w, s, b, idx)
    with pytest.raises(ValueError):  # indices do not match x
        kq.gather_qmv_bias(torch.zeros((3, 2, 64), dtype=torch.float16), w, s, b, idx[:2])
    with pytest.raises(ValueError):  # scores shape
        kq.gather_qmv_mix_bias(torch.zeros((3, 2, 64), dtype=torch.float16), w, s, b, idx, torch.zeros((3, 3)))
    with pytest.raises(ValueError):  # converter: trailing dims disagree
        kq.mxfp4_packed_to_wire(w, s[..., :1])
    with pytest.raises(ValueError):  # converter: wire not a whole number of blocks
        kq.mxfp4_wire_to_packed(torch.zeros((4, 18), dtype=torch.uint8))
    with pytest.raises(RuntimeError):  # valid arguments, but no device: there is no CPU path
        kq.mxfp4_packed_to_wire(w, s)
