"""Helpers shared by the GPU parity tests: torch <-> numpy bit-pattern moves and error metrics."""
import numpy as np
import torch

import oracle_lib as O

TORCH_DT = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def dev():
    return torch.device("cuda:0")


def wire_to_dev(wire):
    return torch.from_numpy(np.ascontiguousarray(wire, dtype=np.uint8)).to(dev())


def bits_to_dev(bits, dtype):
    """numpy storage (f32 or uint16 bit patterns) -> torch tensor of `dtype` on the GPU."""
    if dtype == "float32":
        return torch.from_numpy(np.ascontiguousarray(bits, dtype=np.float32)).to(dev())
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev())
    return t.view(TORCH_DT[dtype])


def dev_to_bits(t):
    """torch tensor -> numpy storage (f32, or uint16 bit patterns for half types)."""
    t = t.detach().contiguous().cpu()
    if t.dtype == torch.float32:
        return t.numpy()
    return t.view(torch.int16).numpy().view(np.uint16)


def make_x(shape, dtype, seed, scale=1.0):
    """Seeded N(0, scale) activations, returned as (numpy storage bits, torch GPU tensor)."""
    x = (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)
    bits = O.f32_to_bits(x, dtype)
    return bits, bits_to_dev(bits, dtype)


def rel_l2(got_bits, want_bits, dtype):
    g = O.bits_to_f32(got_bits, dtype).astype(np.float64)
    w = O.bits_to_f32(want_bits, dtype).astype(np.float64)
    return float(np.linalg.norm(g - w) / (np.linalg.norm(w) + 1e-30))
