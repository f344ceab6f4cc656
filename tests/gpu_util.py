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


def synth_wire_dev(codec, rows, K, seed):
    """Structurally valid random wire minted on the GPU (random code bytes, sane scale fields so that decode stays
    finite) for matrices too large to draw with numpy in a test: uint8 [rows, bytes_per_row]."""
    wpb, bpb = O.geometry(codec)
    nb = rows * (K // wpb)
    g = torch.Generator(device=dev())
    g.manual_seed(seed)
    wire = torch.randint(0, 256, (nb, bpb), dtype=torch.uint8, device=dev(), generator=g)
    d = (torch.rand(nb, 2, device=dev(), generator=g) * 0.006 + 0.004).to(torch.float16).view(torch.uint8).reshape(nb, 4)
    off = {"q4_k": (0, 2), "q5_k": (0, 2), "q4_1": (0, 2), "q5_1": (0, 2), "q6_k": (208,), "q3_k": (108,),
           "q2_k": (80, 82)}.get(codec, (0,))
    if codec == "mxfp4":
        wire[:, 0] = torch.randint(121, 130, (nb,), dtype=torch.uint8, device=dev(), generator=g)
    elif codec == "nvfp4":
        wire[:, 0:4] = torch.randint(0x08, 0x19, (nb, 4), dtype=torch.uint8, device=dev(), generator=g)
    elif codec == "iq1_m":
        raise ValueError("iq1_m keeps its scale in nibbles: mint it with oracle_lib.synth_wire")
    else:
        for i, o in enumerate(off):
            wire[:, o:o + 2] = d[:, 2 * i:2 * i + 2]
    return wire.reshape(rows, K // wpb * bpb)
