#!/usr/bin/env python3
"""Benchmark of the quantized-weight hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-sweep] [--no-cpu]

Headline (the JSON line): q4_k GEMV at M=1 on the Llama-3-8B gate/up projection
(4096 -> 14336, bf16 activations, weights = seeded N(0, 0.02) quantized by kq.quantize),
measured COLD: every step reads a different copy of the wire matrix, the copies together
exceeding twice the 256 MB last-level cache, so the weight bytes come from HBM.
value = quantized weight bytes per step / step time (HIP events on the launching stream).

Every timed call goes through the C ABI of libkq (ctypes) with outputs and workspace allocated
beforehand.  A step is one batch of back-to-back launches (one rotation over the weight copies repeated to
at least 100 launches), captured once into a HIP graph and replayed, so the host's launch rate does not
enter the figure; `us_per_launch` = step time / `launches_per_step`.

Extra fields: `sweep` (the decode projections of the q4_k_m recipe at M in {1,2,4,8}), `prefill`
(q4_k / q5_k / q6_k / q2_k / q3_k / iq4_xs / q8_0 / q4_0 / mxfp4 / nvfp4 / iq3_s / iq2_xxs GEMM 8192 -> 28672 at M in {512, 2048}), `moe` (128 experts, top-8, hidden 2048,
intermediate 768: fused gate/up GLU in q4_k and down in q6_k at 1 and 256 tokens), `lowbit` (M=1
GEMV 8192 -> 8192 in the low-bit codecs), `moe_decode_lowbit` (1 token, 8 of 128 experts, IQ / fp4 / q8_0 stacks),
`read_ceiling` (stock read-only reduction, stock bf16 GEMV and device copy on buffers of the GEMV's sizes, cold),
`dequantize` (whole-matrix decode to f16, wire bytes in plus
2 N K bytes out), `mid_m` (16 ... 64 activation rows on 4096-wide matrices), `no_transpose` (transpose = 0:
128 gathered entries of (M x 128) . (128 x 512), and dense 4096 x 4096), `roofline` for the dominant kernel and `cpu_baseline`
(the CPU oracle timed on this box's host cores on the headline GEMV).
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
MFMA_F16_PEAK_TFLOPS = 2500.0
LLC_BYTES = 256 << 20
# HBM bytes one headline launch moves, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of
# `bench.py --probe` (KiB per dispatch of the GEMV kernel), each counter scaled by what it reads for the probe's
# plain 32256 KiB device copy (32256 / the copy's reading).  Algorithmic bytes are 33,030,144 (weights) + 28,672
# (output).
HEADLINE_FETCH_KIB, HEADLINE_FETCH_SCALE = 16254.3, 1.9984
HEADLINE_WRITE_KIB, HEADLINE_WRITE_SCALE = 28.0, 1.0
HEADLINE_TRAFFIC_BYTES = int(round((HEADLINE_FETCH_KIB * HEADLINE_FETCH_SCALE
                                    + HEADLINE_WRITE_KIB * HEADLINE_WRITE_SCALE) * 1024, -3))
KQ_BF16 = 2


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
    elif codec != "iq1_m":
        for i, o in enumerate(off):
            wire[:, o:o + 2] = d[:, 2 * i:2 * i + 2]
    return wire.reshape(rows, K // wpb * bpb)


def quantized_weights(kq, torch, codec, N, K, seed, device, unique_rows=None):
    """Seeded N(0, 0.02) f32 weights [N, K] encoded by kq.quantize and placed on the GPU.  Codecs with a device
    encoder (legacy and K-quants) are drawn and encoded on the GPU, in slabs of at most 64 Mi weights; the IQ
    codecs go through the host encoder with a uniform importance matrix.  With unique_rows only that many rows
    are drawn and encoded and the slab is repeated down the matrix (the codebook encoders search for ~1 us per
    weight; kernel time does not depend on the values)."""
    rows = min(N, unique_rows) if unique_rows else N
    if kq._load().kq_quantize_dev_supported(kq._load().kq_codec_id(codec.encode())):
        g = torch.Generator(device=device)
        g.manual_seed(seed)
        step = max(1, (64 << 20) // K)
        parts = []
        for r0 in range(0, rows, step):
            w = torch.randn((min(step, rows - r0), K), generator=g, dtype=torch.float32, device=device) * 0.02
            parts.append(kq.quantize(w, codec)[0])
            del w
        wq = parts[0] if len(parts) == 1 else torch.cat(parts)
    else:
        g = torch.Generator()
        g.manual_seed(seed)
        w = torch.randn((rows, K), generator=g, dtype=torch.float32) * 0.02
        wq = kq.quantize(w, codec, torch.ones(K) if codec.startswith("iq") else None)[0].to(device)
    if rows < N:
        wq = wq.repeat((N + rows - 1) // rows, 1)[:N].contiguous()
    return wq


def _time_direct(torch, calls, launches, warm):
    n = len(calls)
    for i in range(warm):
        calls[i % n]()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(launches):
        calls[i % n]()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return ev0.elapsed_time(ev1) / launches, wall_ms / launches


def capture_batch(torch, calls, batch, lanes=1):
    """A HIP graph of `batch` launches rotating over the closures in `calls` (each takes the stream to launch on),
    or None when the calls cannot be captured.  `lanes` > 1 deals the launches round-robin over that many streams
    forked from the capturing one and joined at the end: the graph then orders a launch only after the launches of
    its own lane (valid when the calls share no output or workspace)."""
    n = len(calls)
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(min(n, batch)):  # first calls outside the capture: one-time setup of the library
                calls[i](side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            main = torch.cuda.current_stream()
            if lanes <= 1:
                for i in range(batch):
                    calls[i % n](main.cuda_stream)
            else:
                forks = [torch.cuda.Stream() for _ in range(lanes)]
                for f in forks:
                    f.wait_stream(main)
                for i in range(batch):
                    calls[i % n](forks[i % lanes].cuda_stream)
                for f in forks:
                    main.wait_stream(f)
        return g
    except Exception as e:  # noqa: BLE001
        print(f"bench.py: graph capture unavailable ({e}); timing direct launches", file=sys.stderr)
        torch.cuda.synchronize()
        return None


def time_graph(torch, g, batch, steps, warmup, settle_ms=30.0):
    """`warmup` untimed replays (after enough untimed replays to bring the device to its steady clock), then
    exactly `steps` timed ones between two events.  Returns (ms per replay, wall ms per replay)."""
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    g.replay()
    ev1.record()
    torch.cuda.synchronize()
    one = max(ev0.elapsed_time(ev1), 1e-3)
    for _ in range(int(min(2000, settle_ms / one)) + warmup):
        g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        g.replay()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return ev0.elapsed_time(ev1) / steps, wall_ms / steps


def time_calls(torch, calls, launches, warm, graph=True):
    """Average time (ms) of one launch over about `launches` back-to-back launches rotating over the closures in
    `calls`.  The launches are replays of a HIP graph of one rotation (at least 20 launches), so the host's launch
    rate does not enter; calls that cannot be captured are timed as direct launches."""
    n = len(calls)
    batch = n * max(1, -(-20 // n))
    g = capture_batch(torch, calls, batch) if graph else None
    if g is None:
        direct = [(lambda c=c: c(None)) for c in calls] if graph else calls
        return _time_direct(torch, direct, launches, warm)
    reps = max(1, -(-launches // batch))
    ms, wall = time_graph(torch, g, batch, reps, max(1, warm // batch), settle_ms=10.0)
    return ms / batch, wall / batch


class Abi:
    """Closures over the C ABI with every buffer allocated up front."""

    def __init__(self, kq, torch, dev):
        self.kq, self.torch, self.dev = kq, torch, dev
        self.lib = kq._load()
        self.stream = torch.cuda.current_stream().cuda_stream

    def _check(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.kq_last_error().decode())

    def qmm(self, x, w, codec, N, K):
        torch, lib = self.torch, self.lib
        M = x.shape[0]
        cid = lib.kq_codec_id(codec.encode())
        out = torch.empty((M, N), dtype=x.dtype, device=self.dev)
        nws = lib.kq_qmm_workspace_size(M, N, K, 1, cid, KQ_BF16)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=self.dev)
        args = (x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, 1, cid, KQ_BF16, ws.data_ptr(), nws)
        keep = (x, w, out, ws)

        def call(stream=None, _keep=keep):
            rc = lib.kq_qmm(*args, stream or self.stream)
            if rc:
                self._check(rc)
        return call

    def qmm_nt(self, x, w, codec, K, N):
        """transpose = 0: x [M, K] . W, W stored as K wire rows of N weights."""
        torch, lib = self.torch, self.lib
        M = x.shape[0]
        cid = lib.kq_codec_id(codec.encode())
        out = torch.empty((M, N), dtype=x.dtype, device=self.dev)
        nws = lib.kq_qmm_workspace_size(M, N, K, 0, cid, KQ_BF16)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=self.dev)
        args = (x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, 0, cid, KQ_BF16, ws.data_ptr(), nws)
        keep = (x, w, out, ws)

        def call(stream=None, _keep=keep):
            rc = lib.kq_qmm(*args, stream or self.stream)
            if rc:
                self._check(rc)
        return call

    def gather_nt(self, x, w, codec, rhs, E, K, N):
        """transpose = 0, gathered: entry b = x[b] ([M, K]) . W[rhs[b]], every expert K wire rows of N weights."""
        torch, lib = self.torch, self.lib
        B, M = x.shape[0], x.shape[1]
        cid = lib.kq_codec_id(codec.encode())
        out = torch.empty((B, M, N), dtype=x.dtype, device=self.dev)
        lhs = torch.arange(B, dtype=torch.int32, device=self.dev)
        args = (x.data_ptr(), w.data_ptr(), lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), B, M, E, N, K, M * K,
                w.numel() // E, 0, 0, cid, KQ_BF16, 0, 0)
        keep = (x, w, out, lhs, rhs)

        def call(stream=None, _keep=keep):
            rc = lib.kq_gather_qmm(*args, stream or self.stream)
            if rc:
                self._check(rc)
        return call

    def dequantize(self, w, codec, N, K, out):
        lib = self.lib
        cid = lib.kq_codec_id(codec.encode())
        args = (w.data_ptr(), out.data_ptr(), N * K, cid, 1)  # dtype code 1 = float16
        keep = (w, out)

        def call(stream=None, _keep=keep):
            rc = lib.kq_dequantize(*args, stream or self.stream)
            if rc:
                self._check(rc)
        return call

    def moe_glu(self, x, gate, up, codec, idx, act=0, limit=0.0, alpha=0.0, gate_bias=None, up_bias=None):
        """act: 0 silu, 1 gelu, 2 silu_limit, 3 swiglu_clamp (f32 [E, N] biases)."""
        torch, lib = self.torch, self.lib
        (T, K), (E, N) = x.shape, gate.shape[:2]
        R = idx.shape[1]
        cid = lib.kq_codec_id(codec.encode())
        out = torch.empty((T, R, N), dtype=x.dtype, device=self.dev)
        nws = lib.kq_moe_workspace_size(T, R, E, N, K, 1, cid, KQ_BF16)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=self.dev)
        args = (x.data_ptr(), gate.data_ptr(), up.data_ptr(), idx.data_ptr(),
                gate_bias.data_ptr() if gate_bias is not None else None,
                up_bias.data_ptr() if up_bias is not None else None, out.data_ptr(), T, R, E, N, K,
                act, float(limit), float(alpha), cid, KQ_BF16, ws.data_ptr(), nws)
        keep = (x, gate, up, idx, out, ws, gate_bias, up_bias)

        def call(stream=None, _keep=keep):
            rc = lib.kq_moe_glu_gather(*args, stream or self.stream)
            if rc:
                self._check(rc)
        return call, out

    def gather_qmv(self, h, w, codec, idx, bias=None):
        torch, lib = self.torch, self.lib
        (T, R, K), (E, N) = h.shape, w.shape[:2]
        cid = lib.kq_codec_id(codec.encode())
        out = torch.empty((T, R, N), dtype=h.dtype, device=self.dev)
        nws = lib.kq_moe_workspace_size(T, R, E, N, K, 0, cid, KQ_BF16)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=self.dev)
        args = (h.data_ptr(), w.data_ptr(), idx.data_ptr(), bias.data_ptr() if bias is not None else None,
                out.data_ptr(), T, R, E, N, K, cid, KQ_BF16, ws.data_ptr(), nws)
        keep = (h, w, idx, out, ws, bias)

        def call(stream=None, _keep=keep):
            rc = lib.kq_gather_qmv(*args, stream or self.stream)
            if rc:
                self._check(rc)
        return call


def cold_copies(torch, base, wbytes):
    ncopies = max(2, (2 * LLC_BYTES + wbytes - 1) // wbytes + 1)
    return [base] + [base.clone() for _ in range(ncopies - 1)]


def read_ceiling(torch, dev, sizes):
    """What this box's memory system delivers to stock kernels on buffers of the GEMV's sizes, cold (rotating
    over copies that together exceed twice the last-level cache) and timed like the GEMV (HIP-graph replays):
    a read-only reduction (torch.sum over a float32 view: bytes read), the stock bf16 GEMV of the BLAS library on the
    same bytes taken as a [rows, 4096] bf16 matrix (bytes read), and the runtime's device-to-device copy (bytes read
    + bytes written).  Stated next to the 8 TB/s peak so that a GEMV rate can be compared with what plain readers
    reach on the same part."""
    rows_out = []
    K = 4096
    for label, nbytes in sizes:
        n32 = nbytes // 4
        ncopies = max(2, (2 * LLC_BYTES + nbytes - 1) // nbytes + 1)
        srcs = [torch.randint(-2 ** 31, 2 ** 31 - 1, (n32,), dtype=torch.int32, device=dev) for _ in range(ncopies)]
        acc = torch.empty((), dtype=torch.float32, device=dev)
        dsts = [torch.empty_like(srcs[0]) for _ in range(ncopies)]
        rows = n32 * 2 // K
        xv = torch.randn(K, device=dev).to(torch.bfloat16)
        yv = torch.empty(rows, dtype=torch.bfloat16, device=dev)

        def summer(v):
            return lambda stream=None: torch.sum(v.view(torch.float32), dim=(0,), out=acc)

        def gemv(v):
            m = v.view(torch.bfloat16)[:rows * K].view(rows, K)
            return lambda stream=None: torch.mv(m, xv, out=yv)

        def copier(v, d):
            return lambda stream=None: d.copy_(v)

        ts, _ = time_calls(torch, [summer(v) for v in srcs], 200, 20)
        tg, _ = time_calls(torch, [gemv(v) for v in srcs], 200, 20)
        tc, _ = time_calls(torch, [copier(v, d) for v, d in zip(srcs, dsts)], 200, 20)
        rows_out.append({"buffer": label, "bytes": n32 * 4,
                         "sum_f32_us": round(ts * 1e3, 2), "sum_f32_read_gbs": round(n32 * 4 / (ts * 1e-3) / 1e9, 1),
                         "stock_bf16_gemv_us": round(tg * 1e3, 2),
                         "stock_bf16_gemv_read_gbs": round(rows * K * 2 / (tg * 1e-3) / 1e9, 1),
                         "copy_us": round(tc * 1e3, 2),
                         "copy_read_plus_write_gbs": round(2 * n32 * 4 / (tc * 1e-3) / 1e9, 1)})
        del srcs, dsts
    return rows_out


def cpu_baseline(wire_np, codec, K, M, budget_s=12.0):
    """The CPU oracle (a port of the reference's threaded scalar eval_cpu path) on the same GEMV."""
    import numpy as np
    import oracle_lib as O
    x = O.f32_to_bits(np.random.default_rng(2).standard_normal((M, K)).astype(np.float32), "bfloat16")
    O.qmm(x, wire_np, codec, True, "bfloat16")
    times = []
    t_end = time.perf_counter() + budget_s
    while (time.perf_counter() < t_end or len(times) < 3) and len(times) < 200:
        t0 = time.perf_counter()
        O.qmm(x, wire_np, codec, True, "bfloat16")
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    N = wire_np.shape[0]
    return {"value": round(wire_np.size / med / 1e9, 3), "unit": "GB/s", "cores": int(O.lib.kq_oracle_threads()),
            "kind": "port",
            "sample": f"{codec} GEMV M={M} {K}->{N}, full matrix, median of {len(times)} runs "
                      f"({med * 1e3:.2f} ms each), bf16 activations"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20, help="timed steps; a step is one batch of >= 100 launches")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-sweep", action="store_true", help="skip the sweep, prefill, MoE and low-bit sections")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--gemm-tile", type=int, default=0,
                    help="prefill section: force a tile shape of the prefill GEMM (kq_set_gemm_tile_rows)")
    ap.add_argument("--only", default=None, metavar="SECTIONS",
                    help="comma-separated extra sections to run (sweep, prefill, moe, moe_mxfp4, moe_decode_lowbit, "
                         "lowbit, large_gemv, dequantize, mid_m, no_transpose); default all")
    ap.add_argument("--probe", action="store_true",
                    help="counter probe for `rocprofv3 --pmc`: one device copy of the headline matrix (known bytes) "
                         "followed by 20 cold launches of the headline GEMV, nothing else")
    ap.add_argument("--probe-codec", default=None, metavar="CODEC",
                    help="counter probe for `rocprofv3 --pmc`: 20 launches of the M = 1 GEMV 8192 -> 8192 in CODEC "
                         "(random structurally valid wire; --gemm-tile applies), nothing else")
    ap.add_argument("--probe-prefill", default=None, metavar="CODEC",
                    help="counter probe for `rocprofv3 --pmc`: 5 launches of the prefill GEMM [2048, 8192] x "
                         "[28672, 8192]^T in CODEC (random structurally valid wire), nothing else")
    ap.add_argument("--probe-n", type=int, default=28672, metavar="N",
                    help="weight rows of the --probe-prefill matrix (24576 = whole rounds of 256 x 256 tiles on 256 CUs)")
    ap.add_argument("--probe-moe", type=int, default=None, metavar="TOKENS",
                    help="counter probe for `rocprofv3 --pmc`: 10 launches each of the q4_k GLU op and the q6_k down "
                         "op of the 128-expert top-8 MoE at TOKENS tokens, nothing else")
    ap.add_argument("--probe-moe-mxfp4", type=int, default=None, metavar="TOKENS",
                    help="counter probe for `rocprofv3 --pmc`: 10 launches each of the biased swiglu_clamp GLU op and "
                         "the biased down op of the 32-expert top-4 mxfp4 MoE (2880 x 2880) at TOKENS tokens, nothing else")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); nothing here uses a second GPU.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    import kq

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    abi = Abi(kq, torch, dev)
    gx = torch.Generator(device=dev)
    gx.manual_seed(100)

    def randx(shape, scale=1.0):
        return (torch.randn(shape, device=dev, dtype=torch.float32, generator=gx) * scale).to(torch.bfloat16)

    if args.probe_codec:
        c, n, k = args.probe_codec, 8192, 8192
        w = synth_wire_torch(c, n, k, 7, dev)
        call = abi.qmm(randx((1, k)), w, c, n, k)
        for i in range(20):
            call()
        torch.cuda.synchronize()
        print(json.dumps({"probe": "20 GEMV launches", "codec": c, "N": n, "K": k, "M": 1,
                          "weight_bytes": n * kq.bytes_per_row(c, k)}))
        return

    if args.probe_moe:
        E, H, I, TOPK, T = 128, 2048, 768, 8, args.probe_moe
        gate = synth_wire_torch("q4_k", E * I, H, 11, dev).reshape(E, I, -1)
        up = synth_wire_torch("q4_k", E * I, H, 12, dev).reshape(E, I, -1)
        down = synth_wire_torch("q6_k", E * H, I, 13, dev).reshape(E, H, -1)
        xt = randx((T, H), 0.5)
        touched = []
        for r in range(10):
            idx = torch.randn((T, E), device=dev, generator=gx).topk(TOPK, dim=-1).indices.to(torch.int32).contiguous()
            call, h = abi.moe_glu(xt, gate, up, "q4_k", idx)
            call()
            abi.gather_qmv(h, down, "q6_k", idx)()
            touched.append(int(idx.unique().numel()))
        torch.cuda.synchronize()
        print(json.dumps({"probe": "10 GLU + 10 down launches", "tokens": T, "experts_touched_mean": sum(touched) / 10,
                          "glu_bytes_per_expert": 2 * I * kq.bytes_per_row("q4_k", H),
                          "down_bytes_per_expert": H * kq.bytes_per_row("q6_k", I)}))
        return

    if args.probe_moe_mxfp4:
        E, H, TOPK, T = 32, 2880, 4, args.probe_moe_mxfp4
        gate = synth_wire_torch("mxfp4", E * H, H, 21, dev).reshape(E, H, -1)
        up = synth_wire_torch("mxfp4", E * H, H, 22, dev).reshape(E, H, -1)
        down = synth_wire_torch("mxfp4", E * H, H, 23, dev).reshape(E, H, -1)
        gb, ub, db = (torch.randn((E, H), device=dev, generator=gx) * 0.01 for _ in range(3))
        xt = randx((T, H), 0.5)
        touched = []
        for r in range(10):
            idx = torch.randn((T, E), device=dev, generator=gx).topk(TOPK, dim=-1).indices.to(torch.int32).contiguous()
            call, h = abi.moe_glu(xt, gate, up, "mxfp4", idx, act=3, limit=7.0, alpha=1.702, gate_bias=gb, up_bias=ub)
            call()
            abi.gather_qmv(h, down, "mxfp4", idx, bias=db)()
            touched.append(int(idx.unique().numel()))
        torch.cuda.synchronize()
        print(json.dumps({"probe": "10 GLU + 10 down launches", "tokens": T, "experts_touched_mean": sum(touched) / 10,
                          "glu_bytes_per_expert": 2 * H * kq.bytes_per_row("mxfp4", H),
                          "down_bytes_per_expert": H * kq.bytes_per_row("mxfp4", H)}))
        return

    if args.probe_prefill:
        c, m, n, k = args.probe_prefill, 2048, args.probe_n, 8192
        abi.lib.kq_set_gemm_tile_rows(args.gemm_tile)
        w = synth_wire_torch(c, n, k, 7, dev)
        call = abi.qmm(randx((m, k)), w, c, n, k)
        for i in range(5):
            call()
        torch.cuda.synchronize()
        print(json.dumps({"probe": "5 prefill GEMM launches", "codec": c, "M": m, "N": n, "K": k,
                          "flops": 2 * m * n * k}))
        return

    # ---------------- headline: q4_k gate/up GEMV, M = 1, cold
    codec, N, K, M = "q4_k", 14336, 4096, 1
    wbytes = N * kq.bytes_per_row(codec, K)
    base = quantized_weights(kq, torch, codec, N, K, seed=2, device=dev)
    copies = cold_copies(torch, base, wbytes)
    x = randx((M, K))
    calls = [abi.qmm(x, w, codec, N, K) for w in copies]
    if args.probe:
        dst = torch.empty_like(base)
        torch.cuda.synchronize()
        dst.copy_(copies[1])  # reference dispatch: reads and writes `wbytes` bytes
        torch.cuda.synchronize()
        for i in range(20):
            calls[(i + 2) % len(calls)]()
        torch.cuda.synchronize()
        print(json.dumps({"probe": "copy then 20 cold GEMV launches", "copy_bytes_each_way": wbytes,
                          "gemv_weight_bytes": wbytes}))
        return
    # a step = one rotation over the copies, repeated until it holds at least 100 launches, replayed as one HIP
    # graph: back-to-back launches on one stream with no host work between them
    lps = len(calls) * max(1, -(-100 // len(calls)))
    g = capture_batch(torch, calls, lps)
    if g is not None:
        step_ms, wall_step_ms = time_graph(torch, g, lps, args.steps, args.warmup)
    else:
        ms1, wall1 = _time_direct(torch, [(lambda c=c: c(None)) for c in calls], lps * args.steps, lps * args.warmup)
        step_ms, wall_step_ms = ms1 * lps, wall1 * lps
    ms, wall_ms = step_ms / lps, wall_step_ms / lps
    gbs = wbytes / (ms * 1e-3) / 1e9
    hot_ms, _ = time_calls(torch, calls[:1], 2000, 200)
    # the same launches with no order between them (every call has its own weights, output and workspace): what the
    # kernel streams when the gap between dependent launches, its ramp and its tail overlap other launches.  Not the
    # headline: a decode step's GEMVs mostly depend on each other.
    independent = None
    for lanes in (2, 4):
        gi = capture_batch(torch, calls, lps, lanes=lanes)
        if gi is None:
            break
        ims, _ = time_graph(torch, gi, lps, args.steps, args.warmup, settle_ms=10.0)
        cur = {"lanes": lanes, "us_per_launch": round(ims / lps * 1e3, 3),
               "gbs": round(wbytes / (ims / lps * 1e-3) / 1e9, 1)}
        if independent is None or cur["gbs"] > independent["gbs"]:
            independent = cur
        del gi

    out = {
        "metric": "q4_k GEMV weight-GB/s at M=1 (cold)", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_ms, 6), "launches_per_step": lps,
        "us_per_launch": round(ms * 1e3, 3), "launch_mode": "hip graph replay" if g is not None else "direct",
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic: seeded N(0,0.02) weights quantized by kq.quantize, N(0,1) bf16 activations",
        "config": {"workload": "decode GEMV, Llama-3-8B gate/up projection 4096->14336, q4_k, M=1, bf16 x, "
                               f"cold over {len(copies)} weight copies ({len(copies) * wbytes >> 20} MiB)",
                   "codec": codec, "M": M, "N": N, "K": K},
        "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "hot_gbs": round(wbytes / (hot_ms * 1e-3) / 1e9, 1),
        "wall_ms_per_step": round(wall_step_ms, 6),
        "independent_launches": independent,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": HEADLINE_TRAFFIC_BYTES},
    }
    base_np = base.cpu().numpy() if not args.no_cpu else None
    del copies, calls
    # the box's attainable bandwidth with stock kernels, on the sizes of the headline matrix and of lm_head
    out["read_ceiling"] = read_ceiling(torch, dev, [("gate/up q4_k wire, 33 MB", wbytes),
                                                    ("lm_head q6_k wire, 431 MB", 128256 * kq.bytes_per_row("q6_k", 4096))])

    only = set(args.only.split(",")) if args.only else None

    def want(sec):
        return only is None or sec in only

    if not args.no_sweep:
        steps, warm = 400, 40  # launches per shape
        # ---------------- decode sweep (q4_k_m recipe of Llama-3-8B)
        if want("sweep"):
            sweep = []
            shapes = [("q_proj", "q4_k", 4096, 4096), ("gate/up", "q4_k", 14336, 4096),
                      ("down", "q6_k", 4096, 14336), ("lm_head", "q6_k", 128256, 4096)]
            for name, c, n, k in shapes:
                wb = n * kq.bytes_per_row(c, k)
                wq = base if name == "gate/up" else quantized_weights(kq, torch, c, n, k, 3, dev)
                cps = cold_copies(torch, wq, wb)
                for m in (1, 2, 4, 8):
                    xm = randx((m, k))
                    t, _ = time_calls(torch, [abi.qmm(xm, w, c, n, k) for w in cps], steps, warm)
                    sweep.append({"proj": name, "codec": c, "N": n, "K": k, "M": m, "us": round(t * 1e3, 2),
                                  "cold_gbs": round(wb / (t * 1e-3) / 1e9, 1),
                                  "pct_hbm_peak": round(100 * wb / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)})
                del cps, wq
            out["sweep"] = sweep

        # ---------------- prefill GEMM
        if want("prefill"):
            prefill = []
            abi.lib.kq_set_gemm_tile_rows(args.gemm_tile)
            for c in ("q4_k", "q5_k", "q6_k", "q2_k", "q3_k", "iq4_xs", "q8_0", "q4_0", "mxfp4", "nvfp4", "iq3_s", "iq2_xxs"):
                n, k = 28672, 8192
                # q4_k / q5_k / q6_k / q8_0 / q4_0 / mxfp4 / nvfp4 / iq3_s / iq2_xxs: 256-row tiles for the whole rounds,
                # 128-row tiles for the rest; q2_k / q3_k / iq4_xs: 128 x 256 tiles
                # the fp4 codecs have no encoder (the reference has none either): structurally valid random wire;
                # the codebook encoders search for ~1 us per weight on the host: 512 unique rows, tiled
                if c in ("mxfp4", "nvfp4"):
                    wq = synth_wire_torch(c, n, k, 5, dev)
                else:
                    wq = quantized_weights(kq, torch, c, n, k, 5, dev, unique_rows=512 if c in ("iq3_s", "iq2_xxs") else None)
                for m in (512, 2048):
                    # the device idles while the host encodes the weights: about 30 ms of launches bring it back
                    # to its steady clock before the timed ones (the first shape timed read 6 - 15 % low without)
                    t, _ = time_calls(torch, [abi.qmm(randx((m, k)), wq, c, n, k)], 20, 60 if m <= 512 else 20)
                    tf = 2.0 * m * n * k / (t * 1e-3) / 1e12
                    prefill.append({"codec": c, "M": m, "N": n, "K": k, "ms": round(t, 4), "tflops": round(tf, 1),
                                    "pct_mfma_f16_peak": round(100 * tf / MFMA_F16_PEAK_TFLOPS, 2)})
                del wq
            abi.lib.kq_set_gemm_tile_rows(0)
            out["prefill"] = prefill

        # ---------------- MoE: 128 experts, top-8, hidden 2048, intermediate 768 (weights encoded by kq.quantize)
        if want("moe"):
            E, H, I, TOPK = 128, 2048, 768, 8
            gate = quantized_weights(kq, torch, "q4_k", E * I, H, 11, dev).reshape(E, I, -1)
            up = quantized_weights(kq, torch, "q4_k", E * I, H, 12, dev).reshape(E, I, -1)
            down = quantized_weights(kq, torch, "q6_k", E * H, I, 13, dev).reshape(E, H, -1)
            gu_bytes = 2 * I * kq.bytes_per_row("q4_k", H)
            dn_bytes = H * kq.bytes_per_row("q6_k", I)
            moe = []
            for T in (1, 256):
                xt = randx((T, H), 0.5)
                # 16 different routings, rotated per step, so that a step's experts are not the previous step's
                glu_calls, dn_calls, touched = [], [], []
                for r in range(16):
                    logits = torch.randn((T, E), device=dev, generator=gx)
                    idx = logits.topk(TOPK, dim=-1).indices.to(torch.int32).contiguous()
                    call, h = abi.moe_glu(xt, gate, up, "q4_k", idx)
                    glu_calls.append(call)
                    dn_calls.append(abi.gather_qmv(h, down, "q6_k", idx))
                    touched.append(int(idx.unique().numel()))
                ne = sum(touched) / len(touched)
                tg, _ = time_calls(torch, glu_calls, steps, warm)
                td, _ = time_calls(torch, dn_calls, steps, warm)
                moe.append({"tokens": T, "experts_touched": round(ne, 1), "glu_us": round(tg * 1e3, 2),
                            "down_us": round(td * 1e3, 2),
                            "glu_gbs": round(ne * gu_bytes / (tg * 1e-3) / 1e9, 1),
                            "down_gbs": round(ne * dn_bytes / (td * 1e-3) / 1e9, 1),
                            "pct_hbm_peak": round(100 * ne * (gu_bytes + dn_bytes) / ((tg + td) * 1e-3) / 1e9
                                                  / HBM_PEAK_GBS, 2)})
            del gate, up, down
            out["moe"] = moe

        # ---------------- mxfp4 MoE: 32 experts of 2880 -> 2880, top-4, 64 tokens, f32 biases, swiglu_clamp
        if want("moe_mxfp4"):
            E, H, TOPK, T = 32, 2880, 4, 64
            gate = synth_wire_torch("mxfp4", E * H, H, 21, dev).reshape(E, H, -1)
            up = synth_wire_torch("mxfp4", E * H, H, 22, dev).reshape(E, H, -1)
            down = synth_wire_torch("mxfp4", E * H, H, 23, dev).reshape(E, H, -1)
            gb = torch.randn((E, H), device=dev, generator=gx) * 0.01
            ub = torch.randn((E, H), device=dev, generator=gx) * 0.01
            db = torch.randn((E, H), device=dev, generator=gx) * 0.01
            xt = randx((T, H), 0.5)
            idx = torch.randn((T, E), device=dev, generator=gx).topk(TOPK, dim=-1).indices.to(torch.int32).contiguous()
            glu_call, h = abi.moe_glu(xt, gate, up, "mxfp4", idx, act=3, limit=7.0, alpha=1.702, gate_bias=gb, up_bias=ub)
            dn_call = abi.gather_qmv(h, down, "mxfp4", idx, bias=db)
            tg, _ = time_calls(torch, [glu_call], 100, 20)
            td, _ = time_calls(torch, [dn_call], 100, 20)
            mbytes = H * kq.bytes_per_row("mxfp4", H)
            ne = int(idx.unique().numel())
            out["moe_mxfp4"] = {"tokens": T, "experts_touched": ne, "glu_us": round(tg * 1e3, 1),
                                "down_us": round(td * 1e3, 1),
                                "glu_gbs": round(ne * 2 * mbytes / (tg * 1e-3) / 1e9, 1),
                                "down_gbs": round(ne * mbytes / (td * 1e-3) / 1e9, 1),
                                "note": "block-scaled fp4 MFMA kernel, wire blocks undecoded (f32 biases, swiglu_clamp)"}
            del gate, up, down

        # ---------------- MoE decode (1 token, 8 of 128 experts of 2048 <-> 768) in the low-bit / fp4 codecs
        if want("moe_decode_lowbit"):
            E, H, I, TOPK = 128, 2048, 768, 8
            dec = []
            for c in ("iq4_xs", "iq3_s", "iq2_xxs", "mxfp4", "nvfp4", "q8_0"):
                gate = synth_wire_torch(c, E * I, H, 31, dev).reshape(E, I, -1)
                up = synth_wire_torch(c, E * I, H, 32, dev).reshape(E, I, -1)
                down = synth_wire_torch(c, E * H, I, 33, dev).reshape(E, H, -1)
                calls_g, calls_d = [], []
                for r in range(16):  # 16 routings rotated per step
                    ix = torch.randperm(E, device=dev, generator=gx)[:TOPK].reshape(1, TOPK).to(torch.int32)
                    calls_g.append(abi.moe_glu(randx((1, H), 0.5), gate, up, c, ix)[0])
                    calls_d.append(abi.gather_qmv(randx((1, TOPK, I), 0.5), down, c, ix))
                tg, _ = time_calls(torch, calls_g, 200, 20)
                td, _ = time_calls(torch, calls_d, 200, 20)
                bg, bd = TOPK * 2 * I * kq.bytes_per_row(c, H), TOPK * H * kq.bytes_per_row(c, I)
                dec.append({"codec": c, "tokens": 1, "experts": TOPK, "glu_us": round(tg * 1e3, 2), "down_us": round(td * 1e3, 2),
                            "glu_gbs": round(bg / (tg * 1e-3) / 1e9, 1), "down_gbs": round(bd / (td * 1e-3) / 1e9, 1)})
                del gate, up, down, calls_g, calls_d
            out["moe_decode_lowbit"] = dec

        # ---------------- low-bit codecs (and q8_0, 4-bit block codecs), M = 1, 8192 -> 8192 (minted by kq.quantize)
        if want("lowbit"):
            lowbit = []
            for c in ("q2_k", "q3_k", "iq4_xs", "iq3_s", "iq2_xxs", "q8_0", "q4_0", "iq4_nl", "mxfp4", "nvfp4"):
                n = k = 8192
                wb = n * kq.bytes_per_row(c, k)
                if c in ("mxfp4", "nvfp4"):  # no encoder in the reference: random structurally valid wire
                    wq = synth_wire_torch(c, n, k, 7, dev).reshape(n, -1)
                else:
                    wq = quantized_weights(kq, torch, c, n, k, 7, dev,
                                           unique_rows=None if c in ("q2_k", "q3_k", "iq4_xs", "q8_0", "q4_0") else 512)
                cps = cold_copies(torch, wq, wb)
                t, _ = time_calls(torch, [abi.qmm(x.new_ones((1, k)), w, c, n, k) for w in cps], steps, warm)
                lowbit.append({"codec": c, "N": n, "K": k, "M": 1, "us": round(t * 1e3, 2),
                               "cold_gbs": round(wb / (t * 1e-3) / 1e9, 1),
                               "pct_hbm_peak": round(100 * wb / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)})
                del cps, wq
            out["lowbit"] = lowbit

        # ---------------- long matrices (128256 x 4096, the lm_head shape), M = 1: the launch overheads of the 20 - 70 MB
        # shapes above amortised, to set beside `read_ceiling` (random structurally valid wire)
        if want("large_gemv"):
            large = []
            n, k = 128256, 4096
            for c in ("q8_0", "q4_k", "q5_k", "iq4_xs", "q6_k", "q2_k", "q3_k"):
                wb = n * kq.bytes_per_row(c, k)
                ncopies = max(2, (2 * LLC_BYTES + wb - 1) // wb + 1)
                cps = [synth_wire_torch(c, n, k, 31 + i, dev) for i in range(ncopies)]
                t, _ = time_calls(torch, [abi.qmm(x.new_ones((1, k)), w, c, n, k) for w in cps], 60, 10)
                large.append({"codec": c, "N": n, "K": k, "M": 1, "us": round(t * 1e3, 2),
                              "cold_gbs": round(wb / (t * 1e-3) / 1e9, 1),
                              "pct_hbm_peak": round(100 * wb / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)})
                del cps
            out["large_gemv"] = large

        # ---------------- dequantize to f16 (random structurally valid wire): bytes = wire in + 2 N K out
        if want("dequantize"):
            deq = []
            for c, n, k in (("q4_k", 4096, 4096), ("q4_k", 28672, 8192), ("q6_k", 28672, 8192), ("iq3_s", 28672, 8192),
                            ("q8_0", 28672, 8192)):
                wb = n * kq.bytes_per_row(c, k)
                total = wb + 2 * n * k
                wq = synth_wire_torch(c, n, k, 9, dev)
                # rotate over inputs AND outputs so that neither side is served by the last-level cache
                cps = cold_copies(torch, wq, total)
                outs = [torch.empty((n, k), dtype=torch.float16, device=dev) for _ in cps]
                t, _ = time_calls(torch, [abi.dequantize(w, c, n, k, o) for w, o in zip(cps, outs)], 200, 20)
                deq.append({"codec": c, "N": n, "K": k, "us": round(t * 1e3, 2), "cold_gbs": round(total / (t * 1e-3) / 1e9, 1),
                            "pct_hbm_peak": round(100 * total / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)})
                del cps, outs, wq
            out["dequantize"] = deq

        # ---------------- between decode and prefill: 16 ... 64 rows on matrices with few tiles (K cut over the grid)
        if want("mid_m"):
            mid = []
            for c, n, k, m in (("q4_k", 4096, 4096, 16), ("q4_k", 4096, 4096, 64), ("q4_k", 14336, 4096, 32),
                               ("q6_k", 4096, 4096, 16), ("q8_0", 4096, 4096, 64), ("q2_k", 4096, 4096, 64)):
                wb = n * kq.bytes_per_row(c, k)
                wq = synth_wire_torch(c, n, k, 11, dev)
                cps = cold_copies(torch, wq, wb)
                xm = randx((m, k))
                t, _ = time_calls(torch, [abi.qmm(xm, w, c, n, k) for w in cps], 200, 20)
                mid.append({"codec": c, "N": n, "K": k, "M": m, "us": round(t * 1e3, 2),
                            "tflops": round(2.0 * m * n * k / (t * 1e-3) / 1e12, 1),
                            "cold_gbs": round(wb / (t * 1e-3) / 1e9, 1)})
                del cps, wq
            out["mid_m"] = mid

        # ---------------- transpose = 0 (reduction over wire rows): MLA-shaped gathered entries and dense calls
        if want("no_transpose"):
            nt = []
            for c in ("q4_k", "q8_0"):
                E, k, n = 128, 128, 512
                wq = synth_wire_torch(c, E * k, n, 13, dev)
                rhs = torch.arange(E, dtype=torch.int32, device=dev)
                for m in (1, 64):
                    t, _ = time_calls(torch, [abi.gather_nt(randx((E, m, k)), wq, c, rhs, E, k, n)], 200, 20)
                    nt.append({"codec": c, "entries": E, "M": m, "K": k, "N": n, "us": round(t * 1e3, 2)})
                del wq
            for m in (1, 32, 512, 2048):
                k = n = 4096
                wq = synth_wire_torch("q4_k", k, n, 14, dev)
                t, _ = time_calls(torch, [abi.qmm_nt(randx((m, k)), wq, "q4_k", k, n)], 200, 20)
                nt.append({"codec": "q4_k", "entries": 1, "M": m, "K": k, "N": n, "us": round(t * 1e3, 2),
                           "tflops": round(2.0 * m * n * k / (t * 1e-3) / 1e12, 1)})
                del wq
            out["no_transpose"] = nt

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(base_np, codec, K, M)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
