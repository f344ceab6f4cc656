"""GPU parity: kq.expert_tile_map, kq.gather_qmm_seg and the sorted prefill arm of KQuantSwitchLinear (HIP) vs the
host-built tile map and the CPU oracle; the cases of the reference's tests/test_switch_gemm.py."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3
E, N, K = 8, 128, 512


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _stack(codec, n_experts, n, k, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, n_experts * n * (k // wpb), seed).reshape(n_experts, n, k // wpb * bpb)


def _indices(counts):
    return np.repeat(np.arange(len(counts), dtype=np.int64), counts)


def _host_tiles(counts):
    """(expert, first row, rows <= 64) tiles of every expert's run, in row order (mlx_kquant/nn.py:33-47)."""
    tiles, row = [], 0
    for e, c in enumerate(counts):
        tiles += [(e, row + off, min(64, c - off)) for off in range(0, int(c), 64)]
        row += int(c)
    return np.asarray(tiles, dtype=np.int64).reshape(-1, 3)


def _check_cover(tiles, idx, n_experts):
    """What a valid map must satisfy whatever produced it: tiles of 1..64 rows, one expert each, that cover
    every in-range row exactly once, with at most one partial tile per expert."""
    seen = np.zeros(len(idx), dtype=np.int64)
    partial = {}
    for e, r, n in tiles:
        assert 1 <= n <= 64 and 0 <= e < n_experts and r + n <= len(idx)
        assert np.all(idx[r:r + n] == e)
        seen[r:r + n] += 1
        partial[e] = partial.get(e, 0) + (n < 64)
    assert np.array_equal(seen, (idx < n_experts).astype(np.int64))
    assert all(v <= 1 for v in partial.values())


@pytest.mark.parametrize("counts", [[1, 63, 64, 129, 200, 0, 0, 32], [512], [0, 0, 0, 5], [64] * 8, [65] * 8,
                                    [1, 7, 8, 9, 16, 17, 48, 96]],
                         ids=["ragged", "single", "tiny", "uniform64", "uniform65", "sub_frag"])
def test_expert_tile_map_matches_host(kq, counts):
    idx = _indices(counts)
    m, cnt = kq.expert_tile_map(torch.from_numpy(idx).to(torch.int32).cuda(), len(counts))
    want = _host_tiles(counts)
    assert tuple(m.shape) == (max(len(idx) // 64 + min(len(counts), len(idx)), 1), 3) and tuple(cnt.shape) == (1,)
    n = int(cnt.cpu()[0])
    assert n == len(want)
    got = m.cpu().numpy().astype(np.int64)[:n]
    assert np.array_equal(got, want)  # this build writes the tiles in row order
    _check_cover(got, idx, len(counts))


def test_expert_tile_map_large_and_out_of_range(kq):
    """Many rows per thread of the one-workgroup builder, runs that straddle thread chunks, and rows whose
    expert id is out of range (no tile)."""
    rng = np.random.default_rng(3)
    n_experts = 128
    idx = np.sort(rng.integers(0, n_experts + 2, 70001))
    m, cnt = kq.expert_tile_map(torch.from_numpy(idx).cuda(), n_experts)
    n = int(cnt.cpu()[0])
    got = m.cpu().numpy().astype(np.int64)[:n]
    counts = np.bincount(idx, minlength=n_experts + 2)[:n_experts]
    assert np.array_equal(got, _host_tiles(counts))
    _check_cover(got, idx, n_experts)


@pytest.mark.parametrize("codec", ["iq2_xxs", "q2_k", "q8_0", "q4_k", "q6_k", "mxfp4", "nvfp4"])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_gather_qmm_seg_matches_loop(kq, codec, dtype):
    """Ragged segments: absent experts and partial tiles of 1, 17, 63, 96, 129, 200 and 48 rows; host-built and
    device-built maps; the expected rows are each expert's plain quantized matmul over its run."""
    k = K if codec not in ("mxfp4", "nvfp4") else 320
    wire = _stack(codec, E, N, k, seed=5)
    counts = np.zeros(E, dtype=np.int64)
    counts[[0, 1, 2, 3, 4, 5, 7]] = [1, 17, 63, 96, 129, 200, 48]
    idx = _indices(counts)
    rows = len(idx)
    xb, xt = make_x((rows, k), dtype, seed=23)
    want = O.gather_qmv(xb.reshape(rows, 1, k), wire, codec, idx.reshape(rows, 1), None, dtype).reshape(rows, N)
    w_dev = wire_to_dev(wire)
    scales = torch.zeros(1, dtype=torch.uint8, device="cuda")
    host = _host_tiles(counts)
    maps = {"host": (torch.from_numpy(host).to(torch.int32).cuda(), torch.tensor([len(host)], dtype=torch.int32).cuda()),
            "device": kq.expert_tile_map(torch.from_numpy(idx).to(torch.int32).cuda(), E)}
    for label, (m, c) in maps.items():
        got = kq.gather_qmm_seg(xt, w_dev, scales, codec, m, c)
        assert tuple(got.shape) == (rows, N) and got.dtype == xt.dtype
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype, label)


def test_gather_qmm_seg_unaligned_n_and_few_rows(kq):
    """N that is no multiple of the kernels' slab, then a map of 9 rows (the per-row kernels take it)."""
    n_odd = 72
    wire = _stack("iq2_xxs", 4, n_odd, K, seed=31)
    scales = torch.zeros(1, dtype=torch.uint8, device="cuda")
    for counts in ([65, 0, 3, 64], [4, 0, 5, 0]):
        idx = _indices(counts)
        rows = len(idx)
        xb, xt = make_x((rows, K), "float16", seed=32)
        host = _host_tiles(counts)
        got = kq.gather_qmm_seg(xt, wire_to_dev(wire), scales, "iq2_xxs", torch.from_numpy(host).to(torch.int32).cuda(),
                                torch.tensor([len(host)], dtype=torch.int32).cuda())
        want = O.gather_qmv(xb.reshape(rows, 1, K), wire, "iq2_xxs", idx.reshape(rows, 1), None, "float16")
        assert tuple(got.shape) == (rows, n_odd)
        assert rel_l2(dev_to_bits(got), want.reshape(rows, n_odd), "float16") <= TOL


def test_gather_qmm_seg_counts_bound_the_map(kq):
    """Tiles past counts[0] are ignored: their rows keep what the output buffer held; the valid ones are exact."""
    counts = [40, 70, 30]
    idx = _indices(counts)
    rows = len(idx)
    wire = _stack("q4_k", 3, N, K, seed=41)
    xb, xt = make_x((rows, K), "bfloat16", seed=42)
    host = _host_tiles(counts)  # 4 tiles; only the first 2 (rows 0..103) are declared valid
    got = kq.gather_qmm_seg(xt, wire_to_dev(wire), torch.zeros(1, dtype=torch.uint8, device="cuda"), "q4_k",
                            torch.from_numpy(host).to(torch.int32).cuda(), torch.tensor([2], dtype=torch.int32).cuda())
    want = O.gather_qmv(xb.reshape(rows, 1, K), wire, "q4_k", idx.reshape(rows, 1), None, "bfloat16").reshape(rows, N)
    assert rel_l2(dev_to_bits(got)[:104], want[:104], "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["iq2_xxs", "q2_k", "mxfp4", "nvfp4", "q4_k"])
@pytest.mark.parametrize("rows,experts", [(1024, list(range(E))), (600, [3]), (777, [0, 2, 7])],
                         ids=["all_experts", "single_expert", "sparse_experts"])
def test_sorted_expert_gemm_matches_gather(kq, codec, rows, experts, monkeypatch):
    """The sorted arm of KQuantSwitchLinear against its gather_qmm arm (KQ_SWITCH_GEMM_MIN_ROWS=0) and the oracle."""
    from kq.nn import KQuantSwitchLinear

    k = K if codec not in ("mxfp4", "nvfp4") else 320
    wire = _stack(codec, E, N, k, seed=5)
    sw = KQuantSwitchLinear(E, N, k, False, codec, device="cuda")
    sw.load_wire(wire_to_dev(wire))
    rng = np.random.default_rng(rows)
    idx = np.sort(rng.choice(experts, size=rows)).astype(np.int64)
    xb, xt = make_x((rows, 1, k), "float16", seed=rows + 1)
    idx_dev = torch.from_numpy(idx).to(torch.int32).cuda()
    calls = []
    orig = sw._sorted_expert_gemm
    monkeypatch.setattr(sw, "_sorted_expert_gemm", lambda *a: calls.append(1) or orig(*a))
    monkeypatch.setenv("KQ_SWITCH_GEMM_MIN_ROWS", "512")
    got = sw(xt, idx_dev, sorted_indices=True)
    assert len(calls) == 1
    monkeypatch.setenv("KQ_SWITCH_GEMM_MIN_ROWS", "0")
    ref = sw(xt, idx_dev, sorted_indices=True)
    assert len(calls) == 1
    assert tuple(got.shape) == tuple(ref.shape) == (rows, 1, N) and got.dtype == ref.dtype
    want = O.gather_qmv(xb, wire, codec, idx.reshape(rows, 1), None, "float16")
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL
    assert rel_l2(dev_to_bits(ref), want, "float16") <= TOL


def test_threshold_and_shape_gating(kq, monkeypatch):
    from kq.nn import KQuantSwitchLinear

    sw = KQuantSwitchLinear(E, N, K, False, "iq2_xxs", device="cuda")
    sw.load_wire(wire_to_dev(_stack("iq2_xxs", E, N, K, seed=5)))
    calls = []
    orig = sw._sorted_expert_gemm
    monkeypatch.setattr(sw, "_sorted_expert_gemm", lambda *a: calls.append(1) or orig(*a))
    monkeypatch.setenv("KQ_SWITCH_GEMM_MIN_ROWS", "512")
    rng = np.random.default_rng(0)

    def call(rows, **kw):
        idx = torch.from_numpy(np.sort(rng.integers(0, E, rows))).to(torch.int32).cuda()
        _, xt = make_x((rows, 1, K), "float16", seed=rows)
        return sw(xt, idx, **kw)

    call(64, sorted_indices=True)       # below the threshold
    call(512, sorted_indices=False)     # not promised sorted
    assert not calls
    call(512, sorted_indices=True)
    assert len(calls) == 1
