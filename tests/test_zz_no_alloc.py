"""The no-allocation entry point kq_qmm_noalloc (workspace = a buffer inside the library's code object) gives the
same bits as kq_qmm with a caller-owned workspace, also on a second, smaller call that finds the first call's
contents in the buffer; shapes beyond the built-in buffer are refused."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu

KQ_F16, KQ_BF16 = 1, 2
KQ_ERR_WORKSPACE = -4


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _both(kq, lib, codec, M, N, K, dtype, seed):
    cid = lib.kq_codec_id(codec.encode())
    dt = KQ_F16 if dtype == "float16" else KQ_BF16
    wpb, bpb = O.geometry(codec)
    wire = O.synth_wire(codec, N * K // wpb, seed=seed).reshape(N, K // wpb * bpb)
    w = wire_to_dev(wire)
    xb, xt = make_x((M, K), dtype, seed=seed + 1)
    stream = torch.cuda.current_stream().cuda_stream
    nws = lib.kq_qmm_workspace_size(M, N, K, 1, cid, dt)
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=w.device)
    y_ref = torch.empty((M, N), dtype=xt.dtype, device=w.device)
    y_new = torch.full((M, N), 7.0, dtype=xt.dtype, device=w.device)
    assert lib.kq_qmm(xt.data_ptr(), w.data_ptr(), y_ref.data_ptr(), M, N, K, 1, cid, dt, ws.data_ptr(), nws, stream) == 0
    rc = lib.kq_qmm_noalloc(xt.data_ptr(), w.data_ptr(), y_new.data_ptr(), M, N, K, cid, dt, stream)
    assert rc == 0, lib.kq_last_error()
    torch.cuda.synchronize()
    assert np.array_equal(dev_to_bits(y_new), dev_to_bits(y_ref)), (codec, M, N, K)
    assert rel_l2(dev_to_bits(y_new), O.qmm(xb, wire, codec, True, dtype), dtype) <= 1e-3
    return nws


def test_noalloc_matches_workspace_entry_twice(kq):
    lib = kq._load()
    # split-K GEMV (partial sums in the buffer), then a smaller one of another codec on the used buffer
    n1 = _both(kq, lib, "q4_k", 1, 4096, 4096, "bfloat16", 50)
    n2 = _both(kq, lib, "q6_k", 3, 1024, 2048, "float16", 52)
    assert n1 > 0 and n2 > 0 and n2 < n1
    # prefill GEMM (converted activations and block sums in the buffer), then a smaller one
    n3 = _both(kq, lib, "q4_k", 96, 512, 2048, "bfloat16", 54)
    n4 = _both(kq, lib, "q5_k", 20, 256, 1024, "bfloat16", 56)
    assert n3 > n4 > 0


def test_noalloc_refuses_oversized_workspace(kq):
    lib = kq._load()
    cid = lib.kq_codec_id(b"q4_k")
    M, N, K = 2048, 1024, 8192
    assert lib.kq_qmm_workspace_size(M, N, K, 1, cid, KQ_BF16) > (4 << 20)
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda:0")
    w = torch.zeros((N, K // 256 * 144), dtype=torch.uint8, device="cuda:0")
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda:0")
    rc = lib.kq_qmm_noalloc(x.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K, cid, KQ_BF16,
                            torch.cuda.current_stream().cuda_stream)
    assert rc == KQ_ERR_WORKSPACE
    assert b"workspace" in lib.kq_last_error()


def test_noalloc_leaves_device_memory_alone(kq):
    """The property the entry point exists for: the free device memory reported by the runtime is the same before
    and after a first-of-its-shape call and a repeated call (torch's caching allocator is not involved: every buffer
    is made beforehand, the library's own buffer lives in its code object)."""
    lib = kq._load()
    cid = lib.kq_codec_id(b"q5_k")
    M, N, K = 2, 2048, 4096  # a shape no other test of this file has run: first-use set-up of its kernel included
    wire = O.synth_wire("q5_k", N * K // 256, seed=61).reshape(N, K // 256 * 176)
    w = wire_to_dev(wire)
    xb, xt = make_x((M, K), "bfloat16", seed=62)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device=w.device)
    stream = torch.cuda.current_stream().cuda_stream
    # load the library's code object and take the buffer's address with another shape first
    _both(kq, lib, "q4_k", 1, 512, 1024, "bfloat16", 63)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert lib.kq_qmm_noalloc(xt.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K, cid, KQ_BF16, stream) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert rel_l2(dev_to_bits(y), O.qmm(xb, wire, "q5_k", True, "bfloat16"), "bfloat16") <= 1e-3


def test_noalloc_replayed_from_a_hip_graph(kq):
    """The advertised use: kq_qmm_noalloc captured into a HIP graph after one eager call of the same shape (the
    first call on a device looks the buffer up and sets kernel attributes, which is set-up work and stays outside
    a capture), replayed several times with the built-in buffer dirtied by another shape between the replays."""
    lib = kq._load()
    cid = lib.kq_codec_id(b"q4_k")
    M, N, K = 1, 4096, 4096  # split-K plan: partial sums in the built-in buffer
    wire = O.synth_wire("q4_k", N * K // 256, seed=71).reshape(N, K // 256 * 144)
    w = wire_to_dev(wire)
    xb, xt = make_x((M, K), "bfloat16", seed=72)
    y = torch.zeros((M, N), dtype=torch.bfloat16, device=w.device)
    cur = torch.cuda.current_stream().cuda_stream
    assert lib.kq_qmm_noalloc(xt.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K, cid, KQ_BF16, cur) == 0
    torch.cuda.synchronize()
    eager = dev_to_bits(y).copy()
    assert rel_l2(eager, O.qmm(xb, wire, "q4_k", True, "bfloat16"), "bfloat16") <= 1e-3
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        st = torch.cuda.current_stream().cuda_stream
        assert lib.kq_qmm_noalloc(xt.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K, cid, KQ_BF16, st) == 0
    for rep in range(3):
        _both(kq, lib, "q6_k", 3, 1024, 2048, "float16", 80 + rep)  # another shape writes over the buffer
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dev_to_bits(y), eager), rep
