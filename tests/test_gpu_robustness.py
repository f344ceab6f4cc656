"""GPU behaviour at the edges of the C ABI: calls on a side stream, expert ids outside the stack, more than
65535 activation rows in the [K, N] orientation, and a quantized matmul replayed from a HIP graph."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3
KQ_F16, KQ_BF16 = 1, 2


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _wire(codec, rows, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, rows * (K // wpb), seed).reshape(rows, K // wpb * bpb)


def test_ops_on_a_side_stream_see_their_inputs(kq):
    """stream=: the op runs on the caller's stream after the work already queued on the current stream (the
    preparation of its inputs); as with any torch side stream, the consumer waits for that stream."""
    side = torch.cuda.Stream()
    N, K, M = 512, 2048, 3
    w = wire_to_dev(_wire("q4_k", N, K, 70))
    E, T, R = 4, 6, 2
    gate = wire_to_dev(_wire("q5_k", E * 64, 512, 71)).reshape(E, 64, -1)
    up = wire_to_dev(_wire("q5_k", E * 64, 512, 72)).reshape(E, 64, -1)
    idx = torch.randint(0, E, (T, R), device="cuda:0")
    for rep in range(4):
        # the inputs are produced by a long chain of kernels on the current stream right before the call
        x = torch.randn(M, K, device="cuda:0", dtype=torch.float32)
        for _ in range(20):
            x = x * 1.0001 + 0.0001
        x = x.to(torch.bfloat16)
        xm = torch.randn(T, 512, device="cuda:0", dtype=torch.float32)
        for _ in range(20):
            xm = xm * 0.9999
        xm = xm.to(torch.float16)
        y_side = kq.quantized_matmul(x, w, None, "q4_k", stream=side)
        g_side = kq.moe_glu_gather_kq(xm, gate, up, "q5_k", idx, stream=side)
        torch.cuda.current_stream().wait_stream(side)
        y_side_sum, g_side_sum = y_side.float().sum(), g_side.float().sum()
        y_main = kq.quantized_matmul(x, w, None, "q4_k")
        g_main = kq.moe_glu_gather_kq(xm, gate, up, "q5_k", idx)
        torch.cuda.synchronize()
        assert torch.equal(y_side, y_main), rep
        assert torch.equal(g_side, g_main), rep
        assert float(y_side_sum) == float(y_main.float().sum())
        assert float(g_side_sum) == float(g_main.float().sum())


@pytest.mark.parametrize("T", [4, 12])
@pytest.mark.parametrize("codec,K", [("q4_k", 512), ("q6_k", 256), ("iq4_nl", 256), ("q5_0", 128), ("q8_0", 128),
                                     ("q2_k", 256)])
def test_expert_ids_outside_the_stack_are_skipped(kq, codec, K, T):
    """Entries whose expert id is >= E are left out (their output rows keep what they held); the others are
    computed as usual.  8 entries run the per-entry kernels (streamed, code-level, generic), 24 the grouped ones
    (q4_k / q6_k: still the per-entry streamed kernel)."""
    lib = kq._load()
    cid = lib.kq_codec_id(codec.encode())
    E, N, R = 3, 64, 2
    stack = _wire(codec, E * N, K, 80).reshape(E, N, -1)
    w = wire_to_dev(stack)
    xb, xt = make_x((T * R, K), "float16", seed=81)
    idx = np.tile(np.array([0, 3, 2, 0xFFFFFFFF, 1, 1, 7, 0], dtype=np.uint32), T * R // 8)
    idx_t = torch.from_numpy(idx.view(np.int32).copy()).cuda()
    out = torch.full((T * R, N), 5.0, dtype=torch.float16, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    nws = lib.kq_moe_workspace_size(T, R, E, N, K, 0, cid, KQ_F16)
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device="cuda:0")
    rc = lib.kq_gather_qmv(xt.data_ptr(), w.data_ptr(), idx_t.data_ptr(), None, out.data_ptr(), T, R, E, N, K, cid,
                           KQ_F16, ws.data_ptr(), nws, stream)
    assert rc == 0, lib.kq_last_error()
    torch.cuda.synchronize()
    got = dev_to_bits(out)
    for p in range(T * R):
        if idx[p] >= E:
            assert np.all(O.bits_to_f32(got[p], "float16") == 5.0), (codec, p)
        else:
            want = O.qmm(xb[p:p + 1], stack[idx[p]], codec, True, "float16")
            assert rel_l2(got[p:p + 1], want, "float16") <= TOL, (codec, p)


def test_expert_ids_outside_the_stack_no_transpose(kq):
    lib = kq._load()
    codec, E, K, N, B, M = "q4_0", 2, 16, 64, 4, 2
    cid = lib.kq_codec_id(codec.encode())
    stack = _wire(codec, E * K, N, 82).reshape(E, K, -1)  # [E, K, N / wpb * bpb]
    w = wire_to_dev(stack)
    xb, xt = make_x((B, M, K), "bfloat16", seed=83)
    rhs = np.array([1, 2, 0, 9], dtype=np.uint32)
    lhs = np.arange(B, dtype=np.uint32)
    out = torch.full((B, M, N), 3.0, dtype=torch.bfloat16, device="cuda:0")
    lhs_t = torch.from_numpy(lhs.view(np.int32).copy()).cuda()
    rhs_t = torch.from_numpy(rhs.view(np.int32).copy()).cuda()
    rc = lib.kq_gather_qmm(xt.data_ptr(), w.data_ptr(), lhs_t.data_ptr(), rhs_t.data_ptr(), out.data_ptr(), B, M, E, N, K,
                           M * K, stack.shape[1] * stack.shape[2], 0, 0, cid, KQ_BF16, None, 0,
                           torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.kq_last_error()
    torch.cuda.synchronize()
    got = dev_to_bits(out)
    for b in range(B):
        if rhs[b] >= E:
            assert np.all(O.bits_to_f32(got[b], "bfloat16") == 3.0)
        else:
            want = O.qmm(xb[b], stack[rhs[b]], codec, False, "bfloat16")
            assert rel_l2(got[b], want, "bfloat16") <= TOL


def test_no_transpose_more_rows_than_one_grid_dimension(kq):
    """x [M, K] @ W [K, N] with M above 65535 (the row index does not fit the launch grid's y extent)."""
    codec, K, N, M = "q8_0", 8, 32, 65536 + 37
    wire = _wire(codec, K, N, 84)
    xb, xt = make_x((M, K), "float16", seed=85)
    got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec, transpose=False))
    assert got.shape == (M, N)
    rows = np.r_[0:40, 65500:65573]
    want = O.qmm(xb[rows], wire, codec, False, "float16")
    assert rel_l2(got[rows], want, "float16") <= TOL
    # every row was written: the whole product against a float64 matmul with the decoded weights
    full = O.bits_to_f32(xb, "float16").astype(np.float64) @ O.dequantize(wire, codec).astype(np.float64).reshape(K, N)
    g = O.bits_to_f32(got, "float16").astype(np.float64)
    assert np.linalg.norm(g - full) / np.linalg.norm(full) <= TOL


@pytest.mark.parametrize("codec,M", [("iq2_xxs", 1), ("iq3_s", 4), ("q4_k", 1)])
def test_qmm_replayed_from_a_hip_graph(kq, codec, M):
    """kq_qmm captured into a HIP graph (codebook lookup, workspace and all) gives the eager bits on every replay,
    with eager work and synchronisations between the replays."""
    lib = kq._load()
    cid = lib.kq_codec_id(codec.encode())
    N, K = 1024, 2048
    wire = _wire(codec, N, K, 90)
    w = wire_to_dev(wire)
    xb, xt = make_x((M, K), "bfloat16", seed=91)
    nws = lib.kq_qmm_workspace_size(M, N, K, 1, cid, KQ_BF16)
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device="cuda:0")
    y_eager = torch.empty((M, N), dtype=torch.bfloat16, device="cuda:0")
    y_graph = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda:0")

    def call(y, stream):
        rc = lib.kq_qmm(xt.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K, 1, cid, KQ_BF16, ws.data_ptr(), nws, stream)
        assert rc == 0, lib.kq_last_error()

    call(y_eager, torch.cuda.current_stream().cuda_stream)  # also the first use of the codebooks on this device
    torch.cuda.synchronize()
    assert rel_l2(dev_to_bits(y_eager), O.qmm(xb, wire, codec, True, "bfloat16"), "bfloat16") <= TOL
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(y_graph, torch.cuda.current_stream().cuda_stream)
    for rep in range(4):
        y_graph.zero_()
        ws.fill_(0xAB)  # whatever an earlier user left in the workspace
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager), (codec, rep)
        other = torch.randn(256, 256, device="cuda:0")
        (other @ other).sum().item()  # the program's own eager work between replays


@pytest.mark.parametrize("codec,K", [("q4_k", 1024), ("q6_k", 512)])
def test_fused_gate_up_skips_expert_ids_outside_the_stack(kq, codec, K):
    """kq_moe_glu_gather with 8 entries (the gathered mode of the streamed kernel): entries whose expert id is >= E
    leave their output rows as they were, the others are computed."""
    lib = kq._load()
    cid = lib.kq_codec_id(codec.encode())
    E, N, T, R = 3, 48, 4, 2
    gate = _wire(codec, E * N, K, 95).reshape(E, N, -1)
    up = _wire(codec, E * N, K, 96).reshape(E, N, -1)
    g_dev, u_dev = wire_to_dev(gate), wire_to_dev(up)
    xb, xt = make_x((T, K), "bfloat16", seed=97, scale=0.1)
    idx = np.array([[0, 3], [2, 0xFFFFFFFF], [1, 1], [7, 0]], dtype=np.uint32)
    idx_t = torch.from_numpy(idx.view(np.int32).copy()).cuda()
    out = torch.full((T, R, N), 5.0, dtype=torch.bfloat16, device="cuda:0")
    nws = lib.kq_moe_workspace_size(T, R, E, N, K, 1, cid, KQ_BF16)
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device="cuda:0")
    rc = lib.kq_moe_glu_gather(xt.data_ptr(), g_dev.data_ptr(), u_dev.data_ptr(), idx_t.data_ptr(), None, None,
                               out.data_ptr(), T, R, E, N, K, 0, 0.0, 0.0, cid, KQ_BF16, ws.data_ptr(), nws,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.kq_last_error()
    torch.cuda.synchronize()
    got = dev_to_bits(out)
    for t in range(T):
        for r in range(R):
            if idx[t, r] >= E:
                assert np.all(O.bits_to_f32(got[t, r], "bfloat16") == 5.0), (codec, t, r)
            else:
                want = O.moe_glu_gather(xb[t:t + 1], gate, up, codec, idx[t:t + 1, r:r + 1].astype(np.int64), "silu",
                                        dtype="bfloat16")
                assert rel_l2(got[t:t + 1, r:r + 1], want, "bfloat16") <= TOL, (codec, t, r)
