"""GPU parity: kq.quantized_matmul (HIP) vs the CPU oracle.  Tolerance: rel-L2 <= 1e-3 on the
rounded outputs (fp32 accumulation, one rounding to the activation dtype)."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import bits_to_dev, dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _wire(codec, N, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, N * (K // wpb), seed).reshape(N, K // wpb * bpb)


@pytest.mark.parametrize("codec", O.ALL_CODECS)
@pytest.mark.parametrize("M", [1, 3, 8])
def test_qmm_all_codecs_small(kq, codec, M):
    N, K = 96, 512
    wire = _wire(codec, N, K, seed=31)
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((M, K), dtype, seed=M)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, dtype)
        assert tuple(got.shape) == (M, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, dtype)


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "q5_k", "q8_0", "iq4_xs", "mxfp4"])
@pytest.mark.parametrize("M", [1, 2, 4, 8, 17, 64])
def test_qmm_decode_and_prefill_shapes(kq, codec, M):
    N, K = 256, 2048 if codec != "mxfp4" else 2880
    wire = _wire(codec, N, K, seed=32)
    xb, xt = make_x((M, K), "bfloat16", seed=100 + M)
    got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
    want = O.qmm(xb, wire, codec, True, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, M)


@pytest.mark.parametrize("codec", ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("M,N,K", [(1, 1000, 768), (3, 20000, 256), (8, 520, 4352), (2, 40, 8192), (5, 4100, 1024),
                                   (1, 33, 2048)])
def test_qmm_skinny_ragged_shapes(kq, codec, M, N, K):
    """Row tiles that do not divide N, K of 1 / 3 / 17 superblocks (partial sub-chunks, two chunks)."""
    wire = _wire(codec, N, K, seed=34)
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((M, K), dtype, seed=200 + M)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, N, K, dtype)


NON_K = [c for c in O.ALL_CODECS if c not in ("q2_k", "q3_k", "q4_k", "q5_k", "q6_k")]


@pytest.mark.parametrize("codec", NON_K)
def test_qmm_skinny_codes_ragged(kq, codec):
    """Legacy / IQ / fp4 codecs at M <= 8: K of 7 blocks (a partial last 256-weight step for the 32- and
    64-weight blocks), a partial 128-row tile, a K long enough to be split across workgroups, both dtypes,
    and activations spanning 30 binades (the per-step power-of-two scaling of bf16 inputs)."""
    wpb, _ = O.geometry(codec)
    for M, N, K in ((1, 131, 7 * wpb), (5, 40, 3 * 256), (8, 200, 8192), (2, 300, 2048 + wpb)):
        wire = _wire(codec, N, K, seed=35)
        for dtype in ("bfloat16", "float16"):
            xb, xt = make_x((M, K), dtype, seed=300 + M)
            got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
            want = O.qmm(xb, wire, codec, True, dtype)
            assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, N, K, dtype)
    M, N, K = 4, 64, 1024
    wire = _wire(codec, N, K, seed=36)
    x = np.random.default_rng(37).standard_normal((M, K)).astype(np.float32)
    x *= np.exp2(np.random.default_rng(38).integers(-15, 15, (M, K // 256)).repeat(256, axis=1)).astype(np.float32)
    xb = O.f32_to_bits(x, "bfloat16")
    got = kq.quantized_matmul(bits_to_dev(xb, "bfloat16"), wire_to_dev(wire), None, codec)
    assert rel_l2(dev_to_bits(got), O.qmm(xb, wire, codec, True, "bfloat16"), "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["mxfp4", "q8_0", "q2_k", "iq2_xxs", "q5_0"])
def test_qmm_gemv_unaligned_rows_and_tensor_end(kq, codec):
    """Rows that start at odd byte addresses (17 / 34 / 22-byte blocks, a view 1 byte into an allocation) and
    a last row that ends exactly where the allocation ends."""
    wpb, bpb = O.geometry(codec)
    N, K, M = 37, 5 * wpb, 3
    wire = _wire(codec, N, K, seed=39)
    buf = torch.zeros(wire.size + 1, dtype=torch.uint8, device="cuda:0")
    view = buf[1:].view(N, -1)
    view.copy_(wire_to_dev(wire))
    xb, xt = make_x((M, K), "float16", seed=40)
    got = kq.quantized_matmul(xt, view, None, codec)
    want = O.qmm(xb, wire, codec, True, "float16")
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL


@pytest.mark.parametrize("codec", ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_qmm_skinny_both_variants(kq, codec):
    """Dense skinny calls through every selectable kernel: workgroup-synchronous (1), decoupled-wave (2),
    its two-superblock-unit form (3), the diagonal kernel (4; shapes whose K is not a multiple of 1024
    fall back to the decoupled one) and the streamed kernel (5; q4_k / q5_k / q6_k up to four rows, the rest
    falls back)."""
    lib = kq._load()
    try:
        for variant in (1, 2, 3, 4, 5):
            lib.kq_set_skinny_variant(variant)
            for M, N, K in ((1, 1000, 768), (8, 520, 4352), (3, 4100, 1024), (2, 300, 4096), (5, 4200, 14336),
                            (7, 100, 2048)):
                wire = _wire(codec, N, K, seed=41)
                xb, xt = make_x((M, K), "bfloat16", seed=42)
                got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
                want = O.qmm(xb, wire, codec, True, "bfloat16")
                assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, variant, M, N, K)
    finally:
        lib.kq_set_skinny_variant(0)


@pytest.mark.parametrize("codec", ["q4_k", "q5_k", "q6_k", "q2_k", "q3_k", "iq4_xs", "iq2_xxs", "iq3_s", "q8_0", "iq4_nl",
                                   "q4_0", "mxfp4", "nvfp4"])
@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
def test_qmm_streamed_kernel_shapes(kq, codec, dtype):
    """The streamed kernel (default for up to eight rows of q4_k / q5_k / q6_k): one to eight rows (five and more
    run two groups of four), K ranges that leave waves without a superblock (256, 768), K above 16 superblocks
    (split over grid z), a ragged last row tile, a single row, row counts that level to tiles of fewer than 32
    rows (14336 -> 28, 15000 -> 30), more row tiles than resident workgroups (persistent loop, N = 20000), and
    small shapes of up to four rows that run short tiles (8 or 16 rows, 4096 x 4096, 1000 x 2048, 97 x 4096)
    on eight-wave workgroups instead of a K split."""
    for M, N, K in ((1, 33, 256), (2, 31, 768), (3, 1, 1024), (4, 97, 4096), (1, 20000, 1024), (2, 1030, 5120),
                    (1, 4100, 14336), (4, 2050, 8192), (5, 33, 256), (8, 97, 4096), (7, 1030, 5120), (6, 2050, 8192),
                    (8, 20000, 1024), (5, 1, 768), (1, 14336, 512), (8, 15000, 256), (3, 14336, 1024), (1, 8192, 8192),
                    (2, 300, 6144), (4, 8200, 7936), (1, 4096, 4096), (3, 1000, 2048)):
        wire = _wire(codec, N, K, seed=43)
        xb, xt = make_x((M, K), dtype, seed=44)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype, M, N, K)


@pytest.mark.parametrize("codec", ["mxfp4", "q4_0", "iq4_nl", "q8_0"])
@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
def test_qmm_streamed_kernel_k_ends_inside_a_unit(kq, codec, dtype):
    """The codecs of 32-weight blocks run on the streamed kernel for any K that is a multiple of 32 from 256 up: the
    last 256-weight unit of a row then holds one to seven blocks (K = 2880: 11 units and 2 blocks).  One to eight
    rows, ragged row tiles, a K range cut over grid z (33 units), the whole 2880 x 2880 matrix."""
    for M, N, K in ((1, 100, 288), (3, 64, 2880), (8, 37, 480), (2, 200, 8192 + 96), (1, 2880, 2880), (5, 40, 4096 + 32),
                    (4, 33, 256 + 224)):
        wire = _wire(codec, N, K, seed=71)
        xb, xt = make_x((M, K), dtype, seed=72)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, dtype)
        assert tuple(got.shape) == (M, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype, M, N, K)


@pytest.mark.parametrize("codec", ["mxfp4", "q4_0", "q8_0"])
def test_qmm_k_tail_uses_nothing_past_the_weights(kq, codec):
    """A short last unit is fetched in 16-byte pieces none of which reaches past its row: a matrix that ends exactly
    on a page boundary (as 32 x 2880 x 2880 mxfp4 stacks do) or a few bytes before one, with 0xff bytes (NaN scales)
    around it, gives the oracle's result."""
    N, K, M = 70, 2880, 2
    wire = _wire(codec, N, K, seed=73)
    nbytes = wire.size
    xb, xt = make_x((M, K), "bfloat16", seed=74)
    want = O.qmm(xb, wire, codec, True, "bfloat16")
    buf = torch.full((nbytes + 2 * 4096,), 0xff, dtype=torch.uint8, device="cuda:0")
    for end_in_page in (2048, 4090, 0):
        off = (end_in_page - (buf.data_ptr() + nbytes)) % 4096
        view = buf[off:off + nbytes].view(N, -1)
        view.copy_(wire_to_dev(wire))
        assert (view.data_ptr() + nbytes) % 4096 == end_in_page
        got = kq.quantized_matmul(xt, view, None, codec)
        assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, end_in_page)
        buf.fill_(0xff)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("N,K", [(264, 512), (4096, 4096), (1000, 8192), (33, 256), (97, 320), (20000, 1024)])
def test_qmv_bias_fused_decode(kq, N, K, dtype):
    """q8_0 decode with the bias added to the f32 sum before the single rounding (quantized_matmul_qmv_bias): the
    streamed kernel where K is a multiple of 256 and its plan needs no K split, the code-level kernel otherwise
    (K = 320; 264 x 512 and 33 x 256 are too small to fill the chip unsplit)."""
    wire = _wire("q8_0", N, K, seed=301)
    xb, xt = make_x((1, K), dtype, seed=302)
    b = np.random.default_rng(303).standard_normal(N).astype(np.float32)
    bbits = O.f32_to_bits(b, dtype)
    bt = torch.from_numpy(bbits.view(np.int16)).cuda().view(torch.bfloat16 if dtype == "bfloat16" else torch.float16)
    got = kq.quantized_matmul_qmv_bias(xt, wire_to_dev(wire), None, bt, "q8_0")
    f32 = O.qmm(O.bits_to_f32(xb, dtype).reshape(1, K), wire, "q8_0", True, "float32")
    want = O.f32_to_bits(f32 + O.bits_to_f32(bbits, dtype), dtype)
    assert tuple(got.shape) == (1, N) and got.dtype == xt.dtype
    assert rel_l2(dev_to_bits(got), want, dtype) <= TOL


def test_qmm_skinny_unaligned_q6k_rows(kq):
    """q6_k rows are 210-byte multiples: a wire view that starts 2 bytes into an allocation still decodes."""
    N, K, M = 64, 768, 1
    wire = _wire("q6_k", N, K, seed=35)
    buf = torch.zeros(wire.size + 16, dtype=torch.uint8, device="cuda:0")
    view = buf[2:2 + wire.size].view(N, -1)
    view.copy_(wire_to_dev(wire))
    xb, xt = make_x((M, K), "bfloat16", seed=36)
    got = kq.quantized_matmul(xt, view, None, "q6_k")
    want = O.qmm(xb, wire, "q6_k", True, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q8_0", "iq4_nl"])
def test_qmm_no_transpose(kq, codec):
    K, N, M = 64, 512, 5  # W decodes to [K, N]
    wire = _wire(codec, K, N, seed=33)
    xb, xt = make_x((M, K), "float16", seed=7)
    got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec, transpose=False)
    want = O.qmm(xb, wire, codec, False, "float16")
    assert tuple(got.shape) == (M, N)
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_qmm_no_transpose_every_codec_on_the_matrix_cores(kq, codec):
    """transpose=False (src/kquant_matmul.cpp:455-527 of the reference): the reduction runs over wire rows.  Shapes
    with a ragged last 32-row step, a K that is no multiple of 8, more than 32 activation rows and a column count
    that does not fill the last 128-column tile, in both activation types."""
    shapes = [(1, 128, 512, "bfloat16", 1), (5, 50, 768, "float16", 2), (40, 27, 256, "bfloat16", 3),
              (3, 16, 1280, "float16", 4)]
    if codec in ("q4_k", "q6_k", "q8_0", "iq3_s", "mxfp4"):  # long K, few tiles: the K range is cut over the grid
        shapes += [(3, 1024, 256, "float16", 6), (20, 1000, 256, "bfloat16", 7), (2, 1001, 256, "bfloat16", 11)]
    # 96 rows and more: the kernel that decodes a step once per 128 rows (ragged rows, odd step counts, K cut)
    shapes += [(100, 72, 256, "bfloat16", 8), (200, 33, 512, "float16", 9)]
    if codec in ("q4_k", "q6_k", "q8_0", "iq2_xxs", "nvfp4"):
        shapes.append((130, 1056, 256, "bfloat16", 10))
    if O.geometry(codec)[0] == 32:
        shapes.append((2, 70, 352, "bfloat16", 5))
    for (M, K, N, dtype, seed) in shapes:
        wire = _wire(codec, K, N, seed=70 + seed)
        xb, xt = make_x((M, K), dtype, seed=80 + seed)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec, transpose=False)
        want = O.qmm(xb, wire, codec, False, dtype)
        assert tuple(got.shape) == (M, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, K, N, dtype)


@pytest.mark.parametrize("codec,M,K,N,dtype", [("q4_k", 2048, 64, 4096, "bfloat16"), ("q8_0", 2100, 40, 4096, "float16"),
                                               ("q6_k", 2050, 96, 4096, "bfloat16")])
def test_qmm_no_transpose_many_rows(kq, codec, M, K, N, dtype):
    """transpose=False with thousands of activation rows (a ragged last row tile, a ragged last K step)."""
    wire = _wire(codec, K, N, seed=90)
    xb, xt = make_x((M, K), dtype, seed=91)
    got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec, transpose=False)
    want = O.qmm(xb, wire, codec, False, dtype)
    assert tuple(got.shape) == (M, N)
    assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, K, N, dtype)


def test_qmm_dtype_rules_and_shapes(kq):
    N, K = 64, 256
    wire = _wire("q4_k", N, K, seed=34)
    w = wire_to_dev(wire)
    x32 = torch.from_numpy(np.random.default_rng(1).standard_normal((2, 3, K)).astype(np.float32)).cuda()
    y = kq.quantized_matmul(x32, w, None, "q4_k")
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (2, 3, N)  # f32 -> bf16, x cast first
    xb = O.f32_to_bits(x32.cpu().numpy().reshape(6, K), "bfloat16")
    want = O.qmm(xb, wire, "q4_k", True, "bfloat16")
    assert rel_l2(dev_to_bits(y).reshape(6, N), want, "bfloat16") <= TOL
    with pytest.raises(ValueError):
        kq.quantized_matmul(x32[..., :128], w, None, "q4_k")
    with pytest.raises(ValueError):
        kq.quantized_matmul(x32, w.reshape(1, N, -1), None, "q4_k")
    with pytest.raises(ValueError):
        kq.quantized_matmul(x32.to(torch.int32), w, None, "q4_k")
    empty = kq.quantized_matmul(x32[:0], w, None, "q4_k")
    assert tuple(empty.shape) == (0, 3, N)


@pytest.mark.parametrize("codec", ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_qmm_reference_fixtures(kq, codec):
    import os
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    wire = np.load(os.path.join(gold, f"{codec}.npz"))["wire"]  # [256, bpr], K = 512
    for M in (1, 64):
        xb, xt = make_x((M, 512), "float16", seed=M)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, "float16")
        assert rel_l2(dev_to_bits(got), want, "float16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("M,N,K", [(9, 40, 256), (200, 200, 512), (130, 384, 2304), (512, 256, 4096)])
def test_qmm_prefill_gemm(kq, codec, M, N, K):
    """Prefill GEMM path (M > 8): ragged M and N tiles, several superblocks, both activation dtypes."""
    wire = _wire(codec, N, K, seed=35)
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((M, K), dtype, seed=M + K)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, dtype)
        assert tuple(got.shape) == (M, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, N, K, dtype)


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_qmm_prefill_every_codec(kq, codec):
    """M > 8 for every codec (the tuned K-quant GEMM or the any-codec bf16 matrix-core path), both
    activation dtypes, N that is not a multiple of the 128-row slab, and for the 32-weight-block codecs a K
    that is not a multiple of the 256-weight step."""
    wpb, _ = O.geometry(codec)
    shapes = [(40, 200, 512)] + ([(130, 72, 288)] if wpb == 32 else [(130, 72, 768)])
    for M, N, K in shapes:
        wire = _wire(codec, N, K, seed=61)
        for dtype in ("bfloat16", "float16"):
            xb, xt = make_x((M, K), dtype, seed=62)
            got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
            want = O.qmm(xb, wire, codec, True, dtype)
            assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, M, N, K, dtype)


def test_qmm_prefill_gemm_tile_variants(kq):
    """The 128 x 128, the two-stage 64 x 256 and the 128 x 256 direct-to-LDS tile variants (kq_set_gemm_tile_rows)
    give the same rounded outputs as the 64 x 128 one: all feed the same exact products to f32 accumulators in the
    same order.  N is no multiple of 256, M none of 64, and K spans several steps so that both LDS stages are
    reused (q6_k has no 128 x 256 kernel and falls back)."""
    M, N, K = 200, 384, 2048
    lib = kq._load()
    for codec in ("q4_k", "q5_k", "q6_k"):
        wire = _wire(codec, N, K, seed=37)
        xb, xt = make_x((M, K), "bfloat16", seed=38)
        want = O.qmm(xb, wire, codec, True, "bfloat16")
        outs = []
        try:
            for rows in (128, 256, 512, 513, 64):
                lib.kq_set_gemm_tile_rows(rows)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
                assert rel_l2(got, want, "bfloat16") <= TOL, (codec, rows)
                outs.append(got)
        finally:
            lib.kq_set_gemm_tile_rows(0)
        assert all(np.array_equal(o, outs[-1]) for o in outs[:-1]), codec


@pytest.mark.parametrize("K", [256, 512, 768])
def test_qmm_prefill_gemm_two_stage_short_k(kq, K):
    """The two-stage tile with one, two and three K steps (prologue only, one parked step, stage reuse)."""
    M, N = 70, 264
    lib = kq._load()
    wire = _wire("q4_k", N, K, seed=39)
    xb, xt = make_x((M, K), "float16", seed=40)
    want = O.qmm(xb, wire, "q4_k", True, "float16")
    try:
        lib.kq_set_gemm_tile_rows(256)
        got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, "q4_k"))
    finally:
        lib.kq_set_gemm_tile_rows(0)
    assert rel_l2(got, want, "float16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q5_k"])
def test_qmm_prefill_gemm_128x256_tiles(kq, codec):
    """The direct-to-LDS kernels (512: 128 x 256 tiles, K steps of 128; 513: 128 x 128 tiles, K steps of 64): one,
    two and nine superblocks of K (prologue only, both wire stages, stage reuse), ragged M and N tiles, both
    activation dtypes."""
    lib = kq._load()
    try:
      for rows in (512, 513):
        lib.kq_set_gemm_tile_rows(rows)
        for M, N, K, dtype in ((9, 40, 256, "bfloat16"), (130, 257, 512, "float16"), (300, 520, 2304, "bfloat16"),
                               (128, 256, 1024, "bfloat16")):
            wire = _wire(codec, N, K, seed=63)
            xb, xt = make_x((M, K), dtype, seed=64)
            got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
            want = O.qmm(xb, wire, codec, True, dtype)
            assert rel_l2(got, want, dtype) <= TOL, (codec, rows, M, N, K, dtype)
    finally:
        lib.kq_set_gemm_tile_rows(0)


@pytest.mark.parametrize("codec", ["iq2_xxs", "iq2_xs", "iq2_s", "iq3_xxs", "iq3_s", "iq1_s", "iq1_m"])
def test_qmm_prefill_iq_tall_tiles(kq, codec):
    """The codebook codecs on the 256-row and 128-row tiles (the reference-order decoder with d = 1 as one exact f16
    term, d in the unit of the running sums, codebook in LDS, wire bytes by 4-byte direct-to-LDS loads): one to nine
    superblocks of K, ragged M and N tiles (the matrix's last row sits in every one of these calls: its last dword is
    loaded two bytes early and shifted), both activation dtypes; superblocks with d = 0 and negative d; and the
    automatic choice on a matrix wide enough to be taken."""
    lib = kq._load()
    wpb, bpb = O.geometry(codec)
    try:
        for rows in (1024, 1025):
            lib.kq_set_gemm_tile_rows(rows)
            for M, N, K, dtype in ((128, 40, 256, "bfloat16"), (130, 257, 512, "float16"), (300, 520, 2304, "bfloat16"),
                                   (513, 700, 1024, "float16")):
                wire = _wire(codec, N, K, seed=91)
                xb, xt = make_x((M, K), dtype, seed=92)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
                want = O.qmm(xb, wire, codec, True, dtype)
                assert rel_l2(got, want, dtype) <= TOL, (codec, rows, M, N, K, dtype)
            if codec != "iq1_m":  # iq1_m keeps d in the top nibbles of its scale words
                M, N, K = 140, 300, 1536
                wire = _wire(codec, N, K, seed=93).copy()
                blocks = wire.reshape(N, K // wpb, bpb)
                blocks[::3, ::2, 0:2] = 0      # d = 0: the superblock keeps the unit of the running sums
                blocks[1::3, :, 1] |= 0x80     # negative d
                xb, xt = make_x((M, K), "bfloat16", seed=94)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
                want = O.qmm(xb, wire, codec, True, "bfloat16")
                assert rel_l2(got, want, "bfloat16") <= TOL, (codec, rows, "special blocks")
        lib.kq_set_gemm_tile_rows(0)
        M, N, K = 256, 24600, 256
        wire = _wire(codec, N, K, seed=95)
        xb, xt = make_x((M, K), "float16", seed=96)
        got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
        assert rel_l2(got, O.qmm(xb, wire, codec, True, "float16"), "float16") <= TOL, (codec, "automatic")
    finally:
        lib.kq_set_gemm_tile_rows(0)


@pytest.mark.parametrize("codec", ["mxfp4", "nvfp4"])
def test_qmm_prefill_fp4_tall_tiles(kq, codec):
    """mxfp4 / nvfp4 on the 256-row and 128-row tiles (one exact f16 term per weight out of the hardware's fp4 -> f16
    conversion): one to forty-five K steps of 64, ragged M and N tiles, both activation dtypes; then scale edge cases —
    mxfp4 rows whose block exponents jump by tens of binades from step to step (the per-column exponent offset
    moves and the running sums are rescaled), exponents 0 / 1 / 2, and nvfp4 scale bytes 0x00, 0x7f (both decode to
    0), 0x80, 0xff and the subnormal scales 0x01 ... 0x07; and the automatic choice on a wide matrix."""
    lib = kq._load()
    wpb, bpb = O.geometry(codec)
    try:
        for rows in (1024, 1025):
            lib.kq_set_gemm_tile_rows(rows)
            for M, N, K, dtype in ((128, 40, 64, "bfloat16"), (130, 257, 192, "float16"), (300, 520, 2880, "bfloat16"),
                                   (256, 256, 320, "bfloat16"), (513, 700, 1024, "float16")):
                wire = _wire(codec, N, K, seed=81)
                xb, xt = make_x((M, K), dtype, seed=82)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
                want = O.qmm(xb, wire, codec, True, dtype)
                assert rel_l2(got, want, dtype) <= TOL, (codec, rows, M, N, K, dtype)
            M, N, K = 140, 300, 768
            wire = _wire(codec, N, K, seed=83).copy()
            blocks = wire.reshape(N, K // wpb, bpb)
            if codec == "mxfp4":
                jumps = np.array([120, 122, 180, 170, 60, 75, 131, 104, 140, 150, 20, 1, 0, 2, 200, 190, 127, 127,
                                  90, 117, 118, 91, 127, 100], np.uint8)
                blocks[0::4, :, 0] = jumps[:K // wpb]
                blocks[1::4, :, 0] = np.array([0, 1, 2, 1] * (K // wpb // 4), np.uint8)
                blocks[2::4, ::3, 1:] = 0                                  # blocks of zero codes
            else:
                edge = np.array([0x00, 0x7f, 0x80, 0xff, 0x01, 0x02, 0x03, 0x04, 0x05, 0x06, 0x07, 0x08, 0x7e, 0x38,
                                 0x40, 0x0f], np.uint8)
                for r in range(0, N, 3):
                    blocks[r, :, 0:4] = np.resize(np.roll(edge, r), (K // wpb, 4))
            xb, xt = make_x((M, K), "bfloat16", seed=84)
            got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
            want = O.qmm(xb, wire, codec, True, "bfloat16")
            assert rel_l2(got, want, "bfloat16") <= TOL, (codec, rows, "scale edge cases")
            # row by row as well: a row of tiny weights must not hide behind the large ones
            per_row = [rel_l2(got[:, r:r + 1], want[:, r:r + 1], "bfloat16") for r in range(0, N, 7)]
            assert max(per_row) <= TOL, (codec, rows, "scale edge cases, per weight row", max(per_row))
        lib.kq_set_gemm_tile_rows(0)
        M, N, K = 256, 24600, 128
        wire = _wire(codec, N, K, seed=85)
        xb, xt = make_x((M, K), "float16", seed=86)
        got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
        assert rel_l2(got, O.qmm(xb, wire, codec, True, "float16"), "float16") <= TOL, (codec, "automatic")
    finally:
        lib.kq_set_gemm_tile_rows(0)


@pytest.mark.parametrize("codec", ["q8_0", "q4_0", "iq4_nl", "q4_1", "q5_0", "q5_1"])
def test_qmm_prefill_block32_tall_tiles(kq, codec):
    """q8_0 / q4_0 / iq4_nl / q5_0 / q4_1 / q5_1 on the 256-row and 128-row tiles (every weight d q as two exact f16 terms,
    the block minimum of q4_1 / q5_1 as a third, wire bytes step by step
    through a ring of four slots): one to forty-five K steps of 64 (prologue only, ring wrap, K = 2880), ragged M and N
    tiles, both activation dtypes; blocks with d = 0, negative, subnormal and large d and the extreme codes; and the
    automatic choice on a matrix wide enough to be taken."""
    lib = kq._load()
    wpb, bpb = O.geometry(codec)
    try:
        for rows in (1024, 1025):
            lib.kq_set_gemm_tile_rows(rows)
            for M, N, K, dtype in ((128, 40, 64, "bfloat16"), (130, 257, 192, "float16"), (300, 520, 2880, "bfloat16"),
                                   (256, 256, 320, "bfloat16"), (513, 700, 1024, "float16")):
                wire = _wire(codec, N, K, seed=71)
                xb, xt = make_x((M, K), dtype, seed=72)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
                want = O.qmm(xb, wire, codec, True, dtype)
                assert rel_l2(got, want, dtype) <= TOL, (codec, rows, M, N, K, dtype)
            M, N, K = 140, 300, 512
            wire = _wire(codec, N, K, seed=73).copy()
            blocks = wire.reshape(N, K // wpb, bpb)
            blocks[::5, ::2, 0:2] = 0                                         # d = 0
            blocks[1::5, :, 1] |= 0x80                                        # negative d
            blocks[2::5, 1::2, 0:2] = np.array([0x37, 0x00], np.uint8)        # subnormal d (55 x 2^-24)
            blocks[3::5, ::3, 0:2] = np.frombuffer(np.float16(200.0).tobytes(), np.uint8)
            blocks[:, 1::4, 2:bpb:3] = 0x80 if codec == "q8_0" else 0x0f      # q = -128 / nibbles 15 and 0
            xb, xt = make_x((M, K), "bfloat16", seed=74)
            got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
            want = O.qmm(xb, wire, codec, True, "bfloat16")
            assert rel_l2(got, want, "bfloat16") <= TOL, (codec, rows, "special blocks")
        lib.kq_set_gemm_tile_rows(0)
        M, N, K = 256, 24600, 128
        wire = _wire(codec, N, K, seed=75)
        xb, xt = make_x((M, K), "float16", seed=76)
        got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
        assert rel_l2(got, O.qmm(xb, wire, codec, True, "float16"), "float16") <= TOL, (codec, "automatic")
    finally:
        lib.kq_set_gemm_tile_rows(0)


def test_qmm_prefill_q6k_tall_tiles(kq):
    """q6_k on the 256-row and 128-row tiles of the unit-chain kernel (kq_set_gemm_tile_rows(1024 / 1025); two exact
    terms per weight, wire bytes by half superblocks): one, two, four and nine superblocks of K, ragged M and N tiles,
    fewer rows than a tile, both activation dtypes, and the automatic choice; then a matrix whose blocks hold d = 0,
    negative d and the extreme scales -128 / 127 (products of 4096 that one f16 term could not hold)."""
    lib = kq._load()
    try:
        for rows in (1024, 1025, 0):
            lib.kq_set_gemm_tile_rows(rows)
            for M, N, K, dtype in ((64, 40, 256, "bfloat16"), (130, 257, 512, "float16"), (300, 520, 2304, "bfloat16"),
                                   (256, 256, 1024, "bfloat16"), (513, 700, 1024, "float16")):
                wire = _wire("q6_k", N, K, seed=66)
                xb, xt = make_x((M, K), dtype, seed=67)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, "q6_k"))
                want = O.qmm(xb, wire, "q6_k", True, dtype)
                assert rel_l2(got, want, dtype) <= TOL, (rows, M, N, K, dtype)
            M, N, K = 270, 300, 1024
            wire = _wire("q6_k", N, K, seed=68).copy()
            blocks = wire.reshape(N, K // 256, 210)
            blocks[::3, ::2, 208:210] = 0          # d = 0: the block keeps the unit of the running sums
            blocks[1::3, :, 209] |= 0x80           # negative d
            blocks[:, 1::2, 192:208] = np.tile(np.array([0x80, 0x7f], np.uint8), 8)
            blocks[:, 1::2, 0:192:7] = 0x00        # q = 0 -> (q - 32) = -32 against scale -128
            xb, xt = make_x((M, K), "bfloat16", seed=69)
            got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, "q6_k"))
            want = O.qmm(xb, wire, "q6_k", True, "bfloat16")
            assert rel_l2(got, want, "bfloat16") <= TOL, (rows, "special blocks")
    finally:
        lib.kq_set_gemm_tile_rows(0)


@pytest.mark.parametrize("codec", ["q4_k", "q5_k"])
def test_qmm_prefill_gemm_256x256_tiles(kq, codec):
    """The 256-row kernel (kq_set_gemm_tile_rows(1024): running sums kept in units of the current superblock scale):
    one, two, four and nine superblocks of K (prologue only, both wire stages, stage reuse), ragged M and N tiles,
    fewer rows than a tile, both activation dtypes; and the automatic choice, which splits the column tiles between
    this kernel and the 128-row one."""
    lib = kq._load()
    try:
        for rows in (1024, 0):
            lib.kq_set_gemm_tile_rows(rows)
            for M, N, K, dtype in ((64, 40, 256, "bfloat16"), (130, 257, 512, "float16"), (300, 520, 2304, "bfloat16"),
                                   (256, 256, 1024, "bfloat16"), (513, 700, 1024, "float16")):
                wire = _wire(codec, N, K, seed=63)
                xb, xt = make_x((M, K), dtype, seed=64)
                got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, codec))
                want = O.qmm(xb, wire, codec, True, dtype)
                assert rel_l2(got, want, dtype) <= TOL, (codec, rows, M, N, K, dtype)
    finally:
        lib.kq_set_gemm_tile_rows(0)


def test_qmm_prefill_gemm_256x256_tiles_scale_corner_cases(kq):
    """Superblocks the unit chain of the 256-row kernel must survive: d = 0 with a live dmin (the unit is kept and the
    integers are fed as zeros), a subnormal d next to a large dmin, d falling and rising by 2^20 between neighbouring
    superblocks, dmin = 0, and a first superblock with d = 0.  Every output row is checked on its own."""
    lib = kq._load()
    M, N, K = 256, 256, 2048
    nsb = K // 256
    wire = _wire("q4_k", N, K, seed=91).reshape(N, nsb, 144).copy()

    def put(rows, sb, d, dmin):
        wire[rows, sb, 0:2] = np.frombuffer(np.float16(d).tobytes(), dtype=np.uint8)
        wire[rows, sb, 2:4] = np.frombuffer(np.float16(dmin).tobytes(), dtype=np.uint8)

    put(slice(0, 64), 0, 0.0, 0.01)          # first superblock without a scale
    put(slice(0, 64), 3, 0.0, 0.02)          # d = 0 in the middle, live minima
    put(slice(64, 128), 2, 6e-8, 3.0)        # subnormal d, dmin / d = 5e7
    put(slice(64, 128), 5, 1e-5, 0.0)        # no minima
    put(slice(128, 192), 1, 8.0, 0.001)      # the unit jumps up by about 2^10 ...
    put(slice(128, 192), 2, 1e-5, 0.001)     # ... and down by 2^20
    put(slice(192, 256), 4, 0.0, 0.0)        # an all-zero superblock
    wire = wire.reshape(N, nsb * 144)
    xb, xt = make_x((M, K), "bfloat16", seed=92)
    want = O.bits_to_f32(O.qmm(xb, wire, "q4_k", True, "bfloat16"), "bfloat16").astype(np.float64)
    try:
        lib.kq_set_gemm_tile_rows(1024)
        got = dev_to_bits(kq.quantized_matmul(xt, wire_to_dev(wire), None, "q4_k"))
    finally:
        lib.kq_set_gemm_tile_rows(0)
    g = O.bits_to_f32(got, "bfloat16").astype(np.float64)
    assert np.isfinite(g).all()
    for c0 in range(0, N, 64):  # per group of weight rows: the corner cases do not hide behind the ordinary columns
        blk = slice(c0, c0 + 64)
        assert np.linalg.norm(g[:, blk] - want[:, blk]) / np.linalg.norm(want[:, blk]) <= TOL, c0


def test_qmm_prefill_gemm_wide_dynamic_range(kq):
    """bf16 activations spanning many binades and rows of very different scale: the per-row power-of-two
    scaling of the f16 conversion must keep every row within tolerance."""
    M, N, K = 64, 128, 1024
    wire = _wire("q4_k", N, K, seed=36)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((M, K)).astype(np.float32) * np.exp2(rng.integers(-12, 12, (M, K))).astype(np.float32)
    x *= np.exp2(np.linspace(-60, 60, M)).astype(np.float32)[:, None]
    xb = O.f32_to_bits(x, "bfloat16")
    got = dev_to_bits(kq.quantized_matmul(bits_to_dev(xb, "bfloat16"), wire_to_dev(wire), None, "q4_k"))
    want = O.qmm(xb, wire, "q4_k", True, "bfloat16")
    g, w_ = O.bits_to_f32(got, "bfloat16").astype(np.float64), O.bits_to_f32(want, "bfloat16").astype(np.float64)
    rel_rows = np.linalg.norm(g - w_, axis=1) / np.linalg.norm(w_, axis=1)
    assert rel_rows.max() <= TOL, rel_rows.max()


@pytest.mark.parametrize("codec", ["iq4_xs", "q8_0", "mxfp4", "iq2_xxs"])
def test_qmm_single_row_many_row_tiles(kq, codec):
    """More row tiles than CUs (N = 8300 -> 260 tiles, the last one ragged): single-row calls of the larger
    code-level kernels switch to 4-wave workgroups there; two rows keep 8 waves."""
    N, K = 8300, 512 if codec != "mxfp4" else 288
    wire = _wire(codec, N, K, seed=45)
    for M in (1, 2):
        xb, xt = make_x((M, K), "bfloat16", seed=46 + M)
        got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
        want = O.qmm(xb, wire, codec, True, "bfloat16")
        assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, M)
