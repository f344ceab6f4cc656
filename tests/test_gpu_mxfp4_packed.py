"""GPU parity: the MLX packed-layout mxfp4 ops (kq.moe_glu_gather, kq.gather_qmv_bias, kq.gather_qmv_mix_bias) and the
layout converters, against the CPU oracle on the equivalent GGUF wire and against the layouts' definitions."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3
E2M1 = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.0, -0.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _packed_stack(E, N, K, seed):
    """Random MLX-layout stack: 8 sequential 4-bit codes per uint32 word, e8m0 scale per 32 weights."""
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, (E, N, K), dtype=np.uint8)
    scales = rng.integers(118, 126, (E, N, K // 32), dtype=np.uint8)
    nib = codes.reshape(E, N, K // 8, 8).astype(np.uint32)
    words = np.zeros((E, N, K // 8), dtype=np.uint32)
    for i in range(8):
        words |= nib[..., i] << np.uint32(4 * i)
    return codes, scales, words


def _wire_from_codes(codes, scales):
    """GGUF mxfp4 blocks from sequential codes: scale byte, then code j | code j + 16 << 4 (src/kquant_cpu_decode.cpp
    :403-418 reads them back in that order)."""
    E, N, K = codes.shape
    c = codes.reshape(E, N, K // 32, 32)
    data = c[..., :16] | (c[..., 16:] << 4)
    return np.concatenate([scales[..., None], data], axis=-1).reshape(E, N, K // 32 * 17)


def _dense(codes, scales):
    """The stack's weights from the layout's definition: E2M1(code) * 2^(scale - 127)."""
    return E2M1[codes] * np.repeat(np.exp2(scales.astype(np.float32) - 127.0), 32, axis=-1)


def _dev_words(words):
    return torch.from_numpy(words.view(np.int32)).cuda()


def test_layout_converters(kq):
    E, N, K = 3, 40, 320
    codes, scales, words = _packed_stack(E, N, K, seed=1)
    want = _wire_from_codes(codes, scales)
    wire = kq.mxfp4_packed_to_wire(_dev_words(words), torch.from_numpy(scales).cuda())
    assert wire.dtype == torch.uint8 and tuple(wire.shape) == (E, N, K // 32 * 17)
    assert np.array_equal(wire.cpu().numpy(), want)
    # the wire decodes (oracle = reference decoder) to what the packed layout defines
    assert np.array_equal(O.dequantize(want, "mxfp4").reshape(E, N, K), _dense(codes, scales))
    back_w, back_s = kq.mxfp4_wire_to_packed(wire)
    assert np.array_equal(back_w.cpu().numpy().view(np.uint32), words) and np.array_equal(back_s.cpu().numpy(), scales)


@pytest.mark.parametrize("T,R", [(3, 2), (10, 4), (64, 4)])
def test_packed_ops_match_wire_oracle(kq, T, R):
    """Per-entry (up to 48 pairs) and batched paths; gpt-oss style biases, alpha = 1.702, limit = 7."""
    E, N, K = 4, 64, 576
    rng = np.random.default_rng(7)
    gc, gs, gw = _packed_stack(E, N, K, seed=2)
    uc, us, uw = _packed_stack(E, N, K, seed=3)
    gate, up = _wire_from_codes(gc, gs), _wire_from_codes(uc, us)
    gb = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    ub = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    idx = rng.integers(0, E, (T, R))
    idx_dev = torch.from_numpy(idx).cuda()
    xb, xt = make_x((T, K), "bfloat16", seed=8, scale=0.2)
    dev = lambda a: torch.from_numpy(a).cuda()
    got = kq.moe_glu_gather(xt, _dev_words(gw), dev(gs), dev(gb), _dev_words(uw), dev(us), dev(ub), idx_dev)
    want = O.moe_glu_gather(xb, gate, up, "mxfp4", idx, "swiglu_clamp", 7.0, gb, ub, 1.702, "bfloat16")
    assert tuple(got.shape) == (T, R, N) and got.dtype == torch.bfloat16
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL

    hb, ht = make_x((T, R, K), "bfloat16", seed=9, scale=0.2)
    got = kq.gather_qmv_bias(ht, _dev_words(gw), dev(gs), dev(gb), idx_dev)
    want = O.gather_qmv(hb, gate, "mxfp4", idx, gb, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL

    # routing mix with the bias inside: the definition in float64 on the oracle's decoded weights
    sc = rng.uniform(0.05, 1.0, (T, R)).astype(np.float32)
    got = kq.gather_qmv_mix_bias(ht, _dev_words(gw), dev(gs), dev(gb), idx_dev, dev(sc))
    wd = O.dequantize(gate, "mxfp4").reshape(E, N, K).astype(np.float64)
    hf = O.bits_to_f32(hb, "bfloat16").astype(np.float64)
    ref = np.stack([sum(sc[t, s] * (wd[idx[t, s]] @ hf[t, s] + gb[idx[t, s]]) for s in range(R)) for t in range(T)])
    assert tuple(got.shape) == (T, N)
    g = got.float().cpu().numpy().astype(np.float64)
    assert np.linalg.norm(g - ref) / np.linalg.norm(ref) <= 3e-3  # one bf16 rounding of the result


def test_mix_bias_matches_ns_op_with_zero_bias(kq):
    """With a zero bias the op is gather_qmv_mix_ns_kq on the converted stack, bit for bit."""
    E, N, K, T, S = 4, 64, 320, 5, 3
    codes, scales, words = _packed_stack(E, N, K, seed=4)
    rng = np.random.default_rng(5)
    idx = torch.from_numpy(rng.integers(0, E, (T, S))).cuda()
    sc = torch.from_numpy(rng.uniform(0.1, 1.0, (T, S)).astype(np.float32)).cuda()
    _, ht = make_x((T, S, K), "float16", seed=6, scale=0.2)
    a = kq.gather_qmv_mix_bias(ht, _dev_words(words), torch.from_numpy(scales).cuda(), torch.zeros((E, N), device="cuda"),
                               idx, sc)
    b = kq.gather_qmv_mix_ns_kq(ht, wire_to_dev(_wire_from_codes(codes, scales)), "mxfp4", idx, sc)
    assert torch.equal(a, b)


def test_packed_stack_wire_form_is_kept_and_follows_in_place_changes(kq):
    """By default every call converts the packed stack, so any write to it is seen.  With set_packed_cache(n) a
    stack's wire form is kept between calls: a second call gives the same bytes, an in-place change through torch
    ops is seen by the next call, a write that bypasses torch's version counters is seen after
    invalidate_packed_cache, and a call on another stream uses the kept form correctly."""
    E, N, K, T, R = 3, 64, 288, 5, 2
    rng = np.random.default_rng(17)
    gc, gs, gw = _packed_stack(E, N, K, seed=12)
    gb = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    idx = rng.integers(0, E, (T, R))
    idx_dev = torch.from_numpy(idx).cuda()
    hb, ht = make_x((T, R, K), "bfloat16", seed=19, scale=0.2)
    w_dev, s_dev, b_dev = _dev_words(gw), torch.from_numpy(gs).cuda(), torch.from_numpy(gb).cuda()

    def want(scales):
        return O.gather_qmv(hb, _wire_from_codes(gc, scales), "mxfp4", idx, gb, "bfloat16")

    # default: no cache, a write through .data (which torch's version counter does not see) changes the result
    base = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
    assert rel_l2(dev_to_bits(base), want(gs), "bfloat16") <= TOL
    s_dev.data.add_(1)
    bumped = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
    assert rel_l2(dev_to_bits(bumped), want(gs + 1), "bfloat16") <= TOL
    assert not torch.equal(bumped, base)
    s_dev.data.sub_(1)
    try:
        kq.set_packed_cache(8)
        first = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
        again = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
        assert torch.equal(first, again) and torch.equal(first, base)
        # a consumer on another stream waits for the conversion and reads the same bytes
        side = torch.cuda.Stream()
        other = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev, stream=side)
        side.synchronize()
        assert torch.equal(other, first)
        # double every weight of the stack in place (scale exponents + 1): the kept wire form must not be used
        s_dev.add_(1)
        changed = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
        assert rel_l2(dev_to_bits(changed), want(gs + 1), "bfloat16") <= TOL
        assert not torch.equal(changed, first)
        # a write the version counters miss needs the explicit call
        s_dev.data.add_(1)
        kq.invalidate_packed_cache(w_dev)
        reloaded = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
        assert rel_l2(dev_to_bits(reloaded), want(gs + 2), "bfloat16") <= TOL
        assert not torch.equal(reloaded, changed)
        # eviction at the entry limit keeps the results right
        kq.set_packed_cache(1)
        w2, s2 = w_dev.clone(), s_dev.clone()
        a2 = kq.gather_qmv_bias(ht, w2, s2, b_dev, idx_dev)
        a1 = kq.gather_qmv_bias(ht, w_dev, s_dev, b_dev, idx_dev)
        assert torch.equal(a1, reloaded) and torch.equal(a2, reloaded)
    finally:
        kq.set_packed_cache(0)
