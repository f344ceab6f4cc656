"""Host-side checks of the module layer (no GPU): attributes, placeholder shapes and validation follow
the reference's mlx_kquant/nn.py:50-368."""
import pytest
import torch

import kq.nn as knn
from kq.codec_geometry import bytes_per_row


def test_attributes_and_placeholder_shapes():
    lin = knn.KQuantLinear(512, 96, True, "q4_k")
    assert (lin.mode, lin.kquant_type, lin.group_size, lin.bits, lin.biases) == ("kquant", "q4_k", 256, 4, None)
    assert tuple(lin.weight.shape) == (96, 288) and lin.weight.dtype == torch.uint8
    assert tuple(lin.scales.shape) == (1,) and lin.scales.dtype == torch.uint8
    assert tuple(lin.bias.shape) == (96,)
    assert knn.KQuantLinear(512, 96, False, "q8_0").bias is None
    emb = knn.KQuantEmbedding(1000, 768, "q6_k")
    assert tuple(emb.weight.shape) == (1000, bytes_per_row("q6_k", 768)) and emb.out_dtype == torch.bfloat16
    sw = knn.KQuantSwitchLinear(8, 64, 256, True, "iq4_xs")
    assert tuple(sw.weight.shape) == (8, 64, 136) and tuple(sw.bias.shape) == (8, 64)
    ml = knn.KQuantMultiLinear(512, 128, 16, "q5_k")
    assert tuple(ml.weight.shape) == (16, 128, 352) and ml.num_heads == 16
    # wire bytes and bias are state (buffers), nothing is trainable
    assert set(lin.state_dict()) == {"weight", "scales", "bias"}
    assert list(lin.parameters()) == []
    assert "kquant_type=q4_k" in repr(lin) and "num_experts=8" in repr(sw)


def test_validation():
    with pytest.raises(ValueError):
        knn.KQuantLinear(500, 96, False, "q4_k")  # 500 is not a whole number of 256-weight blocks
    with pytest.raises(ValueError):
        knn.KQuantLinear(512, 96, False, "q9_k")
    lin = knn.KQuantLinear(512, 96, False, "q4_k")
    with pytest.raises(ValueError):
        lin.load_wire(torch.zeros((96, 144), dtype=torch.uint8))
    with pytest.raises(ValueError):
        lin.load_wire(torch.zeros((96, 288), dtype=torch.uint8), bias=torch.zeros(96))
    lin.load_wire(torch.ones((96, 288), dtype=torch.uint8))
    assert int(lin.state_dict()["weight"].sum()) == 96 * 288


def test_host_tile_maps():
    """64-row tiles per expert run, only the last partial, absent experts skipped (reference nn.py:33-47)."""
    m, cnt = knn._host_tile_maps([65, 0, 3, 128])
    assert m.dtype == torch.int32 and cnt.tolist() == [5]
    assert m.tolist() == [[0, 0, 64], [0, 64, 1], [2, 65, 3], [3, 68, 64], [3, 132, 64]]
    m, cnt = knn._host_tile_maps([0, 0])
    assert m.tolist() == [[0, 0, 0]] and cnt.tolist() == [0]


def test_gather_qmm_seg_rejects_bad_inputs():
    """Argument checks run before anything touches a device (reference tests/test_switch_gemm.py:293-319)."""
    import kq

    K, N = 512, 128
    x = torch.zeros((64, K), dtype=torch.float16)
    w = torch.zeros((2, N, 1056), dtype=torch.uint8)  # iq2_xxs bytes per row for K = 4096
    s = torch.zeros((1,), dtype=torch.uint8)
    good = torch.zeros((1, 3), dtype=torch.int32)
    cnt = torch.zeros((1,), dtype=torch.int32)
    with pytest.raises(ValueError):  # K mismatch
        kq.gather_qmm_seg(x, w, s, "iq2_xxs", good, cnt)
    x_ok = torch.zeros((64, 4096), dtype=torch.float16)
    with pytest.raises(ValueError):  # bad map shape
        kq.gather_qmm_seg(x_ok, w, s, "iq2_xxs", torch.zeros((3,), dtype=torch.int32), cnt)
    with pytest.raises(ValueError):  # bad counts shape
        kq.gather_qmm_seg(x_ok, w, s, "iq2_xxs", good, torch.zeros((2,), dtype=torch.int32))
    with pytest.raises(ValueError):  # 3-D x
        kq.gather_qmm_seg(torch.zeros((64, 1, 4096), dtype=torch.float16), w, s, "iq2_xxs", good, cnt)
    with pytest.raises(ValueError):  # float wire
        kq.gather_qmm_seg(x_ok, w.to(torch.float16), s, "iq2_xxs", good, cnt)
    with pytest.raises(ValueError):  # unknown codec
        kq.gather_qmm_seg(x_ok, w, s, "q9_k", good, cnt)
    with pytest.raises(ValueError):  # expert_tile_map: float indices
        kq.expert_tile_map(torch.zeros((8,), dtype=torch.float32), 4)
    with pytest.raises(ValueError):  # expert_tile_map: empty
        kq.expert_tile_map(torch.zeros((0,), dtype=torch.int32), 4)
    with pytest.raises(RuntimeError):  # valid arguments, but no device: there is no CPU path
        kq.gather_qmm_seg(x_ok, w, s, "iq2_xxs", good, cnt)
