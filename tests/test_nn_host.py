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
