"""Host-side checks of arcquant_amd.layers that need no GPU: the module imports, its callers keep the
reference's names and argument order, and building a layer from CPU weights fails loudly."""
import inspect

import pytest
import torch
import torch.nn as nn

from arcquant_amd import layers


def test_qlinear_signature_follows_the_reference():
    # model/qLinearLayer.py:31-38
    params = list(inspect.signature(layers.QLinearLayer.__init__).parameters)
    assert params == ["self", "originalLayer", "select_num", "reorder_index", "out_reorder_index", "quant_type"]
    # model/qLlamaLayer.py:79
    params = list(inspect.signature(layers.reorder_quantize_x).parameters)
    assert params == ["x", "reorder_index", "select_num", "quant_type"]
    assert inspect.signature(layers.reorder_quantize_x).parameters["quant_type"].default == "NVFP4"


def test_tensor_scale_rule():
    t = torch.tensor([[-8.0, 2.0], [1.0, -0.5]])
    assert float(layers._tensor_scale(t, signed=False)) == pytest.approx(8.0 / 2688.0, rel=1e-7)   # max|x|
    assert float(layers._tensor_scale(t, signed=True)) == pytest.approx(2.0 / 2688.0, rel=1e-7)    # signed max
    assert float(layers._tensor_scale(torch.zeros(4), signed=False)) == 1.0


def test_cpu_weights_are_refused():
    lin = nn.Linear(64, 32, bias=False)
    with pytest.raises(RuntimeError, match="GPU"):
        layers.QLinearLayer(lin, 0, torch.arange(64))


def test_rotary_matches_closed_form():
    q = torch.zeros(1, 1, 3, 4)
    q[..., 0] = 1.0                                   # pairs (0, 2) and (1, 3) rotate together
    qe, _ = layers.rotary_pos_emb(q, q.clone(), beg=2)
    # position p, frequency 1 for the first pair: (1, 0) -> (cos p, sin p)
    for i, p in enumerate((2, 3, 4)):
        assert qe[0, 0, i, 0].item() == pytest.approx(torch.cos(torch.tensor(float(p))).item(), abs=1e-6)
        assert qe[0, 0, i, 2].item() == pytest.approx(torch.sin(torch.tensor(float(p))).item(), abs=1e-6)
