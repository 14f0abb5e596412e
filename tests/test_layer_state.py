"""Host logic of the decoder-layer module that needs no GPU: the calibration state
(`iteration`, `static_value`) travels with state_dict()."""
import pytest
import torch

import hyclora_amd  # noqa: F401
from hyclora_amd.models import FusedLlamaLayerIntra, FusedLlamaLayerIntraInterFullFuse


def test_extra_state_round_trip(tmp_path):
    layer = FusedLlamaLayerIntraInterFullFuse()
    sd = layer.state_dict()
    key = next(k for k in sd if k.endswith("_extra_state"))
    assert sd[key]["iteration"] == 0 and sd[key]["static_value"]["x"]["scale"] is None
    layer.iteration = 7
    layer.static_value["x"] = {"outlier_channel_index": torch.tensor([3, 9]),
                               "scale": torch.tensor([0.5, 0.25] * 8).to(torch.bfloat16)}
    layer.static_value["a"]["outlier"] = torch.tensor(0.125)
    torch.save(layer.state_dict(), tmp_path / "s.pt")
    other = FusedLlamaLayerIntraInterFullFuse()
    other.load_state_dict(torch.load(tmp_path / "s.pt", weights_only=True))
    assert other.iteration == 7
    assert torch.equal(other.static_value["x"]["scale"], layer.static_value["x"]["scale"])
    assert other.static_value["x"]["scale"].dtype == torch.bfloat16
    assert other.static_value["a"]["outlier"].item() == 0.125
    assert other.static_value["gate"]["scale"] is None
    # a copy, not an alias
    other.static_value["x"]["scale"].zero_()
    assert layer.static_value["x"]["scale"][0].item() == 0.5
    # dtype conversions of the module leave the statistics' formats alone
    layer.half()
    assert layer.static_value["x"]["scale"].dtype == torch.bfloat16
    assert layer.static_value["a"]["outlier"].dtype == torch.float32
    assert layer.static_value["x"]["outlier_channel_index"].dtype == torch.int64


def test_extra_state_of_another_layer_type_is_rejected():
    src = FusedLlamaLayerIntra()
    dst = FusedLlamaLayerIntraInterFullFuse()
    if set(src.static_value) == set(dst.static_value):
        pytest.skip("same statistics layout")
    with pytest.raises((ValueError, RuntimeError)):
        dst.load_state_dict(src.state_dict())


@pytest.mark.parametrize("channels", [[3, 16], [-1, 2], [5, 5]])
def test_extra_state_with_a_bad_channel_list_is_rejected(channels):
    """The kernels skip an out-of-range outlier channel and keep one copy of a repeated one, so a
    list that enters from a checkpoint is checked where it enters."""
    layer = FusedLlamaLayerIntraInterFullFuse()
    layer.static_value["x_medium"] = {"outlier_channel_index": torch.tensor(channels),
                                      "scale": torch.ones(16).to(torch.bfloat16)}
    state = layer.get_extra_state()
    with pytest.raises(ValueError, match="outlier channel"):
        FusedLlamaLayerIntraInterFullFuse().set_extra_state(state)
