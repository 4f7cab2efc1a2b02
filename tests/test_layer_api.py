"""Host-side behaviour of the layer classes that needs no GPU: constructor / rpu_config API,
state-dict keys and round trip (incl. the traceable layout of the reference's checkpoints),
tile bounds, error paths, C-ABI symbol table."""
import ctypes
import os
import re

import pytest
import torch

from analog_moe_amd import _abi, config as cfg
from analog_moe_amd.moe_layer import AnalogSigmaMoELayer, MoEConifgError, SigmaMoELayer, tile_bounds

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _rpu(learn=True, **fw):
    r = cfg.TorchInferenceRPUConfig()
    r.forward.inp_res = 2 ** 8 - 2
    for k, v in fw.items():
        setattr(r.forward, k, v)
    r.pre_post.input_range.enable = True
    r.pre_post.input_range.learn_input_range = learn
    r.pre_post.input_range.init_value = 3.0
    return r


def test_constructor_and_state_dict_keys():
    layer = AnalogSigmaMoELayer(_rpu(), d_model=32, n_experts=4, expert_size=16, k=2)
    assert layer.keys.shape == (4, 32, 16) and layer.values.shape == (4, 16, 32)
    assert layer.input_range.shape == (2, 4) and isinstance(layer.input_range, torch.nn.Parameter)
    sd = layer.state_dict()
    assert set(sd) == {"keys", "values", "expert_sel.weight", "input_range", "input_range_update_idx"}
    assert sd._metadata[""]["rpu_config"] is layer.rpu_config
    fixed = AnalogSigmaMoELayer(_rpu(learn=False), d_model=32, n_experts=4, expert_size=16, k=2)
    assert not isinstance(fixed.input_range, torch.nn.Parameter) and "input_range" in fixed.state_dict()
    other = AnalogSigmaMoELayer(_rpu(), d_model=32, n_experts=4, expert_size=16, k=2)
    layer.input_range.data[0, 1] = 7.0
    other.load_state_dict(sd)
    assert torch.equal(other.input_range, layer.input_range) and torch.equal(other.keys, layer.keys)


def test_loads_traceable_checkpoint_layout():
    layer = AnalogSigmaMoELayer(_rpu(), d_model=8, n_experts=3, expert_size=4, k=1)
    sd = {k: v.clone() for k, v in layer.state_dict().items()}
    sd.pop("input_range"); sd.pop("input_range_update_idx")
    for i in range(3):
        for name, row in (("keys", 0), ("values", 1)):
            sd[f"{name}.{i}.input_range"] = torch.tensor([1.0 + i + 10 * row])
            sd[f"{name}.{i}.input_range_update_idx"] = torch.tensor([5.0])
            sd[f"{name}.{i}.x_min"] = torch.zeros(1)
            sd[f"{name}.{i}.x_max"] = torch.zeros(1)
    layer.load_state_dict(sd)
    assert torch.equal(layer.input_range.data, torch.tensor([[1.0, 2.0, 3.0], [11.0, 12.0, 13.0]]))
    assert float(layer.input_range_update_idx) == 5.0


def test_tile_split_gives_per_tile_ranges():
    r = _rpu()
    r.mapping.max_input_size = 512
    layer = AnalogSigmaMoELayer(r, d_model=1024, n_experts=2, expert_size=256, k=1)
    assert layer.bounds_up == [0, 512, 1024] and layer.bounds_down is None
    assert layer.input_range.shape == (2, 2, 2)
    assert tile_bounds(10, 4) == [0, 4, 7, 10] and tile_bounds(412, 512) is None


def test_digital_round_trip_and_errors():
    dig = SigmaMoELayer(d_model=16, n_experts=2, expert_size=8, k=1, bias=True)
    ana = AnalogSigmaMoELayer.from_digital(dig, _rpu())
    assert torch.equal(ana.keys, dig.keys) and ana.bias is not None
    back = AnalogSigmaMoELayer.to_digital(ana)
    assert torch.equal(back.values, dig.values) and type(back) is SigmaMoELayer
    with pytest.raises(MoEConifgError):
        ana(torch.zeros(1, 2, 16))                    # CPU tensors: no CPU path
    with pytest.raises(MoEConifgError):
        SigmaMoELayer(d_model=16, n_experts=2, expert_size=8, k=1, traceable=True)


def test_inp_res_mapping_and_weight_modifier():
    assert cfg.kernel_inp_res(2 ** 8 - 2) == pytest.approx(1 / 127)
    assert cfg.kernel_inp_res(1 / (2 ** 8 - 2)) == pytest.approx(1 / 127)
    assert cfg.kernel_inp_res(-1) == -1
    w = torch.randn(3, 8, 5)
    m = cfg.WeightModifierParameter(type=cfg.WeightModifierType.DISCRETIZE_PER_CHANNEL, res=2 ** 4 - 2)
    q = AnalogSigmaMoELayer.modify_weight(w.clone(), m)
    step = w.abs().amax(1, keepdim=True) / 14
    assert torch.allclose(q / step, torch.round(q / step), atol=1e-4)
    m2 = cfg.WeightModifierParameter(type=cfg.WeightModifierType.ADD_NORMAL, std_dev=0.1)
    assert not torch.equal(AnalogSigmaMoELayer.modify_weight(w.clone(), m2), w)
    layer = AnalogSigmaMoELayer(_rpu(), d_model=8, n_experts=3, expert_size=5, k=1)
    layer.rpu_config.clip.type = cfg.WeightClipType.LAYER_GAUSSIAN
    layer.rpu_config.clip.sigma = 1.0
    before = layer.keys.data.abs().max().item()
    layer.post_update_step()
    assert layer.keys.data.abs().max().item() < before


def test_library_exports_every_declared_symbol():
    """Every function declared in include/amoe.h is exported by the built library and has a
    ctypes prototype (no compute call is made)."""
    so = os.path.join(ROOT, "analog_moe_amd", "csrc", "libamoe.so")
    if not os.path.exists(so):
        pytest.skip("libamoe.so not built")
    header = open(os.path.join(ROOT, "include", "amoe.h")).read()
    declared = set(re.findall(r"\b(amoe_[a-z_0-9]+)\s*\(", header))
    declared -= {"amoe_fwd_args", "amoe_bwd_w_args", "amoe_bwd_x_args"}
    assert declared == set(_abi.PROTOTYPES)
    raw = ctypes.CDLL(so)                      # loading needs the HIP runtime library, not a GPU
    for name in declared:
        assert hasattr(raw, name), name
    assert raw.amoe_version() == 100
    assert ctypes.sizeof(_abi.FwdArgs) % 8 == 0
