"""Host-side behaviour of the layer classes that needs no GPU: constructor / rpu_config API,
state-dict keys and round trip (incl. the traceable layout of the reference's checkpoints),
tile bounds, error paths, C-ABI symbol table."""
import ctypes
import os
import re

import pytest
import torch

from analog_moe_amd import _abi, config as cfg
from analog_moe_amd.moe_layer import (AnalogSigmaMoELayer, AnalogSigmaMoELayerAIHWKIT, MoEConifgError, SigmaMoELayer,
                                      tile_bounds)

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
    assert set(sd) == {"keys", "values", "input_range", "input_range_update_idx", "expert_sel.weight",
                       "expert_sel.input_range", "expert_sel.input_range_update_idx"}     # the router is analog too
    digital_router = AnalogSigmaMoELayer(_rpu(), d_model=32, n_experts=4, expert_size=16, k=2, analog_router=False)
    assert set(digital_router.state_dict()) == {"keys", "values", "expert_sel.weight", "input_range",
                                                "input_range_update_idx"}
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


def test_state_dict_layout_conversion_round_trip():
    """moe_layer_aihwkit_lightning.py:33-105, both directions."""
    from analog_moe_amd.moe_layer import non_traceable_to_traceable, traceable_to_non_traceable
    layer = AnalogSigmaMoELayer(_rpu(), d_model=8, n_experts=3, expert_size=4, k=1, analog_router=False)
    layer.input_range.data = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    layer.input_range_update_idx.data.fill_(7.0)
    sd = {"blk." + k: v.clone() for k, v in layer.state_dict().items()}
    non_traceable_to_traceable(sd, "blk.")
    assert "blk.input_range" not in sd and "blk.input_range_update_idx" not in sd
    assert sd["blk.keys.1.input_range"].tolist() == [2.0] and sd["blk.values.2.input_range"].tolist() == [6.0]
    assert sd["blk.values.0.input_range_update_idx"].tolist() == [7.0] and sd["blk.keys.2.x_max"].tolist() == [0.0]
    assert len([k for k in sd if ".input_range" in k or ".x_m" in k]) == 3 * 2 * 4
    traceable_to_non_traceable(sd, "blk.")
    want = {"blk." + k: v for k, v in layer.state_dict().items()}
    assert sd.keys() == want.keys() and all(torch.equal(sd[k], want[k]) for k in want)
    split = _rpu()
    split.mapping.max_input_size = 4
    tiled = AnalogSigmaMoELayer(split, d_model=8, n_experts=2, expert_size=4, k=1, analog_router=False)
    with pytest.raises(MoEConifgError):
        non_traceable_to_traceable(dict(tiled.state_dict()))


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
    # the modifier and the clip are kernels: host tensors are refused, nothing is computed on the CPU
    w = torch.randn(3, 8, 5)
    m = cfg.WeightModifierParameter(type=cfg.WeightModifierType.DISCRETIZE_PER_CHANNEL, res=2 ** 4 - 2)
    with pytest.raises(MoEConifgError, match="GPU only"):
        AnalogSigmaMoELayer.modify_weight(w, m)
    assert AnalogSigmaMoELayer.modify_weight(w, cfg.WeightModifierParameter()) is w          # NONE: untouched
    with pytest.raises(MoEConifgError, match="not supported"):
        AnalogSigmaMoELayer.modify_weight(w, cfg.WeightModifierParameter(type=cfg.WeightModifierType.MULT_NORMAL))
    q = AnalogSigmaMoELayer.modify_weight(w.to("meta"), m)                                    # shape inference only
    assert q.is_meta and q.shape == w.shape
    layer = AnalogSigmaMoELayer(_rpu(), d_model=8, n_experts=3, expert_size=5, k=1)
    layer.rpu_config.clip.type = cfg.WeightClipType.LAYER_GAUSSIAN
    layer.rpu_config.clip.sigma = 1.0
    with pytest.raises(MoEConifgError, match="GPU only"):
        layer.post_update_step()
    layer.rpu_config.clip.type = cfg.WeightClipType.NONE
    layer.post_update_step()


def _aihwkit_rpu(**fw):
    r = cfg.AIHWKITTorchInferenceRPUConfig()
    r.forward.inp_res = 2 ** 8 - 2
    for k, v in fw.items():
        setattr(r.forward, k, v)
    r.pre_post.input_range.enable = True
    return r


def test_aihwkit_flavour_configuration_rules():
    """moe_layer_aihwkit.py:47-61 (constructor checks), :243-258 (is_perfect), :264-279 (remap type picks the
    max |W| behind the noise), cvmm.py:735-739 (abs-max follows the noise management)."""
    kw = dict(d_model=16, n_experts=3, expert_size=8, k=1)
    layer = AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(), **kw)
    assert isinstance(layer.rpu_config, cfg.AIHWKITTorchInferenceRPUConfig) and layer.input_range.shape == (2, 3)
    assert not layer._io_perfect() and not layer._row_abs_max_on() and layer._fusable()
    assert layer._noise_per_channel() is False                               # LAYERWISE_SYMMETRIC
    layer.rpu_config.remap.type = cfg.WeightRemapType.CHANNELWISE_SYMMETRIC
    assert layer._noise_per_channel() is True
    layer.rpu_config.remap.type = cfg.WeightRemapType.NONE
    assert layer._noise_per_channel() is True
    layer.rpu_config.forward.noise_management = cfg.NoiseManagementType.ABS_MAX
    assert layer._row_abs_max_on() and not layer._fusable()
    layer.rpu_config.forward.is_perfect = True
    assert layer._io_perfect() and not layer._row_abs_max_on()
    assert AnalogSigmaMoELayerAIHWKIT(None, **kw).input_range is None          # default config: ranges off
    with pytest.raises(AssertionError):
        AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(inp_bound=2.0), **kw)
    with pytest.raises(AssertionError):
        AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(bound_management="Iterative"), **kw)
    with pytest.raises(MoEConifgError):
        AnalogSigmaMoELayerAIHWKIT(_rpu(), **kw)                             # a lightning config: no is_perfect


def test_aihwkit_flavour_modifier_and_clip():
    """moe_layer_aihwkit.py:144-196 and :313-340."""
    torch.manual_seed(0)
    w = torch.randn(3, 64, 40)
    w[:, :, 0] *= 10
    M, R = cfg.WeightModifierParameter, cfg.WeightRemapType
    mod = AnalogSigmaMoELayerAIHWKIT.modify_weight
    assert mod(w, M(type=cfg.WeightModifierType.NONE), R.LAYERWISE_SYMMETRIC) is w
    assert mod(w, M(type=cfg.WeightModifierType.COPY), R.LAYERWISE_SYMMETRIC) is w
    add = M(type=cfg.WeightModifierType.ADD_NORMAL, std_dev=0.1)
    for bad in (M(type=cfg.WeightModifierType.MULT_NORMAL), M(type=cfg.WeightModifierType.DISCRETIZE),
                M(type=cfg.WeightModifierType.ADD_NORMAL, per_batch_sample=True)):
        with pytest.raises(MoEConifgError):
            mod(w, bad, R.LAYERWISE_SYMMETRIC)
    with pytest.raises(MoEConifgError):
        mod(w, add, R.NONE)
    with pytest.raises(MoEConifgError, match="GPU only"):
        mod(w, add, R.LAYERWISE_SYMMETRIC)
    layer = AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(), d_model=8, n_experts=3, expert_size=5, k=1)
    layer.rpu_config.clip = cfg.WeightClipParameter(type=cfg.WeightClipType.FIXED_VALUE, fixed_value=0.05)
    with pytest.raises(MoEConifgError, match="GPU only"):
        layer.post_update_step()
    with pytest.raises(NotImplementedError):
        layer.clip_weights(cfg.WeightClipParameter(type=cfg.WeightClipType.AVERAGE_CHANNEL_MAX))
    with pytest.raises(MoEConifgError):
        layer.clip_weights(cfg.WeightClipParameter(type=cfg.WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL))


def test_aihwkit_flavour_state_dict_carries_the_config():
    """moe_layer_aihwkit.py:372-436: ``analog_tile_state`` entry, load_rpu_config, compatibility check."""
    kw = dict(d_model=8, n_experts=3, expert_size=4, k=1)
    layer = AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(out_noise=0.07), **kw)
    sd = layer.state_dict()
    assert sd["analog_tile_state"]["rpu_config"] is layer.rpu_config
    assert set(sd) == {"keys", "values", "expert_sel.weight", "input_range", "input_range_update_idx",
                       "analog_tile_state"}
    other = AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(), **kw)
    other.load_state_dict(sd, load_rpu_config=True, strict_rpu_config_check=True)
    assert other.rpu_config.forward.out_noise == 0.07 and torch.equal(other.keys, layer.keys)
    assert "analog_tile_state" in sd                                         # the caller's dict is left alone
    keep = AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(), **kw)
    keep.load_state_dict(sd, load_rpu_config=False)
    assert keep.rpu_config.forward.out_noise == 0.0
    assert layer.compatible_with(cfg.AIHWKITTorchInferenceRPUConfig()) == (True, None)
    ok, msg = layer.compatible_with(object())
    assert ok                                                                # every class derives from object
    ok, msg = layer.compatible_with(3)
    assert not ok and "RPU config mismatch" in msg
    holder = torch.nn.Sequential(AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(out_noise=0.02), **kw))
    twin = torch.nn.Sequential(AnalogSigmaMoELayerAIHWKIT(_aihwkit_rpu(), **kw))
    twin.load_state_dict(holder.state_dict())
    assert twin[0].rpu_config.forward.out_noise == 0.02
    assert layer.get_dtype() == torch.float32


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


def test_library_rejects_bad_arguments_on_the_host():
    """Arguments are validated before anything is launched, so the documented codes of include/amoe.h come
    back from the built library without a GPU: NULL / size / shape / alignment / workspace errors."""
    path = os.path.join(ROOT, "analog_moe_amd", "csrc", "libamoe.so")
    if not os.path.exists(path):
        pytest.skip("libamoe.so has not been built")
    lib = _abi.bind(path)
    EINVAL, ENULL, ESHAPE, EALIGN, EWORKSPACE, EUNSUPPORTED = -1, -2, -3, -4, -5, -6
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)                                   # host memory: only ever looked at as an address
    assert lib.amoe_cvmm_fwd(None, None) == ENULL
    assert lib.amoe_cvmm_bwd_w(None, None) == ENULL
    assert lib.amoe_cvmm_bwd_x(None, None) == ENULL
    # selection
    assert lib.amoe_prepare_sel(p, 0, -1, 4, 2, p, p, p, p, None, p, 4096, None) == EINVAL
    assert lib.amoe_prepare_sel(p, 0, 16, 0, 2, p, p, p, p, None, p, 4096, None) == EINVAL
    assert lib.amoe_prepare_sel(p, 0, 16, 4096, 2, p, p, p, p, None, p, 4096, None) == EUNSUPPORTED
    assert lib.amoe_prepare_sel(None, 0, 16, 4, 2, p, p, p, p, None, p, 4096, None) == ENULL
    assert lib.amoe_prepare_sel(p, 0, 16, 4, 2, p + 2, p, p, p, None, p, 4096, None) == EALIGN
    assert lib.amoe_prepare_sel(p, 0, 16, 4, 2, p, p, p, p, None, p, 0, None) == EWORKSPACE
    assert lib.amoe_offsets_from_sorted(None, 8, 4, p, None) == ENULL
    # forward
    def fwd(**kw):
        a = _abi.FwdArgs(dtype=_abi.AMOE_F32, M=8, N=16, K=32, E=2, n_in_rows=8, n_out_rows=8, x=p, ldx=32, w=p,
                         w_stride_e=512, w_stride_k=16, w_stride_n=1, out=p, ldo=16, sel_sorted=p, offsets=p,
                         in_index=p, inp_res=-1.0, n_tiles=1, out_bound=-1.0, out_res=-1.0)
        a.tile_bounds[0], a.tile_bounds[1] = 0, 32
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    assert lib.amoe_cvmm_fwd(fwd(dtype=7), None) == EINVAL
    assert lib.amoe_cvmm_fwd(fwd(K=0), None) == EINVAL
    assert lib.amoe_cvmm_fwd(fwd(x=None), None) == ENULL
    assert lib.amoe_cvmm_fwd(fwd(ldx=16), None) == ESHAPE
    assert lib.amoe_cvmm_fwd(fwd(w_stride_k=3, w_stride_n=5), None) == EUNSUPPORTED
    assert lib.amoe_cvmm_fwd(fwd(n_tiles=0), None) == EINVAL
    assert lib.amoe_cvmm_fwd(fwd(n_tiles=_abi.AMOE_MAX_TILES + 1), None) == EINVAL
    bad = fwd()
    bad.tile_bounds[1] = 31                                     # the last bound must be K
    assert lib.amoe_cvmm_fwd(bad, None) == ESHAPE
    assert lib.amoe_cvmm_fwd(fwd(out_bound=12.0), None) == ESHAPE          # ADC without max |W|
    assert lib.amoe_cvmm_fwd(fwd(noise_std=0.1), None) == ESHAPE           # generated noise without max |W|
    assert lib.amoe_cvmm_fwd(fwd(xq_out=p), None) == EINVAL                # second output without its range
    assert lib.amoe_cvmm_fwd(fwd(x=p + 2), None) == EALIGN
    # gradients
    def bwd_w(**kw):
        a = _abi.BwdWArgs(dtype=_abi.AMOE_F32, M=8, N=16, K=32, E=2, x=p, ldx=32, g=p, ldg=16, grad_w=p, offsets=p,
                          in_index=p, n_x_rows=8, n_g_rows=8, n_tiles=1)
        a.tile_bounds[0], a.tile_bounds[1] = 0, 32
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    assert lib.amoe_cvmm_bwd_w(bwd_w(dtype=9), None) == EINVAL
    assert lib.amoe_cvmm_bwd_w(bwd_w(grad_w=None), None) == ENULL
    assert lib.amoe_cvmm_bwd_w(bwd_w(ldg=8), None) == ESHAPE
    def bwd_x(**kw):
        a = _abi.BwdXArgs(dtype=_abi.AMOE_F32, M=8, N=16, K=32, E=2, g=p, ldg=16, n_g_rows=8, w=p, w_stride_e=512,
                          w_stride_k=16, grad_x_full=p, ldo=32, offsets=p, g_index=p, out_index=p, n_tiles=1)
        a.tile_bounds[0], a.tile_bounds[1] = 0, 32
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    assert lib.amoe_cvmm_bwd_x(bwd_x(E=0), None) == EINVAL
    assert lib.amoe_cvmm_bwd_x(bwd_x(g_index=None), None) == ENULL
    assert lib.amoe_cvmm_bwd_x(bwd_x(relu_mask=1), None) == ENULL          # a mask needs the forward input
    assert lib.amoe_cvmm_bwd_x(bwd_x(ldo=16), None) == ESHAPE
    # companions
    assert lib.amoe_gate_reduce(_abi.AMOE_F32, p, None, p, 4, 2, 8, None, 0, None) == ENULL
    assert lib.amoe_gate_grad(5, p, p, p, 4, 2, 8, None) == EINVAL
    assert lib.amoe_row_abs_max(_abi.AMOE_F32, p, 4, 8, 16, p, None) == EINVAL          # ldx < K
    assert lib.amoe_weight_abs_max(_abi.AMOE_F32, p, 2, 8, 16, 3, p, None) == EINVAL   # cols is 1 or N
    assert lib.amoe_weight_abs_max_pair(_abi.AMOE_F32, p, 8, 16, p, p, 0, 8, p, 2, None) == EINVAL
    assert lib.amoe_weight_abs_max_pair(_abi.AMOE_F32, p, 8, 16, p, None, 16, 8, p, 2, None) == ENULL
    assert lib.amoe_weight_abs_max_pair(_abi.AMOE_F32, p, 8, 16, p + 2, p, 16, 8, p, 2, None) == EALIGN
    # the layer's four tables: the weight checks of the pair, then the input-range table's own
    F32 = _abi.AMOE_F32
    assert lib.amoe_layer_tables(F32, p, 8, 16, p, p, 16, 8, p, 2, 7, p, 2, 2, p, 1, p, None) == EINVAL      # ir dtype
    assert lib.amoe_layer_tables(F32, p, 8, 16, p, p, 16, 8, p, 2, F32, p, 2, 3, p, 1, p, None) == EINVAL    # n_up > columns
    assert lib.amoe_layer_tables(F32, p, 8, 16, p, p, 16, 8, p, 2, F32, p, 2, 2, None, 1, p, None) == ENULL
    assert lib.amoe_layer_tables(F32, p, 8, 16, p, p, 16, 8, p, 2, F32, p + 2, 2, 2, p, 1, p, None) == EALIGN
    assert lib.amoe_layer_tables(F32, p, 8, 16, None, p, 16, 8, p, 2, F32, p, 2, 2, p, 1, p, None) == ENULL
    # per-expert sums: output type, padding columns within the row stride
    assert lib.amoe_segment_sum(p, p, 2, 1, 5, p, 1, 0, None) == EINVAL                       # output dtype
    assert lib.amoe_segment_sum(p, p, 2, 1, F32, p, 1, 1, None) == EINVAL                     # padding beyond the row
    assert lib.amoe_segment_sum(p, p, 2, 1, F32, None, 2, 1, None) == ENULL
    assert lib.amoe_segment_sum(p, p, 2, 1, F32, p + 2, 2, 1, None) == EALIGN
    # the counter of the gate reductions is an 8-byte word
    assert lib.amoe_gate_reduce(F32, p, p, p, 4, 2, 8, p + 4, 1, None) == EALIGN
    assert lib.amoe_gate_reduce_codes(F32, p, p, p, 1, p, p, 4, 2, 16, p + 4, 1, None) == EALIGN
    # the codes question answers without launching
    assert lib.amoe_fwd_codes_supported(None) == 0
    assert lib.amoe_fwd_codes_supported(fwd()) == 0                                            # fp32, no ADC: values only
    # sum over the heads with the input-range clip
    def ksc(**kw):
        a = _abi.KsumClipArgs(dtype=_abi.AMOE_F32, T=4, k=2, D=32, E=2, full=p, x=p, ldx=32, sel=p, sel_is_i64=1,
                              perm=p, offsets=p, ir=p, n_tiles=1, grad_x=p, ir_grad=p, workspace=p,
                              workspace_bytes=8192)
        a.tile_bounds[0], a.tile_bounds[1] = 0, 32
        for k, v in kw.items():
            setattr(a, k, v)
        return a
    assert lib.amoe_ksum_clip(None, None) == ENULL
    assert lib.amoe_ksum_clip(ksc(dtype=5), None) == EINVAL
    assert lib.amoe_ksum_clip(ksc(k=0), None) == EINVAL
    assert lib.amoe_ksum_clip(ksc(T=0), None) == 0                                       # no tokens: nothing to do
    assert lib.amoe_ksum_clip(ksc(ir=None), None) == ENULL
    assert lib.amoe_ksum_clip(ksc(ldx=16), None) == ESHAPE
    assert lib.amoe_ksum_clip(ksc(x=p + 4), None) == EALIGN
    assert lib.amoe_ksum_clip(ksc(k=9), None) == EUNSUPPORTED                            # more than 8 heads
    two = ksc(n_tiles=2)
    two.tile_bounds[1], two.tile_bounds[2] = 18, 32                                      # a bound inside a 16-byte chunk
    assert lib.amoe_ksum_clip(two, None) == EUNSUPPORTED
    assert lib.amoe_ksum_clip(ksc(workspace_bytes=16), None) == EWORKSPACE
    assert lib.amoe_ksum_clip_workspace(4, 2, 1) >= 4 * 2 * 4
    # weight modifier / clip
    F = _abi.AMOE_F32
    assert lib.amoe_modify_weight(F, p, 2, 8, 16, p, 3, 14.0, 0.0, None, 1, 0, None, p, None) == EINVAL    # wmax cols
    assert lib.amoe_modify_weight(F, p, 2, 8, 16, None, 1, 14.0, 0.0, None, 1, 0, None, p, None) == ENULL
    assert lib.amoe_modify_weight(F, p, 2, 8, 16, p, 1, 14.0, 0.1, p + 2, 1, 0, None, p, None) == EALIGN
    assert lib.amoe_modify_weight(3, p, 2, 8, 16, p, 1, 14.0, 0.1, None, 1, 0, None, p, None) == EINVAL
    assert lib.amoe_weight_std_workspace(2, 8, 16, 1) > 0 and lib.amoe_weight_std_workspace(2, 8, 16, 16) > 0
    assert lib.amoe_weight_std(F, p, 2, 8, 16, 1, p, None, 0, None) == ENULL                # no workspace
    assert lib.amoe_weight_std(F, p, 2, 8, 16, 1, p, p, 8, None) == EWORKSPACE
    assert lib.amoe_weight_std(F, p, 0, 8, 16, 1, p, p, 4096, None) == EINVAL
    assert lib.amoe_clamp_weights(F, p, 2, 8, 16, None, 1, None) == ENULL
    assert lib.amoe_clamp_weights(F, p, 2, 8, 16, p, 5, None) == EINVAL
    # router epilogue
    assert lib.amoe_select_workspace(100, 64) >= 4 * 64
    assert lib.amoe_select_fwd(F, p, 8, 16, 17, p, p, None, None, None, 0, None) == EINVAL      # k > E
    assert lib.amoe_select_fwd(F, p, 8, 1024, 2, p, p, None, None, None, 0, None) == EUNSUPPORTED
    assert lib.amoe_select_fwd(F, p, 8, 16, 2, p, None, None, None, None, 0, None) == ENULL
    assert lib.amoe_select_fwd(F, p, 8, 16, 2, p, p, p, None, None, 0, None) == EINVAL          # reg without reg_c
    assert lib.amoe_select_fwd(F, p, 8, 16, 2, p, p, p, p, p, 4, None) == EWORKSPACE
    assert lib.amoe_select_fwd(F, p, 0, 16, 2, p, p, None, None, None, 0, None) == 0            # no rows: nothing to do
    assert lib.amoe_select_bwd(F, p, 8, 16, 2, None, p, None, None, p, None) == ENULL           # grad_val needs the ids
    assert lib.amoe_select_bwd(F, p, 8, 16, 2, p, p, p, None, p, None) == EINVAL                # reg_c without grad_reg
    for rc in (EINVAL, ENULL, ESHAPE, EALIGN, EWORKSPACE, EUNSUPPORTED):
        assert len(lib.amoe_strerror(rc)) > 0
