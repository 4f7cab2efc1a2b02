"""torch.library registration of the CVMM path: operator schemas, fake implementations and
torch.compile traceability.  Everything here runs on ``meta`` tensors, which reach the operators' fake
implementations only (no kernel runs, no GPU needed); the GPU suite compares compiled and eager results."""
import pytest
import torch
import torch.nn.functional as F

from analog_moe_amd import config as cfgmod
from analog_moe_amd import ffn, library  # noqa: F401
from analog_moe_amd.cvmm import CVMM, AnalogExt, cvmm_prepare_sel2
from analog_moe_amd.moe_layer import AnalogSigmaMoELayer, MoEConifgError


def test_reference_operator_schema():
    """Same argument list as mylib::cvmm_triton_quantized (analog_moe/triton_src/cvmm.py:529)."""
    schema = str(torch.ops.amoe.cvmm_quantized.default._schema)
    assert schema == ("amoe::cvmm_quantized(Tensor x, Tensor sel_index, Tensor sel, Tensor keys, "
                      "Tensor input_ranges, float inp_res, ScalarType out_dtype, Tensor out_index, "
                      "Tensor abs_max, Tensor out_noise) -> Tensor")


def test_fake_of_reference_operator_has_sel_shape_plus_n():
    """cvmm.py:634-642: the abstract implementation returns [*sel.shape, N] in out_dtype."""
    m = dict(device="meta")
    x = torch.empty(3, 5, 32, **m)
    sel = torch.empty(3, 5, 2, dtype=torch.int32, **m)
    idx = torch.empty(30, dtype=torch.int32, **m)
    minus = torch.empty(1, **m)
    out = torch.ops.amoe.cvmm_quantized(x, idx, sel, torch.empty(4, 32, 8, **m), minus, 1 / 127, torch.bfloat16,
                                        idx, minus, minus)
    assert out.shape == (3, 5, 2, 8) and out.dtype == torch.bfloat16


def test_fake_shapes_of_the_fused_operators_and_their_autograd():
    m = dict(device="meta")
    T, D, E, Fs, k = 32, 64, 4, 16, 2
    x = torch.empty(T, D, requires_grad=True, **m)
    keys = torch.empty(E, D, Fs, requires_grad=True, **m)
    values = torch.empty(E, Fs, D, requires_grad=True, **m)
    ir = torch.empty(2, E, 2, requires_grad=True, **m)
    gate = torch.empty(T, k, requires_grad=True, **m)
    idx = torch.empty(T, k, dtype=torch.int64, **m)
    cfg = ffn.FFNConfig(inp_res=1 / 127, bounds_up=[0, 32, 64])
    y, p1, z, perm, in_index, offsets, z_scale = torch.ops.amoe.ffn_fwd(x, keys, values, ir, gate, idx,
                                                                        *ffn.cfg_astuple(cfg))
    assert y.shape == (T, D) and p1.shape == (T * k, Fs) and z.shape == (T * k, D) and z_scale.numel() == 0
    assert perm.shape == in_index.shape == (T * k,) and offsets.shape == (E + 1,) and perm.dtype == torch.int32
    y.sum().backward()
    for t in (x, keys, values, ir, gate):
        assert t.grad.shape == t.shape
    # bf16, 256 output columns, output quantiser, no injected noise: the k-head result is kept as ADC codes
    b = dict(device="meta", dtype=torch.bfloat16)
    xb, kb, vb = torch.empty(T, 256, **b), torch.empty(E, 256, 32, **b), torch.empty(E, 32, 256, **b)
    cfg = ffn.FFNConfig(inp_res=1 / 127, out_bound=12.0, out_res=254.0, noise_std=0.04)
    out = torch.ops.amoe.ffn_fwd(xb, kb, vb, torch.empty(2, E, 1, device="meta"), torch.empty(T, k, **b), idx,
                                 *ffn.cfg_astuple(cfg))
    assert out[2].dtype == torch.uint8 and out[2].shape == (T * k, 256) and out[6].shape == (E, 2)


def _analog_layer(fused: bool, noise: float = 0.04):
    r = cfgmod.TorchInferenceRPUConfig()
    r.forward.inp_res, r.forward.out_noise, r.forward.out_bound, r.forward.out_res = 254, noise, 12.0, 254
    r.pre_post.input_range.enable = True
    r.mapping.max_input_size = 32
    with torch.device("meta"):
        return AnalogSigmaMoELayer(r, d_model=64, n_experts=4, expert_size=16, k=2,
                                   activation=F.relu if fused else F.gelu)


@pytest.mark.parametrize("fused", [True, False])
def test_layer_traces_as_one_graph(fused):
    """fullgraph=True: the forward (router, sort, both projections, noise counter bump) and its backward
    contain nothing the tracer has to break the graph for."""
    torch._dynamo.reset()
    layer = _analog_layer(fused)
    assert layer._fusable() == fused
    layer.use_device_noise_counter()
    x = torch.empty(2, 16, 64, device="meta", requires_grad=True)
    y, reg = torch.compile(layer, backend="aot_eager", fullgraph=True)(x)
    (y.sum() + reg).backward()
    assert y.shape == (2, 16, 64) and x.grad.shape == x.shape
    assert layer.keys.grad.shape == layer.keys.shape and layer.input_range.grad.shape == (2, 4, 2)


def test_cvmm_apply_traces_as_one_graph():
    torch._dynamo.reset()
    m = dict(device="meta")
    E, D, Fs, k = 4, 64, 16, 2
    keys = torch.empty(E, D, Fs, requires_grad=True, **m)
    values = torch.empty(E, Fs, D, requires_grad=True, **m)
    gate = torch.empty(2, 16, k, requires_grad=True, **m)
    idx = torch.empty(2, 16, k, dtype=torch.int64, **m)
    x = torch.empty(2, 16, D, requires_grad=True, **m)
    irt = torch.empty(2, E, requires_grad=True, **m)

    def two_projections(x, keys, values, gate, idx, irt):
        s = cvmm_prepare_sel2(idx, E)
        ext = AnalogExt(offsets=s.offsets)
        h = CVMM.apply(x, s.sel_index, s.sel, keys, 1 / 127, irt[0][s.sel], s.out_index, None, None, None, None, ext)
        return CVMM.apply(F.relu(h), s.out_index, s.sel, values, 1 / 127, irt[1][s.sel], None, gate, None, None,
                          None, ext)

    y = torch.compile(two_projections, backend="aot_eager", fullgraph=True)(x, keys, values, gate, idx, irt)
    y.sum().backward()
    assert y.shape == (2, 16, D)
    for t in (x, keys, values, gate, irt):
        assert t.grad.shape == t.shape


def test_compiled_noisy_layer_needs_the_device_counter():
    """Without it the per-call seed would be a constant of the traced graph."""
    torch._dynamo.reset()
    layer = _analog_layer(True)
    x = torch.empty(2, 16, 64, device="meta")
    with pytest.raises(Exception) as info:
        torch.compile(layer, backend="aot_eager", fullgraph=True)(x)
    assert "use_device_noise_counter" in str(info.value)
    assert issubclass(MoEConifgError, Exception)
