"""``torch.library`` registration of the CVMM path (namespace ``amoe::``).

The reference registers its forward launcher as ``mylib::cvmm_triton_quantized`` with an abstract
implementation (analog_moe/triton_src/cvmm.py:529-530, 634-642) so that ``torch.compile`` can trace
through ``CVMM``.  The HIP kernels here are reached through ctypes calls, which no tracer can follow,
so every group of calls the Python layer makes is one opaque operator with a fake implementation:

  amoe::cvmm_quantized      the reference's operator, same schema and sentinel convention
  amoe::prepare_sel         expert sort                       (cvmm.py:31-34)
  amoe::offsets_from_sorted segment starts from sorted ids
  amoe::expert_std          per-expert std                    (cvmm.py:400-443)
  amoe::weight_abs_max      max |W| per expert / per channel  (moe_layer_aihwkit_lightning.py:476-489)
  amoe::modify_weight       weight modifier of a forward      (moe_layer_aihwkit_lightning.py:313-382)
  amoe::select / select_bwd sigmoid + top-k + usage regulariser of the router's logits
  amoe::cvmm_forward        everything CVMM.forward launches  (cvmm.py:701-769)
  amoe::cvmm_backward       everything CVMM.backward launches (cvmm.py:772-897)
  amoe::ffn_fwd / ffn_bwd   the fused expert feed-forward, with its autograd formula registered

Operators return an empty tensor where the Python interface returns ``None``.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import Tensor

from . import ffn, ops

_EMPTY_SHAPE = (0,)


def _none_if_empty(t: Tensor) -> Optional[Tensor]:
    return None if t.numel() == 0 else t


# --------------------------------------------------------------------------- the reference's operator
def _is_sentinel(t: Tensor, expected_numel: int) -> bool:
    """cvmm.py:583-598: a one-element tensor holding -1 stands for "absent".  A one-element tensor where
    more elements are expected can only be the sentinel, which avoids reading device memory."""
    if t.numel() != 1:
        return False
    if expected_numel != 1:
        return True
    return bool(t.reshape(()) == -1)


@torch.library.custom_op(
    "amoe::cvmm_quantized", mutates_args=(),
    schema="(Tensor x, Tensor sel_index, Tensor sel, Tensor keys, Tensor input_ranges, float inp_res, "
           "ScalarType out_dtype, Tensor out_index, Tensor abs_max, Tensor out_noise) -> Tensor")
def cvmm_quantized(x, sel_index, sel, keys, input_ranges, inp_res, out_dtype, out_index, abs_max, out_noise):
    """cvmm.py:531-631 on the HIP kernel: out[out_index[i]] = Q(x[sel_index[i]]) @ keys[sel[i]] (+ noise),
    shaped [*sel.shape, N].  ``sel`` holds the sorted expert ids."""
    x2 = x.flatten(end_dim=-2)
    if x2.shape[-1] != keys.shape[1]:
        raise RuntimeError("cvmm_quantized: x and keys disagree on the contraction size")
    if out_dtype != x2.dtype:
        x2 = x2.to(out_dtype)
    w = keys if keys.dtype == x2.dtype else keys.to(x2.dtype)
    ssel = sel.reshape(-1).to(torch.int32)
    M, N = ssel.numel(), keys.shape[2]
    offsets = ops.offsets_from_sorted(ssel, keys.shape[0])
    oi = None if _is_sentinel(out_index, M) else out_index.reshape(-1).to(torch.int32)
    ir = None if _is_sentinel(input_ranges, M) else input_ranges.reshape(M, 1)
    am = None if _is_sentinel(abs_max, x2.shape[0]) else abs_max.reshape(-1)
    noise = None
    if not _is_sentinel(out_noise, M * N):
        noise = out_noise.reshape(1, M, N)
    out = ops.cvmm_fwd(x2, w, ssel, offsets, sel_index.reshape(-1).to(torch.int32), oi, M, ir=ir, abs_max=am,
                       inp_res=float(inp_res), noise=noise)
    return out.view(*sel.shape, N)


@cvmm_quantized.register_fake
def _(x, sel_index, sel, keys, input_ranges, inp_res, out_dtype, out_index, abs_max, out_noise):
    return x.new_empty((*sel.shape, keys.shape[2]), dtype=out_dtype)        # cvmm.py:634-642


# --------------------------------------------------------------------------- selection and companions
@torch.library.custom_op("amoe::prepare_sel", mutates_args=(),
                         schema="(Tensor sel, int n_experts, int k) -> (Tensor, Tensor, Tensor, Tensor)")
def prepare_sel(sel, n_experts, k):
    return ops.prepare_sel(sel, n_experts, k)


@prepare_sel.register_fake
def _(sel, n_experts, k):
    M = sel.numel()
    i32 = dict(dtype=torch.int32, device=sel.device)
    return (torch.empty(M, **i32), torch.empty(M, **i32), torch.empty(M, **i32),
            torch.empty(n_experts + 1, **i32))


@torch.library.custom_op("amoe::offsets_from_sorted", mutates_args=(),
                         schema="(Tensor sel_sorted, int n_experts) -> Tensor")
def offsets_from_sorted(sel_sorted, n_experts):
    return ops.offsets_from_sorted(sel_sorted, n_experts)


@offsets_from_sorted.register_fake
def _(sel_sorted, n_experts):
    return torch.empty(n_experts + 1, dtype=torch.int32, device=sel_sorted.device)


@torch.library.custom_op("amoe::expert_std", mutates_args=(),
                         schema="(Tensor x, Tensor in_index, Tensor offsets, int n_experts) -> Tensor")
def expert_std(x, in_index, offsets, n_experts):
    return ops.expert_std(x, in_index, offsets, n_experts)


@expert_std.register_fake
def _(x, in_index, offsets, n_experts):
    return torch.empty(n_experts, dtype=torch.float32, device=x.device)


@torch.library.custom_op("amoe::weight_abs_max", mutates_args=(), schema="(Tensor w, bool per_channel) -> Tensor")
def weight_abs_max(w, per_channel):
    return ops.weight_abs_max(w, per_channel)


@weight_abs_max.register_fake
def _(w, per_channel):
    return torch.empty((w.shape[0], w.shape[2] if per_channel else 1), dtype=torch.float32, device=w.device)


@torch.library.custom_op(
    "amoe::modify_weight", mutates_args=(),
    schema="(Tensor w, bool per_channel, float n_states, float std_dev, Tensor? noise, bool round_noise, "
           "int noise_seed, Tensor? noise_seed_dev) -> Tensor")
def modify_weight(w, per_channel, n_states, std_dev, noise, round_noise, noise_seed, noise_seed_dev):
    """The weight modifier of a training forward (moe_layer_aihwkit_lightning.py:313-382): a copy of
    w [E, K, N] discretised to max |W| / n_states steps and / or with std_dev * max |W| * normal added."""
    wmax = ops.weight_abs_max(w, per_channel)
    return ops.modify_weight(w, wmax, n_states, std_dev, noise, round_noise, noise_seed, noise_seed_dev)


@modify_weight.register_fake
def _(w, per_channel, n_states, std_dev, noise, round_noise, noise_seed, noise_seed_dev):
    return torch.empty(w.shape, dtype=w.dtype, device=w.device)


def _modify_autograd(ctx, grad):
    # straight-through quantiser, noise without gradient (moe_layer_aihwkit_lightning.py:362-377)
    return (grad,) + (None,) * 7


modify_weight.register_autograd(_modify_autograd)


# --------------------------------------------------------------------------- router epilogue
@torch.library.custom_op("amoe::select", mutates_args=(),
                         schema="(Tensor logits, int k, bool want_reg) -> (Tensor, Tensor, Tensor, Tensor)")
def select(logits, k, want_reg):
    """(sel_val [T, k], sel_idx [T, k] int64, reg, reg_c): sigmoid gate values and ids of the top-k experts per
    row of logits [T, E], and the usage regulariser with its derivative table (empty without want_reg)."""
    return ops.select_fwd(logits, k, want_reg)


@select.register_fake
def _(logits, k, want_reg):
    T, E = logits.shape
    f32 = dict(dtype=torch.float32, device=logits.device)
    return (logits.new_empty((T, k)), torch.empty((T, k), dtype=torch.int64, device=logits.device),
            torch.empty((), **f32) if want_reg else torch.empty(_EMPTY_SHAPE, **f32),
            torch.empty(E if want_reg else 0, **f32))


@torch.library.custom_op("amoe::select_bwd", mutates_args=(),
                         schema="(Tensor logits, Tensor sel_idx, Tensor? grad_val, Tensor? reg_c, Tensor? grad_reg) -> Tensor")
def select_bwd(logits, sel_idx, grad_val, reg_c, grad_reg):
    return ops.select_bwd(logits, sel_idx, grad_val, reg_c, grad_reg)


@select_bwd.register_fake
def _(logits, sel_idx, grad_val, reg_c, grad_reg):
    return torch.empty_like(logits)


def _select_setup_context(ctx, inputs, output):
    logits, k, want_reg = inputs
    _, sel_idx, _, reg_c = output
    ctx.save_for_backward(logits, sel_idx, reg_c)
    ctx.want_reg = want_reg
    ctx.set_materialize_grads(False)


def _select_autograd(ctx, grad_val, _grad_idx, grad_reg, _grad_c):
    logits, sel_idx, reg_c = ctx.saved_tensors
    if grad_val is None and (grad_reg is None or not ctx.want_reg):
        return None, None, None
    with_reg = ctx.want_reg and grad_reg is not None
    return (torch.ops.amoe.select_bwd(logits, sel_idx, grad_val, reg_c if with_reg else None,
                                      grad_reg if with_reg else None), None, None)


select.register_autograd(_select_autograd, setup_context=_select_setup_context)


# --------------------------------------------------------------------------- CVMM forward / backward
@torch.library.custom_op(
    "amoe::cvmm_forward", mutates_args=(),
    schema="(Tensor x, Tensor keys, Tensor sel_sorted, Tensor offsets, Tensor sel_index, Tensor? out_index, "
           "Tensor? gate, Tensor? ir, Tensor? noise, bool use_abs_max, float inp_res, int[]? bounds, "
           "Tensor? wmax, float out_bound, float out_res, float noise_std, int noise_seed, "
           "Tensor? noise_seed_dev) -> (Tensor, Tensor)")
def cvmm_forward(x, keys, sel_sorted, offsets, sel_index, out_index, gate, ir, noise, use_abs_max, inp_res,
                 bounds, wmax, out_bound, out_res, noise_std, noise_seed, noise_seed_dev):
    """Returns (result, z): with a gate, z [M, N] is the per-head product and the result [M / k, N] its
    gate-weighted sum over the heads (cvmm.py:757-759); without one the result is [M, N] and z is empty."""
    M = sel_sorted.numel()
    abs_max = ops.row_abs_max(x) if use_abs_max else None
    res = ops.cvmm_fwd(x, keys, sel_sorted, offsets, sel_index, out_index, M, ir=ir, abs_max=abs_max,
                       inp_res=inp_res, bounds=bounds, noise=noise, noise_std=noise_std, noise_seed=noise_seed,
                       noise_seed_dev=noise_seed_dev, wmax=wmax, out_bound=out_bound, out_res=out_res)
    if gate is None:
        return res, res.new_empty(_EMPTY_SHAPE)
    return ops.gate_reduce(res, gate), res


@cvmm_forward.register_fake
def _(x, keys, sel_sorted, offsets, sel_index, out_index, gate, ir, noise, use_abs_max, inp_res, bounds, wmax,
      out_bound, out_res, noise_std, noise_seed, noise_seed_dev):
    M, N = sel_sorted.numel(), keys.shape[2]
    if gate is None:
        return x.new_empty((M, N)), x.new_empty(_EMPTY_SHAPE)
    return x.new_empty((M // gate.shape[-1], N)), x.new_empty((M, N))


@torch.library.custom_op(
    "amoe::cvmm_backward", mutates_args=(),
    schema="(Tensor grad_output, Tensor x, Tensor keys, Tensor offsets, Tensor sel_index, Tensor? out_index, "
           "Tensor? gate, Tensor? ir, Tensor? z, int[]? bounds, bool gradient_relative, float gradient_scale, "
           "float decay, float input_min_percentage) -> (Tensor, Tensor, Tensor, Tensor)")
def cvmm_backward(grad_output, x, keys, offsets, sel_index, out_index, gate, ir, z, bounds, gradient_relative,
                  gradient_scale, decay, input_min_percentage):
    """Returns (grad_x like x, grad_w [E, K, N], ir_grad [M, n_tiles] fp32 or empty, grad_gate or empty)."""
    E, K, N = keys.shape
    M = sel_index.numel()
    grad_output = grad_output.to(x.dtype).contiguous()
    pos_out = sel_index if out_index is None else out_index                     # cvmm.py:828
    irkw = {}
    if ir is not None:
        irkw = dict(gradient_relative=gradient_relative, gradient_scale=gradient_scale, decay=decay,
                    input_min_percentage=input_min_percentage)
    if gate is not None:
        k = gate.shape[-1]
        g_rows = torch.div(pos_out, k, rounding_mode="floor").to(torch.int32)    # cvmm.py:833
        grad_w = ops.cvmm_bwd_w(x, grad_output, E, offsets, sel_index, g_rows, ir=ir, bounds=bounds,
                                g_scale=gate)                                    # cvmm.py:785-789, 812-823
        full, ir_grad = ops.cvmm_bwd_x(grad_output, keys, offsets, g_rows, pos_out, M, x=x, xf_index=sel_index,
                                       gate=gate, ir=ir, bounds=bounds, **irkw)
        grad_x = full.view(x.shape)                                              # cvmm.py:888
        grad_gate = ops.gate_grad(z, grad_output, k).view(gate.shape).to(gate.dtype)   # cvmm.py:889
    else:
        grad_w = ops.cvmm_bwd_w(x, grad_output, E, offsets, sel_index, out_index, ir=ir, bounds=bounds)
        full, ir_grad = ops.cvmm_bwd_x(grad_output, keys, offsets, pos_out, pos_out, M, x=x, xf_index=sel_index,
                                       ir=ir, bounds=bounds, **irkw)
        k = M // max(x.reshape(-1, K).shape[0], 1)
        grad_x = (ops.ksum(full, k) if k > 1 else full).view(x.shape)            # cvmm.py:890-893
        grad_gate = x.new_empty(_EMPTY_SHAPE)
    if ir_grad is None:
        ir_grad = torch.empty(_EMPTY_SHAPE, dtype=torch.float32, device=x.device)
    return grad_x, grad_w, ir_grad, grad_gate


@cvmm_backward.register_fake
def _(grad_output, x, keys, offsets, sel_index, out_index, gate, ir, z, bounds, gradient_relative, gradient_scale,
      decay, input_min_percentage):
    n_tiles = 1 if bounds is None else len(bounds) - 1
    f32 = dict(dtype=torch.float32, device=x.device)
    ir_grad = torch.empty((sel_index.numel(), n_tiles), **f32) if ir is not None else torch.empty(_EMPTY_SHAPE, **f32)
    grad_gate = torch.empty_like(gate) if gate is not None else x.new_empty(_EMPTY_SHAPE)
    return torch.empty_like(x), x.new_empty(tuple(keys.shape)), ir_grad, grad_gate


# --------------------------------------------------------------------------- fused expert feed-forward
_CFG_SCHEMA = ("float inp_res, int[]? bounds_up, int[]? bounds_down, float out_bound, float out_res, "
               "float noise_std, int noise_seed, Tensor? noise_seed_dev, bool noise_per_channel, "
               "bool gradient_relative, float gradient_scale, float decay, float input_min_percentage, "
               "Tensor? noise_up, Tensor? noise_down, Tensor? wmax_up, Tensor? wmax_down")
_N_CFG = len(ffn.CFG_FIELDS)


def _cfg(values) -> ffn.FFNConfig:
    return ffn.FFNConfig(**dict(zip(ffn.CFG_FIELDS, values)))


@torch.library.custom_op(
    "amoe::ffn_fwd", mutates_args=(),
    schema="(Tensor x, Tensor keys, Tensor values, Tensor? input_range, Tensor gate, Tensor sel_idx, "
           + _CFG_SCHEMA + ") -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)")
def ffn_fwd(x, keys, values, input_range, gate, sel_idx, *cfg):
    """(y, p1, z, perm, in_index, offsets, z_scale): the result and what ``amoe::ffn_bwd`` reads again."""
    return ffn.ffn_forward(x, keys, values, input_range, gate, sel_idx, _cfg(cfg))[:7]


@ffn_fwd.register_fake
def _(x, keys, values, input_range, gate, sel_idx, *cfg):
    T, k = x.shape[0], sel_idx.shape[-1]
    M = T * k
    i32 = dict(dtype=torch.int32, device=x.device)
    c = _cfg(cfg)
    E, F, D = values.shape
    # (the same decision ffn_forward makes: a function of shapes and settings only)
    chain = input_range is not None and c.inp_res > 0 and (c.bounds_down is None or len(c.bounds_down) == 2)
    codes = chain and ffn.z_as_codes(x.new_empty((M, F)), values, c)
    z = torch.empty((M, D), dtype=torch.uint8, device=x.device) if codes else x.new_empty((M, D))
    z_scale = torch.empty((E, 2) if codes else (0,), dtype=torch.float32, device=x.device)
    return (x.new_empty((T, D)), x.new_empty((M, keys.shape[2])), z,
            torch.empty(M, **i32), torch.empty(M, **i32), torch.empty(E + 1, **i32), z_scale)


@torch.library.custom_op(
    "amoe::ffn_bwd", mutates_args=(),
    schema="(Tensor dy, Tensor x, Tensor keys, Tensor values, Tensor? input_range, Tensor gate, Tensor sel_idx, "
           "Tensor p1, Tensor z, Tensor z_scale, Tensor perm, Tensor in_index, Tensor offsets, bool want_ir_grad, "
           + _CFG_SCHEMA + ") -> (Tensor, Tensor, Tensor, Tensor, Tensor)")
def ffn_bwd(dy, x, keys, values, input_range, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets, want_ir_grad,
            *cfg):
    """(grad_x, grad_keys, grad_values, grad_input_range or empty, grad_gate)."""
    c = _cfg(cfg)
    ir_up, ir_dn = ffn.ir_tables(input_range, keys.shape[0], c)
    gx, gk, gv, gir, gg = ffn.ffn_backward(dy, x, keys, values, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets,
                                           ir_up, ir_dn, c, want_ir_grad,
                                           torch.float32 if input_range is None else input_range.dtype)
    if gir is None:
        gir = torch.empty(_EMPTY_SHAPE, dtype=torch.float32, device=x.device)
    else:
        gir = gir.reshape(input_range.shape)
    return gx, gk, gv, gir, gg


@ffn_bwd.register_fake
def _(dy, x, keys, values, input_range, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets, want_ir_grad, *cfg):
    if input_range is not None and want_ir_grad:
        gir = torch.empty_like(input_range)
    else:
        gir = torch.empty(_EMPTY_SHAPE, dtype=torch.float32, device=x.device)
    return torch.empty_like(x), torch.empty_like(keys), torch.empty_like(values), gir, torch.empty_like(gate)


def _ffn_setup_context(ctx, inputs, output):
    x, keys, values, input_range, gate, sel_idx = inputs[:6]
    _, p1, z, perm, in_index, offsets, z_scale = output
    ctx.save_for_backward(x, keys, values, input_range, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets)
    ctx.cfg = tuple(inputs[6:])
    ctx.want_ir_grad = input_range is not None and ctx.needs_input_grad[3]
    ctx.set_materialize_grads(False)


def _ffn_autograd(ctx, dy, *_unused):
    x, keys, values, input_range, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets = ctx.saved_tensors
    if dy is None:
        return (None,) * (6 + _N_CFG)
    gx, gk, gv, gir, gg = torch.ops.amoe.ffn_bwd(dy, x, keys, values, input_range, gate, sel_idx, p1, z, z_scale, perm,
                                                 in_index, offsets, ctx.want_ir_grad, *ctx.cfg)
    return (gx, gk, gv, gir if ctx.want_ir_grad else None, gg, None) + (None,) * _N_CFG


ffn_fwd.register_autograd(_ffn_autograd, setup_context=_ffn_setup_context)
