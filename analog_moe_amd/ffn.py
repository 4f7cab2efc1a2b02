"""Fused expert feed-forward of the analog SigmaMoE layer as ONE autograd function.

Same arithmetic as two CVMM calls with a ReLU between them (moe_layer_aihwkit_lightning.py:
384-410, 494-506; cvmm.py:699-897), with the glue folded into the kernels: the ReLU into the
up-projection's store and the down-projection's input gradient, the gate (x) dy outer product
into the weight-gradient loader, the per-position input-range gather into a per-expert table,
and the noise draw into the epilogue.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import ops


@dataclass
class FFNConfig:
    inp_res: float = -1.0                         # kernel step (1/127 for 8 bit); <= 0 off
    bounds_up: Optional[Sequence[int]] = None     # K-tile bounds of the up-projection
    bounds_down: Optional[Sequence[int]] = None
    out_bound: float = -1.0
    out_res: float = -1.0
    noise_std: float = 0.0                        # in-kernel noise, in units of max|W|
    noise_seed: int = 0
    noise_seed_dev: Optional[torch.Tensor] = None  # int64 device word added to the seed by the kernels
    noise_per_channel: bool = False
    gradient_relative: bool = True
    gradient_scale: float = 1.0
    decay: float = 0.0
    input_min_percentage: float = 0.95
    noise_up: Optional[torch.Tensor] = None       # injected noise [n_tiles, T*k, F] (parity runs)
    noise_down: Optional[torch.Tensor] = None
    wmax_up: Optional[torch.Tensor] = None        # max |W| behind noise and ADC when the weights passed in are
    wmax_down: Optional[torch.Tensor] = None      # modified copies (fp32 [E, 1] or [E, N]); None: taken from them
    seed_bump: int = 0                            # added to noise_seed_dev by the forward's last launch (eager calls
                                                  # only: not among the fields the opaque operators take)
    down_ready: Optional["torch.cuda.Event"] = None  # the down-projection's weights and wmax_down are made on another
                                                  # stream: the current one waits for this event before it reads them
                                                  # (eager calls only, as seed_bump)


_SIDE_STREAMS = {}


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority), for the bandwidth-bound companions."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return _SIDE_STREAMS[key]


CFG_FIELDS = ("inp_res", "bounds_up", "bounds_down", "out_bound", "out_res", "noise_std", "noise_seed",
              "noise_seed_dev", "noise_per_channel", "gradient_relative", "gradient_scale", "decay",
              "input_min_percentage", "noise_up", "noise_down", "wmax_up", "wmax_down")


def cfg_astuple(cfg: FFNConfig) -> tuple:
    """The configuration as positional values, in the order the ``amoe::ffn_fwd`` operator takes them."""
    return tuple(getattr(cfg, f) for f in CFG_FIELDS)


def _n_tiles(bounds) -> int:
    return 1 if bounds is None else len(bounds) - 1


def ir_tables(input_range: Optional[torch.Tensor], E: int, cfg: FFNConfig):
    """Per-expert input ranges of the two projections, fp32: [E, n_tiles_up], [E, n_tiles_down]."""
    if input_range is None:
        return None, None
    ir3 = input_range.detach().float().reshape(2, E, -1)
    return ir3[0, :, :_n_tiles(cfg.bounds_up)].contiguous(), ir3[1, :, :_n_tiles(cfg.bounds_down)].contiguous()


def ffn_forward(x, keys, values, input_range, gate, sel_idx, cfg: FFNConfig):
    """Sort, both projections and the gate reduction.  Returns (y, p1, z, perm, in_index, offsets, z_scale, ir_up,
    ir_dn): the result and what the backward pass reads again.  z is the down-projection's k-head result
    [T*k, D], either as values (z_scale empty) or as uint8 ADC codes with z_scale [E, 2] (``ops.dequant_codes``)."""
    T, D = x.shape
    E, _, F = keys.shape
    k = sel_idx.shape[-1]
    M = T * k
    gen = cfg.noise_std > 0 and cfg.noise_up is None
    wu = wd = ir_up = ir_dn = None
    main = torch.cuda.current_stream()
    if cfg.wmax_up is not None:
        wu, wd = cfg.wmax_up, cfg.wmax_down
        ir_up, ir_dn = ir_tables(input_range, E, cfg)
    elif cfg.out_bound > 0 or gen:
        # max |W| per expert and the fp32 input-range tables only read parameters: they run next to the expert
        # sort on a second stream
        side = _side_stream(x.device)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            if cfg.noise_per_channel:
                ir_up, ir_dn = ir_tables(input_range, E, cfg)
                wu = ops.weight_abs_max(keys, True)
                wd = ops.weight_abs_max(values, True)
            elif input_range is None:
                wu, wd = ops.weight_abs_max_pair(keys, values)
            else:                                # both max |W| tables and both fp32 range tables from two launches
                wu, wd, ir_up, ir_dn = ops.layer_tables(keys, values, input_range.reshape(2, E, -1),
                                                        _n_tiles(cfg.bounds_up), _n_tiles(cfg.bounds_down))
        for t in (wu, wd, ir_up, ir_dn):
            if t is not None:
                t.record_stream(main)
    else:
        ir_up, ir_dn = ir_tables(input_range, E, cfg)
    sel_sorted, perm, in_index, offsets = ops.prepare_sel(sel_idx, E, k)
    if wu is not None and cfg.wmax_up is None:
        main.wait_stream(side)
    common = dict(inp_res=cfg.inp_res, out_bound=cfg.out_bound, out_res=cfg.out_res,
                  noise_std=cfg.noise_std if gen else 0.0, ir_by_expert=ir_up is not None)
    # the up-projection also emits the down-projection's DAC image of its result (each row belongs
    # to one expert, so the image is made once instead of once per block of output columns)
    chain = ir_dn is not None and cfg.inp_res > 0 and _n_tiles(cfg.bounds_down) == 1
    p1 = ops.cvmm_fwd(x, keys, sel_sorted, offsets, in_index, perm, M, ir=ir_up, bounds=cfg.bounds_up,
                      noise=cfg.noise_up, noise_seed=cfg.noise_seed, wmax=wu, relu=True,
                      noise_seed_dev=cfg.noise_seed_dev, xq_ir=ir_dn[:, 0].contiguous() if chain else None,
                      xq_inp_res=cfg.inp_res, **common)
    p1, p1q = p1 if chain else (p1, None)
    if cfg.down_ready is not None:
        main.wait_event(cfg.down_ready)
    down = dict(ir=ir_dn, bounds=cfg.bounds_down, noise=cfg.noise_down, noise_seed=cfg.noise_seed + 1, wmax=wd,
                noise_seed_dev=cfg.noise_seed_dev, x_is_quantized=chain, **common)
    # the gate reduction follows the last launch that draws noise: it moves the device seed word on
    bump = (cfg.noise_seed_dev, cfg.seed_bump) if cfg.seed_bump and cfg.noise_seed_dev is not None else ()
    if chain and z_as_codes(p1q, values, cfg):
        # the down-projection's result is read twice more and never as a matrix operand (gate reduction now, gate
        # gradient in the backward pass): it is kept as its ADC codes, one byte per value, with two factors per expert
        z, z_scale = ops.cvmm_fwd(p1q, values, sel_sorted, offsets, perm, None, M, want_codes=True, **down)
        y = ops.gate_reduce_codes(z, z_scale, sel_idx, gate, *bump)
    else:
        z = ops.cvmm_fwd(p1q if chain else p1, values, sel_sorted, offsets, perm, None, M, **down)
        z_scale = torch.empty(0, dtype=torch.float32, device=x.device)
        y = ops.gate_reduce(z, gate, *bump)
    return y, p1, z, perm, in_index, offsets, z_scale, ir_up, ir_dn


def z_as_codes(p1q: torch.Tensor, values: torch.Tensor, cfg: FFNConfig) -> bool:
    """Whether the down-projection leaves its result as ADC codes (a pure function of shapes and settings)."""
    return ops.codes_supported(p1q, values, ir_by_expert=True, inp_res=cfg.inp_res, n_tiles=_n_tiles(cfg.bounds_down),
                               out_bound=cfg.out_bound, out_res=cfg.out_res, noise=cfg.noise_down,
                               per_channel=cfg.noise_per_channel)


def ffn_backward(dy, x, keys, values, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets, ir_up, ir_dn,
                 cfg: FFNConfig, want_ir_grad: bool, ir_dtype: torch.dtype = torch.float32):
    """Returns (grad_x, grad_keys, grad_values, grad_ir [2, E, n_tiles] of type ir_dtype or None, grad_gate)."""
    E = keys.shape[0]
    k = gate.shape[-1]
    M = perm.numel()
    dy = dy.contiguous()
    by = dict(ir_by_expert=ir_up is not None)
    irkw = dict(gradient_relative=cfg.gradient_relative, gradient_scale=cfg.gradient_scale, decay=cfg.decay,
                input_min_percentage=cfg.input_min_percentage)
    tok = in_index                               # token of each sorted position: perm // k, as the sort left it
    # the input gradient reads p1 for its masks anyway; it also leaves gate * clamp(p1), which is the
    # x operand of the weight gradient (otherwise every block of its output columns clips and scales)
    gp1, irg_dn, p1c = ops.cvmm_bwd_x(dy, values, offsets, tok, perm, M, x=p1, xf_index=perm, gate=gate,
                                      ir=ir_dn, bounds=cfg.bounds_down, relu_mask=True, want_xc=True,
                                      **irkw, **by)
    # the clip mask of the up-projection's input gradient depends on the token's input row, which its k heads
    # share: where the sum over the heads can apply it, the GEMM runs without a mask tile and x is read once per
    # token instead of once per head
    late_clip = ir_up is not None and ops.ksum_clip_supported(x, k, cfg.bounds_up)
    if late_clip:
        full, irg_up = ops.cvmm_bwd_x(gp1, keys, offsets, perm, perm, M)
    else:
        full, irg_up = ops.cvmm_bwd_x(gp1, keys, offsets, perm, perm, M, x=x, xf_index=in_index, ir=ir_up,
                                      bounds=cfg.bounds_up, **irkw, **by)
    # the gate gradient and the sum over the k heads only stream z, dy and the per-head input gradient
    # through HBM; they run on a second stream next to the two weight gradients.  With evenly loaded experts the
    # four launches take as long side by side as one after the other (together they are bound by memory traffic);
    # with uneven loads the streaming kernels fill the CUs that the weight gradients' last tiles leave idle
    # (2 - 3 % of the step)
    main, side = torch.cuda.current_stream(), _side_stream(x.device)
    side.wait_stream(main)
    with torch.cuda.stream(side):
        if z.dtype == torch.uint8:
            grad_gate = ops.gate_grad_codes(z, z_scale, sel_idx, dy, k).view(gate.shape)
        else:
            grad_gate = ops.gate_grad(z, dy, k).view(gate.shape)
        if late_clip:
            grad_x, irg_up = ops.ksum_clip(full, x, sel_idx, perm, offsets, ir_up, k, bounds=cfg.bounds_up, **irkw)
            irg_up.record_stream(main)
        else:
            grad_x = ops.ksum(full, k) if k > 1 else full
    grad_gate.record_stream(main)
    grad_x.record_stream(main)
    grad_ir = None
    if ir_up is not None and want_ir_grad:
        ntu, ntd = ir_up.shape[1], ir_dn.shape[1]
        # the two tables of per-expert sums are written where they belong, in the parameter's type, and each launch
        # clears the columns its projection does not have.  The down-projection's sums are issued here, where the
        # second stream keeps the GPU busy, instead of after the join at the end of the step
        nt = max(ntu, ntd)
        grad_ir = torch.empty((2, E, nt), dtype=ir_dtype, device=x.device)
        ops.segment_sum(irg_dn, offsets, E, out=grad_ir[1, :, :ntd], zero_cols=nt - ntd)
    grad_values = ops.cvmm_bwd_w(p1c, dy, E, offsets, perm, tok)
    grad_keys = ops.cvmm_bwd_w(x, gp1, E, offsets, in_index, perm, ir=ir_up, bounds=cfg.bounds_up, **by)
    main.wait_stream(side)
    if grad_ir is not None:
        ops.segment_sum(irg_up, offsets, E, out=grad_ir[0, :, :ntu], zero_cols=nt - ntu)
    return grad_x, grad_keys, grad_values, grad_ir, grad_gate


class AnalogMoEFFN(torch.autograd.Function):
    """y[t] = sum_j gate[t,j] * A(relu(A(x[t], keys[e_tj])), values[e_tj]).
    input_range: [2, E, n_tiles] (row 0 up-, row 1 down-projection) or None."""

    @staticmethod
    def forward(ctx, x, keys, values, input_range, gate, sel_idx, cfg: FFNConfig):
        y, p1, z, perm, in_index, offsets, z_scale, ir_up, ir_dn = ffn_forward(x, keys, values, input_range, gate,
                                                                               sel_idx, cfg)
        ctx.save_for_backward(x, keys, values, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets, ir_up, ir_dn)
        ctx.cfg = cfg
        ctx.ir_shape = None if input_range is None else input_range.shape
        ctx.ir_dtype = None if input_range is None else input_range.dtype
        return y

    @staticmethod
    def backward(ctx, dy):
        x, keys, values, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets, ir_up, ir_dn = ctx.saved_tensors
        grad_x, grad_keys, grad_values, grad_ir, grad_gate = ffn_backward(
            dy, x, keys, values, gate, sel_idx, p1, z, z_scale, perm, in_index, offsets, ir_up, ir_dn, ctx.cfg,
            ctx.needs_input_grad[3], ctx.ir_dtype or torch.float32)
        if grad_ir is not None:
            grad_ir = grad_ir.reshape(ctx.ir_shape)
        return grad_x, grad_keys, grad_values, grad_ir, grad_gate, None, None


def moe_ffn(x, keys, values, input_range, gate, sel_idx, cfg: FFNConfig) -> torch.Tensor:
    """The fused expert feed-forward.  Eagerly this is ``AnalogMoEFFN``; while ``torch.compile`` traces,
    the same two functions are reached through the opaque operators ``amoe::ffn_fwd`` / ``amoe::ffn_bwd``
    (their side streams and ctypes calls are nothing a tracer can follow)."""
    if torch.compiler.is_compiling():
        return torch.ops.amoe.ffn_fwd(x, keys, values, input_range, gate, sel_idx, *cfg_astuple(cfg))[0]
    return AnalogMoEFFN.apply(x, keys, values, input_range, gate, sel_idx, cfg)
