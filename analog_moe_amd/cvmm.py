"""The reference's CVMM operator interface on the HIP kernels.

Same names, argument order and return structure as analog_moe/triton_src/cvmm.py:
``CVMMSel`` (:19-28), ``cvmm_prepare_sel`` (:31-34), ``cvmm_std`` (:400-443) and the autograd
function ``CVMM`` (:699-897, 11 positional arguments).  One optional 12th argument carries what
the reference asserts off or produces elsewhere (K-tile split, ADC, in-kernel noise, segment
offsets); leaving it out gives the reference's behaviour.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import library  # noqa: F401  (registers the amoe:: operators used below)
from .config import enum_name


@dataclass
class CVMMSel:
    raw_sel: torch.Tensor                        # [..., k] expert ids as the router chose them
    sel: torch.Tensor                            # [..., k] ids sorted ascending (flat order)
    sel_index: torch.Tensor                      # [M] input row of each sorted position
    out_index: Optional[torch.Tensor] = None     # [M] output row of each sorted position
    reduction_weight: Optional[torch.Tensor] = None  # [..., k] gate values
    offsets: Optional[torch.Tensor] = None       # [E+1] segment starts (not in the reference)

    def clone(self) -> "CVMMSel":
        return CVMMSel(self.raw_sel, self.sel, self.sel_index, self.out_index, self.reduction_weight,
                       self.offsets)


def cvmm_prepare_sel(sel: torch.Tensor, n_experts: int) -> CVMMSel:
    """cvmm.py:31-34: sorted ids and the permutation; ties keep ascending flat index."""
    ssel, perm, _, offsets = torch.ops.amoe.prepare_sel(sel, n_experts, 1)
    return CVMMSel(sel, ssel.view(sel.shape), perm, None, None, offsets)


def cvmm_prepare_sel2(sel: torch.Tensor, n_experts: int, w: Optional[torch.Tensor] = None) -> CVMMSel:
    """Selection record of a k-head layer as the up-projection uses it: ``sel_index = perm // k``
    (token row), ``out_index = perm`` (cvmm.py:196-205, 828-833)."""
    k = sel.shape[-1]
    ssel, perm, in_index, offsets = torch.ops.amoe.prepare_sel(sel, n_experts, k)
    return CVMMSel(sel, ssel.view(sel.shape), in_index, perm, w, offsets)


def cvmm_std(x: torch.Tensor, sel_index: torch.Tensor, sel: torch.Tensor, n_experts: int) -> torch.Tensor:
    """Per-expert unbiased std of the routed rows' elements (cvmm.py:400-443)."""
    ssel = sel.reshape(-1).to(torch.int32)
    offsets = torch.ops.amoe.offsets_from_sorted(ssel, n_experts)
    return torch.ops.amoe.expert_std(x, sel_index.to(torch.int32), offsets, n_experts).to(x.dtype)


@dataclass
class AnalogExt:
    """What the reference does not pass to CVMM.apply."""
    offsets: Optional[torch.Tensor] = None       # [E+1]; computed from ``sel`` when absent
    bounds: Optional[Sequence[int]] = None       # K-tile bounds (max_input_size split)
    wmax: Optional[torch.Tensor] = None          # [E, 1] or [E, N] max |W| (ADC bound / noise scale)
    out_bound: float = -1.0
    out_res: float = -1.0
    noise_std: float = 0.0                       # generate noise in the kernel from noise_seed
    noise_seed: int = 0
    noise_seed_dev: Optional[torch.Tensor] = None      # int64 device word added to the seed by the kernel


def _abs_max_wanted(ir_params, io_params) -> bool:
    """cvmm.py:727-739."""
    if not hasattr(io_params, "is_perfect"):          # lightning flavour
        return not (ir_params is not None and ir_params.enable)
    return (io_params is not None and not io_params.is_perfect
            and enum_name(io_params.noise_management) == "ABS_MAX")


class CVMM(torch.autograd.Function):
    """cvmm.py:699-897.  The launches sit behind the operators ``amoe::cvmm_forward`` and
    ``amoe::cvmm_backward``; what is left here is shape and dtype glue that ``torch.compile`` can trace."""

    @staticmethod
    def forward(ctx, x, sel_index, sel, keys, inp_res, broadcasted_input_ranges=None, out_index=None,
                reduction_weight=None, out_noise=None, ir_params=None, io_params=None, ext=None):
        ext = ext or AnalogExt()
        E, K, N = keys.shape
        if torch.is_autocast_enabled():
            dt = torch.get_autocast_dtype("cuda")
            if dt not in (torch.bfloat16, torch.float16):       # (the reference autocasts to float16: cvmm.py:716)
                raise RuntimeError("the CVMM kernels autocast to bfloat16 or float16")
            x, keys_op = x.to(dt), keys.to(dt)
        else:
            keys_op = keys if keys.dtype == x.dtype else keys.to(x.dtype)
        ssel = sel.reshape(-1).to(torch.int32)
        offsets = ext.offsets if ext.offsets is not None else torch.ops.amoe.offsets_from_sorted(ssel, E)
        sel_index = sel_index.to(torch.int32)
        out_index = None if out_index is None else out_index.to(torch.int32)
        M = ssel.numel()
        bounds = None if ext.bounds is None else list(ext.bounds)
        n_tiles = 1 if bounds is None else len(bounds) - 1
        bir = None
        if broadcasted_input_ranges is not None:
            bir = broadcasted_input_ranges.detach().reshape(M, n_tiles).float().contiguous()
        noise = None
        if out_noise is not None:
            noise = out_noise.detach().float().reshape(n_tiles, M, N).contiguous()
        gate = None if reduction_weight is None else reduction_weight.detach()
        res, z = torch.ops.amoe.cvmm_forward(
            x, keys_op, ssel, offsets, sel_index, out_index, gate, bir, noise, _abs_max_wanted(ir_params, io_params),
            float(inp_res), bounds, ext.wmax, float(ext.out_bound), float(ext.out_res), float(ext.noise_std),
            int(ext.noise_seed), ext.noise_seed_dev)
        if reduction_weight is None:
            res, z = res.view(*sel.shape, N), None
        else:                                                   # cvmm.py:757-759
            res, z = res.view(*reduction_weight.shape[:-1], N), z.view(*sel.shape, N)
        ctx.save_for_backward(x, keys_op, sel_index, out_index, reduction_weight, bir, z, offsets)
        ctx.ir_grad_args = (bool(getattr(ir_params, "gradient_relative", True)),
                            float(getattr(ir_params, "gradient_scale", 1.0)),
                            float(getattr(ir_params, "decay", 0.0)),
                            float(getattr(ir_params, "input_min_percentage", 0.95)))
        ctx.bir_shape = None if broadcasted_input_ranges is None else broadcasted_input_ranges.shape
        ctx.bir_dtype = None if broadcasted_input_ranges is None else broadcasted_input_ranges.dtype
        ctx.bounds = bounds
        ctx.keys_dtype = keys.dtype
        return res

    @staticmethod
    def backward(ctx, grad_output):
        x, keys, sel_index, out_index, gate, bir, z, offsets = ctx.saved_tensors
        grad_x, grad_w, ir_grad, grad_gate = torch.ops.amoe.cvmm_backward(
            grad_output, x, keys, offsets, sel_index, out_index, gate, bir, z, ctx.bounds, *ctx.ir_grad_args)
        if bir is not None and ctx.needs_input_grad[5]:
            ir_grad = ir_grad.view(ctx.bir_shape).to(ctx.bir_dtype)       # cvmm.py:897
        else:
            ir_grad = None
        return (grad_x, None, None, grad_w.to(ctx.keys_dtype), None, ir_grad, None,
                None if gate is None else grad_gate, None, None, None, None)
