"""Per-expert CPU layer in eager PyTorch.  TEST INFRASTRUCTURE / CPU BASELINE ONLY.

The reference's CPU path is its ``traceable=True`` mode: one analog linear per expert,
looped over experts (moe_layer_aihwkit_lightning.py:165-168, 395-400); the loop body lives
in third-party packages that are not part of the reference checkout.  This file restates
that path: ``for e in experts: y[rows_e] += gate * analog_linear_e(x[rows_e])`` with the
input stage of cvmm.py:145-172, the output stage of cvmm.py:215-229 and the backward rules
of cvmm.py:365-373 (weight gradient from clipped, un-quantised inputs) and cvmm.py:848-881
(strict clip mask, input-range gradient).  It is timed as the CPU baseline of the benchmark
and used in tests as a second, autograd-driven formulation beside the numpy oracle.
Nothing in the shipped package imports it.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch


class _AnalogMVM(torch.autograd.Function):
    """One expert, one K-tile:  (Q(clamp(x, +-ir) / ir) @ W + noise -> ADC) * ir."""

    @staticmethod
    def forward(ctx, x, w, ir, inp_res, noise, wmax, out_bound, out_res, ir_cfg):
        xf = x.float()
        if ir is not None:
            a = torch.minimum(torch.maximum(xf, -ir), ir) / ir
        else:
            a = xf
        if inp_res > 0:
            a = torch.round(a / inp_res) * inp_res
        c = a.to(w.dtype) @ w if w.dtype != torch.float32 else a @ w
        c = c.float()
        if noise is not None:
            c = c + noise
        if out_bound > 0:
            bound = out_bound * wmax
            c = torch.minimum(torch.maximum(c, -bound), bound)
            if out_res > 0:
                half = max(out_res, 1.0 / out_res) * 0.5
                c = torch.round(c * (half / bound)) * (bound / half)
        if ir is not None:
            c = c * ir
        ctx.save_for_backward(x, w, ir)
        ctx.ir_cfg = ir_cfg
        return c.to(x.dtype)

    @staticmethod
    def backward(ctx, g):
        x, w, ir = ctx.saved_tensors
        decay, min_pct, relative, scale, pct_flag = ctx.ir_cfg
        xf = x.float()
        xc = xf if ir is None else torch.minimum(torch.maximum(xf, -ir), ir)
        grad_w = (xc.to(w.dtype).t() @ g.to(w.dtype)).to(w.dtype)
        gx = (g.to(w.dtype) @ w.t()).float()
        grad_ir = None
        if ir is not None:
            upper = xf >= ir
            lower = xf <= -ir
            gi = torch.clamp(upper * gx, max=0.0).sum() - torch.clamp(lower * gx, min=0.0).sum()
            # per-row form of cvmm.py:863-870 summed over the expert's rows (they share one ir)
            if relative:
                gi = gi * ir * scale
            if decay > 0:
                gi = gi + decay * ir * x.shape[0] * pct_flag
            grad_ir = gi.reshape(ir.shape)
            gx = gx * (xf.abs() < ir)
        return gx.to(x.dtype), grad_w, grad_ir, None, None, None, None, None, None


def analog_linear(x, w, ir_tiles, bounds, inp_res, noise, wmax, out_bound, out_res, ir_cfg):
    """Sum over K-tiles of one expert's analog MVM.  ir_tiles: [n_tiles] tensor or None;
    noise: [n_tiles, rows, N] or None."""
    out = None
    for t in range(len(bounds) - 1):
        lo, hi = int(bounds[t]), int(bounds[t + 1])
        ir = None if ir_tiles is None else ir_tiles[t].reshape(1, 1)
        nz = None if noise is None else noise[t]
        c = _AnalogMVM.apply(x[:, lo:hi], w[lo:hi], ir, inp_res, nz, wmax, out_bound, out_res, ir_cfg)
        out = c if out is None else out + c
    return out


def clip_fraction_flag(x_up, x_down, sel_flat, ir, bounds_up, bounds_down, min_pct):
    """Global 'fraction of un-clipped inputs > input_min_percentage' flags of
    cvmm.py:873-877, one for each projection."""
    flags = []
    for x, b, row in ((x_up, bounds_up, 0), (x_down, bounds_down, 1)):
        if ir is None:
            flags.append(0.0)
            continue
        cnt = 0
        for t in range(len(b) - 1):
            r = ir[row][sel_flat, t][:, None]
            cnt += (x[:, int(b[t]):int(b[t + 1])].abs().float() < r).sum().item()
        flags.append(float(cnt / x.numel() > min_pct))
    return flags


def moe_layer_per_expert(x, keys, values, sel_idx, sel_val, ir=None, *, inp_res=-1.0,
                         noise_up=None, noise_down=None, wmax_up=None, wmax_down=None,
                         out_bound=-1.0, out_res=-1.0, bounds_up: Optional[Sequence[int]] = None,
                         bounds_down: Optional[Sequence[int]] = None, decay=0.0,
                         input_min_percentage=0.95, gradient_relative=True, gradient_scale=1.0):
    """x [T, D]; keys [E, D, F]; values [E, F, D]; sel_idx / sel_val [T, k];
    ir [2, E, n_tiles] (row 0 up-projection, row 1 down-projection) or None;
    noise_up [n_tiles, T*k, F], noise_down [n_tiles, T*k, D] indexed by flat (t, k) row.
    Returns y [T, D] = sum_k gate * analog(relu(analog(x, keys[e])), values[e])."""
    T, D = x.shape
    E, _, F = keys.shape
    k = sel_idx.shape[1]
    bounds_up = [0, D] if bounds_up is None else bounds_up
    bounds_down = [0, F] if bounds_down is None else bounds_down
    y = torch.zeros(T, values.shape[2], dtype=torch.float32, device=x.device)
    flat_sel = sel_idx.reshape(-1)
    pct_up = pct_down = 0.0
    if ir is not None and decay > 0:
        # needs the down-projection inputs: run the up-projection once without grad
        with torch.no_grad():
            s = torch.zeros(T * k, F, dtype=x.dtype)
            for e in range(E):
                rows = (flat_sel == e).nonzero().squeeze(-1)
                if rows.numel():
                    nz = None if noise_up is None else noise_up[:, rows]
                    wm = None if wmax_up is None else wmax_up[e]
                    s[rows] = torch.relu(analog_linear(x[rows // k], keys[e], ir[0, e], bounds_up, inp_res,
                                                       nz, wm, out_bound, out_res, (0, 0, True, 1.0, 0.0)))
            pct_up, pct_down = clip_fraction_flag(x[torch.arange(T * k) // k], s, flat_sel, ir,
                                                  bounds_up, bounds_down, input_min_percentage)
    for e in range(E):
        rows = (flat_sel == e).nonzero().squeeze(-1)
        if rows.numel() == 0:
            continue
        tok = rows // k
        nz_u = None if noise_up is None else noise_up[:, rows]
        nz_d = None if noise_down is None else noise_down[:, rows]
        wm_u = None if wmax_up is None else wmax_up[e]
        wm_d = None if wmax_down is None else wmax_down[e]
        cfg_u = (decay, input_min_percentage, gradient_relative, gradient_scale, pct_up)
        cfg_d = (decay, input_min_percentage, gradient_relative, gradient_scale, pct_down)
        h = analog_linear(x[tok], keys[e], None if ir is None else ir[0, e], bounds_up, inp_res,
                          nz_u, wm_u, out_bound, out_res, cfg_u)
        h = torch.relu(h)
        z = analog_linear(h, values[e], None if ir is None else ir[1, e], bounds_down, inp_res,
                          nz_d, wm_d, out_bound, out_res, cfg_d)
        gate = sel_val.reshape(-1)[rows].unsqueeze(-1)
        y = y.index_add(0, tok, (gate.to(z.dtype) * z).float())
    return y.to(x.dtype)
