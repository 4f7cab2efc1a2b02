"""Marshalling layer between tensors and the C ABI (include/amoe.h).

Each function fills the argument struct of one entry point from tensors the caller has
already allocated and calls it on the given library handle and stream.  Nothing here
allocates, chooses a device or falls back: it only reads ``data_ptr()``, strides and shapes.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import torch

from . import _abi
from ._abi import AMOE_BF16, AMOE_F16, AMOE_F32, BwdWArgs, BwdXArgs, FwdArgs, KsumClipArgs, check, set_bounds


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return AMOE_F32
    if t.dtype == torch.bfloat16:
        return AMOE_BF16
    if t.dtype == torch.float16:
        return AMOE_F16
    raise TypeError(f"unsupported dtype {t.dtype}: the CVMM kernels take float32, bfloat16 or float16")


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _i32(t: Optional[torch.Tensor], name: str):
    if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()):
        raise TypeError(f"{name} must be a contiguous int32 tensor")
    return t


def _f32(t: Optional[torch.Tensor], name: str):
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
        raise TypeError(f"{name} must be a contiguous float32 tensor")
    return t


def _rows(t: torch.Tensor, name: str):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with unit column stride")
    return t


def prepare_sel(lib, stream, sel, E: int, k: int, sel_sorted, perm, in_index, offsets, bad_flag, workspace):
    if sel.dtype not in (torch.int32, torch.int64) or not sel.is_contiguous():
        raise TypeError("sel must be a contiguous int32 or int64 tensor")
    M = sel.numel()
    for t, n in ((sel_sorted, "sel_sorted"), (perm, "perm"), (in_index, "in_index"), (offsets, "offsets")):
        _i32(t, n)
    rc = lib.amoe_prepare_sel(_p(sel), int(sel.dtype == torch.int64), M, E, k, _p(sel_sorted), _p(perm),
                              _p(in_index), _p(offsets), _p(bad_flag), _p(workspace),
                              workspace.numel() * workspace.element_size(), stream)
    check(lib, rc, "amoe_prepare_sel")


def offsets_from_sorted(lib, stream, sel_sorted, E: int, offsets):
    _i32(sel_sorted, "sel_sorted"); _i32(offsets, "offsets")
    check(lib, lib.amoe_offsets_from_sorted(_p(sel_sorted), sel_sorted.numel(), E, _p(offsets), stream),
          "amoe_offsets_from_sorted")


def cvmm_fwd(lib, stream, x, w, out, sel_sorted, offsets, in_index, out_index=None, ir=None, abs_max=None,
             inp_res: float = -1.0, bounds: Optional[Sequence[int]] = None, noise=None, noise_std: float = 0.0,
             noise_seed: int = 0, wmax=None, out_bound: float = -1.0, out_res: float = -1.0, relu: bool = False,
             range_flag=None, ir_by_expert: bool = False, noise_seed_dev=None, xq_out=None, xq_ir=None,
             xq_inp_res: float = -1.0, x_is_quantized: bool = False, code_out=None, code_scale_out=None):
    """x [R_in, K]; w [E, K, N] (any strides with K or N contiguous); out [R_out, N] -- or, with code_out
    (uint8 [R_out, N]) and code_scale_out (fp32 [E, 2]), the result as ADC codes and ``out`` a dummy of the
    right shape that is not written."""
    _rows(x, "x"); _rows(out, "out")
    a = FwdArgs()
    a.dtype = dtype_code(x)
    if w.dtype != x.dtype or out.dtype != x.dtype:
        raise TypeError("x, w and out must share one dtype")
    E, K, N = w.shape
    if x.shape[1] != K or out.shape[1] != N:
        raise ValueError("x / w / out shapes do not match")
    if code_out is not None:
        if code_out.dtype != torch.uint8 or code_out.dim() != 2 or code_out.shape[1] != N or not code_out.is_contiguous():
            raise ValueError("code_out must be a contiguous uint8 tensor [rows, N]")
        if code_scale_out is None or code_scale_out.dtype != torch.float32 or code_scale_out.numel() != 2 * E:
            raise ValueError("code_scale_out must be fp32 [E, 2]")
        a.code_out, a.ldcode, a.code_scale_out = _p(code_out), code_out.stride(0), _p(code_scale_out)
    M = in_index.numel()
    a.M, a.N, a.K, a.E = M, N, K, E
    n_out_rows = out.shape[0] if code_out is None else code_out.shape[0]
    a.n_in_rows, a.n_out_rows = x.shape[0], n_out_rows
    a.x, a.ldx = _p(x), x.stride(0)
    a.w, a.w_stride_e, a.w_stride_k, a.w_stride_n = _p(w), w.stride(0), w.stride(1), w.stride(2)
    a.out, a.ldo = (None if code_out is not None and out.numel() == 0 else _p(out)), out.stride(0)
    a.sel_sorted, a.offsets = _p(_i32(sel_sorted, "sel_sorted")), _p(_i32(offsets, "offsets"))
    a.in_index, a.out_index = _p(_i32(in_index, "in_index")), _p(_i32(out_index, "out_index"))
    set_bounds(a, [0, K] if bounds is None else bounds)
    if ir is not None and ir.numel() != (E if ir_by_expert else M) * a.n_tiles:
        raise ValueError("ir must hold one value per sorted position (or expert) and K-tile")
    a.ir_by_expert = int(bool(ir_by_expert))
    a.ir, a.abs_max, a.inp_res = _p(_f32(ir, "ir")), _p(_f32(abs_max, "abs_max")), float(inp_res)
    if noise is not None:
        _f32(noise, "noise")
        if noise.numel() != a.n_tiles * n_out_rows * N:
            raise ValueError("noise must be [n_tiles, out rows, N]")
        a.noise, a.noise_tile_stride, a.ldnoise = _p(noise), n_out_rows * N, N
    a.noise_std, a.noise_seed = float(noise_std), int(noise_seed) & 0xFFFFFFFFFFFFFFFF
    if noise_seed_dev is not None:
        if noise_seed_dev.dtype != torch.int64 or noise_seed_dev.numel() != 1:
            raise ValueError("noise_seed_dev must be one int64 word")
        a.noise_seed_dev = _p(noise_seed_dev)
    if wmax is not None:
        _f32(wmax, "wmax")
        a.wmax, a.wmax_cols = _p(wmax), wmax.numel() // E
    a.out_bound, a.out_res = float(out_bound), float(out_res)
    a.relu, a.range_flag = int(bool(relu)), _p(range_flag)
    if xq_out is not None:
        _rows(xq_out, "xq_out")
        if xq_out.dtype != x.dtype or tuple(xq_out.shape) != (n_out_rows, N):
            raise ValueError("xq_out must match out")
        a.xq_out, a.ldxq, a.xq_ir, a.xq_inp_res = _p(xq_out), xq_out.stride(0), _p(_f32(xq_ir, "xq_ir")), float(xq_inp_res)
    a.x_is_quantized = int(bool(x_is_quantized))
    if x.dtype != torch.float32:
        # the 16-bit kernels feed the DAC codes themselves to the matrix unit: integers are exact up to 256 in
        # bf16 and 2048 in fp16 (the library returns AMOE_EUNSUPPORTED beyond that; say why here)
        most = 256 if x.dtype == torch.bfloat16 else 2048
        for name, res in (("inp_res", inp_res), ("xq_inp_res", xq_inp_res if xq_out is not None else -1.0)):
            if res > 0 and 1.0 / res > most * (1 + 1e-6):
                raise ValueError(f"{name}={res}: an input quantiser with more than {2 * most} steps needs fp32 tensors "
                                 f"({x.dtype} holds the codes exactly only up to +-{most})")
    check(lib, lib.amoe_cvmm_fwd(C.byref(a), stream), "amoe_cvmm_fwd")


def cvmm_bwd_w(lib, stream, x, g, grad_w, offsets, in_index, g_index=None, ir=None,
               bounds: Optional[Sequence[int]] = None, ir_by_expert: bool = False, g_scale=None,
               rows_per_chunk: int = 0):
    """x [*, K]; g [*, N]; grad_w [E, K, N] contiguous."""
    _rows(x, "x"); _rows(g, "g")
    if not grad_w.is_contiguous():
        raise ValueError("grad_w must be contiguous")
    a = BwdWArgs()
    a.dtype = dtype_code(x)
    if g.dtype != x.dtype or grad_w.dtype != x.dtype:
        raise TypeError("x, g and grad_w must share one dtype")
    E, K, N = grad_w.shape
    if x.shape[1] != K or g.shape[1] != N:
        raise ValueError("x / g / grad_w shapes do not match")
    a.M, a.N, a.K, a.E = in_index.numel(), N, K, E
    a.x, a.ldx, a.g, a.ldg, a.grad_w = _p(x), x.stride(0), _p(g), g.stride(0), _p(grad_w)
    a.offsets, a.in_index, a.g_index = _p(_i32(offsets, "offsets")), _p(_i32(in_index, "in_index")), \
        _p(_i32(g_index, "g_index"))
    set_bounds(a, [0, K] if bounds is None else bounds)
    a.ir, a.ir_by_expert = _p(_f32(ir, "ir")), int(bool(ir_by_expert))
    if g_scale is not None and (g_scale.dtype != x.dtype or not g_scale.is_contiguous()):
        raise TypeError("g_scale must be contiguous and share the dtype of x")
    a.g_scale = _p(g_scale)
    a.n_x_rows, a.n_g_rows = x.shape[0], g.shape[0]
    a.rows_per_chunk = int(rows_per_chunk)
    need = lib.amoe_bwd_w_workspace(C.byref(a))
    if need:
        ws = torch.empty(need, dtype=torch.uint8, device=x.device)
        a.workspace, a.workspace_bytes = _p(ws), need
    check(lib, lib.amoe_cvmm_bwd_w(C.byref(a), stream), "amoe_cvmm_bwd_w")


def bwd_x_workspace_bytes(lib, M: int, K: int, n_tiles: int) -> int:
    return lib.amoe_bwd_x_workspace(M, K, n_tiles)


def cvmm_bwd_x(lib, stream, g, w, grad_x_full, offsets, g_index, out_index, x=None, xf_index=None, gate=None,
               ir=None, ir_grad=None, bounds: Optional[Sequence[int]] = None, gradient_relative: bool = True,
               gradient_scale: float = 1.0, decay: float = 0.0, input_min_percentage: float = 0.95,
               relu_mask: bool = False, workspace=None, ir_by_expert: bool = False, xc_out=None):
    """g [*, N]; w [E, K, N] with N contiguous; grad_x_full [R_out, K]; x [*, K] forward input."""
    _rows(g, "g"); _rows(grad_x_full, "grad_x_full")
    a = BwdXArgs()
    a.dtype = dtype_code(g)
    E, K, N = w.shape
    if w.stride(2) != 1:
        raise ValueError("w must have its last dimension contiguous")
    if g.shape[1] != N or grad_x_full.shape[1] != K:
        raise ValueError("g / w / grad_x_full shapes do not match")
    a.M, a.N, a.K, a.E = g_index.numel(), N, K, E
    a.g, a.ldg, a.n_g_rows = _p(g), g.stride(0), g.shape[0]
    a.w, a.w_stride_e, a.w_stride_k = _p(w), w.stride(0), w.stride(1)
    a.grad_x_full, a.ldo = _p(grad_x_full), grad_x_full.stride(0)
    if x is not None:
        _rows(x, "x")
        a.x, a.ldx = _p(x), x.stride(0)
    a.offsets, a.g_index = _p(_i32(offsets, "offsets")), _p(_i32(g_index, "g_index"))
    a.out_index, a.xf_index = _p(_i32(out_index, "out_index")), _p(_i32(xf_index, "xf_index"))
    if gate is not None and (gate.dtype != g.dtype or not gate.is_contiguous()):
        raise TypeError("gate must be contiguous and share the dtype of g")
    a.gate = _p(gate)
    set_bounds(a, [0, K] if bounds is None else bounds)
    a.ir, a.ir_grad = _p(_f32(ir, "ir")), _p(_f32(ir_grad, "ir_grad"))
    a.ir_by_expert = int(bool(ir_by_expert))
    a.gradient_relative, a.gradient_scale = int(bool(gradient_relative)), float(gradient_scale)
    a.decay, a.input_min_percentage = float(decay), float(input_min_percentage)
    a.relu_mask = int(bool(relu_mask))
    if workspace is not None:
        a.workspace, a.workspace_bytes = _p(workspace), workspace.numel() * workspace.element_size()
    if xc_out is not None:
        _rows(xc_out, "xc_out")
        if x is None or xc_out.dtype != x.dtype or xc_out.shape != x.shape:
            raise ValueError("xc_out must match x")
        a.xc_out, a.ldxc = _p(xc_out), xc_out.stride(0)
    check(lib, lib.amoe_cvmm_bwd_x(C.byref(a), stream), "amoe_cvmm_bwd_x")


def _counter(counter):
    """An int64 device word the launch adds to (None: no addition)."""
    if counter is not None and (counter.dtype != torch.int64 or counter.numel() < 1):
        raise ValueError("counter must be an int64 tensor (one word in device memory)")
    return _p(counter)


def gate_reduce(lib, stream, z, gate, y, T: int, k: int, D: int, counter=None, counter_add: int = 0):
    check(lib, lib.amoe_gate_reduce(dtype_code(z), _p(z), _p(gate), _p(y), T, k, D, _counter(counter), counter_add,
                                    stream), "amoe_gate_reduce")


def gate_reduce_codes(lib, stream, codes, scale, sel, gate, y, T: int, k: int, D: int, counter=None,
                      counter_add: int = 0):
    check(lib, lib.amoe_gate_reduce_codes(dtype_code(y), _p(codes), _p(scale), _p(sel), int(sel.dtype == torch.int64),
                                          _p(gate), _p(y), T, k, D, _counter(counter), counter_add, stream),
          "amoe_gate_reduce_codes")


def gate_grad_codes(lib, stream, codes, scale, sel, dy, grad_gate, T: int, k: int, D: int):
    check(lib, lib.amoe_gate_grad_codes(dtype_code(dy), _p(codes), _p(scale), _p(sel), int(sel.dtype == torch.int64),
                                        _p(dy), _p(grad_gate), T, k, D, stream), "amoe_gate_grad_codes")


def ksum(lib, stream, full, out, T: int, k: int, D: int):
    check(lib, lib.amoe_ksum(dtype_code(full), _p(full), _p(out), T, k, D, stream), "amoe_ksum")


def ksum_clip_workspace_bytes(lib, T: int, k: int, n_tiles: int) -> int:
    return lib.amoe_ksum_clip_workspace(T, k, n_tiles)


def ksum_clip(lib, stream, full, x, sel, perm, offsets, ir, grad_x, ir_grad, workspace, T: int, k: int, E: int,
              bounds: Optional[Sequence[int]] = None, gradient_relative: bool = True, gradient_scale: float = 1.0,
              decay: float = 0.0, input_min_percentage: float = 0.95):
    """full [T*k, D] and grad_x [T, D] dense; x [T, D] rows; sel [T*k] int32 or int64; ir [E, n_tiles] fp32;
    ir_grad [T*k, n_tiles] fp32 (by sorted position)."""
    _rows(x, "x")
    if not full.is_contiguous() or not grad_x.is_contiguous():
        raise ValueError("full and grad_x must be contiguous")
    if x.dtype != full.dtype or grad_x.dtype != full.dtype:
        raise TypeError("full, x and grad_x share one dtype")
    if sel.dtype not in (torch.int32, torch.int64) or not sel.is_contiguous() or sel.numel() != T * k:
        raise TypeError("sel must be a contiguous int32 or int64 tensor of T * k experts")
    D = full.shape[1]
    if full.shape[0] != T * k or x.shape != (T, D) or grad_x.shape != (T, D):
        raise ValueError("full / x / grad_x shapes do not match")
    a = KsumClipArgs()
    a.dtype = dtype_code(full)
    a.T, a.k, a.D, a.E = T, k, D, E
    a.full, a.x, a.ldx = _p(full), _p(x), x.stride(0)
    a.sel, a.sel_is_i64 = _p(sel), int(sel.dtype == torch.int64)
    a.perm, a.offsets = _p(_i32(perm, "perm")), _p(_i32(offsets, "offsets"))
    a.ir = _p(_f32(ir, "ir"))
    set_bounds(a, [0, D] if bounds is None else bounds)
    if ir.numel() != E * a.n_tiles:
        raise ValueError("ir must be [E, n_tiles]")
    a.grad_x, a.ir_grad = _p(grad_x), _p(_f32(ir_grad, "ir_grad"))
    a.gradient_relative, a.gradient_scale = int(bool(gradient_relative)), float(gradient_scale)
    a.decay, a.input_min_percentage = float(decay), float(input_min_percentage)
    a.workspace, a.workspace_bytes = _p(workspace), workspace.numel() * workspace.element_size()
    check(lib, lib.amoe_ksum_clip(C.byref(a), stream), "amoe_ksum_clip")


def gate_grad(lib, stream, z, dy, grad_gate, T: int, k: int, D: int):
    check(lib, lib.amoe_gate_grad(dtype_code(z), _p(z), _p(dy), _p(grad_gate), T, k, D, stream), "amoe_gate_grad")


def row_abs_max(lib, stream, x, out):
    _rows(x, "x")
    check(lib, lib.amoe_row_abs_max(dtype_code(x), _p(x), x.stride(0), x.shape[0], x.shape[1],
                                    _p(_f32(out, "abs_max")), stream), "amoe_row_abs_max")


def weight_abs_max(lib, stream, w, cols: int, out):
    if not w.is_contiguous():
        raise ValueError("w must be contiguous")
    E, K, N = w.shape
    check(lib, lib.amoe_weight_abs_max(dtype_code(w), _p(w), E, K, N, cols, _p(_f32(out, "wmax")), stream),
          "amoe_weight_abs_max")


def weight_abs_max_pair(lib, stream, w_a, w_b, out_a, out_b):
    if not w_a.is_contiguous() or not w_b.is_contiguous() or w_a.dtype != w_b.dtype or w_a.shape[0] != w_b.shape[0]:
        raise ValueError("two contiguous weight tensors of one dtype and one expert count")
    E = w_a.shape[0]
    check(lib, lib.amoe_weight_abs_max_pair(dtype_code(w_a), _p(w_a), w_a.shape[1], w_a.shape[2],
                                            _p(_f32(out_a, "wmax_a")), _p(w_b), w_b.shape[1], w_b.shape[2],
                                            _p(_f32(out_b, "wmax_b")), E, stream), "amoe_weight_abs_max_pair")


def layer_tables(lib, stream, w_a, w_b, out_a, out_b, input_range, n_up: int, n_dn: int, ir_up, ir_dn):
    """input_range [2, E, ir_cols] (any of the three dtypes, contiguous) -> ir_up fp32 [E, n_up], ir_dn fp32 [E, n_dn]"""
    if not w_a.is_contiguous() or not w_b.is_contiguous() or w_a.dtype != w_b.dtype or w_a.shape[0] != w_b.shape[0]:
        raise ValueError("two contiguous weight tensors of one dtype and one expert count")
    E = w_a.shape[0]
    if not input_range.is_contiguous() or input_range.numel() % (2 * E):
        raise ValueError("input_range must be contiguous [2, E, tiles]")
    ir_cols = input_range.numel() // (2 * E)
    if tuple(ir_up.shape) != (E, n_up) or tuple(ir_dn.shape) != (E, n_dn) or not ir_up.is_contiguous() or not ir_dn.is_contiguous():
        raise ValueError("ir_up / ir_dn must be contiguous [E, tiles of the projection]")
    check(lib, lib.amoe_layer_tables(dtype_code(w_a), _p(w_a), w_a.shape[1], w_a.shape[2], _p(_f32(out_a, "wmax_a")),
                                     _p(w_b), w_b.shape[1], w_b.shape[2], _p(_f32(out_b, "wmax_b")), E,
                                     dtype_code(input_range), _p(input_range), ir_cols, n_up, _p(_f32(ir_up, "ir_up")),
                                     n_dn, _p(_f32(ir_dn, "ir_dn")), stream), "amoe_layer_tables")


def segment_sum(lib, stream, v, offsets, E: int, n_tiles: int, out, zero_cols: int = 0):
    """out: [E, n_tiles] in any of the three dtypes, rows any stride apart (a slice of a wider table will do); the
    zero_cols columns that follow the slice in that table are cleared"""
    if (out.dim() != 2 or tuple(out.shape) != (E, n_tiles) or (n_tiles > 1 and out.stride(1) != 1) or
            out.stride(0) < n_tiles + zero_cols):
        raise ValueError("out must be [E, n_tiles] with unit column stride and rows at least n_tiles + zero_cols apart")
    check(lib, lib.amoe_segment_sum(_p(_f32(v, "v")), _p(_i32(offsets, "offsets")), E, n_tiles, dtype_code(out),
                                    _p(out), out.stride(0), zero_cols, stream), "amoe_segment_sum")


def expert_std(lib, stream, x, in_index, offsets, E: int, out):
    _rows(x, "x")
    check(lib, lib.amoe_expert_std(dtype_code(x), _p(x), x.stride(0), x.shape[1], _p(_i32(in_index, "in_index")),
                                   _p(_i32(offsets, "offsets")), E, _p(_f32(out, "out")), stream),
          "amoe_expert_std")


def modify_weight(lib, stream, w, wmax, n_states: float, std_dev: float, noise, round_noise: bool, noise_seed: int,
                  noise_seed_dev, out):
    if not w.is_contiguous() or not out.is_contiguous() or out.shape != w.shape or out.dtype != w.dtype:
        raise ValueError("w and out must be contiguous tensors of one shape and dtype")
    E, K, N = w.shape
    cols = wmax.numel() // E
    if wmax.numel() != E * cols or cols not in (1, N):
        raise ValueError("wmax must be [E] or [E, N]")
    if noise is not None and noise.numel() != w.numel():
        raise ValueError("noise must have one value per weight")
    if noise_seed_dev is not None and (noise_seed_dev.dtype != torch.int64 or noise_seed_dev.numel() != 1):
        raise ValueError("noise_seed_dev must be one int64 word")
    check(lib, lib.amoe_modify_weight(dtype_code(w), _p(w), E, K, N, _p(_f32(wmax, "wmax")), cols, float(n_states),
                                      float(std_dev), _p(_f32(noise, "noise")), int(bool(round_noise)),
                                      int(noise_seed) & 0xFFFFFFFFFFFFFFFF, _p(noise_seed_dev), _p(out), stream),
          "amoe_modify_weight")


def weight_std_workspace_bytes(lib, E: int, K: int, N: int, cols: int) -> int:
    return lib.amoe_weight_std_workspace(E, K, N, cols)


def weight_std(lib, stream, w, cols: int, out, workspace):
    if not w.is_contiguous():
        raise ValueError("w must be contiguous")
    E, K, N = w.shape
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib, lib.amoe_weight_std(dtype_code(w), _p(w), E, K, N, cols, _p(_f32(out, "std")), _p(workspace), nbytes,
                                   stream), "amoe_weight_std")


def clamp_weights(lib, stream, w, bound, cols: int):
    if not w.is_contiguous():
        raise ValueError("w must be contiguous")
    E, K, N = w.shape
    if bound.numel() != E * cols:
        raise ValueError("bound must be [E] or [E, N]")
    check(lib, lib.amoe_clamp_weights(dtype_code(w), _p(w), E, K, N, _p(_f32(bound, "bound")), cols, stream),
          "amoe_clamp_weights")


def select_fwd(lib, stream, logits, k: int, sel_val, sel_idx, reg, reg_c, workspace):
    T, E = logits.shape
    if not logits.is_contiguous() or sel_idx.dtype != torch.int64 or sel_val.dtype != logits.dtype:
        raise ValueError("logits must be contiguous, sel_val of its dtype, sel_idx int64")
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    check(lib, lib.amoe_select_fwd(dtype_code(logits), _p(logits), T, E, k, _p(sel_val), _p(sel_idx),
                                   _p(_f32(reg, "reg")), _p(_f32(reg_c, "reg_c")), _p(workspace), nbytes, stream),
          "amoe_select_fwd")


def select_bwd(lib, stream, logits, k: int, sel_idx, grad_val, reg_c, grad_reg, grad_logits):
    T, E = logits.shape
    if not logits.is_contiguous() or not grad_logits.is_contiguous():
        raise ValueError("logits and grad_logits must be contiguous")
    if grad_val is not None and (grad_val.dtype != logits.dtype or not grad_val.is_contiguous()):
        raise ValueError("grad_val must be contiguous and of the logits' dtype")
    check(lib, lib.amoe_select_bwd(dtype_code(logits), _p(logits), T, E, k, _p(sel_idx), _p(grad_val),
                                   _p(_f32(reg_c, "reg_c")), _p(_f32(grad_reg, "grad_reg")), _p(grad_logits), stream),
          "amoe_select_bwd")
