"""Tensor-level entry points of the CVMM path: allocate outputs with torch, run the HIP
kernels of libamoe.so on the current stream.

There is no CPU path and no fallback: the library must have been built
(``python -c "import __graft_entry__ as g; g.build()"``) and every tensor must live on the GPU.
"""
from __future__ import annotations

import os
from typing import Optional, Sequence, Tuple

import torch

from . import _abi, raw

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libamoe.so")
_LIB = None


def lib_path() -> str:
    return _LIB_PATH


def get_lib():
    """The loaded C-ABI library.  Raises if it has not been built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build the HIP library first (__graft_entry__.build()); "
                "analog_moe_amd has no CPU fallback")
        _LIB = _abi.bind(_LIB_PATH)
    return _LIB


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("analog_moe_amd runs on the GPU only: got a CPU tensor (there is no CPU path)")


def _rows2d(t: torch.Tensor) -> torch.Tensor:
    t = t.reshape(-1, t.shape[-1])
    return t if t.stride(1) == 1 else t.contiguous()


def _f32c(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None:
        return None
    return t.detach().to(torch.float32).contiguous()


def _i32c(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None:
        return None
    return t.detach().reshape(-1).to(torch.int32).contiguous()


# ------------------------------------------------------------------------------ selection
def prepare_sel(sel: torch.Tensor, n_experts: int, k: int) -> Tuple[torch.Tensor, ...]:
    """Stable expert sort.  Returns (sel_sorted, perm, in_index = perm // k, offsets[E+1]), int32."""
    _need_gpu(sel)
    lib = get_lib()
    flat = sel.detach().reshape(-1)
    if flat.dtype not in (torch.int32, torch.int64):
        flat = flat.to(torch.int64)
    flat = flat.contiguous()
    M = flat.numel()
    dev = flat.device
    sel_sorted = torch.empty(M, dtype=torch.int32, device=dev)
    perm = torch.empty(M, dtype=torch.int32, device=dev)
    in_index = torch.empty(M, dtype=torch.int32, device=dev)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    ws = torch.empty(max(lib.amoe_prepare_sel_workspace(M, n_experts), 4), dtype=torch.uint8, device=dev)
    raw.prepare_sel(lib, _stream(flat), flat, n_experts, k, sel_sorted, perm, in_index, offsets, None, ws)
    return sel_sorted, perm, in_index, offsets


def offsets_from_sorted(sel_sorted: torch.Tensor, n_experts: int) -> torch.Tensor:
    _need_gpu(sel_sorted)
    s = _i32c(sel_sorted)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=s.device)
    raw.offsets_from_sorted(get_lib(), _stream(s), s, n_experts, offsets)
    return offsets


# ------------------------------------------------------------------------------ forward
def cvmm_fwd(x: torch.Tensor, w: torch.Tensor, sel_sorted: torch.Tensor, offsets: torch.Tensor,
             in_index: torch.Tensor, out_index: Optional[torch.Tensor], n_out_rows: int, *,
             ir: Optional[torch.Tensor] = None, abs_max: Optional[torch.Tensor] = None, inp_res: float = -1.0,
             bounds: Optional[Sequence[int]] = None, noise: Optional[torch.Tensor] = None,
             noise_std: float = 0.0, noise_seed: int = 0, wmax: Optional[torch.Tensor] = None,
             out_bound: float = -1.0, out_res: float = -1.0, relu: bool = False,
             ir_by_expert: bool = False, noise_seed_dev: Optional[torch.Tensor] = None,
             xq_ir: Optional[torch.Tensor] = None, xq_inp_res: float = -1.0, x_is_quantized: bool = False,
             want_codes: bool = False):
    """out[out_index[i]] = analog(x[in_index[i]]) @ w[sel_sorted[i]] -> [n_out_rows, N].
    ir: [M, n_tiles] per sorted position, or the [E, n_tiles] table with ir_by_expert.
    noise_seed_dev: optional int64 device word added to noise_seed by the kernel.
    xq_ir ([E] fp32) + xq_inp_res: also return the input-stage image of the result for the projection
    that follows (-> (out, xq)); x_is_quantized: x is such an image made for this call.
    want_codes: return the result as its ADC codes instead -> (codes uint8 [n_out_rows, N] = code + 128,
    scale fp32 [E, 2]) with result = ((code - 128) * scale[e, 0]) * scale[e, 1]; raises AmoeError (rc
    AMOE_EUNSUPPORTED) where the library has no such kernel for the call (see ``codes_supported``)."""
    _need_gpu(x, w, sel_sorted, offsets, in_index, out_index, ir, abs_max, noise, wmax)
    x2 = _rows2d(x)
    if w.stride(2) != 1 and w.stride(1) != 1:
        w = w.contiguous()
    if want_codes:
        codes = torch.empty((n_out_rows, w.shape[2]), dtype=torch.uint8, device=x2.device)
        scale = torch.empty((w.shape[0], 2), dtype=torch.float32, device=x2.device)
        dummy = torch.empty((0, w.shape[2]), dtype=x2.dtype, device=x2.device)
        raw.cvmm_fwd(get_lib(), _stream(x2), x2, w, dummy, sel_sorted, offsets, in_index, out_index, _f32c(ir),
                     _f32c(abs_max), inp_res, bounds, _f32c(noise), noise_std, noise_seed, _f32c(wmax), out_bound,
                     out_res, relu, None, ir_by_expert, noise_seed_dev, None, None, -1.0, x_is_quantized,
                     code_out=codes, code_scale_out=scale)
        return codes, scale
    out = torch.empty((n_out_rows, w.shape[2]), dtype=x2.dtype, device=x2.device)
    xq = torch.empty_like(out) if xq_ir is not None else None
    raw.cvmm_fwd(get_lib(), _stream(x2), x2, w, out, sel_sorted, offsets, in_index, out_index, _f32c(ir),
                 _f32c(abs_max), inp_res, bounds, _f32c(noise), noise_std, noise_seed, _f32c(wmax), out_bound,
                 out_res, relu, None, ir_by_expert, noise_seed_dev, xq, _f32c(xq_ir), xq_inp_res, x_is_quantized)
    return out if xq is None else (out, xq)


def codes_supported(x: torch.Tensor, w: torch.Tensor, *, ir_by_expert: bool, inp_res: float, n_tiles: int,
                    out_bound: float, out_res: float, noise: Optional[torch.Tensor], per_channel: bool) -> bool:
    """Whether ``cvmm_fwd(..., want_codes=True)`` has a kernel for this call.  The library decides
    (``amoe_fwd_codes_supported``, the same function its launcher asks); only shapes, strides and settings are
    passed, so the answer is a pure function of them and holds for meta tensors under a tracer too.  x and w as
    ``cvmm_fwd`` would hand them over (freshly allocated tensors are 16-byte aligned, which is all that is left)."""
    if x.dtype not in (torch.bfloat16, torch.float16) or w.dtype != x.dtype or w.dim() != 3:
        return False
    E, K, N = w.shape
    if x.dim() < 2 or x.shape[-1] != K or x.stride(-1) != 1 or (w.stride(2) != 1 and w.stride(1) != 1):
        return False
    a = _abi.FwdArgs()
    a.dtype = raw.dtype_code(x)
    a.M, a.N, a.K, a.E = 1, N, K, E
    a.n_in_rows = x.numel() // K
    a.ldx = x.stride(-2)
    a.w_stride_e, a.w_stride_k, a.w_stride_n = w.stride(0), w.stride(1), w.stride(2)
    _abi.set_bounds(a, [0, K])
    a.n_tiles = n_tiles
    flag = 1                       # pointer fields are read as present / absent only
    a.ir, a.ir_by_expert = (flag if ir_by_expert else None), int(bool(ir_by_expert))
    a.inp_res = float(inp_res)
    a.noise = flag if noise is not None else None
    a.wmax, a.wmax_cols = flag, (N if per_channel else 1)
    a.out_bound, a.out_res = float(out_bound), float(out_res)
    a.code_out, a.ldcode, a.code_scale_out = flag, N, flag
    return bool(get_lib().amoe_fwd_codes_supported(a))


def cvmm_bwd_w(x: torch.Tensor, g: torch.Tensor, n_experts: int, offsets: torch.Tensor, in_index: torch.Tensor,
               g_index: Optional[torch.Tensor], *, ir: Optional[torch.Tensor] = None,
               bounds: Optional[Sequence[int]] = None, ir_by_expert: bool = False,
               g_scale: Optional[torch.Tensor] = None, rows_per_chunk: int = 0) -> torch.Tensor:
    """grad_w[e] = sum_i clamp(x[in_index[i]])^T (g_scale[in_index[i]] * g[g_index[i]]).
    rows_per_chunk: 0 lets the library decide how the rows of an expert are shared between workgroups."""
    _need_gpu(x, g, offsets, in_index, g_index, ir, g_scale)
    x2, g2 = _rows2d(x), _rows2d(g)
    grad_w = torch.empty((n_experts, x2.shape[1], g2.shape[1]), dtype=x2.dtype, device=x2.device)
    # the library wants the scale per sorted position
    gs = None if g_scale is None else g_scale.detach().reshape(-1).to(x2.dtype)[in_index.long()].contiguous()
    raw.cvmm_bwd_w(get_lib(), _stream(x2), x2, g2, grad_w, offsets, in_index, g_index, _f32c(ir), bounds,
                   ir_by_expert, gs, rows_per_chunk)
    return grad_w


def cvmm_bwd_x(g: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, g_index: torch.Tensor,
               out_index: torch.Tensor, n_out_rows: int, *, x: Optional[torch.Tensor] = None,
               xf_index: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
               ir: Optional[torch.Tensor] = None, bounds: Optional[Sequence[int]] = None,
               gradient_relative: bool = True, gradient_scale: float = 1.0, decay: float = 0.0,
               input_min_percentage: float = 0.95, relu_mask: bool = False, ir_by_expert: bool = False,
               want_xc: bool = False):
    """Returns (grad_x_full [n_out_rows, K], ir_grad [M, n_tiles] or None) and, with want_xc, also
    gate * clamp(x, +-ir) in the layout of x: the x operand of the weight gradient of the same projection."""
    _need_gpu(g, w, offsets, g_index, out_index, x, xf_index, gate, ir)
    lib = get_lib()
    g2 = _rows2d(g)
    if w.stride(2) != 1:
        w = w.contiguous()
    E, K, N = w.shape
    M = g_index.numel()
    n_tiles = 1 if bounds is None else len(bounds) - 1
    full = torch.empty((n_out_rows, K), dtype=g2.dtype, device=g2.device)
    x2 = None if x is None else _rows2d(x)
    ir32 = _f32c(ir)
    ir_grad = ws = None
    if ir32 is not None:
        ir_grad = torch.empty((M, n_tiles), dtype=torch.float32, device=g2.device)
        ws = torch.empty(max(raw.bwd_x_workspace_bytes(lib, M, K, n_tiles), 4), dtype=torch.uint8, device=g2.device)
    gate_c = None if gate is None else gate.detach().reshape(-1).to(g2.dtype).contiguous()
    xc = torch.empty_like(x2) if (want_xc and x2 is not None) else None
    raw.cvmm_bwd_x(lib, _stream(g2), g2, w, full, offsets, g_index, out_index, x2, xf_index, gate_c, ir32, ir_grad,
                   bounds, gradient_relative, gradient_scale, decay, input_min_percentage, relu_mask, ws,
                   ir_by_expert, xc)
    return (full, ir_grad, xc) if want_xc else (full, ir_grad)


# ------------------------------------------------------------------------------ companions
def gate_reduce(z: torch.Tensor, gate: torch.Tensor, counter: Optional[torch.Tensor] = None,
                counter_add: int = 0) -> torch.Tensor:
    """y[t] = sum_j gate[t, j] * z[t, j]; z [T*k, D] (or [..., k, D]), gate [..., k].  counter: an int64 device word
    to which the same launch adds counter_add (the step counter of the generated noise)."""
    _need_gpu(z, gate, counter)
    k = gate.shape[-1]
    z2 = _rows2d(z).contiguous()
    T, D = z2.shape[0] // k, z2.shape[1]
    gate_c = gate.detach().reshape(-1).to(z2.dtype).contiguous()
    y = torch.empty((T, D), dtype=z2.dtype, device=z2.device)
    raw.gate_reduce(get_lib(), _stream(z2), z2, gate_c, y, T, k, D, counter, counter_add)
    return y


def gate_reduce_codes(codes: torch.Tensor, scale: torch.Tensor, sel: torch.Tensor, gate: torch.Tensor,
                      counter: Optional[torch.Tensor] = None, counter_add: int = 0) -> torch.Tensor:
    """``gate_reduce`` of a k-head tensor stored as ADC codes (``cvmm_fwd(..., want_codes=True)``); sel [..., k]: the
    expert of every (token, head)."""
    _need_gpu(codes, scale, sel, gate, counter)
    k = gate.shape[-1]
    T, D = codes.shape[0] // k, codes.shape[1]
    gate_c = gate.detach().reshape(-1).contiguous()
    sel_c = sel.detach().reshape(-1).contiguous()
    y = torch.empty((T, D), dtype=gate_c.dtype, device=codes.device)
    raw.gate_reduce_codes(get_lib(), _stream(codes), codes, scale, sel_c, gate_c, y, T, k, D, counter, counter_add)
    return y


def gate_grad_codes(codes: torch.Tensor, scale: torch.Tensor, sel: torch.Tensor, dy: torch.Tensor, k: int) -> torch.Tensor:
    _need_gpu(codes, scale, sel, dy)
    d2 = _rows2d(dy).contiguous()
    T, D = d2.shape
    sel_c = sel.detach().reshape(-1).contiguous()
    out = torch.empty((T, k), dtype=d2.dtype, device=d2.device)
    raw.gate_grad_codes(get_lib(), _stream(d2), codes, scale, sel_c, d2, out, T, k, D)
    return out


def dequant_codes(codes: torch.Tensor, scale: torch.Tensor, sel: torch.Tensor) -> torch.Tensor:
    """The values behind a code tensor, fp32 (tests, debugging): ((code - 128) * scale[e, 0]) * scale[e, 1]."""
    e = sel.reshape(-1).long()
    return ((codes.float() - 128.0) * scale[e, 0:1]) * scale[e, 1:2]


def ksum(full: torch.Tensor, k: int) -> torch.Tensor:
    _need_gpu(full)
    f2 = _rows2d(full).contiguous()
    T, D = f2.shape[0] // k, f2.shape[1]
    out = torch.empty((T, D), dtype=f2.dtype, device=f2.device)
    raw.ksum(get_lib(), _stream(f2), f2, out, T, k, D)
    return out


def ksum_clip_supported(x: torch.Tensor, k: int, bounds: Optional[Sequence[int]]) -> bool:
    """Whether ``ksum_clip`` takes this case: 2 to 8 heads, rows of x and K-tile bounds on 16-byte chunks."""
    ch = 4 if x.dtype == torch.float32 else 8
    x2 = _rows2d(x)
    b = [0, x2.shape[1]] if bounds is None else bounds
    return (1 < k <= 8 and all(int(v) % ch == 0 for v in b) and x2.stride(0) % ch == 0
            and x2.data_ptr() % 16 == 0)


def ksum_clip(full: torch.Tensor, x: torch.Tensor, sel: torch.Tensor, perm: torch.Tensor, offsets: torch.Tensor,
              ir: torch.Tensor, k: int, *, bounds: Optional[Sequence[int]] = None, gradient_relative: bool = True,
              gradient_scale: float = 1.0, decay: float = 0.0, input_min_percentage: float = 0.95):
    """``ksum`` of a per-head input gradient made without masks (``cvmm_bwd_x`` without x and ir), with the
    input-range clip of x [T, D] against ir [E, n_tiles] applied on the way (cvmm.py:848-881, 890-891).
    sel [..., k]: the expert of every (token, head).  Returns (grad_x [T, D], ir_grad [T*k, n_tiles] fp32 by
    sorted position, as ``cvmm_bwd_x`` returns it)."""
    _need_gpu(full, x, sel, perm, offsets, ir)
    lib = get_lib()
    f2 = _rows2d(full).contiguous()
    x2 = _rows2d(x)
    T, D = f2.shape[0] // k, f2.shape[1]
    E = offsets.numel() - 1
    ir32 = _f32c(ir)
    n_tiles = 1 if bounds is None else len(bounds) - 1
    grad_x = torch.empty((T, D), dtype=f2.dtype, device=f2.device)
    ir_grad = torch.empty((T * k, n_tiles), dtype=torch.float32, device=f2.device)
    ws = torch.empty(max(raw.ksum_clip_workspace_bytes(lib, T, k, n_tiles), 4), dtype=torch.uint8, device=f2.device)
    raw.ksum_clip(lib, _stream(f2), f2, x2, sel.detach().reshape(-1).contiguous(), perm, offsets, ir32, grad_x, ir_grad,
                  ws, T, k, E, bounds, gradient_relative, gradient_scale, decay, input_min_percentage)
    return grad_x, ir_grad


def gate_grad(z: torch.Tensor, dy: torch.Tensor, k: int) -> torch.Tensor:
    _need_gpu(z, dy)
    z2, d2 = _rows2d(z).contiguous(), _rows2d(dy).contiguous()
    T, D = d2.shape
    out = torch.empty((T, k), dtype=z2.dtype, device=z2.device)
    raw.gate_grad(get_lib(), _stream(z2), z2, d2, out, T, k, D)
    return out


def row_abs_max(x: torch.Tensor) -> torch.Tensor:
    _need_gpu(x)
    x2 = _rows2d(x)
    out = torch.empty(x2.shape[0], dtype=torch.float32, device=x2.device)
    raw.row_abs_max(get_lib(), _stream(x2), x2, out)
    return out


def weight_abs_max(w: torch.Tensor, per_channel: bool) -> torch.Tensor:
    """[E, N] (per channel) or [E, 1] (per expert) max |w|, fp32."""
    _need_gpu(w)
    wc = w.detach().contiguous()
    E, K, N = wc.shape
    cols = N if per_channel else 1
    out = torch.empty((E, cols), dtype=torch.float32, device=wc.device)
    raw.weight_abs_max(get_lib(), _stream(wc), wc, cols, out)
    return out


def weight_abs_max_pair(w_a: torch.Tensor, w_b: torch.Tensor):
    """Per-expert max |w| of two weight tensors of one layer ([E, 1] fp32 each) from one pair of launches."""
    _need_gpu(w_a, w_b)
    a, b = w_a.detach().contiguous(), w_b.detach().contiguous()
    E = a.shape[0]
    both = torch.empty((2, E, 1), dtype=torch.float32, device=a.device)
    raw.weight_abs_max_pair(get_lib(), _stream(a), a, b, both[0], both[1])
    return both[0], both[1]


def layer_tables(w_a: torch.Tensor, w_b: torch.Tensor, input_range: torch.Tensor, n_up: int, n_dn: int):
    """``weight_abs_max_pair`` and the fp32 input-range tables of the two projections (input_range [2, E, tiles] ->
    [E, n_up], [E, n_dn]) from the same two launches.  Returns (wmax_a, wmax_b, ir_up, ir_dn)."""
    _need_gpu(w_a, w_b, input_range)
    a, b = w_a.detach().contiguous(), w_b.detach().contiguous()
    E = a.shape[0]
    ir = input_range.detach().contiguous()
    both = torch.empty((2, E, 1), dtype=torch.float32, device=a.device)
    ir_up = torch.empty((E, n_up), dtype=torch.float32, device=a.device)
    ir_dn = torch.empty((E, n_dn), dtype=torch.float32, device=a.device)
    raw.layer_tables(get_lib(), _stream(a), a, b, both[0], both[1], ir, n_up, n_dn, ir_up, ir_dn)
    return both[0], both[1], ir_up, ir_dn


def segment_sum(v: torch.Tensor, offsets: torch.Tensor, n_experts: int,
                out: Optional[torch.Tensor] = None, zero_cols: int = 0) -> torch.Tensor:
    """out[e, t] = sum of v[i, t] over expert e's sorted rows (fp32 sums, rounded once to out's type).  ``out``:
    [E, columns of v] to write into (its rows may lie further apart than its columns: a slice of a wider table, whose
    next ``zero_cols`` columns are cleared by the same launch)."""
    _need_gpu(v, offsets)
    cols = 1
    for d in v.shape[1:]:
        cols *= d
    v2 = _f32c(v.reshape(v.shape[0], cols))       # (an explicit column count: v may have no rows)
    if out is None:
        out = torch.empty((n_experts, cols), dtype=torch.float32, device=v2.device)
    if v2.shape[0] == 0:                           # no sorted positions at all: nothing to read
        if zero_cols:
            out.as_strided((n_experts, zero_cols), (out.stride(0), 1), out.storage_offset() + cols).zero_()
        return out.zero_()
    raw.segment_sum(get_lib(), _stream(v2), v2, offsets, n_experts, cols, out, zero_cols)
    return out


def expert_std(x: torch.Tensor, in_index: torch.Tensor, offsets: torch.Tensor, n_experts: int) -> torch.Tensor:
    _need_gpu(x, in_index, offsets)
    x2 = _rows2d(x)
    out = torch.empty(n_experts, dtype=torch.float32, device=x2.device)
    raw.expert_std(get_lib(), _stream(x2), x2, _i32c(in_index), offsets, n_experts, out)
    return out


# ------------------------------------------------------------------------------ weight modifier / clip
def modify_weight(w: torch.Tensor, wmax: torch.Tensor, n_states: float = 0.0, std_dev: float = 0.0,
                  noise: Optional[torch.Tensor] = None, round_noise: bool = True, noise_seed: int = 0,
                  noise_seed_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Modified copy of w [E, K, N]: discretised to multiples of wmax / n_states (n_states > 0), plus
    std_dev * wmax * normal (std_dev > 0).  wmax: fp32 [E, 1] or [E, N] as ``weight_abs_max`` returns it."""
    _need_gpu(w, wmax, noise, noise_seed_dev)
    wc = w.detach().contiguous()
    out = torch.empty_like(wc)
    raw.modify_weight(get_lib(), _stream(wc), wc, _f32c(wmax), n_states, std_dev, _f32c(noise), round_noise,
                      noise_seed, noise_seed_dev, out)
    return out


def weight_std(w: torch.Tensor, per_channel: bool) -> torch.Tensor:
    """Unbiased std of w [E, K, N] over (K, N) -> [E, 1, 1] or over K -> [E, 1, N], fp32."""
    _need_gpu(w)
    lib = get_lib()
    wc = w.detach().contiguous()
    E, K, N = wc.shape
    cols = N if per_channel else 1
    out = torch.empty((E, 1, cols), dtype=torch.float32, device=wc.device)
    nbytes = raw.weight_std_workspace_bytes(lib, E, K, N, cols)
    ws = torch.empty(nbytes // 8, dtype=torch.float64, device=wc.device) if nbytes else None
    raw.weight_std(lib, _stream(wc), wc, cols, out, ws)
    return out


def clamp_weights_(w: torch.Tensor, bound: torch.Tensor) -> torch.Tensor:
    """w = clamp(w, -bound, bound) in place; bound broadcasts as [E, 1, 1] or [E, 1, N]."""
    _need_gpu(w, bound)
    if not w.is_contiguous():
        raise ValueError("clamp_weights_ works in place on a contiguous tensor")
    E, K, N = w.shape
    cols = bound.numel() // E
    if cols not in (1, N) or bound.numel() != E * cols:
        raise ValueError("bound must hold one value per expert or per expert and channel")
    raw.clamp_weights(get_lib(), _stream(w), w.detach(), _f32c(bound), cols)
    return w


# ------------------------------------------------------------------------------ router epilogue
SELECT_MAX_EXPERTS = 512


def select_fwd(logits: torch.Tensor, k: int, want_reg: bool):
    """Gate values [T, k] and expert ids [T, k] (int64) of the k largest sigmoid(logits) per row; with want_reg also
    the usage regulariser (fp32 scalar) and its derivative table [E] for ``select_bwd`` (else two empty tensors)."""
    _need_gpu(logits)
    lib = get_lib()
    lg = logits.detach().contiguous()
    T, E = lg.shape
    sel_val = torch.empty((T, k), dtype=lg.dtype, device=lg.device)
    sel_idx = torch.empty((T, k), dtype=torch.int64, device=lg.device)
    reg = reg_c = ws = None
    if want_reg:
        reg = torch.empty((), dtype=torch.float32, device=lg.device)
        reg_c = torch.empty(E, dtype=torch.float32, device=lg.device)
        ws = torch.empty(max(lib.amoe_select_workspace(T, E) // 4, 1), dtype=torch.float32, device=lg.device)
    raw.select_fwd(lib, _stream(lg), lg, k, sel_val, sel_idx, reg, reg_c, ws)
    if not want_reg:
        reg = torch.empty(0, dtype=torch.float32, device=lg.device)
        reg_c = torch.empty(0, dtype=torch.float32, device=lg.device)
    return sel_val, sel_idx, reg, reg_c


def select_bwd(logits: torch.Tensor, sel_idx: torch.Tensor, grad_val: Optional[torch.Tensor],
               reg_c: Optional[torch.Tensor], grad_reg: Optional[torch.Tensor]) -> torch.Tensor:
    _need_gpu(logits, sel_idx, grad_val, reg_c, grad_reg)
    lg = logits.detach().contiguous()
    out = torch.empty_like(lg)
    if lg.numel() == 0:
        return out
    gv = None if grad_val is None else grad_val.detach().to(lg.dtype).contiguous()
    gr = None if grad_reg is None else grad_reg.detach().to(torch.float32).reshape(1).contiguous()
    raw.select_bwd(get_lib(), _stream(lg), lg, sel_idx.shape[-1], sel_idx.contiguous(), gv,
                   None if gr is None else reg_c, gr, out)
    return out
