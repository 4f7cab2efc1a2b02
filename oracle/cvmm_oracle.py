"""CPU oracle for the CVMM hot path of Analog-MoE.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the arithmetic of the reference's
``analog_moe/triton_src/cvmm.py`` so that the HIP kernels can be checked against it.
Nothing in the shipped package imports it; only ``tests/``, the smoke entry point and
the CPU-baseline leg of the benchmark do, and only as the checker.

Pinned functions (checked in tests/test_oracle.py against library routines, closed
forms, brute force and autograd of an independent per-token formulation):
``prepare_sel``, ``dac``, ``cvmm_fwd`` with one tile and no ADC, ``cvmm_bwd_w``,
``cvmm_backward``, ``expert_std``, ``gate_reduce``.

PARITY UNPINNED (the reference asserts these features off, so no reference behaviour
exists to compare with; the definitions here are this build's own):
``tile_bounds`` / the multi-tile path of ``cvmm_fwd`` and ``cvmm_backward``
(``max_input_size`` splitting), the ADC (``out_bound`` / ``out_res``) stage of
``cvmm_fwd``, and ``counter_noise`` (the in-kernel counter-based Gaussian generator,
which replaces the reference's ``torch.randn`` stream).  The oracle's own statements of these
definitions are checked all the same: the multi-tile backward against autograd of a tile-wise surrogate
and an element-by-element brute force, the tile split and the ADC by their closed-form properties, the
generator by its statistics.

All reference citations are relative to the reference checkout.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------------------
def to_bf16(a: np.ndarray) -> np.ndarray:
    """Round fp32 values to the nearest bf16 (ties to even); result kept in fp32."""
    a = np.ascontiguousarray(a, dtype=F32)
    u = a.view(np.uint32).astype(np.uint64)
    nan = np.isnan(a)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = r.view(F32).copy()
    out[nan] = np.nan
    return out


def to_f16(a: np.ndarray) -> np.ndarray:
    """Round fp32 values to the nearest fp16 (ties to even, overflow to infinity); result kept in fp32."""
    with np.errstate(over="ignore"):
        return np.asarray(a, dtype=F32).astype(np.float16).astype(F32)


def _cast(a: np.ndarray, dtype: str) -> np.ndarray:
    """dtype "f32", "bf16" or "f16" (the reference's reduced-precision type, cvmm.py:177-179, 188-189): the values
    as an element of that type holds them, kept in fp32."""
    if dtype == "f32":
        return np.asarray(a, dtype=F32)
    if dtype == "bf16":
        return to_bf16(a)
    if dtype == "f16":
        return to_f16(a)
    raise ValueError(dtype)


# --------------------------------------------------------------------------------------
# selection: sort, index and offset build
# --------------------------------------------------------------------------------------
@dataclass
class SelOracle:
    sel_sorted: np.ndarray  # [M] int32, ascending expert ids
    perm: np.ndarray        # [M] int32, flat (token, head) index of each sorted position
    in_index: np.ndarray    # [M] int32, perm // k  (token row of each sorted position)
    offsets: np.ndarray     # [E+1] int32, segment start of each expert


def prepare_sel(sel: np.ndarray, n_experts: int, k: int = 1) -> SelOracle:
    """``ssel, perm = sort(sel.flatten())`` (cvmm.py:31-34) with the tie order fixed to
    ascending flat index (stable sort).  ``in_index = perm // k`` and ``out_index = perm``
    are the up-projection's gather/scatter rows (cvmm.py:196-205, 828-833)."""
    flat = np.asarray(sel).reshape(-1).astype(np.int64)
    if flat.size and (flat.min() < 0 or flat.max() >= n_experts):
        raise ValueError("expert id out of range")
    perm = np.argsort(flat, kind="stable")
    ssel = flat[perm]
    counts = np.bincount(flat, minlength=n_experts)
    offsets = np.zeros(n_experts + 1, dtype=np.int64)
    np.cumsum(counts, out=offsets[1:])
    return SelOracle(ssel.astype(np.int32), perm.astype(np.int32),
                     (perm // k).astype(np.int32), offsets.astype(np.int32))


# --------------------------------------------------------------------------------------
# analog building blocks
# --------------------------------------------------------------------------------------
def kernel_inp_res(rpu_inp_res: float) -> float:
    """rpu_config.forward.inp_res -> kernel step (moe_layer_aihwkit_lightning.py:451-456)."""
    if rpu_inp_res > 0:
        return 2.0 / rpu_inp_res if rpu_inp_res > 1.0 else 2.0 * rpu_inp_res
    return -1.0


def tile_bounds(K: int, max_input_size: int) -> np.ndarray:
    """BUILD-DEFINED.  Split K input features into ``ceil(K/max_input_size)`` tiles of
    near-equal size (the first ``K % n`` tiles are one longer).  Returns [n+1] bounds."""
    if max_input_size is None or max_input_size <= 0 or max_input_size >= K:
        return np.array([0, K], dtype=np.int32)
    n = -(-K // max_input_size)
    base, rem = divmod(K, n)
    sizes = [base + (1 if i < rem else 0) for i in range(n)]
    return np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)


def dac(a: np.ndarray, ir: Optional[np.ndarray], abs_max: Optional[np.ndarray], inp_res: float):
    """Input stage of cvmm_kernel (cvmm.py:145-172), fp32, in the reference's op order:
    clamp to +-ir, divide by ir, divide by abs_max, then round(a / inp_res) * inp_res.

    ``a`` [R, K]; ``ir`` and ``abs_max`` broadcastable [R, 1] or None.
    Returns (normalised value fed to the matmul, integer codes or None)."""
    a = np.asarray(a, dtype=F32)
    if ir is not None:
        ir = np.asarray(ir, dtype=F32)
        a = np.where(a > ir, ir, a)
        a = np.where(a < -ir, -ir, a)
        a = (a / ir).astype(F32)
    if abs_max is not None:
        a = (a / np.asarray(abs_max, dtype=F32)).astype(F32)
    codes = None
    if inp_res > 0:
        step = F32(inp_res)
        codes = np.rint((a / step).astype(F32)).astype(F32)  # rint: ties to even (cvmm.py:165-166)
        a = (codes * step).astype(F32)
    return a.astype(F32), codes


def adc_params(out_bound: float, out_res: float):
    """BUILD-DEFINED.  Number of ADC states and whether the stage is active."""
    clip = out_bound is not None and out_bound > 0
    quant = clip and out_res is not None and out_res > 0
    n_states = F32(max(out_res, 1.0 / out_res)) if quant else F32(0)
    return clip, quant, n_states


def adc(c: np.ndarray, wmax_row: np.ndarray, out_bound: float, out_res: float) -> np.ndarray:
    """BUILD-DEFINED output stage, applied in the normalised domain before the rescale by
    ir / abs_max: ``bound = out_bound * wmax``; clamp to +-bound; if ``out_res > 0``:
    ``inv_step = (n_states / 2) / bound``, ``step = bound / (n_states / 2)``,
    ``c = rint(c * inv_step) * step`` with ``n_states = max(out_res, 1 / out_res)``."""
    clip, quant, n_states = adc_params(out_bound, out_res)
    if not clip:
        return c
    bound = (F32(out_bound) * np.asarray(wmax_row, dtype=F32)).astype(F32)
    c = np.minimum(np.maximum(c.astype(F32), -bound), bound).astype(F32)
    if quant:
        half = F32(n_states * F32(0.5))
        inv_step = (half / bound).astype(F32)
        step = (bound / half).astype(F32)
        c = (np.rint((c * inv_step).astype(F32)) * step).astype(F32)
    return c


# --------------------------------------------------------------------------------------
# counter-based Gaussian noise (BUILD-DEFINED; replaces torch.randn of
# moe_layer_aihwkit_lightning.py:472-477 so that noise can be produced inside the kernel:
# the noise of a 32 x 32 block of outputs is a product of two matrices of pseudo-random
# signed bytes, which the kernel forms with one 8-bit matrix instruction)
# --------------------------------------------------------------------------------------
def _fmix32(h: np.ndarray) -> np.ndarray:
    h = h.astype(np.uint32)
    h ^= h >> np.uint32(16)
    h = (h.astype(np.uint64) * np.uint64(0x85EBCA6B) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    h ^= h >> np.uint32(13)
    h = (h.astype(np.uint64) * np.uint64(0xC2B2AE35) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    h ^= h >> np.uint32(16)
    return h


def _u32(v) -> np.ndarray:
    return (np.asarray(v, dtype=np.uint64) & np.uint64(0xFFFFFFFF)).astype(np.uint32)


def box_muller_noise(rows: np.ndarray, n_cols: int, tile: int, seed: int) -> np.ndarray:
    """The generator of the weight modifier's normals (``weights_oracle.modifier_normals``): standard-normal
    values for rows ``rows``, all ``n_cols`` columns, stream ``tile``; a pure function of (seed, tile, row, column).

    Columns are paired (2p, 2p+1).  Two 32-bit keys come from the seed halves and the tile.  The
    row gets the key ``fmix32(row ^ ka)``; the pair's word is that key plus ``p * 0x9E3779B9``,
    run through the two multiply / xor-shift rounds of the murmur3 finaliser with the second key
    added between them; the 16-bit halves of the result give u1 in (0,1) and u2 in [0,1);
    Box-Muller gives the pair (r cos 2 pi u2, r sin 2 pi u2), r = sqrt(-2 ln u1).
    n_cols must be even; rows and pair indices are taken modulo 2**32."""
    assert n_cols % 2 == 0
    rows = _u32(np.asarray(rows, dtype=np.uint64)).reshape(-1, 1)
    p = np.arange(n_cols // 2, dtype=np.uint64).reshape(1, -1)
    s_lo, s_hi = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    ka = _fmix32(_u32((s_lo ^ 0x9E3779B9) + tile * 0x632BE5AB))
    kb = _fmix32(_u32((s_hi ^ 0x85EBCA77) + tile * 0x27D4EB2F))
    row_key = _fmix32(rows ^ ka)
    h = _u32(row_key.astype(np.uint64) + p * np.uint64(0x9E3779B9))
    h ^= h >> np.uint32(16)
    h = _u32(h.astype(np.uint64) * np.uint64(0x85EBCA6B))
    h = _u32(h.astype(np.uint64) + np.uint64(kb))
    h ^= h >> np.uint32(13)
    h = _u32(h.astype(np.uint64) * np.uint64(0xC2B2AE35))
    h ^= h >> np.uint32(16)
    u1 = ((h >> np.uint32(16)).astype(F32) + F32(0.5)) * F32(1.0 / 65536.0)
    u2 = (h & np.uint32(0xFFFF)).astype(F32) * F32(1.0 / 65536.0)
    r = np.sqrt(F32(-2.0) * np.log(u1.astype(np.float64)))
    ang = 2.0 * np.pi * u2.astype(np.float64)
    out = np.empty((rows.shape[0], n_cols), dtype=F32)
    out[:, 0::2] = (r * np.cos(ang)).astype(F32)
    out[:, 1::2] = (r * np.sin(ang)).astype(F32)
    return out


NOISE_MULTIPLIERS = (0x9E3779, 0x85EBCB, 0xC2B2AF, 0x27D4EB)
NOISE_HALF_KEY = 0x5BD1E995
NOISE_SCALE = F32(1.0 / (5.656854249492380195 * 5461.5))     # 1 / (sqrt(32) * std of a product of two bytes)


def _noise_words(keys: np.ndarray) -> np.ndarray:
    """keys [...] uint32 -> [..., 32] signed bytes.  Words 0..3 come from the key, words 4..7 from
    ``key ^ NOISE_HALF_KEY``; word j is ``w = (k mod 2^24) * c_(j mod 4) + k``, ``w ^= w >> 15`` with the odd
    24-bit multipliers ``NOISE_MULTIPLIERS``; bytes little-endian."""
    keys = np.asarray(keys, dtype=np.uint32)
    out = np.empty(keys.shape + (32,), dtype=np.int64)
    for j in range(8):
        k = keys ^ np.uint32(NOISE_HALF_KEY if j >= 4 else 0)
        cj = np.uint64(NOISE_MULTIPLIERS[j % 4])
        w = _u32((k & np.uint32(0xFFFFFF)).astype(np.uint64) * cj + k.astype(np.uint64))
        w ^= w >> np.uint32(15)
        for b in range(4):
            v = ((w >> np.uint32(8 * b)) & np.uint32(0xFF)).astype(np.int64)
            out[..., 4 * j + b] = np.where(v >= 128, v - 256, v)
    return out


def counter_noise_int(rows: np.ndarray, block_starts: np.ndarray, n_cols: int, tile: int, seed: int) -> np.ndarray:
    """Integer noise [R, n_cols] for output rows ``rows`` (output-row ids) whose 32-row block starts at sorted
    position ``block_starts[i]``; K-tile ``tile``.  A pure function of (seed, tile, output row, block start,
    column): for the 32 x 32 block of a row block and a column block c // 32,
        z[row][col] = sum_k a[row][k] * b[col][k] - 8
    with the signed bytes  a[row] = words(fmix32(row ^ ka) ^ (col // 32) * 0x632BE5AB)  and
    b[col] = words(fmix32(col * 0x9E3779B1 ^ kb) ^ block_start * 0x27D4EB2F); ka, kb are the two 32-bit keys
    of (seed, tile).  Mean 0, standard deviation 1 / NOISE_SCALE, close to normal (a sum of 32 products)."""
    rows = _u32(np.asarray(rows, dtype=np.uint64)).reshape(-1)
    block_starts = _u32(np.asarray(block_starts, dtype=np.uint64)).reshape(-1)
    s_lo, s_hi = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    ka = _fmix32(_u32((s_lo ^ 0x9E3779B9) + tile * 0x632BE5AB))
    kb = _fmix32(_u32((s_hi ^ 0x85EBCA77) + tile * 0x27D4EB2F))
    row_key = _fmix32(rows ^ ka)                                                     # [R]
    cols = np.arange(n_cols, dtype=np.uint64)
    col_key = _fmix32(_u32(cols * np.uint64(0x9E3779B1)) ^ kb)                       # [N]
    n_cb = (n_cols + 31) // 32
    out = np.zeros((rows.shape[0], n_cols), dtype=np.int64)
    ustarts, inv = np.unique(block_starts, return_inverse=True)
    # b vectors per (block start, column)
    bkeys = col_key[None, :] ^ _u32(ustarts[:, None].astype(np.uint64) * np.uint64(0x27D4EB2F))
    bvec = _noise_words(bkeys)                                                       # [S, N, 32]
    for cb in range(n_cb):
        c0, c1 = cb * 32, min(cb * 32 + 32, n_cols)
        akeys = row_key ^ _u32(np.uint64(cb) * np.uint64(0x632BE5AB))
        avec = _noise_words(akeys)                                                   # [R, 32]
        out[:, c0:c1] = np.einsum("rk,rck->rc", avec, bvec[inv, c0:c1]) - 8
    return out


def counter_noise(rows: np.ndarray, block_starts: np.ndarray, n_cols: int, tile: int, seed: int) -> np.ndarray:
    """``counter_noise_int`` scaled to unit variance (fp32)."""
    return (counter_noise_int(rows, block_starts, n_cols, tile, seed).astype(F32) * NOISE_SCALE).astype(F32)


# --------------------------------------------------------------------------------------
# forward
# --------------------------------------------------------------------------------------
def cvmm_fwd(x, sel_index, sel_sorted, keys, inp_res=-1.0, ir=None, out_index=None,
             abs_max=None, noise=None, *, bounds: Optional[Sequence[int]] = None,
             wmax=None, out_bound=-1.0, out_res=-1.0, noise_std=0.0, noise_seed=None,
             dtype="f32", relu=False, return_codes=False):
    """cvmm_kernel (cvmm.py:89-231) row by row, grouped per expert.

    x [R_in, K]; sel_index [M] input row per sorted position; sel_sorted [M] expert per
    sorted position; keys [E, K, N]; ir [M] or [M, n_tiles] per sorted position (None =
    off); out_index [M] output row per sorted position (None -> sel_index);
    abs_max [R_in] per input row (None = off); noise [n_tiles, M_out, N] or [M_out, N]
    per OUTPUT row, already scaled (None = off), or generated from ``noise_seed`` as
    ``noise_std * wmax[e] * counter_noise``.  wmax [E, N] or [E, 1].

    Per tile t with K-range [b_t, b_t+1):
        c_t = dac(x[:, range]) @ W[e][range, :]  (+ noise_t)  -> adc -> * abs_max * ir_t
    out = sum_t c_t.  With one tile and no ADC this is exactly cvmm.py:136-231.
    dtype "bf16": operands are rounded to bf16 where the kernel feeds them to the matrix
    unit (integer codes are exact in bf16, so with quantisation on only the weights round)
    and the result is rounded to bf16 on store.
    """
    x = np.asarray(x, dtype=F32)
    keys = np.asarray(keys, dtype=F32)
    E, K, N = keys.shape
    M = sel_sorted.shape[0]
    sel_index = np.asarray(sel_index).astype(np.int64)
    oidx = sel_index if out_index is None else np.asarray(out_index).astype(np.int64)
    bounds = np.array([0, K]) if bounds is None else np.asarray(bounds)
    T = len(bounds) - 1
    if ir is not None:
        ir = np.asarray(ir, dtype=F32).reshape(M, -1)
        assert ir.shape[1] == T
    if noise is not None:
        noise = np.asarray(noise, dtype=F32)
        noise = noise.reshape(T, -1, N)
    if wmax is not None:
        wmax = np.asarray(wmax, dtype=F32).reshape(E, -1)
    out = np.zeros((M, N), dtype=F32)
    codes_all = np.zeros((M, K), dtype=F32) if return_codes else None
    w_op = _cast(keys, dtype)
    for e in np.unique(sel_sorted):
        pos = np.nonzero(sel_sorted == e)[0]
        rin = sel_index[pos]
        rout = oidx[pos]
        amax = None if abs_max is None else np.asarray(abs_max, dtype=F32).reshape(-1)[rin][:, None]
        total = np.zeros((len(pos), N), dtype=F32)
        for t in range(T):
            lo, hi = int(bounds[t]), int(bounds[t + 1])
            ir_t = None if ir is None else ir[pos, t][:, None]
            a, codes = dac(x[rin, lo:hi], ir_t, amax, inp_res)
            if return_codes and codes is not None:
                codes_all[pos, lo:hi] = codes
            if dtype != "f32" and codes is None:
                a = _cast(a, dtype)
            c = (a.astype(np.float64) @ w_op[e, lo:hi, :].astype(np.float64)).astype(F32)
            if noise is not None:
                c = (c + noise[t, rout, :]).astype(F32)
            elif noise_seed is not None and noise_std > 0:
                # 32-row blocks are counted from the expert's first sorted position
                starts = pos[0] + (np.arange(len(pos)) // 32) * 32
                zi = counter_noise_int(rout, starts, N, t, noise_seed).astype(F32)
                nz = ((F32(noise_std) * wmax[e][None, :]).astype(F32) * NOISE_SCALE).astype(F32)
                # one fused multiply-add, as the kernel does it (the product is exact in float64)
                c = (zi.astype(np.float64) * nz.astype(np.float64) + c.astype(np.float64)).astype(F32)
            if out_bound is not None and out_bound > 0:
                c = adc(c, wmax[e][None, :], out_bound, out_res)
            if amax is not None:
                c = (c * amax).astype(F32)
            if ir_t is not None:
                c = (c * ir_t).astype(F32)
            total = (total + c).astype(F32)
        if relu:
            total = np.maximum(total, F32(0))
        out[rout] = total
    out = _cast(out, dtype)
    if return_codes:
        return out, codes_all
    return out


def gate_reduce(z: np.ndarray, gate: np.ndarray, dtype="f32") -> np.ndarray:
    """y[t,:] = sum_k gate[t,k] * z[t,k,:]  (cvmm.py:757-759)."""
    T, k = gate.shape
    z = np.asarray(z, dtype=F32).reshape(T, k, -1)
    y = np.einsum("tk,tkd->td", gate.astype(np.float64), z.astype(np.float64))
    return _cast(y.astype(F32), dtype)


# --------------------------------------------------------------------------------------
# backward
# --------------------------------------------------------------------------------------
def _clip_rows(xr, ir, bounds):
    """clamp(x, +-ir) per K-tile, no scaling (cvmm.py:365-373)."""
    if ir is None:
        return xr
    out = xr.copy()
    for t in range(len(bounds) - 1):
        lo, hi = int(bounds[t]), int(bounds[t + 1])
        r = ir[:, t][:, None]
        out[:, lo:hi] = np.minimum(np.maximum(xr[:, lo:hi], -r), r)
    return out


def cvmm_bwd_w(x, sel_index, sel_sorted, grads, ir, n_experts, out_index=None, *,
               bounds=None, dtype="f32"):
    """cvmm_backward_kernel3 (cvmm.py:285-397):
    grad_W[e] = sum_{j in e} clamp(x[sel_index[j]], +-ir_j)^T  g[out_index[j] or sel_index[j]].
    Experts with no rows get zeros (cvmm.py:671)."""
    x = np.asarray(x, dtype=F32)
    grads = np.asarray(grads, dtype=F32)
    K, N = x.shape[1], grads.shape[1]
    M = sel_sorted.shape[0]
    sel_index = np.asarray(sel_index).astype(np.int64)
    gidx = sel_index if out_index is None else np.asarray(out_index).astype(np.int64)
    bounds = np.array([0, K]) if bounds is None else np.asarray(bounds)
    if ir is not None:
        ir = np.asarray(ir, dtype=F32).reshape(M, -1)
    out = np.zeros((n_experts, K, N), dtype=np.float64)
    for e in np.unique(sel_sorted):
        pos = np.nonzero(sel_sorted == e)[0]
        a = _clip_rows(x[sel_index[pos]], None if ir is None else ir[pos], bounds)
        if dtype != "f32":
            a = _cast(a, dtype)
        out[e] = a.astype(np.float64).T @ grads[gidx[pos]].astype(np.float64)
    return _cast(out.astype(F32), dtype)


@dataclass
class BwdOracle:
    grad_x: np.ndarray
    grad_w: np.ndarray
    ir_grad: Optional[np.ndarray]      # [M, n_tiles] in sorted order
    grad_gate: Optional[np.ndarray]    # [T, k]
    grad_x_full: np.ndarray            # [M_out, K] masked, gate-scaled, before the k-sum


def cvmm_backward(grad_output, x, keys, sel_sorted, sel_index, out_index, gate, ir, z, *,
                  k: int, decay=0.0, input_min_percentage=0.95, gradient_relative=True,
                  gradient_scale=1.0, bounds=None, dtype="f32", relu_mask=False):
    """CVMM.backward (cvmm.py:772-897).

    Up-projection call: x [T, K], sel_index = perm // k, out_index = perm, gate None,
    grad_output [M, N].  Down-projection call: x [M, K], sel_index = perm, out_index None,
    gate [T, k], grad_output [T, N], z = un-reduced forward output [M, N].

    Straight-through: quantiser, abs_max scaling, noise and ADC are identity in backward;
    the clip contributes the strict mask |x| < ir (cvmm.py:853, 881).
    ``relu_mask`` (fused-layer extension): additionally multiply grad_x by (x > 0)."""
    x = np.asarray(x, dtype=F32)
    keys = np.asarray(keys, dtype=F32)
    E, K, N = keys.shape
    M = sel_sorted.shape[0]
    g = np.asarray(grad_output, dtype=F32).reshape(-1, N)
    sel_index = np.asarray(sel_index).astype(np.int64)
    bounds = np.array([0, K]) if bounds is None else np.asarray(bounds)
    nt = len(bounds) - 1
    if ir is not None:
        ir = np.asarray(ir, dtype=F32).reshape(M, nt)

    if gate is not None:                                   # cvmm.py:785-789
        gflat = np.asarray(gate, dtype=F32).reshape(-1)
        g_w = _cast((gflat[:, None] * np.repeat(g, k, axis=0)).astype(F32), dtype)
    else:
        gflat = None
        g_w = g
    grad_w = cvmm_bwd_w(x, sel_index, sel_sorted, g_w, ir, E, out_index,
                        bounds=bounds, dtype=dtype)       # cvmm.py:812-823

    # cvmm.py:828-846: plain gather-GEMM-scatter with W^T
    pos_out = sel_index if out_index is None else np.asarray(out_index).astype(np.int64)
    g_rows = pos_out // k if gate is not None else pos_out  # row of grad_output per sorted pos
    w_op = _cast(keys, dtype)
    full = np.zeros((M, K), dtype=F32)                      # indexed by output row
    ir_grad = None if ir is None else np.zeros((M, nt), dtype=F32)
    xs = x[sel_index]                                       # sorted order (cvmm.py:851)
    n_not_clip = 0
    for e in np.unique(sel_sorted):
        pos = np.nonzero(sel_sorted == e)[0]
        full[pos_out[pos]] = (g[g_rows[pos]].astype(np.float64)
                              @ w_op[e].astype(np.float64).T).astype(F32)
    full = _cast(full, dtype) if dtype != "f32" else full
    full_sorted = full[pos_out]                             # cvmm.py:859
    scale_sorted = np.ones((M, 1), dtype=F32) if gflat is None else gflat[pos_out][:, None]
    if ir is not None:
        gs = (full_sorted * scale_sorted).astype(F32)       # cvmm.py:860-861
        mask_sorted = np.zeros((M, K), dtype=bool)
        for t in range(nt):
            lo, hi = int(bounds[t]), int(bounds[t + 1])
            r = ir[:, t][:, None]
            xt = xs[:, lo:hi]
            not_clip = np.abs(xt) < r                       # cvmm.py:853 (strict)
            upper = xt >= r                                 # cvmm.py:856
            lower = xt <= -r                                # cvmm.py:857
            gt = gs[:, lo:hi].astype(np.float64)
            acc = np.minimum(upper * gt, 0.0).sum(-1) - np.maximum(lower * gt, 0.0).sum(-1)
            ir_grad[:, t] = acc.astype(F32)                 # cvmm.py:863-865
            mask_sorted[:, lo:hi] = not_clip
        n_not_clip = mask_sorted.sum()
        if gradient_relative:                               # cvmm.py:868-870
            ir_grad = (ir_grad * ir * F32(gradient_scale)).astype(F32)
        if decay > 0:                                       # cvmm.py:872-878
            pct = F32(n_not_clip) / F32(M * K)
            ir_grad = (ir_grad + F32(decay) * ir * F32(pct > input_min_percentage)).astype(F32)
        full_sorted = full_sorted * mask_sorted             # cvmm.py:881
    if relu_mask:
        full_sorted = full_sorted * (xs > 0)
    full_sorted = (full_sorted * scale_sorted).astype(F32)  # gate scaling (cvmm.py:888)
    full_out = np.zeros((M, K), dtype=F32)
    full_out[pos_out] = full_sorted
    full_out = _cast(full_out, dtype)

    grad_gate = None
    if gate is not None:
        grad_x = full_out.reshape(x.shape)                  # cvmm.py:888
        zz = np.asarray(z, dtype=F32).reshape(-1, k, N)
        grad_gate = np.einsum("tkn,tn->tk", zz.astype(np.float64),
                              g.astype(np.float64)).astype(F32)  # cvmm.py:889
    else:
        grad_x = full_out.reshape(-1, k, K).astype(np.float64).sum(1).astype(F32)  # cvmm.py:890-891
        grad_x = _cast(grad_x, dtype)
    return BwdOracle(grad_x, grad_w, ir_grad, grad_gate, full_out)


# --------------------------------------------------------------------------------------
# per-expert std (input-range initialisation from data)
# --------------------------------------------------------------------------------------
def expert_std(x, sel_index, sel_sorted, n_experts) -> np.ndarray:
    """cvmm_std (cvmm.py:400-443): unbiased std over all elements of the rows routed to
    each expert.  The reference's second kernel launches cdiv(N, BLOCK_N) redundant
    column programs that each add the full row sums (cvmm.py:437-439, 463-465, 480-489),
    which inflates both numerator and count by that factor; this oracle returns the exact
    unbiased estimate sqrt(SS / (n - 1)) the function documents.  An expert with no rows
    gives sqrt(0 / -1) = -0.0, which the caller filters with ``stds > 0``
    (moe_layer_aihwkit_lightning.py:439-443)."""
    x = np.asarray(x, dtype=F32)
    sel_index = np.asarray(sel_index).astype(np.int64)
    out = np.zeros(n_experts, dtype=F32)
    for e in range(n_experts):
        pos = np.nonzero(sel_sorted == e)[0]
        if len(pos) == 0:
            out[e] = F32(-0.0)
            continue
        v = x[sel_index[pos]].astype(np.float64).reshape(-1)
        mean = v.mean()
        ss = ((v - mean) ** 2).sum()
        with np.errstate(divide="ignore", invalid="ignore"):
            out[e] = F32(np.sqrt(ss / (v.size - 1)))
    return out


# --------------------------------------------------------------------------------------
# whole layer: router output -> y, and its backward, composed from the pieces above
# --------------------------------------------------------------------------------------
@dataclass
class LayerOracle:
    y: np.ndarray
    scores: np.ndarray       # [M, F] post-activation up-projection output, flat (t, k) rows
    z: np.ndarray            # [M, D] un-reduced down-projection output
    sel: SelOracle
    grad_x: Optional[np.ndarray] = None
    grad_keys: Optional[np.ndarray] = None
    grad_values: Optional[np.ndarray] = None
    grad_gate: Optional[np.ndarray] = None
    grad_ir: Optional[np.ndarray] = None    # [2, E, n_tiles]: per-expert sums (index backward of
                                            # input_range[sel], moe_layer_aihwkit_lightning.py:447-448)


def layer_fwd_bwd(x, keys, values, sel_idx, sel_val, ir=None, dy=None, *, inp_res=-1.0,
                  noise_up=None, noise_down=None, wmax_up=None, wmax_down=None,
                  noise_std=0.0, noise_seed=None, out_bound=-1.0, out_res=-1.0,
                  bounds_up=None, bounds_down=None, decay=0.0, input_min_percentage=0.95,
                  gradient_relative=True, gradient_scale=1.0, dtype="f32",
                  scores_override=None, z_override=None) -> LayerOracle:
    """SigmaMoE FFN with analog experts: y[t] = sum_h gate[t,h] * A(relu(A(x[t], keys[e])), values[e])
    (per-token form in test_moe_layer_aihwkit_lightning.py:82-107), built from the CVMM
    calls of moe_layer_aihwkit_lightning.py:384-410, 494-506.  ir: [2, E, n_tiles] or None.

    ``scores_override`` / ``z_override``: continue from these stage outputs instead of the
    oracle's own (the returned ``scores`` / ``z`` stay the oracle's).  An output quantiser
    turns a last-bit difference in the accumulation into a whole ADC step for the few values
    that sit on a rounding boundary; checking stage by stage keeps such flips from leaking
    into the comparison of the later stages."""
    x = np.asarray(x, dtype=F32)
    T, D = x.shape
    E, _, Fdim = keys.shape
    k = sel_idx.shape[1]
    s = prepare_sel(sel_idx, E, k)
    bu = np.array([0, D]) if bounds_up is None else np.asarray(bounds_up)
    bd = np.array([0, Fdim]) if bounds_down is None else np.asarray(bounds_down)
    ir_up = ir_dn = None
    if ir is not None:
        ir = np.asarray(ir, dtype=F32).reshape(2, E, -1)
        ir_up = ir[0][s.sel_sorted][:, :len(bu) - 1]
        ir_dn = ir[1][s.sel_sorted][:, :len(bd) - 1]
    seed_up = None if noise_seed is None else noise_seed
    seed_dn = None if noise_seed is None else noise_seed + 1
    p1 = cvmm_fwd(x, s.in_index, s.sel_sorted, keys, inp_res, ir_up, s.perm, None, noise_up,
                  bounds=bu, wmax=wmax_up, out_bound=out_bound, out_res=out_res,
                  noise_std=noise_std, noise_seed=seed_up, dtype=dtype, relu=True)
    p1_own = p1
    if scores_override is not None:
        p1 = np.asarray(scores_override, dtype=F32).reshape(p1.shape)
    z = cvmm_fwd(p1, s.perm, s.sel_sorted, values, inp_res, ir_dn, None, None, noise_down,
                 bounds=bd, wmax=wmax_down, out_bound=out_bound, out_res=out_res,
                 noise_std=noise_std, noise_seed=seed_dn, dtype=dtype)
    z_own = z
    if z_override is not None:
        z = np.asarray(z_override, dtype=F32).reshape(z.shape)
    gate = _cast(np.asarray(sel_val, dtype=F32), dtype)
    y = gate_reduce(z, gate, dtype)
    res = LayerOracle(y, p1_own, z_own, s)
    if dy is None:
        return res
    kw = dict(k=k, decay=decay, input_min_percentage=input_min_percentage,
              gradient_relative=gradient_relative, gradient_scale=gradient_scale, dtype=dtype)
    bdn = cvmm_backward(dy, p1, values, s.sel_sorted, s.perm, None, gate, ir_dn, z,
                        bounds=bd, relu_mask=True, **kw)
    bup = cvmm_backward(bdn.grad_x, x, keys, s.sel_sorted, s.in_index, s.perm, None, ir_up, None,
                        bounds=bu, **kw)
    res.grad_x, res.grad_keys, res.grad_values, res.grad_gate = bup.grad_x, bup.grad_w, bdn.grad_w, bdn.grad_gate
    if ir is not None:
        nt = ir.shape[2]
        gi = np.zeros((2, E, nt), dtype=np.float64)
        np.add.at(gi[0, :, :len(bu) - 1], s.sel_sorted, bup.ir_grad.astype(np.float64))
        np.add.at(gi[1, :, :len(bd) - 1], s.sel_sorted, bdn.ir_grad.astype(np.float64))
        res.grad_ir = gi.astype(F32)
    return res
