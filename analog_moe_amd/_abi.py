"""ctypes declarations of the C ABI in include/amoe.h (struct layouts and prototypes).

Pure declarations: binding a handle does not touch the GPU.  Pointers are passed as plain
integers (``tensor.data_ptr()``), NULL as 0/None.
"""
from __future__ import annotations

import ctypes as C

AMOE_MAX_TILES = 16
AMOE_F32, AMOE_BF16, AMOE_F16 = 0, 1, 2
P = C.c_void_p


class FwdArgs(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("E", C.c_int32),
        ("n_in_rows", C.c_int32), ("n_out_rows", C.c_int32),
        ("x", P), ("ldx", C.c_int64),
        ("w", P), ("w_stride_e", C.c_int64), ("w_stride_k", C.c_int64), ("w_stride_n", C.c_int64),
        ("out", P), ("ldo", C.c_int64),
        ("sel_sorted", P), ("offsets", P), ("in_index", P), ("out_index", P),
        ("ir", P), ("ir_by_expert", C.c_int32), ("abs_max", P), ("inp_res", C.c_float),
        ("n_tiles", C.c_int32), ("tile_bounds", C.c_int32 * (AMOE_MAX_TILES + 1)),
        ("noise", P), ("noise_tile_stride", C.c_int64), ("ldnoise", C.c_int64),
        ("noise_std", C.c_float), ("noise_seed", C.c_uint64), ("noise_seed_dev", C.c_void_p),
        ("wmax", P), ("wmax_cols", C.c_int32),
        ("out_bound", C.c_float), ("out_res", C.c_float),
        ("relu", C.c_int32), ("range_flag", P),
        ("xq_out", P), ("ldxq", C.c_int64), ("xq_ir", P), ("xq_inp_res", C.c_float), ("x_is_quantized", C.c_int32),
        ("code_out", P), ("ldcode", C.c_int64), ("code_scale_out", P),
    ]


class BwdWArgs(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("E", C.c_int32),
        ("x", P), ("ldx", C.c_int64), ("g", P), ("ldg", C.c_int64), ("grad_w", P),
        ("offsets", P), ("in_index", P), ("g_index", P), ("ir", P), ("ir_by_expert", C.c_int32),
        ("g_scale", P), ("n_x_rows", C.c_int64), ("n_g_rows", C.c_int64),
        ("n_tiles", C.c_int32), ("tile_bounds", C.c_int32 * (AMOE_MAX_TILES + 1)),
        ("workspace", P), ("workspace_bytes", C.c_size_t), ("rows_per_chunk", C.c_int32),
    ]


class BwdXArgs(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("E", C.c_int32),
        ("g", P), ("ldg", C.c_int64), ("n_g_rows", C.c_int32),
        ("w", P), ("w_stride_e", C.c_int64), ("w_stride_k", C.c_int64),
        ("grad_x_full", P), ("ldo", C.c_int64),
        ("x", P), ("ldx", C.c_int64),
        ("offsets", P), ("g_index", P), ("out_index", P), ("xf_index", P),
        ("gate", P), ("ir", P), ("ir_by_expert", C.c_int32), ("ir_grad", P),
        ("n_tiles", C.c_int32), ("tile_bounds", C.c_int32 * (AMOE_MAX_TILES + 1)),
        ("gradient_relative", C.c_int32), ("gradient_scale", C.c_float),
        ("decay", C.c_float), ("input_min_percentage", C.c_float),
        ("relu_mask", C.c_int32),
        ("workspace", P), ("workspace_bytes", C.c_size_t), ("xc_out", P), ("ldxc", C.c_int64),
    ]


class KsumClipArgs(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("T", C.c_int64), ("k", C.c_int32), ("D", C.c_int32), ("E", C.c_int32),
        ("full", P), ("x", P), ("ldx", C.c_int64), ("sel", P), ("sel_is_i64", C.c_int32),
        ("perm", P), ("offsets", P), ("ir", P),
        ("n_tiles", C.c_int32), ("tile_bounds", C.c_int32 * (AMOE_MAX_TILES + 1)),
        ("grad_x", P), ("ir_grad", P),
        ("gradient_relative", C.c_int32), ("gradient_scale", C.c_float),
        ("decay", C.c_float), ("input_min_percentage", C.c_float),
        ("workspace", P), ("workspace_bytes", C.c_size_t),
    ]


I32, I64, F32, SZ = C.c_int32, C.c_int64, C.c_float, C.c_size_t

PROTOTYPES = {
    "amoe_version": (C.c_int, []),
    "amoe_strerror": (C.c_char_p, [C.c_int]),
    "amoe_prepare_sel_workspace": (SZ, [I64, I32]),
    "amoe_prepare_sel": (C.c_int, [P, I32, I64, I32, I32, P, P, P, P, P, P, SZ, P]),
    "amoe_noalloc_scratch_bytes": (SZ, []),
    "amoe_prepare_sel_noalloc": (C.c_int, [P, I32, I64, I32, I32, P, P, P, P, P, P]),
    "amoe_offsets_from_sorted": (C.c_int, [P, I64, I32, P, P]),
    "amoe_cvmm_fwd": (C.c_int, [C.POINTER(FwdArgs), P]),
    "amoe_fwd_codes_supported": (C.c_int, [C.POINTER(FwdArgs)]),
    "amoe_bwd_w_workspace": (SZ, [C.POINTER(BwdWArgs)]),
    "amoe_cvmm_bwd_w": (C.c_int, [C.POINTER(BwdWArgs), P]),
    "amoe_bwd_x_workspace": (SZ, [I64, I32, I32]),
    "amoe_cvmm_bwd_x": (C.c_int, [C.POINTER(BwdXArgs), P]),
    "amoe_gate_reduce": (C.c_int, [I32, P, P, P, I64, I32, I32, P, I64, P]),
    "amoe_ksum": (C.c_int, [I32, P, P, I64, I32, I32, P]),
    "amoe_ksum_clip_workspace": (SZ, [I64, I32, I32]),
    "amoe_ksum_clip": (C.c_int, [C.POINTER(KsumClipArgs), P]),
    "amoe_gate_grad": (C.c_int, [I32, P, P, P, I64, I32, I32, P]),
    "amoe_gate_reduce_codes": (C.c_int, [I32, P, P, P, I32, P, P, I64, I32, I32, P, I64, P]),
    "amoe_gate_grad_codes": (C.c_int, [I32, P, P, P, I32, P, P, I64, I32, I32, P]),
    "amoe_row_abs_max": (C.c_int, [I32, P, I64, I64, I32, P, P]),
    "amoe_weight_abs_max": (C.c_int, [I32, P, I32, I32, I32, I32, P, P]),
    "amoe_weight_abs_max_pair": (C.c_int, [I32, P, I32, I32, P, P, I32, I32, P, I32, P]),
    "amoe_layer_tables": (C.c_int, [I32, P, I32, I32, P, P, I32, I32, P, I32, I32, P, I32, I32, P, I32, P, P]),
    "amoe_segment_sum": (C.c_int, [P, P, I32, I32, I32, P, I64, I32, P]),
    "amoe_expert_std": (C.c_int, [I32, P, I64, I32, P, P, I32, P, P]),
    "amoe_modify_weight": (C.c_int, [I32, P, I32, I32, I32, P, I32, F32, F32, P, I32, C.c_uint64, P, P, P]),
    "amoe_weight_std_workspace": (SZ, [I32, I32, I32, I32]),
    "amoe_weight_std": (C.c_int, [I32, P, I32, I32, I32, I32, P, P, SZ, P]),
    "amoe_clamp_weights": (C.c_int, [I32, P, I32, I32, I32, P, I32, P]),
    "amoe_select_workspace": (SZ, [I64, I32]),
    "amoe_select_fwd": (C.c_int, [I32, P, I64, I32, I32, P, P, P, P, P, SZ, P]),
    "amoe_select_bwd": (C.c_int, [I32, P, I64, I32, I32, P, P, P, P, P, P]),
}


def bind(path: str) -> C.CDLL:
    """Load a build of the library and attach the prototypes.  Raises if a symbol is missing."""
    lib = C.CDLL(path)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def set_bounds(args, bounds) -> None:
    n = len(bounds) - 1
    if n < 1 or n > AMOE_MAX_TILES:
        raise ValueError(f"number of K-tiles must be in [1, {AMOE_MAX_TILES}]")
    args.n_tiles = n
    for i, b in enumerate(bounds):
        args.tile_bounds[i] = int(b)


class AmoeError(RuntimeError):
    rc = 0


AMOE_EUNSUPPORTED = -6


def check(lib, rc: int, what: str) -> None:
    if rc != 0:
        err = AmoeError(f"{what}: {lib.amoe_strerror(rc).decode()} (rc={rc})")
        err.rc = rc
        raise err
