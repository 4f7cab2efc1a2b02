"""CPU parity tests of the HIP kernels' own source, compiled for the host with the stand-in
headers of tests/emu (one thread per GPU thread).  They check index arithmetic, masking, tile
scheduling and the analog pro/epilogues against the oracle without a GPU; the matrix
instruction and LDS-transpose stand-ins reproduce the operand layouts measured on MI355X.
The product path is untouched: these tests point analog_moe_amd.ops at the host build by
monkeypatching."""
import os
import subprocess

import numpy as np
import pytest
import torch

from analog_moe_amd import _abi, ops
from oracle import cvmm_oracle as O
from tests import util

HERE = os.path.dirname(os.path.abspath(__file__))
EMU_SO = os.path.join(HERE, "emu", "libamoe_emu.so")


@pytest.fixture(scope="module")
def emu_ops():
    src = [os.path.join(HERE, "..", "analog_moe_amd", "csrc", f) for f in os.listdir(
        os.path.join(HERE, "..", "analog_moe_amd", "csrc")) if f.endswith((".h", ".hip"))]
    src += [os.path.join(HERE, "emu", "gfx950_intrin.h"), os.path.join(HERE, "emu", "hip", "hip_runtime.h")]
    if not os.path.exists(EMU_SO) or any(os.path.getmtime(s) > os.path.getmtime(EMU_SO) for s in src):
        subprocess.run([os.path.join(HERE, "emu", "build_emu.sh")], check=True, capture_output=True)
    lib = _abi.bind(EMU_SO)
    saved = (ops._LIB, ops._stream, ops._need_gpu)
    ops._LIB, ops._stream, ops._need_gpu = lib, (lambda t: None), (lambda *a: None)
    yield ops
    ops._LIB, ops._stream, ops._need_gpu = saved


@pytest.mark.parametrize("M,E,k", [(0, 4, 1), (1, 1, 1), (66, 4, 2), (1500, 8, 2), (5000, 130, 4), (20000, 300, 3)])
def test_prepare_sel_bit_exact(emu_ops, M, E, k):
    M -= M % k
    sel = torch.from_numpy(np.random.default_rng(M).integers(0, E, size=M))
    got = emu_ops.prepare_sel(sel, E, k)
    want = O.prepare_sel(sel.numpy(), E, k)
    for g, w in zip(got, (want.sel_sorted, want.perm, want.in_index, want.offsets)):
        assert np.array_equal(g.numpy(), w)
    assert np.array_equal(emu_ops.offsets_from_sorted(got[0], E).numpy(), want.offsets)
    got32 = emu_ops.prepare_sel(sel.to(torch.int32), E, k)
    assert np.array_equal(got32[1].numpy(), want.perm)


CASES = {
    # name: (problem kwargs, layer kwargs, dtype, tol)
    "f32_plain": (dict(T=48, D=128, E=4, F=64, k=2), dict(), "f32", 1e-5),
    "f32_ir_quant": (dict(T=48, D=128, E=4, F=64, k=2), dict(ir=True, inp_res=1 / 127, decay=0.01,
                                                              input_min_percentage=0.5), "f32", 1e-5),
    "f32_ragged_K": (dict(T=40, D=77, E=3, F=30, k=2), dict(ir=True, inp_res=1 / 127), "f32", 1e-5),
    "f32_split_adc_noise": (dict(T=40, D=96, E=4, F=40, k=2),
                            dict(ir=True, inp_res=1 / 127, bounds_up=[0, 32, 64, 96], bounds_down=[0, 20, 40],
                                 out_bound=12.0, out_res=254.0, noise=0.04), "f32", 1e-5),
    "bf16_plain": (dict(T=48, D=128, E=4, F=64, k=2), dict(), "bf16", 2e-2),
    "bf16_ir_quant": (dict(T=48, D=128, E=4, F=64, k=2), dict(ir=True, inp_res=1 / 127), "bf16", 2e-2),
    "bf16_ragged": (dict(T=40, D=76, E=3, F=36, k=2), dict(ir=True, inp_res=1 / 127), "bf16", 2e-2),
    "bf16_split_adc_noise": (dict(T=40, D=128, E=4, F=48, k=2),
                             dict(ir=True, inp_res=1 / 127, bounds_up=[0, 64, 128], out_bound=12.0, out_res=254.0,
                                  noise=0.04), "bf16", 2e-2),
    "f32_big_tile": (dict(T=200, D=40, E=2, F=136, k=2), dict(ir=True, inp_res=1 / 127), "f32", 1e-5),
    # every tile interior: these run the edge-free instantiations of the row-gather GEMM
    "f32_interior_split": (dict(T=80, D=128, E=3, F=128, k=2),
                           dict(ir=True, inp_res=1 / 127, bounds_up=[0, 64, 128], bounds_down=[0, 32, 128],
                                out_bound=12.0, out_res=254.0, noise=0.04, decay=0.01), "f32", 1e-5),
    "bf16_interior": (dict(T=80, D=128, E=3, F=128, k=2),
                      dict(ir=True, inp_res=1 / 127, out_bound=12.0, out_res=254.0, noise=0.04, decay=0.01),
                      "bf16", 2e-2),
    "bf16_interior_split": (dict(T=80, D=128, E=3, F=256, k=2),
                            dict(ir=True, inp_res=1 / 127, bounds_up=[0, 64, 128], bounds_down=[0, 128, 256],
                                 out_bound=12.0, out_res=254.0, noise=0.04), "bf16", 2e-2),
    "bf16_interior_plain": (dict(T=80, D=128, E=3, F=128, k=2), dict(), "bf16", 2e-2),
    # 256-column interior tiles: the 128 x 256 forward kernel (plain, clip + quantise, ADC without noise)
    "bf16_wide_plain": (dict(T=90, D=256, E=3, F=256, k=2), dict(), "bf16", 2e-2),
    "bf16_wide_ir_quant": (dict(T=90, D=256, E=3, F=256, k=2), dict(ir=True, inp_res=1 / 127, decay=0.01), "bf16", 2e-2),
    # two K-tiles of 256 columns with per-expert ranges: the 128 x 256 input-gradient kernel with its masks
    "bf16_wide_split": (dict(T=90, D=512, E=3, F=256, k=2),
                        dict(ir=True, inp_res=1 / 127, bounds_up=[0, 256, 512], out_bound=12.0, out_res=254.0,
                             decay=0.01), "bf16", 2e-2),
    "bf16_wide_ir_only": (dict(T=90, D=256, E=3, F=256, k=2), dict(ir=True, decay=0.01), "bf16", 2e-2),
    "bf16_wide_adc": (dict(T=90, D=256, E=3, F=256, k=2),
                      dict(ir=True, inp_res=1 / 127, out_bound=12.0, out_res=254.0, bounds_up=[0, 96, 256]), "bf16", 2e-2),
    "f32_interior_ir_only": (dict(T=80, D=128, E=3, F=128, k=2), dict(ir=True, decay=0.01), "f32", 1e-5),
    "f32_interior_quant_only": (dict(T=80, D=128, E=3, F=128, k=2), dict(inp_res=1 / 127), "f32", 1e-5),
    # fp16, the reference's reduced-precision type (cvmm.py:177-179, 188-189): plain, ragged with the analog stages
    # (per-position and per-expert ranges by turns), interior tiles
    "f16_plain": (dict(T=48, D=128, E=4, F=64, k=2), dict(), "f16", 2e-3),
    "f16_ragged_split_adc_noise": (dict(T=40, D=76, E=3, F=36, k=2),
                                   dict(ir=True, inp_res=1 / 127, bounds_up=[0, 40, 76], out_bound=12.0, out_res=254.0,
                                        noise=0.04, decay=0.01), "f16", 2e-3),
    "f16_interior": (dict(T=80, D=128, E=3, F=128, k=2),
                     dict(ir=True, inp_res=1 / 127, out_bound=12.0, out_res=254.0, noise=0.04, decay=0.01),
                     "f16", 2e-3),
    "f16_ir_quant": (dict(T=48, D=128, E=4, F=64, k=2), dict(ir=True, inp_res=1 / 127, decay=0.01), "f16", 2e-3),
    # fp16 on the 128 x 256 kernels (per-expert ranges): plain, and two K-tiles with the analog stages
    "f16_wide_plain": (dict(T=90, D=256, E=3, F=256, k=2), dict(), "f16", 2e-3),
    "f16_wide_split": (dict(T=90, D=512, E=3, F=256, k=2),
                       dict(ir=True, inp_res=1 / 127, bounds_up=[0, 256, 512], out_bound=12.0, out_res=254.0,
                            decay=0.01), "f16", 2e-3),
    # an output quantiser finer than 8 bits (1022 states): its codes do not fit the bytes in which the two-K-tile
    # variant of the 128 x 256 forward kernel parks the first tile, nor the byte-coded result; those launches must
    # fall to the kernels that keep fp32 values.  Per-expert ranges, so that the wide kernels are candidates.
    "bf16_wide_fine_adc_split": (dict(T=90, D=512, E=3, F=256, k=2),
                                 dict(ir=True, inp_res=1 / 127, bounds_up=[0, 256, 512], out_bound=12.0,
                                      out_res=1022.0, by_expert=True), "bf16", 2e-2),
    "bf16_wide_fine_adc": (dict(T=90, D=256, E=3, F=256, k=2),
                           dict(ir=True, inp_res=1 / 127, out_bound=12.0, out_res=1022.0, by_expert=True), "bf16", 2e-2),
    "f16_wide_fine_adc_split": (dict(T=90, D=512, E=3, F=256, k=2),
                                dict(ir=True, inp_res=1 / 127, bounds_up=[0, 256, 512], out_bound=12.0,
                                     out_res=1.0 / 1022.0, by_expert=True), "f16", 2e-3),
    # an input quantiser finer than 8 bits (10 bit: codes up to 511) in fp32, and in fp16, which holds them exactly
    "f32_fine_dac": (dict(T=48, D=128, E=4, F=64, k=2), dict(ir=True, inp_res=2.0 / (2 ** 10 - 2)), "f32", 1e-5),
    "f16_wide_fine_dac": (dict(T=90, D=256, E=3, F=256, k=2),
                          dict(ir=True, inp_res=2.0 / (2 ** 10 - 2), by_expert=True), "f16", 2e-3),
}


@pytest.mark.parametrize("name", list(CASES))
def test_layer_parity_emulated(emu_ops, name):
    pk, lk, dtype, tol = CASES[name]
    lk = dict(lk)
    # alternate between the per-position input-range vector of the reference and the fused
    # per-expert table / in-kernel gate (x) dy product
    lk.setdefault("by_expert", list(CASES).index(name) % 2 == 1)
    tdt = util.TORCH_DTYPE[dtype]
    pr = util.make_problem(7, dtype=tdt, **pk)
    E, k, T, D, F = pk["E"], pk["k"], pk["T"], pk["D"], pk["F"]
    ir = None
    if lk.pop("ir", False):
        nt = max(len(lk.get("bounds_up", [0, 1])), len(lk.get("bounds_down", [0, 1]))) - 1
        ir = torch.from_numpy(np.random.default_rng(1).uniform(0.7, 2.5, size=(2, E, nt)).astype(np.float32))
    nstd = lk.pop("noise", 0.0)
    okw = {n: v for n, v in lk.items() if n != "by_expert"}
    if nstd:
        ntu = len(lk.get("bounds_up", [0, 1])) - 1
        ntd = len(lk.get("bounds_down", [0, 1])) - 1
        g = torch.Generator().manual_seed(3)
        wu = pr["keys"].float().abs().amax((1, 2))[pr["idx"].reshape(-1)].reshape(1, -1, 1)
        wd = pr["values"].float().abs().amax((1, 2))[pr["idx"].reshape(-1)].reshape(1, -1, 1)
        lk["noise_up"] = (torch.randn(ntu, T * k, F, generator=g) * nstd * wu).contiguous()
        lk["noise_down"] = (torch.randn(ntd, T * k, D, generator=g) * nstd * wd).contiguous()
        okw["noise_up"], okw["noise_down"] = lk["noise_up"].numpy(), lk["noise_down"].numpy()
    if lk.get("out_bound", -1) > 0:
        okw["wmax_up"] = pr["keys"].float().abs().amax((1, 2)).reshape(E, 1).numpy()
        okw["wmax_down"] = pr["values"].float().abs().amax((1, 2)).reshape(E, 1).numpy()
    got = util.layer_ops_fwd_bwd(emu_ops, pr, ir, **lk)
    want = util.layer_oracle(pr, ir, dtype, got=got, **okw)
    util.compare_layer(got, want, tol, adc_step=util.adc_steps(pr, ir, lk))


def test_generated_noise_matches_counter_oracle(emu_ops):
    pr = util.make_problem(9, T=40, D=64, E=4, F=32, k=2)
    ir = torch.full((2, 4, 1), 2.0)
    kw = dict(inp_res=1 / 127, noise_std=0.04, noise_seed=0x1234567890, backward=False)
    got = util.layer_ops_fwd_bwd(emu_ops, pr, ir, **kw)
    kw.pop("backward")
    want = util.layer_oracle(pr, ir, "f32", backward=False,
                             wmax_up=pr["keys"].abs().amax((1, 2)).reshape(4, 1).numpy(),
                             wmax_down=pr["values"].abs().amax((1, 2)).reshape(4, 1).numpy(), **kw)
    assert util.rel_err(got["scores"].numpy(), want.scores) < 1e-5
    assert util.rel_err(got["y"].numpy(), want.y) < 1e-5
    clean = util.layer_ops_fwd_bwd(emu_ops, pr, ir, inp_res=1 / 127, backward=False)
    assert (got["z"] - clean["z"]).abs().max() > 1e-3


@pytest.mark.parametrize("split", [False, True])
def test_generated_noise_interior_bf16(emu_ops, split):
    util.check_generated_noise_interior(emu_ops, split=split, T=70)


def test_wide_kernels_with_uneven_experts(emu_ops):
    util.check_wide_kernels_uneven_experts(emu_ops)


def test_bf16_dac_codes_next_to_rounding_ties(emu_ops):
    util.check_bf16_dac_codes_near_ties(emu_ops)


@pytest.mark.parametrize("noisy", [False, True])
def test_result_as_adc_codes(emu_ops, noisy):
    util.check_result_as_codes(emu_ops, noisy=noisy, T=71)


@pytest.mark.parametrize("dtype,noisy", [(torch.bfloat16, True), (torch.bfloat16, False), (torch.float16, True)])
def test_weights_in_registers_kernel(emu_ops, dtype, noisy):
    util.check_weights_in_registers_kernel(emu_ops, dtype=dtype, noisy=noisy)


def test_companions(emu_ops):
    pr = util.make_problem(11, T=30, D=70, E=5, F=20, k=2)
    x = pr["x"]
    assert torch.equal(emu_ops.row_abs_max(x), x.abs().amax(-1))
    assert torch.equal(emu_ops.weight_abs_max(pr["keys"], False), pr["keys"].abs().amax((1, 2)).reshape(5, 1))
    assert torch.equal(emu_ops.weight_abs_max(pr["keys"], True), pr["keys"].abs().amax(1))
    util.check_weight_abs_max(emu_ops)
    util.check_layer_tables(emu_ops)
    util.check_layer_tables(emu_ops, dtype=torch.float32, E=3, n_up=1, n_dn=3)
    util.check_segment_sum_typed(emu_ops)
    util.check_gate_reduce_counter(emu_ops)
    va = pr["values"].to(torch.float16)[:, :, :61].contiguous()                      # 20 x 61: no 16-byte slices
    wa, wb = emu_ops.weight_abs_max_pair(pr["keys"].to(torch.float16), va)
    assert torch.equal(wb, va.float().abs().amax((1, 2)).reshape(5, 1))
    s = emu_ops.prepare_sel(pr["idx"].clamp(max=3), 5, 2)
    std = emu_ops.expert_std(x, s[2], s[3], 5)
    want = O.expert_std(x.numpy(), s[2].numpy(), s[0].numpy(), 5)
    np.testing.assert_allclose(std.numpy()[:4], want[:4], rtol=1e-5)
    assert not (std[4] > 0)


@pytest.mark.parametrize("dtype,kw", [
    (torch.float32, dict(T=50, D=96, k=3, bounds=[0, 32, 96])),
    (torch.float32, dict(T=9, D=260, k=2, E=2, strided_x=True, decay=0.0)),
    (torch.bfloat16, dict(T=40, D=1040, k=8, E=9, bounds=[0, 520, 1040], sel_dtype=torch.int32)),
    (torch.float16, dict(T=33, D=136, k=4, strided_x=True, input_min_percentage=0.99)),
])
def test_head_sum_with_input_range_clip(emu_ops, dtype, kw):
    util.check_ksum_clip(emu_ops, dtype=dtype, **kw)


def test_head_sum_with_clip_rejects_what_it_does_not_take(emu_ops):
    x = torch.randn(4, 64)
    assert not emu_ops.ksum_clip_supported(x, 1, None) and not emu_ops.ksum_clip_supported(x, 9, None)
    assert not emu_ops.ksum_clip_supported(x, 2, [0, 30, 64]) and emu_ops.ksum_clip_supported(x, 2, [0, 32, 64])
    idx = torch.zeros(4, 9, dtype=torch.int64)
    s = emu_ops.prepare_sel(idx, 1, 9)
    with pytest.raises(RuntimeError, match="not supported"):
        emu_ops.ksum_clip(torch.randn(36, 64), x, idx, s[1], s[3], torch.ones(1, 1), 9)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", util.MODIFIER_KINDS)
def test_weight_modifier_matches_oracle(emu_ops, kind, dtype):
    util.check_modify_weight(emu_ops, kind, dtype)
    util.check_modify_weight(emu_ops, kind, dtype, E=2, K=9, N=13)          # ragged rows: the scalar paths


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("per_channel", [False, True])
def test_weight_std_and_clamp_match_oracle(emu_ops, per_channel, dtype):
    util.check_weight_clip(emu_ops, per_channel, dtype)
    util.check_weight_clip(emu_ops, per_channel, dtype, E=2, K=33, N=7)
    if not per_channel:
        util.check_weight_clip(emu_ops, per_channel, dtype, E=2, K=300, N=200)   # several slices per expert


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_epilogue_matches_oracle(emu_ops, dtype):
    util.check_select(emu_ops, dtype, T=37)
    util.check_select(emu_ops, dtype, T=13, E=130, k=8, seed=1)           # three experts per lane, a ragged last wave
    util.check_select(emu_ops, dtype, T=5, E=2, k=2, seed=2)
    util.check_select(emu_ops, dtype, T=9, E=100, k=4, seed=3)            # two experts per lane
    util.check_select(emu_ops, dtype, T=9, E=300, k=5, seed=4)            # eight (five used)


def test_transposed_weight_view(emu_ops):
    """cvmm.py:839 hands the forward launcher `keys.transpose(1, 2)`: k-contiguous weights."""
    pr = util.make_problem(13, T=30, D=72, E=3, F=40, k=2)
    s_sorted, perm, in_index, offsets = emu_ops.prepare_sel(pr["idx"], 3, 2)
    wt = pr["keys"].transpose(1, 2).contiguous().transpose(1, 2)      # [E, D, F] view with D contiguous
    a = emu_ops.cvmm_fwd(pr["x"], wt, s_sorted, offsets, in_index, perm, 60)
    b = emu_ops.cvmm_fwd(pr["x"], pr["keys"], s_sorted, offsets, in_index, perm, 60)
    np.testing.assert_allclose(a.numpy(), b.numpy(), rtol=1e-5, atol=1e-6)
    wt16 = wt.bfloat16().transpose(1, 2).contiguous().transpose(1, 2)
    a16 = emu_ops.cvmm_fwd(pr["x"].bfloat16(), wt16, s_sorted, offsets, in_index, perm, 60)
    b16 = emu_ops.cvmm_fwd(pr["x"].bfloat16(), pr["keys"].bfloat16(), s_sorted, offsets, in_index, perm, 60)
    assert torch.equal(a16, b16)


def test_input_quantiser_finer_than_the_element_type_is_rejected(emu_ops):
    """bf16 holds integers exactly up to 256, fp16 up to 2048: the 16-bit kernels carry the DAC codes themselves, so a
    finer quantiser must be refused (on the host, before anything is launched) instead of truncating codes."""
    pr = util.make_problem(1, T=8, D=16, E=2, F=8, k=2, dtype=torch.bfloat16)
    s_sorted, perm, in_index, offsets = emu_ops.prepare_sel(pr["idx"], 2, 2)
    ir = torch.ones(2, 1)
    args = (pr["x"], pr["keys"], s_sorted, offsets, in_index, perm, 16)
    with pytest.raises(ValueError, match="needs fp32"):
        emu_ops.cvmm_fwd(*args, ir=ir, ir_by_expert=True, inp_res=2.0 / (2 ** 10 - 2))
    emu_ops.cvmm_fwd(*args, ir=ir, ir_by_expert=True, inp_res=1.0 / 256)          # the finest bf16 carries
    with pytest.raises(ValueError, match="xq_inp_res"):
        emu_ops.cvmm_fwd(*args, ir=ir, ir_by_expert=True, inp_res=1.0 / 127, xq_ir=torch.ones(2), xq_inp_res=1.0 / 511)
    h = {n: (t.half() if t.is_floating_point() else t) for n, t in pr.items()}
    argh = (h["x"], h["keys"], s_sorted, offsets, in_index, perm, 16)
    emu_ops.cvmm_fwd(*argh, ir=ir, ir_by_expert=True, inp_res=1.0 / 2047)
    with pytest.raises(ValueError, match="needs fp32"):
        emu_ops.cvmm_fwd(*argh, ir=ir, ir_by_expert=True, inp_res=1.0 / 8191)
    # and by the library itself, for callers that bypass the Python layer
    a = _abi.FwdArgs()
    a.dtype, a.M, a.N, a.K, a.E, a.n_in_rows, a.n_out_rows = _abi.AMOE_BF16, 16, 8, 16, 2, 8, 16
    one = torch.zeros(64)
    for f in ("x", "w", "out", "offsets", "in_index", "ir"):
        setattr(a, f, one.data_ptr())
    a.ldx, a.ldo, a.w_stride_e, a.w_stride_k, a.w_stride_n = 16, 8, 128, 8, 1
    _abi.set_bounds(a, [0, 16])
    a.inp_res = 1.0 / 511
    assert ops.get_lib().amoe_cvmm_fwd(a, None) == _abi.AMOE_EUNSUPPORTED


def test_input_gradient_with_x_but_nothing_that_reads_it(emu_ops):
    """A caller may pass the forward input without an input range, a ReLU mask or a clipped-input output; the
    library asks for xf_index only with one of those, so such a launch must not read through it."""
    pr = util.make_problem(3, T=70, D=256, E=3, F=256, k=2, dtype=torch.bfloat16)
    s_sorted, perm, in_index, offsets = emu_ops.prepare_sel(pr["idx"], 3, 2)
    g = torch.randn(140, 256).bfloat16()
    plain, _ = emu_ops.cvmm_bwd_x(g, pr["keys"], offsets, perm, perm, 140)
    with_x, _ = emu_ops.cvmm_bwd_x(g, pr["keys"], offsets, perm, perm, 140, x=pr["x"])
    assert torch.equal(plain, with_x)


def test_argument_errors(emu_ops):
    lib = ops.get_lib()
    assert lib.amoe_version() == 100
    assert lib.amoe_cvmm_fwd(None, None) == -2
    a = _abi.FwdArgs()
    a.dtype = 7
    assert lib.amoe_cvmm_fwd(a, None) == -1
    pr = util.make_problem(1, T=8, D=16, E=2, F=8, k=2)
    s_sorted, perm, in_index, offsets = emu_ops.prepare_sel(pr["idx"], 2, 2)
    with pytest.raises(_abi.AmoeError, match="inconsistent sizes"):
        emu_ops.cvmm_fwd(pr["x"], pr["keys"], s_sorted, offsets, in_index, perm, 16, bounds=[0, 8, 15])
    with pytest.raises(_abi.AmoeError):
        emu_ops.cvmm_fwd(pr["x"], pr["keys"], s_sorted, offsets, in_index, perm, 16, out_bound=12.0)  # no wmax
    assert b"workspace" in lib.amoe_strerror(-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_chunked_weight_gradient(emu_ops, dtype):
    util.check_row_chunked_wgrad(emu_ops, dtype=dtype, T=200)


def test_row_chunked_weight_gradient_wide_tiles(emu_ops):
    """the 256 x 256 kernel: its partial tiles are laid out as the 128 x 128 tiles the second launch adds"""
    util.check_row_chunked_wgrad(emu_ops, dtype=torch.bfloat16, T=200, D=512, F=256)


@pytest.mark.parametrize("dtype,D,F,T", [(torch.float32, 128, 128, 60), (torch.bfloat16, 128, 128, 60),
                                         (torch.bfloat16, 72, 40, 60), (torch.bfloat16, 256, 256, 70)])
def test_chained_projections(emu_ops, dtype, D, F, T):
    util.check_chained_projections(emu_ops, dtype=dtype, T=T, D=D, F=F)


@pytest.mark.parametrize("dtype,D,F,T", [(torch.float32, 128, 128, 60), (torch.bfloat16, 128, 128, 60),
                                         (torch.bfloat16, 72, 40, 60), (torch.bfloat16, 256, 256, 200)])
def test_clipped_input_for_the_weight_gradient(emu_ops, dtype, D, F, T):
    util.check_clipped_input_output(emu_ops, dtype=dtype, T=T, D=D, F=F)
