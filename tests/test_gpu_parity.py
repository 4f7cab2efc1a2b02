"""GPU parity tests: the HIP kernels, called through the C ABI (analog_moe_amd.ops ->
libamoe.so), against the CPU oracle on the same seeded inputs.
Tolerances: selection bit-exact; fp32 1e-5, bf16 2e-2 and fp16 2e-3 relative to the scale of the
reference tensor (max |a-b| / max |b|)."""
import numpy as np
import pytest
import torch

from oracle import cvmm_oracle as O
from tests import util
from tests.test_emu_kernels import CASES

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-5, "bf16": 2e-2, "f16": 2e-3}


@pytest.fixture(scope="module")
def ops():
    from analog_moe_amd import ops as _ops
    _ops.get_lib()          # fails loudly when libamoe.so has not been built
    return _ops


def _to(pr, dev="cuda"):
    return {n: t.to(dev) for n, t in pr.items()}


@pytest.mark.parametrize("M,E,k,skew", [(0, 4, 1, False), (1, 1, 1, False), (512, 8, 2, False), (32768, 16, 4, False),
                                        (131072, 64, 8, False), (131072, 128, 4, True), (100003, 1000, 1, True),
                                        (3 * 4099, 2048, 3, False)])
def test_prepare_sel_bit_exact(ops, M, E, k, skew):
    rng = np.random.default_rng(M + E)
    if skew:
        p = np.arange(1, E + 1) ** -1.2
        sel = rng.choice(E, size=M, p=p / p.sum())
    else:
        sel = rng.integers(0, E, size=M)
    print(f"prepare_sel M={M} E={E} k={k} skew={skew}", flush=True)
    got = ops.prepare_sel(torch.from_numpy(sel).cuda(), E, k)
    want = O.prepare_sel(sel, E, k)
    for g, w in zip(got, (want.sel_sorted, want.perm, want.in_index, want.offsets)):
        assert np.array_equal(g.cpu().numpy(), w)
    assert np.array_equal(ops.offsets_from_sorted(got[0], E).cpu().numpy(), want.offsets)
    got32 = ops.prepare_sel(torch.from_numpy(sel.astype(np.int32)).cuda(), E, k)
    assert np.array_equal(got32[1].cpu().numpy(), want.perm)


def _run_case(ops, pk, lk, dtype, seed=7, routing="router", by_expert=False):
    lk = dict(lk)
    lk.setdefault("by_expert", by_expert)
    tdt = util.TORCH_DTYPE[dtype]
    pr = util.make_problem(seed, dtype=tdt, routing=routing, **pk)
    E, k, T, D, F = pk["E"], pk["k"], pk["T"], pk["D"], pk["F"]
    ir = None
    irspec = lk.pop("ir", False)
    if irspec:
        nt = max(len(lk.get("bounds_up", [0, 1])), len(lk.get("bounds_down", [0, 1]))) - 1
        if irspec is True:
            ir = torch.from_numpy(np.random.default_rng(1).uniform(0.7, 2.5, size=(2, E, nt)).astype(np.float32))
        else:
            ir = torch.full((2, E, nt), float(irspec))
    nstd = lk.pop("noise", 0.0)
    okw = {n: v for n, v in lk.items() if n != "by_expert"}
    if nstd:
        ntu = len(lk.get("bounds_up", [0, 1])) - 1
        ntd = len(lk.get("bounds_down", [0, 1])) - 1
        g = torch.Generator().manual_seed(3)
        wu = pr["keys"].float().abs().amax((1, 2))[pr["idx"].reshape(-1)].reshape(1, -1, 1)
        wd = pr["values"].float().abs().amax((1, 2))[pr["idx"].reshape(-1)].reshape(1, -1, 1)
        nu = (torch.randn(ntu, T * k, F, generator=g) * nstd * wu).contiguous()
        nd = (torch.randn(ntd, T * k, D, generator=g) * nstd * wd).contiguous()
        lk["noise_up"], lk["noise_down"] = nu.cuda(), nd.cuda()
        okw["noise_up"], okw["noise_down"] = nu.numpy(), nd.numpy()
    if lk.get("out_bound", -1) > 0:
        okw["wmax_up"] = pr["keys"].float().abs().amax((1, 2)).reshape(E, 1).numpy()
        okw["wmax_down"] = pr["values"].float().abs().amax((1, 2)).reshape(E, 1).numpy()
    got = util.layer_ops_fwd_bwd(ops, _to(pr), None if ir is None else ir.cuda(), **lk)
    torch.cuda.synchronize()
    want = util.layer_oracle(pr, ir, dtype, got=got, **okw)
    return util.compare_layer(got, want, TOL[dtype], adc_step=util.adc_steps(pr, ir, lk))


@pytest.mark.parametrize("name", list(CASES))
def test_layer_parity_small(ops, name):
    pk, lk, dtype, _ = CASES[name]
    print("case", name, flush=True)
    print(_run_case(ops, pk, lk, dtype, by_expert=list(CASES).index(name) % 2 == 1))


def test_config1_cpu_runnable_layer(ops):
    """BASELINE config 1: D=128, E=8, F=64, k=2, 4x64 tokens, fp32, fixed input range 3.0,
    8-bit input quantisation, no noise, 8-bit ADC; forward + backward."""
    print("config 1", flush=True)
    errs = _run_case(ops, dict(T=256, D=128, E=8, F=64, k=2),
                     dict(ir=3.0, inp_res=1 / 127, out_bound=12.0, out_res=254.0), "f32", seed=0)
    print(errs)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_config2_paper_scale_layer(ops, dtype):
    """BASELINE config 2: D=412 (not a multiple of the vector width), E=16, F=128, k=4,
    32x256 tokens, per-expert input ranges, 8-bit DAC/ADC, injected output noise 0.04 * max|W|."""
    print("config 2", dtype, flush=True)
    errs = _run_case(ops, dict(T=8192, D=412, E=16, F=128, k=4),
                     dict(ir=True, inp_res=1 / 127, out_bound=12.0, out_res=254.0, noise=0.04, decay=0.01,
                          input_min_percentage=0.9), dtype, seed=0, by_expert=(dtype == "bf16"))
    print(errs)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_wide_tiles_layer(ops, dtype):
    """Several row tiles per expert and several work items per workgroup of the 128 x 256 kernels (forward and
    input gradient): two K-tiles of 256 columns, per-expert ranges, DAC / ADC, injected noise, range decay."""
    print("wide tiles", dtype, flush=True)
    errs = _run_case(ops, dict(T=4096, D=512, E=8, F=256, k=2),
                     dict(ir=True, inp_res=1 / 127, bounds_up=[0, 256, 512], out_bound=12.0, out_res=254.0,
                          noise=0.04, decay=0.01, input_min_percentage=0.9), dtype, seed=0, by_expert=True)
    print(errs)


@pytest.mark.parametrize("dtype,noisy,T,E,D", [(torch.bfloat16, True, 330, 4, 512), (torch.bfloat16, False, 9000, 9, 1024),
                                               (torch.float16, True, 3000, 5, 256)])
def test_weights_in_registers_kernel(ops, dtype, noisy, T, E, D):
    """contraction of 256: the down-projection's forward (as ADC codes, rescaled, plain) and the up-projection's
    input gradient on the kernel that holds the expert's weights in registers"""
    print("weights in registers", dtype, noisy, T, E, D, flush=True)
    print(util.check_weights_in_registers_kernel(ops, device="cuda", dtype=dtype, noisy=noisy, T=T, E=E, D=D))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_wide_kernels_with_uneven_experts(ops, dtype):
    print("wide kernels, uneven experts", dtype, flush=True)
    print(util.check_wide_kernels_uneven_experts(ops, device="cuda", dtype=dtype, T=3000, E=9))


@pytest.mark.parametrize("dtype,kw", [
    (torch.float32, dict(T=700, D=96, k=3, bounds=[0, 32, 96])),
    (torch.float32, dict(T=2100, D=260, k=2, E=2, strided_x=True, decay=0.0)),
    (torch.bfloat16, dict(T=3000, D=1024, N=64, k=8, E=16, bounds=[0, 512, 1024], sel_dtype=torch.int32)),
    (torch.bfloat16, dict(T=9000, D=256, N=32, k=4, E=7)),          # more tokens than one pass of the grid takes
    (torch.float16, dict(T=1033, D=136, k=4, strided_x=True, input_min_percentage=0.99)),
])
def test_head_sum_with_input_range_clip(ops, dtype, kw):
    print("head sum with clip", dtype, kw, flush=True)
    util.check_ksum_clip(ops, device="cuda", dtype=dtype, **kw)


def test_generated_noise_matches_counter_oracle(ops):
    pr = util.make_problem(9, T=500, D=256, E=8, F=128, k=2)
    ir = torch.full((2, 8, 1), 2.0)
    kw = dict(inp_res=1 / 127, noise_std=0.04, noise_seed=0x1234567890)
    got = util.layer_ops_fwd_bwd(ops, _to(pr), ir.cuda(), backward=False, **kw)
    want = util.layer_oracle(pr, ir, "f32", backward=False,
                             wmax_up=pr["keys"].abs().amax((1, 2)).reshape(8, 1).numpy(),
                             wmax_down=pr["values"].abs().amax((1, 2)).reshape(8, 1).numpy(), **kw)
    # the generator is integer arithmetic (a product of byte matrices): the kernel adds the same noise values as the
    # oracle, so the noisy fp32 stages meet the fp32 tolerance of the noise-free path
    assert util.rel_err(got["scores"].cpu().numpy(), want.scores) < 1e-5
    # a last-bit difference in the first stage can move an input of the second across a DAC rounding
    # boundary, so the second stage is checked from the kernel's own first-stage output
    okw = dict(wmax_up=pr["keys"].abs().amax((1, 2)).reshape(8, 1).numpy(),
               wmax_down=pr["values"].abs().amax((1, 2)).reshape(8, 1).numpy(), **kw)
    cont = util.layer_oracle(pr, ir, "f32", backward=False, got=got, **okw)
    assert util.rel_err(got["z"].cpu().numpy(), cont.z) < 1e-5
    assert util.rel_err(got["y"].cpu().numpy(), cont.y) < 1e-5


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_generated_noise_interior(ops, dtype, split):
    """The output stage the benchmark times (edge-free tiles, bf16 codes, noise drawn in the kernel, ADC, one
    max |W| per expert, per-expert input ranges; with and without the K-tile split) against the oracle."""
    print("generated noise, interior tiles", dtype, "split" if split else "one tile", flush=True)
    print(util.check_generated_noise_interior(ops, device="cuda", dtype=dtype, split=split, T=1500))


def test_bf16_dac_codes_next_to_rounding_ties(ops):
    print("bf16 DAC codes next to rounding ties", flush=True)
    util.check_bf16_dac_codes_near_ties(ops, device="cuda", T=960)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("noisy", [False, True])
def test_result_as_adc_codes(ops, noisy, dtype):
    print("result as ADC codes", noisy, dtype, flush=True)
    util.check_result_as_codes(ops, device="cuda", noisy=noisy, T=3000, D=1024, F=256, E=8, k=4, dtype=dtype)


def test_companions(ops):
    pr = _to(util.make_problem(11, T=300, D=70, E=5, F=20, k=2))
    x = pr["x"]
    assert torch.equal(ops.row_abs_max(x), x.abs().amax(-1))
    assert torch.equal(ops.weight_abs_max(pr["keys"], False), pr["keys"].abs().amax((1, 2)).reshape(5, 1))
    assert torch.equal(ops.weight_abs_max(pr["keys"], True), pr["keys"].abs().amax(1))
    s = ops.prepare_sel(pr["idx"].clamp(max=3), 5, 2)
    std = ops.expert_std(x, s[2], s[3], 5).cpu().numpy()
    want = O.expert_std(x.cpu().numpy(), s[2].cpu().numpy(), s[0].cpu().numpy(), 5)
    np.testing.assert_allclose(std[:4], want[:4], rtol=1e-5)
    assert not (std[4] > 0)


def test_cpu_tensors_are_rejected(ops):
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.prepare_sel(torch.zeros(4, dtype=torch.int64), 2, 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_chunked_weight_gradient(ops, dtype):
    util.check_row_chunked_wgrad(ops, device="cuda", dtype=dtype, T=4000)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_row_chunked_weight_gradient_wide_tiles(ops, dtype):
    print("row-chunked weight gradient, 256 x 256 tiles", dtype, flush=True)
    util.check_row_chunked_wgrad(ops, device="cuda", dtype=dtype, T=4000, D=512, F=256)


@pytest.mark.parametrize("dtype,D,F,T", [(torch.float32, 256, 128, 700), (torch.bfloat16, 256, 128, 700),
                                         (torch.bfloat16, 72, 40, 700), (torch.float32, 100, 36, 700),
                                         (torch.bfloat16, 256, 256, 1000), (torch.bfloat16, 512, 256, 1000)])
def test_chained_projections(ops, dtype, D, F, T):
    util.check_chained_projections(ops, device="cuda", dtype=dtype, T=T, D=D, F=F)


@pytest.mark.parametrize("dtype,D,F,T", [(torch.float32, 256, 128, 700), (torch.bfloat16, 256, 128, 700),
                                         (torch.bfloat16, 256, 192, 700), (torch.bfloat16, 72, 40, 700),
                                         (torch.bfloat16, 256, 256, 1000), (torch.bfloat16, 256, 512, 1000),
                                         (torch.bfloat16, 512, 256, 3000)])
def test_clipped_input_for_the_weight_gradient(ops, dtype, D, F, T):
    util.check_clipped_input_output(ops, device="cuda", dtype=dtype, T=T, D=D, F=F)


@pytest.mark.parametrize("name,T,D,E,F,k,routing", [("config3", 16384, 1024, 64, 256, 8, "uniform"),
                                                     ("config4", 32768, 2048, 128, 512, 4, "zipf")])
def test_full_size_properties(ops, name, T, D, E, F, k, routing):
    """BASELINE configs 3 and 4 at full size (bf16), where the oracle is too slow to run whole: sampled
    rows of both forward projections against float64 arithmetic on the kernel's own DAC definition,
    token-permutation invariance (bit-exact), run-to-run identity and exact power-of-two scaling of the
    weight gradient, and the sort invariants."""
    print(name, flush=True)
    pr = _to(util.make_problem(0, T, D, E, F, k, dtype=torch.bfloat16, routing=routing))
    x, keys, values, idx, dy = pr["x"], pr["keys"], pr["values"], pr["idx"], pr["dy"]
    M = T * k
    ss, perm, in_index, offsets = ops.prepare_sel(idx, E, k)
    flat = idx.reshape(-1)
    assert torch.equal(flat[perm.long()].int(), ss) and bool((ss[1:] >= ss[:-1]).all())
    assert torch.equal(offsets.long(), torch.cat([torch.zeros(1, dtype=torch.long, device="cuda"),
                                                  torch.bincount(flat, minlength=E).cumsum(0)]))
    assert torch.equal(in_index, (perm // k).int())
    res = 1 / 127
    ir_up = torch.linspace(2.0, 3.5, E, device="cuda").reshape(E, 1)
    ir_dn = torch.linspace(1.0, 2.0, E, device="cuda").reshape(E, 1)
    fwd_up = lambda xx, ii, oo: ops.cvmm_fwd(xx, keys, ss, offsets, ii, oo, M, ir=ir_up, ir_by_expert=True,
                                             inp_res=res, relu=True)
    p1 = fwd_up(x, in_index, perm)
    z = ops.cvmm_fwd(p1, values, ss, offsets, perm, None, M, ir=ir_dn, ir_by_expert=True, inp_res=res)
    # sampled sorted positions against float64 (codes are exact in bf16; weights are the bf16 values)
    g = torch.Generator().manual_seed(1)
    pos = torch.randint(0, M, (192,), generator=g).cuda()
    e_of = ss[pos].long()

    def ref_rows(inp_rows, w, ir_tab):
        r = ir_tab[e_of].double()
        a = torch.minimum(torch.maximum(inp_rows.double(), -r), r)
        a32 = (a.float() / r.float())                       # fp32 divisions, as the kernel does them
        codes = torch.round(a32 / torch.tensor(res, dtype=torch.float32, device="cuda"))
        out = torch.einsum("rk,rkn->rn", codes.double(), w[e_of].double()) * float(np.float32(res))
        return out * r

    want_p1 = torch.relu(ref_rows(x[in_index[pos].long()], keys, ir_up))
    got_p1 = p1[perm[pos].long()].double()
    assert float((got_p1 - want_p1).abs().max() / want_p1.abs().max()) < 1e-2          # bf16 output rounding
    want_z = ref_rows(p1[perm[pos].long()], values, ir_dn)
    got_z = z[perm[pos].long()].double()
    assert float((got_z - want_z).abs().max() / want_z.abs().max()) < 1e-2
    # shuffling the tokens permutes the outputs identically, bit for bit
    shuf = torch.randperm(T, generator=g).cuda()
    idx2 = idx[shuf]
    ss2, perm2, in2, off2 = ops.prepare_sel(idx2, E, k)
    p1_2 = ops.cvmm_fwd(x[shuf], keys, ss2, off2, in2, perm2, M, ir=ir_up, ir_by_expert=True, inp_res=res, relu=True)
    assert torch.equal(p1_2.view(T, k, F), p1.view(T, k, F)[shuf])
    # weight gradient: identical from run to run, and exactly linear under a power-of-two scale
    tok = (perm // k).int()
    gw = ops.cvmm_bwd_w(p1, dy, E, offsets, perm, tok, ir=ir_dn, ir_by_expert=True)
    assert torch.equal(gw, ops.cvmm_bwd_w(p1, dy, E, offsets, perm, tok, ir=ir_dn, ir_by_expert=True))
    gw4 = ops.cvmm_bwd_w(p1, dy * 4, E, offsets, perm, tok, ir=ir_dn, ir_by_expert=True)
    assert torch.equal(gw4, gw * 4)
    # input gradient of the plain product against float64 on the sampled rows
    full, _ = ops.cvmm_bwd_x(dy, values, offsets, tok, perm, M)
    want_g = torch.einsum("rn,rkn->rk", dy[tok[pos].long()].double(), values[e_of].double())
    got_g = full[perm[pos].long()].double()
    assert float((got_g - want_g).abs().max() / want_g.abs().max()) < 1e-2


@pytest.mark.parametrize("name", ["config1_dac", "config1_dac_adc_split"])
def test_golden_fixture_parity(ops, name):
    """The HIP path on the committed inputs against the committed expected outputs (tests/golden/*.npz)."""
    import os
    from tests.golden import make_golden as G
    fx = np.load(os.path.join(os.path.dirname(G.__file__), name + ".npz"))
    _, _, lk, _ = G.problem(name)
    pr = {n[3:]: torch.from_numpy(fx[n]) for n in fx.files if n.startswith("in_") and n != "in_ir"}
    ir = torch.from_numpy(fx["in_ir"])
    print("fixture", name, flush=True)
    if lk.get("out_bound", -1) > 0:
        lk = dict(lk)          # the layer ops take max |W| themselves
    got = util.layer_ops_fwd_bwd(ops, _to(pr), ir.cuda(), **lk)
    torch.cuda.synchronize()
    want = O.LayerOracle(y=fx["out_y"], scores=fx["out_scores"], z=fx["out_z"],
                         sel=O.SelOracle(*(fx["out_" + n] for n in ("sel_sorted", "perm", "in_index", "offsets"))),
                         grad_x=fx["out_grad_x"], grad_keys=fx["out_grad_keys"], grad_values=fx["out_grad_values"],
                         grad_gate=fx["out_grad_gate"], grad_ir=fx["out_grad_ir"])
    adc = util.adc_steps(pr, ir, lk)
    if adc is None:
        print(util.compare_layer(got, want, TOL["f32"]))
        return
    # with the output quantiser on, a last-bit difference in a sum moves a value by one ADC step, and what follows
    # inherits it: the quantised stages are compared with the step allowance, what follows with a wider tolerance
    errs = util.compare_layer(got, want, 1e-4, adc_step=adc)
    print(errs)
