"""Shared by the CPU (emulated) and GPU parity tests: builds seeded problems, runs the layer
through analog_moe_amd.ops and through the oracle, and compares."""
import numpy as np
import pytest
import torch

from analog_moe_amd.synthetic import make_problem  # noqa: F401  (re-exported: the tests build their inputs with it)
from oracle import cvmm_oracle as O


TORCH_DTYPE = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def dtype_name(dtype) -> str:
    """The oracle's name of a torch dtype."""
    return {v: n for n, v in TORCH_DTYPE.items()}[dtype]


def np32(t):
    return None if t is None else t.detach().float().cpu().numpy()


def layer_ops_fwd_bwd(ops, pr, ir=None, *, inp_res=-1.0, noise_up=None, noise_down=None, noise_std=0.0,
                      noise_seed=None, out_bound=-1.0, out_res=-1.0, bounds_up=None, bounds_down=None, decay=0.0,
                      input_min_percentage=0.95, gradient_relative=True, gradient_scale=1.0, per_channel=False,
                      backward=True, by_expert=False):
    """The layer of oracle.layer_fwd_bwd, through the kernels.  ir [2, E, n_tiles] tensor or None."""
    x, keys, values, idx, gate, dy = (pr[n] for n in ("x", "keys", "values", "idx", "gate", "dy"))
    T, D = x.shape
    E, _, F = keys.shape
    k = idx.shape[1]
    M = T * k
    sel_sorted, perm, in_index, offsets = ops.prepare_sel(idx, E, k)
    sel_l = sel_sorted.long()
    ntu = 1 if bounds_up is None else len(bounds_up) - 1
    ntd = 1 if bounds_down is None else len(bounds_down) - 1
    ir_up = ir_dn = None
    if ir is not None and by_expert:
        ir_up, ir_dn = ir[0][:, :ntu].contiguous(), ir[1][:, :ntd].contiguous()
    elif ir is not None:
        ir_up = ir[0][sel_l][:, :ntu].contiguous()
        ir_dn = ir[1][sel_l][:, :ntd].contiguous()
    be = dict(ir_by_expert=by_expert and ir is not None)
    need_wmax = out_bound > 0 or (noise_seed is not None and noise_std > 0)
    wu = ops.weight_abs_max(keys, per_channel) if need_wmax else None
    wd = ops.weight_abs_max(values, per_channel) if need_wmax else None
    gen = noise_seed is not None and noise_std > 0
    p1 = ops.cvmm_fwd(x, keys, sel_sorted, offsets, in_index, perm, M, ir=ir_up, inp_res=inp_res, bounds=bounds_up,
                      noise=noise_up, noise_std=noise_std if gen else 0.0, noise_seed=noise_seed or 0, wmax=wu,
                      out_bound=out_bound, out_res=out_res, relu=True, **be)
    z = ops.cvmm_fwd(p1, values, sel_sorted, offsets, perm, None, M, ir=ir_dn, inp_res=inp_res, bounds=bounds_down,
                     noise=noise_down, noise_std=noise_std if gen else 0.0, noise_seed=(noise_seed or 0) + 1,
                     wmax=wd, out_bound=out_bound, out_res=out_res, **be)
    y = ops.gate_reduce(z, gate)
    res = dict(y=y, scores=p1, z=z, sel_sorted=sel_sorted, perm=perm, in_index=in_index, offsets=offsets)
    if not backward:
        return res
    irkw = dict(gradient_relative=gradient_relative, gradient_scale=gradient_scale, decay=decay,
                input_min_percentage=input_min_percentage)
    # down-projection backward (cvmm.py:785-889)
    g_tok = torch.div(perm, k, rounding_mode="floor").to(torch.int32)
    if by_expert:   # gate (x) dy formed inside the kernel
        res["grad_values"] = ops.cvmm_bwd_w(p1, dy, E, offsets, perm, g_tok, ir=ir_dn, bounds=bounds_down,
                                            g_scale=gate, **be)
    else:
        g_w = (gate.reshape(-1, 1) * dy.repeat_interleave(k, dim=0)).to(dy.dtype)
        res["grad_values"] = ops.cvmm_bwd_w(p1, g_w, E, offsets, perm, None, ir=ir_dn, bounds=bounds_down)
    gp1, irg_dn = ops.cvmm_bwd_x(dy, values, offsets, g_tok, perm, M, x=p1, xf_index=perm, gate=gate, ir=ir_dn,
                                 bounds=bounds_down, relu_mask=True, **irkw, **be)
    res["grad_gate"] = ops.gate_grad(z, dy, k)
    # up-projection backward
    res["grad_keys"] = ops.cvmm_bwd_w(x, gp1, E, offsets, in_index, perm, ir=ir_up, bounds=bounds_up, **be)
    full, irg_up = ops.cvmm_bwd_x(gp1, keys, offsets, perm, perm, M, x=x, xf_index=in_index, ir=ir_up,
                                  bounds=bounds_up, **irkw, **be)
    res["grad_x"] = ops.ksum(full, k)
    if by_expert and ir is not None and ops.ksum_clip_supported(x, k, bounds_up):
        # the same two results with the clip applied by the sum over the heads (the fused layer's order): the
        # input gradient must not change by a bit; the input-range sums go on to the oracle comparison
        plain, none = ops.cvmm_bwd_x(gp1, keys, offsets, perm, perm, M)
        assert none is None
        late_x, late_irg = ops.ksum_clip(plain, x, idx, perm, offsets, ir_up, k, bounds=bounds_up, **irkw)
        assert torch.equal(late_x, res["grad_x"])
        scale = float(irg_up.abs().max()) + 1e-30
        assert float((late_irg - irg_up).abs().max()) / scale < (1e-5 if x.dtype == torch.float32 else 2e-2)
        irg_up = late_irg
        res["late_clip"] = True
    res["grad_p1"] = gp1
    if ir is not None:
        nt = ir.shape[2]
        gi = torch.zeros(2, E, nt, device=x.device)
        gi[0, :, :ntu] = ops.segment_sum(irg_up, offsets, E)
        gi[1, :, :ntd] = ops.segment_sum(irg_dn, offsets, E)
        res["grad_ir"] = gi
        res["ir_grad_up"], res["ir_grad_dn"] = irg_up, irg_dn
    return res


def layer_oracle(pr, ir=None, dtype="f32", backward=True, got=None, **kw):
    """got: kernel results; when given, the oracle continues from the kernels' own stage outputs
    (scores, z), so each stage is checked on identical inputs."""
    if got is not None:
        kw = dict(kw, scores_override=np32(got["scores"]), z_override=np32(got["z"]))
    return O.layer_fwd_bwd(np32(pr["x"]), np32(pr["keys"]), np32(pr["values"]), pr["idx"].cpu().numpy(),
                           np32(pr["gate"]), None if ir is None else np32(ir), np32(pr["dy"]) if backward else None,
                           dtype=dtype, **kw)


def rel_err(a, b):
    """max |a-b| / max |b|: error relative to the scale of the reference tensor."""
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def adc_flip_check(got, ref, tol, max_step, max_fraction=2e-4):
    """Stage output behind an output quantiser: all but a few elements match to tol; the rest sit on
    a rounding boundary and differ by whole ADC steps (at most one per K-tile, max_step in total)."""
    a, b = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    scale = max(np.abs(b).max(), 1e-30)
    d = np.abs(a - b)
    off = d > tol * scale
    frac = off.mean()
    assert frac <= max_fraction, f"{frac:.2e} of the elements differ"
    if off.any():
        assert d[off].max() <= max_step * 1.001 + tol * scale, (d[off].max(), max_step)
    return float(frac)


def compare_layer(got, want, tol, check_sel=True, skip=(), adc_step=None):
    """got: dict from layer_ops_fwd_bwd; want: LayerOracle.  adc_step: (max step of the scores, max step
    of z) when an output quantiser is on: those two stages are then compared with adc_flip_check."""
    if check_sel:
        assert np.array_equal(got["sel_sorted"].cpu().numpy(), want.sel.sel_sorted)
        assert np.array_equal(got["perm"].cpu().numpy(), want.sel.perm)
        assert np.array_equal(got["in_index"].cpu().numpy(), want.sel.in_index)
        assert np.array_equal(got["offsets"].cpu().numpy(), want.sel.offsets)
    pairs = [("scores", want.scores), ("z", want.z), ("y", want.y), ("grad_values", want.grad_values),
             ("grad_keys", want.grad_keys), ("grad_x", want.grad_x), ("grad_gate", want.grad_gate),
             ("grad_ir", want.grad_ir)]
    errs = {}
    for name, ref in pairs:
        if ref is None or name not in got or name in skip:
            continue
        if adc_step is not None and name in ("scores", "z"):
            errs[name + "_flipped"] = adc_flip_check(np32(got[name]).reshape(ref.shape), ref, tol,
                                                     adc_step[0 if name == "scores" else 1])
            continue
        errs[name] = rel_err(np32(got[name]).reshape(ref.shape), ref)
    bad = {n: e for n, e in errs.items() if not n.endswith("_flipped") and not e <= tol}
    assert not bad, f"relative error above {tol}: {bad} (all: {errs})"
    return errs


def adc_steps(pr, ir, lk):
    """Largest possible ADC-step error of the two forward stages: one step per K-tile, each
    scaled by the largest input range; None when the output quantiser is off."""
    if not (lk.get("out_bound", -1) > 0 and lk.get("out_res", -1) > 0):
        return None
    half = max(lk["out_res"], 1.0 / lk["out_res"]) * 0.5
    irmax = 1.0 if ir is None else float(ir.max())
    ntu = len(lk.get("bounds_up") or [0, 1]) - 1
    ntd = len(lk.get("bounds_down") or [0, 1]) - 1
    su = lk["out_bound"] * float(pr["keys"].float().abs().max()) / half * irmax * ntu
    sd = lk["out_bound"] * float(pr["values"].float().abs().max()) / half * irmax * ntd
    return su, sd


def check_generated_noise_interior(ops, device="cpu", dtype=torch.bfloat16, split=False, T=160, D=256, E=4, F=256,
                                   k=2, seed=0x5EED0123456789):
    """The layer on shapes whose every tile is interior (16-byte aligned operands, column tiles of 128, K tiles
    that are multiples of 64), bf16 DAC codes, noise DRAWN IN THE KERNEL, ADC with one max |W| per expert and a
    per-expert input-range table: the straight-line output stage of the usual training configuration, with and
    without the K-tile split, against the oracle's counter noise.  Stage by stage: the oracle continues from
    the kernel's own first-stage output, and a value next to an ADC rounding boundary may differ by one step."""
    name = dtype_name(dtype)
    pr = make_problem(23, T, D, E, F, k, dtype=dtype)
    bounds_up = [0, D // 2, D] if split else None
    nt = 2 if split else 1
    ir = torch.from_numpy(np.random.default_rng(4).uniform(1.5, 3.0, size=(2, E, nt)).astype(np.float32))
    lk = dict(inp_res=1.0 / 127.0, noise_std=0.04, noise_seed=seed, out_bound=12.0, out_res=254.0,
              bounds_up=bounds_up, decay=0.01, input_min_percentage=0.5)
    dev = {n: t.to(device) for n, t in pr.items()}
    got = layer_ops_fwd_bwd(ops, dev, ir.to(device), by_expert=True, **lk)
    okw = dict(lk, wmax_up=pr["keys"].float().abs().amax((1, 2)).reshape(E, 1).numpy(),
               wmax_down=pr["values"].float().abs().amax((1, 2)).reshape(E, 1).numpy())
    want = layer_oracle(pr, ir, name, got=got, **okw)
    tol = {torch.bfloat16: 2e-2, torch.float16: 2e-3, torch.float32: 1e-5}[dtype]
    errs = compare_layer(got, want, tol, adc_step=adc_steps(pr, ir, lk))
    # the noise is really there, and a different seed gives different noise
    clean = layer_ops_fwd_bwd(ops, dev, ir.to(device), by_expert=True, backward=False,
                              **{n: v for n, v in lk.items() if n not in ("noise_std", "noise_seed")})
    other = layer_ops_fwd_bwd(ops, dev, ir.to(device), by_expert=True, backward=False, **dict(lk, noise_seed=seed + 2))
    assert not torch.equal(got["scores"], clean["scores"]) and not torch.equal(got["z"], clean["z"])
    assert not torch.equal(got["scores"], other["scores"]) and not torch.equal(got["z"], other["z"])
    return errs


def check_wide_kernels_uneven_experts(ops, device="cpu", dtype=torch.bfloat16, T=150, D=256, F=256, E=5, k=2):
    """The 128 x 256 kernels (per-expert ranges, DAC, ADC, range decay) when the experts' segments are as uneven as
    they get: one expert without rows, one with more than a row tile, the rest with partly filled tiles."""
    pr = make_problem(31, T, D, E, F, k, dtype=dtype)
    idx = pr["idx"].clone()
    idx[idx == E - 1] = 0                                # the last expert gets nothing, the first gets its share
    idx[: max(T // 2, 140), 0] = 1                       # and expert 1 more than 128 rows
    pr["idx"] = idx
    counts = torch.bincount(idx.reshape(-1), minlength=E)
    assert int(counts[E - 1]) == 0 and int(counts.max()) > 128
    ir = torch.from_numpy(np.random.default_rng(5).uniform(0.9, 2.5, size=(2, E, 1)).astype(np.float32))
    lk = dict(inp_res=1.0 / 127.0, out_bound=12.0, out_res=254.0, decay=0.01, input_min_percentage=0.5)
    dev = {n: t.to(device) for n, t in pr.items()}
    got = layer_ops_fwd_bwd(ops, dev, ir.to(device), by_expert=True, **lk)
    okw = dict(lk, wmax_up=pr["keys"].float().abs().amax((1, 2)).reshape(E, 1).numpy(),
               wmax_down=pr["values"].float().abs().amax((1, 2)).reshape(E, 1).numpy())
    name = dtype_name(dtype)
    want = layer_oracle(pr, ir, name, got=got, **okw)
    tol = {torch.bfloat16: 2e-2, torch.float16: 2e-3}[dtype]
    errs = compare_layer(got, want, tol, adc_step=adc_steps(pr, ir, lk))
    # the expert without rows gets exact zeros as its weight gradients
    assert float(got["grad_keys"][E - 1].abs().max()) == 0.0 and float(got["grad_values"][E - 1].abs().max()) == 0.0
    return errs


# (input range, bf16 input) pairs whose DAC code is one step off when the two divisions of cvmm.py:154, 163 are
# replaced by one multiplication with (1 / range) * (1 / step): found by enumerating every bf16 value against
# 40 000 random ranges (about one range in a thousand has such a value)
DAC_TIE_PAIRS = [(1.394194483757019, 0.1591796875), (3.8115715980529785, 1.515625), (3.270026445388794, 0.9140625),
                 (1.7780784368515015, 0.70703125), (0.6161530017852783, 0.53125), (1.3566645383834839, 0.26171875)]


def check_bf16_dac_codes_near_ties(ops, device="cpu", T=96):
    """bf16 DAC codes equal the oracle's two-division codes also for values next to a rounding tie, in the input
    stage (seen through identity weights) and in the DAC image the up-projection emits for the down-projection."""
    E, k, D = len(DAC_TIE_PAIRS), 1, 128
    g = torch.Generator().manual_seed(5)
    idx = (torch.arange(T) % E).reshape(T, 1)
    x = torch.randn(T, D, generator=g)
    ir = torch.tensor([[r] for r, _ in DAC_TIE_PAIRS], dtype=torch.float32)
    for t in range(T):                                # a third of every row holds the expert's adversarial value
        v = DAC_TIE_PAIRS[t % E][1]
        x[t, ::3] = v
        x[t, 1::6] = -v
    x = x.bfloat16()
    eye = torch.eye(D).bfloat16().repeat(E, 1, 1).contiguous()
    ss, perm, in_index, offsets = ops.prepare_sel(idx.to(device), E, k)
    res = 1.0 / 127.0
    out, img = ops.cvmm_fwd(x.to(device), eye.to(device), ss, offsets, in_index, perm, T, ir=ir.to(device),
                            ir_by_expert=True, inp_res=res, xq_ir=ir[:, 0].contiguous().to(device), xq_inp_res=res)
    rows = ir.numpy()[idx.reshape(-1).numpy()]
    a, codes = O.dac(np32(x), rows, None, res)
    # the naive product really is off for these inputs (otherwise this test checks nothing)
    kq = (np.float32(1) / rows) * (np.float32(1) / np.float32(res))
    naive = np.rint((np.clip(np32(x), -rows, rows) * kq).astype(np.float32))
    assert (naive != codes).sum() >= T * D // 4
    want = O.to_bf16(((codes * np.float32(res)).astype(np.float32) * rows).astype(np.float32))
    np.testing.assert_array_equal(np32(out), want)
    # the image: the DAC of `out` as stored, against the same range
    _, codes2 = O.dac(np32(out), rows, None, res)
    np.testing.assert_array_equal(np32(img), codes2)


def check_result_as_codes(ops, device="cpu", T=150, D=256, F=128, E=3, k=2, noisy=True, dtype=torch.bfloat16):
    """A forward whose result leaves as ADC codes (one byte per value + two factors per expert): the values behind
    the codes round to exactly the 16-bit result of the ordinary call, and the gate reduction / gate gradient that
    read the codes agree with those that read the values."""
    pr = make_problem(29, T, F, E, D, k, dtype=dtype)                   # (a down-projection: [M, F] -> [M, D])
    M = T * k
    g = torch.Generator().manual_seed(2)
    p1 = torch.relu(torch.randn(M, F, generator=g)).to(dtype).to(device)
    values = (torch.randn(E, F, D, generator=g) / F ** 0.5).to(dtype).to(device)
    idx, gate = pr["idx"].to(device), pr["gate"].to(device)
    dy = torch.randn(T, D, generator=g).to(dtype).to(device)
    ss, perm, in_index, offsets = ops.prepare_sel(idx, E, k)
    ir = torch.linspace(0.6, 1.4, E).reshape(E, 1).to(device)
    wmax = ops.weight_abs_max(values, False)
    kw = dict(ir=ir, ir_by_expert=True, inp_res=1 / 127, out_bound=12.0, out_res=254.0, wmax=wmax,
              noise_std=0.04 if noisy else 0.0, noise_seed=77)
    assert ops.codes_supported(p1, values, ir_by_expert=True, inp_res=1 / 127, n_tiles=1, out_bound=12.0,
                               out_res=254.0, noise=None, per_channel=False)
    z = ops.cvmm_fwd(p1, values, ss, offsets, perm, None, M, **kw)
    codes, scale = ops.cvmm_fwd(p1, values, ss, offsets, perm, None, M, want_codes=True, **kw)
    assert codes.dtype == torch.uint8 and tuple(codes.shape) == (M, D) and tuple(scale.shape) == (E, 2)
    zf = ops.dequant_codes(codes, scale, idx)
    assert torch.equal(zf.to(dtype), z)
    c = codes.cpu().numpy().astype(np.int32) - 128
    assert np.abs(c).max() <= 127 and np.abs(c).max() > 20
    # gate reduction and gate gradient from the codes: against float64 on the exact values, and close to the
    # kernels that read the bf16 values
    # Tolerances, relative to the largest entry: the kernels that read the codes work on the exact values and round
    # their 16-bit result once (2^-9 for bf16, 2^-11 for fp16); the kernels that read z as values start from values
    # that were rounded to the element type first, which adds at most that much again per term.
    one = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -10
    y = ops.gate_reduce_codes(codes, scale, idx, gate)
    want_y = (gate.double().unsqueeze(-1) * zf.double().view(T, k, D)).sum(1)
    assert rel_err(np32(y), want_y.cpu().numpy()) < one
    assert rel_err(np32(y), np32(ops.gate_reduce(z, gate))) < 2 * one
    gg = ops.gate_grad_codes(codes, scale, idx, dy, k)
    want_gg = torch.einsum("tkd,td->tk", zf.double().view(T, k, D), dy.double())
    assert rel_err(np32(gg), want_gg.cpu().numpy()) < one
    assert rel_err(np32(gg), np32(ops.gate_grad(z, dy, k))) < 2 * one
    # codes next to zero under a large common part of dy, in fp32: the terms (code - 128) * dy must be formed from the
    # signed codes (a difference of two sums of byte * dy loses five digits here)
    small = torch.from_numpy((128 + np.random.default_rng(5).integers(-2, 3, size=(M, D))).astype(np.uint8)).to(device)
    dyf = (100.0 + torch.randn(T, D, generator=g)).to(device)
    ggs = ops.gate_grad_codes(small, scale, idx, dyf, k)
    want_s = torch.einsum("tkd,td->tk", ops.dequant_codes(small, scale, idx).double().view(T, k, D), dyf.double())
    assert rel_err(np32(ggs), want_s.cpu().numpy()) < 3e-6


def check_row_chunked_wgrad(ops, device="cpu", dtype=torch.float32, T=600, D=136, F=72):
    """The weight gradient with the rows of an expert shared between workgroups (skewed routing: one
    heavy expert, one empty one) against the oracle, and its run-to-run determinism."""
    E, k = 5, 2
    pr = make_problem(21, T, D, E, F, k, dtype=dtype)
    idx = pr["idx"].clone()
    idx[idx == 4] = 0                                   # expert 4 empty
    idx[: T // 2] = torch.tensor([0, 1])                # expert 0 heavy
    x, g = pr["x"].to(device), torch.randn(T * k, F).to(dtype).to(device)
    ss, perm, in_index, offsets = ops.prepare_sel(idx.to(device), E, k)
    ir = torch.full((E, 1), 0.8, device=device)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    want = O.cvmm_bwd_w(np32(x), in_index.cpu().numpy(), ss.cpu().numpy(), np32(g),
                        np.full((T * k, 1), 0.8, np.float32), E, perm.cpu().numpy(),
                        dtype=dtype_name(dtype))
    outs = []
    for rows_per_chunk in (64, 64, 192, 1 << 20):
        got = ops.cvmm_bwd_w(x, g, E, offsets, in_index, perm, ir=ir, ir_by_expert=True,
                             rows_per_chunk=rows_per_chunk)
        assert rel_err(np32(got), want) < tol
        assert float(got[4].abs().max()) == 0.0
        outs.append(got)
    assert torch.equal(outs[0], outs[1])


def check_chained_projections(ops, device="cpu", dtype=torch.float32, T=100, D=128, F=128, E=3, k=2):
    """The DAC image that the up-projection emits for the down-projection gives bit-identical
    down-projection results to running the down-projection's own input stage."""
    pr = make_problem(17, T, D, E, F, k, dtype=dtype)
    pr = {n: t.to(device) for n, t in pr.items()}
    ss, perm, in_index, offsets = ops.prepare_sel(pr["idx"], E, k)
    M = T * k
    ir_up = torch.linspace(0.9, 1.6, E, device=device).reshape(E, 1)
    ir_dn = torch.linspace(0.5, 1.1, E, device=device).reshape(E, 1)
    res = 1 / 127
    p1, p1q = ops.cvmm_fwd(pr["x"], pr["keys"], ss, offsets, in_index, perm, M, ir=ir_up, ir_by_expert=True,
                           inp_res=res, relu=True, xq_ir=ir_dn[:, 0].contiguous(), xq_inp_res=res)
    p1_alone = ops.cvmm_fwd(pr["x"], pr["keys"], ss, offsets, in_index, perm, M, ir=ir_up, ir_by_expert=True,
                            inp_res=res, relu=True)
    assert torch.equal(p1, p1_alone)
    # rows of p1 are flat (token, head) positions: row i belongs to expert idx.flat[i]
    ir_rows = ir_dn.cpu().numpy()[pr["idx"].reshape(-1).cpu().numpy()]
    want_a, want_codes = O.dac(np32(p1), ir_rows, None, res)
    np.testing.assert_array_equal(np32(p1q), want_a if dtype == torch.float32 else want_codes)
    z_chain = ops.cvmm_fwd(p1q, pr["values"], ss, offsets, perm, None, M, ir=ir_dn, ir_by_expert=True,
                           inp_res=res, x_is_quantized=True)
    z_plain = ops.cvmm_fwd(p1, pr["values"], ss, offsets, perm, None, M, ir=ir_dn, ir_by_expert=True, inp_res=res)
    assert torch.equal(z_chain, z_plain)


def check_clipped_input_output(ops, device="cpu", dtype=torch.float32, T=100, D=128, F=128, E=3, k=2):
    """gate * clamp(x) left by the input gradient feeds the weight gradient: same weight gradient, bit
    for bit, as clipping and scaling inside the weight-gradient kernel."""
    pr = make_problem(19, T, D, E, F, k, dtype=dtype)
    pr = {n: t.to(device) for n, t in pr.items()}
    ss, perm, in_index, offsets = ops.prepare_sel(pr["idx"], E, k)
    M = T * k
    p1 = torch.randn(M, F).to(dtype).to(device)
    ir_dn = torch.linspace(0.5, 1.1, E, device=device).reshape(E, 1)
    tok = torch.div(perm, k, rounding_mode="floor").to(torch.int32)
    gate, dy = pr["gate"], pr["dy"]
    full, irg, p1c = ops.cvmm_bwd_x(dy, pr["values"], offsets, tok, perm, M, x=p1, xf_index=perm, gate=gate,
                                    ir=ir_dn, ir_by_expert=True, relu_mask=True, decay=0.01, want_xc=True)
    full2, irg2 = ops.cvmm_bwd_x(dy, pr["values"], offsets, tok, perm, M, x=p1, xf_index=perm, gate=gate,
                                 ir=ir_dn, ir_by_expert=True, relu_mask=True, decay=0.01)
    assert torch.equal(full, full2) and torch.equal(irg, irg2)
    ir_rows = ir_dn[pr["idx"].reshape(-1).long()]
    want = (torch.minimum(torch.maximum(p1.float(), -ir_rows), ir_rows) * gate.reshape(-1, 1).float()).to(dtype)
    assert torch.equal(p1c, want)
    a = ops.cvmm_bwd_w(p1c, dy, E, offsets, perm, tok)
    b = ops.cvmm_bwd_w(p1, dy, E, offsets, perm, tok, ir=ir_dn, ir_by_expert=True, g_scale=gate)
    assert torch.equal(a, b)


# ---------------------------------------------------------------------------------- weight modifier / clip
MODIFIER_KINDS = ("DISCRETIZE", "DISCRETIZE_PER_CHANNEL", "ADD_NORMAL", "ADD_NORMAL_PER_CHANNEL",
                  "DISCRETIZE_ADD_NORMAL", "DISCRETIZE_ADD_NORMAL_PER_CHANNEL")


def check_ksum_clip(ops, device="cpu", dtype=torch.float32, T=50, D=96, N=40, E=5, k=3, bounds=None, sel_dtype=torch.int64,
                    strided_x=False, decay=0.01, input_min_percentage=0.5):
    """The up-projection's input gradient as the fused layer makes it (plain GEMM, then the sum over the heads
    with the clip) against the oracle's CVMM.backward and, bit for bit, against the masked GEMM followed by ksum."""
    g = torch.Generator().manual_seed(T + D + k)
    x = torch.randn(T, D + (8 if strided_x else 0), generator=g).to(dtype).to(device)[:, :D]
    keys = (torch.randn(E, D, N, generator=g) / N ** 0.5).to(dtype).to(device)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(sel_dtype).to(device)
    grads = torch.randn(T * k, N, generator=g).to(dtype).to(device)
    nt = 1 if bounds is None else len(bounds) - 1
    ir = torch.from_numpy(np.random.default_rng(5).uniform(0.4, 1.6, size=(E, nt)).astype(np.float32)).to(device)
    sel_sorted, perm, in_index, offsets = ops.prepare_sel(idx, E, k)
    M = T * k
    kw = dict(gradient_relative=True, gradient_scale=0.7, decay=decay, input_min_percentage=input_min_percentage)
    assert ops.ksum_clip_supported(x, k, bounds)
    plain, _ = ops.cvmm_bwd_x(grads, keys, offsets, perm, perm, M)
    got_x, got_irg = ops.ksum_clip(plain, x, idx, perm, offsets, ir, k, bounds=bounds, **kw)
    masked, irg2 = ops.cvmm_bwd_x(grads, keys, offsets, perm, perm, M, x=x, xf_index=in_index, ir=ir, bounds=bounds,
                                  ir_by_expert=True, **kw)
    assert torch.equal(got_x, ops.ksum(masked, k))
    name = dtype_name(dtype)
    want = O.cvmm_backward(np32(grads), np32(x), np32(keys), sel_sorted.cpu().numpy(), in_index.cpu().numpy(),
                           perm.cpu().numpy(), None, ir[sel_sorted.long()].cpu().numpy(), None, k=k, bounds=bounds,
                           dtype=name, **kw)
    tol = {"f32": 1e-5, "bf16": 2e-2, "f16": 2e-3}[name]
    assert rel_err(np32(got_x), want.grad_x) < tol
    assert rel_err(got_irg.cpu().numpy(), want.ir_grad) < tol
    clipped = (x.float().abs()[:, None, :] >= 0.4).float().mean()
    assert 0.05 < float(clipped) < 0.95          # both sides of the mask occur


def modifier_weights(seed, E, K, N, dtype=torch.float32, device="cpu"):
    """Weights with one loud channel and one loud expert, so that per-expert and per-channel maxima differ."""
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(E, K, N, generator=g) * 0.1
    w[:, :, 0] *= 7.0
    w[E - 1] *= 3.0
    return w.to(dtype).to(device)


def check_modify_weight(ops, kind, dtype=torch.float32, device="cpu", E=3, K=40, N=24, res=14.0, std_dev=0.07,
                        seed=0x51EDC0DE12345):
    """The kernel against the oracle, bit for bit: once with injected normals, once with its own draws."""
    from oracle import weights_oracle as WO
    name = dtype_name(dtype)
    w = modifier_weights(7, E, K, N, dtype, device)
    per_channel = kind in WO.PER_CHANNEL_WMAX
    wmax = ops.weight_abs_max(w, per_channel)
    n_states = max(res, 1 / res) if kind.startswith("DISCRETIZE") else 0.0
    sd = std_dev if "ADD_NORMAL" in kind else 0.0
    z = torch.randn(E, K, N, generator=torch.Generator().manual_seed(3)).to(dtype)
    got = ops.modify_weight(w, wmax, n_states, sd, noise=z.float().to(device) if sd > 0 else None)
    want = WO.modify_weight(np32(w), kind, res, std_dev, np32(z), name)
    assert got.dtype == dtype and np.array_equal(np32(got), want), kind
    if sd > 0:
        got2 = ops.modify_weight(w, wmax, n_states, sd, noise_seed=seed)
        want2 = WO.modify_weight(np32(w), kind, res, std_dev, WO.modifier_normals(E, K, N, seed), name)
        # the generator's log2 / sin / cos are hardware approximations: the normals agree to ~1e-6, and in bf16 a
        # sum that lands within that of a rounding boundary may fall to the other side
        err = np.abs(np32(got2) - want2)
        noise_err = 1e-5 * std_dev * float(np32(wmax).max())
        if dtype == torch.bfloat16:
            assert err.max() <= 2.0 ** -7 * np.abs(want2).max() and (err > 0).mean() < 0.02, (kind, err.max())
        else:
            assert err.max() <= noise_err, (kind, err.max(), noise_err)
        d = (np32(got2) - WO.modify_weight(np32(w), kind.replace("_ADD_NORMAL", "").replace("ADD_NORMAL", "NONE")
                                           .replace("NONE_PER_CHANNEL", "NONE"), res, 0.0, None, name))
        scale = std_dev * np32(wmax).reshape(E, 1, -1)
        assert abs((d / scale).std() - 1.0) < 0.1 and abs((d / scale).mean()) < 0.1
        assert not torch.equal(got2, ops.modify_weight(w, wmax, n_states, sd, noise_seed=seed + 1))
    return got


def check_weight_clip(ops, per_channel, dtype=torch.float32, device="cpu", E=3, K=50, N=20, sigma=1.5):
    from oracle import weights_oracle as WO
    name = dtype_name(dtype)
    w = (modifier_weights(9, E, K, N) + 0.5).to(dtype).to(device)       # a mean far from zero
    std = ops.weight_std(w, per_channel)
    want_std = WO.weight_std(np32(w), per_channel)
    assert std.shape == want_std.shape
    np.testing.assert_allclose(np32(std), want_std, rtol=2e-7)
    before = w.clone()
    bound = sigma * std.to(dtype)
    out = ops.clamp_weights_(w, bound)
    assert out is w
    kind = "LAYER_GAUSSIAN_PER_CHANNEL" if per_channel else "LAYER_GAUSSIAN"
    # the clamp itself is exact; against the oracle the bound may sit one ulp away where the two exact sums of
    # the std round to different fp32 neighbours
    b = np32(bound).reshape(E, 1, -1)
    assert np.array_equal(np32(w), np.minimum(np.maximum(np32(before), -b), b))
    want = WO.clip_weights(np32(before), kind, sigma, name)
    if dtype == torch.float32:
        np.testing.assert_allclose(np32(w), want, rtol=3e-7, atol=0)
    assert (np32(w) == want).mean() > 0.999
    assert not torch.equal(w, before)


def check_weight_abs_max(ops, device="cpu"):
    """Per-expert and per-channel max |w| over shapes that exercise one lane group per row, several rows per wave,
    several column blocks and ragged rows."""
    for E, K, N, dtype in [(3, 70, 20, torch.float32), (2, 300, 256, torch.bfloat16), (2, 37, 520, torch.float32),
                           (5, 9, 13, torch.bfloat16), (1, 1, 1, torch.float32), (2, 1030, 8, torch.bfloat16)]:
        w = modifier_weights(E + K, E, K, N, dtype, device)
        assert torch.equal(ops.weight_abs_max(w, True), w.abs().amax(1).float()), (E, K, N)
        assert torch.equal(ops.weight_abs_max(w, False), w.abs().amax((1, 2)).float().reshape(E, 1)), (E, K, N)
        # both tables of a layer from one pair of launches: this tensor and its transposed twin of other values
        w2 = (modifier_weights(E + K + 1, E, N, K, dtype, device) * 3).to(dtype)
        wa, wb = ops.weight_abs_max_pair(w, w2)
        assert torch.equal(wa, w.abs().amax((1, 2)).float().reshape(E, 1)), (E, K, N)
        assert torch.equal(wb, w2.abs().amax((1, 2)).float().reshape(E, 1)), (E, K, N)


# ---------------------------------------------------------------------------------- router epilogue
def check_select(ops, dtype=torch.float32, device="cpu", T=70, E=24, k=3, seed=0):
    """select_fwd / select_bwd against the oracle: gate values bit for bit (the chosen ids carry exactly those
    values; where gate values tie, the kernel takes the lower id like the oracle), regulariser and gradients to
    fp32 / bf16 accuracy."""
    from oracle import select_oracle as SO
    name = dtype_name(dtype)
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(T, E, generator=g) * 2.0).to(dtype)
    logits[0, :] = logits[0, 0]                                     # a row of ties
    dev = logits.to(device)
    val, idx, reg, reg_c = ops.select_fwd(dev, k, True)
    want_val, want_idx = SO.select(np32(logits), k, name)
    # expf differs in the last fp32 bit between the device library, the host library and numpy: fp32 gate values
    # agree to an ulp (and the order of two experts whose values differ by less may swap), bf16 ones exactly
    if dtype == torch.bfloat16:
        assert np.array_equal(np32(val), want_val)
        assert np.array_equal(idx.cpu().numpy(), want_idx)
    else:
        np.testing.assert_allclose(np32(val), want_val, rtol=3e-7)
        assert (idx.cpu().numpy() == want_idx).mean() > 0.999
    sig = 1.0 / (1.0 + np.exp(-np32(logits).astype(np.float64)))
    np.testing.assert_allclose(np.take_along_axis(sig, idx.cpu().numpy(), -1), np32(val),
                               rtol=1e-2 if dtype == torch.bfloat16 else 1e-6)
    assert all(len(set(r)) == k for r in idx.cpu().numpy().tolist())
    want_reg, want_c = SO.usage_regulariser(np32(logits))
    np.testing.assert_allclose(float(reg), want_reg, rtol=1e-5)
    np.testing.assert_allclose(np32(reg_c), want_c, rtol=1e-5, atol=1e-6)
    v2, i2, r2, c2 = ops.select_fwd(dev, k, False)
    assert torch.equal(v2, val) and torch.equal(i2, idx) and r2.numel() == 0 and c2.numel() == 0
    gv = torch.randn(T, k, generator=g).to(dtype)
    greg = torch.tensor(0.7)
    tol = dict(rtol=2e-2, atol=2e-3) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-6)
    for use_val, use_reg in ((True, True), (True, False), (False, True)):
        got = ops.select_bwd(dev, idx, gv.to(device) if use_val else None, reg_c if use_reg else None,
                             greg.to(device) if use_reg else None)
        want = SO.select_bwd(np32(logits), idx.cpu().numpy(), np32(gv) if use_val else None,
                             0.7 if use_reg else None, name)
        np.testing.assert_allclose(np32(got), want, **tol)


def check_weights_in_registers_kernel(ops, device="cpu", dtype=torch.bfloat16, T=330, D=512, E=4, k=2, noisy=True):
    """The kernel that keeps an expert's weights in registers (contraction of exactly 256): every variant against
    the oracle, and the byte-coded result bit for bit against the 128 x 256 kernel's value result.  Uneven experts:
    one without rows, one with more rows than a work item takes, the others ending inside a 32-row block."""
    F = 256
    name = dtype_name(dtype)
    tol = {torch.bfloat16: 2e-2, torch.float16: 2e-3}[dtype]
    g = torch.Generator().manual_seed(41)
    idx = torch.randint(0, E - 1, (T, k), generator=g)           # expert E - 1 gets nothing
    idx[: T // 2, 0] = 0                                         # expert 0 gets more than 256 rows
    M = T * k
    res = 1.0 / 127.0
    ir = torch.linspace(0.7, 1.6, E).reshape(E, 1)
    codes_in = torch.randint(-127, 128, (M, F), generator=g).float()
    values = (torch.randn(E, F, D, generator=g) / F ** 0.5).to(dtype)
    ss, perm, in_index, offsets = ops.prepare_sel(idx.to(device), E, k)
    counts = torch.bincount(idx.reshape(-1), minlength=E)
    assert int(counts[E - 1]) == 0 and int(counts[0]) > 256 and any(int(c) % 32 for c in counts)
    sel_np, perm_np = ss.cpu().numpy(), perm.cpu().numpy()
    ir_rows = ir.numpy()[sel_np]                                 # per sorted position
    # the values whose DAC codes codes_in are: row r of the operand belongs to the expert of flat position r
    e_of_row = idx.reshape(-1).numpy()
    x_real = (codes_in.numpy() * np.float32(res)).astype(np.float32) * ir.numpy()[e_of_row]
    wmax = ops.weight_abs_max(values.to(device), False)
    wm_np = values.float().abs().amax((1, 2)).reshape(E, 1).numpy()
    p1q, vals = codes_in.to(dtype).to(device), values.to(device)
    common = dict(ir=ir.to(device), ir_by_expert=True, inp_res=res, x_is_quantized=True)
    analog = dict(out_bound=12.0, out_res=254.0, wmax=wmax, noise_std=0.04 if noisy else 0.0, noise_seed=91)
    okw = dict(inp_res=res, ir=ir_rows, dtype=name)
    # (1) result as ADC codes (weights in registers) == result as values (128 x 256 kernel), and both against the oracle
    codes, scale = ops.cvmm_fwd(p1q, vals, ss, offsets, perm, None, M, want_codes=True, **common, **analog)
    z = ops.cvmm_fwd(p1q, vals, ss, offsets, perm, None, M, **common, **analog)
    zf = ops.dequant_codes(codes, scale, idx.to(device))
    assert torch.equal(zf.to(dtype), z)
    want = O.cvmm_fwd(x_real, perm_np, sel_np, np32(values), out_index=None, wmax=wm_np, out_bound=12.0, out_res=254.0,
                      noise_std=0.04 if noisy else 0.0, noise_seed=91 if noisy else None, **okw)
    step = 12.0 * float(wm_np.max()) / 127.0 * float(ir.max())
    flipped = adc_flip_check(np32(zf.to(dtype)), want, tol, step)
    # (2) codes in, no output stage: the rescaled product
    s_got = ops.cvmm_fwd(p1q, vals, ss, offsets, perm, None, M, **common)
    s_want = O.cvmm_fwd(x_real, perm_np, sel_np, np32(values), out_index=None, **okw)
    assert rel_err(np32(s_got), s_want) < tol
    # (3) the plain product, column-contiguous weights (a forward) and contraction-contiguous weights (an input gradient)
    a = torch.randn(M, F, generator=g).to(dtype)
    p_got = ops.cvmm_fwd(a.to(device), vals, ss, offsets, perm, None, M)
    p_want = O.cvmm_fwd(np32(a), perm_np, sel_np, np32(values), out_index=None, dtype=name)
    assert rel_err(np32(p_got), p_want) < tol
    keys = values.transpose(1, 2).contiguous()                  # [E, D, F]: the up-projection's weights
    g_got, none = ops.cvmm_bwd_x(a.to(device), keys.to(device), offsets, perm, perm, M)
    assert none is None
    assert rel_err(np32(g_got), p_want) < tol                    # G = a @ keys[e]^T is the same product
    assert torch.equal(g_got, p_got)
    return dict(flipped=flipped)


def check_layer_tables(ops, device="cpu", dtype=torch.bfloat16, E=5, D=72, F=40, n_up=2, n_dn=1):
    """The four per-expert tables of a layer from one pair of launches equal what the separate calls give."""
    g = torch.Generator().manual_seed(3)
    keys = (torch.randn(E, D, F, generator=g)).to(dtype).to(device)
    values = (torch.randn(E, F, D, generator=g)).to(dtype).to(device)
    for ir_dtype in (torch.float32, dtype):
        ir = (torch.rand(2, E, max(n_up, n_dn), generator=g) + 0.5).to(ir_dtype).to(device)
        wu, wd, ir_up, ir_dn = ops.layer_tables(keys, values, ir, n_up, n_dn)
        assert torch.equal(wu, ops.weight_abs_max(keys, False)) and torch.equal(wd, ops.weight_abs_max(values, False))
        assert torch.equal(ir_up, ir[0, :, :n_up].float()) and torch.equal(ir_dn, ir[1, :, :n_dn].float())
        assert ir_up.dtype == torch.float32 and ir_up.is_contiguous() and ir_dn.is_contiguous()


def check_segment_sum_typed(ops, device="cpu"):
    """Per-expert sums land in a slice of a wider table, in the table's type, and clear the columns after the slice
    (the index backward of input_range[sel], moe_layer_aihwkit_lightning.py:447-448, sums in the parameter's type)."""
    g = torch.Generator().manual_seed(5)
    offsets = torch.tensor([0, 3, 3, 10, 11, 40, 57], dtype=torch.int32, device=device)      # one expert without rows
    E = offsets.numel() - 1
    v = torch.randn(57, 2, generator=g).to(device)
    want = torch.stack([v[offsets[e]:offsets[e + 1]].double().sum(0) for e in range(E)])
    plain = ops.segment_sum(v, offsets, E)
    assert plain.dtype == torch.float32 and (plain.double() - want).abs().max() < 1e-5
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        table = torch.full((2, E, 4), 7.0, dtype=dt, device=device)
        ops.segment_sum(v, offsets, E, out=table[1, :, :2], zero_cols=1)
        assert torch.equal(table[1, :, :2], plain.to(dt))                    # one rounding of the fp32 sum
        assert bool((table[1, :, 2] == 0).all()) and bool((table[1, :, 3] == 7).all()) and bool((table[0] == 7).all())
    with pytest.raises(ValueError):
        ops.segment_sum(v, offsets, E, out=torch.zeros(E, 2, device=device), zero_cols=1)     # rows too close


def check_gate_reduce_counter(ops, device="cpu"):
    """The gate reductions add to a device word in the same launch (the step counter of the generated noise), also
    when there is nothing to reduce; the reduction itself is unchanged."""
    g = torch.Generator().manual_seed(6)
    T, k, D, E = 9, 3, 32, 4
    z = torch.randn(T * k, D, generator=g).to(device)
    gate = torch.rand(T, k, generator=g).to(device)
    counter = torch.tensor([5], dtype=torch.int64, device=device)
    assert torch.equal(ops.gate_reduce(z, gate, counter, 2), ops.gate_reduce(z, gate)) and int(counter) == 7
    codes = torch.randint(0, 256, (T * k, D), generator=g, dtype=torch.uint8).to(device)
    scale = (torch.rand(E, 2, generator=g) + 0.1).to(device)
    sel = torch.randint(0, E, (T, k), generator=g).to(device)
    assert torch.equal(ops.gate_reduce_codes(codes, scale, sel, gate, counter, 3),
                       ops.gate_reduce_codes(codes, scale, sel, gate)) and int(counter) == 10
    assert ops.gate_reduce(z[:0], gate[:0], counter, 1).shape == (0, D) and int(counter) == 11
    assert ops.gate_reduce_codes(codes[:0], scale, sel[:0], gate[:0], counter, 1).shape == (0, D) and int(counter) == 12
