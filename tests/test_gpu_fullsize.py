"""BASELINE configurations 3 and 4 at full size WITH their analog stages, through the fused feed-forward
(analog_moe_amd.ffn: the path the layer and the benchmark run), on the GPU.

The oracle is too slow at these sizes, so the check is made on samples in float64 torch arithmetic written out
here from the stage definitions (DAC codes by the two fp32 divisions of cvmm.py:150-167; per K-tile: product,
injected noise, ADC, rescale; tiles summed; ReLU): sampled sorted positions of both forward stages (each from the
kernels' own input to that stage, with the whole-ADC-step allowance for values next to a rounding boundary),
whole weight gradients of sampled experts, input gradients of sampled tokens, gate gradients and the per-expert
input-range gradients.  Tolerance: bf16, 2e-2 relative to the tensor's scale."""
import numpy as np
import pytest
import torch

from tests import util

pytestmark = pytest.mark.gpu
RES = 1.0 / 127.0
OUT_BOUND, OUT_RES, NOISE = 12.0, 254.0, 0.04


@pytest.fixture(scope="module")
def ops():
    from analog_moe_amd import ops as _ops
    _ops.get_lib()
    return _ops


def _bounds(K, mis):
    if mis <= 0 or mis >= K:
        return [0, K]
    n = -(-K // mis)
    base, rem = divmod(K, n)
    out = [0]
    for i in range(n):
        out.append(out[-1] + base + (1 if i < rem else 0))
    return out


def _dac_codes(rows, r):
    """rows [R, K] (any float dtype), r [R, 1] fp32 -> integer codes as float64; fp32 arithmetic in the order
    of cvmm.py:146-166."""
    a = rows.float()
    a = torch.minimum(torch.maximum(a, -r), r)
    a = a / r
    a = a / torch.tensor(RES, dtype=torch.float32, device=a.device)
    return torch.round(a).double()


def _stage(rows, w_e, ir_e, bounds, noise_rows, wmax_e):
    """One forward stage for R sampled rows in float64.  rows [R, K]; w_e [R, K, N] (the rows' experts' weights);
    ir_e [R, n_tiles]; noise_rows [n_tiles, R, N]; wmax_e [R, 1].  Returns (result, ADC step * largest range)."""
    half = OUT_RES / 2
    bound = (OUT_BOUND * wmax_e.float())                         # fp32, as the kernel forms it
    inv_step = (torch.tensor(half, dtype=torch.float32, device=rows.device) / bound).double()
    step = (bound / torch.tensor(half, dtype=torch.float32, device=rows.device)).double()
    total = 0
    for t in range(len(bounds) - 1):
        lo, hi = bounds[t], bounds[t + 1]
        r = ir_e[:, t:t + 1].float()
        codes = _dac_codes(rows[:, lo:hi], r)
        c = torch.einsum("rk,rkn->rn", codes, w_e[:, lo:hi].double()) * float(np.float32(RES))
        c = c + noise_rows[t].double()
        c = torch.minimum(torch.maximum(c, -bound.double()), bound.double())
        c = torch.round(c * inv_step) * step
        total = total + c * r.double()
    return total, float((step * ir_e.double().amax(1, keepdim=True)).max())


def _flip_check(got, want, max_step, n_tiles, name):
    """Element by element: the stored bf16 value is within 2^-7 of the float64 one (relative to that element),
    which is far finer than the noise or one ADC step; the few elements next to an ADC rounding boundary differ by
    whole steps instead (at most one per K-tile)."""
    scale = float(want.abs().max())
    d = (got.double() - want).abs()
    off = d > want.abs() * 2.0 ** -7 + 1e-5 * scale
    frac = float(off.double().mean())
    assert frac <= 2e-3, f"{name}: {frac:.2e} of the sampled elements differ"
    if bool(off.any()):
        assert float(d[off].max()) <= n_tiles * max_step * 1.01 + 2.0 ** -7 * scale, (name, float(d[off].max()), max_step)
    return frac


@pytest.mark.parametrize("name,T,D,E,F,k,routing,mis", [("config3", 16384, 1024, 64, 256, 8, "uniform", 512),
                                                         ("config4", 32768, 2048, 128, 512, 4, "zipf", -1)])
def test_full_size_analog_layer(ops, name, T, D, E, F, k, routing, mis):
    from analog_moe_amd import ffn
    print(name, "full size, analog stages, fused path", flush=True)
    dev = "cuda"
    tol = 2e-2
    pr = util.make_problem(0, T, D, E, F, k, dtype=torch.bfloat16, routing=routing)
    pr = {n: t.to(dev) for n, t in pr.items()}
    x, keys, values, idx, gate, dy = (pr[n] for n in ("x", "keys", "values", "idx", "gate", "dy"))
    M = T * k
    bu, bd = _bounds(D, mis), _bounds(F, mis)
    ntu, ntd = len(bu) - 1, len(bd) - 1
    nt = max(ntu, ntd)
    g = torch.Generator(device=dev).manual_seed(11)
    # learned-looking ranges: some inputs clip on every tile of both projections
    ir = torch.empty(2, E, nt, device=dev).uniform_(1.6, 2.6, generator=g)
    ir[1] *= 0.5
    wmax_up = keys.float().abs().amax((1, 2)).reshape(E, 1)
    wmax_dn = values.float().abs().amax((1, 2)).reshape(E, 1)
    flat = idx.reshape(-1)
    noise_up = torch.randn(ntu, M, F, device=dev, generator=g) * (NOISE * wmax_up[flat]).reshape(1, M, 1)
    noise_dn = torch.randn(ntd, M, D, device=dev, generator=g) * (NOISE * wmax_dn[flat]).reshape(1, M, 1)
    decay, min_pct = 0.01, 0.5
    cfg = ffn.FFNConfig(inp_res=RES, bounds_up=bu if ntu > 1 else None, bounds_down=bd if ntd > 1 else None,
                        out_bound=OUT_BOUND, out_res=OUT_RES, noise_std=NOISE, noise_up=noise_up, noise_down=noise_dn,
                        decay=decay, input_min_percentage=min_pct, gradient_relative=True, gradient_scale=1.0)
    y, p1, z, perm, in_index, offsets, z_scale, ir_up, ir_dn = ffn.ffn_forward(x, keys, values, ir, gate, idx, cfg)
    torch.cuda.synchronize()
    print("forward done", flush=True)
    z_kept = z
    if z.dtype == torch.uint8:                       # the k-head result was kept as ADC codes
        z = ops.dequant_codes(z, z_scale, idx)
    ss = flat[perm.long()]
    assert torch.equal(ir_up, ir[0, :, :ntu]) and torch.equal(ir_dn, ir[1, :, :ntd])

    # ---- forward stages on sampled sorted positions
    cpu_g = torch.Generator().manual_seed(1)
    pos = torch.randint(0, M, (128,), generator=cpu_g).to(dev)
    e_of = ss[pos].long()
    flat_pos = perm[pos].long()
    want_p1, step_up = _stage(x[in_index[pos].long()], keys[e_of], ir_up[e_of], bu, noise_up[:, flat_pos],
                              wmax_up[e_of])
    want_p1 = torch.relu(want_p1)
    f1 = _flip_check(p1[flat_pos], want_p1, step_up, ntu, "up-projection")
    want_z, step_dn = _stage(p1[flat_pos], values[e_of], ir_dn[e_of], bd, noise_dn[:, flat_pos], wmax_dn[e_of])
    f2 = _flip_check(z[flat_pos], want_z, step_dn, ntd, "down-projection")
    tk = torch.randint(0, T, (64,), generator=cpu_g).to(dev)
    want_y = (gate[tk].double().unsqueeze(-1) * z.view(T, k, D)[tk].double()).sum(1)
    assert float((y[tk].double() - want_y).abs().max() / want_y.abs().max()) < tol
    print("forward samples ok; elements off by whole ADC steps:", f1, f2, flush=True)

    # ---- backward
    grad_x, grad_keys, grad_values, grad_ir, grad_gate = ffn.ffn_backward(
        dy, x, keys, values, gate, idx, p1, z_kept, z_scale, perm, in_index, offsets, ir_up, ir_dn, cfg, True)
    torch.cuda.synchronize()
    print("backward done", flush=True)
    tok = torch.div(perm, k, rounding_mode="floor").long()

    def tile_range(ir_tab, bounds, e_rows):
        """[R, K] range of every input column of rows whose experts are e_rows."""
        cols = torch.zeros(bounds[-1], dtype=torch.long, device=dev)
        for t in range(len(bounds) - 1):
            cols[bounds[t]:bounds[t + 1]] = t
        return ir_tab[e_rows][:, cols]

    def gp1_rows(positions, e=None):
        """Gradient wrt p1 (ReLU and clip masks applied, gate-scaled; float64, not yet rounded to the bf16 it is
        stored in) of sorted positions, and the same before the masks.  e: the one expert all positions belong to."""
        e_r = ss[positions].long()
        fp = perm[positions].long()
        if e is None:
            G = torch.einsum("rn,rkn->rk", dy[tok[positions]].double(), values[e_r].double())
        else:
            G = dy[tok[positions]].double() @ values[e].double().t()
        p = p1[fp].float()
        r = tile_range(ir_dn, bd, e_r)
        keep = (p.abs() < r) & (p > 0)
        gs = G * gate.reshape(-1)[fp].double().unsqueeze(-1)
        return gs * keep, gs, e_r, fp

    # gate gradient
    gt = grad_gate.reshape(T, k)[tk]
    want_gg = torch.einsum("tkd,td->tk", z.view(T, k, D)[tk].double(), dy[tk].double())
    assert float((gt.double() - want_gg).abs().max() / want_gg.abs().max()) < tol

    # weight gradients of three experts: the most loaded, the least loaded (non-empty) and one in between
    counts = (offsets[1:] - offsets[:-1]).cpu()
    nonempty = torch.nonzero(counts > 0).reshape(-1)
    order = nonempty[torch.argsort(counts[nonempty])]
    picks = sorted({int(order[-1]), int(order[0]), int(order[len(order) // 2])})
    for e in picks:
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        rows = torch.arange(lo, hi, device=dev)
        gp, _, e_r, fp = gp1_rows(rows, e)
        # values: (gate * clamp(p1)) rounded to bf16, transposed, times dy
        r = tile_range(ir_dn, bd, e_r)
        p = p1[fp].float()
        pc = (torch.minimum(torch.maximum(p, -r), r) * gate.reshape(-1)[fp].float().unsqueeze(-1)).bfloat16().double()
        want_gv = pc.t() @ dy[tok[rows]].double()
        err = float((grad_values[e].double() - want_gv).abs().max() / want_gv.abs().max())
        assert err < tol, ("grad_values", e, err)
        # keys: clamp(x) per K-tile, transposed, times the stored (bf16) gradient of p1
        ru = tile_range(ir_up, bu, e_r)
        xr = x[in_index[rows].long()].float()
        xc = torch.minimum(torch.maximum(xr, -ru), ru).double()
        want_gk = xc.t() @ gp.bfloat16().double()
        err = float((grad_keys[e].double() - want_gk).abs().max() / want_gk.abs().max())
        assert err < tol, ("grad_keys", e, err)
    print("weight gradients ok for experts", picks, flush=True)

    # input gradient of sampled tokens: sum over the k heads of mask * (gp1 @ keys[e]^T)
    inv = torch.empty(M, dtype=torch.long, device=dev)
    inv[perm.long()] = torch.arange(M, device=dev)
    tk2 = tk[:32]
    want_gx = torch.zeros(len(tk2), D, dtype=torch.float64, device=dev)
    for j in range(k):
        positions = inv[tk2 * k + j]
        gp, _, e_r, fp = gp1_rows(positions)
        G = torch.einsum("rf,rdf->rd", gp.bfloat16().double(), keys[e_r].double())
        ru = tile_range(ir_up, bu, e_r)
        keep = x[tk2].float().abs() < ru
        want_gx += (G * keep).bfloat16().double()
    err = float((grad_x[tk2].double() - want_gx).abs().max() / want_gx.abs().max())
    assert err < tol, ("grad_x", err)

    # input-range gradients per expert (cvmm.py:863-878 summed over the expert's rows), both projections
    def not_clipped_share(inp, ir_tab, bounds, rows_of):
        tot = 0
        CH = 16384
        for s0 in range(0, M, CH):
            rows = torch.arange(s0, min(s0 + CH, M), device=dev)
            r = tile_range(ir_tab, bounds, ss[rows].long())
            tot += int((inp[rows_of(rows)].float().abs() < r).sum())
        return tot / (M * bounds[-1])
    pct_up = not_clipped_share(x, ir_up, bu, lambda rows: in_index[rows].long())
    pct_dn = not_clipped_share(p1, ir_dn, bd, lambda rows: perm[rows].long())
    assert abs(pct_up - min_pct) > 0.02 and abs(pct_dn - min_pct) > 0.02       # the decay rule is not on its edge
    for e in picks:
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        rows = torch.arange(lo, hi, device=dev)
        gp, gs, e_r, fp = gp1_rows(rows, e)        # gs: gate-scaled gradient wrt the down-projection's input
        p = p1[fp].float()
        for t in range(ntd):
            sl = slice(bd[t], bd[t + 1])
            r = float(ir_dn[e, t])
            s_ = (torch.clamp((p[:, sl] >= r) * gs[:, sl], max=0).sum()
                  - torch.clamp((p[:, sl] <= -r) * gs[:, sl], min=0).sum())
            want = float(s_) * r + (decay * r * (hi - lo) if pct_dn > min_pct else 0.0)
            got = float(grad_ir[1, e, t])
            assert abs(got - want) <= tol * max(abs(want), 1e-3) + 1e-4, ("grad_ir down", e, t, got, want)
        xr = x[in_index[rows].long()].float()
        Gu = gp.bfloat16().double() @ keys[e].double().t()
        for t in range(ntu):
            sl = slice(bu[t], bu[t + 1])
            r = float(ir_up[e, t])
            s_ = (torch.clamp((xr[:, sl] >= r) * Gu[:, sl], max=0).sum()
                  - torch.clamp((xr[:, sl] <= -r) * Gu[:, sl], min=0).sum())
            want = float(s_) * r + (decay * r * (hi - lo) if pct_up > min_pct else 0.0)
            got = float(grad_ir[0, e, t])
            assert abs(got - want) <= tol * max(abs(want), 1e-3) + 1e-4, ("grad_ir up", e, t, got, want)
    print("input and input-range gradients ok", flush=True)


@pytest.mark.parametrize("routing", ["uniform", "near_uniform"])
def test_config3_full_size_generated_noise(ops, routing):
    """The instantiations the benchmark times, at the benchmark's size: configuration 3 with the output noise DRAWN
    IN THE KERNELS (the two-K-tile up-projection with the second output; the down-projection on the kernel that
    holds the weights in registers, its result as ADC codes), sampled rows against float64 with the oracle's
    counter noise.  near_uniform: expert loads that differ by a few percent, so that row tiles and block runs end
    inside experts."""
    from analog_moe_amd import ffn
    from oracle import cvmm_oracle as O
    T, D, E, F, k, mis = 16384, 1024, 64, 256, 8, 512
    print("config3 full size, generated noise", routing, flush=True)
    dev = "cuda"
    pr = util.make_problem(0, T, D, E, F, k, dtype=torch.bfloat16, routing=routing)
    pr = {n: t.to(dev) for n, t in pr.items()}
    x, keys, values, idx, gate = (pr[n] for n in ("x", "keys", "values", "idx", "gate"))
    M = T * k
    bu, bd = _bounds(D, mis), _bounds(F, mis)
    ntu, ntd = len(bu) - 1, len(bd) - 1
    g = torch.Generator(device=dev).manual_seed(11)
    ir = torch.empty(2, E, max(ntu, ntd), device=dev).uniform_(1.6, 2.6, generator=g)
    ir[1] *= 0.5
    wmax_up = keys.float().abs().amax((1, 2)).reshape(E, 1)
    wmax_dn = values.float().abs().amax((1, 2)).reshape(E, 1)
    seed = 0x0123456789ABCDE
    word = torch.tensor([5], dtype=torch.int64, device=dev)          # the device part of the seed
    cfg = ffn.FFNConfig(inp_res=RES, bounds_up=bu, bounds_down=None, out_bound=OUT_BOUND, out_res=OUT_RES,
                        noise_std=NOISE, noise_seed=seed, noise_seed_dev=word)
    y, p1, z, perm, in_index, offsets, z_scale, ir_up, ir_dn = ffn.ffn_forward(x, keys, values, ir, gate, idx, cfg)
    torch.cuda.synchronize()
    assert z.dtype == torch.uint8, "the benchmark's down-projection leaves ADC codes"
    z = ops.dequant_codes(z, z_scale, idx)
    flat = idx.reshape(-1)
    ss = flat[perm.long()]
    cpu_g = torch.Generator().manual_seed(2)
    pos = torch.randint(0, M, (192,), generator=cpu_g)
    pos[:8] = torch.tensor([0, 1, 31, 32, M - 1, M - 32, M // 2, M // 2 + 33])
    pos = pos.to(dev)
    e_of = ss[pos].long()
    flat_pos = perm[pos].long()
    starts = (offsets[e_of] + torch.div(pos - offsets[e_of], 32, rounding_mode="floor") * 32).cpu().numpy()
    out_rows = flat_pos.cpu().numpy()

    def drawn(n_cols, n_tiles, s, wmax_e):
        zi = np.stack([O.counter_noise_int(out_rows, starts, n_cols, t, s) for t in range(n_tiles)]).astype(np.float64)
        scale = ((np.float32(NOISE) * wmax_e.cpu().numpy().astype(np.float32)) * O.NOISE_SCALE).astype(np.float32)
        return torch.from_numpy(zi * scale.astype(np.float64).reshape(1, -1, 1)).to(dev)

    want_p1, step_up = _stage(x[in_index[pos].long()], keys[e_of], ir_up[e_of], bu,
                              drawn(F, ntu, seed + 5, wmax_up[e_of]), wmax_up[e_of])
    f1 = _flip_check(p1[flat_pos], torch.relu(want_p1), step_up, ntu, "up-projection")
    want_z, step_dn = _stage(p1[flat_pos], values[e_of], ir_dn[e_of], bd, drawn(D, ntd, seed + 1 + 5, wmax_dn[e_of]),
                             wmax_dn[e_of])
    f2 = _flip_check(z[flat_pos], want_z, step_dn, ntd, "down-projection")
    print("generated-noise samples ok; elements off by whole ADC steps:", f1, f2, flush=True)
    # the noise is there: the same call with another device word gives another result
    word.add_(2)
    p1_b = ffn.ffn_forward(x, keys, values, ir, gate, idx, cfg)[1]
    assert not torch.equal(p1_b, p1)


@pytest.mark.parametrize("name,T,D,E,F,k,routing,mis", [("config3", 16384, 1024, 64, 256, 8, "uniform", 512)])
def test_full_size_bf16_dac_codes_exact(ops, name, T, D, E, F, k, routing, mis):
    """Every bf16 DAC code of a full-size launch equals round((clamp(x) / r) / res) evaluated by torch in fp32 on
    the same GPU (cvmm.py:146-166): the DAC image the up-projection emits for the down-projection (1.3e8 / 4
    elements), with learned-looking ranges."""
    print(name, "DAC codes at full size", flush=True)
    dev = "cuda"
    pr = util.make_problem(0, T, D, E, F, k, dtype=torch.bfloat16, routing=routing)
    pr = {n: t.to(dev) for n, t in pr.items()}
    M = T * k
    ss, perm, in_index, offsets = ops.prepare_sel(pr["idx"], E, k)
    g = torch.Generator(device=dev).manual_seed(3)
    ir_up = torch.empty(E, 2, device=dev).uniform_(1.5, 3.5, generator=g)
    ir_dn = torch.empty(E, 1, device=dev).uniform_(0.4, 2.0, generator=g)
    p1, img = ops.cvmm_fwd(pr["x"], pr["keys"], ss, offsets, in_index, perm, M, ir=ir_up, ir_by_expert=True,
                           inp_res=RES, bounds=[0, 512, 1024], relu=True, xq_ir=ir_dn[:, 0].contiguous(),
                           xq_inp_res=RES)
    r = ir_dn[pr["idx"].reshape(-1)]                           # rows of p1 are flat (token, head) positions
    want = _dac_codes(p1, r)
    mism = int((img.double() != want).sum())
    assert mism == 0, f"{mism} of {img.numel()} codes differ"
    assert float(want.abs().max()) == 127.0 and int((want == 0).sum()) < want.numel()


# ------------------------------------------------------------------------------- the layer inside its caller
def _decoder(cfgmod, *, vocab, d_model, n_layers, n_heads, context, E, F, k, noise=NOISE, dtype=torch.bfloat16):
    from analog_moe_amd.decoder import SigmaMoEDecoder
    from analog_moe_amd.moe_layer import AnalogSigmaMoELayer

    def make(i):
        r = cfgmod.TorchInferenceRPUConfig()
        r.forward.inp_res = r.forward.out_res = 2 ** 8 - 2
        r.forward.out_bound = OUT_BOUND
        r.forward.out_noise = noise
        ir = r.pre_post.input_range
        ir.enable, ir.learn_input_range, ir.init_value, ir.decay = True, True, 3.0, 0.01
        return AnalogSigmaMoELayer(r, d_model=d_model, n_experts=E, expert_size=F, k=k)
    torch.manual_seed(0)
    model = SigmaMoEDecoder(vocab, d_model, n_layers, n_heads, context, make).cuda().to(dtype)
    model.train()
    for blk in model.blocks:
        blk.ffn.use_device_noise_counter()
    return model


def test_config5_full_size_training_step():
    """BASELINE configuration 5 at full size: one training step (and a second one after the optimizer update) of the
    16-layer decoder -- d_model 1024, 16 heads, 64 experts x 256, k = 8, context 1024, batch 16, vocabulary 8000,
    bf16, 8-bit DAC / ADC, output noise drawn in the kernels, learned input ranges.  The loss is finite, every
    parameter of every block gets a finite gradient, and the feed-forward of a middle block returns exactly what
    the stand-alone layer computes from the captured input under the same noise seed."""
    from analog_moe_amd import config as cfgmod
    print("config 5, full size", flush=True)
    V, D, L, H, S, B = 8000, 1024, 16, 16, 1024, 16
    model = _decoder(cfgmod, vocab=V, d_model=D, n_layers=L, n_heads=H, context=S, E=64, F=256, k=8)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, V, (B, S), generator=g).cuda()
    labels = torch.roll(ids, -1, dims=1)
    ffn = model.blocks[7].ffn
    seen = {}
    h0 = ffn.register_forward_pre_hook(lambda m, a: seen.update(counter=m.noise_counter.clone()))
    h1 = ffn.register_forward_hook(lambda m, a, out: seen.update(x=a[0].detach(), y=out[0].detach(),
                                                                 reg=out[1].detach()))
    opt = torch.optim.AdamW(model.parameters(), lr=1e-4)
    loss, reg = model(ids, labels, reg_weight=0.01)
    h0.remove()
    h1.remove()
    assert torch.isfinite(loss) and torch.isfinite(reg)
    assert abs(float(loss.detach()) - float(np.log(V))) < 1.0          # random initialisation: about log(vocabulary)
    loss.backward()
    missing = [n for n, p in model.named_parameters() if p.requires_grad and p.grad is None]
    assert missing == []
    bad = [n for n, p in model.named_parameters() if p.grad is not None and not bool(torch.isfinite(p.grad).all())]
    assert bad == []
    dead = [n for n, p in model.named_parameters()
            if p.grad is not None and ("keys" in n or "values" in n) and float(p.grad.abs().max()) == 0.0]
    assert dead == []
    # the block's feed-forward against the stand-alone layer: same input, same noise seed word
    assert seen["x"].shape == (B, S, D)
    after = ffn.noise_counter.clone()
    ffn.noise_counter.copy_(seen["counter"])
    with torch.no_grad():
        alone, reg_alone = ffn(seen["x"])
    assert torch.equal(ffn.noise_counter, after)
    assert torch.equal(alone, seen["y"]) and torch.equal(reg_alone, seen["reg"])
    opt.step()
    model.post_update_step()
    opt.zero_grad(set_to_none=True)
    loss2, _ = model(ids, labels, reg_weight=0.01)
    assert torch.isfinite(loss2) and float(loss2.detach()) < float(loss.detach()) + 0.5
    torch.cuda.synchronize()


def test_decoder_step_in_a_hip_graph_matches_eager_steps():
    """The whole training step (forward, loss, backward, AdamW, weight clipping) captured once and replayed: every
    replay's loss against the loss of the same step launched eagerly from the same initial state.  The noise
    seeds advance in device memory, so both sequences draw the same noise; what differs is the order of
    atomic additions in stock PyTorch kernels (embedding gradients), hence the tolerance."""
    from analog_moe_amd import config as cfgmod
    print("decoder step in a HIP graph", flush=True)
    kw = dict(vocab=211, d_model=256, n_layers=2, n_heads=4, context=64, E=8, F=256, k=2)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, 211, (16, 64), generator=g).cuda()
    labels = torch.roll(ids, -1, dims=1)

    def steps(graph, n=6, warm=3):
        model = _decoder(cfgmod, **kw)
        opt = torch.optim.AdamW(model.parameters(), lr=1e-3, capturable=True)

        def step():
            loss, _ = model(ids, labels, reg_weight=0.01)
            loss.backward()
            opt.step()
            model.post_update_step()
            return loss.detach()
        out = []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warm):
                opt.zero_grad(set_to_none=True)
                out.append(float(step()))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        if not graph:
            for _ in range(n):
                opt.zero_grad(set_to_none=True)
                out.append(float(step()))
            return out
        cg = torch.cuda.CUDAGraph()
        opt.zero_grad(set_to_none=True)
        with torch.cuda.graph(cg):
            captured = step()
        for i in range(n - 1):           # (the capture itself does not run the step)
            cg.replay()
            torch.cuda.synchronize()
            out.append(float(captured))
            _ = torch.randn(64, 64, device="cuda").sum().item()      # eager work between the replays
        return out
    eager = steps(False)
    replayed = steps(True)
    print(eager, replayed)
    assert all(np.isfinite(eager)) and all(np.isfinite(replayed))
    assert eager[-1] < eager[0]
    for a, b in zip(eager[:len(replayed)], replayed):
        assert abs(a - b) < 2e-2 * abs(a), (eager, replayed)
