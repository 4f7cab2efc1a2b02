"""Pins the CPU oracle (oracle/cvmm_oracle.py) against things the oracle does not define
itself: library routines (torch.sort, torch.clamp/round, torch.std, einsum), brute-force
per-token loops, autograd of an independent surrogate, closed forms and invariants.
Shapes follow the reference's own tests (D=128, E=4, F=64, k=2, 10x10 tokens:
test_moe_layer_aihwkit_lightning.py:211-217)."""
import os

import numpy as np
import pytest
import torch

from oracle import cvmm_oracle as O

RNG = np.random.default_rng


def _problem(seed=0, T=100, D=128, E=4, F=64, k=2):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, D, generator=g)
    keys = torch.randn(E, D, F, generator=g) / D ** 0.5
    values = torch.randn(E, F, D, generator=g) / F ** 0.5
    router = torch.randn(E, D, generator=g) / D ** 0.5
    gate, idx = torch.sigmoid(x @ router.t()).topk(k, dim=-1, sorted=False)
    return x, keys, values, idx, gate


# ------------------------------------------------------------------ selection
@pytest.mark.parametrize("M,E,k", [(0, 4, 1), (1, 1, 1), (33, 4, 1), (512, 8, 2), (4097, 128, 4), (1000, 1000, 8)])
def test_prepare_sel_matches_stable_sort(M, E, k):
    M = M - M % k
    sel = RNG(M).integers(0, E, size=M)
    s = O.prepare_sel(sel, E, k)
    ssel, perm = torch.sort(torch.from_numpy(sel), stable=True)
    assert np.array_equal(s.sel_sorted, ssel.numpy())
    assert np.array_equal(s.perm, perm.numpy())
    assert np.array_equal(s.in_index, perm.numpy() // k)
    assert np.array_equal(np.sort(s.perm), np.arange(M))
    assert np.array_equal(sel[s.perm], s.sel_sorted)
    assert s.offsets[0] == 0 and s.offsets[-1] == M
    for e in range(E):
        assert np.all(s.sel_sorted[s.offsets[e]:s.offsets[e + 1]] == e)


def test_prepare_sel_rejects_bad_ids():
    with pytest.raises(ValueError):
        O.prepare_sel(np.array([0, 4]), 4)


# ------------------------------------------------------------------ input stage
def test_kernel_inp_res_mapping():
    # moe_layer_aihwkit_lightning.py:451-456: both spellings of "8 bit" give 1/127
    assert O.kernel_inp_res(2 ** 8 - 2) == pytest.approx(1 / 127)
    assert O.kernel_inp_res(1 / (2 ** 8 - 2)) == pytest.approx(1 / 127)
    assert O.kernel_inp_res(-1) == -1 and O.kernel_inp_res(0) == -1


def test_dac_matches_torch_ops_and_codes_are_8bit():
    a = (RNG(1).standard_normal((257, 96)) * 2).astype(np.float32)
    ir = np.abs(RNG(2).standard_normal((257, 1))).astype(np.float32) + 0.3
    res = np.float32(1 / 127)
    v, codes = O.dac(a, ir, None, 1 / 127)
    ta, tir = torch.from_numpy(a), torch.from_numpy(ir)
    t = torch.clamp(ta, -tir, tir) / tir
    t = torch.round(t / float(res)) * float(res)
    assert np.array_equal(v, t.numpy())
    assert np.array_equal(codes, np.rint(codes)) and np.abs(codes).max() <= 127
    assert (np.abs(codes) == 127).any()             # some inputs clip at these ranges
    # quantising an already-quantised, in-range value is the identity
    v2, _ = O.dac(v * ir, ir, None, 1 / 127)
    assert np.allclose(v2, v, atol=1e-7)


def test_dac_ties_round_to_even():
    a = np.array([[0.5, 1.5, 2.5, -0.5, -1.5]], dtype=np.float32) / 127
    v, codes = O.dac(a * np.float32(127) / np.float32(127), None, None, 1 / 127)
    # 0.5/127/(1/127) is not exactly a tie in fp32, so check rint itself
    assert np.array_equal(np.rint(np.array([0.5, 1.5, 2.5, -0.5, -1.5], np.float32)), [0, 2, 2, -0, -2])
    assert np.array_equal(torch.round(torch.tensor([0.5, 1.5, 2.5])).numpy(), [0, 2, 2])


def test_dac_off_is_identity():
    a = RNG(3).standard_normal((5, 7)).astype(np.float32)
    v, codes = O.dac(a, None, None, -1)
    assert codes is None and np.array_equal(v, a)


# ------------------------------------------------------------------ forward
def _brute_fwd(x, W, idx, ir=None, res=-1.0):
    """per-token loop (test_moe_layer_aihwkit_lightning.py:71-80), torch ops only"""
    T, k = idx.shape
    out = torch.zeros(T, k, W.shape[2])
    for t in range(T):
        for h in range(k):
            e = int(idx[t, h])
            a = x[t]
            if ir is not None:
                a = torch.clamp(a, -ir[e], ir[e]) / ir[e]
            if res > 0:
                a = torch.round(a / res) * res
            c = a @ W[e]
            if ir is not None:
                c = c * ir[e]
            out[t, h] = c
    return out


def test_fwd_analog_off_is_per_expert_matmul():
    x, keys, _, idx, _ = _problem()
    s = O.prepare_sel(idx.numpy(), 4, 2)
    out = O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), out_index=s.perm)
    ref = _brute_fwd(x, keys, idx).reshape(-1, 64).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-5)


def test_fwd_clip_quant_matches_per_token_torch():
    x, keys, _, idx, _ = _problem(1)
    ir = torch.tensor([1.0, 2.0, 3.0, 0.5])
    s = O.prepare_sel(idx.numpy(), 4, 2)
    res = float(np.float32(1 / 127))
    out, codes = O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), 1 / 127,
                            ir.numpy()[s.sel_sorted], s.perm, return_codes=True)
    ref = _brute_fwd(x, keys, idx, ir, res).reshape(-1, 64).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=2e-5)
    assert np.abs(codes).max() == 127 and np.array_equal(codes, np.rint(codes))


def test_fwd_down_projection_layout_and_gate_reduce():
    x, keys, values, idx, gate = _problem(2)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    p = np.maximum(O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), out_index=s.perm), 0)
    z = O.cvmm_fwd(p, s.perm, s.sel_sorted, values.numpy())
    y = O.gate_reduce(z, gate.numpy())
    # per-token form: test_moe_layer_aihwkit_lightning.py:96-107
    ref = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for h in range(2):
            e = int(idx[t, h])
            ref[t] += gate[t, h] * (torch.relu(x[t] @ keys[e]) @ values[e])
    np.testing.assert_allclose(y, ref.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(y, torch.einsum("tk,tkd->td", gate, torch.from_numpy(z).view(-1, 2, 128)).numpy(),
                               rtol=1e-5, atol=1e-6)


def test_fwd_abs_max_is_scale_equivariant():
    x, keys, _, idx, _ = _problem(3)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    xn = x.numpy()
    amax = np.abs(xn).max(-1)
    f = lambda v, am: O.cvmm_fwd(v, s.in_index, s.sel_sorted, keys.numpy(), 1 / 127, None, s.perm, am)
    a = f(xn, amax)
    b = f(4 * xn, 4 * amax)                        # power of two: exact in fp32
    np.testing.assert_array_equal(4 * a, b)
    # and it stays within one quantisation step of the un-quantised product
    ref = _brute_fwd(x, keys, idx).reshape(-1, 64).numpy()
    assert np.abs(a - ref).max() < 0.05


def test_fwd_noise_is_added_before_rescale():
    x, keys, _, idx, _ = _problem(4)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    ir = np.array([1.0, 2.0, 3.0, 0.5], np.float32)[s.sel_sorted]
    noise = RNG(5).standard_normal((200, 64)).astype(np.float32) * 0.1
    args = (x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), 1 / 127, ir, s.perm, None)
    clean = O.cvmm_fwd(*args)
    noisy = O.cvmm_fwd(*args, noise)
    ir_by_out = np.empty(200, np.float32)
    ir_by_out[s.perm] = ir
    np.testing.assert_allclose(noisy - clean, noise * ir_by_out[:, None], rtol=0, atol=2e-6)


def test_fwd_within_expert_order_does_not_matter():
    x, keys, _, idx, _ = _problem(5)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    base = O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), 1 / 127, None, s.perm,
                      np.abs(x.numpy()).max(-1))
    perm2 = s.perm.copy()
    for e in range(4):
        seg = slice(s.offsets[e], s.offsets[e + 1])
        perm2[seg] = perm2[seg][::-1]
    other = O.cvmm_fwd(x.numpy(), perm2 // 2, s.sel_sorted, keys.numpy(), 1 / 127, None, perm2,
                       np.abs(x.numpy()).max(-1))
    np.testing.assert_array_equal(base, other)


# ------------------------------------------------------------------ build-defined extensions
def test_tile_bounds():
    assert list(O.tile_bounds(1024, 512)) == [0, 512, 1024]
    assert list(O.tile_bounds(412, 512)) == [0, 412]
    assert list(O.tile_bounds(412, -1)) == [0, 412]
    assert list(O.tile_bounds(10, 4)) == [0, 4, 7, 10]


def test_tile_split_sums_partials():
    x, keys, _, idx, _ = _problem(6)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    ir1 = np.full((200, 1), 100.0, np.float32)
    ir3 = np.full((200, 3), 100.0, np.float32)
    one = O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), -1, ir1, s.perm)
    three = O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), -1, ir3, s.perm,
                       bounds=O.tile_bounds(128, 48))
    np.testing.assert_allclose(one, three, rtol=1e-5, atol=1e-5)
    # with per-tile ranges each tile is its own clip/quantise problem
    ir_t = np.tile(np.array([[0.5, 1.0, 2.0]], np.float32), (200, 1))
    split = O.cvmm_fwd(x.numpy(), s.in_index, s.sel_sorted, keys.numpy(), 1 / 127, ir_t, s.perm,
                       bounds=[0, 43, 86, 128])
    acc = 0
    for t, (lo, hi) in enumerate([(0, 43), (43, 86), (86, 128)]):
        acc = acc + O.cvmm_fwd(x.numpy()[:, lo:hi], s.in_index, s.sel_sorted, keys.numpy()[:, lo:hi], 1 / 127,
                               ir_t[:, t], s.perm)
    np.testing.assert_allclose(split, acc, rtol=1e-6, atol=1e-6)


def test_adc_off_is_identity_and_on_gives_integer_codes():
    c = RNG(7).standard_normal((50, 16)).astype(np.float32) * 3
    wmax = np.full((1, 1), 0.25, np.float32)
    assert O.adc(c, wmax, -1, -1) is c
    q = O.adc(c, wmax, 12.0, 2 ** 8 - 2)
    step = np.float32(12.0 * 0.25 / 127)
    codes = q / step
    np.testing.assert_allclose(codes, np.rint(codes), atol=1e-3)
    assert np.abs(np.rint(codes)).max() <= 127
    assert np.abs(q - np.clip(c, -3, 3)).max() <= step / 2 + 1e-6
    clipped_only = O.adc(c * 10, wmax, 12.0, -1)
    assert np.abs(clipped_only).max() == pytest.approx(3.0)


def test_counter_noise_statistics_and_determinism():
    """The output-noise generator (32 x 32 blocks, each the product of two matrices of pseudo-random signed
    bytes): a pure function of its arguments, standard normal to the accuracy a sample of a million shows
    (moments, Kolmogorov distance), uncorrelated between neighbouring rows, columns, blocks, tiles and seeds, and
    squares only as dependent as the bilinear form makes them (0.012 between entries that share a row or a column of
    a block for ideal random bytes)."""
    from scipy import stats as st
    rows = np.arange(4096) * 7 + 3                       # output rows are scattered ids
    starts = 11 + (np.arange(4096) // 32) * 32           # 32-row blocks from the expert's first sorted position
    a = O.counter_noise(rows, starts, 256, 0, 1234)
    assert a.dtype == np.float32 and a.shape == (4096, 256)
    assert np.array_equal(a, O.counter_noise(rows, starts, 256, 0, 1234))
    assert np.array_equal(a[96:200], O.counter_noise(rows[96:200], starts[96:200], 256, 0, 1234))
    assert np.array_equal(a[:, :70], O.counter_noise(rows, starts, 70, 0, 1234))          # a ragged last block
    zi = O.counter_noise_int(rows[:64], starts[:64], 64, 0, 1234)
    assert np.array_equal(zi.astype(np.float32) * O.NOISE_SCALE, a[:64, :64])
    b = O.counter_noise(rows, starts, 256, 1, 1234)
    c = O.counter_noise(rows, starts, 256, 0, 1235)
    d = O.counter_noise(rows, starts + 32, 256, 0, 1234)   # the same output rows in other blocks
    assert abs(a.mean()) < 4e-3 and abs(a.std() - 1) < 4e-3
    kurt = ((a - a.mean()) ** 4).mean() / a.var() ** 2
    skew = ((a - a.mean()) ** 3).mean() / a.std() ** 3
    assert abs(kurt - 3) < 0.05 and abs(skew) < 0.01
    assert st.kstest(a.ravel()[::4], "norm").statistic < 5e-3
    assert np.abs(a).max() > 4.0                         # tails exist (a sum of 12 uniforms would stop at 6, IH4 at 3.5)
    for other in (b, c):
        assert abs(np.corrcoef(a.ravel(), other.ravel())[0, 1]) < 5e-3
    assert abs(np.corrcoef(a.ravel(), d.ravel())[0, 1]) < 2e-2
    for sh in (1, 2, 31, 32, 33):
        assert abs(np.corrcoef(a[:, :-sh].ravel(), a[:, sh:].ravel())[0, 1]) < 5e-3
        assert abs(np.corrcoef(a[:-sh].ravel(), a[sh:].ravel())[0, 1]) < 5e-3
    sq = a.astype(np.float64) ** 2
    assert abs(np.corrcoef(sq[:, :-1].ravel(), sq[:, 1:].ravel())[0, 1]) < 0.03
    assert abs(np.corrcoef(sq[:-1].ravel(), sq[1:].ravel())[0, 1]) < 0.03
    # the energy of a row over 256 columns scatters like that of 256 independent normals (0.088) -- not more than
    # a quarter above it, as it would if one draw scaled a whole row
    row_energy = sq.mean(1)
    assert row_energy.std() < 1.25 * np.sqrt(2 / 256)


def test_counter_noise_block_is_a_byte_matrix_product():
    """Brute force of one block from the definition: words -> signed bytes -> 32-term products."""
    def fmix(h):
        h &= 0xFFFFFFFF
        h ^= h >> 16; h = (h * 0x85EBCA6B) & 0xFFFFFFFF; h ^= h >> 13; h = (h * 0xC2B2AE35) & 0xFFFFFFFF; h ^= h >> 16
        return h

    def vec(key):
        out = []
        for j in range(8):
            k = key ^ (0x5BD1E995 if j >= 4 else 0)
            w = ((k & 0xFFFFFF) * (0x9E3779, 0x85EBCB, 0xC2B2AF, 0x27D4EB)[j % 4] + k) & 0xFFFFFFFF
            w ^= w >> 15
            for b in range(4):
                v = (w >> (8 * b)) & 0xFF
                out.append(v - 256 if v >= 128 else v)
        return out
    seed, tile = 0xABCDEF0123456789, 2
    ka = fmix((((seed & 0xFFFFFFFF) ^ 0x9E3779B9) + tile * 0x632BE5AB) & 0xFFFFFFFF)
    kb = fmix((((seed >> 32) ^ 0x85EBCA77) + tile * 0x27D4EB2F) & 0xFFFFFFFF)
    rows, start = [5, 900000, 17], 4096 + 64
    got = O.counter_noise_int(np.array(rows), np.full(3, start), 40, tile, seed)
    for i, r in enumerate(rows):
        for c in (0, 1, 31, 32, 39):
            a = vec(fmix(r ^ ka) ^ (((c // 32) * 0x632BE5AB) & 0xFFFFFFFF))
            b = vec(fmix(((c * 0x9E3779B1) & 0xFFFFFFFF) ^ kb) ^ ((start * 0x27D4EB2F) & 0xFFFFFFFF))
            assert got[i, c] == sum(x * y for x, y in zip(a, b)) - 8


# ------------------------------------------------------------------ backward
def _surrogate_layer(x, keys, values, idx, gate, ir):
    """Differentiable surrogate with the same straight-through semantics as CVMM.backward:
    clamp instead of clamp+quantise; per-token loop; autograd supplies every gradient."""
    T, k = idx.shape
    y = torch.zeros(T, values.shape[2])
    zs = torch.zeros(T, k, values.shape[2])
    for t in range(T):
        for h in range(k):
            e = int(idx[t, h])
            a = x[t] if ir is None else torch.clamp(x[t], -ir[0, e], ir[0, e])
            p = torch.relu(a @ keys[e])
            b = p if ir is None else torch.clamp(p, -ir[1, e], ir[1, e])
            z = b @ values[e]
            zs[t, h] = z
            y[t] = y[t] + gate[t, h] * z
    return y, zs


@pytest.mark.parametrize("use_ir", [False, True])
def test_backward_matches_autograd_of_surrogate(use_ir):
    x, keys, values, idx, gate = _problem(8, T=60)
    x.requires_grad_(); keys.requires_grad_(); values.requires_grad_(); gate = gate.detach().requires_grad_()
    ir = torch.tensor([[1.0, 2.0, 3.0, 4.0], [0.5, 1.0, 1.5, 2.0]]) if use_ir else None
    y, _ = _surrogate_layer(x, keys, values, idx, gate, ir)
    dy = torch.randn(y.shape, generator=torch.Generator().manual_seed(1))
    (y * dy).sum().backward()
    r = O.layer_fwd_bwd(x.detach().numpy(), keys.detach().numpy(), values.detach().numpy(), idx.numpy(),
                        gate.detach().numpy(), None if ir is None else ir.numpy()[:, :, None], dy.numpy(),
                        gradient_relative=False)
    np.testing.assert_allclose(r.y, y.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_values, values.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_keys, keys.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_x, x.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_gate, gate.grad.numpy(), rtol=1e-4, atol=1e-5)


def test_ir_grad_closed_form_and_special_cases():
    x, keys, values, idx, gate = _problem(9, T=40)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    g = RNG(1).standard_normal((80, 64)).astype(np.float32)
    irv = np.array([0.7, 1.0, 1.3, 1.6], np.float32)
    ir = irv[s.sel_sorted]
    b = O.cvmm_backward(g, x.numpy(), keys.numpy(), s.sel_sorted, s.in_index, s.perm, None, ir, None, k=2,
                        gradient_relative=True, gradient_scale=0.5)
    # brute force, element by element (cvmm.py:848-870)
    W = keys.numpy().astype(np.float64)
    want = np.zeros(80)
    for j in range(80):
        e, row, o = s.sel_sorted[j], s.in_index[j], s.perm[j]
        G = g[o].astype(np.float64) @ W[e].T
        acc = 0.0
        for n in range(128):
            xv = x[row, n].item()
            if xv >= irv[e]:
                acc += min(G[n], 0.0)
            if xv <= -irv[e]:
                acc -= max(G[n], 0.0)
        want[j] = acc * irv[e] * 0.5
    np.testing.assert_allclose(b.ir_grad[:, 0], want, rtol=1e-4, atol=1e-5)
    assert np.abs(want).max() > 0
    # nothing clips -> zero gradient; decay adds decay*ir when enough inputs are un-clipped
    big = np.full(80, 100.0, np.float32)
    b0 = O.cvmm_backward(g, x.numpy(), keys.numpy(), s.sel_sorted, s.in_index, s.perm, None, big, None, k=2)
    assert np.all(b0.ir_grad == 0)
    b1 = O.cvmm_backward(g, x.numpy(), keys.numpy(), s.sel_sorted, s.in_index, s.perm, None, big, None, k=2,
                         decay=0.01, input_min_percentage=0.95)
    np.testing.assert_allclose(b1.ir_grad[:, 0], 0.01 * big, rtol=1e-6)
    b2 = O.cvmm_backward(g, x.numpy(), keys.numpy(), s.sel_sorted, s.in_index, s.perm, None, ir, None, k=2,
                         decay=0.01, input_min_percentage=0.999, gradient_scale=0.5)
    np.testing.assert_array_equal(b2.ir_grad, b.ir_grad)   # too many inputs clip: no decay term


# ---- K-tile split in the backward: per-tile clip mask, per-tile input-range gradient (cvmm.py:848-881 per tile)
TILES_UP, TILES_DN = [0, 40, 90, 128], [0, 24, 64]          # uneven tiles of D = 128 and F = 64


def _surrogate_layer_tiled(x, keys, values, idx, gate, ir_up, ir_dn):
    """The surrogate above with the contraction cut into K-tiles: every tile clamps its slice of the input
    against its own range, multiplies its slice of the weights, and the tile results are added.  ir_up [E, 3],
    ir_dn [E, 2]; autograd supplies every gradient, including those of the ranges."""
    T, k = idx.shape
    y = torch.zeros(T, values.shape[2])
    for t in range(T):
        for h in range(k):
            e = int(idx[t, h])
            p = 0
            for j in range(len(TILES_UP) - 1):
                lo, hi = TILES_UP[j], TILES_UP[j + 1]
                r = ir_up[e, j]
                p = p + torch.minimum(torch.maximum(x[t, lo:hi], -r), r) @ keys[e, lo:hi]
            p = torch.relu(p)
            z = 0
            for j in range(len(TILES_DN) - 1):
                lo, hi = TILES_DN[j], TILES_DN[j + 1]
                r = ir_dn[e, j]
                z = z + torch.minimum(torch.maximum(p[lo:hi], -r), r) @ values[e, lo:hi]
            y[t] = y[t] + gate[t, h] * z
    return y


def test_tiled_backward_matches_autograd_of_tiled_surrogate():
    """Pins the multi-tile branch of cvmm_backward / cvmm_bwd_w: clip mask and clipped weight-gradient operand
    per K-tile on both projections, through grad_x, both weight gradients and the gate gradient.  (The
    input-range gradient of the reference is not the autograd gradient of a clamp -- it keeps one sign only,
    cvmm.py:863-865 -- so the brute force below pins it.)"""
    x, keys, values, idx, gate = _problem(12, T=50)
    x.requires_grad_(); keys.requires_grad_(); values.requires_grad_(); gate = gate.detach().requires_grad_()
    g = torch.Generator().manual_seed(5)
    ir_up = (torch.rand(4, 3, generator=g) * 1.5 + 0.4)
    ir_dn = (torch.rand(4, 2, generator=g) * 0.8 + 0.2)
    y = _surrogate_layer_tiled(x, keys, values, idx, gate, ir_up, ir_dn)
    dy = torch.randn(y.shape, generator=torch.Generator().manual_seed(1))
    (y * dy).sum().backward()
    ir = np.zeros((2, 4, 3), np.float32)
    ir[0] = ir_up.numpy()
    ir[1, :, :2] = ir_dn.numpy()
    r = O.layer_fwd_bwd(x.detach().numpy(), keys.detach().numpy(), values.detach().numpy(), idx.numpy(),
                        gate.detach().numpy(), ir, dy.numpy(), gradient_relative=False,
                        bounds_up=TILES_UP, bounds_down=TILES_DN)
    np.testing.assert_allclose(r.y, y.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_values, values.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_keys, keys.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_x, x.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r.grad_gate, gate.grad.numpy(), rtol=1e-4, atol=1e-5)
    # the masks did something on every tile of both projections
    xs = x.detach().numpy()
    for j in range(3):
        assert (np.abs(xs[:, TILES_UP[j]:TILES_UP[j + 1]]) >= ir_up.numpy()[:, j].min()).any()


@pytest.mark.parametrize("proj", ["up", "down"])
def test_tiled_ir_grad_brute_force(proj):
    """cvmm.py:848-870 per K-tile, element by element, on both call shapes of CVMM.backward: the
    up-projection (x [T, K] gathered by perm // k, no gate) and the down-projection (x [M, K] gathered by
    perm, gate-scaled gradient), three uneven tiles, relative scaling and the decay rule."""
    x, keys, values, idx, gate = _problem(13, T=40)
    E, k = 4, 2
    s = O.prepare_sel(idx.numpy(), E, k)
    rng = RNG(3)
    if proj == "up":
        W, xin, bounds = keys.numpy(), x.numpy(), TILES_UP
        g = rng.standard_normal((80, 64)).astype(np.float32)
        sel_index, out_index, gt, z = s.in_index, s.perm, None, None
    else:
        W, bounds = values.numpy(), [0, 10, 33, 64]
        xin = np.maximum(rng.standard_normal((80, 64)), 0).astype(np.float32)
        g = rng.standard_normal((40, 128)).astype(np.float32)
        sel_index, out_index, gt = s.perm, None, gate.numpy()
        z = rng.standard_normal((80, 128)).astype(np.float32)
    nt = len(bounds) - 1
    irv = rng.uniform(0.3, 1.4, size=(E, nt)).astype(np.float32)
    ir = irv[s.sel_sorted]
    kw = dict(k=k, gradient_relative=True, gradient_scale=0.25, bounds=bounds, relu_mask=(proj == "down"))
    b = O.cvmm_backward(g, xin, W, s.sel_sorted, sel_index, out_index, gt, ir, z, **kw)
    W64 = W.astype(np.float64)
    want = np.zeros((80, nt))
    want_full = np.zeros((80, W.shape[1]))
    n_not_clip = 0
    for j in range(80):
        e, row = int(s.sel_sorted[j]), int(sel_index[j])
        o = int(s.perm[j])                               # flat (token, head) position = output row
        grow = g[o // k] if proj == "down" else g[o]
        scale = float(gt.reshape(-1)[o]) if proj == "down" else 1.0
        G = np.float32(grow.astype(np.float64) @ W64[e].T).astype(np.float64)
        for t in range(nt):
            acc = 0.0
            for n in range(bounds[t], bounds[t + 1]):
                xv = float(xin[row, n])
                gs = float(np.float32(G[n] * scale))
                if xv >= irv[e, t]:
                    acc += min(gs, 0.0)
                if xv <= -irv[e, t]:
                    acc -= max(gs, 0.0)
                keep = abs(xv) < irv[e, t]
                n_not_clip += keep
                v = G[n] * keep
                if proj == "down":
                    v = v * (xv > 0)
                want_full[o if proj == "up" else row, n] = v * scale
            want[j, t] = acc * irv[e, t] * 0.25
    np.testing.assert_allclose(b.ir_grad, want, rtol=1e-4, atol=1e-5)
    assert (np.abs(want) > 0).any(axis=0).all()          # every tile contributes
    np.testing.assert_allclose(b.grad_x_full, want_full, rtol=1e-4, atol=1e-5)
    # decay: added per tile when the un-clipped share of ALL elements exceeds the threshold (cvmm.py:872-878)
    pct = n_not_clip / (80 * W.shape[1])
    lo_thr, hi_thr = pct - 0.01, pct + 0.01
    bd = O.cvmm_backward(g, xin, W, s.sel_sorted, sel_index, out_index, gt, ir, z, decay=0.02,
                         input_min_percentage=lo_thr, **kw)
    np.testing.assert_allclose(bd.ir_grad, want + 0.02 * ir, rtol=1e-4, atol=1e-5)
    bn = O.cvmm_backward(g, xin, W, s.sel_sorted, sel_index, out_index, gt, ir, z, decay=0.02,
                         input_min_percentage=hi_thr, **kw)
    np.testing.assert_array_equal(bn.ir_grad, b.ir_grad)


def test_bwd_w_empty_expert_is_zero_and_bf16_rounds():
    x, keys, _, idx, _ = _problem(10, T=30, E=4)
    idx = idx.clamp(max=2)                                   # expert 3 gets nothing
    s = O.prepare_sel(idx.numpy(), 4, 2)
    g = RNG(2).standard_normal((60, 64)).astype(np.float32)
    gw = O.cvmm_bwd_w(x.numpy(), s.in_index, s.sel_sorted, g, None, 4, s.perm)
    assert np.all(gw[3] == 0) and np.abs(gw[0]).max() > 0
    gb = O.cvmm_bwd_w(O.to_bf16(x.numpy()), s.in_index, s.sel_sorted, O.to_bf16(g), None, 4, s.perm, dtype="bf16")
    assert np.array_equal(gb, O.to_bf16(gb))
    np.testing.assert_allclose(gb, gw, rtol=3e-2, atol=1e-1)


def test_to_bf16_matches_torch():
    a = RNG(11).standard_normal(10000).astype(np.float32) * 100
    assert np.array_equal(O.to_bf16(a), torch.from_numpy(a).bfloat16().float().numpy())


# ------------------------------------------------------------------ std
def test_expert_std_matches_torch_std():
    x, _, _, idx, _ = _problem(12, E=4)
    idx = idx.clamp(max=2)
    s = O.prepare_sel(idx.numpy(), 4, 2)
    got = O.expert_std(x.numpy(), s.in_index, s.sel_sorted, 4)
    for e in range(3):
        rows = s.in_index[s.sel_sorted == e]
        assert got[e] == pytest.approx(torch.std(x[rows].flatten(), unbiased=True).item(), rel=1e-5)
    assert not (got[3] > 0)                                  # empty expert is filtered by `stds > 0`


# ------------------------------------------------------------------ second formulation
@pytest.mark.parametrize("quant", [False, True])
def test_per_expert_torch_layer_agrees_with_oracle(quant):
    from oracle.layer_cpu import moe_layer_per_expert
    x, keys, values, idx, gate = _problem(13, T=64, E=8, k=2)
    E = 8
    ir = torch.tensor(RNG(3).uniform(0.8, 2.5, size=(2, E, 1)).astype(np.float32))
    wu = keys.abs().amax((1, 2)).reshape(E, 1)
    wd = values.abs().amax((1, 2)).reshape(E, 1)
    nu = torch.randn(1, 128, 64, generator=torch.Generator().manual_seed(5)) * 0.04
    nd = torch.randn(1, 128, 128, generator=torch.Generator().manual_seed(6)) * 0.04
    nus = nu * wu[idx.reshape(-1)].reshape(1, -1, 1)
    nds = nd * wd[idx.reshape(-1)].reshape(1, -1, 1)
    res = 1 / 127 if quant else -1.0
    ob, orr = (12.0, 254.0) if quant else (-1.0, -1.0)
    xs = x.clone().requires_grad_(); ks = keys.clone().requires_grad_(); vs = values.clone().requires_grad_()
    gs = gate.clone().requires_grad_(); irs = ir.clone().requires_grad_()
    y = moe_layer_per_expert(xs, ks, vs, idx, gs, irs, inp_res=res, noise_up=nus, noise_down=nds,
                             wmax_up=wu, wmax_down=wd, out_bound=ob, out_res=orr, decay=0.01,
                             input_min_percentage=0.5)
    dy = torch.randn(y.shape, generator=torch.Generator().manual_seed(7))
    (y * dy).sum().backward()
    r = O.layer_fwd_bwd(x.numpy(), keys.numpy(), values.numpy(), idx.numpy(), gate.numpy(), ir.numpy(), dy.numpy(),
                        inp_res=res, noise_up=nus.numpy(), noise_down=nds.numpy(), wmax_up=wu.numpy(),
                        wmax_down=wd.numpy(), out_bound=ob, out_res=orr, decay=0.01, input_min_percentage=0.5)
    tol = dict(rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(r.y, y.detach().numpy(), **tol)
    np.testing.assert_allclose(r.grad_values, vs.grad.numpy(), **tol)
    np.testing.assert_allclose(r.grad_keys, ks.grad.numpy(), **tol)
    np.testing.assert_allclose(r.grad_x, xs.grad.numpy(), **tol)
    np.testing.assert_allclose(r.grad_gate, gs.grad.numpy(), **tol)
    np.testing.assert_allclose(r.grad_ir, irs.grad.numpy(), rtol=1e-3, atol=1e-3)


# ---------------------------------------------------------------------------------- weight modifier / clip
from oracle import weights_oracle as WO   # noqa: E402
from tests import util   # noqa: E402


def _torch_modify(w, kind, res, std_dev, z):
    """moe_layer_aihwkit_lightning.py:331-381 as tensor operations evaluated by torch on the CPU, with the
    quantiser written as round(w / res) * res."""
    if kind in WO.PER_CHANNEL_WMAX:
        wmax = w.abs().amax(1).unsqueeze(1)
    else:
        wmax = w.view(w.size(0), -1).abs().amax(-1).view(-1, 1, 1)
    if kind.startswith("DISCRETIZE"):
        n_states = max(res, 1 / res)
        step = wmax * torch.tensor(1.0, dtype=torch.float32).div(n_states).item()   # GPU kernels use the reciprocal
        w = torch.round(w / step) * step
    if "ADD_NORMAL" in kind:
        w = w + std_dev * wmax * z
    return w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", util.MODIFIER_KINDS)
def test_modify_weight_oracle_matches_torch_expression(kind, dtype):
    w = util.modifier_weights(1, 3, 30, 10, dtype)
    z = torch.randn(3, 30, 10, generator=torch.Generator().manual_seed(2)).to(dtype)
    want = _torch_modify(w, kind, 14.0, 0.07, z)
    got = WO.modify_weight(util.np32(w), kind, 14.0, 0.07, util.np32(z), "bf16" if dtype == torch.bfloat16 else "f32")
    assert np.array_equal(got, util.np32(want))


def test_modify_weight_oracle_wmax_follows_the_reference_type_list():
    """ADD_NORMAL_PER_CHANNEL is missing from the per-channel list (moe_layer_aihwkit_lightning.py:333-337): its
    noise is scaled by the per-expert maximum, so a quiet channel gets the noise of the loud one."""
    w = util.np32(util.modifier_weights(1, 2, 64, 6))
    z = np.ones_like(w)
    d = WO.modify_weight(w, "ADD_NORMAL_PER_CHANNEL", std_dev=0.1, z=z) - w
    np.testing.assert_allclose(d, np.broadcast_to(0.1 * np.abs(w).max(axis=(1, 2), keepdims=True), w.shape), rtol=1e-5)
    d = WO.modify_weight(w, "DISCRETIZE_ADD_NORMAL_PER_CHANNEL", res=1e6, std_dev=0.1, z=z) - w
    np.testing.assert_allclose(d, np.broadcast_to(0.1 * np.abs(w).max(axis=1, keepdims=True), w.shape), rtol=1e-3,
                               atol=1e-6)
    assert WO.modify_weight(w, "NONE") is not None and np.array_equal(WO.modify_weight(w, "NONE"), w)


@pytest.mark.parametrize("kind", ["DISCRETIZE", "DISCRETIZE_PER_CHANNEL"])
def test_discretize_oracle_is_a_uniform_quantiser(kind):
    """What any quantiser to n_states steps of max |W| must satisfy, whatever its rounding of ties."""
    w = util.np32(util.modifier_weights(4, 3, 50, 8))
    res = 2 ** 4 - 2
    q = WO.modify_weight(w, kind, res)
    wmax = WO.assumed_wmax(w, kind in WO.PER_CHANNEL_WMAX)
    step = wmax / res
    codes = q / step
    np.testing.assert_allclose(codes, np.rint(codes), atol=1e-4)            # multiples of the step
    assert np.abs(codes).max() <= res + 1e-4 and np.abs(codes).max() >= res - 1e-4   # max |W| is the last level
    assert (np.abs(q - w) <= step / 2 * (1 + 1e-5)).all()                      # nearest level
    assert np.array_equal(WO.modify_weight(q, kind, res, wmax=wmax), q)        # idempotent
    assert np.array_equal(WO.modify_weight(w, kind, 1 / res), q)               # res and 1 / res mean the same
    assert len(np.unique(np.rint(codes[0]))) <= 2 * res + 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["LAYER_GAUSSIAN", "LAYER_GAUSSIAN_PER_CHANNEL"])
def test_clip_oracle_matches_numpy_and_torch(kind, dtype):
    w = (util.modifier_weights(5, 3, 40, 12) + 0.3).to(dtype)
    pc = kind.endswith("PER_CHANNEL")
    std = WO.weight_std(util.np32(w), pc)
    np.testing.assert_allclose(std, util.np32(w).astype(np.float64).std(axis=1 if pc else (1, 2), ddof=1,
                                                                        keepdims=True), rtol=1e-6)
    np.testing.assert_allclose(std, util.np32(w.float().std(1 if pc else (1, 2), keepdim=True)), rtol=1e-5)
    # moe_layer_aihwkit_lightning.py:529-541 evaluated by torch
    bound = 2.0 * w.std(1 if pc else (1, 2), keepdim=True)
    want = torch.minimum(torch.maximum(w, -bound), bound)
    got = WO.clip_weights(util.np32(w), kind, 2.0, "bf16" if dtype == torch.bfloat16 else "f32")
    if dtype == torch.float32:
        np.testing.assert_allclose(got, util.np32(want), rtol=1e-6)           # std: fp64 here, fp32 in torch
        assert (got == util.np32(want)).mean() > 0.9
    else:
        assert np.array_equal(got, util.np32(want))
    assert np.array_equal(WO.clip_weights(util.np32(w), "NONE", 2.0), util.np32(w))
    with pytest.raises(ValueError):
        WO.clip_weights(util.np32(w), "FIXED_VALUE", 2.0)


def test_modifier_normals_are_standard_and_keyed():
    z = WO.modifier_normals(4, 64, 33, 99)
    assert z.shape == (4, 64, 33) and abs(z.mean()) < 0.03 and abs(z.std() - 1) < 0.03
    assert np.array_equal(z, WO.modifier_normals(4, 64, 33, 99)) and not np.array_equal(z, WO.modifier_normals(4, 64, 33, 100))
    assert not np.array_equal(z[:, :, :32].reshape(256, 32), O.box_muller_noise(np.arange(256), 32, 0, 99))


# ---------------------------------------------------------------------------------- router epilogue
from oracle import select_oracle as SO   # noqa: E402


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_select_oracle_matches_torch_sigmoid_topk(dtype):
    """tests/test_moe_layer_aihwkit_lightning.py:85-87 evaluated by torch on the CPU."""
    torch.manual_seed(0)
    logits = (torch.randn(200, 32) * 2).to(dtype)
    sel = torch.sigmoid(logits)
    want_val, want_idx = sel.topk(4, dim=-1, sorted=False)
    val, idx = SO.select(util.np32(logits), 4, "bf16" if dtype == torch.bfloat16 else "f32")
    # sorted=False leaves the order open and ties may go to another id: compare the values as sets per row, and
    # the values behind the oracle's ids
    ref = np.sort(util.np32(want_val), axis=-1)[:, ::-1]
    if dtype == torch.bfloat16:
        assert np.array_equal(val, ref)
        assert np.array_equal(np.take_along_axis(util.np32(sel), idx, -1), val)
    else:
        np.testing.assert_allclose(val, ref, rtol=2e-7)
    assert (np.diff(val, axis=-1) <= 0).all() and all(len(set(r)) == 4 for r in idx.tolist())
    tie = SO.select(np.zeros((1, 6), np.float32), 3)[1]
    assert tie.tolist() == [[0, 1, 2]]


def test_regulariser_and_select_bwd_match_torch_autograd():
    torch.manual_seed(1)
    logits = (torch.randn(50, 12) * 2).requires_grad_()
    logp = torch.log_softmax(logits, dim=-1)
    mean_logp = torch.logsumexp(logp, dim=0) - np.log(50)
    reg = (mean_logp.exp() * mean_logp).sum()
    val, idx = torch.sigmoid(logits).topk(3, dim=-1)
    gv = torch.randn(50, 3)
    ((val * gv).sum() + 0.7 * reg).backward()
    got_reg, c = SO.usage_regulariser(logits.detach().numpy())
    assert abs(float(got_reg) - float(reg.detach())) < 1e-6
    uniform_reg, _ = SO.usage_regulariser(np.zeros((7, 8), np.float32))
    assert abs(float(uniform_reg) + np.log(8)) < 1e-6                       # uniform usage: minus log E
    got = SO.select_bwd(logits.detach().numpy(), idx.numpy(), gv.numpy(), 0.7)
    np.testing.assert_allclose(got, logits.grad.numpy(), rtol=1e-4, atol=1e-7)
    only_reg = SO.select_bwd(logits.detach().numpy(), idx.numpy(), None, 1.0)
    np.testing.assert_allclose(only_reg.sum(axis=-1), 0.0, atol=1e-7)       # softmax gradients sum to zero per row


# ---------------------------------------------------------------------------------- golden fixtures
@pytest.mark.parametrize("name", ["config1_dac", "config1_dac_adc_split"])
def test_oracle_reproduces_golden_fixture(name):
    """The committed vectors (tests/golden/*.npz, written by tests/golden/make_golden.py) still come out of the
    oracle: a change to the oracle's arithmetic has to be deliberate."""
    from tests.golden import make_golden as G
    fx = np.load(os.path.join(os.path.dirname(G.__file__), name + ".npz"))
    pr, ir, lk, okw = G.problem(name)
    for n, t in pr.items():
        assert np.array_equal(fx["in_" + n], t.numpy()), n          # the generator still makes the same inputs
    want = util.layer_oracle({n: torch.from_numpy(fx["in_" + n]) for n in pr}, torch.from_numpy(fx["in_ir"]), "f32", **okw)
    for n in ("sel_sorted", "perm", "in_index", "offsets"):
        assert np.array_equal(getattr(want.sel, n), fx["out_" + n])
    for n in ("y", "scores", "z", "grad_x", "grad_keys", "grad_values", "grad_gate", "grad_ir"):
        # BLAS builds differ in summation order: one ADC step where a sum lands on a rounding boundary
        got, ref = getattr(want, n), fx["out_" + n]
        close = np.isclose(got, ref, rtol=1e-5, atol=1e-6 * np.abs(ref).max())
        assert close.mean() > 0.999, (n, close.mean())


def test_div_by_is_the_correctly_rounded_quotient(tmp_path):
    """The fp32 DAC stage's "codes match exactly" rests on amoe::div_by (csrc/common.h: a / b from one multiplication
    and two fused multiply-adds with y = 1 / b) being the IEEE quotient that torch's two divisions give
    (cvmm.py:154, 163).  The kernels' own source is compiled for the host and compared with `/`: every one of the
    2^23 dividend mantissas (both signs, three binades) against the 8-bit step 1/127 and three other divisors, and
    4 x 10^7 random pairs of the DAC's operand ranges including divisors with all-ones mantissas, divisors next to a
    power of two and the quantisation steps of 2 to 13 bits."""
    import ctypes
    import os
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    so = str(tmp_path / "libdivcheck.so")
    subprocess.run(["/opt/rocm/llvm/bin/clang++", "-x", "c++", "-std=c++20", "-O2", "-fPIC", "-shared",
                    "-ffp-contract=off", "-Wno-psabi", "-I", os.path.join(here, "emu"),
                    "-I", os.path.join(here, "..", "include"), "-I", os.path.join(here, "..", "analog_moe_amd", "csrc"),
                    os.path.join(here, "emu", "div_by_check.cpp"), "-o", so], check=True)
    lib = ctypes.CDLL(so)
    lib.div_by_mismatches_all_mantissas.restype = ctypes.c_longlong
    lib.div_by_mismatches_all_mantissas.argtypes = [ctypes.c_float]
    lib.div_by_mismatches_random.restype = ctypes.c_longlong
    lib.div_by_mismatches_random.argtypes = [ctypes.c_uint64, ctypes.c_longlong, ctypes.c_int]
    for b in (1.0 / 127.0, 2.0 / 254.0, 3.0, 1.4142135):
        assert lib.div_by_mismatches_all_mantissas(b) == 0, b
    for kind in range(4):
        assert lib.div_by_mismatches_random(kind + 1, 10_000_000, kind) == 0, kind
