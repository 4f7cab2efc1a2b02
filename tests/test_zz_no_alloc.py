"""The allocation-free selection entry point (amoe_prepare_sel_noalloc) through the C ABI: bit-identical to
amoe_prepare_sel on two calls in a row, the second with a smaller input (the library's scratch array keeps the
first call's contents), and the size limit is enforced."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib, raw_mod, sel, E, k, noalloc):
    M = sel.numel()
    dev = sel.device
    out = [torch.full((M,), -7, dtype=torch.int32, device=dev) for _ in range(3)]
    offsets = torch.full((E + 1,), -7, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    if noalloc:
        rc = lib.amoe_prepare_sel_noalloc(sel.data_ptr(), int(sel.dtype == torch.int64), M, E, k, out[0].data_ptr(),
                                          out[1].data_ptr(), out[2].data_ptr(), offsets.data_ptr(), None, stream)
    else:
        ws = torch.empty(max(lib.amoe_prepare_sel_workspace(M, E), 4), dtype=torch.uint8, device=dev)
        rc = lib.amoe_prepare_sel(sel.data_ptr(), int(sel.dtype == torch.int64), M, E, k, out[0].data_ptr(),
                                  out[1].data_ptr(), out[2].data_ptr(), offsets.data_ptr(), None, ws.data_ptr(),
                                  ws.numel(), stream)
    assert rc == 0, lib.amoe_strerror(rc)
    torch.cuda.synchronize()
    return out + [offsets]


def test_prepare_sel_noalloc_matches_prepare_sel():
    from analog_moe_amd import ops, raw
    from oracle import cvmm_oracle as O
    lib = ops.get_lib()
    assert lib.amoe_noalloc_scratch_bytes() == 2 << 20
    rng = np.random.default_rng(5)
    # two calls in a row on the same GPU; the second is smaller and has fewer experts
    for M, E, k, dt in [(131072, 64, 8, torch.int64), (3000, 16, 4, torch.int32), (0, 4, 1, torch.int64),
                        (32768 * 4, 128, 4, torch.int64), (513, 5, 1, torch.int32)]:
        print("noalloc prepare_sel", M, E, k, dt, flush=True)
        sel_np = rng.integers(0, E, size=M)
        sel = torch.from_numpy(sel_np).to(dt).cuda()
        got = _run(lib, raw, sel, E, k, noalloc=True)
        want = _run(lib, raw, sel, E, k, noalloc=False)
        for g, w in zip(got, want):
            assert torch.equal(g, w)
        o = O.prepare_sel(sel_np, E, k)
        for g, w in zip(got, (o.sel_sorted, o.perm, o.in_index, o.offsets)):
            assert np.array_equal(g.cpu().numpy(), w)
    # beyond the library's array: rejected on the host, nothing launched
    M, E = 1 << 20, 2048
    assert lib.amoe_prepare_sel_workspace(M, E) > lib.amoe_noalloc_scratch_bytes()
    sel = torch.zeros(M, dtype=torch.int32, device="cuda")
    buf = torch.empty(M, dtype=torch.int32, device="cuda")
    off = torch.empty(E + 1, dtype=torch.int32, device="cuda")
    rc = lib.amoe_prepare_sel_noalloc(sel.data_ptr(), 0, M, E, 1, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(),
                                      off.data_ptr(), None, torch.cuda.current_stream().cuda_stream)
    assert rc == -5 and b"scratch" in lib.amoe_strerror(rc)
