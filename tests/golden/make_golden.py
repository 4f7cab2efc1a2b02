"""Writes the golden fixtures of this directory: inputs and the CPU oracle's outputs for one analog SigmaMoE layer,
forward and backward, in the shape of the reference's CPU-runnable test (d_model 128, top-2, fp32, input range 3.0,
8-bit inputs: tests/test_moe_layer_aihwkit_lightning.py:191-284), with 4 experts of size 32 and 64 tokens to keep
the files small; seed 0.

    python -m tests.golden.make_golden        (from the repository root)

The reference's own tests hold no vectors on disk, and nothing of the reference is imported or run here: the fixtures
freeze ``oracle.cvmm_oracle.layer_fwd_bwd`` as it was when they were written, so that a later change to the oracle or
to the kernels shows up against data instead of against a moving target.
"""
import os

import numpy as np
import torch

from oracle import cvmm_oracle as O
from tests import util

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    # name: keyword arguments of the layer (input range 3.0 on every expert, as the reference's tests set it)
    "config1_dac": dict(inp_res=1 / 127, decay=0.01, input_min_percentage=0.95),
    "config1_dac_adc_split": dict(inp_res=1 / 127, out_bound=12.0, out_res=254.0, bounds_up=[0, 64, 128],
                                  decay=0.0, input_min_percentage=0.5),
}
SHAPE = dict(T=64, D=128, E=4, F=32, k=2)


def problem(name):
    pr = util.make_problem(0, **SHAPE)
    lk = dict(CASES[name])
    nt = len(lk.get("bounds_up", [0, 1])) - 1
    ir = torch.full((2, SHAPE["E"], nt), 3.0)
    ir[0, :, 0] = torch.linspace(1.0, 3.0, SHAPE["E"])          # some experts clip N(0, 1) inputs, some do not
    okw = dict(lk)
    if lk.get("out_bound", -1) > 0:
        okw["wmax_up"] = pr["keys"].abs().amax((1, 2)).reshape(-1, 1).numpy()
        okw["wmax_down"] = pr["values"].abs().amax((1, 2)).reshape(-1, 1).numpy()
    return pr, ir, lk, okw


def main():
    for name in CASES:
        pr, ir, lk, okw = problem(name)
        want = util.layer_oracle(pr, ir, "f32", **okw)
        arrays = {"in_" + n: t.numpy() for n, t in pr.items()}
        arrays["in_ir"] = ir.numpy()
        for n in ("y", "scores", "z", "grad_x", "grad_keys", "grad_values", "grad_gate", "grad_ir"):
            arrays["out_" + n] = np.asarray(getattr(want, n), dtype=np.float32)
        for n in ("sel_sorted", "perm", "in_index", "offsets"):
            arrays["out_" + n] = getattr(want.sel, n)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrays)
        print(path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
