"""CPU oracle for the router's epilogue (sigmoid gate, top-k, usage regulariser).  TEST INFRASTRUCTURE ONLY.

The reference's layer inherits this step from ``sigma_moe.SigmaMoELayer``, which is not in the reference checkout;
what the checkout fixes is the per-token form in tests/test_moe_layer_aihwkit_lightning.py:82-90
(``sel = sigmoid(expert_sel(x)); sel_val, sel_idx = sel.topk(k, dim=-1, sorted=False)``).  ``select`` restates that
and is pinned against torch's ``sigmoid`` / ``topk`` on the CPU (tests/test_oracle.py); the order within a row
(descending, ties to the lower id) is this build's choice, ``sorted=False`` leaves it open.

PARITY UNPINNED: the regulariser.  ``usage_regulariser`` is minus the entropy of the mean expert usage,
``sum_e pbar_e log pbar_e`` with ``pbar = mean_t softmax(logits[t])`` -- this build's definition of the ``reg_loss``
the layer returns second (the reference only unpacks it, :260-262).  It and ``select_bwd`` are pinned against
torch's autograd of the same expression on the CPU.
"""
from __future__ import annotations

import numpy as np

from .cvmm_oracle import F32, _cast


def select(logits: np.ndarray, k: int, dtype: str = "f32"):
    """(sel_val [T, k], sel_idx [T, k]): the k largest sigmoid(logits) per row, in descending order, ties to the
    lower expert id; gate values rounded to ``dtype`` before they are compared, as a tensor of that type holds them."""
    x = _cast(logits, dtype)
    s = _cast(F32(1.0) / (F32(1.0) + np.exp(-x, dtype=F32)), dtype)
    order = np.argsort(-s, axis=-1, kind="stable")[:, :k]
    return np.take_along_axis(s, order, axis=-1), order.astype(np.int64)


def softmax_rows(logits: np.ndarray) -> np.ndarray:
    x = np.asarray(logits, dtype=np.float64)
    ex = np.exp(x - x.max(axis=-1, keepdims=True))
    return ex / ex.sum(axis=-1, keepdims=True)


def usage_regulariser(logits: np.ndarray):
    """(reg, c): reg = sum_e pbar_e log pbar_e;  c_e = d reg / d pbar_e = 1 + log pbar_e."""
    pbar = softmax_rows(logits).mean(axis=0)
    return F32((pbar * np.log(pbar)).sum()), (1.0 + np.log(pbar)).astype(F32)


def select_bwd(logits: np.ndarray, sel_idx: np.ndarray, grad_val, grad_reg, dtype: str = "f32") -> np.ndarray:
    """grad of (sum(sel_val * grad_val) + grad_reg * reg) with respect to the logits."""
    x = _cast(logits, dtype)
    T, E = x.shape
    g = np.zeros((T, E), dtype=np.float64)
    if grad_reg is not None:
        p = softmax_rows(x)
        _, c = usage_regulariser(x)
        g += float(grad_reg) / T * p * (c[None, :] - (p * c[None, :]).sum(axis=-1, keepdims=True))
    if grad_val is not None:
        s = _cast(F32(1.0) / (F32(1.0) + np.exp(-x, dtype=F32)), dtype).astype(np.float64)
        ds = s * (1.0 - s)
        rows = np.arange(T)[:, None]
        np.add.at(g, (rows, sel_idx), np.asarray(grad_val, dtype=np.float64) * ds[rows, sel_idx])
    return _cast(g.astype(F32), dtype)
