"""SigmaMoE feed-forward layer (digital base) and its analog, hardware-aware version.

``AnalogSigmaMoELayer`` keeps the constructor, the ``rpu_config`` API, the overridable hooks
``compute_scores`` / ``cvmm_wrapper`` and the state-dict keys of the reference's
``AnalogSigmaMoELayerAIHWKITLightning`` (analog_moe/moe_layer_aihwkit_lightning.py:134-570).
Its base class there comes from the third-party ``sigma_moe`` package; ``SigmaMoELayer`` here
restates the part of that contract the reference relies on (constructor keywords
:261-276, attributes :220-233, forward = router -> top-k -> selection record ->
compute_scores -> down-projection with gate reduction, as in the per-token form of
test_moe_layer_aihwkit_lightning.py:82-107).

Differences from the reference, all opt-in through ``rpu_config``: ``mapping.max_input_size``
(K-tile split with one input range per tile), ``forward.out_bound`` / ``out_res`` (ADC) are
implemented instead of asserted off (:152-160); output noise is drawn inside the kernel unless
``noise_mode="injected"`` is chosen.  The router is an analog linear layer on the same kernels
(``AnalogLinear``; ``analog_router=False`` keeps a digital ``nn.Linear``).
"""
from __future__ import annotations

import contextlib
import math
from functools import partial
from typing import Callable, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from .config import (AIHWKITTorchInferenceRPUConfig, TorchInferenceRPUConfig, enum_name, kernel_inp_res)
from .cvmm import CVMM, AnalogExt, CVMMSel, cvmm_prepare_sel2, cvmm_std
from . import library  # noqa: F401  (registers the amoe:: operators)
from . import ops
from .ffn import FFNConfig, _side_stream, moe_ffn


class MoEConifgError(Exception):
    """Exceptions related to MoE configuration (name as in the reference)."""


class _PerfectIO:
    """io_params of a digital call: no abs-max scaling (cvmm.py:735-739)."""
    is_perfect = True
    noise_management = "NONE"


def tile_bounds(K: int, max_input_size: int):
    """Near-equal K-tiles of at most ``max_input_size`` features; None for a single tile."""
    if max_input_size is None or max_input_size <= 0 or max_input_size >= K:
        return None
    n = -(-K // max_input_size)
    base, rem = divmod(K, n)
    b = [0]
    for i in range(n):
        b.append(b[-1] + base + (1 if i < rem else 0))
    return b


class SigmaMoELayer(nn.Module):
    def __init__(self, d_model: int, n_experts: int, expert_size: int, k: int, dropout: float = 0.0,
                 selection_mode: str = "sigmoid", activation_after_topk: bool = False,
                 activation: Callable = F.relu, bias: bool = False, v_dim: Optional[int] = None,
                 sinkhorn_n_iters: int = 3, expert_dropout: float = 0.0, traceable: bool = False):
        super().__init__()
        if traceable:
            raise MoEConifgError("traceable=True (per-expert module lists on the CPU) is not part of this "
                                 "GPU-only package")
        if selection_mode not in ("sigmoid", "softmax"):
            raise MoEConifgError(f"selection_mode {selection_mode!r} is not implemented")
        self.k_dim = d_model
        self.v_dim = v_dim if v_dim is not None else d_model
        self.n_experts = n_experts
        self.expert_size = expert_size
        self.size = n_experts * expert_size
        self.dropout = dropout
        self.selection_mode = selection_mode
        self.activation_after_topk = activation_after_topk
        self.activation = activation
        self.n_heads = k
        self.sinkhorn_n_iters = sinkhorn_n_iters
        self.expert_dropout = expert_dropout
        self.traceable = traceable
        self.keys = nn.Parameter(torch.empty(n_experts, self.k_dim, expert_size))
        self.values = nn.Parameter(torch.empty(n_experts, expert_size, self.v_dim))
        self.expert_sel = nn.Linear(self.k_dim, n_experts, bias=False)
        if bias:
            self.bias = nn.Parameter(torch.zeros(n_experts, expert_size))
            self.o_bias = nn.Parameter(torch.zeros(self.v_dim))
        else:
            self.bias = None
            self.o_bias = None
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.keys, std=1.0 / math.sqrt(self.k_dim))
        nn.init.normal_(self.values, std=1.0 / math.sqrt(self.expert_size))
        nn.init.normal_(self.expert_sel.weight, std=1.0 / math.sqrt(self.k_dim))

    # -- hooks the analog layer overrides ------------------------------------------------------
    def cvmm_wrapper(self, inputs: Tensor, sel_indices: CVMMSel, weights: Tensor) -> Tensor:
        return CVMM.apply(inputs, sel_indices.sel_index, sel_indices.sel, weights, -1.0, None,
                          sel_indices.out_index, sel_indices.reduction_weight, None, None, _PerfectIO(),
                          AnalogExt(offsets=sel_indices.offsets))

    def compute_scores(self, inp: Tensor, index: CVMMSel, expert_scores: Optional[Tensor] = None) -> Tensor:
        scores = self.cvmm_wrapper(inp, index, self.keys)
        if self.bias is not None:
            scores = scores + self.bias[index.raw_sel]
        scores = self.activation(scores)
        if expert_scores is not None:
            scores = scores * expert_scores[..., None]
        if self.dropout > 0:
            scores = F.dropout(scores, self.dropout, training=self.training)
        return scores

    # -- router ------------------------------------------------------------------------------------
    def select(self, x: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
        """Gate values and expert ids [..., k] of the top-k experts, and the regularisation loss."""
        logits = self.expert_sel(x)
        if self._fused_select(logits):
            # sigmoid, top-k and the regulariser in one pass over the logits (and one for their gradient)
            val, idx, reg, _ = torch.ops.amoe.select(logits.reshape(-1, self.n_experts), self.n_heads, self.training)
            lead = logits.shape[:-1]
            return (val.view(*lead, self.n_heads), idx.view(*lead, self.n_heads),
                    reg if self.training else x.new_zeros(()))
        reg_loss = x.new_zeros(())
        if self.training and logits.numel() > 0:
            logp = F.log_softmax(logits.float(), dim=-1).flatten(end_dim=-2)
            mean_logp = torch.logsumexp(logp, dim=0) - math.log(logp.shape[0])
            reg_loss = (mean_logp.exp() * mean_logp).sum()          # minus entropy of the mean usage
        sel = logits if self.activation_after_topk else self._sel_activation(logits)
        if self.training and self.expert_dropout > 0:
            mask = torch.rand_like(sel) < self.expert_dropout
            sel = sel.masked_fill(mask, float("-inf"))
        sel_val, sel_idx = sel.topk(self.n_heads, dim=-1, sorted=False)
        if self.activation_after_topk:
            sel_val = self._sel_activation(sel_val)
        return sel_val, sel_idx, reg_loss

    def _fused_select(self, logits: Tensor) -> bool:
        """The plain router (sigmoid before top-k, no expert dropout) on the GPU takes the fused kernels."""
        return ((logits.is_cuda or logits.is_meta) and self.selection_mode == "sigmoid"
                and not self.activation_after_topk and not (self.training and self.expert_dropout > 0)
                and self.n_heads <= self.n_experts <= ops.SELECT_MAX_EXPERTS and logits.numel() > 0
                and logits.dtype in (torch.float32, torch.bfloat16, torch.float16))

    def _sel_activation(self, t: Tensor) -> Tensor:
        return torch.sigmoid(t) if self.selection_mode == "sigmoid" else F.softmax(t, dim=-1)

    def forward_selected(self, x: Tensor, sel_val: Tensor, sel_idx: Tensor) -> Tensor:
        """Expert feed-forward for a given routing decision (what follows the router in forward)."""
        if not (x.is_cuda or x.is_meta):
            raise MoEConifgError("MoE layer executed on CPU: this package runs on the GPU only "
                                 "(moe_layer_aihwkit_lightning.py:395-400 raises the same way)")
        sel_indices = cvmm_prepare_sel2(sel_idx, self.n_experts)
        scores = self.compute_scores(x, sel_indices)
        down = sel_indices.clone()
        down.reduction_weight = sel_val
        down.sel_index = sel_indices.out_index
        down.out_index = None
        out = self.cvmm_wrapper(scores, down, self.values)
        if self.o_bias is not None:
            out = out + self.o_bias
        return out

    def forward(self, x: Tensor) -> Tuple[Tensor, Tensor]:
        sel_val, sel_idx, reg_loss = self.select(x)
        return self.forward_selected(x, sel_val, sel_idx), reg_loss


class AnalogLinear(nn.Module):
    """An analog linear layer ``y = A(x) @ weight.T`` on the CVMM kernels: one analog tile per K-tile, which the
    kernels see as a one-expert selection (every row belongs to expert 0, in order).

    The reference turns the router ``expert_sel`` into an analog layer with aihwkit-lightning's
    ``convert_to_analog`` (moe_layer_aihwkit_lightning.py:195-200), so the expert selection itself sees the
    input range, the DAC, the output noise and the ADC.  That package is third-party; this class applies the
    same stages with the definitions of this build (they are the expert projections' own): parameters
    ``weight [out, in]`` as in ``nn.Linear`` (no bias), ``input_range [n_tiles]``, ``input_range_update_idx``.
    """

    def __init__(self, in_features: int, out_features: int, rpu_config, noise_mode: str = "kernel"):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.rpu_config = rpu_config
        self.noise_mode = noise_mode
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        self.register_parameter("bias", None)
        self.bounds = tile_bounds(in_features, getattr(rpu_config.mapping, "max_input_size", -1))
        self.n_tiles = 1 if self.bounds is None else len(self.bounds) - 1
        self.input_range = None
        irp = rpu_config.pre_post.input_range
        if irp.enable:
            self.input_range_update_idx = nn.Parameter(torch.tensor(0.0), requires_grad=False)
            ir = torch.full((self.n_tiles,), float(irp.init_value))
            if irp.learn_input_range:
                self.input_range = nn.Parameter(ir)
            else:
                del self.input_range
                self.register_buffer("input_range", ir)
        self._init_done = False
        self._noise_calls = 0
        self._noise_seed_base = 0
        self.noise_counter: Optional[Tensor] = None
        self._rows = {}                           # one-expert selection per row count

    def _selection(self, T: int, device) -> CVMMSel:
        def make():
            i32 = dict(dtype=torch.int32, device=device)
            zeros = torch.zeros(T, **i32)
            return CVMMSel(zeros, zeros, torch.arange(T, **i32), None, None, torch.arange(2, **i32) * T)
        if torch.compiler.is_compiling():
            return make()
        key = (T, str(device))
        if key not in self._rows:
            self._rows[key] = make()
        return self._rows[key]

    def _init_pending(self) -> bool:
        n = self.rpu_config.pre_post.input_range.init_from_data
        if n <= 0 or self._init_done:
            return False
        if not bool(self.input_range_update_idx < n):
            self._init_done = True
            return False
        return True

    def _seed(self) -> int:
        salt = 0x5851F42D4C957F2D                  # a seed stream of its own, apart from the expert projections'
        if self.noise_counter is not None:
            return (self._noise_seed_base ^ salt) & (2 ** 63 - 1)
        if torch.compiler.is_compiling():
            raise MoEConifgError("a compiled noisy forward would freeze the host-side noise seed: call "
                                 "use_device_noise_counter() on the layer before torch.compile")
        self._noise_calls += 1
        return ((torch.initial_seed() * 0x9E3779B97F4A7C15 + self._noise_calls * 0xD1B54A32D192ED03) ^ salt) \
            & (2 ** 63 - 1)

    def forward(self, x: Tensor) -> Tensor:
        if not (x.is_cuda or x.is_meta):
            raise MoEConifgError("Analog MoE executed on CPU. This package runs on the GPU only.")
        fwd = self.rpu_config.forward
        irp = self.rpu_config.pre_post.input_range
        x2 = x.reshape(-1, self.in_features)
        sel = self._selection(x2.shape[0], x.device)
        perfect = bool(getattr(fwd, "is_perfect", False))
        bir = None
        if self.input_range is not None:
            if self.training and self._init_pending():
                std = cvmm_std(x2, sel.sel_index, sel.sel, 1).float()
                if bool(std[0] > 0):
                    idx = self.input_range_update_idx
                    self.input_range.data = ((self.input_range.data * idx + irp.init_std_alpha * std[0]) / (idx + 1)
                                             ).abs().to(self.input_range.dtype)
                    self.input_range_update_idx.data += 1
            bir = self.input_range.reshape(1, self.n_tiles).expand(x2.shape[0], self.n_tiles)
        w = self.weight.t().unsqueeze(0)                               # [1, in, out]: a transposed view
        modified = w
        drew = False                                   # a launch of this forward read the device seed word
        if (self.training or self.rpu_config.modifier.enable_during_test) and \
                enum_name(self.rpu_config.modifier.type) not in ("NONE", "COPY"):
            modified = AnalogSigmaMoELayer.modify_weight(
                w, self.rpu_config.modifier, injected=self.noise_mode == "injected", seed_dev=self.noise_counter,
                seed=None if self.noise_mode == "injected" else self._seed() ^ _MODIFIER_ROUTER_SEED)
            drew = self.noise_mode != "injected"
        ext = AnalogExt(offsets=sel.offsets, bounds=self.bounds,
                        out_bound=-1.0 if perfect else float(getattr(fwd, "out_bound", -1)),
                        out_res=-1.0 if perfect else float(getattr(fwd, "out_res", -1)))
        per_channel = bool(getattr(fwd, "out_noise_per_channel", False))
        noisy = self.training and fwd.out_noise > 0 and not perfect
        if ext.out_bound > 0 or noisy:
            ext.wmax = torch.ops.amoe.weight_abs_max(w.detach().contiguous(), per_channel)
        out_noise = None
        if noisy and self.noise_mode == "kernel":
            ext.noise_std, ext.noise_seed, ext.noise_seed_dev = float(fwd.out_noise), self._seed(), self.noise_counter
        elif noisy:
            out_noise = torch.randn(self.n_tiles, x2.shape[0], self.out_features, device=x.device) \
                * fwd.out_noise * ext.wmax[0]
        y = CVMM.apply(x2, sel.sel_index, sel.sel, modified, -1.0 if perfect else kernel_inp_res(fwd.inp_res), bir,
                       None, None, out_noise, irp, fwd, ext)
        if self.noise_counter is not None and (drew or ext.noise_seed_dev is not None):
            self.noise_counter.add_(1)                 # the next forward (or graph replay) draws anew
        return y.view(*x.shape[:-1], self.out_features)

    @torch.no_grad()
    def clip_weights(self) -> None:
        kind = enum_name(self.rpu_config.clip.type)
        out, inp = self.weight.shape
        if kind == "LAYER_GAUSSIAN":                  # one bound for the whole matrix
            _gaussian_clip_(self.weight.data.view(1, out, inp), self.rpu_config.clip.sigma, False)
        elif kind == "LAYER_GAUSSIAN_PER_CHANNEL":    # one per output channel = per row of weight [out, in]
            _gaussian_clip_(self.weight.data.view(out, inp, 1), self.rpu_config.clip.sigma, False)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, tiles={self.n_tiles}"


_LIGHTNING_MODIFIERS = ("DISCRETIZE", "DISCRETIZE_PER_CHANNEL", "ADD_NORMAL", "ADD_NORMAL_PER_CHANNEL",
                        "DISCRETIZE_ADD_NORMAL", "DISCRETIZE_ADD_NORMAL_PER_CHANNEL")
_MODIFIER_DOWN_SEED = 0x5851F42D4C957F2D     # keep the draws for the weight tensors of a layer apart
_MODIFIER_ROUTER_SEED = 0x2545F4914F6CDD1D
_STATIC_MODIFIER_CALLS = [0]


def _need_device(w: Tensor, what: str) -> None:
    if not (w.is_cuda or w.is_meta):
        raise MoEConifgError(f"{what} on CPU tensors. This package runs on the GPU only.")


def _modify_on_device(w: Tensor, per_channel: bool, n_states: float, std_dev: float, round_noise: bool,
                      seed: Optional[int], seed_dev: Optional[Tensor], injected: bool) -> Tensor:
    """One pass of the weight-modifier kernel over w [E, K, N] (``amoe::modify_weight``)."""
    _need_device(w, "Weight modifier")
    noise = None
    if std_dev > 0 and injected:
        with torch.no_grad():
            noise = torch.randn_like(w) if round_noise else torch.randn(w.shape, device=w.device)
    elif std_dev > 0 and seed is None:
        # a call without a layer behind it (the reference's static method): torch's seed and a call count
        _STATIC_MODIFIER_CALLS[0] += 1
        seed = (torch.initial_seed() * 0x9E3779B97F4A7C15 + _STATIC_MODIFIER_CALLS[0] * 0xD1B54A32D192ED03) & (2 ** 63 - 1)
    return torch.ops.amoe.modify_weight(w, per_channel, n_states, std_dev, noise, round_noise, int(seed or 0),
                                        seed_dev if std_dev > 0 and noise is None else None)


def _gaussian_clip_(w: Tensor, sigma: float, per_channel: bool, max_bound: float = -1.0) -> None:
    """w = clamp(w, +-sigma * std) in place, std per expert or per channel, rounded as ``sigma * w.std(...)``
    rounds (moe_layer_aihwkit_lightning.py:529-541); max_bound > 0 caps the bound (moe_layer_aihwkit.py:332-333)."""
    _need_device(w, "Weight clipping")
    if w.is_meta:
        return
    bound = sigma * ops.weight_std(w, per_channel).to(w.dtype)
    if max_bound > 0:
        bound = bound.clamp(max=max_bound)
    ops.clamp_weights_(w, bound)


def non_traceable_to_traceable(state_dict, prefix: str = "") -> None:
    """In place: ``input_range [2, E]`` and its counter become the per-expert entries of the reference's
    traceable layout -- ``keys.{i}.input_range``, ``.input_range_update_idx``, ``.x_min``, ``.x_max`` and the same
    under ``values.{i}`` (moe_layer_aihwkit_lightning.py:33-63).  Input ranges of a K-tile split layer
    ([2, E, n_tiles]) have no counterpart in that layout and are refused."""
    input_range = state_dict[prefix + "input_range"]
    update_idx = state_dict[prefix + "input_range_update_idx"]
    if input_range.dim() != 2:
        raise MoEConifgError("the traceable layout holds one input range per expert and projection")
    for i in range(input_range.size(1)):
        for row, name in enumerate(("keys", "values")):
            state_dict[prefix + f"{name}.{i}.input_range"] = input_range[row, i].view(1)
            state_dict[prefix + f"{name}.{i}.input_range_update_idx"] = update_idx.view(1)
            state_dict[prefix + f"{name}.{i}.x_min"] = torch.zeros(1, device=input_range.device, dtype=input_range.dtype)
            state_dict[prefix + f"{name}.{i}.x_max"] = torch.zeros(1, device=input_range.device, dtype=input_range.dtype)
    state_dict.pop(prefix + "input_range")
    state_dict.pop(prefix + "input_range_update_idx")


def traceable_to_non_traceable(state_dict, prefix: str = "") -> None:
    """In place, the inverse (moe_layer_aihwkit_lightning.py:66-105): per-expert entries, in expert order, are
    stacked into ``input_range [2, E]``; the counter is taken from the first entry; ``x_min`` / ``x_max`` go."""
    import re
    pat = re.compile(rf"^{re.escape(prefix)}(keys|values)\.(\d+)\.(input_range|input_range_update_idx|x_min|x_max)$")
    found, idx, drop = {}, None, []
    for key in list(state_dict):
        m = pat.match(key)
        if not m:
            continue
        drop.append(key)
        if m.group(3) == "input_range":
            found[(m.group(1), int(m.group(2)))] = state_dict[key]
        elif m.group(3) == "input_range_update_idx" and idx is None:
            idx = state_dict[key]
    if not found:
        return
    n = 1 + max(i for _, i in found)
    state_dict[prefix + "input_range"] = torch.stack([
        torch.cat([found[("keys", i)].reshape(1) for i in range(n)]),
        torch.cat([found[("values", i)].reshape(1) for i in range(n)])])
    if idx is not None:
        state_dict[prefix + "input_range_update_idx"] = idx.reshape(())
    for key in drop:
        state_dict.pop(key)


def load_state_dict_pre_hook(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
    """Accept checkpoints written in the traceable layout (moe_layer_aihwkit_lightning.py:108-131; this package
    has the non-traceable layer only, so that is the one direction a load can need)."""
    if prefix + "input_range" not in state_dict:
        traceable_to_non_traceable(state_dict, prefix)


class AnalogSigmaMoELayer(SigmaMoELayer):
    """Analog SigmaMoE layer; ``rpu_config`` first, then the digital layer's keywords
    (moe_layer_aihwkit_lightning.py:135-138).  ``noise_mode``: "kernel" draws the output noise in
    the GEMM epilogue from a counter-based generator; "injected" materialises ``randn`` tensors as
    the reference does (:472-492) and hands them to the kernel."""

    def __init__(self, rpu_config: Optional[TorchInferenceRPUConfig] = None, *args, noise_mode: str = "kernel",
                 analog_router: bool = True, **kwargs):
        super().__init__(*args, **kwargs)
        self.rpu_config = TorchInferenceRPUConfig() if rpu_config is None else rpu_config
        if noise_mode not in ("kernel", "injected"):
            raise MoEConifgError("noise_mode must be 'kernel' or 'injected'")
        self.noise_mode = noise_mode
        if analog_router:                  # moe_layer_aihwkit_lightning.py:195-200: the router is analog too
            digital = self.expert_sel
            self.expert_sel = AnalogLinear(self.k_dim, self.n_experts, self.rpu_config, noise_mode)
            self.expert_sel.weight.data = digital.weight.data.clone()
        self._noise_calls = 0
        self._noise_seed_base = 0
        self._init_done = False            # host-side latch of "input_range_update_idx reached init_from_data"
        self.noise_counter: Optional[Tensor] = None     # see use_device_noise_counter()
        self._register_load_state_dict_pre_hook(load_state_dict_pre_hook)
        mis = getattr(self.rpu_config.mapping, "max_input_size", -1)
        self.bounds_up = tile_bounds(self.k_dim, mis)
        self.bounds_down = tile_bounds(self.expert_size, mis)
        self.n_tiles = max(1 if self.bounds_up is None else len(self.bounds_up) - 1,
                           1 if self.bounds_down is None else len(self.bounds_down) - 1)
        self.input_range = None
        ir_params = self.rpu_config.pre_post.input_range
        if ir_params.enable:
            self.input_range_update_idx = nn.Parameter(torch.tensor(0.0), requires_grad=False)
            shape = (2, self.n_experts) if self.n_tiles == 1 else (2, self.n_experts, self.n_tiles)
            ir = torch.full(shape, float(ir_params.init_value))
            if ir_params.learn_input_range:
                self.input_range = nn.Parameter(ir)
            else:
                del self.input_range
                self.register_buffer("input_range", ir)

    # -- conversion ---------------------------------------------------------------------------------
    @classmethod
    def from_digital(cls, module: SigmaMoELayer, rpu_config: TorchInferenceRPUConfig) -> "AnalogSigmaMoELayer":
        layer = cls(rpu_config=rpu_config, d_model=module.k_dim, n_experts=module.n_experts,
                    expert_size=module.expert_size, k=module.n_heads, dropout=module.dropout,
                    selection_mode=module.selection_mode, activation_after_topk=module.activation_after_topk,
                    activation=module.activation, bias=module.bias is not None, v_dim=module.v_dim,
                    sinkhorn_n_iters=module.sinkhorn_n_iters, expert_dropout=module.expert_dropout,
                    traceable=module.traceable)
        layer.set_weights(module.expert_sel, module.keys, module.values, module.bias, module.o_bias)
        return layer.to(device=module.keys.device, dtype=module.keys.dtype)

    @classmethod
    def to_digital(cls, module: "AnalogSigmaMoELayer") -> SigmaMoELayer:
        layer = SigmaMoELayer(d_model=module.k_dim, n_experts=module.n_experts, expert_size=module.expert_size,
                              k=module.n_heads, dropout=module.dropout, selection_mode=module.selection_mode,
                              activation_after_topk=module.activation_after_topk, activation=module.activation,
                              bias=module.bias is not None, v_dim=module.v_dim,
                              sinkhorn_n_iters=module.sinkhorn_n_iters, expert_dropout=module.expert_dropout)
        layer.keys.data = module.keys.data.detach().clone()
        layer.values.data = module.values.data.detach().clone()
        layer.expert_sel.weight.data = module.expert_sel.weight.data.detach().clone()
        if module.bias is not None:
            layer.bias.data = module.bias.data.detach().clone()
            layer.o_bias.data = module.o_bias.data.detach().clone()
        return layer.to(device=module.keys.device, dtype=module.values.dtype)

    def set_weights(self, expert_sel: nn.Linear, keys: Tensor, values: Tensor, bias: Optional[Tensor] = None,
                    o_bias: Optional[Tensor] = None) -> None:
        self.expert_sel.weight.data = expert_sel.weight.detach().clone()
        if expert_sel.bias is not None and self.expert_sel.bias is not None:
            self.expert_sel.bias.data = expert_sel.bias.detach().clone()
        self.keys.data = keys.detach().clone()
        self.values.data = values.detach().clone()
        if bias is not None and self.bias is not None:
            self.bias.data = bias.detach().clone()
        if o_bias is not None and self.o_bias is not None:
            self.o_bias.data = o_bias.detach().clone()

    # -- what differs between the two flavours of the reference -------------------------------------------
    def _io_perfect(self) -> bool:
        """True switches the DAC, the ADC and the output noise off (only the AIHWKIT flavour can)."""
        return False

    def _noise_per_channel(self) -> bool:
        return bool(getattr(self.rpu_config.forward, "out_noise_per_channel", False))

    def _modifier_on(self) -> bool:
        return enum_name(self.rpu_config.modifier.type) != "NONE"

    def _modified(self, weights: Tensor, is_down: bool = False) -> Tensor:
        return self.modify_weight(weights, self.rpu_config.modifier, **self._modifier_draw(is_down))

    def _row_abs_max_on(self) -> bool:
        """Whether CVMM will scale every input row by its abs-max (cvmm.py:727-739)."""
        return self.input_range is None

    def _modifier_draw(self, is_down: bool) -> dict:
        """Where the modifier's normals come from: the layer's seed (and its device counter) for the kernel's
        generator, or -- ``noise_mode="injected"`` -- torch's own stream, as the reference draws them."""
        if self.noise_mode == "injected":
            return dict(injected=True)
        seed = self._noise_seed() ^ (_MODIFIER_DOWN_SEED if is_down else 0)
        return dict(seed=seed, seed_dev=self.noise_counter)

    # -- weight modifier / clipping (moe_layer_aihwkit_lightning.py:313-382, 509-543) -----------------
    @staticmethod
    def modify_weight(inp_weight: Tensor, modifier, *, seed: Optional[int] = None, seed_dev: Optional[Tensor] = None,
                      injected: bool = False) -> Tensor:
        """A modified copy of ``inp_weight`` [E, K, N] (one kernel pass; the reference clones and modifies in
        place).  The gradient of the result reaches ``inp_weight`` unchanged."""
        kind = enum_name(modifier.type)
        if kind == "NONE":
            return inp_weight
        if kind not in _LIGHTNING_MODIFIERS:
            raise MoEConifgError(f"Weight modifier {modifier} not supported")
        # per-channel max |W| for the two discretising per-channel types only: the reference's list
        # (moe_layer_aihwkit_lightning.py:333-337) names DISCRETIZE_ADD_NORMAL_PER_CHANNEL twice and leaves
        # ADD_NORMAL_PER_CHANNEL out, so that type scales its noise by the per-expert maximum -- kept as it is
        per_channel = kind in ("DISCRETIZE_PER_CHANNEL", "DISCRETIZE_ADD_NORMAL_PER_CHANNEL")
        n_states = float(max(modifier.res, 1 / modifier.res)) if kind.startswith("DISCRETIZE") else 0.0
        std_dev = float(modifier.std_dev) if "ADD_NORMAL" in kind else 0.0
        return _modify_on_device(inp_weight, per_channel, n_states, std_dev, True, seed, seed_dev, injected)

    def post_update_step(self) -> None:
        if hasattr(self.rpu_config, "clip") and enum_name(self.rpu_config.clip.type) != "NONE":
            self.clip_weights()
            if isinstance(self.expert_sel, AnalogLinear):
                self.expert_sel.clip_weights()

    @torch.no_grad()
    def clip_weights(self) -> None:
        kind = enum_name(self.rpu_config.clip.type)
        if kind == "NONE":
            return
        sigma = self.rpu_config.clip.sigma
        assert sigma > 0, "Clip sigma must be greater than 0"
        if kind not in ("LAYER_GAUSSIAN", "LAYER_GAUSSIAN_PER_CHANNEL"):
            raise ValueError(f"Unknown clip type {self.rpu_config.clip.type}")
        for w in (self.keys, self.values):
            _gaussian_clip_(w.data, sigma, kind == "LAYER_GAUSSIAN_PER_CHANNEL")

    # -- the analog matmul ------------------------------------------------------------------------------
    def _update_input_range_from_data(self, inputs: Tensor, sel_indices: CVMMSel, ir_idx: int) -> None:
        """Running average of init_std_alpha * std during the first init_from_data calls; one counter
        for both projections (moe_layer_aihwkit_lightning.py:432-445)."""
        ir_params = self.rpu_config.pre_post.input_range
        if not self._init_from_data_pending():
            return
        idx = self.input_range_update_idx
        stds = cvmm_std(inputs, sel_indices.sel_index, sel_indices.sel, self.n_experts).float()
        ok = stds > 0.0
        if ok.any():
            ir = self.input_range.data[ir_idx]
            upd = (ir * idx + ir_params.init_std_alpha * (stds if ir.dim() == 1 else stds[:, None])) / (idx + 1)
            ir[ok] = upd[ok].to(ir.dtype)
            self.input_range_update_idx.data += 1
        self.input_range.data = self.input_range.data.abs()

    def _init_from_data_pending(self) -> bool:
        """True while the input ranges are still being initialised from data.  Costs no device
        synchronisation when init_from_data is 0, and none after the initialisation has ended."""
        n = self.rpu_config.pre_post.input_range.init_from_data
        if n <= 0 or self._init_done:
            return False
        if not bool(self.input_range_update_idx < n):
            self._init_done = True
            return False
        return True

    def use_device_noise_counter(self) -> Tensor:
        """Keep the per-call part of the noise seed in device memory (one int64 word that every noisy
        launch reads and every forward bumps on the stream).  A forward captured in a HIP graph then
        draws new noise on each replay; without it the seed is a launch argument frozen at capture.  The
        same holds for a forward traced by ``torch.compile``.  Calling this again re-reads torch's seed."""
        if self.noise_counter is None:
            self.noise_counter = torch.zeros(1, dtype=torch.int64, device=self.keys.device)
        # the host part of the seed is read here, once: a traced or captured forward cannot ask for it
        self._noise_seed_base = (torch.initial_seed() * 0x9E3779B97F4A7C15) & (2 ** 63 - 1)
        if isinstance(self.expert_sel, AnalogLinear):       # the router draws from the same counter
            self.expert_sel.noise_counter = self.noise_counter
            self.expert_sel._noise_seed_base = self._noise_seed_base
        return self.noise_counter

    def _noise_seed(self) -> int:
        if self.noise_counter is not None:       # the call count lives on the device
            return self._noise_seed_base
        if torch.compiler.is_compiling():
            raise MoEConifgError("a compiled noisy forward would freeze the host-side noise seed: call "
                                 "use_device_noise_counter() on the layer before torch.compile")
        self._noise_calls += 1
        return (torch.initial_seed() * 0x9E3779B97F4A7C15 + self._noise_calls * 0xD1B54A32D192ED03) & (2 ** 63 - 1)

    def cvmm_wrapper(self, inputs: Tensor, sel_indices: CVMMSel, weights: Tensor) -> Tensor:
        """moe_layer_aihwkit_lightning.py:412-507."""
        if not (inputs.is_cuda or inputs.is_meta):
            raise MoEConifgError("Analog MoE executed on CPU. This package runs on the GPU only.")
        fwd = self.rpu_config.forward
        is_up = inputs.ndim == 3
        ir_idx = 0 if is_up else 1
        bounds = self.bounds_up if is_up else self.bounds_down
        nt = 1 if bounds is None else len(bounds) - 1
        bir = None
        if self.input_range is not None:
            if self.training:
                self._update_input_range_from_data(inputs, sel_indices, ir_idx)
            ir = self.input_range[ir_idx]
            if ir.dim() == 2:
                ir = ir[:, :nt]
            bir = ir[sel_indices.sel]                                   # [..., k(, n_tiles)]
        perfect = self._io_perfect()
        inp_res = -1.0 if perfect else kernel_inp_res(fwd.inp_res)
        modified = weights
        drew = False                                   # a launch of this call read the device seed word
        if (self.training or self.rpu_config.modifier.enable_during_test) and self._modifier_on():
            modified = self._modified(weights, is_down=not is_up)
            drew = self.noise_mode != "injected"
        ext = AnalogExt(offsets=sel_indices.offsets, bounds=bounds,
                        out_bound=-1.0 if perfect else float(getattr(fwd, "out_bound", -1)),
                        out_res=-1.0 if perfect else float(getattr(fwd, "out_res", -1)))
        per_channel = self._noise_per_channel()
        noisy = self.training and fwd.out_noise > 0 and not perfect
        if ext.out_bound > 0 or noisy:
            ext.wmax = torch.ops.amoe.weight_abs_max(weights.detach(), per_channel)
        out_noise = None
        if noisy and self.noise_mode == "kernel":
            ext.noise_std, ext.noise_seed = float(fwd.out_noise), self._noise_seed()
            ext.noise_seed_dev = self.noise_counter
        elif noisy:
            shape = (nt, *sel_indices.raw_sel.shape, weights.shape[-1])
            out_noise = torch.randn(shape, device=inputs.device) * fwd.out_noise * ext.wmax[sel_indices.raw_sel]
        res = CVMM.apply(inputs, sel_indices.sel_index, sel_indices.sel, modified, inp_res, bir,
                         sel_indices.out_index, sel_indices.reduction_weight, out_noise,
                         self.rpu_config.pre_post.input_range, fwd, ext)
        if self.noise_counter is not None and (drew or ext.noise_seed_dev is not None):
            self.noise_counter.add_(1)                 # output noise or a weight modifier drew from it
        return res

    # -- fused path ---------------------------------------------------------------------------------------
    def _fusable(self) -> bool:
        return (self.activation is F.relu and self.bias is None and self.dropout == 0 and
                self.input_range is not None and not self._row_abs_max_on() and
                not (self.training and self._init_from_data_pending()))

    def forward_selected(self, x: Tensor, sel_val: Tensor, sel_idx: Tensor) -> Tensor:
        if not (x.is_cuda or x.is_meta) or not self._fusable():
            return super().forward_selected(x, sel_val, sel_idx)
        fwd = self.rpu_config.forward
        irp = self.rpu_config.pre_post.input_range
        perfect = self._io_perfect()
        noisy = self.training and fwd.out_noise > 0 and not perfect
        cfg = FFNConfig(inp_res=-1.0 if perfect else kernel_inp_res(fwd.inp_res), bounds_up=self.bounds_up,
                        bounds_down=self.bounds_down,
                        out_bound=-1.0 if perfect else float(getattr(fwd, "out_bound", -1)),
                        out_res=-1.0 if perfect else float(getattr(fwd, "out_res", -1)),
                        noise_std=float(fwd.out_noise) if noisy else 0.0, noise_seed=self._noise_seed() if noisy else 0,
                        noise_seed_dev=self.noise_counter if noisy else None,
                        noise_per_channel=self._noise_per_channel(),
                        gradient_relative=getattr(irp, "gradient_relative", True),
                        gradient_scale=getattr(irp, "gradient_scale", 1.0), decay=irp.decay,
                        input_min_percentage=irp.input_min_percentage)
        if noisy and self.noise_mode == "injected":
            E, k = self.n_experts, self.n_heads
            M = sel_idx.numel()
            flat = sel_idx.reshape(-1)
            pc = cfg.noise_per_channel
            wu = torch.ops.amoe.weight_abs_max(self.keys.detach(), pc)
            wd = torch.ops.amoe.weight_abs_max(self.values.detach(), pc)
            ntu = 1 if self.bounds_up is None else len(self.bounds_up) - 1
            ntd = 1 if self.bounds_down is None else len(self.bounds_down) - 1
            cfg.noise_up = torch.randn(ntu, M, self.expert_size, device=x.device) * fwd.out_noise * wu[flat]
            cfg.noise_down = torch.randn(ntd, M, self.v_dim, device=x.device) * fwd.out_noise * wd[flat]
        keys, values = self.keys, self.values
        drew = False
        if (self.training or self.rpu_config.modifier.enable_during_test) and self._modifier_on():
            drew = self.noise_mode != "injected"
            # The modified copies depend on the parameters only: called eagerly they are made on a second stream, the
            # up-projection's next to the expert sort and the down-projection's next to the up-projection (which
            # waits for its own copy only).  The output noise and the ADC keep following the max |W| of the
            # unmodified weights (moe_layer_aihwkit_lightning.py:458-489)
            want_wmax = noisy or cfg.out_bound > 0
            fork = x.is_cuda and not torch.compiler.is_compiling()
            main = torch.cuda.current_stream() if fork else None
            side = _side_stream(x.device) if fork else None
            if fork:
                side.wait_stream(main)
            with (torch.cuda.stream(side) if fork else contextlib.nullcontext()):
                if want_wmax:
                    cfg.wmax_up = torch.ops.amoe.weight_abs_max(keys.detach(), cfg.noise_per_channel)
                keys = self._modified(keys, is_down=False)
                if fork:
                    main.wait_event(side.record_event())
                if want_wmax:
                    cfg.wmax_down = torch.ops.amoe.weight_abs_max(values.detach(), cfg.noise_per_channel)
                values = self._modified(values, is_down=True)
                if fork:
                    cfg.down_ready = side.record_event()
            if fork:
                for t in (keys, values, cfg.wmax_up, cfg.wmax_down):
                    if t is not None:
                        t.record_stream(main)
        lead = x.shape[:-1]
        if torch.is_autocast_enabled():            # as CVMM.forward does (cvmm.py:716): compute in the autocast type
            dt = torch.get_autocast_dtype("cuda")
            if dt not in (torch.bfloat16, torch.float16):
                raise MoEConifgError("the CVMM kernels autocast to bfloat16 or float16")
            x = x.to(dt)
        # the two projections use seed + 0 and seed + 1, so the device word moves by 2 per call; a weight modifier alone
        # (no output noise) must see a new word too.  Called eagerly, the layer's last forward launch adds it; under
        # torch.compile (opaque operators that declare no mutation) the addition stays a torch operation
        bump_here = self.noise_counter is not None and (drew or cfg.noise_seed_dev is not None)
        if bump_here and cfg.noise_seed_dev is not None and not torch.compiler.is_compiling():
            cfg.seed_bump, bump_here = 2, False
        y = moe_ffn(x.reshape(-1, x.shape[-1]), keys.to(x.dtype), values.to(x.dtype),
                    self.input_range, sel_val.reshape(-1, self.n_heads).to(x.dtype),
                    sel_idx.reshape(-1, self.n_heads), cfg)
        if bump_here:
            self.noise_counter.add_(2)
        y = y.view(*lead, self.v_dim)
        if self.o_bias is not None:
            y = y + self.o_bias
        return y

    # -- checkpointing: the config travels with the state dict (:545-570) ------------------------------------
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        destination._metadata[prefix.split(".")[0]]["rpu_config"] = self.rpu_config

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)
        if "rpu_config" in local_metadata:
            self.rpu_config = local_metadata["rpu_config"]
        self._init_done = False


class AnalogSigmaMoELayerAIHWKIT(AnalogSigmaMoELayer):
    """The reference's second flavour (analog_moe/moe_layer_aihwkit.py:29-436) on the same kernels.  What it
    does differently from the lightning flavour:

    * ``forward.is_perfect`` switches quantisation and output noise off (:243-258);
    * the row abs-max scaling follows ``forward.noise_management`` instead of the input range
      (cvmm.py:735-739), and the bound management must be off (:59-61);
    * the max |W| behind the output noise and the weight modifier follows ``remap.type`` (:172-182, 264-279);
    * the weight modifier knows ADD_NORMAL only (:144-196), the clip FIXED_VALUE and LAYER_GAUSSIAN
      (:313-340);
    * the configuration travels in the state dict under ``analog_tile_state`` (:372-415).

    AIHWKIT's tile objects (``AnalogContext``, the analog optimizer hooks) are third-party and not part of
    this package; the K-tile split and the ADC, which the reference asserts off (:50-58), stay available."""

    def __init__(self, rpu_config=None, *args, **kwargs):
        rpu_config = AIHWKITTorchInferenceRPUConfig() if rpu_config is None else rpu_config
        fwd = rpu_config.forward
        if not hasattr(fwd, "is_perfect"):
            raise MoEConifgError("the AIHWKIT flavour needs an rpu_config whose forward has is_perfect "
                                 "(an aihwkit TorchInferenceRPUConfig or AIHWKITTorchInferenceRPUConfig)")
        assert getattr(fwd, "inp_bound", 1.0) in [-1, 1.0], "inp_bound must be 1.0 or off (=-1)"
        assert enum_name(getattr(fwd, "bound_management", "NONE")) == "NONE", "bound_management must be NONE"
        # this flavour keeps the router it is given (moe_layer_aihwkit.py:88-94, 135-142): converting it is left
        # to the caller's conversion of the whole model
        kwargs.setdefault("analog_router", False)
        super().__init__(rpu_config, *args, **kwargs)

    # -- flavour hooks ---------------------------------------------------------------------------------------
    def _remap(self) -> str:
        remap = getattr(self.rpu_config, "remap", None)
        return "NONE" if remap is None else enum_name(remap.type)

    def _io_perfect(self) -> bool:
        return bool(self.rpu_config.forward.is_perfect)

    def _noise_per_channel(self) -> bool:
        kind = self._remap()                                  # moe_layer_aihwkit.py:264-279
        if kind in ("CHANNELWISE_SYMMETRIC", "NONE"):
            return True
        if kind == "LAYERWISE_SYMMETRIC":
            return False
        raise MoEConifgError(f"Weight remap type {self.rpu_config.remap.type} not supported")

    def _modifier_on(self) -> bool:
        return enum_name(self.rpu_config.modifier.type) not in ("NONE", "COPY")

    def _modified(self, weights: Tensor, is_down: bool = False) -> Tensor:
        return self.modify_weight(weights, self.rpu_config.modifier, self.rpu_config.remap.type,
                                  **self._modifier_draw(is_down))

    def _row_abs_max_on(self) -> bool:
        fwd = self.rpu_config.forward
        return not fwd.is_perfect and enum_name(fwd.noise_management) == "ABS_MAX"

    @staticmethod
    def modify_weight(inp_weight: Tensor, modifier, remap_type=None, *, seed: Optional[int] = None,
                      seed_dev: Optional[Tensor] = None, injected: bool = False) -> Tensor:
        """moe_layer_aihwkit.py:144-196: ADD_NORMAL only, max |W| by remap type, fp32 normals."""
        if getattr(modifier, "per_batch_sample", False):
            raise MoEConifgError("per_batch_sample not implemented")
        kind = enum_name(modifier.type)
        if kind in ("NONE", "COPY"):
            return inp_weight
        if kind == "MULT_NORMAL":
            raise MoEConifgError("MULT_NORMAL not implemented")
        remap = enum_name(remap_type)
        if remap not in ("CHANNELWISE_SYMMETRIC", "LAYERWISE_SYMMETRIC"):
            raise MoEConifgError(f"Weight remap type {remap_type} not supported")
        if kind == "DISCRETIZE":
            raise MoEConifgError("DISCRETIZE not implemented")
        if kind != "ADD_NORMAL":
            raise MoEConifgError(f"Weight modifier {modifier} not supported")
        return _modify_on_device(inp_weight, remap == "CHANNELWISE_SYMMETRIC", 0.0, float(modifier.std_dev), False,
                                 seed, seed_dev, injected)

    def post_update_step(self) -> None:
        if hasattr(self.rpu_config, "clip") and enum_name(self.rpu_config.clip.type) != "NONE":
            self.clip_weights(self.rpu_config.clip)

    @torch.no_grad()
    def clip_weights(self, clip=None) -> None:
        """moe_layer_aihwkit.py:313-340."""
        clip = self.rpu_config.clip if clip is None else clip
        kind = enum_name(clip.type)
        if kind == "FIXED_VALUE":
            for w in (self.keys, self.values):
                _need_device(w, "Weight clipping")
                if not w.is_meta:
                    ops.clamp_weights_(w.data, torch.full((w.shape[0],), float(clip.fixed_value), device=w.device))
        elif kind == "LAYER_GAUSSIAN":
            for w in (self.keys, self.values):
                _gaussian_clip_(w.data, clip.sigma, False, max_bound=clip.fixed_value)
        elif kind == "AVERAGE_CHANNEL_MAX":
            raise NotImplementedError("AVERAGE_CHANNEL_MAX not implemented")
        else:
            raise MoEConifgError(f"Unknown clip type {clip.type}")

    def get_dtype(self) -> torch.dtype:
        return self.keys.dtype

    # -- checkpointing (moe_layer_aihwkit.py:372-436) --------------------------------------------------------------
    def load_state_dict(self, state_dict, strict: bool = True, load_rpu_config: Optional[bool] = None,
                        strict_rpu_config_check: Optional[bool] = None, **kwargs):
        state_dict = state_dict.copy()
        analog_tile_state = state_dict.pop("analog_tile_state", None)
        if analog_tile_state is not None:
            if strict_rpu_config_check:
                ok, msg = self.compatible_with(analog_tile_state["rpu_config"])
                if not ok:
                    raise MoEConifgError(msg)
            if load_rpu_config or load_rpu_config is None:
                self.rpu_config = analog_tile_state["rpu_config"]
        self._init_done = False
        return nn.Module.load_state_dict(self, state_dict, strict, **kwargs)

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        nn.Module._save_to_state_dict(self, destination, prefix, keep_vars)
        destination[prefix + "analog_tile_state"] = {"rpu_config": self.rpu_config}

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        analog_tile_state = state_dict.pop(prefix + "analog_tile_state", None)
        if analog_tile_state is not None:
            self.rpu_config = analog_tile_state["rpu_config"]
        nn.Module._load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                                        unexpected_keys, error_msgs)
        self._init_done = False

    def compatible_with(self, rpu_config) -> Tuple[bool, Optional[str]]:
        if not isinstance(self.rpu_config, type(rpu_config)) and not isinstance(rpu_config, type(self.rpu_config)):
            return False, ("RPU config mismatch: Cannot replace "
                           f"{rpu_config.__class__.__name__} with {self.rpu_config.__class__.__name__}")
        return True, None


# Name under which the reference exports its lightning flavour (analog_moe/__init__.py).
AnalogSigmaMoELayerAIHWKITLightning = AnalogSigmaMoELayer
