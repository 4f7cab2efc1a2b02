"""A minimal SigmaMoE decoder: the caller of the CVMM path in the full training step.

The reference's example trains ``sigma_moe.SigmaMoEForCausalLM`` (example_aihwkit.py:6, 86-100), a
third-party model whose feed-forward blocks are the SigmaMoE layers this package implements.  That model is
not part of the reference checkout; this module provides the smallest stand-in that exercises the layer the
same way: token + position embedding, pre-norm blocks of causal self-attention and an analog SigmaMoE
feed-forward, final norm and language-model head.  Attention, norms and embeddings are stock PyTorch; the
MoE feed-forward is ``AnalogSigmaMoELayer`` (or any module with its ``forward(x) -> (y, reg_loss)``).
"""
from __future__ import annotations

from typing import Callable, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn


class CausalSelfAttention(nn.Module):
    def __init__(self, d_model: int, n_heads: int):
        super().__init__()
        if d_model % n_heads:
            raise ValueError("d_model must be a multiple of n_heads")
        self.n_heads = n_heads
        self.qkv = nn.Linear(d_model, 3 * d_model, bias=False)
        self.proj = nn.Linear(d_model, d_model, bias=False)

    def forward(self, x: Tensor) -> Tensor:
        B, S, D = x.shape
        q, k, v = self.qkv(x).view(B, S, 3, self.n_heads, D // self.n_heads).permute(2, 0, 3, 1, 4)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.proj(a.transpose(1, 2).reshape(B, S, D))


class DecoderBlock(nn.Module):
    def __init__(self, d_model: int, n_heads: int, ffn: nn.Module):
        super().__init__()
        self.ln_attn = nn.LayerNorm(d_model)
        self.attn = CausalSelfAttention(d_model, n_heads)
        self.ln_ffn = nn.LayerNorm(d_model)
        self.ffn = ffn

    def forward(self, x: Tensor) -> Tuple[Tensor, Tensor]:
        x = x + self.attn(self.ln_attn(x))
        y, reg = self.ffn(self.ln_ffn(x))
        return x + y, reg


class SigmaMoEDecoder(nn.Module):
    """``make_ffn(layer_index) -> module`` builds the feed-forward of each block."""

    def __init__(self, vocab_size: int, d_model: int, n_layers: int, n_heads: int, context: int,
                 make_ffn: Callable[[int], nn.Module]):
        super().__init__()
        self.tok = nn.Embedding(vocab_size, d_model)
        self.pos = nn.Embedding(context, d_model)
        self.blocks = nn.ModuleList(DecoderBlock(d_model, n_heads, make_ffn(i)) for i in range(n_layers))
        self.ln_out = nn.LayerNorm(d_model)
        self.head = nn.Linear(d_model, vocab_size, bias=False)

    def forward(self, ids: Tensor, labels: Optional[Tensor] = None, reg_weight: float = 0.0):
        """Logits [B, S, V] and the summed regularisation loss of the MoE layers; with ``labels`` the scalar
        training loss (cross-entropy in fp32 + reg_weight * regularisation) instead of the logits."""
        B, S = ids.shape
        x = self.tok(ids) + self.pos(torch.arange(S, device=ids.device))
        reg = x.new_zeros((), dtype=torch.float32)
        for blk in self.blocks:
            x, r = blk(x)
            reg = reg + r.float()
        logits = self.head(self.ln_out(x))
        if labels is None:
            return logits, reg
        loss = F.cross_entropy(logits.float().view(B * S, -1), labels.reshape(-1))
        return loss + reg_weight * reg, reg

    def post_update_step(self) -> None:
        """Weight clipping of the analog layers after an optimizer step (moe_layer_aihwkit_lightning.py:509-517)."""
        for blk in self.blocks:
            if hasattr(blk.ffn, "post_update_step"):
                blk.ffn.post_update_step()
