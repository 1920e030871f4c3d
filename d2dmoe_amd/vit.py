"""ViT with MoE FFN layers: the model-level drop-in for the reference's converted vision transformers.

A plain VisionTransformer with the module tree and parameter names of torchvision's (which the reference forks in
architectures/vit.py): `conv_proj`, `class_token`, `encoder.pos_embedding`, `encoder.layers.encoder_layer_<i>.{ln_1,
self_attention, ln_2, mlp.0, mlp.3}`, `encoder.ln`, `heads.head` -- so a torchvision or reference state dict loads
unchanged -- and the patched forwards that return the gating data of every MoE layer
(architectures/moe/moe_models.py:55-78, 103-127).  Attention, LayerNorm, patch embedding and the head stay stock
PyTorch; the FFNs become `MoeficationMoE` layers through `gpt2.replace_with_moes`, which recognises both backbones.
"""
from __future__ import annotations

from collections import OrderedDict
from functools import partial

import torch
from torch import nn

from .layer import MoELayer


class MLPBlock(nn.Sequential):
    """Linear, GELU, Dropout, Linear, Dropout -- index-addressed as in torchvision (`mlp.0`, `mlp.3`)."""

    def __init__(self, in_dim: int, mlp_dim: int, dropout: float):
        super().__init__(nn.Linear(in_dim, mlp_dim), nn.GELU(), nn.Dropout(dropout), nn.Linear(mlp_dim, in_dim),
                         nn.Dropout(dropout))


class EncoderBlock(nn.Module):
    def __init__(self, num_heads: int, hidden_dim: int, mlp_dim: int, dropout: float, attention_dropout: float):
        super().__init__()
        self.num_heads = num_heads
        self.ln_1 = nn.LayerNorm(hidden_dim, eps=1e-6)
        self.self_attention = nn.MultiheadAttention(hidden_dim, num_heads, dropout=attention_dropout, batch_first=True)
        self.dropout = nn.Dropout(dropout)
        self.ln_2 = nn.LayerNorm(hidden_dim, eps=1e-6)
        self.mlp = MLPBlock(hidden_dim, mlp_dim, dropout)

    def forward(self, input: torch.Tensor):
        x = self.ln_1(input)
        x, _ = self.self_attention(x, x, x, need_weights=False)
        x = self.dropout(x) + input
        return x + self.mlp(self.ln_2(x))


class Encoder(nn.Module):
    def __init__(self, seq_length, num_layers, num_heads, hidden_dim, mlp_dim, dropout, attention_dropout):
        super().__init__()
        self.pos_embedding = nn.Parameter(torch.empty(1, seq_length, hidden_dim).normal_(std=0.02))
        self.dropout = nn.Dropout(dropout)
        self.layers = nn.Sequential(OrderedDict(
            (f'encoder_layer_{i}', EncoderBlock(num_heads, hidden_dim, mlp_dim, dropout, attention_dropout))
            for i in range(num_layers)))
        self.ln = nn.LayerNorm(hidden_dim, eps=1e-6)

    def forward(self, input: torch.Tensor):
        return self.ln(self.layers(self.dropout(input + self.pos_embedding)))


class VisionTransformer(nn.Module):
    """ViT-B/16 by default: 224 x 224 images, 196 patches + class token = 197 tokens, D = 768, d_ff = 3072."""

    def __init__(self, image_size=224, patch_size=16, num_layers=12, num_heads=12, hidden_dim=768, mlp_dim=3072,
                 dropout=0.0, attention_dropout=0.0, num_classes=1000):
        super().__init__()
        assert image_size % patch_size == 0
        self.image_size, self.patch_size, self.hidden_dim = image_size, patch_size, hidden_dim
        self.conv_proj = nn.Conv2d(3, hidden_dim, kernel_size=patch_size, stride=patch_size)
        seq_length = (image_size // patch_size) ** 2 + 1
        self.class_token = nn.Parameter(torch.zeros(1, 1, hidden_dim))
        self.encoder = Encoder(seq_length, num_layers, num_heads, hidden_dim, mlp_dim, dropout, attention_dropout)
        self.seq_length = seq_length
        self.heads = nn.Sequential(OrderedDict(head=nn.Linear(hidden_dim, num_classes)))

    def _process_input(self, x: torch.Tensor) -> torch.Tensor:
        n, _, h, w = x.shape
        assert h == self.image_size and w == self.image_size, f'expected {self.image_size} x {self.image_size} images'
        x = self.conv_proj(x)                               # (n, hidden, h/p, w/p)
        return x.reshape(n, self.hidden_dim, -1).permute(0, 2, 1)

    def forward(self, x: torch.Tensor):
        x = self._process_input(x)
        x = torch.cat([self.class_token.expand(x.shape[0], -1, -1), x], dim=1)
        return self.heads(self.encoder(x)[:, 0])


# ---- patched forwards (reference: moe_models.py:55-78, 103-127) -----------------------------------------------------
def moe_vit_block_forward(self, input: torch.Tensor):
    """Encoder block that returns (output, gating data); no NaN probe on the input (it would synchronise)."""
    gating_data = {}
    x = self.ln_1(input)
    x, _ = self.self_attention(x, x, x, need_weights=False)
    x = self.dropout(x) + input
    y = self.ln_2(x)
    if isinstance(self.mlp, MoELayer):
        y, ffn_gating_data = self.mlp(y)
        gating_data.update(ffn_gating_data)
    else:
        y = self.mlp(y)
    return x + y, gating_data


def moe_vit_encoder_forward(self, input: torch.Tensor):
    x = self.dropout(input + self.pos_embedding)
    gating_data = {}
    for layer in self.layers:
        x, block_gating_data = layer(x)
        gating_data.update(block_gating_data)
    return self.ln(x), gating_data


def moe_vit_main_forward(self, x: torch.Tensor, return_gating_data: bool = False):
    x = self._process_input(x)
    x = torch.cat([self.class_token.expand(x.shape[0], -1, -1), x], dim=1)
    x, gating_data = self.encoder(x)
    x = self.heads(x[:, 0])
    return (x, gating_data) if return_gating_data else x


def patch_forwards(model: VisionTransformer) -> None:
    for block in model.encoder.layers:
        block.forward = partial(moe_vit_block_forward, block)
    model.encoder.forward = partial(moe_vit_encoder_forward, model.encoder)
    model.forward = partial(moe_vit_main_forward, model)
