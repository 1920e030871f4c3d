"""GPT-2 with dynamic-k MoE feed-forward layers: the model-level harness around the MoE-FFN path.

The model follows the reference's GPT (architectures/gpt.py:27-262): same module tree and parameter names
(``transformer.wte / wpe / h.{i}.ln_1 / attn.c_attn / attn.c_proj / ln_2 / mlp.c_fc / mlp.c_proj / ln_f``, tied
``lm_head``), same initialisation (N(0, 0.02), residual projections scaled by 1/sqrt(2 n_layer)), so a reference
``state_dict`` loads.  Attention is PyTorch's scaled_dot_product_attention (causal); only the feed-forward layers are
this package's business.

Model surgery mirrors ``replace_with_moes`` / ``split_original_parameters`` (architectures/moe/moefication.py:104-202,
205-306) and the patched forwards (architectures/moe/moe_models.py:79-100, 194-218):

* ``replace_with_moes(model, num_experts=..., experts_class='hip_kernel')`` returns a deep copy whose ``Block.mlp`` are
  ``MoeficationMoE`` layers (plus the ``dropout`` child the reference hangs on them) and whose block / model forwards
  also return the gating data.  The reference's block forward starts with ``torch.any(torch.isnan(input))``, a host
  synchronisation per block; it is left out here.
* ``split_original_parameters(original, moe_model, names, labels=None)`` moves the dense FFN weights into the experts:
  neuron ``n`` of ``c_fc`` / ``c_proj`` becomes neuron ``j`` of expert ``labels[n]`` (``w1[e, :, j] = W_fc[n]``,
  ``b1[e, j] = b_fc[n]``, ``w2[e, j] = W_proj[:, n]``, ``last_bias = b_proj``).  The reference takes ``labels`` from
  balanced k-means over the normalised ``c_fc`` rows (``k_means_constrained``, not available here); any balanced
  labelling gives the same function when every expert runs, and the default is contiguous blocks of neurons.
"""
from __future__ import annotations

import math
from copy import deepcopy
from dataclasses import dataclass
from functools import partial
from typing import Dict, List, Optional, Sequence

import torch
from torch import nn
from torch.nn import functional as F

from .layer import MoELayer, MoeficationMoE


@dataclass
class GPTConfig:
    block_size: int = 1024
    vocab_size: int = 50304   # GPT-2's 50257 padded to a multiple of 64
    n_layer: int = 12
    n_head: int = 12
    n_embd: int = 768
    dropout: float = 0.0
    bias: bool = True
    activation: str = 'gelu'


class LayerNorm(nn.Module):
    """LayerNorm with an optional bias (architectures/gpt.py:27-36)."""

    def __init__(self, ndim, bias):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(ndim))
        self.bias = nn.Parameter(torch.zeros(ndim)) if bias else None

    def forward(self, x):
        return F.layer_norm(x, self.weight.shape, self.weight, self.bias, 1e-5)


class CausalSelfAttention(nn.Module):
    def __init__(self, config):
        super().__init__()
        assert config.n_embd % config.n_head == 0
        self.c_attn = nn.Linear(config.n_embd, 3 * config.n_embd, bias=config.bias)
        self.c_proj = nn.Linear(config.n_embd, config.n_embd, bias=config.bias)
        self.resid_dropout = nn.Dropout(config.dropout)
        self.n_head = config.n_head
        self.n_embd = config.n_embd
        self.dropout = config.dropout

    def forward(self, x):
        B, T, C = x.size()
        q, k, v = self.c_attn(x).split(self.n_embd, dim=2)
        q = q.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        k = k.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        v = v.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=self.dropout if self.training else 0.0,
                                           is_causal=True)
        y = y.transpose(1, 2).contiguous().view(B, T, C)
        return self.resid_dropout(self.c_proj(y))


class MLP(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.c_fc = nn.Linear(config.n_embd, 4 * config.n_embd, bias=config.bias)
        if config.activation in ('gelu', None):
            self.act = nn.GELU()
        elif config.activation == 'relu':
            self.act = nn.ReLU()
        else:
            raise NotImplementedError(config.activation)
        self.c_proj = nn.Linear(4 * config.n_embd, config.n_embd, bias=config.bias)
        self.dropout = nn.Dropout(config.dropout)

    def forward(self, x):
        return self.dropout(self.c_proj(self.act(self.c_fc(x))))


class Block(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.ln_1 = LayerNorm(config.n_embd, bias=config.bias)
        self.attn = CausalSelfAttention(config)
        self.ln_2 = LayerNorm(config.n_embd, bias=config.bias)
        self.mlp = MLP(config)

    def forward(self, x):
        x = x + self.attn(self.ln_1(x))
        return x + self.mlp(self.ln_2(x))


class GPT(nn.Module):
    def __init__(self, config: GPTConfig):
        super().__init__()
        self.config = config
        self.transformer = nn.ModuleDict(dict(
            wte=nn.Embedding(config.vocab_size, config.n_embd),
            wpe=nn.Embedding(config.block_size, config.n_embd),
            drop=nn.Dropout(config.dropout),
            h=nn.ModuleList([Block(config) for _ in range(config.n_layer)]),
            ln_f=LayerNorm(config.n_embd, bias=config.bias),
        ))
        self.lm_head = nn.Linear(config.n_embd, config.vocab_size, bias=False)
        self.transformer.wte.weight = self.lm_head.weight   # weight tying
        self.apply(self._init_weights)
        for name, p in self.named_parameters():
            if name.endswith('c_proj.weight'):
                torch.nn.init.normal_(p, mean=0.0, std=0.02 / math.sqrt(2 * config.n_layer))

    @staticmethod
    def _init_weights(module):
        if isinstance(module, nn.Linear):
            torch.nn.init.normal_(module.weight, mean=0.0, std=0.02)
            if module.bias is not None:
                torch.nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            torch.nn.init.normal_(module.weight, mean=0.0, std=0.02)

    def embed(self, idx):
        b, t = idx.size()
        assert t <= self.config.block_size, f'sequence of length {t} exceeds the block size {self.config.block_size}'
        pos = torch.arange(0, t, dtype=torch.long, device=idx.device)
        return self.transformer.drop(self.transformer.wte(idx) + self.transformer.wpe(pos))

    def forward(self, idx):
        x = self.embed(idx)
        for block in self.transformer.h:
            x = block(x)
        return self.lm_head(self.transformer.ln_f(x))


# ------------------------------------------------------------------------------------------- patched forwards
def moe_gpt_block_forward(self, input: torch.Tensor):
    """Block forward that also returns the gating data of its MoE layer (moe_models.py:79-100, without the NaN check
    that synchronises the host)."""
    torch._assert(input.dim() == 3, f'Expected (batch_size, seq_length, hidden_dim) got {input.shape}')
    gating_data = {}
    h = input + self.attn(self.ln_1(input))
    ln2 = self.ln_2(h)
    if isinstance(self.mlp, MoELayer):
        mlp_out, ffn_gating_data = self.mlp(ln2)
        mlp_out = self.mlp.dropout(mlp_out)
        gating_data.update(ffn_gating_data)
    else:
        mlp_out = self.mlp(ln2)
    return h + mlp_out, gating_data


def moe_gpt_main_forward(self, x: torch.Tensor, return_gating_data: bool = False):
    """Model forward collecting the gating data of every block (moe_models.py:194-218)."""
    x = self.embed(x)
    gating_data = {}
    for block in self.transformer.h:
        x, block_gating_data = block(x)
        gating_data.update(block_gating_data)
    x = self.lm_head(self.transformer.ln_f(x))
    return (x, gating_data) if return_gating_data else x


# ------------------------------------------------------------------------------------------- model surgery
def is_gated_ffn(ffn: nn.Module) -> bool:
    """A LLaMA/Gemma-style gated FFN: Linear submodules gate_proj, up_proj, down_proj and an activation act_fn (the
    layout of transformers' GemmaMLP, which the reference converts with intermediate gating, moefication.py:115-129)."""
    return all(isinstance(getattr(ffn, n, None), nn.Linear) for n in ('gate_proj', 'up_proj', 'down_proj')) and \
        isinstance(getattr(ffn, 'act_fn', None), nn.Module)


def ffn_parts(ffn: nn.Module):
    """(first Linear, activation module, second Linear, dropout probability) of a dense FFN block: this file's `MLP`
    (c_fc, act, c_proj, dropout), an index-addressed Linear/act/Dropout/Linear/Dropout sequence (torchvision's
    MLPBlock, `vit.MLPBlock`), or a gated FFN, whose first Linear is the gate projection (`ffn.up_proj` is its third)."""
    if isinstance(ffn, MLP):
        return ffn.c_fc, ffn.act, ffn.c_proj, ffn.dropout.p
    if isinstance(ffn, nn.Sequential) and len(ffn) == 5 and isinstance(ffn[0], nn.Linear) and isinstance(ffn[3], nn.Linear):
        return ffn[0], ffn[1], ffn[3], ffn[4].p if isinstance(ffn[4], nn.Dropout) else 0.0
    if is_gated_ffn(ffn):
        return ffn.gate_proj, ffn.act_fn, ffn.down_proj, 0.0
    raise ValueError(f'Unsupported ffn type: {type(ffn)}')


def ffn_filter_condition(_model: nn.Module, m: nn.Module) -> bool:
    if isinstance(m, MLP) or is_gated_ffn(m):
        return True
    return isinstance(m, nn.Sequential) and len(m) == 5 and isinstance(m[0], nn.Linear) and isinstance(m[3], nn.Linear)


def find_module_names(model: nn.Module, condition=None) -> List[str]:
    condition = condition or ffn_filter_condition
    return [name for name, m in model.named_modules() if condition(model, m)]


def _parent_and_attr(model: nn.Module, name: str):
    parts = name.split('.')
    parent = model
    for p in parts[:-1]:
        parent = parent[int(p)] if p.isdigit() and isinstance(parent, (nn.ModuleList, nn.Sequential)) else getattr(parent, p)
    return parent, parts[-1]


def get_module_by_name(model: nn.Module, name: str) -> nn.Module:
    parent, attr = _parent_and_attr(model, name)
    return parent[int(attr)] if attr.isdigit() and isinstance(parent, (nn.ModuleList, nn.Sequential)) else getattr(parent, attr)


def set_module_by_name(model: nn.Module, name: str, module: Optional[nn.Module]):
    parent, attr = _parent_and_attr(model, name)
    if attr.isdigit() and isinstance(parent, (nn.ModuleList, nn.Sequential)):
        parent[int(attr)] = module
    else:
        setattr(parent, attr, module)


def replace_layer_with_moe(model: nn.Module, name: str, num_experts=None, expert_size=None, experts_class='hip_kernel'):
    original = get_module_by_name(model, name)
    w1, act, _, dropout_p = ffn_parts(original)
    hidden_dim, d_ff = w1.in_features, w1.out_features
    if num_experts is not None:
        assert d_ff % num_experts == 0, 'd_ff has to be divisible by the number of experts'
        expert_size = d_ff // num_experts
    else:
        assert d_ff % expert_size == 0, 'd_ff has to be divisible by the expert size'
        num_experts = d_ff // expert_size
    gated = is_gated_ffn(original)
    moe_layer = MoeficationMoE(name, hidden_dim, num_experts, w1.bias is not None, expert_size, type(act), experts_class,
                               add_intermediate_gating=gated)
    moe_layer = moe_layer.to(device=w1.weight.device, dtype=w1.weight.dtype)
    set_module_by_name(model, name, moe_layer)
    if not gated:
        set_module_by_name(model, f'{name}.dropout', nn.Dropout(dropout_p))


def replace_with_moes(original_model: nn.Module, num_experts: int = None, expert_size: int = None,
                      experts_class: str = 'hip_kernel', module_filter_condition=None):
    """Deep copy of `original_model` (this package's GPT or VisionTransformer) with every selected FFN replaced by a MoE
    layer and the forwards patched to return gating data; returns (model, names of the replaced modules)."""
    from . import vit
    assert (num_experts is None) != (expert_size is None), 'pass exactly one of num_experts and expert_size'
    if not isinstance(original_model, (GPT, vit.VisionTransformer)):
        raise ValueError(f'Unsupported model type: {type(original_model)}')
    original_model.eval()
    model = deepcopy(original_model)
    names = find_module_names(original_model, module_filter_condition)
    for name in names:
        replace_layer_with_moe(model, name, num_experts, expert_size, experts_class)
    if isinstance(model, GPT):
        for block in model.transformer.h:
            block.forward = partial(moe_gpt_block_forward, block)
        model.forward = partial(moe_gpt_main_forward, model)
    else:
        vit.patch_forwards(model)
    return model, names


def param_split(ffn: nn.Module, moe_layer: MoeficationMoE, labels: Optional[Sequence[int]] = None):
    """Moves the dense FFN's neurons into the experts: neuron n goes to expert labels[n], in order of appearance (what the
    reference's param_clustering_split does with its clustering labels, moefication.py:205-285).  Works for every
    experts container of this package; for a gated FFN the gate projection is the first layer and the up projection is
    split alongside it."""
    ex = moe_layer.experts
    E, Ed = moe_layer.num_experts, moe_layer.expert_dim
    fc1, _, fc2, _ = ffn_parts(ffn)
    up = ffn.up_proj if is_gated_ffn(ffn) else None
    d_ff = fc1.out_features
    D = fc1.in_features
    if labels is None:
        labels = torch.arange(d_ff) // Ed
    labels = torch.as_tensor(labels, dtype=torch.long)
    assert labels.numel() == d_ff and torch.equal(torch.bincount(labels, minlength=E), torch.full((E,), Ed)), \
        'every expert takes exactly expert_dim neurons'
    # position of each neuron inside its expert = its rank among the neurons with the same label
    order = torch.argsort(labels, stable=True)          # neurons grouped by expert, original order kept
    slot = torch.empty_like(order)
    slot[order] = torch.arange(d_ff) % Ed
    ref = next(ex.parameters())
    with torch.no_grad():
        w1 = torch.empty(E, D, Ed, dtype=ref.dtype)
        w2 = torch.empty(E, Ed, D, dtype=ref.dtype)
        w1[labels, :, slot] = fc1.weight.detach().cpu().to(ref.dtype)               # fc1.weight [d_ff, D]
        w2[labels, slot, :] = fc2.weight.detach().cpu().t().to(ref.dtype)           # fc2.weight [D, d_ff]
        b1 = w_up = None
        if moe_layer.bias:
            b1 = torch.empty(E, Ed, dtype=ref.dtype)
            b1[labels, slot] = fc1.bias.detach().cpu().to(ref.dtype)
        if up is not None:
            w_up = torch.empty(E, D, Ed, dtype=ref.dtype)
            w_up[labels, :, slot] = up.weight.detach().cpu().to(ref.dtype)
        dev = ref.device
        ex.load_operands(w1.to(dev), None if b1 is None else b1.to(dev), w2.to(dev), None if w_up is None else w_up.to(dev))
        if moe_layer.bias:
            moe_layer.last_bias.copy_(fc2.bias.detach().view(1, -1))


def split_original_parameters(original_model: nn.Module, moe_model: nn.Module, replaced_module_names: List[str],
                              labels: Optional[Dict[str, Sequence[int]]] = None):
    assert len(replaced_module_names) > 0
    original_model.eval()
    for name in replaced_module_names:
        param_split(get_module_by_name(original_model, name), get_module_by_name(moe_model, name),
                    None if labels is None else labels[name])
