"""Experts containers: the plugin boundary of the MoE layer.

Mirrors the reference's experts-container interface (architectures/moe/moe_layers.py):
``cls(dim, num_experts, depth, expert_dim, bias, activation, intermediate_gating)`` and
``forward(x[N, D], routing_tensor[N, E]) -> [N, D]``, chosen by name through ``MOE_IMPL_MAP``
(moe_layers.py:402-407).  Parameter names and shapes equal the reference's so its state_dicts load unchanged.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn

from . import ops
from .hip_abi import D2DMoEError

# activation module -> kernel activation name (reference: moe_layers.py:11-16, extended for gated experts)
ACTIVATION_TO_NAME = {
    nn.GELU: 'gelu',
    nn.Tanh: 'tanh',
    nn.ReLU: 'relu',
    nn.LeakyReLU: 'leaky_relu',
    nn.SiLU: 'silu',
    nn.Identity: 'identity',
}


def activation_name(module_or_cls) -> str:
    """Kernel name of an activation class or instance; GELU(approximate='tanh') maps to 'gelu_tanh'."""
    cls = module_or_cls if isinstance(module_or_cls, type) else type(module_or_cls)
    if cls.__name__ in ('PytorchGELUTanh', 'GELUTanh', 'NewGELUActivation'):
        return 'gelu_tanh'
    if cls not in ACTIVATION_TO_NAME:
        raise NotImplementedError(f'{cls} has no HIP kernel activation')
    if cls is nn.GELU and not isinstance(module_or_cls, type) and getattr(module_or_cls, 'approximate', 'none') == 'tanh':
        return 'gelu_tanh'
    return ACTIVATION_TO_NAME[cls]


def init_(p: torch.Tensor) -> torch.Tensor:
    """U(+-1/sqrt(size of last dim)), in place (reference: moe_layers.py:19-24)."""
    bound = 1.0 / math.sqrt(p.size(-1))
    with torch.no_grad():
        p.uniform_(-bound, bound)
    return p


class ExpertsLayer(nn.Module):
    pass


class _IntermediateStub(nn.Module):
    """Hook point for router training: dense first-layer activations [E,N,Ed] (reference: moe_layers.py:116-124)."""

    def forward(self, x, w1, b1, act):
        h = torch.einsum('eni,eio->eno', x, w1) + b1.unsqueeze(-2)
        return act(h)


class _OutputStub(nn.Module):
    """Hook point for router training: dense per-expert outputs [E,N,D] (reference: moe_layers.py:127-133)."""

    def forward(self, h, w2):
        return torch.einsum('eni,eio->eno', h, w2)


class _PackedCache:
    """Derived MFMA-ordered weight buffer, rebuilt when any source parameter changes (in-place version counter,
    storage pointer, device or dtype)."""

    def __init__(self):
        self.slots = {}   # with / without router section -> (key, buffer)

    def get(self, shape, tensors):
        key = tuple((t.data_ptr(), t._version, t.dtype, t.device) if t is not None else None for t in tensors)
        key = key + (shape.d_model, shape.n_experts, shape.expert_dim, shape.gated, shape.router_width,
                     shape.router_activation, shape.router_output_activation)
        slot = shape.router_width > 0
        cached = self.slots.get(slot)
        if cached is None or cached[0] != key:
            cached = (key, ops.pack_weights(shape, *tensors))
            self.slots[slot] = cached
        return cached[1]


def _grad_wanted(*tensors) -> bool:
    """True when autograd is on and one of the tensors asks for a gradient: the HIP kernels have no backward, so such a
    call has to be refused (the reference's kernel wrappers raise in backward, moe_impls.py:60-64)."""
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class _HipContainer(ExpertsLayer):
    """What every experts container of this package shares: the route to the HIP kernels.

    A container names its weights in the kernels' layout through ``hip_operands()`` ->
    ``(w1 [E,D,Ed], b1 [E,Ed] | None, w2 [E,Ed,D], w_up [E,D,Ed] | None, activation name)``; the derived MFMA-ordered
    buffer is cached on those tensors and rebuilt when one of them changes."""

    HIP_MODES = ('hip', 'triton', 'triton_atomic')

    def _init_hip(self):
        self.kernel_path = 'auto'
        self._packed = _PackedCache()

    def hip_operands(self):
        raise NotImplementedError

    def packed_weights(self, router_w1=None, router_w2=None, router_activation='relu', router_output_activation='abs'):
        w1, b1, w2, w_up, act = self.hip_operands()
        if not w1.is_cuda or w1.dtype not in (torch.bfloat16, torch.float32, torch.float16):
            return None
        sh = ops.make_shape(0, w1.size(1), w1.size(0), w1.size(2), router_w1.size(0) if router_w1 is not None else 0,
                            ops._dtype_code(w1), act, gated=w_up is not None, router_activation=router_activation,
                            router_output_activation=router_output_activation)
        return self._packed.get(sh, (w1, b1, w2, w_up, router_w1, router_w2))

    def forward_hip(self, x, routing_tensor, last_bias=None, add_residual=False):
        if not x.is_cuda:
            raise D2DMoEError("forward_mode 'hip' needs a ROCm device; use a PyTorch mode on the CPU")
        w1, b1, w2, w_up, act = self.hip_operands()
        if _grad_wanted(x, routing_tensor, w1, b1, w2, w_up, last_bias):
            # inference-only, like the reference's kernel wrappers (moe_impls.py:60-64)
            raise NotImplementedError("the HIP experts path has no backward; wrap the call in torch.no_grad()")
        return ops.experts(x.contiguous(), routing_tensor.contiguous(), w1, b1, w2, w_up, last_bias, act, add_residual,
                           self.kernel_path, self.packed_weights())


class HipKernelExperts(_HipContainer):
    """Two-layer experts with the first-layer bias only, run by the gfx950 HIP kernels.

    Drop-in for the reference's CustomKernelExperts (moe_layers.py:136-264): same constructor, same parameters
    ``w1 [E,D,Ed]``, ``b1 [E,Ed]``, ``w2 [E,Ed,D]``, same ``forward_mode`` property.  Modes:
      'masked'  dense PyTorch einsum over all experts, gate-weighted (reference forward_all); keeps the two stub
                submodules that router training hooks into
      'naive'   PyTorch per-expert loop (reference forward_naive); the CPU path
      'hip'     the HIP kernels; 'triton' and 'triton_atomic' are accepted as aliases so reference scripts that
                select the Triton kernels get this path
    """

    def __init__(self, dim, num_experts, depth=2, expert_dim=None, bias=True, activation=nn.GELU,
                 intermediate_gating=False):
        if intermediate_gating:
            raise NotImplementedError('use HipExecuteAllExperts for gated experts')
        super().__init__()
        assert depth == 2, 'only two-layer experts'
        assert bias == 'without_last', 'bias must be "without_last" (first-layer bias only)'
        self.activation_str = activation_name(activation)
        self.num_experts = num_experts
        self.depth = depth
        self.expert_dim = dim * 2 if expert_dim is None else expert_dim
        self.hidden_dim = dim
        self.bias_mode = bias
        self.w1 = init_(nn.Parameter(torch.empty(num_experts, dim, self.expert_dim)))
        self.b1 = init_(nn.Parameter(torch.empty(num_experts, self.expert_dim)))
        self.w2 = init_(nn.Parameter(torch.empty(num_experts, self.expert_dim, dim)))
        self.act = activation()
        self._forward_mode = 'masked'
        self._init_hip()
        self.intermediate_activation_extraction_stub = _IntermediateStub()
        self.output_activation_extraction_stub = _OutputStub()
        self._norms_packed = None   # (key, buffer) of the derived buffer output_norms() uses

    @property
    def forward_mode(self):
        return self._forward_mode

    @forward_mode.setter
    def forward_mode(self, value):
        self._forward_mode = value

    # -- derived buffers --------------------------------------------------------------------
    def hip_operands(self):
        return self.w1, self.b1, self.w2, None, self.activation_str

    def load_operands(self, w1, b1, w2, w_up=None):
        assert w_up is None
        with torch.no_grad():
            self.w1.copy_(w1)
            self.w2.copy_(w2)
            if b1 is not None:
                self.b1.copy_(b1)

    def output_norms(self, x):
        """L2 norm of every expert's output for every token, [E,N]: the router-training targets the reference reads off
        a forward hook on `output_activation_extraction_stub` in 'masked' mode (train_routers.py:49-86,
        utils.py:353-369).  On a ROCm device in bf16 or float16, with D a multiple of 256 up to 2048 and experts of at most
        64 neurons, one HIP kernel computes them without forming the [E,N,D] outputs; anything else (float32, other
        widths) takes the reference's own route through the stubs."""
        assert x.dim() == 2, f'{x.size()=}'
        if x.is_cuda and not (torch.is_grad_enabled() and (x.requires_grad or self.w1.requires_grad)):
            sh = ops.make_shape(0, self.hidden_dim, self.num_experts, self.expert_dim, 0, ops._dtype_code(x),
                                self.activation_str) if x.dtype in (torch.bfloat16, torch.float32, torch.float16) else None
            if sh is not None and x.dtype == self.w1.dtype:
                key = tuple((t.data_ptr(), t._version, t.dtype, t.device) for t in (self.w1, self.b1, self.w2))
                if self._norms_packed is None or self._norms_packed[0] != key:
                    self._norms_packed = (key, ops.pack_norms(sh, self.w1, self.b1, self.w2))
                if self._norms_packed[1] is not None:
                    return ops.expert_output_norms(x.contiguous(), self.w1, self.b1, self.w2, self.activation_str,
                                                   self._norms_packed[1])
        h = self.intermediate_activation_extraction_stub(x.unsqueeze(0), self.w1, self.b1, self.act)
        y = self.output_activation_extraction_stub(h, self.w2)
        return torch.linalg.vector_norm(y, ord=2, dim=-1)

    # -- forward ----------------------------------------------------------------------------
    def forward(self, x, routing_tensor):
        assert x.dim() == 2, f'{x.size()=}'
        mode = self._forward_mode
        if mode == 'masked':
            return self.forward_all(x, routing_tensor)
        if mode == 'naive':
            return self.forward_naive(x, routing_tensor)
        if mode in self.HIP_MODES:
            return self.forward_hip(x, routing_tensor)
        raise NotImplementedError(f'Unsupported forward_mode: {mode}')

    def forward_all(self, x, routing_tensor):
        h = self.intermediate_activation_extraction_stub(x.unsqueeze(0), self.w1, self.b1, self.act)
        y = self.output_activation_extraction_stub(h, self.w2)
        return torch.einsum('end,ne->nd', y, routing_tensor)

    def forward_naive(self, x, routing_tensor):
        out = torch.zeros_like(x)
        for e in range(self.num_experts):
            mask = routing_tensor[:, e] > 0.0
            out[mask] += self.act(x[mask] @ self.w1[e] + self.b1[e]) @ self.w2[e]
        return out

    # the reference exposes these two as static methods of the container (moe_layers.py:213-224, 241-249)
    @staticmethod
    def extract_indices(routing_tensor):
        if routing_tensor.is_cuda:
            _, _, s, u, c = ops.build_permutation(routing_tensor.contiguous(), reference_layout=True)
            return s, u, c
        r = routing_tensor.to(torch.int32)
        s = r.argsort(dim=0, descending=True, stable=True)
        return s, s.argsort(dim=0), r.sum(dim=0)

    @staticmethod
    def extract_indices_atomic(routing_tensor):
        s, _, c = HipKernelExperts.extract_indices(routing_tensor)
        return s, c


class _ExecuteAllLayer(nn.Module):
    """One batched expert layer, parameters ``w [E,in,out]`` and optional ``b [E,1,out]``
    (reference: moe_layers.py:32-47)."""

    def __init__(self, in_dim, out_dim, num_experts, bias, activation):
        super().__init__()
        self.bias = bias
        self.w = init_(nn.Parameter(torch.empty(num_experts, in_dim, out_dim)))
        if self.bias:
            self.b = init_(nn.Parameter(torch.empty(num_experts, 1, out_dim)))
        self.act = activation()

    def forward(self, x):
        x = torch.einsum('eni,eio->eno', x, self.w)
        if self.bias:
            x = x + self.b
        return self.act(x)


class HipExecuteAllExperts(_HipContainer):
    """Depth-2 experts, optionally with LLaMA/Gemma-style intermediate gating, parameters named as the reference's
    ExecuteAllExperts (moe_layers.py:50-101): ``layers.0.w`` first/gate projection, ``layers.1.w`` down projection,
    ``layers.2.w`` up projection (gated only).  ``forward_mode`` 'masked' is the reference's dense einsum; 'hip'
    runs the HIP kernels, skipping experts that are not routed to."""

    def __init__(self, dim, num_experts, depth=2, expert_dim=None, bias=True, activation=nn.GELU,
                 intermediate_gating=False):
        super().__init__()
        assert depth == 2, 'only two-layer experts'
        self.num_experts = num_experts
        self.depth = depth
        self.dim = dim
        self.expert_dim = dim * 2 if expert_dim is None else expert_dim
        self.bias_mode = bias
        self.activation = activation
        self.intermediate_gating = intermediate_gating
        first_bias = True if bias == 'without_last' else bias
        last_bias = False if bias == 'without_last' else bias
        self.layers = nn.ModuleList()
        if intermediate_gating:
            self.layers.append(_ExecuteAllLayer(dim, self.expert_dim, num_experts, first_bias, activation))
            self.layers.append(_ExecuteAllLayer(self.expert_dim, dim, num_experts, first_bias, nn.Identity))
            self.layers.append(_ExecuteAllLayer(dim, self.expert_dim, num_experts, first_bias, nn.Identity))
        else:
            self.layers.append(_ExecuteAllLayer(dim, self.expert_dim, num_experts, first_bias, activation))
            self.layers.append(_ExecuteAllLayer(self.expert_dim, dim, num_experts, last_bias, nn.Identity))
        self.forward_mode = 'masked'
        self._init_hip()

    def hip_operands(self):
        if self.layers[1].bias or (self.intermediate_gating and self.layers[0].bias):
            raise NotImplementedError('the HIP path covers first-layer bias (ungated) or no bias (gated)')
        b1 = self.layers[0].b.squeeze(1) if self.layers[0].bias else None   # a view: shares storage and version counter
        w_up = self.layers[2].w if self.intermediate_gating else None
        return self.layers[0].w, b1, self.layers[1].w, w_up, activation_name(self.layers[0].act)

    def load_operands(self, w1, b1, w2, w_up=None):
        """Fills the parameters from kernel-layout tensors (what the reference's param_clustering_split writes entry by
        entry, moefication.py:253-271)."""
        assert (w_up is not None) == self.intermediate_gating
        with torch.no_grad():
            self.layers[0].w.copy_(w1)
            self.layers[1].w.copy_(w2)
            if b1 is not None:
                self.layers[0].b.copy_(b1.unsqueeze(1))
            if w_up is not None:
                self.layers[2].w.copy_(w_up)

    def forward(self, x, routing_tensor):
        assert x.dim() == 2, f'{x.size()=}'
        if self.forward_mode in self.HIP_MODES:
            return self.forward_hip(x, routing_tensor)
        x = x.unsqueeze(0)
        if self.intermediate_gating:
            x = self.layers[1](self.layers[0](x) * self.layers[2](x))
        else:
            for layer in self.layers:
                x = layer(x)
        return torch.einsum('end,ne->nd', x, routing_tensor)


class _GLUExpert(nn.Module):
    """One gated expert as a module (reference: moe_layers.py:104-113; same submodule names)."""

    def __init__(self, d_model, d_intermediate, activation, bias, last_bias):
        super().__init__()
        self.gate = nn.Linear(d_model, d_intermediate, bias=bias)
        self.up_scale = nn.Linear(d_model, d_intermediate, bias=bias)
        self.activation = activation()
        self.down_scale = nn.Linear(d_intermediate, d_model, bias=last_bias)

    def forward(self, x):
        return self.down_scale(self.activation(self.gate(x)) * self.up_scale(x))


def _loop_over_experts(x, routing_tensor, num_experts, expert_fn):
    """The reference's per-expert loop of its module containers (moe_layers.py:311-326, 385-399): every expert runs on the
    rows routed to it and its output is scaled by the routing value.  (The reference first asserts that x holds no NaN,
    which costs a host synchronisation per call; that check is left out.)"""
    outputs = torch.zeros_like(x)
    for i in range(num_experts):
        col = routing_tensor[:, i]
        mask = col != 0.0
        outputs[mask] += expert_fn(x[mask], i) * col[mask].unsqueeze(1)
    return outputs


class _StackedOperands:
    """Kernel-layout copies ([E,D,Ed] / [E,Ed] / [E,Ed,D]) of weights a container keeps per expert, rebuilt when one of the
    source parameters changes (storage pointer or in-place version counter)."""

    def __init__(self):
        self.key = None
        self.value = None

    def get(self, sources, build):
        key = tuple((t.data_ptr(), t._version, t.dtype, t.device) for t in sources)
        if key != self.key:
            with torch.no_grad():
                self.value = build()
            self.key = key
        return self.value


class HipModuleBatchedExperts(_HipContainer):
    """Experts kept as one small module each, with the reference's ModuleBatchedExperts names (moe_layers.py:267-326):
    ``e.<i>.0`` / ``e.<i>.2`` Linear layers (``e.<i>.gate`` / ``up_scale`` / ``down_scale`` for gated experts), so its
    state_dicts load unchanged.  ``forward_mode`` 'naive' (the default) is the reference's per-expert loop; 'hip' runs the
    HIP kernels on stacked copies of the weights (inference only)."""

    def __init__(self, dim, num_experts, depth=2, expert_dim=None, bias=True, activation=nn.GELU,
                 intermediate_gating=False):
        super().__init__()
        assert depth == 2, 'only two-layer experts'
        self.num_experts = num_experts
        self.depth = depth
        self.expert_dim = dim * 2 if expert_dim is None else expert_dim
        self.bias_mode = bias
        self.intermediate_gating = intermediate_gating
        first_bias = True if bias == 'without_last' else bias
        last_bias = False if bias == 'without_last' else bias
        self.e = nn.ModuleList()
        for _ in range(num_experts):
            if intermediate_gating:
                self.e.append(_GLUExpert(dim, self.expert_dim, activation, bool(bias), bool(last_bias)))
            else:
                self.e.append(nn.Sequential(nn.Linear(dim, self.expert_dim, bias=first_bias), activation(),
                                            nn.Linear(self.expert_dim, dim, bias=last_bias)))
        self.forward_mode = 'naive'
        self._init_hip()
        self._stacked = _StackedOperands()

    def hip_operands(self):
        if self.intermediate_gating:
            first = [m.gate for m in self.e]
            up = [m.up_scale for m in self.e]
            last = [m.down_scale for m in self.e]
            act = activation_name(self.e[0].activation)
            if first[0].bias is not None:
                raise NotImplementedError('the HIP path covers gated experts without biases')
        else:
            first = [m[0] for m in self.e]
            up = None
            last = [m[2] for m in self.e]
            act = activation_name(self.e[0][1])
        if last[0].bias is not None:
            raise NotImplementedError('the HIP path has no per-expert output bias')
        sources = [l.weight for l in first] + [l.weight for l in last]
        sources += [l.bias for l in first if l.bias is not None] + ([l.weight for l in up] if up else [])

        def build():
            w1 = torch.stack([l.weight.t() for l in first]).contiguous()
            b1 = torch.stack([l.bias for l in first]).contiguous() if first[0].bias is not None else None
            w2 = torch.stack([l.weight.t() for l in last]).contiguous()
            w_up = torch.stack([l.weight.t() for l in up]).contiguous() if up else None
            return w1, b1, w2, w_up

        return (*self._stacked.get(sources, build), act)

    def load_operands(self, w1, b1, w2, w_up=None):
        assert (w_up is not None) == self.intermediate_gating
        with torch.no_grad():
            for i, m in enumerate(self.e):
                first, last = (m.gate, m.down_scale) if self.intermediate_gating else (m[0], m[2])
                first.weight.copy_(w1[i].t())
                last.weight.copy_(w2[i].t())
                if b1 is not None:
                    first.bias.copy_(b1[i])
                if w_up is not None:
                    m.up_scale.weight.copy_(w_up[i].t())

    def forward(self, x, routing_tensor):
        assert x.dim() == 2, f'{x.size()=}'
        if self.forward_mode in self.HIP_MODES:
            return self.forward_hip(x, routing_tensor)
        return _loop_over_experts(x, routing_tensor, self.num_experts, lambda rows, i: self.e[i](rows))


class HipBatchedExperts(_HipContainer):
    """Experts kept as stacked tensors in parameter lists, with the reference's BatchedExperts names
    (moe_layers.py:329-399): ``weights.0 [E,D,Ed]``, ``weights.1 [E,Ed,D]``, ``biases.<i> [E,1,*]``.  As there, the list
    of biases under bias='without_last' also holds an (unused) entry for the last layer.  ``forward_mode`` 'naive' (the
    default) is the reference's per-expert loop; 'hip' runs the HIP kernels (inference only)."""

    def __init__(self, dim, num_experts, depth=2, expert_dim=None, bias=True, activation=nn.GELU,
                 intermediate_gating=False):
        super().__init__()
        assert depth == 2, 'only two-layer experts'
        if intermediate_gating:
            raise NotImplementedError()
        self.num_experts = num_experts
        self.depth = depth
        self.expert_dim = dim * 2 if expert_dim is None else expert_dim
        self.bias_mode = bias
        has_bias = True if bias == 'without_last' else bias
        self.weights = nn.ParameterList([init_(nn.Parameter(torch.empty(num_experts, dim, self.expert_dim))),
                                         init_(nn.Parameter(torch.empty(num_experts, self.expert_dim, dim)))])
        if has_bias:
            self.biases = nn.ParameterList([nn.Parameter(torch.zeros(num_experts, 1, self.expert_dim)),
                                            nn.Parameter(torch.zeros(num_experts, 1, dim))])
        self.act = activation()
        self.forward_mode = 'naive'
        self._init_hip()

    def expert_forward(self, x, expert_index):
        if self.bias_mode is True:
            x = self.act(x @ self.weights[0][expert_index] + self.biases[0][expert_index])
            return x @ self.weights[1][expert_index] + self.biases[1][expert_index]
        if self.bias_mode == 'without_last':
            x = self.act(x @ self.weights[0][expert_index] + self.biases[0][expert_index])
            return x @ self.weights[1][expert_index]
        return self.act(x @ self.weights[0][expert_index]) @ self.weights[1][expert_index]

    def hip_operands(self):
        if self.bias_mode is True:
            raise NotImplementedError('the HIP path has no per-expert output bias')
        b1 = self.biases[0].squeeze(1) if self.bias_mode == 'without_last' else None
        return self.weights[0], b1, self.weights[1], None, activation_name(self.act)

    def load_operands(self, w1, b1, w2, w_up=None):
        assert w_up is None
        with torch.no_grad():
            self.weights[0].copy_(w1)
            self.weights[1].copy_(w2)
            if b1 is not None:
                self.biases[0].copy_(b1.unsqueeze(1))

    def forward(self, x, routing_tensor):
        assert x.dim() == 2, f'{x.size()=}'
        if self.forward_mode in self.HIP_MODES:
            return self.forward_hip(x, routing_tensor)
        return _loop_over_experts(x, routing_tensor, self.num_experts, self.expert_forward)


MOE_IMPL_MAP = {
    'hip_kernel': HipKernelExperts,
    'custom_kernel': HipKernelExperts,     # the reference's name for its Triton-backed container
    'hip_execute_all': HipExecuteAllExperts,
    'execute_all': HipExecuteAllExperts,   # the reference's dense container (the one its Gemma runs use)
    'module': HipModuleBatchedExperts,     # one module per expert (the reference's default experts_class)
    'batched': HipBatchedExperts,          # stacked tensors in parameter lists
}
