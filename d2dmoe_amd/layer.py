"""The dynamic-k MoE layer and its router, with the reference's module interface
(architectures/moe/moefication.py:28-101 and :309-354), backed by the gfx950 HIP kernels.

``MoeficationMoE.forward(x[B,T,D]) -> (out[B,T,D], {name: (routing_tensor[B,T,E],)})``; the attributes
``forward_mode`` ('all' | 'topk' | 'dynk' | 'dynk_max'), ``tau``, ``k``, ``router``, ``experts``, ``last_bias``,
``add_residual_connection`` keep their meaning.  ``tau`` keeps the reference's convention: an expert is kept when
``norm >= max_norm * (1.0 - tau)``.

When ``forward_mode == 'dynk_max'``, the input is on a ROCm device and the experts container is in its 'hip' mode,
the whole layer (router MLP, selection, experts, bias/residual epilogue) runs as one d2dmoe_forward call without any
host synchronisation.  Every other combination is composed from the same parts in PyTorch, as the reference does.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
from torch import nn

from . import ops
from .experts import MOE_IMPL_MAP, _HipContainer, _grad_wanted
from .hip_abi import ACT


class _Abs(nn.Module):
    def forward(self, x):
        return torch.abs(x)


# name -> module class (reference: common.py:159-169)
ACTIVATION_NAME_MAP = {
    'relu': nn.ReLU,
    'gelu': nn.GELU,
    'sigmoid': nn.Sigmoid,
    'tanh': nn.Tanh,
    'leaky_relu': nn.LeakyReLU,
    'softplus': nn.Softplus,
    'silu': nn.SiLU,
    'abs': _Abs,
    'identity': nn.Identity,
}


class _CallCache:
    """Holder of a layer's prepared library call.  It is derived state: copies and pickles of the layer start empty."""
    __slots__ = ('entry',)

    def __init__(self):
        self.entry = None

    def __deepcopy__(self, memo):
        return _CallCache()

    def __reduce__(self):
        return (_CallCache, ())


class MoELayer(nn.Module):
    def __init__(self, name, num_experts):
        super().__init__()
        self.name = name
        self.num_experts = num_experts


class MoeficationRouter(nn.Module):
    """MLP predicting per-expert output norms (reference: moefication.py:309-339).  ``layers`` holds
    Linear / activation modules in the reference's order, so ``router.layers.0.weight`` etc. load unchanged."""

    def __init__(self, hidden_dim, num_experts, width=128, depth=2, bias=False, activation='tanh',
                 output_activation='identity', test_override_outputs_p=None):
        super().__init__()
        self.layers = nn.ModuleList()
        if depth == 1:
            self.layers.append(nn.Linear(hidden_dim, num_experts, bias=bias))
        else:
            self.layers.append(nn.Linear(hidden_dim, width, bias=bias))
            self.layers.append(ACTIVATION_NAME_MAP[activation]())
            for _ in range(depth - 2):
                self.layers.append(nn.Linear(width, width, bias=bias))
                self.layers.append(ACTIVATION_NAME_MAP[activation]())
            self.layers.append(nn.Linear(width, num_experts, bias=bias))
        self.layers.append(ACTIVATION_NAME_MAP[output_activation]())
        self.depth = depth
        self.activation = activation
        self.output_activation = output_activation
        self.test_override_outputs_p = test_override_outputs_p
        if test_override_outputs_p is not None:
            self.response_cache = {}

    def hip_compatible(self) -> bool:
        """True when d2dmoe_router covers this router: depth 2, no biases, activations known to the kernels."""
        return (self.depth == 2 and self.layers[0].bias is None and self.layers[2].bias is None
                and self.activation in ACT and self.output_activation in ACT)

    def forward(self, x):
        if (x.is_cuda and not torch.is_grad_enabled() and self.hip_compatible()
                and x.dtype in (torch.float32, torch.bfloat16, torch.float16)):
            lead = x.shape[:-1]
            x = ops.router(x.reshape(-1, x.size(-1)).contiguous(), self.layers[0].weight, self.layers[2].weight,
                           self.activation, self.output_activation).view(*lead, -1)
        else:
            for layer in self.layers:
                x = layer(x)
        if self.test_override_outputs_p is not None:
            # test hook: replace the outputs by Bernoulli draws, cached per (batch, sequence) shape
            key = (x.size(0), x.size(1))
            if key in self.response_cache:
                x = self.response_cache[key]
            else:
                with torch.no_grad():
                    x.bernoulli_(self.test_override_outputs_p)
                    self.response_cache[key] = x
        return x


class MoeficationMoE(MoELayer):
    def __init__(self, name, hidden_dim, num_experts, bias, expert_dim, activation, experts_class='hip_kernel',
                 add_residual_connection=False, add_intermediate_gating=False):
        super().__init__(name, num_experts)
        self.hidden_dim = hidden_dim
        self.expert_dim = expert_dim
        self.num_experts = num_experts
        self.bias = bias
        self.experts = MOE_IMPL_MAP[experts_class](dim=hidden_dim,
                                                   num_experts=num_experts,
                                                   depth=2,
                                                   expert_dim=expert_dim,
                                                   bias=False if not bias else 'without_last',
                                                   activation=activation,
                                                   intermediate_gating=add_intermediate_gating)
        if self.bias:
            self.last_bias = nn.Parameter(torch.zeros(1, hidden_dim))
        self.forward_mode = 'all'
        self.router: Optional[MoeficationRouter] = None
        self.k = None
        self.tau = None
        self.add_residual_connection = add_residual_connection
        # Cost accounting (the reference sums (routing > 0) over the dense routing tensor on the host side of every
        # batch, eval.py:176-177): with collect_counts set, the fused HIP call also returns the per-expert number of
        # routed tokens from its own device-side counters; it stays on the device, nothing synchronises.
        self.collect_counts = False
        self._prepared = _CallCache()   # (key, ops.PreparedForward) of the fused call
        self.last_expert_counts: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------------------ gating
    def gate(self, x):
        mode = self.forward_mode
        if mode == 'all':
            return torch.ones(x.size(0), x.size(1), self.num_experts, dtype=x.dtype, device=x.device)
        if mode == 'topk':
            scores = self.router(x)
            top = torch.topk(scores, k=self.k, dim=-1)[1]
            return torch.zeros_like(scores).scatter_(2, top, 1.0)
        if mode == 'dynk':
            norms = self.router(x)
            shares = norms / norms.sum(dim=-1, keepdim=True)
            sorted_shares, order = torch.sort(shares, dim=-1, descending=True)
            keep = torch.cumsum(sorted_shares, dim=-1) < self.tau
            keep = keep.roll(shifts=1, dims=-1)
            keep[..., 0] = True   # the expert that crosses the threshold is kept too; at least one expert runs
            return keep.gather(dim=-1, index=order.argsort(dim=-1)).to(x.dtype)
        if mode == 'dynk_max':
            norms = self.router(x)
            if norms.is_cuda and norms.dtype in (torch.float32, torch.bfloat16, torch.float16):
                routing, _ = ops.select(norms.reshape(-1, norms.size(-1)).contiguous(), float(1.0 - self.tau))
                return routing.view(norms.shape)
            max_norms, _ = norms.max(dim=-1, keepdim=True)
            thresholds = max_norms * (1.0 - self.tau)
            routing = torch.zeros_like(norms)
            routing[norms >= thresholds] = 1.0
            return routing
        raise ValueError(f'Unsupported forward_mode: {mode}')

    # ------------------------------------------------------------------------------ forward
    def _fused_ok(self, x) -> bool:
        """True when the whole layer can run as one d2dmoe_forward call.  Raises, as the experts containers do, when that
        call would be taken under autograd with a tensor that asks for a gradient: the kernels have no backward
        (the reference's wrappers raise there too, moe_impls.py:60-64), and an output silently cut off from the graph
        would leave the parameters without gradients."""
        if self.forward_mode != 'dynk_max' or not x.is_cuda or x.dtype not in (torch.float32, torch.bfloat16, torch.float16):
            return False
        ex = self.experts
        if not isinstance(ex, _HipContainer) or ex.forward_mode not in ex.HIP_MODES:
            return False
        if self.router is None or not (self.router.test_override_outputs_p is not None or self.router.hip_compatible()):
            return False
        if torch.is_grad_enabled() and _grad_wanted(x, *self.parameters()):
            raise NotImplementedError(f"MoE layer {getattr(self, 'name', None)!r}: the HIP layer path has no backward; wrap the "
                                      "call in torch.no_grad() / torch.inference_mode() or call requires_grad_(False) on "
                                      "the layer, or switch the experts to a PyTorch forward_mode for training")
        return True

    def _router_operands(self):
        """(router_w1, router_w2, hidden activation, output activation) as the fused HIP call takes them; the weights are
        None when the router's outputs are overridden (test hook) and the norms are passed in instead."""
        router = self.router
        if router.test_override_outputs_p is not None:
            rw1 = rw2 = None
        else:
            rw1, rw2 = router.layers[0].weight, router.layers[2].weight
        ract = router.activation if router.activation in ACT else 'relu'
        roact = router.output_activation if router.output_activation in ACT else 'abs'
        return rw1, rw2, ract, roact

    def packed_weights(self):
        """The derived, MFMA-ordered weight buffer the fused forward of this layer uses (built on first use, rebuilt when
        a parameter changes); None where no MFMA kernel applies.  Calling it ahead of time moves the packing out of the
        first forward."""
        if not isinstance(self.experts, _HipContainer) or self.router is None or not self.router.hip_compatible():
            return None
        return self.experts.packed_weights(*self._router_operands())

    def _prepared_forward(self, x):
        """The layer's ops.PreparedForward, rebuilt when a parameter was replaced or updated in place, the dtype or device
        changed, or a setting it bakes in did (residual, bias, router override)."""
        ex = self.experts
        rw1, rw2, ract, roact = self._router_operands()
        w1, b1, w2, w_up, act = ex.hip_operands()
        last_bias = self.last_bias if self.bias else None
        sources = (rw1, rw2, w1, b1, w2, w_up, last_bias)
        key = tuple((t.data_ptr(), t._version) if t is not None else None for t in sources) + \
            (x.dtype, x.device, act, ract, roact, self.add_residual_connection)
        cached = self._prepared.entry
        if cached is None or cached[0] != key:
            prepared = ops.PreparedForward(self.hidden_dim, x.dtype, rw1, rw2, w1, b1, w2, w_up,
                                           last_bias.view(-1) if last_bias is not None else None, act,
                                           self.add_residual_connection, ex.packed_weights(rw1, rw2, ract, roact), ract, roact)
            cached = self._prepared.entry = (key, prepared)
        return cached[1]

    def forward(self, x):
        orig_size = x.size()
        if self._fused_ok(x):
            x2 = x.reshape(-1, orig_size[-1]).contiguous()
            router = self.router
            norms_in = None
            if router.test_override_outputs_p is not None:
                norms_in = router(x).reshape(-1, self.num_experts).contiguous()
            out, routing, _, counts = self._prepared_forward(x)(x2, float(1.0 - self.tau), norms_in,
                                                                want_counts=self.collect_counts,
                                                                path=self.experts.kernel_path)
            routing_tensor = routing.view(*orig_size[:-1], self.num_experts)
            self.last_expert_counts = counts
            return out.view(orig_size), {self.name: (routing_tensor,)}
        routing_tensor = self.gate(x)
        x2 = x.reshape(-1, x.size(-1))
        out = self.experts(x2, routing_tensor.view(-1, routing_tensor.size(-1)))
        if self.bias:
            out = out + self.last_bias
        if self.add_residual_connection:
            out = out + x2
        return out.view(orig_size), {self.name: (routing_tensor,)}


def add_routers(model: nn.Module, router_args: Dict) -> Dict[str, MoeficationMoE]:
    """Attaches a fresh router to every MoE layer of `model` (reference: moefication.py:342-354)."""
    found = {}
    for name, module in model.named_modules():
        if isinstance(module, MoeficationMoE):
            module.router = MoeficationRouter(module.hidden_dim, module.num_experts, **router_args)
            found[name] = module
    assert len(found) > 0
    return found
