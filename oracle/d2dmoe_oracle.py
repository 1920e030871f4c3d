"""CPU oracle for the dynamic-k MoE-FFN forward path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain PyTorch CPU ops, the algorithm of the reference's MoE forward path.
It is the checker that the HIP kernels are compared against; nothing in the product package may
import it (only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do).

Every function names the reference lines it follows (paths relative to the reference checkout).

How each function is pinned (the reference ships no golden vectors for this path, so the pins are
mathematical; they live in tests/test_oracle_pins.py):

  router_forward        pinned: float64 recomputation with numpy matmul; abs/relu closed forms
  gate_dynk_max         pinned: python brute force on small inputs; tau=1 -> all ones; all-zero row ->
                        all ones; arg-max always kept; NaN row -> zeros; monotone in tau
  gate_all / gate_topk  pinned: closed forms (ones; exactly k ones on the k largest, brute force)
  gate_dynk             pinned: brute-force loop (sort shares, accumulate until share >= tau)
  extract_indices       pinned: nonzero()-based construction, inverse(perm) == id, counts == column sums,
                        equality with torch.argsort(stable=True, descending=True), set equality with
                        the unstable argsort the reference calls
  experts_forward_all   pinned: per-token brute force in numpy float64; all-ones routing reduces to a dense
                        FFN through two library GEMMs; all-zero routing -> zeros; one-hot -> one small MLP
  experts_forward_naive pinned: equals experts_forward_all for 0/1 routing (fp64), same special cases
  experts_first_layer / experts_second_merge
                        pinned: composition equals experts_forward_all on 0/1 routing
  gated variants        pinned: same three formulations with act(gate) * up
  moe_layer_forward     pinned: composition of the above + bias/residual closed form
  expert_output_norms   pinned: per-(token, expert) brute force in numpy float64; the Gram identity
                        |h W2|^2 = h (W2 W2^T) h^T; zero second layer -> zeros; one expert, identity
                        activation -> |x A| for the product matrix A through a library GEMM
  activations           pinned: torch.nn.functional counterparts / closed forms in float64

No function is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional, Tuple

import torch
import torch.nn.functional as F

# --------------------------------------------------------------------------------------------
# activations  (reference: utils.py:730-756 for the kernel-side definitions,
#               common.py:159-169 for the name -> torch module map)
# --------------------------------------------------------------------------------------------


def act_relu(x):
    return F.relu(x)


def act_leaky_relu(x):
    # utils.py:735-737: slope 0.01 (also nn.LeakyReLU's default)
    return F.leaky_relu(x, 0.01)


def act_tanh(x):
    # utils.py:740-743 writes tanh as 2*sigmoid(2x)-1; mathematically identical to tanh
    return torch.tanh(x)


def act_gelu(x):
    # utils.py:754-756: x * 0.5 * (1 + erf(x / sqrt(2)))  == nn.GELU() (erf form)
    return F.gelu(x)


def act_gelu_tanh(x):
    # utils.py:749-751 (gelu_approx); the activation of stock Gemma MLPs
    return F.gelu(x, approximate='tanh')


def act_silu(x):
    return F.silu(x)


def act_identity(x):
    return x


def act_abs(x):
    return torch.abs(x)


ACTIVATIONS: Dict[str, Callable[[torch.Tensor], torch.Tensor]] = {
    'relu': act_relu,
    'gelu': act_gelu,
    'tanh': act_tanh,
    'leaky_relu': act_leaky_relu,
    'gelu_tanh': act_gelu_tanh,
    'silu': act_silu,
    'identity': act_identity,
    'abs': act_abs,
}

# --------------------------------------------------------------------------------------------
# parameter creation (reference: moe_layers.py:19-24, 157-159; moefication.py:313-323)
# --------------------------------------------------------------------------------------------


def make_layer_params(d_model: int, n_experts: int, expert_dim: int, router_width: int,
                      seed: int, gated: bool = False, bias: bool = True,
                      dtype: torch.dtype = torch.float32) -> Dict[str, torch.Tensor]:
    """Seeded weights in the reference's creation order.

    Experts: w1 [E,D,Ed], b1 [E,Ed], w2 [E,Ed,D] each through init_ (moe_layers.py:157-159);
    gated experts: gate [E,D,Ed], down [E,Ed,D], up [E,D,Ed] (moe_layers.py:71-78: layer 0 is the gate,
    1 the output, 2 the up-projection).  last_bias zeros [1,D] (moefication.py:46-47).
    Router: two bias-free nn.Linear layers, default init = U(+-1/sqrt(fan_in)) (moefication.py:313-323).
    """
    g = torch.Generator().manual_seed(seed)

    def uni(*shape, fan):
        b = 1.0 / math.sqrt(fan)
        return (torch.rand(*shape, generator=g) * 2 - 1) * b

    p: Dict[str, torch.Tensor] = {}
    if gated:
        p['w_gate'] = uni(n_experts, d_model, expert_dim, fan=expert_dim)
        p['w_down'] = uni(n_experts, expert_dim, d_model, fan=d_model)
        p['w_up'] = uni(n_experts, d_model, expert_dim, fan=expert_dim)
    else:
        p['w1'] = uni(n_experts, d_model, expert_dim, fan=expert_dim)
        if bias:
            p['b1'] = uni(n_experts, expert_dim, fan=expert_dim)
        p['w2'] = uni(n_experts, expert_dim, d_model, fan=d_model)
    if bias:
        p['last_bias'] = torch.zeros(1, d_model)
    p['router_w1'] = uni(router_width, d_model, fan=d_model)
    p['router_w2'] = uni(n_experts, router_width, fan=router_width)
    return {k: v.to(dtype) for k, v in p.items()}


# --------------------------------------------------------------------------------------------
# router (reference: moefication.py:309-339)
# --------------------------------------------------------------------------------------------


def router_forward(x: torch.Tensor, router_w1: torch.Tensor, router_w2: torch.Tensor,
                   activation: str = 'relu', output_activation: str = 'abs') -> torch.Tensor:
    """Depth-2 bias-free router: out_act(act(x W1^T) W2^T)  (moefication.py:313-323, 328-330).

    x [..., D], router_w1 [W, D], router_w2 [E, W] (nn.Linear stores [out, in]).  Each F.linear
    rounds its result to x.dtype, as the reference's eager nn.Linear does.
    """
    h = ACTIVATIONS[activation](F.linear(x, router_w1))
    return ACTIVATIONS[output_activation](F.linear(h, router_w2))


# --------------------------------------------------------------------------------------------
# gating (reference: moefication.py:54-88)
# --------------------------------------------------------------------------------------------


def gate_all(x: torch.Tensor, n_experts: int) -> torch.Tensor:
    # moefication.py:56-58
    return torch.ones(*x.shape[:-1], n_experts, dtype=x.dtype)


def gate_topk(scores: torch.Tensor, k: int) -> torch.Tensor:
    # moefication.py:59-63
    top = torch.topk(scores, k=k, dim=-1)[1]
    routing = torch.zeros_like(scores)
    routing.scatter_(-1, top, 1.0)
    return routing


def gate_dynk(norms: torch.Tensor, tau: float) -> torch.Tensor:
    # moefication.py:64-79: keep the largest-share experts until their cumulative share crosses tau
    total = norms.sum(dim=-1, keepdim=True)
    shares = norms / total
    sorted_shares, order = torch.sort(shares, dim=-1, descending=True)
    cum = torch.cumsum(sorted_shares, dim=-1)
    keep_sorted = cum < tau
    keep_sorted = keep_sorted.roll(shifts=1, dims=-1)
    keep_sorted[..., 0] = True
    return keep_sorted.gather(dim=-1, index=order.argsort(dim=-1)).to(norms.dtype)


def gate_dynk_max(norms: torch.Tensor, tau: float) -> torch.Tensor:
    """Keep expert e iff norms[e] >= max_e(norms) * (1.0 - tau)   (moefication.py:80-85).

    The product is taken as the reference takes it: tensor (in its own dtype) times the python float
    (1.0 - tau); the result is rounded to the tensor's dtype before the comparison.
    """
    max_norms, _ = norms.max(dim=-1, keepdim=True)
    thresholds = max_norms * (1.0 - tau)
    routing = torch.zeros_like(norms)
    routing[norms >= thresholds] = 1.0
    return routing


def gate_dynk_max_scaled(norms: torch.Tensor, thr_scale: float) -> torch.Tensor:
    """Same rule with the multiplier given directly (thr_scale plays the role of 1.0 - tau)."""
    max_norms, _ = norms.max(dim=-1, keepdim=True)
    thresholds = max_norms * thr_scale
    routing = torch.zeros_like(norms)
    routing[norms >= thresholds] = 1.0
    return routing


# --------------------------------------------------------------------------------------------
# token -> expert permutation (reference: moe_layers.py:213-224, 241-249)
# --------------------------------------------------------------------------------------------


def extract_indices(routing: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Canonical form of the reference's extract_indices.

    The reference sorts each expert column of routing.to(int32) in descending order with an UNSTABLE
    argsort; only the set held by the first expert_bincounts[e] rows of column e is defined by it
    (that prefix is all its kernels read: moe_impls.py:124-133, 270-293).  The canonical permutation
    fixes the order as the stable one: active tokens ascending, then inactive tokens ascending.

    Returns (sort_indices [N,E] int64, unsort_indices [N,E] int64, expert_bincounts [E] int64), where
    unsort_indices is the per-column inverse permutation (moe_layers.py:223).
    """
    r = routing.to(torch.int32)
    sort_indices = torch.argsort(r, dim=0, descending=True, stable=True)
    expert_bincounts = r.sum(dim=0).to(torch.int64)
    unsort_indices = torch.argsort(sort_indices, dim=0, stable=True)
    return sort_indices, unsort_indices, expert_bincounts


def permutation_csr(routing: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Compact form of the same permutation: offsets [E+1] int32 (exclusive prefix sum of the counts) and
    token_idx [P] int32 = for each expert in ascending order, its active tokens in ascending order."""
    active = routing > 0
    counts = active.sum(dim=0)
    offsets = torch.zeros(routing.size(1) + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
    # nonzero on the transposed mask lists (expert, token) pairs in expert-major, token-ascending order
    token_idx = active.t().nonzero()[:, 1].to(torch.int32)
    return offsets, token_idx


# --------------------------------------------------------------------------------------------
# experts (reference: moe_layers.py:116-133, 193-211; moe_impls.py:124-180, 485-514)
# --------------------------------------------------------------------------------------------


def experts_forward_all(x: torch.Tensor, routing: torch.Tensor, w1: torch.Tensor,
                        b1: Optional[torch.Tensor], w2: torch.Tensor, activation: str = 'relu') -> torch.Tensor:
    """Dense 'masked' formulation, gate-weighted  (moe_layers.py:193-198, stubs :116-133).

    x [N,D], routing [N,E], w1 [E,D,Ed], b1 [E,Ed] or None, w2 [E,Ed,D] -> [N,D].
    """
    h = torch.einsum('eni,eio->eno', x.unsqueeze(0).expand(w1.size(0), -1, -1), w1)
    if b1 is not None:
        h = h + b1.unsqueeze(-2)
    h = ACTIVATIONS[activation](h)
    y = torch.einsum('eni,eio->eno', h, w2)
    return torch.einsum('end,ne->nd', y, routing)


def expert_output_norms(x: torch.Tensor, w1: torch.Tensor, b1: Optional[torch.Tensor], w2: torch.Tensor,
                        activation: str = 'relu') -> torch.Tensor:
    """L2 norm of every expert's output for every token: the regression targets of router training.

    The reference runs the layer in 'masked' mode, captures the output of
    `output_activation_extraction_stub` ([E,N,D], moe_layers.py:125-133, 193-198) with a forward hook and takes
    `torch.linalg.vector_norm(output, ord=2, dim=-1)` (utils.py:353-369, train_routers.py:49-86).
    x [N,D], w1 [E,D,Ed], b1 [E,Ed] or None, w2 [E,Ed,D] -> [E,N].
    """
    h = torch.einsum('eni,eio->eno', x.unsqueeze(0).expand(w1.size(0), -1, -1), w1)
    if b1 is not None:
        h = h + b1.unsqueeze(-2)
    h = ACTIVATIONS[activation](h)
    y = torch.einsum('eni,eio->eno', h, w2)
    return torch.linalg.vector_norm(y, ord=2, dim=-1)


def experts_forward_naive(x: torch.Tensor, routing: torch.Tensor, w1: torch.Tensor,
                          b1: Optional[torch.Tensor], w2: torch.Tensor, activation: str = 'relu') -> torch.Tensor:
    """Per-expert boolean-mask loop, unweighted  (moe_layers.py:200-211).  The reference's CPU path."""
    act = ACTIVATIONS[activation]
    out = torch.zeros_like(x)
    for e in range(w1.size(0)):
        mask = routing[:, e] > 0.0
        xe = x[mask]
        he = xe @ w1[e]
        if b1 is not None:
            he = he + b1[e]
        out[mask] += act(he) @ w2[e]
    return out


def experts_first_layer(x, sort_indices, expert_bincounts, w1, b1, activation='relu'):
    """inter[e, j, :] = act(x[sort_indices[j, e]] @ w1[e] + b1[e]) for j < count[e]
    (moe_impls.py:124-180); rows j >= count[e] are left at zero here (uninitialised in the reference)."""
    E, D, Ed = w1.shape
    N = x.size(0)
    act = ACTIVATIONS[activation]
    inter = torch.zeros(E, N, Ed, dtype=x.dtype)
    for e in range(E):
        c = int(expert_bincounts[e])
        if c == 0:
            continue
        rows = sort_indices[:c, e]
        h = x[rows].float() @ w1[e].float()
        if b1 is not None:
            h = h + b1[e].float()
        inter[e, :c] = act(h).to(x.dtype)
    return inter


def experts_second_merge(inter, unsort_indices, routing, w2):
    """Deterministic second layer: per-expert product, then per token an ascending-expert float32 sum and
    one final cast  (moe_impls.py:430-464 for the product, :485-514 for the merge order)."""
    E, N, Ed = inter.shape
    D = w2.size(-1)
    per_expert = torch.einsum('eni,eio->eno', inter.float(), w2.float()).to(inter.dtype)
    out = torch.zeros(N, D, dtype=torch.float32)
    for n in range(N):
        for e in range(E):
            if routing[n, e] > 0:
                out[n] += per_expert[e, unsort_indices[n, e]].float()
    return out.to(inter.dtype)


def experts_gated_forward_all(x, routing, w_gate, w_up, w_down, activation='gelu_tanh'):
    """Gated experts, dense and gate-weighted: sum_e r[n,e] * ((act(x Wg[e]) * (x Wu[e])) Wd[e])
    (moe_layers.py:86-96 with layers 0/2/1 = gate/up/down, no biases for Gemma)."""
    xe = x.unsqueeze(0).expand(w_gate.size(0), -1, -1)
    g = ACTIVATIONS[activation](torch.einsum('eni,eio->eno', xe, w_gate))
    u = torch.einsum('eni,eio->eno', xe, w_up)
    y = torch.einsum('eni,eio->eno', g * u, w_down)
    return torch.einsum('end,ne->nd', y, routing)


def experts_gated_forward_loop(x, routing, w_gate, w_up, w_down, activation='gelu_tanh'):
    """Gated experts as a per-expert loop with score weighting (moe_layers.py:104-113, 310-324)."""
    act = ACTIVATIONS[activation]
    out = torch.zeros_like(x)
    for e in range(w_gate.size(0)):
        mask = routing[:, e] != 0.0
        scores = routing[:, e][mask].unsqueeze(1)
        xe = x[mask]
        ye = (act(xe @ w_gate[e]) * (xe @ w_up[e])) @ w_down[e]
        out[mask] += ye * scores
    return out


# --------------------------------------------------------------------------------------------
# the layer (reference: moefication.py:90-101)
# --------------------------------------------------------------------------------------------


def moe_layer_forward(x: torch.Tensor, params: Dict[str, torch.Tensor], tau: float,
                      activation: str = 'relu', experts_mode: str = 'naive',
                      add_residual: bool = False, norms_override: Optional[torch.Tensor] = None,
                      router_activation: str = 'relu', router_output_activation: str = 'abs'
                      ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """x [B,T,D] -> (out [B,T,D], routing [B,T,E], norms [B,T,E]) with the dynk_max gate.

    Router -> gate -> experts -> + last_bias -> (+ x)  (moefication.py:90-101).  norms_override replaces
    the router output the way the reference's router test hook does (moefication.py:331-338).
    """
    if norms_override is None:
        norms = router_forward(x, params['router_w1'], params['router_w2'],
                               router_activation, router_output_activation)
    else:
        norms = norms_override
    routing = gate_dynk_max(norms, tau)
    out = layer_from_routing(x, params, routing, activation, experts_mode, add_residual)
    return out, routing, norms


def layer_from_routing(x: torch.Tensor, params: Dict[str, torch.Tensor], routing: torch.Tensor,
                       activation: str = 'relu', experts_mode: str = 'naive', add_residual: bool = False) -> torch.Tensor:
    """Experts + epilogue for a given routing tensor (moefication.py:93-100).  x [..., D], routing [..., E];
    routing is cast to x's dtype so a float64 evaluation can reuse a mask computed in the storage dtype."""
    x2 = x.reshape(-1, x.size(-1))
    r2 = routing.reshape(-1, routing.size(-1)).to(x.dtype)
    if 'w_gate' in params:
        fn = experts_gated_forward_all if experts_mode == 'all' else experts_gated_forward_loop
        out = fn(x2, r2, params['w_gate'], params['w_up'], params['w_down'], activation)
    else:
        fn = experts_forward_all if experts_mode == 'all' else experts_forward_naive
        out = fn(x2, r2, params['w1'], params.get('b1'), params['w2'], activation)
    if 'last_bias' in params:
        out = out + params['last_bias']
    if add_residual:
        out = out + x2
    return out.view(x.shape)


def upcast(params: Dict[str, torch.Tensor], dtype=torch.float64) -> Dict[str, torch.Tensor]:
    return {k: v.to(dtype) for k, v in params.items()}
