"""Pins for the CPU oracle.  The reference ships no golden vectors for the MoE forward path, so each oracle
function is checked against something the mathematics fixes: numpy float64 brute force on small inputs,
closed forms, and special cases that reduce to a library routine.  None of these re-type the oracle's own
formula: the brute-force versions are scalar python/numpy loops written per (token, expert, neuron)."""
import math

import numpy as np
import pytest
import torch

from oracle import d2dmoe_oracle as O


def _np(t):
    return t.detach().double().numpy()


def _rand_layer(N=10, D=16, E=4, Ed=6, W=8, seed=0, gated=False, dtype=torch.float64):
    p = O.make_layer_params(D, E, Ed, W, seed=seed, gated=gated, dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1000)
    x = torch.randn(N, D, generator=g).to(dtype)
    routing = (torch.rand(N, E, generator=g) < 0.5).to(dtype)
    if 'b1' in p:
        p['last_bias'] = torch.randn(1, D, generator=g).to(dtype) * 0.1
    return x, routing, p


# ---------------------------------------------------------------- activations ---------------


def test_activation_closed_forms():
    x = torch.linspace(-4, 4, 101, dtype=torch.float64)
    xn = x.numpy()
    erf = np.vectorize(math.erf)
    assert np.allclose(_np(O.act_relu(x)), np.where(xn >= 0, xn, 0.0), atol=0)
    assert np.allclose(_np(O.act_leaky_relu(x)), np.where(xn >= 0, xn, 0.01 * xn), atol=1e-15)
    # reference kernel writes tanh as 2*sigmoid(2x)-1
    assert np.allclose(_np(O.act_tanh(x)), 2.0 / (1.0 + np.exp(-2 * xn)) - 1.0, atol=1e-14)
    assert np.allclose(_np(O.act_gelu(x)), xn * 0.5 * (1 + erf(xn / math.sqrt(2))), atol=1e-14)
    ka = math.sqrt(2.0 / math.pi)
    assert np.allclose(_np(O.act_gelu_tanh(x)), 0.5 * xn * (1 + np.tanh(ka * (xn + 0.044715 * xn ** 3))), atol=1e-14)
    assert np.allclose(_np(O.act_silu(x)), xn / (1 + np.exp(-xn)), atol=1e-14)
    assert np.array_equal(_np(O.act_abs(x)), np.abs(xn))


# ---------------------------------------------------------------- init ----------------------


def test_param_shapes_bounds_and_order():
    p = O.make_layer_params(32, 8, 4, 16, seed=3)
    assert p['w1'].shape == (8, 32, 4) and p['b1'].shape == (8, 4) and p['w2'].shape == (8, 4, 32)
    assert p['last_bias'].shape == (1, 32) and torch.count_nonzero(p['last_bias']) == 0
    assert p['router_w1'].shape == (16, 32) and p['router_w2'].shape == (8, 16)
    # bounds follow the LAST dim of each tensor: w1,b1 -> 1/sqrt(Ed); w2 -> 1/sqrt(D); linears -> 1/sqrt(fan_in)
    assert p['w1'].abs().max() <= 1 / math.sqrt(4) and p['w1'].abs().max() > 0.9 / math.sqrt(4)
    assert p['w2'].abs().max() <= 1 / math.sqrt(32) and p['w2'].abs().max() > 0.9 / math.sqrt(32)
    assert p['router_w1'].abs().max() <= 1 / math.sqrt(32)
    assert p['router_w2'].abs().max() <= 1 / math.sqrt(16)
    q = O.make_layer_params(32, 8, 4, 16, seed=3)
    assert all(torch.equal(p[k], q[k]) for k in p)
    g = O.make_layer_params(32, 8, 4, 16, seed=3, gated=True, bias=False)
    assert set(g) == {'w_gate', 'w_down', 'w_up', 'router_w1', 'router_w2'}
    assert g['w_gate'].shape == (8, 32, 4) and g['w_down'].shape == (8, 4, 32) and g['w_up'].shape == (8, 32, 4)


# ---------------------------------------------------------------- router --------------------


def test_router_against_numpy_float64():
    x, _, p = _rand_layer(N=7, D=16, E=5, W=9)
    got = _np(O.router_forward(x, p['router_w1'], p['router_w2']))
    xn, w1, w2 = _np(x), _np(p['router_w1']), _np(p['router_w2'])
    want = np.zeros((7, 5))
    for n in range(7):
        hidden = [max(0.0, sum(xn[n, d] * w1[w, d] for d in range(16))) for w in range(9)]
        for e in range(5):
            want[n, e] = abs(sum(hidden[w] * w2[e, w] for w in range(9)))
    assert np.allclose(got, want, rtol=1e-12, atol=1e-14)
    assert (got >= 0).all()


def test_router_fp32_close_to_float64():
    x, _, p = _rand_layer(N=64, D=768, E=128, W=128, dtype=torch.float32)
    a = O.router_forward(x, p['router_w1'], p['router_w2']).double()
    b = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    assert (a - b).abs().max() / b.abs().max() < 1e-5


# ---------------------------------------------------------------- gates ---------------------


def _brute_dynk_max(norms, scale):
    N, E = norms.shape
    out = np.zeros((N, E))
    for n in range(N):
        m = max(norms[n])
        for e in range(E):
            out[n, e] = 1.0 if norms[n, e] >= m * scale else 0.0
    return out


@pytest.mark.parametrize('tau', [0.0, 0.1, 0.5, 0.9, 0.99, 1.0])
def test_dynk_max_brute_force(tau):
    g = torch.Generator().manual_seed(5)
    norms = torch.randn(33, 12, generator=g, dtype=torch.float64).abs()
    got = _np(O.gate_dynk_max(norms, tau))
    assert np.array_equal(got, _brute_dynk_max(_np(norms), 1.0 - tau))


def test_dynk_max_special_cases():
    g = torch.Generator().manual_seed(6)
    norms = torch.randn(50, 16, generator=g).abs()
    # tau = 1 -> threshold 0 -> every (non-negative) norm passes
    assert torch.equal(O.gate_dynk_max(norms, 1.0), torch.ones_like(norms))
    # tau = 0 -> only the maxima survive
    r0 = O.gate_dynk_max(norms, 0.0)
    assert torch.equal(r0, (norms == norms.max(-1, keepdim=True)[0]).float())
    # the arg-max expert is always kept; monotone in tau
    prev = r0
    for tau in [0.1, 0.3, 0.5, 0.9, 0.99]:
        r = O.gate_dynk_max(norms, tau)
        assert (r.gather(-1, norms.argmax(-1, keepdim=True)) == 1).all()
        assert (r >= prev).all()
        prev = r
    # all-zero row -> threshold 0 -> all experts on; NaN row -> none
    z = norms.clone()
    z[3] = 0.0
    z[4, 2] = float('nan')
    rz = O.gate_dynk_max(z, 0.5)
    assert (rz[3] == 1).all() and (rz[4] == 0).all()
    # output keeps the input dtype and is exactly 0/1
    rb = O.gate_dynk_max(norms.bfloat16(), 0.9)
    assert rb.dtype == torch.bfloat16 and set(rb.unique().tolist()) <= {0.0, 1.0}


def test_dynk_max_threshold_rounding_matches_scalar_rule():
    """threshold = round_to_dtype(float32(max) * float32(1 - tau)); checked with numpy float32 arithmetic."""
    g = torch.Generator().manual_seed(7)
    for dtype in (torch.float32, torch.bfloat16):
        norms = torch.randn(257, 32, generator=g).abs().to(dtype)
        for tau in (0.1, 0.5, 0.9, 0.95):
            scale = np.float32(1.0 - tau)
            m = norms.float().numpy().max(-1, keepdims=True)
            thr = torch.from_numpy((m * scale).astype(np.float32)).to(dtype).float().numpy()
            want = (norms.float().numpy() >= thr).astype(np.float32)
            assert np.array_equal(O.gate_dynk_max(norms, tau).float().numpy(), want)
            assert np.array_equal(O.gate_dynk_max_scaled(norms, float(scale)).float().numpy(), want)


def test_gate_all_and_topk():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 3, 10, generator=g)
    assert torch.equal(O.gate_all(x, 7), torch.ones(2, 3, 7))
    s = torch.randn(2, 5, 9, generator=g)
    for k in (1, 3, 9):
        r = O.gate_topk(s, k)
        assert (r.sum(-1) == k).all()
        # every kept score is >= every dropped score
        kept_min = torch.where(r > 0, s, torch.full_like(s, float('inf'))).min(-1)[0]
        drop_max = torch.where(r > 0, torch.full_like(s, float('-inf')), s).max(-1)[0]
        assert (kept_min >= drop_max).all()


def test_gate_dynk_brute_force():
    g = torch.Generator().manual_seed(9)
    norms = torch.rand(40, 11, generator=g, dtype=torch.float64) + 1e-3
    for tau in (0.05, 0.3, 0.7, 0.999):
        got = _np(O.gate_dynk(norms, tau))
        nn_ = _np(norms)
        for n in range(nn_.shape[0]):
            shares = nn_[n] / nn_[n].sum()
            order = sorted(range(len(shares)), key=lambda e: -shares[e])
            want = np.zeros(len(shares))
            cum = 0.0
            for e in order:  # take experts, largest first, until the cumulative share reaches tau
                want[e] = 1.0
                cum += shares[e]
                if not (cum < tau):
                    break
            assert np.array_equal(got[n], want), (n, tau)


# ---------------------------------------------------------------- permutation ---------------


@pytest.mark.parametrize('shape,p', [((1, 1), 1.0), ((64, 4), 0.5), ((197, 128), 0.02), ((300, 7), 0.8),
                                     ((129, 33), 0.0), ((65, 5), 1.0)])
def test_extract_indices_invariants(shape, p):
    g = torch.Generator().manual_seed(11)
    routing = (torch.rand(*shape, generator=g) < p).float()
    sort_idx, unsort_idx, counts = O.extract_indices(routing)
    N, E = shape
    assert sort_idx.dtype == torch.int64 and unsort_idx.dtype == torch.int64 and counts.dtype == torch.int64
    assert torch.equal(counts, routing.sum(0).long())
    offsets, token_idx = O.permutation_csr(routing)
    assert offsets[0] == 0 and torch.equal(offsets[1:].long(), counts.cumsum(0))
    ar = torch.arange(N)
    for e in range(E):
        active = routing[:, e].nonzero().flatten()
        inactive = (routing[:, e] == 0).nonzero().flatten()
        c = int(counts[e])
        assert torch.equal(sort_idx[:c, e], active)          # prefix = active tokens, ascending
        assert torch.equal(sort_idx[c:, e], inactive)        # suffix = inactive tokens, ascending
        assert torch.equal(sort_idx[unsort_idx[:, e], e], ar)  # inverse o perm = id
        assert torch.equal(unsort_idx[sort_idx[:, e], e], ar)
        assert torch.equal(token_idx[int(offsets[e]):int(offsets[e + 1])].long(), active)
    # the reference's (unstable) call defines the same prefix SETS
    unstable = routing.to(torch.int32).argsort(dim=0, descending=True)
    for e in range(E):
        c = int(counts[e])
        assert set(unstable[:c, e].tolist()) == set(sort_idx[:c, e].tolist())


# ---------------------------------------------------------------- experts -------------------


def _brute_experts(x, routing, w1, b1, w2, act, weighted):
    """Scalar loops: out[n] = sum_{e active} r * act(x_n w1_e + b1_e) w2_e, in numpy float64."""
    x, routing, w1, w2 = _np(x), _np(routing), _np(w1), _np(w2)
    b1 = None if b1 is None else _np(b1)
    N, D = x.shape
    E, _, Ed = w1.shape
    f = lambda v: _np(O.ACTIVATIONS[act](torch.tensor(v, dtype=torch.float64)))
    out = np.zeros((N, D))
    for n in range(N):
        for e in range(E):
            if routing[n, e] == 0:
                continue
            h = np.array([sum(x[n, d] * w1[e, d, j] for d in range(D)) + (0 if b1 is None else b1[e, j])
                          for j in range(Ed)])
            h = f(h)
            scale = routing[n, e] if weighted else 1.0
            for c in range(D):
                out[n, c] += scale * sum(h[j] * w2[e, j, c] for j in range(Ed))
    return out


@pytest.mark.parametrize('act', ['relu', 'gelu', 'tanh', 'leaky_relu'])
@pytest.mark.parametrize('bias', [True, False])
def test_experts_three_formulations_agree(act, bias):
    x, routing, p = _rand_layer(N=9, D=12, E=5, Ed=3, seed=21)
    b1 = p['b1'] if bias else None
    brute = _brute_experts(x, routing, p['w1'], b1, p['w2'], act, weighted=False)
    a = _np(O.experts_forward_all(x, routing, p['w1'], b1, p['w2'], act))
    b = _np(O.experts_forward_naive(x, routing, p['w1'], b1, p['w2'], act))
    assert np.allclose(a, brute, rtol=1e-11, atol=1e-13)
    assert np.allclose(b, brute, rtol=1e-11, atol=1e-13)
    # first-layer + merge composition (the reference's deterministic kernel pair)
    s, u, c = O.extract_indices(routing)
    inter = O.experts_first_layer(x, s, c, p['w1'], b1, act)
    m = _np(O.experts_second_merge(inter, u, routing, p['w2']))
    assert np.allclose(m, brute, rtol=1e-6, atol=1e-7)   # that pair accumulates in float32


def test_experts_forward_all_is_gate_weighted():
    x, routing, p = _rand_layer(N=8, D=10, E=4, Ed=3, seed=22)
    weights = routing * torch.rand(8, 4, dtype=torch.float64)
    brute = _brute_experts(x, weights, p['w1'], p['b1'], p['w2'], 'relu', weighted=True)
    assert np.allclose(_np(O.experts_forward_all(x, weights, p['w1'], p['b1'], p['w2'], 'relu')), brute,
                       rtol=1e-11, atol=1e-13)


def test_experts_special_cases_reduce_to_library_routines():
    x, routing, p = _rand_layer(N=33, D=24, E=6, Ed=5, seed=23)
    E, D, Ed = p['w1'].shape
    # all experts on  ==  a dense FFN with the experts concatenated along the hidden axis
    ones = torch.ones_like(routing)
    W1 = p['w1'].permute(1, 0, 2).reshape(D, E * Ed)
    B1 = p['b1'].reshape(E * Ed)
    W2 = p['w2'].reshape(E * Ed, D)
    dense = torch.relu(x @ W1 + B1) @ W2
    for fn in (O.experts_forward_all, O.experts_forward_naive):
        assert torch.allclose(fn(x, ones, p['w1'], p['b1'], p['w2'], 'relu'), dense, rtol=1e-11, atol=1e-13)
        # nothing routed -> zeros
        assert torch.count_nonzero(fn(x, torch.zeros_like(routing), p['w1'], p['b1'], p['w2'], 'relu')) == 0
        # one-hot routing -> one small MLP per token
        onehot = torch.zeros_like(routing)
        pick = torch.arange(33) % E
        onehot[torch.arange(33), pick] = 1
        want = torch.stack([torch.relu(x[n] @ p['w1'][pick[n]] + p['b1'][pick[n]]) @ p['w2'][pick[n]]
                            for n in range(33)])
        assert torch.allclose(fn(x, onehot, p['w1'], p['b1'], p['w2'], 'relu'), want, rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize('act', ['gelu_tanh', 'relu', 'silu'])
def test_gated_experts_formulations_agree(act):
    x, routing, p = _rand_layer(N=7, D=10, E=4, Ed=3, seed=24, gated=True)
    xn, rn = _np(x), _np(routing)
    wg, wu, wd = _np(p['w_gate']), _np(p['w_up']), _np(p['w_down'])
    f = lambda v: _np(O.ACTIVATIONS[act](torch.tensor(v, dtype=torch.float64)))
    brute = np.zeros((7, 10))
    for n in range(7):
        for e in range(4):
            if rn[n, e] == 0:
                continue
            gate = f(np.array([sum(xn[n, d] * wg[e, d, j] for d in range(10)) for j in range(3)]))
            up = np.array([sum(xn[n, d] * wu[e, d, j] for d in range(10)) for j in range(3)])
            for c in range(10):
                brute[n, c] += rn[n, e] * sum(gate[j] * up[j] * wd[e, j, c] for j in range(3))
    a = _np(O.experts_gated_forward_all(x, routing, p['w_gate'], p['w_up'], p['w_down'], act))
    b = _np(O.experts_gated_forward_loop(x, routing, p['w_gate'], p['w_up'], p['w_down'], act))
    assert np.allclose(a, brute, rtol=1e-11, atol=1e-13)
    assert np.allclose(b, brute, rtol=1e-11, atol=1e-13)
    # all-ones routing == dense gated FFN with concatenated experts
    E, D, Ed = p['w_gate'].shape
    Wg = p['w_gate'].permute(1, 0, 2).reshape(D, E * Ed)
    Wu = p['w_up'].permute(1, 0, 2).reshape(D, E * Ed)
    Wd = p['w_down'].reshape(E * Ed, D)
    dense = (O.ACTIVATIONS[act](x @ Wg) * (x @ Wu)) @ Wd
    ones = torch.ones_like(routing)
    assert torch.allclose(O.experts_gated_forward_all(x, ones, p['w_gate'], p['w_up'], p['w_down'], act), dense,
                          rtol=1e-11, atol=1e-13)


# ---------------------------------------------------------------- layer ---------------------


def test_layer_forward_composition_and_epilogue():
    x, _, p = _rand_layer(N=12, D=16, E=6, Ed=4, W=8, seed=25)
    x3 = x.view(3, 4, 16)
    out, routing, norms = O.moe_layer_forward(x3, p, tau=0.5, experts_mode='naive')
    assert out.shape == x3.shape and routing.shape == (3, 4, 6) and norms.shape == (3, 4, 6)
    assert torch.equal(routing, O.gate_dynk_max(O.router_forward(x3, p['router_w1'], p['router_w2']), 0.5))
    brute = _brute_experts(x, routing.view(12, 6), p['w1'], p['b1'], p['w2'], 'relu', weighted=False)
    assert np.allclose(_np(out.view(12, 16)), brute + _np(p['last_bias']), rtol=1e-11, atol=1e-13)
    out_r, _, _ = O.moe_layer_forward(x3, p, tau=0.5, experts_mode='all', add_residual=True)
    assert torch.allclose(out_r, out + x3, rtol=1e-11, atol=1e-13)
    # the router override hook feeds synthetic norms straight to the gate
    fake = torch.rand(3, 4, 6, dtype=torch.float64)
    _, r2, n2 = O.moe_layer_forward(x3, p, tau=0.5, norms_override=fake)
    assert torch.equal(n2, fake) and torch.equal(r2, O.gate_dynk_max(fake, 0.5))


def test_threshold_fraction_round_trip():
    # the bench takes the threshold fraction f ("0.9 x max") and sets module tau = 1 - f
    assert 1.0 - 0.1 == 0.9


def test_expert_output_norms_brute_force_gram_identity_and_special_cases():
    g = torch.Generator().manual_seed(17)
    N, D, E, Ed = 9, 12, 5, 7
    x = torch.randn(N, D, generator=g, dtype=torch.float64)
    w1 = torch.randn(E, D, Ed, generator=g, dtype=torch.float64)
    b1 = torch.randn(E, Ed, generator=g, dtype=torch.float64)
    w2 = torch.randn(E, Ed, D, generator=g, dtype=torch.float64)
    got = O.expert_output_norms(x, w1, b1, w2, 'relu')
    assert got.shape == (E, N)
    xn, w1n, b1n, w2n = x.numpy(), w1.numpy(), b1.numpy(), w2.numpy()
    for e in range(E):
        for n in range(N):
            h = np.maximum(xn[n] @ w1n[e] + b1n[e], 0.0)
            y = h @ w2n[e]
            assert abs(got[e, n].item() - math.sqrt(float((y * y).sum()))) < 1e-10
            # the quadratic form over the expert's Gram matrix gives the same number
            gram = w2n[e] @ w2n[e].T
            assert abs(got[e, n].item() ** 2 - float(h @ gram @ h)) < 1e-8
    # a zero second layer gives zero norms; norms are non-negative and scale with the second layer
    assert torch.equal(O.expert_output_norms(x, w1, b1, torch.zeros_like(w2), 'relu'), torch.zeros(E, N, dtype=torch.float64))
    assert (got >= 0).all()
    assert torch.allclose(O.expert_output_norms(x, w1, b1, -3.0 * w2, 'relu'), 3.0 * got, rtol=1e-12)
    # one expert, identity activation, no bias: |x (W1 W2)| through a library GEMM
    a = w1[0] @ w2[0]
    want = torch.linalg.vector_norm(x @ a, dim=-1)
    assert torch.allclose(O.expert_output_norms(x, w1[:1], None, w2[:1], 'identity')[0], want, rtol=1e-12)
