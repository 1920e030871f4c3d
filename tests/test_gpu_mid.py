"""GPU parity of the compacted two-kernel path (D2DMOE_PATH_MFMA_MID): work proportional to the routed pairs for routing of
middling density.  Outputs against the float64 oracle (2e-2, max|got - want| / max|want|, bf16), against the dense sweep on
the same routing, run-to-run bit equality, and the expert-major permutation it leaves behind against the oracle's."""
import pytest
import torch

from oracle import d2dmoe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

DEV = 'cuda:0'


def _say(*a):
    print(*a, flush=True)


def _ops():
    from d2dmoe_amd import ops
    return ops


def _packed(d, act='relu', E=128, Ed=24, with_router=False):
    ops = _ops()
    sh = ops.make_shape(0, 768, E, Ed, 128 if with_router else 0, 1, act)
    return ops.pack_weights(sh, d['w1'], d.get('b1'), d['w2'], None, d['router_w1'] if with_router else None,
                            d['router_w2'] if with_router else None)


@pytest.mark.parametrize('N,E,Ed,density', [(1, 128, 24, 0.2), (31, 128, 24, 0.2), (32, 128, 24, 0.2), (33, 128, 24, 0.3),
                                            (197, 128, 24, 0.18), (300, 128, 24, 0.02), (300, 128, 24, 0.36), (1576, 128, 24, 0.18),
                                            (1576, 128, 24, 0.06), (700, 96, 30, 0.25), (520, 16, 31, 0.5), (700, 100, 24, 0.2), (1000, 40, 7, 0.4), (260, 8, 5, 0.6),
                                            (4100, 128, 24, 0.3), (2048, 144, 16, 0.1)])
def test_mid_path_matches_oracle(N, E, Ed, density):
    _say('mid', N, E, Ed, density)
    x, routing, p = H.random_case(N, 768, E, Ed, 128, seed=N + E, dtype=torch.bfloat16, density=density)
    d = H.to_dev(p, DEV)
    ops = _ops()
    packed = _packed(d, 'relu', E, Ed)
    lb = d['last_bias'].view(-1)
    out = ops.experts(x.to(DEV), routing.to(DEV), d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_mid', packed)
    want = O.layer_from_routing(x.double(), O.upcast(p), routing.double(), 'relu', 'all')
    err = H.rel_err(out.cpu(), want)
    _say(f'  rel err {err:.2e}')
    assert err < H.TOL_BF16
    again = ops.experts(x.to(DEV), routing.to(DEV), d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_mid', packed)
    assert torch.equal(out, again)                         # fixed summation order: bit-reproducible
    dense = ops.experts(x.to(DEV), routing.to(DEV), d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_dense', packed)
    assert H.rel_err(out, dense) < 1e-2


@pytest.mark.parametrize('act', ['relu', 'gelu', 'tanh', 'leaky_relu'])
def test_mid_path_activations_weights_residual_edges(act):
    """Weighted routing (the 'masked' semantics), residual, no last_bias, rows without any expert, an expert nobody uses, an
    expert everybody uses, and a NaN-free result for all-zero routing."""
    N, E, Ed = 777, 128, 24
    x, routing, p = H.random_case(N, 768, E, Ed, 128, seed=5, dtype=torch.bfloat16, density=0.15)
    g = torch.Generator().manual_seed(1)
    routing = routing * (torch.rand(N, E, generator=g) + 0.25).bfloat16()
    routing[::7] = 0                  # tokens without experts
    routing[:, 3] = 0                 # an unused expert
    routing[:, 5] = 1                 # an expert every token uses
    d = H.to_dev(p, DEV)
    ops = _ops()
    packed = _packed(d, act)
    out = ops.experts(x.to(DEV), routing.to(DEV), d['w1'], d['b1'], d['w2'], None, None, act, True, 'mfma_mid', packed)
    pp = {k: v for k, v in p.items() if k != 'last_bias'}
    want = O.layer_from_routing(x.double(), O.upcast(pp), routing.double(), act, 'all', add_residual=True)
    assert H.rel_err(out.cpu(), want) < H.TOL_BF16
    zero = ops.experts(x.to(DEV), torch.zeros_like(routing).to(DEV), d['w1'], d['b1'], d['w2'], None, d['last_bias'].view(-1),
                       act, False, 'mfma_mid', packed)
    assert torch.equal(zero.cpu(), p['last_bias'].expand(N, -1))


@pytest.mark.parametrize('thr', [0.5, 0.3, 0.9, 0.1])
def test_mid_path_full_size_layer(thr):
    """Whole layer at 50 432 tokens with the path forced: the mask is the oracle's gate on the GPU's own norms, outputs against
    the float64 oracle on row slices; where the routed pairs exceed the capacity (threshold 0.1 of the maximum: about 100
    experts per token) the device-side switch hands the call to the dense sweep and the result is still right."""
    _say('mid full size', thr)
    N, D, E, Ed, W = 50432, 768, 128, 24, 128
    x, _, p = H.random_case(N, D, E, Ed, W, seed=61, dtype=torch.bfloat16)
    d = H.to_dev(p, DEV)
    ops = _ops()
    packed = _packed(d, 'relu', with_router=True)
    out, routing, norms, counts = ops.forward(x.to(DEV), d['router_w1'], d['router_w2'], float(thr), d['w1'], d['b1'], d['w2'],
                                              None, d['last_bias'].view(-1), 'relu', False, None, True, True, 'mfma_mid', packed)
    routing = routing.cpu()
    assert torch.equal(routing, O.gate_dynk_max_scaled(norms.cpu(), thr))
    rows = torch.cat([torch.arange(64), torch.arange(30000, 30064), torch.arange(N - 64, N)])
    want = O.layer_from_routing(x[rows].double(), O.upcast(p), routing[rows].double(), 'relu', 'all')
    err = H.rel_err(out.cpu()[rows], want)
    _say(f'  experts/token {routing.sum(1).mean().item():.1f}, rel err {err:.2e}')
    assert err < H.TOL_BF16
    dense, r2, _, _ = ops.forward(x.to(DEV), d['router_w1'], d['router_w2'], float(thr), d['w1'], d['b1'], d['w2'], None,
                                  d['last_bias'].view(-1), 'relu', False, None, True, True, 'mfma_dense', packed)
    assert torch.equal(r2.cpu(), routing)
    assert H.rel_err(out, dense) < 1e-2
    # a random permutation of the tokens permutes the outputs bit for bit: every token's sum runs over its experts in
    # ascending order whatever tile it sits in
    if thr >= 0.3:
        perm = torch.randperm(N, generator=torch.Generator().manual_seed(3))
        xp = x[perm].contiguous().to(DEV)
        rp = routing[perm].contiguous().to(DEV)
        a = ops.experts(x.to(DEV), routing.to(DEV), d['w1'], d['b1'], d['w2'], None, d['last_bias'].view(-1), 'relu', False,
                        'mfma_mid', packed)
        b = ops.experts(xp, rp, d['w1'], d['b1'], d['w2'], None, d['last_bias'].view(-1), 'relu', False, 'mfma_mid', packed)
        assert torch.equal(a.cpu()[perm], b.cpu())
