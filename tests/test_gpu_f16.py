"""float16 storage (the reference benches float32 and float16, scripts/test_moe_implementations.py:223-228) through the C
ABI: the generic kernels and the tiled MFMA products take it; the kernels written for bfloat16 do not.

Bars: masks, counts and permutations bit-exact for the same norms; outputs within 4e-3 of the float64 oracle on the same
stored inputs (max|got - want| / max|want|; float16 keeps 11 significant bits where bfloat16 keeps 8).
"""
import pytest
import torch

from oracle import d2dmoe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

DEV = 'cuda:0'
F16 = torch.float16
TOL_F16 = H.TOL_F16


def _ops():
    from d2dmoe_amd import ops
    return ops


def _say(*a):
    print(*a, flush=True)


def _want(x, routing, p, act, residual=False):
    return O.layer_from_routing(x.double(), O.upcast(p), routing.double(), act, 'all', residual)


def _got(x, routing, p, act, residual=False, path='auto', packed=None):
    d = H.to_dev(p, DEV)
    lb = d['last_bias'].view(-1) if 'last_bias' in d else None
    if 'w_gate' in d:
        return _ops().experts(x.to(DEV), routing.to(DEV), d['w_gate'], None, d['w_down'], d['w_up'], lb, act, residual, path,
                              packed).cpu()
    return _ops().experts(x.to(DEV), routing.to(DEV), d['w1'], d.get('b1'), d['w2'], None, lb, act, residual, path, packed).cpu()


def _pack(p, D, E, Ed, W, act, gated):
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 2, act, gated=gated)
    if gated:
        return _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    return _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])


@pytest.mark.parametrize('N,D,W,E', [(1, 64, 128, 4), (197, 768, 128, 128), (70, 100, 37, 19), (1576, 768, 128, 128),
                                     (40, 2048, 256, 256), (33, 128, 64, 96)])
def test_router_and_select_f16(N, D, W, E):
    _say('f16 router+select', N, D, W, E)
    x, _, p = H.random_case(N, D, E, 8, W, seed=N + D, dtype=F16)
    norms = _ops().router(x.to(DEV), p['router_w1'].to(DEV), p['router_w2'].to(DEV))
    want64 = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    assert norms.dtype == F16
    assert H.rel_err(norms.cpu(), want64) < TOL_F16
    for tau in (0.9, 0.5, 0.1):
        routing, counts = _ops().select(norms, float(1.0 - tau), want_counts=True)
        want = O.gate_dynk_max(norms.cpu(), tau)
        assert torch.equal(routing.cpu(), want)
        assert torch.equal(counts.cpu().long(), (want > 0).sum(0))


@pytest.mark.parametrize('N,D,W,E', [(197, 768, 128, 128), (50432, 768, 128, 128), (4096, 2048, 256, 256), (33, 768, 128, 128)])
def test_fused_router_select_f16(N, D, W, E):
    """The fused router + selection kernels with float16 storage: norms against the float64 oracle, the mask bit-exact with
    the oracle's gate on the kernel's own norms (thresholds 0.1, 0.5 and 0.9 of the maximum), counts."""
    _say('f16 fused router', N, D, W, E)
    Ed = 24 if D == 768 else 8
    x, _, p = H.random_case(N, D, E, Ed, W, seed=N + D, dtype=F16)
    d = H.to_dev(p, DEV)
    packed = _pack(p, D, E, Ed, W, 'relu', False)
    assert packed is not None
    want64 = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    for tau in (0.9, 0.5, 0.1):
        routing, norms, counts = _ops().router_select(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), packed, E,
                                                      Ed, want_norms=True, want_counts=True)
        assert H.rel_err(norms.cpu(), want64) < TOL_F16
        want = O.gate_dynk_max(norms.cpu(), tau)
        assert torch.equal(routing.cpu(), want)
        assert torch.equal(counts.cpu().long(), (want > 0).sum(0))


def test_select_special_rows_f16():
    norms = torch.rand(64, 32).half()
    norms[3] = 0.0                       # all-zero row: every expert kept
    norms[5] = 7.0                       # all-equal row
    norms[9, 4] = float('nan')           # NaN row: nothing kept
    norms[11, 2] = float('inf')
    routing, _ = _ops().select(norms.to(DEV), 0.1)
    assert torch.equal(routing.cpu(), O.gate_dynk_max(norms, 0.9))


@pytest.mark.parametrize('N,E', [(7, 5), (197, 128), (1576, 128)])
def test_build_permutation_f16(N, E):
    _say('f16 permutation', N, E)
    g = torch.Generator().manual_seed(N)
    routing = (torch.rand(N, E, generator=g) < 0.3).half()
    offsets, token_idx, sort_idx, unsort_idx, bincounts = _ops().build_permutation(routing.to(DEV), reference_layout=True)
    want_sort, want_unsort, want_counts = O.extract_indices(routing)
    assert torch.equal(sort_idx.cpu(), want_sort)
    assert torch.equal(unsort_idx.cpu(), want_unsort)
    assert torch.equal(bincounts.cpu(), want_counts)
    off = offsets.cpu().long()
    assert torch.equal(off[1:] - off[:-1], want_counts)
    for e in range(0, E, max(E // 7, 1)):
        assert torch.equal(token_idx.cpu()[off[e]:off[e + 1]].long(), want_sort[:want_counts[e], e])


@pytest.mark.parametrize('N,D,E,Ed,gated,act', [(10, 64, 4, 32, False, 'relu'), (197, 768, 128, 24, False, 'gelu'),
                                               (50, 100, 7, 5, False, 'tanh'), (20, 2048, 16, 64, True, 'gelu_tanh')])
def test_experts_generic_f16(N, D, E, Ed, gated, act):
    _say('f16 generic', N, D, E, Ed, gated, act)
    x, routing, p = H.random_case(N, D, E, Ed, 8, seed=N + E, dtype=F16, gated=gated, bias=not gated)
    got = _got(x, routing, p, act, path='generic')
    assert got.dtype == F16
    assert H.rel_err(got, _want(x, routing, p, act)) < TOL_F16
    g = torch.Generator().manual_seed(3)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).half()
    assert H.rel_err(_got(x, weights, p, act, residual=True, path='generic'), _want(x, weights, p, act, True)) < TOL_F16


@pytest.mark.parametrize('N,D,E,Ed,W,gated,act,density', [(300, 768, 128, 24, 128, False, 'relu', 0.8),
                                                         (1576, 768, 128, 24, 128, False, 'gelu', 0.1),
                                                         (700, 512, 16, 64, 128, True, 'silu', 0.5),
                                                         (257, 2048, 32, 64, 256, True, 'gelu_tanh', 0.7),
                                                         (40, 256, 6, 20, 128, False, 'relu', 0.5)])
def test_tiled_products_f16(N, D, E, Ed, W, gated, act, density):
    """v_mfma_f32_32x32x16_f16 in the tiled products: against the float64 oracle, against the generic kernel, with weighted
    routing and the residual, and for all-zero routing."""
    _say('f16 tiled products', N, D, E, Ed, gated, act)
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=N + E, dtype=F16, gated=gated, bias=not gated, density=density)
    packed = _pack(p, D, E, Ed, W, act, gated)
    assert packed is not None
    got = _got(x, routing, p, act, path='mfma_gemm', packed=packed)
    assert H.rel_err(got, _want(x, routing, p, act)) < TOL_F16
    assert H.rel_err(got, _got(x, routing, p, act, path='generic')) < TOL_F16
    if gated or D != 768:
        assert torch.equal(got, _got(x, routing, p, act, path='auto', packed=packed))    # AUTO takes the tiled products
    assert torch.equal(got, _got(x, routing, p, act, path='mfma_gemm', packed=packed))   # run to run
    g = torch.Generator().manual_seed(3)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).half()
    got = _got(x, weights, p, act, residual=True, path='mfma_gemm', packed=packed)
    assert H.rel_err(got, _want(x, weights, p, act, True)) < TOL_F16
    zero = _got(x, torch.zeros_like(routing), p, act, path='mfma_gemm', packed=packed)
    lbias = p['last_bias'].expand(N, -1).float() if 'last_bias' in p else torch.zeros(N, D)
    assert torch.equal(zero.float(), lbias)


@pytest.mark.parametrize('N,E,Ed,density,act', [(197, 128, 24, 0.8, 'relu'), (1576, 128, 24, 0.79, 'gelu'), (65, 128, 24, 0.05, 'relu'),
                                                (1, 128, 24, 0.5, 'relu'), (300, 24, 128, 0.5, 'relu'), (700, 100, 30, 0.3, 'tanh'),
                                                (9000, 128, 24, 0.6, 'relu')])
def test_dense_sweep_f16(N, E, Ed, density, act):
    """The fused sweep (D = 768) with v_mfma_f32_32x32x16_f16: against the float64 oracle, against the tiled products,
    weighted routing + residual, zero routing, run-to-run bit equality; AUTO takes it."""
    _say('f16 dense sweep', N, E, Ed, density, act)
    D, W = 768, 128
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=N + E, dtype=F16, density=density)
    packed = _pack(p, D, E, Ed, W, act, False)
    got = _got(x, routing, p, act, path='mfma_dense', packed=packed)
    assert H.rel_err(got, _want(x, routing, p, act)) < TOL_F16
    assert H.rel_err(got, _got(x, routing, p, act, path='mfma_gemm', packed=packed)) < TOL_F16
    assert torch.equal(got, _got(x, routing, p, act, path='mfma_dense', packed=packed))
    if N > 16:
        assert torch.equal(got, _got(x, routing, p, act, path='auto', packed=packed))
    g = torch.Generator().manual_seed(3)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).half()
    got = _got(x, weights, p, act, residual=True, path='mfma_dense', packed=packed)
    assert H.rel_err(got, _want(x, weights, p, act, True)) < TOL_F16
    zero = _got(x, torch.zeros_like(routing), p, act, path='mfma_dense', packed=packed)
    assert torch.equal(zero.float(), p['last_bias'].expand(N, -1).float())


@pytest.mark.parametrize('N,E,Ed,density,act', [(197, 128, 24, 0.02, 'relu'), (1576, 128, 24, 0.03, 'gelu'), (65, 128, 24, 0.05, 'relu'),
                                                (1, 128, 24, 0.2, 'relu'), (300, 24, 128, 0.1, 'relu'), (700, 100, 30, 0.06, 'tanh'),
                                                (600, 64, 40, 0.06, 'relu'), (50432, 128, 24, 0.017, 'relu')])
def test_expert_major_f16(N, E, Ed, density, act):
    """The expert-major path (plan, experts, ordered combine) with float16 storage: against the float64 oracle (on row
    slices at 50 432 tokens), single-expert and no-expert tokens, weighted routing + residual, the over-capacity
    fall-back to the sweep, run-to-run bit equality."""
    _say('f16 expert-major', N, E, Ed, density, act)
    D, W = 768, 128
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=N + E, dtype=F16, density=density)
    if N > 4:
        routing[1] = 0
        routing[2] = 0
        routing[2, E // 2] = 1      # one expert: finished inside the experts kernel
        routing[3] = 1              # every expert
    packed = _pack(p, D, E, Ed, W, act, False)
    got = _got(x, routing, p, act, path='mfma_sparse', packed=packed)
    rows = slice(0, N) if N <= 4096 else slice(N - 3000, N)
    pr = {k: v for k, v in p.items()}
    assert H.rel_err(got[rows], _want(x[rows], routing[rows], pr, act)) < TOL_F16
    assert torch.equal(got, _got(x, routing, p, act, path='mfma_sparse', packed=packed))
    assert H.rel_err(got, _got(x, routing, p, act, path='mfma_dense', packed=packed)) < TOL_F16
    if N <= 4096:
        g = torch.Generator().manual_seed(3)
        weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).half()
        got = _got(x, weights, p, act, residual=True, path='mfma_sparse', packed=packed)
        assert H.rel_err(got, _want(x, weights, p, act, True)) < TOL_F16
        dense_routing = (torch.rand(N, E, generator=g) < 0.9).half()     # beyond the capacity: the sweep does the work
        got = _got(x, dense_routing, p, act, path='mfma_sparse', packed=packed)
        assert H.rel_err(got, _want(x, dense_routing, p, act)) < TOL_F16


@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_layer_f16_vit_shape(tau):
    """Whole layer (router -> dynamic-k selection -> experts) at the ViT-B shape, 1576 tokens, float16 storage."""
    N, D, E, Ed, W = 1576, 768, 128, 24, 128
    _say('f16 layer', tau)
    x, _, p = H.random_case(N, D, E, Ed, W, seed=11, dtype=F16)
    d = H.to_dev(p, DEV)
    packed = _pack(p, D, E, Ed, W, 'relu', False)
    out, routing, norms, counts = _ops().forward(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), d['w1'], d['b1'],
                                                 d['w2'], None, d['last_bias'].view(-1), 'relu', False, None, True, True, 'auto',
                                                 packed)
    want64 = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    assert H.rel_err(norms.cpu(), want64) < TOL_F16
    assert torch.equal(routing.cpu(), O.gate_dynk_max(norms.cpu(), tau))
    assert torch.equal(counts.cpu().long(), (routing.cpu() > 0).sum(0))
    assert H.rel_err(out.cpu(), _want(x, routing.cpu(), p, 'relu')) < TOL_F16


_GEMMA = (2048, 256, 64, 256, True, 'gelu_tanh')
_VITB = (768, 128, 24, 128, False, 'relu')
_WIDE = (1024, 64, 40, 128, False, 'gelu')


@pytest.mark.parametrize('N,D,E,Ed,W,gated,act', [(n,) + c for c in (_GEMMA, _VITB, _WIDE) for n in (1, 7, 16)] + [(40,) + _GEMMA])
def test_small_batch_path_f16(N, D, E, Ed, W, gated, act):
    """The small-batch kernels (at most 16 tokens per pass, gated experts up to 48 tokens) with float16 storage: experts
    against the float64 oracle with weighted routing and residual; the whole layer (three launches) bit-equal to the staged
    entry points router -> select -> experts under both tau readings, mask exact for its own norms."""
    _say('f16 small batch', N, D, E, Ed, gated, act)
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=5 * N + E, dtype=F16, gated=gated, bias=not gated, density=0.6)
    packed = _pack(p, D, E, Ed, W, act, gated)
    g = torch.Generator().manual_seed(4)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).half()
    got = _got(x, weights, p, act, residual=True, path='mfma_decode', packed=packed)
    assert H.rel_err(got, _want(x, weights, p, act, True)) < TOL_F16
    assert torch.equal(got, _got(x, weights, p, act, residual=True, path='auto', packed=packed))
    if N > 16:
        return
    d = H.to_dev(p, DEV)
    lb = d['last_bias'].view(-1) if 'last_bias' in d else None
    ew = (d['w_gate'], None, d['w_down'], d['w_up']) if gated else (d['w1'], d['b1'], d['w2'], None)
    xd = x.to(DEV)
    for tau in (0.9, 0.1):
        out, r, norms, counts = _ops().forward(xd, d['router_w1'], d['router_w2'], float(1.0 - tau), *ew, lb, act, True, None,
                                               True, True, 'auto', packed)
        norms2 = _ops().router(xd, d['router_w1'], d['router_w2'])
        r2, counts2 = _ops().select(norms2, float(1.0 - tau), want_counts=True)
        assert torch.equal(norms, norms2) and torch.equal(r, r2) and torch.equal(counts, counts2)
        assert torch.equal(r.cpu(), O.gate_dynk_max(norms.cpu(), tau))
        out2 = _got(x, r2.cpu(), p, act, residual=True, path='mfma_decode', packed=packed)
        assert torch.equal(out.cpu(), out2)
        assert H.rel_err(out.cpu(), _want(x, r2.cpu(), p, act, True)) < TOL_F16


@pytest.mark.parametrize('N,E,Ed,density', [(100, 256, 64, 0.01), (1030, 256, 64, 0.009), (300, 64, 40, 0.1), (1, 256, 64, 0.02)])
def test_gated_expert_major_f16(N, E, Ed, density):
    """The gated expert-major path (Gemma shape, D = 2048) with float16 storage: against the float64 oracle and the tiled
    products, weighted routing + residual, run-to-run bit equality; and the whole layer under the literal rule."""
    _say('f16 gated expert-major', N, E, Ed, density)
    D, W, act = 2048, 256, 'gelu_tanh'
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=N + E, dtype=F16, gated=True, bias=False, density=density)
    if N > 4:
        routing[1] = 0
        routing[2] = 0
        routing[2, E // 2] = 1
    packed = _pack(p, D, E, Ed, W, act, True)
    got = _got(x, routing, p, act, path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _want(x, routing, p, act)) < TOL_F16
    assert torch.equal(got, _got(x, routing, p, act, path='mfma_sparse', packed=packed))
    if N > 16:
        assert H.rel_err(got, _got(x, routing, p, act, path='mfma_gemm', packed=packed)) < TOL_F16
    g = torch.Generator().manual_seed(6)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).half()
    got = _got(x, weights, p, act, residual=True, path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _want(x, weights, p, act, True)) < TOL_F16
    if E == 256 and N > 16:
        d = H.to_dev(p, DEV)
        out, r, norms, counts = _ops().forward(x.to(DEV), d['router_w1'], d['router_w2'], 0.9, d['w_gate'], None, d['w_down'],
                                               d['w_up'], None, act, False, None, True, True, 'auto', packed)
        assert torch.equal(r.cpu(), O.gate_dynk_max(norms.cpu(), 0.1))
        assert H.rel_err(out.cpu(), _want(x, r.cpu(), p, act)) < TOL_F16


def test_bf16_only_paths_refuse_f16():
    from d2dmoe_amd.hip_abi import D2DMoEError
    x, routing, p = H.random_case(64, 768, 128, 24, 128, seed=1, dtype=F16)
    packed = _pack(p, 768, 128, 24, 128, 'relu', False)
    for path in ('mfma_mid',):
        with pytest.raises(D2DMoEError):
            _got(x, routing, p, 'relu', path=path, packed=packed)
