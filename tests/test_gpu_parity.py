"""Parity of the HIP path against the CPU oracle, through the C ABI (d2dmoe_amd.ops binds include/d2dmoe.h).

Bars:  routing masks, counts and permutations bit-exact given the same predicted norms;
       layer outputs within 1e-5 (float32) / 2e-2 (bfloat16) relative error, measured as
       max|got - want| / max|want| against the oracle evaluated in float64 on the same stored inputs.
"""
import hashlib

import numpy as np
import pytest
import torch

from oracle import d2dmoe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

DEV = 'cuda:0'
DTYPES = [torch.float32, torch.bfloat16]


def _ops():
    from d2dmoe_amd import ops
    return ops


def _say(*a):
    print(*a, flush=True)


# =================================================================== router ===========================
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('N,D,W,E', [(1, 64, 128, 4), (10, 64, 128, 4), (197, 768, 128, 128), (1576, 768, 128, 128),
                                     (16, 2048, 256, 256), (70, 100, 37, 19),
                                     # widths that are multiples of 32: the float32 layers run on the matrix cores
                                     (33, 96, 160, 32), (50, 32, 32, 64), (100, 64, 96, 288)])
def test_router_matches_oracle(dtype, N, D, W, E):
    _say('router', dtype, N, D, W, E)
    x, _, p = H.random_case(N, D, E, 8, W, seed=N + D, dtype=dtype)
    got = _ops().router(x.to(DEV), p['router_w1'].to(DEV), p['router_w2'].to(DEV)).cpu()
    want64 = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    assert got.dtype == dtype and got.shape == (N, E)
    assert H.rel_err(got, want64) < H.tol_for(dtype)
    if dtype == torch.bfloat16:
        # against the oracle evaluated in bf16 itself: the same values except where the accumulation order moves a
        # result across a rounding boundary (one bf16 ulp = 2^-8 relative)
        want = O.router_forward(x, p['router_w1'], p['router_w2']).float()
        diff = (got.float() - want).abs()
        assert (diff <= want.abs() * 2 ** -6 + 1e-3).all()
        assert (diff == 0).float().mean() > 0.9


@pytest.mark.parametrize('dtype', DTYPES)
def test_router_other_activations(dtype):
    x, _, p = H.random_case(33, 96, 12, 8, 40, seed=5, dtype=dtype)
    for act, oact in [('tanh', 'identity'), ('gelu', 'abs'), ('leaky_relu', 'relu')]:
        got = _ops().router(x.to(DEV), p['router_w1'].to(DEV), p['router_w2'].to(DEV), act, oact).cpu()
        want = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double(), act, oact)
        assert H.rel_err(got, want) < H.tol_for(dtype), (act, oact)


# =================================================================== select ===========================
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('N,E', [(1, 1), (7, 5), (197, 128), (1576, 128), (50432, 128), (16, 256), (33, 1000), (64, 64)])
def test_select_bit_exact(dtype, N, E):
    _say('select', dtype, N, E)
    g = torch.Generator().manual_seed(N * 31 + E)
    norms = torch.randn(N, E, generator=g).abs().to(dtype)
    if N >= 7:
        norms[3] = 0.0                  # all-zero row -> everything selected
        norms[5, E // 2] = float('nan')  # NaN row -> nothing selected
        norms[6] = norms[6, 0]           # all-equal row
    for tau in (0.0, 0.1, 0.5, 0.9, 0.99, 1.0):
        scale = float(1.0 - tau)
        routing, counts = _ops().select(norms.to(DEV), scale, want_counts=True)
        want = O.gate_dynk_max(norms, tau)
        assert routing.dtype == dtype
        assert torch.equal(routing.cpu(), want), (tau, (routing.cpu() != want).sum().item())
        assert torch.equal(counts.cpu().long(), want.float().sum(0).long())


def test_select_threshold_fraction_convention():
    """The bench's "threshold fraction f" enters as thr_scale = f; the module's tau enters as 1 - tau."""
    g = torch.Generator().manual_seed(1)
    norms = torch.randn(500, 128, generator=g).abs().bfloat16()
    r, _ = _ops().select(norms.to(DEV), 0.9)
    assert torch.equal(r.cpu(), O.gate_dynk_max_scaled(norms, 0.9))
    assert torch.equal(r.cpu(), O.gate_dynk_max(norms, 1.0 - 0.9))


# =================================================================== permutation ======================
def _check_perm(routing_cpu):
    N, E = routing_cpu.shape
    off, tok, s, u, c = _ops().build_permutation(routing_cpu.to(DEV), reference_layout=True)
    so, uo, co = O.extract_indices(routing_cpu)
    oo, to = O.permutation_csr(routing_cpu)
    assert torch.equal(off.cpu(), oo)
    P = int(oo[-1])
    assert torch.equal(tok.cpu()[:P], to)
    assert torch.equal(c.cpu(), co)
    assert torch.equal(s.cpu(), so), 'sort_indices differ from argsort(stable, descending)'
    assert torch.equal(u.cpu(), uo), 'unsort_indices differ'
    off2, tok2 = _ops().build_permutation(routing_cpu.to(DEV))
    assert torch.equal(off2.cpu(), oo) and torch.equal(tok2.cpu()[:P], to)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('N,E,p', [(1, 1, 1.0), (1, 128, 0.5), (63, 4, 0.5), (64, 4, 0.5), (65, 5, 0.5), (197, 128, 0.02),
                                   (1576, 128, 0.8), (1000, 33, 0.0), (1000, 33, 1.0), (4096, 256, 0.3),
                                   (1111, 130, 0.6), (50432, 128, 0.79)])
def test_permutation_bit_exact(dtype, N, E, p):
    _say('perm', dtype, N, E, p)
    g = torch.Generator().manual_seed(N + E)
    routing = (torch.rand(N, E, generator=g) < p).to(dtype)
    _check_perm(routing)


def test_permutation_skewed_and_empty():
    # Zipf-like expert popularity: a few experts take most tokens
    g = torch.Generator().manual_seed(3)
    w = torch.arange(1, 129).float() ** -1.2
    routing = (torch.rand(5000, 128, generator=g) < (w * 3).clamp(max=1.0)).bfloat16()
    _check_perm(routing)
    # no tokens at all
    off, tok = _ops().build_permutation(torch.empty(0, 16, dtype=torch.float32, device=DEV))
    assert torch.equal(off.cpu(), torch.zeros(17, dtype=torch.int32))


# =================================================================== experts ==========================
def _experts_want(x, routing, p, act, residual=False):
    return O.layer_from_routing(x.double(), O.upcast(p), routing.double(), act, 'all', residual)


def _experts_got(x, routing, p, act, residual=False, path='generic', packed=None):
    d = H.to_dev(p, DEV)
    lb = d['last_bias'].view(-1) if 'last_bias' in d else None
    if 'w_gate' in d:
        return _ops().experts(x.to(DEV), routing.to(DEV), d['w_gate'], None, d['w_down'], d['w_up'], lb, act,
                              residual, path, packed).cpu()
    return _ops().experts(x.to(DEV), routing.to(DEV), d['w1'], d.get('b1'), d['w2'], None, lb, act, residual, path,
                          packed).cpu()


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('N,D,E,Ed,density', [(10, 64, 4, 32, 0.5), (1, 64, 4, 32, 1.0), (197, 768, 128, 24, 0.8),
                                              (197, 768, 128, 24, 0.02), (1576, 768, 128, 24, 0.79),
                                              (77, 768, 24, 128, 0.5), (50, 100, 7, 5, 0.5), (20, 2048, 16, 64, 0.5)])
def test_experts_generic_matches_oracle(dtype, N, D, E, Ed, density):
    _say('experts generic', dtype, N, D, E, Ed, density)
    x, routing, p = H.random_case(N, D, E, Ed, 8, seed=N + E, dtype=dtype, density=density)
    got = _experts_got(x, routing, p, 'relu')
    assert got.dtype == dtype
    assert H.rel_err(got, _experts_want(x, routing, p, 'relu')) < H.tol_for(dtype)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('act', ['relu', 'gelu', 'tanh', 'leaky_relu'])
def test_experts_generic_activations_bias_residual(dtype, act):
    x, routing, p = H.random_case(70, 96, 10, 12, 8, seed=11, dtype=dtype)
    assert H.rel_err(_experts_got(x, routing, p, act, residual=True), _experts_want(x, routing, p, act, True)) < H.tol_for(dtype)
    q = {k: v for k, v in p.items() if k not in ('b1', 'last_bias')}
    assert H.rel_err(_experts_got(x, routing, q, act), _experts_want(x, routing, q, act)) < H.tol_for(dtype)


@pytest.mark.parametrize('dtype', DTYPES)
def test_experts_generic_special_cases(dtype):
    x, routing, p = H.random_case(40, 64, 6, 8, 8, seed=12, dtype=dtype)
    # nothing routed -> last_bias only
    got = _experts_got(x, torch.zeros_like(routing), p, 'relu')
    assert torch.equal(got, p['last_bias'].expand(40, -1))
    # everything routed == dense FFN with the experts concatenated (two library GEMMs)
    ones = torch.ones_like(routing)
    E, D, Ed = p['w1'].shape
    W1 = p['w1'].double().permute(1, 0, 2).reshape(D, E * Ed)
    dense = torch.relu(x.double() @ W1 + p['b1'].double().reshape(-1)) @ p['w2'].double().reshape(E * Ed, D)
    dense = dense + p['last_bias'].double()
    assert H.rel_err(_experts_got(x, ones, p, 'relu'), dense) < H.tol_for(dtype)
    # weighted routing == the reference's 'masked' formulation
    g = torch.Generator().manual_seed(1)
    weights = (routing.float() * torch.rand(40, 6, generator=g)).to(dtype)
    assert H.rel_err(_experts_got(x, weights, p, 'relu'), _experts_want(x, weights, p, 'relu')) < H.tol_for(dtype)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('act', ['gelu_tanh', 'relu', 'silu'])
def test_experts_generic_gated(dtype, act):
    x, routing, p = H.random_case(16, 256, 16, 64, 8, seed=13, dtype=dtype, gated=True, bias=False)
    assert H.rel_err(_experts_got(x, routing, p, act), _experts_want(x, routing, p, act)) < H.tol_for(dtype)


# =================================================================== experts, bf16 MFMA ===============
def _packed_for(p, act='relu', with_router=False):
    d = H.to_dev(p, DEV)
    E, D, Ed = d['w1'].shape
    W = d['router_w1'].size(0) if with_router else 0
    sh = _ops().make_shape(0, D, E, Ed, W, 1, act)
    packed = _ops().pack_weights(sh, d['w1'], d.get('b1'), d['w2'], None, d['router_w1'] if with_router else None,
                                 d['router_w2'] if with_router else None)
    assert packed is not None, 'no MFMA kernel for this shape'
    return packed


@pytest.mark.parametrize('N,E,Ed,density', [(197, 128, 24, 0.8), (197, 128, 24, 0.02), (1576, 128, 24, 0.79), (64, 128, 24, 1.0),
                                            (65, 128, 24, 0.5), (1, 128, 24, 0.5), (300, 24, 128, 0.5), (130, 100, 30, 0.5),
                                            (100, 7, 5, 0.5), (70, 16, 192, 0.5), (96, 160, 16, 0.3)])
def test_experts_mfma_dense_matches_oracle(N, E, Ed, density):
    _say('experts mfma', N, E, Ed, density)
    x, routing, p = H.random_case(N, 768, E, Ed, 8, seed=N + E, dtype=torch.bfloat16, density=density)
    packed = _packed_for(p)
    got = _experts_got(x, routing, p, 'relu', path='mfma_dense', packed=packed)
    assert H.rel_err(got, _experts_want(x, routing, p, 'relu')) < H.TOL_BF16
    # the two HIP paths share their rounding points (h rounded to bf16, float32 sums, one final rounding)
    assert H.rel_err(got, _experts_got(x, routing, p, 'relu')) < 1e-2


@pytest.mark.parametrize('act', ['relu', 'gelu', 'tanh', 'leaky_relu'])
def test_experts_mfma_dense_activations_bias_residual_weights(act):
    x, routing, p = H.random_case(200, 768, 128, 24, 8, seed=21, dtype=torch.bfloat16, density=0.6)
    packed = _packed_for(p, act)
    got = _experts_got(x, routing, p, act, residual=True, path='mfma_dense', packed=packed)
    assert H.rel_err(got, _experts_want(x, routing, p, act, True)) < H.TOL_BF16
    q = {k: v for k, v in p.items() if k not in ('b1', 'last_bias')}
    got = _experts_got(x, routing, q, act, path='mfma_dense', packed=_packed_for(q, act))
    assert H.rel_err(got, _experts_want(x, routing, q, act)) < H.TOL_BF16
    g = torch.Generator().manual_seed(2)
    weights = (routing.float() * torch.rand(200, 128, generator=g)).bfloat16()
    got = _experts_got(x, weights, p, act, path='mfma_dense', packed=packed)
    assert H.rel_err(got, _experts_want(x, weights, p, act)) < H.TOL_BF16
    # nothing routed -> last_bias only (every chunk is skipped)
    got = _experts_got(x, torch.zeros_like(routing), p, act, path='mfma_dense', packed=packed)
    assert torch.equal(got, p['last_bias'].expand(200, -1))


@pytest.mark.parametrize('N,E,Ed,density,act', [(197, 128, 32, 0.8, 'gelu'), (197, 128, 32, 0.02, 'gelu'), (1600, 128, 32, 0.79, 'gelu'),
                                                (64, 64, 64, 1.0, 'relu'), (65, 128, 24, 0.5, 'relu'), (1, 128, 32, 0.5, 'gelu'),
                                                (300, 24, 128, 0.5, 'relu'), (130, 100, 30, 0.5, 'tanh'), (100, 7, 5, 0.5, 'relu'),
                                                (96, 160, 16, 0.3, 'leaky_relu'), (4200, 16, 256, 0.6, 'gelu')])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_experts_mfma_dense_at_width_1024(N, E, Ed, density, act, dtype):
    """The fused sweep at D = 1024 (GPT-2 medium, BERT-large, ViT-L; hidden size up to 4096): chunks of 128 neurons,
    routing values fetched from global memory one chunk ahead, first product accumulated in vector registers.  Against
    the float64 oracle and the tiled products; nothing routed, weighted routing with residual, no biases, run-to-run
    bits; the last shape (experts of 256 neurons) has no sweep and must still take the tiled products under AUTO."""
    _say('experts mfma D=1024', N, E, Ed, density, act, dtype)
    tol = H.TOL_BF16 if dtype == torch.bfloat16 else 4e-3
    x, routing, p = H.random_case(N, 1024, E, Ed, 8, seed=N + E, dtype=dtype, density=density)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, 1024, E, Ed, 0, _ops()._dtype_code(x), act)
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    assert packed is not None
    want = _experts_want(x, routing, p, act)
    if Ed > 128:
        got = _experts_got(x, routing, p, act, path='auto', packed=packed)
        assert torch.equal(got, _experts_got(x, routing, p, act, path='mfma_gemm', packed=packed))
        assert H.rel_err(got, want) < tol
        return
    got = _experts_got(x, routing, p, act, path='mfma_dense', packed=packed)
    assert H.rel_err(got, want) < tol
    assert H.elem_err(got, want) < tol
    assert H.rel_err(got, _experts_got(x, routing, p, act, path='mfma_gemm', packed=packed)) < (1e-2 if dtype == torch.bfloat16 else 2e-3)
    if N > 16:
        assert torch.equal(got, _experts_got(x, routing, p, act, path='auto', packed=packed))
    assert torch.equal(got, _experts_got(x, routing, p, act, path='mfma_dense', packed=packed))
    zero = _experts_got(x, torch.zeros_like(routing), p, act, path='mfma_dense', packed=packed)
    assert torch.equal(zero, p['last_bias'].expand(N, -1))
    g = torch.Generator().manual_seed(5)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).to(dtype)
    got = _experts_got(x, weights, p, act, residual=True, path='mfma_dense', packed=packed)
    assert H.rel_err(got, _experts_want(x, weights, p, act, True)) < tol
    q = {k: v for k, v in p.items() if k not in ('b1', 'last_bias')}
    dq = H.to_dev(q, DEV)
    packed_q = _ops().pack_weights(sh, dq['w1'], None, dq['w2'], None, None, None)
    got = _experts_got(x, routing, q, act, path='mfma_dense', packed=packed_q)
    assert H.rel_err(got, _experts_want(x, routing, q, act)) < tol


@pytest.mark.parametrize('E,Ed,act,dtype', [(128, 32, 'gelu', torch.float16), (128, 30, 'relu', torch.bfloat16),
                                            (100, 30, 'gelu', torch.float16), (128, 24, 'tanh', torch.bfloat16),
                                            (64, 64, 'relu', torch.float16), (96, 20, 'leaky_relu', torch.float16)])
def test_experts_mfma_dense_at_width_1024_whole_tiles(E, Ed, act, dtype):
    """8320 tokens are 130 whole tiles of 64: the two-token-tile form of every instance of the D = 1024 sweep (storage type
    x compiled-in or run-time activation x expert sizes that are / are not multiples of 8), against the tiled products on
    all rows and the float64 oracle on a slice; and the same instances as the expert-major path's device-side fall-back
    (one workgroup per CU walking the tiles), which must give the same bits."""
    _say('experts mfma D=1024 whole tiles', E, Ed, act, dtype)
    N = 8320
    tol = H.TOL_BF16 if dtype == torch.bfloat16 else 4e-3
    x, routing, p = H.random_case(N, 1024, E, Ed, 8, seed=E + Ed, dtype=dtype, density=0.7)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, 1024, E, Ed, 0, _ops()._dtype_code(x), act)
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    xg, rg, lb = x.to(DEV), routing.to(DEV), d['last_bias'].view(-1)
    a = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, act, True, 'mfma_dense', packed)
    t = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, act, True, 'mfma_gemm', packed)
    assert H.rel_err(a, t) < (1e-2 if dtype == torch.bfloat16 else 2e-3)
    rows = torch.cat([torch.arange(0, 96), torch.arange(N - 64, N)])
    want = _experts_want(x[rows], routing[rows], p, act, True)
    assert H.rel_err(a.cpu()[rows], want) < tol
    assert H.elem_err(a.cpu()[rows], want) < tol
    if Ed <= 64:   # the expert-major path exists; 0.7 * E experts per token are far beyond its capacity
        f = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, act, True, 'mfma_sparse', packed)
        assert torch.equal(f, a)


def test_experts_mfma_dense_at_width_1024_full_size_properties():
    """GPT-2-medium layer at 16 384 tokens (128 experts x 32, GELU): oracle on a slice of rows, the tiled products on all
    rows, two runs give identical bits, and permuting the tokens permutes the output rows bit for bit."""
    N = 16384
    x, routing, p = H.random_case(N, 1024, 128, 32, 8, seed=41, dtype=torch.bfloat16, density=0.79)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, 1024, 128, 32, 0, 1, 'gelu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    xg, rg = x.to(DEV), routing.to(DEV)
    lb = d['last_bias'].view(-1)
    a = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'gelu', True, 'mfma_dense', packed)
    b = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'gelu', True, 'mfma_dense', packed)
    assert torch.equal(a, b)
    t = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'gelu', True, 'mfma_gemm', packed)
    assert H.rel_err(a, t) < 1e-2
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(9)).to(DEV)
    c = _ops().experts(xg[perm].contiguous(), rg[perm].contiguous(), d['w1'], d['b1'], d['w2'], None, lb, 'gelu', True,
                       'mfma_dense', packed)
    assert torch.equal(c, a[perm])
    rows = torch.cat([torch.arange(0, 128), torch.arange(8000, 8064), torch.arange(N - 64, N)])
    want = _experts_want(x[rows], routing[rows], p, 'gelu', True)
    assert H.rel_err(a.cpu()[rows], want) < H.TOL_BF16
    assert H.elem_err(a.cpu()[rows], want) < H.TOL_BF16


def _structured_routing(kind, N, E, seed):
    """Routings whose experts are used unevenly, the cases in which a tile of the sweep works through fewer blocks of
    hidden neurons than the layer has."""
    g = torch.Generator().manual_seed(seed)
    r = torch.zeros(N, E)
    if kind == 'hot':            # every token picks 2 of the same 5 experts
        hot = torch.randperm(E, generator=g)[:5]
        pick = torch.stack([hot[torch.randperm(5, generator=g)[:2]] for _ in range(N)])
        r.scatter_(1, pick, 1.0)
    elif kind == 'one_dense':    # a few hot experts, and one token in a hundred routes to half of all experts
        hot = torch.randperm(E, generator=g)[:3]
        r[:, hot] = (torch.rand(N, 3, generator=g) < 0.7).float()
        dense = torch.rand(N, generator=g) < 0.01
        r[dense] = (torch.rand(int(dense.sum()), E, generator=g) < 0.5).float()
    elif kind == 'by_tile':      # tokens of one 64-token tile share a window of experts that moves from tile to tile
        for t0 in range(0, N, 64):
            e0 = (t0 // 64 * 7) % E
            idx = (e0 + torch.arange(6)) % E
            r[t0:t0 + 64, idx] = (torch.rand(min(64, N - t0), 6, generator=g) < 0.6).float()
    elif kind == 'last_only':    # only the last expert (the last block, partly padding when hidden % 32 != 0)
        r[:, E - 1] = 1.0
    elif kind == 'zipf':         # norms |randn| * rank^-1.2 under the 0.1 * max rule
        w = (torch.randperm(E, generator=g).float() + 1.0) ** -1.2
        n = torch.randn(N, E, generator=g).abs() * w
        r = (n >= 0.1 * n.max(1, keepdim=True).values).float()
    return r


@pytest.mark.parametrize('kind', ['hot', 'one_dense', 'by_tile', 'last_only', 'zipf'])
@pytest.mark.parametrize('N,D,E,Ed,act,dtype', [(1000, 768, 128, 24, 'relu', torch.bfloat16), (8320, 768, 128, 24, 'gelu', torch.bfloat16),
                                                (700, 768, 100, 30, 'relu', torch.float16), (900, 768, 24, 128, 'relu', torch.bfloat16),
                                                (1000, 1024, 128, 32, 'gelu', torch.bfloat16), (8320, 1024, 100, 30, 'relu', torch.float16),
                                                (300, 768, 7, 5, 'relu', torch.bfloat16)])
def test_experts_mfma_dense_uneven_expert_use(kind, N, D, E, Ed, act, dtype):
    """The sweep gathers its chunks from the blocks of 32 hidden neurons that a tile's tokens use.  Routings with hot
    experts, a rare dense token, expert windows that move from tile to tile, a single expert at the end of the layer, and
    Zipf-weighted norms: against the float64 oracle and the generic kernel (small cases).  Where every tile is a whole
    one (8320 tokens), a random permutation of the tokens -- tiles then hold other tokens and gather other blocks -- must
    permute the output rows bit for bit: a block a tile works through for its other tokens adds exact zeros to a row."""
    _say('experts mfma uneven use', kind, N, D, E, Ed, act, dtype)
    tol = H.TOL_BF16 if dtype == torch.bfloat16 else 4e-3
    x, _, p = H.random_case(N, D, E, Ed, 8, seed=N + E, dtype=dtype, density=0.5)
    routing = _structured_routing(kind, N, E, seed=E + Ed).to(dtype)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, 0, _ops()._dtype_code(x), act)
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    got = _experts_got(x, routing, p, act, residual=True, path='mfma_dense', packed=packed)
    rows = torch.arange(N) if N <= 1000 else torch.cat([torch.arange(0, 200), torch.arange(N - 200, N)])
    want = _experts_want(x[rows], routing[rows], p, act, True)
    assert H.rel_err(got[rows], want) < tol
    assert H.elem_err(got[rows], want) < tol
    if N <= 1000 and D == 768:
        assert H.rel_err(got, _experts_got(x, routing, p, act, residual=True, path='generic')) < (1e-2 if dtype == torch.bfloat16 else 2e-3)
    if N == 8320:     # whole tiles only (the tail tiles sum their chunk ranges in a second step)
        perm = torch.randperm(N, generator=torch.Generator().manual_seed(4))
        got_p = _experts_got(x[perm].contiguous(), routing[perm].contiguous(), p, act, residual=True, path='mfma_dense', packed=packed)
        assert torch.equal(got_p, got[perm])


def test_experts_mfma_dense_full_size_properties():
    """50432 tokens (the headline workload): oracle on a slice of rows, the generic HIP kernel on all rows, and
    determinism (two runs give identical bits)."""
    N = 50432
    x, routing, p = H.random_case(N, 768, 128, 24, 8, seed=31, dtype=torch.bfloat16, density=0.79)
    packed = _packed_for(p)
    d = H.to_dev(p, DEV)
    xg, rg = x.to(DEV), routing.to(DEV)
    lb = d['last_bias'].view(-1)
    a = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_dense', packed)
    b = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_dense', packed)
    assert torch.equal(a, b)
    gen = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'generic', None)
    assert H.rel_err(a, gen) < 1e-2
    rows = torch.cat([torch.arange(0, 128), torch.arange(25000, 25064), torch.arange(N - 64, N)])
    want = _experts_want(x[rows], routing[rows], p, 'relu')
    assert H.rel_err(a.cpu()[rows], want) < H.TOL_BF16
    assert H.elem_err(a.cpu()[rows], want) < H.TOL_BF16


@pytest.mark.parametrize('N,E,Ed,density', [(197, 128, 24, 0.02), (1576, 128, 24, 0.0165), (65, 128, 24, 0.05), (1, 128, 24, 0.05),
                                            (300, 24, 128, 0.1), (130, 100, 30, 0.05), (333, 16, 64, 0.2), (100, 7, 5, 0.3),
                                            (1576, 128, 24, 0.5)])
def test_experts_mfma_sparse_matches_oracle(N, E, Ed, density):
    """Expert-major path: plan -> grouped per-expert kernel -> ordered combine.  The last case routes 64 experts per
    token, more than the path is provisioned for, so the device-side flag hands the call to the dense sweep."""
    _say('experts sparse', N, E, Ed, density)
    x, routing, p = H.random_case(N, 768, E, Ed, 8, seed=N + E + 1, dtype=torch.bfloat16, density=density)
    packed = _packed_for(p)
    got = _experts_got(x, routing, p, 'relu', path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _experts_want(x, routing, p, 'relu')) < H.TOL_BF16
    assert H.rel_err(got, _experts_got(x, routing, p, 'relu', path='mfma_dense', packed=packed)) < 1e-2
    assert torch.equal(got, _experts_got(x, routing, p, 'relu', path='mfma_sparse', packed=packed))   # deterministic


def test_layer_big_experts_auto_paths():
    """d2dmoe_forward under AUTO with 24 experts of 128 neurons (the reference benchmark's split): with the norms
    handed in (the Bernoulli override of scripts/test_moe_implementations.py:136-142, tau 0.99) the expert-major path
    runs whatever the threshold, and above its capacity the sweep takes over on the device; behind the real router a low
    threshold fraction goes straight to the sweep and a high one to the expert-major path.  Each result must be, bit for
    bit, what the experts entry point gives for the same routing on the path named."""
    N, D, E, Ed, W = 3000, 768, 24, 128, 128
    x, _, p = H.random_case(N, D, E, Ed, W, seed=5, dtype=torch.bfloat16)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, 'relu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    lb = d['last_bias'].view(-1)
    xd = x.to(DEV)

    def layer(thr_scale, norms_in):
        return _ops().forward(xd, d['router_w1'], d['router_w2'], thr_scale, d['w1'], d['b1'], d['w2'], None, lb, 'relu',
                              False, norms_in, False, False, 'auto', packed)

    def experts(routing, path):
        return _ops().experts(xd, routing, d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, path, packed)

    for k_frac, path in ((0.1, 'mfma_sparse'), (0.9, 'mfma_dense')):
        g = torch.Generator().manual_seed(int(k_frac * 10))
        norms_in = (torch.rand(N, E, generator=g) < k_frac).to(torch.bfloat16).to(DEV)
        out, routing, _, _ = layer(0.01, norms_in)
        assert torch.equal(routing.cpu(), O.gate_dynk_max(norms_in.cpu(), 0.99))
        assert torch.equal(out, experts(routing, path)), (k_frac, path)
        assert H.rel_err(out.cpu(), _experts_want(x, routing.cpu(), p, 'relu')) < H.TOL_BF16
    for thr_scale, path in ((0.1, 'mfma_dense'), (0.9, 'mfma_sparse')):
        out, routing, _, _ = layer(thr_scale, None)
        assert torch.equal(out, experts(routing, path)), (thr_scale, path)
        assert H.rel_err(out.cpu(), _experts_want(x, routing.cpu(), p, 'relu')) < H.TOL_BF16


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('N,D,E,Ed', [(300, 768, 24, 128), (300, 768, 128, 24), (300, 768, 16, 64), (300, 1024, 64, 32),
                                      (300, 1280, 40, 32), (2600, 768, 3, 128), (1, 768, 1, 24)])
def test_experts_mfma_sparse_degenerate_routings(N, D, E, Ed, dtype):
    """Expert-major path on routings that leave the plan with empty or lopsided lists: no pair at all (the output is
    last_bias), every token on the last expert only (one list, every token finished inside the experts kernel), one
    token on every expert (E lists of one pair), and one expert per token round-robin with the residual added."""
    _say('experts sparse degenerate', N, D, E, Ed, dtype)
    x, _, p = H.random_case(N, D, E, Ed, 8, seed=N + E, dtype=dtype)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, 0, 1 if dtype == torch.bfloat16 else 2, 'relu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    assert packed is not None
    zeros = torch.zeros(N, E)
    last = zeros.clone(); last[:, E - 1] = 1
    one_token = zeros.clone(); one_token[N // 2] = 1
    diag = zeros.clone(); diag[torch.arange(N), torch.arange(N) % E] = 1
    for routing, residual in ((zeros, False), (last, False), (one_token, False), (diag, True)):
        routing = routing.to(dtype)
        got = _experts_got(x, routing, p, 'relu', residual=residual, path='mfma_sparse', packed=packed)
        assert H.rel_err(got, _experts_want(x, routing, p, 'relu', residual)) < H.tol_for(dtype)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('N,E,Ed,density,act', [(5000, 24, 128, 0.1, 'relu'), (2000, 10, 100, 0.3, 'gelu'), (33, 24, 128, 0.2, 'relu'),
                                                (1, 24, 128, 0.5, 'relu'), (9000, 3, 128, 0.5, 'tanh'),
                                                (50432, 24, 128, 0.1, 'relu'), (50432, 24, 128, 0.5, 'relu')])
def test_experts_mfma_sparse_big_experts(N, E, Ed, density, act, dtype):
    """Expert-major path for experts of more than 64 neurons (the reference's own benchmark shape, 24 experts x 128:
    scripts/test_moe_implementations.py:109-126): groups of up to 8 tiles of 32 pairs per weight load.  Against the
    float64 oracle (row slices at 50 432 tokens) and the dense sweep; tokens with no / one / every expert; weighted
    routing + residual; run-to-run bit equality; AUTO takes this path for such experts; at density 0.5 the pairs exceed
    the provisioned capacity and the device-side flag hands over to the sweep, whose result must then be the sweep's
    own, bit for bit."""
    _say('experts sparse big', N, E, Ed, density, act, dtype)
    tol = H.tol_for(dtype)
    x, routing, p = H.random_case(N, 768, E, Ed, 8, seed=N + E + Ed, dtype=dtype, density=density)
    if N > 4:
        routing[1] = 0
        routing[2] = 0
        routing[2, E // 2] = 1
        routing[3] = 1
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, 768, E, Ed, 0, 1 if dtype == torch.bfloat16 else 2, act)
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    assert packed is not None
    got = _experts_got(x, routing, p, act, path='mfma_sparse', packed=packed)
    rows = slice(0, N) if N <= 5000 else slice(N - 2500, N)
    assert H.rel_err(got[rows], _experts_want(x[rows], routing[rows], p, act)) < tol
    assert torch.equal(got, _experts_got(x, routing, p, act, path='mfma_sparse', packed=packed))
    if N > 16:
        assert torch.equal(got, _experts_got(x, routing, p, act, path='auto', packed=packed))
    dense = _experts_got(x, routing, p, act, path='mfma_dense', packed=packed)
    if routing.float().sum().item() > 8 * N:
        assert torch.equal(got, dense)          # over capacity: the sweep ran
    else:
        assert H.rel_err(got, dense) < tol
    if N <= 5000:
        g = torch.Generator().manual_seed(5)
        weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).to(dtype)
        got = _experts_got(x, weights, p, act, residual=True, path='mfma_sparse', packed=packed)
        assert H.rel_err(got, _experts_want(x, weights, p, act, True)) < tol


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('N,D,E,Ed,density,act', [(300, 1024, 128, 32, 0.03, 'gelu'), (1576, 1024, 128, 32, 0.02, 'relu'),
                                                  (700, 1024, 64, 64, 0.05, 'relu'), (333, 1024, 100, 20, 0.04, 'tanh'),
                                                  (1, 1024, 128, 32, 0.05, 'relu'), (900, 1280, 160, 32, 0.03, 'gelu'),
                                                  (20000, 1024, 128, 32, 0.017, 'gelu')])
def test_experts_mfma_sparse_wide_models(N, D, E, Ed, density, act, dtype):
    """The expert-major path at the widths of GPT-2 medium / BERT-large / ViT-L (D = 1024) and GPT-2 large (D = 1280): against
    the float64 oracle (row slices at 20 000 tokens) and the tiled products, single-expert / no-expert / all-expert
    tokens, weighted routing + residual, run-to-run bit equality, and the over-capacity fall-back, which at these widths
    is the tiled products working behind the plan in the same workspace."""
    _say('experts sparse wide', N, D, E, Ed, density, act, dtype)
    tol = H.tol_for(dtype)
    x, routing, p = H.random_case(N, D, E, Ed, 8, seed=N + D + E, dtype=dtype, density=density)
    if N > 4:
        routing[1] = 0
        routing[2] = 0
        routing[2, E // 2] = 1
        routing[3] = 1
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, 0, 1 if dtype == torch.bfloat16 else 2, act)
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    assert packed is not None
    got = _experts_got(x, routing, p, act, path='mfma_sparse', packed=packed)
    rows = slice(0, N) if N <= 4096 else slice(N - 2500, N)
    assert H.rel_err(got[rows], _experts_want(x[rows], routing[rows], p, act)) < tol
    assert torch.equal(got, _experts_got(x, routing, p, act, path='mfma_sparse', packed=packed))
    if N > 16:
        assert H.rel_err(got, _experts_got(x, routing, p, act, path='mfma_gemm', packed=packed)) < tol
    if N <= 4096:
        g = torch.Generator().manual_seed(5)
        weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).to(dtype)
        got = _experts_got(x, weights, p, act, residual=True, path='mfma_sparse', packed=packed)
        assert H.rel_err(got, _experts_want(x, weights, p, act, True)) < tol
        dense_routing = (torch.rand(N, E, generator=g) < 0.6).to(dtype)   # beyond the capacity
        got = _experts_got(x, dense_routing, p, act, path='mfma_sparse', packed=packed)
        assert H.rel_err(got, _experts_want(x, dense_routing, p, act)) < tol


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('N,E,Ed', [(1200, 512, 32), (700, 320, 24), (600, 256, 64)])
def test_experts_mfma_sparse_d768_without_a_fused_sweep(N, E, Ed, dtype):
    """D = 768 layers the fused sweep does not cover (more than 256 experts, more than 8192 hidden neurons): the
    expert-major path's device-side fall-back is the tiled products working behind the plan in the same workspace, whose
    size the query must cover.  Sparse routing (expert-major kernels) and dense routing (fall-back) against the oracle."""
    _say('experts sparse D=768, no sweep', N, E, Ed, dtype)
    tol = H.tol_for(dtype)
    x, routing, p = H.random_case(N, 768, E, Ed, 8, seed=N + E, dtype=dtype, density=4.0 / E)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, 768, E, Ed, 0, 1 if dtype == torch.bfloat16 else 2, 'relu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    assert packed is not None
    got = _experts_got(x, routing, p, 'relu', path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _experts_want(x, routing, p, 'relu')) < tol
    g = torch.Generator().manual_seed(3)
    dense_routing = (torch.rand(N, E, generator=g) < 0.5).to(dtype)   # far beyond the capacity: the fall-back runs
    got = _experts_got(x, dense_routing, p, 'relu', path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _experts_want(x, dense_routing, p, 'relu')) < tol
    assert torch.equal(got, _experts_got(x, dense_routing, p, 'relu', path='mfma_gemm', packed=packed))


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('D', [192, 384])
def test_layer_at_widths_with_a_router_section_only(D, dtype):
    """ViT-Tiny / ViT-Small widths (multiples of 64 but not of 256): the packed buffer holds the router section only; the
    layer runs the fused router kernel and the generic experts, through ops.forward and through the module."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    N, E, Ed, W = 394, 64, 4 * D // 64, 128
    _say('layer router-section-only', D, dtype)
    x, _, p = H.random_case(N, D, E, Ed, W, seed=D, dtype=dtype)
    d = H.to_dev(p, DEV)
    code = 1 if dtype == torch.bfloat16 else 2
    ops = _ops()
    assert ops.packed_bytes(ops.make_shape(0, D, E, Ed, 0, code)) == 0
    packed = ops.pack_weights(ops.make_shape(0, D, E, Ed, W, code), d['w1'], d['b1'], d['w2'], None, d['router_w1'],
                              d['router_w2'])
    assert packed is not None
    for tau in (0.9, 0.1):
        out, routing, norms, counts = ops.forward(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), d['w1'], d['b1'],
                                                  d['w2'], None, d['last_bias'].view(-1), 'relu', False, None, True, True, 'auto',
                                                  packed)
        assert torch.equal(routing.cpu(), O.gate_dynk_max(norms.cpu(), tau))
        assert torch.equal(counts.cpu().long(), (routing.cpu() > 0).sum(0))
        want = O.layer_from_routing(x.double(), O.upcast(p), routing.cpu().double(), 'relu', 'all')
        assert H.rel_err(out.cpu(), want) < H.tol_for(dtype)
    moe = MoeficationMoE('mlp', D, E, True, Ed, torch.nn.ReLU, experts_class='custom_kernel')
    moe.router = MoeficationRouter(D, E, width=W, depth=2, bias=False, activation='relu', output_activation='abs')
    moe = moe.to(DEV).to(dtype).eval()
    moe.forward_mode, moe.tau = 'dynk_max', 0.9
    moe.experts.forward_mode = 'hip'
    with torch.no_grad():
        out, gating = moe(x.to(DEV).view(2, N // 2, D))
    (routing,) = gating['mlp']
    q = {'w1': moe.experts.w1, 'b1': moe.experts.b1, 'w2': moe.experts.w2, 'last_bias': moe.last_bias}
    q = {k: v.detach().cpu() for k, v in q.items()}
    want = O.layer_from_routing(x.double(), O.upcast(q), routing.view(N, E).cpu().double(), 'relu', 'all')
    assert H.rel_err(out.view(N, D).cpu(), want) < H.tol_for(dtype)


@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_layer_wide_model_auto(tau):
    """Whole layer at D = 1024 (128 experts x 32, GELU) under AUTO at 2000 tokens: the literal rule takes the expert-major
    path, the module reading the tiled products; mask exact for the kernel's own norms, output against the oracle."""
    N, D, E, Ed, W = 2000, 1024, 128, 32, 128
    _say('layer wide', tau)
    x, _, p = H.random_case(N, D, E, Ed, W, seed=21, dtype=torch.bfloat16)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, 'gelu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    out, routing, norms, counts = _ops().forward(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), d['w1'], d['b1'],
                                                 d['w2'], None, d['last_bias'].view(-1), 'gelu', False, None, True, True, 'auto',
                                                 packed)
    assert torch.equal(routing.cpu(), O.gate_dynk_max(norms.cpu(), tau))
    assert torch.equal(counts.cpu().long(), (routing.cpu() > 0).sum(0))
    assert H.rel_err(out.cpu(), _experts_want(x, routing.cpu(), p, 'gelu')) < H.TOL_BF16


@pytest.mark.parametrize('act', ['relu', 'gelu', 'tanh'])
def test_experts_mfma_sparse_activations_weights_edges(act):
    x, routing, p = H.random_case(500, 768, 128, 24, 8, seed=41, dtype=torch.bfloat16, density=0.03)
    packed = _packed_for(p, act)
    got = _experts_got(x, routing, p, act, residual=True, path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _experts_want(x, routing, p, act, True)) < H.TOL_BF16
    g = torch.Generator().manual_seed(2)
    weights = (routing.float() * (torch.rand(500, 128, generator=g) + 0.5)).bfloat16()
    got = _experts_got(x, weights, p, act, path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _experts_want(x, weights, p, act)) < H.TOL_BF16
    # nothing routed -> last_bias only; a single expert taking every token (maximal skew)
    got = _experts_got(x, torch.zeros_like(routing), p, act, path='mfma_sparse', packed=packed)
    assert torch.equal(got, p['last_bias'].expand(500, -1))
    one = torch.zeros_like(routing)
    one[:, 77] = 1
    got = _experts_got(x, one, p, act, path='mfma_sparse', packed=packed)
    assert H.rel_err(got, _experts_want(x, one, p, act)) < H.TOL_BF16
    # tokens with ONE routed expert are finished inside the experts kernel: weighted, with the residual, without last_bias
    lone = torch.zeros_like(routing)
    lone[torch.arange(500), torch.arange(500) % 128] = 0.75
    lone[::7, 5] = 1.0   # some tokens get a second expert and go through the combine kernel
    q = {k: v for k, v in p.items() if k != 'last_bias'}
    got = _experts_got(x, lone, q, act, residual=True, path='mfma_sparse', packed=_packed_for(q, act))
    assert H.rel_err(got, _experts_want(x, lone, q, act, True)) < H.TOL_BF16


def test_experts_mfma_sparse_full_size_and_auto_switch():
    """50432 tokens with ~2 experts per token: the oracle on slices of rows, the dense sweep on all rows; and the
    whole-layer call picks the expert-major path by itself for a high threshold fraction."""
    N = 50432
    x, routing, p = H.random_case(N, 768, 128, 24, 128, seed=51, dtype=torch.bfloat16, density=0.0165)
    packed = _packed_for(p, with_router=True)
    d = H.to_dev(p, DEV)
    xg, rg = x.to(DEV), routing.to(DEV)
    lb = d['last_bias'].view(-1)
    a = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_sparse', packed)
    b = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', False, 'mfma_dense', packed)
    assert H.rel_err(a, b) < 1e-2
    rows = torch.cat([torch.arange(0, 128), torch.arange(25000, 25064), torch.arange(N - 64, N)])
    assert H.rel_err(a.cpu()[rows], _experts_want(x[rows], routing[rows], p, 'relu')) < H.TOL_BF16
    assert H.elem_err(a.cpu()[rows], _experts_want(x[rows], routing[rows], p, 'relu')) < H.TOL_BF16
    out_auto, r_auto, _, _ = _ops().forward(xg, d['router_w1'], d['router_w2'], 0.9, d['w1'], d['b1'], d['w2'], None, lb,
                                            'relu', False, None, False, False, 'auto', packed)
    out_dense, r_dense, _, _ = _ops().forward(xg, d['router_w1'], d['router_w2'], 0.9, d['w1'], d['b1'], d['w2'], None, lb,
                                              'relu', False, None, False, False, 'mfma_dense', packed)
    assert torch.equal(r_auto, r_dense) and H.rel_err(out_auto, out_dense) < 1e-2
    want = O.layer_from_routing(x[rows].double(), O.upcast(p), r_auto.cpu()[rows].double(), 'relu', 'all')
    assert H.rel_err(out_auto.cpu()[rows], want) < H.TOL_BF16
    assert H.elem_err(out_auto.cpu()[rows], want) < H.TOL_BF16
def test_full_size_token_permutation_equivariance():
    """50432 tokens: a token's output does not depend on where in the batch it sits.  Expert-major path: bit-exact under
    a random permutation of the tokens (every token's sum runs over its experts in ascending order, whatever its
    neighbours).  Token-tile-major sweep: bit-exact for tokens that sit in full 64-token tiles before and after (the
    tail tiles add their chunk ranges' float32 sums in a second step, which may move the last bf16 bit), and within
    one bf16 ulp everywhere."""
    N = 50432
    g = torch.Generator().manual_seed(77)
    perm = torch.randperm(N, generator=g)
    x, routing, p = H.random_case(N, 768, 128, 24, 8, seed=78, dtype=torch.bfloat16, density=0.0165)
    packed = _packed_for(p)
    d = H.to_dev(p, DEV)
    lb = d['last_bias'].view(-1)
    xg, rg, pg = x.to(DEV), routing.to(DEV), perm.to(DEV)
    xp, rp = xg[pg].contiguous(), rg[pg].contiguous()
    a = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', True, 'mfma_sparse', packed)
    b = _ops().experts(xp, rp, d['w1'], d['b1'], d['w2'], None, lb, 'relu', True, 'mfma_sparse', packed)
    assert torch.equal(a[pg], b)
    x2, routing2, _ = H.random_case(N, 768, 128, 24, 8, seed=79, dtype=torch.bfloat16, density=0.79)
    xg, rg = x2.to(DEV), routing2.to(DEV)
    xp, rp = xg[pg].contiguous(), rg[pg].contiguous()
    a = _ops().experts(xg, rg, d['w1'], d['b1'], d['w2'], None, lb, 'relu', True, 'mfma_dense', packed)
    b = _ops().experts(xp, rp, d['w1'], d['b1'], d['w2'], None, lb, 'relu', True, 'mfma_dense', packed)
    full = (N // (64 * 256)) * 64 * 256          # tokens in whole rounds of 64-token tiles on 256 CUs at most
    pos_after = torch.empty(N, dtype=torch.long, device=DEV)
    pos_after[pg] = torch.arange(N, device=DEV)   # token n sits at row pos_after[n] of the permuted batch
    both_full = (torch.arange(N, device=DEV) < full) & (pos_after < full)
    assert both_full.float().mean() > 0.8
    assert torch.equal(a[both_full], b[pos_after[both_full]])
    diff = (a.float() - b[pos_after].float()).abs()
    assert (diff <= a.float().abs() * 2 ** -7 + 1e-6).all()


def test_packed_weights_cache_tracks_parameter_updates():
    from d2dmoe_amd import HipKernelExperts
    torch.manual_seed(0)
    ex = HipKernelExperts(768, 128, 2, 24, 'without_last', torch.nn.ReLU).to(DEV).bfloat16()
    ex.forward_mode = 'hip'
    x = torch.randn(70, 768, device=DEV, dtype=torch.bfloat16)
    r = (torch.rand(70, 128, device=DEV) < 0.5).bfloat16()
    with torch.no_grad():
        a = ex(x, r)
        assert ex._packed.slots[False][1] is not None
        ex.w2.mul_(2.0)           # in-place update bumps the version counter -> repack
        b = ex(x, r)
    assert H.rel_err(b, 2 * a.float()) < 1e-2


# =================================================================== fused router + select (MFMA) =====
@pytest.mark.parametrize('N', [16384, 16385, 50432, 50401])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_router_select_resident(N, dtype):
    """From 16 384 tokens on, the ViT-B router runs with its weights resident in registers and x staged through LDS
    (one workgroup per CU walking the tiles).  Checked: the mask is the oracle's gate applied to the kernel's own
    norms; the counts are the column sums of the mask; a token's result does not depend on where it stands in the
    batch (bit-exact under a permutation of the tokens); and, since every kernel accumulates over K in ascending order,
    the rows equal, bit for bit, what the tiled kernels (one wave or one workgroup per 32 tokens) give on slices."""
    _say('router resident', N, dtype)
    D, W, E, Ed = 768, 128, 128, 24
    x, _, p = H.random_case(N, D, E, Ed, W, seed=N, dtype=dtype)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1 if dtype == torch.bfloat16 else 2, 'relu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    xd = x.to(DEV)
    want64 = O.router_forward(x[:4096].double(), p['router_w1'].double(), p['router_w2'].double())
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(N)).to(DEV)
    for thr in (0.1, 0.9):
        r, n, c = _ops().router_select(xd, d['router_w1'], d['router_w2'], thr, packed, E, Ed, True, True)
        assert torch.equal(c.long(), (r > 0).sum(0))
        assert torch.equal(r.cpu(), O.gate_dynk_max(n.cpu(), 1.0 - thr))
        assert H.rel_err(n[:4096].cpu(), want64) < (H.TOL_BF16 if dtype == torch.bfloat16 else H.TOL_F16)
        rp, np_, cp = _ops().router_select(xd[perm].contiguous(), d['router_w1'], d['router_w2'], thr, packed, E, Ed, True, True)
        assert torch.equal(np_, n[perm]) and torch.equal(rp, r[perm]) and torch.equal(cp, c)
        for lo, hi in ((0, 4096), (N - 12001, N), (5000, 5033)):
            r2, n2, _ = _ops().router_select(xd[lo:hi].contiguous(), d['router_w1'], d['router_w2'], thr, packed, E, Ed, True, True)
            assert torch.equal(n[lo:hi], n2) and torch.equal(r[lo:hi], r2), (lo, hi)
    # without the optional outputs
    r3, n3, c3 = _ops().router_select(xd, d['router_w1'], d['router_w2'], 0.9, packed, E, Ed, False, False)
    assert n3 is None and c3 is None and torch.equal(r3, r)


@pytest.mark.parametrize('N,D,W,E', [(197, 768, 128, 128), (1, 768, 128, 128), (33, 768, 128, 128), (1576, 768, 128, 128),
                                     (50432, 768, 128, 128), (16, 2048, 256, 256), (300, 2048, 256, 256),
                                     (8191, 768, 128, 128), (4100, 2048, 256, 256),
                                     (1576, 768, 128, 24), (50432, 768, 128, 24), (300, 768, 128, 64), (700, 1024, 128, 200),
                                     (33, 1280, 128, 160), (500, 2048, 256, 96), (1, 768, 128, 8)])
@pytest.mark.parametrize('tau', [0.1, 0.9])
def test_router_select_mfma(N, D, W, E, tau):
    """Fused router + selection: norms within tolerance of the float64 router, mask bit-exact for the kernel's own
    norms (stage-wise exactness), counts exact, and few mask flips against the oracle's bf16 router.  Expert counts
    other than the router's hidden width (any multiple of 8 up to 256: the reference benchmark's 24, 64, 96, 160, 200)
    run on zero-padded tiles of 32 experts."""
    _say('router+select mfma', N, D, W, E, tau)
    Ed = 24 if D == 768 else 8
    x, _, p = H.random_case(N, D, E, Ed, W, seed=N + D, dtype=torch.bfloat16)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, 'relu')
    packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    assert packed is not None
    out, routing, norms, counts = _ops().forward(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), d['w1'],
                                                 d['b1'], d['w2'], None, None, 'relu', False, None, True, True, 'auto', packed)
    want64 = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    assert H.rel_err(norms.cpu(), want64) < H.TOL_BF16
    assert torch.equal(routing.cpu(), O.gate_dynk_max(norms.cpu(), tau))
    assert torch.equal(counts.cpu().long(), routing.cpu().float().sum(0).long())
    # the stand-alone entry point runs the same fused kernel
    r2, n2, c2 = _ops().router_select(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), packed, E, Ed, True, True)
    assert torch.equal(r2, routing) and torch.equal(n2, norms) and torch.equal(c2, counts)
    # ... and without the packed buffer it composes the generic router and select kernels
    r3, n3, c3 = _ops().router_select(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), None, E, Ed, True, True)
    assert torch.equal(r3.cpu(), O.gate_dynk_max(n3.cpu(), tau)) and torch.equal(c3.cpu().long(), r3.cpu().float().sum(0).long())
    # the generic (non-MFMA) HIP router rounds at the same points; both masks come from the same rule
    norms_g = _ops().router(x.to(DEV), d['router_w1'], d['router_w2'])
    assert (norms_g.float() - norms.float()).abs().max() <= norms_g.float().abs().max() * 2 ** -7
    flips = (routing.cpu() != O.gate_dynk_max(O.router_forward(x, p['router_w1'], p['router_w2']), tau)).float().mean().item()
    _say(f'  mask flips vs oracle bf16 router: {flips:.2e}')
    assert flips < 2e-2
    if N <= 2000:
        want = O.layer_from_routing(x.double(), O.upcast({k: v for k, v in p.items() if k != 'last_bias'}),
                                    routing.cpu().double(), 'relu', 'all')
        assert H.rel_err(out.cpu(), want) < H.TOL_BF16


# =================================================================== small-batch (decode) path ========
@pytest.mark.parametrize('N', [1, 5, 16, 17, 40, 48])
@pytest.mark.parametrize('D,E,Ed,W,gated,act', [(2048, 256, 64, 256, True, 'gelu_tanh'), (2048, 256, 64, 256, True, 'relu'),
                                               (768, 128, 24, 128, False, 'relu'), (768, 24, 128, 128, False, 'gelu'),
                                               (1024, 16, 32, 128, True, 'silu')])
def test_decode_path_matches_oracle(N, D, E, Ed, W, gated, act):
    """16 tokens per pass, at most three passes: one workgroup per expert streams its packed weights; the Gemma-2B FFN is
    the first shape.  AUTO takes the path up to 16 tokens, for gated experts up to 48."""
    _say('decode', N, D, E, Ed, gated, act)
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=N + E, dtype=torch.bfloat16, gated=gated, bias=not gated, density=0.7)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, act, gated=gated)
    if gated:
        packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    else:
        packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    assert packed is not None
    got = _experts_got(x, routing, p, act, path='mfma_decode', packed=packed)
    assert H.rel_err(got, _experts_want(x, routing, p, act)) < H.TOL_BF16
    assert H.rel_err(got, _experts_got(x, routing, p, act, path='generic')) < 1e-2
    if N <= 16 or gated:
        assert torch.equal(got, _experts_got(x, routing, p, act, path='auto', packed=packed))
    # nothing routed / one expert for everybody / weighted routing
    zero = _experts_got(x, torch.zeros_like(routing), p, act, path='mfma_decode', packed=packed)
    lbias = p['last_bias'].expand(N, -1).float() if 'last_bias' in p else torch.zeros(N, D)
    assert torch.equal(zero.float(), lbias)
    g = torch.Generator().manual_seed(3)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).bfloat16()
    got = _experts_got(x, weights, p, act, residual=True, path='mfma_decode', packed=packed)
    assert H.rel_err(got, _experts_want(x, weights, p, act, True)) < H.TOL_BF16
    # whole layer: skinny router kernels + select + decode experts
    out, r, norms, counts = _forward(x, p, 0.9, act, packed=packed)
    want64 = O.router_forward(x.double(), p['router_w1'].double(), p['router_w2'].double())
    assert H.rel_err(norms.cpu(), want64) < H.TOL_BF16
    assert torch.equal(r.cpu(), O.gate_dynk_max(norms.cpu(), 0.9))
    want = O.layer_from_routing(x.double(), O.upcast(p), r.cpu().double(), act, 'all')
    assert H.rel_err(out.cpu(), want) < H.TOL_BF16


@pytest.mark.parametrize('N', [1, 7, 16])
@pytest.mark.parametrize('D,E,Ed,W,gated,act', [(2048, 256, 64, 256, True, 'gelu_tanh'), (768, 128, 24, 128, False, 'relu')])
@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_small_batch_layer_equals_staged_calls(N, D, E, Ed, W, gated, act, tau):
    """d2dmoe_forward runs a layer of at most 16 tokens as two launches (first router layer beside the experts' first
    layer; second router layer and selection inside the output kernel).  Norms, routing, counts and outputs must be the
    bits the stand-alone entry points produce: router -> select -> experts."""
    _say('small batch layer vs staged', N, D, E, gated, tau)
    x, _, p = H.random_case(N, D, E, Ed, W, seed=3 * N + E, dtype=torch.bfloat16, gated=gated, bias=not gated)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, act, gated=gated)
    if gated:
        packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    else:
        packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    out, routing, norms, counts = _forward(x, p, tau, act, packed=packed, residual=True)
    xd = x.to(DEV)
    norms2 = _ops().router(xd, d['router_w1'], d['router_w2'])
    routing2, counts2 = _ops().select(norms2, float(1.0 - tau), want_counts=True)
    assert torch.equal(norms, norms2)
    assert torch.equal(routing, routing2)
    assert torch.equal(counts, counts2)
    out2 = _experts_got(x, routing2.cpu(), p, act, residual=True, path='mfma_decode', packed=packed)
    assert torch.equal(out.cpu(), out2)
    assert torch.equal(routing.cpu(), O.gate_dynk_max(norms.cpu(), tau))


@pytest.mark.parametrize('N,D,E,Ed,W,gated,act', [(16, 2048, 256, 64, 256, True, 'gelu_tanh'), (3, 2048, 256, 64, 256, True, 'gelu_tanh'),
                                                  (16, 768, 128, 24, 128, False, 'relu')])
def test_small_batch_layer_back_to_back_calls_keep_their_bits(N, D, E, Ed, W, gated, act):
    """The output kernel's workgroups each sum a range of experts and the last to arrive adds the ranges; the arrival
    counters and the partial sums live in the workspace and are reused by the next call.  150 calls on two alternating
    inputs with no host synchronisation in between: every result must be the bits of the first call on that input (a sum
    that picked up another call's partials, or a counter left over, would show)."""
    _say('small batch back to back', N, D, E, gated)
    xa, _, p = H.random_case(N, D, E, Ed, W, seed=11 + N, dtype=torch.bfloat16, gated=gated, bias=not gated)
    xb = torch.roll(xa, 1, dims=1).contiguous()
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, act, gated=gated)
    if gated:
        packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    else:
        packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    lb = d['last_bias'].view(-1) if 'last_bias' in d else None

    def layer(x):
        if gated:
            return _ops().forward(x, d['router_w1'], d['router_w2'], 0.1, d['w_gate'], None, d['w_down'], d['w_up'], lb, act,
                                  True, None, True, True, 'auto', packed)
        return _ops().forward(x, d['router_w1'], d['router_w2'], 0.1, d['w1'], d['b1'], d['w2'], None, lb, act, True, None,
                              True, True, 'auto', packed)

    xs = {'a': xa.to(DEV), 'b': xb.to(DEV)}
    first = {name: layer(x) for name, x in xs.items()}
    torch.cuda.synchronize()
    assert not torch.equal(first['a'][0], first['b'][0])
    for name, x in (('a', xa), ('b', xb)):
        want = O.layer_from_routing(x.double(), O.upcast(p), first[name][1].cpu().double(), act, 'all', True)
        assert H.rel_err(first[name][0].cpu(), want) < H.TOL_BF16
    got = [('ab'[i & 1], layer(xs['ab'[i & 1]])) for i in range(150)]
    torch.cuda.synchronize()
    for name, res in got:
        for a, b in zip(res, first[name]):
            assert torch.equal(a, b)


# =================================================================== tiled products (gated, or ungated at other widths) ===
@pytest.mark.parametrize('N,D,E,Ed,W,act,gated', [(300, 256, 6, 24, 128, 'silu', True), (700, 512, 16, 64, 128, 'relu', True),
                                                  (257, 1024, 5, 128, 128, 'gelu', True), (9000, 256, 4, 32, 128, 'gelu_tanh', True),
                                                  (1030, 2048, 256, 64, 256, 'gelu_tanh', True),
                                                  (300, 1024, 16, 48, 128, 'relu', False), (530, 768, 128, 24, 128, 'gelu', False),
                                                  (40, 1280, 7, 32, 128, 'leaky_relu', False)])
@pytest.mark.parametrize('dtype', DTYPES)
def test_tiled_products_path_matches_oracle(N, D, E, Ed, W, act, gated, dtype):
    """More than 16 tokens: up product with the routing value as a factor, hidden activations kept as fragments, down
    product with K splits.  Gated experts (the Gemma-2B FFN is the fifth shape) and ungated experts with bias at widths
    the fused sweep is not built for (GPT-2 medium / large, BERT-large) or, on request, at 768.  9000 tokens take two
    passes of the token slab."""
    _say('tiled products', N, D, E, Ed, act, gated, dtype)
    tol = H.TOL_F32 if dtype == torch.float32 else H.TOL_BF16
    x, routing, p = H.random_case(N, D, E, Ed, W, seed=N + E, dtype=dtype, gated=gated, bias=not gated, density=0.7)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 0 if dtype == torch.float32 else 1, act, gated=gated)
    if gated:
        packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    else:
        packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
    assert packed is not None
    rows = torch.arange(N) if N * E * D * Ed < 2e10 else torch.cat([torch.arange(40), torch.arange(N - 40, N)])
    got = _experts_got(x, routing, p, act, path='mfma_gemm', packed=packed)
    assert H.rel_err(got[rows], _experts_want(x[rows], routing[rows], p, act)) < tol
    if dtype == torch.float32 or gated or D not in (768, 1024):   # AUTO picks it for N > 16 unless the fused sweep covers the shape
        assert torch.equal(got, _experts_got(x, routing, p, act, path='auto', packed=packed))
    if N <= 1100 and D <= 1280:
        assert H.rel_err(got, _experts_got(x, routing, p, act, path='generic')) < (1e-2 if dtype == torch.bfloat16 else 1e-5)
    # nothing routed -> last_bias only (zeros for gated experts, which carry no biases); weighted routing + residual
    zero = _experts_got(x, torch.zeros_like(routing), p, act, path='mfma_gemm', packed=packed)
    lbias = p['last_bias'].expand(N, -1).float() if 'last_bias' in p else torch.zeros(N, D)
    assert torch.equal(zero.float(), lbias)
    g = torch.Generator().manual_seed(3)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).to(dtype)
    got = _experts_got(x, weights, p, act, residual=True, path='mfma_gemm', packed=packed)
    assert H.rel_err(got[rows], _experts_want(x[rows], weights[rows], p, act, True)) < tol
    # run-to-run reproducibility: fixed summation order, no atomics
    assert torch.equal(got, _experts_got(x, weights, p, act, residual=True, path='mfma_gemm', packed=packed))


@pytest.mark.parametrize('N,E,Ed,density,act', [(300, 16, 64, 0.15, 'gelu_tanh'), (4096, 256, 64, 0.009, 'gelu_tanh'),
                                                (77, 8, 40, 0.3, 'relu'), (1, 4, 64, 0.5, 'silu'), (33, 40, 64, 0.05, 'gelu_tanh'),
                                                (200, 64, 64, 0.7, 'gelu_tanh'), (200, 16, 64, 0.7, 'gelu_tanh'),
                                                (16400, 16, 64, 0.2, 'gelu_tanh')])
def test_gated_expert_major_path_matches_oracle(N, E, Ed, density, act):
    """Gated experts at D = 2048 with few experts per token: plan -> per-expert gated kernel -> ordered combine.  The
    last but one case routes 45 pairs per token, more than the 32 the path is provisioned for; the device-side flag then
    hands the call to the tiled products, which work in the same workspace.  The next (11 per token) stays expert-major;
    the last has more than 16 384 tokens, where the capacity is 8 per token and the fall-back runs in three passes."""
    _say('gated expert-major', N, E, Ed, density, act)
    D = 2048
    x, routing, p = H.random_case(N, D, E, Ed, 64, seed=N + E, dtype=torch.bfloat16, gated=True, bias=False, density=density)
    routing[0] = 0
    routing[0, E - 1] = 1            # a token with a single expert
    if N > 2:
        routing[2] = 0               # a token with none: zeros (gated experts carry no biases)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, 64, 1, act, gated=True)
    packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    assert packed is not None
    rows = torch.arange(N) if N <= 400 else torch.cat([torch.arange(64), torch.arange(N - 64, N)])
    got = _experts_got(x, routing, p, act, path='mfma_sparse', packed=packed)
    assert H.rel_err(got[rows], _experts_want(x[rows], routing[rows], p, act)) < H.TOL_BF16
    if N > 2:
        assert torch.equal(got[2].float(), torch.zeros(D))
    assert torch.equal(got, _experts_got(x, routing, p, act, path='mfma_sparse', packed=packed))   # deterministic
    # against the tiled products on every row
    assert H.rel_err(got, _experts_got(x, routing, p, act, path='mfma_gemm', packed=packed)) < 1e-2
    # weighted routing + residual
    g = torch.Generator().manual_seed(5)
    weights = (routing.float() * (torch.rand(N, E, generator=g) + 0.5)).to(torch.bfloat16)
    got = _experts_got(x, weights, p, act, residual=True, path='mfma_sparse', packed=packed)
    assert H.rel_err(got[rows], _experts_want(x[rows], weights[rows], p, act, True)) < H.TOL_BF16


def test_gated_layer_takes_the_expert_major_path_for_a_high_threshold():
    """Whole gated layer at the Gemma shape, 4096 tokens, keep norm >= 0.9 * max: AUTO plans on the device and runs the
    expert-major kernels; the result equals the tiled products' on the same routing within the bf16 tolerance."""
    N, D, E, Ed, W = 4096, 2048, 256, 64, 256
    x, _, p = H.random_case(N, D, E, Ed, W, seed=7, dtype=torch.bfloat16, gated=True, bias=False)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, 'gelu_tanh', gated=True)
    packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    out_a, r_a, _, _ = _forward(x, p, 0.1, 'gelu_tanh', path='auto', packed=packed)
    out_g, r_g, _, _ = _forward(x, p, 0.1, 'gelu_tanh', path='mfma_gemm', packed=packed)
    assert torch.equal(r_a, r_g)
    assert 1.0 <= r_a.float().sum(1).mean().item() < 8.0
    assert H.rel_err(out_a, out_g) < 1e-2
    rows = torch.cat([torch.arange(48), torch.arange(N - 48, N)])
    want = O.layer_from_routing(x[rows].double(), O.upcast(p), r_a.cpu()[rows].double(), 'gelu_tanh', 'all')
    assert H.rel_err(out_a.cpu()[rows], want) < H.TOL_BF16


@pytest.mark.parametrize('N', [17, 40, 48, 49, 100, 128, 129])
@pytest.mark.parametrize('tau', [0.1, 0.9])
def test_gated_layer_between_small_batch_and_tiled_products(N, tau):
    """Whole gated layer at token counts where AUTO changes hands: small-batch kernels in passes of 16 (up to 48 tokens),
    expert-major kernels (up to 128 tokens whatever the routing, beyond that for a high threshold fraction), tiled products
    otherwise.  Outputs against the float64 oracle on the kernel's own routing; the routing against the oracle gate on
    the kernel's own norms."""
    D, E, Ed, W = 2048, 32, 64, 256
    x, _, p = H.random_case(N, D, E, Ed, W, seed=N, dtype=torch.bfloat16, gated=True, bias=False)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, 'gelu_tanh', gated=True)
    packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
    out, r, norms, counts = _forward(x, p, tau, 'gelu_tanh', path='auto', packed=packed)
    assert torch.equal(r.cpu(), O.gate_dynk_max(norms.cpu(), tau))
    assert torch.equal(counts.cpu().long(), r.cpu().float().sum(0).long())
    want = O.layer_from_routing(x.double(), O.upcast(p), r.cpu().double(), 'gelu_tanh', 'all')
    assert H.rel_err(out.cpu(), want) < H.TOL_BF16


# =================================================================== whole layer ======================
def _forward(x, p, tau, act='relu', norms_in=None, path='auto', packed=None, residual=False):
    d = H.to_dev(p, DEV)
    lb = d['last_bias'].view(-1) if 'last_bias' in d else None
    x2 = x.reshape(-1, x.size(-1)).to(DEV)
    nin = None if norms_in is None else norms_in.reshape(-1, norms_in.size(-1)).to(DEV).contiguous()
    if 'w_gate' in d:
        return _ops().forward(x2, d['router_w1'], d['router_w2'], float(1.0 - tau), d['w_gate'], None, d['w_down'],
                              d['w_up'], lb, act, residual, nin, True, True, path, packed)
    return _ops().forward(x2, d['router_w1'], d['router_w2'], float(1.0 - tau), d['w1'], d.get('b1'), d['w2'], None, lb,
                          act, residual, nin, True, True, path, packed)


@pytest.mark.parametrize('case', ['toy', 'vit197', 'gpt64', 'gated16'])
@pytest.mark.parametrize('dtype', DTYPES)
def test_layer_against_golden_fixture(case, dtype):
    """Parity mode: the oracle's predicted norms go in, so every later stage must reproduce the fixture."""
    _say('fixture', case, dtype)
    fx, x, p, c = H.fixture_inputs(case, dtype)
    dt = 'f32' if dtype == torch.float32 else 'bf16'
    norms = O.router_forward(x, p['router_w1'], p['router_w2'])
    for tau in c['taus']:
        tag = f'{dt}_tau{tau}'
        out, routing, _, counts = _forward(x, p, tau, c['act'], norms_in=norms)
        want_r = H.routing_from_bits(fx[f'routing_bits_{tag}'], c['E'])
        assert torch.equal(routing.cpu().float(), want_r)
        assert torch.equal(counts.cpu().long(), want_r.sum(0).long())
        assert H.rel_err(out.cpu()[:32], torch.from_numpy(fx[f'out_{tag}'])) < H.tol_for(dtype)
        if dtype == torch.bfloat16 and c['D'] == 768:
            out_m, routing_m, _, _ = _forward(x, p, tau, c['act'], norms_in=norms, path='mfma_dense',
                                              packed=_packed_for(p, c['act']))
            assert torch.equal(routing_m, routing)
            assert H.rel_err(out_m.cpu()[:32], torch.from_numpy(fx[f'out_{tag}'])) < H.TOL_BF16
        off, tok, s, u, _ = _ops().build_permutation(routing, reference_layout=True)
        assert np.array_equal(off.cpu().numpy(), fx[f'offsets_{tag}'])
        assert np.array_equal(tok.cpu().numpy()[:int(off[-1])], fx[f'token_idx_{tag}'])
        assert hashlib.sha256(s.cpu().numpy().tobytes()).hexdigest() == str(fx[f'sort_crc_{tag}'])
        assert hashlib.sha256(u.cpu().numpy().tobytes()).hexdigest() == str(fx[f'unsort_crc_{tag}'])


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('tau', [0.1, 0.9])
def test_layer_end_to_end_vit_shape(dtype, tau):
    """Full path including the router on the GPU (the ViT-B shape the CPU baseline runs, 8 x 197 tokens).  The mask is a hard
    compare on router outputs, so a different accumulation order can flip entries that sit within rounding of the
    threshold; their number is reported and bounded, and outputs are compared on rows whose mask agrees."""
    _say('e2e', dtype, tau)
    N, D, E, Ed, W = 1576, 768, 128, 24, 128
    x, _, p = H.random_case(N, D, E, Ed, W, seed=77, dtype=dtype)
    packed = _packed_for(p, with_router=True) if dtype == torch.bfloat16 else None
    out, routing, norms, counts = _forward(x, p, tau, packed=packed)
    norms_o = O.router_forward(x, p['router_w1'], p['router_w2'])
    routing_o = O.gate_dynk_max(norms_o, tau)
    mism = (routing.cpu() != routing_o)
    frac = mism.float().mean().item()
    _say(f'  mask mismatches vs oracle router: {int(mism.sum())} of {N * E} ({frac:.2e})')
    assert frac < (1e-4 if dtype == torch.float32 else 2e-2)
    # stage-wise: the GPU mask is exactly the oracle's gate applied to the GPU's own norms
    assert torch.equal(routing.cpu(), O.gate_dynk_max(norms.cpu(), tau))
    assert torch.equal(counts.cpu().long(), routing.cpu().float().sum(0).long())
    want = O.layer_from_routing(x.double(), O.upcast(p), routing.cpu().double(), 'relu', 'all')
    assert H.rel_err(out.cpu(), want) < H.tol_for(dtype)
    assert H.elem_err(out.cpu(), want) < H.tol_for(dtype)
    same_rows = ~mism.any(dim=1)
    want_o = O.layer_from_routing(x.double(), O.upcast(p), routing_o.double(), 'relu', 'all')
    assert same_rows.float().mean() > 0.5
    assert H.rel_err(out.cpu()[same_rows], want_o[same_rows]) < H.tol_for(dtype)


def test_layer_skewed_norms_override():
    """The skewed-routing workload in miniature: the router is bypassed by synthetic predicted norms |N(0,1)| x Zipf(1.2)."""
    N, D, E, Ed = 2048, 768, 128, 24
    x, _, p = H.random_case(N, D, E, Ed, 128, seed=5, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(9)
    w = (torch.randperm(E, generator=g) + 1).float() ** -1.2
    norms = (torch.randn(N, E, generator=g).abs() * (w / w.max())).bfloat16()
    out, routing, _, counts = _forward(x, p, 1.0 - 0.9, norms_in=norms)
    want_r = O.gate_dynk_max_scaled(norms, 0.9)
    assert torch.equal(routing.cpu(), want_r)
    assert torch.equal(counts.cpu().long(), want_r.float().sum(0).long())
    want = O.layer_from_routing(x.double(), O.upcast(p), want_r.double(), 'relu', 'all')
    assert H.rel_err(out.cpu(), want) < H.TOL_BF16
    _say('  skew: max/mean tokens per expert =', (counts.max() / counts.float().mean()).item())


# =================================================================== module drop-in ===================
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('mode', ['naive', 'hip', 'triton_atomic'])
def test_module_modes_agree_and_do_not_sync(dtype, mode):
    """The reference's own check (scripts/test_moe_implementations.py:36-85): every forward mode against 'masked'
    on B=5, T=2, D=64, Ed=32, E=4, ReLU, dynk_max, tau=0.5; the kernel path must not synchronise with the host."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    for rep in range(3):
        torch.manual_seed(100 + rep)
        moe = MoeficationMoE('test_moe', 64, 4, True, 32, torch.nn.ReLU, experts_class='custom_kernel')
        moe.router = MoeficationRouter(64, 4, width=128, depth=2, bias=False, activation='relu', output_activation='abs')
        moe = moe.to(DEV).to(dtype).eval()
        moe.forward_mode = 'dynk_max'
        moe.tau = 0.5
        x = torch.randn(5, 2, 64, device=DEV, dtype=dtype)
        with torch.no_grad():
            want, gating = moe(x)
            moe.experts.forward_mode = mode
            moe(x)  # first call builds caches / workspaces
            if mode != 'naive':
                torch.cuda.set_sync_debug_mode('error')
            try:
                got, gating2 = moe(x)
            finally:
                torch.cuda.set_sync_debug_mode('default')
        assert torch.equal(gating['test_moe'][0], gating2['test_moe'][0])
        assert H.rel_err(got, want) < H.tol_for(dtype)


def test_module_execute_all_gated_hip():
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    torch.manual_seed(3)
    moe = MoeficationMoE('g', 256, 16, False, 64, torch.nn.GELU, experts_class='execute_all', add_intermediate_gating=True)
    moe.router = MoeficationRouter(256, 16, width=32, depth=2, bias=False, activation='relu', output_activation='abs')
    moe = moe.to(DEV).bfloat16().eval()
    moe.forward_mode, moe.tau = 'dynk_max', 0.9
    x = torch.randn(1, 16, 256, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        want, g1 = moe(x)
        moe.experts.forward_mode = 'hip'
        got, g2 = moe(x)
    assert torch.equal(g1['g'][0], g2['g'][0])
    assert H.rel_err(got, want) < 3e-2   # both sides are bf16 evaluations here


# =================================================================== GPT-2 model-level drop-in ========
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('shape', ['tiny', 'gpt2_width'])
def test_gpt_with_hip_moe_layers(shape, dtype):
    """Model surgery on the GPU: with every expert running, the MoE model (HIP experts) reproduces the dense model's
    logits; under dynk_max the fused layer returns the gating data of every block without a host synchronisation."""
    from d2dmoe_amd import add_routers, gpt2
    _say('gpt', shape, dtype)
    torch.manual_seed(0)
    if shape == 'tiny':
        cfg = gpt2.GPTConfig(block_size=32, vocab_size=96, n_layer=2, n_head=2, n_embd=64)
        kw, width = dict(expert_size=16), 16
    else:   # GPT-2-small width, MFMA kernels in bf16: 128 experts x 24 neurons, GELU, biases
        cfg = gpt2.GPTConfig(block_size=128, vocab_size=512, n_layer=2, n_head=12, n_embd=768)
        kw, width = dict(num_experts=128), 128
    model = gpt2.GPT(cfg).eval()
    with torch.no_grad():
        for n, prm in model.named_parameters():
            if n.endswith('bias'):
                prm.normal_(0.0, 0.05)
    model = model.to(DEV).to(dtype)
    moe, names = gpt2.replace_with_moes(model, experts_class='hip_kernel', **kw)
    gpt2.split_original_parameters(model, moe, names)
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode = 'all'
        layer.experts.forward_mode = 'hip'
    idx = torch.randint(0, cfg.vocab_size, (4, cfg.block_size), generator=torch.Generator().manual_seed(1)).to(DEV)
    with torch.no_grad():
        want = model.float()(idx) if dtype == torch.float32 else model(idx)
        got, gating = moe(idx, return_gating_data=True)
    tol = 2e-4 if dtype == torch.float32 else H.TOL_BF16
    assert H.rel_err(got.float().cpu(), want.float().cpu()) < tol
    assert set(gating) == set(names)
    # dynamic-k mode through the fused layer call
    add_routers(moe, dict(width=width, depth=2, bias=False, activation='relu', output_activation='abs'))
    moe = moe.to(DEV).to(dtype)
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode, layer.tau = 'dynk_max', 0.5
    # packing ahead of time: the buffers the first forward would build, and the forward then reuses them
    from d2dmoe_amd import prepack
    nbytes = prepack(moe)
    layers = [gpt2.get_module_by_name(moe, n) for n in names]
    if dtype == torch.bfloat16 and shape != 'tiny':
        assert nbytes > 0
    ahead = [layer.packed_weights() for layer in layers]
    assert nbytes == sum(pk.numel() * pk.element_size() for pk in ahead if pk is not None)
    with torch.no_grad():
        moe(idx)
        torch.cuda.synchronize()
    for layer, pk in zip(layers, ahead):
        now = layer.packed_weights()
        assert (now is None and pk is None) or now.data_ptr() == pk.data_ptr()
    with torch.no_grad():
        torch.cuda.set_sync_debug_mode('error')
        try:
            out, gating = moe(idx, return_gating_data=True)
        finally:
            torch.cuda.set_sync_debug_mode('default')
    frac = gating[names[-1]][0].float().mean().item()
    assert out.shape == (4, cfg.block_size, cfg.vocab_size) and 0.0 < frac < 1.0
    # cost accounting: executed (token, expert) pairs per layer from the kernel's own counters
    last = gpt2.get_module_by_name(moe, names[-1])
    last.collect_counts = True
    with torch.no_grad():
        _, gating = moe(idx, return_gating_data=True)
    assert torch.equal(last.last_expert_counts.long().cpu(), (gating[names[-1]][0] > 0).long().sum((0, 1)).cpu())
    assert torch.isfinite(out.float()).all()


# =================================================================== HIP graph capture ================
@pytest.mark.parametrize('case', ['vit_dense', 'vit_sparse', 'gemma_decode', 'gemma_tiled'])
def test_layer_replays_from_a_hip_graph(case):
    """The whole layer captured into a HIP graph (no allocation, memset or host sync inside the C ABI calls) and
    replayed on new inputs, with eager work and synchronisations between the replays: every replay equals eager."""
    _say('graph', case)
    if case.startswith('vit'):
        N, D, E, Ed, W, act, gated, tau = 300, 768, 128, 24, 128, 'relu', False, (0.9 if case == 'vit_dense' else 0.1)
    elif case == 'gemma_decode':
        N, D, E, Ed, W, act, gated, tau = 16, 2048, 256, 64, 256, 'gelu_tanh', True, 0.9
    else:
        N, D, E, Ed, W, act, gated, tau = 300, 2048, 256, 64, 256, 'gelu_tanh', True, 0.9
    x, _, p = H.random_case(N, D, E, Ed, W, seed=11, dtype=torch.bfloat16, gated=gated, bias=not gated)
    d = H.to_dev(p, DEV)
    sh = _ops().make_shape(0, D, E, Ed, W, 1, act, gated=gated)
    if gated:
        packed = _ops().pack_weights(sh, d['w_gate'], None, d['w_down'], d['w_up'], d['router_w1'], d['router_w2'])
        args = (d['w_gate'], None, d['w_down'], d['w_up'], None)
    else:
        packed = _ops().pack_weights(sh, d['w1'], d['b1'], d['w2'], None, d['router_w1'], d['router_w2'])
        args = (d['w1'], d['b1'], d['w2'], None, d['last_bias'].view(-1))

    def layer(inp):
        return _ops().forward(inp, d['router_w1'], d['router_w2'], float(1.0 - tau), *args, act, False, None, False, True,
                              'auto', packed)

    static_x = x.to(DEV).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            layer(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_routing, _, g_counts = layer(static_x)
    for rep in range(3):
        new_x = (torch.randn(N, D, generator=torch.Generator().manual_seed(100 + rep)) * (1.0 + rep)).bfloat16().to(DEV)
        want_out, want_routing, _, want_counts = layer(new_x)       # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(new_x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_routing, want_routing) and torch.equal(g_counts, want_counts), (case, rep)
        assert torch.equal(g_out, want_out), (case, rep)


# =================================================================== argument checks on real device pointers ==========
def test_entry_points_reject_bad_workspace_alignment_and_paths():
    """Status codes instead of launches: workspace too small or misaligned, tensor pointer off by 2 bytes, a path the
    shape has no kernel for, packed buffer missing for an MFMA path."""
    import ctypes
    from d2dmoe_amd import hip_abi as abi
    ops = _ops()
    lib = abi.load()
    N, D, E, Ed = 64, 768, 128, 24
    x, routing, p = H.random_case(N, D, E, Ed, 128, seed=3, dtype=torch.bfloat16)
    d = H.to_dev(p, DEV)
    xg, rg = x.to(DEV), routing.to(DEV)
    out = torch.empty_like(xg)
    sh = ops.make_shape(N, D, E, Ed, 0, abi.BF16)
    packed = ops.pack_weights(sh, d['w1'], d['b1'], d['w2'], None, None, None)
    need = lib.d2dmoe_workspace_bytes(ctypes.byref(sh))
    ws = torch.empty(need + 512, dtype=torch.uint8, device=DEV)
    base = ws.data_ptr() + (-ws.data_ptr()) % 256
    stream = torch.cuda.current_stream().cuda_stream

    def call(xp=xg.data_ptr(), path='mfma_sparse', wsp=base, wsb=need, pk=packed.data_ptr(), shape=sh):
        return lib.d2dmoe_experts(ctypes.byref(shape), xp, rg.data_ptr(), d['w1'].data_ptr(), d['b1'].data_ptr(),
                                  d['w2'].data_ptr(), None, None, pk, None if pk is None else ctypes.byref(packed.desc),
                                  out.data_ptr(), abi.PATH[path], wsp, wsb, stream)

    assert call() == 0
    assert call(wsb=1024) == -5                  # workspace too small for the expert-major plan
    assert call(wsp=base + 16) == -5             # workspace not 256-byte aligned
    assert call(xp=xg.data_ptr() + 2) == -7      # x not 16-byte aligned
    assert call(pk=None, path='mfma_dense') == -1
    assert call(path='mfma_decode') == -6        # more than 48 tokens
    f32 = ops.make_shape(N, D, E, Ed, 0, abi.F32)
    assert call(shape=f32, path='mfma_dense') == -9   # the buffer was packed for bf16
    assert call(shape=f32, path='mfma_dense', pk=None) == -6
    torch.cuda.synchronize()
    # the call that went through left a correct result behind
    assert H.rel_err(out.cpu(), _experts_want(x, routing, {k: v for k, v in p.items() if k != 'last_bias'}, 'relu')) < H.TOL_BF16


# ---------------------------------------------------------------------------------------------------------------------
# Router-training targets: per-expert output norms (reference: train_routers.py:49-86, utils.py:353-369)
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16], ids=['bf16', 'f16'])
@pytest.mark.parametrize('N,D,E,Ed,act', [(197, 768, 128, 24, 'relu'), (65, 768, 100, 30, 'gelu'), (1, 768, 7, 5, 'relu'),
                                          (300, 768, 16, 32, 'tanh'), (130, 768, 9, 24, 'leaky_relu'),
                                          # experts of 33-64 neurons (two slots of 32 each), other widths, 32-token tiles
                                          (150, 768, 24, 64, 'relu'), (70, 768, 5, 33, 'gelu'), (129, 1024, 128, 32, 'gelu'),
                                          (200, 1024, 19, 48, 'relu'), (97, 256, 11, 8, 'relu'), (64, 512, 16, 64, 'gelu'),
                                          (100, 1280, 40, 32, 'gelu'), (33, 2048, 12, 40, 'relu'), (31, 1536, 9, 16, 'tanh')])
def test_expert_output_norms_match_oracle(N, D, E, Ed, act, dtype):
    _say('expert output norms', N, D, E, Ed, act, dtype)
    tol = H.tol_for(dtype)
    x, _, p = H.random_case(N, D, E, Ed, 8, seed=N + E + 5, dtype=dtype)
    d = H.to_dev(p, DEV)
    got = _ops().expert_output_norms(x.to(DEV), d['w1'], d['b1'], d['w2'], act)
    assert got.shape == (E, N) and got.dtype == dtype
    q = O.upcast(p)
    want = O.expert_output_norms(x.double(), q['w1'], q['b1'], q['w2'], act)
    assert H.rel_err(got.cpu(), want) < tol
    # element-wise as well: a norm is a sum of squares, there is no cancellation to hide behind
    rel = ((got.cpu().double() - want).abs() / want.clamp_min(1e-3 * want.max().item())).max().item()
    assert rel < tol, rel
    # without the first-layer bias
    got = _ops().expert_output_norms(x.to(DEV), d['w1'], None, d['w2'], act)
    want = O.expert_output_norms(x.double(), q['w1'], None, q['w2'], act)
    assert H.rel_err(got.cpu(), want) < tol


@pytest.mark.gpu
@pytest.mark.parametrize('Ed', [24, 64])
def test_expert_output_norms_float16_second_layer_of_any_magnitude(Ed):
    """The Gram matrix of the second layer is stored in float16 scaled by a power of two per expert: second-layer
    weights whose squared row norms leave the float16 range at either end (the outputs themselves do not) give the norms
    of the oracle, each expert with a magnitude of its own."""
    N, D, E = 130, 768, 12
    _say('expert output norms, float16, scaled second layers', Ed)
    x, _, p = H.random_case(N, D, E, Ed, 8, seed=77, dtype=torch.float16)
    scale = torch.tensor([2.0 ** k for k in (-14, -10, -6, -2, 0, 1, 3, 5, 7, 9, 10, 11)]).view(E, 1, 1)
    w2 = p['w2'].float()
    w2 = w2 / w2.abs().amax(dim=(1, 2), keepdim=True) * scale     # largest entry of expert e: 2^k
    p['w2'] = w2.half()
    assert torch.isfinite(p['w2']).all()
    assert (p['w2'][-1].float().pow(2).sum(-1) > 65504).any() and (p['w2'][0].float().pow(2).sum(-1) < 6.1e-5).all()
    p['w1'] = (p['w1'].float() * 0.05).half()      # hidden activations small enough for the outputs to stay finite
    d = H.to_dev(p, DEV)
    got = _ops().expert_output_norms(x.to(DEV), d['w1'], d['b1'], d['w2'], 'relu').cpu()
    q = O.upcast(p)
    want = O.expert_output_norms(x.double(), q['w1'], q['b1'], q['w2'], 'relu')
    assert torch.isfinite(want.half()).all(), 'the case is meant to stay inside the float16 range'
    for e in range(E):    # per expert: every magnitude on its own scale
        big = want[e] > 6.2e-5        # normal float16 results
        assert big.any() or e < 2
        rel = ((got[e].double() - want[e]).abs()[big] / want[e][big]).max().item() if big.any() else 0.0
        assert rel < H.TOL_F16, (e, rel)
        assert ((got[e].double() - want[e]).abs()[~big] <= 2.0 ** -24 + H.TOL_F16 * want[e][~big]).all()


@pytest.mark.gpu
def test_expert_output_norms_module_method_and_full_size():
    from d2dmoe_amd import HipKernelExperts
    torch.manual_seed(0)
    ex = HipKernelExperts(768, 128, 2, 24, 'without_last', torch.nn.ReLU).to(DEV).bfloat16()
    with torch.no_grad():
        ex.b1.normal_(0.0, 0.1)
    N = 50432
    x = torch.randn(N, 768, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
    with torch.no_grad():
        got = ex.output_norms(x)                       # HIP kernel
        assert got.shape == (128, N)
        rows = torch.cat([torch.arange(0, 96), torch.arange(N - 70, N)]).to(DEV)
        ref = torch.linalg.vector_norm(ex.output_activation_extraction_stub(
            ex.intermediate_activation_extraction_stub(x[rows].unsqueeze(0), ex.w1, ex.b1, ex.act), ex.w2), ord=2, dim=-1)
        assert H.rel_err(got[:, rows].float().cpu(), ref.float().cpu()) < H.TOL_BF16
        want = O.expert_output_norms(x[rows].double().cpu(), ex.w1.double().cpu(), ex.b1.double().cpu(), ex.w2.double().cpu(), 'relu')
        assert H.rel_err(got[:, rows].cpu(), want) < H.TOL_BF16
        assert torch.equal(got, ex.output_norms(x))    # deterministic
        # the packed buffer follows parameter updates
        ex.w2.mul_(2.0)
        assert H.rel_err(ex.output_norms(x)[:, rows].cpu(), 2.0 * want) < H.TOL_BF16
        # float32 parameters: the reference's own route through the stubs
        ex32 = HipKernelExperts(768, 16, 2, 24, 'without_last', torch.nn.ReLU).to(DEV)
        x32 = x[:40].float()
        got32 = ex32.output_norms(x32)
        want32 = O.expert_output_norms(x32.double().cpu(), ex32.w1.double().cpu(), ex32.b1.double().cpu(), ex32.w2.double().cpu(), 'relu')
        assert H.rel_err(got32.cpu(), want32) < H.TOL_F32


@pytest.mark.gpu
def test_vit_with_hip_moe_layers():
    """ViT-B width on the GPU in bf16: 2 encoder blocks, 197 tokens per image; with every expert running the MoE model
    (HIP experts) reproduces the dense model's logits; under dynk_max the fused layers return their gating data."""
    from d2dmoe_amd import add_routers, gpt2, vit
    torch.manual_seed(0)
    m = vit.VisionTransformer(image_size=224, patch_size=16, num_layers=2, num_heads=12, hidden_dim=768, mlp_dim=3072,
                              num_classes=100).eval()
    with torch.no_grad():
        for n, prm in m.named_parameters():
            if n.endswith('bias'):
                prm.normal_(0.0, 0.05)
    m = m.to(DEV).bfloat16()
    moe, names = gpt2.replace_with_moes(m, num_experts=128, experts_class='hip_kernel')
    gpt2.split_original_parameters(m, moe, names)
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode = 'all'
        layer.experts.forward_mode = 'hip'
    x = torch.randn(4, 3, 224, 224, generator=torch.Generator().manual_seed(1)).to(DEV).bfloat16()
    with torch.no_grad():
        want = m(x)
        got, gating = moe(x, return_gating_data=True)
    assert H.rel_err(got.float().cpu(), want.float().cpu()) < H.TOL_BF16
    assert set(gating) == set(names) and tuple(gating[names[0]][0].shape) == (4, 197, 128)
    add_routers(moe, dict(width=128, depth=2, bias=False, activation='relu', output_activation='abs'))
    moe = moe.to(DEV).bfloat16()
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode, layer.tau = 'dynk_max', 0.5
    with torch.no_grad():
        out, gating = moe(x, return_gating_data=True)
    frac = gating[names[-1]][0].float().mean().item()
    assert out.shape == (4, 100) and 0.0 < frac < 1.0 and torch.isfinite(out.float()).all()
