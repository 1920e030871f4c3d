"""GPU parity of the module-level drop-in: every experts container of the registry on the HIP kernels, the gates other
than dynk_max feeding them, the gated (Gemma-shape) module on the product kernels, and the benchmark configurations at
their full sizes (GPT-2-small forward, skewed routing at 50 432 tokens).

Bars as in test_gpu_parity.py: masks bit-exact given the same predicted norms; outputs within 1e-5 (float32) / 2e-2
(bfloat16) of the float64 oracle, as max|got - want| / max|want| -- the per-element relative error is reported next to it.
"""
import pytest
import torch
from torch import nn

from oracle import d2dmoe_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

DEV = 'cuda:0'


def _say(*a):
    print(*a, flush=True)


def _ops():
    from d2dmoe_amd import ops
    return ops


def _gpu_ms(fn, reps=30, warm=5):
    """Median GPU time of fn() in milliseconds (events on torch's current stream, which the C ABI launches on)."""
    for _ in range(warm):
        fn()
    times = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    return sorted(times)[len(times) // 2]


def _layer_params(moe):
    """The module's weights as the oracle's parameter dictionary (CPU copies)."""
    w1, b1, w2, w_up, act = moe.experts.hip_operands()
    p = {}
    if w_up is not None:
        p.update(w_gate=w1, w_up=w_up, w_down=w2)
    else:
        p.update(w1=w1, w2=w2)
        if b1 is not None:
            p['b1'] = b1
    if moe.bias:
        p['last_bias'] = moe.last_bias
    if moe.router is not None:
        p.update(router_w1=moe.router.layers[0].weight, router_w2=moe.router.layers[2].weight)
    return {k: v.detach().cpu() for k, v in p.items()}, act


# =================================================================== gated module on the product kernels =========
@pytest.mark.parametrize('N', [16, 100, 4096])
@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_gated_module_reaches_the_product_kernels(N, tau):
    """MoeficationMoE(experts_class='execute_all', add_intermediate_gating=True) at the Gemma shape: the module's forward is
    the fused d2dmoe_forward with the packed weights (bit-equal to calling it directly) and agrees with the float64
    oracle; the cost of the module call and of the direct call are printed side by side."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    _say('gated module', N, tau)
    D, E, Ed, W = 2048, 256, 64, 256
    torch.manual_seed(11)
    moe = MoeficationMoE('mlp', D, E, False, Ed, H.GELUTanh, experts_class='execute_all', add_intermediate_gating=True)
    moe.router = MoeficationRouter(D, E, width=W, depth=2, bias=False, activation='relu', output_activation='abs')
    moe = moe.to(DEV).bfloat16().eval()
    moe.forward_mode, moe.tau = 'dynk_max', tau
    moe.experts.forward_mode = 'hip'
    x = torch.randn(1, N, D, generator=torch.Generator().manual_seed(N)).bfloat16().to(DEV)
    p, act = _layer_params(moe)
    assert act == 'gelu_tanh'
    with torch.no_grad():
        out, gating = moe(x)
        (routing,) = gating['mlp']
        packed = moe.packed_weights()
        assert packed is not None
        d = {k: v.to(DEV) for k, v in p.items()}

        def direct():
            return _ops().forward(x.view(N, D), d['router_w1'], d['router_w2'], float(1.0 - tau), d['w_gate'], None,
                                  d['w_down'], d['w_up'], None, act, False, None, True, False, 'auto', packed)
        out_d, routing_d, norms_d, _ = direct()
    assert torch.equal(routing.view(N, E), routing_d) and torch.equal(out.view(N, D), out_d)
    assert torch.equal(routing_d.cpu(), O.gate_dynk_max(norms_d.cpu(), tau))
    rows = torch.arange(N) if N <= 100 else torch.cat([torch.arange(40), torch.arange(N - 40, N)])
    want = O.layer_from_routing(x.view(N, D).cpu()[rows].double(), O.upcast(p), routing_d.cpu()[rows].double(), act, 'all')
    err = H.rel_err(out.view(N, D).cpu()[rows], want)
    _say(f'  experts/token {routing_d.float().sum(1).mean().item():.1f}, rel err {err:.2e}')
    assert err < H.TOL_BF16
    # cost: the module call against the direct call
    with torch.no_grad():
        t_mod = _gpu_ms(lambda: moe(x))
        t_dir = _gpu_ms(direct)
    # printed, not asserted: a parity run must not turn red on a slow box (path identity is the bit-equality above)
    _say(f'  module {t_mod * 1e3:.0f} us, direct {t_dir * 1e3:.0f} us')


# =================================================================== every container in its 'hip' mode =================
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('experts_class,gated', [('custom_kernel', False), ('execute_all', False), ('execute_all', True),
                                                 ('module', False), ('module', True), ('batched', False)])
def test_every_container_runs_the_hip_kernels(experts_class, gated, dtype):
    """Whole layer under dynk_max with each container of MOE_IMPL_MAP: 'hip' mode against the float64 oracle on the
    module's own weights, at a width the MFMA paths cover (D = 768 ungated, 2048 gated) and at an odd one."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    for D, E, Ed, N in ((2048, 16, 64, 70) if gated else (768, 128, 24, 70), (80, 6, 10, 33)):
        _say('container', experts_class, gated, dtype, D)
        torch.manual_seed(5)
        bias = not gated
        moe = MoeficationMoE('m', D, E, bias, Ed, nn.ReLU, experts_class=experts_class, add_intermediate_gating=gated)
        if bias:
            with torch.no_grad():
                moe.last_bias.normal_(0, 0.05)
                if experts_class == 'batched':
                    moe.experts.biases[0].uniform_(-0.1, 0.1)
        moe.router = MoeficationRouter(D, E, width=128, depth=2, bias=False, activation='relu', output_activation='abs')
        moe = moe.to(DEV).to(dtype).eval()
        moe.forward_mode, moe.tau = 'dynk_max', 0.6
        moe.experts.forward_mode = 'hip'
        x = torch.randn(2, N // 2, D, generator=torch.Generator().manual_seed(1)).to(dtype).to(DEV)
        with torch.no_grad():
            out, gating = moe(x)
            moe.collect_counts = True
            out2, _ = moe(x)
        routing = gating['m'][0].reshape(-1, E).cpu()
        assert torch.equal(out, out2)
        assert torch.equal(moe.last_expert_counts.cpu().long(), routing.float().sum(0).long())
        p, act = _layer_params(moe)
        want = O.layer_from_routing(x.reshape(-1, D).cpu().double(), O.upcast(p), routing.double(), act, 'all')
        assert H.rel_err(out.reshape(-1, D).cpu(), want) < H.tol_for(dtype)
        assert 0 < routing.sum() < routing.numel()


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_wide_model_layer_through_the_module(tau, dtype):
    """A converted FFN of GPT-2-medium / BERT-large width (D = 1024, 128 experts x 32, GELU) through MoeficationMoE in 'hip'
    mode, 2 x 1000 tokens: under the literal reading the fused call takes the expert-major kernels, under module tau 0.9
    the tiled products; mask from the oracle gate on the module's own norms, output against the float64 oracle."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    _say('wide module', tau, dtype)
    D, E, Ed = 1024, 128, 32
    torch.manual_seed(9)
    moe = MoeficationMoE('m', D, E, True, Ed, nn.GELU, experts_class='custom_kernel')
    with torch.no_grad():
        moe.last_bias.normal_(0, 0.05)
    moe.router = MoeficationRouter(D, E, width=128, depth=2, bias=False, activation='relu', output_activation='abs')
    moe = moe.to(DEV).to(dtype).eval()
    moe.forward_mode, moe.tau = 'dynk_max', tau
    moe.experts.forward_mode = 'hip'
    x = torch.randn(2, 1000, D, generator=torch.Generator().manual_seed(2)).to(dtype).to(DEV)
    with torch.no_grad():
        moe.collect_counts = True
        out, gating = moe(x)
    routing = gating['m'][0].reshape(-1, E).cpu()
    assert torch.equal(moe.last_expert_counts.cpu().long(), routing.float().sum(0).long())
    p, act = _layer_params(moe)
    norms = O.router_forward(x.reshape(-1, D).cpu(), p['router_w1'], p['router_w2'])
    flips = (routing != O.gate_dynk_max(norms, tau)).float().mean().item()
    assert flips < 2e-3
    want = O.layer_from_routing(x.reshape(-1, D).cpu().double(), O.upcast(p), routing.double(), act, 'all')
    assert H.rel_err(out.reshape(-1, D).cpu(), want) < H.tol_for(dtype)
    k = routing.sum(1).mean().item()
    assert (k < 8) if tau < 0.5 else (k > 50)


# =================================================================== the other gates feed the HIP experts (a3) ============
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('mode', ['all', 'topk', 'dynk'])
def test_other_gate_modes_feed_the_hip_experts(mode, dtype):
    """forward_mode 'all' / 'topk' / 'dynk' (moefication.py:56-79): the gate runs in PyTorch on the device, on router
    outputs from the HIP router kernel, and its routing tensor drives the HIP experts.  The mask equals the oracle's gate
    on the same predicted norms; the output is within tolerance of the float64 oracle."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    _say('gate', mode, dtype)
    D, E, Ed, N = 768, 128, 24, 394
    torch.manual_seed(8)
    moe = MoeficationMoE('m', D, E, True, Ed, nn.GELU, experts_class='custom_kernel')
    moe.router = MoeficationRouter(D, E, width=128, depth=2, bias=False, activation='relu', output_activation='abs')
    with torch.no_grad():
        moe.last_bias.normal_(0, 0.05)
    moe = moe.to(DEV).to(dtype).eval()
    moe.forward_mode, moe.k, moe.tau = mode, 7, 0.35
    moe.experts.forward_mode = 'hip'
    x = torch.randn(2, N // 2, D, generator=torch.Generator().manual_seed(2)).to(dtype).to(DEV)
    with torch.no_grad():
        out, gating = moe(x)
        norms = moe.router(x)
    routing = gating['m'][0].cpu()
    want_r = {'all': lambda: O.gate_all(x.cpu(), E), 'topk': lambda: O.gate_topk(norms.cpu(), 7),
              'dynk': lambda: O.gate_dynk(norms.cpu(), 0.35)}[mode]()
    if mode == 'topk':
        # ties inside a row may be broken differently on the device: the kept set has k entries, all >= the k-th value
        kth = norms.cpu().float().topk(7, dim=-1)[0][..., -1:]
        assert torch.equal(routing.sum(-1), torch.full(routing.shape[:-1], 7.0, dtype=routing.dtype))
        assert bool(((routing == 0) | (norms.cpu().float() >= kth)).all())
    elif mode == 'dynk':
        # The cumulative share is a running sum in the storage type; its last bits depend on the device's sort and scan,
        # so rows whose sum sits on tau can differ from the CPU gate (they are counted and reported).  What every valid
        # dynk mask satisfies, whatever the summation order: the kept experts are the largest shares, the largest one is
        # always kept, dropping the smallest kept share leaves less than tau, and a row that drops anything holds at
        # least tau -- the last two up to the rounding of a sum of E shares in the storage type.
        differing = (routing != want_r).any(-1).float().mean().item()
        _say(f'  dynk rows differing from the CPU gate: {differing:.2e}')
        if dtype == torch.float32:
            assert differing < 2e-2
        nd = norms.cpu().double()
        shares = (nd / nd.sum(-1, keepdim=True)).reshape(-1, E)
        kept = routing.reshape(-1, E) > 0
        eps = 1e-5 if dtype == torch.float32 else 2e-2
        big = torch.finfo(torch.float64).max
        min_kept = torch.where(kept, shares, torch.full_like(shares, big)).min(-1)[0]
        max_dropped = torch.where(kept, torch.full_like(shares, -1.0), shares).max(-1)[0]
        slack = 1e-6 if dtype == torch.float32 else 2.0 ** -6      # shares that tie after rounding to the storage type
        assert bool((kept.sum(-1) >= 1).all()) and bool((min_kept >= max_dropped * (1.0 - slack)).all())
        kept_sum = (shares * kept).sum(-1)
        assert bool((kept_sum - min_kept < 0.35 + eps).all())
        assert bool((kept.all(-1) | (kept_sum >= 0.35 - eps)).all())
    else:
        assert torch.equal(routing, want_r)
    p, act = _layer_params(moe)
    want = O.layer_from_routing(x.cpu().double(), O.upcast(p), routing.double(), act, 'all')
    assert H.rel_err(out.cpu(), want) < H.tol_for(dtype)
    _say(f'  experts/token {routing.float().sum(-1).mean().item():.1f}')


def test_hip_layer_refuses_autograd():
    """With autograd on and trainable parameters the fused layer call raises (the kernels have no backward), as the
    experts containers do on their own and as the reference's kernel wrappers do (moe_impls.py:60-64)."""
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    moe = MoeficationMoE('m', 64, 4, True, 32, nn.ReLU, experts_class='custom_kernel')
    moe.router = MoeficationRouter(64, 4, width=128, depth=2, bias=False, activation='relu', output_activation='abs')
    moe = moe.to(DEV).eval()
    moe.forward_mode, moe.tau = 'dynk_max', 0.5
    moe.experts.forward_mode = 'hip'
    x = torch.randn(2, 3, 64, device=DEV)
    with pytest.raises(NotImplementedError, match='no backward'):
        moe(x)
    with pytest.raises(NotImplementedError, match='no backward'):
        moe.experts(x.view(-1, 64), torch.ones(6, 4, device=DEV))
    for prm in moe.parameters():
        prm.requires_grad_(False)
    out, _ = moe(x)                      # frozen parameters, plain input: nothing asks for a gradient
    assert out.shape == x.shape
    with pytest.raises(NotImplementedError, match='no backward'):
        moe(x.clone().requires_grad_(True))
    with torch.no_grad():
        out2, _ = moe(x.clone().requires_grad_(True))
    assert torch.equal(out, out2)


def test_packed_buffer_of_another_shape_is_refused():
    """The descriptor that travels with a packed buffer is checked by the library: a buffer packed for another layer is
    refused (status -9) before anything is launched; a buffer that lost its descriptor (a slice, a plain copy) is refused
    by the wrapper, and packed_from_header() recovers it from the buffer's first bytes.  A buffer packed without the router
    section still serves the layer: the router then runs on the unfused kernels, with the same mask."""
    from d2dmoe_amd import D2DMoEError
    x, routing, p = H.random_case(64, 768, 128, 24, 128, seed=1, dtype=torch.bfloat16, device=DEV)
    _, _, q = H.random_case(64, 768, 64, 48, 128, seed=2, dtype=torch.bfloat16, device=DEV)
    ops = _ops()
    other = ops.pack_weights(ops.make_shape(0, 768, 64, 48, 128, 1, 'relu'), q['w1'], q['b1'], q['w2'], None, q['router_w1'],
                             q['router_w2'])
    with pytest.raises(D2DMoEError, match='status -9'):
        ops.forward(x, p['router_w1'], p['router_w2'], 0.1, p['w1'], p['b1'], p['w2'], None, None, 'relu', packed=other)
    with pytest.raises(D2DMoEError, match='status -9'):
        ops.experts(x, routing, p['w1'], p['b1'], p['w2'], packed=other)
    full = ops.pack_weights(ops.make_shape(0, 768, 128, 24, 128, 1, 'relu'), p['w1'], p['b1'], p['w2'], None, p['router_w1'],
                            p['router_w2'])
    with pytest.raises(D2DMoEError, match='packed buffer'):
        ops.experts(x, routing, p['w1'], p['b1'], p['w2'], packed=full[:1024])
    with pytest.raises(D2DMoEError, match='packed buffer'):
        ops.experts(x, routing, p['w1'], p['b1'], p['w2'], packed=full.clone())
    want = ops.experts(x, routing, p['w1'], p['b1'], p['w2'], packed=full)
    again = ops.packed_from_header(full.clone())
    assert bytes(again.desc) == bytes(full.desc)
    assert torch.equal(ops.experts(x, routing, p['w1'], p['b1'], p['w2'], packed=again), want)
    assert torch.equal(ops.experts(x, routing, p['w1'], p['b1'], p['w2'], packed=ops.clone_packed(full)), want)
    bare = ops.pack_weights(ops.make_shape(0, 768, 128, 24, 0, 1, 'relu'), p['w1'], p['b1'], p['w2'])
    o1, r1, _, _ = ops.forward(x, p['router_w1'], p['router_w2'], 0.1, p['w1'], p['b1'], p['w2'], None, None, 'relu', packed=bare)
    o2, r2, _, _ = ops.forward(x, p['router_w1'], p['router_w2'], 0.1, p['w1'], p['b1'], p['w2'], None, None, 'relu', packed=full)
    assert torch.equal(r1, r2) and torch.equal(o1, o2)


# =================================================================== router rounding and the mask (bf16, f32) =========
def _ulp(t: torch.Tensor, dtype) -> torch.Tensor:
    """Spacing of `dtype` at the magnitude of t (float64 tensor)."""
    mant = 8 if dtype == torch.bfloat16 else 24
    return torch.pow(2.0, torch.floor(torch.log2(t.abs().clamp_min(1e-300))) - (mant - 1))


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('tau', [0.1, 0.9])
@pytest.mark.parametrize('N', [1576, 50432])
def test_mask_flips_sit_on_the_threshold(N, tau, dtype):
    """End to end (router on the GPU) the mask can differ from the oracle's only where a predicted norm sits on the
    threshold: the GPU's router sums in another order, so a norm, or the row maximum the threshold is made from, may land
    on the neighbouring representable value.  Every differing entry must have its oracle norm within two spacings of the
    storage type of the oracle threshold (one for the norm, one for the threshold), and there must be few of them."""
    _say('flips', N, tau, dtype)
    D, E, Ed, W = 768, 128, 24, 128
    x, _, p = H.random_case(N, D, E, Ed, W, seed=21, dtype=dtype)
    d = H.to_dev(p, DEV)
    ops = _ops()
    packed = None
    if dtype == torch.bfloat16:
        packed = ops.pack_weights(ops.make_shape(0, D, E, Ed, W, 1, 'relu'), d['w1'], d['b1'], d['w2'], None,
                                  d['router_w1'], d['router_w2'])
    routing, norms, _ = ops.router_select(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), packed, E, Ed, True)
    routing, norms = routing.cpu(), norms.cpu()
    assert torch.equal(routing, O.gate_dynk_max(norms, tau))          # stage-wise exact on the GPU's own norms
    norms_o = O.router_forward(x, p['router_w1'], p['router_w2'])
    routing_o = O.gate_dynk_max(norms_o, tau)
    thr_o = (norms_o.max(dim=-1, keepdim=True)[0] * (1.0 - tau)).double()
    flips = routing != routing_o
    n_flips = int(flips.sum())
    margin = ((norms_o.double() - thr_o).abs() / _ulp(thr_o, dtype))[flips]
    worst = margin.max().item() if n_flips else 0.0
    _say(f'  {n_flips} of {N * E} entries differ ({n_flips / (N * E):.2e}); worst margin {worst:.2f} spacings')
    assert worst <= 2.0
    assert n_flips <= (1e-5 if dtype == torch.bfloat16 else 2e-6) * N * E


# =================================================================== GPT-2-small configuration at its size ===================
@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_gpt2_layer_at_full_size(tau):
    """One converted GPT-2-small FFN (GELU, biases, 128 x 24) on 16 x 1024 tokens: mask from the oracle gate on the GPU's
    norms, output against the float64 oracle on row slices (module tau and the literal keep-if->=0.9*max reading)."""
    _say('gpt2 layer', tau)
    N, D, E, Ed, W = 16 * 1024, 768, 128, 24, 128
    x, _, p = H.random_case(N, D, E, Ed, W, seed=31, dtype=torch.bfloat16)
    d = H.to_dev(p, DEV)
    ops = _ops()
    packed = ops.pack_weights(ops.make_shape(0, D, E, Ed, W, 1, 'gelu'), d['w1'], d['b1'], d['w2'], None, d['router_w1'],
                              d['router_w2'])
    out, routing, norms, counts = ops.forward(x.to(DEV), d['router_w1'], d['router_w2'], float(1.0 - tau), d['w1'], d['b1'],
                                              d['w2'], None, d['last_bias'].view(-1), 'gelu', False, None, True, True, 'auto',
                                              packed)
    routing = routing.cpu()
    assert torch.equal(routing, O.gate_dynk_max(norms.cpu(), tau))
    assert torch.equal(counts.cpu().long(), routing.float().sum(0).long())
    rows = torch.cat([torch.arange(64), torch.arange(8000, 8064), torch.arange(N - 64, N)])
    want = O.layer_from_routing(x[rows].double(), O.upcast(p), routing[rows].double(), 'gelu', 'all')
    got = out.cpu()[rows]
    elem = H.elem_err(got, want)
    _say(f'  experts/token {routing.sum(1).mean().item():.1f}, rel err {H.rel_err(got, want):.2e}, per element {elem:.2e}')
    assert H.rel_err(got, want) < H.TOL_BF16
    assert elem < H.TOL_BF16


def test_gpt2_small_forward_at_full_size():
    """The GPT-2-small benchmark configuration as named: 12 layers, d_model 768, 12 heads, vocabulary 50257, every FFN converted to 128 experts of
    24 neurons with its own 768->128->128 router, batch 16 x 1024, bf16, module tau 0.9.  The model returns finite logits
    and one routing tensor per layer; each layer's mask is a valid dynamic-k mask (at least one expert per token); the
    last layer's output is checked against the float64 oracle on the layer's own input rows."""
    from d2dmoe_amd import add_routers, gpt2
    _say('gpt2-small full forward')
    torch.manual_seed(0)
    cfg = gpt2.GPTConfig(block_size=1024, vocab_size=50257, n_layer=12, n_head=12, n_embd=768)
    dense = gpt2.GPT(cfg).eval().to(DEV).bfloat16()
    moe, names = gpt2.replace_with_moes(dense, num_experts=128, experts_class='hip_kernel')
    gpt2.split_original_parameters(dense, moe, names)
    del dense
    add_routers(moe, dict(width=128, depth=2, bias=False, activation='relu', output_activation='abs'))
    moe = moe.to(DEV).bfloat16().eval()
    captured = {}
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode, layer.tau = 'dynk_max', 0.9
        layer.experts.forward_mode = 'hip'
    last = gpt2.get_module_by_name(moe, names[-1])
    hook = last.register_forward_hook(lambda m, args, res: captured.update(x=args[0].detach(), out=res[0].detach()))
    idx = torch.randint(0, cfg.vocab_size, (16, 1024), generator=torch.Generator().manual_seed(1)).to(DEV)
    with torch.no_grad():
        logits, gating = moe(idx, return_gating_data=True)
    hook.remove()
    assert logits.shape == (16, 1024, 50257)
    assert bool(torch.isfinite(logits[:, ::64].float()).all()) and bool(torch.isfinite(logits[-1, -1].float()).all())
    assert len(gating) == 12 and set(gating) == set(names)
    for n in names:
        (r,) = gating[n]
        assert r.shape == (16, 1024, 128)
        per_token = r.float().sum(-1)
        assert bool((per_token >= 1).all()) and bool(((r == 0) | (r == 1)).all())
    _say('  experts/token per layer:', [round(gating[n][0].float().sum(-1).mean().item(), 1) for n in names])
    p, act = _layer_params(last)
    rows = torch.cat([torch.arange(48), torch.arange(16 * 1024 - 48, 16 * 1024)])
    xin = captured['x'].reshape(-1, 768).cpu()[rows]
    r = gating[names[-1]][0].reshape(-1, 128).cpu()[rows]
    want = O.layer_from_routing(xin.double(), O.upcast(p), r.double(), act, 'all')
    assert H.rel_err(captured['out'].reshape(-1, 768).cpu()[rows], want) < H.TOL_BF16


# =================================================================== skewed-routing configuration at its size ===================
@pytest.mark.parametrize('tau', [0.9, 0.1])
def test_skewed_routing_at_full_size(tau):
    """50 432 tokens, router bypassed by |N(0,1)| x Zipf(1.2) predicted norms: mask bit-exact with the oracle gate, counts
    exact, outputs against the float64 oracle on row slices, under the module reading of tau = 0.9 and the literal one."""
    _say('skew', tau)
    N, D, E, Ed = 50432, 768, 128, 24
    x, _, p = H.random_case(N, D, E, Ed, 128, seed=41, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(9)
    w = (torch.randperm(E, generator=g) + 1).float() ** -1.2
    norms = (torch.randn(N, E, generator=g).abs() * (w / w.max())).bfloat16()
    d = H.to_dev(p, DEV)
    ops = _ops()
    packed = ops.pack_weights(ops.make_shape(0, D, E, Ed, 0, 1, 'relu'), d['w1'], d['b1'], d['w2'])
    out, routing, _, counts = ops.forward(x.to(DEV), None, None, float(1.0 - tau), d['w1'], d['b1'], d['w2'], None,
                                          d['last_bias'].view(-1), 'relu', False, norms.to(DEV), False, True, 'auto', packed)
    want_r = O.gate_dynk_max(norms, tau)
    assert torch.equal(routing.cpu(), want_r)
    assert torch.equal(counts.cpu().long(), want_r.float().sum(0).long())
    rows = torch.cat([torch.arange(64), torch.arange(25000, 25064), torch.arange(N - 64, N)])
    want = O.layer_from_routing(x[rows].double(), O.upcast(p), want_r[rows].double(), 'relu', 'all')
    err = H.rel_err(out.cpu()[rows], want)
    c = counts.float()
    _say(f'  experts/token {want_r.float().sum(1).mean().item():.1f}, max/mean load {(c.max() / c.mean()).item():.1f}, '
         f'rel err {err:.2e}, per element {H.elem_err(out.cpu()[rows], want):.2e}')
    assert err < H.TOL_BF16
    assert H.elem_err(out.cpu()[rows], want) < H.TOL_BF16
