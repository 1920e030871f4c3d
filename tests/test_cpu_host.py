"""CPU-side checks: the oracle against the committed golden fixtures, the host-side module logic, and that the
C-ABI library loads and exports every symbol that include/d2dmoe.h declares (no compute calls without a GPU)."""
import ctypes
import hashlib
import os
import re

import numpy as np
import pytest
import torch
from torch import nn

from oracle import d2dmoe_oracle as O
from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------ oracle vs golden fixtures ----------
@pytest.mark.parametrize('case', ['toy', 'vit197', 'gpt64', 'gated16'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_oracle_reproduces_fixture(case, dtype):
    fx, x, p, c = H.fixture_inputs(case, dtype)
    dt = 'f32' if dtype == torch.float32 else 'bf16'
    norms = O.router_forward(x, p['router_w1'], p['router_w2'])
    assert np.array_equal(norms.float().numpy().reshape(-1, c['E'])[:32], fx[f'norms_{dt}'])
    for tau in c['taus']:
        tag = f'{dt}_tau{tau}'
        routing = O.gate_dynk_max(norms, tau).reshape(-1, c['E'])
        assert torch.equal(routing.float(), H.routing_from_bits(fx[f'routing_bits_{tag}'], c['E']))
        s, u, cnt = O.extract_indices(routing)
        off, tok = O.permutation_csr(routing)
        assert np.array_equal(off.numpy(), fx[f'offsets_{tag}']) and np.array_equal(tok.numpy(), fx[f'token_idx_{tag}'])
        assert hashlib.sha256(s.numpy().tobytes()).hexdigest() == str(fx[f'sort_crc_{tag}'])
        assert hashlib.sha256(u.numpy().tobytes()).hexdigest() == str(fx[f'unsort_crc_{tag}'])
        # the storage-dtype evaluation (what the reference's eager path would compute) stays within the parity
        # tolerance of the stored float64 result.  The per-expert loop in bf16 rounds its running sum to bf16 after
        # every expert (up to ~100 roundings per token here), so it is held to a looser bound.
        want = torch.from_numpy(fx[f'out_{tag}'])
        for mode in ('all', 'naive'):
            got = O.layer_from_routing(x, p, routing.view(*x.shape[:-1], -1), c['act'], mode)
            tol = 6e-2 if (mode == 'naive' and dtype == torch.bfloat16) else H.tol_for(dtype)
            assert H.rel_err(got.reshape(-1, c['D'])[:32], want) < tol, (case, dtype, tau, mode)


# ------------------------------------------------------------------ C ABI: load + exports ---------------
def test_library_exports_every_declared_symbol():
    from d2dmoe_amd import hip_abi as abi
    header = open(os.path.join(ROOT, 'include', 'd2dmoe.h')).read()
    declared = set(re.findall(r'\b(d2dmoe_[a-z_]+)\s*\(', header))
    assert declared == set(abi.EXPORTS), declared ^ set(abi.EXPORTS)
    lib = abi.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.d2dmoe_version() == int(re.search(r'#define D2DMOE_VERSION (\d+)', header).group(1))
    assert lib.d2dmoe_status_string(0) == b'ok'
    assert b'workspace' in lib.d2dmoe_status_string(-5)


def test_shape_struct_matches_header_and_argument_checks():
    from d2dmoe_amd import hip_abi as abi, ops
    header = open(os.path.join(ROOT, 'include', 'd2dmoe.h')).read()
    body = re.search(r'typedef struct d2dmoe_shape \{(.*?)\} d2dmoe_shape;', header, re.S).group(1)
    fields = re.findall(r'(int64_t|int32_t)\s+(\w+);', body)
    assert [f for _, f in fields] == [f for f, _ in abi.Shape._fields_]
    for (ctype, _), (_, pyt) in zip(fields, abi.Shape._fields_):
        assert ctypes.sizeof(pyt) == (8 if ctype == 'int64_t' else 4)
    lib = abi.load()
    sh = ops.make_shape(50432, 768, 128, 24, 128, abi.BF16)
    ws = lib.d2dmoe_workspace_bytes(ctypes.byref(sh))
    assert ws >= 50432 * 128 * 2 * 2 and ws % 256 == 0
    # rejected arguments come back as negative status codes before anything touches a device
    bad = ops.make_shape(10, 768, 128, 24, 128, abi.BF16)
    bad.dtype = 9
    assert lib.d2dmoe_workspace_bytes(ctypes.byref(bad)) == 0
    assert lib.d2dmoe_experts(ctypes.byref(bad), None, None, None, None, None, None, None, None, None, None, 0, None, 0,
                              None) == -3
    ok = ops.make_shape(10, 768, 128, 24, 128, abi.BF16)
    assert lib.d2dmoe_experts(ctypes.byref(ok), None, None, None, None, None, None, None, None, None, None, 0, None, 0,
                              None) == -1
    assert lib.d2dmoe_select(None, None, None, 4, 8, 0, ctypes.c_float(0.5), None) == -1
    assert lib.d2dmoe_select(1, 1, None, 4, 5000, 0, ctypes.c_float(0.5), None) == -2
    assert lib.d2dmoe_router(1, 1, 1, 1, 4, 8, 8, 8, 0, 99, 0, None, 0, None) == -4
    assert lib.d2dmoe_build_permutation(None, 4, 8, 0, None, None, None, None, None, None, 0, None) == -1
    with pytest.raises(abi.D2DMoEError):
        abi.check(-6, 'x')


def test_packed_and_workspace_sizes_follow_the_documented_layouts():
    """Host-only size queries (no device is touched): packed sections and workspace of the shapes the benchmarks use."""
    from d2dmoe_amd import hip_abi as abi, ops
    lib = abi.load()
    lib.d2dmoe_packed_bytes.restype = ctypes.c_size_t
    # Gemma-2B FFN: expert-major section (gate, up, down fragments + padded bias) + small-batch section (gate|up + down,
    # 3 matrices + padded bias) + tiled-products section (3 matrices + bias) + router section
    mat = 256 * 64 * 2048 * 2
    g = ops.make_shape(4096, 2048, 256, 64, 256, abi.BF16, 'gelu_tanh', gated=True)
    want = 3 * (3 * mat + 256 * 64 * 2) + (256 * 2048 + 256 * 256) * 2
    got = lib.d2dmoe_packed_bytes(ctypes.byref(g))
    assert want <= got <= want + 6 * 256 and got % 256 == 0
    # workspace at 4096 tokens: router hidden + norms, then the expert-major plan (under 2 MB of counts, offsets and
    # lists) and its per-pair result rows, provisioned for 32 routed experts per token (32 x 4096 rows of 2048 bf16); the
    # fall-back, the tiled products, works in the same region (H fragments 4096 x 16384 bf16 + 2 float32 partial sums:
    # smaller)
    ws = lib.d2dmoe_workspace_bytes(ctypes.byref(g))
    want_ws = 4096 * 256 * 2 * 2 + 32 * 4096 * 2048 * 2
    assert want_ws <= ws <= want_ws + (2 << 20)
    assert 32 * 4096 * 2048 * 2 >= 4096 * 16384 * 2 + 2 * 4096 * 2048 * 4
    # 16 tokens: the small-batch path needs the hidden fragments and one flag per expert only; the size query also covers
    # the expert-major path on request, whose fall-back works on one 256-token tile of H fragments (8 MB)
    g16 = ops.make_shape(16, 2048, 256, 64, 256, abi.BF16, 'gelu_tanh', gated=True)
    assert lib.d2dmoe_workspace_bytes(ctypes.byref(g16)) < 10 << 20
    # float32 layers: the tiled-products section only (hidden size 128 x 24 = 3072 neurons, float32 fragments)
    f = ops.make_shape(100, 768, 128, 24, 128, abi.F32)
    want_f = (2 * 3072 * 768 + 3072) * 4
    assert want_f <= lib.d2dmoe_packed_bytes(ctypes.byref(f)) <= want_f + 256
    odd = ops.make_shape(100, 700, 128, 24, 128, abi.F32)   # width not a multiple of 256: generic kernel only
    assert lib.d2dmoe_packed_bytes(ctypes.byref(odd)) == 0
    # ViT-B shape: dense-sweep stream (4 waves x 12 chunks x 192 fragments of 1 KB) is part of the buffer
    v = ops.make_shape(50432, 768, 128, 24, 128, abi.BF16)
    assert lib.d2dmoe_packed_bytes(ctypes.byref(v)) >= 4 * 12 * 192 * 1024
    # router section: W2 is padded with zero rows to the next of 32 / 64 / 128 / 256 experts, so the same layer with and
    # without a router differs by W1 + padded W2; 24 experts take one tile of 32, 100 experts have no fused router
    for E, Ed, pad in ((24, 128, 32), (64, 48, 64), (128, 24, 128)):
        with_r = lib.d2dmoe_packed_bytes(ctypes.byref(ops.make_shape(0, 768, E, Ed, 128, abi.BF16)))
        without = lib.d2dmoe_packed_bytes(ctypes.byref(ops.make_shape(0, 768, E, Ed, 0, abi.BF16)))
        assert 0 <= with_r - without - (128 * 768 + pad * 128) * 2 < 512, (E, with_r - without)
    e100 = ops.make_shape(0, 768, 100, 30, 128, abi.BF16)
    assert lib.d2dmoe_packed_bytes(ctypes.byref(e100)) == lib.d2dmoe_packed_bytes(
        ctypes.byref(ops.make_shape(0, 768, 100, 30, 0, abi.BF16)))
    # expert-major workspace at D = 768: provisioned for 8 routed experts per token whatever the expert size (rows of
    # 768 16-bit values per pair, token and slot lists of 4 bytes each)
    for E, Ed in ((128, 24), (48, 64), (24, 128)):
        ws = lib.d2dmoe_workspace_bytes(ctypes.byref(ops.make_shape(50432, 768, E, Ed, 128, abi.BF16)))
        want = 8 * 50432 * (768 * 2 + 8)
        assert want <= ws <= want + (64 << 20), (E, Ed, ws)


def test_norms_buffer_size_follows_the_documented_layout():
    """d2dmoe_norms_packed_bytes: four wave streams of first-layer fragments (16 bytes per lane; experts padded to 32
    neurons, to 64 from 33 neurons on, 8 such slots of 32 per chunk, one ring of 32 fragments of padding per wave), bias,
    Gram fragments in two 16-bit parts (one 32 x 32 block per small expert, 2 x 2 per big one), one scale per slot; 0 for
    what the kernel does not cover."""
    from d2dmoe_amd import hip_abi as abi, ops
    lib = abi.load()
    for D, E, Ed in ((768, 128, 24), (768, 100, 30), (1024, 128, 32), (768, 24, 64), (2048, 9, 33), (256, 7, 5), (1280, 160, 32)):
        for dt in (abi.BF16, abi.F16):
            got = lib.d2dmoe_norms_packed_bytes(ctypes.byref(ops.make_shape(0, D, E, Ed, 0, dt)))
            slots = E * (2 if Ed > 32 else 1)
            chunks = (slots + 7) // 8
            stream = 4 * (chunks * 2 * (D // 16) + 32) * 64 * 16
            bias = chunks * 8 * 32 * 2
            gram = chunks * 8 * (8 if Ed > 32 else 4) * 64 * 16
            scale = chunks * 8 * 4
            assert stream + bias + gram + scale <= got < stream + bias + gram + scale + 768, (D, E, Ed, dt)
    for D, E, Ed, dt, gated in ((768, 128, 24, abi.F32, False), (800, 128, 24, abi.BF16, False), (2304, 16, 24, abi.BF16, False),
                                (768, 16, 65, abi.BF16, False), (2048, 256, 64, abi.BF16, True)):
        sh = ops.make_shape(0, D, E, Ed, 0, dt, 'gelu_tanh' if gated else 'relu', gated=gated)
        assert lib.d2dmoe_norms_packed_bytes(ctypes.byref(sh)) == 0, (D, E, Ed, dt, gated)


def test_expert_major_workspace_covers_its_tiled_products_fallback():
    """Ungated D = 768 layers the fused sweep does not cover (more than 256 experts, or more than 32 chunks of 256 hidden
    neurons) fall back, behind the expert-major plan, to the tiled products, which work in the workspace BEHIND the plan:
    the size query must cover router scratch + the plan's lists + the products' own need (hidden fragments of whole
    256-token tiles + float32 partial sums)."""
    from d2dmoe_amd import hip_abi as abi, ops
    lib = abi.load()
    for N, E, Ed in ((4096, 512, 32), (4096, 320, 32), (1000, 256, 64), (8192, 384, 24), (300, 1024, 8)):
        for dt in (abi.BF16, abi.F16):
            ws = lib.d2dmoe_workspace_bytes(ctypes.byref(ops.make_shape(N, 768, E, Ed, 128, dt)))
            edp = Ed if Ed % 4 == 0 else (Ed + 31) // 32 * 32
            hp = (E * edp + 255) // 256 * 256
            n_ttiles = (min(N, 8192) + 255) // 256
            tiles, ks2, ksplit = n_ttiles * 3, hp // 16, 1
            while ksplit < 8 and tiles * ksplit < 256 and (ks2 // (ksplit * 2)) % 4 == 0:
                ksplit *= 2
            gemm = n_ttiles * 256 * hp * 2 + ksplit * min(N, 8192) * 768 * 4
            plan_lists = 2 * 8 * N * 4 + (N + 1) * 4
            router = N * (128 + E) * 2
            assert ws >= router + plan_lists + gemm, (N, E, Ed, dt, ws, router + plan_lists + gemm)


def test_packed_descriptor_is_checked_on_the_host_before_anything_is_launched():
    """Every entry point that takes `packed` takes its descriptor and refuses, with D2DMOE_E_PACKED and before any other
    argument is looked at, a buffer that comes without one or was packed for another layer, element type, router or
    layout version.  No device is touched: the packed pointer is a dummy, and a descriptor that passes is followed by the
    NULL-pointer error for x."""
    from d2dmoe_amd import hip_abi as abi, ops
    lib = abi.load()
    dummy = 256                                    # a non-NULL "device pointer" that is never dereferenced
    sh = ops.make_shape(100, 768, 128, 24, 128, abi.BF16)
    good = abi.PackedDesc()
    assert lib.d2dmoe_packed_describe(ctypes.byref(sh), ctypes.byref(good)) == 0
    assert ctypes.sizeof(good) == 64 and good.magic == abi.PACKED_MAGIC
    assert good.bytes == lib.d2dmoe_packed_bytes(ctypes.byref(sh)) and good.router_width == 128
    assert good.sections & 32 and good.sections & 1        # router and dense-sweep sections
    assert lib.d2dmoe_packed_describe(ctypes.byref(ops.make_shape(10, 700, 128, 24, 128, abi.F32)), ctypes.byref(good)) == -6
    assert lib.d2dmoe_packed_describe(ctypes.byref(sh), ctypes.byref(good)) == 0

    def experts(desc, shape=sh):
        return lib.d2dmoe_experts(ctypes.byref(shape), None, None, None, None, None, None, None, dummy,
                                  None if desc is None else ctypes.byref(desc), None, 0, None, 0, None)

    def forward(desc, shape=sh):
        return lib.d2dmoe_forward(ctypes.byref(shape), None, None, None, ctypes.c_float(0.1), None, None, None, None, None,
                                  dummy, None if desc is None else ctypes.byref(desc), None, None, dummy, None, dummy, 0,
                                  None, 0, None)

    def forward_static(desc, shape=sh):
        return lib.d2dmoe_forward_static(ctypes.byref(shape), None, None, None, ctypes.c_float(0.1), None, None, None, None,
                                         None, dummy, None if desc is None else ctypes.byref(desc), None, None, dummy, None,
                                         dummy, 0, None)

    def router_select(desc, shape=sh):
        return lib.d2dmoe_router_select(ctypes.byref(shape), None, None, None, dummy,
                                        None if desc is None else ctypes.byref(desc), ctypes.c_float(0.1), None, dummy, None,
                                        None, 0, None)

    def variant(**kw):
        d = abi.PackedDesc.from_buffer_copy(bytes(good))
        for k, v in kw.items():
            setattr(d, k, v)
        return d

    for call in (experts, forward, router_select):
        assert call(good) == -1, call.__name__               # descriptor accepted: the next check is x == NULL
        assert call(None) == abi.E_PACKED, call.__name__     # a buffer without its descriptor
        for bad in (variant(magic=0), variant(layout_version=good.layout_version + 1), variant(dtype=abi.F16),
                    variant(d_model=1024), variant(n_experts=64), variant(expert_dim=48), variant(gated=1),
                    variant(bytes=good.bytes - 256), variant(sections=good.sections & ~1),
                    variant(router_width=256)):
            assert call(bad) == abi.E_PACKED, call.__name__
    # the static entry point looks at the workspace limit first (this shape fits), then at the descriptor
    assert forward_static(None) == abi.E_PACKED and forward_static(variant(dtype=abi.F16)) == abi.E_PACKED
    # a buffer packed WITH the router serves a call whose shape names none (experts only) ...
    assert experts(good, ops.make_shape(100, 768, 128, 24, 0, abi.BF16)) == -1
    # ... and one packed without it passes too (the router then runs on the unfused kernels); only its size must be its own
    bare_shape = ops.make_shape(100, 768, 128, 24, 0, abi.BF16)
    bare = abi.PackedDesc()
    assert lib.d2dmoe_packed_describe(ctypes.byref(bare_shape), ctypes.byref(bare)) == 0
    assert bare.router_width == 0 and not (bare.sections & 32) and bare.bytes < good.bytes
    assert forward(bare) == -1 and experts(bare) == -1
    assert forward(variant(router_width=0)) == abi.E_PACKED   # claims "no router" at the size of a buffer with one
    # the header of a buffer, copied back to the host, yields the descriptor again
    back = abi.PackedDesc()
    assert lib.d2dmoe_packed_desc_from_header(bytes(good), ctypes.byref(back)) == 0 and bytes(back) == bytes(good)
    assert lib.d2dmoe_packed_desc_from_header(bytes(64), ctypes.byref(back)) == abi.E_PACKED
    assert b'packed' in lib.d2dmoe_status_string(abi.E_PACKED)


# ------------------------------------------------------------------ host-side module mirror -------------
def _toy_layer(act=nn.ReLU, experts_class='hip_kernel'):
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter
    torch.manual_seed(0)
    moe = MoeficationMoE('blk3.mlp', 64, 4, True, 32, act, experts_class=experts_class)
    moe.router = MoeficationRouter(64, 4, width=128, depth=2, bias=False, activation='relu', output_activation='abs')
    moe.forward_mode = 'dynk_max'
    moe.tau = 0.5
    return moe.eval()


def test_module_interface_and_state_dict_keys():
    moe = _toy_layer()
    keys = set(moe.state_dict().keys())
    assert keys == {'last_bias', 'experts.w1', 'experts.b1', 'experts.w2', 'router.layers.0.weight',
                    'router.layers.2.weight'}
    assert moe.experts.w1.shape == (4, 64, 32) and moe.experts.b1.shape == (4, 32) and moe.experts.w2.shape == (4, 32, 64)
    assert moe.last_bias.shape == (1, 64)
    assert moe.experts.w1.abs().max() <= 1 / np.sqrt(32) and moe.experts.w2.abs().max() <= 1 / np.sqrt(64)
    x = torch.randn(5, 2, 64)
    with torch.no_grad():
        out, gating = moe(x)
    assert out.shape == x.shape and list(gating) == ['blk3.mlp']
    (routing,) = gating['blk3.mlp']
    assert routing.shape == (5, 2, 4) and routing.dtype == x.dtype
    # the CPU module path agrees with the oracle (same weights)
    p = {'w1': moe.experts.w1.data, 'b1': moe.experts.b1.data, 'w2': moe.experts.w2.data,
         'last_bias': moe.last_bias.data, 'router_w1': moe.router.layers[0].weight.data,
         'router_w2': moe.router.layers[2].weight.data}
    want, r_want, _ = O.moe_layer_forward(x, p, 0.5, experts_mode='all')
    assert torch.equal(routing, r_want) and torch.allclose(out, want, rtol=1e-5, atol=1e-6)
    moe.experts.forward_mode = 'naive'
    with torch.no_grad():
        out_naive, _ = moe(x)
    assert torch.allclose(out_naive, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize('mode', ['all', 'topk', 'dynk', 'dynk_max'])
def test_gate_modes_match_oracle(mode):
    moe = _toy_layer()
    moe.forward_mode = mode
    moe.k = 2
    moe.tau = 0.6
    x = torch.randn(3, 7, 64)
    with torch.no_grad():
        r = moe.gate(x)
        scores = moe.router(x)
    want = {'all': lambda: O.gate_all(x, 4), 'topk': lambda: O.gate_topk(scores, 2),
            'dynk': lambda: O.gate_dynk(scores, 0.6), 'dynk_max': lambda: O.gate_dynk_max(scores, 0.6)}[mode]()
    assert torch.equal(r, want)


def test_hip_mode_fails_loudly_without_a_gpu():
    from d2dmoe_amd import D2DMoEError
    moe = _toy_layer()
    moe.experts.forward_mode = 'hip'
    with pytest.raises(D2DMoEError):
        with torch.no_grad():
            moe(torch.randn(2, 3, 64))
    with pytest.raises(NotImplementedError):
        moe.experts.forward_mode = 'triton_optimized'
        with torch.no_grad():
            moe(torch.randn(2, 3, 64))


def test_router_override_hook_and_add_routers():
    from d2dmoe_amd import MoeficationMoE, MoeficationRouter, add_routers
    r = MoeficationRouter(64, 4, width=16, depth=2, activation='relu', output_activation='abs',
                          test_override_outputs_p=0.5)
    x = torch.randn(2, 5, 64)
    a = r(x)
    b = r(torch.randn(2, 5, 64))
    assert a is b and set(a.unique().tolist()) <= {0.0, 1.0}    # cached per (batch, sequence) shape
    model = nn.Sequential(MoeficationMoE('a', 64, 4, True, 8, nn.GELU), MoeficationMoE('b', 64, 4, True, 8, nn.GELU))
    found = add_routers(model, dict(width=16, depth=2, bias=False, activation='relu', output_activation='abs'))
    assert set(found) == {'0', '1'} and all(m.router is not None for m in found.values())
    assert found['0'].router.hip_compatible()
    assert not MoeficationRouter(64, 4, depth=3).hip_compatible()


def test_execute_all_container_names_and_masked_forward():
    from d2dmoe_amd import MOE_IMPL_MAP
    torch.manual_seed(1)
    ex = MOE_IMPL_MAP['execute_all'](dim=32, num_experts=4, depth=2, expert_dim=8, bias=False, activation=nn.GELU,
                                     intermediate_gating=True)
    assert set(ex.state_dict()) == {'layers.0.w', 'layers.1.w', 'layers.2.w'}
    x = torch.randn(6, 32)
    routing = (torch.rand(6, 4) < 0.5).float()
    with torch.no_grad():
        got = ex(x, routing)
    want = O.experts_gated_forward_all(x, routing, ex.layers[0].w.data, ex.layers[2].w.data, ex.layers[1].w.data, 'gelu')
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_extract_indices_cpu_matches_oracle():
    from d2dmoe_amd import HipKernelExperts
    routing = (torch.rand(100, 6) < 0.3).float()
    s, u, c = HipKernelExperts.extract_indices(routing)
    so, uo, co = O.extract_indices(routing)
    assert torch.equal(s, so) and torch.equal(u, uo) and torch.equal(c.long(), co)


# ------------------------------------------------------------------------------------- GPT-2 model surgery
def _tiny_gpt(seed=0, activation='gelu'):
    from d2dmoe_amd import gpt2
    torch.manual_seed(seed)
    cfg = gpt2.GPTConfig(block_size=32, vocab_size=96, n_layer=2, n_head=2, n_embd=64, activation=activation)
    model = gpt2.GPT(cfg).eval()
    with torch.no_grad():   # make the zero-initialised biases matter
        for n, p in model.named_parameters():
            if n.endswith('bias'):
                p.normal_(0.0, 0.05)
    return gpt2, model


@pytest.mark.parametrize('labelling', ['contiguous', 'shuffled'])
def test_gpt_surgery_all_experts_reproduces_the_dense_model(labelling):
    """replace_with_moes + split_original_parameters: with every expert running ('all'), the MoE model is the dense
    model, whatever balanced labelling moved the neurons (reference: moefication.py:157-202, 205-306)."""
    gpt2, model = _tiny_gpt()
    moe, names = gpt2.replace_with_moes(model, expert_size=16, experts_class='hip_kernel')
    assert names == ['transformer.h.0.mlp', 'transformer.h.1.mlp']
    labels = None
    if labelling == 'shuffled':
        g = torch.Generator().manual_seed(5)
        labels = {n: (torch.arange(256) // 16)[torch.randperm(256, generator=g)] for n in names}
    gpt2.split_original_parameters(model, moe, names, labels)
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        assert layer.num_experts == 16 and layer.expert_dim == 16 and isinstance(layer.dropout, nn.Dropout)
        layer.forward_mode = 'all'
        layer.experts.forward_mode = 'masked'
    idx = torch.randint(0, 96, (3, 20), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        want = model(idx)
        got, gating = moe(idx, return_gating_data=True)
        assert torch.equal(moe(idx), got)
    assert set(gating) == set(names) and gating[names[0]][0].shape == (3, 20, 16)
    assert H.rel_err(got, want) < 1e-5
    # state_dict keys of a MoE block follow the reference layer's
    keys = [k for k in moe.state_dict() if k.startswith('transformer.h.0.mlp')]
    assert keys == ['transformer.h.0.mlp.last_bias', 'transformer.h.0.mlp.experts.w1', 'transformer.h.0.mlp.experts.b1',
                    'transformer.h.0.mlp.experts.w2']


def test_gpt_dynk_max_on_cpu_matches_oracle_layer():
    from d2dmoe_amd import add_routers
    gpt2, model = _tiny_gpt(activation='relu')
    moe, names = gpt2.replace_with_moes(model, num_experts=8)
    gpt2.split_original_parameters(model, moe, names)
    add_routers(moe, dict(width=16, depth=2, bias=False, activation='relu', output_activation='abs'))
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode, layer.tau = 'dynk_max', 0.6
        layer.experts.forward_mode = 'masked'
    idx = torch.randint(0, 96, (2, 16), generator=torch.Generator().manual_seed(2))
    captured = {}
    layer0 = gpt2.get_module_by_name(moe, names[0])
    hook = layer0.register_forward_hook(lambda m, inp, out: captured.update(x=inp[0], out=out[0], routing=out[1][names[0]][0]))
    with torch.no_grad():
        moe(idx)
    hook.remove()
    p = dict(w1=layer0.experts.w1.detach(), b1=layer0.experts.b1.detach(), w2=layer0.experts.w2.detach(),
             last_bias=layer0.last_bias.detach(), router_w1=layer0.router.layers[0].weight.detach(),
             router_w2=layer0.router.layers[2].weight.detach())
    want_out, want_routing, _ = O.moe_layer_forward(captured["x"], p, 0.6, "relu", "all")
    assert torch.equal(captured['routing'], want_routing.view_as(captured['routing']))
    assert H.rel_err(captured['out'], want_out.view_as(captured['out'])) < 1e-5
    assert 0 < captured['routing'].mean().item() < 1


# ---------------------------------------------------------------------------------------------------------------------
# Checkpoint import (reference: train.py:295-320 writes final.pth; utils.py:580-672 rebuilds and load_state_dict()s)
# ---------------------------------------------------------------------------------------------------------------------
def _tiny_moe_gpt(seed):
    from d2dmoe_amd import add_routers, gpt2
    torch.manual_seed(seed)
    cfg = gpt2.GPTConfig(block_size=16, vocab_size=64, n_layer=2, n_head=2, n_embd=32)
    dense = gpt2.GPT(cfg).eval()
    moe, names = gpt2.replace_with_moes(dense, num_experts=8, experts_class='hip_kernel')
    gpt2.split_original_parameters(dense, moe, names)
    add_routers(moe, dict(width=16, depth=2, bias=False, activation='relu', output_activation='abs'))
    return moe, names


def test_reference_checkpoint_layout_loads_unchanged(tmp_path):
    import d2dmoe_amd as P
    src, names = _tiny_moe_gpt(0)
    state = src.state_dict()
    # the parameter names and shapes a reference model_state carries for a MoE layer
    n0 = names[0]
    assert tuple(state[f'{n0}.experts.w1'].shape) == (8, 32, 16)
    assert tuple(state[f'{n0}.experts.b1'].shape) == (8, 16)
    assert tuple(state[f'{n0}.experts.w2'].shape) == (8, 16, 32)
    assert tuple(state[f'{n0}.last_bias'].shape) == (1, 32)
    assert tuple(state[f'{n0}.router.layers.0.weight'].shape) == (16, 32)
    assert tuple(state[f'{n0}.router.layers.2.weight'].shape) == (8, 16)
    # final.pth as the reference's driver writes it, minus the arbitrary `args` object; keys wrapped as accelerate
    # / DataParallel / torch.compile leave them
    path = tmp_path / 'final.pth'
    wrapped = {'module._orig_mod.' + k: v for k, v in state.items()}
    torch.save({'model_state': wrapped, 'final_score': 0.5, 'model_flops': 123}, path)
    got = P.read_model_state(path)
    assert set(got) == set(state)
    dst, _ = _tiny_moe_gpt(1)
    assert not torch.equal(dst.state_dict()[f'{n0}.experts.w1'], state[f'{n0}.experts.w1'])
    missing, unexpected = P.load_model_state(dst, got)
    assert missing == [] and unexpected == []
    for k, v in state.items():
        assert torch.equal(dst.state_dict()[k], v), k
    idx = torch.randint(0, 64, (2, 16), generator=torch.Generator().manual_seed(3))
    from d2dmoe_amd import gpt2
    for m in (src, dst):
        for n in names:
            layer = gpt2.get_module_by_name(m, n)
            layer.forward_mode, layer.tau = 'dynk_max', 0.9
            layer.experts.forward_mode = 'naive'
    with torch.no_grad():
        assert torch.equal(src(idx)[0], dst(idx)[0])
    # a bare state dict is accepted as well
    torch.save(state, tmp_path / 'bare.pth')
    assert set(P.read_model_state(tmp_path / 'bare.pth')) == set(state)


def test_checkpoint_import_refuses_what_it_should(tmp_path):
    import argparse
    import d2dmoe_amd as P
    src, names = _tiny_moe_gpt(0)
    # an arbitrary Python object in the file: the safe loader refuses it and the error says what to do
    torch.save({'args': argparse.Namespace(lr=0.1), 'model_state': src.state_dict()}, tmp_path / 'with_args.pth')
    with pytest.raises(ValueError, match='weights_only'):
        P.read_model_state(tmp_path / 'with_args.pth')
    torch.save({'model_state': [1, 2, 3]}, tmp_path / 'junk.pth')
    with pytest.raises(ValueError, match='state dict'):
        P.read_model_state(tmp_path / 'junk.pth')
    # converted with another number of experts: named shape error instead of a wall of mismatches
    from d2dmoe_amd import gpt2
    torch.manual_seed(0)
    cfg = gpt2.GPTConfig(block_size=16, vocab_size=64, n_layer=2, n_head=2, n_embd=32)
    other, _ = gpt2.replace_with_moes(gpt2.GPT(cfg).eval(), num_experts=4, experts_class='hip_kernel')
    state = {k: v for k, v in src.state_dict().items() if 'router' not in k}
    with pytest.raises(ValueError, match='number of experts'):
        P.load_model_state(other, state)
    # prefixes are only stripped when every key carries them
    mixed = {'module.a': torch.zeros(1), 'b': torch.zeros(1)}
    assert set(P.strip_wrapper_prefixes(mixed)) == {'module.a', 'b'}
    # without a GPU there is nothing to pack
    assert P.prepack(src) == 0


def test_output_norms_on_cpu_follow_the_reference_route():
    """Without a GPU the router-training targets come from the two stub submodules, as in the reference."""
    from d2dmoe_amd import HipKernelExperts
    torch.manual_seed(0)
    ex = HipKernelExperts(48, 6, 2, 8, 'without_last', torch.nn.GELU)
    with torch.no_grad():
        ex.b1.normal_(0.0, 0.1)
    x = torch.randn(11, 48)
    seen = {}
    h = ex.output_activation_extraction_stub.register_forward_hook(lambda m, i, o: seen.__setitem__('y', o))
    got = ex.output_norms(x)
    h.remove()
    assert got.shape == (6, 11) and tuple(seen['y'].shape) == (6, 11, 48)
    want = O.expert_output_norms(x.double(), ex.w1.double(), ex.b1.double(), ex.w2.double(), 'gelu')
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-6)


def test_vit_surgery_keeps_the_function_and_the_parameter_names():
    """ViT with torchvision's module tree: FFNs (mlp.0 / mlp.3) -> MoE layers, same logits with every expert running,
    gating data of every block from the patched forwards (reference: moe_models.py:55-78, 103-127)."""
    from d2dmoe_amd import add_routers, gpt2, vit
    torch.manual_seed(0)
    m = vit.VisionTransformer(image_size=32, patch_size=8, num_layers=2, num_heads=2, hidden_dim=32, mlp_dim=64,
                              num_classes=10).eval()
    with torch.no_grad():
        for n, prm in m.named_parameters():
            if n.endswith('bias'):
                prm.normal_(0.0, 0.05)
        m.class_token.normal_(0.0, 0.02)
    keys = set(m.state_dict())
    for k in ('conv_proj.weight', 'class_token', 'encoder.pos_embedding', 'encoder.layers.encoder_layer_1.ln_2.bias',
              'encoder.layers.encoder_layer_0.self_attention.in_proj_weight',
              'encoder.layers.encoder_layer_0.mlp.0.weight', 'encoder.layers.encoder_layer_0.mlp.3.bias',
              'encoder.ln.weight', 'heads.head.weight'):
        assert k in keys, k
    moe, names = gpt2.replace_with_moes(m, num_experts=8, experts_class='hip_kernel')
    assert names == ['encoder.layers.encoder_layer_0.mlp', 'encoder.layers.encoder_layer_1.mlp']
    labels = {n: torch.randperm(64, generator=torch.Generator().manual_seed(i)) % 8 for i, n in enumerate(names)}
    gpt2.split_original_parameters(m, moe, names, labels)
    x = torch.randn(3, 3, 32, 32, generator=torch.Generator().manual_seed(5))
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode = 'all'
        layer.experts.forward_mode = 'naive'
    with torch.no_grad():
        want = m(x)
        got, gating = moe(x, return_gating_data=True)
    assert H.rel_err(got, want) < 1e-5 and set(gating) == set(names)
    assert tuple(gating[names[0]][0].shape) == (3, 17, 8)
    add_routers(moe, dict(width=16, depth=2, bias=False, activation='relu', output_activation='abs'))
    for n in names:
        layer = gpt2.get_module_by_name(moe, n)
        layer.forward_mode, layer.tau = 'dynk_max', 0.5
    with torch.no_grad():
        out, gating = moe(x, return_gating_data=True)
    frac = gating[names[1]][0].float().mean().item()
    assert out.shape == (3, 10) and 0.0 < frac < 1.0


def test_bench_refuses_more_than_one_gpu():
    """The path is measured on one GPU; asking bench.py for more ends with a message that says so, before any GPU call."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert 'single-GPU' in (res.stderr + res.stdout)
    # ... and its usage text prints (argparse formats every help string with %)
    res = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--help'], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0 and '--workload' in res.stdout, res.stderr[-400:]


# ------------------------------------------------------------------ every experts container of the registry ----
def test_registry_holds_the_reference_keys():
    from d2dmoe_amd import MOE_IMPL_MAP
    assert {'execute_all', 'module', 'batched', 'custom_kernel'} <= set(MOE_IMPL_MAP)   # moe_layers.py:402-407


def _container_params(ex):
    """(w1, b1, w2, w_up) in the kernels' layout, read through the container's own accessor."""
    w1, b1, w2, w_up, _ = ex.hip_operands()
    return {'w1': w1.detach(), 'b1': None if b1 is None else b1.detach(), 'w2': w2.detach(),
            'w_up': None if w_up is None else w_up.detach()}


@pytest.mark.parametrize('experts_class,gated', [('custom_kernel', False), ('execute_all', False), ('execute_all', True),
                                                 ('module', False), ('module', True), ('batched', False)])
def test_container_pytorch_modes_match_oracle(experts_class, gated):
    from d2dmoe_amd import MoeficationMoE
    torch.manual_seed(3)
    bias = not gated
    moe = MoeficationMoE('m', 48, 5, bias, 12, nn.GELU, experts_class=experts_class, add_intermediate_gating=gated).eval()
    ex = moe.experts
    if bias and experts_class == 'batched':
        with torch.no_grad():
            ex.biases[0].uniform_(-0.2, 0.2)     # the reference initialises them to zero; make them count
    x = torch.randn(11, 48)
    routing = (torch.rand(11, 5) < 0.5).float() * torch.rand(11, 5)      # weighted routing, some zeros
    p = _container_params(ex)
    if gated:
        want = O.experts_gated_forward_all(x.double(), routing.double(), p['w1'].double(), p['w_up'].double(),
                                           p['w2'].double(), 'gelu')
    else:
        want = O.experts_forward_all(x.double(), routing.double(), p['w1'].double(), p['b1'].double(), p['w2'].double(),
                                     'gelu')
    with torch.no_grad():
        got = ex(x, routing)
    assert H.rel_err(got, want) < 1e-5
    # state_dict names follow the reference's containers
    keys = set(ex.state_dict())
    if experts_class == 'module':
        assert ('e.0.gate.weight' in keys and 'e.4.down_scale.weight' in keys) if gated else \
            ({'e.0.0.weight', 'e.0.0.bias', 'e.4.2.weight'} <= keys and 'e.0.2.bias' not in keys)
    if experts_class == 'batched':
        assert keys == {'weights.0', 'weights.1', 'biases.0', 'biases.1'}
    if experts_class == 'execute_all':
        assert 'layers.0.w' in keys and ('layers.2.w' in keys) == gated


class _GatedMLP(nn.Module):
    """The submodule layout of transformers' GemmaMLP."""

    def __init__(self, d, dff):
        super().__init__()
        self.gate_proj = nn.Linear(d, dff, bias=False)
        self.up_proj = nn.Linear(d, dff, bias=False)
        self.down_proj = nn.Linear(dff, d, bias=False)
        self.act_fn = H.GELUTanh()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


@pytest.mark.parametrize('experts_class,gated', [('custom_kernel', False), ('execute_all', False), ('execute_all', True),
                                                 ('module', False), ('module', True), ('batched', False)])
def test_param_split_fills_every_container(experts_class, gated):
    """With every expert running, the converted layer reproduces the dense FFN, for contiguous and shuffled labels."""
    from d2dmoe_amd import MoeficationMoE, gpt2
    torch.manual_seed(4)
    D, dff, E = 32, 48, 6
    if gated:
        ffn = _GatedMLP(D, dff).eval()
    else:
        ffn = nn.Sequential(nn.Linear(D, dff), nn.GELU(), nn.Dropout(0.0), nn.Linear(dff, D), nn.Dropout(0.0)).eval()
    assert gpt2.ffn_filter_condition(None, ffn)
    x = torch.randn(3, 4, D)
    with torch.no_grad():
        want = ffn(x)
    for labels in (None, torch.randperm(dff) % E):
        holder = nn.ModuleDict({'ffn': ffn})
        holder = __import__('copy').deepcopy(holder)
        gpt2.replace_layer_with_moe(holder, 'ffn', num_experts=E, experts_class=experts_class)
        moe = holder['ffn']
        assert isinstance(moe, MoeficationMoE) and moe.forward_mode == 'all'
        gpt2.param_split(ffn, moe, labels)
        with torch.no_grad():
            got, gating = moe(x)
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-5), (experts_class, gated)
        assert gating['ffn'][0].shape == (3, 4, E)


def test_operand_dtype_mismatch_is_refused_before_any_device_call():
    from d2dmoe_amd import D2DMoEError, ops
    x = torch.randn(4, 64).bfloat16()
    routing = torch.ones(4, 4).bfloat16()
    w1, b1, w2 = torch.randn(4, 64, 32), torch.randn(4, 32), torch.randn(4, 32, 64)    # float32 weights
    with pytest.raises(D2DMoEError, match='w1 is torch.float32'):
        ops.experts(x, routing, w1, b1, w2)
    with pytest.raises(D2DMoEError, match='routing is torch.float32'):
        ops.experts(x, routing.float(), w1.bfloat16(), b1.bfloat16(), w2.bfloat16())
    with pytest.raises(D2DMoEError, match='router_w1'):
        ops.forward(x, torch.randn(128, 64), torch.randn(4, 128).bfloat16(), 0.1, w1.bfloat16(), b1.bfloat16(), w2.bfloat16())


def test_grad_predicate_of_the_hip_paths():
    from d2dmoe_amd.experts import _grad_wanted
    w = nn.Parameter(torch.zeros(2))
    x = torch.zeros(2)
    assert _grad_wanted(x, w) and not _grad_wanted(x, None)
    with torch.no_grad():
        assert not _grad_wanted(x, w)
    w.requires_grad_(False)
    assert not _grad_wanted(x, w)
