"""d2dmoe_forward_static: the whole layer with the workspace inside the library (no allocation by the entry point).

Called through the C ABI; its outputs are compared bit for bit with d2dmoe_forward's (same kernels, caller-owned
workspace) on two calls in a row, the second with a smaller input, so that whatever the first call left in the array is
there when the second runs.  Covers a path per workspace use: dense sweep with chunk-split tail (float32 partial sums),
expert-major (plan, per-pair rows, device flag; also with the plan's first pass written by the router kernel, and at
D = 1024 with the tiled products' region behind it), small batch (hidden fragments, expert flags), tiled products.
"""
import ctypes

import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu

DEV = 'cuda:0'


def _call(static, x, d, tau, act, gated, packed, bufs=None):
    from d2dmoe_amd import ops
    w1, b1, w2, w_up = (d['w_gate'], None, d['w_down'], d['w_up']) if gated else (d['w1'], d['b1'], d['w2'], None)
    lb = d['last_bias'].view(-1) if 'last_bias' in d else None
    kw = dict(bufs or {})
    return ops.forward(x, d['router_w1'], d['router_w2'], float(1.0 - tau), w1, b1, w2, w_up, lb, act, True, None, True, True,
                       'auto', packed, static_workspace=static, **kw)


@pytest.mark.parametrize('name,D,E,Ed,W,act,gated,tau,sizes', [
    ('vit dense sweep', 768, 128, 24, 128, 'relu', False, 0.9, (1576, 300)),
    ('vit expert-major', 768, 128, 24, 128, 'gelu', False, 0.1, (1576, 197)),
    ('gemma small batch', 2048, 256, 64, 256, 'gelu_tanh', True, 0.9, (16, 5)),
    ('gemma tiled products', 2048, 256, 64, 256, 'gelu_tanh', True, 0.9, (600, 200)),
    ('gemma expert-major', 2048, 256, 64, 256, 'gelu_tanh', True, 0.1, (300, 100)),
    # from 16 384 tokens on the router kernel also writes the expert-major plan's per-segment counts into the workspace
    ('vit expert-major, resident router', 768, 128, 24, 128, 'relu', False, 0.1, (16500, 16390)),
    ('gpt2-medium width expert-major', 1024, 128, 32, 128, 'gelu', False, 0.1, (2000, 700)),
])
def test_static_workspace_forward_equals_forward(name, D, E, Ed, W, act, gated, tau, sizes):
    from d2dmoe_amd import ops
    print('static', name, flush=True)
    _, _, p = H.random_case(8, D, E, Ed, W, seed=3, dtype=torch.bfloat16, gated=gated, bias=not gated)
    d = H.to_dev(p, DEV)
    sh = ops.make_shape(0, D, E, Ed, W, 1, act, gated=gated)
    packed = ops.pack_weights(sh, d['w_gate'] if gated else d['w1'], d.get('b1'), d['w_down'] if gated else d['w2'],
                              d.get('w_up'), d['router_w1'], d['router_w2'])
    got = None
    for i, n in enumerate(sizes):
        del got                                                  # the previous round's tensors go before the count below
        x = torch.randn(n, D, generator=torch.Generator().manual_seed(50 + i)).bfloat16().to(DEV)
        want = _call(False, x, d, tau, act, gated, packed)
        # caller-owned outputs, filled with a pattern first: the entry point has to write all of them
        bufs = dict(out=torch.full_like(x, 7.0), routing=torch.full((n, E), 7.0, dtype=x.dtype, device=DEV),
                    norms=torch.full((n, E), 7.0, dtype=x.dtype, device=DEV),
                    counts=torch.full((E,), -1, dtype=torch.int32, device=DEV))
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        got = _call(True, x, d, tau, act, gated, packed, bufs)
        assert torch.cuda.memory_allocated() == before          # nothing came from torch's allocator either
        torch.cuda.synchronize()
        for g, w_, what in zip(got, want, ('out', 'routing', 'norms', 'counts')):
            assert torch.equal(g, w_), (name, n, what)
        assert got[0].data_ptr() == bufs['out'].data_ptr()
        k = got[1].float().sum(1).mean().item()
        print(f'  {n} tokens: {k:.1f} experts/token, outputs bit-equal', flush=True)


def test_static_workspace_limit_is_reported():
    """A shape whose workspace exceeds the array is refused before anything is launched, with its own status code."""
    from d2dmoe_amd import hip_abi as abi, ops
    lib = abi.load()
    sh = ops.make_shape(50432, 768, 128, 24, 128, abi.BF16)
    assert lib.d2dmoe_workspace_bytes(ctypes.byref(sh)) > abi.STATIC_WORKSPACE_BYTES
    dummy = torch.zeros(64, dtype=torch.bfloat16, device=DEV)
    ptr = dummy.data_ptr()
    st = lib.d2dmoe_forward_static(ctypes.byref(sh), ptr, ptr, ptr, ctypes.c_float(0.1), ptr, ptr, ptr, None, None, None,
                                   None, None, None, ptr, None, ptr, 0, None)
    assert st == abi.E_STATIC_LIMIT
    assert b'static' in lib.d2dmoe_status_string(st)
    small = ops.make_shape(1576, 768, 128, 24, 128, abi.BF16)
    assert 0 < lib.d2dmoe_workspace_bytes(ctypes.byref(small)) <= abi.STATIC_WORKSPACE_BYTES
