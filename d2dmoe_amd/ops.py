"""Tensor-level wrappers over the C ABI: they take torch tensors living on a ROCm device, hand their device
pointers and torch's current HIP stream to libd2dmoe_hip.so, and return torch tensors.  torch is used for device
memory and streams only; all arithmetic happens in the HIP kernels.  None of these functions synchronises with
the host or copies device data back (the reference's kernel path has the same rule:
scripts/test_moe_implementations.py:78-83)."""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Tuple

import torch

from . import hip_abi as abi

_DTYPES = {torch.float32: abi.F32, torch.bfloat16: abi.BF16}
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise abi.D2DMoEError(f'unsupported dtype {t.dtype}: the HIP path handles float32 and bfloat16') from None


def _require_gpu(*tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise abi.D2DMoEError('the HIP path needs tensors on a ROCm device; there is no CPU fallback')
        if not t.is_contiguous():
            raise abi.D2DMoEError('the HIP path needs contiguous tensors')
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise abi.D2DMoEError('all tensors must live on the same device')
    return dev


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """Per-(device, stream) scratch buffer, grown on demand and reused between calls on that stream."""
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


def make_shape(n_tokens: int, d_model: int, n_experts: int, expert_dim: int, router_width: int, dtype_code: int,
               activation: str = 'relu', gated: bool = False, add_residual: bool = False,
               router_activation: str = 'relu', router_output_activation: str = 'abs') -> abi.Shape:
    for a in (activation, router_activation, router_output_activation):
        if a not in abi.ACT:
            raise abi.D2DMoEError(f'activation {a!r} has no HIP kernel (known: {sorted(abi.ACT)})')
    return abi.Shape(n_tokens, d_model, n_experts, expert_dim, router_width, dtype_code, abi.ACT[activation],
                     int(gated), int(add_residual), abi.ACT[router_activation], abi.ACT[router_output_activation])


def router(x: torch.Tensor, router_w1: torch.Tensor, router_w2: torch.Tensor, activation: str = 'relu',
           output_activation: str = 'abs') -> torch.Tensor:
    """norms [N,E] = out_act(act(x W1^T) W2^T) through d2dmoe_router."""
    dev = _require_gpu(x, router_w1, router_w2)
    lib = abi.load()
    n, d = x.shape
    w, e = router_w1.size(0), router_w2.size(0)
    assert router_w1.shape == (w, d) and router_w2.shape == (e, w)
    norms = torch.empty(n, e, dtype=x.dtype, device=dev)
    need = max(n * w * x.element_size(), 16)
    ws = _workspace(dev, need)
    abi.check(lib.d2dmoe_router(_ptr(x), _ptr(router_w1), _ptr(router_w2), _ptr(norms), n, d, w, e, _dtype_code(x),
                                abi.ACT[activation], abi.ACT[output_activation], _ptr(ws), ws.numel(), _stream()),
              'd2dmoe_router')
    return norms


def select(norms: torch.Tensor, thr_scale: float, want_counts: bool = False
           ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """routing [N,E] (0/1, dtype of norms) and optionally int32 counts [E] through d2dmoe_select."""
    dev = _require_gpu(norms)
    lib = abi.load()
    n, e = norms.shape
    routing = torch.empty_like(norms)
    counts = torch.empty(e, dtype=torch.int32, device=dev) if want_counts else None
    abi.check(lib.d2dmoe_select(_ptr(norms), _ptr(routing), _ptr(counts), n, e, _dtype_code(norms),
                                ctypes.c_float(thr_scale), _stream()), 'd2dmoe_select')
    return routing, counts


def router_select(x: torch.Tensor, router_w1: torch.Tensor, router_w2: torch.Tensor, thr_scale: float,
                  packed: Optional[torch.Tensor] = None, n_experts: Optional[int] = None, expert_dim: int = 1,
                  want_norms: bool = False, want_counts: bool = False, activation: str = 'relu',
                  output_activation: str = 'abs'):
    """Router MLP + dynamic-k selection through d2dmoe_router_select (one fused MFMA kernel when `packed` carries a
    router section for this shape).  Returns (routing [N,E], norms or None, counts or None)."""
    dev = _require_gpu(x, router_w1, router_w2, packed)
    lib = abi.load()
    n, d = x.shape
    w, e = router_w1.size(0), router_w2.size(0)
    sh = make_shape(n, d, e, expert_dim, w, _dtype_code(x), 'relu', router_activation=activation,
                    router_output_activation=output_activation)
    routing = torch.empty(n, e, dtype=x.dtype, device=dev)
    norms = torch.empty(n, e, dtype=x.dtype, device=dev) if want_norms else None
    counts = torch.empty(e, dtype=torch.int32, device=dev) if want_counts else None
    ws = _workspace(dev, max(lib.d2dmoe_workspace_bytes(ctypes.byref(sh)), 256))
    abi.check(lib.d2dmoe_router_select(ctypes.byref(sh), _ptr(x), _ptr(router_w1), _ptr(router_w2), _ptr(packed),
                                       ctypes.c_float(thr_scale), _ptr(norms), _ptr(routing), _ptr(counts), _ptr(ws),
                                       ws.numel(), _stream()), 'd2dmoe_router_select')
    return routing, norms, counts


def build_permutation(routing: torch.Tensor, reference_layout: bool = False):
    """offsets int32 [E+1], token_idx int32 [N*E] (first offsets[E] entries valid); with reference_layout also
    sort_indices / unsort_indices int64 [N,E] and bincounts int64 [E] as the reference's extract_indices returns."""
    dev = _require_gpu(routing)
    lib = abi.load()
    n, e = routing.shape
    offsets = torch.empty(e + 1, dtype=torch.int32, device=dev)
    token_idx = torch.empty(max(n * e, 1), dtype=torch.int32, device=dev)
    sort_idx = unsort_idx = bincounts = None
    if reference_layout:
        sort_idx = torch.empty(n, e, dtype=torch.int64, device=dev)
        unsort_idx = torch.empty(n, e, dtype=torch.int64, device=dev)
        bincounts = torch.empty(e, dtype=torch.int64, device=dev)
    sh = make_shape(n, 1, e, 1, 0, _dtype_code(routing))
    need = max(lib.d2dmoe_workspace_bytes(ctypes.byref(sh)), 16)
    ws = _workspace(dev, need)
    abi.check(lib.d2dmoe_build_permutation(_ptr(routing), n, e, _dtype_code(routing), _ptr(offsets), _ptr(token_idx),
                                           _ptr(sort_idx), _ptr(unsort_idx), _ptr(bincounts), _ptr(ws), ws.numel(),
                                           _stream()), 'd2dmoe_build_permutation')
    if reference_layout:
        return offsets, token_idx, sort_idx, unsort_idx, bincounts
    return offsets, token_idx


def packed_bytes(shape: abi.Shape) -> int:
    return abi.load().d2dmoe_packed_bytes(ctypes.byref(shape))


def pack_weights(shape: abi.Shape, w1, b1, w2, w_up=None, router_w1=None, router_w2=None) -> Optional[torch.Tensor]:
    """Derived MFMA-fragment-ordered weight buffer, or None when the shape has no MFMA kernel."""
    dev = _require_gpu(w1, b1, w2, w_up, router_w1, router_w2)
    lib = abi.load()
    nbytes = lib.d2dmoe_packed_bytes(ctypes.byref(shape))
    if nbytes == 0:
        return None
    packed = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    abi.check(lib.d2dmoe_pack_weights(ctypes.byref(shape), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(w_up), _ptr(router_w1),
                                      _ptr(router_w2), _ptr(packed), nbytes, _stream()), 'd2dmoe_pack_weights')
    return packed


def pack_norms(shape: abi.Shape, w1, b1, w2) -> Optional[torch.Tensor]:
    """Derived buffer of d2dmoe_expert_output_norms (first-layer fragments, bias, per-expert Gram matrices), or None
    when the kernel does not cover the shape."""
    dev = _require_gpu(w1, b1, w2)
    lib = abi.load()
    nbytes = lib.d2dmoe_norms_packed_bytes(ctypes.byref(shape))
    if nbytes == 0:
        return None
    packed = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    abi.check(lib.d2dmoe_pack_norms(ctypes.byref(shape), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(packed), nbytes, _stream()),
              'd2dmoe_pack_norms')
    return packed


def expert_output_norms(x: torch.Tensor, w1: torch.Tensor, b1: Optional[torch.Tensor], w2: torch.Tensor,
                        activation: str = 'relu', packed: Optional[torch.Tensor] = None) -> torch.Tensor:
    """norms [E,N] = | act(x w1[e] + b1[e]) w2[e] |_2 through d2dmoe_expert_output_norms (bf16, D = 768, Ed <= 32)."""
    dev = _require_gpu(x, w1, b1, w2, packed)
    lib = abi.load()
    n, d = x.shape
    e, _, ed = w1.shape
    sh = make_shape(n, d, e, ed, 0, _dtype_code(x), activation)
    if packed is None:
        packed = pack_norms(sh, w1, b1, w2)
    if packed is None:
        raise abi.D2DMoEError('d2dmoe_expert_output_norms does not cover this shape (bf16, D = 768, experts of <= 32 neurons)')
    out = torch.empty(e, n, dtype=x.dtype, device=dev)
    abi.check(lib.d2dmoe_expert_output_norms(ctypes.byref(sh), _ptr(x), _ptr(packed), _ptr(out), _stream()),
              'd2dmoe_expert_output_norms')
    return out


def experts(x: torch.Tensor, routing: torch.Tensor, w1: torch.Tensor, b1: Optional[torch.Tensor], w2: torch.Tensor,
            w_up: Optional[torch.Tensor] = None, last_bias: Optional[torch.Tensor] = None, activation: str = 'relu',
            add_residual: bool = False, path: str = 'auto', packed: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [N,D] = sum_e routing[n,e] * expert_e(x[n]) (+ last_bias) (+ x) through d2dmoe_experts."""
    dev = _require_gpu(x, routing, w1, b1, w2, w_up, last_bias, packed)
    lib = abi.load()
    n, d = x.shape
    e, _, ed = w1.shape
    assert routing.shape == (n, e) and w2.shape == (e, ed, d) and routing.dtype == x.dtype
    sh = make_shape(n, d, e, ed, 0, _dtype_code(x), activation, gated=w_up is not None, add_residual=add_residual)
    out = torch.empty_like(x)
    need = max(lib.d2dmoe_workspace_bytes(ctypes.byref(sh)), 16)
    ws = _workspace(dev, need)
    abi.check(lib.d2dmoe_experts(ctypes.byref(sh), _ptr(x), _ptr(routing), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(w_up),
                                 _ptr(last_bias), _ptr(packed), _ptr(out), abi.PATH[path], _ptr(ws), ws.numel(),
                                 _stream()), 'd2dmoe_experts')
    return out


def forward(x: torch.Tensor, router_w1: Optional[torch.Tensor], router_w2: Optional[torch.Tensor], thr_scale: float,
            w1: torch.Tensor, b1: Optional[torch.Tensor], w2: torch.Tensor, w_up: Optional[torch.Tensor] = None,
            last_bias: Optional[torch.Tensor] = None, activation: str = 'relu', add_residual: bool = False,
            norms_in: Optional[torch.Tensor] = None, want_norms: bool = False, want_counts: bool = False,
            path: str = 'auto', packed: Optional[torch.Tensor] = None, router_activation: str = 'relu',
            router_output_activation: str = 'abs'):
    """Whole layer through d2dmoe_forward.  x [N,D] -> (out [N,D], routing [N,E], norms or None, counts or None)."""
    dev = _require_gpu(x, router_w1, router_w2, w1, b1, w2, w_up, last_bias, norms_in, packed)
    lib = abi.load()
    n, d = x.shape
    e, _, ed = w1.shape
    w = router_w1.size(0) if router_w1 is not None else 0
    sh = make_shape(n, d, e, ed, w, _dtype_code(x), activation, gated=w_up is not None, add_residual=add_residual,
                    router_activation=router_activation, router_output_activation=router_output_activation)
    out = torch.empty_like(x)
    routing = torch.empty(n, e, dtype=x.dtype, device=dev)
    norms = torch.empty(n, e, dtype=x.dtype, device=dev) if (want_norms and norms_in is None) else None
    counts = torch.empty(e, dtype=torch.int32, device=dev) if want_counts else None
    need = max(lib.d2dmoe_workspace_bytes(ctypes.byref(sh)), 256)
    ws = _workspace(dev, need)
    abi.check(lib.d2dmoe_forward(ctypes.byref(sh), _ptr(x), _ptr(router_w1), _ptr(router_w2), ctypes.c_float(thr_scale),
                                 _ptr(w1), _ptr(b1), _ptr(w2), _ptr(w_up), _ptr(last_bias), _ptr(packed),
                                 _ptr(norms_in), _ptr(norms), _ptr(routing), _ptr(counts), _ptr(out), abi.PATH[path],
                                 _ptr(ws), ws.numel(), _stream()), 'd2dmoe_forward')
    return out, routing, (norms_in if norms_in is not None else norms), counts
