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

_DTYPES = {torch.float32: abi.F32, torch.bfloat16: abi.BF16, torch.float16: abi.F16}
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise abi.D2DMoEError(f'unsupported dtype {t.dtype}: the HIP path handles float32, bfloat16 and float16') from None


def _require_same_dtype(what: str, ref: torch.Tensor, **tensors: Optional[torch.Tensor]) -> None:
    """The kernels read every operand with the element type of `ref` (d2dmoe_shape.dtype): an operand of another dtype
    would be reinterpreted byte by byte, so it is refused here, before any pointer reaches the library."""
    for name, t in tensors.items():
        if t is not None and t.dtype != ref.dtype:
            raise abi.D2DMoEError(f'{what}: {name} is {t.dtype} but the activations are {ref.dtype}; the HIP path needs one '
                                  'element type for activations, routing and weights')


class PackedWeights(torch.Tensor):
    """The buffer d2dmoe_pack_weights wrote (a uint8 tensor) together with its descriptor, `desc` (abi.PackedDesc): what it
    was packed for.  Every call that takes the buffer hands the descriptor to the library, which refuses a buffer packed
    for another layer.  Tensor operations return plain tensors; use clone_packed() for a copy that keeps the descriptor."""

    @staticmethod
    def wrap(buf: torch.Tensor, desc: 'abi.PackedDesc') -> 'PackedWeights':
        out = buf.as_subclass(PackedWeights)
        out.desc = desc
        return out

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **(kwargs or {}))


def clone_packed(packed: 'PackedWeights') -> 'PackedWeights':
    """A copy of a packed buffer (other memory, same contents) with the same descriptor."""
    return PackedWeights.wrap(torch.Tensor.clone(packed), _desc_of(packed))


def packed_from_header(buf: torch.Tensor) -> 'PackedWeights':
    """Re-attaches the descriptor to a packed buffer that lost it (saved and loaded, copied): the buffer's first 64 bytes
    hold it.  Copies those bytes to the host (a synchronising copy)."""
    head = bytes(buf.view(torch.uint8)[:64].cpu().numpy())
    desc = abi.PackedDesc()
    abi.check(abi.load().d2dmoe_packed_desc_from_header(head, ctypes.byref(desc)), 'd2dmoe_packed_desc_from_header')
    return PackedWeights.wrap(buf, desc)


def _desc_of(packed: Optional[torch.Tensor]):
    if packed is None:
        return None
    desc = getattr(packed, 'desc', None)
    if desc is None:
        raise abi.D2DMoEError('packed buffer without its descriptor: pass what pack_weights returned (clone_packed() copies '
                              'it, packed_from_header() recovers the descriptor from a raw buffer)')
    return desc


def _pd(packed: Optional[torch.Tensor]):
    """The descriptor argument of a C call: a pointer to the buffer's descriptor, or NULL without a buffer."""
    desc = _desc_of(packed)
    return None if desc is None else ctypes.byref(desc)


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


def _workspace(dev: torch.device, nbytes: int, stream: Optional[int] = None) -> torch.Tensor:
    """Per-(device, stream) scratch buffer, grown on demand and reused between calls on that stream."""
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _stream() if stream is None else stream)
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
    _require_same_dtype('router', x, router_w1=router_w1, router_w2=router_w2)
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
    _require_same_dtype('router_select', x, router_w1=router_w1, router_w2=router_w2)
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
    abi.check(lib.d2dmoe_router_select(ctypes.byref(sh), _ptr(x), _ptr(router_w1), _ptr(router_w2), _ptr(packed), _pd(packed),
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
    _require_same_dtype('pack_weights', w1, b1=b1, w2=w2, w_up=w_up, router_w1=router_w1, router_w2=router_w2)
    if _dtype_code(w1) != shape.dtype:
        raise abi.D2DMoEError(f'pack_weights: the weights are {w1.dtype} but the shape names dtype code {shape.dtype}')
    dev = _require_gpu(w1, b1, w2, w_up, router_w1, router_w2)
    lib = abi.load()
    nbytes = lib.d2dmoe_packed_bytes(ctypes.byref(shape))
    if nbytes == 0:
        return None
    packed = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    desc = abi.PackedDesc()
    abi.check(lib.d2dmoe_pack_weights(ctypes.byref(shape), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(w_up), _ptr(router_w1),
                                      _ptr(router_w2), _ptr(packed), nbytes, ctypes.byref(desc), _stream()),
              'd2dmoe_pack_weights')
    return PackedWeights.wrap(packed, desc)


def pack_norms(shape: abi.Shape, w1, b1, w2) -> Optional[torch.Tensor]:
    """Derived buffer of d2dmoe_expert_output_norms (first-layer fragments, bias, per-expert Gram matrices), or None
    when the kernel does not cover the shape."""
    _require_same_dtype('pack_norms', w1, b1=b1, w2=w2)
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
    """norms [E,N] = | act(x w1[e] + b1[e]) w2[e] |_2 through d2dmoe_expert_output_norms (bf16 or float16, D a multiple of
    256 up to 2048, ungated experts of at most 64 neurons)."""
    _require_same_dtype('expert_output_norms', x, w1=w1, b1=b1, w2=w2)
    dev = _require_gpu(x, w1, b1, w2, packed)
    lib = abi.load()
    n, d = x.shape
    e, _, ed = w1.shape
    sh = make_shape(n, d, e, ed, 0, _dtype_code(x), activation)
    if packed is None:
        packed = pack_norms(sh, w1, b1, w2)
    if packed is None:
        raise abi.D2DMoEError('d2dmoe_expert_output_norms does not cover this shape (bf16 / float16, D a multiple of 256 up to 2048, '
                              'ungated experts of <= 64 neurons)')
    out = torch.empty(e, n, dtype=x.dtype, device=dev)
    abi.check(lib.d2dmoe_expert_output_norms(ctypes.byref(sh), _ptr(x), _ptr(packed), _ptr(out), _stream()),
              'd2dmoe_expert_output_norms')
    return out


def experts(x: torch.Tensor, routing: torch.Tensor, w1: torch.Tensor, b1: Optional[torch.Tensor], w2: torch.Tensor,
            w_up: Optional[torch.Tensor] = None, last_bias: Optional[torch.Tensor] = None, activation: str = 'relu',
            add_residual: bool = False, path: str = 'auto', packed: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [N,D] = sum_e routing[n,e] * expert_e(x[n]) (+ last_bias) (+ x) through d2dmoe_experts."""
    _require_same_dtype('experts', x, routing=routing, w1=w1, b1=b1, w2=w2, w_up=w_up, last_bias=last_bias)
    dev = _require_gpu(x, routing, w1, b1, w2, w_up, last_bias, packed)
    lib = abi.load()
    n, d = x.shape
    e, _, ed = w1.shape
    assert routing.shape == (n, e) and w2.shape == (e, ed, d)
    sh = make_shape(n, d, e, ed, 0, _dtype_code(x), activation, gated=w_up is not None, add_residual=add_residual)
    out = torch.empty_like(x)
    need = max(lib.d2dmoe_workspace_bytes(ctypes.byref(sh)), 16)
    ws = _workspace(dev, need)
    abi.check(lib.d2dmoe_experts(ctypes.byref(sh), _ptr(x), _ptr(routing), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(w_up),
                                 _ptr(last_bias), _ptr(packed), _pd(packed), _ptr(out), abi.PATH[path], _ptr(ws), ws.numel(),
                                 _stream()), 'd2dmoe_experts')
    return out


class PreparedForward:
    """d2dmoe_forward for one layer with everything that does not change from call to call resolved once: operand checks
    (device, contiguity, one element type, packed-buffer size), the weights' device pointers, the d2dmoe_shape and
    workspace size per token count.  A call then allocates the outputs, looks the stream and workspace up and makes the one
    library call.  The object keeps references to the tensors it was built from; build a new one when a weight tensor is
    replaced (in-place updates keep the pointers valid, but a packed buffer has to be rebuilt from them first)."""

    def __init__(self, d_model: int, dtype: torch.dtype, router_w1, router_w2, w1, b1, w2, w_up=None, last_bias=None,
                 activation: str = 'relu', add_residual: bool = False, packed=None, router_activation: str = 'relu',
                 router_output_activation: str = 'abs'):
        self.tensors = (router_w1, router_w2, w1, b1, w2, w_up, last_bias, packed)
        for name, t in zip(('router_w1', 'router_w2', 'w1', 'b1', 'w2', 'w_up', 'last_bias'), self.tensors):
            if t is not None and t.dtype != dtype:
                raise abi.D2DMoEError(f'forward: {name} is {t.dtype} but the activations are {dtype}; the HIP path needs '
                                      'one element type for activations, routing and weights')
        self.dtype = dtype
        self.code = _DTYPES.get(dtype)
        if self.code is None:
            raise abi.D2DMoEError(f'unsupported dtype {dtype}: the HIP path handles float32, bfloat16 and float16')
        self.dev = _require_gpu(*self.tensors)
        self.lib = abi.load()
        self.d = d_model
        self.e, _, self.ed = w1.shape
        assert w1.size(1) == d_model and w2.shape == (self.e, self.ed, d_model)
        self.w = router_w1.size(0) if router_w1 is not None else 0
        self.kw = dict(activation=activation, gated=w_up is not None, add_residual=add_residual,
                       router_activation=router_activation, router_output_activation=router_output_activation)
        self.ptrs = tuple(_ptr(t) for t in self.tensors)
        self.shapes = {}
        # the router section is the last one of a packed buffer: a buffer packed without it serves calls that bring their
        # own predicted norms (norms_in), and only those
        # the buffer's descriptor says what it was packed for; the library checks it against the shape of every call.  A
        # buffer packed without the router section serves calls that bring their own predicted norms (norms_in) -- and
        # calls that run the router on the unfused kernels.
        self.packed_desc = _desc_of(packed)
        self.pd = None if self.packed_desc is None else ctypes.byref(self.packed_desc)

    def shape_for(self, n: int):
        got = self.shapes.get(n)
        if got is None:
            sh = make_shape(n, self.d, self.e, self.ed, self.w, self.code, **self.kw)
            got = (sh, ctypes.byref(sh), max(self.lib.d2dmoe_workspace_bytes(ctypes.byref(sh)), 256))
            if len(self.shapes) > 64:
                self.shapes.clear()
            self.shapes[n] = got
        return got

    def __call__(self, x: torch.Tensor, thr_scale: float, norms_in=None, want_norms=False, want_counts=False,
                 path: str = 'auto', static_workspace: bool = False, out=None, routing=None, norms=None, counts=None):
        if x.dtype != self.dtype or (norms_in is not None and norms_in.dtype != self.dtype):
            raise abi.D2DMoEError(f'forward: the activations are {x.dtype} but the layer was prepared for {self.dtype}')
        if _require_gpu(x, norms_in, out, routing, norms, counts) != self.dev:
            raise abi.D2DMoEError('all tensors must live on the same device')
        n, d = x.shape
        assert d == self.d
        e = self.e
        _, shref, need = self.shape_for(n)
        dev = self.dev
        out = torch.empty_like(x) if out is None else out
        routing = torch.empty(n, e, dtype=x.dtype, device=dev) if routing is None else routing
        assert out.shape == x.shape and out.dtype == x.dtype and routing.shape == (n, e) and routing.dtype == x.dtype
        if norms is None and want_norms and norms_in is None:
            norms = torch.empty(n, e, dtype=x.dtype, device=dev)
        if counts is None and want_counts:
            counts = torch.empty(e, dtype=torch.int32, device=dev)
        rw1, rw2, w1, b1, w2, w_up, lb, pk = self.ptrs
        stream = _stream()
        if static_workspace:
            abi.check(self.lib.d2dmoe_forward_static(shref, x.data_ptr(), rw1, rw2, ctypes.c_float(thr_scale), w1, b1, w2,
                                                     w_up, lb, pk, self.pd, _ptr(norms_in), _ptr(norms), routing.data_ptr(),
                                                     _ptr(counts), out.data_ptr(), abi.PATH[path], stream),
                      'd2dmoe_forward_static')
        else:
            ws = _workspace(dev, need, stream)
            abi.check(self.lib.d2dmoe_forward(shref, x.data_ptr(), rw1, rw2, ctypes.c_float(thr_scale), w1, b1, w2, w_up, lb,
                                              pk, self.pd, _ptr(norms_in), _ptr(norms), routing.data_ptr(), _ptr(counts),
                                              out.data_ptr(), abi.PATH[path], ws.data_ptr(), ws.numel(), stream),
                      'd2dmoe_forward')
        return out, routing, (norms_in if norms_in is not None else norms), counts


def forward(x: torch.Tensor, router_w1: Optional[torch.Tensor], router_w2: Optional[torch.Tensor], thr_scale: float,
            w1: torch.Tensor, b1: Optional[torch.Tensor], w2: torch.Tensor, w_up: Optional[torch.Tensor] = None,
            last_bias: Optional[torch.Tensor] = None, activation: str = 'relu', add_residual: bool = False,
            norms_in: Optional[torch.Tensor] = None, want_norms: bool = False, want_counts: bool = False,
            path: str = 'auto', packed: Optional[torch.Tensor] = None, router_activation: str = 'relu',
            router_output_activation: str = 'abs', static_workspace: bool = False, out: Optional[torch.Tensor] = None,
            routing: Optional[torch.Tensor] = None, norms: Optional[torch.Tensor] = None,
            counts: Optional[torch.Tensor] = None):
    """Whole layer through d2dmoe_forward.  x [N,D] -> (out [N,D], routing [N,E], norms or None, counts or None).

    static_workspace=True goes through d2dmoe_forward_static instead: the workspace is the array inside the library, and
    when the caller also hands over `out` / `routing` (/ `norms` / `counts`) nothing at all is allocated by the call."""
    prepared = PreparedForward(x.size(1), x.dtype, router_w1, router_w2, w1, b1, w2, w_up, last_bias, activation,
                               add_residual, packed, router_activation, router_output_activation)
    return prepared(x, thr_scale, norms_in, want_norms, want_counts, path, static_workspace, out, routing, norms, counts)
