"""ctypes binding of the C ABI in include/d2dmoe.h (libd2dmoe_hip.so, built in-tree by d2dmoe_amd.build).

The library is the only compute path of this package: there is no CPU or eager fallback behind these calls.
If the shared object is missing or fails to load, every call raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_size_t, c_uint32, c_uint64, c_void_p

LIB_NAME = 'libd2dmoe_hip.so'
# D2DMOE_LIB names another build of the same library (a full path); default is the in-tree one.
LIB_PATH = os.environ.get('D2DMOE_LIB') or os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

# enums of include/d2dmoe.h
F32, BF16, F16 = 0, 1, 2
E_STATIC_LIMIT = -8
E_PACKED = -9
PACKED_MAGIC = 0x4b50324d
STATIC_WORKSPACE_BYTES = 256 << 20
ACT = {'relu': 0, 'gelu': 1, 'tanh': 2, 'leaky_relu': 3, 'gelu_tanh': 4, 'silu': 5, 'identity': 6, 'abs': 7}
PATH = {'auto': 0, 'generic': 1, 'mfma_dense': 2, 'mfma_sparse': 3, 'mfma_decode': 4, 'mfma_gemm': 5,
        'mfma_mid': 6}

# every extern "C" symbol the header declares
EXPORTS = (
    'd2dmoe_version', 'd2dmoe_status_string', 'd2dmoe_workspace_bytes', 'd2dmoe_router', 'd2dmoe_select',
    'd2dmoe_router_select',
    'd2dmoe_build_permutation', 'd2dmoe_experts', 'd2dmoe_packed_bytes', 'd2dmoe_pack_weights', 'd2dmoe_forward',
    'd2dmoe_norms_packed_bytes', 'd2dmoe_pack_norms', 'd2dmoe_expert_output_norms', 'd2dmoe_forward_static',
    'd2dmoe_packed_desc_from_header', 'd2dmoe_packed_describe',
)


class Shape(Structure):
    """struct d2dmoe_shape"""
    _fields_ = [
        ('n_tokens', c_int64), ('d_model', c_int32), ('n_experts', c_int32), ('expert_dim', c_int32),
        ('router_width', c_int32), ('dtype', c_int32), ('activation', c_int32), ('gated', c_int32),
        ('add_residual', c_int32), ('router_activation', c_int32), ('router_output_activation', c_int32),
    ]


class PackedDesc(Structure):
    """struct d2dmoe_packed_desc: what a packed buffer was packed for (64 bytes)"""
    _fields_ = [
        ('magic', c_uint32), ('layout_version', c_uint32), ('dtype', c_int32), ('d_model', c_int32), ('n_experts', c_int32),
        ('expert_dim', c_int32), ('gated', c_int32), ('router_width', c_int32), ('sections', c_uint32),
        ('reserved0', c_uint32), ('bytes', c_uint64), ('reserved1', c_uint64 * 2),
    ]


class D2DMoEError(RuntimeError):
    pass


_lib = None


def load() -> ctypes.CDLL:
    """Loads the in-tree shared library (once) and declares the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise D2DMoEError(f'{LIB_PATH} is missing: build it with `python -m d2dmoe_amd.build` '
                          f'(or __graft_entry__.build()); there is no fallback path')
    lib = ctypes.CDLL(LIB_PATH)
    P, I32, I64, SZ = c_void_p, c_int32, c_int64, c_size_t
    SH = POINTER(Shape)
    PD = POINTER(PackedDesc)
    lib.d2dmoe_version.restype = ctypes.c_int
    lib.d2dmoe_version.argtypes = []
    lib.d2dmoe_status_string.restype = c_char_p
    lib.d2dmoe_status_string.argtypes = [ctypes.c_int]
    lib.d2dmoe_workspace_bytes.restype = SZ
    lib.d2dmoe_workspace_bytes.argtypes = [SH]
    lib.d2dmoe_router.restype = ctypes.c_int
    lib.d2dmoe_router.argtypes = [P, P, P, P, I64, I32, I32, I32, I32, I32, I32, P, SZ, P]
    lib.d2dmoe_select.restype = ctypes.c_int
    lib.d2dmoe_select.argtypes = [P, P, P, I64, I32, I32, c_float, P]
    lib.d2dmoe_router_select.restype = ctypes.c_int
    lib.d2dmoe_router_select.argtypes = [SH, P, P, P, P, PD, c_float, P, P, P, P, SZ, P]
    lib.d2dmoe_build_permutation.restype = ctypes.c_int
    lib.d2dmoe_build_permutation.argtypes = [P, I64, I32, I32, P, P, P, P, P, P, SZ, P]
    lib.d2dmoe_experts.restype = ctypes.c_int
    lib.d2dmoe_experts.argtypes = [SH, P, P, P, P, P, P, P, P, PD, P, I32, P, SZ, P]
    lib.d2dmoe_packed_bytes.restype = SZ
    lib.d2dmoe_packed_bytes.argtypes = [SH]
    lib.d2dmoe_pack_weights.restype = ctypes.c_int
    lib.d2dmoe_pack_weights.argtypes = [SH, P, P, P, P, P, P, P, SZ, PD, P]
    lib.d2dmoe_forward.restype = ctypes.c_int
    lib.d2dmoe_forward.argtypes = [SH, P, P, P, c_float, P, P, P, P, P, P, PD, P, P, P, P, P, I32, P, SZ, P]
    lib.d2dmoe_forward_static.restype = ctypes.c_int
    lib.d2dmoe_forward_static.argtypes = [SH, P, P, P, c_float, P, P, P, P, P, P, PD, P, P, P, P, P, I32, P]
    lib.d2dmoe_norms_packed_bytes.restype = SZ
    lib.d2dmoe_norms_packed_bytes.argtypes = [SH]
    lib.d2dmoe_pack_norms.restype = ctypes.c_int
    lib.d2dmoe_pack_norms.argtypes = [SH, P, P, P, P, SZ, P]
    lib.d2dmoe_expert_output_norms.restype = ctypes.c_int
    lib.d2dmoe_expert_output_norms.argtypes = [SH, P, P, P, P]
    lib.d2dmoe_packed_describe.restype = ctypes.c_int
    lib.d2dmoe_packed_describe.argtypes = [SH, PD]
    lib.d2dmoe_packed_desc_from_header.restype = ctypes.c_int
    lib.d2dmoe_packed_desc_from_header.argtypes = [P, PD]
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().d2dmoe_status_string(status).decode()
        raise D2DMoEError(f'{what} failed with status {status}: {msg}')
