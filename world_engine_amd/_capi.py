"""ctypes binding of the C ABI declared in ``include/we_attn.h`` (``libwe_attn.so``, the product)
and of the measurement library declared in ``include/we_attn_probe.h`` (``libwe_probe.so``, loaded
only by the benchmark and by the tests of its entry points).

Both are built in-tree by ``world_engine_amd/build.py`` (``hipcc`` for gfx950).  There is no
fallback: if a library is missing, every call into it raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwe_attn.so")
PROBE_LIB_PATH = os.path.join(_HERE, "libwe_probe.so")

WE_DTYPE_BF16, WE_DTYPE_F16, WE_DTYPE_F32 = 0, 1, 2
WE_MAX_SLOTS = 256
WE_STATIC_SCRATCH_BYTES = 32 << 20
WE_PLAN_FIELDS = 5
WE_CLOCK_SLOTS = 16
WE_ERR_SCRATCH_LIMIT = -7
WE_ERR_NOT_READY = -8

_I64x3 = POINTER(c_int64)

class AttnExtras(ctypes.Structure):
    """``we_attn_extras`` of include/we_attn.h."""
    _fields_ = [("qk_norm_eps", ctypes.c_float), ("v1", c_void_p), ("v1_strides", ctypes.c_int64 * 3),
                ("v_lamb", c_void_p), ("gate", c_void_p), ("gate_strides", ctypes.c_int64 * 3),
                ("gate_x", c_void_p), ("gate_x_strides", ctypes.c_int64 * 2), ("gate_w", c_void_p)]


class QkvProj(ctypes.Structure):
    """``we_qkv_proj`` of include/we_attn.h."""
    _fields_ = [("x", c_void_p), ("x_strides", ctypes.c_int64 * 2), ("w", c_void_p), ("w_row_stride", c_int64),
                ("d_model", c_int32), ("v_out", c_void_p), ("v_out_strides", ctypes.c_int64 * 3)]


# name -> (restype, argtypes); must list every symbol include/we_attn.h declares
SIGNATURES = {
    "we_version": (c_int32, []),
    "we_error_string": (c_char_p, [c_int32]),
    "we_rope_kv_store": (c_int32, [
        c_void_p, c_void_p, c_void_p,              # q, k, v
        _I64x3, _I64x3, _I64x3,                    # strides
        c_void_p,                                  # q_out
        c_void_p, c_void_p, c_int64,               # cos, sin, table_rows
        c_void_p, c_void_p, c_void_p,              # t_pos, y_pos, x_pos
        c_int64, c_int64, c_int64,                 # pos_stride_b, grid_h, grid_w
        c_void_p, c_void_p,                        # kv, written
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_int32, c_int32, c_void_p,       # dilation, is_frozen, dtype, stream
    ]),
    "we_rope_apply": (c_int32, [
        c_void_p, _I64x3, c_void_p,                # x, strides, x_out
        c_void_p, c_void_p, c_int64,               # cos, sin, table_rows
        c_void_p, c_void_p, c_void_p,              # t_pos, y_pos, x_pos
        c_int64, c_int64, c_int64,                 # pos_stride_b, grid_h, grid_w
        c_int32, c_int32, c_int32, c_int32,        # B H T Dh
        c_int32, c_void_p,                         # dtype, stream
    ]),
    "we_init": (c_int32, []),
    "we_attn_auto_splits": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int64]),
    "we_attn_plan": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_int32,
                               POINTER(c_int32)]),
    "we_attn_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32]),
    "we_attn_ring_fwd": (c_int32, [
        c_void_p, _I64x3,                          # q, q_strides
        c_void_p, c_void_p, c_void_p,              # kv, written, t_pos
        c_void_p, _I64x3,                          # out, out_strides
        c_void_p, c_size_t,                        # workspace, bytes
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_float, c_int32, c_int32, c_int32, c_void_p,  # dilation scale n_splits q_tile dtype stream
    ]),
    "we_attn_ring_fwd_static": (c_int32, [
        c_void_p, _I64x3,                          # q, q_strides
        c_void_p, c_void_p, c_void_p,              # kv, written, t_pos
        c_void_p, _I64x3,                          # out, out_strides
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_float, c_int32, c_int32, c_int32, c_void_p,  # dilation scale n_splits q_tile dtype stream
    ]),
    "we_rope_kv_attn_fwd": (c_int32, [
        c_void_p, c_void_p, c_void_p,              # q, k, v
        _I64x3, _I64x3, _I64x3,                    # strides
        c_void_p,                                  # q_out
        c_void_p, c_void_p, c_int64,               # cos, sin, table_rows
        c_void_p, c_void_p, c_void_p,              # t_pos, y_pos, x_pos
        c_int64, c_int64, c_int64,                 # pos_stride_b, grid_h, grid_w
        c_void_p, c_void_p,                        # kv, written
        c_void_p, _I64x3,                          # out, out_strides
        c_void_p, c_size_t,                        # workspace, bytes
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_int32, c_float, c_int32, c_int32, c_int32,  # dilation frozen scale n_splits q_tile dtype
        c_void_p, c_void_p,                        # extras (we_attn_extras* or NULL), stream
    ]),
    "we_qkv_rope_kv_store": (c_int32, [
        c_void_p, c_void_p,                        # proj (we_qkv_proj*), q_out
        c_void_p, c_void_p, c_int64,               # cos, sin, table_rows
        c_void_p, c_void_p, c_void_p,              # t_pos, y_pos, x_pos
        c_int64, c_int64, c_int64,                 # pos_stride_b, grid_h, grid_w
        c_void_p, c_void_p,                        # kv, written
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_int32, c_int32,                 # dilation, is_frozen, dtype
        c_void_p, c_void_p,                        # extras, stream
    ]),
    "we_qkv_rope_kv_attn_fwd": (c_int32, [
        c_void_p, c_void_p,                        # proj (we_qkv_proj*), q_out
        c_void_p, c_void_p, c_int64,               # cos, sin, table_rows
        c_void_p, c_void_p, c_void_p,              # t_pos, y_pos, x_pos
        c_int64, c_int64, c_int64,                 # pos_stride_b, grid_h, grid_w
        c_void_p, c_void_p,                        # kv, written
        c_void_p, _I64x3,                          # out, out_strides
        c_void_p, c_size_t,                        # workspace, bytes
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_int32, c_float, c_int32, c_int32, c_int32,  # dilation frozen scale n_splits q_tile dtype
        c_void_p, c_void_p,                        # extras, stream
    ]),
}

# the measurement library exports these on top of everything above; must list every symbol
# include/we_attn_probe.h declares
PROBE_SIGNATURES = {
    "we_attn_ring_fwd_clocked": (c_int32, [
        c_void_p, _I64x3,                          # q, q_strides
        c_void_p, c_void_p, c_void_p,              # kv, written, t_pos
        c_void_p, _I64x3,                          # out, out_strides
        c_void_p, c_size_t,                        # workspace, bytes
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,   # B H Hkv T Dh L
        c_int32, c_float, c_int32, c_int32, c_int32,            # dilation scale n_splits q_tile dtype
        c_void_p, c_size_t, c_void_p,              # clocks, clocks_len, stream
    ]),
    "we_stream_probe": (c_int32, [c_void_p, c_size_t, c_int32, c_int32, c_int32, c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension has not been built "
                "(run `python -m world_engine_amd.build`). There is no CPU or PyTorch fallback."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


_probe_lib = None


def probe_lib() -> ctypes.CDLL:
    """Load the measurement library once (benchmark and probe tests only); raise if it has not
    been built.  It carries its own copy of the product's entry points and per-device state."""
    global _probe_lib
    if _probe_lib is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise RuntimeError(f"{PROBE_LIB_PATH} is missing (run `python -m world_engine_amd.build`)")
        handle = ctypes.CDLL(PROBE_LIB_PATH)
        for name, (res, args) in {**SIGNATURES, **PROBE_SIGNATURES}.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _probe_lib = handle
    return _probe_lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().we_error_string(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")


def i64x3(a: int, b: int, c: int):
    return (c_int64 * 3)(a, b, c)
