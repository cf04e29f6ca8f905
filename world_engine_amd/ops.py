"""Python entry points of the HIP kernels (thin wrappers over the C ABI, no fallbacks).

Every function enqueues on the calling thread's current torch stream and returns at once; no
host synchronisation happens here, so calls can be captured into a HIP graph.  Tensors must live
on a ROCm device; anything else raises.
"""
from __future__ import annotations

import ctypes
import math
from typing import Mapping, Optional, Tuple

import torch

from . import _capi

Tensor = torch.Tensor

_DTYPE_CODE = {torch.bfloat16: _capi.WE_DTYPE_BF16, torch.float16: _capi.WE_DTYPE_F16,
               torch.float32: _capi.WE_DTYPE_F32}


def _dtype_code(t: Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported element type {t.dtype}") from None


def _need_device(*tensors: Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise RuntimeError("world_engine_amd kernels run on a ROCm GPU only; got a tensor on "
                               f"{t.device} (there is no CPU path)")
        if t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def _stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


_initialised = set()   # (library handle id, device index) pairs whose one-time set-up has run


def init(device=None, probe: bool = False) -> None:
    """One-time set-up of a device for the library (``we_init``): kernel LDS limits, the static
    scratch buffer's address, the compute-unit count.  Every wrapper here does it on first use;
    code that captures HIP graphs without an eager warm-up call calls this first (the set-up's
    runtime calls do not belong into a capture)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    lib = _capi.probe_lib() if probe else _capi.lib()
    key = (id(lib), dev.index)
    if key in _initialised:
        return
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("world_engine_amd: the first call on a device cannot be made under graph capture; call "
                           "world_engine_amd.ops.init(device) (or make one eager call) beforehand")
    with torch.cuda.device(dev):
        _capi.check(lib.we_init(), "we_init")
    _initialised.add(key)


def _call(dev: torch.device, fn, *args, probe: bool = False):
    """Call a library entry point with the tensors' device current: the library launches its
    kernels on the device that is current when it is called and keeps per-device facts (LDS limits,
    the static scratch buffer's address).  No overhead when it already is."""
    if (id(_capi.probe_lib() if probe else _capi.lib()), dev.index) not in _initialised:
        init(dev, probe)
    if dev.index == torch.cuda.current_device():
        return fn(*args)
    with torch.cuda.device(dev):
        return fn(*args)


def _bhtd_strides(t: Tensor, what: str):
    if t.dim() != 4 or t.stride(3) != 1:
        raise RuntimeError(f"{what} must be [B, H, T, Dh] with a contiguous last dimension")
    return _capi.i64x3(t.stride(0), t.stride(1), t.stride(2))


def _pos_triplet(pos_ids: Mapping[str, Tensor], B: int, T: int, need_yx: bool):
    """Returns (t_pos, y_pos, x_pos, row_stride); y/x are None when not needed."""
    t_pos = pos_ids["t_pos"]
    if tuple(t_pos.shape) != (B, T):
        raise RuntimeError("t_pos must be [B, T]")
    if t_pos.dtype != torch.long:
        raise RuntimeError("position ids must be int64")
    if not need_yx:
        if t_pos.stride(1) != 1 and T > 1:
            t_pos = t_pos.contiguous()
        return t_pos, None, None, t_pos.stride(0)
    y_pos, x_pos = pos_ids["y_pos"], pos_ids["x_pos"]
    for p in (y_pos, x_pos):
        if tuple(p.shape) != (B, T) or p.dtype != torch.long:
            raise RuntimeError("y_pos / x_pos must be int64 [B, T]")
    same = all(p.stride(1) == 1 and p.stride(0) == t_pos.stride(0) for p in (t_pos, y_pos, x_pos))
    if not same:
        t_pos, y_pos, x_pos = (p.contiguous() for p in (t_pos, y_pos, x_pos))
    return t_pos, y_pos, x_pos, t_pos.stride(0)


def _check_cache(kv: Tensor, written: Tensor, B: int, Hkv: int, T: int, Dh: int, L: int) -> None:
    if kv.dim() != 5 or tuple(kv.shape) != (2, B, Hkv, L + T, Dh) or not kv.is_contiguous():
        raise RuntimeError("kv must be a contiguous [2, B, Hkv, L+T, Dh] buffer; "
                           "KV cache expects exactly one frame per upsert")
    if written.dtype != torch.bool or written.numel() != L + T or not written.is_contiguous():
        raise RuntimeError("written must be a contiguous bool [L+T] tensor")


def _check_tables(cos_table: Tensor, sin_table: Tensor, Dh: int) -> None:
    if (cos_table.dtype != torch.float32 or sin_table.dtype != torch.float32
            or cos_table.shape != sin_table.shape or cos_table.dim() != 2 or cos_table.shape[1] != Dh // 2
            or not cos_table.is_contiguous() or not sin_table.is_contiguous()):
        raise RuntimeError("cos/sin tables must be contiguous fp32 [rows, Dh/2]")


def rope_kv_store(q: Optional[Tensor], k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor],
                  cos_table: Optional[Tensor], sin_table: Optional[Tensor],
                  grid_h: int, grid_w: int, kv: Tensor, written: Tensor, L: int, dilation: int,
                  is_frozen: bool) -> Optional[Tensor]:
    """Fused RoPE(q), RoPE(k) + tail / ring-slot store of (k, v) + ``written`` update.

    Replaces ``src/model/attn.py:110`` and ``src/model/kv_cache.py:191-193,126-151`` of the
    reference for one frame.  ``kv`` ``[2,B,Hkv,L+T,Dh]`` and ``written`` ``[L+T]`` are mutated
    in place.  With ``cos_table is None`` nothing is rotated (k already rotated by the caller).
    Returns RoPE(q) (contiguous ``[B,H,T,Dh]``) or ``None`` when ``q`` is ``None``.
    """
    dev = _need_device(k, v, kv, written, q, cos_table, sin_table, pos_ids["t_pos"])
    if k.dim() != 4 or k.shape != v.shape:
        raise RuntimeError("k and v must both be [B, Hkv, T, Dh]")
    B, Hkv, T, Dh = k.shape
    if k.dtype != kv.dtype or v.dtype != kv.dtype or (q is not None and q.dtype != kv.dtype):
        raise RuntimeError("q/k/v must have the cache's element type")
    _check_cache(kv, written, B, Hkv, T, Dh, L)
    H = Hkv
    q_out = None
    if q is not None:
        if q.dim() != 4 or q.shape[0] != B or q.shape[2] != T or q.shape[3] != Dh:
            raise RuntimeError("q must be [B, H, T, Dh] matching k")
        H = q.shape[1]
        q_out = torch.empty((B, H, T, Dh), dtype=q.dtype, device=dev)
    rotate = cos_table is not None
    if rotate:
        _check_tables(cos_table, sin_table, Dh)
    t_pos, y_pos, x_pos, ps = _pos_triplet(pos_ids, B, T, rotate)
    code = _call(
        dev, _capi.lib().we_rope_kv_store,
        q.data_ptr() if q is not None else None, k.data_ptr(), v.data_ptr(),
        _bhtd_strides(q, "q") if q is not None else None, _bhtd_strides(k, "k"), _bhtd_strides(v, "v"),
        q_out.data_ptr() if q_out is not None else None,
        cos_table.data_ptr() if rotate else None, sin_table.data_ptr() if rotate else None,
        cos_table.shape[0] if rotate else 0,
        t_pos.data_ptr(), y_pos.data_ptr() if rotate else None, x_pos.data_ptr() if rotate else None,
        ps, grid_h, grid_w, kv.data_ptr(), written.data_ptr(),
        B, H, Hkv, T, Dh, L, dilation, int(bool(is_frozen)), _dtype_code(kv), _stream_ptr(dev))
    _capi.check(code, "we_rope_kv_store")
    return q_out


def rope_apply(x: Tensor, pos_ids: Mapping[str, Tensor], cos_table: Tensor, sin_table: Tensor,
               grid_h: int, grid_w: int) -> Tensor:
    """Stand-alone RoPE of one ``[B,H,T,Dh]`` tensor (``src/model/attn.py:33-40``)."""
    dev = _need_device(x, cos_table, sin_table, pos_ids["t_pos"])
    if x.dim() != 4:
        raise RuntimeError("x must be [B, H, T, Dh]")
    B, H, T, Dh = x.shape
    if cos_table.dtype != torch.float32 or sin_table.dtype != torch.float32:
        raise RuntimeError("cos/sin tables must be fp32")
    if cos_table.shape != sin_table.shape or cos_table.dim() != 2 or cos_table.shape[1] != Dh // 2:
        raise RuntimeError("cos/sin tables must be [rows, Dh/2]")
    t_pos, y_pos, x_pos, ps = _pos_triplet(pos_ids, B, T, True)
    out = torch.empty((B, H, T, Dh), dtype=x.dtype, device=dev)
    code = _call(
        dev, _capi.lib().we_rope_apply,
        x.data_ptr(), _bhtd_strides(x, "x"), out.data_ptr(),
        cos_table.contiguous().data_ptr(), sin_table.contiguous().data_ptr(), cos_table.shape[0],
        t_pos.data_ptr(), y_pos.data_ptr(), x_pos.data_ptr(), ps, grid_h, grid_w,
        B, H, T, Dh, _dtype_code(x), _stream_ptr(dev))
    _capi.check(code, "we_rope_apply")
    return out


def attn_auto_splits(B: int, H: int, Hkv: int, T: int, Dh: int, L: int) -> int:
    return int(_capi.lib().we_attn_auto_splits(B, H, Hkv, T, Dh, L))


def attn_workspace_bytes(B: int, H: int, Hkv: int, T: int, Dh: int, L: int, n_splits: int = 0,
                         q_tile: int = 0) -> int:
    """Bytes of split-context workspace ``attn_ring`` needs for these sizes and knobs."""
    return int(_capi.lib().we_attn_workspace_bytes(B, H, Hkv, T, Dh, L, n_splits, q_tile))


def attn_plan(B: int, H: int, Hkv: int, T: int, Dh: int, L: int, n_splits: int = 0, q_tile: int = 0,
              compute_units: int = 0) -> dict:
    """What the library would do with an attention call of these sizes (``we_attn_plan``; launches
    nothing, needs no GPU when ``compute_units`` is given)."""
    out = (ctypes.c_int32 * _capi.WE_PLAN_FIELDS)()
    code = _capi.lib().we_attn_plan(B, H, Hkv, T, Dh, L, n_splits, q_tile, compute_units, out)
    _capi.check(code, "we_attn_plan")
    return {"q_tile": out[0], "n_splits": out[1], "units_whole": out[2], "workgroups": out[3], "compute_units": out[4]}


def attn_ring(q: Tensor, kv: Tensor, written: Tensor, t_pos: Tensor, L: int, dilation: int,
              scale: Optional[float] = None, n_splits: int = 0, q_tile: int = 0,
              out: Optional[Tensor] = None, workspace: Optional[Tensor] = None,
              token_major_out: bool = True, clocks: Optional[Tensor] = None) -> Tensor:
    """Attention of one frame's queries over the visible part of the ring buffer.

    Replaces ``make_block_mask`` + ``flex_attention`` (``src/model/kv_cache.py:141-144``,
    ``src/model/attn.py:116``).  ``q`` ``[B,H,T,Dh]`` (any batch/head/token strides), ``kv``
    ``[2,B,Hkv,L+T,Dh]``, ``written`` ``[L+T]`` bool, ``t_pos`` int64 with the frame index at
    element 0.  Returns ``[B,H,T,Dh]``; with ``token_major_out`` its memory is ``[B,T,H,Dh]`` so
    that ``y.transpose(1, 2).reshape(B, T, H*Dh)`` is a view (``src/patch_model.py:139``).
    ``workspace`` (split-context scratch, uint8, ``attn_workspace_bytes`` long) is allocated when not given.
    ``clocks`` (int64 device tensor): the call goes through the measurement library
    (``libwe_probe.so``, ``we_attn_ring_fwd_clocked``), which also leaves, per workgroup of the main
    kernel, its duration in shader-clock cycles and in ticks of the constant 100 MHz counter.
    """
    dev = _need_device(q, kv, written, t_pos)
    if q.dim() != 4:
        raise RuntimeError("q must be [B, H, T, Dh]")
    B, H, T, Dh = q.shape
    if kv.dim() != 5 or kv.shape[0] != 2 or kv.shape[1] != B or kv.shape[3] != L + T or kv.shape[4] != Dh:
        raise RuntimeError("kv must be [2, B, Hkv, L+T, Dh] matching q")
    if not kv.is_contiguous() or kv.dtype != q.dtype:
        raise RuntimeError("kv must be contiguous and of q's element type")
    Hkv = kv.shape[2]
    if written.dtype != torch.bool or written.numel() != L + T or not written.is_contiguous():
        raise RuntimeError("written must be a contiguous bool [L+T] tensor")
    if t_pos.dtype != torch.long or t_pos.numel() < 1:
        raise RuntimeError("t_pos must be a non-empty int64 tensor")
    scale = 1.0 / math.sqrt(Dh) if scale is None else float(scale)
    lib = _capi.probe_lib() if clocks is not None else _capi.lib()
    with torch.cuda.device(dev):      # (the size depends on the device's compute-unit count)
        ws_bytes = int(lib.we_attn_workspace_bytes(B, H, Hkv, T, Dh, L, n_splits, q_tile))
    if ws_bytes and (workspace is None or workspace.numel() * workspace.element_size() < ws_bytes):
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    if out is None:
        if token_major_out:
            out = torch.empty((B, T, H, Dh), dtype=q.dtype, device=dev).transpose(1, 2)
        else:
            out = torch.empty((B, H, T, Dh), dtype=q.dtype, device=dev)
    elif tuple(out.shape) != (B, H, T, Dh) or out.dtype != q.dtype or out.device != dev:
        raise RuntimeError("out must be [B, H, T, Dh] of q's element type on q's device")
    common = (q.data_ptr(), _bhtd_strides(q, "q"), kv.data_ptr(), written.data_ptr(), t_pos.data_ptr(),
              out.data_ptr(), _bhtd_strides(out, "out"),
              workspace.data_ptr() if ws_bytes else None,
              workspace.numel() * workspace.element_size() if ws_bytes else 0,
              B, H, Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, _dtype_code(q))
    if clocks is not None:
        if clocks.dtype != torch.int64 or not clocks.is_contiguous() or clocks.device != dev:
            raise RuntimeError("clocks must be a contiguous int64 tensor on q's device")
        code = _call(dev, lib.we_attn_ring_fwd_clocked, *common, clocks.data_ptr(), clocks.numel(), _stream_ptr(dev),
                     probe=True)
        _capi.check(code, "we_attn_ring_fwd_clocked")
    else:
        code = _call(dev, lib.we_attn_ring_fwd, *common, _stream_ptr(dev))
        _capi.check(code, "we_attn_ring_fwd")
    return out


def attn_ring_static(q: Tensor, kv: Tensor, written: Tensor, t_pos: Tensor, L: int, dilation: int, out: Tensor,
                     scale: Optional[float] = None, n_splits: int = 0, q_tile: int = 0) -> Tensor:
    """``attn_ring`` through ``we_attn_ring_fwd_static``: no workspace argument and no allocation
    anywhere (``out`` must be given); the split-context partial results go to a buffer inside the
    library's device image (``_capi.WE_STATIC_SCRATCH_BYTES``).  Sizes that need more raise.  Calls
    that overlap on one GPU race on that buffer.  No counterpart in the reference; for callers
    that cannot allocate."""
    dev = _need_device(q, kv, written, t_pos, out)
    if q.dim() != 4:
        raise RuntimeError("q must be [B, H, T, Dh]")
    B, H, T, Dh = q.shape
    if kv.dim() != 5 or kv.shape[0] != 2 or kv.shape[1] != B or kv.shape[3] != L + T or kv.shape[4] != Dh:
        raise RuntimeError("kv must be [2, B, Hkv, L+T, Dh] matching q")
    if not kv.is_contiguous() or kv.dtype != q.dtype:
        raise RuntimeError("kv must be contiguous and of q's element type")
    if written.dtype != torch.bool or written.numel() != L + T or not written.is_contiguous():
        raise RuntimeError("written must be a contiguous bool [L+T] tensor")
    if t_pos.dtype != torch.long or t_pos.numel() < 1:
        raise RuntimeError("t_pos must be a non-empty int64 tensor")
    if tuple(out.shape) != (B, H, T, Dh) or out.dtype != q.dtype:
        raise RuntimeError("out must be [B, H, T, Dh] of q's element type on q's device")
    scale = 1.0 / math.sqrt(Dh) if scale is None else float(scale)
    code = _call(   # (the buffer's address is per device: the call must see q's device as current)
        dev, _capi.lib().we_attn_ring_fwd_static,
        q.data_ptr(), _bhtd_strides(q, "q"), kv.data_ptr(), written.data_ptr(), t_pos.data_ptr(),
        out.data_ptr(), _bhtd_strides(out, "out"), B, H, kv.shape[2], T, Dh, L, dilation, scale, n_splits, q_tile,
        _dtype_code(q), _stream_ptr(dev))
    _capi.check(code, "we_attn_ring_fwd_static")
    return out


def stream_probe(buf: Tensor, workgroups: int, tiles: int, share: int = 1) -> None:
    """Measurement library (``libwe_probe.so``, ``we_stream_probe``): ``workgroups`` workgroups each stream ``tiles`` 16-KB
    tiles of ``buf`` into LDS the way the attention kernel fetches K/V tiles at 256-token frames,
    ``share`` workgroups per region, and compute nothing.  Time the launches from outside."""
    dev = _need_device(buf)
    if not buf.is_contiguous():
        raise RuntimeError("buf must be contiguous")
    code = _call(dev, _capi.probe_lib().we_stream_probe, buf.data_ptr(), buf.numel() * buf.element_size(), workgroups,
                 tiles, share, _stream_ptr(dev), probe=True)
    _capi.check(code, "we_stream_probe")


def _build_extras(dtype, B, H, Hkv, T, Dh, qk_norm_eps, v1, v_lamb, gate, gate_x, gate_w):
    """``we_attn_extras`` for a call, or None.  Returns (pointer or None, object to keep alive)."""
    if not (qk_norm_eps or v1 is not None or gate is not None or gate_w is not None):
        return None, None
    ex = _capi.AttnExtras()
    ex.qk_norm_eps = float(qk_norm_eps)
    if v1 is not None:
        if (v_lamb is None or v_lamb.numel() != 1 or v_lamb.dtype != dtype or tuple(v1.shape) != (B, Hkv, T, Dh)
                or v1.dtype != dtype):
            raise RuntimeError("v1 must match v and v_lamb must be one element of the same type")
        _need_device(v1, v_lamb)
        ex.v1, ex.v_lamb = v1.data_ptr(), v_lamb.data_ptr()
        ex.v1_strides = _bhtd_strides(v1, "v1")
    if gate is not None:
        if tuple(gate.shape) != (B, H, T) or gate.dtype != dtype:
            raise RuntimeError("gate must be [B, H, T] of q's element type")
        _need_device(gate)
        ex.gate = gate.data_ptr()
        ex.gate_strides = _capi.i64x3(*gate.stride())
    if gate_w is not None:
        if gate is not None:
            raise RuntimeError("give either gate or gate_x / gate_w")
        if (gate_x is None or gate_x.dim() != 3 or tuple(gate_x.shape) != (B, T, H) or gate_x.stride(2) != 1
                or gate_x.dtype != dtype or tuple(gate_w.shape) != (H, H) or gate_w.dtype != dtype
                or not gate_w.is_contiguous()):
            raise RuntimeError("gate_x must be [B, T, H] (contiguous channels) and gate_w a contiguous [H, H], "
                               "both of q's element type")
        _need_device(gate_x, gate_w)
        ex.gate_x, ex.gate_w = gate_x.data_ptr(), gate_w.data_ptr()
        ex.gate_x_strides = (ctypes.c_int64 * 2)(gate_x.stride(0), gate_x.stride(1))
    return ctypes.byref(ex), ex


def rope_kv_attn(q: Tensor, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], cos_table: Tensor,
                 sin_table: Tensor, grid_h: int, grid_w: int, kv: Tensor, written: Tensor, L: int,
                 dilation: int, is_frozen: bool, scale: Optional[float] = None, n_splits: int = 0,
                 q_tile: int = 0, out: Optional[Tensor] = None, workspace: Optional[Tensor] = None,
                 token_major_out: bool = True, qk_norm_eps: float = 0.0, v1: Optional[Tensor] = None,
                 v_lamb: Optional[Tensor] = None, gate: Optional[Tensor] = None,
                 gate_x: Optional[Tensor] = None, gate_w: Optional[Tensor] = None, q_rot: Optional[Tensor] = None):
    """``rope_kv_store`` followed by ``attn_ring`` in one library call (``we_rope_kv_attn_fwd``):
    the per-layer sequence of the reference from ``q, k = rope(q), rope(k)`` to the
    ``flex_attention`` call (``src/model/attn.py:110-116``), validated as a whole before the first
    launch.  Returns ``(out, q_rot)``; results are those of the two separate calls, bit for bit.
    ``out``, ``workspace`` and ``q_rot`` (contiguous ``[B,H,T,Dh]``) are allocated when not given.

    Optional neighbours of the path done inside the kernels (``src/model/attn.py:105-109,117-119``):
    ``qk_norm_eps > 0`` RMS-normalises q and k rows first (``F.rms_norm`` without weight; torch's
    epsilon for low-precision inputs is ``torch.finfo(torch.float32).eps``); ``v1`` ``[B,Hkv,T,Dh]``
    with the one-element ``v_lamb`` stores ``lerp(v, v1, v_lamb)``; ``gate`` ``[B,H,T]`` (any
    strides, sigmoid applied) multiplies the output rows.  These match the separate torch operations
    to 1 ulp of the element type (row reduction order, fused multiply-add in the lerp)."""
    dev = _need_device(q, k, v, kv, written, cos_table, sin_table, pos_ids["t_pos"])
    if k.dim() != 4 or k.shape != v.shape:
        raise RuntimeError("k and v must both be [B, Hkv, T, Dh]")
    B, Hkv, T, Dh = k.shape
    if q.dim() != 4 or q.shape[0] != B or q.shape[2] != T or q.shape[3] != Dh:
        raise RuntimeError("q must be [B, H, T, Dh] matching k")
    H = q.shape[1]
    if k.dtype != kv.dtype or v.dtype != kv.dtype or q.dtype != kv.dtype:
        raise RuntimeError("q/k/v must have the cache's element type")
    _check_cache(kv, written, B, Hkv, T, Dh, L)
    _check_tables(cos_table, sin_table, Dh)
    t_pos, y_pos, x_pos, ps = _pos_triplet(pos_ids, B, T, True)
    scale = 1.0 / math.sqrt(Dh) if scale is None else float(scale)
    lib = _capi.lib()
    with torch.cuda.device(dev):
        ws_bytes = int(lib.we_attn_workspace_bytes(B, H, Hkv, T, Dh, L, n_splits, q_tile))
    if ws_bytes and (workspace is None or workspace.numel() * workspace.element_size() < ws_bytes):
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    if q_rot is None:
        q_rot = torch.empty((B, H, T, Dh), dtype=q.dtype, device=dev)
    elif tuple(q_rot.shape) != (B, H, T, Dh) or q_rot.dtype != q.dtype or q_rot.device != dev or not q_rot.is_contiguous():
        raise RuntimeError("q_rot must be a contiguous [B, H, T, Dh] tensor of q's element type on q's device")
    if out is None:
        if token_major_out:
            out = torch.empty((B, T, H, Dh), dtype=q.dtype, device=dev).transpose(1, 2)
        else:
            out = torch.empty((B, H, T, Dh), dtype=q.dtype, device=dev)
    elif tuple(out.shape) != (B, H, T, Dh) or out.dtype != q.dtype or out.device != dev:
        raise RuntimeError("out must be [B, H, T, Dh] of q's element type on q's device")
    extras, _keep = _build_extras(q.dtype, B, H, Hkv, T, Dh, qk_norm_eps, v1, v_lamb, gate, gate_x, gate_w)
    code = _call(
        dev, lib.we_rope_kv_attn_fwd,
        q.data_ptr(), k.data_ptr(), v.data_ptr(), _bhtd_strides(q, "q"), _bhtd_strides(k, "k"), _bhtd_strides(v, "v"),
        q_rot.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(), cos_table.shape[0],
        t_pos.data_ptr(), y_pos.data_ptr(), x_pos.data_ptr(), ps, grid_h, grid_w, kv.data_ptr(), written.data_ptr(),
        out.data_ptr(), _bhtd_strides(out, "out"),
        workspace.data_ptr() if ws_bytes else None,
        workspace.numel() * workspace.element_size() if ws_bytes else 0,
        B, H, Hkv, T, Dh, L, dilation, int(bool(is_frozen)), scale, n_splits, q_tile, _dtype_code(kv),
        extras, _stream_ptr(dev))
    _capi.check(code, "we_rope_kv_attn_fwd")
    return out, q_rot


def qkv_rope_kv_attn(x: Tensor, w_qkv: Tensor, n_heads: int, n_kv_heads: int, pos_ids: Mapping[str, Tensor],
                     cos_table: Tensor, sin_table: Tensor, grid_h: int, grid_w: int, kv: Tensor, written: Tensor,
                     L: int, dilation: int, is_frozen: bool, scale: Optional[float] = None, n_splits: int = 0,
                     q_tile: int = 0, attend: bool = True, want_v: bool = False, qk_norm_eps: float = 0.0,
                     v1: Optional[Tensor] = None, v_lamb: Optional[Tensor] = None, gate: Optional[Tensor] = None,
                     gate_x: Optional[Tensor] = None, gate_w: Optional[Tensor] = None,
                     buffers: Optional[dict] = None):
    """The module's merged q/k/v projection, RoPE, the cache write and (``attend``) the attention
    over the ring in one library call (``we_qkv_rope_kv_attn_fwd`` / ``we_qkv_rope_kv_store``):
    ``src/patch_model.py:116-134`` from ``self.qkv_proj(x)`` to the ``flex_attention`` call.  The
    projection runs in the library's own kernel with the store's work as its epilogue, so q, k, v
    never exist as a ``[B, T, (H + 2 Hkv) Dh]`` tensor.

    ``x`` ``[B, T, d_model]`` (channel stride 1), ``w_qkv`` ``[(H + 2 Hkv) Dh, d_model]`` =
    ``qkv_proj.weight``.  Returns ``(out or None, q_rot, v or None)``: ``out`` ``[B, H, T, Dh]`` in
    token-major memory, ``q_rot`` the rotated (normalised) queries, ``v`` (``want_v``) the projected
    value rows ``[B, Hkv, T, Dh]`` before the value blend - what the first layer returns as ``v1``.
    Projection rows are fp32 sums rounded once to the element type in a fixed order that differs
    from a BLAS library's: they can differ from ``F.linear``'s in the last bit.
    ``buffers``: a dict the call keeps its ``q_rot`` / ``out`` / ``workspace`` tensors in and takes
    them from next time (shapes permitting), for callers that step the same layer again and again."""
    dev = _need_device(x, w_qkv, kv, written, cos_table, sin_table, pos_ids["t_pos"])
    if x.dim() != 3 or x.stride(2) != 1:
        raise RuntimeError("x must be [B, T, d_model] with contiguous channels")
    B, T, d_model = x.shape
    if kv.dim() != 5:
        raise RuntimeError("kv must be [2, B, Hkv, L+T, Dh]")
    Dh = kv.shape[4]
    H, Hkv = n_heads, n_kv_heads
    if w_qkv.dim() != 2 or tuple(w_qkv.shape) != ((H + 2 * Hkv) * Dh, d_model) or w_qkv.stride(1) != 1:
        raise RuntimeError("w_qkv must be [(H + 2 Hkv) * Dh, d_model] with contiguous rows")
    if x.dtype != kv.dtype or w_qkv.dtype != kv.dtype:
        raise RuntimeError("x and w_qkv must have the cache's element type")
    _check_cache(kv, written, B, Hkv, T, Dh, L)
    _check_tables(cos_table, sin_table, Dh)
    t_pos, y_pos, x_pos, ps = _pos_triplet(pos_ids, B, T, True)
    scale = 1.0 / math.sqrt(Dh) if scale is None else float(scale)
    lib = _capi.lib()
    def buf(name, make):
        if buffers is None:
            return make()
        key = (name, B, H, Hkv, T, Dh, x.dtype, dev)
        if key not in buffers:
            buffers[key] = make()
        return buffers[key]

    q_rot = buf("q_rot", lambda: torch.empty((B, H, T, Dh), dtype=x.dtype, device=dev))
    proj = _capi.QkvProj()
    proj.x, proj.w, proj.d_model = x.data_ptr(), w_qkv.data_ptr(), d_model
    proj.x_strides = (ctypes.c_int64 * 2)(x.stride(0), x.stride(1))
    proj.w_row_stride = w_qkv.stride(0)
    v_raw = None
    if want_v:   # token-major like the projection output the module would have sliced it from
        v_raw = torch.empty((B, T, Hkv, Dh), dtype=x.dtype, device=dev).transpose(1, 2)
        proj.v_out = v_raw.data_ptr()
        proj.v_out_strides = _bhtd_strides(v_raw, "v_out")
    extras, _keep = _build_extras(x.dtype, B, H, Hkv, T, Dh, qk_norm_eps, v1, v_lamb, gate, gate_x, gate_w)
    head = (ctypes.byref(proj), q_rot.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(), cos_table.shape[0],
            t_pos.data_ptr(), y_pos.data_ptr(), x_pos.data_ptr(), ps, grid_h, grid_w, kv.data_ptr(),
            written.data_ptr())
    if not attend:
        code = _call(dev, lib.we_qkv_rope_kv_store, *head, B, H, Hkv, T, Dh, L, dilation, int(bool(is_frozen)),
                     _dtype_code(kv), extras, _stream_ptr(dev))
        _capi.check(code, "we_qkv_rope_kv_store")
        return None, q_rot, v_raw
    with torch.cuda.device(dev):
        ws_bytes = int(lib.we_attn_workspace_bytes(B, H, Hkv, T, Dh, L, n_splits, q_tile))
    workspace = buf(("workspace", ws_bytes), lambda: torch.empty(ws_bytes, dtype=torch.uint8, device=dev)) if ws_bytes else None
    out = buf("out", lambda: torch.empty((B, T, H, Dh), dtype=x.dtype, device=dev).transpose(1, 2))
    code = _call(dev, lib.we_qkv_rope_kv_attn_fwd, *head, out.data_ptr(), _bhtd_strides(out, "out"),
                 workspace.data_ptr() if ws_bytes else None, ws_bytes,
                 B, H, Hkv, T, Dh, L, dilation, int(bool(is_frozen)), scale, n_splits, q_tile, _dtype_code(kv),
                 extras, _stream_ptr(dev))
    _capi.check(code, "we_qkv_rope_kv_attn_fwd")
    return out, q_rot, v_raw


# --------------------------------------------------------------------------------------------
# torch.library registration: opaque ops that survive torch.compile(fullgraph=True), the way the
# reference wraps its one native kernel (src/quantize.py:17-42).
# --------------------------------------------------------------------------------------------
@torch.library.custom_op("world_engine_amd::rope_kv_store", mutates_args=("kv", "written"))
def rope_kv_store_op(q: Tensor, k: Tensor, v: Tensor, t_pos: Tensor, y_pos: Tensor, x_pos: Tensor,
                     cos_table: Tensor, sin_table: Tensor, grid_h: int, grid_w: int,
                     kv: Tensor, written: Tensor, L: int, dilation: int, is_frozen: bool) -> Tensor:
    pos = {"t_pos": t_pos, "y_pos": y_pos, "x_pos": x_pos}
    return rope_kv_store(q, k, v, pos, cos_table, sin_table, grid_h, grid_w, kv, written, L,
                         dilation, is_frozen)


@rope_kv_store_op.register_fake
def _rope_kv_store_fake(q, k, v, t_pos, y_pos, x_pos, cos_table, sin_table, grid_h, grid_w,
                        kv, written, L, dilation, is_frozen):
    return q.new_empty(q.shape)


@torch.library.custom_op("world_engine_amd::attn_ring", mutates_args=())
def attn_ring_op(q: Tensor, kv: Tensor, written: Tensor, t_pos: Tensor, L: int, dilation: int,
                 scale: float) -> Tensor:
    return attn_ring(q, kv, written, t_pos, L, dilation, scale)


@attn_ring_op.register_fake
def _attn_ring_fake(q, kv, written, t_pos, L, dilation, scale):
    B, H, T, Dh = q.shape
    return q.new_empty((B, T, H, Dh)).transpose(1, 2)


@torch.library.custom_op("world_engine_amd::rope_kv_attn", mutates_args=("kv", "written"))
def rope_kv_attn_op(q: Tensor, k: Tensor, v: Tensor, t_pos: Tensor, y_pos: Tensor, x_pos: Tensor,
                    cos_table: Tensor, sin_table: Tensor, grid_h: int, grid_w: int,
                    kv: Tensor, written: Tensor, L: int, dilation: int, is_frozen: bool, scale: float,
                    qk_norm_eps: float = 0.0, v1: Optional[Tensor] = None, v_lamb: Optional[Tensor] = None,
                    gate: Optional[Tensor] = None, gate_x: Optional[Tensor] = None,
                    gate_w: Optional[Tensor] = None) -> Tensor:
    pos = {"t_pos": t_pos, "y_pos": y_pos, "x_pos": x_pos}
    return rope_kv_attn(q, k, v, pos, cos_table, sin_table, grid_h, grid_w, kv, written, L, dilation,
                        is_frozen, scale, qk_norm_eps=qk_norm_eps, v1=v1, v_lamb=v_lamb, gate=gate,
                        gate_x=gate_x, gate_w=gate_w)[0]


@rope_kv_attn_op.register_fake
def _rope_kv_attn_fake(q, k, v, t_pos, y_pos, x_pos, cos_table, sin_table, grid_h, grid_w, kv, written, L,
                       dilation, is_frozen, scale, qk_norm_eps=0.0, v1=None, v_lamb=None, gate=None, gate_x=None,
                       gate_w=None):
    B, H, T, Dh = q.shape
    return q.new_empty((B, T, H, Dh)).transpose(1, 2)


@torch.library.custom_op("world_engine_amd::qkv_rope_kv_attn", mutates_args=("kv", "written"))
def qkv_rope_kv_attn_op(x: Tensor, w_qkv: Tensor, n_heads: int, n_kv_heads: int, t_pos: Tensor, y_pos: Tensor,
                        x_pos: Tensor, cos_table: Tensor, sin_table: Tensor, grid_h: int, grid_w: int,
                        kv: Tensor, written: Tensor, L: int, dilation: int, is_frozen: bool, scale: float,
                        qk_norm_eps: float = 0.0, v1: Optional[Tensor] = None, v_lamb: Optional[Tensor] = None,
                        gate_x: Optional[Tensor] = None, gate_w: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Returns (attention output, projected v rows before the value blend)."""
    pos = {"t_pos": t_pos, "y_pos": y_pos, "x_pos": x_pos}
    out, _, v = qkv_rope_kv_attn(x, w_qkv, n_heads, n_kv_heads, pos, cos_table, sin_table, grid_h, grid_w, kv,
                                 written, L, dilation, is_frozen, scale, want_v=True, qk_norm_eps=qk_norm_eps,
                                 v1=v1, v_lamb=v_lamb, gate_x=gate_x, gate_w=gate_w)
    return out, v


@qkv_rope_kv_attn_op.register_fake
def _qkv_rope_kv_attn_fake(x, w_qkv, n_heads, n_kv_heads, t_pos, y_pos, x_pos, cos_table, sin_table, grid_h, grid_w,
                           kv, written, L, dilation, is_frozen, scale, qk_norm_eps=0.0, v1=None, v_lamb=None,
                           gate_x=None, gate_w=None):
    B, T = x.shape[:2]
    Dh = kv.shape[4]
    return (x.new_empty((B, T, n_heads, Dh)).transpose(1, 2), x.new_empty((B, T, n_kv_heads, Dh)).transpose(1, 2))
