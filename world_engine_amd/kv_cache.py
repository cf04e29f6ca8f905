"""Ring-buffer KV cache with the reference's class interface, backed by the HIP kernels.

Interface kept from ``src/model/kv_cache.py`` of world_engine: ``LayerKVCache(B, H, L, Dh, dtype,
tokens_per_frame, pinned_dilation)`` with buffers ``kv`` ``[2,B,H,L+T,Dh]``, ``written``
``[L+T]``, ``frame_offsets``, ``current_idx`` and methods ``reset`` / ``upsert`` (:64-154);
``StaticKVCache(config, batch_size, dtype)`` with ``layers``, ``reset``, ``set_frozen``,
``upsert(k, v, pos_ids, layer)`` (:157-193).  After every call ``kv`` and ``written`` hold
exactly the bits the reference's buffers would.

What differs by design: ``upsert`` returns a :class:`RingMask` (a view of the cache state) where
the reference returns a flex-attention ``BlockMask`` (:12-61, :144).  The only consumer of that
object in the reference is the attention call this package also replaces.  The cache writes are
one fused kernel launch; the slot is computed on the device from ``t_pos[0, 0]`` (:126-131), so
no host synchronisation happens outside the optional eager input checks (:112-124).
"""
from __future__ import annotations

from typing import Mapping, Optional, Tuple

import torch
from torch import Tensor, nn

from . import ops


class RingMask:
    """Which cache rows the current frame may attend to, described by reference to the cache
    state instead of a materialised mask: row ``j`` is visible iff it is in the tail or lies in
    a written ring slot other than the one the current frame replaces on a persisting frame
    (``src/model/kv_cache.py:141-143``)."""

    __slots__ = ("kv", "written", "t_pos", "L", "tpf", "dilation")

    def __init__(self, kv: Tensor, written: Tensor, t_pos: Tensor, L: int, tpf: int, dilation: int):
        self.kv, self.written, self.t_pos = kv, written, t_pos
        self.L, self.tpf, self.dilation = L, tpf, dilation

    def dense(self) -> Tensor:
        """The equivalent bool ``[L+T]`` mask (debugging aid; runs small device ops)."""
        n = self.L // self.tpf
        t = self.t_pos.reshape(-1)[0]
        slot = torch.div(t + (self.dilation - 1), self.dilation, rounding_mode="floor") % (n // self.dilation)
        hide = (t % self.dilation) == 0
        rows = torch.arange(self.L + self.tpf, device=self.written.device)
        in_slot = (rows >= slot * self.tpf) & (rows < (slot + 1) * self.tpf)
        return self.written & ~(in_slot & hide)


class LayerKVCache(nn.Module):
    """One layer's ring: ``L`` history rows in ``L/T`` frame slots plus a ``T``-row tail that
    always holds the current frame."""

    def __init__(self, B: int, H: int, L: int, Dh: int, dtype: torch.dtype, tokens_per_frame: int,
                 pinned_dilation: int = 1):
        super().__init__()
        T = tokens_per_frame
        if L % T != 0 or (L // T) % pinned_dilation != 0:
            raise AssertionError("L must be a multiple of tokens_per_frame and L/T of pinned_dilation")
        self.tpf = T
        self.L = L
        self.capacity = L + T
        self.pinned_dilation = pinned_dilation
        self.num_buckets = (L // T) // pinned_dilation
        self.check_inputs = True  # eager-mode sanity checks like the reference's (they sync)

        self.register_buffer("kv", torch.zeros(2, B, H, self.capacity, Dh, dtype=dtype), persistent=False)
        written = torch.zeros(self.capacity, dtype=torch.bool)
        written[L:] = True
        self.register_buffer("written", written, persistent=False)
        offsets = torch.arange(T, dtype=torch.long)
        self.register_buffer("frame_offsets", offsets, persistent=False)
        self.register_buffer("current_idx", offsets + L, persistent=False)
        # per-layer call buffers (rotated q, attention output, split-context workspace) of the eager
        # path, sized on first use and dropped whenever the module is moved or cast
        self._call_buffers = {}

    def _apply(self, fn, *args, **kwargs):
        self._call_buffers = {}
        return super()._apply(fn, *args, **kwargs)

    def _reusable(self, reuse: bool):
        """The buffer dict for an eager call, or None where every call must own its tensors (under
        torch.compile the opaque op allocates; under stream capture the graph owns what it captured)."""
        if not reuse or torch.compiler.is_compiling() or torch.cuda.is_current_stream_capturing():
            return None
        return self._call_buffers

    def reset(self) -> None:
        self.kv.zero_()
        self.written.zero_()
        self.written[self.L:].fill_(True)

    # -- input checks of the reference's eager path (src/model/kv_cache.py:112-124) ------------
    def _check(self, k: Tensor, pos_ids: Mapping[str, Tensor], rope=None) -> None:
        t_pos = pos_ids["t_pos"]
        ops._need_device(k, self.kv, t_pos)
        if k.size(2) != self.tpf:
            raise RuntimeError("KV cache expects exactly one frame per upsert")
        if tuple(t_pos.shape) != (k.size(0), self.tpf):
            raise RuntimeError("t_pos must be [B, T]")
        if self.check_inputs and not torch.compiler.is_compiling() and not torch.cuda.is_current_stream_capturing():
            if not bool((t_pos >= 0).all().item()):
                raise RuntimeError("t_pos must be non-negative during inference")
            if not bool((t_pos == t_pos[:, :1]).all().item()):
                raise RuntimeError("t_pos must be constant within frame")
            if rope is not None:   # the bounds check of the reference's RoPE (src/model/attn.py:25-30)
                rope.check_pos_ids(pos_ids)

    def _mask(self, pos_ids: Mapping[str, Tensor]) -> RingMask:
        return RingMask(self.kv, self.written, pos_ids["t_pos"], self.L, self.tpf, self.pinned_dilation)

    def upsert_kv(self, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], is_frozen: bool):
        """Store already-rotated ``k`` and ``v`` ``[B,H,T,Dh]`` (no stacking copy)."""
        self._check(k, pos_ids)
        ops.rope_kv_store(None, k, v, pos_ids, None, None, 1, 1, self.kv, self.written, self.L,
                          self.pinned_dilation, is_frozen)
        return self.kv[0], self.kv[1], self._mask(pos_ids)

    def upsert(self, kv: Tensor, pos_ids: Mapping[str, Tensor], is_frozen: bool):
        """Reference signature: ``kv`` is ``[2,B,H,T,Dh]`` (``src/model/kv_cache.py:104``)."""
        return self.upsert_kv(kv[0], kv[1], pos_ids, is_frozen)

    def rope_upsert(self, q: Tensor, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], rope,
                    is_frozen: bool):
        """Fused path used by the attention module: rotate q and k with ``rope``'s tables, store
        k/v, return ``(RoPE(q), k_all, v_all, mask)`` from a single kernel launch."""
        self._check(k, pos_ids, rope)
        q_rot = ops.rope_kv_store(q, k, v, pos_ids, rope.cos, rope.sin, rope.height, rope.width,
                                  self.kv, self.written, self.L, self.pinned_dilation, is_frozen)
        return q_rot, self.kv[0], self.kv[1], self._mask(pos_ids)

    def rope_upsert_attend(self, q: Tensor, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], rope,
                           is_frozen: bool, scale: Optional[float] = None, qk_norm_eps: float = 0.0,
                           v1: Optional[Tensor] = None, v_lamb: Optional[Tensor] = None,
                           gate: Optional[Tensor] = None, gate_x: Optional[Tensor] = None,
                           gate_w: Optional[Tensor] = None, reuse_buffers: bool = False) -> Tensor:
        """``rope_upsert`` followed by the attention over the ring, as one library call
        (``src/model/attn.py:110-116`` of the reference from RoPE to ``flex_attention``).  Under
        ``torch.compile`` the registered opaque op is used instead of the eager wrapper.

        ``reuse_buffers``: the rotated q, the output and the split-context workspace live in
        per-layer tensors that the next eager call of this layer uses again, so a serving loop
        allocates nothing after its first frame.  The returned tensor is then only valid until
        that next call (the attention module consumes it at once); off by default."""
        if torch.compiler.is_compiling():
            s = float(scale) if scale is not None else float(q.shape[-1]) ** -0.5
            return torch.ops.world_engine_amd.rope_kv_attn(
                q, k, v, pos_ids["t_pos"], pos_ids["y_pos"], pos_ids["x_pos"], rope.cos, rope.sin, rope.height,
                rope.width, self.kv, self.written, self.L, self.pinned_dilation, bool(is_frozen), s,
                float(qk_norm_eps), v1, v_lamb, gate, gate_x, gate_w)
        self._check(k, pos_ids, rope)
        kept = self._reusable(reuse_buffers)
        bufs = {}
        if kept is not None:
            B, H, T, Dh = q.shape
            key = ("attn", B, H, k.shape[1], T, Dh, q.dtype, q.device)
            if key not in kept:
                ws_bytes = ops.attn_workspace_bytes(B, H, k.shape[1], T, Dh, self.L)
                kept[key] = dict(q_rot=torch.empty((B, H, T, Dh), dtype=q.dtype, device=q.device),
                                 out=torch.empty((B, T, H, Dh), dtype=q.dtype, device=q.device).transpose(1, 2),
                                 workspace=torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None)
            bufs = kept[key]
        return ops.rope_kv_attn(q, k, v, pos_ids, rope.cos, rope.sin, rope.height, rope.width, self.kv,
                                self.written, self.L, self.pinned_dilation, is_frozen, scale,
                                qk_norm_eps=qk_norm_eps, v1=v1, v_lamb=v_lamb, gate=gate, gate_x=gate_x,
                                gate_w=gate_w, **bufs)[0]

    def qkv_rope_upsert_attend(self, x: Tensor, w_qkv: Tensor, n_heads: int, pos_ids: Mapping[str, Tensor], rope,
                               is_frozen: bool, scale: Optional[float] = None, want_v: bool = False,
                               qk_norm_eps: float = 0.0, v1: Optional[Tensor] = None,
                               v_lamb: Optional[Tensor] = None, gate_x: Optional[Tensor] = None,
                               gate_w: Optional[Tensor] = None, reuse_buffers: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
        """``rope_upsert_attend`` with the module's merged q/k/v projection in front, as one
        library call (``src/patch_model.py:116-134`` from ``self.qkv_proj(x)`` to the attention
        output).  Returns ``(y, v)``: ``v`` (``want_v``) is the projected value rows before the
        value blend, what the first layer hands on as ``v1``."""
        n_kv = self.kv.shape[2]
        if torch.compiler.is_compiling():
            s = float(scale) if scale is not None else float(self.kv.shape[4]) ** -0.5
            y, v = torch.ops.world_engine_amd.qkv_rope_kv_attn(
                x, w_qkv, n_heads, n_kv, pos_ids["t_pos"], pos_ids["y_pos"], pos_ids["x_pos"], rope.cos, rope.sin,
                rope.height, rope.width, self.kv, self.written, self.L, self.pinned_dilation, bool(is_frozen), s,
                float(qk_norm_eps), v1, v_lamb, gate_x, gate_w)
            return y, (v if want_v else None)
        self._check(x.unsqueeze(1), pos_ids, rope)
        y, _, v = ops.qkv_rope_kv_attn(x, w_qkv, n_heads, n_kv, pos_ids, rope.cos, rope.sin, rope.height, rope.width,
                                       self.kv, self.written, self.L, self.pinned_dilation, is_frozen, scale,
                                       want_v=want_v, qk_norm_eps=qk_norm_eps, v1=v1, v_lamb=v_lamb, gate_x=gate_x,
                                       gate_w=gate_w, buffers=self._reusable(reuse_buffers))
        return y, v


class StaticKVCache(nn.Module):
    """Per-layer rings with local/global windows chosen as in ``src/model/kv_cache.py:157-181``."""

    def __init__(self, config, batch_size: int, dtype: torch.dtype):
        super().__init__()
        self.tpf = config.tokens_per_frame
        period = config.global_attn_period
        off = getattr(config, "global_attn_offset", 0) % period
        n_kv = getattr(config, "n_kv_heads", config.n_heads)
        d_head = config.d_model // config.n_heads
        layers = []
        for idx in range(config.n_layers):
            is_global = (idx - off) % period == 0
            frames = config.global_window if is_global else config.local_window
            dilation = config.global_pinned_dilation if is_global else 1
            layers.append(LayerKVCache(batch_size, n_kv, frames * self.tpf, d_head, dtype, self.tpf, dilation))
        self.layers = nn.ModuleList(layers)
        self._is_frozen = True

    def reset(self) -> None:
        for layer in self.layers:
            layer.reset()
        self._is_frozen = True

    def set_frozen(self, is_frozen: bool) -> None:
        self._is_frozen = is_frozen

    def upsert(self, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], layer: int):
        return self.layers[layer].upsert_kv(k, v, pos_ids, self._is_frozen)

    def rope_upsert(self, q: Tensor, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], rope, layer: int):
        return self.layers[layer].rope_upsert(q, k, v, pos_ids, rope, self._is_frozen)

    def rope_upsert_attend(self, q: Tensor, k: Tensor, v: Tensor, pos_ids: Mapping[str, Tensor], rope, layer: int,
                           scale: Optional[float] = None, **extras) -> Tensor:
        return self.layers[layer].rope_upsert_attend(q, k, v, pos_ids, rope, self._is_frozen, scale, **extras)

    def qkv_rope_upsert_attend(self, x: Tensor, w_qkv: Tensor, n_heads: int, pos_ids: Mapping[str, Tensor], rope,
                               layer: int, scale: Optional[float] = None, **extras):
        return self.layers[layer].qkv_rope_upsert_attend(x, w_qkv, n_heads, pos_ids, rope, self._is_frozen, scale,
                                                         **extras)
