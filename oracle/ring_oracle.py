"""CPU oracle for the frame-causal ring-buffer attention path.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU, the algorithm that world_engine runs once per DiT layer per
model forward: rotary embedding of q/k, the ring-buffer K/V write, the visibility mask and the
masked softmax attention.  It exists so that the HIP kernels can be checked against it.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
it; nothing under ``world_engine_amd/`` does, and the product path never falls back to it.

Reference sources followed (paths relative to the world_engine checkout):

* ``src/model/kv_cache.py:70-102``  buffers, ``written`` initial state, ``reset``
* ``src/model/kv_cache.py:104-154`` ``LayerKVCache.upsert`` (slot arithmetic, tail write, mask,
  unfrozen ring write)
* ``src/model/kv_cache.py:12-61``   meaning of the block mask: key j is visible iff mask[j]
* ``src/model/kv_cache.py:157-193`` per-layer window/dilation choice, frozen flag, k/v stacking
* ``src/model/attn.py:22-40``       table-driven RoPE (fp32 math, de-interleaved output)
* ``src/model/attn.py:99-122`` / ``src/patch_model.py:116-141``  order of operations, incl. the
  module's element-wise steps around the path: value-residual lerp (``attn.py:105-107``), weightless
  QK RMS norm (``attn.py:109``, ``src/model/nn.py:55-56``), sigmoid head gate (``attn.py:117-119``)
* ``src/patch_model.py:102-122``    merged q/k/v projection in front of the path (weight rows q | k | v,
  split, ``[B,T,H,Dh] -> [B,H,T,Dh]`` views)
* ``src/world_engine.py:139-152``   frozen denoise passes followed by one unfrozen cache pass
* ``torch/_higher_order_ops/flex_attention.py:159-267`` (torch 2.10, third-party) dtype flow
  of eager ``flex_attention``: fp32 scores, ``* scale``, ``where(mask, s, -inf)``, softmax,
  ``P.to(q.dtype) @ V``; default scale ``1/sqrt(Dh)``
  (``torch/nn/attention/flex_attention.py:1543-1544``).

Pinning status (see tests/test_oracle_pins.py; the reference ships no tests or golden vectors):

* ``slot_and_write_step``            pinned: brute-force frame-retention model + closed forms
* ``OracleLayerKVCache`` / ``OracleStaticKVCache``  pinned: independent dict-of-frames model,
  invariants (tail == latest call, frozen leaves ring untouched, unwritten rows zero)
* ``visible_mask``                   pinned: N_vis closed form, retention model
* ``rope_apply`` / ``rope_angles``   pinned: complex-rotation closed form in fp64, zero-angle
  case, norm preservation, relative-position property
* ``attention_reference_path`` / ``attention_fp32``  pinned: torch's own eager
  ``flex_attention`` with a ``BlockMask.from_kv_blocks`` mask (library routine), SDPA on the
  gathered visible keys, key-permutation invariance, fp64 brute force
* ``rms_norm`` / ``value_lerp`` / ``gate_output``  pinned: torch's own ``F.rms_norm`` / ``torch.lerp``
  (library routines, the calls the reference makes) bit for bit on the CPU, plus closed cases
  (unit RMS, power-of-two scale invariance, lerp end points, gate 0 / 1)
* ``qkv_project``                    pinned: exact integer arithmetic on dyadic inputs (every
  summation order gives the same fp32 sum there), fp64 sums rounded once on random inputs
  (within one unit in the last place), torch's own ``F.linear`` + the reference's
  split / reshape / transpose for the layout
* ``rope_table_1d``                  synthetic table of the benchmark configurations (not a
  reference function); checked against direct fp64 evaluation
* ``ortho_rope_table``               parity unpinned: depends on ``rotary_embedding_torch``
  internals (``src/model/attn.py:52-67``) that are not available offline; off the hot path
  because every kernel consumes tables.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# slot arithmetic                                     src/model/kv_cache.py:126-131,140
# --------------------------------------------------------------------------------------
def slot_and_write_step(frame_t: int, n_slots: int, dilation: int) -> Tuple[int, bool]:
    """Ring slot a frame maps to and whether the frame is persisted.

    ``bucket = ceil(frame_t / dilation)``, ``slot = bucket mod (n_slots / dilation)``;
    a frame is persisted (``write_step``) only when ``frame_t`` is a multiple of ``dilation``.
    Python's ``//`` and ``%`` are floor operations like torch's on int64 tensors.
    """
    num_buckets = n_slots // dilation
    bucket = (frame_t + (dilation - 1)) // dilation
    return bucket % num_buckets, (frame_t % dilation) == 0


# --------------------------------------------------------------------------------------
# RoPE                                                      src/model/attn.py:22-40
# --------------------------------------------------------------------------------------
def rope_table_1d(n_rows: int, d_head: int, base: float = 10000.0) -> Tuple[Tensor, Tensor]:
    """cos/sin tables ``[n_rows, d_head/2]`` fp32 for a 1-D rotary embedding over the absolute
    token position: ``angle[p, i] = p * base**(-2 i / d_head)``, evaluated in fp64."""
    half = d_head // 2
    inv = torch.pow(torch.tensor(base, dtype=torch.float64),
                    -2.0 * torch.arange(half, dtype=torch.float64) / d_head)
    ang = torch.arange(n_rows, dtype=torch.float64)[:, None] * inv[None, :]
    return ang.cos().float().contiguous(), ang.sin().float().contiguous()


def ortho_rope_table(height: int, width: int, n_frames: int, d_head: int) -> Tuple[Tensor, Tensor]:
    """Three-axis table in the spirit of ``OrthoRoPE.get_freqs`` (src/model/attn.py:52-67):
    columns ``[X | Y | T]`` with ``d_head/8 + d_head/8 + d_head/4`` angles, rows ordered (t h w).

    PARITY UNPINNED: the per-axis spectra come from ``rotary_embedding_torch`` whose source is
    not in this environment.  The formulas used here are the package's documented ones
    ('pixel': ``linspace(1, max_freq/2, dim/2) * pi``; 'lang': ``10000**(-2i/dim)``; every
    frequency repeated twice), recalled, not verified.
    """
    def repeat2(f):
        return f.repeat_interleave(2, dim=-1)

    max_freq = min(height, width) * 0.8
    dim_xy, dim_t = d_head // 8, d_head // 4
    pix = torch.linspace(1.0, max_freq / 2, dim_xy // 2) * math.pi
    lang = 1.0 / (10000.0 ** (torch.arange(0, dim_t, 2)[: dim_t // 2].float() / dim_t))
    xs = torch.linspace(-1 + 1 / width, 1 - 1 / width, width)
    ys = torch.linspace(-1 + 1 / height, 1 - 1 / height, height)
    fx = repeat2(xs[:, None] * pix[None, :])[None, :, :].expand(height, width, -1)
    fy = repeat2(ys[:, None] * pix[None, :])[:, None, :].expand(height, width, -1)
    ft = repeat2(torch.arange(n_frames).float()[:, None] * lang[None, :])
    hw = height * width
    table = torch.cat([
        fx.reshape(1, hw, -1).expand(n_frames, hw, -1),
        fy.reshape(1, hw, -1).expand(n_frames, hw, -1),
        ft[:, None, :].expand(n_frames, hw, -1),
    ], dim=-1).reshape(n_frames * hw, -1)
    return table.cos().contiguous(), table.sin().contiguous()


def rope_angles(pos_ids: Dict[str, Tensor], cos_table: Tensor, sin_table: Tensor,
                height: int, width: int) -> Tuple[Tensor, Tensor]:
    """Gather table rows by ``flat = t*(H*W) + y*W + x`` (src/model/attn.py:22-31).
    Returns cos, sin of shape ``[B, 1, T, Dh/2]``."""
    t, y, x = pos_ids["t_pos"], pos_ids["y_pos"], pos_ids["x_pos"]
    flat = t * (height * width) + y * width + x
    idx = flat.reshape(-1).long()
    cos = cos_table.index_select(0, idx).view(*flat.shape, -1)
    sin = sin_table.index_select(0, idx).view(*flat.shape, -1)
    return cos[:, None], sin[:, None]


def rope_apply(x: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """Rotate even/odd lane pairs in fp32 and return the de-interleaved halves
    ``[y0 | y1]`` in ``x``'s dtype (src/model/attn.py:33-40).  Each product and the
    sum/difference is a separately rounded fp32 operation, as in eager torch."""
    xf = x.float()
    x0 = xf[..., 0::2]
    x1 = xf[..., 1::2]
    y0 = x0 * cos - x1 * sin
    y1 = x1 * cos + x0 * sin
    return torch.cat((y0, y1), dim=-1).to(x.dtype)


# --------------------------------------------------------------------------------------
# ring-buffer KV cache                               src/model/kv_cache.py:64-193
# --------------------------------------------------------------------------------------
class OracleLayerKVCache:
    """CPU restatement of one layer's ring buffer (src/model/kv_cache.py:64-154).

    ``kv``       ``[2, B, Hkv, L + T, Dh]``: rows ``[0, L)`` are ``L/T`` frame slots, rows
                 ``[L, L+T)`` (the tail) always hold the current frame.
    ``written``  ``[L + T]`` bool, tail always True.
    """

    def __init__(self, B: int, H: int, L: int, Dh: int, dtype: torch.dtype,
                 tokens_per_frame: int, pinned_dilation: int = 1):
        T = tokens_per_frame
        if L % T != 0 or (L // T) % pinned_dilation != 0:
            raise ValueError("ring length must hold a whole number of frames and dilation groups")
        self.tpf, self.L, self.capacity = T, L, L + T
        self.pinned_dilation = pinned_dilation
        self.n_slots = L // T
        self.num_buckets = self.n_slots // pinned_dilation
        self.kv = torch.zeros(2, B, H, self.capacity, Dh, dtype=dtype)
        self.written = torch.zeros(self.capacity, dtype=torch.bool)
        self.written[L:] = True

    def reset(self) -> None:                       # src/model/kv_cache.py:99-102
        self.kv.zero_()
        self.written.zero_()
        self.written[self.L:] = True

    def upsert(self, kv: Tensor, pos_ids: Dict[str, Tensor], is_frozen: bool):
        """``kv``: ``[2, B, Hkv, T, Dh]`` of one frame.  Returns full-capacity ``k``, ``v``
        views and the bool visibility mask ``[L + T]`` the attention must apply."""
        T, L = self.tpf, self.L
        t_pos = pos_ids["t_pos"]
        if kv.shape[3] != T:
            raise RuntimeError("KV cache expects exactly one frame per upsert")
        if tuple(t_pos.shape) != (kv.shape[1], T):
            raise RuntimeError("t_pos must be [B, T]")
        if bool((t_pos < 0).any()):
            raise RuntimeError("t_pos must be non-negative during inference")
        if not bool((t_pos == t_pos[:, :1]).all()):
            raise RuntimeError("t_pos must be constant within frame")

        frame_t = int(t_pos[0, 0])
        slot, write_step = slot_and_write_step(frame_t, self.n_slots, self.pinned_dilation)
        lo = slot * T

        # the tail always receives the current frame              kv_cache.py:138
        self.kv[:, :, :, L:L + T] = kv

        # visibility: everything written so far, minus the slot this frame is about to
        # replace when it is a persisting frame                   kv_cache.py:140-143
        mask = self.written.clone()
        if write_step:
            mask[lo:lo + T] = False

        # unfrozen: persist into the ring (or, off-dilation, re-write the tail) and mark it
        if not is_frozen:                                       # kv_cache.py:147-151
            dst = slice(lo, lo + T) if write_step else slice(L, L + T)
            self.kv[:, :, :, dst] = kv
            self.written[dst] = True

        return self.kv[0], self.kv[1], mask


class OracleStaticKVCache:
    """One ring per layer with local/global windows (src/model/kv_cache.py:157-193).

    ``config`` needs ``tokens_per_frame, local_window, global_window, global_attn_period,
    global_pinned_dilation, n_layers, n_heads, d_model`` and optionally ``n_kv_heads``,
    ``global_attn_offset``.
    """

    def __init__(self, config, batch_size: int, dtype: torch.dtype):
        self.tpf = config.tokens_per_frame
        period = config.global_attn_period
        off = getattr(config, "global_attn_offset", 0) % period
        hkv = getattr(config, "n_kv_heads", config.n_heads)
        dh = config.d_model // config.n_heads
        self.layers: List[OracleLayerKVCache] = []
        for i in range(config.n_layers):
            is_global = (i - off) % period == 0
            window = config.global_window if is_global else config.local_window
            dil = config.global_pinned_dilation if is_global else 1
            self.layers.append(OracleLayerKVCache(batch_size, hkv, window * self.tpf, dh, dtype,
                                                  self.tpf, dil))
        self._is_frozen = True

    def reset(self) -> None:
        for layer in self.layers:
            layer.reset()
        self._is_frozen = True

    def set_frozen(self, is_frozen: bool) -> None:
        self._is_frozen = is_frozen

    def upsert(self, k: Tensor, v: Tensor, pos_ids: Dict[str, Tensor], layer: int):
        return self.layers[layer].upsert(torch.stack([k, v], dim=0), pos_ids, self._is_frozen)


def visible_mask(written: Tensor, frame_t: int, T: int, n_slots: int, dilation: int) -> Tensor:
    """Mask the attention applies given the cache's ``written`` state *before or after* the
    call's own ring write (the slot it touches is hidden either way on a persisting frame)."""
    slot, write_step = slot_and_write_step(frame_t, n_slots, dilation)
    mask = written.clone()
    if write_step:
        mask[slot * T:(slot + 1) * T] = False
    mask[n_slots * T:] = True
    return mask


# --------------------------------------------------------------------------------------
# masked attention                  torch/_higher_order_ops/flex_attention.py:159-267
# --------------------------------------------------------------------------------------
def _expand_gqa(q: Tensor, k: Tensor, v: Tensor) -> Tuple[Tensor, Tensor]:
    g = q.shape[1] // k.shape[1]
    if g > 1:
        k = k.repeat_interleave(g, dim=1)
        v = v.repeat_interleave(g, dim=1)
    return k, v


def attention_reference_path(q: Tensor, k_all: Tensor, v_all: Tensor, mask: Tensor,
                             scale: Optional[float] = None) -> Tensor:
    """Dense restatement of what the reference's attention call computes, with its dtype flow:
    fp32 scores, scale, ``-inf`` on hidden keys, softmax, probabilities cast to the input dtype
    before ``P @ V``.  ``q`` ``[B,H,T,Dh]``; ``k_all``/``v_all`` ``[B,Hkv,cap,Dh]``; ``mask``
    ``[cap]`` bool (the same for every batch element, head and query)."""
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    k_all, v_all = _expand_gqa(q, k_all, v_all)
    wp = torch.float64 if q.dtype == torch.float64 else torch.float32
    s = (q.to(wp) @ k_all.to(wp).transpose(-2, -1)) * scale
    s = torch.where(mask.view(1, 1, 1, -1), s, torch.tensor(float("-inf"), dtype=wp))
    p = torch.softmax(s, dim=-1)
    return p.to(q.dtype) @ v_all


def attention_fp32(q: Tensor, k_all: Tensor, v_all: Tensor, mask: Tensor,
                   scale: Optional[float] = None, dtype: torch.dtype = torch.float32) -> Tensor:
    """The numerical yardstick: the same masked softmax attention computed entirely in
    ``dtype`` (fp32, or fp64 for brute-force checks) on the gathered visible keys."""
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    k_all, v_all = _expand_gqa(q, k_all, v_all)
    idx = mask.nonzero().flatten()
    kk = k_all.index_select(2, idx).to(dtype)
    vv = v_all.index_select(2, idx).to(dtype)
    s = (q.to(dtype) @ kk.transpose(-2, -1)) * scale
    return torch.softmax(s, dim=-1) @ vv


# --------------------------------------------------------------------------------------
# the module's element-wise steps around the path
#                     src/model/attn.py:105-109,117-119, src/model/nn.py:55-56
# --------------------------------------------------------------------------------------
def rms_norm(x: Tensor, eps: Optional[float] = None) -> Tensor:
    """Weightless RMS norm over the last dimension, ``F.rms_norm(x, (x.size(-1),))``
    (src/model/nn.py:55-56): ``x / sqrt(mean(x^2) + eps)`` evaluated in fp32 for low-precision
    inputs and rounded to ``x``'s dtype.  torch's default epsilon is the machine epsilon of the
    arithmetic type, i.e. fp32's for bf16 / f16 / fp32 inputs."""
    wp = torch.float64 if x.dtype == torch.float64 else torch.float32
    if eps is None:
        eps = torch.finfo(wp).eps
    xf = x.to(wp)
    ms = xf.pow(2).mean(dim=-1, keepdim=True)
    return (xf * torch.rsqrt(ms + eps)).to(x.dtype)


def value_lerp(v: Tensor, v1: Tensor, weight: Tensor) -> Tensor:
    """Value residual ``torch.lerp(v, v1, weight)`` (src/model/attn.py:105-107): fp32 arithmetic for
    low-precision tensors, ``v + w (v1 - v)`` below ``w = 0.5`` and ``v1 - (v1 - v)(1 - w)`` from
    there on (the formula torch switches between to stay monotonic), rounded to ``v``'s dtype."""
    wp = torch.float64 if v.dtype == torch.float64 else torch.float32
    a, b = v.to(wp), v1.to(wp)
    w = weight.to(wp)
    d = b - a
    out = torch.where(w.abs() < 0.5, a + w * d, b - d * (1 - w))
    return out.to(v.dtype)


def gate_output(y: Tensor, gates: Tensor) -> Tensor:
    """Head gate (src/model/attn.py:117-119): ``y * gates.permute(0, 2, 1).unsqueeze(-1)`` with
    ``y`` ``[B,H,T,Dh]`` and ``gates`` ``[B,T,H]`` (sigmoid already applied), a product of two
    tensors of the element type, rounded to it."""
    return y * gates.permute(0, 2, 1).unsqueeze(-1)


# --------------------------------------------------------------------------------------
# the merged projection in front of the path              src/patch_model.py:102-122
# --------------------------------------------------------------------------------------
def qkv_project(x: Tensor, w_qkv: Tensor, n_heads: int, n_kv_heads: int) -> Tuple[Tensor, Tensor, Tensor]:
    """``q, k, v = self.qkv_proj(x).split((H Dh, Hkv Dh, Hkv Dh), dim=-1)`` followed by the
    ``[B,T,h,Dh] -> [B,h,T,Dh]`` views (src/patch_model.py:116-122; the weight's rows are the q,
    k and v projections' rows one after the other, :102-114).  A bias-free linear layer of the
    element type: every output is the fp32 sum of the products, rounded once to ``x``'s dtype.
    The order of the fp32 additions is the BLAS library's business in the reference; here it is
    torch's CPU matmul on fp32 copies."""
    B, T, _ = x.shape
    d_head = w_qkv.shape[0] // (n_heads + 2 * n_kv_heads)
    wp = torch.float64 if x.dtype == torch.float64 else torch.float32
    y = (x.to(wp) @ w_qkv.to(wp).t()).to(x.dtype)
    q, k, v = y.split((n_heads * d_head, n_kv_heads * d_head, n_kv_heads * d_head), dim=-1)
    return (q.reshape(B, T, n_heads, d_head).transpose(1, 2), k.reshape(B, T, n_kv_heads, d_head).transpose(1, 2),
            v.reshape(B, T, n_kv_heads, d_head).transpose(1, 2))


# --------------------------------------------------------------------------------------
# one attention-layer step in the reference's order of operations
#                                  src/model/attn.py:105-119, src/patch_model.py:124-137
# --------------------------------------------------------------------------------------
def layer_step(cache: OracleStaticKVCache, layer: int, q: Tensor, k: Tensor, v: Tensor,
               pos_ids: Dict[str, Tensor], cos_table: Tensor, sin_table: Tensor,
               height: int, width: int, scale: Optional[float] = None,
               reference_dtype_flow: bool = True, qk_norm: bool = False,
               v1: Optional[Tensor] = None, v_lamb: Optional[Tensor] = None,
               gates: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """[lerp(v, v1, v_lamb)] -> [rms_norm(q), rms_norm(k)] -> RoPE(q), RoPE(k) -> cache upsert ->
    masked attention -> [gate].  The bracketed steps are the module's optional ones and are off
    by default.  Returns ``(out, q_rot)``; with ``reference_dtype_flow=False`` the attention (and
    the gate multiply) are evaluated in fp32 on the element-type inputs."""
    if v1 is not None:
        v = value_lerp(v, v1.view_as(v), v_lamb)
    if qk_norm:
        q, k = rms_norm(q), rms_norm(k)
    cos, sin = rope_angles(pos_ids, cos_table, sin_table, height, width)
    q_rot = rope_apply(q, cos, sin)
    k_rot = rope_apply(k, cos, sin)
    k_all, v_all, mask = cache.upsert(k_rot, v, pos_ids, layer)
    fn = attention_reference_path if reference_dtype_flow else attention_fp32
    out = fn(q_rot, k_all, v_all, mask, scale)
    if gates is not None:
        out = gate_output(out, gates if reference_dtype_flow else gates.float())
    return out, q_rot


# --------------------------------------------------------------------------------------
# synthetic inputs shared by tests, smoke and bench
# --------------------------------------------------------------------------------------
def synth_qkv(cfg_id: int, step: int, substep: int, B: int, H: int, Hkv: int, T: int, Dh: int,
              dtype: torch.dtype, outlier: bool = False) -> Tuple[Tensor, Tensor, Tensor]:
    """q, k, v ~ N(0,1) drawn in fp32 from ``seed = 10000*cfg + 100*step + substep`` on the CPU
    generator and cast to ``dtype``.  With ``outlier`` one K channel chosen from the seed is
    multiplied by 8 (the softmax-stability case)."""
    g = torch.Generator(device="cpu").manual_seed(10_000 * cfg_id + 100 * step + substep)
    q = torch.randn(B, H, T, Dh, generator=g, dtype=torch.float32)
    k = torch.randn(B, Hkv, T, Dh, generator=g, dtype=torch.float32)
    v = torch.randn(B, Hkv, T, Dh, generator=g, dtype=torch.float32)
    if outlier:
        ch = int(torch.randint(0, Dh, (1,), generator=g))
        k[..., ch] *= 8.0
    return q.to(dtype), k.to(dtype), v.to(dtype)


def synth_dyadic_linear(seed: int, B: int, T: int, d_model: int, feats: int,
                        dtype: torch.dtype) -> Tuple[Tensor, Tensor]:
    """x ``[B,T,d_model]`` and w ``[feats,d_model]`` whose values are multiples of 1/8 in [-1, 1]:
    every product is a multiple of 1/64 and every partial sum of up to 2^17 of them is an exact
    fp32 number, so a linear layer's fp32 sums do not depend on the order of the additions."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = (torch.randint(-8, 9, (B, T, d_model), generator=g).float() / 8).to(dtype)
    w = (torch.randint(-8, 9, (feats, d_model), generator=g).float() / 8).to(dtype)
    return x, w


def synth_pos_ids(frame_t: int, B: int, T: int, width: int) -> Dict[str, Tensor]:
    """Position ids of one frame (src/model/world_model.py:245-249,280-284): ``t_pos`` constant,
    ``y = idx // W``, ``x = idx % W``; int64 ``[B, T]``."""
    idx = torch.arange(T, dtype=torch.long)
    return {
        "t_pos": torch.full((B, T), frame_t, dtype=torch.long),
        "y_pos": (idx // width)[None].expand(B, T).contiguous(),
        "x_pos": (idx % width)[None].expand(B, T).contiguous(),
    }
