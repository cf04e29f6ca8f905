"""Self-attention module with the reference's ``forward(x, pos_ids, v1, kv_cache)`` contract.

``RingAttn`` takes the place of ``Attn`` / ``MergedQKVAttn`` (``src/model/attn.py:70-122``,
``src/patch_model.py:92-141``): same parameters and state-dict keys, same call signature, same
order of operations.  The part between the q/k/v projection and the output projection - RoPE,
cache update, masked attention - runs as two HIP kernel launches (three with context splits)
instead of the reference's eager/compiled op sequence.  Projections stay ordinary torch ops.  The
weightless RMS norm, the value-residual lerp and the head gate are torch ops by default and move
into the two kernels with ``fuse_elementwise=True`` (results then agree to 1 ulp instead of bit
for bit).
"""
from __future__ import annotations

import math
from typing import Mapping, Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops
from .kv_cache import RingMask


class RoPE(nn.Module):
    """Table-driven rotary embedding (``src/model/attn.py:12-40``).  ``cos``/``sin`` are fp32
    ``[n_frames*height*width, Dh/2]`` buffers that ignore dtype casts of the parent model (the
    reference keeps them fp32 through ``NoCastModule``); the row of token ``(t, y, x)`` is
    ``t*height*width + y*width + x``.

    As in the reference (``src/model/nn.py:10-24``), a dtype cast of a parent module leaves the
    buffers fp32 but their *values* pass through the requested type: after ``model.to(bfloat16)``
    the tables hold cos / sin rounded to bf16 precision.  This is what the reference's own tables
    hold once ``WorldEngine`` has cast the model (``src/world_engine.py:56``), so it is kept; code
    that wants full-precision angles must build the module after the cast, or move it with
    ``.to(device)`` only."""

    def __init__(self, cos: Tensor, sin: Tensor, height: int, width: int):
        super().__init__()
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape:
            raise AssertionError("RoPE tables must be fp32 and of equal shape")
        self.height, self.width = height, width
        self.register_buffer("cos", cos.contiguous(), persistent=False)
        self.register_buffer("sin", sin.contiguous(), persistent=False)

    def _apply(self, fn, *args, **kwargs):
        def keep_dtype(t):
            out = fn(t)
            return out if out.dtype == t.dtype else out.to(dtype=t.dtype)
        return super()._apply(keep_dtype, *args, **kwargs)

    @classmethod
    def one_dimensional(cls, n_rows: int, d_head: int, height: int, width: int, base: float = 10000.0):
        """1-D rotary table over the absolute token position: ``angle[p,i] = p * base**(-2i/Dh)``
        (computed in fp64, stored fp32)."""
        inv = torch.pow(torch.tensor(base, dtype=torch.float64),
                        -2.0 * torch.arange(d_head // 2, dtype=torch.float64) / d_head)
        ang = torch.arange(n_rows, dtype=torch.float64)[:, None] * inv[None, :]
        return cls(ang.cos().float(), ang.sin().float(), height, width)

    @classmethod
    def three_axis(cls, n_frames: int, d_head: int, height: int, width: int):
        """Table of the reference's ``OrthoRoPE`` (``src/model/attn.py:46-67``): angle columns
        ``[X | Y | T]`` of ``Dh/8 + Dh/8 + Dh/4``, rows ordered ``(t, y, x)``.  X and Y use a linear
        "pixel" spectrum over positions ``linspace(-1 + 1/n, 1 - 1/n, n)`` with top frequency
        ``0.8 * min(height, width)``; T uses the geometric "lang" spectrum over the frame index.

        The per-axis spectra are those of ``rotary_embedding_torch`` (>= 0.8.8 per the reference's
        ``pyproject.toml:14``), a package that is not available offline: 'pixel' is
        ``linspace(1, max_freq/2, dim/2) * pi``, 'lang' is ``10000**(-2i/dim)``, each frequency
        taken twice in a row.  These formulas are restated from the package's published source and
        have not been checked against it here; the kernels consume any table, so only positions of
        real checkpoints depend on this builder."""
        if d_head % 16 != 0:
            raise AssertionError("d_head must be a multiple of 16 for the three-axis table")
        dim_xy, dim_t = d_head // 8, d_head // 4
        pixel = torch.linspace(1.0, min(height, width) * 0.8 / 2, dim_xy // 2) * math.pi
        lang = 1.0 / (10000.0 ** (torch.arange(0, dim_t, 2)[: dim_t // 2].float() / dim_t))
        x_pos = torch.linspace(-1 + 1 / width, 1 - 1 / width, width)
        y_pos = torch.linspace(-1 + 1 / height, 1 - 1 / height, height)
        ang_x = (x_pos[:, None] * pixel[None, :]).repeat_interleave(2, dim=-1)              # [W, Dh/8]
        ang_y = (y_pos[:, None] * pixel[None, :]).repeat_interleave(2, dim=-1)              # [H, Dh/8]
        ang_t = (torch.arange(n_frames).float()[:, None] * lang[None, :]).repeat_interleave(2, dim=-1)
        table = torch.cat([
            ang_x[None, None, :, :].expand(n_frames, height, width, -1),
            ang_y[None, :, None, :].expand(n_frames, height, width, -1),
            ang_t[:, None, None, :].expand(n_frames, height, width, -1),
        ], dim=-1).reshape(n_frames * height * width, d_head // 2)
        return cls(table.cos(), table.sin(), height, width)

    def check_pos_ids(self, pos_ids: Mapping[str, Tensor]) -> None:
        """Eager-mode bounds check of the position ids, as the reference's ``get_angles`` has it
        (``src/model/attn.py:25-30``): ``y < height`` and ``x < width`` are asserted, and a table
        row past the end raises like its ``index_select``.  The kernels clamp the row for memory
        safety only, so without this check a table that is too short would rotate by wrong angles
        silently.  Synchronises; skipped under ``torch.compile`` and stream capture."""
        t, y, x = pos_ids["t_pos"], pos_ids["y_pos"], pos_ids["x_pos"]
        if torch.compiler.is_compiling() or (t.is_cuda and torch.cuda.is_current_stream_capturing()):
            return
        flat = t * (self.height * self.width) + y * self.width + x
        y_max, x_max, f_min, f_max = (int(v) for v in torch.stack([y.max(), x.max(), flat.min(), flat.max()]).tolist())
        if not (y_max < self.height and x_max < self.width):
            raise AssertionError(f"pos_ids out of bounds, {y_max}, {x_max}")
        if f_min < 0 or f_max >= self.cos.shape[0]:
            raise IndexError(f"index out of range in self: RoPE table has {self.cos.shape[0]} rows, position ids "
                             f"select rows {f_min}..{f_max}")

    def forward(self, x: Tensor, pos_ids: Mapping[str, Tensor]) -> Tensor:
        self.check_pos_ids(pos_ids)
        return ops.rope_apply(x, pos_ids, self.cos, self.sin, self.height, self.width)


def ring_attention(q: Tensor, k: Tensor, v: Tensor, block_mask: RingMask, enable_gqa: bool = False,
                   scale: Optional[float] = None) -> Tensor:
    """Call-compatible stand-in for ``flex_attention(q, k, v, block_mask=bm, enable_gqa=...)`` at
    ``src/model/attn.py:116``: ``k``/``v`` must be the cache planes that ``upsert`` returned
    together with ``block_mask``."""
    kv = block_mask.kv
    if k.data_ptr() != kv[0].data_ptr() or v.data_ptr() != kv[1].data_ptr():
        raise RuntimeError("ring_attention needs the k/v views returned by the cache's upsert")
    if not enable_gqa and q.shape[1] != k.shape[1]:
        raise RuntimeError("query and key head counts differ but enable_gqa is False")
    return ops.attn_ring(q, kv, block_mask.written, block_mask.t_pos, block_mask.L,
                         block_mask.dilation, scale)


class RingAttn(nn.Module):
    """Drop-in for the reference's attention module.

    ``config`` provides ``d_model, n_heads`` and optionally ``n_kv_heads, value_residual,
    gated_attn`` (``src/model/attn.py:76-96``).  ``rope`` is a shared :class:`RoPE`.  With
    ``merged_qkv`` the three projections are one ``qkv_proj`` as after the reference's inference
    patch (``src/patch_model.py:102-114``); otherwise the keys are ``q_proj/k_proj/v_proj``.

    ``fuse_elementwise`` moves the module's element-wise neighbours of the attention (QK RMS
    norm, value-residual lerp, head gate incl. its H x H projection and sigmoid) into the two
    kernels: seven to nine launches fewer per layer, results within 1 ulp of the separate torch operations instead of bit-identical, which
    is why it is off unless asked for.

    ``fuse_projection`` (on top of ``merged_qkv`` and ``fuse_elementwise``) also runs the merged
    q/k/v projection in the library, in one kernel with the cache write: x goes in, the rotated q
    and the cache rows come out, the ``[B, T, (H + 2 Hkv) Dh]`` projection output never exists.
    Its rows are fp32 sums rounded once like the BLAS routine's, in another order of additions.
    That kernel is built for the frames this path is slow on - a few hundred tokens, where the
    projection streams its weights once and is bound by memory latency: 64 tokens x 128 features
    per workgroup, one workgroup per CU.  Where the shape needs more workgroups than the 256 CUs
    (``fused_projection_max_workgroups``) the projection is a matrix-core-bound GEMM, the BLAS
    routine is the faster one (measured at 16 heads of 128, d_model 2048, per call: 256 tokens
    16.5 us against 23.4 us for linear layer + store kernel; 1024 tokens 45 against 36; 4096
    tokens of 24 heads, d_model 3072: 356 against 214), and ``forward`` takes the linear layer
    followed by the ``fuse_elementwise`` call instead.
    """

    # one round of workgroups on the 256 CUs of an MI355X
    fused_projection_max_workgroups = 256

    def __init__(self, config, layer_idx: int, rope: RoPE, merged_qkv: bool = False,
                 fuse_elementwise: bool = False, fuse_projection: bool = False):
        super().__init__()
        if fuse_projection and not (merged_qkv and fuse_elementwise):
            raise AssertionError("fuse_projection needs merged_qkv and fuse_elementwise")
        self.fuse_elementwise = fuse_elementwise
        self.fuse_projection = fuse_projection
        self.config = config
        self.layer_idx = layer_idx
        self.n_heads = config.n_heads
        self.n_kv_heads = getattr(config, "n_kv_heads", config.n_heads)
        if config.d_model % self.n_heads != 0:
            raise AssertionError("d_model must be divisible by n_heads")
        self.d_head = config.d_model // self.n_heads
        self.enable_gqa = self.n_heads != self.n_kv_heads
        self.q_out = self.n_heads * self.d_head
        self.kv_out = self.n_kv_heads * self.d_head
        if fuse_projection and (config.d_model % 128 or (self.q_out + 2 * self.kv_out) % 128 or self.d_head not in (64, 128)):
            raise AssertionError("fuse_projection needs d_model and (n_heads + 2 n_kv_heads) * d_head to be multiples "
                                 "of 128 and a head dim of 64 or 128")

        self.value_residual = getattr(config, "value_residual", False)
        if self.value_residual:
            self.v_lamb = nn.Parameter(torch.tensor(0.5))

        self.merged_qkv = merged_qkv
        if merged_qkv:
            self.qkv_proj = nn.Linear(config.d_model, self.q_out + 2 * self.kv_out, bias=False)
        else:
            self.q_proj = nn.Linear(config.d_model, self.q_out, bias=False)
            self.k_proj = nn.Linear(config.d_model, self.kv_out, bias=False)
            self.v_proj = nn.Linear(config.d_model, self.kv_out, bias=False)
        self.out_proj = nn.Linear(config.d_model, config.d_model, bias=False)
        self.rope = rope

        self.gated_attn = getattr(config, "gated_attn", False)
        if self.gated_attn:
            self.gate_proj = nn.Linear(self.n_heads, self.n_heads, bias=False)
            nn.init.zeros_(self.gate_proj.weight)

    @classmethod
    def from_reference(cls, src: nn.Module, config, rope: RoPE, merged_qkv: bool = True,
                       fuse_elementwise: bool = False, fuse_projection: bool = False):
        """Build from an ``Attn``-like module (anything with ``layer_idx`` and a matching state
        dict), the way the reference's ``MergedQKVAttn(src, config)`` does
        (``src/patch_model.py:92-114``): same device and dtype as the source's weights, its
        train / eval mode, ``q_proj | k_proj | v_proj`` rows concatenated into ``qkv_proj`` (or
        split again when ``merged_qkv`` is off and the source is already merged).  Where the
        reference loads with ``strict=False``, a key that has no place in the new module - or a
        parameter of the new module that the source does not provide - raises here: a silently
        random projection is not a state anyone wants."""
        new = cls(config, src.layer_idx, rope, merged_qkv=merged_qkv, fuse_elementwise=fuse_elementwise,
                  fuse_projection=fuse_projection)
        ref_w = next(src.parameters())
        new.to(device=ref_w.device, dtype=ref_w.dtype)
        state = {k: v for k, v in src.state_dict().items() if not k.startswith("rope.")}
        if merged_qkv and "q_proj.weight" in state:
            state["qkv_proj.weight"] = torch.cat(
                [state.pop("q_proj.weight"), state.pop("k_proj.weight"), state.pop("v_proj.weight")], dim=0)
        elif not merged_qkv and "qkv_proj.weight" in state:
            q_w, k_w, v_w = state.pop("qkv_proj.weight").split((new.q_out, new.kv_out, new.kv_out), dim=0)
            state.update({"q_proj.weight": q_w, "k_proj.weight": k_w, "v_proj.weight": v_w})
        own = {k for k in new.state_dict() if not k.startswith("rope.")}
        missing, unexpected = sorted(own - set(state)), sorted(set(state) - own)
        if missing or unexpected:
            raise RuntimeError(f"cannot build RingAttn from {type(src).__name__} (layer {src.layer_idx}): "
                               f"missing keys {missing}, unexpected keys {unexpected}")
        new.load_state_dict(state, strict=False)      # (strict=False only for the shared rope's buffers)
        new.train(src.training)
        return new

    def _forward_fused_projection(self, x: Tensor, pos_ids, v1: Optional[Tensor], kv_cache):
        """x -> [projection + norm + RoPE + value blend + cache write] -> [attention + gate] -> out_proj."""
        B, T = x.shape[:2]
        extras = {"qk_norm_eps": torch.finfo(torch.float32).eps}
        first = self.value_residual and v1 is None
        if self.value_residual and not first:
            extras.update(v1=v1.view(B, self.n_kv_heads, T, self.d_head), v_lamb=self.v_lamb)
        if self.gated_attn:
            extras.update(gate_x=x[..., : self.n_heads], gate_w=self.gate_proj.weight)
        y, v = kv_cache.qkv_rope_upsert_attend(x, self.qkv_proj.weight, self.n_heads, pos_ids, self.rope,
                                               self.layer_idx, want_v=first, reuse_buffers=True, **extras)
        if first:
            v1 = v
        return self.out_proj(y.transpose(1, 2).reshape(B, T, -1)), v1

    def projection_workgroups(self, B: int, T: int) -> int:
        """Workgroups the fused projection kernel launches for x ``[B, T, d_model]``."""
        return B * ((T + 63) // 64) * ((self.q_out + 2 * self.kv_out) // 128)

    def uses_fused_projection(self, B: int, T: int) -> bool:
        return self.fuse_projection and self.projection_workgroups(B, T) <= self.fused_projection_max_workgroups

    def forward(self, x: Tensor, pos_ids: Mapping[str, Tensor], v1: Optional[Tensor], kv_cache):
        B, T = x.shape[:2]
        if (self.uses_fused_projection(B, T) and hasattr(kv_cache, "qkv_rope_upsert_attend")
                and x.dtype in (torch.bfloat16, torch.float16) and x.stride(-1) == 1):
            return self._forward_fused_projection(x, pos_ids, v1, kv_cache)
        if self.merged_qkv:
            q, k, v = self.qkv_proj(x).split((self.q_out, self.kv_out, self.kv_out), dim=-1)
        else:
            q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        q = q.reshape(B, T, self.n_heads, self.d_head).transpose(1, 2)
        k = k.reshape(B, T, self.n_kv_heads, self.d_head).transpose(1, 2)
        v = v.reshape(B, T, self.n_kv_heads, self.d_head).transpose(1, 2)

        fuse = self.fuse_elementwise and hasattr(kv_cache, "rope_upsert_attend") and x.dtype != torch.float32
        extras = {}
        if self.value_residual:
            first = v1 is None
            v1 = v if first else v1
            if not fuse:
                v = torch.lerp(v, v1.view_as(v), self.v_lamb)
            elif not first:                      # lerp(v, v, w) is v
                extras.update(v1=v1.view_as(v), v_lamb=self.v_lamb)

        gates = None
        if self.gated_attn and not fuse:
            gates = torch.sigmoid(self.gate_proj(x[..., : self.n_heads]))
        if fuse:
            extras["qk_norm_eps"] = torch.finfo(torch.float32).eps     # F.rms_norm's epsilon for these inputs
            if self.gated_attn:      # projection + sigmoid + multiply all happen in the kernels' epilogues
                extras.update(gate_x=x[..., : self.n_heads], gate_w=self.gate_proj.weight)
        else:
            q = F.rms_norm(q, (self.d_head,))
            k = F.rms_norm(k, (self.d_head,))

        # RoPE(q), RoPE(k), cache write (one launch) and attention over the ring (one or two), all
        # behind one library call; a cache without it gets the reference's sequence of calls
        if hasattr(kv_cache, "rope_upsert_attend"):
            # (y lives in the layer's own buffer until this layer's next call; out_proj below reads it now)
            y = kv_cache.rope_upsert_attend(q, k, v, pos_ids, self.rope, self.layer_idx, reuse_buffers=True, **extras)
        else:
            q, k_all, v_all, ring = kv_cache.rope_upsert(q, k, v, pos_ids, self.rope, self.layer_idx)
            y = ring_attention(q, k_all, v_all, ring, enable_gqa=self.enable_gqa)

        if gates is not None and not fuse:
            y = y * gates.permute(0, 2, 1).unsqueeze(-1)

        y = y.transpose(1, 2).reshape(B, T, -1)
        return self.out_proj(y), v1


def install_ring_attention(model: nn.Module, rope: Optional[RoPE], attn_types: tuple, merged_qkv: bool = True,
                           fuse_elementwise: bool = False, fuse_projection: bool = False) -> int:
    """Swap every submodule that is an instance of ``attn_types`` for a :class:`RingAttn`, the
    same ``set_submodule`` walk the reference uses for its merged-QKV patch
    (``src/patch_model.py:144-147``).  ``rope=None`` takes the tables of the modules' own ``.rope``
    (``cos`` / ``sin`` buffers, grid from ``model.config.height / width``): modules that share one
    rotary module (``src/model/world_model.py:199-202``) share one :class:`RoPE` afterwards too.
    Returns the number of modules replaced."""
    n = 0
    ropes = {}
    for name, mod in list(model.named_modules()):
        if isinstance(mod, attn_types) and not isinstance(mod, RingAttn):
            r = rope
            if r is None:
                src = mod.rope
                if id(src) not in ropes:
                    ropes[id(src)] = RoPE(src.cos.detach().clone(), src.sin.detach().clone(), model.config.height,
                                          model.config.width).to(src.cos.device)
                r = ropes[id(src)]
            model.set_submodule(name, RingAttn.from_reference(mod, model.config, r, merged_qkv, fuse_elementwise,
                                                                 fuse_projection))
            n += 1
    return n
