"""MI355X-native frame-causal ring-buffer attention for world_engine's per-frame hot path.

Public surface mirrors the reference's for this path: :class:`StaticKVCache`,
:class:`LayerKVCache` (``src/model/kv_cache.py``), :class:`RingAttn` for ``Attn`` /
``MergedQKVAttn`` and :class:`RoPE` (``src/model/attn.py``, ``src/patch_model.py``).
All compute goes through hand-written gfx950 kernels in ``libwe_attn.so``; there is no CPU or
eager fallback.
"""
from .kv_cache import LayerKVCache, RingMask, StaticKVCache
from .attn import RingAttn, RoPE, install_ring_attention, ring_attention
from . import ops

__all__ = ["LayerKVCache", "StaticKVCache", "RingMask", "RingAttn", "RoPE", "ring_attention",
           "install_ring_attention", "ops"]
