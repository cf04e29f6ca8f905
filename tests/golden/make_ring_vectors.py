#!/usr/bin/env python3
"""Writes tests/golden/ring_cfg0_bf16.npz: a frozen snapshot of the smallest benchmark
configuration (one layer, B=1, H=8, Dh=64, 64 tokens per frame, 4-slot ring, 8 frame-steps so the
ring wraps twice) at bf16.

The reference holds no golden vectors for this path and its modules do not import in this
environment (tensordict, rotary_embedding_torch and omegaconf are absent), so the expected values
are produced by the CPU oracle, whose functions are pinned independently in
tests/test_oracle_pins.py.  The snapshot guards both sides against drift: the CPU suite checks
that the oracle still reproduces it, the GPU suite checks the HIP path against it.

Contents: for every step the SHA-256 of the cache buffer bytes and of `written` after the store;
for steps 1, 4 and 7 the fp32 attention output [B, H, T, Dh] and the bf16 bits of RoPE(q).
Inputs are regenerated from the seeds (oracle.ring_oracle.synth_qkv) and are not stored.

Run from the repository root:  python tests/golden/make_ring_vectors.py
"""
import hashlib
import os
import sys
from types import SimpleNamespace

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ring_oracle as ro  # noqa: E402

CFG = dict(cfg_id=0, B=1, H=8, Hkv=8, Dh=64, T=64, n_slots=4, steps=8, keep=(1, 4, 7))


def digest(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def run(cfg=CFG):
    B, H, Hkv, Dh, T, n = cfg["B"], cfg["H"], cfg["Hkv"], cfg["Dh"], cfg["T"], cfg["n_slots"]
    W = 8
    conf = SimpleNamespace(tokens_per_frame=T, local_window=n, global_window=n, global_attn_period=1,
                           global_pinned_dilation=1, n_layers=1, n_heads=H, n_kv_heads=Hkv, d_model=H * Dh)
    cache = ro.OracleStaticKVCache(conf, B, torch.bfloat16)
    cache.set_frozen(False)
    cos_t, sin_t = ro.rope_table_1d(64 * T, Dh)
    out = {"kv_sha256": [], "written_sha256": []}
    for step in range(cfg["steps"]):
        q, k, v = ro.synth_qkv(cfg["cfg_id"], step, 0, B, H, Hkv, T, Dh, torch.bfloat16)
        pos = ro.synth_pos_ids(step, B, T, W)
        cos, sin = ro.rope_angles(pos, cos_t, sin_t, T // W, W)
        q_r, k_r = ro.rope_apply(q, cos, sin), ro.rope_apply(k, cos, sin)
        k_all, v_all, mask = cache.upsert(k_r, v, pos, 0)
        out["kv_sha256"].append(digest(cache.layers[0].kv))
        out["written_sha256"].append(digest(cache.layers[0].written))
        if step in cfg["keep"]:
            out[f"attn_fp32_step{step}"] = ro.attention_fp32(q_r, k_all, v_all, mask).numpy()
            out[f"q_rot_bits_step{step}"] = q_r.contiguous().view(torch.int16).numpy()
    return out


if __name__ == "__main__":
    res = run()
    res["kv_sha256"] = np.array(res["kv_sha256"])
    res["written_sha256"] = np.array(res["written_sha256"])
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ring_cfg0_bf16.npz")
    np.savez_compressed(path, **res)
    print(path, os.path.getsize(path), "bytes")
