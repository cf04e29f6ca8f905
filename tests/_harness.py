"""Shared driver for the GPU parity tests: runs the same seeded frame schedule through the CPU
oracle and through the HIP path (the package's classes, which call the C ABI) and compares."""
from __future__ import annotations

import math
from types import SimpleNamespace
from typing import Dict, Iterable, Optional

import torch

from oracle import ring_oracle as ro
import world_engine_amd as wea
from world_engine_amd import ops

# north-star tolerance for attention outputs on bf16 inputs against the fp32 oracle
MAX_ABS, MEAN_ABS = 2e-2, 2e-3

# Worst errors against the fp32 oracle recorded with the present kernels on the benchmark
# configurations (max-abs, mean-abs over the steps the tests check).  The tests fail when either
# doubles, long before a regression reaches the tolerance above.
RECORDED_MARGIN = {"cfg1": (2.3e-3, 1.6e-4), "cfg2": (9.1e-3, 2.0e-4), "cfg3": (2.2e-3, 9.3e-5), "cfg4": (2.2e-3, 1.6e-4)}


def assert_margin(name: str, worst):
    mx, mean = worst
    lim_mx, lim_mean = RECORDED_MARGIN[name]
    print(f"margin {name}: worst max-abs {mx:.3e} mean-abs {mean:.3e} (recorded {lim_mx:.1e} / {lim_mean:.1e})", flush=True)
    assert mx <= 2 * lim_mx and mean <= 2 * lim_mean, (
        f"{name}: error against the fp32 oracle grew: max-abs {mx:.3e} (recorded {lim_mx:.1e}), "
        f"mean-abs {mean:.3e} (recorded {lim_mean:.1e})")


def make_config(T, n_slots, H, Hkv, Dh, n_layers=1, d=1):
    return SimpleNamespace(tokens_per_frame=T, local_window=n_slots, global_window=n_slots,
                           global_attn_period=1, global_pinned_dilation=d, n_layers=n_layers,
                           n_heads=H, n_kv_heads=Hkv, d_model=H * Dh)


def to_dev(pos: Dict[str, torch.Tensor], dev):
    return {k: v.to(dev) for k, v in pos.items()}


def merged_views(q, k, v):
    """Lay q/k/v out the way the merged projection produces them (src/patch_model.py:117-122):
    one [B, T, (H+2Hkv)*Dh] buffer, viewed as transposed [B, H, T, Dh] slices."""
    B, H, T, Dh = q.shape
    Hkv = k.shape[1]
    buf = torch.cat([q.transpose(1, 2).reshape(B, T, H * Dh), k.transpose(1, 2).reshape(B, T, Hkv * Dh),
                     v.transpose(1, 2).reshape(B, T, Hkv * Dh)], dim=-1).contiguous()
    qq, kk, vv = buf.split((H * Dh, Hkv * Dh, Hkv * Dh), dim=-1)
    return (qq.reshape(B, T, H, Dh).transpose(1, 2), kk.reshape(B, T, Hkv, Dh).transpose(1, 2),
            vv.reshape(B, T, Hkv, Dh).transpose(1, 2))


class Pair:
    """One oracle cache and one HIP cache fed identical inputs."""

    def __init__(self, dev, dtype, B, H, Hkv, T, Dh, n_slots, d=1, n_layers=1, table_rows=None, cfg_id=0):
        self.dev, self.dtype = dev, dtype
        self.B, self.H, self.Hkv, self.T, self.Dh, self.n, self.d = B, H, Hkv, T, Dh, n_slots, d
        self.W = int(math.isqrt(T))
        if self.W * self.W != T:          # not a square patch grid: treat the frame as one row
            self.W = T
        self.Hgrid = T // self.W
        self.cfg_id = cfg_id
        cfg = make_config(T, n_slots, H, Hkv, Dh, n_layers, d)
        self.oracle = ro.OracleStaticKVCache(cfg, B, dtype)
        self.hip = wea.StaticKVCache(cfg, B, dtype).to(dev)
        for layer in self.hip.layers:
            layer.check_inputs = False
        rows = table_rows or 64 * T
        self.cos, self.sin = ro.rope_table_1d(rows, Dh)
        self.rope = wea.RoPE(self.cos, self.sin, self.Hgrid, self.W).to(dev)

    def set_frozen(self, f):
        self.oracle.set_frozen(f)
        self.hip.set_frozen(f)

    def inputs(self, step, sub=0, outlier=False):
        q, k, v = ro.synth_qkv(self.cfg_id, step, sub, self.B, self.H, self.Hkv, self.T, self.Dh,
                               self.dtype, outlier)
        return q, k, v, ro.synth_pos_ids(step, self.B, self.T, self.W)

    def store(self, q, k, v, pos, layer=0, strided=True):
        """RoPE + upsert on both sides.  Returns oracle (q_rot, k_all, v_all, mask) and HIP
        (q_rot, ring descriptor)."""
        cos, sin = ro.rope_angles(pos, self.cos, self.sin, self.Hgrid, self.W)
        q_o, k_o = ro.rope_apply(q, cos, sin), ro.rope_apply(k, cos, sin)
        k_all, v_all, mask = self.oracle.upsert(k_o, v, pos, layer)
        qd, kd, vd = q.to(self.dev), k.to(self.dev), v.to(self.dev)
        if strided:
            qd, kd, vd = merged_views(qd, kd, vd)
        q_h, k_h, v_h, ring = self.hip.rope_upsert(qd, kd, vd, to_dev(pos, self.dev), self.rope, layer)
        return (q_o, k_all, v_all, mask), (q_h, ring)

    def assert_state_equal(self, layer=0, what=""):
        o, h = self.oracle.layers[layer], self.hip.layers[layer]
        assert torch.equal(h.written.cpu(), o.written), f"written differs {what}"
        assert_bits_equal(h.kv, o.kv, f"kv buffer {what}")

    def attend(self, q_h, ring, **kw):
        return ops.attn_ring(q_h, ring.kv, ring.written, ring.t_pos, ring.L, ring.dilation, **kw)


def assert_bits_equal(a: torch.Tensor, b: torch.Tensor, what=""):
    """Bit-for-bit equality.  NaNs only have to be NaN on both sides: torch's own fp32->bf16
    conversions disagree on the NaN bit pattern (0x7FC0 scalar, 0xFFFF vectorised)."""
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    assert a.shape == b.shape and a.dtype == b.dtype, what
    if torch.equal(a.view(torch.uint8), b.view(torch.uint8)):
        return
    ib = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[a.element_size()]
    bad = (a.view(ib) != b.view(ib)) & ~(a.isnan() & b.isnan())
    if bad.any():
        idx = bad.nonzero()
        raise AssertionError(f"bit mismatch: {what}: {idx.shape[0]} elements, first at {idx[0].tolist()}")


def assert_attn_close(out_hip: torch.Tensor, ref32: torch.Tensor, what=""):
    diff = (out_hip.float().cpu() - ref32.float()).abs()
    mx, mean = diff.max().item(), diff.mean().item()
    assert math.isfinite(mx), f"non-finite output {what}"
    assert mx <= MAX_ABS and mean <= MEAN_ABS, f"{what}: max-abs {mx:.3e} (<= {MAX_ABS}), mean-abs {mean:.3e} (<= {MEAN_ABS})"
    return mx, mean


def assert_ulp_close(a, b, what, ulps=1):
    """Element-type tensors equal up to `ulps` units in the last place of the largest value of
    their row (a last-bit difference in a normalised input moves a rotated pair, a difference of
    products, by that much whatever the size of the result).  Returns the fraction that differs."""
    a32, b32 = a.float().cpu(), b.float().cpu()
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[a.dtype]
    tol = 2 * ulps * eps * b32.abs().amax(dim=-1, keepdim=True).clamp_min(2.0 ** -100)
    bad = (a32 - b32).abs() > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off by more than {ulps} ulp of their row's largest"
    return float((a32 != b32).float().mean())
