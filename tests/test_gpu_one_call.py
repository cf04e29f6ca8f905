"""GPU parity of the one-call path (we_rope_kv_attn_fwd): RoPE + K/V store + attention.

Cache rows, ``written`` and RoPE(q) must equal the oracle's bit for bit (and so the two-call
path's); attention within max-abs 2e-2 / mean-abs 2e-3 of the fp32 oracle.
"""
import pytest
import torch

from oracle import ring_oracle as ro
from _harness import Pair, assert_attn_close, assert_bits_equal, merged_views, to_dev
from world_engine_amd import ops

pytestmark = pytest.mark.gpu


def _one_call_step(p, t, sub, frozen, layer=0, outlier=False, strided=True, **kw):
    """One schedule step through the oracle and through ops.rope_kv_attn; returns the two outputs."""
    p.set_frozen(frozen)
    q, k, v, pos = p.inputs(t, sub, outlier)
    cos, sin = ro.rope_angles(pos, p.cos, p.sin, p.Hgrid, p.W)
    q_o, k_o = ro.rope_apply(q, cos, sin), ro.rope_apply(k, cos, sin)
    k_all, v_all, mask = p.oracle.upsert(k_o, v, pos, layer)
    ref = ro.attention_fp32(q_o, k_all, v_all, mask)
    qd, kd, vd = q.to(p.dev), k.to(p.dev), v.to(p.dev)
    if strided:
        qd, kd, vd = merged_views(qd, kd, vd)
    lay = p.hip.layers[layer]
    out, q_rot = ops.rope_kv_attn(qd, kd, vd, to_dev(pos, p.dev), p.rope.cos, p.rope.sin, p.rope.height,
                                  p.rope.width, lay.kv, lay.written, lay.L, lay.pinned_dilation, frozen, **kw)
    assert_bits_equal(q_rot, q_o, f"RoPE(q) t={t} sub={sub}")
    p.assert_state_equal(layer=layer, what=f"t={t} sub={sub} frozen={frozen}")
    return out, ref


@pytest.mark.parametrize("dtype,Dh", [(torch.bfloat16, 128), (torch.float16, 128), (torch.bfloat16, 64)])
def test_one_call_schedule_small_frames(gpu_device, dtype, Dh):
    """Frozen substeps + persisting call over more than two wraps, warm-up frames included."""
    print(f"one call dtype={dtype} Dh={Dh}", flush=True)
    p = Pair(gpu_device, dtype, B=1, H=4, Hkv=4, T=128, Dh=Dh, n_slots=5, cfg_id=31)
    for t in range(12):
        for sub, frozen in ((0, True), (1, False)):
            out, ref = _one_call_step(p, t, sub, frozen, strided=(t % 2 == 0))
            assert_attn_close(out, ref, f"t={t} sub={sub}")


def test_one_call_cfg1_shape(gpu_device):
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, cfg_id=1)
    for t in list(range(0, 20)) + [31, 32, 33]:
        out, ref = _one_call_step(p, t, 0, False)
        assert_attn_close(out, ref, f"t={t}")


@pytest.mark.parametrize("kw", [{"n_splits": 1}, {"n_splits": 2}, {"n_splits": 5}, {"n_splits": 16}])
def test_one_call_split_counts(gpu_device, kw):
    p = Pair(gpu_device, torch.bfloat16, B=2, H=2, Hkv=2, T=128, Dh=128, n_slots=6, cfg_id=32)
    for t in range(9):
        out, ref = _one_call_step(p, t, 0, t % 3 == 1, **kw)
        assert_attn_close(out, ref, f"t={t} {kw}")


def test_one_call_grouped_heads_and_dilation(gpu_device):
    """Two query heads per kv head and a pinned dilation of 2 (frames that do not persist leave
    the ring alone)."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=4, Hkv=2, T=64, Dh=128, n_slots=8, d=2, cfg_id=33)
    for t in range(13):
        out, ref = _one_call_step(p, t, 0, False)
        assert_attn_close(out, ref, f"t={t}")


def test_one_call_large_frames(gpu_device):
    """1024-token frames (256-query workgroups) behind the same entry point."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=2, Hkv=2, T=1024, Dh=128, n_slots=2, cfg_id=34)
    for t in range(3):
        out, ref = _one_call_step(p, t, 0, False)
        assert_attn_close(out, ref, f"t={t}")


def test_one_call_outlier_channel(gpu_device):
    p = Pair(gpu_device, torch.bfloat16, B=1, H=4, Hkv=4, T=256, Dh=128, n_slots=4, cfg_id=35)
    for t in range(6):
        out, ref = _one_call_step(p, t, 0, False, outlier=True)
        assert_attn_close(out, ref, f"t={t}")


def test_module_forward_compiles_as_one_graph(gpu_device):
    """RingAttn under torch.compile(fullgraph=True): the cache call is the registered opaque op
    (the reference wraps its one native kernel the same way, src/quantize.py:17-42); results and
    cache state equal the eager module's."""
    import types
    import world_engine_amd as wea
    torch.manual_seed(0)
    cfg = types.SimpleNamespace(d_model=256, n_heads=4, n_kv_heads=2, value_residual=True, gated_attn=True,
                                tokens_per_frame=64, local_window=3, global_window=3, global_attn_period=1,
                                global_pinned_dilation=1, n_layers=1)
    cos, sin = ro.rope_table_1d(16 * 64, 64)
    rope = wea.RoPE(cos, sin, 8, 8).to(gpu_device)
    mod = wea.RingAttn(cfg, 0, rope, merged_qkv=True).to(gpu_device, torch.bfloat16)
    with torch.no_grad():
        mod.gate_proj.weight.normal_(0, 0.5)
    caches = [wea.StaticKVCache(cfg, 1, torch.bfloat16).to(gpu_device) for _ in range(2)]
    for c in caches:
        c.set_frozen(False)
        for layer in c.layers:
            layer.check_inputs = False
    compiled = torch.compile(mod, backend="eager", fullgraph=True)
    for t in range(5):
        x = torch.randn(1, 64, 256, device=gpu_device, dtype=torch.bfloat16)
        pos = to_dev(ro.synth_pos_ids(t, 1, 64, 8), gpu_device)
        with torch.no_grad():
            y_e, _ = mod(x, pos, None, caches[0])
            y_c, _ = compiled(x, pos, None, caches[1])
        assert torch.equal(y_e, y_c), f"t={t}"
        assert_bits_equal(caches[0].layers[0].kv, caches[1].layers[0].kv, f"cache t={t}")
        assert torch.equal(caches[0].layers[0].written, caches[1].layers[0].written)
