"""GPU parity on the edges of the path's domain, each against the CPU oracle driven the same way:
frame indices beyond 32 bits (the kernels' 64-bit slot arithmetic), batch rows with different
frame indices, the largest ring the library takes, non-finite values in V across context splits,
negative and boundary value-residual weights."""
import pytest
import torch

from oracle import ring_oracle as ro
from _harness import Pair, assert_attn_close, assert_bits_equal, assert_ulp_close, merged_views, to_dev
import world_engine_amd as wea
from world_engine_amd import _capi, ops

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


@pytest.mark.parametrize("base", [2 ** 31 + 5, 2 ** 33 + 7])
@pytest.mark.parametrize("d", [1, 3])
def test_frame_indices_beyond_32_bits(gpu_device, base, d):
    """The reference computes the slot in int64 throughout (src/model/kv_cache.py:126-131,140); the
    kernels take a 32-bit shortcut for small frame indices and 64-bit floor division beyond.  Keys
    are stored as given (no table has 2^31 rows), then attended: cache state bit-exact, output in
    tolerance, over more frames than the ring has buckets."""
    _say(f"frame index base {base} dilation {d}")
    n = 2 * d if d > 1 else 4
    dev = gpu_device
    p = Pair(dev, torch.bfloat16, B=1, H=4, Hkv=2, T=64, Dh=64, n_slots=n, d=d, cfg_id=91)
    for i in range(3 * n + 2):
        t = base + i
        frozen = i % 4 == 3
        p.set_frozen(frozen)
        q, k, v, _ = p.inputs(i)
        pos = ro.synth_pos_ids(t, 1, 64, p.W)
        assert int(pos["t_pos"][0, 0]) == t
        k_all, v_all, mask = p.oracle.upsert(k, v, pos, 0)
        kh, vh, ring = p.hip.upsert(k.to(dev), v.to(dev), to_dev(pos, dev), 0)
        p.assert_state_equal(what=f"t={t} frozen={frozen}")
        assert torch.equal(ring.dense().cpu(), mask), f"mask t={t}"
        for kw in ({}, {"n_splits": 2}):
            out = ops.attn_ring(q.to(dev), ring.kv, ring.written, ring.t_pos, ring.L, ring.dilation, **kw)
            assert_attn_close(out, ro.attention_fp32(q, k_all, v_all, mask), f"t={t} {kw}")


def test_batch_rows_with_different_frame_indices(gpu_device):
    """The ring slot comes from t_pos[0, 0] (src/model/kv_cache.py:126), the rotary table row from
    every row's own t (src/model/attn.py:27): batch row 0 at frame 5, row 1 at frame 9."""
    dev = gpu_device
    p = Pair(dev, torch.bfloat16, B=2, H=4, Hkv=2, T=64, Dh=128, n_slots=4, cfg_id=92)
    p.set_frozen(False)
    for step, (t0, t1) in enumerate([(5, 9), (6, 2), (7, 7), (8, 30), (9, 0)]):
        q, k, v, _ = p.inputs(step)
        pos = ro.synth_pos_ids(t0, 2, 64, p.W)
        pos["t_pos"][1] = t1
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        assert_bits_equal(q_h, q_o, f"RoPE(q) rows at frames {t0}, {t1}")
        p.assert_state_equal(what=f"frames {t0}, {t1}")
        slot, _ = ro.slot_and_write_step(t0, 4, 1)
        assert bool(p.hip.layers[0].written[slot * 64]), "the slot is row 0's"
        if t1 != t0:   # the two batch rows really were rotated by different angles
            same = ro.rope_apply(q, *ro.rope_angles(ro.synth_pos_ids(t0, 2, 64, p.W), p.cos, p.sin, p.Hgrid, p.W))
            assert not torch.equal(same[1], q_o[1])
        assert_attn_close(p.attend(q_h, ring), ro.attention_fp32(q_o, k_all, v_all, mask), f"frames {t0}, {t1}")


def test_largest_ring_runs_through_a_wrap_and_one_more_slot_is_refused(gpu_device):
    """WE_MAX_SLOTS = 256 ring slots: filled, wrapped and attended; 257 slots are refused with
    WE_ERR_UNSUPPORTED before anything is launched."""
    dev = gpu_device
    n = _capi.WE_MAX_SLOTS
    T = 32
    p = Pair(dev, torch.bfloat16, B=1, H=2, Hkv=1, T=T, Dh=64, n_slots=n, cfg_id=93, table_rows=(n + 8) * T)
    p.set_frozen(False)
    checks = {0, 1, 63, 64, 65, 127, 128, 255, 256, 257, 259}
    for t in range(n + 4):
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        if t in checks:
            _say(f"256 slots: frame {t}")
            p.assert_state_equal(what=f"t={t}")
            assert int(mask.sum()) == (min(t, n - 1) + 1) * T
            for kw in ({}, {"n_splits": 5}):
                assert_attn_close(p.attend(q_h, ring, **kw), ro.attention_fp32(q_o, k_all, v_all, mask), f"t={t} {kw}")
    big = wea.LayerKVCache(1, 1, (n + 1) * T, 64, torch.bfloat16, T).to(dev)
    qz = torch.zeros(1, 2, T, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="not covered"):
        ops.attn_ring(qz, big.kv, big.written, torch.zeros(1, T, dtype=torch.long, device=dev), (n + 1) * T, 1)


def test_non_finite_values_in_v_poison_the_same_columns_however_the_context_is_split(gpu_device):
    """An infinity or a NaN in a visible V row makes exactly that head-dim column non-finite for
    the queries that see it - in a single pass as in the reference's P @ V - and the same must hold
    when the context is split and the parts are merged; a row whose values are tiny (below 2^-126)
    must come back as zeros or tiny values, not as NaN."""
    dev = gpu_device
    p = Pair(dev, torch.bfloat16, B=1, H=8, Hkv=8, T=128, Dh=128, n_slots=4, cfg_id=94)
    p.set_frozen(False)
    for t in range(3):
        q, k, v, pos = p.inputs(t)
        if t == 1:
            v[0, 0, 5, 17] = float("inf")
            v[0, 1, 77, 3] = float("nan")
            v[0, 2, 9, 40] = -float("inf")
            v[0, 3] = v[0, 3] * 1e-38            # subnormal-sized values in every column of head 3's new frame
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
    single = p.attend(q_h, ring, n_splits=1).float().cpu()
    assert torch.isinf(single[0, 0, :, 17]).all() and torch.isnan(single[0, 1, :, 3]).all()
    assert (single[0, 2, :, 40] == -float("inf")).all()
    assert torch.isfinite(single[0, 3]).all()
    for n_splits in (2, 3, 6):
        split = p.attend(q_h, ring, n_splits=n_splits).float().cpu()
        assert torch.equal(torch.isnan(split), torch.isnan(single)), f"{n_splits} parts: NaN pattern differs"
        assert torch.equal(torch.isinf(split), torch.isinf(single)), f"{n_splits} parts: infinity pattern differs"
        fin = torch.isfinite(single)
        assert torch.equal(split[~fin & ~torch.isnan(single)], single[~fin & ~torch.isnan(single)])
        d = (split[fin] - single[fin]).abs()
        assert d.max().item() <= 2e-2 and d.mean().item() <= 2e-3, (n_splits, d.max().item())


@pytest.mark.parametrize("lamb", [-0.75, 0.5, -0.5, 0.498046875])
def test_value_blend_weight_signs_and_the_switch_point(gpu_device, lamb):
    """torch.lerp switches formula at |w| = 0.5 (ATen/native/Lerp.h), not at w = 0.5: a learned
    v_lamb at or below -0.5 takes the second formula.  Cache rows against the oracle's value_lerp
    (pinned to torch.lerp bit for bit) within 1 ulp (the kernel's fused multiply-add)."""
    dev = gpu_device
    dtype = torch.bfloat16
    p = Pair(dev, dtype, B=1, H=2, Hkv=2, T=64, Dh=64, n_slots=2, cfg_id=95)
    layer = p.hip.layers[0]
    g = torch.Generator("cpu").manual_seed(11)
    w = torch.tensor(lamb, dtype=dtype)
    for t in range(3):
        p.set_frozen(False)
        q, k, v, pos = p.inputs(t)
        v1 = torch.randn(v.shape, generator=g).to(dtype)
        ref, _ = ro.layer_step(p.oracle, 0, q, k, v, pos, p.cos, p.sin, p.Hgrid, p.W, reference_dtype_flow=False, v1=v1, v_lamb=w)
        qd, kd, vd = merged_views(q.to(dev), k.to(dev), v.to(dev))
        out, _ = ops.rope_kv_attn(qd, kd, vd, to_dev(pos, dev), p.rope.cos, p.rope.sin, p.rope.height, p.rope.width,
                                  layer.kv, layer.written, layer.L, 1, False, v1=v1.to(dev), v_lamb=w.to(dev))
        assert_bits_equal(layer.kv[0], p.oracle.layers[0].kv[0], f"K plane t={t}")
        frac = assert_ulp_close(layer.kv[1], p.oracle.layers[0].kv[1], f"blended V plane, weight {lamb}, t={t}")
        assert frac < 0.05, frac
        assert_attn_close(out, ref, f"weight {lamb} t={t}")
