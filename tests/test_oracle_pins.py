"""Pins for the CPU oracle (oracle/ring_oracle.py).

The reference ships no tests, golden vectors or fixtures for this path, so every oracle function
is pinned against something that does not restate its formula: an independent frame-retention
model for the ring, closed forms and invariants for RoPE, and torch's own library routines
(eager ``flex_attention`` with a ``BlockMask``, ``scaled_dot_product_attention``) plus fp64
brute force for the attention.
"""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import ring_oracle as ro


# ----------------------------------------------------------------------------------------
# slot arithmetic and ring contents: independent retention model
# ----------------------------------------------------------------------------------------
class RetentionModel:
    """What the ring is *for*, written without slot formulas: persisting frames (multiples of
    the dilation) are kept, the ring holds the most recent ``n_slots/d`` of them in a FIFO: the
    first frames fill positions 0, 1, 2, ... in arrival order, after that a new persisting
    frame takes the position of the oldest kept one.  Nothing else ever moves."""

    def __init__(self, n_slots, d):
        self.cap = n_slots // d
        self.d = d
        self.where = {}          # kept frame -> position in the ring
        self.order = []          # kept frames, oldest first

    def persist(self, frame):
        assert frame % self.d == 0 and frame not in self.where
        if len(self.order) < self.cap:
            pos = len(self.order)
        else:
            pos = self.where.pop(self.order.pop(0))
        self.where[frame] = pos
        self.order.append(frame)
        return pos


@pytest.mark.parametrize("n_slots,d", [(4, 1), (16, 1), (8, 2), (8, 4), (12, 3), (32, 1)])
def test_slot_sequence_against_retention_model(n_slots, d):
    model = RetentionModel(n_slots, d)
    for t in range(0, 3 * n_slots * d + 5):
        slot, ws = ro.slot_and_write_step(t, n_slots, d)
        assert ws == (t % d == 0)
        assert 0 <= slot < n_slots // d
        if ws:
            pos = model.persist(t)
            assert pos == slot, (t, pos, slot)
        else:
            # an off-dilation frame maps to the slot the NEXT persisting frame will take
            nxt = ((t // d) + 1) * d
            assert slot == ro.slot_and_write_step(nxt, n_slots, d)[0]


def test_slot_sequences_of_the_benchmark_configs():
    # d = 1: slot = t mod n; cfg0 wraps twice over 8 steps, cfg1 over 32
    assert [ro.slot_and_write_step(t, 4, 1)[0] for t in range(8)] == [0, 1, 2, 3, 0, 1, 2, 3]
    assert [ro.slot_and_write_step(t, 16, 1)[0] for t in range(32)] == list(range(16)) * 2
    # d = 2 with 8 slots: 4 buckets, frames 0,2,4,6,8 -> slots 0,1,2,3,0
    assert [ro.slot_and_write_step(t, 8, 2)[0] for t in (0, 2, 4, 6, 8)] == [0, 1, 2, 3, 0]


def _frame_kv(frame, sub, B, H, T, Dh, dtype):
    g = torch.Generator().manual_seed(1000 * frame + sub)
    return torch.randn(2, B, H, T, Dh, generator=g).to(dtype)


@pytest.mark.parametrize("n_slots,d", [(4, 1), (6, 2), (8, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ring_contents_against_dict_of_frames(n_slots, d, dtype):
    """Drive the oracle with the engine's schedule (frozen passes, then one unfrozen pass,
    src/world_engine.py:139-152) and rebuild the expected buffers from scratch each step."""
    B, H, T, Dh = 2, 2, 8, 16
    L = n_slots * T
    cache = ro.OracleLayerKVCache(B, H, L, Dh, dtype, T, d)
    kept = {}                                   # slot -> kv of the frame living there
    for t in range(3 * n_slots * d + 2):
        pos = {"t_pos": torch.full((B, T), t)}
        slot, ws = ro.slot_and_write_step(t, n_slots, d)
        for sub, frozen in ((0, True), (1, True), (2, False)):
            new = _frame_kv(t, sub, B, H, T, Dh, dtype)
            ring_before = cache.kv[:, :, :, :L].clone()
            written_before = cache.written.clone()
            k_all, v_all, mask = cache.upsert(new, pos, frozen)
            # tail always equals the latest call's K/V
            assert torch.equal(cache.kv[:, :, :, L:], new)
            if frozen:
                assert torch.equal(cache.kv[:, :, :, :L], ring_before)
                assert torch.equal(cache.written, written_before)
            elif ws:
                kept[slot] = new
            # expected visibility: kept frames except the one this persisting frame replaces
            exp_mask = torch.zeros(L + T, dtype=torch.bool)
            exp_mask[L:] = True
            for s in kept:
                exp_mask[s * T:(s + 1) * T] = True
            if ws:      # the frame about to be replaced is hidden, before and after the write
                exp_mask[slot * T:(slot + 1) * T] = False
            assert torch.equal(mask, exp_mask), (t, sub)
            assert k_all.data_ptr() == cache.kv[0].data_ptr() and v_all.shape == (B, H, L + T, Dh)
        # rebuild the whole buffer from the dict of kept frames
        exp = torch.zeros(2, B, H, L + T, Dh, dtype=dtype)
        exp_written = torch.zeros(L + T, dtype=torch.bool)
        exp_written[L:] = True
        for s, f in kept.items():
            exp[:, :, :, s * T:(s + 1) * T] = f
            exp_written[s * T:(s + 1) * T] = True
        exp[:, :, :, L:] = new
        assert torch.equal(cache.kv, exp)
        assert torch.equal(cache.written, exp_written)
        # slots beyond the cycled buckets are never touched
        assert not cache.written[(n_slots // d) * T:L].any()
    cache.reset()
    assert not cache.kv.any() and cache.written[L:].all() and not cache.written[:L].any()


@pytest.mark.parametrize("n_slots", [4, 16])
def test_visible_count_closed_form(n_slots):
    """d = 1: N_vis(t) = min(t, n-1)*T + T (steady state L, not L+T)."""
    B, H, T, Dh = 1, 1, 4, 16
    cache = ro.OracleLayerKVCache(B, H, n_slots * T, Dh, torch.float32, T, 1)
    for t in range(3 * n_slots):
        _, _, mask = cache.upsert(torch.zeros(2, B, H, T, Dh), {"t_pos": torch.full((B, T), t)}, False)
        assert int(mask.sum()) == min(t, n_slots - 1) * T + T
        assert torch.equal(mask, ro.visible_mask(cache.written, t, T, n_slots, 1))


def test_oracle_input_checks():
    cache = ro.OracleLayerKVCache(1, 1, 16, 16, torch.float32, 4, 1)
    with pytest.raises(RuntimeError):
        cache.upsert(torch.zeros(2, 1, 1, 3, 16), {"t_pos": torch.zeros(1, 3, dtype=torch.long)}, True)
    with pytest.raises(RuntimeError):
        cache.upsert(torch.zeros(2, 1, 1, 4, 16), {"t_pos": torch.tensor([[0, 0, 1, 0]])}, True)
    with pytest.raises(RuntimeError):
        cache.upsert(torch.zeros(2, 1, 1, 4, 16), {"t_pos": torch.full((1, 4), -1)}, True)


def test_static_cache_layer_geometry():
    cfg = SimpleNamespace(tokens_per_frame=4, local_window=2, global_window=8, global_attn_period=3,
                          global_attn_offset=1, global_pinned_dilation=4, n_layers=7, n_heads=4,
                          n_kv_heads=2, d_model=64)
    c = ro.OracleStaticKVCache(cfg, 1, torch.float32)
    is_global = [i in (1, 4) for i in range(7)]
    for layer, g in zip(c.layers, is_global):
        assert layer.L == (32 if g else 8) and layer.pinned_dilation == (4 if g else 1)
        assert layer.kv.shape == (2, 1, 2, layer.L + 4, 16)
    assert c._is_frozen
    c.set_frozen(False)
    c.reset()
    assert c._is_frozen


# ----------------------------------------------------------------------------------------
# RoPE
# ----------------------------------------------------------------------------------------
def test_rope_table_1d_matches_direct_fp64():
    cos, sin = ro.rope_table_1d(50, 32)
    for p in (0, 1, 17, 49):
        for i in (0, 5, 15):
            ang = p * 10000.0 ** (-2.0 * i / 32)
            assert abs(cos[p, i].item() - math.cos(ang)) < 1e-7
            assert abs(sin[p, i].item() - math.sin(ang)) < 1e-7


def test_rope_is_complex_rotation_with_deinterleaved_output():
    torch.manual_seed(0)
    B, H, T, Dh, W = 2, 3, 16, 32, 4
    cos_t, sin_t = ro.rope_table_1d(5 * T, Dh)
    x = torch.randn(B, H, T, Dh)
    pos = ro.synth_pos_ids(3, B, T, W)
    cos, sin = ro.rope_angles(pos, cos_t, sin_t, T // W, W)
    y = ro.rope_apply(x, cos, sin)
    # closed form: (x_even + i x_odd) * exp(i*angle), angle row = 3*T + token
    z = torch.complex(x[..., 0::2].double(), x[..., 1::2].double())
    inv = 10000.0 ** (-2.0 * torch.arange(Dh // 2, dtype=torch.float64) / Dh)
    ang = (3 * T + torch.arange(T, dtype=torch.float64))[:, None] * inv[None]
    zr = z * torch.polar(torch.ones_like(ang), ang)
    exp = torch.cat([zr.real, zr.imag], dim=-1)
    assert (y.double() - exp).abs().max() < 5e-6
    # norm of each pair is preserved
    n_in = x[..., 0::2] ** 2 + x[..., 1::2] ** 2
    n_out = y[..., : Dh // 2] ** 2 + y[..., Dh // 2:] ** 2
    assert torch.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)


def test_rope_zero_angle_is_pure_deinterleave():
    x = torch.randn(1, 2, 4, 16).to(torch.bfloat16)
    cos = torch.ones(1, 1, 4, 8)
    sin = torch.zeros(1, 1, 4, 8)
    y = ro.rope_apply(x, cos, sin)
    assert torch.equal(y, torch.cat([x[..., 0::2], x[..., 1::2]], dim=-1))
    assert y.dtype == torch.bfloat16


def test_rope_relative_position_property():
    """<rope(q,p), rope(k,p')> depends only on p - p' for a 1-D table."""
    torch.manual_seed(1)
    Dh = 64
    cos_t, sin_t = ro.rope_table_1d(64, Dh)
    q, k = torch.randn(Dh), torch.randn(Dh)

    def rot(x, p):
        return ro.rope_apply(x.view(1, 1, 1, Dh), cos_t[p].view(1, 1, 1, -1), sin_t[p].view(1, 1, 1, -1)).flatten()

    d0 = torch.dot(rot(q, 10), rot(k, 3))
    d1 = torch.dot(rot(q, 40), rot(k, 33))
    assert abs(d0 - d1) < 1e-4


def test_rope_angles_flat_index():
    cos_t = torch.arange(24, dtype=torch.float32).view(24, 1)
    pos = {"t_pos": torch.tensor([[1, 1, 1]]), "y_pos": torch.tensor([[0, 1, 2]]), "x_pos": torch.tensor([[1, 0, 1]])}
    cos, _ = ro.rope_angles(pos, cos_t, cos_t, 3, 2)       # flat = t*6 + y*2 + x
    assert cos.shape == (1, 1, 3, 1) and cos.flatten().tolist() == [7.0, 8.0, 11.0]


# ----------------------------------------------------------------------------------------
# attention: torch's own flex_attention (eager) with a BlockMask is the library yardstick
# ----------------------------------------------------------------------------------------
def _flex_with_block_mask(q, k_all, v_all, mask, T):
    """torch's eager flex_attention over the full-capacity cache with a block mask built from a
    per-key bool vector, i.e. the call the reference makes (src/model/attn.py:116) expressed with
    library routines only."""
    from torch.nn.attention.flex_attention import BlockMask, flex_attention, _DEFAULT_SPARSE_BLOCK_SIZE as BS
    cap = mask.numel()
    nkv, nq = (cap + BS - 1) // BS, (T + BS - 1) // BS
    blocks = torch.nn.functional.pad(mask, (0, nkv * BS - cap)).view(nkv, BS)
    any_b, all_b = blocks.any(-1), blocks.all(-1)

    def ordered(dense):
        dense = dense[None].expand(nq, nkv)
        num = dense.sum(-1, dtype=torch.int32)[None, None].contiguous()
        idx = dense.int().argsort(dim=-1, descending=True, stable=True).int()[None, None].contiguous()
        return num, idx

    pn, pi = ordered(any_b & ~all_b)
    fn, fi = ordered(all_b)
    bm = BlockMask.from_kv_blocks(pn, pi, fn, fi, BLOCK_SIZE=BS, mask_mod=lambda b, h, qi, ki: mask[ki],
                                  seq_lengths=(T, cap))
    return flex_attention(q, k_all, v_all, block_mask=bm, enable_gqa=q.shape[1] != k_all.shape[1])


def _run_steps(dtype, B, H, Hkv, T, Dh, n_slots, steps, cfg_id=0, d=1):
    W = int(math.isqrt(T))
    cfg = SimpleNamespace(tokens_per_frame=T, local_window=n_slots, global_window=n_slots,
                          global_attn_period=1, global_pinned_dilation=d, n_layers=1, n_heads=H,
                          n_kv_heads=Hkv, d_model=H * Dh)
    cache = ro.OracleStaticKVCache(cfg, B, dtype)
    cache.set_frozen(False)
    cos_t, sin_t = ro.rope_table_1d(steps * T, Dh)
    for s in range(steps):
        q, k, v = ro.synth_qkv(cfg_id, s, 0, B, H, Hkv, T, Dh, dtype)
        pos = ro.synth_pos_ids(s, B, T, W)
        cos, sin = ro.rope_angles(pos, cos_t, sin_t, T // W, W)
        q_rot, k_rot = ro.rope_apply(q, cos, sin), ro.rope_apply(k, cos, sin)
        k_all, v_all, mask = cache.upsert(k_rot, v, pos, 0)
        yield s, q_rot, k_all, v_all, mask


def test_cfg0_cpu_plumbing_fp32_against_flex_and_fp64():
    """Benchmark configuration 0: B=1,H=8,Dh=64,T=64, 4 slots, fp32, 8 steps (ring wraps twice)."""
    for s, q, k_all, v_all, mask in _run_steps(torch.float32, 1, 8, 8, 64, 64, 4, 8):
        assert int(mask.sum()) == min(s, 3) * 64 + 64
        ref_path = ro.attention_reference_path(q, k_all, v_all, mask)
        flex = _flex_with_block_mask(q, k_all, v_all, mask, 64)
        f64 = ro.attention_fp32(q, k_all, v_all, mask, dtype=torch.float64)
        f32 = ro.attention_fp32(q, k_all, v_all, mask)
        assert (ref_path - flex).abs().max() < 2e-6
        assert (ref_path.double() - f64).abs().max() < 1e-5
        assert (f32.double() - f64).abs().max() < 1e-5


def test_bf16_reference_path_matches_flex_and_is_near_fp32():
    for s, q, k_all, v_all, mask in _run_steps(torch.bfloat16, 1, 4, 2, 64, 64, 4, 6, cfg_id=7):
        ref_path = ro.attention_reference_path(q, k_all, v_all, mask)
        flex = _flex_with_block_mask(q, k_all, v_all, mask, 64)
        assert ref_path.dtype == torch.bfloat16
        assert (ref_path.float() - flex.float()).abs().max() <= 2 ** -6   # a bf16 ulp or two at |y|~1
        f32 = ro.attention_fp32(q, k_all, v_all, mask)
        assert (ref_path.float() - f32).abs().max() < 2e-2
        assert (ref_path.float() - f32).abs().mean() < 2e-3


def test_step0_is_unmasked_sdpa_over_the_tail():
    s, q, k_all, v_all, mask = next(_run_steps(torch.float32, 2, 4, 4, 16, 32, 4, 1))
    L = 4 * 16
    sdpa = torch.nn.functional.scaled_dot_product_attention(q, k_all[:, :, L:], v_all[:, :, L:])
    assert (ro.attention_fp32(q, k_all, v_all, mask) - sdpa).abs().max() < 2e-6
    assert (ro.attention_reference_path(q, k_all, v_all, mask) - sdpa).abs().max() < 2e-6


def test_attention_is_invariant_to_slot_order_and_to_hidden_garbage():
    steps = list(_run_steps(torch.float32, 1, 2, 2, 16, 32, 4, 7))
    s, q, k_all, v_all, mask = steps[-1]
    base = ro.attention_fp32(q, k_all, v_all, mask)
    # rotate the three visible ring slots among themselves: softmax is permutation invariant
    T = 16
    vis = [i for i in range(4) if mask[i * T]]
    perm = vis[1:] + vis[:1]
    k2, v2 = k_all.clone(), v_all.clone()
    for a, b in zip(vis, perm):
        k2[:, :, a * T:(a + 1) * T] = k_all[:, :, b * T:(b + 1) * T]
        v2[:, :, a * T:(a + 1) * T] = v_all[:, :, b * T:(b + 1) * T]
    assert (ro.attention_fp32(q, k2, v2, mask) - base).abs().max() < 2e-6
    # large finite values in the hidden slot change nothing
    hid = [i for i in range(4) if not mask[i * T]][0]
    k2, v2 = k_all.clone(), v_all.clone()
    k2[:, :, hid * T:(hid + 1) * T] = 1e4
    v2[:, :, hid * T:(hid + 1) * T] = -1e4
    assert torch.equal(ro.attention_fp32(q, k2, v2, mask), base)
    assert (ro.attention_reference_path(q, k2, v2, mask) - base).abs().max() < 2e-6


def test_gqa_matches_explicit_head_repeat():
    s, q, k_all, v_all, mask = list(_run_steps(torch.float32, 1, 4, 2, 16, 32, 2, 3))[-1]
    a = ro.attention_fp32(q, k_all, v_all, mask)
    b = ro.attention_fp32(q, k_all.repeat_interleave(2, 1), v_all.repeat_interleave(2, 1), mask)
    assert torch.equal(a, b)


def test_outlier_channel_softmax_is_stable():
    q, k, v = ro.synth_qkv(2, 0, 0, 1, 2, 2, 64, 128, torch.bfloat16, outlier=True)
    mask = torch.ones(64, dtype=torch.bool)
    out = ro.attention_fp32(q, k, v, mask)
    f64 = ro.attention_fp32(q, k, v, mask, dtype=torch.float64)
    assert torch.isfinite(out).all() and (out.double() - f64).abs().max() < 1e-4
    assert (k.float().abs().amax(dim=(0, 1, 2)) > 12).sum() == 1     # exactly one hot channel


def test_synth_inputs_are_reproducible():
    a = ro.synth_qkv(1, 5, 2, 1, 2, 2, 8, 16, torch.bfloat16)
    b = ro.synth_qkv(1, 5, 2, 1, 2, 2, 8, 16, torch.bfloat16)
    c = ro.synth_qkv(1, 5, 3, 1, 2, 2, 8, 16, torch.bfloat16)
    assert all(torch.equal(x, y) for x, y in zip(a, b)) and not torch.equal(a[0], c[0])
    pos = ro.synth_pos_ids(9, 2, 16, 4)
    assert pos["t_pos"].unique().tolist() == [9] and pos["y_pos"][0].tolist() == [i // 4 for i in range(16)]


# ------------------------------------------------------------------------------------------
# the module's element-wise steps around the path (src/model/attn.py:105-109,117-119)
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rms_norm_matches_torch_and_closed_cases(dtype):
    """The oracle's weightless RMS norm against F.rms_norm - the call the reference makes
    (src/model/nn.py:55-56) - bit for bit, and against what the formula fixes."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(2, 3, 17, 128, generator=g) * 3).to(dtype)
    got = ro.rms_norm(x)
    assert got.dtype == dtype and torch.equal(got, F.rms_norm(x, (128,)))
    # rows come out with unit root-mean-square (up to the rounding of the element type)
    rms = got.float().pow(2).mean(-1).sqrt()
    assert (rms - 1).abs().max().item() < {torch.bfloat16: 4e-3, torch.float16: 5e-4, torch.float32: 1e-6}[dtype]
    # without the epsilon, scaling a row by a power of two changes nothing at all; with it, nothing
    # beyond the last bit of a few elements (the epsilon is 1e-7 of a mean square near 9)
    base0 = ro.rms_norm(x, eps=0.0)
    assert torch.equal(ro.rms_norm(x * 4, eps=0.0), base0) and torch.equal(ro.rms_norm(x * 16, eps=0.0), base0)
    assert (ro.rms_norm(x * 4) != got).float().mean().item() < 0.01
    # a row of equal magnitudes normalises to +-1 exactly
    c = torch.full((1, 1, 1, 64), 3.0).to(dtype)
    c[..., ::2] = -3.0
    out = ro.rms_norm(c)
    assert torch.equal(out.abs(), torch.ones_like(out)) and torch.equal(out.sign(), c.sign())
    # an all-zero row stays zero (eps keeps the reciprocal root finite)
    assert torch.equal(ro.rms_norm(torch.zeros(1, 4, dtype=dtype)), torch.zeros(1, 4, dtype=dtype))
    # a dropped mean (sum instead of mean) or a missing square root would not survive this
    one = torch.zeros(1, 16, dtype=dtype)
    one[0, 5] = 2.0
    assert abs(ro.rms_norm(one)[0, 5].item() - 4.0) < 1e-5     # 2 / sqrt(4 / 16 + eps)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_value_lerp_matches_torch_and_end_points(dtype):
    g = torch.Generator().manual_seed(4)
    v = torch.randn(2, 3, 33, 64, generator=g).to(dtype)
    v1 = torch.randn(2, 3, 33, 64, generator=g).to(dtype)
    for w in (0.0, 0.25, 0.37, 0.5, 0.62, 1.0):
        wt = torch.tensor(w, dtype=dtype)
        got, want = ro.value_lerp(v, v1, wt), torch.lerp(v, v1, wt)
        if dtype == torch.float32:      # torch contracts a + w*d into a fused multiply-add in fp32
            assert (got - want).abs().max().item() <= 2.4e-7 * max(1.0, want.abs().max().item())
        else:
            assert torch.equal(got, want), f"w={w}"
    assert torch.equal(ro.value_lerp(v, v1, torch.tensor(0.0, dtype=dtype)), v)
    assert torch.equal(ro.value_lerp(v, v1, torch.tensor(1.0, dtype=dtype)), v1)
    assert torch.equal(ro.value_lerp(v, v, torch.tensor(0.37, dtype=dtype)), v)
    # direction: the weight moves the result towards v1, not away from it
    a, b = torch.tensor([1.0], dtype=dtype), torch.tensor([3.0], dtype=dtype)
    assert ro.value_lerp(a, b, torch.tensor(0.25, dtype=dtype)).item() == 1.5


def test_gate_output_layout_and_rounding():
    g = torch.Generator().manual_seed(5)
    y = torch.randn(2, 4, 8, 16, generator=g).to(torch.bfloat16)          # [B, H, T, Dh]
    gates = torch.rand(2, 8, 4, generator=g).to(torch.bfloat16)           # [B, T, H]
    got = ro.gate_output(y, gates)
    for b in range(2):
        for h in range(4):
            for t in range(8):
                want = (y[b, h, t].float() * gates[b, t, h].float()).to(torch.bfloat16)
                assert torch.equal(got[b, h, t], want)
    assert torch.equal(ro.gate_output(y, torch.ones(2, 8, 4, dtype=torch.bfloat16)), y)
    assert not ro.gate_output(y, torch.zeros(2, 8, 4, dtype=torch.bfloat16)).any()


def test_layer_step_with_module_steps_equals_their_composition():
    """layer_step with norm / lerp / gate switched on is exactly: torch's own lerp and rms_norm in
    front of, and the tensor multiply behind, the plain layer_step (src/model/attn.py:105-119)."""
    import torch.nn.functional as F
    from types import SimpleNamespace
    B, H, Hkv, T, Dh, n = 1, 4, 2, 16, 32, 2
    cfg = SimpleNamespace(tokens_per_frame=T, local_window=n, global_window=n, global_attn_period=1,
                          global_pinned_dilation=1, n_layers=1, n_heads=H, n_kv_heads=Hkv, d_model=H * Dh)
    a, b = ro.OracleStaticKVCache(cfg, B, torch.bfloat16), ro.OracleStaticKVCache(cfg, B, torch.bfloat16)
    a.set_frozen(False), b.set_frozen(False)
    cos, sin = ro.rope_table_1d(8 * T, Dh)
    g = torch.Generator().manual_seed(6)
    lamb = torch.tensor(0.3, dtype=torch.bfloat16)
    for t in range(4):
        q, k, v = ro.synth_qkv(7, t, 0, B, H, Hkv, T, Dh, torch.bfloat16)
        v1 = torch.randn(v.shape, generator=g).to(torch.bfloat16)
        gates = torch.sigmoid(torch.randn(B, T, H, generator=g)).to(torch.bfloat16)
        pos = ro.synth_pos_ids(t, B, T, 4)
        out_a, qa = ro.layer_step(a, 0, q, k, v, pos, cos, sin, 4, 4, qk_norm=True, v1=v1, v_lamb=lamb, gates=gates)
        out_b, qb = ro.layer_step(b, 0, F.rms_norm(q, (Dh,)), F.rms_norm(k, (Dh,)), torch.lerp(v, v1, lamb), pos,
                                  cos, sin, 4, 4)
        out_b = out_b * gates.permute(0, 2, 1).unsqueeze(-1)
        assert torch.equal(qa, qb) and torch.equal(out_a, out_b)
        assert torch.equal(a.layers[0].kv, b.layers[0].kv) and torch.equal(a.layers[0].written, b.layers[0].written)


# ----------------------------------------------------------------------------------------
# the merged q/k/v projection in front of the path
# ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_qkv_project_exact_integer_case_and_layout(dtype):
    """On dyadic operands the projection is integer arithmetic: the oracle must equal the int64
    matrix product scaled by 1/64 and rounded once to the element type, and its q / k / v must be
    the reference's views (src/patch_model.py:116-122) of that matrix - checked element by element
    for the head / token / channel each output came from."""
    B, T, d_model, H, Hkv, Dh = 2, 5, 96, 3, 1, 16
    feats = (H + 2 * Hkv) * Dh
    x, w = ro.synth_dyadic_linear(11, B, T, d_model, feats, dtype)
    xi, wi = (x.double() * 8).long(), (w.double() * 8).long()
    y = (torch.einsum("btk,nk->btn", xi, wi).double() / 64).to(dtype)          # exact, then one rounding
    q, k, v = ro.qkv_project(x, w, H, Hkv)
    assert q.shape == (B, H, T, Dh) and k.shape == (B, Hkv, T, Dh) and v.shape == (B, Hkv, T, Dh)
    for b in range(B):
        for t in range(T):
            for h in range(H):
                assert torch.equal(q[b, h, t], y[b, t, h * Dh:(h + 1) * Dh])
            for h in range(Hkv):
                assert torch.equal(k[b, h, t], y[b, t, (H + h) * Dh:(H + h + 1) * Dh])
                assert torch.equal(v[b, h, t], y[b, t, (H + Hkv + h) * Dh:(H + Hkv + h + 1) * Dh])


def test_qkv_project_matches_torch_linear_and_fp64():
    """Against the call the reference makes (F.linear on element-type tensors, then split) and
    against fp64 sums rounded once: identical on dyadic operands, within one unit in the last
    place on random ones (the BLAS routine's summation order is not the oracle's)."""
    import torch.nn.functional as F
    B, T, d_model, H, Hkv, Dh = 1, 12, 256, 2, 2, 32
    feats = (H + 2 * Hkv) * Dh
    x, w = ro.synth_dyadic_linear(12, B, T, d_model, feats, torch.bfloat16)
    q, k, v = ro.qkv_project(x, w, H, Hkv)
    ql, kl, vl = F.linear(x, w).split((H * Dh, Hkv * Dh, Hkv * Dh), dim=-1)
    assert torch.equal(q, ql.reshape(B, T, H, Dh).transpose(1, 2))
    assert torch.equal(k, kl.reshape(B, T, Hkv, Dh).transpose(1, 2))
    assert torch.equal(v, vl.reshape(B, T, Hkv, Dh).transpose(1, 2))
    g = torch.Generator().manual_seed(13)
    x = torch.randn(B, T, d_model, generator=g).to(torch.bfloat16)
    w = (torch.randn(feats, d_model, generator=g) / 16).to(torch.bfloat16)
    got = torch.cat([t_.transpose(1, 2).reshape(B, T, -1) for t_ in ro.qkv_project(x, w, H, Hkv)], dim=-1)
    want64 = x.double() @ w.double().t()
    ulp = 2.0 ** (torch.floor(torch.log2(want64.abs().clamp_min(1e-30))) - 7)       # bf16: 8 significant bits
    assert ((got.double() - want64).abs() <= 0.5 * ulp + 1e-6 * want64.abs()).all()
    lin = F.linear(x, w)
    assert ((got.double() - lin.double()).abs() <= ulp).all()
