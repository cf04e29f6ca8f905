"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on identical seeded inputs.

Bars: ring-buffer contents, ``written`` and RoPE outputs bit-exact; attention output within
max-abs 2e-2 / mean-abs 2e-3 of the fp32 oracle on bf16 inputs.
"""
import math

import pytest
import torch

from oracle import ring_oracle as ro
from _harness import Pair, assert_attn_close, assert_bits_equal, assert_margin, merged_views, to_dev, MAX_ABS, MEAN_ABS
import world_engine_amd as wea
from world_engine_amd import _capi, ops

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------------------------------
# RoPE + ring store: bit-exact
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("d", [1, 2, 4])
@pytest.mark.parametrize("hkv", [4, 2])
def test_store_bit_exact_over_wraps(gpu_device, dtype, d, hkv):
    _say(f"store dtype={dtype} d={d} hkv={hkv}")
    n = 4 * d if d > 1 else 4
    p = Pair(gpu_device, dtype, B=2, H=4, Hkv=hkv, T=64, Dh=64, n_slots=n, d=d, cfg_id=11)
    for t in range(3 * n + 2):
        for sub, frozen in ((0, True), (1, True), (2, False)):
            p.set_frozen(frozen)
            q, k, v, pos = p.inputs(t, sub)
            (q_o, _, _, mask), (q_h, ring) = p.store(q, k, v, pos, strided=(t % 2 == 0))
            assert_bits_equal(q_h, q_o, f"RoPE(q) t={t} sub={sub}")
            p.assert_state_equal(what=f"t={t} sub={sub} frozen={frozen}")
            assert torch.equal(ring.dense().cpu(), mask), f"mask t={t} sub={sub}"


def test_store_cfg1_shape_bit_exact(gpu_device):
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, cfg_id=1)
    p.set_frozen(False)
    for t in (0, 1, 15, 16, 17, 40):
        q, k, v, pos = p.inputs(t)
        (q_o, *_), (q_h, _) = p.store(q, k, v, pos)
        assert_bits_equal(q_h, q_o, f"RoPE(q) t={t}")
        p.assert_state_equal(what=f"t={t}")


def test_reference_signature_upsert_without_rope(gpu_device):
    """StaticKVCache.upsert(k, v, pos_ids, layer) / LayerKVCache.upsert(kv, pos_ids, frozen) with
    an already rotated k, as the reference's own attention module would call them."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=2, Hkv=2, T=64, Dh=128, n_slots=3, n_layers=2, cfg_id=12)
    p.set_frozen(False)
    for t in range(8):
        q, k, v, pos = p.inputs(t)
        p.oracle.upsert(k, v, pos, 1)
        k_all, v_all, ring = p.hip.upsert(k.to(gpu_device), v.to(gpu_device), to_dev(pos, gpu_device), 1)
        assert k_all.shape == (1, 2, 4 * 64, 128) and k_all.data_ptr() == p.hip.layers[1].kv[0].data_ptr()
        p.assert_state_equal(layer=1, what=f"t={t}")
        # layer API with the stacked tensor
        p.oracle.layers[0].upsert(torch.stack([k, v]), pos, t % 2 == 0)
        p.hip.layers[0].upsert(torch.stack([k, v]).to(gpu_device), to_dev(pos, gpu_device), t % 2 == 0)
        p.assert_state_equal(layer=0, what=f"layer api t={t}")
    p.hip.reset()
    p.oracle.reset()
    p.assert_state_equal(layer=0, what="after reset")
    assert p.hip._is_frozen


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_standalone_rope_bit_exact(gpu_device, dtype):
    p = Pair(gpu_device, dtype, B=2, H=3, Hkv=3, T=64, Dh=128, n_slots=2, cfg_id=13)
    q, k, v, pos = p.inputs(5)
    cos, sin = ro.rope_angles(pos, p.cos, p.sin, p.Hgrid, p.W)
    got = p.rope(merged_views(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device))[0], to_dev(pos, gpu_device))
    assert_bits_equal(got, ro.rope_apply(q, cos, sin), "stand-alone RoPE")


def test_rope_special_values_round_like_torch(gpu_device):
    """NaN, infinities, denormals and ties go through the same fp32 -> bf16 rounding as torch."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=1, Hkv=1, T=64, Dh=64, n_slots=2, cfg_id=14)
    q, k, v, pos = p.inputs(1)
    k[0, 0, 0, :8] = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -0.0, 1e-40, 3.3895e38, -1e-38])
    (q_o, *_), (q_h, _) = p.store(q, k, v, pos)
    p.assert_state_equal(what="special values")


# ------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------
def _run_and_check(p, steps, frozen_subs=0, check_steps=None, outlier=False, layer=0, **attn_kw):
    worst = (0.0, 0.0)
    for t in range(steps):
        for sub in range(frozen_subs + 1):
            frozen = sub < frozen_subs
            p.set_frozen(frozen)
            q, k, v, pos = p.inputs(t, sub, outlier)
            (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos, layer=layer)
            out = p.attend(q_h, ring, **attn_kw)
            p.assert_state_equal(layer=layer, what=f"t={t} sub={sub}")
            if check_steps is None or t in check_steps:
                ref = ro.attention_fp32(q_o, k_all, v_all, mask)
                mx, mean = assert_attn_close(out, ref, f"t={t} sub={sub} kw={attn_kw}")
                worst = (max(worst[0], mx), max(worst[1], mean))
    return worst


def test_attention_cfg0_shapes_bf16(gpu_device):
    """Benchmark configuration 0 geometry (B=1,H=8,Dh=64,T=64, 4 slots, 8 steps) in bf16 on the GPU."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=8, Hkv=8, T=64, Dh=64, n_slots=4, cfg_id=0)
    worst = _run_and_check(p, 8)
    _say(f"cfg0 shapes: worst max-abs {worst[0]:.2e} mean-abs {worst[1]:.2e}")


def test_attention_cfg0_fp32(gpu_device):
    """Benchmark configuration 0 as stated (fp32, B=1, H=8, Dh=64, 64-token frames, 4 slots, 8 steps, the
    ring wraps twice) through the fp32 kernel: fp32 arithmetic throughout, so the bar is 1e-5."""
    p = Pair(gpu_device, torch.float32, B=1, H=8, Hkv=8, T=64, Dh=64, n_slots=4, cfg_id=0)
    p.set_frozen(False)
    for t in range(8):
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        out = p.attend(q_h, ring)
        p.assert_state_equal(what=f"t={t}")
        ref = ro.attention_reference_path(q_o, k_all, v_all, mask)     # fp32 inputs: the reference's own flow
        diff = (out.cpu() - ref).abs()
        assert diff.max().item() <= 1e-5, f"t={t}: max-abs {diff.max().item():.2e}"
        assert out.transpose(1, 2).is_contiguous()


@pytest.mark.parametrize("Dh,hkv,T", [(128, 2, 128), (64, 4, 192)])
def test_attention_fp32_other_shapes(gpu_device, Dh, hkv, T):
    """fp32 kernel with grouped heads, both head dims, several query tiles and a dilated ring."""
    p = Pair(gpu_device, torch.float32, B=2, H=4, Hkv=hkv, T=T, Dh=Dh, n_slots=4, d=2, cfg_id=41)
    for t in range(7):
        p.set_frozen(t % 3 == 2)
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        out = p.attend(q_h, ring)
        ref = ro.attention_fp32(q_o, k_all, v_all, mask)
        assert (out.cpu() - ref).abs().max().item() <= 1e-5, f"t={t}"


def test_attention_cfg1_all_32_steps(gpu_device):
    """Benchmark configuration 1: B=1,H=16,Dh=128,T=256, 16 slots, 32 steps (warm-up + steady wrap)."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, cfg_id=1)
    worst = _run_and_check(p, 32)
    assert_margin("cfg1", worst)


@pytest.mark.parametrize("n_splits", [1, 2, 3, 7, 16])
@pytest.mark.parametrize("q_tile", [128, 256])
def test_attention_split_and_tile_variants(gpu_device, n_splits, q_tile):
    _say(f"variants n_splits={n_splits} q_tile={q_tile}")
    p = Pair(gpu_device, torch.bfloat16, B=2, H=4, Hkv=2, T=128, Dh=128, n_slots=6, cfg_id=21)
    _run_and_check(p, 9, n_splits=n_splits, q_tile=q_tile)


@pytest.mark.parametrize("dtype,Dh,T", [(torch.float16, 128, 64), (torch.float16, 64, 128),
                                        (torch.bfloat16, 64, 192), (torch.bfloat16, 128, 320)])
def test_attention_dtypes_head_dims_and_ragged_tiles(gpu_device, dtype, Dh, T):
    """T values that are not a multiple of the query tile exercise the partial last tile."""
    _say(f"dtype={dtype} Dh={Dh} T={T}")
    p = Pair(gpu_device, dtype, B=1, H=6, Hkv=3, T=T, Dh=Dh, n_slots=3, cfg_id=22)
    for kw in ({}, {"n_splits": 2, "q_tile": 128}, {"n_splits": 1, "q_tile": 128}, {"n_splits": 1, "q_tile": 256},
               {"n_splits": 3, "q_tile": 256}):
        p.hip.reset()
        p.oracle.reset()
        _run_and_check(p, 5, **kw)


@pytest.mark.parametrize("T,Dh,kw", [(80, 128, {}), (96, 64, {}), (40, 128, {}), (200, 128, {"n_splits": 3}),
                                     (330, 64, {"q_tile": 256, "n_splits": 2}), (24, 128, {"n_splits": 1}),
                                     (136, 128, {"q_tile": 256})])
def test_attention_frame_lengths_off_the_tile_grid(gpu_device, T, Dh, kw):
    """Frame lengths that are not multiples of the 64-key tile (or of 32, or below one block):
    the last tile of every slot is short, its missing keys must not count and the rows behind it
    (the next slot's frame, or the end of the buffer for the tail) must not be read as keys."""
    _say(f"ragged T={T} Dh={Dh} {kw}")
    p = Pair(gpu_device, torch.bfloat16, B=2, H=2, Hkv=1, T=T, Dh=Dh, n_slots=3, cfg_id=51)
    _run_and_check(p, 8, frozen_subs=1, **kw)


@pytest.mark.parametrize("T,n_slots,kw", [(8, 3, {}), (24, 2, {"n_splits": 2}), (96, 3, {"n_splits": 4}),
                                          (96, 3, {"n_splits": 1, "q_tile": 128}), (64, 3, {"n_splits": 2}),
                                          (256, 4, {})])
def test_attention_all_logits_far_below_zero(gpu_device, T, n_slots, kw):
    """Every logit is near -290 in the log2 domain (one channel of q and k carries +48 / -48): a
    softmax only sees differences, so the result is an ordinary one, but any reference exponent
    that is not taken from the data (a wavefront that starts on an empty 32-key block of a short
    tile, a split without keys) would make every probability underflow to zero.  With 96-token
    frames and 4 splits two of the splits start on the short second tile of a slot."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=2, Hkv=2, T=T, Dh=128, n_slots=n_slots, cfg_id=27)
    p.set_frozen(False)
    for t in range(n_slots + 2):
        q, k, v, pos = p.inputs(t)
        q[..., 126] = 48.0
        k[..., 126] = -48.0
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        out = p.attend(q_h, ring, **kw)
        p.assert_state_equal(what=f"t={t}")
        ref = ro.attention_fp32(q_o, k_all, v_all, mask)
        s = (q_o.float() @ k_all.float().transpose(-1, -2))[..., mask] * (128 ** -0.5) * 1.4427
        assert s.max().item() < -200.0
        assert ref.abs().max().item() > 0.1
        assert_attn_close(out, ref, f"T={T} t={t} {kw}")


def test_attention_fp32_ragged_frame(gpu_device):
    p = Pair(gpu_device, torch.float32, B=1, H=2, Hkv=2, T=72, Dh=64, n_slots=3, cfg_id=52)
    for t in range(7):
        p.set_frozen(False)
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        assert (p.attend(q_h, ring).cpu() - ro.attention_fp32(q_o, k_all, v_all, mask)).abs().max().item() <= 1e-5


@pytest.mark.parametrize("n_slots,T,Dh,kw", [(80, 64, 64, {"n_splits": 1}), (130, 64, 128, {}),
                                             (70, 96, 64, {"n_splits": 2, "q_tile": 256})])
def test_attention_rings_longer_than_one_wavefront(gpu_device, n_slots, T, Dh, kw):
    """More ring slots than a wavefront has lanes, and more tiles per workgroup than one batch of
    precomputed tile offsets holds: the slot list spans several rounds and the offsets are
    reloaded inside the tile loop.  Runs until the ring has wrapped."""
    _say(f"long ring n_slots={n_slots} T={T} Dh={Dh} {kw}")
    p = Pair(gpu_device, torch.bfloat16, B=1, H=2, Hkv=1, T=T, Dh=Dh, n_slots=n_slots, cfg_id=53,
             table_rows=(n_slots + 12) * T)
    steps = n_slots + 8
    _run_and_check(p, steps, check_steps={0, 1, 63, 64, 65, 66, n_slots - 1, n_slots, n_slots + 1, steps - 1}, **kw)


def test_attention_partial_round_tail_split(gpu_device):
    """320 workgroups = one full round of 256 CUs plus a quarter round: the library splits the
    context of the last 64 heads only (mixed direct-output and workspace rows in one call).  With
    160 heads the same frame is one round of 160 256-query workgroups and nothing is split."""
    assert ops.attn_auto_splits(1, 160, 160, 256, 64, 512) == 1
    assert ops.attn_workspace_bytes(1, 160, 160, 256, 64, 512) == 0
    assert ops.attn_auto_splits(1, 320, 320, 256, 64, 512) == 2
    assert ops.attn_workspace_bytes(1, 320, 320, 256, 64, 512) == 2 * 64 * 256 * (64 * 2 + 16)
    p = Pair(gpu_device, torch.bfloat16, B=1, H=320, Hkv=320, T=256, Dh=64, n_slots=2, cfg_id=27)
    _run_and_check(p, 4)
    p = Pair(gpu_device, torch.bfloat16, B=1, H=160, Hkv=160, T=256, Dh=64, n_slots=2, cfg_id=27)
    _run_and_check(p, 3)


@pytest.mark.parametrize("d", [2, 4])
def test_attention_with_pinned_dilation(gpu_device, d):
    p = Pair(gpu_device, torch.bfloat16, B=1, H=2, Hkv=2, T=64, Dh=128, n_slots=4 * d, d=d, cfg_id=23)
    _run_and_check(p, 4 * d * 2 + 3, frozen_subs=1)


def test_attention_cfg2_outlier_channel_three_layers(gpu_device):
    """Benchmark configuration 2 semantics (each layer its own ring, K with one x8 channel) on 3 layers."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, n_layers=3, cfg_id=2)
    p.set_frozen(False)
    for t in (0, 1, 2, 17):
        for layer in range(3):
            q, k, v, pos = ro.synth_qkv(2, t, layer, 1, 16, 16, 256, 128, torch.bfloat16, outlier=True) + (ro.synth_pos_ids(t, 1, 256, 16),)
            (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos, layer=layer)
            out = p.attend(q_h, ring)
            p.assert_state_equal(layer=layer, what=f"t={t} layer={layer}")
            assert_attn_close(out, ro.attention_fp32(q_o, k_all, v_all, mask), f"cfg2 t={t} layer={layer}")


def test_attention_cfg2_full_depth_24_layers(gpu_device):
    """Benchmark configuration 2 at full depth: 24 layers, each with its own 16-slot ring (856 MB in
    all), one K channel x8, 19 frames (the ring wraps after 16).  Cache buffers and `written` of
    all 24 layers are compared bit for bit after every frame; the attention of four layers per
    frame (rotating, so every layer is covered) against the fp32 oracle."""
    L_ = 24
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, n_layers=L_, cfg_id=2)
    p.set_frozen(False)
    worst = (0.0, 0.0)
    for t in range(19):
        _say(f"cfg2 full depth: frame {t}")
        pos = ro.synth_pos_ids(t, 1, 256, 16)
        checked = {(4 * t + i) % L_ for i in range(4)}
        for layer in range(L_):
            q, k, v = ro.synth_qkv(2, t, layer, 1, 16, 16, 256, 128, torch.bfloat16, outlier=True)
            (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos, layer=layer)
            out = p.attend(q_h, ring)
            if layer in checked:
                mx, mean = assert_attn_close(out, ro.attention_fp32(q_o, k_all, v_all, mask), f"cfg2 t={t} layer={layer}")
                worst = (max(worst[0], mx), max(worst[1], mean))
        for layer in range(L_):
            p.assert_state_equal(layer=layer, what=f"t={t} layer={layer}")
    assert_margin("cfg2", worst)


def test_attention_cfg4_frozen_substeps_schedule(gpu_device):
    """Benchmark configuration 4: 32 slots, 4 frozen substeps re-attending the same ring + 1 persisting
    call per frame.  State is compared after every call; outputs on the first frames and around
    the wrap."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=32, cfg_id=4)
    assert_margin("cfg4", _run_and_check(p, 35, frozen_subs=4, check_steps={0, 1, 31, 32, 34}))


def test_attention_cfg3_full_size(gpu_device):
    """Benchmark configuration 3 at full size (B=4,H=24,T=1024, 8 slots): oracle on three steps, plus
    size-independent properties on the steady state."""
    p = Pair(gpu_device, torch.bfloat16, B=4, H=24, Hkv=24, T=1024, Dh=128, n_slots=8, cfg_id=3)
    assert_margin("cfg3", _run_and_check(p, 10, check_steps={0, 9}))
    # steady state: permuting the visible slots' contents must not change the result
    q, k, v, pos = p.inputs(10)
    p.set_frozen(True)
    (_, _, _, mask), (q_h, ring) = p.store(q, k, v, pos)
    base = p.attend(q_h, ring).clone()
    kv = p.hip.layers[0].kv
    T = 1024
    vis = [s for s in range(8) if mask[s * T]]
    assert len(vis) == 7
    rolled = kv.clone()
    for a, b in zip(vis, vis[1:] + vis[:1]):
        rolled[:, :, :, a * T:(a + 1) * T] = kv[:, :, :, b * T:(b + 1) * T]
    out2 = ops.attn_ring(q_h, rolled, ring.written, ring.t_pos, ring.L, ring.dilation)
    d = (out2.float() - base.float()).abs()
    assert d.max().item() <= 1e-2 and d.mean().item() <= 1e-3
    # the hidden slot's contents are irrelevant (large finite garbage)
    hid = [s for s in range(8) if not mask[s * T]][0]
    rolled.copy_(kv)
    rolled[:, :, :, hid * T:(hid + 1) * T] = 3e4
    out3 = ops.attn_ring(q_h, rolled, ring.written, ring.t_pos, ring.L, ring.dilation)
    assert torch.equal(out3, base)
    # split count does not matter beyond rounding
    out4 = p.attend(q_h, ring, n_splits=3)
    d = (out4.float() - base.float()).abs()
    assert d.max().item() <= 1e-2 and d.mean().item() <= 1e-3


def test_output_layout_and_out_argument(gpu_device):
    p = Pair(gpu_device, torch.bfloat16, B=2, H=2, Hkv=2, T=64, Dh=64, n_slots=2, cfg_id=24)
    p.set_frozen(False)
    q, k, v, pos = p.inputs(0)
    (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
    a = p.attend(q_h, ring)
    assert a.shape == (2, 2, 64, 64) and a.transpose(1, 2).is_contiguous()
    b = p.attend(q_h, ring, token_major_out=False)
    assert b.is_contiguous() and torch.equal(a, b)
    out = torch.empty_like(b)
    c = p.attend(q_h, ring, out=out)
    assert c.data_ptr() == out.data_ptr() and torch.equal(out, b)


@pytest.mark.parametrize("T,Dh", [(256, 128), (72, 64)])
def test_query_rows_far_apart_take_the_register_path(gpu_device, T, Dh):
    """128-query workgroups fetch their Q tile by DMA with 32-bit row offsets; a q whose rows lie
    more than 2 GiB / T apart (here: a view into a 2.1 GB buffer) has its fragments loaded lane by
    lane instead.  Same values, same arithmetic: the outputs must be bit-identical."""
    _say(f"far-apart query rows T={T} Dh={Dh}")
    H = 2
    p = Pair(gpu_device, torch.bfloat16, B=1, H=H, Hkv=1, T=T, Dh=Dh, n_slots=3, cfg_id=27)
    row = (1 << 31) // (2 * T) + 64                  # elements between two tokens' rows
    far = torch.empty(T, row, dtype=torch.bfloat16, device=gpu_device)
    for t in range(4):
        p.set_frozen(t == 2)
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
        far[:, : H * Dh] = q_h.transpose(1, 2).reshape(T, H * Dh)
        q_far = far[:, : H * Dh].view(1, T, H, Dh).transpose(1, 2)
        assert q_far.stride(2) * T * 2 >= 1 << 31
        for kw in ({"q_tile": 128}, {"q_tile": 128, "n_splits": 2}):
            a = p.attend(q_h, ring, **kw)
            b = p.attend(q_far, ring, **kw)
            assert torch.equal(a, b), (t, kw)
        assert_attn_close(a, ro.attention_fp32(q_o, k_all, v_all, mask), f"t={t}")


def test_stream_probe_runs_and_validates(gpu_device):
    """The tile-stream measurement aid: launches on a buffer that covers its regions, refuses one
    that does not, and writes nothing."""
    _say("stream probe")
    buf = torch.full((96 * 23 * 16384,), 7, dtype=torch.uint8, device=gpu_device)
    ops.stream_probe(buf, 192, 23, 2)
    ops.stream_probe(buf, 8, 1, 1)
    torch.cuda.synchronize()
    assert bool((buf == 7).all())
    with pytest.raises(RuntimeError, match="we_stream_probe"):
        ops.stream_probe(buf, 192, 23, 1)            # 192 regions do not fit
    with pytest.raises(RuntimeError, match="we_stream_probe"):
        ops.stream_probe(buf, 100, 23, 2)            # not a multiple of 8 workgroups
    with pytest.raises(RuntimeError, match="we_stream_probe"):
        ops.stream_probe(buf, 192, 0, 2)


def test_clocked_entry_point_same_output_and_plausible_clocks(gpu_device):
    """``we_attn_ring_fwd_clocked`` is ``we_attn_ring_fwd`` plus two counters per workgroup: the
    output has the same bits, every workgroup reports a duration, and cycles per 100 MHz tick is a
    shader frequency the part can run at."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=4, Hkv=2, T=128, Dh=128, n_slots=4, cfg_id=27)
    p.set_frozen(False)
    for t in range(5):
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
    plain = p.attend(q_h, ring, n_splits=2)
    assert_attn_close(plain, ro.attention_fp32(q_o, k_all, v_all, mask), "plain")
    clocks = torch.zeros(_capi.WE_CLOCK_SLOTS * 1024, dtype=torch.int64, device=gpu_device)
    timed = p.attend(q_h, ring, n_splits=2, clocks=clocks)
    assert_bits_equal(timed, plain, "clocked output")
    rec = clocks.view(-1, _capi.WE_CLOCK_SLOTS).cpu()
    c = rec[:, :2]
    c = c[c[:, 0] != 0]
    _say(f"clocked: {c.shape[0]} workgroups, cycles {c[:4, 0].tolist()} ticks {c[:4, 1].tolist()}")
    # 1 query tile x 2 query heads per kv head x (2 kv heads x 2 context parts); grid slots past
    # the last part leave early and report nothing
    assert c.shape[0] == 1 * 2 * (2 * 2), "one report per working workgroup"
    assert torch.all(c[:, 1] > 0)
    ghz = (c[:, 0].double() / c[:, 1].double()).median().item() * 0.1
    assert 0.3 < ghz < 3.0, f"implausible shader clock {ghz} GHz"
    with pytest.raises(RuntimeError, match="we_attn_ring_fwd_clocked"):
        p.attend(q_h, ring, n_splits=2, clocks=clocks[:2])
    with pytest.raises(RuntimeError, match="int64"):
        p.attend(q_h, ring, n_splits=2, clocks=clocks.to(torch.int32))


# ------------------------------------------------------------------------------------------
# module-level drop-in and graph capture
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("fuse", ["none", "elementwise", "projection"])
def test_ring_attn_module_matches_cpu_composition(gpu_device, fuse):
    """RingAttn.forward (merged QKV, GQA, value residual, head gate) against the same sequence
    composed on the CPU from torch linears, F.rms_norm and the oracle - with the module's torch
    operations around the library call, with the element-wise ones inside the kernels, and with
    the q/k/v projection inside the store kernel as well."""
    import torch.nn.functional as F
    from types import SimpleNamespace
    torch.manual_seed(5)
    T, H, Hkv, Dh, n = 64, 4, 2, 64, 3
    cfg = SimpleNamespace(tokens_per_frame=T, local_window=n, global_window=n, global_attn_period=1,
                          global_pinned_dilation=1, n_layers=1, n_heads=H, n_kv_heads=Hkv, d_model=H * Dh,
                          value_residual=True, gated_attn=True)
    cos, sin = ro.rope_table_1d(16 * T, Dh)
    rope = wea.RoPE(cos, sin, 8, 8)
    mod = wea.RingAttn(cfg, 0, rope, merged_qkv=True, fuse_elementwise=fuse != "none",
                       fuse_projection=fuse == "projection")
    with torch.no_grad():
        mod.gate_proj.weight.normal_(0, 0.5)
    mod = mod.to(torch.bfloat16)
    cpu_sd = {k: v.clone() for k, v in mod.state_dict().items()}
    mod = mod.to(gpu_device)
    cache = wea.StaticKVCache(cfg, 1, torch.bfloat16).to(gpu_device)
    ocache = ro.OracleStaticKVCache(cfg, 1, torch.bfloat16)
    v1_h = v1_o = None
    for t in range(5):
        frozen = t % 2 == 1
        cache.set_frozen(frozen)
        ocache.set_frozen(frozen)
        x = torch.randn(1, T, H * Dh).to(torch.bfloat16)
        pos = ro.synth_pos_ids(t, 1, T, 8)
        y_h, v1_h = mod(x.to(gpu_device), to_dev(pos, gpu_device), v1_h, cache)
        # CPU composition
        qkv = F.linear(x, cpu_sd["qkv_proj.weight"])
        q, k, v = qkv.split((H * Dh, Hkv * Dh, Hkv * Dh), dim=-1)
        q = q.reshape(1, T, H, Dh).transpose(1, 2)
        k = k.reshape(1, T, Hkv, Dh).transpose(1, 2)
        v = v.reshape(1, T, Hkv, Dh).transpose(1, 2)
        v1_o = v if v1_o is None else v1_o
        v = torch.lerp(v, v1_o.view_as(v), cpu_sd["v_lamb"])
        q, k = F.rms_norm(q, (Dh,)), F.rms_norm(k, (Dh,))
        y, _ = ro.layer_step(ocache, 0, q, k, v, pos, cos, sin, 8, 8)
        gates = torch.sigmoid(F.linear(x[..., :H], cpu_sd["gate_proj.weight"]))
        y = y * gates.permute(0, 2, 1).unsqueeze(-1)
        y_o = F.linear(y.transpose(1, 2).reshape(1, T, -1), cpu_sd["out_proj.weight"])
        d = (y_h.float().cpu() - y_o.float()).abs()
        assert d.max().item() < 3e-2 and d.mean().item() < 3e-3, (t, d.max().item(), d.mean().item())
        assert torch.equal(cache.layers[0].written.cpu(), ocache.layers[0].written)


def test_calls_from_a_worker_thread(gpu_device):
    """The reference generates frames from a worker thread (asyncio.to_thread(engine.gen_frame, ...),
    examples/simple_client.py:23-25) and from its own stream.  The library launches on the calling
    thread's current stream and keeps no per-thread state: frames stepped alternately by the main
    thread and by a worker thread on a side stream must leave the same cache state and outputs as
    the oracle."""
    import threading
    p = Pair(gpu_device, torch.bfloat16, B=1, H=4, Hkv=2, T=128, Dh=128, n_slots=3, cfg_id=28)
    p.set_frozen(False)
    side = torch.cuda.Stream(device=gpu_device)
    results, errors = {}, []

    def one_frame(t, use_side):
        try:
            q, k, v, pos = p.inputs(t)
            if use_side:
                side.wait_stream(torch.cuda.default_stream(gpu_device))
                with torch.cuda.stream(side):
                    (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
                    out = p.attend(q_h, ring)
                side.synchronize()
            else:
                (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
                out = p.attend(q_h, ring)
                torch.cuda.synchronize()
            results[t] = (out, ro.attention_fp32(q_o, k_all, v_all, mask))
        except Exception as e:          # noqa: BLE001 - re-raised in the main thread
            errors.append((t, e))

    for t in range(6):
        _say(f"worker thread frame {t}")
        if t % 2:
            th = threading.Thread(target=one_frame, args=(t, True))
            th.start()
            th.join()
        else:
            one_frame(t, False)
        assert not errors, errors
        p.assert_state_equal(what=f"t={t}")
        assert_attn_close(*results[t], f"t={t}")


def test_hip_graph_replay_matches_eager(gpu_device):
    """One frame step (store + attention) captured in a HIP graph and replayed for successive
    frames by updating only device tensors; every replay must equal the eager result."""
    p = Pair(gpu_device, torch.bfloat16, B=1, H=4, Hkv=4, T=128, Dh=128, n_slots=4, cfg_id=25)
    p.set_frozen(False)
    eager = Pair(gpu_device, torch.bfloat16, B=1, H=4, Hkv=4, T=128, Dh=128, n_slots=4, cfg_id=25)
    eager.set_frozen(False)
    dev = gpu_device
    qs, ks, vs = (torch.empty(1, 4, 128, 128, dtype=torch.bfloat16, device=dev) for _ in range(3))
    pos_s = to_dev(ro.synth_pos_ids(0, 1, 128, p.W), dev)
    layer = p.hip.layers[0]
    out_s = torch.empty(1, 4, 128, 128, dtype=torch.bfloat16, device=dev)
    n_splits = 2
    ws = torch.empty(ops.attn_workspace_bytes(1, 4, 4, 128, 128, layer.L, n_splits), dtype=torch.uint8, device=dev)

    def step():
        q_rot = ops.rope_kv_store(qs, ks, vs, pos_s, p.rope.cos, p.rope.sin, p.Hgrid, p.W, layer.kv,
                                  layer.written, layer.L, 1, False)
        ops.attn_ring(q_rot, layer.kv, layer.written, pos_s["t_pos"], layer.L, 1, n_splits=n_splits,
                      out=out_s, workspace=ws)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                               # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    layer.reset()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    layer.reset()
    for t in range(10):
        q, k, v, pos = p.inputs(t)
        qs.copy_(q); ks.copy_(k); vs.copy_(v)
        pos_s["t_pos"].fill_(t)
        graph.replay()
        torch.cuda.synchronize()
        (_, _, _, _), (q_h, ring) = eager.store(q, k, v, pos, strided=False)
        ref = eager.attend(q_h, ring, n_splits=n_splits, token_major_out=False)
        assert torch.equal(out_s, ref), f"replay {t} differs from eager"
        assert torch.equal(layer.kv, eager.hip.layers[0].kv) and torch.equal(layer.written, eager.hip.layers[0].written)


# ------------------------------------------------------------------------------------------
# error behaviour through the C ABI
# ------------------------------------------------------------------------------------------
def test_bad_inputs_raise(gpu_device):
    p = Pair(gpu_device, torch.bfloat16, B=1, H=2, Hkv=2, T=64, Dh=64, n_slots=2, cfg_id=26)
    q, k, v, pos = p.inputs(0)
    dev = gpu_device
    with pytest.raises(RuntimeError, match="one frame per upsert"):
        p.hip.upsert(k[:, :, :32].to(dev), v[:, :, :32].to(dev), to_dev(pos, dev), 0)
    p.hip.layers[0].check_inputs = True
    bad = to_dev(pos, dev)
    bad["t_pos"] = bad["t_pos"].clone()
    bad["t_pos"][0, 3] = 7
    with pytest.raises(RuntimeError, match="constant within frame"):
        p.hip.upsert(k.to(dev), v.to(dev), bad, 0)
    bad["t_pos"].fill_(-1)
    with pytest.raises(RuntimeError, match="non-negative"):
        p.hip.upsert(k.to(dev), v.to(dev), bad, 0)
    # a RoPE table that is too short for the frame index raises instead of clamping
    # (src/model/attn.py:25-30: index_select on the flat position)
    short = wea.RoPE(*ro.rope_table_1d(2 * 64, 64), p.Hgrid, p.W).to(dev)
    good = to_dev(p.inputs(1)[3], dev)
    late = to_dev(p.inputs(2)[3], dev)
    p.hip.rope_upsert(q.to(dev), k.to(dev), v.to(dev), good, short, 0)
    before = p.hip.layers[0].kv.clone()
    with pytest.raises(IndexError, match="index out of range"):
        p.hip.rope_upsert(q.to(dev), k.to(dev), v.to(dev), late, short, 0)
    with pytest.raises(IndexError, match="index out of range"):
        p.hip.rope_upsert_attend(q.to(dev), k.to(dev), v.to(dev), late, short, 0)
    with pytest.raises(IndexError, match="index out of range"):
        short(q.to(dev), late)
    assert torch.equal(p.hip.layers[0].kv, before), "a refused call must not touch the cache"
    narrow = wea.RoPE(*ro.rope_table_1d(64 * 64, 64), p.Hgrid // 2, p.W).to(dev)
    with pytest.raises(AssertionError, match="pos_ids out of bounds"):
        p.hip.rope_upsert(q.to(dev), k.to(dev), v.to(dev), good, narrow, 0)
    # unsupported head dim for the attention kernel
    layer = wea.LayerKVCache(1, 1, 64, 32, torch.bfloat16, 64).to(dev)
    with pytest.raises(RuntimeError, match="not covered"):
        ops.attn_ring(torch.zeros(1, 1, 64, 32, dtype=torch.bfloat16, device=dev), layer.kv, layer.written,
                      torch.zeros(1, 64, dtype=torch.long, device=dev), 64, 1)
    # fp32 caches run the one-pass kernel: asking for a context split is refused
    with pytest.raises(RuntimeError, match="not covered"):
        lay32 = wea.LayerKVCache(1, 1, 128, 64, torch.float32, 64).to(dev)
        ops.attn_ring(torch.zeros(1, 1, 64, 64, dtype=torch.float32, device=dev), lay32.kv, lay32.written,
                      torch.zeros(1, 64, dtype=torch.long, device=dev), 128, 1, n_splits=2)
