"""CPU-side checks: the C-ABI library loads and exports every declared symbol, argument
validation returns the documented codes before anything touches a GPU, and the host classes
mirror the reference's interface."""
import ctypes
import os
import re
from types import SimpleNamespace

import pytest
import torch

import world_engine_amd as wea
from world_engine_amd import _capi, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header="we_attn.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(we_[a-z0-9_]+)\s*\(", text)))


def _exported(path):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line and line.split()[-1].startswith("we_")}


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert {"we_version", "we_error_string", "we_init", "we_rope_kv_store", "we_rope_apply", "we_attn_auto_splits",
            "we_attn_workspace_bytes", "we_attn_plan", "we_attn_ring_fwd"} <= set(names)
    assert set(names) == set(_capi.SIGNATURES), "ctypes signatures and header disagree"
    lib = _capi.lib()
    for n in names:
        assert hasattr(lib, n), f"{n} not exported"
    assert lib.we_version() >= 100
    assert lib.we_error_string(0) == b"ok" and b"unknown" in lib.we_error_string(-99)
    # the product library is the drop-in surface and nothing else: no measurement entry points
    assert _exported(_capi.LIB_PATH) == set(names)


def test_measurement_library_exports_both_headers():
    """libwe_probe.so (benchmark and probe tests only) carries the entry points of
    include/we_attn_probe.h on top of the product's."""
    probe_names = _declared_symbols("we_attn_probe.h")
    assert set(probe_names) == set(_capi.PROBE_SIGNATURES) == {"we_attn_ring_fwd_clocked", "we_stream_probe"}
    plib = _capi.probe_lib()
    for n in probe_names + _declared_symbols():
        assert hasattr(plib, n), f"{n} not exported by the measurement library"
    assert _exported(_capi.PROBE_LIB_PATH) == set(probe_names) | set(_declared_symbols())
    assert plib.we_version() == _capi.lib().we_version()


def test_validation_codes_without_gpu():
    lib = _capi.lib()
    s3 = _capi.i64x3(8, 8, 8)
    fake = ctypes.c_void_p(4096)     # never dereferenced: validation fails first
    # null pointers
    assert lib.we_attn_ring_fwd(None, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64, 1, 0.1, 1, 0, 0, None) == -1
    # L not a multiple of T
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 100, 1, 0.1, 1, 0, 0, None) == -2
    # H % Hkv != 0
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 3, 2, 64, 64, 64, 1, 0.1, 1, 0, 0, None) == -2
    # unsupported head dim / dtype / slot count
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 96, 64, 1, 0.1, 1, 0, 0, None) == -3
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64, 1, 0.1, 1, 0, 3, None) == -3
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64, 1, 0.1, 2, 0, 2, None) == -3   # fp32: no splits
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64 * 257, 1, 0.1, 1, 0, 0, None) == -3
    # misaligned pointer / stride
    assert lib.we_attn_ring_fwd(ctypes.c_void_p(4100), s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64, 1, 0.1, 1, 0, 0, None) == -4
    assert lib.we_attn_ring_fwd(fake, _capi.i64x3(8, 8, 4), fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64, 1, 0.1, 1, 0, 0, None) == -4
    # splits without workspace
    assert lib.we_attn_ring_fwd(fake, s3, fake, fake, fake, fake, s3, None, 0, 1, 1, 1, 64, 64, 64, 1, 0.1, 2, 0, 0, None) == -5
    # store: q without q_out, tables without y/x, dilation not dividing the slot count
    assert lib.we_rope_kv_store(fake, fake, fake, s3, s3, s3, None, None, None, 0, fake, None, None, 0, 1, 1, fake, fake,
                                1, 1, 1, 64, 64, 64, 1, 0, 0, None) == -1
    assert lib.we_rope_kv_store(None, fake, fake, None, s3, s3, None, fake, fake, 10, fake, None, None, 0, 1, 1, fake, fake,
                                1, 1, 1, 64, 64, 64, 1, 0, 0, None) == -1
    assert lib.we_rope_kv_store(None, fake, fake, None, s3, s3, None, None, None, 0, fake, None, None, 0, 1, 1, fake, fake,
                                1, 1, 1, 64, 64, 192, 2, 0, 0, None) == -2


def test_workspace_and_split_planning():
    lib = _capi.lib()
    assert lib.we_attn_workspace_bytes(1, 16, 16, 256, 128, 4096, 1, 0) == 0
    assert lib.we_attn_workspace_bytes(1, 16, 16, 256, 128, 4096, 4, 0) == 4 * 16 * 256 * (128 * 2 + 16)
    # 256-token frames: every unit is split, into three quarters of the parts that would give every CU a workgroup
    s = lib.we_attn_auto_splits(1, 16, 16, 256, 128, 4096)
    assert s == 6
    # ... and the workgroups of a call never outnumber the 256 CUs: 48, 80, 96, 160 unsplit workgroups
    for heads, want in ((24, 5), (40, 3), (48, 2), (80, 1)):
        assert lib.we_attn_auto_splits(1, heads, heads, 256, 128, 4096) == want, heads
    assert lib.we_attn_workspace_bytes(1, 16, 16, 256, 128, 4096, 0, 0) == s * 16 * 256 * (128 * 2 + 16)
    # long contexts (32 slots and more) take about 240 workgroups; 32 heads are cut in four (all 256 CUs);
    # beyond sixteen parts about 160 workgroups
    assert lib.we_attn_auto_splits(1, 16, 16, 256, 128, 8192) == 7
    assert lib.we_attn_auto_splits(1, 12, 12, 256, 128, 8192) == 10
    assert lib.we_attn_auto_splits(1, 32, 32, 256, 128, 4096) == 4
    assert lib.we_attn_auto_splits(1, 4, 4, 256, 128, 4096) == 20
    assert lib.we_attn_auto_splits(1, 4, 4, 256, 128, 8192) == 20
    # 1024-token frames with 96 heads: 384 workgroups of 256 queries = 1.5 rounds of 256 CUs, so only
    # the last 32 of the 96 units (128 workgroups) are split in two
    assert lib.we_attn_auto_splits(4, 24, 24, 1024, 128, 8192) == 2
    assert lib.we_attn_workspace_bytes(4, 24, 24, 1024, 128, 8192, 0, 0) == 2 * 32 * 1024 * (128 * 2 + 16)
    # whole rounds: nothing to split
    assert lib.we_attn_auto_splits(4, 32, 32, 1024, 128, 8192) == 1
    assert lib.we_attn_workspace_bytes(4, 32, 32, 1024, 128, 8192, 0, 0) == 0
    # never more splits than half the 64-key tiles of the context
    assert lib.we_attn_auto_splits(1, 1, 1, 64, 64, 128) <= 1


def test_planner_over_other_shapes_and_cu_counts():
    """Invariants of the split planner over shapes and parts other than the benchmark's: a split
    call never launches more workgroups than there are CUs, every part keeps at least two 64-key
    tiles, unsplit calls stay unsplit, and the counts scale with the CU count."""
    for cus in (64, 104, 228, 256, 304):
        for B, H, Hkv, T, n_slots in ((1, 4, 4, 256, 16), (1, 12, 4, 256, 24), (2, 8, 8, 128, 8), (1, 40, 40, 256, 32),
                                      (1, 6, 2, 64, 3), (3, 5, 5, 192, 12), (1, 16, 16, 256, 64), (1, 2, 2, 512, 4)):
            pl = ops.attn_plan(B, H, Hkv, T, 128, n_slots * T, compute_units=cus)
            unsplit = B * H * -(-T // pl["q_tile"])
            tiles = n_slots * T // 64
            assert pl["compute_units"] == cus and pl["n_splits"] >= 1
            if pl["n_splits"] > 1 and pl["units_whole"] == 0:
                assert pl["workgroups"] <= cus, (cus, B, H, T, n_slots, pl)
                assert pl["workgroups"] == unsplit * pl["n_splits"]
                assert tiles // pl["n_splits"] >= 2, (cus, B, H, T, n_slots, pl)
                assert pl["workgroups"] * 2 > cus or pl["n_splits"] == max(1, tiles // 2), "split calls use most of the chip"
            if unsplit >= cus and unsplit % cus == 0:
                assert pl["n_splits"] == 1
    # the benchmark's 16-head call on half and on twice the CUs
    assert ops.attn_plan(1, 16, 16, 256, 128, 4096, compute_units=128)["n_splits"] == 4
    assert ops.attn_plan(1, 16, 16, 256, 128, 4096, compute_units=512)["n_splits"] == 12
    assert ops.attn_plan(1, 16, 16, 256, 128, 4096, compute_units=256) == {
        "q_tile": 128, "n_splits": 6, "units_whole": 0, "workgroups": 192, "compute_units": 256}
    p3 = ops.attn_plan(4, 24, 24, 1024, 128, 8192, compute_units=256)
    assert (p3["q_tile"], p3["n_splits"], p3["units_whole"], p3["workgroups"]) == (256, 2, 64, 512)
    # the partial last round: 384 workgroups on 256 CUs split their last 128; on 128 CUs they are three whole rounds
    assert ops.attn_plan(4, 24, 24, 1024, 128, 8192, compute_units=128)["n_splits"] == 1


def test_no_cpu_fallback():
    cache = wea.LayerKVCache(1, 2, 128, 64, torch.bfloat16, 64)
    k = torch.zeros(1, 2, 64, 64, dtype=torch.bfloat16)
    pos = {"t_pos": torch.zeros(1, 64, dtype=torch.long)}
    with pytest.raises(RuntimeError, match="ROCm GPU only"):
        cache.upsert_kv(k, k, pos, False)
    with pytest.raises(RuntimeError, match="ROCm GPU only"):
        ops.attn_ring(k, cache.kv, cache.written, pos["t_pos"], 128, 1)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", "/nonexistent/libwe_attn.so")
    with pytest.raises(RuntimeError, match="has not been built"):
        _capi.lib()


def test_cache_classes_mirror_reference_interface():
    cfg = SimpleNamespace(tokens_per_frame=64, local_window=4, global_window=8, global_attn_period=2,
                          global_attn_offset=1, global_pinned_dilation=2, n_layers=4, n_heads=8,
                          n_kv_heads=4, d_model=512)
    c = wea.StaticKVCache(cfg, 1, torch.bfloat16)
    assert isinstance(c.layers, torch.nn.ModuleList) and len(c.layers) == 4
    assert [(l.L, l.pinned_dilation, l.num_buckets) for l in c.layers] == [(256, 1, 4), (512, 2, 4), (256, 1, 4), (512, 2, 4)]
    l0 = c.layers[0]
    assert l0.kv.shape == (2, 1, 4, 320, 64) and l0.kv.dtype == torch.bfloat16 and l0.capacity == 320 and l0.tpf == 64
    assert l0.written.dtype == torch.bool and l0.written[256:].all() and not l0.written[:256].any()
    assert l0.frame_offsets.tolist() == list(range(64)) and l0.current_idx[0] == 256
    assert len(c.state_dict()) == 0                      # non-persistent buffers, like the reference
    assert c._is_frozen
    c.set_frozen(False)
    assert not c._is_frozen
    l0.written[:64] = True
    l0.kv.fill_(1)
    c.reset()
    assert c._is_frozen and not l0.kv.any() and not l0.written[:256].any() and l0.written[256:].all()
    with pytest.raises(AssertionError):
        wea.LayerKVCache(1, 1, 100, 64, torch.bfloat16, 64)
    with pytest.raises(AssertionError):
        wea.LayerKVCache(1, 1, 192, 64, torch.bfloat16, 64, pinned_dilation=2)


def test_attention_module_parameters_and_casting():
    cfg = SimpleNamespace(n_heads=8, n_kv_heads=2, d_model=512, value_residual=True, gated_attn=True)
    rope = wea.RoPE.one_dimensional(128, 64, 8, 8)
    split = wea.RingAttn(cfg, 3, rope)
    assert {"q_proj.weight", "k_proj.weight", "v_proj.weight", "out_proj.weight", "v_lamb", "gate_proj.weight"} == set(split.state_dict())
    assert split.layer_idx == 3 and split.enable_gqa and split.d_head == 64
    assert not split.gate_proj.weight.any()
    merged = wea.RingAttn.from_reference(split, cfg, rope, merged_qkv=True)
    assert merged.qkv_proj.weight.shape == (512 + 2 * 128, 512)
    assert torch.equal(merged.qkv_proj.weight[:512], split.q_proj.weight)
    assert torch.equal(merged.qkv_proj.weight[512:640], split.k_proj.weight)
    assert torch.equal(merged.out_proj.weight, split.out_proj.weight)
    merged = merged.to(torch.bfloat16)
    assert merged.rope.cos.dtype == torch.float32 and merged.qkv_proj.weight.dtype == torch.bfloat16
    assert rope.cos.shape == (128, 32)

    class Holder(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.config = cfg
            self.blocks = torch.nn.ModuleList([wea.RingAttn(cfg, i, rope) for i in range(2)])

    class Legacy(wea.RingAttn):
        pass

    m = Holder()
    assert wea.install_ring_attention(m, rope, (Legacy,)) == 0


def test_fused_projection_is_chosen_by_shape():
    """fuse_projection runs the library's projection kernel where its workgroups (64 tokens x
    128 features each) fit the CUs in one round, and the linear layer + store call beyond."""
    rope = wea.RoPE.one_dimensional(128, 128, 16, 16)
    cfg = SimpleNamespace(n_heads=16, n_kv_heads=16, d_model=2048)
    m = wea.RingAttn(cfg, 0, rope, merged_qkv=True, fuse_elementwise=True, fuse_projection=True)
    assert m.projection_workgroups(1, 256) == 4 * 48 and m.uses_fused_projection(1, 256)
    assert m.projection_workgroups(1, 264) == 5 * 48 and m.uses_fused_projection(1, 264)
    assert m.projection_workgroups(1, 1024) == 16 * 48 and not m.uses_fused_projection(1, 1024)
    assert not m.uses_fused_projection(4, 256)
    assert m.uses_fused_projection(1, 8)
    plain = wea.RingAttn(cfg, 0, rope, merged_qkv=True, fuse_elementwise=True)
    assert not plain.uses_fused_projection(1, 256)
    wide = wea.RingAttn(SimpleNamespace(n_heads=24, n_kv_heads=24, d_model=3072), 0, rope, merged_qkv=True,
                        fuse_elementwise=True, fuse_projection=True)
    assert wide.projection_workgroups(1, 256) == 288 and not wide.uses_fused_projection(1, 256)
    assert wide.uses_fused_projection(1, 192)


def test_custom_ops_registered_with_fake_kernels():
    q = torch.empty(1, 4, 64, 64, dtype=torch.bfloat16, device="meta")
    kv = torch.empty(2, 1, 4, 192, 64, dtype=torch.bfloat16, device="meta")
    written = torch.empty(192, dtype=torch.bool, device="meta")
    t = torch.empty(1, 64, dtype=torch.long, device="meta")
    out = torch.ops.world_engine_amd.attn_ring(q, kv, written, t, 128, 1, 0.125)
    assert out.shape == (1, 4, 64, 64) and out.transpose(1, 2).is_contiguous()
    tab = torch.empty(64, 32, device="meta")
    qr = torch.ops.world_engine_amd.rope_kv_store(q, q, q, t, t, t, tab, tab, 8, 8, kv, written, 128, 1, False)
    assert qr.shape == q.shape
    y = torch.ops.world_engine_amd.rope_kv_attn(q, q, q, t, t, t, tab, tab, 8, 8, kv, written, 128, 1, False, 0.125)
    assert y.shape == (1, 4, 64, 64) and y.transpose(1, 2).is_contiguous()


def test_one_call_entry_point_validates_both_halves():
    lib = _capi.lib()
    s3 = _capi.i64x3(8, 8, 8)
    fake = ctypes.c_void_p(4096)     # never dereferenced: validation fails first
    args = lambda **kw: [kw.get("q", fake), fake, fake, s3, s3, s3, kw.get("q_out", fake), kw.get("cos", fake), fake, 10,
                         fake, fake, fake, 64, 8, 8, fake, fake, kw.get("out", fake), s3, None, 0,
                         1, 1, 1, 64, kw.get("Dh", 64), kw.get("L", 64), 1, 0, 0.1, kw.get("n_splits", 1), 0,
                         kw.get("dtype", 0), kw.get("extras"), None]
    assert lib.we_rope_kv_attn_fwd(*args(q=None)) == -1
    assert lib.we_rope_kv_attn_fwd(*args(q_out=None)) == -1
    assert lib.we_rope_kv_attn_fwd(*args(cos=None)) == -1
    assert lib.we_rope_kv_attn_fwd(*args(out=None)) == -1            # attention half
    assert lib.we_rope_kv_attn_fwd(*args(L=100)) == -2
    assert lib.we_rope_kv_attn_fwd(*args(Dh=96)) == -3               # store accepts it, attention does not
    assert lib.we_rope_kv_attn_fwd(*args(dtype=2, n_splits=2)) == -3 # fp32 runs the one-pass kernel only
    assert lib.we_rope_kv_attn_fwd(*args(dtype=3)) == -3
    assert lib.we_rope_kv_attn_fwd(*args(n_splits=2)) == -5          # splits without workspace
    # extras: lerp needs both the residual and its weight; negative epsilon; norm needs Dh/16 a power of two
    ex = _capi.AttnExtras()
    ex.v1 = 4096
    assert lib.we_rope_kv_attn_fwd(*args(extras=ctypes.byref(ex))) == -1
    ex = _capi.AttnExtras()
    ex.qk_norm_eps = -1.0
    assert lib.we_rope_kv_attn_fwd(*args(extras=ctypes.byref(ex))) == -2


def test_stream_probe_validates_before_launching():
    """The tile-stream probe of the measurement library refuses bad arguments with a status code (no GPU needed)."""
    lib = _capi.probe_lib()
    fake = ctypes.c_void_p(4096)
    region = 23 * 16384
    assert lib.we_stream_probe(None, 96 * region, 192, 23, 2, None) == -1            # null buffer
    assert lib.we_stream_probe(fake, 96 * region, 100, 23, 2, None) == -2            # workgroups not a multiple of 8
    assert lib.we_stream_probe(fake, 96 * region, 192, 0, 2, None) == -2             # no tiles
    assert lib.we_stream_probe(fake, 96 * region, 192, 23, 5, None) == -2            # 24 workgroups per XCD do not share in fives
    assert lib.we_stream_probe(ctypes.c_void_p(4100), 96 * region, 192, 23, 2, None) == -4   # misaligned
    assert lib.we_stream_probe(fake, 96 * region - 1, 192, 23, 2, None) == -5        # buffer does not cover the regions


def test_projection_entry_points_validate_before_launching():
    """we_qkv_rope_kv_store / we_qkv_rope_kv_attn_fwd refuse bad operands with a status code and
    launch nothing (no GPU is needed to see that)."""
    lib = _capi.lib()
    s3 = _capi.i64x3(8, 8, 8)
    fake = ctypes.c_void_p(4096)     # never dereferenced: validation fails first

    def proj(**kw):
        pr = _capi.QkvProj()
        pr.x, pr.w = kw.get("x", 4096), kw.get("w", 4096)
        pr.d_model = kw.get("d_model", 256)
        pr.x_strides = (ctypes.c_int64 * 2)(64 * 256, kw.get("xs_t", 256))
        pr.w_row_stride = kw.get("ws", 256)
        return pr

    def store(pr, **kw):
        return lib.we_qkv_rope_kv_store(ctypes.byref(pr) if pr is not None else None, kw.get("q_out", fake), kw.get("cos", fake),
                                        fake, 10, fake, fake, fake, 64, 8, 8, fake, fake,
                                        1, kw.get("H", 2), kw.get("Hkv", 2), 64, kw.get("Dh", 64), kw.get("L", 64), 1, 0,
                                        kw.get("dtype", 0), kw.get("extras"), None)

    assert store(None) == -1
    assert store(proj(x=None)) == -1
    assert store(proj(), q_out=None) == -1
    assert store(proj(), cos=None) == -1               # the projection always rotates
    assert store(proj(), L=100) == -2
    assert store(proj(), dtype=2) == -3                # bf16 / f16 only
    assert store(proj(), Dh=32) == -3
    assert store(proj(d_model=192, xs_t=192, ws=192)) == -3    # contraction length not a multiple of 128
    assert store(proj(), H=1, Hkv=1) == -3             # (H + 2 Hkv) Dh = 192 is not a whole number of feature tiles
    assert store(proj(ws=128)) == -2                   # weight rows shorter than the contraction
    assert store(proj(xs_t=260)) == -4                 # token stride not a multiple of 8 elements
    ex = _capi.AttnExtras()
    ex.v1 = 4096
    assert store(proj(), extras=ctypes.byref(ex)) == -1        # residual without its weight
    pr = proj()
    rc = lib.we_qkv_rope_kv_attn_fwd(ctypes.byref(pr), fake, fake, fake, 10, fake, fake, fake, 64, 8, 8, fake, fake,
                                     None, s3, None, 0, 1, 2, 2, 64, 64, 64, 1, 0, 0.1, 1, 0, 0, None, None)
    assert rc == -1                                    # attention half: no output
    rc = lib.we_qkv_rope_kv_attn_fwd(ctypes.byref(pr), fake, fake, fake, 10, fake, fake, fake, 64, 8, 8, fake, fake,
                                     fake, s3, None, 0, 1, 2, 2, 64, 64, 64, 1, 0, 0.1, 2, 0, 0, None, None)
    assert rc == -5                                    # splits without workspace
    # the opaque op has a fake kernel with the module's output layouts
    x = torch.empty(1, 64, 256, dtype=torch.bfloat16, device="meta")
    w = torch.empty(8 * 64, 256, dtype=torch.bfloat16, device="meta")
    kv = torch.empty(2, 1, 2, 192, 64, dtype=torch.bfloat16, device="meta")
    written = torch.empty(192, dtype=torch.bool, device="meta")
    t = torch.empty(1, 64, dtype=torch.long, device="meta")
    tab = torch.empty(64, 32, device="meta")
    y, v = torch.ops.world_engine_amd.qkv_rope_kv_attn(x, w, 4, 2, t, t, t, tab, tab, 8, 8, kv, written, 128, 1, False, 0.125)
    assert y.shape == (1, 4, 64, 64) and y.transpose(1, 2).is_contiguous()
    assert v.shape == (1, 2, 64, 64) and v.transpose(1, 2).is_contiguous()


def test_attention_kernels_keep_their_state_in_registers():
    """Compile-time guard: the MFMA kernels hold accumulators, fragments and softmax state in
    VGPRs.  A source change that makes the compiler place those arrays in scratch memory still
    passes every parity test and is an order of magnitude slower, so the compiler's own resource
    report is checked: at most a few spilled registers per lane, never whole arrays."""
    import re
    import shutil
    import subprocess
    from world_engine_amd import build as wbuild
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    src = os.path.join(wbuild.CSRC, "attn_ring.hip")
    r = subprocess.run([hipcc, *[f for f in wbuild.HIPCC_FLAGS if f not in ("-shared", "-fPIC")], "-c", src, "-o", os.devnull,
                        "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    sizes = [int(m) for m in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", r.stderr)]
    assert len(sizes) == 16, sizes          # bf16/f16 x Dh 64/128 x 128/256 queries x ragged or not
    assert max(sizes) <= 160, sizes
    # the projection kernel: accumulators in registers, two wavefronts per SIMD
    src = os.path.join(wbuild.CSRC, "qkv_proj_store.hip")
    r = subprocess.run([hipcc, *[f for f in wbuild.HIPCC_FLAGS if f not in ("-shared", "-fPIC")], "-c", src, "-o", os.devnull,
                        "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    sizes = [int(m) for m in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", r.stderr)]
    vgprs = [int(m) for m in re.findall(r" VGPRs: (\d+)", r.stderr)]
    assert len(sizes) == 2 and max(sizes) == 0 and max(vgprs) <= 256, (sizes, vgprs)


def test_three_axis_rope_table_structure():
    """What the geometry fixes about the three-axis table (the per-axis spectra themselves come
    from a package that is not available here, so their values stay unpinned): block widths, which
    coordinate each block depends on, doubled frequencies, mirror symmetry of the pixel axes,
    angles below Nyquist, a unit first temporal frequency; and the oracle's restatement agrees."""
    from oracle import ring_oracle as ro
    Hh, Ww, n_frames, Dh = 6, 10, 5, 64
    rope = wea.RoPE.three_axis(n_frames, Dh, Hh, Ww)
    assert rope.cos.shape == rope.sin.shape == (n_frames * Hh * Ww, Dh // 2) and rope.cos.dtype == torch.float32
    ang = torch.atan2(rope.sin, rope.cos).view(n_frames, Hh, Ww, Dh // 2)
    bx, by = slice(0, Dh // 8), slice(Dh // 8, Dh // 4)
    bt = slice(Dh // 4, Dh // 2)
    cos = rope.cos.view(n_frames, Hh, Ww, -1)
    sin = rope.sin.view(n_frames, Hh, Ww, -1)
    # X depends on x only, Y on y only, T on t only
    assert torch.equal(cos[..., bx], cos[:1, :1, :, bx].expand(n_frames, Hh, Ww, -1))
    assert torch.equal(cos[..., by], cos[:1, :, :1, by].expand(n_frames, Hh, Ww, -1))
    assert torch.equal(sin[..., bt], sin[:, :1, :1, bt].expand(n_frames, Hh, Ww, -1))
    # each frequency appears twice in a row
    assert torch.equal(cos[..., 0::2], cos[..., 1::2]) and torch.equal(sin[..., 0::2], sin[..., 1::2])
    # pixel positions are symmetric about the centre: angle(x) = -angle(W-1-x)
    assert torch.allclose(cos[..., bx], cos[..., bx].flip(2), atol=1e-6)
    assert torch.allclose(sin[..., bx], -sin[..., bx].flip(2), atol=1e-6)
    assert torch.allclose(sin[..., by], -sin[..., by].flip(1), atol=1e-6)
    # neighbouring pixels differ by less than pi in every column (below Nyquist), and by more than 0
    step_x = (ang[0, 0, 1, bx] - ang[0, 0, 0, bx]).remainder(2 * torch.pi)
    assert (step_x > 0).all() and (step_x < torch.pi).all()
    # frame 0 is the identity rotation on the temporal block; the first temporal frequency is 1 rad/frame
    assert torch.equal(cos[0, ..., bt], torch.ones_like(cos[0, ..., bt])) and not sin[0, ..., bt].any()
    assert torch.allclose(ang[1, 0, 0, bt][0], torch.tensor(1.0), atol=1e-6)
    assert (ang[1, 0, 0, bt][0::2].diff() < 0).all()      # geometric spectrum: decreasing
    o_cos, o_sin = ro.ortho_rope_table(Hh, Ww, n_frames, Dh)
    assert torch.allclose(rope.cos, o_cos, atol=1e-6) and torch.allclose(rope.sin, o_sin, atol=1e-6)


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 on its own, and a C program that
    includes it must link against the built library and get the documented status codes back
    from calls that are rejected before anything touches a GPU."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    lib_path = _capi.library_path() if hasattr(_capi, "library_path") else os.path.join(ROOT, "world_engine_amd", "libwe_attn.so")
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include "we_attn.h"
#include <stdio.h>
int main(void) {
  int64_t s[3] = {8, 8, 8};
  /* NULL pointers are refused first */
  int rc_null = we_attn_ring_fwd(0, s, 0, 0, 0, 0, s, 0, 0, 1, 1, 1, 64, 64, 128, 1, 0.125f, 0, 0, WE_DTYPE_BF16, 0);
  size_t ws = we_attn_workspace_bytes(1, 16, 16, 256, 128, 4096, 4, 0);
  printf("%d %d %zu %s\n", we_version(), rc_null, ws, we_error_string(WE_ERR_WORKSPACE));
  return 0;
}
''')
    exe = tmp_path / "abi"
    r = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{os.path.join(ROOT, 'include')}",
                        str(src), "-o", str(exe), lib_path, f"-Wl,-rpath,{os.path.dirname(lib_path)}",
                        "-Wl,-rpath,/opt/rocm/lib", "-Wl,--allow-shlib-undefined"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    version, rc_null, ws, msg = out.stdout.strip().split(" ", 3)
    lib = _capi.lib()
    assert int(version) == lib.we_version()
    assert int(rc_null) == -1                                    # WE_ERR_NULL_POINTER
    assert int(ws) == 4 * 16 * 256 * (128 * 2 + 16)
    assert "workspace" in msg


def test_rope_position_ids_are_bounds_checked_in_eager_mode():
    """The reference asserts y < height, x < width and its index_select raises on a table row past
    the end (src/model/attn.py:25-30); the kernels only clamp, so the host check must raise."""
    from oracle import ring_oracle as ro
    rope = wea.RoPE.one_dimensional(4 * 16, 32, 4, 4)            # rows for frames 0..3 of a 4x4 grid
    rope.check_pos_ids(ro.synth_pos_ids(3, 1, 16, 4))            # last frame the table holds
    with pytest.raises(IndexError, match="index out of range"):
        rope.check_pos_ids(ro.synth_pos_ids(4, 1, 16, 4))        # one frame past the table
    with pytest.raises(AssertionError, match="pos_ids out of bounds"):
        rope.check_pos_ids(ro.synth_pos_ids(0, 1, 16, 2))        # y runs to 7 on a grid of height 4
    neg = ro.synth_pos_ids(0, 1, 16, 4)
    neg["t_pos"] = neg["t_pos"] - 1
    with pytest.raises(IndexError):
        rope.check_pos_ids(neg)
    # the oracle raises on the same inputs (index_select), so both sides fail alike
    cos, sin = ro.rope_table_1d(4 * 16, 32)
    with pytest.raises((IndexError, RuntimeError)):
        ro.rope_angles(ro.synth_pos_ids(4, 1, 16, 4), cos, sin, 4, 4)
