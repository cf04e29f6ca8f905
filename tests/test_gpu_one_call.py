"""GPU parity of the one-call path (we_rope_kv_attn_fwd): RoPE + K/V store + attention.

Cache rows, ``written`` and RoPE(q) must equal the oracle's bit for bit (and so the two-call
path's); attention within max-abs 2e-2 / mean-abs 2e-3 of the fp32 oracle.
"""
import pytest
import torch

from oracle import ring_oracle as ro
from _harness import Pair, assert_attn_close, assert_bits_equal, assert_ulp_close, merged_views, to_dev
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_one_call_cfg1_shape(gpu_device, dtype):
    p = Pair(gpu_device, dtype, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, cfg_id=1)
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


@pytest.mark.parametrize("backend,fuse", [("eager", False), ("inductor", False), ("inductor", True)])
def test_module_forward_compiles_as_one_graph(gpu_device, backend, fuse):
    """RingAttn under torch.compile(fullgraph=True), also with the backend the reference compiles
    its passes with (src/world_engine.py:139): the cache call is the registered opaque op (the
    reference wraps its one native kernel the same way, src/quantize.py:17-42); results and cache
    state equal the eager module's."""
    import types
    import world_engine_amd as wea
    torch.manual_seed(0)
    cfg = types.SimpleNamespace(d_model=256, n_heads=4, n_kv_heads=2, value_residual=True, gated_attn=True,
                                tokens_per_frame=64, local_window=3, global_window=3, global_attn_period=1,
                                global_pinned_dilation=1, n_layers=1)
    cos, sin = ro.rope_table_1d(16 * 64, 64)
    rope = wea.RoPE(cos, sin, 8, 8).to(gpu_device)
    mod = wea.RingAttn(cfg, 0, rope, merged_qkv=True, fuse_elementwise=fuse).to(gpu_device, torch.bfloat16)
    with torch.no_grad():
        mod.gate_proj.weight.normal_(0, 0.5)
    caches = [wea.StaticKVCache(cfg, 1, torch.bfloat16).to(gpu_device) for _ in range(2)]
    for c in caches:
        c.set_frozen(False)
        for layer in c.layers:
            layer.check_inputs = False
    compiled = torch.compile(mod, backend=backend, fullgraph=True)
    for t in range(5):
        x = torch.randn(1, 64, 256, device=gpu_device, dtype=torch.bfloat16)
        pos = to_dev(ro.synth_pos_ids(t, 1, 64, 8), gpu_device)
        with torch.no_grad():
            y_e, _ = mod(x, pos, None, caches[0])
            y_c, _ = compiled(x, pos, None, caches[1])
        # the projections around the call may be fused differently by the compiler: tolerance there,
        # bits for what the library writes
        assert (y_e.float() - y_c.float()).abs().max().item() <= 2e-2, f"t={t}"
        assert_bits_equal(caches[0].layers[0].kv, caches[1].layers[0].kv, f"cache t={t}")
        assert torch.equal(caches[0].layers[0].written, caches[1].layers[0].written)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_neighbours_match_torch_ops(gpu_device, dtype):
    """qk RMS norm, value-residual lerp and head gate inside the kernels against the same torch
    operations in front of / behind the plain call: cache rows and RoPE(q) within 1 ulp (and
    mostly identical), `written` identical, gated output within the attention bar."""
    dev = gpu_device
    B, H, Hkv, T, Dh, n = 2, 4, 2, 128, 128, 3
    p_f = Pair(dev, dtype, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, cfg_id=61)     # fused
    p_u = Pair(dev, dtype, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, cfg_id=61)     # torch ops + plain call
    eps = torch.finfo(torch.float32).eps
    g = torch.Generator("cpu").manual_seed(7)
    lamb = torch.tensor(0.37, dtype=dtype, device=dev)
    for t in range(7):
        frozen = t % 3 == 1
        q, k, v, pos = p_f.inputs(t)
        v1 = torch.randn(v.shape, generator=g).to(dtype)
        gate = torch.sigmoid(torch.randn(B, T, H, generator=g)).to(dtype).to(dev).permute(0, 2, 1)   # strided [B,H,T]
        qd, kd, vd = merged_views(q.to(dev), k.to(dev), v.to(dev))
        v1d = v1.to(dev)
        posd = to_dev(pos, dev)
        lf, lu = p_f.hip.layers[0], p_u.hip.layers[0]
        out_f, qrot_f = ops.rope_kv_attn(qd, kd, vd, posd, p_f.rope.cos, p_f.rope.sin, p_f.rope.height, p_f.rope.width,
                                         lf.kv, lf.written, lf.L, 1, frozen, qk_norm_eps=eps, v1=v1d, v_lamb=lamb,
                                         gate=gate)
        qn = torch.nn.functional.rms_norm(qd, (Dh,))
        kn = torch.nn.functional.rms_norm(kd, (Dh,))
        vl = torch.lerp(vd, v1d, lamb)
        out_u, qrot_u = ops.rope_kv_attn(qn, kn, vl, posd, p_u.rope.cos, p_u.rope.sin, p_u.rope.height, p_u.rope.width,
                                         lu.kv, lu.written, lu.L, 1, frozen)
        out_u = out_u * gate.unsqueeze(-1)
        frac = assert_ulp_close(qrot_f, qrot_u, f"RoPE(norm(q)) t={t}")
        frac_kv = assert_ulp_close(lf.kv, lu.kv, f"cache t={t}")
        assert frac < 0.02 and frac_kv < 0.02, (frac, frac_kv)
        assert torch.equal(lf.written, lu.written)
        assert_attn_close(out_f, out_u.float().cpu(), f"gated output t={t}")


@pytest.mark.parametrize("gate_mode", ["given", "projected"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_neighbours_match_the_oracle(gpu_device, dtype, gate_mode):
    """The one-call entry point with qk RMS norm, value-residual lerp and head gate inside the
    kernels against the CPU oracle's layer_step with the same steps switched on
    (src/model/attn.py:105-119): cache rows and RoPE(norm(q)) within 1 ulp of their row's largest
    value (the kernel's row reduction order, rsqrt and the lerp's fused multiply-add differ in the
    last bit), `written` identical, the gated output within 2e-2 / 2e-3 of the fp32 flow.  The
    gate is either handed over ready-made or projected from the module's input inside the kernels
    (sigmoid(gate_proj(x[..., :H])), src/model/attn.py:117-118)."""
    dev = gpu_device
    B, H, Hkv, T, Dh, n = 2, 4, 2, 128, 128, 3
    p = Pair(dev, dtype, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, cfg_id=62)
    eps = torch.finfo(torch.float32).eps
    g = torch.Generator("cpu").manual_seed(8)
    lamb = torch.tensor(0.37, dtype=dtype)
    layer = p.hip.layers[0]
    for t in range(8):
        frozen = t % 3 == 1
        p.set_frozen(frozen)
        q, k, v, pos = p.inputs(t)
        q, k = q * 3, k * 0.5                                   # rows that are not already normalised
        v1 = torch.randn(v.shape, generator=g).to(dtype)
        if gate_mode == "given":
            gates = torch.sigmoid(torch.randn(B, T, H, generator=g)).to(dtype)      # [B, T, H] as the module has them
            gate_kw = dict(gate=gates.to(dev).permute(0, 2, 1))
        else:
            x_full = (torch.randn(B, T, 3 * H, generator=g) * 2).to(dtype)          # the module's input; the gate reads its first H channels
            w_gate = (torch.randn(H, H, generator=g) * 0.7).to(dtype)
            gates = torch.sigmoid(torch.nn.functional.linear(x_full[..., :H], w_gate))
            gate_kw = dict(gate_x=x_full.to(dev)[..., :H], gate_w=w_gate.to(dev))
        ref, q_rot = ro.layer_step(p.oracle, 0, q, k, v, pos, p.cos, p.sin, p.Hgrid, p.W, reference_dtype_flow=False,
                                   qk_norm=True, v1=v1, v_lamb=lamb, gates=gates)
        qd, kd, vd = merged_views(q.to(dev), k.to(dev), v.to(dev))
        out, qrot_h = ops.rope_kv_attn(qd, kd, vd, to_dev(pos, dev), p.rope.cos, p.rope.sin, p.rope.height, p.rope.width,
                                       layer.kv, layer.written, layer.L, 1, frozen, qk_norm_eps=eps, v1=v1.to(dev),
                                       v_lamb=lamb.to(dev), **gate_kw)
        frac_q = assert_ulp_close(qrot_h, q_rot, f"RoPE(norm(q)) t={t}")
        frac_kv = assert_ulp_close(layer.kv, p.oracle.layers[0].kv, f"cache t={t}")
        assert frac_q < 0.02 and frac_kv < 0.02, (frac_q, frac_kv)
        assert torch.equal(layer.written.cpu(), p.oracle.layers[0].written)
        assert_attn_close(out, ref, f"gated output t={t}")


def test_module_with_fused_neighbours(gpu_device):
    """RingAttn(fuse_elementwise=True) against the same module with the torch operations."""
    import types
    import world_engine_amd as wea
    torch.manual_seed(1)
    cfg = types.SimpleNamespace(d_model=512, n_heads=4, n_kv_heads=4, value_residual=True, gated_attn=True,
                                tokens_per_frame=64, local_window=3, global_window=3, global_attn_period=1,
                                global_pinned_dilation=1, n_layers=2)
    cos, sin = ro.rope_table_1d(16 * 64, 128)
    rope = wea.RoPE(cos, sin, 8, 8).to(gpu_device)
    plain = [wea.RingAttn(cfg, i, rope, merged_qkv=True).to(gpu_device, torch.bfloat16) for i in range(2)]
    fused = [wea.RingAttn(cfg, i, rope, merged_qkv=True, fuse_elementwise=True).to(gpu_device, torch.bfloat16)
             for i in range(2)]
    for a, b in zip(plain, fused):
        with torch.no_grad():
            a.gate_proj.weight.normal_(0, 0.5)
            a.v_lamb.fill_(0.3)
        b.load_state_dict(a.state_dict())
    caches = [wea.StaticKVCache(cfg, 1, torch.bfloat16).to(gpu_device) for _ in range(2)]
    for c in caches:
        c.set_frozen(False)
    for t in range(5):
        x = torch.randn(1, 64, 512, device=gpu_device, dtype=torch.bfloat16)
        pos = to_dev(ro.synth_pos_ids(t, 1, 64, 8), gpu_device)
        with torch.no_grad():
            ya, v1a = plain[0](x, pos, None, caches[0])
            ya2, _ = plain[1](ya, pos, v1a, caches[0])
            yb, v1b = fused[0](x, pos, None, caches[1])
            yb2, _ = fused[1](yb, pos, v1b, caches[1])
        d1 = (ya.float() - yb.float()).abs().max().item()
        d2 = (ya2.float() - yb2.float()).abs().max().item()
        scale = ya2.float().abs().max().item()
        assert d1 <= 2e-2 * max(1.0, ya.float().abs().max().item()) and d2 <= 3e-2 * max(1.0, scale), (t, d1, d2)
        for li in range(2):
            assert_ulp_close(caches[1].layers[li].kv, caches[0].layers[li].kv, f"layer {li} cache t={t}", ulps=2 if li else 1)


def test_eager_loop_reuses_its_per_layer_buffers(gpu_device):
    """A serving loop in eager mode: with ``reuse_buffers`` the rotated q, the output and the
    split-context workspace of a layer are allocated on its first call and used again by every
    later one - the allocator's event count stays flat over 50 frames - and the results are those
    of a twin cache whose calls allocate afresh.  Moving the cache drops the buffers."""
    dev = gpu_device
    B, H, Hkv, T, Dh, n = 1, 8, 8, 128, 128, 4
    p = Pair(dev, torch.bfloat16, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, n_layers=2, cfg_id=63)
    twin = Pair(dev, torch.bfloat16, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, n_layers=2, cfg_id=63)
    p.set_frozen(False)
    twin.set_frozen(False)
    assert ops.attn_workspace_bytes(B, H, Hkv, T, Dh, n * T) > 0, "the case must need a workspace"
    frames = []
    for t in range(50):
        q, k, v, pos = p.inputs(t % 7)
        pos = ro.synth_pos_ids(t, B, T, p.W)
        frames.append((q.to(dev), k.to(dev), v.to(dev), to_dev(pos, dev)))
    torch.cuda.synchronize()
    events = None
    for t, (q, k, v, pos) in enumerate(frames):
        outs = []
        for layer in range(2):
            y = p.hip.rope_upsert_attend(q, k, v, pos, p.rope, layer, reuse_buffers=True)
            ref = twin.hip.rope_upsert_attend(q, k, v, pos, twin.rope, layer)
            assert torch.equal(y, ref), f"frame {t} layer {layer}: reused buffers change the result"
            outs.append(y.data_ptr())
        if t == 0:
            first_ptrs = outs
        assert outs == first_ptrs and outs[0] != outs[1], "every layer keeps its own output buffer"
        del y, ref
        if t == 1:                               # steady state from the second frame on
            events = _alloc_events_of_reusing_calls(p, frames[1])
    assert events == 0, f"{events} allocations per frame in the steady state of the reusing path"
    assert len(p.hip.layers[0]._call_buffers) == 1
    p.hip.to(dev, torch.bfloat16)
    assert len(p.hip.layers[0]._call_buffers) == 0, "moving or casting the cache drops the call buffers"


def _alloc_events_of_reusing_calls(p, frame):
    """Allocator events (torch.cuda.memory_stats) caused by one more frame through the reusing path."""
    q, k, v, pos = frame
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    for layer in range(2):
        p.hip.rope_upsert_attend(q, k, v, pos, p.rope, layer, reuse_buffers=True)
    torch.cuda.synchronize()
    return torch.cuda.memory_stats()["allocation.all.allocated"] - before
