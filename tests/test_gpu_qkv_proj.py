"""GPU parity of the merged q/k/v projection fused with RoPE + the K/V store
(we_qkv_rope_kv_store / we_qkv_rope_kv_attn_fwd; src/patch_model.py:116-122 in front of
src/model/attn.py:105-116).

On dyadic operands (multiples of 1/8) every fp32 sum of the projection is exact whatever the
order of the additions, so everything the kernel writes - RoPE(q), cache rows, ``written``, the
projected v rows - must equal the oracle's bit for bit.  On random operands the projection may
differ from the oracle's in the last bit of the element type (summation order), so rows are
compared to 1 ulp of their largest value and the attention output to the usual 2e-2 / 2e-3.
"""
import pytest
import torch

from oracle import ring_oracle as ro
from _harness import Pair, assert_attn_close, assert_bits_equal, assert_ulp_close, to_dev
from world_engine_amd import ops

pytestmark = pytest.mark.gpu


def _operands(kind, seed, B, T, d_model, feats, dtype):
    if kind == "dyadic":
        return ro.synth_dyadic_linear(seed, B, T, d_model, feats, dtype)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, d_model, generator=g).to(dtype)
    w = (torch.randn(feats, d_model, generator=g) / d_model ** 0.5).to(dtype)
    return x, w


def _proj_step(p, t, frozen, x, w, attend=True, exact=True, **kw):
    """One frame through the oracle (projection, then layer_step) and through the fused call."""
    p.set_frozen(frozen)
    pos = ro.synth_pos_ids(t, p.B, p.T, p.W)
    q, k, v = ro.qkv_project(x, w, p.H, p.Hkv)
    ref, q_o = ro.layer_step(p.oracle, 0, q, k, v, pos, p.cos, p.sin, p.Hgrid, p.W, reference_dtype_flow=False,
                             qk_norm=bool(kw.get("qk_norm_eps")), v1=kw.get("v1"), v_lamb=kw.get("v_lamb"))
    lay = p.hip.layers[0]
    dkw = {k_: (v_.to(p.dev) if torch.is_tensor(v_) else v_) for k_, v_ in kw.items()}
    out, q_rot, v_raw = ops.qkv_rope_kv_attn(x.to(p.dev), w.to(p.dev), p.H, p.Hkv, to_dev(pos, p.dev), p.rope.cos,
                                             p.rope.sin, p.rope.height, p.rope.width, lay.kv, lay.written, lay.L,
                                             lay.pinned_dilation, frozen, attend=attend, want_v=True, **dkw)
    what = f"t={t} frozen={frozen}"
    assert torch.equal(lay.written.cpu(), p.oracle.layers[0].written), f"written {what}"
    if exact:
        assert_bits_equal(q_rot, q_o, f"RoPE(q) {what}")
        assert_bits_equal(v_raw, v, f"projected v {what}")
        p.assert_state_equal(what=what)
    else:
        assert_ulp_close(q_rot, q_o, f"RoPE(q) {what}")
        assert_ulp_close(v_raw, v, f"projected v {what}")
        assert_ulp_close(lay.kv, p.oracle.layers[0].kv, f"cache {what}")
    return out, ref


@pytest.mark.parametrize("dtype,Dh,H,Hkv,T,B,d_model", [
    (torch.bfloat16, 128, 4, 4, 128, 1, 256),
    (torch.bfloat16, 128, 4, 2, 96, 2, 128),     # grouped heads, a short last token tile, one contraction step
    (torch.float16, 128, 2, 2, 64, 1, 384),      # three contraction steps: the ring wraps exactly once
    (torch.bfloat16, 64, 6, 2, 72, 2, 512),      # two heads per feature tile, 10 x 64 features
    (torch.bfloat16, 64, 3, 1, 40, 1, 640),      # (H + 2 Hkv) Dh = 320 is not a whole number of feature tiles: refused
])
def test_projection_store_bit_exact_on_dyadic_operands(gpu_device, dtype, Dh, H, Hkv, T, B, d_model):
    print(f"qkv store dtype={dtype} Dh={Dh} H={H} Hkv={Hkv} T={T} B={B} d_model={d_model}", flush=True)
    feats = (H + 2 * Hkv) * Dh
    p = Pair(gpu_device, dtype, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=3, cfg_id=71)
    if feats % 128 != 0:
        x, w = ro.synth_dyadic_linear(0, B, T, d_model, feats, dtype)
        with pytest.raises(RuntimeError, match="we_qkv_rope_kv_store"):
            _proj_step(p, 0, False, x, w, attend=False)
        return
    for t in range(8):
        x, w = ro.synth_dyadic_linear(100 * t + 1, B, T, d_model, feats, dtype)
        _proj_step(p, t, t % 3 == 1, x, w, attend=False)


def test_projection_attend_cfg1_shape(gpu_device):
    """cfg1's module shapes (d_model 2048, 16 heads of 128, 256-token frames, 16-slot ring): exact
    on dyadic operands, then random operands to 1 ulp and the attention bar."""
    B, H, Hkv, T, Dh, d_model = 1, 16, 16, 256, 128, 2048
    feats = (H + 2 * Hkv) * Dh
    p = Pair(gpu_device, torch.bfloat16, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=16, cfg_id=72)
    for t in range(3):
        print(f"cfg1 dyadic t={t}", flush=True)
        x, w = ro.synth_dyadic_linear(200 + t, B, T, d_model, feats, torch.bfloat16)
        out, ref = _proj_step(p, t, False, x, w)
        # these v rows are sums of 2048 terms (magnitudes up to ~40, not ~4 as for unit-variance rows): the
        # absolute bar is applied to outputs brought to unit scale by an exact power of two
        assert_attn_close(out.float() / 16, ref / 16, f"dyadic t={t}")
    p = Pair(gpu_device, torch.bfloat16, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=16, cfg_id=73)
    _, w = _operands("random", 300, B, T, d_model, feats, torch.bfloat16)
    for t in list(range(4)) + [17, 18]:
        print(f"cfg1 random t={t}", flush=True)
        x, _ = _operands("random", 301 + t, B, T, d_model, feats, torch.bfloat16)
        out, ref = _proj_step(p, t, t == 2, x, w, exact=False)
        assert_attn_close(out, ref, f"random t={t}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_projection_with_norm_and_value_blend(gpu_device, dtype):
    """The store's optional steps behind the projection: weightless RMS norm of q and k rows and
    the value blend, against the oracle's layer_step with the same steps (1 ulp of a row's largest
    value, as for the store kernel); the projected v handed back is the one before the blend."""
    B, H, Hkv, T, Dh, d_model = 2, 4, 2, 128, 128, 256
    feats = (H + 2 * Hkv) * Dh
    p = Pair(gpu_device, dtype, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=3, cfg_id=74)
    eps = torch.finfo(torch.float32).eps
    g = torch.Generator().manual_seed(9)
    lamb = torch.tensor(0.37, dtype=dtype)
    for t in range(6):
        print(f"norm+blend dtype={dtype} t={t}", flush=True)
        x, w = ro.synth_dyadic_linear(400 + t, B, T, d_model, feats, dtype)
        v1 = torch.randn(B, Hkv, T, Dh, generator=g).to(dtype)
        out, ref = _proj_step(p, t, t % 3 == 1, x, w, exact=False, qk_norm_eps=eps, v1=v1, v_lamb=lamb)
        assert_attn_close(out, ref, f"t={t}")


def test_projection_rejects_bad_operands(gpu_device):
    dev = gpu_device
    p = Pair(dev, torch.bfloat16, B=1, H=2, Hkv=2, T=64, Dh=128, n_slots=2, cfg_id=75)
    lay = p.hip.layers[0]
    pos = to_dev(ro.synth_pos_ids(0, 1, 64, p.W), dev)
    args = (p.rope.cos, p.rope.sin, p.rope.height, p.rope.width, lay.kv, lay.written, lay.L, 1, False)
    x = torch.zeros(1, 64, 192, device=dev, dtype=torch.bfloat16)          # d_model not a multiple of 128
    w = torch.zeros(6 * 128, 192, device=dev, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.qkv_rope_kv_attn(x, w, 2, 2, pos, *args)
    x = torch.zeros(1, 64, 256, device=dev, dtype=torch.bfloat16)
    w = torch.zeros(5 * 128, 256, device=dev, dtype=torch.bfloat16)        # wrong number of weight rows
    with pytest.raises(RuntimeError):
        ops.qkv_rope_kv_attn(x, w, 2, 2, pos, *args)
    before = lay.kv.clone()
    torch.cuda.synchronize()
    assert torch.equal(before, lay.kv)


@pytest.mark.parametrize("compiled", [False, True])
def test_module_with_fused_projection(gpu_device, compiled):
    """RingAttn(fuse_projection=True) - x in, out_proj's input out, two library kernels and the
    combine in between - against the same module with the projection as a torch linear layer, two
    layers deep so that the first layer's projected v reaches the second as the value residual;
    also under torch.compile(fullgraph=True), where the call is the registered opaque op."""
    import types
    import world_engine_amd as wea
    torch.manual_seed(2)
    dev = gpu_device
    cfg = types.SimpleNamespace(d_model=512, n_heads=4, n_kv_heads=2, value_residual=True, gated_attn=True,
                                tokens_per_frame=64, local_window=3, global_window=3, global_attn_period=1,
                                global_pinned_dilation=1, n_layers=2)
    cos, sin = ro.rope_table_1d(16 * 64, 128)
    rope = wea.RoPE(cos, sin, 8, 8).to(dev)
    plain = [wea.RingAttn(cfg, i, rope, merged_qkv=True, fuse_elementwise=True).to(dev, torch.bfloat16)
             for i in range(2)]
    fused = [wea.RingAttn(cfg, i, rope, merged_qkv=True, fuse_elementwise=True, fuse_projection=True)
             .to(dev, torch.bfloat16) for i in range(2)]
    for a, b in zip(plain, fused):
        with torch.no_grad():
            a.gate_proj.weight.normal_(0, 0.5)
            a.v_lamb.fill_(0.3)
        b.load_state_dict(a.state_dict())
    run = [torch.compile(m, fullgraph=True) for m in fused] if compiled else fused
    caches = [wea.StaticKVCache(cfg, 1, torch.bfloat16).to(dev) for _ in range(2)]
    for c in caches:
        c.set_frozen(False)
        for layer in c.layers:
            layer.check_inputs = False
    for t in range(5):
        print(f"module fused projection compiled={compiled} t={t}", flush=True)
        x = torch.randn(1, 64, 512, device=dev, dtype=torch.bfloat16)
        pos = to_dev(ro.synth_pos_ids(t, 1, 64, 8), dev)
        with torch.no_grad():
            ya, v1a = plain[0](x, pos, None, caches[0])
            ya2, _ = plain[1](ya, pos, v1a, caches[0])
            yb, v1b = run[0](x, pos, None, caches[1])
            yb2, _ = run[1](yb, pos, v1b, caches[1])
        assert v1b.shape == v1a.shape
        assert_ulp_close(v1b, v1a, f"v1 t={t}")
        d1 = (ya.float() - yb.float()).abs().max().item()
        d2 = (ya2.float() - yb2.float()).abs().max().item()
        assert d1 <= 2e-2 * max(1.0, ya.float().abs().max().item()), (t, d1)
        assert d2 <= 3e-2 * max(1.0, ya2.float().abs().max().item()), (t, d2)
        for li in range(2):
            assert_ulp_close(caches[1].layers[li].kv, caches[0].layers[li].kv, f"layer {li} cache t={t}",
                             ulps=2 if li else 1)
            assert torch.equal(caches[1].layers[li].written, caches[0].layers[li].written)


def test_module_takes_the_linear_layer_beyond_one_round_of_workgroups(gpu_device):
    """1024-token frames of 16 heads need 768 projection workgroups: RingAttn(fuse_projection=True)
    takes the linear layer + the fuse_elementwise call there, so it matches the module built
    without fuse_projection bit for bit; a 256-token frame of the same module (192 workgroups)
    takes the projection kernel and agrees to rounding."""
    import types
    import world_engine_amd as wea
    torch.manual_seed(5)
    dev = gpu_device
    cos, sin = ro.rope_table_1d(8 * 1024, 128)
    for T, side in ((1024, 32), (256, 16)):
        cfg = types.SimpleNamespace(d_model=2048, n_heads=16, n_kv_heads=16, value_residual=False, gated_attn=False,
                                    tokens_per_frame=T, local_window=2, global_window=2, global_attn_period=1,
                                    global_pinned_dilation=1, n_layers=1)
        rope = wea.RoPE(cos, sin, side, side).to(dev)
        plain = wea.RingAttn(cfg, 0, rope, merged_qkv=True, fuse_elementwise=True).to(dev, torch.bfloat16)
        fused = wea.RingAttn(cfg, 0, rope, merged_qkv=True, fuse_elementwise=True, fuse_projection=True).to(dev, torch.bfloat16)
        fused.load_state_dict(plain.state_dict())
        assert fused.uses_fused_projection(1, T) == (T == 256)
        caches = [wea.StaticKVCache(cfg, 1, torch.bfloat16).to(dev) for _ in range(2)]
        for c in caches:
            c.set_frozen(False)
        for t in range(3):
            print(f"shape rule T={T} t={t}", flush=True)
            x = torch.randn(1, T, 2048, device=dev, dtype=torch.bfloat16)
            pos = to_dev(ro.synth_pos_ids(t, 1, T, side), dev)
            with torch.no_grad():
                ya, _ = plain(x, pos, None, caches[0])
                yb, _ = fused(x, pos, None, caches[1])
            if T == 1024:
                assert torch.equal(ya, yb), t
                assert torch.equal(caches[0].layers[0].kv, caches[1].layers[0].kv), t
            else:
                assert_ulp_close(caches[1].layers[0].kv, caches[0].layers[0].kv, f"cache t={t}")
                d = (ya.float() - yb.float()).abs().max().item()
                assert d <= 2e-2 * max(1.0, ya.float().abs().max().item()), (t, d)
            assert torch.equal(caches[0].layers[0].written, caches[1].layers[0].written)


def _proj_case(seed):
    import random
    r = random.Random(1000 + seed)
    Dh = r.choice([64, 128])
    while True:
        hkv = r.choice([1, 2, 3, 4])
        H = hkv * r.choice([1, 1, 2, 4])
        if (H + 2 * hkv) * Dh % 128 == 0:
            break
    d = r.choice([1, 1, 2])
    return dict(dtype=r.choice([torch.bfloat16, torch.bfloat16, torch.float16]), B=r.choice([1, 1, 2, 3]), Hkv=hkv, H=H,
                T=r.choice([8, 16, 40, 64, 72, 100, 128, 136, 200, 256, 320]), Dh=Dh, d=d, n_slots=d * r.choice([1, 2, 3]),
                d_model=128 * r.choice([1, 2, 3, 4, 5, 8, 9]), steps=r.choice([3, 5]), norm=r.choice([False, True]),
                blend=r.choice([False, True]))


@pytest.mark.parametrize("seed", list(range(16)))
def test_projection_random_geometry(gpu_device, seed):
    """Seeded sweep over the projection's shapes: batch, grouped heads, both head dims, frame
    lengths on and off the 64-token tile, contraction lengths of one to nine ring slots (fewer and
    more than the ring holds), pinned dilation, frozen calls, with and without the norm and the
    value blend.  Dyadic operands: without the norm / blend everything written is bit-identical to
    the oracle's; with them rows agree to 1 ulp of their largest value, as for the store kernel."""
    c = _proj_case(seed)
    print(f"projection seed {seed}: {c}", flush=True)
    feats = (c["H"] + 2 * c["Hkv"]) * c["Dh"]
    p = Pair(gpu_device, c["dtype"], B=c["B"], H=c["H"], Hkv=c["Hkv"], T=c["T"], Dh=c["Dh"], n_slots=c["n_slots"],
             d=c["d"], cfg_id=90 + seed)
    g = torch.Generator().manual_seed(seed)
    lamb = torch.tensor(0.3, dtype=c["dtype"])
    for t in range(c["steps"]):
        x, w = ro.synth_dyadic_linear(7000 + 10 * seed + t, c["B"], c["T"], c["d_model"], feats, c["dtype"])
        kw = {}
        if c["norm"]:
            kw["qk_norm_eps"] = torch.finfo(torch.float32).eps
        if c["blend"]:
            kw.update(v1=torch.randn(c["B"], c["Hkv"], c["T"], c["Dh"], generator=g).to(c["dtype"]), v_lamb=lamb)
        out, ref = _proj_step(p, t, t % 3 == 1, x, w, exact=not kw, **kw)
        # dyadic v rows have a standard deviation of about 0.4 sqrt(d_model): the absolute bar is applied to
        # outputs brought to unit scale by an exact power of two
        import math
        s = 2.0 ** math.ceil(math.log2(0.4 * math.sqrt(c["d_model"])))
        assert_attn_close(out.float() / s, ref / s, f"t={t}")
