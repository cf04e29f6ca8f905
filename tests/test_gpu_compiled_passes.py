"""The reference compiles a whole denoise pass and a whole cache pass - S-1 frozen forwards,
then one persisting forward, over every layer - with
``torch.compile(fullgraph=True, mode="max-autotune", dynamic=False)``
(``src/world_engine.py:139-152``).  The same here, over a stack of four ``RingAttn`` layers with
mixed local / global windows and a pinned dilation (``src/model/kv_cache.py:157-181``): no graph
break, and what the library is given inside the compiled passes is checked call by call against
the oracle - cache rows and ``written`` bit for bit, attention within max-abs 2e-2 / mean-abs 2e-3.

The projections, norms and Euler updates around the library call are Inductor's own code and may
round differently from eager PyTorch, so the oracle is fed the very q / k / v each library call
received (recorded whenever the op's Python body runs, which it does not when a captured graph
of the pass is replayed; the cache state is then compared with a second, eagerly driven stack)."""
from types import SimpleNamespace

import pytest
import torch
from torch import nn

import world_engine_amd as wea
from world_engine_amd import ops
from oracle import ring_oracle as ro
from _harness import assert_attn_close, assert_bits_equal, to_dev

pytestmark = pytest.mark.gpu


class Stack(nn.Module):
    """Four attention layers with residual connections: the part of WorldDiT.forward that touches
    the cache (src/model/world_model.py:204-208, :166)."""

    def __init__(self, cfg, rope):
        super().__init__()
        self.blocks = nn.ModuleList([wea.RingAttn(cfg, i, rope, merged_qkv=True) for i in range(cfg.n_layers)])

    def forward(self, x, pos_ids, kv_cache):
        v1 = None
        for blk in self.blocks:
            y, v1 = blk(x, pos_ids, v1, kv_cache)
            x = x + y
        return x


def test_compiled_denoise_and_cache_passes(gpu_device, monkeypatch):
    dev = gpu_device
    B, H, Hkv, Dh, T, W, n_layers, n_frames = 1, 4, 2, 64, 64, 8, 4, 7
    cfg = SimpleNamespace(d_model=H * Dh, n_heads=H, n_kv_heads=Hkv, value_residual=True, gated_attn=True,
                          tokens_per_frame=T, local_window=2, global_window=4, global_attn_period=2,
                          global_attn_offset=1, global_pinned_dilation=2, n_layers=n_layers)
    torch.manual_seed(11)
    rope = wea.RoPE.one_dimensional(n_frames * T, Dh, W, W).to(dev)
    model = Stack(cfg, rope).to(dev, torch.bfloat16)
    # the tables as the kernels see them: a dtype cast of the parent model leaves them fp32 but
    # passes their values through the requested type, exactly as the reference's NoCastModule
    # does to its RoPE buffers (src/model/nn.py:10-24)
    cos, sin = rope.cos.cpu(), rope.sin.cpu()
    assert cos.dtype == torch.float32 and torch.equal(cos, cos.bfloat16().float())
    with torch.no_grad():
        for blk in model.blocks:
            blk.gate_proj.weight.normal_(0, 0.5)
            blk.v_lamb.fill_(0.3)
            blk.out_proj.weight.mul_(0.25)
    sigmas = torch.tensor([1.0, 0.6, 0.25, 0.0])           # three frozen forwards per frame
    steps = list(zip(sigmas.tolist(), sigmas.diff().tolist()))

    def denoise_pass(x, pos_ids, kv_cache):                # src/world_engine.py:139-146
        kv_cache.set_frozen(True)
        for _sig, dsig in steps:
            v = model(x, pos_ids, kv_cache)
            x = x + dsig * v
        return x

    def cache_pass(x, pos_ids, kv_cache):                  # src/world_engine.py:148-152
        kv_cache.set_frozen(False)
        model(x, pos_ids, kv_cache)

    compiled_cache = wea.StaticKVCache(cfg, B, torch.bfloat16).to(dev)
    eager_cache = wea.StaticKVCache(cfg, B, torch.bfloat16).to(dev)
    oracle = ro.OracleStaticKVCache(cfg, B, torch.bfloat16)
    layer_of = {l.kv.data_ptr(): i for i, l in enumerate(compiled_cache.layers)}
    assert [(l.L // T, l.pinned_dilation) for l in compiled_cache.layers] == [(2, 1), (4, 2), (2, 1), (4, 2)]

    # record what every library call inside the compiled passes receives and returns
    calls = []
    real = ops.rope_kv_attn

    def recording(q, k, v, pos_ids, *args, **kw):
        res = real(q, k, v, pos_ids, *args, **kw)
        kv = args[4]
        if kv.data_ptr() in layer_of and not torch.cuda.is_current_stream_capturing():
            # host copies: device memory allocated here would sit in the compiled pass's graph pool
            calls.append(dict(layer=layer_of[kv.data_ptr()], q=q.cpu(), k=k.cpu(), v=v.cpu(),
                              pos={n: p.cpu() for n, p in pos_ids.items()}, frozen=bool(args[8]), out=res[0].cpu()))
        return res

    monkeypatch.setattr(ops, "rope_kv_attn", recording)
    c_denoise = torch.compile(denoise_pass, fullgraph=True, mode="max-autotune", dynamic=False)
    c_cache = torch.compile(cache_pass, fullgraph=True, mode="max-autotune", dynamic=False)

    def check_calls(expected, what):
        """Every recorded call against the oracle, in order; returns False when the pass ran as a
        replayed graph (nothing recorded)."""
        if not calls:
            return False
        assert len(calls) == expected, f"{what}: {len(calls)} library calls recorded, {expected} expected"
        for i, c in enumerate(calls):
            oracle.set_frozen(c["frozen"])
            ref, _ = ro.layer_step(oracle, c["layer"], c["q"], c["k"], c["v"], c["pos"], cos, sin, W, W,
                                   reference_dtype_flow=False)
            assert_attn_close(c["out"], ref, f"{what} call {i} layer {c['layer']}")
        calls.clear()
        return True

    def check_state(what):
        for l in range(n_layers):
            assert_bits_equal(compiled_cache.layers[l].kv, oracle.layers[l].kv, f"{what}: kv layer {l}")
            assert torch.equal(compiled_cache.layers[l].written.cpu(), oracle.layers[l].written), f"{what}: written layer {l}"

    def adopt_state():
        for l in range(n_layers):
            oracle.layers[l].kv.copy_(compiled_cache.layers[l].kv.cpu())
            oracle.layers[l].written.copy_(compiled_cache.layers[l].written.cpu())

    recorded_passes = 0
    with torch.no_grad():
        for t in range(n_frames):
            print(f"compiled passes: frame {t}", flush=True)
            x = torch.randn(B, T, H * Dh, device=dev, dtype=torch.bfloat16)
            pos = to_dev(ro.synth_pos_ids(t, B, T, W), dev)
            x0 = c_denoise(x, pos, compiled_cache).clone()
            torch.cuda.synchronize()
            if check_calls(len(steps) * n_layers, f"denoise pass t={t}"):
                check_state(f"after the denoise pass t={t}")
                recorded_passes += 1
            else:
                adopt_state()
            c_cache(x0, pos, compiled_cache)
            torch.cuda.synchronize()
            if check_calls(n_layers, f"cache pass t={t}"):
                check_state(f"after the cache pass t={t}")
                recorded_passes += 1
            else:
                adopt_state()
            # the same two passes driven eagerly on a second cache, from the same inputs
            monkeypatch.setattr(ops, "rope_kv_attn", real)
            x0_e = denoise_pass(x, pos, eager_cache)
            cache_pass(x0, pos, eager_cache)               # from the compiled pass's x0: same K/V up to rounding
            monkeypatch.setattr(ops, "rope_kv_attn", recording)
            torch.cuda.synchronize()
            d = (x0.float() - x0_e.float()).abs()
            assert d.max().item() <= 6e-2 * max(1.0, x0_e.float().abs().max().item()), f"t={t}: compiled vs eager x0 {d.max().item():.3e}"
            for l in range(n_layers):
                a, b = compiled_cache.layers[l], eager_cache.layers[l]
                assert torch.equal(a.written, b.written)
                dk = (a.kv.float() - b.kv.float()).abs().max().item()
                assert dk <= 2.0 ** -6 * max(1.0, b.kv.float().abs().max().item()), f"t={t} layer {l}: caches differ by {dk:.3e}"
    assert recorded_passes >= 2, "the library calls of at least the first frame's passes must have been checked one by one"
    # the ring wrapped on the local layers and pinned every second frame on the global ones
    assert compiled_cache.layers[0].written[: 2 * T].all() and compiled_cache.layers[1].written[: 2 * T].all()
    assert not compiled_cache.layers[1].written[2 * T: 4 * T].any()
