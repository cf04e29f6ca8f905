"""A whole frame step - S forwards over every layer - captured in ONE HIP graph and replayed frame
after frame (``src/world_engine.py:139-152`` under ``mode="max-autotune"``): S-1 frozen calls, then
the persisting one, on a cache with mixed local/global windows and a pinned dilation above one
(``src/model/kv_cache.py:157-181``), positions from a three-axis rotary table.

Every replay is checked: cache rows and ``written`` bit for bit against the oracle's state
machine, attention within max-abs 2e-2 / mean-abs 2e-3 of the fp32 oracle, and outputs bit for
bit against the same calls launched eagerly on a second cache.
"""
from types import SimpleNamespace

import pytest
import torch

import world_engine_amd as wea
from oracle import ring_oracle as ro
from _harness import assert_attn_close, assert_bits_equal, to_dev

pytestmark = pytest.mark.gpu


def test_frame_step_graph_mixed_windows_and_dilation(gpu_device):
    dev = gpu_device
    B, H, Hkv, Dh, T, W, S, n_layers, n_frames = 1, 4, 2, 64, 64, 8, 3, 4, 14
    cfg = SimpleNamespace(tokens_per_frame=T, local_window=3, global_window=8, global_attn_period=2,
                          global_attn_offset=1, global_pinned_dilation=2, n_layers=n_layers, n_heads=H,
                          n_kv_heads=Hkv, d_model=H * Dh)
    rope = wea.RoPE.three_axis(n_frames, Dh, W, W).to(dev)
    cos, sin = rope.cos.cpu(), rope.sin.cpu()
    graph_cache = wea.StaticKVCache(cfg, B, torch.bfloat16).to(dev)
    eager_cache = wea.StaticKVCache(cfg, B, torch.bfloat16).to(dev)
    oracle_cache = ro.OracleStaticKVCache(cfg, B, torch.bfloat16)
    assert [(l.L // T, l.pinned_dilation) for l in graph_cache.layers] == [(3, 1), (8, 2), (3, 1), (8, 2)]

    shape_q, shape_kv = (B, H, T, Dh), (B, Hkv, T, Dh)
    q_s = [[torch.empty(shape_q, dtype=torch.bfloat16, device=dev) for _ in range(n_layers)] for _ in range(S)]
    k_s = [[torch.empty(shape_kv, dtype=torch.bfloat16, device=dev) for _ in range(n_layers)] for _ in range(S)]
    v_s = [[torch.empty(shape_kv, dtype=torch.bfloat16, device=dev) for _ in range(n_layers)] for _ in range(S)]
    pos_s = to_dev(ro.synth_pos_ids(0, B, T, W), dev)

    def frame(cache, outs):
        for u in range(S):
            cache.set_frozen(u < S - 1)
            for l in range(n_layers):
                outs[u][l] = cache.rope_upsert_attend(q_s[u][l], k_s[u][l], v_s[u][l], pos_s, rope, l)

    def fill(t):
        host = [[ro.synth_qkv(61, t, u * n_layers + l, B, H, Hkv, T, Dh, torch.bfloat16) for l in range(n_layers)]
                for u in range(S)]
        for u in range(S):
            for l in range(n_layers):
                q, k, v = host[u][l]
                q_s[u][l].copy_(q); k_s[u][l].copy_(k); v_s[u][l].copy_(v)
        pos_s["t_pos"].fill_(t)
        return host

    graph_out = [[None] * n_layers for _ in range(S)]
    eager_out = [[None] * n_layers for _ in range(S)]
    fill(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        frame(graph_cache, graph_out)        # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph_cache.reset()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        frame(graph_cache, graph_out)
    graph_cache.reset()

    for t in range(n_frames):
        print(f"frame graph replay t={t}", flush=True)
        host = fill(t)
        graph.replay()
        torch.cuda.synchronize()
        frame(eager_cache, eager_out)
        torch.cuda.synchronize()
        pos = ro.synth_pos_ids(t, B, T, W)
        for u in range(S):
            oracle_cache.set_frozen(u < S - 1)
            for l in range(n_layers):
                q, k, v = host[u][l]
                ref, _ = ro.layer_step(oracle_cache, l, q, k, v, pos, cos, sin, W, W, reference_dtype_flow=False)
                assert torch.equal(graph_out[u][l], eager_out[u][l]), f"graph != eager at t={t} u={u} layer={l}"
                assert_attn_close(graph_out[u][l], ref, f"t={t} u={u} layer={l}")
        for l in range(n_layers):
            assert_bits_equal(graph_cache.layers[l].kv, oracle_cache.layers[l].kv, f"kv t={t} layer={l}")
            assert torch.equal(graph_cache.layers[l].written.cpu(), oracle_cache.layers[l].written), (t, l)
            assert torch.equal(graph_cache.layers[l].kv, eager_cache.layers[l].kv)
