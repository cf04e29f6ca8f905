"""The committed snapshot tests/golden/ring_cfg0_bf16.npz (written by
tests/golden/make_ring_vectors.py) against the CPU oracle (drift guard, CPU suite) and against the
HIP path through the C ABI (GPU suite).  Cache bytes and RoPE(q) are compared bit for bit (SHA-256 /
raw bits); attention within max-abs 2e-2 / mean-abs 2e-3 of the stored fp32 result."""
import hashlib
import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
NPZ = os.path.join(HERE, "golden", "ring_cfg0_bf16.npz")

spec = importlib.util.spec_from_file_location("make_ring_vectors", os.path.join(HERE, "golden", "make_ring_vectors.py"))
gen = importlib.util.module_from_spec(spec)
spec.loader.exec_module(gen)


def load():
    return np.load(NPZ, allow_pickle=False)


def test_fixture_is_complete():
    g = load()
    assert len(g["kv_sha256"]) == gen.CFG["steps"] == len(g["written_sha256"])
    for s in gen.CFG["keep"]:
        assert g[f"attn_fp32_step{s}"].shape == (1, 8, 64, 64) and g[f"attn_fp32_step{s}"].dtype == np.float32
        assert g[f"q_rot_bits_step{s}"].dtype == np.int16
    assert len(set(g["kv_sha256"].tolist())) == gen.CFG["steps"]          # every step changes the cache


def test_oracle_reproduces_fixture():
    g, now = load(), gen.run()
    assert now["kv_sha256"] == g["kv_sha256"].tolist()
    assert now["written_sha256"] == g["written_sha256"].tolist()
    for s in gen.CFG["keep"]:
        assert np.array_equal(now[f"q_rot_bits_step{s}"], g[f"q_rot_bits_step{s}"])
        np.testing.assert_allclose(now[f"attn_fp32_step{s}"], g[f"attn_fp32_step{s}"], rtol=0, atol=2e-6)


@pytest.mark.gpu
def test_hip_path_matches_fixture():
    from types import SimpleNamespace
    from oracle import ring_oracle as ro          # seeded inputs and the RoPE table only
    import world_engine_amd as wea
    from world_engine_amd import ops
    from _harness import merged_views, MAX_ABS, MEAN_ABS

    g, c = load(), gen.CFG
    dev = torch.device("cuda:0")
    B, H, Hkv, Dh, T, n = c["B"], c["H"], c["Hkv"], c["Dh"], c["T"], c["n_slots"]
    conf = SimpleNamespace(tokens_per_frame=T, local_window=n, global_window=n, global_attn_period=1,
                           global_pinned_dilation=1, n_layers=1, n_heads=H, n_kv_heads=Hkv, d_model=H * Dh)
    cache = wea.StaticKVCache(conf, B, torch.bfloat16).to(dev)
    cache.set_frozen(False)
    cos_t, sin_t = ro.rope_table_1d(64 * T, Dh)
    rope = wea.RoPE(cos_t, sin_t, 8, 8).to(dev)

    def digest(t):
        return hashlib.sha256(t.cpu().contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()

    for step in range(c["steps"]):
        q, k, v = ro.synth_qkv(c["cfg_id"], step, 0, B, H, Hkv, T, Dh, torch.bfloat16)
        pos = {kk: vv.to(dev) for kk, vv in ro.synth_pos_ids(step, B, T, 8).items()}
        qd, kd, vd = merged_views(q.to(dev), k.to(dev), v.to(dev))
        q_rot, _, _, ring = cache.rope_upsert(qd, kd, vd, pos, rope, 0)
        assert digest(cache.layers[0].kv) == g["kv_sha256"][step], f"cache bytes differ at step {step}"
        assert digest(cache.layers[0].written) == g["written_sha256"][step], f"written differs at step {step}"
        if step in c["keep"]:
            assert np.array_equal(q_rot.cpu().contiguous().view(torch.int16).numpy(), g[f"q_rot_bits_step{step}"])
            out = ops.attn_ring(q_rot, ring.kv, ring.written, ring.t_pos, ring.L, ring.dilation)
            diff = np.abs(out.float().cpu().numpy() - g[f"attn_fp32_step{step}"])
            assert diff.max() <= MAX_ABS and diff.mean() <= MEAN_ABS, (step, diff.max(), diff.mean())
