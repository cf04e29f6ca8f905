"""The allocation-free entry point (we_attn_ring_fwd_static, split-context partials in a buffer that
is part of the library's device image) against we_attn_ring_fwd with a caller-owned workspace:
same kernels, so outputs are compared bit for bit, and against the fp32 oracle at the usual
tolerance.  Two calls in a row, the second on a smaller input, so that whatever the first call
left in the shared buffer is there when the second runs."""
import ctypes

import pytest
import torch

from oracle import ring_oracle as ro
from world_engine_amd import _capi, ops
from _harness import Pair, assert_attn_close

pytestmark = pytest.mark.gpu


def _both(p, t, n_splits=0, q_tile=0):
    """One frame through store + both attention entry points; returns (static out, workspace out, oracle)."""
    q, k, v, pos = p.inputs(t)
    (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
    base = ops.attn_ring(q_h, ring.kv, ring.written, ring.t_pos, ring.L, ring.dilation, n_splits=n_splits, q_tile=q_tile)
    out = torch.full_like(base, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]        # hipMemGetInfo: what the driver itself has handed out
    ops.attn_ring_static(q_h, ring.kv, ring.written, ring.t_pos, ring.L, ring.dilation, out, n_splits=n_splits,
                         q_tile=q_tile)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before, "the static entry point must not allocate through torch"
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point must not allocate device memory at all"
    return out, base, ro.attention_fp32(q_o, k_all, v_all, mask)


def test_static_scratch_entry_point_matches_workspace_entry_point(gpu_device):
    print("no-alloc: large call (B=1 H=16 T=256 Dh=128, 6 slots, auto splits)", flush=True)
    big = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=6, cfg_id=71)
    big.set_frozen(False)
    assert ops.attn_workspace_bytes(1, 16, 16, 256, 128, 6 * 256) > 0, "the case must use the split-context scratch"
    for t in range(8):                      # through the wrap, so later frames see a full ring
        out, base, ref = _both(big, t)
        assert torch.equal(out, base), f"large call, frame {t}: static and workspace entry points differ"
        assert_attn_close(out, ref, f"large call, frame {t}")
    print("no-alloc: smaller call right after (B=2 H=4 Hkv=2 T=128 Dh=64, 3 slots, 3 splits)", flush=True)
    small = Pair(gpu_device, torch.bfloat16, B=2, H=4, Hkv=2, T=128, Dh=64, n_slots=3, cfg_id=72)
    small.set_frozen(False)
    for t in range(5):
        out, base, ref = _both(small, t, n_splits=3)
        assert torch.equal(out, base), f"small call, frame {t}: static and workspace entry points differ"
        assert_attn_close(out, ref, f"small call, frame {t}")
    # and the large one again: the buffer now holds the small call's partials
    out, base, ref = _both(big, 8)
    assert torch.equal(out, base)
    assert_attn_close(out, ref, "large call after the small one")


def test_static_scratch_limit_and_unsplit_calls(gpu_device):
    lib = _capi.lib()
    dev = gpu_device
    # a call that needs no scratch (single pass) works and matches
    p = Pair(dev, torch.bfloat16, B=1, H=2, Hkv=2, T=64, Dh=64, n_slots=2, cfg_id=73)
    p.set_frozen(False)
    out, base, ref = _both(p, 0, n_splits=1)
    assert torch.equal(out, base)
    # sizes whose partials do not fit the buffer are refused before anything is launched:
    # B=8, H=32, T=256 with 8 splits needs 8 * 65536 rows * 272 bytes = 136 MiB
    need = ops.attn_workspace_bytes(8, 32, 32, 256, 128, 4 * 256, 8, 0)
    assert need > _capi.WE_STATIC_SCRATCH_BYTES
    s3 = _capi.i64x3(256 * 128, 128, 128 * 32)
    fake = ctypes.c_void_p(4096)             # never dereferenced: the size check comes first
    rc = lib.we_attn_ring_fwd_static(fake, s3, fake, fake, fake, fake, s3, 8, 32, 32, 256, 128, 4 * 256, 1, 0.1, 8, 0, 0, None)
    assert rc == _capi.WE_ERR_SCRATCH_LIMIT
    assert b"static buffer" in lib.we_error_string(rc)
    # argument errors are those of we_attn_ring_fwd
    assert lib.we_attn_ring_fwd_static(None, s3, fake, fake, fake, fake, s3, 1, 1, 1, 64, 64, 64, 1, 0.1, 1, 0, 0, None) == -1
    assert lib.we_attn_ring_fwd_static(fake, s3, fake, fake, fake, fake, s3, 1, 1, 1, 64, 96, 64, 1, 0.1, 1, 0, 0, None) == -3


def test_static_entry_point_under_graph_capture(gpu_device):
    """What the entry point is for: captured into a HIP graph (after the device's one-time set-up,
    which an eager call or ops.init() does and a capture cannot), replayed with eager work and
    synchronisations in between, every replay compared with the workspace entry point's result."""
    dev = gpu_device
    ops.init(dev)
    p = Pair(dev, torch.bfloat16, B=1, H=8, Hkv=8, T=128, Dh=128, n_slots=4, cfg_id=74)
    eager = Pair(dev, torch.bfloat16, B=1, H=8, Hkv=8, T=128, Dh=128, n_slots=4, cfg_id=74)
    p.set_frozen(False)
    eager.set_frozen(False)
    layer = p.hip.layers[0]
    q_s = torch.empty(1, 8, 128, 128, dtype=torch.bfloat16, device=dev)
    out_s = torch.empty(1, 8, 128, 128, dtype=torch.bfloat16, device=dev)
    t_s = torch.zeros(1, 128, dtype=torch.long, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                    # one eager call before the capture
        ops.attn_ring_static(q_s, layer.kv, layer.written, t_s, layer.L, 1, out_s, n_splits=3)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.attn_ring_static(q_s, layer.kv, layer.written, t_s, layer.L, 1, out_s, n_splits=3)
    for t in range(6):
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos, strided=False)     # eager store into the captured cache
        q_s.copy_(q_h)
        t_s.fill_(t)
        graph.replay()
        torch.cuda.synchronize()
        (_, _, _, _), (q_e, ring_e) = eager.store(q, k, v, pos, strided=False)
        base = eager.attend(q_e, ring_e, n_splits=3, token_major_out=False)
        assert torch.equal(out_s, base), f"replay {t}: static entry point under a graph differs from the workspace entry point"
        assert_attn_close(out_s, ro.attention_fp32(q_o, k_all, v_all, mask), f"replay {t}")
    assert torch.cuda.mem_get_info()[0] >= free_before - (8 << 20), "replays must not grow device memory"
