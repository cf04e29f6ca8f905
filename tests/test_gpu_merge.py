"""Split-context parts merged by the main kernel itself (the last workgroup of a query tile to
arrive reads the others' partial rows out of its XCD's L2) against the same call with the second
kernel doing the merge (``two_pass``): the two routes share their arithmetic, so outputs are
compared bit for bit, and both against the fp32 oracle at the usual tolerance.  The arrival
counters at the start of the workspace must be back at zero after every call."""
import pytest
import torch

from oracle import ring_oracle as ro
from world_engine_amd import _capi, ops
from _harness import Pair, assert_attn_close, assert_bits_equal

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


def _frames(p, n_frames, frozen_subs=0, **kw):
    """Runs the schedule; every call once per route with its own workspace."""
    dev = p.dev
    L = p.n * p.T
    nbytes = ops.attn_workspace_bytes(p.B, p.H, p.Hkv, p.T, p.Dh, L, kw.get("n_splits", 0), kw.get("q_tile", 0))
    assert nbytes > _capi.WE_WS_COUNTER_BYTES, "the case must split the context"
    ws_a, ws_b = ops.new_workspace(nbytes, dev), ops.new_workspace(nbytes, dev)
    ws_a[_capi.WE_WS_COUNTER_BYTES:].fill_(0x7f)      # whatever the partial rows held before must not matter
    for t in range(n_frames):
        for sub in range(frozen_subs + 1):
            p.set_frozen(sub < frozen_subs)
            q, k, v, pos = p.inputs(t, sub)
            (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos)
            merged = p.attend(q_h, ring, workspace=ws_a, **kw)
            two = p.attend(q_h, ring, workspace=ws_b, two_pass=True, **kw)
            assert_bits_equal(merged, two, f"in-kernel merge vs second kernel, t={t} sub={sub} {kw}")
            assert_attn_close(merged, ro.attention_fp32(q_o, k_all, v_all, mask), f"t={t} sub={sub} {kw}")
            assert not ws_a[: _capi.WE_WS_COUNTER_BYTES].any(), f"arrival counters not back at zero, t={t}"
            assert not ws_b[: _capi.WE_WS_COUNTER_BYTES].any(), "the two-pass route must not touch the counters"


def test_device_passes_the_xcd_check(gpu_device):
    """On an MI355X workgroup id % 8 names the XCD, so the merge route is what the library picks."""
    ops.init(gpu_device)
    assert ops.attn_plan(1, 8, 8, 128, 64, 4 * 128, 2, xcd_merge=None)["merge_in_kernel"], "the device failed the XCD check"
    p = Pair(gpu_device, torch.bfloat16, B=1, H=8, Hkv=8, T=128, Dh=64, n_slots=4, cfg_id=81)
    p.set_frozen(False)
    q, k, v, pos = p.inputs(0)
    (_, _, _, _), (q_h, ring) = p.store(q, k, v, pos)
    ws = ops.new_workspace(ops.attn_workspace_bytes(1, 8, 8, 128, 64, 4 * 128, 2), gpu_device)
    ws[_capi.WE_WS_COUNTER_BYTES:].fill_(0xff)       # fp16 NaN patterns: a part that nobody wrote would show
    sentinel = ws.clone()
    p.attend(q_h, ring, workspace=ws, n_splits=2, two_pass=True)
    torch.cuda.synchronize()
    assert not torch.equal(ws, sentinel)
    # the in-kernel route writes the same partial rows (and merges them itself)
    ws2 = sentinel.clone()
    p.attend(q_h, ring, workspace=ws2, n_splits=2)
    torch.cuda.synchronize()
    assert torch.equal(ws2, ws), "both routes leave the same partial results in the workspace"


def test_cfg1_shape_all_32_steps(gpu_device):
    _say("merge: cfg1 shape")
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=16, cfg_id=1)
    _frames(p, 20)


def test_cfg4_shape_with_frozen_substeps(gpu_device):
    _say("merge: cfg4 shape")
    p = Pair(gpu_device, torch.bfloat16, B=1, H=16, Hkv=16, T=256, Dh=128, n_slots=32, cfg_id=4)
    _frames(p, 3, frozen_subs=2)


def test_cfg3_tail_split(gpu_device):
    """Benchmark configuration 3: 64 whole units and 32 units cut in two in one launch of 256-query
    workgroups; the halves are merged by whichever finishes second."""
    _say("merge: cfg3 shape")
    p = Pair(gpu_device, torch.bfloat16, B=4, H=24, Hkv=24, T=1024, Dh=128, n_slots=8, cfg_id=3)
    _frames(p, 2)


@pytest.mark.parametrize("dtype,B,H,Hkv,T,Dh,n_slots,kw", [
    (torch.bfloat16, 2, 16, 8, 128, 128, 6, {"n_splits": 3}),                 # grouped heads, two batches
    (torch.float16, 1, 8, 8, 128, 64, 5, {"n_splits": 4}),
    (torch.bfloat16, 1, 8, 8, 200, 128, 4, {"n_splits": 3}),                  # frame length off the tile grid, ragged query tile
    (torch.bfloat16, 1, 16, 8, 72, 64, 6, {"n_splits": 2, "q_tile": 256}),
    (torch.bfloat16, 1, 8, 8, 128, 128, 20, {"n_splits": 12}),                # more parts than one batch of the merge
    (torch.bfloat16, 1, 8, 8, 64, 128, 24, {}),                               # the planner's own choice for a small call (12 parts)
    (torch.bfloat16, 8, 2, 1, 320, 64, 3, {"n_splits": 2, "q_tile": 128}),
    (torch.bfloat16, 1, 64, 64, 128, 64, 6, {"n_splits": 8}),                 # 512 workgroups: nobody waits, the last part in merges every share
    (torch.bfloat16, 1, 8, 8, 128, 128, 40, {"n_splits": 16}),                # sixteen parts, two batches per item
])
def test_shapes(gpu_device, dtype, B, H, Hkv, T, Dh, n_slots, kw):
    _say(f"merge: {dtype} B={B} H={H} Hkv={Hkv} T={T} Dh={Dh} slots={n_slots} {kw}")
    plan = ops.attn_plan(B, H, Hkv, T, Dh, n_slots * T, kw.get("n_splits", 0), kw.get("q_tile", 0))
    assert plan["merge_in_kernel"], plan
    p = Pair(gpu_device, dtype, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n_slots, cfg_id=82)
    _frames(p, n_slots + 2 if n_slots <= 6 else 3, **kw)


def test_merge_with_head_gate(gpu_device):
    """The head gate of the one-call entry point is applied by whoever merges."""
    dev = gpu_device
    B, H, Hkv, T, Dh, n = 1, 8, 8, 128, 128, 4
    p = Pair(dev, torch.bfloat16, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, cfg_id=83)
    g = torch.Generator("cpu").manual_seed(3)
    layer = p.hip.layers[0]
    twin = Pair(dev, torch.bfloat16, B=B, H=H, Hkv=Hkv, T=T, Dh=Dh, n_slots=n, cfg_id=83).hip.layers[0]
    for t in range(5):
        q, k, v, pos = p.inputs(t)
        gate = torch.sigmoid(torch.randn(B, T, H, generator=g)).to(torch.bfloat16).to(dev).permute(0, 2, 1)
        posd = {k_: v_.to(dev) for k_, v_ in pos.items()}
        args = (q.to(dev), k.to(dev), v.to(dev), posd, p.rope.cos, p.rope.sin, p.rope.height, p.rope.width)
        a, _ = ops.rope_kv_attn(*args, layer.kv, layer.written, layer.L, 1, False, n_splits=3, gate=gate)
        b, _ = ops.rope_kv_attn(*args, twin.kv, twin.written, twin.L, 1, False, n_splits=3, gate=gate,
                                q_tile=_capi.WE_SPLIT_TWO_PASS)
        assert_bits_equal(a, b, f"gated output t={t}")


def test_graph_replay_of_the_merging_kernel(gpu_device):
    """Captured once (after the device's set-up), replayed for ten frames with eager work in
    between: the counters reset themselves, so every replay must equal the eager two-pass result."""
    dev = gpu_device
    p = Pair(dev, torch.bfloat16, B=1, H=8, Hkv=8, T=128, Dh=128, n_slots=4, cfg_id=84)
    p.set_frozen(False)
    eager = Pair(dev, torch.bfloat16, B=1, H=8, Hkv=8, T=128, Dh=128, n_slots=4, cfg_id=84)
    eager.set_frozen(False)
    qs, ks, vs = (torch.empty(1, 8, 128, 128, dtype=torch.bfloat16, device=dev) for _ in range(3))
    pos_s = {k_: v_.to(dev) for k_, v_ in ro.synth_pos_ids(0, 1, 128, p.W).items()}
    layer = p.hip.layers[0]
    out_s = torch.empty(1, 8, 128, 128, dtype=torch.bfloat16, device=dev)
    ws = ops.new_workspace(ops.attn_workspace_bytes(1, 8, 8, 128, 128, layer.L, 4), dev)

    def step():
        q_rot = ops.rope_kv_store(qs, ks, vs, pos_s, p.rope.cos, p.rope.sin, p.Hgrid, p.W, layer.kv,
                                  layer.written, layer.L, 1, False)
        ops.attn_ring(q_rot, layer.kv, layer.written, pos_s["t_pos"], layer.L, 1, n_splits=4, out=out_s, workspace=ws)

    ops.init(dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
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
        ref = eager.attend(q_h, ring, n_splits=4, token_major_out=False, two_pass=True)
        assert torch.equal(out_s, ref), f"replay {t} differs from the eager two-pass result"
        assert not ws[: _capi.WE_WS_COUNTER_BYTES].any()
