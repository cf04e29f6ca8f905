#!/usr/bin/env python3
"""Benchmark of the frame-causal ring-buffer attention hot path on one MI355X.

A *step* is one frame-step of one attention layer: the fused RoPE + ring-slot K/V store followed
by the attention over the ring (one we_rope_kv_store call + one we_attn_ring_fwd call through the
C ABI).  The default workload is benchmark configuration 1 (B=1, H=16, Dh=128, 256 tokens per frame,
16-slot ring, bf16); ``--config 2|3|4`` select the other single-GPU configurations.  Inputs are
synthetic N(0,1) tensors already resident in HBM, laid out like the merged QKV projection output.
The timed region replays a HIP graph holding exactly K consecutive steps (the ring advances every
step, as in the real schedule), bracketed by device synchronisation.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0       # MI355X HBM3E, published
PEAK_BF16_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published

# HBM-side bytes per attention call (attn_ring_kernel + attn_combine_kernel, reads + writes) from
# two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) with the library's own split/tile choice, each
# scaled by the same counter's reading for a 256 MiB copy kernel (FETCH_SIZE x2.000, WRITE_SIZE
# x1.000); the summaries are profiles/attn_ring_cfg{1,3}_hbm_traffic.txt.
MEASURED_TRAFFIC = {1: 60658972, 3: 496861378}

CONFIGS = {
    1: dict(name="cfg1: B=1 H=16 Dh=128 T=256 16-slot ring (4096-token context) bf16, steady-state wrap",
            B=1, H=16, Hkv=16, Dh=128, T=256, slots=16, layers=1, frozen_subs=0, bound="hbm"),
    2: dict(name="cfg2: 24 layers x cfg1 shapes, own ring per layer, K outlier channel",
            B=1, H=16, Hkv=16, Dh=128, T=256, slots=16, layers=24, frozen_subs=0, bound="hbm", outlier=True),
    3: dict(name="cfg3: B=4 H=24 Dh=128 T=1024 8-slot ring (8192-token context) bf16",
            B=4, H=24, Hkv=24, Dh=128, T=1024, slots=8, layers=1, frozen_subs=0, bound="mfma"),
    4: dict(name="cfg4: B=1 H=16 Dh=128 T=256 32-slot ring, 4 frozen substeps + 1 persisting call per frame",
            B=1, H=16, Hkv=16, Dh=128, T=256, slots=32, layers=1, frozen_subs=4, bound="hbm"),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_work(c, n_vis):
    """Per attention call: flops = 4*B*H*T*N_vis*Dh; bytes = 2*[2*B*Hkv*N_vis*Dh + 2*B*H*T*Dh]
    (bf16 K and V of the visible keys read once, Q read, O written)."""
    flops = 4.0 * c["B"] * c["H"] * c["T"] * n_vis * c["Dh"]
    byts = 2.0 * (2.0 * c["B"] * c["Hkv"] * n_vis * c["Dh"] + 2.0 * c["B"] * c["H"] * c["T"] * c["Dh"])
    return flops, byts


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--config", type=int, default=1, choices=sorted(CONFIGS))
    ap.add_argument("--n-splits", type=int, default=0, help="context splits (0 = library's choice)")
    ap.add_argument("--q-tile", type=int, default=0, help="queries per workgroup (0 = library's choice)")
    ap.add_argument("--eager", action="store_true", help="launch from Python per call instead of a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--two-calls", action="store_true",
                    help="we_rope_kv_store + we_attn_ring_fwd instead of the one-call we_rope_kv_attn_fwd")
    ap.add_argument("--attn-iters", type=int, default=200, help="attention-only launches for the roofline timing")
    ap.add_argument("--batch", type=int, default=0, help="override the configuration's batch size (experiments)")
    ap.add_argument("--peaks", action="store_true",
                    help="also measure what this box reaches on a plain bf16 GEMM (hipBLASLt through torch) and on a "
                         "streaming copy, and add them to the JSON as measured_peaks")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="also launch 20 plain copy kernels (read MiB, write MiB each) so a counter run holds "
                         "a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the single-GPU hot path only: this build has no multi-GPU path "
              "(heads and batch streams would shard with no communication); run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from oracle import ring_oracle as ro           # inputs + the cpu_baseline leg only
    import world_engine_amd as wea
    from world_engine_amd import ops

    c = dict(CONFIGS[args.config])
    if args.batch:
        c["B"] = args.batch
        c["name"] += f" [batch overridden to {args.batch}]"
    B, H, Hkv, Dh, T, n, layers = c["B"], c["H"], c["Hkv"], c["Dh"], c["T"], c["slots"], c["layers"]
    L = n * T
    W = int(math.isqrt(T))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    dtype = torch.bfloat16
    K, Wm = args.steps, args.warmup
    subs = c["frozen_subs"] + 1                      # attention calls per frame
    frames_total = (Wm + K + subs - 1) // subs + n + 2

    cache = wea.StaticKVCache(
        __import__("types").SimpleNamespace(tokens_per_frame=T, local_window=n, global_window=n,
                                            global_attn_period=1, global_pinned_dilation=1,
                                            n_layers=layers, n_heads=H, n_kv_heads=Hkv, d_model=H * Dh),
        B, dtype).to(dev)
    for layer in cache.layers:
        layer.check_inputs = False                   # the eager sanity checks synchronise
    cos, sin = ro.rope_table_1d(frames_total * T, Dh)
    rope = wea.RoPE(cos, sin, T // W, W).to(dev)

    # synthetic inputs, resident in HBM, in the merged-QKV layout the real module produces
    n_in = 4
    inputs = []
    for i in range(n_in):
        q, k, v = ro.synth_qkv(args.config, i, 0, B, H, Hkv, T, Dh, dtype, outlier=c.get("outlier", False))
        buf = torch.cat([q.transpose(1, 2).reshape(B, T, H * Dh), k.transpose(1, 2).reshape(B, T, Hkv * Dh),
                         v.transpose(1, 2).reshape(B, T, Hkv * Dh)], dim=-1).contiguous().to(dev)
        qq, kk, vv = buf.split((H * Dh, Hkv * Dh, Hkv * Dh), dim=-1)
        inputs.append((qq.reshape(B, T, H, Dh).transpose(1, 2), kk.reshape(B, T, Hkv, Dh).transpose(1, 2),
                       vv.reshape(B, T, Hkv, Dh).transpose(1, 2)))
    idx = torch.arange(T, dtype=torch.long)
    y_pos = (idx // W)[None].expand(B, T).contiguous().to(dev)
    x_pos = (idx % W)[None].expand(B, T).contiguous().to(dev)
    t_pos_all = torch.arange(frames_total, dtype=torch.long)[:, None, None].expand(frames_total, B, T).contiguous().to(dev)

    n_splits = args.n_splits or ops.attn_auto_splits(B, H, Hkv, T, Dh, L)
    ws = torch.empty(max(ops.attn_workspace_bytes(B, H, Hkv, T, Dh, L, args.n_splits, args.q_tile), 16), dtype=torch.uint8, device=dev)
    out = torch.empty((B, T, H, Dh), dtype=dtype, device=dev).transpose(1, 2)

    def one_step(step_idx):
        """One attention call of the schedule for every layer: substeps 0..frozen_subs-1 of a
        frame are frozen, the last one persists (src/world_engine.py:139-152)."""
        frame, sub = divmod(step_idx, subs)
        frozen = sub < c["frozen_subs"]
        pos = {"t_pos": t_pos_all[frame], "y_pos": y_pos, "x_pos": x_pos}
        for li, layer in enumerate(cache.layers):
            q, k, v = inputs[(step_idx + li) % n_in]
            if args.two_calls:
                q_rot = ops.rope_kv_store(q, k, v, pos, rope.cos, rope.sin, rope.height, rope.width,
                                          layer.kv, layer.written, layer.L, 1, frozen)
                ops.attn_ring(q_rot, layer.kv, layer.written, pos["t_pos"], layer.L, 1, n_splits=args.n_splits,
                              q_tile=args.q_tile, out=out, workspace=ws)
            else:
                ops.rope_kv_attn(q, k, v, pos, rope.cos, rope.sin, rope.height, rope.width, layer.kv,
                                 layer.written, layer.L, 1, frozen, n_splits=args.n_splits, q_tile=args.q_tile,
                                 out=out, workspace=ws)

    if args.calibrate_copy:
        # elementwise copy through a kernel (a same-dtype copy_() could take the DMA engines and
        # would then be invisible to the shader counters); int32 + 0 keeps the bytes unchanged
        n_el = args.calibrate_copy * (1 << 20) // 4
        src = torch.arange(n_el, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(20):
            torch.add(src, 0, out=dst)
        torch.cuda.synchronize()
        assert torch.equal(src[-4096:], dst[-4096:])
        log(f"[bench] calibration: 20 copy kernels of {args.calibrate_copy} MiB read + {args.calibrate_copy} MiB written")
        del src, dst

    # ---- fill the ring (untimed, not counted), then W warm-up steps ----
    fill_steps = n * subs
    for s in range(fill_steps):
        one_step(s)
    for s in range(fill_steps, fill_steps + Wm):
        one_step(s)
    torch.cuda.synchronize()
    first = fill_steps + Wm

    # ---- timed region: exactly K steps ----
    if args.eager:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(first, first + K):
            one_step(s)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    else:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for s in range(first, first + K):
                one_step(s)
        torch.cuda.synchronize()                      # capture records, it does not execute
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / K
    us_per_layer_step = ms_per_step * 1e3 / layers
    log(f"[bench] {c['name']}: {ms_per_step * 1e3:.2f} us per step ({K} steps, n_splits={n_splits})")

    # ---- attention-only timing at steady state for the roofline (HIP events on the launch stream) ----
    layer0 = cache.layers[0]
    pos = {"t_pos": t_pos_all[(first + K) // subs + 1], "y_pos": y_pos, "x_pos": x_pos}
    q_rot = ops.rope_kv_store(*inputs[0], pos, rope.cos, rope.sin, rope.height, rope.width,
                              layer0.kv, layer0.written, layer0.L, 1, True)
    iters = args.attn_iters

    def attn_only():
        ops.attn_ring(q_rot, layer0.kv, layer0.written, pos["t_pos"], layer0.L, 1, n_splits=args.n_splits,
                      q_tile=args.q_tile, out=out, workspace=ws)

    for _ in range(5):
        attn_only()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if args.eager:
        e0.record()
        for _ in range(iters):
            attn_only()
        e1.record()
    else:
        g2 = torch.cuda.CUDAGraph()
        side2 = torch.cuda.Stream()
        side2.wait_stream(torch.cuda.current_stream())
        with torch.cuda.graph(g2, stream=side2):
            for _ in range(iters):
                attn_only()
        torch.cuda.synchronize()
        g2.replay()
        torch.cuda.synchronize()
        e0.record()
        g2.replay()
        e1.record()
    torch.cuda.synchronize()
    attn_us = e0.elapsed_time(e1) * 1e3 / iters
    n_vis = L                                        # steady state: n-1 ring slots + the tail
    flops, byts = algorithmic_work(c, n_vis)
    tflops = flops / (attn_us * 1e-6) / 1e12
    gbps = byts / (attn_us * 1e-6) / 1e9
    if c["bound"] == "hbm":
        roof = {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": None}
    else:
        roof = {"bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": None}
    if not (args.n_splits or args.q_tile or args.batch):
        roof["traffic"] = MEASURED_TRAFFIC.get(args.config)
    roof.update({"kernel": "attn_ring_kernel" + (" + attn_combine_kernel" if n_splits > 1 else ""),
                 "us_per_launch": round(attn_us, 3), "algorithmic_bytes": byts, "algorithmic_flops": flops,
                 "n_splits": n_splits})
    log(f"[bench] attention call: {attn_us:.2f} us -> {tflops:.1f} TFLOP/s, {gbps:.0f} GB/s algorithmic")

    # ---- CPU baseline: the oracle's restatement of the reference path on the host cores ----
    cpu = None
    if not args.no_cpu_baseline:
        cfg1l = __import__("types").SimpleNamespace(tokens_per_frame=T, local_window=n, global_window=n,
                                                    global_attn_period=1, global_pinned_dilation=1, n_layers=1,
                                                    n_heads=H, n_kv_heads=Hkv, d_model=H * Dh)
        oc = ro.OracleStaticKVCache(cfg1l, B, dtype)
        oc.set_frozen(False)
        oc.layers[0].kv.normal_()                    # steady state: every slot written
        oc.layers[0].written[:] = True
        q, k, v = ro.synth_qkv(args.config, 0, 0, B, H, Hkv, T, Dh, dtype)
        done, spent = 0, 0.0
        budget = 12.0 if c["B"] * c["H"] * c["T"] <= 16 * 256 else 20.0
        ro.layer_step(oc, 0, q, k, v, ro.synth_pos_ids(n, B, T, W), cos, sin, T // W, W)   # untimed warm-up
        while spent < budget and done < 1000:    # about 12 s of host work (20 s for the large shapes)
            pos_c = ro.synth_pos_ids(n + 1 + done, B, T, W)
            t0c = time.perf_counter()
            ro.layer_step(oc, 0, q, k, v, pos_c, cos, sin, T // W, W)
            spent += time.perf_counter() - t0c
            done += 1
        cpu = {"value": round(spent / done * 1e6, 1), "unit": "us per frame-step (one layer)",
               "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"{done} steady-state frame-steps of the same shape through oracle/ring_oracle.layer_step "
                         f"(eager PyTorch CPU, bf16 inputs, fp32 scores), host cpu_count={os.cpu_count()}"}
        log(f"[bench] cpu baseline: {cpu['value']:.0f} us per frame-step on {cpu['cores']} threads")

    peaks = None
    if args.peaks:
        # achievable rates on this box next to the published ones the roofline is priced against
        a = torch.randn(8192, 8192, device=dev, dtype=dtype)
        b2 = torch.randn(8192, 8192, device=dev, dtype=dtype)
        src = torch.empty(1 << 28, dtype=torch.int32, device=dev)          # 1 GiB
        dst = torch.empty_like(src)

        def timed(fn, n):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record()
            for _ in range(n):
                fn()
            s1.record()
            torch.cuda.synchronize()
            return s0.elapsed_time(s1) * 1e-3 / n

        t_mm = timed(lambda: torch.matmul(a, b2), 20)
        t_cp = timed(lambda: torch.add(src, 0, out=dst), 20)
        peaks = {"bf16_gemm_8192_tflops": round(2 * 8192 ** 3 / t_mm / 1e12, 1),
                 "copy_1gib_read_plus_write_gbps": round(2 * src.numel() * 4 / t_cp / 1e9, 1)}
        log(f"[bench] measured on this box: {peaks}")
        del a, b2, src, dst

    result = {
        "metric": "attn_us_per_frame_step",
        "value": round(ms_per_step * 1e3, 3),
        "unit": "us",
        "n_gpus": 1,
        "steps": K,
        "warmup": Wm,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": c["name"], "launch": "eager" if args.eager else "hip_graph",
                   "calls_per_step": f"{layers} x " + ("(we_rope_kv_store + we_attn_ring_fwd)" if args.two_calls
                                                       else "we_rope_kv_attn_fwd (store kernel + attention kernels)"),
                   "n_splits": n_splits, "q_tile": args.q_tile or "auto"},
        "us_per_layer_step": round(us_per_layer_step, 3),
        "attn_tflops": round(tflops, 2),
        "attn_algorithmic_gbps": round(gbps, 1),
        "roofline": roof,
        "cpu_baseline": cpu,
    }
    if peaks is not None:
        result["measured_peaks"] = peaks
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
