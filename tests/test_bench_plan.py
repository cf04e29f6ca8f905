"""CPU-side checks of bench.py's own arithmetic: every leg of every configuration stays inside the
RoPE table it builds, the CPU leg runs past its frame window without leaving the table, and the
traffic figure is read from the committed counter summaries."""
import argparse
import os
import re

import pytest
import torch

import bench
from oracle import ring_oracle as ro


@pytest.mark.parametrize("steps,warmup", [(1, 0), (20, 5), (128, 16), (512, 32)])
@pytest.mark.parametrize("cfg_id", sorted(bench.CONFIGS))
def test_every_leg_stays_inside_the_rope_table(cfg_id, steps, warmup):
    c = bench.CONFIGS[cfg_id]
    plan = bench.schedule_plan(c, steps, warmup)
    T = c["T"]
    rows = plan["table_frames"] * T
    subs = c["frozen_subs"] + 1
    assert plan["subs"] == subs and plan["fill_steps"] == c["slots"] * subs
    # the schedule: fill + warm-up + timed steps, step s belongs to frame s // subs
    timed_frames = {s // subs for s in range(plan["first"] + steps)}
    assert max(timed_frames) == plan["last_timed_frame"]
    legs = {"schedule": max(timed_frames), "attention-only": plan["attn_frame"], "cpu": max(plan["cpu_frames"])}
    for leg, frame in legs.items():
        assert bench.max_table_row(frame, T) < rows, f"{leg} leg reads table row past the end"
    # the ring is full before the first timed step, whatever the warm-up
    assert plan["first"] // subs >= c["slots"]
    # legs use distinct frames in increasing order (the attention-only frame follows the schedule)
    assert plan["attn_frame"] > plan["last_timed_frame"] and min(plan["cpu_frames"]) > plan["attn_frame"]


def test_cpu_leg_cycles_inside_its_window():
    # a tiny shape, so that the leg does far more steps than its window holds frames
    c = dict(name="tiny", B=1, H=2, Hkv=1, Dh=16, T=16, slots=2, layers=3, frozen_subs=1, bound="hbm",
             cpu_budget_s=0.2)
    args = argparse.Namespace(steps=20, warmup=5)
    cpu = bench.run_cpu(0, c, args, torch, ro)
    n = int(re.match(r"(\d+) steady-state", cpu["sample"]).group(1))
    assert n > len(bench.schedule_plan(c, 20, 5)["cpu_frames"])
    assert cpu["kind"] == "port" and cpu["value"] > 0 and cpu["cores"] >= 1
    assert "3 layers" in cpu["unit"]
    one = bench.run_cpu(0, c, args, torch, ro, threads=1, budget=0.05)
    assert one["cores"] == 1 and torch.get_num_threads() >= 1


def test_algorithmic_work_matches_the_stated_figures():
    # steady state: N_vis = L (n - 1 ring slots + the tail)
    f1, b1 = bench.algorithmic_work(bench.CONFIGS[1], 16 * 256)
    f3, b3 = bench.algorithmic_work(bench.CONFIGS[3], 8 * 1024)
    f4, b4 = bench.algorithmic_work(bench.CONFIGS[4], 32 * 256)
    assert round(f1 / 1e9, 3) == 8.590 and round(b1 / 1e6, 2) == 35.65
    assert round(f3 / 1e9, 1) == 412.3 and round(b3 / 1e6, 1) == 453.0
    assert round(f4 / 1e9, 2) == 17.18 and round(b4 / 1e6, 2) == 69.21


def test_percentiles():
    xs = [5.0, 1.0, 3.0, 2.0, 4.0]
    s = bench.spread(xs)
    assert s["median"] == 3.0 and s["p10"] == pytest.approx(1.4) and s["p90"] == pytest.approx(4.6)
    assert bench.spread([7.0]) == {"median": 7.0, "p10": 7.0, "p90": 7.0, "samples": 1}


def test_traffic_comes_from_the_committed_summaries():
    for cfg_id in (1, 3):
        path = os.path.join(bench.ROOT, "profiles", f"attn_ring_cfg{cfg_id}_hbm_traffic.txt")
        if not os.path.exists(path):
            pytest.skip("no counter summary for this configuration")
        val, src = bench.read_traffic(cfg_id)
        assert isinstance(val, int) and val > 0 and f"cfg{cfg_id}_hbm_traffic" in src
        assert str(val) in open(path).read()
    assert bench.read_traffic(99) == (None, None)
