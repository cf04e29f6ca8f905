"""Build ``libwe_attn.so`` (HIP, gfx950) in-tree: ``python -m world_engine_amd.build``.

Every source is compiled to its own object, in parallel (the main attention kernel once per
element type / head dim family), and the objects are linked into the shared library."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_obj")
# (source, extra defines, object name)
_RING = [("attn_ring.hip", [f"-DWE_RING_PART={i}"], f"attn_ring_{name}.o")
         for i, name in enumerate(("bf16_128", "bf16_64", "f16_128", "f16_64"))]
_SHARED = [("rope_kv_store.hip", [], "rope_kv_store.o"),
           ("qkv_proj_store.hip", [], "qkv_proj_store.o"),
           ("attn_ring_f32.hip", [], "attn_ring_f32.o"),
           ("attn_combine.hip", [], "attn_combine.o")]
# the product: libwe_attn.so
UNITS = _SHARED + _RING + [("device_state.hip", [], "device_state.o"), ("capi.hip", [], "capi.o")]
# the measurement library: the same kernels plus their clocked instantiations and the tile-stream
# probe (its own copies of the objects that hold state or differ; the rest are the product's)
PROBE_UNITS = _SHARED + [(src, defs + ["-DWE_WITH_PROBES"], "probe_" + obj) for src, defs, obj in _RING] + [
    ("device_state.hip", [], "probe_device_state.o"), ("capi.hip", [], "probe_capi_base.o"),
    ("probe_capi.hip", [], "probe_capi.o"), ("stream_probe.hip", [], "stream_probe.o")]
SOURCES = sorted({u[0] for u in UNITS + PROBE_UNITS})
OUT = os.path.join(HERE, "libwe_attn.so")
PROBE_OUT = os.path.join(HERE, "libwe_probe.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep fp32 arithmetic scalar: packed fp32 instructions are avoided on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("packed-fp32-ops", "Reserved registers on the clobber list", "warnings generated", "warning generated")
    lines = res.stderr.splitlines()
    err = "\n".join(l for l in lines if not any(n in l for n in noise))
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}\n{err}")
    return err


def build(verbose: bool = False, jobs: int = 8) -> str:
    """Compile every unit once and link ``libwe_attn.so`` and ``libwe_probe.so``; returns the product's path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    units = list({u[2]: u for u in UNITS + PROBE_UNITS}.values())   # one compile per object
    cmds = [[hipcc, *HIPCC_FLAGS, *defs, "-c", os.path.join(CSRC, src), "-o", os.path.join(OBJ_DIR, obj)]
            for src, defs, obj in units]
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(cmds)))) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    for out, group in ((OUT, UNITS), (PROBE_OUT, PROBE_UNITS)):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[os.path.join(OBJ_DIR, u[2]) for u in group], "-o", out],
             verbose)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
