"""Seeded sweep over valid geometries: batch, grouped heads, frame lengths on and off the tile
grid, both head dims and element types, ring sizes from one slot up, pinned dilation, frozen and
persisting calls, automatic and explicit split / tile choices - each a short schedule against the
oracle (cache bit-exact, attention within max-abs 2e-2 / mean-abs 2e-3)."""
import random

import pytest
import torch

from oracle import ring_oracle as ro
from _harness import Pair, assert_attn_close, assert_bits_equal

pytestmark = pytest.mark.gpu


def _case(seed):
    r = random.Random(seed)
    d = r.choice([1, 1, 1, 2, 3])
    hkv = r.choice([1, 2, 3])
    return dict(
        dtype=r.choice([torch.bfloat16, torch.bfloat16, torch.float16]),
        B=r.choice([1, 1, 2, 3]), Hkv=hkv, H=hkv * r.choice([1, 1, 2, 4]),
        T=r.choice([8, 16, 24, 48, 64, 72, 100, 128, 136, 192, 200, 256, 264, 320]),
        Dh=r.choice([64, 128]), n_slots=d * r.choice([1, 2, 3, 5]), d=d,
        n_splits=r.choice([0, 0, 1, 2, 3, 5]), q_tile=r.choice([0, 0, 128, 256]),
        steps=r.choice([4, 6, 9]), frozen_every=r.choice([0, 2, 3]))


@pytest.mark.parametrize("seed", list(range(36)))
def test_random_geometry(gpu_device, seed):
    c = _case(seed)
    print(f"seed {seed}: {c}", flush=True)
    p = Pair(gpu_device, c["dtype"], B=c["B"], H=c["H"], Hkv=c["Hkv"], T=c["T"], Dh=c["Dh"], n_slots=c["n_slots"],
             d=c["d"], cfg_id=70 + seed)
    for t in range(c["steps"]):
        frozen = c["frozen_every"] > 0 and t % c["frozen_every"] == 1
        p.set_frozen(frozen)
        q, k, v, pos = p.inputs(t)
        (q_o, k_all, v_all, mask), (q_h, ring) = p.store(q, k, v, pos, strided=(t % 2 == 0))
        assert_bits_equal(q_h, q_o, f"RoPE(q) t={t}")
        p.assert_state_equal(what=f"t={t}")
        out = p.attend(q_h, ring, n_splits=c["n_splits"], q_tile=c["q_tile"])
        assert_attn_close(out, ro.attention_fp32(q_o, k_all, v_all, mask), f"t={t}")
