"""The install path end to end: a model-shaped module tree whose attention modules look like the
reference's ``Attn`` (``q_proj / k_proj / v_proj / out_proj``, ``v_lamb``, ``gate_proj``, their own
``.rope``, ``layer_idx``; ``src/model/attn.py:70-96``) sits in a holder with ``.config`` and a
shared rotary module (``src/model/world_model.py:199-202``); ``install_ring_attention`` walks it
the way the reference's merged-QKV patch does (``src/patch_model.py:92-114,144-147``).  Checked:
what gets replaced, the state-dict mapping, mode / dtype / device carry-over, loud failure on
state that does not fit, and - on the GPU - four frames of forward through the installed modules
against the same sequence composed on the CPU from torch's own operations and the oracle."""
from types import SimpleNamespace

import pytest
import torch
import torch.nn.functional as F
from torch import nn

from oracle import ring_oracle as ro
import world_engine_amd as wea

T, H, HKV, DH, N_SLOTS, GRID = 64, 4, 2, 64, 3, 8


def _config(n_layers=2):
    return SimpleNamespace(tokens_per_frame=T, local_window=N_SLOTS, global_window=N_SLOTS, global_attn_period=1,
                           global_pinned_dilation=1, n_layers=n_layers, n_heads=H, n_kv_heads=HKV, d_model=H * DH,
                           value_residual=True, gated_attn=True, height=GRID, width=GRID, n_frames=16)


class TableRope(nn.Module):
    """Stand-in for the reference's rotary module: fp32 ``cos`` / ``sin`` buffers, not persistent."""

    def __init__(self, cfg):
        super().__init__()
        cos, sin = ro.rope_table_1d(cfg.n_frames * cfg.height * cfg.width, cfg.d_model // cfg.n_heads)
        self.register_buffer("cos", cos, persistent=False)
        self.register_buffer("sin", sin, persistent=False)

    def _apply(self, fn, *args, **kwargs):       # tables stay fp32 under dtype casts
        def keep(t):
            out = fn(t)
            return out if out.dtype == t.dtype else out.to(t.dtype)
        return super()._apply(keep, *args, **kwargs)


class SplitAttn(nn.Module):
    """Attention module with the reference's attribute and parameter names; never run."""

    def __init__(self, cfg, layer_idx):
        super().__init__()
        self.config, self.layer_idx = cfg, layer_idx
        d, dh = cfg.d_model, cfg.d_model // cfg.n_heads
        self.v_lamb = nn.Parameter(torch.tensor(0.5))
        self.q_proj = nn.Linear(d, cfg.n_heads * dh, bias=False)
        self.k_proj = nn.Linear(d, cfg.n_kv_heads * dh, bias=False)
        self.v_proj = nn.Linear(d, cfg.n_kv_heads * dh, bias=False)
        self.out_proj = nn.Linear(d, d, bias=False)
        self.rope = TableRope(cfg)
        self.gate_proj = nn.Linear(cfg.n_heads, cfg.n_heads, bias=False)


class Block(nn.Module):
    def __init__(self, cfg, idx):
        super().__init__()
        self.attn = SplitAttn(cfg, idx)
        self.mlp = nn.Linear(cfg.d_model, cfg.d_model)


class Model(nn.Module):
    def __init__(self, cfg):
        super().__init__()
        self.config = cfg
        self.transformer = nn.Module()
        self.transformer.blocks = nn.ModuleList([Block(cfg, i) for i in range(cfg.n_layers)])
        shared = self.transformer.blocks[0].attn.rope
        for blk in self.transformer.blocks[1:]:
            blk.attn.rope = shared


def _model(seed=0, dtype=torch.bfloat16):
    torch.manual_seed(seed)
    m = Model(_config())
    with torch.no_grad():
        for i, blk in enumerate(m.transformer.blocks):
            blk.attn.gate_proj.weight.normal_(0, 0.5)
            blk.attn.v_lamb.fill_(0.3 + 0.3 * i)
    return m.to(dtype).eval()


@pytest.mark.parametrize("merged_qkv", [False, True])
def test_install_replaces_and_maps_state(merged_qkv):
    m = _model()
    m.transformer.blocks[1].attn.train()           # the mode is carried over module by module
    before = [{k: v.clone() for k, v in blk.attn.state_dict().items()} for blk in m.transformer.blocks]
    n = wea.install_ring_attention(m, None, (SplitAttn,), merged_qkv=merged_qkv)
    assert n == 2
    assert wea.install_ring_attention(m, None, (SplitAttn,), merged_qkv=merged_qkv) == 0, "nothing left to replace"
    attns = [blk.attn for blk in m.transformer.blocks]
    assert all(isinstance(a, wea.RingAttn) for a in attns)
    assert isinstance(m.transformer.blocks[0].mlp, nn.Linear), "only attention modules are touched"
    assert attns[0].rope is attns[1].rope, "modules that shared a rotary module share one afterwards"
    assert attns[0].rope.cos.dtype == torch.float32 and (attns[0].rope.height, attns[0].rope.width) == (GRID, GRID)
    for i, (a, sd) in enumerate(zip(attns, before)):
        assert a.layer_idx == i and a.training == (i == 1)
        assert a.out_proj.weight.dtype == torch.bfloat16
        new = a.state_dict()
        if merged_qkv:
            assert set(new) == {"qkv_proj.weight", "out_proj.weight", "v_lamb", "gate_proj.weight"}
            rows = torch.cat([sd["q_proj.weight"], sd["k_proj.weight"], sd["v_proj.weight"]], dim=0)
            assert torch.equal(new["qkv_proj.weight"], rows), "merged rows are q | k | v"
        else:
            assert set(new) == set(sd)
            for k in ("q_proj.weight", "k_proj.weight", "v_proj.weight"):
                assert torch.equal(new[k], sd[k])
        for k in ("out_proj.weight", "v_lamb", "gate_proj.weight"):
            assert torch.equal(new[k], sd[k]), k


def test_merged_source_can_be_split_again_and_bad_state_fails_loudly():
    cfg = _config()
    rope = wea.RoPE(*ro.rope_table_1d(64, DH), GRID, GRID)
    merged = wea.RingAttn(cfg, 0, rope, merged_qkv=True)
    split = wea.RingAttn.from_reference(merged, cfg, rope, merged_qkv=False)
    assert torch.equal(torch.cat([split.q_proj.weight, split.k_proj.weight, split.v_proj.weight]), merged.qkv_proj.weight)

    class Extra(SplitAttn):
        def __init__(self, cfg, idx):
            super().__init__(cfg, idx)
            self.k_norm_scale = nn.Parameter(torch.ones(4))

    with pytest.raises(RuntimeError, match=r"unexpected keys \['k_norm_scale'\]"):
        wea.RingAttn.from_reference(Extra(cfg, 0), cfg, rope)

    class NoGate(SplitAttn):
        def __init__(self, cfg, idx):
            super().__init__(cfg, idx)
            del self.gate_proj

    with pytest.raises(RuntimeError, match=r"missing keys \['gate_proj.weight'\]"):
        wea.RingAttn.from_reference(NoGate(cfg, 0), cfg, rope)


def _cpu_forward(sd, cfg, x, pos, v1, ocache, layer, cos, sin):
    """The reference module's forward (src/model/attn.py:99-122) from torch's own CPU operations
    and the oracle's cache + attention."""
    B = x.shape[0]
    q = F.linear(x, sd["q_proj.weight"]).reshape(B, T, H, DH).transpose(1, 2)
    k = F.linear(x, sd["k_proj.weight"]).reshape(B, T, HKV, DH).transpose(1, 2)
    v = F.linear(x, sd["v_proj.weight"]).reshape(B, T, HKV, DH).transpose(1, 2)
    v1 = v if v1 is None else v1
    v = torch.lerp(v, v1.view_as(v), sd["v_lamb"])
    q, k = F.rms_norm(q, (DH,)), F.rms_norm(k, (DH,))
    y, _ = ro.layer_step(ocache, layer, q, k, v, pos, cos, sin, GRID, GRID)
    gates = torch.sigmoid(F.linear(x[..., :H], sd["gate_proj.weight"]))
    y = y * gates.permute(0, 2, 1).unsqueeze(-1)
    return F.linear(y.transpose(1, 2).reshape(B, T, -1), sd["out_proj.weight"]), v1


@pytest.mark.gpu
@pytest.mark.parametrize("merged_qkv,fuse_elementwise", [(False, False), (True, False), (False, True), (True, True)])
def test_installed_modules_run_four_frames_like_the_cpu_composition(gpu_device, merged_qkv, fuse_elementwise):
    print(f"install path: merged_qkv={merged_qkv} fuse_elementwise={fuse_elementwise}", flush=True)
    dev = gpu_device
    m = _model(seed=3)
    cfg = m.config
    sds = [{k: v.clone() for k, v in blk.attn.state_dict().items()} for blk in m.transformer.blocks]
    cos, sin = m.transformer.blocks[0].attn.rope.cos.clone(), m.transformer.blocks[0].attn.rope.sin.clone()
    m = m.to(dev)                                    # installed after the move, as the reference patches after .to()
    assert wea.install_ring_attention(m, None, (SplitAttn,), merged_qkv=merged_qkv, fuse_elementwise=fuse_elementwise) == 2
    attns = [blk.attn for blk in m.transformer.blocks]
    assert all(a.out_proj.weight.device.type == "cuda" and a.rope.cos.device.type == "cuda" for a in attns)
    cache = wea.StaticKVCache(cfg, 1, torch.bfloat16).to(dev)
    ocache = ro.OracleStaticKVCache(cfg, 1, torch.bfloat16)
    g = torch.Generator("cpu").manual_seed(9)
    for t in range(4):
        frozen = t == 1
        cache.set_frozen(frozen)
        ocache.set_frozen(frozen)
        x = torch.randn(1, T, H * DH, generator=g).to(torch.bfloat16)
        pos = ro.synth_pos_ids(t, 1, T, GRID)
        posd = {k: v.to(dev) for k, v in pos.items()}
        xh, v1h = x.to(dev), None
        xo, v1o = x, None
        with torch.no_grad():
            for layer in range(2):                   # two layers chained, the second fed the first one's v1
                yh, v1h = attns[layer](xh, posd, v1h, cache)
                yo, v1o = _cpu_forward(sds[layer], cfg, xo, pos, v1o, ocache, layer, cos, sin)
                d = (yh.float().cpu() - yo.float()).abs()
                assert d.max().item() < 4e-2 and d.mean().item() < 4e-3, (t, layer, d.max().item(), d.mean().item())
                xh, xo = yh, yh.cpu()                # both sides continue from the GPU's output
        for layer in range(2):
            assert torch.equal(cache.layers[layer].written.cpu(), ocache.layers[layer].written), (t, layer)
            if not fuse_elementwise:                 # torch's own norm / lerp on both sides: the cache rows agree closely
                dk = (cache.layers[layer].kv.float().cpu() - ocache.layers[layer].kv.float()).abs()
                assert dk.max().item() <= 6e-2, (t, layer, dk.max().item())
