"""Seeded small Lenisun checkpoints for tests: a config dict and a {name: bfloat16 tensor} dict in the family's tensor
naming.  Sizes are arguments; nothing here equals a published model.  TEST INFRASTRUCTURE ONLY."""
from typing import Dict, List, Optional, Tuple

import torch


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.25, q_temp=(0.5, 16), v_mix=False, mlp=None) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": mlp}


def wkv_layer(heads=3, dim=16, mlp=None) -> dict:
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def dense_mlp(ff=64, limit=1.5) -> dict:
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe_mlp(ff=32, experts=6, top=2, shared_ff: Optional[int] = 24) -> dict:
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff}
    return f


def make_config(layers: List[dict], width=64, vocab=96, eps=1e-5, embed_scale=0.7) -> dict:
    return {"architecture": "Lenisun", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}}


def make_tensors(config: dict, seed: int = 0, decay_rank: int = 8) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = torch.randn(n, k, generator=g) * gain * k ** -0.5

    def vec(name, n, mean=0.0, std=0.1):
        t[name] = mean + torch.randn(n, generator=g) * std

    t["embed"] = torch.randn(config["vocab"], W, generator=g)
    for i, lay in enumerate(config["layers"]):
        m = lay["mixer"]
        for n in ("norm1", "norm1b"):
            vec(f"l{i}.{n}", W)
        p = f"l{i}.mix"
        if lay["type"] == "attention":
            H, G, dk, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
            lin(f"{p}.q", H * dk, W)
            lin(f"{p}.k", G * dk, W)
            lin(f"{p}.v", G * dv, W)
            vec(f"{p}.q.norm", dk, 1.0, 0.2)
            vec(f"{p}.k.norm", dk, 1.0, 0.2)
            if m.get("v_mix"):
                t[f"{p}.vmix"] = torch.rand((), generator=g) * 0.6 + 0.2
            lin(f"{p}.o", W, H * dv)
        else:
            H, d = m["heads"], m["dim"]
            for s in ("r", "k", "v", "g", "w"):
                t[f"{p}.mu.{s}"] = torch.rand(W, generator=g)
            for s in ("r", "k", "v", "g"):
                lin(f"{p}.{s}", H * d, W)
            lin(f"{p}.w1", decay_rank, W)
            lin(f"{p}.w2", H * d, decay_rank)
            vec(f"{p}.w0", H * d, -0.5, 0.7)
            t[f"{p}.u"] = torch.randn(H, d, generator=g) * 0.4
            vec(f"{p}.norm", H * d, 1.0, 0.2)
            lin(f"{p}.o", W, H * d)
        f = lay.get("mlp")
        if not f:
            continue
        for n in ("norm2", "norm2b"):
            vec(f"l{i}.{n}", W)
        q = f"l{i}.mlp"
        if f["kind"] == "dense":
            lin(f"{q}.gate", f["ff"], W, 2.0)
            lin(f"{q}.up", f["ff"], W, 2.0)
            lin(f"{q}.down", W, f["ff"])
        else:
            for e in range(f["router"]["experts"]):
                lin(f"{q}.e{e}.gate", f["expert"]["ff"], W)
                lin(f"{q}.e{e}.up", f["expert"]["ff"], W)
                lin(f"{q}.e{e}.down", W, f["expert"]["ff"])
            lin(f"{q}.router", f["router"]["experts"], W, 2.0)
            if f.get("shared"):
                lin(f"{q}.shared.gate", f["shared"]["ff"], W)
                lin(f"{q}.shared.up", f["shared"]["ff"], W)
                lin(f"{q}.shared.down", W, f["shared"]["ff"])
                lin(f"{q}.shared.sg", 1, W)
    vec("final.norm", W)
    lin("head", config["vocab"], W)
    return {k: v.to(torch.bfloat16) for k, v in t.items()}


def standard(seed: int = 0) -> Tuple[dict, Dict[str, torch.Tensor]]:
    """Every mechanism once, sizes unlike any other fixture: attention first (GQA 6:3, dk 24, dv 40, blending), a recurrent
    layer without a feed-forward, a blending attention layer with MHA and equal widths and no query gain, a recurrent
    layer with top-2 experts and no shared expert."""
    layers = [
        attention_layer(heads=6, kv_heads=3, dim=24, vdim=40, scale=0.3, q_temp=(0.4, 8), v_mix=True, mlp=dense_mlp(72, 1.0)),
        wkv_layer(heads=2, dim=48, mlp=None),
        attention_layer(heads=3, kv_heads=3, dim=40, vdim=40, scale=0.2, q_temp=None, v_mix=True, mlp=moe_mlp(40, 5, 2, 24)),
        wkv_layer(heads=5, dim=16, mlp=moe_mlp(24, 7, 3, None)),
        attention_layer(heads=2, kv_heads=1, dim=8, vdim=16, scale=0.5, q_temp=(1.0, 1), v_mix=False, mlp=None),
    ]
    cfg = make_config(layers, width=80, vocab=120, eps=1e-4, embed_scale=1.3)
    return cfg, make_tensors(cfg, seed)
