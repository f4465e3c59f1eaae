"""Seeded small Senadra checkpoints for tests: a config dict and a {name: tensor} dict in the family's tensor naming.
Sizes are arguments; nothing here equals a published model.  TEST INFRASTRUCTURE ONLY."""
from typing import Dict, List, Optional

import torch


def attention_layer(heads=6, kv_heads=3, dim=32, vdim=64, scale=0.2, chunk: Optional[int] = 48, kv_from: Optional[int] = None,
                    mlp=None) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        m["mask"] = {"size": chunk}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent_layer(heads=4, dim=32, rot_dim=16, vdim=48, kv_rank=48, q_rank=40, scale=0.15, base=1000.0, rot_dims=None, mlp=None) -> dict:
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "scale": scale, "rot": {"base": base, "dims": rot_dims if rot_dims is not None else rot_dim}}}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=32, conv=3, mlp=None) -> dict:
    return {"type": "channel_delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def dense_mlp(ff=96) -> dict:
    return {"kind": "dense", "ff": ff}


def make_config(layers: List[dict], width=64, vocab=96, eps=1e-5, residual_mult=0.5, side_dim: Optional[int] = 8,
                softcap: Optional[float] = 20.0) -> dict:
    c = {"architecture": "Senadra", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
         "residual_mult": residual_mult}
    if side_dim:
        c["token_side"] = {"dim": side_dim}
    if softcap:
        c["logit_softcap"] = softcap
    return c


def make_tensors(config: dict, seed: int = 0, low_rank: int = 8, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """N(0, 1 / fan_in) projections (wider for what feeds a softmax), gains around one, decays spread over (0, 1).
    Values are rounded to `dtype` (what a checkpoint stores)."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = torch.randn(n, k, generator=g) * gain * k ** -0.5

    def vec(name, n, mean=0.0, std=0.1):
        t[name] = mean + torch.randn(n, generator=g) * std

    t["embed"] = torch.randn(config["vocab"], W, generator=g)
    side = (config.get("token_side") or {}).get("dim", 0)
    if side:
        t["side.embed"] = torch.randn(config["vocab"], side * len(config["layers"]), generator=g)
    for i, lay in enumerate(config["layers"]):
        m, p = lay["mixer"], f"l{i}.mix"
        vec(f"l{i}.norm1", W, 1.0)
        if lay["type"] == "attention":
            H, dk = m["heads"], m["dim"]
            G, dv = m.get("kv_heads", H), m.get("vdim", dk)
            lin(f"{p}.q", H * dk, W, 2.0)
            if m.get("kv_from") is None:
                lin(f"{p}.k", G * dk, W, 2.0)
                lin(f"{p}.v", G * dv, W)
            t[f"{p}.r1"] = torch.rand(H, generator=g) * 0.8 + 0.1
            t[f"{p}.r2"] = torch.rand(H, generator=g) * 0.5 + 0.05
            lin(f"{p}.g", H * dv, W)
            lin(f"{p}.o", W, H * dv)
        elif lay["type"] == "latent_attention":
            H, dn, dr, dv, rk, rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            lin(f"{p}.dq", rq, W)
            vec(f"{p}.dq.norm", rq, 1.0)
            lin(f"{p}.uq", H * (dn + dr), rq, 2.0)
            lin(f"{p}.dkv", rk + dr, W, 1.5)
            vec(f"{p}.dkv.norm", rk, 1.0)
            lin(f"{p}.uk", H * dn, rk, 2.0)
            lin(f"{p}.uv", H * dv, rk)
            lin(f"{p}.g", H * dv, W)
            lin(f"{p}.o", W, H * dv)
        else:
            H, dk, dv, taps = m["heads"], m["dim"], m["vdim"], m["conv"]
            G = m.get("kv_heads", H)
            for n_, c_ in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                lin(f"{p}.{n_}", c_, W)
                t[f"{p}.{n_}.conv"] = torch.randn(c_, taps, generator=g) * 0.5
            lin(f"{p}.b", H, W)
            t[f"{p}.A_log"] = torch.log(torch.rand(H, generator=g) * 2.0 + 0.2)
            vec(f"{p}.norm", dv, 1.0)
            lin(f"{p}.a1", low_rank, W)
            lin(f"{p}.a2", H * dk, low_rank)
            vec(f"{p}.dt_bias", H * dk, -1.0, 1.0)
            lin(f"{p}.g1", low_rank, W)
            lin(f"{p}.g2", H * dv, low_rank)
            lin(f"{p}.o", W, H * dv)
        f = lay.get("mlp")
        if f:
            vec(f"l{i}.norm2", W, 1.0)
            lin(f"l{i}.mlp.up", f["ff"], W)
            lin(f"l{i}.mlp.down", W, f["ff"])
            t[f"l{i}.mlp.act"] = torch.tensor([0.3, -0.4]) + torch.randn(2, generator=g) * 0.2
        if side:
            lin(f"l{i}.side.gate", side, W)
            lin(f"l{i}.side.proj", W, side)
            vec(f"l{i}.side.norm", W, 1.0)
    vec("final.norm", W, 1.0)
    lin("head", config["vocab"], W)
    return {k: v.to(dtype) for k, v in t.items()}


def standard_layers() -> List[dict]:
    """Every mixer, an attention layer that reads another's cache, a layer without a feed-forward."""
    return [attention_layer(mlp=dense_mlp()), delta_layer(mlp=dense_mlp(80)), latent_layer(mlp=dense_mlp()),
            delta_layer(heads=3, kv_heads=3, dim=32, vdim=16, conv=4, mlp=None), attention_layer(kv_from=0, mlp=dense_mlp(72))]
