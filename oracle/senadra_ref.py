"""Plain CPU restatement of the Senadra decoder, one function per mechanism.  TEST INFRASTRUCTURE ONLY: nothing of the
serving path imports this file and it imports nothing of the serving path.

Senadra is a pre-norm hybrid stack over an fp32 residual stream x with a residual multiplier m:
    x <- x + m mixer(N1(x));   x <- x + m ff(N2(x))   (if the layer has a feed-forward);   x <- x + m N_s(side(x, token))
with N(z) = z / sqrt(mean(z^2) + eps) * w.  Mixers:
  * "attention": GQA softmax attention without a rotation; values are unit-RMS per head before they are cached; the score
    loses r1_h ln(1 + r2_h (i - j)) with the distance; a query sees only keys of its own block of `mask.size` positions; a
    sigmoid output gate; a layer may read another layer's keys and values (`kv_from`).
  * "latent_attention": queries and keys/values through normed low-rank latents; a per-head unrotated part and one rotated
    key part shared by the heads (interleaved pairs); causal; sigmoid output gate.  The cache is the latent and the rotated part.
  * "channel_delta": a gated delta rule with one decay per head and key channel; q, k, v through a short causal
    convolution and SiLU; q and k unit vectors; per-head unit-RMS output, gain and a low-rank sigmoid gate.
The feed-forward is W_down xielu(W_up h).  The side input of a layer gates a slice of a second token embedding with a
GELU of a projection of x, projects it back and norms it.  Logits are soft-capped by a tanh.

All arithmetic is in `DT` (float64) on the CPU; weights are taken as stored.  A sequence is processed whole (`forward`) or
in any portions through an explicit per-sequence state (`new_state` / `advance`).
"""
import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def rms_unit(z: torch.Tensor, eps: float) -> torch.Tensor:
    return z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def xielu(z, pq):
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    ap, aq = softplus(pq[0]), 0.5 + softplus(pq[1])
    neg = torch.clamp(z, max=0.0)
    return torch.where(z > 0, ap * z * z + 0.5 * z, aq * (torch.expm1(neg) - neg) + 0.5 * z)


def rotate_pairs(x, pos, base: float, dims: int):
    """x [T, ..., D]: the first `dims` channels are rotated, channel 2i with 2i + 1, by pos * base^(-2i / dims)."""
    i = torch.arange(dims // 2, dtype=DT)
    ang = pos.to(DT)[:, None] * base ** (-2.0 * i / dims)  # [T, dims/2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def attention_mixer(h, pos, p: Dict[str, torch.Tensor], m: dict, eps: float, past_k=None, past_v=None, shared=None):
    """h [T, W] new tokens at positions pos [T].  past_k [P, G, dk], past_v [P, G, dv]: what the cache holds.  shared =
    (keys, values) of ALL P + T positions from the layer this one reads its cache from (then no projections of its own).
    Returns (out [T, W], keys [P + T, G, dk], values [P + T, G, dv])."""
    H, dk = m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", dk)
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, dk)
    if shared is None:
        k = (h @ p["k"].T).view(T, G, dk)
        v = rms_unit((h @ p["v"].T).view(T, G, dv), eps)
        if past_k is not None:
            k, v = torch.cat([past_k, k], 0), torch.cat([past_v, v], 0)
    else:
        k, v = shared
    P = k.shape[0] - T
    size = (m.get("mask") or {}).get("size")
    j = torch.arange(P + T)[None, :]
    i = pos[:, None]
    hidden = j > i
    if size:
        hidden = hidden | (torch.div(i, size, rounding_mode="floor") != torch.div(j, size, rounding_mode="floor"))
    dist = torch.clamp(i - j, min=0).to(DT)
    out = torch.zeros(T, H, dv, dtype=DT)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if "r1" in p:
            s = s - p["r1"][hd] * torch.log1p(p["r2"][hd] * dist)
        s = s.masked_fill(hidden, float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ p["g"].T)
    return out @ p["o"].T, k, v


def latent_attention_mixer(h, pos, p: Dict[str, torch.Tensor], m: dict, eps: float, past_c=None, past_r=None):
    """Cache: past_c [P, kv_rank] normed latents, past_r [P, rot_dim] rotated shared key parts.
    Returns (out, latents [P + T, kv_rank], rotated parts [P + T, rot_dim])."""
    H, dn, dr, dv, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    rot = m["rot"]
    cq = rms_unit(h @ p["dq"].T, eps) * p["dq.norm"]
    q = (cq @ p["uq"].T).view(T, H, dn + dr)
    q_n, q_r = q[..., :dn], rotate_pairs(q[..., dn:], pos, rot["base"], rot["dims"])
    ckv = h @ p["dkv"].T
    c = rms_unit(ckv[:, :rk], eps) * p["dkv.norm"]
    r = rotate_pairs(ckv[:, rk:], pos, rot["base"], rot["dims"])
    if past_c is not None:
        c, r = torch.cat([past_c, c], 0), torch.cat([past_r, r], 0)
    N = c.shape[0]
    k_n = (c @ p["uk"].T).view(N, H, dn)
    v = (c @ p["uv"].T).view(N, H, dv)
    hidden = torch.arange(N)[None, :] > pos[:, None]
    out = torch.zeros(T, H, dv, dtype=DT)
    for hd in range(H):
        s = (q_n[:, hd] @ k_n[:, hd].T + q_r[:, hd] @ r.T) * m["scale"]
        s = s.masked_fill(hidden, float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ v[:, hd]
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ p["g"].T)
    return out @ p["o"].T, c, r


def short_conv(x, w, tail):
    """Causal per-channel convolution.  x [T, C], w [C, taps] (last column = current token), tail [taps - 1, C] = the inputs
    before x[0] (zeros at the start of a sequence).  Returns (y [T, C], new tail)."""
    taps = w.shape[1]
    full = torch.cat([tail, x], 0)  # [taps - 1 + T, C]
    y = torch.zeros_like(x)
    for t in range(taps):
        y = y + full[t:t + x.shape[0]] * w[:, t]
    return y, full[full.shape[0] - (taps - 1):]


def delta_recurrence(q, k, v, beta, decay, S):
    """One head group at a time: q, k [T, H, dk]; v [T, H, dv]; beta [T, H]; decay [T, H, dk]; S [H, dk, dv].
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T = q.shape[0]
    out = torch.zeros_like(v)
    for t in range(T):
        S = S * decay[t][:, :, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out, S


def channel_delta_mixer(h, p: Dict[str, torch.Tensor], m: dict, eps: float, state=None):
    """state = {"S": [H, dk, dv], "q": tail, "k": tail, "v": tail} or None at the start of a sequence."""
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    taps = m["conv"]
    T = h.shape[0]
    if state is None:
        state = {"S": torch.zeros(H, dk, dv, dtype=DT), "q": torch.zeros(taps - 1, G * dk, dtype=DT),
                 "k": torch.zeros(taps - 1, G * dk, dtype=DT), "v": torch.zeros(taps - 1, H * dv, dtype=DT)}
    new = {}
    act = {}
    for n in ("q", "k", "v"):
        y, new[n] = short_conv(h @ p[n].T, p[n + ".conv"], state[n])
        act[n] = y * torch.sigmoid(y)
    unit = lambda z: z / torch.sqrt((z * z).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q = (unit(act["q"].view(T, G, dk)) * dk ** -0.5).repeat_interleave(rep, dim=1)
    k = unit(act["k"].view(T, G, dk)).repeat_interleave(rep, dim=1)
    v = act["v"].view(T, H, dv)
    beta = torch.sigmoid(h @ p["b"].T)
    dt = softplus((h @ p["a1"].T) @ p["a2"].T + p["dt_bias"]).view(T, H, dk)
    decay = torch.exp(-torch.exp(p["A_log"])[None, :, None] * dt)
    o, new["S"] = delta_recurrence(q, k, v, beta, decay, state["S"])
    o = rms_unit(o, eps) * p["norm"] * torch.sigmoid((h @ p["g1"].T) @ p["g2"].T).view(T, H, dv)
    return o.reshape(T, H * dv) @ p["o"].T, new


def dense_ff(h, p):
    return xielu(h @ p["up"].T, p["act"]) @ p["down"].T


def side_input(x, tokens, layer: int, table, p, dim: int, eps: float):
    """The normed per-layer token input (before the residual multiplier)."""
    e = table[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ p["gate"].T) * e) @ p["proj"].T
    return rms_unit(y, eps) * p["norm"]


def layer_params(tensors, i: int, part: str) -> Dict[str, torch.Tensor]:
    pre = f"l{i}.{part}."
    return {k[len(pre):]: v.to(DT) for k, v in tensors.items() if k.startswith(pre)}


def new_state(config: dict) -> dict:
    return {"len": 0, "layers": [None] * len(config["layers"])}


def advance(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], state: dict, trace: Optional[list] = None):
    """Feed `tokens` after what `state` holds; returns logits [T, vocab]."""
    eps, mult = config["norm"]["eps"], config.get("residual_mult", 1.0)
    tok = torch.tensor(tokens, dtype=torch.long)
    T = len(tokens)
    pos = torch.arange(state["len"], state["len"] + T)
    x = tensors["embed"].to(DT)[tok]
    side = config.get("token_side")
    for i, lay in enumerate(config["layers"]):
        m, st = lay["mixer"], state["layers"][i]
        p = layer_params(tensors, i, "mix")
        h = rms_unit(x, eps) * tensors[f"l{i}.norm1"].to(DT)
        if lay["type"] == "attention":
            if m.get("kv_from") is not None:
                src = state["layers"][m["kv_from"]]
                y, _, _ = attention_mixer(h, pos, p, m, eps, shared=(src["k"], src["v"]))
            else:
                y, k, v = attention_mixer(h, pos, p, m, eps, st["k"] if st else None, st["v"] if st else None)
                state["layers"][i] = {"k": k, "v": v}
        elif lay["type"] == "latent_attention":
            y, c, r = latent_attention_mixer(h, pos, p, m, eps, st["c"] if st else None, st["r"] if st else None)
            state["layers"][i] = {"c": c, "r": r}
        elif lay["type"] == "channel_delta":
            y, state["layers"][i] = channel_delta_mixer(h, p, m, eps, st)
        else:
            raise ValueError(lay["type"])
        x = x + mult * y
        if lay.get("mlp"):
            h = rms_unit(x, eps) * tensors[f"l{i}.norm2"].to(DT)
            x = x + mult * dense_ff(h, layer_params(tensors, i, "mlp"))
        if side:
            x = x + mult * side_input(x, tok, i, tensors["side.embed"].to(DT), layer_params(tensors, i, "side"), side["dim"], eps)
        if trace is not None:
            trace.append(x.clone())
    state["len"] += T
    logits = (rms_unit(x, eps) * tensors["final.norm"].to(DT)) @ tensors["head"].to(DT).T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def forward(config, tensors, tokens, trace=None):
    return advance(config, tensors, tokens, new_state(config), trace)
