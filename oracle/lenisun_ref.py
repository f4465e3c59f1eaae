"""Plain CPU restatement of the Lenisun decoder, one function per mechanism.  TEST INFRASTRUCTURE ONLY: nothing of the
serving path imports this file and it imports nothing of the serving path.

Lenisun is a hybrid stack over an fp32 residual stream x.  Every layer is
    x <- x + N_1b(mixer(N_1(x)));   x <- x + N_2b(ff(N_2(x)))        (the second line only if the layer has a feed-forward)
with N(z) = z / sqrt(mean(z^2) + eps) * (1 + g) ("one-plus" RMS norm).  The mixer is either softmax attention without a
rotation (per-head RMS norm of q and k, a query gain that grows with the logarithm of the position, optional blending of
the values with those of the first blending layer) or an RWKV-style linear recurrence with a per-channel data-dependent decay
and a bonus for the current token.  The feed-forward is either a clamped gated unit or a sigmoid-routed mixture of experts
whose routing weight scales the expert's INPUT, plus a sigmoid-gated shared expert.

All arithmetic is float64 on the CPU; weights are taken as stored.  Sequences are processed one at a time and whole
(`forward`), or in any portions through an explicit per-sequence state (`new_state` / `advance`), so that tests of the cache
and state handling have an independent statement of what "the state" is.
"""
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms_unit(z: torch.Tensor, eps: float) -> torch.Tensor:
    """z divided by its root mean square over the last axis, eps inside the root."""
    return z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)


def norm_one_plus(z, g, eps):
    return rms_unit(z, eps) * (1.0 + g)


def query_gain(pos: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) for integer positions p."""
    return 1.0 + coef * torch.log(torch.div(pos + 1, every, rounding_mode="floor").to(F64) + 1.0)


def attention_mixer(h, pos, p: Dict[str, torch.Tensor], m: dict, eps: float, past_k=None, past_v=None, v_first=None,
                    blend: bool = False):
    """h [T, W] are the new tokens at positions pos [T]; past_k [P, G, dk] / past_v [P, G, dv] the cached ones.
    Returns (out [T, W], keys [P + T, G, dk], values [P + T, G, dv] as cached, values before blending [T, G, dv])."""
    H, dk = m["heads"], m["dim"]
    G = m.get("kv_heads", H)
    dv = m.get("vdim", dk)
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, dk)
    k = (h @ p["k"].T).view(T, G, dk)
    v = (h @ p["v"].T).view(T, G, dv)
    q = rms_unit(q, eps) * p["q.norm"]
    k = rms_unit(k, eps) * p["k.norm"]
    qt = m.get("q_temp")
    if qt:
        q = q * query_gain(pos, qt["coef"], qt["every"])[:, None, None]
    v_raw = v
    if blend:  # every blending layer but the first
        lam = p["vmix"]
        v = (1.0 - lam) * v + lam * v_first
    if past_k is not None:
        k = torch.cat([past_k, k], 0)
        v = torch.cat([past_v, v], 0)
    P = k.shape[0] - T
    out = torch.zeros(T, H, dv, dtype=F64)
    rep = H // G
    for hd in range(H):
        g = hd // rep
        s = (q[:, hd] @ k[:, g].T) * m["scale"]  # [T, P + T]
        j = torch.arange(P + T)[None, :]
        i = (torch.arange(T) + P)[:, None]
        s = s.masked_fill(j > i, float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(T, H * dv) @ p["o"].T, k, v, v_raw


def wkv_mixer(h, p: Dict[str, torch.Tensor], m: dict, eps: float, prev_h=None, state=None):
    """h [T, W]; prev_h [W] the input of the token before h[0] (zeros at the start of a sequence); state [H, d, d]
    indexed [head, key channel, value channel].  Returns (out [T, W], last h, state)."""
    H, d = m["heads"], m["dim"]
    T, W = h.shape
    if prev_h is None:
        prev_h = torch.zeros(W, dtype=F64)
    if state is None:
        state = torch.zeros(H, d, d, dtype=F64)
    shifted = torch.cat([prev_h[None], h[:-1]], 0)
    mix = lambda s: h + (shifted - h) * p[f"mu.{s}"]
    r = (mix("r") @ p["r"].T).view(T, H, d)
    k = (mix("k") @ p["k"].T).view(T, H, d)
    v = (mix("v") @ p["v"].T).view(T, H, d)
    gate = torch.nn.functional.silu(mix("g") @ p["g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix("w") @ p["w1"].T) @ p["w2"].T + p["w0"])).view(T, H, d)
    u = p["u"]  # [H, d]
    o = torch.zeros(T, H, d, dtype=F64)
    S = state.clone()
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]  # [H, d(key), d(value)]
        o[t] = torch.einsum("hij,hi->hj", S + u[:, :, None] * kv, r[t])
        S = decay[t][:, :, None] * S + kv
    o = rms_unit(o, eps).reshape(T, H * d) * p["norm"] * gate
    return o @ p["o"].T, h[-1], S


def dense_ff(h, p, f: dict):
    lim = f["limit"]
    g = torch.clamp(h @ p["gate"].T, max=lim)
    u = torch.clamp(h @ p["up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ p["down"].T


def expert_ff(h, p, prefix: str):
    a = torch.nn.functional.silu(h @ p[f"{prefix}gate"].T) * (h @ p[f"{prefix}up"].T)
    return a @ p[f"{prefix}down"].T


def moe_ff(h, p, f: dict):
    E, top = f["router"]["experts"], f["router"]["top"]
    s = torch.sigmoid(h @ p["router"].T)  # [T, E]
    w, idx = torch.topk(s, top, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += expert_ff((w[t, j] * h[t])[None], p, f"e{e}.")[0]
    if f.get("shared"):
        out = out + torch.sigmoid(h @ p["shared.sg"].T) * expert_ff(h, p, "shared.")
    return out


class LenisunRef:
    def __init__(self, config: dict, tensors: Dict[str, torch.Tensor]):
        self.c = config
        self.t = {k: v.to(F64) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]
        self.layers = config["layers"]
        blenders = [i for i, l in enumerate(self.layers) if l["type"] == "attention" and l["mixer"].get("v_mix")]
        self.first_blender = blenders[0] if blenders else None

    def sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {k[len(prefix):]: v for k, v in self.t.items() if k.startswith(prefix)}

    def new_state(self):
        return {"pos": 0, "layers": [dict() for _ in self.layers]}

    def advance(self, tokens: List[int], st: dict, trace: Optional[list] = None) -> torch.Tensor:
        """Feed `tokens` after what `st` already holds; returns logits [T, vocab] and updates st."""
        T = len(tokens)
        pos = torch.arange(st["pos"], st["pos"] + T)
        x = self.t["embed"][torch.tensor(tokens)] * self.c["embedding"]["scale"]
        v_first = None
        for i, (lay, ls) in enumerate(zip(self.layers, st["layers"])):
            p = self.sub(f"l{i}.mix.")
            h = norm_one_plus(x, self.t[f"l{i}.norm1"], self.eps)
            if lay["type"] == "attention":
                blends = bool(lay["mixer"].get("v_mix"))
                y, ls["k"], ls["v"], v_raw = attention_mixer(
                    h, pos, p, lay["mixer"], self.eps, ls.get("k"), ls.get("v"), v_first,
                    blend=blends and i != self.first_blender)
                if i == self.first_blender:
                    v_first = v_raw
            elif lay["type"] == "wkv":
                y, ls["h"], ls["S"] = wkv_mixer(h, p, lay["mixer"], self.eps, ls.get("h"), ls.get("S"))
            else:
                raise ValueError(lay["type"])
            x = x + norm_one_plus(y, self.t[f"l{i}.norm1b"], self.eps)
            f = lay.get("mlp")
            if f:
                h = norm_one_plus(x, self.t[f"l{i}.norm2"], self.eps)
                fp = self.sub(f"l{i}.mlp.")
                y = dense_ff(h, fp, f) if f["kind"] == "dense" else moe_ff(h, fp, f)
                x = x + norm_one_plus(y, self.t[f"l{i}.norm2b"], self.eps)
            if trace is not None:
                trace.append(x.clone())
        st["pos"] += T
        return norm_one_plus(x, self.t["final.norm"], self.eps) @ self.t["head"].T

    def forward(self, tokens: List[int], trace: Optional[list] = None) -> torch.Tensor:
        return self.advance(tokens, self.new_state(), trace)

    def generate_greedy(self, prompt: List[int], n: int) -> List[int]:
        st = self.new_state()
        logits = self.advance(prompt, st)
        out = []
        for _ in range(n):
            out.append(int(logits[-1].argmax()))
            logits = self.advance([out[-1]], st)
        return out
