"""Senadra: a pre-norm hybrid decoder over an fp32 residual stream with a residual multiplier m —

    x <- x + m mixer(N1(x));    x <- x + m ff(N2(x));    x <- x + m Ns(side(x, token))         N(z) = z / sqrt(mean(z^2) + eps) * w

with three mixers in any order: block-masked softmax attention with a logarithmic distance bias (optionally reading another
layer's cache), latent attention (low-rank query and key/value latents with one rotated key part), and a gated delta rule
with per-channel decay.  The feed-forward is W_down xielu(W_up h); every layer ends with a gated slice of a second token
embedding; logits are soft-capped.

config.json gives `width`, `vocab`, `layers[i].type|mixer|mlp`, `norm.eps`, `residual_mult`, `token_side.dim`, `logit_softcap`;
tensors are named `embed`, `side.embed`, `l<i>.norm1|norm2`, `l<i>.mix.*`, `l<i>.mlp.*`, `l<i>.side.*`, `final.norm`, `head`.
This file only maps those keys and names onto the mechanisms of utils/mixers.py; the step (ragged: portions of prompts beside
decoded tokens), the paged KV pool and the recurrent state slots are FlashCausalLM's (models/flash_causal_lm.py)."""
import json
from typing import List, Optional

import torch

from tgis_amd import native
from tgis_amd.utils.layers import FastLinear
from tgis_amd.utils.mixers import ActivatedMLP, BlockBiasedAttention, DeltaRuleMixer, LatentAttention, TokenSideInput, _f32

# the unit vectors of the delta rule are x / sqrt(|x|^2 + this): a constant of the design
DELTA_UNIT_EPS = 1e-6
MIXER_TYPES = ("attention", "latent_attention", "channel_delta")


class SenadraConfig:
    model_type = "senadra"

    def __init__(self, width: int, vocab: int, layers: List[dict], norm: dict, residual_mult: float = 1.0,
                 token_side: Optional[dict] = None, logit_softcap: Optional[float] = None, **kwargs):
        self.width, self.vocab, self.layers = int(width), int(vocab), layers
        self.eps = float(norm["eps"])
        self.residual_mult = float(residual_mult)
        self.side_dim = int(token_side["dim"]) if token_side else 0
        self.logit_softcap = float(logit_softcap) if logit_softcap else 0.0
        # the names the serving path shares with the other families
        self.hidden_size, self.vocab_size, self.num_hidden_layers = self.width, self.vocab, len(layers)
        self.pad_token_id = self.bos_token_id = self.eos_token_id = None
        self.quantize = None
        for k, v in kwargs.items():
            setattr(self, k, v)
        for i, lay in enumerate(layers):
            if lay["type"] not in MIXER_TYPES:
                raise ValueError(f"layer {i}: unknown mixer type {lay['type']!r}")
            f = lay.get("mlp")
            if f and f.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
            src = lay["mixer"].get("kv_from")
            if src is not None:
                if lay["type"] != "attention" or not (0 <= src < len(layers)) or layers[src]["type"] != "attention" \
                        or layers[src]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from must name an attention layer with keys and values of its own")

    @classmethod
    def from_json(cls, path: str) -> "SenadraConfig":
        with open(path) as f:
            return cls(**json.load(f))

    def to_dict(self):
        d = {"architecture": "Senadra", "width": self.width, "vocab": self.vocab, "layers": self.layers, "norm": {"eps": self.eps},
             "residual_mult": self.residual_mult}
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        return d


class SenadraLayer:
    def __init__(self, i: int, config: SenadraConfig, weights, side_table: Optional[torch.Tensor]):
        lay = config.layers[i]
        m = lay["mixer"]
        self.layer_id, self.kind = i, lay["type"]
        self.norm1 = _f32(weights.get_tensor(f"l{i}.norm1"))
        self.kv_shape = self.state_shape = None
        if self.kind == "attention":
            heads = int(m["heads"])
            self.mixer = BlockBiasedAttention(
                weights, f"l{i}.mix", i, heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(m["dim"]),
                vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]), eps=config.eps,
                chunk=int((m.get("mask") or {}).get("size", 0)), kv_source=m.get("kv_from"))
            if self.mixer.own_kv:
                self.kv_shape = (self.mixer.G, self.mixer.dk, self.mixer.dv)
        elif self.kind == "latent_attention":
            rot = m.get("rot") or {}
            self.mixer = LatentAttention(
                weights, f"l{i}.mix", i, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                kv_rank=int(m["kv_rank"]), scale=float(m["scale"]), eps=config.eps, rot_base=float(rot.get("base", 10000.0)),
                rot_dims=int(rot.get("dims", m["rot_dim"])))
            self.kv_shape = self.mixer.kv_shape
        else:
            heads = int(m["heads"])
            self.mixer = DeltaRuleMixer(
                weights, f"l{i}.mix", i, heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(m["dim"]),
                vdim=int(m.get("vdim", m["dim"])), taps=int(m["conv"]), eps=config.eps, unit_eps=DELTA_UNIT_EPS)
            self.state_shape = self.mixer.state_shape
        self.ff = None
        if lay.get("mlp"):
            self.norm2 = _f32(weights.get_tensor(f"l{i}.norm2"))
            self.ff = ActivatedMLP(weights, f"l{i}.mlp")
        self.side = TokenSideInput(weights, f"l{i}.side", i, side_table, config.side_dim) if side_table is not None else None


class FlashSenadraModel:
    def __init__(self, config: SenadraConfig, weights):
        if weights.process_group.size() != 1:
            raise NotImplementedError("Senadra is served by one process per model: its layers are not sharded")
        self.config = config
        self.dtype = weights.dtype
        self.embed = weights.get_tensor("embed").contiguous()
        self.side_table = weights.get_tensor("side.embed").contiguous() if config.side_dim else None
        self.layers = [SenadraLayer(i, config, weights, self.side_table) for i in range(len(config.layers))]
        self.final_norm = _f32(weights.get_tensor("final.norm"))
        # cache geometry, read by FlashCausalLM (layers that read another layer's keys and values have none)
        self.kv_layer_shapes = [l.kv_shape for l in self.layers]
        self.state_layer_shapes = [l.state_shape for l in self.layers]
        shapes = [s for s in self.kv_layer_shapes if s is not None]
        att = [l.mixer for l in self.layers if l.kind != "channel_delta"]
        self.num_heads = max([a.H for a in att], default=1)
        self.num_key_value_heads = max([s[0] for s in shapes], default=1)
        self.head_size = max([s[1] for s in shapes], default=8)
        self.supports_ragged_steps = True

    def forward(self, input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds, kv):
        if inputs_embeds is not None:
            raise NotImplementedError("prompt prefixes (inputs_embeds) are not wired into the fp32-residual path")
        cfg, dt = self.config, self.dtype
        m, eps = cfg.residual_mult, cfg.eps
        kv.cu_seqlens_q = cu_seqlens_q
        x = native.embedding_scaled_f32(input_ids, self.embed, 1.0)
        # the normed input of layer 0; afterwards every sublayer's output is added (times m) and the sum normed in one launch
        h = native.residual_update_f32(x, None, None, self.layers[0].norm1, eps, dt)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            y = layer.mixer.forward(h, position_ids, kv)
            if layer.ff is not None:
                h = native.residual_update_f32(x, y, None, layer.norm2, eps, dt, post_scale=m)
                y = layer.ff(h, partial=True)
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            if layer.side is not None:
                # the side input reads the residual stream itself: it leaves the sum rounded to the activation dtype
                x_act = native.residual_update_f32(x, y, None, None, eps, dt, post_scale=m, cast=True)
                y = layer.side(x_act, input_ids)
                h = native.residual_update_f32(x, y, layer.side.gain, nxt, eps, dt, post_scale=m)
            else:
                h = native.residual_update_f32(x, y, None, nxt, eps, dt, post_scale=m)
            if kv.residual_trace is not None:
                kv.residual_trace.append(x.clone())
        return h  # final-normed, in the serving dtype

    __call__ = forward


class FlashSenadraForCausalLM:
    def __init__(self, config: SenadraConfig, weights):
        self.config = config
        self.model = FlashSenadraModel(config, weights)
        self.lm_head = FastLinear(weights.get_tensor("head").contiguous(), None)
        self.supports_ragged_steps = True

    def get_input_embeddings(self):
        return None

    @property
    def num_layers(self):
        return len(self.model.layers)

    def forward(self, input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds=None, kv=None,
                lm_head_indices: Optional[torch.Tensor] = None):
        """fp32 logits [T or len(lm_head_indices), vocab], soft-capped."""
        hidden = self.model(input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds, kv)
        if lm_head_indices is not None:
            hidden = hidden.index_select(0, lm_head_indices)
        if hidden.shape[0] == 0:
            return torch.empty((0, self.config.vocab), dtype=torch.float32, device=hidden.device)
        # fp32 logits from the weight-streaming kernel's fp32 accumulators, 256 rows at a time (the library GEMM above that
        # size would round them to the serving dtype first)
        if hidden.shape[0] <= 256:
            logits = self.lm_head(hidden, out_f32=True)
        else:
            logits = torch.cat([self.lm_head(hidden[i:i + 256], out_f32=True) for i in range(0, hidden.shape[0], 256)], 0)
        if self.config.logit_softcap:
            native.logit_softcap(logits, self.config.logit_softcap)
        return logits

    __call__ = forward
