"""Lenisun: a hybrid decoder over an fp32 residual stream — softmax-attention layers and RWKV-style recurrent layers in any
order, each followed (optionally) by a clamped gated unit or a routed mixture of experts, with an RMS norm before AND after
every sublayer:

    x <- x + N(mixer(N(x)));    x <- x + N(ff(N(x)))        N(z) = z / sqrt(mean(z^2) + eps) * (1 + gain)

config.json gives the layer list (`layers[i].type`, `.mixer`, `.mlp`), `width`, `vocab`, `norm.eps`, `embedding.scale`;
tensors are named `embed`, `l<i>.norm1|norm1b|norm2|norm2b`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
This file only maps those keys and names onto the mechanisms of utils/mixers.py; the step (ragged: portions of prompts beside
decoded tokens), the paged KV pool and the recurrent state slots are FlashCausalLM's (models/flash_causal_lm.py)."""
import json
import os
from typing import List, Optional

import torch

from tgis_amd import native
from tgis_amd.utils.layers import FastLinear
from tgis_amd.utils.mixers import GatedUnit, NormedQKAttention, RoutedExperts, WkvMixer, _f32

# the sigmoid slope of the clamped gated unit is a constant of the design
CLAMPED_UNIT_ALPHA = 1.702


class LenisunConfig:
    model_type = "lenisun"

    def __init__(self, width: int, vocab: int, layers: List[dict], norm: dict, embedding: Optional[dict] = None, **kwargs):
        self.width, self.vocab, self.layers = int(width), int(vocab), layers
        self.eps = float(norm["eps"])
        self.embedding_scale = float((embedding or {}).get("scale", 1.0))
        # the names the serving path shares with the other families
        self.hidden_size, self.vocab_size, self.num_hidden_layers = self.width, self.vocab, len(layers)
        self.pad_token_id = self.bos_token_id = self.eos_token_id = None
        self.quantize = None
        for k, v in kwargs.items():
            setattr(self, k, v)
        for i, lay in enumerate(layers):
            if lay["type"] not in ("attention", "wkv"):
                raise ValueError(f"layer {i}: unknown mixer type {lay['type']!r}")
            f = lay.get("mlp")
            if f and f.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")

    @classmethod
    def from_json(cls, path: str) -> "LenisunConfig":
        with open(path) as f:
            return cls(**json.load(f))

    def to_dict(self):
        return {"architecture": "Lenisun", "width": self.width, "vocab": self.vocab, "layers": self.layers,
                "norm": {"eps": self.eps}, "embedding": {"scale": self.embedding_scale}}


class LenisunLayer:
    def __init__(self, i: int, config: LenisunConfig, weights, blends: bool):
        lay = config.layers[i]
        m = lay["mixer"]
        self.layer_id = i
        self.kind = lay["type"]
        self.norm1, self.norm1b = (_f32(weights.get_tensor(f"l{i}.{n}")) for n in ("norm1", "norm1b"))
        if self.kind == "attention":
            heads = int(m["heads"])
            temp = m.get("q_temp") or {}
            self.mixer = NormedQKAttention(
                weights, f"l{i}.mix", i, heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(m["dim"]),
                vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]), eps=config.eps,
                gain_coef=float(temp.get("coef", 0.0)), gain_every=int(temp.get("every", 0)) if temp else 0, blend=blends)
            self.kv_shape = (self.mixer.G, self.mixer.dk, self.mixer.dv)
            self.state_shape = None
        else:
            self.mixer = WkvMixer(weights, f"l{i}.mix", i, heads=int(m["heads"]), dim=int(m["dim"]), eps=config.eps)
            self.kv_shape = None
            self.state_shape = (self.mixer.H, self.mixer.d)
        f = lay.get("mlp")
        self.ff = None
        self.dense_ff = bool(f) and f["kind"] == "dense"
        if f:
            self.norm2, self.norm2b = (_f32(weights.get_tensor(f"l{i}.{n}")) for n in ("norm2", "norm2b"))
            if f["kind"] == "dense":
                self.ff = GatedUnit(weights, f"l{i}.mlp", mode="clamped", alpha=CLAMPED_UNIT_ALPHA, limit=float(f["limit"]))
            else:
                self.ff = RoutedExperts(weights, f"l{i}.mlp", experts=int(f["router"]["experts"]), top=int(f["router"]["top"]),
                                        shared=bool(f.get("shared")))


class FlashLenisunModel:
    def __init__(self, config: LenisunConfig, weights):
        if weights.process_group.size() != 1:
            raise NotImplementedError("Lenisun is served by one process per model: its layers are not sharded")
        self.config = config
        self.dtype = weights.dtype
        self.embed = weights.get_tensor("embed").contiguous()
        # value blending: every layer that asks for it but the first blends with the first one's values of the same token
        blenders = [i for i, l in enumerate(config.layers) if l["type"] == "attention" and l["mixer"].get("v_mix")]
        self.first_blender = blenders[0] if blenders else None
        self.layers = [LenisunLayer(i, config, weights, blends=i in blenders[1:]) for i in range(len(config.layers))]
        self.final_norm = _f32(weights.get_tensor("final.norm"))
        # cache geometry, read by FlashCausalLM
        self.kv_layer_shapes = [l.kv_shape for l in self.layers]
        self.state_layer_shapes = [l.state_shape for l in self.layers]
        att = [l.mixer for l in self.layers if l.kind == "attention"]
        self.num_heads = max([a.H for a in att], default=1)
        self.num_key_value_heads = max([a.G for a in att], default=1)
        self.head_size = max([a.dk for a in att], default=8)
        self.supports_ragged_steps = True

    def forward(self, input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds, kv):
        if inputs_embeds is not None:
            raise NotImplementedError("prompt prefixes (inputs_embeds) are not wired into the fp32-residual path")
        cfg, dt = self.config, self.dtype
        kv.cu_seqlens_q = cu_seqlens_q
        x = native.embedding_scaled_f32(input_ids, self.embed, cfg.embedding_scale)
        first = self.layers[0]
        # the normed input of layer 0; afterwards every sublayer's output is normed, added and normed again in one launch
        h = native.sandwich_norm_f32(x, None, None, first.norm1, cfg.eps, torch.float32 if first.kind == "wkv" else dt)
        v_first = None
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            if layer.kind == "attention":
                y, qkv = layer.mixer.forward(h, position_ids, kv, v_first)
                if i == self.first_blender:
                    v_first = layer.mixer.values_of(qkv)
            else:
                y = layer.mixer.forward(h, position_ids, kv, dt)
            nxt = self.layers[i + 1] if i + 1 < n else None
            after_dtype = torch.float32 if (nxt is not None and nxt.kind == "wkv") else dt
            after_gain = nxt.norm1 if nxt is not None else self.final_norm
            if layer.ff is not None:
                h = native.sandwich_norm_f32(x, y, layer.norm1b, layer.norm2, cfg.eps, dt)
                y = layer.ff(h, partial=True) if layer.dense_ff else layer.ff(h)
                h = native.sandwich_norm_f32(x, y, layer.norm2b, after_gain, cfg.eps, after_dtype)
            else:
                h = native.sandwich_norm_f32(x, y, layer.norm1b, after_gain, cfg.eps, after_dtype)
            if kv.residual_trace is not None:
                kv.residual_trace.append(x.clone())
        return h  # final-normed, in the serving dtype

    __call__ = forward


class FlashLenisunForCausalLM:
    def __init__(self, config: LenisunConfig, weights):
        self.config = config
        self.model = FlashLenisunModel(config, weights)
        self.lm_head = FastLinear(weights.get_tensor("head").contiguous(), None)
        self.supports_ragged_steps = True

    def get_input_embeddings(self):
        return None

    @property
    def num_layers(self):
        return len(self.model.layers)

    def forward(self, input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds=None, kv=None,
                lm_head_indices: Optional[torch.Tensor] = None):
        """fp32 logits [T or len(lm_head_indices), vocab]."""
        hidden = self.model(input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds, kv)
        if lm_head_indices is not None:
            hidden = hidden.index_select(0, lm_head_indices)
        # fp32 logits from the weight-streaming kernel's fp32 accumulators, 256 rows at a time (the library GEMM above
        # that size would round them to the serving dtype first)
        if hidden.shape[0] == 0:
            return torch.empty((0, self.config.vocab), dtype=torch.float32, device=hidden.device)
        if hidden.shape[0] <= 256:
            return self.lm_head(hidden, out_f32=True)
        return torch.cat([self.lm_head(hidden[i:i + 256], out_f32=True) for i in range(0, hidden.shape[0], 256)], 0)

    __call__ = forward
