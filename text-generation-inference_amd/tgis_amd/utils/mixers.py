"""Sequence mixers and feed-forward blocks for decoders with an fp32 residual stream, built on the ragged-step kernels of
libtgis_hip.so (csrc/residual_f32.hip, attn_varlen.hip, wkv.hip, moe.hip).  Every constant of a mechanism is a constructor
argument, so that a model file only maps its config keys and tensor names onto them.

  NormedQKAttention   softmax attention without a rotation: per-head RMS norm of q and k, optional position-dependent query
                      gain, optional blending of the values with another layer's, separate key / value widths, GQA
  WkvMixer            RWKV-style linear recurrence: token shift, low-rank data-dependent decay, bonus for the current token,
                      per-head unit norm, output gate; state in a RecurrentStateCache slot
  GatedUnit           W_down(act(W_gate h) * W_up h) with the plain SiLU form or the clamped sigmoid(alpha g) * (u + 1) form
  RoutedExperts       sigmoid-scored top-k mixture of GatedUnit experts whose routing weight scales the expert input, plus an
                      optional shared expert behind a sigmoid gate

Activations between kernels are in the serving dtype (bfloat16 or float32); what has to be 32-bit (norm statistics, scores,
softmax weights, router logits, decays, recurrent state) is 32-bit inside the kernels whatever the serving dtype.
All of them run ragged steps: a step's tokens are concatenated by sequence and described by a `StepArgs`-like object with
`cu_seqlens_q`, `ctx_lens`, `slots`, `block_tables`, `state_slots`, `cache`, `state` (models.custom_modeling KVArgs)."""
from typing import Optional

import torch

from tgis_amd import native
from tgis_amd.utils.layers import SKINNY_MAX_M, FastLinear, workspace

# rows up to which the clamped gated unit runs in the epilogue of the weight-streaming GEMM
CLAMPED_EPILOGUE_MAX_M = SKINNY_MAX_M


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


def can_defer(lin: FastLinear) -> bool:
    """May this projection leave its split-K sum to the sandwich norm behind it (decode-sized steps)?  The norm takes the
    slabs with 16-byte loads: widths that are multiples of 4, up to 8192."""
    return lin.streams and lin.out_features % 4 == 0 and lin.out_features <= 8192


def load_linear(weights, name: str) -> FastLinear:
    return FastLinear(weights.get_tensor(name).contiguous(), None)


def load_stacked_linear(weights, names) -> FastLinear:
    """Several [out_i, in] weights that read the same input, as one GEMM."""
    return FastLinear(torch.cat([weights.get_tensor(n) for n in names], dim=0).contiguous(), None)


class NormedQKAttention:
    def __init__(self, weights, prefix: str, layer_id: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 eps: float, gain_coef: float = 0.0, gain_every: int = 0, blend: bool = False):
        self.layer_id = layer_id
        self.H, self.G, self.dk, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.eps = float(scale), float(eps)
        self.gain_coef, self.gain_every = float(gain_coef), int(gain_every)
        self.qkv = load_stacked_linear(weights, [f"{prefix}.q", f"{prefix}.k", f"{prefix}.v"])
        self.o = load_linear(weights, f"{prefix}.o")
        self.q_gain = _f32(weights.get_tensor(f"{prefix}.q.norm"))
        self.k_gain = _f32(weights.get_tensor(f"{prefix}.k.norm"))
        # blend: v <- (1 - lambda) v + lambda v_other, lambda a learned scalar kept on the device
        self.v_lambda = _f32(weights.get_tensor(f"{prefix}.vmix")).reshape(1) if blend else None
        self.defer = can_defer(self.o)

    def values_of(self, qkv: torch.Tensor) -> torch.Tensor:
        """The value columns of a projected step (what another layer blends with)."""
        return qkv[:, (self.H + self.G) * self.dk:]

    def forward(self, h: torch.Tensor, position_ids, step, v_other: Optional[torch.Tensor] = None):
        """h [T, W] -> (out [T, W], qkv [T, H dk + G dk + G dv] with q normed in place)."""
        qkv = self.qkv(h)
        cache = step.cache
        k_pool, v_pool = cache.k_pool(self.layer_id), cache.v_pool(self.layer_id)
        native.qk_norm_kv_write(qkv, position_ids, step.slots, self.q_gain, self.k_gain, self.eps, self.gain_coef,
                                self.gain_every, v_other if self.v_lambda is not None else None, self.v_lambda, k_pool, v_pool,
                                self.H, self.G, self.dk, self.dv)
        att = native.attn_varlen(qkv, k_pool, v_pool, step.block_tables, step.ctx_lens, step.cu_seqlens_q, self.H, self.G,
                                 self.dk, self.dv, self.scale, max_q_len=step.max_q_len, max_ctx=step.max_ctx)
        return self.o(att, partial=self.defer), qkv


class WkvMixer:
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, weights, prefix: str, layer_id: int, heads: int, dim: int, eps: float):
        self.layer_id = layer_id
        self.H, self.d, self.eps = heads, dim, float(eps)
        self.mu = torch.stack([_f32(weights.get_tensor(f"{prefix}.mu.{s}")) for s in self.MIXES]).contiguous()
        self.proj = [load_linear(weights, f"{prefix}.{s}") for s in ("r", "k", "v", "g")]
        self.w1 = load_linear(weights, f"{prefix}.w1")
        self.w2t = _f32(weights.get_tensor(f"{prefix}.w2")).t().contiguous()  # [rank, H d]
        self.w0 = _f32(weights.get_tensor(f"{prefix}.w0"))
        self.u = _f32(weights.get_tensor(f"{prefix}.u")).reshape(-1)
        self.gain = _f32(weights.get_tensor(f"{prefix}.norm"))
        self.o = load_linear(weights, f"{prefix}.o")
        self.defer = can_defer(self.o)

    def forward(self, h32: torch.Tensor, position_ids, step, dtype):
        """h32 [T, W] fp32 (the normed mixer input, kept in fp32 because it is also the shift state)."""
        st = step.state
        state, shift = st.state[self.layer_id], st.shift[self.layer_id]
        mixes = native.token_shift_mix(h32, shift, step.state_slots, step.cu_seqlens_q, position_ids, self.mu, dtype)
        T = h32.shape[0]
        HD = self.H * self.d
        rkvg = torch.empty((4, T, HD), dtype=dtype, device=h32.device)
        for i, lin in enumerate(self.proj):
            lin(mixes[i], out=rkvg[i])
        logw = native.wkv_decay(self.w1(mixes[4]), self.w2t, self.w0)
        out = native.wkv_scan(rkvg[0], rkvg[1], rkvg[2], rkvg[3], logw, self.u, self.gain, state, shift, h32, step.state_slots,
                              step.cu_seqlens_q, position_ids, self.H, self.d, self.eps)
        return self.o(out, partial=self.defer)


class GatedUnit:
    """mode "silu": silu(g) * u.  mode "clamped": g = min(g, limit), u = clamp(u, +-limit), g * sigmoid(alpha g) * (u + 1)."""

    def __init__(self, weights, prefix: str, mode: str = "silu", alpha: float = 1.0, limit: float = 0.0):
        self.gate_up = load_stacked_linear(weights, [f"{prefix}.gate", f"{prefix}.up"])
        self.down = load_linear(weights, f"{prefix}.down")
        self.ff = self.gate_up.out_features // 2
        self.mode = {"silu": 0, "clamped": 1}[mode]
        self.alpha, self.limit = float(alpha), float(limit)
        # the plain SiLU form is the epilogue the weight-streaming kernel already has for the Llama MLP (act 2 on a
        # gate | up image); the clamped form is a launch of its own
        self.fused = self.mode == 0 and self.gate_up.streams and self.ff % 16 == 0
        if self.fused:
            self.gate_up.gate_up = True
        # the clamped form at decode sizes: the same gate | up image with the clamped unit in the epilogue (a second image
        # of the weight; longer steps take the library GEMM on the checkpoint layout and the activation launch)
        self.clamped_image = None
        if self.mode == 1 and self.gate_up.streams and self.ff % 16 == 0 and self.limit > 0:
            self.clamped_image = native.DenseWeight(self.gate_up.weight, gate_up=True)

    def forward(self, h: torch.Tensor, partial: bool = False):
        """partial: the consumer is a sandwich norm, which can finish the down projection's split-K sum itself."""
        partial = partial and can_defer(self.down)
        if self.fused:
            return self.down(self.gate_up(h), partial=partial)
        if self.clamped_image is not None and h.shape[0] <= CLAMPED_EPILOGUE_MAX_M:
            act = native.dense_gemm_clamped_glu(h, self.clamped_image, workspace(h.device), self.alpha, self.limit)
            return self.down(act, partial=partial)
        return self.down(native.glu(self.gate_up(h), self.ff, self.mode, self.alpha, self.limit), partial=partial)

    __call__ = forward


class RoutedExperts:
    def __init__(self, weights, prefix: str, experts: int, top: int, shared: bool):
        self.E, self.k = experts, top
        self.router = _f32(weights.get_tensor(f"{prefix}.router"))
        pad8 = lambda n: (n + 7) // 8 * 8
        gate = [weights.get_tensor(f"{prefix}.e{e}.gate") for e in range(experts)]
        ff, W = gate[0].shape
        # the grouped GEMM reads 16-byte fragments along its inner dimension: widths that are not multiples of 8 are padded
        # with zero rows / columns once, here (silu(0) * 0 = 0 keeps a padded hidden channel out of the result)
        self.W, self.Wp, self.ff = W, pad8(W), pad8(ff)
        pad = lambda t, rows, cols: torch.nn.functional.pad(t, (0, cols - t.shape[1], 0, rows - t.shape[0]))
        # [E, 2 ff, W] (gate rows, then up rows) and [E, W, ff]
        self.w_gate_up = torch.stack([torch.cat([pad(gate[e], self.ff, self.Wp),
                                                 pad(weights.get_tensor(f"{prefix}.e{e}.up"), self.ff, self.Wp)], 0)
                                      for e in range(experts)]).contiguous()
        self.w_down = torch.stack([pad(weights.get_tensor(f"{prefix}.e{e}.down"), W, self.ff) for e in range(experts)]).contiguous()
        self.shared = GatedUnit(weights, f"{prefix}.shared") if shared else None
        self.shared_gate = _f32(weights.get_tensor(f"{prefix}.shared.sg")).reshape(-1) if shared else None

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        T, W = h.shape
        idx, weight, sg = native.moe_route(h, self.router, self.shared_gate, self.k)
        sorted_, tile_expert, pos, n_tiles = native.moe_align(idx, self.E)
        cap = sorted_.shape[0]
        hp = h if self.Wp == W else torch.nn.functional.pad(h, (0, self.Wp - W))
        act = native.moe_gemm(hp, self.w_gate_up, self.ff, tile_expert, n_tiles, cap, sorted_=sorted_, pair_div=self.k,
                              pair_scale=weight.view(-1), glu_act=True)
        rows = native.moe_gemm(act, self.w_down, W, tile_expert, n_tiles, cap)
        shared = self.shared(h) if self.shared is not None else None
        return native.moe_combine(rows, pos, self.k, T, shared=shared, shared_gate=sg)

    __call__ = forward
