"""GPU: the Senadra family on the kernels (FlashCausalLM + utils/mixers.py + csrc/residual_f32, attn_varlen, delta_rule)
against the plain float64 restatement in oracle/senadra_ref.py, on small seeded checkpoints of their own sizes.

float32 serving is compared tightly (it differs from the oracle by accumulation order only); bfloat16 serving against a
bound that scales with bf16 rounding.  Schedules (whole prompts, token by token, portions down to two tokens, mixed batches,
pages and slots that change hands) are compared with the oracle run whole, where only rounding may differ."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import senadra_ref as ref
from oracle import senadra_tiny as tiny

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-4, torch.bfloat16: 0.15}
DTYPES = [torch.float32, torch.bfloat16]


def build_lm(cfg, tensors, dtype, pages=64, slots=4, tokenizer=None):
    from tgis_amd.inference_engine.synthetic import InferenceEngine
    from tgis_amd.models.custom_modeling.flash_senadra_modeling import SenadraConfig
    from tgis_amd.models.flash_causal_lm import FlashCausalLM

    eng = InferenceEngine({k: v.clone() for k, v in tensors.items()}, SenadraConfig(**cfg), dtype, None, tokenizer=tokenizer)
    return FlashCausalLM("synthetic", None, "synthetic", dtype, None, engine=eng, kv_cache_pages=pages, state_slots=slots)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest row error: rms of the centred difference over the rms of the centred reference row."""
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def rand_tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.fixture(scope="module")
def std():
    cfg = tiny.make_config(tiny.standard_layers())
    return cfg, tiny.make_tensors(cfg, seed=3)


# ---- whole model -----------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [75, 300])
def test_whole_prompt_matches_oracle_layer_by_layer(gpu_device, std, dtype, n):
    """75 tokens: the decode-sized GEMM path (split-K sums finished by the residual update behind them); 300: the library
    GEMMs.  Both cross several attention blocks of 48 positions."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(n, cfg["vocab"], 1)
    want_trace = []
    want = ref.forward(cfg, tensors, toks, want_trace)
    with lm.context_manager():
        seq = lm.open_sequence()
        trace = []
        got = lm.step_sequences([(seq, toks)], None, residual_trace=trace)
    assert len(trace) == len(want_trace)
    for i, (g, w) in enumerate(zip(trace, want_trace)):
        assert rel_err(g, w) <= TOL[dtype], f"layer {i}"
    assert rel_err(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_by_token_and_portions_equal_whole(gpu_device, std, dtype):
    """Prefill against decoding one token at a time, and portions of several sizes down to two tokens, some of them ending or
    starting on a page border (32) or on a block border of the attention mask (48)."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(101, cfg["vocab"], 2)
    want = ref.forward(cfg, tensors, toks)
    with lm.context_manager():
        for cuts in ([1] * 101, [2] * 50 + [1], [31, 1, 2, 30, 3, 29, 5], [32, 32, 32, 5], [48, 48, 5], [47, 2, 2, 50], [7, 57, 37]):
            assert sum(cuts) == 101
            seq = lm.open_sequence()
            at, outs = 0, []
            for n in cuts:
                outs.append(lm.step_sequences([(seq, toks[at:at + n])], None))
                at += n
            assert rel_err(torch.cat(outs), want) <= TOL[dtype], cuts
            lm.close_sequence(seq)


@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reuse_pages_and_slots(gpu_device, std, dtype):
    """Up to four live requests of unequal length, portions of some beside single tokens of others, in a pool that is too
    small to hold all requests at once: pages and slots go back and are handed out again, to other requests."""
    cfg, tensors = std
    lens = [70, 33, 95, 5, 64, 40, 1]
    prompts = [rand_tokens(n, cfg["vocab"], 10 + i) for i, n in enumerate(lens)]
    want = [ref.forward(cfg, tensors, p) for p in prompts]
    lm = build_lm(cfg, tensors, dtype, pages=9, slots=4)  # 9 pages = 288 tokens < sum(lens)
    rng = np.random.default_rng(0)
    got = [[] for _ in prompts]
    done = [0] * len(prompts)
    live, waiting = {}, list(range(len(prompts)))
    with lm.context_manager():
        while waiting or live:
            while waiting and len(live) < 4:
                i = waiting[0]
                if sum((lens[j] + 31) // 32 for j in live) + (lens[i] + 31) // 32 > 9:
                    break
                live[waiting.pop(0)] = lm.open_sequence()
            entries, who = [], []
            for i, seq in live.items():
                left = lens[i] - done[i]
                n = 1 if (left == 1 or rng.random() < 0.4) else int(rng.integers(2, min(left, 40) + 1))
                entries.append((seq, prompts[i][done[i]:done[i] + n]))
                who.append((i, n))
            logits = lm.step_sequences(entries, None)
            at = 0
            for i, n in who:
                got[i].append(logits[at:at + n])
                at += n
                done[i] += n
                if done[i] == lens[i]:
                    lm.close_sequence(live.pop(i))
    assert lm.kv_cache.free_pages == 9 and lm.state_cache.free_slots == 4
    for i in range(len(prompts)):
        assert rel_err(torch.cat(got[i]), want[i]) <= TOL[dtype], i


def test_stale_slot_and_pages_do_not_leak(gpu_device, std):
    """A request that takes over a slot and pages still holding another request's state, convolution tail and keys computes
    what it computes in a fresh pool; also its first tokens (position 0: zero state, zeros before the start)."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, torch.float32, pages=4, slots=1)
    a, b = rand_tokens(120, cfg["vocab"], 5), rand_tokens(50, cfg["vocab"], 6)
    with lm.context_manager():
        s = lm.open_sequence()
        lm.step_sequences([(s, a)], None)
        lm.close_sequence(s)
        s = lm.open_sequence()
        got = torch.cat([lm.step_sequences([(s, b[:1])], None), lm.step_sequences([(s, b[1:3])], None),
                         lm.step_sequences([(s, b[3:])], None)])
    assert rel_err(got, ref.forward(cfg, tensors, b)) <= TOL[torch.float32]


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(gpu_device, std, dtype):
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(40 + 200, cfg["vocab"], 8)
    want = ref.forward(cfg, tensors, toks)
    with lm.context_manager():
        s = lm.open_sequence()
        outs = [lm.step_sequences([(s, toks[:40])], None)]
        for t in toks[40:]:
            outs.append(lm.step_sequences([(s, [t])], None))
    assert rel_err(torch.cat(outs), want) <= TOL[dtype]


OTHER_SHAPES = {
    # odd widths everywhere (the general attention kernel, library GEMMs), no side input, no soft cap, multiplier 1,
    # a delta rule first, block size 1 (every token sees itself only) and an unmasked attention layer
    "odd": dict(layers=[tiny.delta_layer(heads=2, kv_heads=1, dim=20, vdim=12, conv=2, mlp=tiny.dense_mlp(50)),
                        tiny.attention_layer(heads=3, kv_heads=3, dim=12, vdim=20, scale=0.3, chunk=None, mlp=None),
                        tiny.latent_layer(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=22, q_rank=18, rot_dims=4, mlp=tiny.dense_mlp(34)),
                        tiny.attention_layer(heads=3, kv_heads=3, dim=12, vdim=20, scale=0.3, chunk=1, kv_from=1, mlp=tiny.dense_mlp(30))],
                width=36, vocab=50, residual_mult=1.0, side_dim=None, softcap=None, low_rank=5),
    # matrix-core shapes: wide heads, MQA, a key width of 176 for the latent layer's pages, five taps, block = one page
    "wide": dict(layers=[tiny.latent_layer(heads=8, dim=48, rot_dim=16, vdim=64, kv_rank=160, q_rank=56, scale=0.1, mlp=tiny.dense_mlp(128)),
                         tiny.attention_layer(heads=8, kv_heads=1, dim=128, vdim=128, scale=0.09, chunk=32, mlp=tiny.dense_mlp(64)),
                         tiny.delta_layer(heads=2, kv_heads=2, dim=128, vdim=64, conv=5, mlp=None),
                         tiny.delta_layer(heads=4, kv_heads=1, dim=64, vdim=128, conv=4, mlp=tiny.dense_mlp(64))],
                 width=128, vocab=120, residual_mult=0.25, side_dim=16, softcap=8.0, low_rank=16),
    # a single layer of each kind
    "attn": dict(layers=[tiny.attention_layer(heads=4, kv_heads=2, dim=16, vdim=32, chunk=33, mlp=None)], width=32, vocab=40),
    "latent": dict(layers=[tiny.latent_layer(mlp=None)], width=32, vocab=40, side_dim=4),
    "delta": dict(layers=[tiny.delta_layer(mlp=None)], width=32, vocab=40, softcap=3.0),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(OTHER_SHAPES))
def test_other_sizes_and_layer_orders(gpu_device, dtype, shape):
    """Whole, then in portions with single tokens, for configurations that share no size with the standard one."""
    kw = dict(OTHER_SHAPES[shape])
    low_rank = kw.pop("low_rank", 8)
    cfg = tiny.make_config(**kw)
    tensors = tiny.make_tensors(cfg, seed=21, low_rank=low_rank)
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(90, cfg["vocab"], 4)
    want = ref.forward(cfg, tensors, toks)
    with lm.context_manager():
        for cuts in ([90], [33, 1, 1, 2, 30, 23]):
            seq = lm.open_sequence()
            at, outs = 0, []
            for n in cuts:
                outs.append(lm.step_sequences([(seq, toks[at:at + n])], None))
                at += n
            assert rel_err(torch.cat(outs), want) <= TOL[dtype], cuts
            lm.close_sequence(seq)


# ---- attention: keys that must or must not be seen -------------------------------------------------------------------------
def _planted(dtype, key_pos, n_ctx, q_chunks, chunk, H, G, dk, dv, bias):
    """q of the LAST token and k of token `key_pos` are made parallel and large, v of that token is a marker: the last
    token's output is the marker iff the kernel sees that key.  Returns (output of the last token, marker per head)."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(key_pos * 1000 + n_ctx)
    qkv = torch.randn(n_ctx, (H + G) * dk + G * dv, generator=g) * 0.1
    direction = torch.nn.functional.normalize(torch.randn(dk, generator=g), dim=0) * 6
    for h in range(H):
        qkv[n_ctx - 1, h * dk:(h + 1) * dk] = direction
    for gg in range(G):
        qkv[key_pos, (H + gg) * dk:(H + gg + 1) * dk] = direction
    marker = torch.arange(1, G * dv + 1, dtype=torch.float32) * 0.25 + 50
    qkv[key_pos, (H + G) * dk:] = marker
    cache = PagedKVCache(1, G, dk, 40, dtype, dev, layer_shapes=[(G, dk, dv)])
    pages = cache.alloc((n_ctx + PAGE - 1) // PAGE)
    np.random.default_rng(1).shuffle(pages)  # pages of a sequence are scattered over the pool
    bt = torch.tensor([pages], dtype=torch.int32, device=dev)
    r1 = torch.full((H,), 0.2, device=dev) if bias else None
    r2 = torch.full((H,), 0.5, device=dev) if bias else None
    out_last, at = None, 0
    for n in q_chunks:
        pos = torch.arange(at, at + n)
        slots = (torch.tensor(pages, dtype=torch.int64)[pos // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
        x = qkv[at:at + n].to(dtype).to(dev).contiguous()
        native.kv_norm_write(x, H * dk, (H + G) * dk, slots, cache.k_pool(0), cache.v_pool(0), G, dk, dv, False, 1e-6)
        ctx = torch.tensor([at + n], dtype=torch.int32, device=dev)
        cu = torch.tensor([0, n], dtype=torch.int32, device=dev)
        o = native.attn_varlen_ext(x, cache.k_pool(0), cache.v_pool(0), bt, ctx, cu, H, G, dk, dv, 1.0, r1, r2, chunk, max_q_len=n,
                                   max_ctx=at + n)
        out_last = o[-1]
        at += n
    torch.cuda.synchronize()
    return out_last.float().cpu(), marker.view(G, dv).repeat_interleave(H // G, 0).reshape(-1)


# (H, G, dk, dv): the general kernel (odd widths) and the matrix-core kernel's shapes under bf16 (narrow: staged; wide: direct)
GEOMETRIES = [(4, 2, 12, 8), (8, 2, 64, 64), (4, 4, 128, 64), (8, 1, 32, 96)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", GEOMETRIES)
@pytest.mark.parametrize("chunk", [0, 224, 96, 50])
def test_attention_sees_its_block_and_nothing_before_it(gpu_device, dtype, geom, chunk):
    """700 tokens; the query is the last one (position 699).  Keys inside its block — its first position, a page border, the
    query's neighbour — must be found; the key just before the block, far keys and position 0 must not (without a mask all
    are found).  In a prompt run whole, cut into portions (one of two tokens), and with the last token decoded alone."""
    n = 700
    start = (n - 1) // chunk * chunk if chunk else 0
    inside = sorted({start, start + 1, min(start + 31, n - 1), min(start + 32, n - 1), n - 2, n - 1} |
                    ({33, 255, 256} if not chunk else set()))
    outside = [] if not chunk else sorted({0, 1, start - 1, start - 2, start - 33, 31, 32} - set(range(start, n)))
    for chunks in ([n], [300, 2, 397, 1], [n - 1, 1]):
        for key_pos in inside:
            got, want = _planted(dtype, key_pos, n, chunks, chunk, *geom, bias=True)
            assert torch.allclose(got, want, atol=0.3 if dtype == torch.bfloat16 else 1e-2, rtol=0.01), (chunks, key_pos, got[:3], want[:3])
        for key_pos in outside:
            got, _ = _planted(dtype, key_pos, n, chunks, chunk, *geom, bias=False)
            assert float(got.abs().max()) < 5.0, (chunks, key_pos, got[:3])


def _plain_block_attention(q, k, v, scale, H, G, chunk, r1, r2):
    n_q, n = q.shape[0], k.shape[0]
    out = torch.zeros(n_q, H, v.shape[2], dtype=torch.float64)
    i = (torch.arange(n_q) + n - n_q)[:, None]
    j = torch.arange(n)[None, :]
    hidden = j > i
    if chunk:
        hidden = hidden | (i // chunk != j // chunk)
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale - r1[h] * torch.log1p(r2[h] * (i - j).clamp(min=0).double())
        out[:, h] = torch.softmax(s.masked_fill(hidden, float("-inf")), -1) @ v[:, h // (H // G)]
    return out.reshape(n_q, -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", GEOMETRIES + [(16, 1, 64, 128), (2, 2, 256, 256), (34, 2, 32, 32), (3, 1, 48, 72)])
@pytest.mark.parametrize("chunk", [0, 77])
def test_attention_ragged_batch_against_plain_softmax(gpu_device, dtype, geom, chunk):
    """A step of unequal sequences — whole prompts, a portion that continues a long context, single decoded tokens, one of
    them behind 3000 cached keys — through both kernels (where the matrix-core one applies) against plain softmax with the
    distance bias, the block mask and unit-RMS values."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    H, G, dk, dv = geom
    dev = torch.device("cuda:0")
    cached = [0, 200, 3000, 31, 0, 64]
    new = [70, 45, 1, 1, 1, 33]
    g = torch.Generator().manual_seed(H * 1000 + dk)
    cache = PagedKVCache(1, G, dk, 130, dtype, dev, layer_shapes=[(G, dk, dv)])
    r1, r2 = torch.rand(H, generator=g) * 0.5, torch.rand(H, generator=g) * 0.3
    kcol, vcol = H * dk, (H + G) * dk
    full, pages = [], []
    for c, n in zip(cached, new):
        x = (torch.randn(c + n, (H + G) * dk + G * dv, generator=g) * (2.0 / dk ** 0.25)).to(dtype)
        pg = cache.alloc((c + n + PAGE - 1) // PAGE)
        if c:  # what earlier steps left in the cache (c >= 512 goes through the transposing value writer)
            pos = torch.arange(c)
            slots = (torch.tensor(pg)[pos // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
            native.kv_norm_write(x[:c].to(dev).contiguous(), kcol, vcol, slots, cache.k_pool(0), cache.v_pool(0), G, dk, dv, True, 1e-5)
        full.append(x)
        pages.append(pg)
    step = torch.cat([x[c:] for x, c in zip(full, cached)]).to(dev).contiguous()
    slots = torch.cat([(torch.tensor(pg)[torch.arange(c, c + n) // PAGE] * PAGE + torch.arange(c, c + n) % PAGE)
                       for pg, c, n in zip(pages, cached, new)]).to(torch.int32).to(dev)
    native.kv_norm_write(step, kcol, vcol, slots, cache.k_pool(0), cache.v_pool(0), G, dk, dv, True, 1e-5)
    bt = torch.zeros(len(pages), max(len(p) for p in pages), dtype=torch.int32)
    for i, p in enumerate(pages):
        bt[i, :len(p)] = torch.tensor(p)
    ctx = torch.tensor([c + n for c, n in zip(cached, new)], dtype=torch.int32, device=dev)
    cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32, device=dev)
    want = []
    for x, c, n in zip(full, cached, new):
        xd = x.double()
        v = ref.rms_unit(xd[:, vcol:].view(c + n, G, dv), 1e-5).to(dtype).double()
        want.append(_plain_block_attention(xd[c:, :kcol].view(n, H, dk), xd[:, kcol:vcol].view(c + n, G, dk), v, 0.5, H, G, chunk,
                                           r1.double(), r2.double()))
    want = torch.cat(want)
    impls = [1] + ([2] if dtype == torch.bfloat16 and dk % 16 == 0 and dv % 32 == 0 else [])
    gate = torch.randn(want.shape[0], H * dv, generator=g).to(dtype)
    for impl in impls:
        got = native.attn_varlen_ext(step, cache.k_pool(0), cache.v_pool(0), bt.to(dev), ctx, cu, H, G, dk, dv, 0.5, r1.to(dev), r2.to(dev),
                                     chunk, max_q_len=max(new), max_ctx=3001, impl=impl)
        err = (got.double().cpu() - want).abs().max() / want.abs().max()
        assert float(err) <= (2e-5 if dtype == torch.float32 else 2e-2), (impl, float(err))
        # the sigmoid output gate in the kernel's epilogue
        got = native.attn_varlen_ext(step, cache.k_pool(0), cache.v_pool(0), bt.to(dev), ctx, cu, H, G, dk, dv, 0.5, r1.to(dev), r2.to(dev),
                                     chunk, gate.to(dev), max_q_len=max(new), max_ctx=3001, impl=impl)
        err = (got.double().cpu() - want * torch.sigmoid(gate.double())).abs().max() / want.abs().max()
        assert float(err) <= (2e-5 if dtype == torch.float32 else 2e-2), ("gated", impl, float(err))
    if 2 in impls:  # decode-only steps take the key-split form of the matrix-core kernel
        sel = [i for i, n in enumerate(new) if n == 1]
        rows = [int(cu[i]) for i in sel]
        got = native.attn_varlen_ext(step[rows].contiguous(), cache.k_pool(0), cache.v_pool(0), bt[sel].contiguous().to(dev),
                                     ctx[sel].contiguous(), torch.arange(len(sel) + 1, dtype=torch.int32, device=dev), H, G, dk, dv, 0.5,
                                     r1.to(dev), r2.to(dev), chunk, gate[rows].contiguous().to(dev), max_q_len=1, max_ctx=3001, impl=2)
        err = (got.double().cpu() - (want * torch.sigmoid(gate.double()))[rows]).abs().max() / want.abs().max()
        assert float(err) <= 2e-2, float(err)
        # with scratch memory the pages of these few sequences are dealt to several workgroups and combined afterwards
        ws = native.Workspace(8 << 20, dev)
        got2 = native.attn_varlen_ext(step[rows].contiguous(), cache.k_pool(0), cache.v_pool(0), bt[sel].contiguous().to(dev),
                                      ctx[sel].contiguous(), torch.arange(len(sel) + 1, dtype=torch.int32, device=dev), H, G, dk, dv, 0.5,
                                      r1.to(dev), r2.to(dev), chunk, gate[rows].contiguous().to(dev), max_q_len=1, max_ctx=3001, impl=2, ws=ws)
        err = (got2.double().cpu() - (want * torch.sigmoid(gate.double()))[rows]).abs().max() / want.abs().max()
        assert float(err) <= 2e-2, ("key splits", float(err))
        assert torch.all(ws.buf[:4096] == 0)  # the GEMMs' arrival counters are not scratch


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------
def _dict_weights(tensors, dtype):
    from tgis_amd.utils.dist import FakeGroup
    from tgis_amd.utils.weights import DictWeights

    return DictWeights(tensors, device=torch.device("cuda:0"), dtype=dtype, process_group=FakeGroup(0, 1))


def _f64(tensors, prefix):
    return {k[len(prefix):]: v.double() for k, v in tensors.items() if k.startswith(prefix)}


def _kv_step(cache, pages, at, m, state=None, slot=None):
    from tgis_amd.models.custom_modeling.flash_llama_modeling import KVArgs
    from tgis_amd.utils.kv_cache import PAGE

    dev = torch.device("cuda:0")
    pos = torch.arange(at, at + m)
    return KVArgs(cache=cache, block_tables=torch.tensor([pages], dtype=torch.int32, device=dev) if pages else None,
                  ctx_lens=torch.tensor([at + m], dtype=torch.int32, device=dev),
                  slots=(torch.tensor(pages)[pos // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev) if pages else None,
                  max_q_len=m, max_ctx=at + m, cu_seqlens_q=torch.tensor([0, m], dtype=torch.int32, device=dev), state=state,
                  state_slots=torch.tensor([slot], dtype=torch.int32, device=dev) if slot is not None else None), pos.to(torch.int32).to(dev)


@pytest.mark.parametrize("dtype", DTYPES)
def test_residual_update(gpu_device, dtype):
    """x += m delta (plain, normed with a gain, from split-K slabs); y = norm(x) w, or x rounded."""
    from tgis_amd import native
    from tgis_amd.utils.layers import FastLinear

    g = torch.Generator().manual_seed(0)
    for E in (8, 36, 257, 1024):
        x = torch.randn(5, E, generator=g)
        delta = (torch.randn(5, E, generator=g) * 3).to(dtype)
        wb, w = torch.randn(E, generator=g), torch.randn(E, generator=g)
        tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
        xd = x.cuda()
        y = native.residual_update_f32(xd, delta.cuda(), None, w.cuda(), 1e-3, dtype, post_scale=0.3)
        want_x = x.double() + 0.3 * delta.double()
        assert torch.allclose(xd.cpu().double(), want_x, atol=1e-5, rtol=1e-5)
        assert torch.allclose(y.cpu().double(), ref.rms_unit(want_x, 1e-3) * w.double(), **tol)
        y = native.residual_update_f32(xd, delta.cuda(), wb.cuda(), None, 1e-3, dtype, post_scale=0.7, cast=True)
        want_x = want_x + 0.7 * ref.rms_unit(delta.double(), 1e-3) * wb.double()
        assert torch.allclose(xd.cpu().double(), want_x, atol=1e-5, rtol=1e-5)
        assert torch.allclose(y.cpu().double(), want_x, **tol)
        assert native.residual_update_f32(xd, delta.cuda(), None, None, 1e-3, post_scale=-1.0) is None
        assert torch.allclose(xd.cpu().double(), want_x - delta.double(), atol=1e-5, rtol=1e-5)
    if dtype == torch.bfloat16:
        for M, K, N in ((1, 512, 256), (33, 2048, 512)):
            wt = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype).cuda()
            a = torch.randn(M, K, generator=g).to(dtype).cuda()
            x = torch.randn(M, N, generator=g).cuda()
            wn = torch.randn(N, generator=g).cuda()
            part = FastLinear(wt, None)(a, partial=True)
            assert isinstance(part, native.Partial)
            x_ref = x.double().cpu() + 0.5 * (a.double().cpu() @ wt.double().cpu().T)
            y = native.residual_update_f32(x, part, None, wn, 1e-5, torch.float32, post_scale=0.5)
            assert torch.allclose(x.double().cpu(), x_ref, atol=2e-3, rtol=1e-3)
            assert torch.allclose(y.double().cpu(), ref.rms_unit(x_ref, 1e-5) * wn.double().cpu(), atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_small_kernels(gpu_device, dtype):
    """xIELU on both sides of zero, the gated lookup, the output gate, latent norms and the soft cap."""
    from tgis_amd import native

    g = torch.Generator().manual_seed(1)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    z = (torch.randn(7, 50, generator=g) * 3).to(dtype)
    pq = torch.tensor([0.4, -0.7], dtype=torch.float64)
    ap, an = float(ref.softplus(pq[0])), 0.5 + float(ref.softplus(pq[1]))
    assert torch.allclose(native.xielu(z.cuda(), ap, an).cpu().double(), ref.xielu(z.double(), pq), **tol)
    gate = torch.randn(7, 50, generator=g).to(dtype)
    assert torch.allclose(native.sigmoid_gate_mul(z.cuda(), gate.cuda()).cpu().double(), z.double() * torch.sigmoid(gate.double()), **tol)
    table = torch.randn(11, 30, generator=g).to(dtype)
    ids = torch.randint(0, 11, (7,), generator=g)
    t = torch.randn(7, 6, generator=g).to(dtype)
    want = ref.gelu_tanh(t.double()) * table.double()[ids][:, 12:18]
    assert torch.allclose(native.gelu_gated_lookup(t.cuda(), ids.cuda(), table.cuda(), 12).cpu().double(), want, **tol)
    w = torch.randn(50, generator=g)
    assert torch.allclose(native.rms_norm_rows(z.cuda()[:, :50], w.cuda(), 1e-4).cpu().double(), ref.rms_unit(z.double(), 1e-4) * w.double(), **tol)
    lg = torch.randn(3, 40, generator=g) * 20
    assert torch.allclose(native.logit_softcap(lg.cuda(), 7.0).cpu().double(), 7.0 * torch.tanh(lg.double() / 7.0), atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [37, 300])
def test_activated_mlp_and_side_input(gpu_device, dtype, T):
    from tgis_amd.utils.mixers import ActivatedMLP, TokenSideInput

    cfg = tiny.make_config([tiny.delta_layer(mlp=tiny.dense_mlp(72)), tiny.delta_layer(mlp=None)], width=48, side_dim=8)
    tensors = tiny.make_tensors(cfg, 1)
    wts = _dict_weights(tensors, dtype)
    g = torch.Generator().manual_seed(2)
    h = torch.randn(T, 48, generator=g).to(dtype)
    mlp = ActivatedMLP(wts, "l0.mlp")
    assert rel_err(mlp(h.cuda()), ref.dense_ff(h.double(), _f64(tensors, "l0.mlp."))) <= TOL[dtype]
    side = TokenSideInput(wts, "l1.side", 1, wts.get_tensor("side.embed"), 8)
    side.defer = False
    ids = torch.randint(0, cfg["vocab"], (T,), generator=g)
    got = side(h.cuda(), ids.cuda())
    p = _f64(tensors, "l1.side.")
    want = (ref.gelu_tanh(h.double() @ p["gate"].T) * tensors["side.embed"].double()[ids][:, 8:16]) @ p["proj"].T
    assert rel_err(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,taps", [(4, 2, 16, 32, 3), (3, 3, 32, 16, 4), (2, 1, 20, 12, 2), (2, 2, 128, 64, 5),
                                                          (1, 1, 64, 128, 4), (2, 1, 200, 40, 3), (2, 2, 16, 16, 1)])
def test_delta_rule_mixer_and_its_state(gpu_device, dtype, heads, kv_heads, dim, vdim, taps):
    """Whole sequence against the oracle, then in steps of 17, 2, 1 and the rest through a slot with stale contents: what the
    recurrence and the convolution carry from step to step is the oracle's."""
    from tgis_amd.utils.mixers import DeltaRuleMixer
    from tgis_amd.utils.state_cache import RecurrentStateCache

    W = 40
    lay = tiny.delta_layer(heads, kv_heads, dim, vdim, taps)
    cfg = tiny.make_config([lay], width=W)
    tensors = tiny.make_tensors(cfg, heads * 100 + dim)
    mixer = DeltaRuleMixer(_dict_weights(tensors, dtype), "l0.mix", 0, heads, kv_heads, dim, vdim, taps, 1e-4)
    mixer.defer = False  # a finished tensor, not split-K slabs for a residual update behind it
    dev = torch.device("cuda:0")
    h = torch.randn(45, W, generator=torch.Generator().manual_seed(dim)).to(dtype)
    want, _ = ref.channel_delta_mixer(h.double(), _f64(tensors, "l0.mix."), lay["mixer"], 1e-4)
    state = RecurrentStateCache([mixer.state_shape], W, 3, dev)
    slot = state.alloc(3)[1]
    state.state[0].fill_(7.0)  # stale: position 0 must ignore it
    state.shift[0].fill_(7.0)
    outs, at = [], 0
    for m in (17, 2, 1, 25):
        kv, pos = _kv_step(None, None, at, m, state, slot)
        outs.append(mixer.forward(h[at:at + m].to(dev), pos, kv))
        at += m
    assert rel_err(torch.cat(outs), want) <= TOL[dtype]
    assert torch.all(state.state[0][0] == 7.0) and torch.all(state.shift[0][2] == 7.0)  # other slots untouched


def test_delta_rule_keeps_a_far_write(gpu_device):
    """A key written at the start with beta = 1 and no decay is read back 300 tokens later by a matching query: the
    recurrence neither loses nor smears it, across LDS stages and steps."""
    from tgis_amd import native

    dev = torch.device("cuda:0")
    H, dk, dv, taps, n = 1, 32, 32, 2, 300
    C = 2 * dk + dv
    conv = torch.zeros(n, C)
    e0, e1 = torch.zeros(dk), torch.zeros(dk)
    e0[3], e1[7] = 1.0, 1.0
    conv[:, :dk] = e1           # queries that read nothing ...
    conv[:, dk:2 * dk] = e1     # ... and keys that overwrite their own row with zeros
    conv[0, dk:2 * dk] = e0     # the planted key
    marker = torch.arange(1, dv + 1, dtype=torch.float32)
    conv[0, 2 * dk:] = marker
    conv[n - 1, :dk] = e0       # the last query asks for it
    a = torch.full((n, dk), -60.0)          # softplus -> 0: no decay
    b = torch.full((n, 1), 60.0)            # beta = 1
    gate = torch.full((n, dv), 60.0)        # sigmoid = 1
    state = torch.zeros(2, H, native.delta_state_floats(dk, dv), device=dev)
    tail = torch.zeros(2, taps - 1, C, device=dev)
    out, at = None, 0
    for m in (100, 2, 197, 1):
        sl = slice(at, at + m)
        out = native.delta_scan(conv[sl].to(dev).contiguous(), a[sl].to(dev), b[sl].to(dev), gate[sl].to(dev), torch.zeros(H, device=dev),
                                torch.zeros(H * dk, device=dev), torch.ones(dv, device=dev), state, tail, torch.zeros(m, C, device=dev),
                                torch.tensor([1], dtype=torch.int32, device=dev), torch.tensor([0, m], dtype=torch.int32, device=dev),
                                torch.arange(at, at + m, dtype=torch.int32, device=dev), H, H, dk, dv, taps, 1e-12, 1e-12, 1.0)
        at += m
    want = marker / marker.pow(2).mean().sqrt()
    assert torch.allclose(out[-1].cpu(), want, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [dict(), dict(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=22, q_rank=18, rot_dims=4),
                                  dict(heads=8, dim=48, rot_dim=16, vdim=64, kv_rank=160, q_rank=56, scale=0.1)])
def test_latent_attention_alone(gpu_device, dtype, geom):
    """Whole and in portions: what the pages hold (normed latent, rotated shared part) serves later steps; positions far
    from zero rotate by the same angles as the oracle's."""
    from tgis_amd.utils.kv_cache import PagedKVCache
    from tgis_amd.utils.mixers import LatentAttention

    W = 56
    lay = tiny.latent_layer(**geom)
    m = lay["mixer"]
    cfg = tiny.make_config([lay], width=W)
    tensors = tiny.make_tensors(cfg, 5)
    dev = torch.device("cuda:0")
    att = LatentAttention(_dict_weights(tensors, dtype), "l0.mix", 0, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                          m["scale"], 1e-4, m["rot"]["base"], m["rot"]["dims"])
    att.defer = False
    n = 600
    h = torch.randn(n, W, generator=torch.Generator().manual_seed(4)).to(dtype)
    want, _, _ = ref.latent_attention_mixer(h.double(), torch.arange(n), _f64(tensors, "l0.mix."), m, 1e-4)
    cache = PagedKVCache(1, 1, 8, 24, dtype, dev, layer_shapes=[att.kv_shape])
    pages = cache.alloc(19)[::-1]
    outs, at = [], 0
    for step in (33, 2, 41, 1, 520, 3):
        kv, pos = _kv_step(cache, pages, at, step)
        outs.append(att.forward(h[at:at + step].to(dev), pos, kv))
        at += step
    assert rel_err(torch.cat(outs), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_biased_attention_alone_and_shared_cache(gpu_device, dtype):
    """One attention layer with GQA, unequal key / value widths, the mask, the bias, unit-RMS values and the gate, in portions;
    then a second layer that has no keys and values of its own and reads the first one's pages with its own queries."""
    from tgis_amd.utils.kv_cache import PagedKVCache
    from tgis_amd.utils.mixers import BlockBiasedAttention

    W, H, G, dk, dv = 48, 6, 2, 24, 16
    lays = [tiny.attention_layer(H, G, dk, dv, scale=0.3, chunk=20), tiny.attention_layer(H, G, dk, dv, scale=0.2, chunk=35, kv_from=0)]
    cfg = tiny.make_config(lays, width=W)
    tensors = tiny.make_tensors(cfg, 9)
    dev = torch.device("cuda:0")
    wts = _dict_weights(tensors, dtype)
    a0 = BlockBiasedAttention(wts, "l0.mix", 0, H, G, dk, dv, 0.3, 1e-4, chunk=20)
    a1 = BlockBiasedAttention(wts, "l1.mix", 1, H, G, dk, dv, 0.2, 1e-4, chunk=35, kv_source=0)
    a0.defer = a1.defer = False
    n = 77
    h = torch.randn(n, W, generator=torch.Generator().manual_seed(4)).to(dtype)
    h1 = torch.randn(n, W, generator=torch.Generator().manual_seed(5)).to(dtype)
    pos_all = torch.arange(n)
    want0, k, v = ref.attention_mixer(h.double(), pos_all, _f64(tensors, "l0.mix."), lays[0]["mixer"], 1e-4)
    want1, _, _ = ref.attention_mixer(h1.double(), pos_all, _f64(tensors, "l1.mix."), lays[1]["mixer"], 1e-4, shared=(k, v))
    cache = PagedKVCache(2, G, dk, 6, dtype, dev, layer_shapes=[(G, dk, dv), None])
    pages = cache.alloc(3)[::-1]
    o0, o1, at = [], [], 0
    for m in (33, 2, 41, 1):
        kv, pos = _kv_step(cache, pages, at, m)
        o0.append(a0.forward(h[at:at + m].to(dev), pos, kv))
        o1.append(a1.forward(h1[at:at + m].to(dev), pos, kv))
        at += m
    assert rel_err(torch.cat(o0), want0) <= TOL[dtype]
    assert rel_err(torch.cat(o1), want1) <= TOL[dtype]


# ---- the framework's own entry point and scheduler -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 16])
def test_greedy_generation_through_batches(gpu_device, std, dtype, chunk, monkeypatch):
    """from_pb -> generate_token(first) -> decode steps (captured graphs) with a second batch prefilled, concatenated and
    one request pruned on the way; prompts prefilled whole or in portions of 16.  Token ids against the oracle's greedy
    continuation, teacher-forced where bf16 may flip a near tie."""
    from tgis_amd.testing import SyntheticTokenizer, make_batch_pb

    cfg, tensors = std
    monkeypatch.setenv("TGIS_PREFILL_CHUNK", str(chunk))
    tok = SyntheticTokenizer(cfg["vocab"])
    lm = build_lm(cfg, tensors, dtype, pages=40, slots=6, tokenizer=tok)
    steps = 12
    with lm.context_manager():
        b1, errs = lm.batch_type.from_pb(make_batch_pb([37, 5, 50], steps, batch_id=0), tok, lm.dtype, lm.device, None, None, True)
        assert not errs
        prompts = {r.id: b1.all_input_ids_tensor[i, :l].tolist() for i, (r, l) in enumerate(zip(b1.requests, b1.input_lengths))}
        out = {r.id: [] for r in b1.requests}
        for t in lm.generate_token(b1, first=True)[0]:
            out[t.request_id].append(t.token_id)
        for _ in range(3):
            for t in lm.generate_token(b1)[0]:
                out[t.request_id].append(t.token_id)
        b2, _ = lm.batch_type.from_pb(make_batch_pb([20, 33], steps, batch_id=1, first_request_id=3), tok, lm.dtype, lm.device, None, None, True)
        for i, (r, l) in enumerate(zip(b2.requests, b2.input_lengths)):
            prompts[r.id] = b2.all_input_ids_tensor[i, :l].tolist()
            out[r.id] = []
        for t in lm.generate_token(b2, first=True)[0]:
            out[t.request_id].append(t.token_id)
        batch = lm.batch_type.concatenate([b1, b2])
        for _ in range(3):
            for t in lm.generate_token(batch)[0]:
                out[t.request_id].append(t.token_id)
        batch = lm.batch_type.prune(batch, [1])
        assert lm.state_cache.free_slots == 6 - 4
        for _ in range(4):
            for t in lm.generate_token(batch)[0]:
                out[t.request_id].append(t.token_id)
        batch.release()
    assert lm.kv_cache.free_pages == 40 and lm.state_cache.free_slots == 6
    for rid, ids in out.items():
        # the oracle, fed the engine's own tokens: at every step the engine's choice must be the oracle's argmax, or a
        # near tie of it under bf16
        st = ref.new_state(cfg)
        logits = ref.advance(cfg, tensors, prompts[rid], st)[-1]
        for k, t in enumerate(ids):
            best = int(logits.argmax())
            if t != best:
                gap = float(logits[best] - logits[t])
                assert dtype == torch.bfloat16 and gap < 0.05 * float(logits.std()), (rid, k, t, best, gap)
            logits = ref.advance(cfg, tensors, [t], st)[-1]


# ---- the trace runner, as a user starts it ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_a_schedule(gpu_device, tmp_path, dtype):
    """A checkpoint folder of its own shape written to disk and replayed by bin/trace_run in a child process: requests admitted
    at different steps, portions beside single tokens, a request that sits a step out, a pool of 6 pages for 3 live requests,
    slots and pages handed on to later requests."""
    from safetensors.torch import save_file

    layers = [tiny.delta_layer(heads=4, kv_heads=4, dim=32, vdim=32, conv=4, mlp=tiny.dense_mlp(48)),
              tiny.attention_layer(heads=8, kv_heads=1, dim=16, vdim=32, scale=0.25, chunk=40, mlp=None),
              tiny.latent_layer(heads=2, dim=16, rot_dim=16, vdim=32, kv_rank=32, q_rank=24, mlp=tiny.dense_mlp(96)),
              tiny.attention_layer(heads=8, kv_heads=1, dim=16, vdim=32, scale=0.2, chunk=24, kv_from=1, mlp=tiny.dense_mlp(40))]
    cfg = tiny.make_config(layers, width=64, vocab=70, eps=1e-6, residual_mult=0.4, side_dim=12, softcap=15.0)
    tensors = tiny.make_tensors(cfg, seed=11, low_rank=16)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(model_dir / "model.safetensors"))
    prompts = {"a": rand_tokens(60, 70, 1), "b": rand_tokens(33, 70, 2), "c": rand_tokens(64, 70, 3), "d": rand_tokens(40, 70, 4)}
    want = {k: ref.forward(cfg, tensors, v) for k, v in prompts.items()}
    schedule = [[("a", 31)], [("a", 2), ("b", 30)], [("a", 1), ("b", 1), ("c", 33)], [("a", 26), ("c", 1)], [("b", 2), ("c", 30)],
                [("d", 2)], [("d", 37), ("c", 0)], [("d", 1)]]
    done = {k: 0 for k in prompts}
    lines, expect = [], []
    for n, step in enumerate(schedule):
        entries, rows, end = [], [], []
        for rid, cnt in step:
            if cnt == 0:
                continue
            lo = done[rid]
            entries.append({"id": rid, "tokens": prompts[rid][lo:lo + cnt], "want": list(range(cnt))})
            rows.append(want[rid][lo:lo + cnt])
            done[rid] += cnt
            if done[rid] == len(prompts[rid]):
                end.append(rid)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        expect.append(torch.cat(rows))
    out_dir = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", "192", "--slots", "3"],
                       input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=280)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {n}" for n in range(len(schedule))]
    tol = TOL[torch.float32 if dtype == "float32" else torch.bfloat16]
    for n, e in enumerate(expect):
        got = torch.from_numpy(np.fromfile(out_dir / f"{n}.f32", dtype="<f4").reshape(e.shape).copy())
        assert rel_err(got, e) <= tol, n
