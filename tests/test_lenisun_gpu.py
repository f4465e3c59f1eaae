"""GPU: the Lenisun family on the kernels (FlashCausalLM + utils/mixers.py + csrc/residual_f32, attn_varlen, wkv, moe)
against the plain float64 restatement in oracle/lenisun_ref.py, on small seeded checkpoints of their own sizes.

float32 serving is compared tightly (it differs from the oracle by accumulation order only); bfloat16 serving against a
bound that scales with bf16 rounding.  Schedules (whole prompts, token-by-token, portions down to two tokens, mixed batches,
pages and slots that change hands) are compared with the SAME model run whole, where only rounding may differ."""
import numpy as np
import pytest
import torch

from oracle import lenisun_ref as ref
from oracle import lenisun_tiny as tiny

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-4, torch.bfloat16: 0.15}


def build_lm(cfg, tensors, dtype, pages=64, slots=4, tokenizer=None):
    from tgis_amd.inference_engine.synthetic import InferenceEngine
    from tgis_amd.models.custom_modeling.flash_lenisun_modeling import LenisunConfig
    from tgis_amd.models.flash_causal_lm import FlashCausalLM

    eng = InferenceEngine({k: v.clone() for k, v in tensors.items()}, LenisunConfig(**cfg), dtype, None, tokenizer=tokenizer)
    return FlashCausalLM("synthetic", None, "synthetic", dtype, None, engine=eng, kv_cache_pages=pages, state_slots=slots)


def rel_err(got: torch.Tensor, want: torch.Tensor, dtype=torch.float32) -> float:
    """Row errors (rms of the centred difference over the rms of the centred reference row) condensed into one number
    that is compared with TOL: their maximum — except that under bf16 rounding a router may settle a near tie the other
    way for a token or two, which changes that token's row wholesale; so up to 5 % of the rows may be off by up to ten
    times the bound, and the rest decide."""
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    e = (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).flatten()
    if dtype == torch.bfloat16 and e.numel() >= 20:
        k = max(1, int(0.95 * e.numel()))
        return max(float(e.sort().values[k - 1]), float(e.max()) / 10)
    return float(e.max())


def rand_tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.fixture(scope="module")
def std():
    return tiny.standard(seed=3)


@pytest.fixture(scope="module")
def std_ref(std):
    return ref.LenisunRef(*std)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [75, 300])
def test_whole_prompt_matches_oracle_layer_by_layer(gpu_device, std, std_ref, dtype, n):
    """75 tokens: the decode-sized GEMM path (split-K sums finished by the norm behind them); 300: the library GEMMs."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(n, cfg["vocab"], 1)
    want_trace = []
    want = std_ref.forward(toks, want_trace)
    with lm.context_manager():
        seq = lm.open_sequence()
        trace = []
        got = lm.step_sequences([(seq, toks)], None, residual_trace=trace)
    assert len(trace) == len(want_trace)
    for i, (g, w) in enumerate(zip(trace, want_trace)):
        assert rel_err(g, w, dtype) <= TOL[dtype], f"layer {i}"
    assert rel_err(got, want, dtype) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_by_token_and_portions_equal_whole(gpu_device, std, std_ref, dtype):
    """Prefill against decoding one token at a time, and portions of several sizes down to two tokens, some of them ending
    or starting on a page border (32)."""
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(101, cfg["vocab"], 2)
    want = std_ref.forward(toks)
    with lm.context_manager():
        for cuts in ([1] * 101, [2] * 50 + [1], [31, 1, 2, 30, 3, 29, 5], [32, 32, 32, 5], [63, 2, 2, 34], [7, 57, 37]):
            assert sum(cuts) == 101
            seq = lm.open_sequence()
            at, outs = 0, []
            for n in cuts:
                outs.append(lm.step_sequences([(seq, toks[at:at + n])], None))
                at += n
            got = torch.cat(outs)
            assert rel_err(got, want, dtype) <= TOL[dtype], cuts
            lm.close_sequence(seq)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_batches_reuse_pages_and_slots(gpu_device, std, std_ref, dtype):
    """Up to four live requests of unequal length, portions of some beside single tokens of others, in a pool that is too
    small to hold all requests at once: pages and slots go back and are handed out again, to other requests."""
    cfg, tensors = std
    lens = [70, 33, 95, 5, 64, 40, 1]
    prompts = [rand_tokens(n, cfg["vocab"], 10 + i) for i, n in enumerate(lens)]
    want = [std_ref.forward(p) for p in prompts]
    lm = build_lm(cfg, tensors, dtype, pages=9, slots=4)  # 9 pages = 288 tokens < sum(lens)
    rng = np.random.default_rng(0)
    got = [[] for _ in prompts]
    done = [0] * len(prompts)
    live, waiting = {}, list(range(len(prompts)))
    with lm.context_manager():
        while waiting or live:
            while waiting and len(live) < 4:
                i = waiting[0]
                pages_needed = (lens[i] + 31) // 32
                held = sum((lens[j] + 31) // 32 for j in live)
                if held + pages_needed > 9:
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
        assert rel_err(torch.cat(got[i]), want[i], dtype) <= TOL[dtype], i


def test_stale_slot_and_pages_do_not_leak(gpu_device, std, std_ref):
    """A request that takes over a slot and pages still holding another request's state and keys computes what it computes
    in a fresh pool; also its first tokens (position 0: zero state, zero shift)."""
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
    assert rel_err(got, std_ref.forward(b)) <= TOL[torch.float32]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_decoding(gpu_device, std, std_ref, dtype):
    cfg, tensors = std
    lm = build_lm(cfg, tensors, dtype)
    toks = rand_tokens(40 + 200, cfg["vocab"], 8)
    want = std_ref.forward(toks)
    with lm.context_manager():
        s = lm.open_sequence()
        outs = [lm.step_sequences([(s, toks[:40])], None)]
        for t in toks[40:]:
            outs.append(lm.step_sequences([(s, [t])], None))
    assert rel_err(torch.cat(outs), want, dtype) <= TOL[dtype]


# ---- attention: keys that must or must not be seen -------------------------------------------------------------------------
def _planted_attention(dtype, key_pos, n_ctx, q_chunks, H=4, G=2, dk=16, dv=8):
    """q of the LAST token and k of token `key_pos` are made parallel and large, v of that token is a marker: the output of
    the last token is the marker iff the kernel sees exactly that key.  Returns (output of the last token, marker)."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(key_pos * 1000 + n_ctx)
    qkv = torch.randn(n_ctx, (H + G) * dk + G * dv, generator=g) * 0.1
    direction = torch.nn.functional.normalize(torch.randn(dk, generator=g), dim=0)
    for h in range(H):
        qkv[n_ctx - 1, h * dk:(h + 1) * dk] = direction * 3
    for gg in range(G):
        qkv[key_pos, (H + gg) * dk:(H + gg + 1) * dk] = direction * 3
    marker = torch.arange(1, G * dv + 1, dtype=torch.float32) * 0.25
    qkv[key_pos, (H + G) * dk:] = marker
    cache = PagedKVCache(1, G, dk, 40, dtype, dev, layer_shapes=[(G, dk, dv)])
    pages = cache.alloc((n_ctx + PAGE - 1) // PAGE)
    rng = np.random.default_rng(1)
    rng.shuffle(pages)  # pages of a sequence are scattered over the pool
    bt = torch.tensor([pages], dtype=torch.int32, device=dev)
    ones = torch.ones(dk, dtype=torch.float32, device=dev)
    out_last, at = None, 0
    for n in q_chunks:
        pos = torch.arange(at, at + n, dtype=torch.int32)
        slots = (torch.tensor(pages, dtype=torch.int64)[pos.long() // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
        x = qkv[at:at + n].to(dtype).to(dev).contiguous()
        # eps tiny and unit gains: the norm only rescales q and k to rms 1 -> |q| = |k| = sqrt(dk); scale 4 makes the
        # planted score 4 dk against |other| <~ 4 dk * cos(random)
        native.qk_norm_kv_write(x, pos.to(dev), slots, ones, ones, 1e-12, 0.0, 0, None, None, cache.k_pool(0), cache.v_pool(0), H, G, dk, dv)
        ctx = torch.tensor([at + n], dtype=torch.int32, device=dev)
        cu = torch.tensor([0, n], dtype=torch.int32, device=dev)
        o = native.attn_varlen(x, cache.k_pool(0), cache.v_pool(0), bt, ctx, cu, H, G, dk, dv, 4.0, max_q_len=n)
        out_last = o[-1]
        at += n
    torch.cuda.synchronize()
    want = marker.view(G, dv).repeat_interleave(H // G, 0).reshape(-1)
    return out_last.float().cpu(), want


# (H, G, dk, dv): the general kernel (odd widths), and the matrix-core kernel's shapes under bf16
GEOMETRIES = [(4, 2, 16, 8), (4, 2, 32, 32), (8, 2, 64, 32), (4, 4, 128, 64), (3, 1, 48, 96)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", GEOMETRIES)
@pytest.mark.parametrize("key_pos", [0, 1, 31, 32, 33, 63, 64, 255, 256, 500, 698])
def test_attention_finds_one_key_among_hundreds(gpu_device, dtype, key_pos, geom):
    """Far keys, keys on both sides of page borders, the first keys: in a prompt run whole, in a prompt cut into portions
    (one of two tokens), and with the last token decoded alone."""
    n = 700
    for chunks in ([n], [300, 2, 397, 1], [n - 1, 1]):
        got, want = _planted_attention(dtype, key_pos, n, chunks, *geom)
        assert torch.allclose(got, want, atol=0.02 if dtype == torch.bfloat16 else 1e-3, rtol=0.01), (chunks, got[:4], want[:4])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_is_causal_at_every_offset(gpu_device, dtype):
    """The planted key sits one past the query: it must not be seen (in a portion, the tokens behind a query are in the
    cache already when the kernel runs)."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    dev = torch.device("cuda:0")
    n = 70
    for qpos, (H, G, dk, dv) in [(p, g) for p in (0, 30, 31, 32, 63, 64, 68) for g in ((2, 1, 8, 8), (4, 2, 32, 32), (2, 2, 64, 64))]:
        g = torch.Generator().manual_seed(qpos)
        qkv = torch.randn(n, (H + G) * dk + G * dv, generator=g) * 0.1
        d = torch.nn.functional.normalize(torch.randn(dk, generator=g), dim=0)
        qkv[qpos, :H * dk] = d.repeat(H) * 3
        qkv[qpos + 1, H * dk:(H + G) * dk] = d.repeat(G) * 3
        qkv[qpos + 1, (H + G) * dk:] = 100.0
        cache = PagedKVCache(1, G, dk, 8, dtype, dev, layer_shapes=[(G, dk, dv)])
        pages = cache.alloc(3)
        pos = torch.arange(n, dtype=torch.int32)
        slots = (torch.tensor(pages)[pos.long() // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
        x = qkv.to(dtype).to(dev)
        ones = torch.ones(dk, dtype=torch.float32, device=dev)
        native.qk_norm_kv_write(x, pos.to(dev), slots, ones, ones, 1e-12, 0.0, 0, None, None, cache.k_pool(0), cache.v_pool(0), H, G, dk, dv)
        o = native.attn_varlen(x, cache.k_pool(0), cache.v_pool(0), torch.tensor([pages], dtype=torch.int32, device=dev),
                               torch.tensor([n], dtype=torch.int32, device=dev), torch.tensor([0, n], dtype=torch.int32, device=dev),
                               H, G, dk, dv, 4.0, max_q_len=n)
        assert float(o[qpos].float().abs().max()) < 1.0, qpos


def _plain_attention(q, k, v, scale, H, G):
    """q [n_q, H, dk] are the last n_q tokens of a sequence whose keys / values are k [n, G, dk], v [n, G, dv]."""
    n_q, n = q.shape[0], k.shape[0]
    out = torch.zeros(n_q, H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale
        vis = torch.arange(n)[None, :] <= (torch.arange(n_q) + n - n_q)[:, None]
        out[:, h] = torch.softmax(s.masked_fill(~vis, float("-inf")), -1) @ v[:, h // (H // G)]
    return out.reshape(n_q, -1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", GEOMETRIES + [(16, 1, 64, 128), (32, 2, 32, 32), (2, 2, 256, 256), (40, 1, 16, 8), (34, 2, 32, 32)])
def test_attention_ragged_batch_against_plain_softmax(gpu_device, dtype, geom):
    """A step of unequal sequences — whole prompts, a portion that continues a long context, single decoded tokens, one of
    them behind 3000 cached keys — through both kernels (where the matrix-core one applies) against plain softmax."""
    from tgis_amd import native
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache

    H, G, dk, dv = geom
    dev = torch.device("cuda:0")
    cached = [0, 200, 3000, 31, 0, 64]
    new = [70, 45, 1, 1, 1, 33]
    g = torch.Generator().manual_seed(H * 1000 + dk)
    cache = PagedKVCache(1, G, dk, 130, dtype, dev, layer_shapes=[(G, dk, dv)])
    ones = torch.ones(dk, dtype=torch.float32, device=dev)
    full, pages = [], []
    for c, n in zip(cached, new):
        x = (torch.randn(c + n, (H + G) * dk + G * dv, generator=g) * 1.5).to(dtype)
        pg = cache.alloc((c + n + PAGE - 1) // PAGE)
        pos = torch.arange(c, dtype=torch.int32)
        if c:  # what earlier steps left in the cache
            slots = (torch.tensor(pg)[pos.long() // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev)
            native.qk_norm_kv_write(x[:c].to(dev).contiguous(), pos.to(dev), slots, ones, ones, 1e-6, 0.0, 0, None, None,
                                    cache.k_pool(0), cache.v_pool(0), H, G, dk, dv)
        full.append(x)
        pages.append(pg)
    step = torch.cat([x[c:] for x, c in zip(full, cached)]).to(dev).contiguous()
    pos = torch.cat([torch.arange(c, c + n, dtype=torch.int32) for c, n in zip(cached, new)])
    slots = torch.cat([(torch.tensor(pg)[torch.arange(c, c + n) // PAGE] * PAGE + torch.arange(c, c + n) % PAGE)
                       for pg, c, n in zip(pages, cached, new)]).to(torch.int32).to(dev)
    native.qk_norm_kv_write(step, pos.to(dev), slots, ones, ones, 1e-6, 0.0, 0, None, None, cache.k_pool(0), cache.v_pool(0), H, G, dk, dv)
    width = max(len(p) for p in pages)
    bt = torch.zeros(len(pages), width, dtype=torch.int32)
    for i, p in enumerate(pages):
        bt[i, :len(p)] = torch.tensor(p)
    ctx = torch.tensor([c + n for c, n in zip(cached, new)], dtype=torch.int32, device=dev)
    cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32, device=dev)
    want = []
    for x, c, n in zip(full, cached, new):
        xd = x.double()
        q = ref.rms_unit(xd[c:, :H * dk].view(n, H, dk), 1e-6).to(dtype).double()
        k = ref.rms_unit(xd[:, H * dk:(H + G) * dk].view(c + n, G, dk), 1e-6).to(dtype).double()
        want.append(_plain_attention(q, k, xd[:, (H + G) * dk:].view(c + n, G, dv), 0.5, H, G))
    want = torch.cat(want)
    impls = [1] + ([2] if dtype == torch.bfloat16 and dk % 16 == 0 and dv % 32 == 0 else [])
    for impl in impls:
        for max_q in (max(new),):
            got = native.attn_varlen(step, cache.k_pool(0), cache.v_pool(0), bt.to(dev), ctx, cu, H, G, dk, dv, 0.5,
                                     max_q_len=max_q, max_ctx=3001, impl=impl)
            err = (got.double().cpu() - want).abs().max() / want.abs().max()
            assert float(err) <= (2e-5 if dtype == torch.float32 else 2e-2), (impl, float(err))
    if 2 in impls:  # decode-only steps take the key-split form of the matrix-core kernel
        sel = [i for i, n in enumerate(new) if n == 1]
        rows = [int(cu[i]) for i in sel]
        got = native.attn_varlen(step[rows].contiguous(), cache.k_pool(0), cache.v_pool(0), bt[sel].contiguous().to(dev), ctx[sel].contiguous(),
                                 torch.arange(len(sel) + 1, dtype=torch.int32, device=dev), H, G, dk, dv, 0.5, max_q_len=1,
                                 max_ctx=3001, impl=2)
        err = (got.double().cpu() - want[rows]).abs().max() / want.abs().max()
        assert float(err) <= 2e-2, float(err)


# ---- mechanisms alone ----------------------------------------------------------------------------------------------------
def _dict_weights(tensors, dtype):
    from tgis_amd.utils.dist import FakeGroup
    from tgis_amd.utils.weights import DictWeights

    return DictWeights(tensors, device=torch.device("cuda:0"), dtype=dtype, process_group=FakeGroup(0, 1))


def _f64(tensors, prefix):
    return {k[len(prefix):]: v.double() for k, v in tensors.items() if k.startswith(prefix)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sandwich_norm(gpu_device, dtype):
    from tgis_amd import native

    g = torch.Generator().manual_seed(0)
    for E in (8, 80, 257, 1024):
        x = torch.randn(5, E, generator=g)
        delta = (torch.randn(5, E, generator=g) * 3).to(dtype)
        wb, w = torch.randn(E, generator=g) * 0.2, torch.randn(E, generator=g) * 0.2
        xd = x.cuda()
        y = native.sandwich_norm_f32(xd, delta.cuda(), wb.cuda(), w.cuda(), 1e-3, dtype)
        want_x = x.double() + ref.norm_one_plus(delta.double(), wb.double(), 1e-3)
        want_y = ref.norm_one_plus(want_x, w.double(), 1e-3)
        assert torch.allclose(xd.cpu().double(), want_x, atol=1e-5, rtol=1e-5)
        assert torch.allclose(y.cpu().double(), want_y, atol=1e-5 if dtype == torch.float32 else 2e-2, rtol=1e-5 if dtype == torch.float32 else 1e-2)


def test_sandwich_norm_takes_split_k_slabs(gpu_device):
    """The norm behind a decode-sized projection sums the projection's split-K slabs itself."""
    from tgis_amd import native
    from tgis_amd.utils.layers import FastLinear

    g = torch.Generator().manual_seed(3)
    for M, K, N in ((1, 512, 256), (33, 2048, 512), (70, 4096, 1024)):
        w = (torch.randn(N, K, generator=g) * K ** -0.5).to(torch.bfloat16).cuda()
        a = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
        x = torch.randn(M, N, generator=g).cuda()
        wb, wn = (torch.randn(N, generator=g) * 0.2).cuda(), (torch.randn(N, generator=g) * 0.2).cuda()
        part = FastLinear(w, None)(a, partial=True)
        assert isinstance(part, native.Partial)
        x_ref = x.double().cpu() + ref.norm_one_plus(a.double().cpu() @ w.double().cpu().T, wb.double().cpu(), 1e-5)
        y = native.sandwich_norm_f32(x, part, wb, wn, 1e-5, torch.float32)
        assert torch.allclose(x.double().cpu(), x_ref, atol=2e-3, rtol=1e-3)
        assert torch.allclose(y.double().cpu(), ref.norm_one_plus(x_ref, wn.double().cpu(), 1e-5), atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["clamped", "silu"])
@pytest.mark.parametrize("T", [37, 300])
def test_gated_unit(gpu_device, dtype, kind, T):
    """37 rows: the activation in the epilogue of the weight-streaming GEMM (two-byte dtypes); 300: library GEMM + launch."""
    from tgis_amd.utils.mixers import GatedUnit

    cfg = tiny.make_config([tiny.wkv_layer(mlp=tiny.dense_mlp(72, 0.8))], width=48)
    tensors = tiny.make_tensors(cfg, 1)
    unit = GatedUnit(_dict_weights(tensors, dtype), "l0.mlp", mode=kind, alpha=1.702, limit=0.8)
    h = torch.randn(T, 48, generator=torch.Generator().manual_seed(2)).to(dtype)
    got = unit(h.cuda())
    p = _f64(tensors, "l0.mlp.")
    if kind == "clamped":
        want = ref.dense_ff(h.double(), p, {"limit": 0.8})
    else:
        want = ref.expert_ff(h.double(), p, "")
    assert rel_err(got, want, dtype) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,shared,T,W,ff", [(6, 2, 24, 70, 64, 32), (16, 1, 8, 3, 64, 32), (3, 3, None, 33, 64, 32),
                                                       (40, 4, 16, 300, 64, 32), (5, 2, 12, 41, 36, 20), (4, 1, 7, 9, 30, 13)])
def test_routed_experts(gpu_device, dtype, experts, top, shared, T, W, ff):
    """Also widths that are not multiples of 8 (padded once at load) and more tokens than a tile."""
    from tgis_amd.utils.mixers import RoutedExperts

    f = tiny.moe_mlp(ff, experts, top, shared)
    cfg = tiny.make_config([tiny.wkv_layer(mlp=f)], width=W)
    tensors = tiny.make_tensors(cfg, experts)
    moe = RoutedExperts(_dict_weights(tensors, dtype), "l0.mlp", experts, top, bool(shared))
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(T)).to(dtype)
    got = moe(h.cuda())
    want = ref.moe_ff(h.double(), _f64(tensors, "l0.mlp."), f)
    assert rel_err(got, want, dtype) <= TOL[dtype]


def test_router_picks_the_largest_scores(gpu_device):
    from tgis_amd import native

    g = torch.Generator().manual_seed(0)
    h, w = torch.randn(50, 40, generator=g), torch.randn(11, 40, generator=g)
    idx, weight, sg = native.moe_route(h.cuda(), w.cuda(), torch.randn(40, generator=g).cuda(), 4)
    s = torch.sigmoid(h.double() @ w.double().T)
    wv, wi = torch.topk(s, 4, dim=-1)
    assert torch.equal(idx.cpu().long(), wi)
    assert torch.allclose(weight.cpu().double(), wv, atol=1e-6)
    assert sg.shape == (50,)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim", [(3, 16), (2, 48), (1, 64), (2, 128), (4, 20)])
def test_wkv_mixer_and_its_state(gpu_device, dtype, heads, dim):
    """Whole sequence against the oracle, then the same sequence in two steps through a slot: the state that the first
    step leaves is the oracle's, and so is what the second step computes from it."""
    from tgis_amd.models.custom_modeling.flash_llama_modeling import KVArgs
    from tgis_amd.utils.mixers import WkvMixer
    from tgis_amd.utils.state_cache import RecurrentStateCache

    W = 40
    cfg = tiny.make_config([tiny.wkv_layer(heads, dim)], width=W)
    tensors = tiny.make_tensors(cfg, heads * 100 + dim)
    mixer = WkvMixer(_dict_weights(tensors, dtype), "l0.mix", 0, heads, dim, 1e-4)
    mixer.defer = False  # a finished tensor, not split-K slabs for a norm behind it
    dev = torch.device("cuda:0")
    h = torch.randn(45, W, generator=torch.Generator().manual_seed(dim))
    p = _f64(tensors, "l0.mix.")
    want, want_h, want_S = ref.wkv_mixer(h.double(), p, cfg["layers"][0]["mixer"], 1e-4)
    state = RecurrentStateCache([(heads, dim)], W, 3, dev)
    slot = state.alloc(3)[1]
    state.state[0].fill_(7.0)  # stale: position 0 must ignore it
    state.shift[0].fill_(7.0)

    def run(lo, hi):
        kv = KVArgs(cache=None, block_tables=None, ctx_lens=None, slots=None, max_q_len=hi - lo, max_ctx=hi, state=state,
                    state_slots=torch.tensor([slot], dtype=torch.int32, device=dev),
                    cu_seqlens_q=torch.tensor([0, hi - lo], dtype=torch.int32, device=dev))
        return mixer.forward(h[lo:hi].to(dev), torch.arange(lo, hi, dtype=torch.int32, device=dev), kv, dtype)

    got = torch.cat([run(0, 17), run(17, 19), run(19, 45)])
    assert rel_err(got, want, dtype) <= TOL[dtype]
    assert torch.allclose(state.state[0][slot].cpu().double(), want_S, atol=TOL[dtype] * float(want_S.abs().max()))
    assert torch.allclose(state.shift[0][slot].cpu().double(), want_h, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_mixer_alone(gpu_device, dtype):
    """One attention layer with GQA, unequal key / value widths, query gain and blending, whole and in portions."""
    from tgis_amd.models.custom_modeling.flash_llama_modeling import KVArgs
    from tgis_amd.utils.kv_cache import PAGE, PagedKVCache
    from tgis_amd.utils.mixers import NormedQKAttention

    W, H, G, dk, dv = 48, 6, 2, 24, 16
    lay = tiny.attention_layer(H, G, dk, dv, scale=0.3, q_temp=(0.7, 4), v_mix=True)
    cfg = tiny.make_config([lay], width=W)
    tensors = tiny.make_tensors(cfg, 9)
    dev = torch.device("cuda:0")
    att = NormedQKAttention(_dict_weights(tensors, dtype), "l0.mix", 0, H, G, dk, dv, 0.3, 1e-4, 0.7, 4, blend=True)
    att.defer = False  # a finished tensor, not split-K slabs for a norm behind it
    n = 77
    g = torch.Generator().manual_seed(4)
    h = torch.randn(n, W, generator=g).to(dtype)
    v_other = torch.randn(n, G * dv, generator=g).to(dtype)
    want, _, _, _ = ref.attention_mixer(h.double(), torch.arange(n), _f64(tensors, "l0.mix."), lay["mixer"], 1e-4,
                                        v_first=v_other.double().view(n, G, dv), blend=True)
    cache = PagedKVCache(1, G, dk, 6, dtype, dev, layer_shapes=[(G, dk, dv)])
    pages = cache.alloc(3)[::-1]
    outs, at = [], 0
    for m in (33, 2, 41, 1):
        pos = torch.arange(at, at + m, dtype=torch.int32)
        kv = KVArgs(cache=cache, block_tables=torch.tensor([pages], dtype=torch.int32, device=dev),
                    ctx_lens=torch.tensor([at + m], dtype=torch.int32, device=dev),
                    slots=(torch.tensor(pages)[pos.long() // PAGE] * PAGE + pos % PAGE).to(torch.int32).to(dev), max_q_len=m,
                    max_ctx=at + m, cu_seqlens_q=torch.tensor([0, m], dtype=torch.int32, device=dev))
        out, _ = att.forward(h[at:at + m].to(dev), pos.to(dev), kv, v_other[at:at + m].to(dev))
        outs.append(out)
        at += m
    assert rel_err(torch.cat(outs), want, dtype) <= TOL[dtype]


# ---- the framework's own entry point and scheduler -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk", [0, 16])
def test_greedy_generation_through_batches(gpu_device, std, std_ref, dtype, chunk, monkeypatch):
    """from_pb -> generate_token(first) -> decode steps (captured graphs) with a second batch prefilled, concatenated and
    one request pruned on the way; prompts prefilled whole or in portions of 16.  Token ids against the oracle's greedy
    continuation, teacher-forced where bf16 may flip a near tie."""
    from tgis_amd.testing import SyntheticTokenizer, make_batch_pb

    cfg, tensors = std
    monkeypatch.setenv("TGIS_PREFILL_CHUNK", str(chunk))
    tok = SyntheticTokenizer(cfg["vocab"])
    lm = build_lm(cfg, tensors, dtype, pages=40, slots=6, tokenizer=tok)
    assert lm.prefill_chunk == chunk
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
        st = std_ref.new_state()
        logits = std_ref.advance(prompts[rid], st)[-1]
        for k, t in enumerate(ids):
            best = int(logits.argmax())
            if t != best:
                gap = float(logits[best] - logits[t])
                assert dtype == torch.bfloat16 and gap < 0.05 * float(logits.std()), (rid, k, t, best, gap)
            logits = std_ref.advance([t], st)[-1]


# ---- the trace runner, as a user starts it ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_a_schedule(gpu_device, tmp_path, dtype):
    """A checkpoint folder of its own shape (recurrent layer first, MQA with 40 query heads, an attention layer without a
    feed-forward, no blending, top-3 of 5 experts without a shared one) written to disk and replayed by bin/trace_run in a
    child process: requests admitted at different steps, portions beside single tokens, a request that sits a step out,
    a pool of 6 pages for 3 live requests, slots and pages handed on to later requests."""
    import json
    import os
    import subprocess
    import sys

    from safetensors.torch import save_file

    layers = [
        tiny.wkv_layer(heads=4, dim=32, mlp=tiny.moe_mlp(16, 5, 3, None)),
        tiny.attention_layer(heads=40, kv_heads=1, dim=16, vdim=32, scale=0.25, q_temp=(0.3, 5), v_mix=False, mlp=None),
        tiny.attention_layer(heads=4, kv_heads=4, dim=32, vdim=32, scale=0.2, q_temp=None, v_mix=False, mlp=tiny.dense_mlp(96, 3.0)),
    ]
    cfg = tiny.make_config(layers, width=64, vocab=70, eps=1e-6, embed_scale=2.0)
    tensors = tiny.make_tensors(cfg, seed=11, decay_rank=12)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(model_dir / "model.safetensors"))
    oracle = ref.LenisunRef(cfg, tensors)
    prompts = {"a": rand_tokens(60, 70, 1), "b": rand_tokens(33, 70, 2), "c": rand_tokens(64, 70, 3), "d": rand_tokens(40, 70, 4)}
    want = {k: oracle.forward(v) for k, v in prompts.items()}
    # (request, tokens in this step); every token's logits are asked for
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
        assert rel_err(got, e, torch.float32 if dtype == "float32" else torch.bfloat16) <= tol, n
