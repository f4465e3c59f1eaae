"""CPU: what the Lenisun family needs and a GPU does not — the oracle's own consistency (whole sequence == token by token
== portions through its explicit state), the config reader, model dispatch by config.json, the recurrent state slots, the
per-layer KV pool bookkeeping, and the trace runner's command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

from oracle import lenisun_ref as ref
from oracle import lenisun_tiny as tiny

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rand_tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def test_oracle_portions_equal_whole():
    """The oracle's state (keys, values as cached, recurrent matrix, last mixer input) carries everything: any cut of a
    sequence gives the logits of the whole, to float64 rounding."""
    cfg, tensors = tiny.standard(seed=1)
    model = ref.LenisunRef(cfg, tensors)
    toks = rand_tokens(41, cfg["vocab"], 0)
    whole = model.forward(toks)
    for cuts in ([1] * 41, [2] * 20 + [1], [17, 1, 23], [40, 1]):
        st, outs, at = model.new_state(), [], 0
        for n in cuts:
            outs.append(model.advance(toks[at:at + n], st))
            at += n
        assert torch.allclose(torch.cat(outs), whole, atol=1e-9, rtol=1e-9), cuts


def test_oracle_mechanisms_against_definitions():
    """Hand-checkable instances of each equation."""
    z = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(ref.rms_unit(z, 0.0), z / (12.5 ** 0.5))
    assert torch.allclose(ref.norm_one_plus(z, torch.tensor([1.0, -1.0], dtype=torch.float64), 0.0), torch.tensor([[2 * 3 / 12.5 ** 0.5, 0.0]], dtype=torch.float64))
    # query gain: 1 + coef * ln(floor((p + 1) / every) + 1)
    g = ref.query_gain(torch.tensor([0, 6, 7, 15, 16]), 0.5, 8)
    want = 1 + 0.5 * torch.log(torch.tensor([1.0, 1.0, 2.0, 3.0, 3.0], dtype=torch.float64))
    assert torch.allclose(g, want)
    # clamped unit: gate above the limit saturates, up is clamped on both sides
    p = {"gate": torch.tensor([[10.0]], dtype=torch.float64), "up": torch.tensor([[-10.0]], dtype=torch.float64),
         "down": torch.tensor([[1.0]], dtype=torch.float64)}
    y = ref.dense_ff(torch.tensor([[1.0]], dtype=torch.float64), p, {"limit": 2.0})
    assert torch.allclose(y, torch.tensor([[2.0 * torch.sigmoid(torch.tensor(1.702 * 2.0, dtype=torch.float64)) * (-2.0 + 1.0)]]))
    # recurrence with one head of width 1: o_t = r_t (S + u k_t v_t), S <- w_t S + k_t v_t
    m = {"heads": 1, "dim": 1}
    one = lambda v: torch.tensor([[v]], dtype=torch.float64)
    pw = {f"mu.{s}": torch.zeros(1, dtype=torch.float64) for s in "rkvgw"}
    pw.update({"r": one(1.0), "k": one(2.0), "v": one(3.0), "g": one(1.0), "w1": one(0.0), "w2": one(0.0),
               "w0": torch.tensor([0.0], dtype=torch.float64), "u": one(0.5), "norm": torch.ones(1, dtype=torch.float64), "o": one(1.0)})
    h = torch.tensor([[1.0], [1.0]], dtype=torch.float64)
    _, _, S = ref.wkv_mixer(h, pw, m, 0.0)
    decay = torch.exp(-torch.exp(torch.tensor(0.0, dtype=torch.float64)))
    assert torch.allclose(S, (decay * 6.0 + 6.0).reshape(1, 1, 1))


def test_moe_weight_scales_the_expert_input():
    """The routing weight goes INTO the expert (a nonlinear unit), not onto its output."""
    f = tiny.moe_mlp(ff=8, experts=3, top=1, shared_ff=None)
    cfg = tiny.make_config([tiny.wkv_layer(mlp=f)], width=8)
    t = {k[len("l0.mlp."):]: v.double() for k, v in tiny.make_tensors(cfg, 0).items() if k.startswith("l0.mlp.")}
    h = torch.randn(4, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    s = torch.sigmoid(h @ t["router"].T)
    w, idx = s.max(-1)
    want = torch.stack([ref.expert_ff((w[i] * h[i])[None], t, f"e{int(idx[i])}.")[0] for i in range(4)])
    assert torch.allclose(ref.moe_ff(h, t, f), want)
    outside = torch.stack([w[i] * ref.expert_ff(h[i][None], t, f"e{int(idx[i])}.")[0] for i in range(4)])
    assert not torch.allclose(want, outside)


def test_config_reader_and_dispatch(tmp_path):
    from tgis_amd.models import config_model_type
    from tgis_amd.models.custom_modeling.flash_lenisun_modeling import LenisunConfig

    cfg, _ = tiny.standard()
    c = LenisunConfig(**cfg)
    assert (c.width, c.vocab, c.eps, c.embedding_scale) == (80, 120, 1e-4, 1.3)
    assert c.hidden_size == 80 and c.vocab_size == 120 and c.num_hidden_layers == 5 and c.model_type == "lenisun"
    assert config_model_type(cfg) == "lenisun" and config_model_type({"model_type": "llama"}) == "llama"
    with pytest.raises(ValueError):
        LenisunConfig(**{**cfg, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(ValueError):
        LenisunConfig(**{**cfg, "layers": [{"type": "wkv", "mixer": {"heads": 1, "dim": 8}, "mlp": {"kind": "gru"}}]})
    # the engine's config loader takes the family's own reader for a config.json without a model_type
    from tgis_amd.inference_engine.engine import BaseInferenceEngine

    (tmp_path / "config.json").write_text(json.dumps(cfg))
    loaded = BaseInferenceEngine._load_config(str(tmp_path))
    assert isinstance(loaded, LenisunConfig) and loaded.layers == cfg["layers"]
    assert BaseInferenceEngine._load_tokenizer(str(tmp_path)) is None  # ids-only checkpoint
    # no GPU here: the flash path refuses instead of falling back
    if not torch.cuda.is_available():
        from tgis_amd.models import get_model

        with pytest.raises(NotImplementedError):
            get_model(str(tmp_path), None, "tgis_native", "bfloat16", None, None)


def test_recurrent_state_slots():
    from tgis_amd.utils.state_cache import OutOfSlots, RecurrentStateCache

    st = RecurrentStateCache([None, (2, 4), None, (3, 8)], width=16, num_slots=3, device="cpu")
    assert st.state[0] is None and st.state[1].shape == (4, 2, 4, 4) and st.state[3].shape == (4, 3, 8, 8)
    assert st.shift[1].shape == (4, 16) and st.null_slot == 3
    assert st.bytes_per_slot() == 4 * ((2 * 16 + 16) + (3 * 64 + 16))
    a = st.alloc(2)
    assert a == [0, 1] and st.free_slots == 1
    with pytest.raises(OutOfSlots):
        st.alloc(2)
    assert st.free_slots == 1  # all or nothing
    st.free([0])
    assert st.alloc(2) == [0, 2]  # lowest ids first, freed ones again


def test_kv_pool_with_layer_shapes():
    from tgis_amd.utils.kv_cache import PAGE, OutOfPages, PagedKVCache

    kv = PagedKVCache(3, 2, 8, 5, torch.float32, "cpu", layer_shapes=[(2, 8, 4), None, (1, 16, 16)])
    assert kv.k_pool(0).shape == (6, 2, PAGE * 8) and kv.v_pool(0).shape == (6, 2, 4 * PAGE)
    assert kv.k_pool(1) is None and kv.v_pool(2).shape == (6, 1, 16 * PAGE)
    assert kv.bytes_per_token() == 4 * (2 * 12 + 32) and kv.null_page == 5
    p = kv.alloc(5)
    with pytest.raises(OutOfPages):
        kv.alloc(1)
    kv.free(p[1:3])
    assert kv.alloc(2) == sorted(p[1:3])


def test_trace_runner_command_line():
    """The runner's help names its arguments; a model folder it cannot serve without a GPU ends with an error, not a hang."""
    exe = os.path.join(ROOT, "bin", "trace_run")
    assert os.access(exe, os.X_OK)
    out = subprocess.run([sys.executable, exe, "--help"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0
    for flag in ("--model", "--dtype", "--out", "--max-tokens"):
        assert flag in out.stdout
    bad = subprocess.run([sys.executable, exe, "--model", "/nonexistent", "--dtype", "float16", "--out", "/tmp/x", "--max-tokens", "64"],
                         capture_output=True, text=True, timeout=120)
    assert bad.returncode == 2 and "invalid choice" in bad.stderr


def test_family_build_units_exist():
    from tgis_amd import buildlib

    for family, units in buildlib.FAMILY_UNITS.items():
        for u in units:
            assert os.path.exists(os.path.join(buildlib.CSRC, u + ".hip")), (family, u)
    assert buildlib.library_path().endswith("libtgis_hip.so")
    assert buildlib.library_path("lenisun").endswith("libtgis_hip.lenisun.so")
