"""CPU: what the Senadra family needs and a GPU does not — the oracle's own consistency (whole sequence == token by token ==
portions through its explicit state), hand-checkable instances of its equations, the config reader, model dispatch by
config.json, the state slots with per-mixer shapes, and the family's build units."""
import json
import math
import os

import pytest
import torch

from oracle import senadra_ref as ref
from oracle import senadra_tiny as tiny

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
D = torch.float64


def rand_tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def test_oracle_portions_equal_whole():
    """The oracle's state (keys and unit-RMS values, latents and rotated parts, the delta rule's matrix and convolution tails)
    carries everything: any cut of a sequence gives the logits of the whole, to float64 rounding."""
    cfg = tiny.make_config(tiny.standard_layers())
    tensors = tiny.make_tensors(cfg, seed=1)
    toks = rand_tokens(61, cfg["vocab"], 0)
    whole = ref.forward(cfg, tensors, toks)
    for cuts in ([1] * 61, [2] * 30 + [1], [17, 1, 43], [47, 2, 12], [60, 1]):
        st, outs, at = ref.new_state(cfg), [], 0
        for n in cuts:
            outs.append(ref.advance(cfg, tensors, toks[at:at + n], st))
            at += n
        assert torch.allclose(torch.cat(outs), whole, atol=1e-9, rtol=1e-9), cuts


def test_oracle_mechanisms_against_definitions():
    z = torch.tensor([[3.0, 4.0]], dtype=D)
    assert torch.allclose(ref.rms_unit(z, 0.0), z / (12.5 ** 0.5))
    # xIELU: both branches meet at zero with slope 1/2; quadratic growth on the right, bounded curvature on the left
    pq = torch.tensor([0.0, 0.0], dtype=D)
    sp = math.log(2.0)
    assert torch.allclose(ref.xielu(torch.tensor([2.0, 0.0, -1.0], dtype=D), pq),
                          torch.tensor([sp * 4 + 1.0, 0.0, (0.5 + sp) * (math.exp(-1.0) - 1 + 1.0) - 0.5], dtype=D))
    # rotation of pairs: (1, 0) at position p turns to (cos a, sin a) with a = p base^(-2i / dims); channels past dims pass
    x = torch.tensor([[1.0, 0.0, 1.0, 0.0, 5.0, 6.0]], dtype=D)
    r = ref.rotate_pairs(x, torch.tensor([3]), 100.0, 4)
    assert torch.allclose(r, torch.tensor([[math.cos(3.0), math.sin(3.0), math.cos(0.3), math.sin(0.3), 5.0, 6.0]], dtype=D))
    # short convolution: the last column of the weight multiplies the current token; zeros before the start
    y, tail = ref.short_conv(torch.tensor([[1.0], [2.0], [3.0]], dtype=D), torch.tensor([[10.0, 1.0]], dtype=D), torch.zeros(1, 1, dtype=D))
    assert torch.allclose(y, torch.tensor([[1.0], [12.0], [23.0]], dtype=D)) and torch.allclose(tail, torch.tensor([[3.0]], dtype=D))
    # delta rule, one head of width 1: S <- g S; u = beta (v - S k); S <- S + k u; o = S q
    one = lambda v: torch.tensor([[[v]]], dtype=D)
    o, S = ref.delta_recurrence(torch.cat([one(1.0), one(1.0)]), torch.cat([one(2.0), one(1.0)]), torch.cat([one(3.0), one(5.0)]),
                                torch.tensor([[1.0], [0.5]], dtype=D), torch.cat([one(0.5), one(0.5)]), torch.zeros(1, 1, 1, dtype=D))
    # t0: S = 0; u = 3; S = 6; o = 6.   t1: S = 3; u = 0.5 (5 - 3) = 1; S = 4; o = 4
    assert torch.allclose(o.flatten(), torch.tensor([6.0, 4.0], dtype=D)) and float(S) == 4.0


def test_block_mask_and_distance_bias_in_the_oracle():
    """With a huge bias slope the nearest visible key wins; a block border hides everything before it."""
    W, H, dk, dv = 8, 1, 4, 4
    p = {"q": torch.zeros(H * dk, W, dtype=D), "k": torch.zeros(dk, W, dtype=D), "v": torch.eye(dv, W, dtype=D),
         "g": torch.zeros(dv, W, dtype=D), "o": torch.eye(W, dv, dtype=D), "r1": torch.tensor([50.0], dtype=D), "r2": torch.tensor([1.0], dtype=D)}
    h = torch.randn(6, W, generator=torch.Generator().manual_seed(0), dtype=D)
    m = {"heads": 1, "kv_heads": 1, "dim": dk, "vdim": dv, "scale": 1.0, "mask": {"size": 3}}
    out, _, v = ref.attention_mixer(h, torch.arange(6), p, m, 1e-6)
    # scores are zero, so the bias alone decides: every token attends (almost) only to itself; gate = sigmoid(0) = 1/2
    assert torch.allclose(out[:, :dv], 0.5 * v[:, 0], atol=1e-6)
    p["r1"] = torch.tensor([0.0], dtype=D)
    out, _, v = ref.attention_mixer(h, torch.arange(6), p, m, 1e-6)
    # without a bias: the mean of the block so far — token 3 starts a new block and sees itself only
    assert torch.allclose(out[3, :dv], 0.5 * v[3, 0]) and torch.allclose(out[5, :dv], 0.5 * v[3:6, 0].mean(0))
    assert torch.allclose(out[2, :dv], 0.5 * v[0:3, 0].mean(0))


def test_config_reader_and_dispatch(tmp_path):
    from tgis_amd.models import config_model_type
    from tgis_amd.models.custom_modeling.flash_senadra_modeling import SenadraConfig

    cfg = tiny.make_config(tiny.standard_layers(), width=64, vocab=96, eps=1e-5, residual_mult=0.5, side_dim=8, softcap=20.0)
    c = SenadraConfig(**cfg)
    assert (c.width, c.vocab, c.eps, c.residual_mult, c.side_dim, c.logit_softcap) == (64, 96, 1e-5, 0.5, 8, 20.0)
    assert c.hidden_size == 64 and c.vocab_size == 96 and c.num_hidden_layers == 5 and c.model_type == "senadra"
    assert config_model_type(cfg) == "senadra"
    plain = SenadraConfig(**tiny.make_config([tiny.delta_layer()], side_dim=None, softcap=None))
    assert plain.side_dim == 0 and plain.logit_softcap == 0.0
    with pytest.raises(ValueError):
        SenadraConfig(**{**cfg, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(ValueError):
        SenadraConfig(**{**cfg, "layers": [tiny.delta_layer(mlp={"kind": "moe"})]})
    with pytest.raises(ValueError):  # a layer may only borrow keys and values from an attention layer that has its own
        SenadraConfig(**{**cfg, "layers": [tiny.delta_layer(), tiny.attention_layer(kv_from=0)]})
    from tgis_amd.inference_engine.engine import BaseInferenceEngine

    (tmp_path / "config.json").write_text(json.dumps(cfg))
    loaded = BaseInferenceEngine._load_config(str(tmp_path))
    assert isinstance(loaded, SenadraConfig) and loaded.layers == cfg["layers"] and loaded.to_dict() == cfg
    if not torch.cuda.is_available():
        from tgis_amd.models import get_model

        with pytest.raises(NotImplementedError):
            get_model(str(tmp_path), None, "tgis_native", "bfloat16", None, None)


def test_state_slots_with_mixer_shapes():
    from tgis_amd.utils.state_cache import RecurrentStateCache

    st = RecurrentStateCache([None, {"matrix": (3, 2048), "memory": (2, 40)}, (2, 4)], width=16, num_slots=3, device="cpu")
    assert st.state[0] is None and st.state[1].shape == (4, 3, 2048) and st.shift[1].shape == (4, 2, 40)
    assert st.state[2].shape == (4, 2, 4, 4) and st.shift[2].shape == (4, 16)
    assert st.bytes_per_slot() == 4 * ((3 * 2048 + 80) + (2 * 16 + 16))


def test_family_build_units_and_state_size():
    from tgis_amd import buildlib, native

    for u in buildlib.FAMILY_UNITS["senadra"]:
        assert os.path.exists(os.path.join(buildlib.CSRC, u + ".hip")), u
    lib = native.load_library()
    assert lib.tgis_delta_state_floats(32, 64) == 32 * 64 and lib.tgis_delta_state_floats(20, 12) == 32 * 32
    assert lib.tgis_delta_state_floats(300, 64) == -1
