"""CPU: what the Mananex family needs and a GPU does not — the oracle's own consistency (whole sequence == token by token ==
portions through its explicit state), hand-checkable instances of its equations, the config reader, model dispatch by
config.json, the state slot shapes, and the family's build units."""
import json
import math
import os

import pytest
import torch

from oracle import mananex_ref as ref
from oracle import mananex_tiny as tiny

D = torch.float64


def rand_tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def test_oracle_portions_equal_whole():
    """The oracle's state (rotated keys, values, the recurrence's matrices) carries everything: any cut of a sequence gives the
    logits of the whole, to float64 rounding."""
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
    assert torch.allclose(ref.offset_norm(z, torch.tensor([0.0, 1.0], dtype=D), 0.0), torch.tensor([[3.0, 8.0]], dtype=D) / 12.5 ** 0.5)
    # rotation of pairs: (1, 0) at position p turns to (cos a, sin a) with a = p base^(-2i / dims); channels past dims pass
    x = torch.tensor([[[1.0, 0.0, 1.0, 0.0, 5.0, 6.0]]], dtype=D)
    r = ref.rotate_pairs(x, torch.tensor([3]), 100.0, 4)
    assert torch.allclose(r[0, 0], torch.tensor([math.cos(3.0), math.sin(3.0), math.cos(0.3), math.sin(0.3), 5.0, 6.0], dtype=D))
    # the window and the kept first positions: position 9 with a window of 3 keeping 2 sees 0, 1 and 7, 8, 9
    assert ref.visible(torch.tensor([9]), 12, 3, 2)[0].nonzero().flatten().tolist() == [0, 1, 7, 8, 9]
    assert ref.visible(torch.tensor([2]), 12, None, 0)[0].nonzero().flatten().tolist() == [0, 1, 2]
    # a sink equal to the only score halves the weight; no value goes with it
    w = ref.sink_softmax(torch.tensor([[0.7, float("-inf")]], dtype=D), torch.tensor(0.7, dtype=D))
    assert torch.allclose(w, torch.tensor([[0.5, 0.0]], dtype=D))
    # the forget gate stays above its lower bound
    f = ref.forget_gate(torch.tensor([-50.0, 0.0, 50.0], dtype=D), torch.tensor(0.6, dtype=D))
    assert torch.allclose(f, torch.tensor([0.6, 0.8, 1.0], dtype=D))
    # recurrence, one head of width 1: S <- f S + (1 - f) v; o = S q, read after the update
    one = lambda v: torch.tensor([[[v]]], dtype=D)
    o, S = ref.gated_linear_recurrence(torch.cat([one(2.0), one(1.0)]), torch.cat([one(0.5), one(0.25)]), torch.cat([one(4.0), one(8.0)]),
                                       torch.zeros(1, 1, 1, dtype=D))
    # t0: S = 2, o = 4.   t1: S = 0.5 + 6 = 6.5, o = 6.5
    assert torch.allclose(o.flatten(), torch.tensor([4.0, 6.5], dtype=D)) and float(S) == 6.5
    # top-2 of three logits, softmaxed among themselves
    p = {"router": torch.eye(3, dtype=D), "router.b": torch.tensor([0.0, 0.0, 1.0], dtype=D)}
    idx, wt = ref.route_top_softmax(torch.tensor([[2.0, 0.5, 1.0]], dtype=D), p, 2)
    assert sorted(idx[0].tolist()) == [0, 2] and torch.allclose(wt, torch.tensor([[0.5, 0.5]], dtype=D))


def test_layer_equation_in_the_oracle():
    """With zero projections in both sublayers a layer hands on only the mix over depth: x' = a[0] Y_0 + a[1] Y_0."""
    cfg = tiny.make_config([tiny.layer(mlp=tiny.dense_mlp(8))], width=16, vocab=12)
    t = tiny.make_tensors(cfg, seed=0)
    for k in list(t):
        if k.endswith(".o") or k.endswith("mlp.down") or k.endswith("mlp.down.b"):
            t[k] = torch.zeros_like(t[k])
    t["l0.dwa"] = torch.tensor([0.25, 0.5])
    trace = []
    ref.forward(cfg, t, [1, 2, 3], trace)
    assert torch.allclose(trace[0], 0.75 * t["embed"].double()[[1, 2, 3]])


def test_config_reader_and_dispatch(tmp_path):
    from tgis_amd.models import config_model_type
    from tgis_amd.models.custom_modeling.flash_mananex_modeling import MananexConfig

    cfg = tiny.make_config(tiny.standard_layers(), width=64, vocab=96, eps=1e-5)
    c = MananexConfig(**cfg)
    assert (c.width, c.vocab, c.eps) == (64, 96, 1e-5)
    assert c.hidden_size == 64 and c.vocab_size == 96 and c.num_hidden_layers == 4 and c.model_type == "mananex"
    assert config_model_type(cfg) == "mananex"
    with pytest.raises(ValueError):
        MananexConfig(**{**cfg, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(ValueError):
        MananexConfig(**{**cfg, "layers": [tiny.layer(mlp={"kind": "sparse"})]})
    from tgis_amd.inference_engine.engine import BaseInferenceEngine

    (tmp_path / "config.json").write_text(json.dumps(cfg))
    loaded = BaseInferenceEngine._load_config(str(tmp_path))
    assert isinstance(loaded, MananexConfig) and loaded.layers == cfg["layers"] and loaded.to_dict() == cfg
    if not torch.cuda.is_available():
        from tgis_amd.models import get_model

        with pytest.raises(NotImplementedError):
            get_model(str(tmp_path), None, "tgis_native", "bfloat16", None, None)


def test_state_slot_shapes_and_build_units():
    from tgis_amd import buildlib
    from tgis_amd.utils.state_cache import RecurrentStateCache

    st = RecurrentStateCache([{"matrix": (3, 16, 32), "memory": (1,)}, None], width=16, num_slots=2, device="cpu")
    assert st.state[0].shape == (3, 3, 16, 32) and st.shift[0].shape == (3, 1) and st.state[1] is None
    for u in buildlib.FAMILY_UNITS["mananex"]:
        assert os.path.exists(os.path.join(buildlib.CSRC, u + ".hip")), u
