"""CPU: what the Tatevik family needs and a GPU does not — the oracle's own consistency (whole sequence == token by token ==
portions through its explicit state), hand-checkable instances of its equations, the config reader with its layer runs, model
dispatch by config.json, the state slot shapes, and the family's build units."""
import json
import math
import os

import pytest
import torch

from oracle import tatevik_ref as ref
from oracle import tatevik_tiny as tiny

D = torch.float64


def rand_tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def test_oracle_portions_equal_whole():
    cfg = tiny.make_config(tiny.standard_layers(), loop={"start": 1, "stop": 3, "times": 3})
    model = ref.TatevikRef(cfg, tiny.make_tensors(cfg, seed=1))
    toks = rand_tokens(61, cfg["vocab"], 0)
    whole = model.forward(toks)
    for cuts in ([1] * 61, [2] * 30 + [1], [17, 1, 43], [47, 2, 12], [60, 1]):
        st, outs, at = model.new_state(), [], 0
        for n in cuts:
            outs.append(model.advance(st, toks[at:at + n]))
            at += n
        assert torch.allclose(torch.cat(outs), whole, atol=1e-9, rtol=1e-9), cuts


def test_oracle_mechanisms_against_definitions():
    # layer norm: mean-free, unit variance, a gain, no bias
    z = torch.tensor([[1.0, 3.0]], dtype=D)
    assert torch.allclose(ref.layer_norm(z, torch.tensor([2.0, 0.5], dtype=D), 0.0), torch.tensor([[-2.0, 0.5]], dtype=D))
    # convolution: the last column of the filter meets the current token; the tail holds the inputs before the portion
    x = torch.tensor([[1.0], [2.0], [3.0]], dtype=D)
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=D)
    y, tail = ref.causal_conv(x, w, torch.zeros(2, 1, dtype=D))
    assert y.flatten().tolist() == [1.0, 12.0, 123.0] and tail.flatten().tolist() == [2.0, 3.0]
    y2, tail2 = ref.causal_conv(torch.tensor([[4.0]], dtype=D), w, tail)
    assert y2.flatten().tolist() == [234.0] and tail2.flatten().tolist() == [3.0, 4.0]
    # rotation of pairs: (1, 0) at position p turns to (cos a, sin a) with a = p base^(-2i / dims); channels past dims pass
    x = torch.tensor([[[1.0, 0.0, 1.0, 0.0, 5.0, 6.0]]], dtype=D)
    r = ref.rotate_pairs(x, torch.tensor([3]), 100.0, 4)
    assert torch.allclose(r[0, 0], torch.tensor([math.cos(3.0), math.sin(3.0), math.cos(0.3), math.sin(0.3), 5.0, 6.0], dtype=D))
    # mixing the heads' scores: with M = [[0, 1], [1, 0]] head 0 weighs the keys by head 1's scores
    q = torch.tensor([[[1.0], [0.0]]], dtype=D)           # head 0 asks, head 1 does not
    K = torch.tensor([[[0.0]], [[5.0]]], dtype=D)          # one kv head, two keys
    V = torch.tensor([[[1.0]], [[2.0]]], dtype=D)
    o = ref.attend_mixed(q, K, V, torch.tensor([1]), torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=D), 1.0, 0)
    assert abs(float(o[0, 0, 0]) - 1.5) < 1e-12            # head 0 gets head 1's flat scores: the mean of the values
    assert abs(float(o[0, 1, 0]) - (1 + 2 * math.exp(5)) / (1 + math.exp(5))) < 1e-12
    # the window: position 9 with a window of 3 sees 7, 8, 9
    o = ref.attend_mixed(torch.zeros(1, 1, 1, dtype=D), torch.zeros(12, 1, 1, dtype=D), torch.arange(12, dtype=D).view(12, 1, 1),
                         torch.tensor([9]), torch.eye(1, dtype=D), 1.0, 3)
    assert abs(float(o) - 8.0) < 1e-12
    # linear attention, one head of width 1: S <- a S + k v, o = S q, read after the update
    one = lambda *v: torch.tensor(v, dtype=D).view(-1, 1, 1)
    o, S = ref.linear_attention(one(2.0, 1.0), one(1.0, 3.0), one(4.0, 5.0), one(0.5, 0.25), torch.zeros(1, 1, 1, dtype=D))
    # t0: S = 4, o = 8.   t1: S = 1 + 15 = 16, o = 16
    assert o.flatten().tolist() == [8.0, 16.0] and float(S) == 16.0
    # the selective scan with one channel and one state: S <- exp(-d) S + d x B, y = S C + D x
    p = {"in": torch.tensor([[1.0], [0.0]], dtype=D), "conv": torch.tensor([[1.0]], dtype=D), "conv.b": torch.zeros(1, dtype=D),
         "x": torch.tensor([[0.0], [1.0], [1.0]], dtype=D), "dt": torch.zeros(1, 1, dtype=D), "dt.b": torch.tensor([math.log(math.e - 1)], dtype=D),
         "A_log": torch.zeros(1, 1, dtype=D), "D": torch.tensor([2.0], dtype=D), "o": torch.ones(1, 1, dtype=D)}
    st = {"S": torch.zeros(1, 1, dtype=D), "tail": torch.zeros(0, 1, dtype=D)}
    y = ref.selective_scan_mixer(torch.tensor([[1.0]], dtype=D), p, {"inner": 1, "state": 1, "dt_rank": 1, "conv": 1}, st)
    xs = 1 / (1 + math.exp(-1.0))                          # silu(1); d = softplus(bias) = 1; B = C = xs; z = 0: silu(z) = 0
    assert abs(float(st["S"]) - xs * xs) < 1e-12 and float(y) == 0.0
    # routing: scores are the softmax; the correction only chooses; groups that lose count as minus infinity
    p = {"router": torch.eye(4, dtype=D), "correction": torch.tensor([0.0, 0.0, 0.0, 0.7], dtype=D)}
    h = torch.tensor([[2.0, 1.0, 0.0, 0.0]], dtype=D)
    s = torch.softmax(h, -1)[0]
    idx, wt, _, _ = ref.route(h, p, {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}})
    assert sorted(idx[0].tolist()) == [2, 3]               # the corrected expert 3 makes its group the best one
    assert torch.allclose(wt[0].sum(), torch.tensor(1.0, dtype=D)) and torch.allclose(wt[0, idx[0].tolist().index(3)], s[3] / (s[2] + s[3]))
    idx, _, _, _ = ref.route(h, p, {"experts": 4, "top": 2, "groups": {"count": 1, "keep": 1}})
    assert sorted(idx[0].tolist()) == [0, 3]
    # the polynomial of unit-RMS powers
    q = {"up": torch.eye(2, dtype=D), "down": torch.eye(2, dtype=D), "act": torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=D)}
    z = torch.tensor([[1.0, -1.0]], dtype=D)
    assert torch.allclose(ref.power_norm_mlp(z, q, 0.0), torch.tensor([[1 + 2 + 3 + 4.0, -1 + 2 - 3 + 4.0]], dtype=D))


def test_layer_runs_and_loop_entry():
    cfg = tiny.make_config([tiny.scan_layer(inner=8, state=2, dt_rank=2, conv=2), tiny.channel_decay_layer(heads=1, dim=4, vdim=4, rank=2)],
                           width=8, vocab=12, taps=0, loop={"start": 1, "stop": 2, "times": 2})
    assert ref.layer_runs(cfg) == [(0, None, False), (1, 0, True), (1, 1, True)]
    assert ref.layer_runs({**cfg, "loop": None}) == [(0, None, False), (1, None, False)]
    t = tiny.make_tensors(cfg, seed=0)
    for k in list(t):
        if k.endswith(".o"):
            t[k] = torch.zeros_like(t[k])                   # no mixer contributes: the stream is what the loop's entries make of it
    trace = []
    ref.TatevikRef(cfg, t).forward([1, 2], trace)
    x0 = t["embed"].double()[[1, 2]] * cfg["embedding"]["scale"]
    w, step = t["loop.in"].double(), t["loop.step"].double()
    x1 = torch.cat([x0, x0], -1) @ w.T + step[0]
    x2 = torch.cat([x1, x0], -1) @ w.T + step[1]
    assert torch.allclose(trace[0], x0) and torch.allclose(trace[1], x1) and torch.allclose(trace[2], x2)


def test_config_reader_and_dispatch(tmp_path):
    from tgis_amd.models import config_model_type
    from tgis_amd.models.custom_modeling.flash_tatevik_modeling import TatevikConfig

    cfg = tiny.make_config(tiny.standard_layers(), width=64, vocab=96, eps=1e-5, loop={"start": 2, "stop": 5, "times": 2})
    c = TatevikConfig(**cfg)
    assert (c.width, c.vocab, c.eps, c.canon_taps, c.embedding_scale) == (64, 96, 1e-5, 4, 0.7)
    assert [i for i, _ in c.runs] == [0, 1, 2, 3, 4, 2, 3, 4, 5] and [t for _, t in c.runs] == [None, None, 0, None, None, 1, None, None, None]
    assert c.hidden_size == 64 and c.vocab_size == 96 and c.num_hidden_layers == 9 and c.model_type == "tatevik"
    assert config_model_type(cfg) == "tatevik"
    assert TatevikConfig(**{k: v for k, v in cfg.items() if k not in ("loop", "canon", "embedding")}).runs == [(i, None) for i in range(6)]
    with pytest.raises(ValueError):
        TatevikConfig(**{**cfg, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(ValueError):
        TatevikConfig(**{**cfg, "layers": [tiny.scan_layer(mlp={"kind": "sparse"})]})
    with pytest.raises(ValueError):
        TatevikConfig(**{**cfg, "loop": {"start": 3, "stop": 9, "times": 2}})
    from tgis_amd.inference_engine.engine import BaseInferenceEngine

    (tmp_path / "config.json").write_text(json.dumps(cfg))
    loaded = BaseInferenceEngine._load_config(str(tmp_path))
    assert isinstance(loaded, TatevikConfig) and loaded.layers == cfg["layers"] and loaded.to_dict() == cfg
    if not torch.cuda.is_available():
        from tgis_amd.models import get_model

        with pytest.raises(NotImplementedError):
            get_model(str(tmp_path), None, "tgis_native", "bfloat16", None, None)


def test_state_slot_shapes_and_build_units():
    from tgis_amd import buildlib
    from tgis_amd.utils.state_cache import RecurrentStateCache

    st = RecurrentStateCache([{"matrix": (96, 12), "memory": (3 * 72 + 3 * 96,)}, {"matrix": (3, 24, 40), "memory": (216,)}], width=72,
                             num_slots=2, device="cpu")
    assert st.state[0].shape == (3, 96, 12) and st.shift[0].shape == (3, 504) and st.state[1].shape == (3, 3, 24, 40)
    for u in buildlib.FAMILY_UNITS["tatevik"]:
        assert os.path.exists(os.path.join(buildlib.CSRC, u + ".hip")), u
