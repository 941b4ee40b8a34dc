"""Tatevik: a decoder of PARALLEL layers over an fp32 residual stream with per-channel scales on both sublayers, an input
convolution in front of each of them, and an optional loop over a run of layers —

    h = LN(x);   x <- x + s1 * mixer(h + C1(h)) + s2 * ff(h + C2(h))          LN: mean-free, unit variance, a gain, no bias

with C1, C2 short causal per-channel convolutions over time (their last inputs are part of a sequence's state).  Layers
`loop.start .. loop.stop - 1` run `loop.times` times in a row with the same weights; every pass has caches and states of its
own and starts from x <- W_in [x; x0] + step[pass], x0 the scaled embedding.  Mixers: `mamba1` (selective state-space scan),
`parallel` (softmax attention with scores mixed over the heads, beside a linear attention with one decay per head; both
results RMS-normed over the width and averaged) and `gla` (linear attention with a learned decay per key channel).
Feed-forwards: `dense` (a polynomial of unit-RMS powers between two projections) or `moe` (SiLU gated experts chosen among the
best groups by softmax scores plus a correction) or none.  A final LN and an untied head.

config.json gives `width`, `vocab`, `norm.eps`, `embedding.scale`, `canon.taps`, `loop` and `layers[i].type|mixer|mlp`;
tensors are named `embed`, `loop.in`, `loop.step`, `l<i>.norm1`, `l<i>.ls1|ls2`, `l<i>.canon1|canon2`, `l<i>.mix.*`,
`l<i>.mlp.*`, `final.norm`, `head`.  This file only maps those keys and names onto the mechanisms of utils/mixers.py; the
step (ragged: portions of prompts beside decoded tokens), the paged KV pool and the recurrent state slots are FlashCausalLM's
(models/flash_causal_lm.py).  A layer that runs in several passes appears once per pass in the model's list of layer runs:
that list, not the list of weights, is what the caches are made for."""
import json
from typing import List, Optional

import torch

from tgis_amd import native
from tgis_amd.utils.layers import FastLinear
from tgis_amd.utils.mixers import (DecayedLinearAttention, InputConvolutions, MixedHeadAttention, NormedPairMixers, PowerNormMLP,
                                   RoutedExperts, SelectiveScanMixer, SingleMixer, _f32, load_linear)

MIXER_TYPES = ("mamba1", "parallel", "gla")
# the two side-by-side mixers are averaged
PAIR_COEF = 0.5
# what guards the sum of the chosen experts' scores
ROUTER_RENORM_EPS = 1e-20
# rows up to which the pair's average rides in the residual update
PAIR_FUSED_MAX_ROWS = 256


class TatevikConfig:
    model_type = "tatevik"

    def __init__(self, width: int, vocab: int, layers: List[dict], norm: dict, embedding: Optional[dict] = None,
                 canon: Optional[dict] = None, loop: Optional[dict] = None, **kwargs):
        self.width, self.vocab, self.layers = int(width), int(vocab), layers
        self.eps = float(norm["eps"])
        self.embedding_scale = float((embedding or {}).get("scale", 1.0))
        self.canon_taps = int((canon or {}).get("taps", 0))
        self.loop = dict(loop) if loop else None
        for k, v in kwargs.items():
            setattr(self, k, v)
        for i, lay in enumerate(layers):
            if lay["type"] not in MIXER_TYPES:
                raise ValueError(f"layer {i}: unknown mixer type {lay['type']!r}")
            f = lay.get("mlp")
            if f and f.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        self.runs = self.layer_runs()
        # the names the serving path shares with the other families (a "layer" of the caches is a layer RUN)
        self.hidden_size, self.vocab_size, self.num_hidden_layers = self.width, self.vocab, len(self.runs)
        self.pad_token_id = self.bos_token_id = self.eos_token_id = None
        self.quantize = None

    def layer_runs(self):
        """[(layer index, pass number or None)] in execution order; a pass number is given where a pass begins."""
        n = len(self.layers)
        if not self.loop:
            return [(i, None) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        if not (0 <= a < b <= n and times >= 1):
            raise ValueError(f"loop over layers {a} .. {b - 1}, {times} times, of {n} layers")
        runs = [(i, None) for i in range(a)]
        for t in range(times):
            runs += [(i, t if i == a else None) for i in range(a, b)]
        return runs + [(i, None) for i in range(b, n)]

    @classmethod
    def from_json(cls, path: str) -> "TatevikConfig":
        with open(path) as f:
            return cls(**json.load(f))

    def to_dict(self):
        d = {"architecture": "Tatevik", "width": self.width, "vocab": self.vocab, "layers": self.layers, "norm": {"eps": self.eps},
             "embedding": {"scale": self.embedding_scale}}
        if self.canon_taps:
            d["canon"] = {"taps": self.canon_taps}
        if self.loop:
            d["loop"] = self.loop
        return d


class TatevikLayer:
    """The weights of one layer (shared by its runs)."""

    def __init__(self, i: int, config: TatevikConfig, weights):
        lay = config.layers[i]
        m, eps = lay["mixer"], config.eps
        self.kind = lay["type"]
        self.norm1 = _f32(weights.get_tensor(f"l{i}.norm1"))
        self.ls1 = _f32(weights.get_tensor(f"l{i}.ls1"))
        f = lay.get("mlp")
        self.ls2 = _f32(weights.get_tensor(f"l{i}.ls2")) if f else None
        self.canon = None
        if config.canon_taps:
            names = [f"l{i}.canon1"] + ([f"l{i}.canon2"] if f else [])
            self.canon = InputConvolutions(weights, names, config.width, config.canon_taps)
        self.kv_shape = None
        if self.kind == "mamba1":
            self.mixer = SelectiveScanMixer(weights, f"l{i}.mix", inner=int(m["inner"]), state=int(m["state"]), dt_rank=int(m["dt_rank"]),
                                            taps=int(m["conv"]))
            self.state_matrix, self.mixer_floats = self.mixer.state_matrix, self.mixer.memory_floats
        elif self.kind == "parallel":
            l, r = m["left"], m["right"]
            heads = int(l["heads"])
            mask, rot = l.get("mask") or {}, l.get("rot") or {}
            left = MixedHeadAttention(weights, f"l{i}.mix.left", heads=heads, kv_heads=int(l.get("kv_heads", heads)), dim=int(l["dim"]),
                                      vdim=int(l.get("vdim", l["dim"])), scale=float(l["scale"]), eps=eps, window=int(mask.get("size", 0)),
                                      rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)))
            right = DecayedLinearAttention(weights, f"l{i}.mix.right", heads=int(r["heads"]), dim=int(r["dim"]),
                                           vdim=int(r.get("vdim", r["dim"])), eps=eps, decay="head", head_decay=r["decay"], act=True,
                                           norm="row", gate="sigmoid")
            self.mixer = NormedPairMixers(weights, left, right, f"l{i}.mix.left.out", f"l{i}.mix.right.out", eps, coef=PAIR_COEF)
            self.kv_shape = left.kv_shape
            self.state_matrix, self.mixer_floats = right.state_matrix, 0
        else:
            dim = int(m["dim"])
            gla = DecayedLinearAttention(weights, f"l{i}.mix", heads=int(m["heads"]), dim=dim, vdim=int(m.get("vdim", dim)), eps=eps,
                                         decay="channel", tau=float(m["tau"]), q_scale=dim ** -0.5, norm="head", gate="silu")
            self.mixer = SingleMixer(weights, gla)
            self.state_matrix, self.mixer_floats = gla.state_matrix, 0
        self.ff = None
        if f:
            if f["kind"] == "dense":
                self.ff = PowerNormMLP(weights, f"l{i}.mlp", eps)
            else:
                r = f["router"]
                g = r.get("groups") or {}
                count = int(g.get("count", 1))
                self.ff = RoutedExperts(weights, f"l{i}.mlp", experts=int(r["experts"]), top=int(r["top"]), shared=False,
                                        weight_on_input=False, grouped_softmax=True, groups=count, keep_groups=int(g.get("keep", count)),
                                        renorm_eps=ROUTER_RENORM_EPS)
        # a slot's memory of this layer: the input convolutions' tail, then the mixer's own
        self.canon_floats = self.canon.floats if self.canon is not None else 0
        self.state_shape = {"matrix": self.state_matrix, "memory": (max(self.canon_floats + self.mixer_floats, 1),)}


class TatevikRun:
    """One execution of a layer: the layer's weights and the run's place in the caches."""

    def __init__(self, layer: TatevikLayer, cache_id: int, pass_number: Optional[int]):
        self.layer, self.cache_id, self.pass_number = layer, cache_id, pass_number


class FlashTatevikModel:
    def __init__(self, config: TatevikConfig, weights):
        if weights.process_group.size() != 1:
            raise NotImplementedError("Tatevik is served by one process per model: its layers are not sharded")
        self.config = config
        self.dtype = weights.dtype
        self.embed = weights.get_tensor("embed").contiguous()
        self.weights_of = [TatevikLayer(i, config, weights) for i in range(len(config.layers))]
        self.layers = [TatevikRun(self.weights_of[i], r, t) for r, (i, t) in enumerate(config.runs)]
        self.loop_in = self.loop_step = None
        if config.loop:
            self.loop_in = load_linear(weights, "loop.in")
            self.loop_step = _f32(weights.get_tensor("loop.step"))
            if self.loop_step.shape[0] < int(config.loop["times"]):
                raise ValueError(f"loop.step has {self.loop_step.shape[0]} rows for {config.loop['times']} passes")
        self.final_norm = _f32(weights.get_tensor("final.norm"))
        # cache geometry, read by FlashCausalLM: one entry per layer RUN
        self.kv_layer_shapes = [r.layer.kv_shape for r in self.layers]
        self.state_layer_shapes = [r.layer.state_shape for r in self.layers]
        att = [l.mixer.left for l in self.weights_of if l.kind == "parallel"]
        self.num_heads = max([a.H for a in att], default=1)
        self.num_key_value_heads = max([a.G for a in att], default=1)
        self.head_size = max([a.dk for a in att], default=8)
        self.supports_ragged_steps = True

    def forward(self, input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds, kv):
        if inputs_embeds is not None:
            raise NotImplementedError("prompt prefixes (inputs_embeds) are not wired into the fp32-residual path")
        cfg, dt = self.config, self.dtype
        eps, n = cfg.eps, len(self.layers)
        kv.cu_seqlens_q = cu_seqlens_q
        x0 = native.embedding_scaled_f32(input_ids, self.embed, cfg.embedding_scale)
        x = x0
        # the normed input of the first run; afterwards a run's residual update also norms for the next one, unless a pass
        # begins there
        x, h = self.enter(x, x0, self.layers[0], eps, dt)
        for r, run in enumerate(self.layers):
            layer = run.layer
            memory = kv.state.shift[run.cache_id]
            if layer.canon is not None:
                hs = layer.canon(h, memory[:, :layer.canon_floats] if layer.canon_floats else None, position_ids, kv, dt)
                h1, h2 = hs[0], hs[-1]
            else:
                h1 = h2 = h
            state = kv.state.state[run.cache_id]
            pair = None
            if layer.kind == "mamba1":
                tail = memory[:, layer.canon_floats:layer.canon_floats + layer.mixer_floats] if layer.mixer_floats else None
                y = layer.mixer.forward(h1, position_ids, kv, state, tail)
            elif layer.kind == "parallel":
                # decode-sized steps: the two mixers' rows are normed and averaged by the residual update below (one launch
                # less); long steps keep the launch of their own (the fused form reads both rows twice)
                y = layer.mixer.forward(h1, position_ids, kv, run.cache_id, state, defer=h1.shape[0] <= PAIR_FUSED_MAX_ROWS)
                if isinstance(y, tuple):
                    y, pair = y
            else:
                y = layer.mixer.forward(h1, position_ids, kv, run.cache_id, state)
            y_ff = layer.ff(h2) if layer.ff is not None else None
            nxt = self.layers[r + 1] if r + 1 < n else None
            fused = nxt is None or nxt.pass_number is None
            gain = (nxt.layer.norm1 if nxt is not None else self.final_norm) if fused else None
            last = nxt is None
            x, h = native.scaled_residual_norm(x, y, layer.ls1, y_ff, layer.ls2, None, gain, eps, dt, x_out=None if x is x0 else x,
                                               h_f32=not last and cfg.canon_taps > 0, pair=pair)
            if kv.residual_trace is not None:
                kv.residual_trace.append(x.clone())
            if not fused:
                x, h = self.enter(x, x0, nxt, eps, dt)
        return h  # final-normed, in the serving dtype

    def enter(self, x, x0, run: TatevikRun, eps: float, dt):
        """What comes in front of a run that the run before it did not prepare: where a pass begins, the pass's mix with the
        embedding and its step vector; then the layer's norm.  Returns (the stream, the normed input)."""
        h_f32 = self.config.canon_taps > 0
        if run.pass_number is None:
            return x, native.scaled_residual_norm(x, None, None, None, None, None, run.layer.norm1, eps, dt, h_f32=h_f32, keep_x=False)[1]
        both = torch.cat([x, x0], dim=1).to(dt)
        mixed = self.loop_in(both, out_f32=True)
        return native.scaled_residual_norm(mixed, None, None, None, None, self.loop_step[run.pass_number], run.layer.norm1, eps, dt,
                                           x_out=mixed, h_f32=h_f32)

    __call__ = forward


class FlashTatevikForCausalLM:
    def __init__(self, config: TatevikConfig, weights):
        self.config = config
        self.model = FlashTatevikModel(config, weights)
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
        if hidden.shape[0] == 0:
            return torch.empty((0, self.config.vocab), dtype=torch.float32, device=hidden.device)
        # fp32 logits from the weight-streaming kernel's fp32 accumulators, 256 rows at a time (the library GEMM above that
        # size would round them to the serving dtype first)
        if hidden.shape[0] <= 256:
            return self.lm_head(hidden, out_f32=True)
        return torch.cat([self.lm_head(hidden[i:i + 256], out_f32=True) for i in range(0, hidden.shape[0], 256)], 0)

    __call__ = forward
