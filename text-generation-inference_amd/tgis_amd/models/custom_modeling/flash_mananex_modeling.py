"""Mananex: a decoder of PARALLEL layers over an fp32 residual stream with gated residuals and a learned mix over depth —

    h = N(x);   y = x + sigmoid(R1 h + b1) * mixer(h) + sigmoid(R2 h + b2) * ff(h);   x' = sum_{j <= i + 1} a_i[j] Y_j

with N(z) = z / sqrt(mean(z^2) + eps) * (1 + w), Y_0 the embedding output and Y_(j+1) layer j's y.  The mixer runs two mixers
side by side on the same h: windowed softmax attention with kept first positions, a sink logit and a per-head output gate
("left"), and an HGRN2-style gated linear recurrence ("right"); their results are added with two fixed weights.  The
feed-forward is a SiLU gated unit with biases or a mixture of bias-free gated experts whose top-k router logits are softmaxed
among themselves.  The head is the embedding table.

config.json gives `width`, `vocab`, `norm.eps` and `layers[i].type|mixer|mlp`; tensors are named `embed`, `l<i>.norm1`,
`l<i>.mix.left.*`, `l<i>.mix.right.*`, `l<i>.mlp.*`, `l<i>.rg1|rg2(.b)`, `l<i>.dwa`, `final.norm`.  This file only maps those keys
and names onto the mechanisms of utils/mixers.py; the step (ragged: portions of prompts beside decoded tokens), the paged KV
pool and the recurrent state slots are FlashCausalLM's (models/flash_causal_lm.py)."""
import json
from typing import List, Optional

import torch

from tgis_amd import native
from tgis_amd.utils.layers import FastLinear
from tgis_amd.utils.mixers import GatedLinearRecurrence, GatedUnit, RoutedExperts, SideBySideMixers, WindowSinkAttention, _f32

MIXER_TYPES = ("parallel",)
# the gain of every norm of the design is stored as an offset from one
NORM_GAIN_OFFSET = 1.0


class MananexConfig:
    model_type = "mananex"

    def __init__(self, width: int, vocab: int, layers: List[dict], norm: dict, **kwargs):
        self.width, self.vocab, self.layers = int(width), int(vocab), layers
        self.eps = float(norm["eps"])
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
            if f and f.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")

    @classmethod
    def from_json(cls, path: str) -> "MananexConfig":
        with open(path) as f:
            return cls(**json.load(f))

    def to_dict(self):
        return {"architecture": "Mananex", "width": self.width, "vocab": self.vocab, "layers": self.layers, "norm": {"eps": self.eps}}


class MananexLayer:
    def __init__(self, i: int, config: MananexConfig, weights):
        lay = config.layers[i]
        m = lay["mixer"]
        self.layer_id = i
        self.norm1 = _f32(weights.get_tensor(f"l{i}.norm1"))
        left, right = m["left"], m["right"]
        mask, rot = left.get("mask") or {}, left.get("rot") or {}
        heads = int(left["heads"])
        self.attention = WindowSinkAttention(
            weights, f"l{i}.mix.left", i, heads=heads, kv_heads=int(left.get("kv_heads", heads)), dim=int(left["dim"]),
            vdim=int(left.get("vdim", left["dim"])), scale=float(left["scale"]), window=int(mask.get("size", 0)),
            keep_first=int(mask.get("keep_first", 0)), rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)))
        self.recurrence = GatedLinearRecurrence(weights, f"l{i}.mix.right", i, heads=int(right["heads"]), dim=int(right["dim"]),
                                                vdim=int(right.get("vdim", right["dim"])), eps=config.eps)
        f = lay.get("mlp")
        # the residual gates read h too: they ride in the mixers' stacked projection
        self.gate_names = [f"l{i}.rg1"] + ([f"l{i}.rg2"] if f else [])
        self.mixer = SideBySideMixers(weights, [self.attention, self.recurrence],
                                      [float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))], extra_in=self.gate_names)
        self.gate_bias = [weights.get_tensor(n + ".b").contiguous() for n in self.gate_names]
        self.ff = None
        self.dense_ff = bool(f) and f["kind"] == "dense"
        if f:
            if self.dense_ff:
                self.ff = GatedUnit(weights, f"l{i}.mlp", mode="silu", bias=True)
            else:
                self.ff = RoutedExperts(weights, f"l{i}.mlp", experts=int(f["router"]["experts"]), top=int(f["router"]["top"]),
                                        shared=False, router_bias=True, softmax_top=True, weight_on_input=False)
        # x' = sum_j mix[j] Y_j over the embedding output and the results of layers 0 .. i
        self.depth_mix = _f32(weights.get_tensor(f"l{i}.dwa")).reshape(-1)
        if self.depth_mix.shape[0] != i + 2:
            raise ValueError(f"layer {i}: the depth mix has {self.depth_mix.shape[0]} coefficients, not {i + 2}")
        self.kv_shape, self.state_shape = self.attention.kv_shape, self.recurrence.state_shape


class FlashMananexModel:
    def __init__(self, config: MananexConfig, weights):
        if weights.process_group.size() != 1:
            raise NotImplementedError("Mananex is served by one process per model: its layers are not sharded")
        self.config = config
        self.dtype = weights.dtype
        self.embed = weights.get_tensor("embed").contiguous()
        self.layers = [MananexLayer(i, config, weights) for i in range(len(config.layers))]
        self.final_norm = _f32(weights.get_tensor("final.norm"))
        # cache geometry, read by FlashCausalLM
        self.kv_layer_shapes = [l.kv_shape for l in self.layers]
        self.state_layer_shapes = [l.state_shape for l in self.layers]
        self.num_heads = max(l.attention.H for l in self.layers)
        self.num_key_value_heads = max(l.attention.G for l in self.layers)
        self.head_size = max(l.attention.dk for l in self.layers)
        self.supports_ragged_steps = True

    def forward(self, input_ids, position_ids, cu_seqlens_q, max_s, inputs_embeds, kv):
        if inputs_embeds is not None:
            raise NotImplementedError("prompt prefixes (inputs_embeds) are not wired into the fp32-residual path")
        cfg, dt = self.config, self.dtype
        eps, n = cfg.eps, len(self.layers)
        kv.cu_seqlens_q = cu_seqlens_q
        T = input_ids.shape[0]
        # Y_0 .. Y_n of this step's tokens: what the mix over depth reads
        hist = torch.empty((n + 1, T, cfg.width), dtype=torch.float32, device=input_ids.device)
        native.embedding_scaled_f32(input_ids, self.embed, 1.0, out=hist[0])
        x = torch.empty((T, cfg.width), dtype=torch.float32, device=input_ids.device)
        h = native.residual_update_f32(hist[0], None, None, self.layers[0].norm1, eps, dt, pre_add=NORM_GAIN_OFFSET)
        for i, layer in enumerate(self.layers):
            y_mix, proj = layer.mixer.forward(h, position_ids, kv)
            W = cfg.width
            gates = [proj[:, c:c + W] for c in (layer.mixer.extra_cols[g] for g in layer.gate_names)]
            y_ff = None
            if layer.ff is not None:
                y_ff = layer.ff(h, partial=True) if layer.dense_ff else layer.ff(h)
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            h = native.parallel_residual_f32(hist[0] if i == 0 else x, y_mix, gates[0], layer.gate_bias[0], y_ff,
                                             gates[1] if y_ff is not None else None, layer.gate_bias[1] if y_ff is not None else None,
                                             dt, hist, i + 1, layer.depth_mix, x, nxt, eps, dt, pre_add=NORM_GAIN_OFFSET)
            if kv.residual_trace is not None:
                kv.residual_trace.append(x.clone())
        return h  # final-normed, in the serving dtype

    __call__ = forward


class FlashMananexForCausalLM:
    def __init__(self, config: MananexConfig, weights):
        self.config = config
        self.model = FlashMananexModel(config, weights)
        # the head is the embedding table
        self.lm_head = FastLinear(self.model.embed, None)
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
