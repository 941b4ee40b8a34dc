"""Engine for seeded synthetic checkpoints held in memory (benchmarks, smoke and parity tests): same model
classes, same `Weights` interface and TP slicing as tgis_native, no files and no tokenizer download.
The weight recipe is the one SURVEY.md §8(d) defines (N(0, 0.02) dense; GPTQ: random nibbles, random zero nibbles in 0..13,
scales U(0.5,1.5)*2/15*0.02, g_idx = k // group) — there is no network for real checkpoints."""
import os
from typing import Any, Dict, Optional

import torch

from tgis_amd.inference_engine.engine import BaseInferenceEngine
from tgis_amd.inference_engine.tgis_native import _barrier, model_class_for
from tgis_amd.utils.dist import initialize_torch_distributed
from tgis_amd.utils.weights import DictWeights


class InferenceEngine(BaseInferenceEngine):
    def __init__(self, tensors: Dict[str, torch.Tensor], model_config: Any, dtype: torch.dtype,
                 quantize: Optional[str], tokenizer=None, gptq_bits: int = 4, gptq_groupsize: int = 128):
        super().__init__(None, model_config, tokenizer=tokenizer)
        model_class, _aliases = model_class_for(self._config)
        self._config.quantize = quantize
        self.process_group = initialize_torch_distributed(self.world_size, self.rank)
        _barrier(self.process_group)
        weights = DictWeights(tensors, device=self.device, dtype=dtype, process_group=self.process_group)
        if quantize == "gptq":
            weights.gptq_bits, weights.gptq_groupsize = gptq_bits, gptq_groupsize
        model = model_class(self._config, weights)
        _barrier(self.process_group)
        if not hasattr(model, "config"):
            model.config = self._config
        self.model = model


def llama_tensors(config, quantize: Optional[str], seed: int, groupsize: int = 128, device="cpu",
                  dtype=torch.float16, head_scale: float = 1.0) -> Dict[str, torch.Tensor]:
    """Seeded full (unsharded) Llama checkpoint as a name -> tensor dict in HF naming."""
    g = torch.Generator(device=device).manual_seed(seed)
    E, I, V = config.hidden_size, config.intermediate_size, config.vocab_size
    D = E // config.num_attention_heads
    Hkv = config.num_key_value_heads
    t: Dict[str, torch.Tensor] = {}

    def dense(name, n, k, std=0.02):
        t[f"{name}.weight"] = (torch.randn(n, k, generator=g, device=device) * std).to(dtype)

    def gptq(name, n, k):
        G = k // groupsize
        t[f"{name}.qweight"] = torch.randint(-2**31, 2**31 - 1, (k // 8, n), generator=g, device=device,
                                             dtype=torch.int32)
        # stored zero nibbles 0..13 (true zero points 1..14, mean 7.5 = the mean nibble): with 0..15 the dequantised
        # weights carry a common -1 * scale offset, a rank-one term that overflows fp16 activations within a few layers
        zn = torch.randint(0, 14, (G, n // 8, 8), generator=g, device=device, dtype=torch.int64)
        zw = (zn << (4 * torch.arange(8, device=device, dtype=torch.int64))).sum(-1)
        t[f"{name}.qzeros"] = torch.where(zw >= 2**31, zw - 2**32, zw).to(torch.int32)
        t[f"{name}.scales"] = ((torch.rand(G, n, generator=g, device=device) + 0.5) * (2.0 / 15.0) * 0.02
                               ).to(torch.float16)
        t[f"{name}.g_idx"] = (torch.arange(k, device=device, dtype=torch.int32) // groupsize)

    lin = gptq if quantize == "gptq" else dense
    t["model.embed_tokens.weight"] = (torch.randn(V, E, generator=g, device=device) * 0.02).to(dtype)
    for i in range(config.num_hidden_layers):
        p = f"model.layers.{i}"
        lin(f"{p}.self_attn.q_proj", E, E)
        lin(f"{p}.self_attn.k_proj", Hkv * D, E)
        lin(f"{p}.self_attn.v_proj", Hkv * D, E)
        lin(f"{p}.self_attn.o_proj", E, E)
        lin(f"{p}.mlp.gate_proj", I, E)
        lin(f"{p}.mlp.up_proj", I, E)
        lin(f"{p}.mlp.down_proj", E, I)
        t[f"{p}.input_layernorm.weight"] = torch.ones(E, device=device, dtype=dtype)
        t[f"{p}.post_attention_layernorm.weight"] = torch.ones(E, device=device, dtype=dtype)
    t["model.norm.weight"] = torch.ones(E, device=device, dtype=dtype)
    t["lm_head.weight"] = (torch.randn(V, E, generator=g, device=device) * 0.02 * head_scale).to(dtype)
    return t


class BigCodeConfig:
    """The fields of HF's GPTBigCodeConfig that FlashSantacoderForCausalLM reads (multi-query attention)."""
    model_type = "gpt_bigcode"

    def __init__(self, vocab_size=49152, hidden_size=6144, n_inner=24576, num_hidden_layers=40, num_attention_heads=48,
                 layer_norm_epsilon=1e-5, n_positions=8192, activation_function="gelu_pytorch_tanh"):
        self.vocab_size, self.hidden_size, self.n_inner = vocab_size, hidden_size, n_inner
        self.num_hidden_layers, self.num_attention_heads = num_hidden_layers, num_attention_heads
        self.layer_norm_epsilon, self.n_positions = layer_norm_epsilon, n_positions
        self.activation_function = activation_function
        self.multi_query = True
        self.architectures = ["GPTBigCodeForCausalLM"]
        self.transpose = False
        self.pad_token_id, self.bos_token_id, self.eos_token_id = 0, 0, 0
        self.tie_word_embeddings = True
        # the names the benchmark's byte accounting shares with Llama
        self.intermediate_size = n_inner
        self.num_key_value_heads = 1


def bigcode_tensors(config, seed: int, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Seeded full GPT-BigCode checkpoint in HF naming (tied head): N(0, 1/sqrt(fan_in)) weights, small biases."""
    g = torch.Generator(device=device).manual_seed(seed)
    E, I, V = config.hidden_size, config.n_inner, config.vocab_size
    D = E // config.num_attention_heads
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k):
        t[f"{name}.weight"] = (torch.randn(n, k, generator=g, device=device) * k ** -0.5).to(dtype)
        t[f"{name}.bias"] = (torch.randn(n, generator=g, device=device) * 0.02).to(dtype)

    def ln(name):
        t[f"{name}.weight"] = torch.ones(E, device=device, dtype=dtype)
        t[f"{name}.bias"] = torch.zeros(E, device=device, dtype=dtype)

    t["transformer.wte.weight"] = (torch.randn(V, E, generator=g, device=device) * 0.02).to(dtype)
    t["transformer.wpe.weight"] = (torch.randn(config.n_positions, E, generator=g, device=device) * 0.02).to(dtype)
    for i in range(config.num_hidden_layers):
        p = f"transformer.h.{i}"
        ln(f"{p}.ln_1")
        lin(f"{p}.attn.c_attn", E + 2 * D, E)
        lin(f"{p}.attn.c_proj", E, E)
        ln(f"{p}.ln_2")
        lin(f"{p}.mlp.c_fc", I, E)
        lin(f"{p}.mlp.c_proj", E, I)
    ln("transformer.ln_f")
    return t


def lenisun_tensors(config, seed: int, device="cpu", dtype=torch.bfloat16, decay_rank: int = 64) -> Dict[str, torch.Tensor]:
    """Seeded full Lenisun checkpoint in the family's tensor naming for a `LenisunConfig`: N(0, 1 / fan_in) projections,
    small norm gains around zero, decays spread over (0, 1)."""
    g = torch.Generator(device=device).manual_seed(seed)
    W = config.width
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = (torch.randn(n, k, generator=g, device=device) * gain * k ** -0.5).to(dtype)

    def vec(name, n, mean=0.0, std=0.05):
        t[name] = (mean + torch.randn(n, generator=g, device=device) * std).to(dtype)

    t["embed"] = torch.randn(config.vocab, W, generator=g, device=device).to(dtype)
    for i, lay in enumerate(config.layers):
        m, p = lay["mixer"], f"l{i}.mix"
        vec(f"l{i}.norm1", W)
        vec(f"l{i}.norm1b", W)
        if lay["type"] == "attention":
            H, dk = m["heads"], m["dim"]
            G, dv = m.get("kv_heads", H), m.get("vdim", dk)
            lin(f"{p}.q", H * dk, W)
            lin(f"{p}.k", G * dk, W)
            lin(f"{p}.v", G * dv, W)
            vec(f"{p}.q.norm", dk, 1.0)
            vec(f"{p}.k.norm", dk, 1.0)
            if m.get("v_mix"):
                t[f"{p}.vmix"] = torch.full((), 0.5, device=device).to(dtype)
            lin(f"{p}.o", W, H * dv)
        else:
            H, d = m["heads"], m["dim"]
            for s in ("r", "k", "v", "g", "w"):
                t[f"{p}.mu.{s}"] = torch.rand(W, generator=g, device=device).to(dtype)
            for s in ("r", "k", "v", "g"):
                lin(f"{p}.{s}", H * d, W)
            lin(f"{p}.w1", decay_rank, W)
            lin(f"{p}.w2", H * d, decay_rank)
            vec(f"{p}.w0", H * d, -1.0, 1.0)
            t[f"{p}.u"] = (torch.randn(H, d, generator=g, device=device) * 0.3).to(dtype)
            vec(f"{p}.norm", H * d, 1.0)
            lin(f"{p}.o", W, H * d)
        f = lay.get("mlp")
        if not f:
            continue
        vec(f"l{i}.norm2", W)
        vec(f"l{i}.norm2b", W)
        q = f"l{i}.mlp"
        if f["kind"] == "dense":
            for n_, (o_, i_) in (("gate", (f["ff"], W)), ("up", (f["ff"], W)), ("down", (W, f["ff"]))):
                lin(f"{q}.{n_}", o_, i_)
        else:
            for e in range(f["router"]["experts"]):
                lin(f"{q}.e{e}.gate", f["expert"]["ff"], W)
                lin(f"{q}.e{e}.up", f["expert"]["ff"], W)
                lin(f"{q}.e{e}.down", W, f["expert"]["ff"])
            lin(f"{q}.router", f["router"]["experts"], W)
            if f.get("shared"):
                lin(f"{q}.shared.gate", f["shared"]["ff"], W)
                lin(f"{q}.shared.up", f["shared"]["ff"], W)
                lin(f"{q}.shared.down", W, f["shared"]["ff"])
                lin(f"{q}.shared.sg", 1, W)
    vec("final.norm", W)
    lin("head", config.vocab, W)
    return t


def senadra_tensors(config, seed: int, device="cpu", dtype=torch.bfloat16, low_rank: int = 64) -> Dict[str, torch.Tensor]:
    """Seeded full Senadra checkpoint in the family's tensor naming for a `SenadraConfig`: N(0, 1 / fan_in) projections, gains
    around one, decays spread over (0, 1), mild distance biases."""
    g = torch.Generator(device=device).manual_seed(seed)
    W = config.width
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = (torch.randn(n, k, generator=g, device=device) * gain * k ** -0.5).to(dtype)

    def vec(name, n, mean=0.0, std=0.05):
        t[name] = (mean + torch.randn(n, generator=g, device=device) * std).to(dtype)

    t["embed"] = torch.randn(config.vocab, W, generator=g, device=device).to(dtype)
    side = config.side_dim
    if side:
        t["side.embed"] = torch.randn(config.vocab, side * len(config.layers), generator=g, device=device).to(dtype)
    for i, lay in enumerate(config.layers):
        m, p = lay["mixer"], f"l{i}.mix"
        vec(f"l{i}.norm1", W, 1.0)
        if lay["type"] == "attention":
            H, dk = m["heads"], m["dim"]
            G, dv = m.get("kv_heads", H), m.get("vdim", dk)
            lin(f"{p}.q", H * dk, W)
            if m.get("kv_from") is None:
                lin(f"{p}.k", G * dk, W)
                lin(f"{p}.v", G * dv, W)
            t[f"{p}.r1"] = (torch.rand(H, generator=g, device=device) * 0.5).to(dtype)
            t[f"{p}.r2"] = (torch.rand(H, generator=g, device=device) * 0.2).to(dtype)
            lin(f"{p}.g", H * dv, W)
            lin(f"{p}.o", W, H * dv)
        elif lay["type"] == "latent_attention":
            H, dn, dr, dv, rk, rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            lin(f"{p}.dq", rq, W)
            vec(f"{p}.dq.norm", rq, 1.0)
            lin(f"{p}.uq", H * (dn + dr), rq)
            lin(f"{p}.dkv", rk + dr, W)
            vec(f"{p}.dkv.norm", rk, 1.0)
            lin(f"{p}.uk", H * dn, rk)
            lin(f"{p}.uv", H * dv, rk)
            lin(f"{p}.g", H * dv, W)
            lin(f"{p}.o", W, H * dv)
        else:
            H, dk, dv, taps = m["heads"], m["dim"], m.get("vdim", m["dim"]), m["conv"]
            G = m.get("kv_heads", H)
            for n_, c_ in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                lin(f"{p}.{n_}", c_, W)
                t[f"{p}.{n_}.conv"] = (torch.randn(c_, taps, generator=g, device=device) * 0.5).to(dtype)
            lin(f"{p}.b", H, W)
            t[f"{p}.A_log"] = torch.log(torch.rand(H, generator=g, device=device) * 2.0 + 0.2).to(dtype)
            vec(f"{p}.norm", dv, 1.0)
            lin(f"{p}.a1", low_rank, W)
            lin(f"{p}.a2", H * dk, low_rank)
            vec(f"{p}.dt_bias", H * dk, -1.0, 1.0)
            lin(f"{p}.g1", low_rank, W)
            lin(f"{p}.g2", H * dv, low_rank)
            lin(f"{p}.o", W, H * dv)
        f = lay.get("mlp")
        if f:
            vec(f"l{i}.norm2", W, 1.0)
            lin(f"l{i}.mlp.up", f["ff"], W)
            lin(f"l{i}.mlp.down", W, f["ff"])
            t[f"l{i}.mlp.act"] = torch.tensor([0.3, -0.4], device=device).to(dtype)
        if side:
            lin(f"l{i}.side.gate", side, W)
            lin(f"l{i}.side.proj", W, side)
            vec(f"l{i}.side.norm", W, 1.0)
    vec("final.norm", W, 1.0)
    lin("head", config.vocab, W)
    return t


def mananex_tensors(config, seed: int, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Seeded full Mananex checkpoint in the family's tensor naming for a `MananexConfig`: N(0, 1 / fan_in) projections, norm
    gains around zero (offsets from one), lower bounds of the forget gates spread over (0, 1), depth-mix coefficients that
    weigh the newest entry most."""
    g = torch.Generator(device=device).manual_seed(seed)
    W = config.width
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = (torch.randn(n, k, generator=g, device=device) * gain * k ** -0.5).to(dtype)

    def vec(name, n, mean=0.0, std=0.05):
        t[name] = (mean + torch.randn(n, generator=g, device=device) * std).to(dtype)

    t["embed"] = torch.randn(config.vocab, W, generator=g, device=device).to(dtype)
    for i, lay in enumerate(config.layers):
        m = lay["mixer"]
        vec(f"l{i}.norm1", W)
        a, p = m["left"], f"l{i}.mix.left"
        H, dk = a["heads"], a["dim"]
        G, dv = a.get("kv_heads", H), a.get("vdim", dk)
        lin(f"{p}.q", H * dk, W)
        lin(f"{p}.k", G * dk, W)
        lin(f"{p}.v", G * dv, W)
        vec(f"{p}.sink", H, 0.0, 1.0)
        lin(f"{p}.g", H, W)
        lin(f"{p}.o", W, H * dv)
        r, p = m["right"], f"l{i}.mix.right"
        Hr, dkr, dvr = r["heads"], r["dim"], r.get("vdim", r["dim"])
        lin(f"{p}.q", Hr * dkr, W)
        lin(f"{p}.f", Hr * dkr, W)
        vec(f"{p}.f.b", Hr * dkr, 0.5, 1.0)
        t[f"{p}.lower"] = (torch.rand(Hr * dkr, generator=g, device=device) * 0.9).to(dtype)
        lin(f"{p}.v", Hr * dvr, W)
        vec(f"{p}.norm", dvr, 1.0)
        lin(f"{p}.o", W, Hr * dvr)
        lin(f"l{i}.rg1", W, W)
        vec(f"l{i}.rg1.b", W, 0.5, 0.5)
        f = lay.get("mlp")
        if f:
            q = f"l{i}.mlp"
            lin(f"l{i}.rg2", W, W)
            vec(f"l{i}.rg2.b", W, 0.5, 0.5)
            if f["kind"] == "dense":
                for n_, (o_, i_) in (("gate", (f["ff"], W)), ("up", (f["ff"], W)), ("down", (W, f["ff"]))):
                    lin(f"{q}.{n_}", o_, i_)
                    vec(f"{q}.{n_}.b", o_, 0.0, 0.1)
            else:
                for e in range(f["router"]["experts"]):
                    lin(f"{q}.e{e}.gate", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.up", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.down", W, f["expert"]["ff"])
                lin(f"{q}.router", f["router"]["experts"], W)
                vec(f"{q}.router.b", f["router"]["experts"], 0.0, 0.5)
        c = torch.randn(i + 2, generator=g, device=device) * (0.3 / (i + 2))
        c[-1] += 0.9
        t[f"l{i}.dwa"] = c.to(dtype)
    vec("final.norm", W)
    return t


def tatevik_tensors(config, seed: int, device="cpu", dtype=torch.bfloat16, decay_rank: int = 64) -> Dict[str, torch.Tensor]:
    """Seeded full Tatevik checkpoint in the family's tensor naming for a `TatevikConfig`: N(0, 1 / fan_in) projections, norm
    gains around one, sublayer scales around 0.5, head-mixing matrices near the identity, step sizes and decays in the range a
    trained model of the kind uses."""
    g = torch.Generator(device=device).manual_seed(seed)
    W = config.width
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = (torch.randn(n, k, generator=g, device=device) * gain * k ** -0.5).to(dtype)

    def vec(name, n, mean=0.0, std=0.05):
        t[name] = (mean + torch.randn(n, generator=g, device=device) * std).to(dtype)

    taps = config.canon_taps
    t["embed"] = torch.randn(config.vocab, W, generator=g, device=device).to(dtype)
    if config.loop:
        lin("loop.in", W, 2 * W)
        vec("loop.step", int(config.loop["times"]) * W, 0.0, 0.1)
        t["loop.step"] = t["loop.step"].view(-1, W)
    for i, lay in enumerate(config.layers):
        m, p = lay["mixer"], f"l{i}.mix"
        vec(f"l{i}.norm1", W, 1.0)
        vec(f"l{i}.ls1", W, 0.5, 0.1)
        if taps:
            t[f"l{i}.canon1"] = (torch.randn(W, taps, generator=g, device=device) * 0.3).to(dtype)
        if lay["type"] == "mamba1":
            inner, N, R, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            lin(f"{p}.in", 2 * inner, W)
            t[f"{p}.conv"] = (torch.randn(inner, K, generator=g, device=device) * 0.4).to(dtype)
            vec(f"{p}.conv.b", inner, 0.0, 0.1)
            lin(f"{p}.x", R + 2 * N, inner)
            lin(f"{p}.dt", inner, R)
            vec(f"{p}.dt.b", inner, -2.0, 1.0)
            t[f"{p}.A_log"] = torch.log(torch.rand(inner, N, generator=g, device=device) * 8 + 0.5).to(dtype)
            vec(f"{p}.D", inner, 1.0, 0.2)
            lin(f"{p}.o", W, inner)
        elif lay["type"] == "parallel":
            a, q = m["left"], f"{p}.left"
            H, dk = a["heads"], a["dim"]
            G, dv = a.get("kv_heads", H), a.get("vdim", dk)
            for n_, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                lin(f"{q}.{n_}", rows, W)
                vec(f"{q}.{n_}.b", rows, 0.0, 0.1)
            t[f"{q}.talk"] = (torch.eye(H, device=device) + torch.randn(H, H, generator=g, device=device) * (0.5 / H)).to(dtype)
            lin(f"{q}.g", H * dv, W)
            lin(f"{q}.o", W, H * dv)
            vec(f"{q}.o.b", W, 0.0, 0.1)
            r, q = m["right"], f"{p}.right"
            Hr, dkr, dvr = r["heads"], r["dim"], r.get("vdim", r["dim"])
            lin(f"{q}.q", Hr * dkr, W)
            lin(f"{q}.k", Hr * dkr, W)
            lin(f"{q}.v", Hr * dvr, W)
            lin(f"{q}.g", Hr * dvr, W)
            lin(f"{q}.o", W, Hr * dvr)
            vec(f"{q}.norm", Hr * dvr, 1.0)
            vec(f"{p}.left.out", W, 1.0)
            vec(f"{p}.right.out", W, 1.0)
        else:
            H, dk, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
            lin(f"{p}.q", H * dk, W)
            lin(f"{p}.k", H * dk, W)
            lin(f"{p}.v", H * dv, W)
            lin(f"{p}.g", H * dv, W)
            lin(f"{p}.o", W, H * dv)
            vec(f"{p}.norm", dv, 1.0)
            lin(f"{p}.a1", decay_rank, W)
            lin(f"{p}.a2", H * dk, decay_rank)
            vec(f"{p}.a2.b", H * dk, 3.0, 1.0)
        f = lay.get("mlp")
        if f:
            q = f"l{i}.mlp"
            vec(f"l{i}.ls2", W, 0.5, 0.1)
            if taps:
                t[f"l{i}.canon2"] = (torch.randn(W, taps, generator=g, device=device) * 0.3).to(dtype)
            if f["kind"] == "dense":
                lin(f"{q}.up", f["ff"], W)
                lin(f"{q}.down", W, f["ff"])
                t[f"{q}.act"] = torch.tensor([0.9, 0.3, -0.1, 0.05], device=device).to(dtype)
            else:
                E = f["router"]["experts"]
                for e in range(E):
                    lin(f"{q}.e{e}.gate", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.up", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.down", W, f["expert"]["ff"])
                lin(f"{q}.router", E, W)
                vec(f"{q}.correction", E, 0.0, 0.05)
    vec("final.norm", W, 1.0)
    lin("head", config.vocab, W)
    return t
