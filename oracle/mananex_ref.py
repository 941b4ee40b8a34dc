"""Plain CPU restatement of the Mananex decoder, one function per mechanism.  TEST INFRASTRUCTURE ONLY: nothing of the
serving path imports this file and it imports nothing of the serving path.

Mananex is a stack of PARALLEL layers over an fp32 residual stream.  With h = N(x), N(z) = z / sqrt(mean(z^2) + eps) * (1 + w),
a layer computes
    y = x + sigmoid(R1 h + b1) * mixer(h) + sigmoid(R2 h + b2) * ff(h)          (one norm, both sublayers read it; gated residual)
and hands on a learned mix over depth of everything computed so far,
    x' = sum_{j <= i + 1} a_i[j] Y_j,        Y_0 = the embedding output, Y_(j+1) = layer j's y.
The mixer runs two mixers side by side on the same h and adds them with two fixed weights:
  * left: GQA softmax attention with an interleaved-pair rotation of the first `rot.dims` channels, a sliding window that
    also keeps the first `keep_first` positions of the sequence, one learned sink logit per head in the softmax denominator,
    and one sigmoid output gate per head;
  * right: an HGRN2-style gated linear recurrence, S <- diag(f) S + (1 - f) v^T, o = S^T q with q = silu(W_q h) and a forget
    gate bounded below, f = l + (1 - l) sigmoid(W_f h + b); per-head RMS norm of o with a gain shared by the heads.
The feed-forward is a SiLU gated unit with biases, or a mixture of bias-free SiLU gated experts: the top-k router logits
(with a bias) are softmaxed among themselves.  The head is the embedding table.

All arithmetic is in `DT` (float64) on the CPU; weights are taken as stored.  A sequence is processed whole (`forward`) or
in any portions through an explicit per-sequence state (`new_state` / `advance`)."""
from typing import Dict, List, Optional

import torch

DT = torch.float64


def rms_unit(z: torch.Tensor, eps: float) -> torch.Tensor:
    return z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)


def offset_norm(z, w, eps: float):
    """RMS norm whose stored gain is an offset from one."""
    return rms_unit(z, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def rotate_pairs(x, pos, base: float, dims: int):
    """x [T, heads, D]: channels (2i, 2i + 1), 2i + 1 < dims, turn by pos * base^(-2i / dims); the rest pass."""
    if not dims:
        return x
    i = torch.arange(dims // 2, dtype=DT)
    ang = pos.to(DT)[:, None] * base ** (-2.0 * i / dims)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(pos, n_keys: int, window: Optional[int], keep_first: int):
    """[T, n_keys] bool: key j is seen from position i iff j <= i and (i - j < window or j < keep_first)."""
    j = torch.arange(n_keys)[None, :]
    i = pos[:, None]
    ok = j <= i
    if window:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def sink_softmax(s, sink):
    """softmax over the last axis whose denominator also holds exp(sink): a slot without key or value.  s may hold -inf."""
    m = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - m))


def window_sink_attention(h, pos, p: Dict[str, torch.Tensor], m: dict, past_k=None, past_v=None):
    """h [T, W] at positions pos.  past_k [P, G, dk] (rotated), past_v [P, G, dv].  Returns (out [T, W], keys, values)."""
    H, dk = m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", dk)
    T = h.shape[0]
    rot = m.get("rot") or {}
    rd, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
    q = rotate_pairs((h @ p["q"].T).view(T, H, dk), pos, base, rd)
    k = rotate_pairs((h @ p["k"].T).view(T, G, dk), pos, base, rd)
    v = (h @ p["v"].T).view(T, G, dv)
    if past_k is not None:
        k, v = torch.cat([past_k, k], 0), torch.cat([past_v, v], 0)
    mask = m.get("mask") or {}
    ok = visible(pos, k.shape[0], mask.get("size"), int(mask.get("keep_first", 0)))
    out = torch.zeros(T, H, dv, dtype=DT)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~ok, float("-inf"))
        if "sink" in p:
            w = sink_softmax(s, p["sink"][hd])
        else:
            w = torch.softmax(s, -1)
        out[:, hd] = w @ v[:, g]
    if "g" in p:
        out = out * torch.sigmoid(h @ p["g"].T)[:, :, None]
    return out.reshape(T, H * dv) @ p["o"].T, k, v


# when a list: gated_linear_recurrence appends, per token, the smallest |S^T q| / (|S|^T |q|) over the heads: how much of the
# read-out is left after its terms cancel (the per-head norm that follows divides by it)
READOUT_CONDITION = None


def forget_gate(z, lower):
    """f = l + (1 - l) sigmoid(z): a forget gate that cannot fall below l."""
    return lower + (1.0 - lower) * torch.sigmoid(z)


def gated_linear_recurrence(q, f, v, S):
    """q, f [T, H, dk]; v [T, H, dv]; S [H, dk, dv].  S <- diag(f) S + (1 - f) v^T;  o = S^T q (the new state is read)."""
    out = torch.zeros_like(v)
    for t in range(q.shape[0]):
        S = S * f[t][:, :, None] + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
        if READOUT_CONDITION is not None:
            bound = torch.einsum("hkv,hk->hv", S.abs(), q[t].abs())
            READOUT_CONDITION.append(float((out[t].norm(dim=-1) / bound.norm(dim=-1).clamp_min(1e-300)).min()))
    return out, S


def hgrn_mixer(h, p: Dict[str, torch.Tensor], m: dict, eps: float, S=None):
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    if S is None:
        S = torch.zeros(H, dk, dv, dtype=DT)
    q = silu(h @ p["q"].T).view(T, H, dk)
    f = forget_gate(h @ p["f"].T + p["f.b"], p["lower"]).view(T, H, dk)
    v = (h @ p["v"].T).view(T, H, dv)
    o, S = gated_linear_recurrence(q, f, v, S)
    o = rms_unit(o, eps) * p["norm"]
    return o.reshape(T, H * dv) @ p["o"].T, S


def gated_unit(h, p, prefix=""):
    g = h @ p[prefix + "gate"].T
    u = h @ p[prefix + "up"].T
    if prefix + "gate.b" in p:
        g, u = g + p[prefix + "gate.b"], u + p[prefix + "up.b"]
    y = (silu(g) * u) @ p[prefix + "down"].T
    return y + p[prefix + "down.b"] if prefix + "down.b" in p else y


# when a list: route_top_softmax appends, per call, the smallest gap between a chosen and an unchosen logit (how close the
# routing of these tokens is to falling the other way)
ROUTER_MARGINS = None


def route_top_softmax(h, p, top: int):
    """(indices [T, top], weights [T, top]): the largest logits, softmaxed among themselves."""
    z = h @ p["router"].T + p["router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    if ROUTER_MARGINS is not None and top < z.shape[-1]:
        ROUTER_MARGINS.append(float((val[:, -1] - torch.topk(z, top + 1, dim=-1).values[:, -1]).min()))
    return idx, torch.softmax(val, -1)


def clear_cut_tokens(config, tensors, n: int, seed: int, margin: float = 0.3, condition: float = 0.1) -> List[int]:
    """n random tokens, each drawn again until no router of the model is within `margin` of choosing other experts for it and
    no head's read-out of the recurrence cancels to less than `condition` of its terms before it is normed: what a
    reduced-precision run computes for them differs from this restatement by rounding, not by a decision or a division that
    rounding tips."""
    global ROUTER_MARGINS, READOUT_CONDITION
    g = torch.Generator().manual_seed(seed)
    state, toks = new_state(config), []
    try:
        while len(toks) < n:
            for _ in range(50):
                t = int(torch.randint(0, config["vocab"], (1,), generator=g))
                trial = {"len": state["len"], "layers": list(state["layers"])}
                ROUTER_MARGINS, READOUT_CONDITION = [], []
                advance(config, tensors, [t], trial)
                if all(m >= margin for m in ROUTER_MARGINS) and all(c >= condition for c in READOUT_CONDITION):
                    break
            state = trial
            toks.append(t)
    finally:
        ROUTER_MARGINS = READOUT_CONDITION = None
    return toks


def expert_mixture(h, p, f: dict):
    idx, w = route_top_softmax(h, p, int(f["router"]["top"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            out[t] += we * gated_unit(h[t:t + 1], p, f"e{e}.")[0]
    return out


def feed_forward(h, p, f: Optional[dict]):
    if not f:
        return None
    return gated_unit(h, p) if f["kind"] == "dense" else expert_mixture(h, p, f)


def residual_gate(h, tensors, name: str):
    return torch.sigmoid(h @ tensors[name].to(DT).T + tensors[name + ".b"].to(DT))


def layer_params(tensors, i: int, part: str) -> Dict[str, torch.Tensor]:
    pre = f"l{i}.{part}."
    return {k[len(pre):]: v.to(DT) for k, v in tensors.items() if k.startswith(pre)}


def sub_params(p: Dict[str, torch.Tensor], part: str) -> Dict[str, torch.Tensor]:
    return {k[len(part) + 1:]: v for k, v in p.items() if k.startswith(part + ".")}


def new_state(config: dict) -> dict:
    return {"len": 0, "layers": [None] * len(config["layers"])}


def advance(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], state: dict, trace: Optional[list] = None):
    """Feed `tokens` after what `state` holds; returns logits [T, vocab]."""
    eps = config["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    T = len(tokens)
    pos = torch.arange(state["len"], state["len"] + T)
    x = tensors["embed"].to(DT)[tok]
    history = [x]
    for i, lay in enumerate(config["layers"]):
        if lay["type"] != "parallel":
            raise ValueError(lay["type"])
        m = lay["mixer"]
        st = state["layers"][i] or {}
        p = layer_params(tensors, i, "mix")
        h = offset_norm(x, tensors[f"l{i}.norm1"].to(DT), eps)
        left, k, v = window_sink_attention(h, pos, sub_params(p, "left"), m["left"], st.get("k"), st.get("v"))
        right, S = hgrn_mixer(h, sub_params(p, "right"), m["right"], eps, st.get("S"))
        state["layers"][i] = {"k": k, "v": v, "S": S}
        y = x + residual_gate(h, tensors, f"l{i}.rg1") * (m["left_scale"] * left + m["right_scale"] * right)
        ff = feed_forward(h, layer_params(tensors, i, "mlp"), lay.get("mlp"))
        if ff is not None:
            y = y + residual_gate(h, tensors, f"l{i}.rg2") * ff
        history.append(y)
        a = tensors[f"l{i}.dwa"].to(DT)
        x = sum(a[j] * history[j] for j in range(i + 2))
        if trace is not None:
            trace.append(x.clone())
    state["len"] += T
    return offset_norm(x, tensors["final.norm"].to(DT), eps) @ tensors["embed"].to(DT).T


def forward(config, tensors, tokens, trace=None):
    return advance(config, tensors, tokens, new_state(config), trace)
