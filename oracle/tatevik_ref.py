"""Plain CPU restatement of the Tatevik decoder, one function per mechanism.  TEST INFRASTRUCTURE ONLY: nothing of the
serving path imports this file and it imports nothing of the serving path.

Tatevik is a stack of PARALLEL layers over an fp32 residual stream.  With h = LN(x) (mean-free, unit variance, a gain and no
bias) a layer computes
    x <- x + s1 * mixer(h + C1(h)) + s2 * ff(h + C2(h))
where s1, s2 are learned per-channel scales and C1, C2 short causal per-channel convolutions over time.  A run of layers may be
repeated (`loop`): every pass has caches and states of its own, starts from x <- W_in [x; x0] + step[pass] with x0 the scaled
embedding, and shares the layers' weights with the other passes.  Mixers:
  * mamba1    a selective state-space scan (input-dependent step size, diagonal transition, per-channel state vectors);
  * parallel  windowed GQA softmax attention whose scores are mixed over the heads before the softmax (left) beside a linear
              attention with one fixed decay per head (right); each result is RMS-normed over the width, then they are averaged;
  * gla       linear attention with a learned decay per key channel.
Feed-forwards: W_down P(W_up h) with P a polynomial of unit-RMS powers, or a mixture of SiLU gated experts chosen among the
best groups of neighbouring experts by softmax scores plus a correction, weighted by the uncorrected scores.

All arithmetic is in `DT` (float64) on the CPU; weights are taken as stored.  A sequence is processed in any portions through
an explicit per-sequence state (`new_state` / `advance`); `forward` is one portion from an empty state."""
import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


# ---- small pieces ---------------------------------------------------------------------------------------------------------
def rms_unit(z, eps: float):
    return z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)


def layer_norm(z, w, eps: float):
    d = z - z.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def causal_conv(x, w, tail, bias=None):
    """x [T, C], w [C, taps] (last column = the current token), tail [taps - 1, C] = the inputs before x (zeros at a
    sequence's start).  Returns (y [T, C], the new tail)."""
    taps = w.shape[1]
    full = torch.cat([tail, x], 0)
    T = x.shape[0]
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + full[j:j + T] * w[:, j]
    if bias is not None:
        y = y + bias
    return y, full[full.shape[0] - (taps - 1):] if taps > 1 else full[:0]


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


# ---- mixers ---------------------------------------------------------------------------------------------------------------
def selective_scan_mixer(h, p: Dict[str, torch.Tensor], m: dict, st: dict):
    """st: {"S": [inner, state], "tail": [conv - 1, inner]}."""
    inner, N, R = int(m["inner"]), int(m["state"]), int(m["dt_rank"])
    xz = h @ p["in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x, st["tail"] = causal_conv(x, p["conv"], st["tail"], p["conv.b"])
    x = silu(x)
    low = x @ p["x"].T
    dt = softplus(low[:, :R] @ p["dt"].T + p["dt.b"])
    Bm, Cm = low[:, R:R + N], low[:, R + N:R + 2 * N]
    A = -torch.exp(p["A_log"])
    S = st["S"]
    ys = []
    for t in range(h.shape[0]):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * Bm[t][None, :]
        ys.append(S @ Cm[t] + p["D"] * x[t])
    st["S"] = S
    y = torch.stack(ys) * silu(z)
    return y @ p["o"].T


def mixed_head_attention(h, pos, p: Dict[str, torch.Tensor], m: dict, eps: float, st: dict):
    """st: {"k": [n, G, dk], "v": [n, G, dv]} of the positions before this portion."""
    H, dk = int(m["heads"]), int(m["dim"])
    G, dv = int(m.get("kv_heads", H)), int(m.get("vdim", dk))
    T = h.shape[0]
    q = (h @ p["q"].T + p["q.b"]).view(T, H, dk)
    k = (h @ p["k"].T + p["k.b"]).view(T, G, dk)
    v = (h @ p["v"].T + p["v.b"]).view(T, G, dv)
    rot = m.get("rot") or {}
    q = rotate_pairs(q, pos, float(rot.get("base", 10000.0)), int(rot.get("dims", 0)))
    k = rotate_pairs(k, pos, float(rot.get("base", 10000.0)), int(rot.get("dims", 0)))
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    st["k"], st["v"] = torch.cat([st["k"], k], 0), torch.cat([st["v"], v], 0)
    window = int((m.get("mask") or {}).get("size", 0))
    o = attend_mixed(q, st["k"], st["v"], pos, p["talk"], float(m["scale"]), window).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T + p["o.b"]


def attend_mixed(q, K, V, pos, talk, scale: float, window: int):
    """q [T, H, dk] at positions pos; K [n, G, dk], V [n, G, dv] of positions 0 .. n - 1.  The scaled scores of the H heads are
    mixed by talk [H, H] before the softmax over the visible keys (j <= i, and i - j < window if window).  -> [T, H, dv]."""
    H, G, n = q.shape[1], K.shape[1], K.shape[0]
    grp = torch.arange(H) // (H // G)
    raw = torch.einsum("thd,nhd->htn", q, K[:, grp]) * scale  # [H, T, n]
    mixed = torch.einsum("hg,gtn->htn", talk, raw)
    j = torch.arange(n)[None, :]
    i = pos[:, None]
    ok = (j <= i)
    if window:
        ok = ok & (i - j < window)
    mixed = mixed.masked_fill(~ok[None], float("-inf"))
    w = torch.softmax(mixed, -1)
    return torch.einsum("htn,nhd->thd", w, V[:, grp])


# When these are lists, route() appends how far each token is from another choice of experts and linear_attention() how much of
# a read-out's terms survive their cancellation (clear_cut_tokens uses them to draw prompts that rounding cannot tip).
ROUTER_MARGINS: Optional[list] = None
READOUT_CONDITION: Optional[list] = None


def linear_attention(q, k, v, decay, S, S_abs=None):
    """S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head.  q, k [T, H, dk], v [T, H, dv], decay [T, H, dk]
    (broadcastable), S [H, dk, dv].  Returns (o [T, H, dv], S)."""
    outs = []
    for t in range(q.shape[0]):
        S = decay[t][..., None] * S + k[t][..., None] * v[t][:, None, :]
        o = torch.einsum("hkv,hk->hv", S, q[t])
        outs.append(o)
        if READOUT_CONDITION is not None and S_abs is not None:
            S_abs[0] = decay[t][..., None] * S_abs[0] + k[t].abs()[..., None] * v[t].abs()[:, None, :]
            terms = torch.einsum("hkv,hk->hv", S_abs[0], q[t].abs())
            READOUT_CONDITION.append(float((o.norm(dim=-1) / terms.norm(dim=-1).clamp_min(1e-300)).min()))
    return torch.stack(outs), S


def fixed_decay_attention(h, p, m: dict, eps: float, st: dict):
    """q, k, v through SiLU; one decay per head; the heads' read-outs normed together, gated by a sigmoid."""
    H, dk = int(m["heads"]), int(m["dim"])
    dv = int(m.get("vdim", dk))
    T = h.shape[0]
    q = silu(h @ p["q"].T).view(T, H, dk)
    k = silu(h @ p["k"].T).view(T, H, dk)
    v = silu(h @ p["v"].T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=DT).view(1, H, 1).expand(T, H, dk)
    o, st["S"] = linear_attention(q, k, v, decay, st["S"], st.setdefault("S_abs", [torch.zeros_like(st["S"])]))
    o = rms_unit(o.reshape(T, H * dv), eps) * p["norm"] * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T


def side_by_side(h, pos, p, m: dict, eps: float, st: dict):
    left = mixed_head_attention(h, pos, {k[5:]: v for k, v in p.items() if k.startswith("left.")}, m["left"], eps, st["left"])
    right = fixed_decay_attention(h, {k[6:]: v for k, v in p.items() if k.startswith("right.")}, m["right"], eps, st["right"])
    return 0.5 * (rms_unit(left, eps) * p["left.out"] + rms_unit(right, eps) * p["right.out"])


def channel_decay_attention(h, p, m: dict, eps: float, st: dict):
    """Linear attention with a decay per key channel, sigmoid(z)^(1 / tau); per-head norm; SiLU gate."""
    H, dk = int(m["heads"]), int(m["dim"])
    dv = int(m.get("vdim", dk))
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ p["k"].T).view(T, H, dk)
    v = (h @ p["v"].T).view(T, H, dv)
    z = (h @ p["a1"].T) @ p["a2"].T + p["a2.b"]
    decay = torch.exp(torch.nn.functional.logsigmoid(z) / float(m["tau"])).view(T, H, dk)
    o, st["S"] = linear_attention(q, k, v, decay, st["S"], st.setdefault("S_abs", [torch.zeros_like(st["S"])]))
    o = (rms_unit(o, eps) * p["norm"]).reshape(T, H * dv) * silu(h @ p["g"].T)
    return o @ p["o"].T


# ---- feed-forwards --------------------------------------------------------------------------------------------------------
def power_norm_mlp(h, p, eps: float):
    z = h @ p["up"].T
    a, b, c, e = [float(x) for x in p["act"]]
    act = a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e
    return act @ p["down"].T


def route(h, p, r: dict):
    """(chosen [T, top], weights [T, top], scores [T, E], choice scores with excluded groups at -inf)."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(h @ p["router"].T, -1)
    c = s + p["correction"]
    groups = r.get("groups") or {}
    count, keep = int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1)))
    if count > 1 and keep < count:
        best = c.view(-1, count, E // count).max(-1).values
        if ROUTER_MARGINS is not None:
            b = best.sort(-1, descending=True).values
            ROUTER_MARGINS.extend((b[:, keep - 1] - b[:, keep]).tolist())
        kept = best.topk(keep, -1).indices
        allow = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        c = c.masked_fill(~allow[:, :, None].expand(-1, -1, E // count).reshape(-1, E), float("-inf"))
    if ROUTER_MARGINS is not None and top < E:
        b = c.sort(-1, descending=True).values
        ROUTER_MARGINS.extend(float(x) for x in (b[:, top - 1] - b[:, top]).tolist() if x == x and x != float("inf"))
    idx = c.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20), s, c


def expert_mixture(h, p, f: dict):
    idx, w, _, _ = route(h, p, f["router"])
    out = torch.zeros(h.shape[0], p["e0.down"].shape[0], dtype=DT)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            y = (silu(h[t] @ p[f"e{e}.gate"].T) * (h[t] @ p[f"e{e}.up"].T)) @ p[f"e{e}.down"].T
            out[t] += we * y
    return out


# ---- the model ------------------------------------------------------------------------------------------------------------
def layer_runs(config: dict) -> List[tuple]:
    """[(layer index, pass number or None, first of its pass)] in execution order."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    return runs + [(i, None, False) for i in range(b, n)]


class TatevikRef:
    def __init__(self, config: dict, tensors: Dict[str, torch.Tensor]):
        self.c = config
        self.t = {k: v.to(DT) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])
        self.W = int(config["width"])
        self.taps = int((config.get("canon") or {}).get("taps", 0))
        self.runs = layer_runs(config)

    def sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {k[len(prefix):]: v for k, v in self.t.items() if k.startswith(prefix)}

    def new_state(self) -> dict:
        runs = []
        for i, _, _ in self.runs:
            lay = self.c["layers"][i]
            m = lay["mixer"]
            s = {"canon1": torch.zeros(max(self.taps - 1, 0), self.W, dtype=DT), "canon2": torch.zeros(max(self.taps - 1, 0), self.W, dtype=DT)}
            if lay["type"] == "mamba1":
                s["mix"] = {"S": torch.zeros(int(m["inner"]), int(m["state"]), dtype=DT), "tail": torch.zeros(int(m["conv"]) - 1, int(m["inner"]), dtype=DT)}
            elif lay["type"] == "parallel":
                l, r = m["left"], m["right"]
                G = int(l.get("kv_heads", l["heads"]))
                s["mix"] = {"left": {"k": torch.zeros(0, G, int(l["dim"]), dtype=DT), "v": torch.zeros(0, G, int(l.get("vdim", l["dim"])), dtype=DT)},
                            "right": {"S": torch.zeros(int(r["heads"]), int(r["dim"]), int(r.get("vdim", r["dim"])), dtype=DT)}}
            elif lay["type"] == "gla":
                s["mix"] = {"S": torch.zeros(int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), dtype=DT)}
            else:
                raise ValueError(lay["type"])
            runs.append(s)
        return {"runs": runs, "n": 0}

    def layer(self, i: int, x, pos, st: dict, parts: Optional[dict] = None):
        lay = self.c["layers"][i]
        t, eps = self.t, self.eps
        h = layer_norm(x, t[f"l{i}.norm1"], eps)
        h1 = h
        if self.taps:
            c1, st["canon1"] = causal_conv(h, t[f"l{i}.canon1"], st["canon1"])
            h1 = h + c1
        p = self.sub(f"l{i}.mix.")
        if lay["type"] == "mamba1":
            y = selective_scan_mixer(h1, p, lay["mixer"], st["mix"])
        elif lay["type"] == "parallel":
            y = side_by_side(h1, pos, p, lay["mixer"], eps, st["mix"])
        else:
            y = channel_decay_attention(h1, p, lay["mixer"], eps, st["mix"])
        out = x + y * t[f"l{i}.ls1"]
        f = lay.get("mlp")
        if parts is not None:
            parts.update(h=h, h1=h1, mixer=y)
        if f:
            h2 = h
            if self.taps:
                c2, st["canon2"] = causal_conv(h, t[f"l{i}.canon2"], st["canon2"])
                h2 = h + c2
            q = self.sub(f"l{i}.mlp.")
            ff = power_norm_mlp(h2, q, eps) if f["kind"] == "dense" else expert_mixture(h2, q, f)
            out = out + ff * t[f"l{i}.ls2"]
            if parts is not None:
                parts.update(h2=h2, ff=ff)
        return out

    def advance(self, state: dict, tokens: List[int], trace: Optional[list] = None) -> torch.Tensor:
        """Feeds the next tokens of a sequence; returns the logits [len(tokens), vocab]."""
        t = self.t
        n0 = state["n"]
        pos = torch.arange(n0, n0 + len(tokens))
        x0 = t["embed"][torch.tensor(tokens)] * float((self.c.get("embedding") or {}).get("scale", 1.0))
        x = x0
        for (i, number, first), st in zip(self.runs, state["runs"]):
            if first:
                x = torch.cat([x, x0], -1) @ t["loop.in"].T + t["loop.step"][number]
            x = self.layer(i, x, pos, st)
            if trace is not None:
                trace.append(x.clone())
        state["n"] = n0 + len(tokens)
        return layer_norm(x, t["final.norm"], self.eps) @ t["head"].T

    def forward(self, tokens: List[int], trace: Optional[list] = None) -> torch.Tensor:
        return self.advance(self.new_state(), tokens, trace)


def clear_cut_tokens(config: dict, tensors, n: int, seed: int, margin: float = 0.05, condition: float = 0.05) -> List[int]:
    """n random tokens, each drawn again until no router of the model is within `margin` (in score) of choosing other experts
    or groups for it and no read-out of a linear attention cancels to less than `condition` of its terms before it is normed:
    what a reduced-precision run computes for them differs from this restatement by rounding, not by a decision or a division
    that rounding tips."""
    import copy

    global ROUTER_MARGINS, READOUT_CONDITION
    g = torch.Generator().manual_seed(seed)
    ref = TatevikRef(config, tensors)
    state, toks = ref.new_state(), []
    try:
        while len(toks) < n:
            for _ in range(50):
                t = int(torch.randint(0, config["vocab"], (1,), generator=g))
                trial = copy.deepcopy(state)
                ROUTER_MARGINS, READOUT_CONDITION = [], []
                ref.advance(trial, [t])
                if all(m >= margin for m in ROUTER_MARGINS) and all(c >= condition for c in READOUT_CONDITION):
                    break
            state = trial
            toks.append(t)
    finally:
        ROUTER_MARGINS = READOUT_CONDITION = None
    return toks
