"""Seeded small Tatevik checkpoints for tests: a config dict and a {name: tensor} dict in the family's tensor naming.
Sizes are arguments; nothing here equals a published model.  TEST INFRASTRUCTURE ONLY."""
from typing import Dict, List, Optional

import torch


def scan_layer(inner=96, state=12, dt_rank=8, conv=4, mlp=None) -> dict:
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}, "mlp": mlp}


def attention_part(heads=6, kv_heads=3, dim=32, vdim=24, scale=0.3, window: Optional[int] = 40, rot_dims=16, rot_base=5000.0) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot_dims:
        m["rot"] = {"base": rot_base, "dims": rot_dims}
    return m


def fixed_decay_part(heads=3, dim=24, vdim=40, decay=(0.7, 0.93, 0.995)) -> dict:
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def pair_layer(left: Optional[dict] = None, right: Optional[dict] = None, mlp=None) -> dict:
    return {"type": "parallel", "mixer": {"left": left or attention_part(), "right": right or fixed_decay_part()}, "mlp": mlp}


def channel_decay_layer(heads=3, dim=24, vdim=40, tau=8.0, rank=8, mlp=None) -> dict:
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}, "mlp": mlp}


def dense_mlp(ff=104) -> dict:
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts=6, top=2, ff=40, groups=3, keep=2) -> dict:
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def make_config(layers: List[dict], width=72, vocab=112, eps=1e-5, taps=4, scale=0.7, loop: Optional[dict] = None) -> dict:
    c = {"architecture": "Tatevik", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps}, "embedding": {"scale": scale}}
    if taps:
        c["canon"] = {"taps": taps}
    if loop:
        c["loop"] = loop
    return c


def make_tensors(config: dict, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """N(0, 1 / fan_in) projections (wider for what feeds a softmax, a router or a gate), gains around one, sublayer scales
    around 0.5, head-mixing matrices near the identity.  Values are rounded to `dtype` (what a checkpoint stores)."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = torch.randn(n, k, generator=g) * gain * k ** -0.5

    def vec(name, n, mean=0.0, std=0.1):
        t[name] = mean + torch.randn(n, generator=g) * std

    taps = int((config.get("canon") or {}).get("taps", 0))
    t["embed"] = torch.randn(config["vocab"], W, generator=g)
    if config.get("loop"):
        lin("loop.in", W, 2 * W, 1.4)
        t["loop.step"] = torch.randn(int(config["loop"]["times"]), W, generator=g) * 0.3
    for i, lay in enumerate(config["layers"]):
        m, p = lay["mixer"], f"l{i}.mix"
        vec(f"l{i}.norm1", W, 1.0)
        vec(f"l{i}.ls1", W, 0.5, 0.2)
        if taps:
            t[f"l{i}.canon1"] = torch.randn(W, taps, generator=g) * 0.4
        if lay["type"] == "mamba1":
            inner, N, R, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            lin(f"{p}.in", 2 * inner, W)
            t[f"{p}.conv"] = torch.randn(inner, K, generator=g) * 0.5
            vec(f"{p}.conv.b", inner, 0.0, 0.2)
            lin(f"{p}.x", R + 2 * N, inner)
            lin(f"{p}.dt", inner, R, 2.0)
            vec(f"{p}.dt.b", inner, -1.0, 1.0)
            t[f"{p}.A_log"] = torch.log(torch.rand(inner, N, generator=g) * 4 + 0.05)
            vec(f"{p}.D", inner, 1.0, 0.3)
            lin(f"{p}.o", W, inner)
        elif lay["type"] == "parallel":
            a, q = m["left"], f"{p}.left"
            H, dk = a["heads"], a["dim"]
            G, dv = a.get("kv_heads", H), a.get("vdim", dk)
            for n_, rows, gain in (("q", H * dk, 2.0), ("k", G * dk, 2.0), ("v", G * dv, 1.0)):
                lin(f"{q}.{n_}", rows, W, gain)
                vec(f"{q}.{n_}.b", rows, 0.0, 0.3)
            t[f"{q}.talk"] = torch.eye(H) + torch.randn(H, H, generator=g) * 0.3
            lin(f"{q}.g", H * dv, W, 2.0)
            lin(f"{q}.o", W, H * dv)
            vec(f"{q}.o.b", W, 0.0, 0.2)
            r, q = m["right"], f"{p}.right"
            Hr, dkr, dvr = r["heads"], r["dim"], r.get("vdim", r["dim"])
            lin(f"{q}.q", Hr * dkr, W, 1.5)
            lin(f"{q}.k", Hr * dkr, W, 1.5)
            lin(f"{q}.v", Hr * dvr, W, 1.5)
            lin(f"{q}.g", Hr * dvr, W, 2.0)
            lin(f"{q}.o", W, Hr * dvr)
            vec(f"{q}.norm", Hr * dvr, 1.0)
            vec(f"{p}.left.out", W, 1.0)
            vec(f"{p}.right.out", W, 1.0)
        else:
            H, dk, dv, rank = m["heads"], m["dim"], m.get("vdim", m["dim"]), m.get("rank", 8)
            lin(f"{p}.q", H * dk, W)
            lin(f"{p}.k", H * dk, W)
            lin(f"{p}.v", H * dv, W)
            lin(f"{p}.g", H * dv, W, 2.0)
            lin(f"{p}.o", W, H * dv)
            vec(f"{p}.norm", dv, 1.0)
            lin(f"{p}.a1", rank, W, 2.0)
            lin(f"{p}.a2", H * dk, rank, 2.0)
            vec(f"{p}.a2.b", H * dk, 2.0, 1.5)
        f = lay.get("mlp")
        if f:
            q = f"l{i}.mlp"
            vec(f"l{i}.ls2", W, 0.5, 0.2)
            if taps:
                t[f"l{i}.canon2"] = torch.randn(W, taps, generator=g) * 0.4
            if f["kind"] == "dense":
                lin(f"{q}.up", f["ff"], W)
                lin(f"{q}.down", W, f["ff"])
                t[f"{q}.act"] = torch.tensor([0.9, 0.4, -0.2, 0.1]) + torch.randn(4, generator=g) * 0.1
            else:
                E = f["router"]["experts"]
                for e in range(E):
                    lin(f"{q}.e{e}.gate", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.up", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.down", W, f["expert"]["ff"], 2.0)
                lin(f"{q}.router", E, W, 1.5)
                vec(f"{q}.correction", E, 0.0, 0.15)
    vec("final.norm", W, 1.0)
    lin("head", config["vocab"], W)
    return {k: v.to(dtype) for k, v in t.items()}


def standard_layers() -> List[dict]:
    """Every mixer and feed-forward kind, a layer without a feed-forward, GQA and MHA, a window and none, full and partial
    rotation, states that are not a multiple of 8, one group of experts and several."""
    return [scan_layer(mlp=dense_mlp()),
            pair_layer(mlp=moe_mlp()),
            channel_decay_layer(mlp=None),
            pair_layer(left=attention_part(heads=4, kv_heads=4, dim=16, vdim=16, window=None, rot_dims=16),
                       right=fixed_decay_part(heads=2, dim=32, vdim=16, decay=(0.5, 0.99)), mlp=dense_mlp(ff=64)),
            scan_layer(inner=80, state=16, dt_rank=5, conv=2, mlp=moe_mlp(experts=4, top=1, ff=56, groups=1, keep=1)),
            channel_decay_layer(heads=2, dim=40, vdim=24, tau=3.0, rank=16, mlp=moe_mlp(experts=8, top=3, ff=32, groups=4, keep=2))]


def random_config(seed: int) -> dict:
    """A configuration drawn from the design's whole space: 2 .. 5 layers of any kinds in any order, any feed-forward or none,
    a loop (anywhere, 1 .. 3 passes) or none, 0 .. 5 taps, widths that need not be multiples of 8."""
    import random

    rnd = random.Random(seed)
    pick = rnd.choice

    def mlp():
        kind = pick(["dense", "moe", "moe", None])
        if kind == "dense":
            return dense_mlp(ff=pick([24, 40, 66, 128]))
        if kind == "moe":
            count = pick([1, 2, 3, 4])
            per = pick([1, 2, 3])
            keep = rnd.randint(1, count)
            return moe_mlp(experts=count * per, top=rnd.randint(1, keep * per), ff=pick([16, 24, 40]), groups=count, keep=keep)
        return None

    def one():
        kind = pick(["mamba1", "parallel", "gla"])
        if kind == "mamba1":
            return scan_layer(inner=pick([24, 48, 80, 128]), state=pick([1, 4, 7, 16, 24, 40]), dt_rank=pick([1, 3, 8, 12]), conv=pick([1, 2, 4, 6]), mlp=mlp())
        if kind == "gla":
            return channel_decay_layer(heads=pick([1, 2, 3, 5]), dim=pick([8, 12, 32, 40]), vdim=pick([8, 20, 32, 64]), tau=pick([1.0, 4.0, 16.0, 30.0]),
                                       rank=pick([2, 8, 12]), mlp=mlp())
        G = pick([1, 2, 3, 4])
        H = G * pick([1, 2, 3, 4])
        dk = pick([8, 16, 24, 32, 48, 64])
        Hr = pick([1, 2, 4, 5])
        left = attention_part(heads=H, kv_heads=G, dim=dk, vdim=pick([8, 16, 32, 48, 80]), scale=pick([0.1, 0.25, dk ** -0.5]),
                              window=pick([None, 1, 7, 32, 50, 64, 100, 160]), rot_dims=pick([0, 2, dk // 2 // 2 * 2, dk]), rot_base=pick([100.0, 10000.0, 500000.0]))
        right = fixed_decay_part(heads=Hr, dim=pick([8, 16, 40]), vdim=pick([8, 24, 64]), decay=[rnd.uniform(0.3, 1.0) for _ in range(Hr)])
        return pair_layer(left=left, right=right, mlp=mlp())

    n = rnd.randint(2, 5)
    layers = [one() for _ in range(n)]
    loop = None
    if rnd.random() < 0.7:
        a = rnd.randint(0, n - 1)
        loop = {"start": a, "stop": rnd.randint(a + 1, n), "times": rnd.randint(1, 3)}
    return make_config(layers, width=pick([24, 36, 40, 64, 100]), vocab=pick([31, 64, 97]), eps=pick([1e-5, 1e-6]), taps=pick([0, 1, 2, 3, 5]),
                       scale=pick([0.5, 1.0, 3.0]), loop=loop)
