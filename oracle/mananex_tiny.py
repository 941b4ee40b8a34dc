"""Seeded small Mananex checkpoints for tests: a config dict and a {name: tensor} dict in the family's tensor naming.
Sizes are arguments; nothing here equals a published model.  TEST INFRASTRUCTURE ONLY."""
from typing import Dict, List, Optional

import torch


def attention_part(heads=6, kv_heads=3, dim=32, vdim=64, scale=0.2, window: Optional[int] = 24, keep_first=3, rot_dims=8,
                   rot_base=1000.0) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first}
    if rot_dims:
        m["rot"] = {"base": rot_base, "dims": rot_dims}
    return m


def recurrent_part(heads=3, dim=16, vdim=32) -> dict:
    return {"heads": heads, "dim": dim, "vdim": vdim}


def layer(left: Optional[dict] = None, right: Optional[dict] = None, left_scale=0.8, right_scale=1.3, mlp=None) -> dict:
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left or attention_part(), "right": right or recurrent_part(), "left_scale": left_scale, "right_scale": right_scale}}


def dense_mlp(ff=96) -> dict:
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts=6, top=2, ff=40) -> dict:
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers: List[dict], width=64, vocab=96, eps=1e-5) -> dict:
    return {"architecture": "Mananex", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps}}


def make_tensors(config: dict, seed: int = 0, dtype=torch.bfloat16, sink_mean: float = 0.5) -> Dict[str, torch.Tensor]:
    """N(0, 1 / fan_in) projections (wider for what feeds a softmax or a router), norm gains around zero (they are offsets
    from one), lower bounds of the forget gates spread over (0, 1), depth-mix coefficients that weigh the newest entry most.
    Values are rounded to `dtype` (what a checkpoint stores)."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    t: Dict[str, torch.Tensor] = {}

    def lin(name, n, k, gain=1.0):
        t[name] = torch.randn(n, k, generator=g) * gain * k ** -0.5

    def vec(name, n, mean=0.0, std=0.1):
        t[name] = mean + torch.randn(n, generator=g) * std

    t["embed"] = torch.randn(config["vocab"], W, generator=g)
    for i, lay in enumerate(config["layers"]):
        m = lay["mixer"]
        vec(f"l{i}.norm1", W)
        a, p = m["left"], f"l{i}.mix.left"
        H, dk = a["heads"], a["dim"]
        G, dv = a.get("kv_heads", H), a.get("vdim", dk)
        lin(f"{p}.q", H * dk, W, 2.0)
        lin(f"{p}.k", G * dk, W, 2.0)
        lin(f"{p}.v", G * dv, W)
        vec(f"{p}.sink", H, sink_mean, 1.0)
        lin(f"{p}.g", H, W, 2.0)
        lin(f"{p}.o", W, H * dv)
        r, p = m["right"], f"l{i}.mix.right"
        Hr, dkr, dvr = r["heads"], r["dim"], r.get("vdim", r["dim"])
        lin(f"{p}.q", Hr * dkr, W)
        lin(f"{p}.f", Hr * dkr, W, 2.0)
        vec(f"{p}.f.b", Hr * dkr, 0.5, 1.0)
        t[f"{p}.lower"] = torch.rand(Hr * dkr, generator=g) * 0.9
        lin(f"{p}.v", Hr * dvr, W)
        vec(f"{p}.norm", dvr, 1.0)
        lin(f"{p}.o", W, Hr * dvr)
        lin(f"l{i}.rg1", W, W, 2.0)
        vec(f"l{i}.rg1.b", W, 0.5, 0.5)
        f = lay.get("mlp")
        if f:
            q = f"l{i}.mlp"
            lin(f"l{i}.rg2", W, W, 2.0)
            vec(f"l{i}.rg2.b", W, 0.5, 0.5)
            if f["kind"] == "dense":
                for n_, (o_, i_) in (("gate", (f["ff"], W)), ("up", (f["ff"], W)), ("down", (W, f["ff"]))):
                    lin(f"{q}.{n_}", o_, i_)
                    vec(f"{q}.{n_}.b", o_, 0.0, 0.3)
            else:
                for e in range(f["router"]["experts"]):
                    lin(f"{q}.e{e}.gate", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.up", f["expert"]["ff"], W)
                    lin(f"{q}.e{e}.down", W, f["expert"]["ff"], 2.0)
                lin(f"{q}.router", f["router"]["experts"], W, 4.0)
                vec(f"{q}.router.b", f["router"]["experts"], 0.0, 0.5)
        c = torch.randn(i + 2, generator=g) * 0.15
        c[-1] += 0.9
        t[f"l{i}.dwa"] = c
    vec("final.norm", W)
    return {k: v.to(dtype) for k, v in t.items()}


def standard_layers() -> List[dict]:
    """Dense and routed feed-forwards, a layer without one, GQA and MHA, windows of several sizes, a layer without a window,
    full and partial rotation."""
    return [layer(mlp=dense_mlp()),
            layer(left=attention_part(heads=4, kv_heads=4, dim=16, vdim=32, scale=0.3, window=40, keep_first=0, rot_dims=16),
                  right=recurrent_part(heads=2, dim=32, vdim=16), mlp=moe_mlp()),
            layer(left=attention_part(heads=6, kv_heads=2, dim=32, vdim=32, window=None, rot_dims=12), mlp=None),
            layer(left=attention_part(window=33, keep_first=34), right=recurrent_part(heads=1, dim=24, vdim=40), mlp=moe_mlp(experts=5, top=1, ff=56))]
