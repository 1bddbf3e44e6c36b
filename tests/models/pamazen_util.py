"""Helpers of the Pamazen tests: small configurations and random checkpoints written from the naming rules of
the checkpoint layout (not from the model class).  The engine, the schedule driver and the error measures are
those of the Lenitar and Malinex tests."""

from __future__ import annotations

import copy
import math
from typing import Dict, List, Optional, Tuple

import torch

from tests.models.lenitar_util import engine, rel_err, run_schedule, write_checkpoint  # noqa: F401
from tests.models.malinex_util import rel_errs  # noqa: F401


def att(heads=4, kv_heads=2, dim=8, vdim=6, scale=None, rot_dims=4, base=100.0, factor=1.5, v_mix=True):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.5 * dim ** -0.5,
         "v_mix": v_mix}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    return {"type": "attention", "mixer": m}


def par(heads=4, kv_heads=2, dim=6, window=7, keep=2, cap=5.0, scale=None, rheads=3, rdim=5, rank=4, ls=0.7, rs=1.3):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else 2.0 * dim ** -0.5,
            "mask": {"size": window, "keep_first": keep}}
    if cap:
        left["softcap"] = cap
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "dim": rdim}, "left_scale": ls, "right_scale": rs},
            "_rank": rank}


def moe(experts=6, top=2, ff=10, shared=12, identity=2, groups=2, keep=1):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity,
                                                         "groups": {"count": groups, "keep": keep}}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers: List[Tuple[dict, Optional[dict]]], width=20, vocab=50, eps=1e-5, streams=3, mult=0.6, cap=8.0) -> dict:
    cfg = {"architecture": "Pamazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "layers": [dict(copy.deepcopy(m), mlp=copy.deepcopy(f)) for m, f in layers]}
    if streams:
        cfg["streams"] = streams
    if cap:
        cfg["logit_softcap"] = cap
    return cfg


def clean(cfg: dict) -> dict:
    """The configuration as a checkpoint carries it (without the helpers' private keys)."""
    out = dict(cfg)
    out["layers"] = [{k: v for k, v in s.items() if not k.startswith("_")} for s in cfg["layers"]]
    return out


def without_choice(cfg: dict) -> dict:
    """The configuration with routers that choose every expert (one group, top = all): nothing can flip under
    bf16 rounding.  Tensor shapes stay."""
    out = copy.deepcopy(cfg)
    for s in out["layers"]:
        f = s.get("mlp")
        if f is not None:
            r = f["router"]
            r["top"] = r["experts"] + r.get("identity", 0)
            r["groups"] = {"count": 1, "keep": 1}
    return out


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams", 0)

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).bfloat16().float()

    def vec(n, mean=0.0, std=1.0):
        return (mean + std * torch.randn(n, generator=g)).bfloat16().float()

    def one(mean=1.0, std=0.2):
        return vec(1, mean, std).reshape(())

    out = {"embed": vec(cfg["vocab"] * W).view(cfg["vocab"], W), "head": lin(cfg["vocab"], W, 2.0), "final.norm": one()}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        subs = ["1"] + (["2"] if layer.get("mlp") is not None else [])
        for q in subs:
            out[p + "norm" + q] = one()
            if S:
                out[f"{p}hc{q}.in"] = vec(S, 1.0 / S, 0.3)
                out[f"{p}hc{q}.out"] = vec(S, 1.0, 0.4)
                out[f"{p}hc{q}.mix"] = (torch.eye(S) + 0.25 * torch.randn(S, S, generator=g)).bfloat16().float()
        q = p + "mix."
        if layer["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({q + "q": lin(H * dk, W, 2.0), q + "k": lin(G * dk, W, 2.0), q + "v": lin(G * dv, W), q + "o": lin(W, H * dv),
                        q + "vmix": one(0.4, 0.2)})
        else:
            l, r, rank = m["left"], m["right"], layer.get("_rank", 4)
            H, G, dk = l["heads"], l["kv_heads"], l["dim"]
            out.update({q + "left.q": lin(H * dk, W, 2.0), q + "left.k": lin(G * dk, W, 2.0), q + "left.q.norm": vec(dk, 1.0, 0.3),
                        q + "left.k.norm": vec(dk, 1.0, 0.3), q + "left.sink": vec(H, 0.0, 1.5), q + "left.o": lin(W, H * dk)})
            n = r["heads"] * r["dim"]
            out.update({q + "right.r": lin(n, W, 1.5), q + "right.k": lin(n, W, 1.5), q + "right.v": lin(n, W), q + "right.g": lin(n, W, 2.0),
                        q + "right.a": lin(n, W, 2.0), q + "right.a.b": vec(n, 0.0, 1.0), q + "right.w1": lin(rank, W, 2.0),
                        q + "right.w2": lin(n, rank, 2.0), q + "right.w0": vec(n, -1.0, 1.5), q + "right.norm": vec(n, 1.0, 0.2),
                        q + "right.o": lin(W, n)})
        f = layer.get("mlp")
        if f is None:
            continue
        r = f["router"]
        E, n, ff = r["experts"], r["experts"] + r.get("identity", 0), f["expert"]["ff"]
        out[p + "mlp.router"], out[p + "mlp.correction"] = lin(n, W, 4.0), vec(n, 0.0, 0.15)
        for e in range(E):
            out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"], out[f"{p}mlp.e{e}.down"] = lin(ff, W, 2.0), lin(ff, W), lin(W, ff)
        if f.get("shared"):
            s = f["shared"]["ff"]
            out.update({p + "mlp.shared.gate": lin(s, W, 2.0), p + "mlp.shared.up": lin(s, W), p + "mlp.shared.down": lin(W, s),
                        p + "mlp.shared.sg": lin(1, W, 3.0)})
    return out
