"""Helpers of the Malinex tests: small configurations and random checkpoints written from the naming
rules of the checkpoint layout (not from the model class).  The engine, the schedule driver and the error
measure are those of the Lenitar tests."""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

from tests.models.lenitar_util import engine, rel_err, run_schedule, write_checkpoint  # noqa: F401


def gla(heads=3, dim=6, vdim=10, tau=4.0, rank=5):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "_rank": rank}


def att(heads=4, kv_heads=2, dim=8, vdim=6, scale=None, coef=0.4, every=5):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 2.0 * dim ** -0.5}
    if coef is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def dense(ff=28):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=10, shared=12):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers: List[Tuple[dict, Optional[dict]]], width=20, vocab=50, eps=1e-5, logit_scale=0.7, max_positions=320,
           share: Optional[Dict[int, int]] = None) -> dict:
    """``share`` = {layer: the layer whose weights it runs}."""
    specs = []
    for i, (m, f) in enumerate(layers):
        spec = dict(m, mlp=f)
        if share and i in share:
            j = share[i]
            spec = dict(layers[j][0], mlp=layers[j][1], weights_of=j)
        specs.append(spec)
    return {"architecture": "Malinex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "max_positions": max_positions, "layers": specs}


def clean(cfg: dict) -> dict:
    """The configuration as a checkpoint carries it (without the helpers' private keys)."""
    out = dict(cfg)
    out["layers"] = [{k: v for k, v in s.items() if not k.startswith("_")} for s in cfg["layers"]]
    return out


def without_experts(cfg: dict) -> dict:
    """The configuration with every routed feed-forward replaced by a dense one."""
    out = dict(cfg)
    out["layers"] = []
    for s in cfg["layers"]:
        f = s.get("mlp")
        if f is not None and f.get("kind") == "moe":
            s = dict(s, mlp=dense(f["expert"]["ff"] * f["router"]["top"]))
        out["layers"].append(s)
    return out


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).bfloat16().float()

    def vec(n, mean=0.0, std=1.0):
        return (mean + std * torch.randn(n, generator=g)).bfloat16().float()

    out = {"embed": vec(cfg["vocab"] * W).view(cfg["vocab"], W), "pos": vec(cfg["max_positions"] * W, 0.0, 0.5).view(-1, W),
           "head": lin(cfg["vocab"], W), "final.norm": vec(W, 1.0, 0.2)}
    for i, layer in enumerate(cfg["layers"]):
        if "weights_of" in layer:
            continue
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm1b"):
            out[p + n] = vec(W, 1.0, 0.2)
        out[p + "rg1"], out[p + "rg1.b"] = lin(W, W, 2.0), vec(W, 0.0, 1.0)
        q = p + "mix."
        if layer["type"] == "gla":
            H, dk, dv, r = m["heads"], m["dim"], m["vdim"], layer.get("_rank", 5)
            out.update({q + "q": lin(H * dk, W, 2.0), q + "k": lin(H * dk, W, 2.0), q + "v": lin(H * dv, W), q + "g": lin(H * dv, W, 2.0),
                        q + "o": lin(W, H * dv), q + "norm": vec(dv, 1.0, 0.2), q + "a1": lin(r, W, 2.0), q + "a2": lin(H * dk, r, 2.0),
                        q + "a2.b": vec(H * dk, 1.5, 1.0)})
        else:
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({q + "q": lin(H * dk, W, 2.0), q + "k": lin(G * dk, W, 2.0), q + "v": lin(G * dv, W), q + "g": lin(H, W, 2.0),
                        q + "o": lin(W, H * dv), q + "q.b": vec(H * dk, 0.0, 0.3), q + "k.b": vec(G * dk, 0.0, 0.3),
                        q + "v.b": vec(G * dv, 0.0, 0.3), q + "q.norm": vec(H * dk, 1.0, 0.2), q + "k.norm": vec(G * dk, 1.0, 0.2),
                        q + "r1": vec(H, 0.5, 0.3).abs(), q + "r2": vec(H, 0.6, 0.4).abs(), q + "pb": vec(H, -1.0, 1.0)})
        f = layer.get("mlp")
        if f is None:
            continue
        for n in ("norm2", "norm2b"):
            out[p + n] = vec(W, 1.0, 0.2)
        out[p + "rg2"], out[p + "rg2.b"] = lin(W, W, 2.0), vec(W, 0.0, 1.0)
        if f["kind"] == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"] = lin(f["ff"], W, 2.0), lin(W, f["ff"])
        else:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            out[p + "mlp.router"], out[p + "mlp.correction"] = lin(E, W, 4.0), vec(E, 0.0, 0.15)
            for e in range(E):
                out[f"{p}mlp.e{e}.up"], out[f"{p}mlp.e{e}.down"] = lin(ff, W, 2.0), lin(W, ff)
            if f.get("shared"):
                out[p + "mlp.shared.up"], out[p + "mlp.shared.down"] = lin(f["shared"]["ff"], W, 2.0), lin(W, f["shared"]["ff"])
    return out


def rel_errs(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: RMS difference of the centred logits, relative to the RMS of the wanted ones."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()
