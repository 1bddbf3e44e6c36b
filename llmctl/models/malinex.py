"""Malinex: a decoder-only design of sequential layers with norms on both sides of every sublayer and
gated residuals.

* Embedding plus a learned position vector; the residual stream x is fp32.
* A layer: ``h = norm1(x)``, ``x += norm1b(mixer(h) * sigmoid(W_rg1 h + b))``, then the same with
  ``norm2`` / the feed-forward / ``W_rg2`` / ``norm2b`` (RMS norms with plain weights).  The gate reads what the
  sublayer reads, so its rows ride on the sublayer's fused input projection (``side`` rows of the mixers).
* Mixers, chosen per layer: ``gla`` = :class:`~llmctl.models.mixers.GatedLinearAttention` (state slot per
  sequence) and ``attention`` = :class:`~llmctl.models.mixers.SigmoidAttention` (paged rows ``[v | k]``).
* Feed-forward: ``dense`` = :class:`~llmctl.models.mixers.DenseFF` with the exact GELU, or ``moe`` =
  :class:`~llmctl.models.moe.BiasedSoftmaxMoE` (softmax router with a selection bias, squared-ReLU experts,
  a shared expert), or none.
* A layer entry with ``weights_of: j`` runs layer j's weights again with a cache entry or state of its own:
  the model holds one module per weight set and one cache entry per layer.
* Final RMS norm, then ``logits = head x * logit_scale``.

Checkpoint layout: ``config.json`` (``architecture``, ``vocab``, ``width``, ``norm.eps``, ``logit_scale``,
``max_positions``, ``layers`` = one entry per layer with ``type``, ``mixer``, ``mlp`` or null, optional
``weights_of``) and ``model.safetensors`` with ``embed``, ``pos``, ``l<i>.norm1|norm1b|norm2|norm2b``,
``l<i>.rg1|rg2[.b]``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``; linear weights ``[out, in]``.
"""

from __future__ import annotations

import copy
import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from llmctl.ops import hybrid as hops

from .mixers import DenseFF, GatedLinearAttention, SigmoidAttention, StepBatch
from .moe import BiasedSoftmaxMoE

ARCHITECTURE = "Malinex"


@dataclass
class MalinexConfig:
    name: str = "malinex"
    architecture: str = ARCHITECTURE
    vocab_size: int = 512
    hidden: int = 256
    layer_specs: List[Dict[str, Any]] = field(default_factory=list)
    layer_norm_eps: float = 1e-5
    logit_scale: float = 1.0
    max_position_embeddings: int = 8192
    decay_ranks: Dict[int, int] = field(default_factory=dict)  # gla layers: rank of the decay projection
    extra: Dict[str, Any] = field(default_factory=dict)

    tie_word_embeddings = False

    @property
    def is_moe(self) -> bool:
        return any((s.get("mlp") or {}).get("kind") == "moe" for s in self.layer_specs)

    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    def source(self, i: int) -> int:
        """The layer whose weights layer i runs."""
        return int(self.layer_specs[i].get("weights_of", i))

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MalinexConfig":
        d = copy.deepcopy(dict(d))
        kw = dict(architecture=d.pop("architecture", ARCHITECTURE), vocab_size=int(d.pop("vocab")),
                  hidden=int(d.pop("width")), layer_specs=list(d.pop("layers")),
                  layer_norm_eps=float(d.pop("norm")["eps"]), logit_scale=float(d.pop("logit_scale", 1.0)),
                  max_position_embeddings=int(d.pop("max_positions", d.pop("max_position_embeddings", 8192))))
        if "name" in d:
            kw["name"] = d.pop("name")
        if "decay_ranks" in d:
            kw["decay_ranks"] = {int(k): int(v) for k, v in d.pop("decay_ranks").items()}
        n = len(kw["layer_specs"])
        for i, spec in enumerate(kw["layer_specs"]):
            if spec["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown mixer type {spec['type']!r} (known: {sorted(MIXER_TYPES)})")
            mlp = spec.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") not in ("dense", "moe"):
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            j = spec.get("weights_of")
            if j is not None and (not 0 <= int(j) < n or "weights_of" in kw["layer_specs"][int(j)]):
                raise ValueError(f"layer {i}: weights_of must name a layer with weights of its own")
        return cls(extra=d, **kw)

    @classmethod
    def from_file(cls, path) -> "MalinexConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architecture, "name": self.name, "vocab": self.vocab_size, "width": self.hidden,
             "norm": {"eps": self.layer_norm_eps}, "logit_scale": self.logit_scale,
             "max_positions": self.max_position_embeddings, "layers": copy.deepcopy(self.layer_specs)}
        if self.decay_ranks:
            d["decay_ranks"] = {str(k): v for k, v in self.decay_ranks.items()}
        d.update(self.extra)
        return d

    def num_parameters(self, include_embedding: bool = True) -> int:
        with torch.device("meta"):
            m = MalinexLM(self, dtype=torch.bfloat16)
        n = sum(p.numel() for p in m.parameters())
        return n if include_embedding else n - 2 * self.vocab_size * self.hidden


def _gla(width, m, eps, rank, **kw):
    return GatedLinearAttention(width, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), tau=float(m["tau"]),
                                decay_rank=int(rank or m.get("decay_rank") or max(int(m["dim"]) // 4, 1)), eps=eps, **kw)


def _attention(width, m, eps, rank, **kw):
    qt = m.get("q_temp") or {}
    return SigmoidAttention(width, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                            vdim=int(m["vdim"]), scale=float(m["scale"]), eps=eps, temp_coef=float(qt.get("coef", 0.0)),
                            temp_every=int(qt.get("every", 1)), **kw)


MIXER_TYPES = {"gla": _gla, "attention": _attention}


class MalinexLayer(nn.Module):
    def __init__(self, cfg: MalinexConfig, i: int, device=None, dtype=None):
        super().__init__()
        spec, W = cfg.layer_specs[i], cfg.hidden
        f32 = dict(device=device, dtype=torch.float32)
        kw = dict(device=device, dtype=dtype)
        self.norm1 = nn.Parameter(torch.ones(W, **f32))
        self.norm1b = nn.Parameter(torch.ones(W, **f32))
        self.mixer = MIXER_TYPES[spec["type"]](W, spec["mixer"], cfg.layer_norm_eps, cfg.decay_ranks.get(i), side=W, **kw)
        mlp = spec.get("mlp")
        self.ff = None
        if mlp is not None:
            if mlp.get("kind", "dense") == "dense":
                self.ff = DenseFF(W, int(mlp["ff"]), "gelu", side=W, **kw)
            else:
                r = mlp["router"]
                self.ff = BiasedSoftmaxMoE(W, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), "relu2",
                                           shared_ff=int((mlp.get("shared") or {}).get("ff", 0)), side=W, **kw)
            self.norm2 = nn.Parameter(torch.ones(W, **f32))
            self.norm2b = nn.Parameter(torch.ones(W, **f32))


class MalinexLM(nn.Module):
    is_hybrid = True

    def __init__(self, cfg: MalinexConfig, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        kw = dict(device=device, dtype=dtype)
        W = cfg.hidden
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W, **kw))
        self.pos = nn.Parameter(torch.empty(cfg.max_position_embeddings, W, **kw))
        # one module per weight set; ``order[i]`` names the module that layer i runs
        own = [i for i in range(cfg.layers) if cfg.source(i) == i]
        self.blocks = nn.ModuleDict({str(i): MalinexLayer(cfg, i, **kw) for i in own})
        self.order = [cfg.source(i) for i in range(cfg.layers)]
        self.final_norm = nn.Parameter(torch.ones(W, device=device, dtype=torch.float32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W, **kw))
        with torch.no_grad():
            self.embed.normal_(0.0, 0.02)
            self.pos.normal_(0.0, 0.02)
            self.lm_head.normal_(0.0, 0.02)

    @property
    def dtype(self):
        return self.embed.dtype

    def block(self, i: int) -> MalinexLayer:
        return self.blocks[str(self.order[i])]

    @property
    def layers(self) -> List[MalinexLayer]:
        return [self.block(i) for i in range(len(self.order))]

    @property
    def has_recurrent_state(self) -> bool:
        return any(len(l.mixer.state_shapes()) > 0 for l in self.layers)

    @property
    def position_limit(self) -> int:
        """Positions the engine may ask for (rows of the learned position table)."""
        return self.pos.shape[0]

    def head_weight(self):
        return self.lm_head

    def cache_kinds(self):
        """One cache entry per layer (layers that share weights keep entries of their own): the mixer's
        paged rows, or its state pools."""
        out = []
        for l in self.layers:
            m = l.mixer
            out.append(("latent", m.cache_row) if m.cache_kind == "latent" else ("state", m.state_shapes()))
        return out

    # ------------------------------------------------------------------ serving step
    def step(self, b: StepBatch, cache, rows: Optional[torch.Tensor] = None, trail: Optional[list] = None):
        """Run the step's packed tokens through all layers against the engine's cache (``cache.layer(i)``:
        the rows or the state pools of layer i).  Returns the fp32 residual stream of ``rows`` (all rows
        if None) after the last layer; ``trail`` collects it after every layer."""
        eps, dt = self.cfg.layer_norm_eps, self.dtype
        n = len(self.order)
        if n == 0:
            x, _ = hops.embed_rmsnorm_f32(b.ids, b.pos, self.embed, self.pos, self.final_norm, eps, dt)
            return x if rows is None else x.index_select(0, rows)
        x, h = hops.embed_rmsnorm_f32(b.ids, b.pos, self.embed, self.pos, self.block(0).norm1, eps, dt)
        for i in range(n):
            layer = self.block(i)
            nxt = self.block(i + 1).norm1 if i + 1 < n else None
            y, r = layer.mixer.step(h, b, cache.layer(i))
            h = hops.gated_norm_add_norm_f32_(x, y, r, layer.norm1b, layer.norm2 if layer.ff is not None else nxt, eps, dt)
            if layer.ff is not None:
                y, r = layer.ff(h)
                h = hops.gated_norm_add_norm_f32_(x, y, r, layer.norm2b, nxt, eps, dt)
            if trail is not None:
                trail.append(x.clone())
        return x if rows is None else x.index_select(0, rows)

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        xn, _ = hops.add_rmsnorm2_f32_(x.contiguous(), None, None, self.final_norm, None, self.cfg.layer_norm_eps, False,
                                       self.dtype)
        return F.linear(xn, self.lm_head).float() * self.cfg.logit_scale

    # ------------------------------------------------------------------ checkpoint names
    @torch.no_grad()
    def load_named(self, W: Dict[str, torch.Tensor]) -> None:
        """Copy a checkpoint's tensors (its names, see the module docstring) into the fused parameters."""
        def put(dst, src):
            if tuple(dst.shape) != tuple(src.shape):
                raise ValueError(f"shape {tuple(src.shape)} does not fit {tuple(dst.shape)}")
            dst.copy_(src.to(dst.dtype))

        def zeros(n):
            return torch.zeros(n, dtype=torch.float32)

        put(self.embed, W["embed"])
        put(self.pos, W["pos"])
        put(self.lm_head, W["head"])
        put(self.final_norm, W["final.norm"])
        for key, layer in self.blocks.items():
            p = f"l{key}."
            put(layer.norm1, W[p + "norm1"])
            put(layer.norm1b, W[p + "norm1b"])
            m, q = layer.mixer, p + "mix."
            if isinstance(m, GatedLinearAttention):
                put(m.w_in, torch.cat([W[q + "q"], W[q + "k"], W[q + "v"], W[q + "g"], W[q + "a1"], W[p + "rg1"]], 0))
                put(m.b_in, torch.cat([zeros(m.cols), W[p + "rg1.b"].float()]))
                put(m.w_a2, W[q + "a2"])
                put(m.b_a2, W[q + "a2.b"])
                put(m.norm, W[q + "norm"])
            else:
                put(m.w_in, torch.cat([W[q + "q"], W[q + "k"], W[q + "v"], W[q + "g"], W[p + "rg1"]], 0))
                put(m.b_in, torch.cat([W[q + "q.b"].float(), W[q + "k.b"].float(), W[q + "v.b"].float(), zeros(m.H),
                                       W[p + "rg1.b"].float()]))
                put(m.q_norm, W[q + "q.norm"])
                put(m.k_norm, W[q + "k.norm"])
                put(m.dist_a, W[q + "r1"])
                put(m.dist_b, W[q + "r2"])
                put(m.bias, W[q + "pb"])
            put(m.w_o, W[q + "o"])
            ff, f = layer.ff, p + "mlp."
            if ff is None:
                continue
            put(layer.norm2, W[p + "norm2"])
            put(layer.norm2b, W[p + "norm2b"])
            if isinstance(ff, DenseFF):
                put(ff.w_up, torch.cat([W[f + "up"], W[p + "rg2"]], 0))
                put(ff.b_up, torch.cat([zeros(ff.ff), W[p + "rg2.b"].float()]))
                put(ff.w_down, W[f + "down"])
            else:
                put(ff.w_router, W[f + "router"])
                put(ff.bias, W[f + "correction"])
                for e in range(ff.E):
                    put(ff.experts_up[e], W[f"{f}e{e}.up"])
                    put(ff.experts_down[e], W[f"{f}e{e}.down"])
                if ff.shared_ff:
                    put(ff.w_sup, torch.cat([W[f + "shared.up"], W[p + "rg2"]], 0))
                    put(ff.w_sdown, W[f + "shared.down"])
                else:
                    put(ff.w_sup, W[p + "rg2"])
                put(ff.b_sup, torch.cat([zeros(ff.shared_ff), W[p + "rg2.b"].float()]))

    @torch.no_grad()
    def export_named(self) -> Dict[str, torch.Tensor]:
        """The inverse of :meth:`load_named`: tensors under the checkpoint's names."""
        out = {"embed": self.embed, "pos": self.pos, "head": self.lm_head, "final.norm": self.final_norm}
        for key, layer in self.blocks.items():
            p = f"l{key}."
            out[p + "norm1"], out[p + "norm1b"] = layer.norm1, layer.norm1b
            m, q = layer.mixer, p + "mix."
            if isinstance(m, GatedLinearAttention):
                a, c, e = m.H * m.dk, 2 * m.H * m.dk, 2 * m.H * m.dk + m.H * m.dv
                out.update({q + "q": m.w_in[:a], q + "k": m.w_in[a:c], q + "v": m.w_in[c:e], q + "g": m.w_in[e:e + m.H * m.dv],
                            q + "a1": m.w_in[e + m.H * m.dv:m.cols], q + "a2": m.w_a2, q + "a2.b": m.b_a2, q + "norm": m.norm})
            else:
                a, c, e = m.H * m.dk, (m.H + m.G) * m.dk, (m.H + m.G) * m.dk + m.G * m.dv
                out.update({q + "q": m.w_in[:a], q + "k": m.w_in[a:c], q + "v": m.w_in[c:e], q + "g": m.w_in[e:m.cols],
                            q + "q.b": m.b_in[:a], q + "k.b": m.b_in[a:c], q + "v.b": m.b_in[c:e], q + "q.norm": m.q_norm,
                            q + "k.norm": m.k_norm, q + "r1": m.dist_a, q + "r2": m.dist_b, q + "pb": m.bias})
            out.update({q + "o": m.w_o, p + "rg1": m.w_in[m.cols:], p + "rg1.b": m.b_in[m.cols:]})
            ff, f = layer.ff, p + "mlp."
            if ff is None:
                continue
            out[p + "norm2"], out[p + "norm2b"] = layer.norm2, layer.norm2b
            if isinstance(ff, DenseFF):
                out.update({f + "up": ff.w_up[:ff.ff], f + "down": ff.w_down, p + "rg2": ff.w_up[ff.ff:], p + "rg2.b": ff.b_up[ff.ff:]})
            else:
                out[f + "router"], out[f + "correction"] = ff.w_router, ff.bias
                for e in range(ff.E):
                    out[f"{f}e{e}.up"], out[f"{f}e{e}.down"] = ff.experts_up[e], ff.experts_down[e]
                if ff.shared_ff:
                    out[f + "shared.up"], out[f + "shared.down"] = ff.w_sup[:ff.shared_ff], ff.w_sdown
                out[p + "rg2"], out[p + "rg2.b"] = ff.w_sup[ff.shared_ff:], ff.b_sup[ff.shared_ff:]
        return {k: v.detach().clone().contiguous() for k, v in out.items()}


def load_malinex(ck: Path, cfg: MalinexConfig, device=None, dtype=torch.bfloat16) -> MalinexLM:
    from safetensors import safe_open

    with safe_open(str(ck / "model.safetensors"), framework="pt", device="cpu") as f:
        W = {k: f.get_tensor(k) for k in f.keys()}
    # sizes that only the tensors give: the rank of the decay projection, the number of positions
    for i, spec in enumerate(cfg.layer_specs):
        if spec["type"] == "gla" and cfg.source(i) == i:
            cfg.decay_ranks[i] = int(W[f"l{i}.mix.a1"].shape[0])
    cfg.max_position_embeddings = int(W["pos"].shape[0])
    model = MalinexLM(cfg, device=device, dtype=dtype)
    model.load_named(W)
    return model


def malinex_template(width: int = 256, layers: int = 4, heads: int = 4, kv_heads: int = 2, vocab: int = 512, every: int = 3,
                     ff: Optional[int] = None, experts: int = 0, top: int = 2, expert_ff: Optional[int] = None,
                     head_dim: Optional[int] = None, share: bool = False, max_positions: int = 8192) -> MalinexConfig:
    """A random-init configuration for benchmarks and smoke runs: gated linear attention in every layer but
    each ``every``-th, which is sigmoid attention; dense feed-forwards, or routed experts when ``experts`` > 0;
    ``share``: the last gated-linear-attention layer runs the weights of the one before it."""
    d = head_dim or width // heads
    gla = {"heads": heads, "dim": max(d // 2, 1), "vdim": d, "tau": 8.0}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d, "scale": d ** -0.5, "q_temp": {"coef": 0.2, "every": 512}}
    if experts:
        mlp = {"kind": "moe", "expert": {"ff": expert_ff or width // 2}, "router": {"experts": experts, "top": top},
               "shared": {"ff": expert_ff or width // 2}}
    else:
        mlp = {"kind": "dense", "ff": ff or 2 * width}
    specs = [{"type": "attention" if (i + 1) % every == 0 else "gla",
              "mixer": copy.deepcopy(att if (i + 1) % every == 0 else gla), "mlp": copy.deepcopy(mlp)} for i in range(layers)]
    if share:
        g = [i for i, s in enumerate(specs) if s["type"] == "gla"]
        if len(g) >= 2:
            specs[g[-1]]["weights_of"] = g[-2]
    return MalinexConfig(name=f"malinex-w{width}-l{layers}", vocab_size=vocab, hidden=width, layer_specs=specs,
                         layer_norm_eps=1e-5, logit_scale=1.0, max_position_embeddings=max_positions,
                         decay_ranks={i: max(width // 32, 4) for i, s in enumerate(specs) if s["type"] == "gla"})
