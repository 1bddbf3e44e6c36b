"""Pamazen: a decoder-only design of pre-norm layers over several residual streams (hyper-connections).

* ``x = embed[token]``; every one of ``streams`` residual streams starts as x (fp32).
* A sublayer q of layer i (1: the mixer, 2: the feed-forward) reads ``u = sum_s in_q[s] x_s`` through an RMS
  norm with a single weight, and its result y enters all streams at once:
  ``x_t <- sum_s mix_q[s, t] x_s + residual_mult * out_q[t] * y``.  Without ``streams`` in the config there is one
  stream and the plain sum ``x += residual_mult * y``.  After the last layer x is the sum of the streams.
* Mixers, chosen per layer: ``attention`` = :class:`~llmctl.models.mixers.GroupedAttention` without q / k norms:
  rotary on neighbour pairs of the first ``rot.dims`` entries with linearly scaled frequencies, causal, one added
  to the softmax denominator, and the values of every ``v_mix`` layer after the first one blended with the
  first one's (same token) before they are cached; ``parallel`` = :class:`~llmctl.models.mixers.ParallelMixers`
  of a windowed attention (q / k norms, no rotation, values = the projected keys, capped scores, a window that
  keeps the first tokens, a learned sink) and a :class:`~llmctl.models.mixers.DeltaRule` memory.
* Feed-forward: :class:`~llmctl.models.moe.BiasedSoftmaxMoE` with gated experts, group-limited choice by
  ``score + correction``, weights that are the scores themselves, identity experts and a gated shared expert; or none.
* Final RMS norm (single weight), ``logits = head x``, then ``cap * tanh(logits / cap)``.

Checkpoint layout: ``config.json`` (``architecture``, ``vocab``, ``width``, ``norm.eps``, ``residual_mult``,
``streams``, ``logit_softcap``, ``layers`` = one entry per layer with ``type``, ``mixer``, ``mlp`` or null) and
``model.safetensors`` with ``embed``, ``l<i>.norm1|norm2``, ``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``; linear weights ``[out, in]``.
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

from .mixers import DeltaRule, GroupedAttention, ParallelMixers, StepBatch
from .moe import BiasedSoftmaxMoE

ARCHITECTURE = "Pamazen"


@dataclass
class PamazenConfig:
    name: str = "pamazen"
    architecture: str = ARCHITECTURE
    vocab_size: int = 512
    hidden: int = 256
    layer_specs: List[Dict[str, Any]] = field(default_factory=list)
    layer_norm_eps: float = 1e-6
    residual_mult: float = 1.0
    streams: int = 0  # 0: one stream with the plain residual sum (no hyper-connection tensors)
    logit_softcap: float = 0.0
    decay_ranks: Dict[int, int] = field(default_factory=dict)  # parallel layers: rank of the decay projection
    max_position_embeddings: int = 1 << 20
    extra: Dict[str, Any] = field(default_factory=dict)

    tie_word_embeddings = False

    @property
    def is_moe(self) -> bool:
        return any(s.get("mlp") is not None for s in self.layer_specs)

    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    def value_mix_roles(self) -> List[Optional[str]]:
        """Per layer: "source" for the first attention layer with ``v_mix``, "mix" for the later ones, else None."""
        out, seen = [], False
        for s in self.layer_specs:
            if s["type"] == "attention" and s["mixer"].get("v_mix"):
                out.append("mix" if seen else "source")
                seen = True
            else:
                out.append(None)
        return out

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PamazenConfig":
        d = copy.deepcopy(dict(d))
        kw = dict(architecture=d.pop("architecture", ARCHITECTURE), vocab_size=int(d.pop("vocab")),
                  hidden=int(d.pop("width")), layer_specs=list(d.pop("layers")),
                  layer_norm_eps=float(d.pop("norm")["eps"]), residual_mult=float(d.pop("residual_mult", 1.0)),
                  streams=int(d.pop("streams", 0) or 0), logit_softcap=float(d.pop("logit_softcap", 0.0) or 0.0))
        if "name" in d:
            kw["name"] = d.pop("name")
        if "decay_ranks" in d:
            kw["decay_ranks"] = {int(k): int(v) for k, v in d.pop("decay_ranks").items()}
        widths = set()
        for i, spec in enumerate(kw["layer_specs"]):
            if spec["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown mixer type {spec['type']!r} (known: {sorted(MIXER_TYPES)})")
            mlp = spec.get("mlp")
            if mlp is not None and mlp.get("kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            m = spec["mixer"]
            if spec["type"] == "attention" and m.get("v_mix"):
                widths.add((int(m.get("kv_heads", m["heads"])), int(m["vdim"])))
        if len(widths) > 1:
            raise ValueError("layers that mix their values with the first one's need values of one size")
        return cls(extra=d, **kw)

    @classmethod
    def from_file(cls, path) -> "PamazenConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architecture, "name": self.name, "vocab": self.vocab_size, "width": self.hidden,
             "norm": {"eps": self.layer_norm_eps}, "residual_mult": self.residual_mult, "layers": copy.deepcopy(self.layer_specs)}
        if self.streams:
            d["streams"] = self.streams
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.decay_ranks:
            d["decay_ranks"] = {str(k): v for k, v in self.decay_ranks.items()}
        d.update(self.extra)
        return d

    def num_parameters(self, include_embedding: bool = True) -> int:
        with torch.device("meta"):
            m = PamazenLM(self, dtype=torch.bfloat16)
        n = sum(p.numel() for p in m.parameters())
        return n if include_embedding else n - 2 * self.vocab_size * self.hidden


def _attention(width, m, eps, rank, role, **kw):
    rot = m.get("rot") or {}
    return GroupedAttention(width, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                            vdim=int(m["vdim"]), rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)),
                            scale=float(m["scale"]), eps=eps, rot_scaling=rot.get("scaling"), interleaved=True,
                            sink=0.0, qk_norm=False, value_mix=role, **kw)


def _parallel(width, m, eps, rank, role, **kw):
    l, r = m["left"], m["right"]
    mask = l.get("mask") or {}
    left = GroupedAttention(width, heads=int(l["heads"]), kv_heads=int(l.get("kv_heads", l["heads"])), dim=int(l["dim"]),
                            vdim=int(l.get("vdim", l["dim"])), rot_base=10000.0, rot_dims=0, scale=float(l["scale"]), eps=eps,
                            interleaved=True, window=mask.get("size"), keep_first=int(mask.get("keep_first", 0)),
                            sink=True, qk_norm=True, values="keys", softcap=float(l.get("softcap", 0.0) or 0.0), **kw)
    right = DeltaRule(width, heads=int(r["heads"]), dim=int(r["dim"]),
                      decay_rank=int(rank or r.get("decay_rank") or max(int(r["dim"]) // 4, 1)), eps=eps, **kw)
    return ParallelMixers(left, right, float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))


MIXER_TYPES = {"attention": _attention, "parallel": _parallel}


class HyperConnection(nn.Module):
    """The coefficients of one sublayer over ``streams`` residual streams: ``c_in [S]`` weighs the streams into the
    sublayer's input, ``mix [S, S]`` (from, to) carries the old streams over, ``c_out [S]`` spreads the result."""

    def __init__(self, streams: int, device=None):
        super().__init__()
        f32 = dict(device=device, dtype=torch.float32)
        self.c_in = nn.Parameter(torch.full((streams,), 1.0 / streams, **f32))
        self.c_out = nn.Parameter(torch.ones(streams, **f32))
        self.mix = nn.Parameter(torch.eye(streams, **f32))


class PamazenLayer(nn.Module):
    def __init__(self, cfg: PamazenConfig, i: int, role: Optional[str], device=None, dtype=None):
        super().__init__()
        spec, W = cfg.layer_specs[i], cfg.hidden
        f32 = dict(device=device, dtype=torch.float32)
        kw = dict(device=device, dtype=dtype)
        S = max(cfg.streams, 1)
        self.norm1 = nn.Parameter(torch.ones(1, **f32))  # an RMS norm with one weight for all coordinates
        self.hc1 = HyperConnection(S, device)
        self.mixer = MIXER_TYPES[spec["type"]](W, spec["mixer"], cfg.layer_norm_eps, cfg.decay_ranks.get(i), role, **kw)
        # a checkpoint carries a mixing factor for every attention layer; layers that do not mix keep theirs unread
        self.vmix_unread = (nn.Parameter(torch.zeros(1, **f32))
                            if spec["type"] == "attention" and self.mixer.vmix is None else None)
        mlp = spec.get("mlp")
        self.ff = None
        if mlp is not None:
            r = mlp["router"]
            g = r.get("groups") or {}
            shared = int((mlp.get("shared") or {}).get("ff", 0))
            self.ff = BiasedSoftmaxMoE(W, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), "swiglu", shared_ff=shared,
                                       groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))), renorm=False,
                                       identity=int(r.get("identity", 0)), shared_gate=shared > 0, **kw)
            self.norm2 = nn.Parameter(torch.ones(1, **f32))
            self.hc2 = HyperConnection(S, device)

    def sublayers(self):
        """(norm weight, hyper-connection, run) per sublayer, in order."""
        out = [(self.norm1, self.hc1)]
        if self.ff is not None:
            out.append((self.norm2, self.hc2))
        return out


class PamazenLM(nn.Module):
    is_hybrid = True

    def __init__(self, cfg: PamazenConfig, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        kw = dict(device=device, dtype=dtype)
        W = cfg.hidden
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W, **kw))
        roles = cfg.value_mix_roles()
        self.layers = nn.ModuleList([PamazenLayer(cfg, i, roles[i], **kw) for i in range(cfg.layers)])
        self.final_norm = nn.Parameter(torch.ones(1, device=device, dtype=torch.float32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W, **kw))
        self._fn, self._fn_key = None, None
        with torch.no_grad():
            self.embed.normal_(0.0, 0.02)
            self.lm_head.normal_(0.0, 0.02)

    @property
    def dtype(self):
        return self.embed.dtype

    @property
    def has_recurrent_state(self) -> bool:
        return any(len(l.mixer.state_shapes()) > 0 for l in self.layers)

    def head_weight(self):
        return self.lm_head

    def cache_kinds(self):
        """One cache entry per layer: the mixer's paged rows, or rows and state pools for a pair of mixers."""
        out = []
        for l in self.layers:
            m = l.mixer
            if m.cache_kind == "rows+state":
                out.append(("rows+state", (m.cache_row, m.state_shapes())))
            else:
                out.append(("latent", m.cache_row) if m.cache_kind == "latent" else ("state", m.state_shapes()))
        return out

    # ------------------------------------------------------------------ serving step
    def step(self, b: StepBatch, cache, rows: Optional[torch.Tensor] = None, trail: Optional[list] = None):
        """Run the step's packed tokens through all layers against the engine's cache (``cache.layer(i)``).
        Returns the fp32 sum of the residual streams of ``rows`` (all rows if None) after the last layer;
        ``trail`` collects it after every layer."""
        eps, dt, mult = self.cfg.layer_norm_eps, self.dtype, self.cfg.residual_mult
        S = max(self.cfg.streams, 1)
        subs = [(i, q, n, hc) for i, l in enumerate(self.layers) for q, (n, hc) in enumerate(l.sublayers())]
        if not subs:
            X, _ = hops.hc_embed_norm(b.ids, self.embed, S, torch.ones(S, device=self.embed.device), self.final_norm, eps, dt)
        else:
            X, h = hops.hc_embed_norm(b.ids, self.embed, S, subs[0][3].c_in, subs[0][2], eps, dt)
        for j, (i, q, _, hc) in enumerate(subs):
            layer = self.layers[i]
            nxt = subs[j + 1] if j + 1 < len(subs) else None
            if q == 0:
                y = layer.mixer.step(h, b, cache.layer(i))
            else:
                y = layer.ff(h)
            (y1, s1), (y2, s2) = (y if isinstance(y, tuple) else ((y, 1.0), (None, 0.0)))
            h = hops.hc_update_norm_(X, y1, s1, y2, s2, hc.mix, hc.c_out, mult, nxt[3].c_in if nxt else None,
                                     nxt[2] if nxt else None, eps, dt)
            if trail is not None and (nxt is None or nxt[0] != i):
                trail.append(X.sum(1))
        if rows is not None:
            X = X.index_select(0, rows)
        return X.sum(1)

    def _final_norm_row(self) -> torch.Tensor:
        """The final norm's single weight as a row of ``width`` (made once; serving weights are static)."""
        w = self.final_norm
        key = (w.data_ptr(), w._version, w.device)
        if self._fn_key != key:
            self._fn, self._fn_key = w.detach().float().expand(self.cfg.hidden).contiguous(), key
        return self._fn

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        xn, _ = hops.add_rmsnorm2_f32_(x.contiguous(), None, None, self._final_norm_row(), None, self.cfg.layer_norm_eps, False,
                                       self.dtype)
        z = F.linear(xn, self.lm_head).float()
        return hops.softcap_(z, self.cfg.logit_softcap) if self.cfg.logit_softcap > 0 else z

    # ------------------------------------------------------------------ checkpoint names
    @torch.no_grad()
    def load_named(self, W: Dict[str, torch.Tensor]) -> None:
        """Copy a checkpoint's tensors (its names, see the module docstring) into the fused parameters."""
        def put(dst, src):
            src = src.reshape(dst.shape) if src.numel() == dst.numel() and src.dim() != dst.dim() else src
            if tuple(dst.shape) != tuple(src.shape):
                raise ValueError(f"shape {tuple(src.shape)} does not fit {tuple(dst.shape)}")
            dst.copy_(src.to(dst.dtype))

        put(self.embed, W["embed"])
        put(self.lm_head, W["head"])
        put(self.final_norm, W["final.norm"])
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.norm1, W[p + "norm1"])
            hcs = [(layer.hc1, "hc1.")]
            if layer.ff is not None:
                put(layer.norm2, W[p + "norm2"])
                hcs.append((layer.hc2, "hc2."))
            if self.cfg.streams:
                for hc, n in hcs:
                    put(hc.c_in, W[p + n + "in"])
                    put(hc.c_out, W[p + n + "out"])
                    put(hc.mix, W[p + n + "mix"])
            else:
                for hc, _ in hcs:
                    hc.c_in.fill_(1.0)
            m, q = layer.mixer, p + "mix."
            if isinstance(m, ParallelMixers):
                a, ql = m.left, q + "left."
                put(a.w_qkv, torch.cat([W[ql + "q"], W[ql + "k"]], 0))
                put(a.q_norm, W[ql + "q.norm"])
                put(a.k_norm, W[ql + "k.norm"])
                put(a.sink, W[ql + "sink"])
                put(a.w_o, W[ql + "o"])
                d, qr = m.right, q + "right."
                put(d.w_in, torch.cat([W[qr + n] for n in ("r", "k", "v", "g", "a", "w1")], 0))
                put(d.w_w2, W[qr + "w2"])
                put(d.w0, W[qr + "w0"])
                put(d.b_a, W[qr + "a.b"])
                put(d.norm, W[qr + "norm"])
                put(d.w_o, W[qr + "o"])
            else:
                put(m.w_qkv, torch.cat([W[q + "q"], W[q + "k"], W[q + "v"]], 0))
                put(m.w_o, W[q + "o"])
                if q + "vmix" in W:
                    put(m.vmix if m.vmix is not None else layer.vmix_unread, W[q + "vmix"])
            ff, f = layer.ff, p + "mlp."
            if ff is None:
                continue
            put(ff.w_router, W[f + "router"])
            if f + "correction" in W:
                put(ff.bias, W[f + "correction"])
            for e in range(ff.E):
                put(ff.w_up[e], torch.cat([W[f"{f}e{e}.gate"], W[f"{f}e{e}.up"]], 0))
                put(ff.w_down[e], W[f"{f}e{e}.down"])
            if ff.shared_ff:
                put(ff.w_sup, torch.cat([W[f + "shared.gate"], W[f + "shared.up"], W[f + "shared.sg"].reshape(1, -1)], 0))
                put(ff.w_sdown, W[f + "shared.down"])

    @torch.no_grad()
    def export_named(self) -> Dict[str, torch.Tensor]:
        """The inverse of :meth:`load_named`: tensors under the checkpoint's names."""
        out = {"embed": self.embed, "head": self.lm_head, "final.norm": self.final_norm.reshape(())}
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = layer.norm1.reshape(())
            hcs = [(layer.hc1, "hc1.")]
            if layer.ff is not None:
                out[p + "norm2"] = layer.norm2.reshape(())
                hcs.append((layer.hc2, "hc2."))
            if self.cfg.streams:
                for hc, n in hcs:
                    out[p + n + "in"], out[p + n + "out"], out[p + n + "mix"] = hc.c_in, hc.c_out, hc.mix
            m, q = layer.mixer, p + "mix."
            if isinstance(m, ParallelMixers):
                a, ql = m.left, q + "left."
                nq = a.H * a.dk
                out.update({ql + "q": a.w_qkv[:nq], ql + "k": a.w_qkv[nq:], ql + "q.norm": a.q_norm, ql + "k.norm": a.k_norm,
                            ql + "sink": a.sink, ql + "o": a.w_o})
                d, qr = m.right, q + "right."
                n = d.H * d.d
                for j, name in enumerate(("r", "k", "v", "g", "a")):
                    out[qr + name] = d.w_in[j * n:(j + 1) * n]
                out.update({qr + "w1": d.w_in[5 * n:], qr + "w2": d.w_w2, qr + "w0": d.w0, qr + "a.b": d.b_a, qr + "norm": d.norm,
                            qr + "o": d.w_o})
            else:
                a, c = m.H * m.dk, (m.H + m.G) * m.dk
                out.update({q + "q": m.w_qkv[:a], q + "k": m.w_qkv[a:c], q + "v": m.w_qkv[c:], q + "o": m.w_o})
                out[q + "vmix"] = (m.vmix if m.vmix is not None else layer.vmix_unread).reshape(())
            ff, f = layer.ff, p + "mlp."
            if ff is None:
                continue
            out[f + "router"], out[f + "correction"] = ff.w_router, ff.bias
            for e in range(ff.E):
                out[f"{f}e{e}.gate"], out[f"{f}e{e}.up"], out[f"{f}e{e}.down"] = ff.w_up[e, :ff.ff], ff.w_up[e, ff.ff:], ff.w_down[e]
            if ff.shared_ff:
                s = ff.shared_ff
                out.update({f + "shared.gate": ff.w_sup[:s], f + "shared.up": ff.w_sup[s:2 * s], f + "shared.sg": ff.w_sup[2 * s:2 * s + 1],
                            f + "shared.down": ff.w_sdown})
        return {k: v.detach().clone().contiguous() for k, v in out.items()}


def load_pamazen(ck: Path, cfg: PamazenConfig, device=None, dtype=torch.bfloat16) -> PamazenLM:
    from safetensors import safe_open

    with safe_open(str(ck / "model.safetensors"), framework="pt", device="cpu") as f:
        W = {k: f.get_tensor(k) for k in f.keys()}
    # a size that only the tensors give: the rank of the decay projection
    for i, spec in enumerate(cfg.layer_specs):
        if spec["type"] == "parallel":
            cfg.decay_ranks[i] = int(W[f"l{i}.mix.right.w1"].shape[0])
    model = PamazenLM(cfg, device=device, dtype=dtype)
    model.load_named(W)
    return model


def pamazen_template(width: int = 256, layers: int = 4, heads: int = 4, kv_heads: int = 2, vocab: int = 512, every: int = 3,
                     experts: int = 8, top: int = 2, expert_ff: Optional[int] = None, head_dim: Optional[int] = None,
                     streams: int = 4, window: int = 1024, identity: int = 0, groups: int = 1) -> PamazenConfig:
    """A random-init configuration for benchmarks and smoke runs: rotary attention in every layer but each
    ``every``-th, which is the parallel pair of windowed attention and delta-rule memory; routed gated experts with
    a shared one."""
    d = head_dim or width // heads
    att = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d, "scale": d ** -0.5, "v_mix": True,
           "rot": {"base": 10000.0, "dims": d // 2 * 2, "scaling": {"factor": 8.0}}}
    par = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d, "scale": d ** -0.5, "softcap": 50.0,
                    "mask": {"size": window, "keep_first": 8}},
           "right": {"heads": heads, "dim": max(d // 2, 1)}, "left_scale": 0.5, "right_scale": 0.5}
    ff = expert_ff or width // 2
    mlp = {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": ff},
           "router": {"experts": experts, "top": top, "identity": identity, "groups": {"count": groups, "keep": max(groups // 2, 1)}}}
    specs = [{"type": "parallel" if (i + 1) % every == 0 else "attention",
              "mixer": copy.deepcopy(par if (i + 1) % every == 0 else att), "mlp": copy.deepcopy(mlp)} for i in range(layers)]
    return PamazenConfig(name=f"pamazen-w{width}-l{layers}", vocab_size=vocab, hidden=width, layer_specs=specs,
                         layer_norm_eps=1e-6, residual_mult=0.5, streams=streams, logit_softcap=30.0,
                         decay_ranks={i: max(width // 32, 4) for i, s in enumerate(specs) if s["type"] == "parallel"})
