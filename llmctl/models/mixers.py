"""Sequence mixers beside softmax attention, for serving steps over packed tokens.

* :class:`LatentAttention` — attention whose keys and values are up-projections of one small
  latent per token; only the latent and one rotary key part shared by all heads are cached.  With
  ``k = W_uk c`` the score ``q . k`` equals ``(W_uk^T q) . c``, so the step carries the query into the
  latent space once and attends the cache rows directly (one "head" of width ``rank + rot`` serves all
  query heads), and the value up-projection is applied to the attended latent afterwards.  Options:
  sliding window, a per-head softmax sink, a sigmoid output gate, a low-rank query path.
* :class:`GroupedAttention` — grouped-query softmax attention over a paged row cache ``[v | k]`` per
  kv head, with the options of small recent designs as parameters: short causal convolutions on the
  projected q / k / v, per-head RMS norm of q and k, rotary positions (neighbour or half pairs, YaRN
  or linear frequency scaling), values turned by their position and the head outputs turned back, a learned
  per-head temperature, capped scores, chunked or windowed masks, a window that spares the first tokens, a learned or
  fixed softmax sink, values that are the key projection's output, values blended with an earlier layer's.
* :class:`CausalConv` — a short causal convolution over time per channel, its last inputs carried in a
  state slot; :class:`ClampedGLU` — a gated feed-forward with clamped branches.
* :class:`GatedLinearAttention` — a matrix memory per head whose key rows decay by a data-dependent
  factor per key channel (low-rank decay projection, temperature ``tau``), read out with the query,
  RMS-normed per head and gated by ``silu``; its state lives in a slot pool like the mLSTM's.
* :class:`SigmoidAttention` — grouped-query causal attention without softmax over the same paged row
  cache ``[v | k]``: biases on q / k / v, RMS norm over the whole of q and of k, a query temperature that
  grows with the logarithm of the position, a logarithmic distance penalty per head, key weights
  ``sigmoid(score + head bias)`` that are not normalised, one sigmoid output gate per head.
* :class:`DenseFF` — an ungated feed-forward ``W_down act(W_up h)``.
* :class:`DeltaRule` — the generalized delta rule: a matrix memory per head that decays per key channel, removes
  what it holds along the current unit key at a learned rate and then writes ``k v^T``; low-rank decay projection
  through a ``tanh``, per-head unit RMS, weight and sigmoid gate on the read-out; state in a slot pool.
* :class:`ParallelMixers` — two mixers on the same input whose results are added with fixed factors (one input GEMM
  on the stacked weights; paged rows for the one, state pools for the other).
* :class:`MLSTM` — the xLSTM matrix memory: per head a ``[dk, dv]`` state with exponential input gate,
  sigmoid forget gate (both soft-capped) and a running log-scale stabiliser; state lives in a slot
  pool of the engine's cache, one slot per live sequence.

The mixers take ``side`` extra output rows on their fused input projection (a layer's own gate or
the like, which reads the same input) and hand those columns back beside their result.

All read a :class:`StepBatch` (the engine's description of one step: packed prompt portions first,
then one row per decoding sequence) and the layer's part of the engine's cache.  Projections are
vendor GEMMs on fused weights; everything else is a kernel of :mod:`llmctl.ops.hybrid`.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from llmctl.ops import hybrid as hops


@dataclass
class StepBatch:
    """One engine step over T packed tokens: rows [0, Tp) are prompt portions of ``len(p_ctx)``
    sequences (row offsets ``p_cu``), rows [Tp, T) one decoded token each."""
    ids: torch.Tensor  # int64 [T]
    pos: torch.Tensor  # int32 [T]
    slots: torch.Tensor  # int64 [T] cache slot of every token (block * block_size + offset)
    Tp: int
    p_cu: Optional[torch.Tensor]  # int32 [np + 1]
    p_ctx: Optional[torch.Tensor]  # int32 [np] context length after the step
    p_bt: Optional[torch.Tensor]  # int32 [np, max_blocks]
    d_ctx: Optional[torch.Tensor]  # int32 [nd]
    d_bt: Optional[torch.Tensor]  # int32 [nd, max_blocks]
    # all sequences (portions, then decodes): row offsets, first position, recurrent-state slot
    cu: torch.Tensor  # int32 [n + 1]
    start: torch.Tensor  # int32 [n]
    state: torch.Tensor  # int32 [n]
    max_q: int = 0  # the longest prompt portion of the step
    cu_host: Optional[list] = None  # ``cu`` on the host (chunk-parallel scans split long portions)
    seq_of: Optional[torch.Tensor] = None  # int32 [T] index (into cu / start / state) of every row's sequence
    d_max_ctx: int = 0  # the longest context among the decoding sequences
    fresh: bool = False  # every row belongs to a prompt portion that starts at position 0 (no earlier context)
    scratch: dict = field(default_factory=dict)  # what layers derive from the step alone and share (chunk plans of scans)


def rotary_frequencies(base: float, dims: int, scaling: Optional[dict] = None, device=None):
    """Per-pair rotary frequencies ``base^(-2i/dims)`` (fp32 ``[dims/2]``) and the factor on cos and sin.
    ``scaling`` = ``{factor, original, fast, slow}`` applies YaRN: with ``where(t) = dims ln(original /
    (2 pi t)) / (2 ln base)`` the pairs below ``floor(where(fast))`` keep their frequency, those above
    ``ceil(where(slow))`` are divided by ``factor``, a linear ramp lies between; cos and sin are multiplied
    by ``0.1 ln(factor) + 1``.  ``scaling`` = ``{factor}`` alone is linear scaling: every frequency is divided
    by ``factor``."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(dims, 1))
    amp = 1.0
    if scaling and "original" not in scaling:
        f = f / float(scaling.get("factor", 1.0))
    elif scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        where = lambda t: dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(float(base)))
        lo = max(math.floor(where(float(scaling["fast"]))), 0)
        hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device), amp


def _init(t: torch.Tensor, std: float) -> None:
    with torch.no_grad():
        t.normal_(0.0, std)


class LatentAttention(nn.Module):
    """Options: ``q_rank`` None = a full-rank query projection; ``window`` None = plain causal; ``sink``
    / ``gate`` False = no softmax sink / no sigmoid output gate; ``rot_scaling`` = YaRN (see
    :func:`rotary_frequencies`); ``interleaved`` = rotary pairs are neighbours (2i, 2i+1), not halves."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, q_rank: Optional[int],
                 rot_base: float, rot_dims: int, scale: float, window: Optional[int], eps: float, device=None, dtype=None,
                 sink: bool = True, gate: bool = True, rot_scaling: Optional[dict] = None, interleaved: bool = False):
        super().__init__()
        self.width, self.H, self.dn, self.dr, self.dv = width, heads, dim, rot_dim, vdim
        self.rk, self.qr, self.rot_dims, self.scale, self.eps = kv_rank, q_rank, rot_dims, scale, eps
        self.window = int(window) if window else hops.NO_LIMIT
        self.has_gate, self.interleaved = gate, interleaved
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError("rotary dims must be even and fit the rotated part")
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        # one GEMM for everything that reads the layer input: [W_dq or W_q ; W_dkv ; W_g]
        self.q_cols = q_rank if q_rank else heads * (dim + rot_dim)
        self.w_in = nn.Parameter(torch.empty(self.q_cols + kv_rank + rot_dim + (heads * vdim if gate else 0), width, **kw))
        self.w_uq = nn.Parameter(torch.empty(heads * (dim + rot_dim), q_rank, **kw)) if q_rank else None
        self.w_uk = nn.Parameter(torch.empty(heads, dim, kv_rank, **kw))  # per head [dn, rank]
        self.w_uv = nn.Parameter(torch.empty(heads, vdim, kv_rank, **kw))  # per head [dv, rank]
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        self.q_norm = nn.Parameter(torch.ones(q_rank, **f32)) if q_rank else None
        self.kv_norm = nn.Parameter(torch.ones(kv_rank, **f32))
        self.sink = nn.Parameter(torch.zeros(heads, **f32)) if sink else None
        for w in (self.w_in, self.w_uq, self.w_uk, self.w_uv, self.w_o):
            if w is not None:
                _init(w, 0.02)
        inv_freq, self.rot_amp = rotary_frequencies(rot_base, rot_dims, rot_scaling, device)
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    cache_kind = "latent"

    @property
    def cache_row(self) -> int:
        return self.rk + self.dr

    def state_shapes(self):
        return []

    EXPAND_MIN_TOKENS = 128

    def _expand(self, b: StepBatch) -> bool:
        """Whole prompts (no earlier context) attend per-head keys and values expanded from the step's own
        latents when that is the cheaper product: a score then costs dim + rot and a value vdim per head
        instead of rank + rot and rank.  Steps with earlier context, and decode rows, attend the cached rows."""
        return (b.fresh and b.Tp >= self.EXPAND_MIN_TOKENS
                and 2 * self.rk + self.dr > 2 * (self.dn + self.dr + self.dv))

    def _w_uvk(self) -> torch.Tensor:
        """[W_uv ; W_uk] per head as one weight [H * (vdim + dim), rank] (made once; serving weights are static)."""
        key = (self.w_uv.data_ptr(), self.w_uv._version, self.w_uk._version)
        if getattr(self, "_uvk_key", None) != key:
            self._uvk = torch.cat([self.w_uv.detach(), self.w_uk.detach()], 1).reshape(-1, self.rk).contiguous()
            self._uvk_key = key
        return self._uvk

    def _attend_expanded(self, q: torch.Tensor, b: StepBatch, cache: torch.Tensor) -> torch.Tensor:
        T, H, dn, dr, dv = q.shape[0], self.H, self.dn, self.dr, self.dv
        lat = cache.view(-1, self.rk + dr).index_select(0, b.slots)  # the rows just written: [latent | rotary key]
        rows = torch.empty(T, H, dv + dn + dr, device=q.device, dtype=q.dtype)  # per head [v | k | shared rotary key]
        rows[:, :, :dv + dn] = F.linear(lat[:, :self.rk], self._w_uvk()).view(T, H, dv + dn)
        rows[:, :, dv + dn:] = lat[:, None, self.rk:]
        qa = hops.latent_q_assemble(q[:, :, :dn], q, b.pos, self.inv_freq, self.rot_dims, dn, self.interleaved, self.rot_amp)
        # the step's rows as a cache of one-token pages: sequence n's position j is row p_cu[n] + j
        bt = (b.p_cu[:-1, None] + torch.arange(b.max_q, device=q.device, dtype=torch.int32)[None, :]).clamp_(max=T - 1)
        o = hops.latent_attention_prefill(qa, rows.view(T, 1, -1), bt.contiguous(), b.p_cu, b.p_ctx, self.window, self.sink,
                                          self.scale, dv, b.max_q, groups=H, koff=dv)
        return o.reshape(T, H * dv)

    def step(self, h: torch.Tensor, b: StepBatch, cache) -> torch.Tensor:
        if isinstance(cache, tuple):  # (paged rows, recurrent states): this mixer keeps no state
            cache = cache[0]
        T, H = h.shape[0], self.H
        z = F.linear(h, self.w_in)
        a, c = self.q_cols, self.q_cols + self.rk + self.dr
        hops.latent_kv_write(z[:, a:c], self.kv_norm, self.eps, b.pos, self.inv_freq, self.rot_dims, cache, b.slots,
                             self.interleaved, self.rot_amp)
        if self.qr:
            cq = hops.rmsnorm_cols(z[:, :a], self.q_norm, self.eps, self.qr, h.dtype)
            q = F.linear(cq, self.w_uq).view(T, H, self.dn + self.dr)
        else:
            q = z[:, :a].unflatten(1, (H, self.dn + self.dr))  # a view: rows keep z's pitch
        if self._expand(b):
            o = self._attend_expanded(q, b, cache)
            if self.has_gate:
                o = hops.sigmoid_gate_mul(o, z[:, c:])
            return F.linear(o, self.w_o)
        q_lat = torch.bmm(q[:, :, :self.dn].transpose(0, 1), self.w_uk).transpose(0, 1)  # [T, H, rank]
        qa = hops.latent_q_assemble(q_lat, q, b.pos, self.inv_freq, self.rot_dims, self.dn, self.interleaved, self.rot_amp)
        outs = []
        if b.Tp:
            outs.append(hops.latent_attention_prefill(qa[:b.Tp], cache, b.p_bt, b.p_cu, b.p_ctx, self.window,
                                                      self.sink, self.scale, self.rk, b.max_q))
        if T > b.Tp:
            outs.append(hops.latent_attention_decode(qa[b.Tp:], cache, b.d_bt, b.d_ctx, self.window, self.sink,
                                                     self.scale, self.rk, max_ctx=b.d_max_ctx))
        o_lat = outs[0] if len(outs) == 1 else torch.cat(outs)
        o = torch.bmm(o_lat.transpose(0, 1), self.w_uv.transpose(1, 2)).transpose(0, 1).reshape(T, H * self.dv)
        if self.has_gate:
            o = hops.sigmoid_gate_mul(o, z[:, c:])
        return F.linear(o, self.w_o)


class CausalConv(nn.Module):
    """A short causal convolution over time on every channel (weights fp32 ``[channels, taps]``):
    ``y_t = (u_t if residual) + sum_j w[:, j] u_(t - taps + 1 + j)``; the last ``taps - 1`` inputs of a
    sequence are its state (one fp32 ``[taps - 1, channels]`` entry per state slot)."""

    def __init__(self, channels: int, taps: int, residual: bool, device=None):
        super().__init__()
        self.channels, self.taps, self.residual = channels, taps, residual
        self.weight = nn.Parameter(torch.zeros(channels, taps, device=device, dtype=torch.float32))
        self._wt, self._wt_key = None, None

    def state_shape(self):
        return (self.taps - 1, self.channels)

    def tap_major(self) -> torch.Tensor:
        """The weights as the kernels read them, ``[taps, channels]`` (made once; serving weights are static)."""
        w = self.weight
        if self._wt is None or self._wt_key != (w.data_ptr(), w._version, w.device):
            self._wt, self._wt_key = w.detach().t().contiguous(), (w.data_ptr(), w._version, w.device)
        return self._wt

    def forward(self, u: torch.Tensor, b: StepBatch, state: torch.Tensor) -> torch.Tensor:
        return hops.causal_conv(u, self.tap_major(), state, b.seq_of, b.cu, b.start, b.state, self.residual,
                                max_len=max(b.max_q, 1 if u.shape[0] > b.Tp else 0))


class GroupedAttention(nn.Module):
    """Grouped-query attention (``heads`` query heads over ``kv_heads`` key / value heads; key size
    ``dim``, value size ``vdim``) with, each optional: ``conv_taps`` short causal convolutions on the
    projected q, k, v; ``qk_norm``: per-head RMS norm of q and k; rotary on the first ``rot_dims`` entries (YaRN
    or linear scaling by ``rot_scaling``, neighbour pairs when ``interleaved``); ``rotate_values``: the value of position j
    is cached turned by ``j * rot_base^(-2m/vdim)`` per pair m and a head's output at position i is
    turned back by i, so the sum weighs values by their relative position; ``temperature``: a learned
    per-head factor on the scaled scores; ``softcap`` c: the scaled score becomes ``c tanh(score / c)``;
    ``chunk``: position i sees j <= i of its own chunk of that many positions only; ``window``, of which
    ``keep_first`` exempts the first positions of the sequence; ``sink``: True = a learned per-head logit that
    joins the softmax denominator (not scaled, not capped, no value), a number = that logit fixed for all heads
    (0.0: one is added to the denominator).  ``values="keys"``: there is no value projection; a token's value is
    the output of its key projection, taken ahead of norm and rotary.  ``value_mix``: ``"source"`` leaves the step's projected values
    where a later layer finds them, ``"mix"`` replaces v by ``(1 - vmix) v + vmix v_source`` (same token, one learned
    number) before it is cached.  The cache row of a token is ``[v | k]`` per kv head."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, rot_base: float, rot_dims: int,
                 scale: float, eps: float, conv_taps: int = 0, rot_scaling: Optional[dict] = None,
                 interleaved: bool = True, rotate_values: bool = False, temperature: bool = False,
                 chunk: Optional[int] = None, window: Optional[int] = None, sink=False, qk_norm: bool = True,
                 values: str = "own", value_mix: Optional[str] = None, softcap: float = 0.0, keep_first: int = 0,
                 device=None, dtype=None):
        super().__init__()
        if heads % kv_heads or rot_dims % 2 or rot_dims > dim:
            raise ValueError("kv heads must divide the heads; rotary dims must be even and fit the head")
        if rotate_values and (vdim % 2 or not interleaved):
            raise ValueError("turned values need an even value size and neighbour pairs")
        if values not in ("own", "keys") or (values == "keys" and (vdim != dim or rotate_values or value_mix or conv_taps)):
            raise ValueError("values that are the keys have the keys' size and are neither turned, mixed nor convolved")
        if value_mix not in (None, "source", "mix"):
            raise ValueError("value_mix: None, 'source' or 'mix'")
        self.width, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.rot_dims, self.scale, self.eps, self.interleaved = rot_dims, scale, eps, interleaved
        self.chunk = int(chunk) if chunk else hops.NO_LIMIT
        self.window = int(window) if window else hops.NO_LIMIT
        self.softcap, self.keep_first = float(softcap or 0.0), int(keep_first or 0)
        self.v_from_k, self.value_mix = values == "keys", value_mix
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        cols = (heads + kv_heads) * dim + (0 if self.v_from_k else kv_heads * vdim)
        self.cols = cols
        self.w_qkv = nn.Parameter(torch.empty(cols, width, **kw))  # [W_q ; W_k ; W_v]: the input is read once
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        self.conv = CausalConv(cols, conv_taps, residual=False, device=device) if conv_taps else None
        self.q_norm = nn.Parameter(torch.ones(dim, **f32)) if qk_norm else None
        self.k_norm = nn.Parameter(torch.ones(dim, **f32)) if qk_norm else None
        self.temp = nn.Parameter(torch.ones(heads, **f32)) if temperature else None
        if sink is True:
            self.sink = nn.Parameter(torch.zeros(heads, **f32))
        elif sink is False or sink is None:
            self.sink = None
        else:
            self.register_buffer("sink", torch.full((heads,), float(sink), **f32), persistent=False)
        self.vmix = nn.Parameter(torch.zeros(1, **f32)) if value_mix else None
        for w in (self.w_qkv, self.w_o):
            _init(w, 0.02)
        inv_freq, self.rot_amp = rotary_frequencies(rot_base, rot_dims, rot_scaling, device)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        vf = rotary_frequencies(rot_base, vdim, None, device)[0] if rotate_values else None
        self.register_buffer("v_freq", vf, persistent=False)

    cache_kind = "latent"  # a paged pool of rows
    VALUE_SOURCE = "values_of_first_mixing_layer"  # key in StepBatch.scratch

    @property
    def cache_row(self) -> int:
        return self.G * (self.dv + self.dk)

    @property
    def w_in(self):
        return self.w_qkv

    def state_shapes(self):
        return [self.conv.state_shape()] if self.conv is not None else []

    def step(self, h: torch.Tensor, b: StepBatch, cache, z: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``z``: the input projection ``h W_qkv^T`` if the caller has made it (as columns of a wider product)."""
        rows, states = cache if isinstance(cache, tuple) else (cache, ())
        T = h.shape[0]
        if z is None:
            z = F.linear(h, self.w_qkv)
        if self.conv is not None:
            z = self.conv(z, b, states[0])
        v_first = None
        if self.value_mix is not None:
            v0 = (self.H + self.G) * self.dk
            if self.value_mix == "source":
                b.scratch[self.VALUE_SOURCE] = z[:, v0:v0 + self.G * self.dv]
            else:
                v_first = b.scratch[self.VALUE_SOURCE]
        q = hops.attn_qkv_prep(z, self.H, self.G, self.dk, self.dv, self.q_norm, self.k_norm, self.eps, b.pos,
                               self.inv_freq, self.rot_dims, self.interleaved, self.rot_amp, self.v_freq, rows, b.slots,
                               v_from_k=self.v_from_k, v_first=v_first, v_lambda=self.vmix if v_first is not None else None)
        opt = dict(groups=self.G, koff=self.dv, chunk=self.chunk, hscale=self.temp, ofreq=self.v_freq,
                   softcap=self.softcap, keep_first=self.keep_first)
        outs = []
        if b.Tp:
            outs.append(hops.latent_attention_prefill(q[:b.Tp], rows, b.p_bt, b.p_cu, b.p_ctx, self.window, self.sink,
                                                      self.scale, self.dv, b.max_q, **opt))
        if T > b.Tp:
            outs.append(hops.latent_attention_decode(q[b.Tp:], rows, b.d_bt, b.d_ctx, self.window, self.sink, self.scale,
                                                     self.dv, max_ctx=b.d_max_ctx, **opt))
        o = outs[0] if len(outs) == 1 else torch.cat(outs)
        return F.linear(o.reshape(T, self.H * self.dv), self.w_o)


class ClampedGLU(nn.Module):
    """Gated feed-forward with clamped branches: ``g = min(W_gate h, limit)``, ``u = clamp(W_up h,
    -limit, limit)``, ``W_down (g sigmoid(alpha g) (u + 1))``; gate and up are one weight."""

    def __init__(self, width: int, ff: int, limit: float, alpha: float = 1.702, device=None, dtype=None):
        super().__init__()
        self.ff, self.limit, self.alpha = ff, float(limit), float(alpha)
        self.w_gu = nn.Parameter(torch.empty(2 * ff, width, device=device, dtype=dtype))
        self.w_down = nn.Parameter(torch.empty(width, ff, device=device, dtype=dtype))
        _init(self.w_gu, 0.02)
        _init(self.w_down, 0.02)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(hops.clamped_glu(F.linear(h, self.w_gu), self.limit, self.alpha), self.w_down)


class MLSTM(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, device=None,
                 dtype=None):
        super().__init__()
        self.width, self.H, self.dk, self.dv, self.cap, self.eps = width, heads, dim, vdim, float(gate_cap), eps
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        # [W_q ; W_k ; W_v ; W_g] in one GEMM; the two gate rows per head stay fp32
        self.w_in = nn.Parameter(torch.empty(2 * heads * dim + 2 * heads * vdim, width, **kw))
        self.w_if = nn.Parameter(torch.empty(2 * heads, width, **f32))
        self.b_i = nn.Parameter(torch.zeros(heads, **f32))
        self.b_f = nn.Parameter(torch.full((heads,), 3.0, **f32))
        self.norm = nn.Parameter(torch.ones(heads * vdim, **f32))
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        for w in (self.w_in, self.w_if, self.w_o):
            _init(w, 0.02)

    cache_kind = "state"

    def state_shapes(self):
        return [(self.H, self.dk, self.dv), (self.H, self.dk), (self.H,)]

    def step(self, h: torch.Tensor, b: StepBatch, state) -> torch.Tensor:
        T, H, dk, dv = h.shape[0], self.H, self.dk, self.dv
        z = F.linear(h, self.w_in)
        q, k = z[:, :H * dk].view(T, H, dk), z[:, H * dk:2 * H * dk].view(T, H, dk)
        v = z[:, 2 * H * dk:2 * H * dk + H * dv].view(T, H, dv)
        g = z[:, 2 * H * dk + H * dv:]
        gates = F.linear(h.float(), self.w_if)  # fp32 [T, 2H]
        S, n, m = state
        o = hops.mlstm_scan(q, k, v, gates, self.b_i, self.b_f, self.cap, 1.0 / math.sqrt(dk), S, n, m, b.state,
                            b.cu, b.start, cu_host=b.cu_host)
        return F.linear(hops.headnorm_gate(o, self.norm, g, self.eps, h.dtype), self.w_o)


def _mm_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w^T`` with an fp32 result (inputs in their own dtype, fp32 accumulation)."""
    if x.dtype == torch.float32:
        return F.linear(x, w)
    try:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    except (TypeError, RuntimeError):
        return F.linear(x, w).float()


class GatedLinearAttention(nn.Module):
    """Per head a memory ``S [dim, vdim]``: ``S_t = diag(a_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` with
    ``q = W_q h * dim^-1/2`` and the decay ``a_t = sigmoid(W_a2 (W_a1 h) + b)^(1/tau)`` per key channel.
    Each head's ``o`` is RMS-normed over vdim (one weight ``[vdim]`` for all heads), the heads are
    concatenated, multiplied by ``silu(W_g h)`` and projected by ``W_o``.  The fused input weight is
    ``[W_q ; W_k ; W_v ; W_g ; W_a1 ; side rows]``."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, tau: float, decay_rank: int, eps: float,
                 side: int = 0, device=None, dtype=None):
        super().__init__()
        self.width, self.H, self.dk, self.dv, self.tau, self.rank, self.eps = width, heads, dim, vdim, float(tau), decay_rank, eps
        self.side = side
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        self.cols = 2 * heads * dim + 2 * heads * vdim + decay_rank
        self.w_in = nn.Parameter(torch.empty(self.cols + side, width, **kw))
        self.b_in = nn.Parameter(torch.zeros(self.cols + side, **kw)) if side else None  # only side rows carry a bias
        self.w_a2 = nn.Parameter(torch.empty(heads * dim, decay_rank, **kw))
        self.b_a2 = nn.Parameter(torch.zeros(heads * dim, **f32))
        self.norm = nn.Parameter(torch.ones(vdim, **f32))
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        for w in (self.w_in, self.w_a2, self.w_o):
            _init(w, 0.02)
        self._nw = None

    cache_kind = "state"
    cache_row = 0

    def state_shapes(self):
        return [(self.H, self.dk, self.dv)]

    def _norm_rows(self) -> torch.Tensor:
        """The per-head norm weight repeated for every head (made once; serving weights are static)."""
        key = (self.norm.data_ptr(), self.norm._version, self.norm.device)
        if self._nw is None or self._nw[0] != key:
            self._nw = (key, self.norm.detach().repeat(self.H).contiguous())
        return self._nw[1]

    def step(self, h: torch.Tensor, b: StepBatch, state):
        if isinstance(state, tuple) and len(state) == 2 and isinstance(state[1], tuple):  # (rows, states)
            state = state[1]
        T, H, dk, dv = h.shape[0], self.H, self.dk, self.dv
        z = F.linear(h, self.w_in, self.b_in)
        a, c, e = H * dk, 2 * H * dk, 2 * H * dk + H * dv
        q, k = z[:, :a].unflatten(1, (H, dk)), z[:, a:c].unflatten(1, (H, dk))
        v = z[:, c:e].unflatten(1, (H, dv))
        g = z[:, e:e + H * dv]
        decay = _mm_f32(z[:, e + H * dv:self.cols], self.w_a2)  # fp32 [T, H * dk]
        if "gla_plan" not in b.scratch:
            b.scratch["gla_plan"] = hops.gla_chunk_plan(b.cu_host, h.device) if h.is_cuda else None
        o = hops.gla_scan(q, k, v, decay, self.b_a2, self.tau, dk ** -0.5, state[0], b.state, b.cu, b.start,
                          plan=b.scratch["gla_plan"])
        y = F.linear(hops.headnorm_gate(o, self._norm_rows(), g, self.eps, h.dtype, silu=True), self.w_o)
        return (y, z[:, self.cols:]) if self.side else y


class SigmoidAttention(nn.Module):
    """Grouped-query causal attention whose key weights are ``sigmoid(score + bias_h)``, not a softmax
    (``heads`` query heads over ``kv_heads`` key / value heads; key size ``dim``, value size ``vdim``):
    q, k, v with biases; RMS norm over all of q and all of k before the split into heads; no rotation;
    ``q *= 1 + temp_coef ln(floor((p + 1) / temp_every) + 1)`` at position p; ``score = q . k * scale -
    r1_h ln(1 + r2_h (i - j))``; head h's output times ``sigmoid(W_g h)_h``.  The cache row of a token is
    ``[v | k]`` per kv head; the fused input weight is ``[W_q ; W_k ; W_v ; W_g ; side rows]``."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
                 temp_coef: float = 0.0, temp_every: int = 1, window: Optional[int] = None, side: int = 0,
                 device=None, dtype=None):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("kv heads must divide the heads")
        self.width, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.scale, self.eps, self.temp_coef, self.temp_every = float(scale), eps, float(temp_coef), int(temp_every)
        self.window = int(window) if window else hops.NO_LIMIT
        self.side = side
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        self.cols = (heads + kv_heads) * dim + kv_heads * vdim + heads
        self.w_in = nn.Parameter(torch.empty(self.cols + side, width, **kw))
        self.b_in = nn.Parameter(torch.zeros(self.cols + side, **kw))
        self.q_norm = nn.Parameter(torch.ones(heads * dim, **f32))
        self.k_norm = nn.Parameter(torch.ones(kv_heads * dim, **f32))
        self.dist_a = nn.Parameter(torch.zeros(heads, **f32))  # r1
        self.dist_b = nn.Parameter(torch.zeros(heads, **f32))  # r2
        self.bias = nn.Parameter(torch.zeros(heads, **f32))
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        for w in (self.w_in, self.w_o):
            _init(w, 0.02)

    cache_kind = "latent"  # a paged pool of rows

    @property
    def cache_row(self) -> int:
        return self.G * (self.dv + self.dk)

    def state_shapes(self):
        return []

    def step(self, h: torch.Tensor, b: StepBatch, cache):
        rows = cache[0] if isinstance(cache, tuple) else cache
        T, H, G, dk, dv = h.shape[0], self.H, self.G, self.dk, self.dv
        z = F.linear(h, self.w_in, self.b_in)
        q = hops.qk_fullnorm_prep(z, H, G, dk, dv, self.q_norm, self.k_norm, self.eps, b.pos, self.temp_coef,
                                  self.temp_every, rows, b.slots)
        opt = dict(groups=G, koff=dv, sig_bias=self.bias, dist_a=self.dist_a, dist_b=self.dist_b)
        outs = []
        if b.Tp:
            outs.append(hops.latent_attention_prefill(q[:b.Tp], rows, b.p_bt, b.p_cu, b.p_ctx, self.window, None,
                                                      self.scale, dv, b.max_q, **opt))
        if T > b.Tp:
            outs.append(hops.latent_attention_decode(q[b.Tp:], rows, b.d_bt, b.d_ctx, self.window, None, self.scale, dv,
                                                     max_ctx=b.d_max_ctx, **opt))
        o = outs[0] if len(outs) == 1 else torch.cat(outs)
        g0 = self.cols - H
        y = F.linear(hops.sigmoid_gate_mul(o.reshape(T, H * dv), z[:, g0:self.cols]), self.w_o)
        return (y, z[:, self.cols:]) if self.side else y


class DenseFF(nn.Module):
    """``W_down act(W_up h)`` with ``act`` one of :func:`llmctl.ops.hybrid.act_any`'s kinds; the up
    projection carries ``side`` extra output rows (with a bias) that are handed back."""

    def __init__(self, width: int, ff: int, act: str = "gelu", side: int = 0, device=None, dtype=None):
        super().__init__()
        self.ff, self.act, self.side = ff, act, side
        kw = dict(device=device, dtype=dtype)
        self.w_up = nn.Parameter(torch.empty(ff + side, width, **kw))
        self.b_up = nn.Parameter(torch.zeros(ff + side, **kw)) if side else None
        self.w_down = nn.Parameter(torch.empty(width, ff, **kw))
        _init(self.w_up, 0.02)
        _init(self.w_down, 0.02)

    def forward(self, h: torch.Tensor):
        z = F.linear(h, self.w_up, self.b_up)
        y = F.linear(hops.act_any(z[:, :self.ff], self.act), self.w_down)
        return (y, z[:, self.ff:]) if self.side else y


class DeltaRule(nn.Module):
    """The generalized delta rule: per head a memory ``S [dim, dim]`` with ``S_t = diag(w_t) S_(t-1) - (a_t u_t)
    (u_t^T S_(t-1)) + k_t v_t^T`` (both terms read the old memory) and ``o_t = S_t^T r_t``, where ``r, k, v = W_r h,
    W_k h, W_v h``, the decay per key channel is ``w = exp(-decay_coef sigmoid(W_w2 tanh(W_w1 h) + w0))``, the removal
    rate ``a = sigmoid(W_a h + b_a)`` and ``u = k / sqrt(sum k^2 + key_eps)`` the unit key of the head.  Each head's
    ``o`` is divided by its root mean square, the heads are concatenated, multiplied by the weight ``norm`` and by
    ``sigmoid(W_g h)``, then projected by ``W_o``.  The memory is fp32 and lives in a state slot per sequence.
    The fused input weight is ``[W_r ; W_k ; W_v ; W_g ; W_a ; W_w1]``."""

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, eps: float, decay_coef: float = math.exp(-0.5),
                 key_eps: float = 1e-6, device=None, dtype=None):
        super().__init__()
        self.width, self.H, self.d, self.rank, self.eps = width, heads, dim, decay_rank, eps
        self.decay_coef, self.key_eps = float(decay_coef), float(key_eps)
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        n = heads * dim
        self.cols = 5 * n + decay_rank
        self.w_in = nn.Parameter(torch.empty(self.cols, width, **kw))
        self.w_w2 = nn.Parameter(torch.empty(n, decay_rank, **kw))
        self.w0 = nn.Parameter(torch.zeros(n, **f32))
        self.b_a = nn.Parameter(torch.zeros(n, **f32))
        self.norm = nn.Parameter(torch.ones(n, **f32))
        self.w_o = nn.Parameter(torch.empty(width, n, **kw))
        for w in (self.w_in, self.w_w2, self.w_o):
            _init(w, 0.02)

    cache_kind = "state"
    cache_row = 0

    def state_shapes(self):
        return [(self.H, self.d, self.d)]

    def step(self, h: torch.Tensor, b: StepBatch, state, z: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(state, tuple) and len(state) == 2 and isinstance(state[1], tuple):  # (rows, states)
            state = state[1]
        T, H, d = h.shape[0], self.H, self.d
        n = H * d
        if z is None:
            z = F.linear(h, self.w_in)
        r, k, v = (z[:, i * n:(i + 1) * n].unflatten(1, (H, d)) for i in range(3))
        g, za = z[:, 3 * n:4 * n], z[:, 4 * n:5 * n]
        zw = _mm_f32(hops.tanh_act(z[:, 5 * n:self.cols]), self.w_w2)  # fp32 [T, H * d]
        if "gla_plan" not in b.scratch:
            b.scratch["gla_plan"] = hops.gla_chunk_plan(b.cu_host, h.device) if h.is_cuda else None
        o = hops.delta_scan(r, k, v, zw, self.w0, za, self.b_a, self.decay_coef, self.key_eps, state[0], b.state, b.cu,
                            b.start, plan=b.scratch["gla_plan"])
        return F.linear(hops.headnorm_gate(o, self.norm, g, self.eps, h.dtype), self.w_o)


class ParallelMixers(nn.Module):
    """Two mixers side by side on the same input: the result is ``left_scale * left(h) + right_scale * right(h)``.
    ``step`` returns the two results with their factors (the layer's residual pass sums them); both input
    projections run as one product on the stacked weights, so the input is read once.  The cache entry is the
    pair the members need: paged rows for the one that attends, state pools for the one that recurs."""

    def __init__(self, left: nn.Module, right: nn.Module, left_scale: float, right_scale: float):
        super().__init__()
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self._w, self._w_key = None, None

    @property
    def cache_kind(self):
        return "rows+state"

    @property
    def cache_row(self) -> int:
        return int(self.left.cache_row) + int(self.right.cache_row)

    def state_shapes(self):
        return list(self.left.state_shapes()) + list(self.right.state_shapes())

    def _stacked(self) -> torch.Tensor:
        """[W_in left ; W_in right] (made once; serving weights are static)."""
        a, c = self.left.w_in, self.right.w_in
        key = (a.data_ptr(), a._version, c.data_ptr(), c._version)
        if self._w_key != key:
            self._w, self._w_key = torch.cat([a.detach(), c.detach()], 0).contiguous(), key
        return self._w

    def step(self, h: torch.Tensor, b: StepBatch, cache):
        rows, states = cache
        nl = len(self.left.state_shapes())
        z = F.linear(h, self._stacked())
        cl = self.left.w_in.shape[0]
        yl = self.left.step(h, b, (rows, tuple(states[:nl])), z=z[:, :cl])
        yr = self.right.step(h, b, (rows, tuple(states[nl:])), z=z[:, cl:])
        return (yl, self.left_scale), (yr, self.right_scale)
