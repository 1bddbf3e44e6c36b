"""Mixture-of-experts MLP with expert parallelism (Mixtral-style top-k SwiGLU experts).

Not in the reference (SURVEY §2.3 "EP (expert parallel / MoE)": absent, all reference
templates are dense); added as a model family (``mixtral-8x7b``, ``tiny-moe``) with the EP
dimension the MI355X plan carries.

Per layer, on token-major activations ``x [T, h]``:

1. router: ``softmax(x W_r^T)`` in fp32, top-k experts per token, weights renormalised over
   the k picks; Switch/GShard load-balancing loss ``E * sum_e f_e * P_e`` (``f_e`` share of
   routed slots, ``P_e`` mean router probability) is kept on the module for the model loss;
2. dispatch: token copies are sorted by expert (one stable argsort) into contiguous
   per-expert segments;
3. expert parallel (``ep > 1``): experts are sharded rank-major over the EP group (rank j owns
   experts ``[j*E/ep, (j+1)*E/ep)``); per-expert counts go through one small all-to-all, then
   the token rows through a variable-split ``all_to_all_single`` (RCCL over the xGMI mesh: on
   a K8 node every pair of GPUs has its own link, so the all-to-all uses all 7 links at once);
   received rows are regrouped by local expert.  The only host sync per layer is the split
   sizes (dropless routing: no capacity factor, no dropped tokens);
4. experts: per local expert ``down(swiglu(up(x_e)))`` on its contiguous segment (hipBLASLt
   GEMMs + the SwiGLU HIP kernel on GPU);
5. the reverse all-to-all and a weighted ``index_add`` back to token order.

Gradients flow through the same path (the all-to-all's backward is the reverse all-to-all).
Expert parameters carry ``p.expert = True``: the engine reduces their gradients over the
expert-DP group instead of the full DP group (``llmctl.parallel.groups``).
"""

from __future__ import annotations

import math
from typing import List, Optional

import torch
import torch.distributed as dist
import torch.nn as nn

from llmctl import ops
from llmctl.exec.linear import linear


class _AllToAll(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, send_splits: List[int], recv_splits: List[int], group):
        ctx.group, ctx.send, ctx.recv = group, send_splits, recv_splits
        out = x.new_empty((sum(recv_splits),) + tuple(x.shape[1:]))
        dist.all_to_all_single(out, x.contiguous(), recv_splits, send_splits, group=group)
        return out

    @staticmethod
    def backward(ctx, g):
        out = g.new_empty((sum(ctx.send),) + tuple(g.shape[1:]))
        dist.all_to_all_single(out, g.contiguous(), ctx.send, ctx.recv, group=ctx.group)
        return out, None, None, None


class MoEMLP(nn.Module):
    def __init__(self, cfg, num_layers: int, ep_group=None, ep_size: int = 1, ep_rank: int = 0, device=None,
                 dtype=None):
        super().__init__()
        E, k = cfg.num_experts, cfg.experts_per_token
        if E % ep_size:
            raise ValueError(f"num_experts={E} not divisible by expert_parallel={ep_size}")
        self.E, self.k, self.ep, self.ep_group = E, k, ep_size, ep_group
        self.El = E // ep_size
        self.e0 = ep_rank * self.El  # global index of this rank's first expert
        h, f = cfg.hidden, cfg.moe_ffn
        kw = dict(device=device, dtype=dtype)
        self.w_router = nn.Parameter(torch.empty(E, h, **kw))
        self.experts_up = nn.ParameterList([nn.Parameter(torch.empty(2 * f, h, **kw)) for _ in range(self.El)])
        self.experts_down = nn.ParameterList([nn.Parameter(torch.empty(h, f, **kw)) for _ in range(self.El)])
        with torch.no_grad():
            self.w_router.normal_(0.0, 0.02)
            # every rank draws all E experts in order and keeps its own: the initial weights do
            # not depend on the EP layout (equivalence tests, resharding)
            for e in range(E):
                up = torch.empty(2 * f, h, **kw).normal_(0.0, 0.02)
                down = torch.empty(h, f, **kw).normal_(0.0, 0.02 / math.sqrt(2 * num_layers))
                if self.e0 <= e < self.e0 + self.El:
                    self.experts_up[e - self.e0].copy_(up)
                    self.experts_down[e - self.e0].copy_(down)
        for p in list(self.experts_up) + list(self.experts_down):
            p.expert = True
        self.aux_loss: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------ names (global expert ids)
    def global_expert_index(self, local: int) -> int:
        return self.e0 + local

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        T, h = x.shape
        E, k = self.E, self.k
        probs = linear(x, self.w_router).float().softmax(-1)  # [T, E]
        topw, topi = probs.topk(k, dim=-1)
        topw = topw / topw.sum(-1, keepdim=True)
        flat = topi.reshape(-1)  # [T*k] expert of each token copy
        counts = torch.bincount(flat, minlength=E)
        self.aux_loss = E * (counts.float() / float(T * k) * probs.mean(0)).sum()
        order = torch.argsort(flat, stable=True)
        tok = torch.div(order, k, rounding_mode="floor")
        xs = x.index_select(0, tok)  # token copies grouped by expert
        if self.ep > 1:
            g = self.ep_group
            cnt_recv = torch.empty_like(counts)
            dist.all_to_all_single(cnt_recv, counts, group=g)  # [src rank, local expert]
            host = torch.cat([counts, cnt_recv]).tolist()  # the layer's one host sync
            c_send = [sum(host[r * self.El:(r + 1) * self.El]) for r in range(self.ep)]
            c_recv2 = [host[E + r * self.El:E + (r + 1) * self.El] for r in range(self.ep)]
            c_recv = [sum(c) for c in c_recv2]
            xr = _AllToAll.apply(xs, c_send, c_recv, g)  # src-major, expert-minor
            # regroup the received rows by local expert (expert-major, src-minor)
            starts, o = [], 0
            for r in range(self.ep):
                row = []
                for e in range(self.El):
                    row.append(o)
                    o += c_recv2[r][e]
                starts.append(row)
            perm = [i for e in range(self.El) for r in range(self.ep)
                    for i in range(starts[r][e], starts[r][e] + c_recv2[r][e])]
            perm_t = torch.tensor(perm, dtype=torch.long, device=x.device)
            xe = xr.index_select(0, perm_t)
            local_counts = [sum(c_recv2[r][e] for r in range(self.ep)) for e in range(self.El)]
        else:
            xe = xs
            local_counts = counts.tolist()
        pad = self._pad_rows(xe, local_counts)
        if pad is not None:
            # every expert's rows padded with zero rows to a multiple of 256: all expert GEMMs -- the
            # token-deep weight gradients included -- then take gemm64's shapes (hipBLASLt's
            # weight-gradient layout runs ~1.0 PF); zero rows contribute zero outputs and gradients
            dst, padded = pad
            xp = xe.new_zeros((sum(padded), h)).index_copy(0, dst, xe)
            outs, o = [], 0
            for e, n in enumerate(padded):
                if n:
                    outs.append(linear(ops.swiglu(linear(xp[o:o + n], self.experts_up[e])), self.experts_down[e]))
                    o += n
            ye = torch.cat(outs, 0).index_select(0, dst) if outs else xe.new_zeros((0, h))
        else:
            ye = run_expert_segments(xe, local_counts, self.experts_up, self.experts_down)
        if self.ep > 1:
            inv = torch.empty_like(perm_t)
            inv[perm_t] = torch.arange(perm_t.numel(), device=x.device)
            ys = _AllToAll.apply(ye.index_select(0, inv), c_recv, c_send, self.ep_group)
        else:
            ys = ye
        w = topw.reshape(-1).index_select(0, order).to(ys.dtype).unsqueeze(-1)
        return torch.zeros_like(x).index_add(0, tok, ys * w)


    def _pad_rows(self, xe: torch.Tensor, counts: List[int]):
        """(destination row of every expert row in the padded buffer, padded count per expert), or
        None: GPU only (gemm64 shapes), knob ``moe_pad``."""
        from llmctl.config.knobs import knobs

        if not (knobs().moe_pad and xe.is_cuda and xe.dtype == torch.bfloat16 and xe.shape[1] % 128 == 0
                and self.experts_up[0].shape[0] % 256 == 0 and self.experts_down[0].shape[0] % 256 == 0
                and self.experts_down[0].shape[1] % 128 == 0):
            return None
        padded = [(n + 255) // 256 * 256 for n in counts]
        idx, o = [], 0
        for n, npad in zip(counts, padded):
            idx.append(torch.arange(o, o + n))
            o += npad
        dst = torch.cat(idx).to(xe.device, non_blocking=True) if idx else torch.zeros(0, dtype=torch.long,
                                                                                       device=xe.device)
        return dst, padded


def run_expert_segments(xe: torch.Tensor, counts: List[int], ups, downs, act=None, pad: int = 0) -> torch.Tensor:
    """``down_e(act(up_e(x)))`` on each expert's contiguous row segment of ``xe`` (rows sorted by
    expert, ``counts[e]`` rows each).

    ``pad`` > 0: an expert's GEMMs also take the rows that follow its segment, up to the next multiple of
    ``pad`` rows (of 16 for segments of at most 16 rows), and the results of those rows are dropped; ``xe``
    must then hold ``pad`` spare rows after the last segment.  The GEMM library picks a kernel per shape and
    remembers the pick: row counts that change with every step's routing cost ~60 us of host time per GEMM
    for the lookup, a few recurring ones cost none."""
    act = act or ops.swiglu
    outs, o = [], 0
    for e, n in enumerate(counts):
        if n == 0:
            continue
        m = n
        if pad:
            m = 16 if n <= 16 else (n + pad - 1) // pad * pad
            m = min(m, xe.shape[0] - o)
        y = linear(act(linear(xe[o:o + m], ups[e])), downs[e])
        outs.append(y[:n] if m != n else y)
        o += n
    return torch.cat(outs, 0) if outs else xe.new_zeros((0, downs[0].shape[0]))


class GroupLimitedMoE(nn.Module):
    """Routed SwiGLU experts with sigmoid scores and group-limited choice (serving forward).

    Router logits are an fp32 product; scores ``sigmoid(z)``; experts form ``groups`` equal groups of
    neighbours, a group is scored by the sum of its two best experts, only the ``keep`` best groups are
    eligible and the ``top`` best eligible experts are used, weighted by their own scores (no
    renormalisation).  Token copies are sorted by expert and run through per-expert GEMMs on
    contiguous segments (the dispatch of :class:`MoEMLP`); the weighted sum is accumulated in fp32."""

    def __init__(self, width: int, ff: int, experts: int, top: int, groups: int, keep: int, device=None, dtype=None):
        super().__init__()
        if experts % groups or not (0 < keep <= groups) or not (0 < top <= keep * (experts // groups)):
            raise ValueError("router: experts must split into equal groups and top must fit the kept groups")
        self.E, self.top, self.groups, self.keep, self.ff = experts, top, groups, keep, ff
        kw = dict(device=device, dtype=dtype)
        self.w_router = nn.Parameter(torch.empty(experts, width, device=device, dtype=torch.float32))
        self.experts_up = nn.ParameterList([nn.Parameter(torch.empty(2 * ff, width, **kw)) for _ in range(experts)])
        self.experts_down = nn.ParameterList([nn.Parameter(torch.empty(width, ff, **kw)) for _ in range(experts)])
        with torch.no_grad():
            self.w_router.normal_(0.0, 0.02)
            for p in list(self.experts_up) + list(self.experts_down):
                p.normal_(0.0, 0.02)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [T, width] -> fp32 [T, width]."""
        from llmctl.ops import hybrid as hops

        T = x.shape[0]
        topi, topw = hops.group_topk_router(torch.nn.functional.linear(x.float(), self.w_router), self.top,
                                            self.groups, self.keep)
        flat = topi.reshape(-1)
        counts = torch.bincount(flat, minlength=self.E).tolist()  # the layer's one host sync
        order = torch.argsort(flat, stable=True)
        tok = torch.div(order, self.top, rounding_mode="floor")
        ye = run_expert_segments(x.index_select(0, tok), counts, self.experts_up, self.experts_down, hops.swiglu_any)
        w = topw.reshape(-1).index_select(0, order).unsqueeze(-1)
        return torch.zeros(T, x.shape[1], dtype=torch.float32, device=x.device).index_add_(0, tok, ye.float() * w)


class BiasedSoftmaxMoE(nn.Module):
    """Routed experts chosen by softmax scores plus a selection bias (serving forward).  Router logits are an
    fp32 product; ``s = softmax(z)``; the ``top`` experts with the largest ``s + bias`` are used, weighted by their
    own ``s`` (over the sum of the chosen ones when ``renorm``); an optional shared expert of the same form runs
    for every token.  Experts: ``W_down act(W_up h)`` with ``act`` = ``relu2`` / ``gelu``, or gated, ``W_down
    (silu(W_gate h) * W_up h)``, with ``act="swiglu"`` (gate and up are one weight ``[gate ; up]``).  Options:
    ``groups`` / ``keep``: the router's outputs form equal groups of neighbours, a group scores as its best choice
    score, and only experts of the ``keep`` best groups can be chosen; ``identity``: the last that many router
    outputs are experts without weights whose output is their input; ``shared_gate``: the shared expert's output is
    multiplied by ``sigmoid(w_sg . h)``, one number per token, whose row rides on the shared up projection.
    Dispatch as in :class:`GroupLimitedMoE`
    (token copies sorted by expert, per-expert GEMMs on contiguous segments, fp32 weighted sum).  Steps of
    few tokens that between them reach about every expert anyway (decode batches) take the dense form
    instead: all experts on all rows in one up GEMM, one activation pass and one batched down GEMM on the
    stacked weights, the unchosen experts weighted by zero; that form has no host synchronisation and a
    quarter of the launches.  Longer steps run one pair of GEMMs per expert.  (A third form, all experts as one
    batch of equal-sized segments through two batched GEMMs on the stacked weights, is written and agrees with
    the others on the CPU and on small GPU steps, but a 2048-token step through it ended in a GPU memory fault
    whose cause is not found: ``BATCHED`` keeps it off on GPUs.)  The shared expert's up projection carries ``side`` extra output rows (with a
    bias) that are handed back; without a shared expert they are a projection of their own."""

    def __init__(self, width: int, ff: int, experts: int, top: int, act: str = "relu2", shared_ff: int = 0,
                 side: int = 0, groups: int = 1, keep: int = 1, renorm: bool = True, identity: int = 0,
                 shared_gate: bool = False, device=None, dtype=None):
        super().__init__()
        n = experts + identity
        if not (0 < top <= n):
            raise ValueError("router: top must lie in 1 .. experts")
        if groups < 1 or n % groups or not (0 < keep <= groups) or top > keep * (n // groups):
            raise ValueError("router: its outputs must split into equal groups and top must fit the kept groups")
        if shared_gate and not shared_ff:
            raise ValueError("a gate on the shared expert needs a shared expert")
        self.E, self.top, self.ff, self.act, self.shared_ff, self.side = experts, top, ff, act, shared_ff, side
        self.groups, self.keep, self.renorm, self.identity, self.shared_gate = groups, keep, renorm, identity, shared_gate
        self.up_rows = 2 * ff if act == "swiglu" else ff  # rows of an expert's first projection
        self.sup_rows = 2 * shared_ff if act == "swiglu" else shared_ff
        extra = self.sup_rows + (1 if shared_gate else 0) + side
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        self.w_router = nn.Parameter(torch.empty(n, width, **f32))
        self.bias = nn.Parameter(torch.zeros(n, **f32))
        self.w_up = nn.Parameter(torch.empty(experts, self.up_rows, width, **kw))  # stacked: expert e is w_up[e]
        self.w_down = nn.Parameter(torch.empty(experts, width, ff, **kw))
        self.w_sup = nn.Parameter(torch.empty(extra, width, **kw)) if extra else None
        self.b_sup = nn.Parameter(torch.zeros(extra, **kw)) if side else None
        self.w_sdown = nn.Parameter(torch.empty(width, shared_ff, **kw)) if shared_ff else None
        with torch.no_grad():
            self.w_router.normal_(0.0, 0.02)
            for p in (self.w_up, self.w_down, self.w_sup, self.w_sdown):
                if p is not None:
                    p.normal_(0.0, 0.02)

    @property
    def experts_up(self):
        return self.w_up.unbind(0)

    @property
    def experts_down(self):
        return self.w_down.unbind(0)

    PAD = 64  # expert segments run in multiples of this many rows
    DENSE_ROWS = 64  # steps of at most this many rows may take the dense form

    def _dense(self, T: int) -> bool:
        return T <= self.DENSE_ROWS and T * self.top >= self.E

    BATCHED = False  # the batched-segment form on GPUs: off (see the class docstring)

    def _batched(self, N: int, C: int) -> bool:
        """N token copies in segments padded to C rows each: worth it unless the padding doubles the work."""
        return (self.BATCHED or not self.w_up.is_cuda) and self.E * C <= 2 * N + self.E * self.PAD

    def _run_batched(self, xs: torch.Tensor, counts: List[int], C: int, act) -> torch.Tensor:
        """``xs``: the token copies sorted by expert, zero rows from row N on.  Gathers every expert's segment
        into ``[E, C, width]`` (missing rows = the zero row N), runs both projections as batched GEMMs and
        gathers the N real rows back in sorted order."""
        import numpy as np

        E, N, W = self.E, sum(counts), xs.shape[1]
        gi = np.full(E * C, N, dtype=np.int64)
        back = np.empty(N, dtype=np.int64)
        o = 0
        for e, n in enumerate(counts):
            gi[e * C:e * C + n] = np.arange(o, o + n)
            back[o:o + n] = np.arange(e * C, e * C + n)
            o += n
        # a blocking copy: the host array is a temporary, and an asynchronous copy from pageable memory of this
        # size may read it after it has been released
        both = torch.from_numpy(np.concatenate([gi, back])).to(xs.device)
        xg = xs.index_select(0, both[:E * C]).view(E, C, W)
        a = act(torch.bmm(xg, self.w_up.transpose(1, 2)).view(E * C, self.up_rows))
        y = torch.bmm(a.view(E, C, self.ff), self.w_down.transpose(1, 2)).view(E * C, W)
        return y.index_select(0, both[E * C:])

    def forward(self, x: torch.Tensor):
        """x [T, width] -> fp32 [T, width] (and the side columns)."""
        from llmctl.ops import hybrid as hops

        T = x.shape[0]
        act = hops.swiglu_any if self.act == "swiglu" else (lambda u: hops.act_any(u, self.act))
        topi, topw = hops.bias_topk_router(torch.nn.functional.linear(x.float(), self.w_router), self.bias, self.top,
                                           self.groups, self.keep, self.renorm)
        if self._dense(T):
            E, ff, W = self.E, self.ff, x.shape[1]
            a = act(torch.nn.functional.linear(x, self.w_up.view(E * self.up_rows, W)).view(T * E, self.up_rows))  # [T * E, ff]
            y = torch.bmm(a.view(T, E, ff).transpose(0, 1), self.w_down.transpose(1, 2))  # [E, T, W]
            dw = torch.zeros(T, E + self.identity, dtype=torch.float32, device=x.device).scatter_(1, topi, topw)
            out = (y.float() * dw[:, :E].t().unsqueeze(-1)).sum(0)
            if self.identity:
                out += x.float() * dw[:, E:].sum(1, keepdim=True)
        else:
            flat = topi.reshape(-1)
            counts = torch.bincount(flat, minlength=self.E + self.identity).tolist()  # the layer's one host sync
            order = torch.argsort(flat, stable=True)
            tok = torch.div(order, self.top, rounding_mode="floor")
            xs = x.new_zeros((tok.shape[0] + self.PAD, x.shape[1]))  # spare rows: see run_expert_segments
            torch.index_select(x, 0, tok, out=xs[:tok.shape[0]])
            real = sum(counts[:self.E])  # copies that go to experts with weights; the identity experts' follow
            big = max(counts[:self.E]) if self.E else 0
            C = 16 if big <= 16 else (big + self.PAD - 1) // self.PAD * self.PAD
            if not self.identity and self._batched(tok.shape[0], C):
                ye = self._run_batched(xs, counts, C, act)
            else:
                ye = run_expert_segments(xs, counts[:self.E], self.experts_up, self.experts_down, act, pad=self.PAD)
                if real < tok.shape[0]:
                    ye = torch.cat([ye, xs[real:tok.shape[0]]], 0)
            w = topw.reshape(-1).index_select(0, order).unsqueeze(-1)
            out = torch.zeros(T, x.shape[1], dtype=torch.float32, device=x.device).index_add_(0, tok, ye.float() * w)
        side = None
        if self.w_sup is not None:
            z = torch.nn.functional.linear(x, self.w_sup, self.b_sup)
            if self.shared_ff:
                ys = torch.nn.functional.linear(act(z[:, :self.sup_rows]), self.w_sdown)
                if self.shared_gate:
                    out = hops.gated_add_f32_(out, ys, z[:, self.sup_rows:self.sup_rows + 1])
                else:
                    out += ys
            side = z[:, self.sup_rows + (1 if self.shared_gate else 0):]
        return (out, side) if self.side else out


def expert_param_global_name(name: str, module_e0: int) -> str:
    """``...experts_up.<local>`` -> ``...experts_up.<global>`` (and the inverse with -e0)."""
    parts = name.split(".")
    for i, p in enumerate(parts[:-1]):
        if p in ("experts_up", "experts_down"):
            parts[i + 1] = str(int(parts[i + 1]) + module_e0)
            return ".".join(parts)
    return name
