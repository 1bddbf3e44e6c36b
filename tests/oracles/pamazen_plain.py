"""A plain float64 implementation of the Pamazen design over whole sequences, one function per mechanism.

It shares no code with ``llmctl``: full score matrices with explicit masks, a token loop for the
recurrence, a per-token loop over the chosen experts.  ``W`` maps checkpoint tensor names to tensors,
``cfg`` is the parsed ``config.json``.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_pairs(x, base, dims, factor):
    """x [T, H, d]: neighbours (2i, 2i + 1), i < dims / 2, are turned by p * base^(-2i / dims) / factor, p = 0 .. T-1."""
    return rotate_pairs_at(x, torch.arange(x.shape[0], dtype=F64), base, dims, factor)


def rotate_pairs_at(x, pos, base, dims, factor):
    out = x.clone()
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims) / factor
        ang = pos * f
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


def softmax_with_extra(scores, visible, extra):
    """Rows of ``scores [H, T, T]`` over the visible keys; ``extra [H]`` is one more logit in the denominator
    (it has no value)."""
    s = scores.masked_fill(~visible, float("-inf"))
    e = extra.view(-1, 1, 1).expand(s.shape[0], s.shape[1], 1)
    top = torch.maximum(s.max(-1, keepdim=True).values, e)
    w = torch.exp(s - top)
    return w / (w.sum(-1, keepdim=True) + torch.exp(e - top))


def rotary_attention(h, W, p, m, v_first, first):
    """The 'attention' mixer.  Returns (output [T, width], the value projection's output [T, G, vdim])."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).view(T, H, dk)
    k = (h @ W[p + "k"].T).view(T, G, dk)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    v_own = v
    if m.get("v_mix") and not first:
        lam = W[p + "vmix"].reshape(())
        v = (1.0 - lam) * v + lam * v_first
    rot = m.get("rot")
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotate_pairs(q, rot["base"], int(rot["dims"]), factor)
        k = rotate_pairs(k, rot["base"], int(rot["dims"]), factor)
    rep = H // G
    kk, vv = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * float(m["scale"])
    i = torch.arange(T)
    vis = (i[None, :] <= i[:, None])[None]
    wgt = softmax_with_extra(s, vis, torch.zeros(H, dtype=F64))
    o = torch.einsum("hij,jhd->ihd", wgt, vv).reshape(T, H * dv)
    return o @ W[p + "o"].T, v_own


def window_attention(h, W, p, m, eps):
    """The left half of the 'parallel' mixer."""
    T = h.shape[0]
    H, G, dk = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"])
    q = (h @ W[p + "q"].T).view(T, H, dk)
    k = (h @ W[p + "k"].T).view(T, G, dk)
    v = k  # no value projection: the key projection's output serves
    q = rms_unit(q, eps) * W[p + "q.norm"]
    kn = rms_unit(k, eps) * W[p + "k.norm"]
    rep = H // G
    s = torch.einsum("ihd,jhd->hij", q, kn.repeat_interleave(rep, 1)) * float(m["scale"])
    cap = m.get("softcap")
    if cap:
        s = float(cap) * torch.tanh(s / float(cap))
    i = torch.arange(T)
    d = i[:, None] - i[None, :]
    mask = m.get("mask") or {}
    size, keep = int(mask.get("size", T + 1)), int(mask.get("keep_first", 0))
    vis = ((d >= 0) & ((d < size) | (i[None, :] < keep)))[None]
    wgt = softmax_with_extra(s, vis, W[p + "sink"].to(F64))
    o = torch.einsum("hij,jhd->ihd", wgt, v.repeat_interleave(rep, 1)).reshape(T, -1)
    return o @ W[p + "o"].T


def delta_rule(h, W, p, m, eps):
    """The right half of the 'parallel' mixer: a token loop over the memory."""
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    r = (h @ W[p + "r"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, d)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).view(T, H, d)
    a = torch.sigmoid(h @ W[p + "a"].T + W[p + "a.b"]).view(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d, dtype=F64)
    o = torch.zeros(T, H, d, dtype=F64)
    for t in range(T):
        uS = torch.einsum("hk,hkv->hv", u[t], S)
        S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, r[t])
    o = rms_unit(o, eps).reshape(T, H * d) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    return (float(m["left_scale"]) * window_attention(h, W, p + "left.", m["left"], eps)
            + float(m["right_scale"]) * delta_rule(h, W, p + "right.", m["right"], eps))


def glu_expert(h, W, p):
    z = h @ W[p + "gate"].T
    return ((z * torch.sigmoid(z)) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, r):
    """Per token: (chosen expert ids, their weights)."""
    E, ident, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    n = E + ident
    s = torch.softmax(h @ W[p + "router"].T, -1)
    choice = s + (W[p + "correction"] if p + "correction" in W else 0.0)
    groups = r.get("groups") or {}
    count, keep = int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1)))
    per = n // count
    picks = []
    for t in range(h.shape[0]):
        c = choice[t].clone()
        gscore = c.view(count, per).max(-1).values
        best = torch.argsort(gscore, descending=True, stable=True)[:keep].tolist()
        for g in range(count):
            if g not in best:
                c[g * per:(g + 1) * per] = float("-inf")
        ids = torch.argsort(c, descending=True, stable=True)[:top].tolist()
        picks.append((ids, [float(s[t, e]) for e in ids]))
    return picks


def moe(h, W, p, mlp):
    r = mlp["router"]
    E = int(r["experts"])
    out = torch.zeros_like(h)
    for t, (ids, ws) in enumerate(route(h, W, p, r)):
        for e, w in zip(ids, ws):
            out[t] += w * (glu_expert(h[t:t + 1], W, f"{p}e{e}.")[0] if e < E else h[t])
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * glu_expert(h, W, p + "shared.")
    return out


def forward(cfg, W, tokens):
    """Returns (logits [T, vocab], [the stream after every layer])."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    S = int(cfg.get("streams", 0))
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = [x0.clone() for _ in range(max(S, 1))]
    trail = []
    v_first, seen_vmix = None, False

    def sublayer(xs, q, i, fn):
        g = W[f"l{i}.norm{q}"].reshape(())
        if S:
            cin, cout, cm = W[f"l{i}.hc{q}.in"], W[f"l{i}.hc{q}.out"], W[f"l{i}.hc{q}.mix"]
            u = sum(cin[s] * xs[s] for s in range(S))
            y = fn(rms_unit(u, eps) * g)
            return [sum(cm[s, t] * xs[s] for s in range(S)) + mult * cout[t] * y for t in range(S)]
        return [xs[0] + mult * fn(rms_unit(xs[0], eps) * g)]

    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}.mix."
        if spec["type"] == "attention":
            m = spec["mixer"]
            first = bool(m.get("v_mix")) and not seen_vmix
            box = {}

            def run(hh, m=m, p=p, first=first):
                y, box["v"] = rotary_attention(hh, W, p, m, v_first, first or not m.get("v_mix"))
                return y

            xs = sublayer(xs, 1, i, run)
            if first:
                v_first, seen_vmix = box["v"], True
        elif spec["type"] == "parallel":
            xs = sublayer(xs, 1, i, lambda hh, m=spec["mixer"], p=p: parallel_mixer(hh, W, p, m, eps))
        else:
            raise ValueError(spec["type"])
        if spec.get("mlp") is not None:
            xs = sublayer(xs, 2, i, lambda hh, mlp=spec["mlp"], i=i: moe(hh, W, f"l{i}.mlp.", mlp))
        trail.append(sum(xs))
    x = rms_unit(sum(xs), eps) * W["final.norm"].reshape(())
    logits = x @ W["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits, trail
