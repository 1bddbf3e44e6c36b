"""A plain whole-sequence implementation of the Malinex design in float64, one function per mechanism.

It shares no code with ``llmctl``: full score matrices with explicit masks, a token loop for the
recurrence, a per-token loop over the chosen experts.  ``cfg`` is the checkpoint's ``config.json`` as a
dict, ``W`` maps the checkpoint's tensor names to tensors.  Everything runs on one sequence at a time,
positions 0 .. T-1.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x over its root mean square (eps inside the root), last dim."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms_unit(x, eps) * w.to(F64)


def lin(W, name, h, bias=False):
    y = h @ W[name].to(F64).t()
    return y + W[name + ".b"].to(F64) if bias else y


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def relu2(z):
    return torch.relu(z).pow(2)


# ------------------------------------------------------------------ mixers
def decayed_memory(q, k, v, alpha, S0=None):
    """q, k, alpha [T, H, dk], v [T, H, dv] -> (o [T, H, dv], the memory after the last token):
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=F64) if S0 is None else S0.to(F64).clone()
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t].to(F64)[:, :, None] * S + k[t].to(F64)[:, :, None] * v[t].to(F64)[:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t].to(F64))
    return o, S


def sigmoid_weights(q, k, scale, r1, r2, bias, first=0):
    """q [Tq, H, dk] at positions first .. first + Tq - 1, k [Tk, H, dk] at positions 0 .. Tk - 1 (heads already
    expanded) -> weights [H, Tq, Tk]: sigmoid(q . k * scale - r1 ln(1 + r2 (i - j)) + bias) for j <= i, else 0."""
    Tq, Tk = q.shape[0], k.shape[0]
    i = torch.arange(first, first + Tq, dtype=F64)[:, None]
    j = torch.arange(Tk, dtype=F64)[None, :]
    s = torch.einsum("ihd,jhd->hij", q.to(F64), k.to(F64)) * scale
    s = s - r1.to(F64).view(-1, 1, 1) * torch.log(1.0 + r2.to(F64).view(-1, 1, 1) * (i - j).clamp(min=0.0))
    return torch.where(j <= i, torch.sigmoid(s + bias.to(F64).view(-1, 1, 1)), torch.zeros((), dtype=F64))


def gla(W, p, m, h, eps, state=None):
    """Gated linear attention: per head a [dim, vdim] memory whose key rows decay by alpha_t.
    h [T, width] -> [T, width]; ``state`` ([H, dim, vdim], optional) is the memory before the first token."""
    T = h.shape[0]
    H, dk, dv, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    q = (lin(W, p + "q", h) * dk ** -0.5).view(T, H, dk)
    k = lin(W, p + "k", h).view(T, H, dk)
    v = lin(W, p + "v", h).view(T, H, dv)
    z = lin(W, p + "a2", lin(W, p + "a1", h), bias=True).view(T, H, dk)
    alpha = torch.sigmoid(z).pow(1.0 / tau)
    o, _ = decayed_memory(q, k, v, alpha, state)
    o = rms_unit(o, eps) * W[p + "norm"].to(F64)  # per head over vdim, one weight for all heads
    g = lin(W, p + "g", h)
    return lin(W, p + "o", o.reshape(T, H * dv) * (g * torch.sigmoid(g)))


def sigmoid_attention(W, p, m, h, eps):
    """Grouped causal attention without softmax: a visible key's weight is sigmoid(score + head bias),
    the score being the scaled product minus a logarithmic distance penalty."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    q = norm(lin(W, p + "q", h, True), W[p + "q.norm"], eps)  # over the whole projection, before the split
    k = norm(lin(W, p + "k", h, True), W[p + "k.norm"], eps)
    v = lin(W, p + "v", h, True).view(T, G, dv)
    pos = torch.arange(T, dtype=F64)
    qt = m.get("q_temp")
    if qt:
        q = q * (1.0 + float(qt["coef"]) * torch.log(torch.floor((pos + 1.0) / float(qt["every"])) + 1.0))[:, None]
    q = q.view(T, H, dk)
    k = k.view(T, G, dk).repeat_interleave(H // G, 1)  # query head h reads kv head h // (H / G)
    v = v.repeat_interleave(H // G, 1)
    w = sigmoid_weights(q, k, float(m["scale"]), W[p + "r1"], W[p + "r2"], W[p + "pb"])
    gate = torch.sigmoid(lin(W, p + "g", h))  # [T, H]: one number per head
    out = torch.einsum("hij,jhd->ihd", w, v) * gate[:, :, None]
    return lin(W, p + "o", out.reshape(T, H * dv))


MIXERS = {"gla": gla, "attention": sigmoid_attention}


# ------------------------------------------------------------------ feed-forward
def dense_ff(W, p, h):
    return lin(W, p + "down", gelu_erf(lin(W, p + "up", h)))


def expert(W, p, h):
    return lin(W, p + "down", relu2(lin(W, p + "up", h)))


def route(W, p, f, h):
    """(chosen experts [T, top], their weights [T, top])."""
    s = torch.softmax(lin(W, p + "router", h), -1)
    idx = torch.topk(s + W[p + "correction"].to(F64), int(f["router"]["top"]), dim=-1).indices
    w = torch.gather(s, 1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(W, p, f, h):
    idx, w = route(W, p, f, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            out[t] += we * expert(W, f"{p}e{e}.", h[t:t + 1])[0]
    if f.get("shared"):
        out = out + expert(W, p + "shared.", h)
    return out


def feed_forward(W, p, f, h):
    return dense_ff(W, p, h) if f.get("kind", "dense") == "dense" else moe_ff(W, p, f, h)


# ------------------------------------------------------------------ the model
def layer(cfg, W, i, x):
    spec = cfg["layers"][i]
    p = f"l{spec.get('weights_of', i)}."
    eps = float(cfg["norm"]["eps"])
    h = norm(x, W[p + "norm1"], eps)
    y = MIXERS[spec["type"]](W, p + "mix.", spec["mixer"], h, eps)
    y = y * torch.sigmoid(lin(W, p + "rg1", h, True))
    x = x + norm(y, W[p + "norm1b"], eps)
    f = spec.get("mlp")
    if f is not None:
        h = norm(x, W[p + "norm2"], eps)
        y = feed_forward(W, p + "mlp.", f, h) * torch.sigmoid(lin(W, p + "rg2", h, True))
        x = x + norm(y, W[p + "norm2b"], eps)
    return x


def forward(cfg, W, tokens, trail=None):
    """Logits [T, vocab] (float64) of one sequence; ``trail`` collects the stream after every layer."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = W["embed"].to(F64)[ids] + W["pos"].to(F64)[:len(ids)]
    for i in range(len(cfg["layers"])):
        x = layer(cfg, W, i, x)
        if trail is not None:
            trail.append(x.clone())
    x = norm(x, W["final.norm"], float(cfg["norm"]["eps"]))
    return lin(W, "head", x) * float(cfg.get("logit_scale", 1.0))
