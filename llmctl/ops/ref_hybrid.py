"""CPU (fp32 torch) forms of the hybrid-mixer ops in :mod:`llmctl.ops.hybrid`.

Same signatures and cache / state layouts as the HIP kernels in ``csrc/hybrid``: the engine's
CPU path (gloo tests, no GPU) runs on these, and the kernel tests compare the HIP kernels with an
independent plain implementation, not with this file.
"""

from __future__ import annotations

from typing import Optional

import torch


def layernorm_f32(x, w, b, eps, out_dtype):
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    var = (xf - mu).pow(2).mean(-1, keepdim=True)
    return ((xf - mu) * torch.rsqrt(var + eps) * w.float() + b.float()).to(out_dtype)


def residual_add_(x, a, b):
    x += a.float()
    if b is not None:
        x += b.float()
    return x


def rmsnorm_cols(x, w, eps, n, out_dtype):
    xf = x[:, :n].float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def _rotate(x, pos, inv_freq, dims, interleaved=False, amp=1.0):
    """x f32 [T, ..., n]: entries [0, dims) rotated; pairs are halves (i, i + dims/2) or neighbours
    (2i, 2i + 1); cos and sin are scaled by ``amp``."""
    half = dims // 2
    ang = pos.float()[:, None] * inv_freq.float()[None, :]  # fp32 angles
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape) * amp, torch.sin(ang).view(shape) * amp
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        r = torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)
        return torch.cat([r, x[..., dims:]], -1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def latent_kv_write(dkv, norm_w, eps, pos, inv_freq, rot_dims, cache, slots, interleaved=False, amp=1.0):
    rk = norm_w.shape[0]
    c = rmsnorm_cols(dkv, norm_w, eps, rk, torch.float32)
    kr = _rotate(dkv[:, rk:].float(), pos, inv_freq, rot_dims, interleaved, amp)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = row[ok]


def latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims, dn, interleaved=False, amp=1.0):
    qr = _rotate(q[..., dn:].float(), pos, inv_freq, rot_dims, interleaved, amp)
    return torch.cat([q_lat.float(), qr], -1).to(q.dtype)


def latent_attention(qa, cache, bt, cu, ctx, window, sink, scale, rk, groups=1, koff=0, chunk=1 << 30, hscale=None,
                     ofreq=None, sig_bias=None, dist_a=None, dist_b=None, softcap=0.0, keep_first=0):
    """Attention over a paged row cache.  Sequence n owns query rows [cu[n], cu[n+1]); its last query
    sits at position ctx[n] - 1.  A token's cache row holds ``groups`` sub-rows; query head h reads
    sub-row h / (H / groups), whose entries [koff, koff + R) are the key and whose first ``rk`` entries
    are the value (latent attention: one sub-row, key = the whole row).  Position i sees j <= i inside
    its window (i - j < window) and its chunk (i // chunk == j // chunk); ``sink`` [H] joins the softmax
    denominator; ``hscale`` [H] multiplies the scores; ``ofreq`` [rk / 2] turns the output's neighbour
    pairs back by -position * ofreq.  ``dist_a``, ``dist_b`` [H]: ``dist_a ln(1 + dist_b (i - j))`` is taken
    off the scaled score; ``sig_bias`` [H]: no softmax, a visible key weighs sigmoid(score + sig_bias).
    ``softcap`` c > 0: the scaled score becomes c tanh(score / c); ``keep_first`` n: the window does not hide
    the keys at positions below n."""
    T, H, R = qa.shape
    bs = cache.shape[1]
    G = groups
    rs = cache.shape[2] // G
    out = torch.zeros(T, H, rk, dtype=torch.float32)
    flat = cache.view(-1, G, rs)
    cu_l, ctx_l = [int(v) for v in cu], [int(v) for v in ctx]
    hs = hscale.float().view(H, 1, 1) if hscale is not None else 1.0
    for n in range(len(ctx_l)):
        a, b = cu_l[n], cu_l[n + 1]
        if b == a:
            continue
        p0 = ctx_l[n] - (b - a)  # position of the first query row
        lo = max(0, p0 - window + 1, (p0 // chunk) * chunk)
        if keep_first > 0:
            lo = max(0, (p0 // chunk) * chunk)
        kpos = torch.arange(lo, ctx_l[n])
        rows = flat[bt[n, (kpos // bs).long()].long() * bs + kpos % bs].float()  # [K, G, rs]
        rows = rows.repeat_interleave(H // G, 1)  # [K, H, rs]
        s = torch.einsum("thr,khr->htk", qa[a:b].float(), rows[:, :, koff:koff + R]) * scale * hs
        if softcap > 0.0:
            s = softcap * torch.tanh(s / softcap)
        qpos = torch.arange(p0, ctx_l[n])
        d = qpos[:, None] - kpos[None, :]
        vis = (d >= 0) & ((d < window) | (kpos[None, :] < keep_first)) & (qpos[:, None] // chunk == kpos[None, :] // chunk)
        if dist_a is not None:
            s = s - dist_a.float().view(H, 1, 1) * torch.log1p(dist_b.float().view(H, 1, 1) * d.clamp(min=0).float())
        if sig_bias is not None:
            wgt = torch.sigmoid(s + sig_bias.float().view(H, 1, 1)).masked_fill(~vis, 0.0)
            out[a:b] = torch.einsum("htk,khr->thr", wgt, rows[:, :, :rk])
            continue
        s = s.masked_fill(~vis, float("-inf"))
        top = s.max(-1, keepdim=True).values
        if sink is not None:
            sk = sink.float().view(H, 1, 1)
            top = torch.maximum(top, sk)
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sk - top)
        o = torch.einsum("htk,khr->thr", e / den, rows[:, :, :rk])
        if ofreq is not None:
            o = _rotate(o, -qpos, ofreq, rk, True)
        out[a:b] = o
    return out.to(qa.dtype)


def add_rmsnorm2_f32_(x, a, b, w1, w2, eps, one_plus, out_dtype):
    if a is not None:
        x += a.float() + b.float() if b is not None else a.float()
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    plus = 1.0 if one_plus else 0.0
    h1 = (y * (plus + w1.float())).to(out_dtype)
    return h1, ((y * (plus + w2.float())).to(out_dtype) if w2 is not None else h1)


def clamped_glu(gu, limit, alpha):
    f = gu.shape[-1] // 2
    g, u = gu[..., :f].float().clamp(max=limit), gu[..., f:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def causal_conv(u, w, state, seq_of, cu, start, sslot, add_input):
    """y_t = (u_t if add_input) + sum_j w[j] u_(t - taps + 1 + j) (w tap-major [taps, C]) per sequence of the packed rows; the
    last taps - 1 inputs of a sequence live in ``state[slot]`` ([taps - 1, C], oldest first) between steps
    and are ignored by a sequence that starts at position 0."""
    T, C = u.shape
    taps = w.shape[0]
    y = torch.zeros(T, C, dtype=torch.float32)
    cu_l = [int(v) for v in cu]
    for s in range(len(cu_l) - 1):
        a, b = cu_l[s], cu_l[s + 1]
        if a == b:
            continue
        slot = int(sslot[s])
        old = state[slot].clone() if int(start[s]) > 0 else torch.zeros(taps - 1, C)
        if 0 < int(start[s]) < taps - 1:  # entries of positions before 0
            old[:taps - 1 - int(start[s])] = 0.0
        ext = torch.cat([old, u[a:b].float()], 0)
        n = b - a
        acc = torch.zeros(n, C)
        for j in range(taps):
            acc += ext[j:j + n] * w[j].float()
        y[a:b] = acc + (u[a:b].float() if add_input else 0.0)
        if taps > 1:
            state[slot] = ext[-(taps - 1):]
    return y.to(u.dtype)


def attn_qkv_prep(z, H, G, dk, dv, q_norm, k_norm, eps, pos, freq, rot_dims, interleaved, amp, vfreq, cache, slots,
                  v_from_k=False, v_first=None, v_lambda=None):
    """z [T, H*dk + G*dk + G*dv] = [q | k | v]: per-head RMS norm (skipped when the weights are None) and rotary
    of q and k, optional turn of v over all of dv; k and v go to the token's cache row [G, dv + dk] = [v | k];
    returns q [T, H, dk].  ``v_from_k``: z = [q | k] and the value is the key projection's output (ahead of norm and
    rotary).  ``v_first`` [T, G*dv] with ``v_lambda`` (one number): v <- (1 - lambda) v + lambda v_first."""
    T = z.shape[0]
    zf = z.float()
    q, k = zf[:, :H * dk].view(T, H, dk), zf[:, H * dk:(H + G) * dk].view(T, G, dk)
    v = k if v_from_k else zf[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv)
    if v_first is not None:
        lam = v_lambda.float().reshape(())
        v = (1.0 - lam) * v + lam * v_first.float().view(T, G, dv)
    unit = lambda x: x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    if q_norm is not None:
        q, k = unit(q) * q_norm.float(), unit(k) * k_norm.float()
    q = _rotate(q, pos, freq, rot_dims, interleaved, amp)
    k = _rotate(k, pos, freq, rot_dims, interleaved, amp)
    if vfreq is not None:
        v = _rotate(v, pos, vfreq, dv, interleaved)
    row = torch.cat([v, k], -1).reshape(T, G * (dv + dk)).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = row[ok]
    return q.to(z.dtype)


def sigmoid_gate_mul(o, g):
    gate = torch.sigmoid(g.float())
    if g.shape[-1] != o.shape[-1]:  # one gate per group of neighbouring columns
        gate = gate.repeat_interleave(o.shape[-1] // g.shape[-1], -1)
    return (o.float() * gate).to(g.dtype)


def mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, cu, start):
    """Token-by-token matrix-memory recurrence.  State pools S [slots, H, dk, dv], n [slots, H, dk],
    m [slots, H] (fp32) are read at ``state_slots[seq]`` (zeros when the sequence starts at
    position 0) and written back after the sequence's last token of this step."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    ig = cap * torch.tanh((if_raw[:, :H].float() + b_i.float()) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((if_raw[:, H:].float() + b_f.float()) / cap))
    cu_l = [int(x) for x in cu]
    for s in range(len(cu_l) - 1):
        a, b = cu_l[s], cu_l[s + 1]
        if a == b:
            continue
        slot = int(state_slots[s])
        if int(start[s]) == 0:
            Ss, ns, ms = torch.zeros_like(S[slot]), torch.zeros_like(n[slot]), torch.zeros_like(m[slot])
        else:
            Ss, ns, ms = S[slot].clone(), n[slot].clone(), m[slot].clone()
        for t in range(a, b):
            qt, kt, vt = q[t].float() * qscale, k[t].float(), v[t].float()
            m_new = torch.maximum(fg[t] + ms, ig[t])
            da, db = torch.exp(fg[t] + ms - m_new), torch.exp(ig[t] - m_new)
            Ss = da[:, None, None] * Ss + db[:, None, None] * kt[:, :, None] * vt[:, None, :]
            ns = da[:, None] * ns + db[:, None] * kt
            ms = m_new
            num = torch.einsum("hkv,hk->hv", Ss, qt)
            den = torch.maximum((ns * qt).sum(-1).abs(), torch.exp(-ms)) + 1e-6
            out[t] = num / den[:, None]
        S[slot], n[slot], m[slot] = Ss, ns, ms
    return out


def headnorm_gate(o, w, g, eps, out_dtype, silu=False):
    T, H, dv = o.shape
    of = o.float()
    y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps)
    gf = g.float()
    gate = gf * torch.sigmoid(gf) if silu else torch.sigmoid(gf)
    return (y.reshape(T, H * dv) * w.float() * gate).to(out_dtype)


def group_topk_router(logits, top, groups, keep):
    T, E = logits.shape
    s = torch.sigmoid(logits.float())
    per = E // groups
    gs = s.view(T, groups, per).topk(min(2, per), -1).values.sum(-1)
    best = gs.topk(keep, -1).indices
    ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
    ok = ok[:, :, None].expand(T, groups, per).reshape(T, E)
    idx = s.masked_fill(~ok, -1.0).topk(top, -1).indices
    return idx, s.gather(1, idx)


def swiglu_any(gu):
    f = gu.shape[-1] // 2
    g, u = gu[..., :f].float(), gu[..., f:].float()
    return (g * torch.sigmoid(g) * u).to(gu.dtype)


def gated_norm_add_norm_f32_(x, y, r, w_post, w_next, eps, out_dtype):
    g = y.float() * torch.sigmoid(r.float())
    x += g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps) * w_post.float()
    if w_next is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w_next.float()).to(out_dtype)


def embed_rmsnorm_f32(ids, pos, table, pos_table, w, eps, out_dtype):
    x = table[ids].float() + pos_table[pos.long()].float()
    return x, (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def gla_scan(q, k, v, z, z_bias, tau, qscale, S, state_slots, cu, start):
    """Token-by-token decayed matrix memory.  The state pool S [slots, H, dk, dv] (fp32) is read at
    ``state_slots[seq]`` (zeros when the sequence starts at position 0) and written back after the
    sequence's last token of this step."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    alpha = torch.exp(torch.nn.functional.logsigmoid(z.float() + z_bias.float()) / tau).view(T, H, dk)
    cu_l = [int(x) for x in cu]
    for s in range(len(cu_l) - 1):
        a, b = cu_l[s], cu_l[s + 1]
        if a == b:
            continue
        slot = int(state_slots[s])
        Ss = torch.zeros_like(S[slot]) if int(start[s]) == 0 else S[slot].clone()
        for t in range(a, b):
            Ss = alpha[t][:, :, None] * Ss + k[t].float()[:, :, None] * v[t].float()[:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", Ss, q[t].float() * qscale)
        S[slot] = Ss
    return out


def qk_fullnorm_prep(z, H, G, dk, dv, q_norm, k_norm, eps, pos, temp_coef, temp_every, cache, slots):
    """z [T, >= H*dk + G*dk + G*dv] = [q | k | v | ...]: RMS norm of all of q and of all of k (weights [H*dk],
    [G*dk]); q times 1 + temp_coef ln(floor((p + 1) / temp_every) + 1); k and v go to the token's cache row
    [G, dv + dk] = [v | k]; returns q [T, H, dk]."""
    T = z.shape[0]
    zf = z.float()
    unit = lambda x: x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    q = unit(zf[:, :H * dk]) * q_norm.float()
    k = unit(zf[:, H * dk:(H + G) * dk]) * k_norm.float()
    v = zf[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv)
    if temp_coef != 0.0:
        q = q * (1.0 + temp_coef * torch.log(torch.floor((pos.float() + 1.0) / float(temp_every)) + 1.0))[:, None]
    row = torch.cat([v, k.view(T, G, dk)], -1).reshape(T, G * (dv + dk)).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = row[ok]
    return q.view(T, H, dk).to(z.dtype)


def bias_topk_router(logits, bias, top, groups=1, keep=1, renorm=True):
    s = torch.softmax(logits.float(), -1)
    c = s + bias.float() if bias is not None else s
    if groups > 1:
        T, E = c.shape
        per = E // groups
        best = c.view(T, groups, per).max(-1).values.topk(keep, -1).indices
        ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        c = c.masked_fill(~ok[:, :, None].expand(T, groups, per).reshape(T, E), float("-inf"))
    idx = c.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx, (w / (w.sum(-1, keepdim=True) + 1e-20) if renorm else w)


def act_any(x, kind):
    xf = x.float()
    if kind == "relu2":
        y = torch.relu(xf).pow(2)
    elif kind == "gelu":
        y = 0.5 * xf * (1.0 + torch.erf(xf * 0.7071067811865476))
    else:
        raise ValueError(f"unknown activation {kind!r}")
    return y.to(x.dtype)


def hc_embed_norm(ids, table, streams, c_in, g, eps, out_dtype):
    """Every one of ``streams`` residual streams starts as the embedding; returns (X fp32 [T, S, W], the first
    sublayer's input ``norm(sum_s c_in[s] x_s) * g``)."""
    x = table[ids].float()
    X = x[:, None, :].repeat(1, streams, 1).contiguous()
    u = x * c_in.float().sum()
    return X, (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * g.float().reshape(())).to(out_dtype)


def hc_update_norm_(X, y1, s1, y2, s2, mix, c_out, mult, c_in, g, eps, out_dtype):
    """A sublayer's result into ``streams`` residual streams X fp32 [T, S, W], all at once from the old ones:
    ``x_t <- sum_s mix[s, t] x_s + mult c_out[t] (s1 y1 + s2 y2)``; then, when ``c_in`` is given, the next
    sublayer's input ``norm(sum_t c_in[t] x_t) * g`` (else None)."""
    y = y1.float() * s1
    if y2 is not None:
        y = y + y2.float() * s2
    new = torch.einsum("st,nsw->ntw", mix.float(), X) + mult * c_out.float()[None, :, None] * y[:, None, :]
    X.copy_(new)
    if c_in is None:
        return None
    u = torch.einsum("t,ntw->nw", c_in.float(), X)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * g.float().reshape(())).to(out_dtype)


def delta_scan(r, k, v, zw, w0, za, ab, decay_coef, key_eps, S, state_slots, cu, start):
    """Token-by-token generalized delta rule.  Per head a memory S [dk, dv]: with the decay ``w = exp(-decay_coef
    sigmoid(zw + w0))``, the removal rate ``a = sigmoid(za + ab)`` and the unit key ``u = k / sqrt(sum k^2 + key_eps)``,
    ``S_t = diag(w) S_(t-1) - (a u) (u^T S_(t-1)) + k v^T`` and ``o_t = S_t^T r``.  The state pool S [slots, H, dk, dv]
    (fp32) is read at ``state_slots[seq]`` (zeros when the sequence starts at position 0) and written back after
    the sequence's last token of this step."""
    T, H, dk = r.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    w = torch.exp(-decay_coef * torch.sigmoid(zw.float() + w0.float())).view(T, H, dk)
    a = torch.sigmoid(za.float() + ab.float()).view(T, H, dk)
    kf = k.float()
    u = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + key_eps)
    cu_l = [int(x) for x in cu]
    for s in range(len(cu_l) - 1):
        lo, hi = cu_l[s], cu_l[s + 1]
        if lo == hi:
            continue
        slot = int(state_slots[s])
        Ss = torch.zeros_like(S[slot]) if int(start[s]) == 0 else S[slot].clone()
        for t in range(lo, hi):
            uS = torch.einsum("hk,hkv->hv", u[t], Ss)
            Ss = w[t][:, :, None] * Ss - (a[t] * u[t])[:, :, None] * uS[:, None, :] + kf[t][:, :, None] * v[t].float()[:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", Ss, r[t].float())
        S[slot] = Ss
    return out


def tanh_act(x):
    return torch.tanh(x.float()).to(x.dtype)


def softcap_(x, cap):
    return x.copy_(cap * torch.tanh(x / cap))


def gated_add_f32_(out, y, g):
    out += y.float() * torch.sigmoid(g.float())
    return out
