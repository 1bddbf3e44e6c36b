"""Ops of the hybrid sequence mixers: latent attention (compressed K/V cache, sliding window,
softmax sink), grouped attention over paged rows (softmax or sigmoid weights, distance penalty), the
mLSTM matrix memory, gated linear attention, the generalized delta rule, the group-limited sigmoid router and the
softmax router with a selection bias (optionally group-limited), and the fp32 residual stream of parallel layers, of
layers with a gated residual between two norms, and of layers over several residual streams (hyper-connections).

GPU tensors run the HIP kernels of ``csrc/hybrid`` (``torch.ops.llmctl_hybrid.*``, library
``_llmctl_hybrid.so``); CPU tensors run :mod:`llmctl.ops.ref_hybrid`.  All activations are
token-major ``[T, features]`` over the step's packed tokens; sequences are described by ``cu``
(row offsets, int32 [n + 1]), ``ctx`` (context length after the step, int32 [n]) and block tables.

Precision: norms, rotary angles, attention scores / softmax, the recurrence with its gates and the
residual stream are fp32 inside every kernel whatever the activation dtype (bf16 or fp32).
"""

from __future__ import annotations

import torch

from . import ref_hybrid as ref
from ._lib import native_hybrid, use_native


def layernorm_f32(x, w, b, eps: float, out_dtype):
    """LayerNorm of the fp32 residual stream ``x [T, W]`` -> ``out_dtype``."""
    if use_native(x):
        return native_hybrid().layernorm_f32(x, w, b, eps, out_dtype == torch.bfloat16)
    return ref.layernorm_f32(x, w, b, eps, out_dtype)


def residual_add_(x, a, b=None):
    """``x += a (+ b)`` on the fp32 residual stream (a, b: any float dtype)."""
    if use_native(x):
        native_hybrid().residual_add_(x, a, b)
        return x
    return ref.residual_add_(x, a, b)


def add_layernorm_f32_(x, a, b, w, bias, eps: float, out_dtype):
    """``x += a (+ b)`` in place, then LayerNorm(x) -> ``out_dtype``: the parallel layer's residual
    update and the next layer's norm in one pass over the stream."""
    if use_native(x):
        return native_hybrid().add_layernorm_f32_(x, a, b, w, bias, eps, out_dtype == torch.bfloat16)
    ref.residual_add_(x, a, b)
    return ref.layernorm_f32(x, w, bias, eps, out_dtype)


def rmsnorm_cols(x, w, eps: float, n: int, out_dtype):
    """RMS norm (weight ``w [n]``) of the first ``n`` columns of ``x [T, N]`` -> ``[T, n]``."""
    if use_native(x):
        return native_hybrid().rmsnorm_cols(x, w, eps, n, out_dtype == torch.bfloat16)
    return ref.rmsnorm_cols(x, w, eps, n, out_dtype)


def latent_kv_write(dkv, norm_w, eps: float, pos, inv_freq, rot_dims: int, cache, slots, interleaved: bool = False,
                    amp: float = 1.0):
    """The down-projected K/V row ``dkv [T, rank + rot]``: RMS norm of the latent part, rotary on
    the shared key part (pairs: halves, or neighbours when ``interleaved``; cos and sin times ``amp``),
    both written to the paged cache row ``[rank | rot]`` at ``slots``."""
    if use_native(dkv):
        native_hybrid().latent_kv_write(dkv, norm_w, eps, pos, inv_freq, rot_dims, cache, slots, interleaved, amp)
    else:
        ref.latent_kv_write(dkv, norm_w, eps, pos, inv_freq, rot_dims, cache, slots, interleaved, amp)


def latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims: int, dn: int, interleaved: bool = False, amp: float = 1.0):
    """Query rows in the cache's layout: ``[q_lat | rotary(q[..., dn:])]`` per head, where ``q_lat
    [T, H, rank]`` is the unrotated query part carried into the latent space (q W_uk)."""
    if use_native(q):
        return native_hybrid().latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims, dn, interleaved, amp)
    return ref.latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims, dn, interleaved, amp)


NO_LIMIT = 1 << 30  # a window or chunk that never masks


def latent_attention_prefill(qa, cache, bt, cu, ctx, window: int, sink, scale: float, rk: int, max_q: int,
                             mfma: bool = True, groups: int = 1, koff: int = 0, chunk: int = NO_LIMIT, hscale=None,
                             ofreq=None, sig_bias=None, dist_a=None, dist_b=None, softcap: float = 0.0, keep_first: int = 0):
    """Prompt portions: sequence n's query rows ``[cu[n], cu[n+1])`` end at position ``ctx[n]-1``;
    ``max_q``: the longest portion (sizes the launch).  bf16 shapes that fit run on the matrix cores
    (``mfma=False`` forces the generic fp32-SIMT kernel, which also serves fp32).

    The general form reads a paged row cache whose token rows hold ``groups`` sub-rows (one per kv
    group; query head h reads sub-row ``h // (H // groups)``): entries ``[koff, koff + R)`` of a sub-row
    are the key, its first ``rk`` entries the value.  Latent attention is ``groups=1, koff=0``.  Masks:
    ``window`` (i - j < window) and ``chunk`` (i // chunk == j // chunk), :data:`NO_LIMIT` for none.
    ``sink`` (fp32 [H] or None) joins the softmax denominator; ``hscale`` (fp32 [H]) multiplies a head's
    scores; ``ofreq`` (fp32 [rk/2]) turns the output's neighbour pairs back by ``-position * ofreq``.
    ``dist_a``, ``dist_b`` (fp32 [H], together): ``dist_a ln(1 + dist_b (i - j))`` is taken off the scaled score.
    ``sig_bias`` (fp32 [H]): the weights are not a softmax; a visible key weighs ``sigmoid(score + sig_bias)``
    and nothing is normalised over the keys (no sink then).  ``softcap`` c > 0: the scaled score becomes
    ``c tanh(score / c)`` before masks and softmax; ``keep_first`` n > 0: the window does not hide the keys at
    positions below n (nothing is renumbered: such keys are addressed by their own positions)."""
    if use_native(qa):
        return native_hybrid().latent_attn_prefill(qa, cache, bt, cu, ctx, window, sink, scale, rk, max_q, mfma, groups,
                                                   koff, chunk, hscale, ofreq, sig_bias, dist_a, dist_b, softcap, keep_first)
    return ref.latent_attention(qa, cache, bt, cu, ctx, window, sink, scale, rk, groups, koff, chunk, hscale, ofreq,
                                sig_bias, dist_a, dist_b, softcap, keep_first)


def latent_attention_decode(qa, cache, bt, ctx, window: int, sink, scale: float, rk: int, mfma: bool = True,
                            groups: int = 1, koff: int = 0, chunk: int = NO_LIMIT, hscale=None, ofreq=None,
                            max_ctx: int = 0, sig_bias=None, dist_a=None, dist_b=None, softcap: float = 0.0,
                            keep_first: int = 0):
    """One query row per sequence, at position ``ctx[n] - 1`` (options as in the prefill form;
    ``max_ctx``: the longest context if the host knows it, it sizes the split of the keys)."""
    if use_native(qa):
        return native_hybrid().latent_attn_decode(qa, cache, bt, ctx, window, sink, scale, rk, mfma, groups, koff, chunk,
                                                  hscale, ofreq, max_ctx, sig_bias, dist_a, dist_b, softcap, keep_first)
    cu = torch.arange(qa.shape[0] + 1, dtype=torch.int32)
    return ref.latent_attention(qa, cache, bt, cu, ctx, window, sink, scale, rk, groups, koff, chunk, hscale, ofreq,
                                sig_bias, dist_a, dist_b, softcap, keep_first)


def add_rmsnorm2_f32_(x, a, b, w1, w2, eps: float, one_plus: bool, out_dtype):
    """``x += a (+ b)`` in place on the fp32 residual stream (skipped when ``a`` is None), then RMS norms
    of the same x with weights ``w1`` and (optional) ``w2``: ``x / sqrt(mean(x^2) + eps) * (w + one_plus)``.
    Returns (h1, h2) in ``out_dtype`` (h2 is h1 when ``w2`` is None)."""
    if use_native(x):
        return native_hybrid().add_rmsnorm2_f32_(x, a, b, w1, w2, eps, one_plus, out_dtype == torch.bfloat16)
    return ref.add_rmsnorm2_f32_(x, a, b, w1, w2, eps, one_plus, out_dtype)


def residual_add_act_(x, a, b=None):
    """``x += a (+ b)`` on the fp32 residual stream, a and b in the activation dtype."""
    if use_native(x):
        native_hybrid().residual_add_act_(x, a, b)
        return x
    return ref.residual_add_(x, a, b)


def clamped_glu(gu, limit: float, alpha: float):
    """``gu [T, 2F] = [gate | up]`` -> ``g * sigmoid(alpha g) * (u + 1)`` with ``g = min(gate, limit)``,
    ``u = clamp(up, -limit, limit)``."""
    if use_native(gu):
        return native_hybrid().clamped_glu(gu.contiguous(), limit, alpha)
    return ref.clamped_glu(gu, limit, alpha)


def causal_conv(u, w, state, seq_of, cu, start, sslot, add_input: bool, max_len: int = 0):
    """Short causal convolution over time per channel of the packed rows ``u [T, C]`` (``w`` fp32, tap-major
    ``[taps, C]``): ``y_t = (u_t if add_input) + sum_j w[j] u_(t - taps + 1 + j)``.  ``state`` (fp32
    ``[slots, taps - 1, C]``) carries each live sequence's last ``taps - 1`` inputs between steps (read
    at ``sslot[seq]`` unless the sequence starts at position 0, then updated in place).  ``max_len``: the
    longest portion of the step if the host knows it (steps of short portions take a one-launch form)."""
    if use_native(u):
        return native_hybrid().causal_conv(u, w, state, seq_of, cu, start, sslot, add_input, max_len)
    return ref.causal_conv(u, w, state, seq_of, cu, start, sslot, add_input)


def attn_qkv_prep(z, H: int, G: int, dk: int, dv: int, q_norm, k_norm, eps: float, pos, freq, rot_dims: int,
                  interleaved: bool, amp: float, vfreq, cache, slots, v_from_k: bool = False, v_first=None, v_lambda=None):
    """``z [T, H*dk + G*dk + G*dv] = [q | k | v]``: per-head RMS norm (weights fp32 [dk]; both None: no norm) and
    rotary of q and k, optional turn of v over all of dv by ``position * vfreq``; k and v are written to the
    token's cache row ``[G, dv + dk] = [v | k]`` at ``slots``; returns q ``[T, H, dk]``.  ``v_from_k``: ``z = [q | k]``
    and a token's value is the output of its key projection, taken ahead of norm and rotary (``dv == dk``).  ``v_first`` (``[T, G*dv]``,
    row-strided views allowed) with ``v_lambda`` (fp32, one number): ``v <- (1 - lambda) v + lambda v_first`` before
    the write."""
    if use_native(z):
        return native_hybrid().attn_qkv_prep(z, H, G, dk, dv, q_norm, k_norm, eps, pos, freq, rot_dims, interleaved, amp,
                                             vfreq, cache, slots, v_from_k, v_first, v_lambda)
    return ref.attn_qkv_prep(z, H, G, dk, dv, q_norm, k_norm, eps, pos, freq, rot_dims, interleaved, amp, vfreq, cache, slots,
                             v_from_k, v_first, v_lambda)


def sigmoid_gate_mul(o, g):
    """``o * sigmoid(g)`` -> g's dtype.  ``g`` may have fewer columns than ``o [T, C]``: ``g [T, H]`` gates
    every run of ``C / H`` neighbouring columns (one number per head)."""
    if use_native(g):
        return native_hybrid().sigmoid_gate_mul(o, g)
    return ref.sigmoid_gate_mul(o, g)


MLSTM_CHUNK = 128  # tokens per chunk of the chunk-parallel scan; portions of >= 2 chunks take it


def mlstm_scan(q, k, v, if_raw, b_i, b_f, cap: float, qscale: float, S, n, m, state_slots, cu, start, slab: bool = False,
               cu_host=None):
    """mLSTM recurrence over the step's tokens; returns the un-normalised head outputs fp32
    ``[T, H, dv]`` and updates the state pools in place.  ``slab`` forces the block-per-tile kernel
    (the form for key dims above 128) where the wave-per-tile one would run.  ``cu_host`` (the row
    offsets as a host list) lets long portions run chunk-parallel (:func:`_mlstm_scan_chunked`)."""
    if use_native(q):
        if (cu_host is not None and not slab and q.shape[-1] <= 128
                and max((b - a for a, b in zip(cu_host[:-1], cu_host[1:])), default=0) >= 2 * MLSTM_CHUNK):
            return _mlstm_scan_chunked(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, start, cu_host)
        return native_hybrid().mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, cu, start, slab)
    return ref.mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, cu, start)


def _mlstm_scan_chunked(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, start, cu_host):
    """The same token-by-token recurrence with the chunks of a portion running side by side.  The state
    is linear in its past: over a chunk with summed log forget gates F and own contribution (S_loc, m_loc)
    -- the chunk run from a zero state with m = -inf -- the carried state becomes m' = max(F + m, m_loc),
    S' = e^(F + m - m') S + e^(m_loc - m') S_loc, and m' is exactly the stabiliser the sequential run
    reaches.  Three passes: (1) every chunk's own contribution, all chunks at once, no outputs; (2) the
    states at every chunk's first token, chunk after chunk (elementwise); (3) every chunk again from its
    true state, all at once, writing the outputs token by token as the sequential form does.  A single
    prompt thus fills chunks x heads x value-tiles waves instead of heads x value-tiles."""
    nat = native_hybrid()
    dev = q.device
    H, dk, dv = q.shape[1], q.shape[2], v.shape[2]
    pcu, base = [0], [0]
    for a, b in zip(cu_host[:-1], cu_host[1:]):
        t = a
        while t < b:
            t = min(t + MLSTM_CHUNK, b)
            pcu.append(t)
        base.append(len(pcu) - 1)
    P = len(pcu) - 1
    i32 = lambda x: torch.tensor(x, dtype=torch.int32).to(dev, non_blocking=True)
    pcu_d, base_d, ident = i32(pcu), i32(base), torch.arange(P, dtype=torch.int32, device=dev)
    f32 = dict(dtype=torch.float32, device=dev)
    locS, locn, locm = torch.empty(P, H, dk, dv, **f32), torch.empty(P, H, dk, **f32), torch.empty(P, H, **f32)
    fsum = torch.empty(P, H, **f32)
    nat.mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, locS, locn, locm, ident, pcu_d,
                   torch.full((P,), -1, dtype=torch.int32, device=dev), False, fsum, False)
    iS, in_, im = torch.empty_like(locS), torch.empty_like(locn), torch.empty_like(locm)
    nat.mlstm_chunk_combine(S, n, m, state_slots, start, base_d, locS, locn, locm, fsum, iS, in_, im)
    out = nat.mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, iS, in_, im, ident, pcu_d,
                         torch.ones(P, dtype=torch.int32, device=dev), False, None, True)
    live = [s for s in range(len(base) - 1) if base[s + 1] > base[s]]
    if live:  # the last chunk's final state is the sequence's new carried state
        last = torch.tensor([base[s + 1] - 1 for s in live], dtype=torch.long).to(dev, non_blocking=True)
        dst = state_slots.long()[torch.tensor(live, dtype=torch.long).to(dev, non_blocking=True)]
        S.index_copy_(0, dst, iS.index_select(0, last))
        n.index_copy_(0, dst, in_.index_select(0, last))
        m.index_copy_(0, dst, im.index_select(0, last))
    return out


def headnorm_gate(o, w, g, eps: float, out_dtype, silu: bool = False):
    """Per-head unit-RMS of ``o [T, H, dv]`` (fp32), times ``w [H*dv]``, times ``sigmoid(g)`` (``silu``:
    times ``g sigmoid(g)``)."""
    if use_native(o):
        return native_hybrid().headnorm_gate(o, w, g, eps, out_dtype == torch.bfloat16, silu)
    return ref.headnorm_gate(o, w, g, eps, out_dtype, silu)


def group_topk_router(logits, top: int, groups: int, keep: int):
    """Sigmoid scores of ``logits [T, E]`` (fp32); experts in ``groups`` equal groups of neighbours,
    a group scored by the sum of its two best experts, the ``top`` best experts of the ``keep`` best
    groups chosen.  Returns (expert ids int64 [T, top], their scores fp32 [T, top])."""
    if use_native(logits):
        return native_hybrid().group_topk_router(logits, top, groups, keep)
    return ref.group_topk_router(logits, top, groups, keep)


def swiglu_any(gu):
    """``silu(gate) * up`` of ``gu [..., 2F]`` = ``[gate | up]``, bf16 or fp32."""
    if use_native(gu):
        return native_hybrid().swiglu_any(gu.contiguous())
    return ref.swiglu_any(gu)


def gated_norm_add_norm_f32_(x, y, r, w_post, w_next, eps: float, out_dtype):
    """A sublayer's result into the fp32 residual stream of a layer with norms on both sides and a
    gated residual, in one pass: ``g = y sigmoid(r)``; ``x += g / rms(g) * w_post`` in place; returns
    ``x / rms(x) * w_next`` -> ``out_dtype`` (the next sublayer's input), or None when ``w_next`` is None.
    ``y`` and ``r`` are ``[T, W]`` in the activation dtype or fp32 (row-strided views allowed)."""
    if use_native(x):
        h = native_hybrid().gated_norm_add_norm_f32_(x, y, r, w_post, w_next, eps, out_dtype == torch.bfloat16)
        return h if w_next is not None else None
    return ref.gated_norm_add_norm_f32_(x, y, r, w_post, w_next, eps, out_dtype)


def embed_rmsnorm_f32(ids, pos, table, pos_table, w, eps: float, out_dtype):
    """``x = table[ids] + pos_table[pos]`` (learned absolute positions) as the fp32 residual stream, and
    its RMS norm with weight ``w`` -> ``out_dtype``.  Returns (x, h)."""
    if use_native(table):
        return native_hybrid().embed_rmsnorm_f32(ids, pos, table, pos_table, w, eps, out_dtype == torch.bfloat16)
    return ref.embed_rmsnorm_f32(ids, pos, table, pos_table, w, eps, out_dtype)


GLA_CHUNK = 64  # tokens per chunk of the chunk-parallel scan; portions of >= 4 chunks take it


def gla_chunk_plan(cu_host, device):
    """The chunks of a step's portions for the chunk-parallel scan, or None when no portion is long enough:
    (chunk row offsets, first chunk of every sequence, 0 .. P-1, P zeros, P ones) on ``device`` and P.  It
    depends on the step only, so the layers of a model share one."""
    if cu_host is None or max((b - a for a, b in zip(cu_host[:-1], cu_host[1:])), default=0) < 4 * GLA_CHUNK:
        return None
    pcu, base = [0], [0]
    for a, b in zip(cu_host[:-1], cu_host[1:]):
        t = a
        while t < b:
            t = min(t + GLA_CHUNK, b)
            pcu.append(t)
        base.append(len(pcu) - 1)
    P = len(pcu) - 1
    both = torch.tensor(pcu + base, dtype=torch.int32).to(device)  # blocking: the host tensor is a temporary
    ident = torch.arange(P, dtype=torch.int32, device=device)
    return (both[:P + 1], both[P + 1:], ident, torch.zeros(P, dtype=torch.int32, device=device),
            torch.ones(P, dtype=torch.int32, device=device), P)


def gla_scan(q, k, v, z, z_bias, tau: float, qscale: float, S, state_slots, cu, start, cu_host=None, plan=None):
    """Gated linear attention over the step's tokens: per head a memory ``S [dk, dv]`` with a decay per
    key channel, ``a_t = sigmoid(z_t + z_bias)^(1/tau)`` (computed as ``exp(log_sigmoid / tau)`` in fp32),
    ``S_t = diag(a_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T (q_t qscale)``.  ``q, k [T, H, dk]``, ``v [T, H, dv]``
    (row-strided views allowed), ``z [T, H*dk]`` fp32, ``z_bias`` fp32 ``[H*dk]``.
    Returns fp32 ``[T, H, dv]`` and updates the state pool ``S [slots, H, dk, dv]`` in place at
    ``state_slots[seq]`` (a sequence with ``start == 0`` begins from zeros).  ``cu_host`` (the row offsets on
    the host) or ``plan`` (:func:`gla_chunk_plan` of them) lets long portions run chunk-parallel."""
    if use_native(q):
        nat = native_hybrid()
        if plan is None and cu_host is not None:
            plan = gla_chunk_plan(cu_host, q.device)
        if plan is not None:
            return _gla_scan_chunked(nat, q, k, v, z, z_bias, tau, qscale, S, state_slots, start, plan)
        return nat.gla_scan(q, k, v, z, z_bias, tau, qscale, S, state_slots, cu, start, None, True, True)
    return ref.gla_scan(q, k, v, z, z_bias, tau, qscale, S, state_slots, cu, start)


def _gla_scan_chunked(nat, q, k, v, z, z_bias, tau, qscale, S, state_slots, start, plan):
    """The same recurrence with the chunks of a portion side by side.  The memory is linear in its past:
    over a chunk with total decay D (the product of its a_t per key channel) and own contribution S_loc (the
    chunk run from zeros), S_end = diag(D) S_begin + S_loc.  Three passes: (1) every chunk from zeros, all at
    once, no outputs, giving (S_loc, log D); (2) the memory at every chunk's first token, chunk after chunk
    (elementwise), and the sequence's new carried memory; (3) every chunk again from its true memory, all at
    once, writing outputs token by token."""
    pcu_d, base_d, ident, zeros, ones, P = plan
    H, dk, dv = q.shape[1], q.shape[2], v.shape[2]
    f32 = dict(dtype=torch.float32, device=q.device)
    loc, logd = torch.empty(P, H, dk, dv, **f32), torch.empty(P, H, dk, **f32)
    nat.gla_scan(q, k, v, z, z_bias, tau, qscale, loc, ident, pcu_d, zeros, logd, False, True)
    init = torch.empty_like(loc)
    nat.gla_chunk_combine(S, state_slots, start, base_d, loc, logd, init)
    return nat.gla_scan(q, k, v, z, z_bias, tau, qscale, init, ident, pcu_d, ones, None, True, False)


def qk_fullnorm_prep(z, H: int, G: int, dk: int, dv: int, q_norm, k_norm, eps: float, pos, temp_coef: float,
                     temp_every: int, cache, slots):
    """``z [T, >= H*dk + G*dk + G*dv] = [q | k | v | ...]`` (biases already added): RMS norm over the whole
    of q and over the whole of k before the split into heads (weights fp32 ``[H*dk]``, ``[G*dk]``); the query
    temperature ``1 + temp_coef ln(floor((p + 1) / temp_every) + 1)`` at position p (``temp_coef`` 0: none);
    k and v are written to the token's cache row ``[G, dv + dk] = [v | k]`` at ``slots``; returns q ``[T, H, dk]``."""
    if use_native(z):
        return native_hybrid().qk_fullnorm_prep(z, H, G, dk, dv, q_norm, k_norm, eps, pos, temp_coef, temp_every, cache, slots)
    return ref.qk_fullnorm_prep(z, H, G, dk, dv, q_norm, k_norm, eps, pos, temp_coef, temp_every, cache, slots)


def bias_topk_router(logits, bias, top: int, groups: int = 1, keep: int = 1, renorm: bool = True):
    """Softmax scores of ``logits [T, E]`` (fp32); the ``top`` experts with the largest ``score + bias`` (the
    choice score; ``bias`` None: the score) are chosen (ties: the lower index).  ``groups`` > 1: the experts
    form that many equal groups of neighbours, a group's score is its largest choice score, and only experts
    of the ``keep`` best groups can be chosen.  The weights are the chosen experts' own scores (without the
    bias), over their sum (+ 1e-20) when ``renorm``.  Returns (expert ids int64 [T, top], weights fp32 [T, top])."""
    if use_native(logits):
        return native_hybrid().bias_topk_router(logits, bias, top, groups, keep, renorm)
    return ref.bias_topk_router(logits, bias, top, groups, keep, renorm)


def act_any(x, kind: str):
    """Elementwise activation of ``x`` (bf16 or fp32, computed in fp32): ``relu2`` = relu(x)^2, ``gelu`` = the
    exact (erf) GELU."""
    if use_native(x):
        return native_hybrid().act_any(x, {"relu2": 0, "gelu": 1}[kind])
    return ref.act_any(x, kind)


def hc_embed_norm(ids, table, streams: int, c_in, g, eps: float, out_dtype):
    """The start of ``streams`` residual streams (hyper-connections): every stream is the embedding row.
    Returns (``X`` fp32 ``[T, streams, W]``, the first sublayer's input ``norm(sum_s c_in[s] x_s) * g`` ->
    ``out_dtype``); ``c_in`` fp32 ``[streams]``, ``g`` fp32, one number (an RMS norm with a single weight)."""
    if use_native(table):
        return native_hybrid().hc_embed_norm(ids, table, streams, c_in, g, eps, out_dtype == torch.bfloat16)
    return ref.hc_embed_norm(ids, table, streams, c_in, g, eps, out_dtype)


def hc_update_norm_(X, y1, s1: float, y2, s2: float, mix, c_out, mult: float, c_in, g, eps: float, out_dtype):
    """A sublayer's result into the residual streams ``X`` (fp32 ``[T, S, W]``, in place), all streams at once
    from the old ones: ``x_t <- sum_s mix[s, t] x_s + mult c_out[t] (s1 y1 + s2 y2)`` (``y2`` may be None; ``y``
    ``[T, W]`` in the activation dtype or fp32, row-strided views allowed), and the next sublayer's input
    ``norm(sum_t c_in[t] x_t) * g`` -> ``out_dtype`` in the same pass over the row (None when ``c_in`` is None).
    One stream with ``mix = c_out = c_in = 1`` is the plain residual sum with a pre-norm."""
    if use_native(X):
        h = native_hybrid().hc_update_norm_(X, y1, s1, y2, s2, mix, c_out, mult, c_in, g, eps, out_dtype == torch.bfloat16)
        return h if c_in is not None else None
    return ref.hc_update_norm_(X, y1, s1, y2, s2, mix, c_out, mult, c_in, g, eps, out_dtype)


def delta_scan(r, k, v, zw, w0, za, ab, decay_coef: float, key_eps: float, S, state_slots, cu, start, cu_host=None, plan=None):
    """The generalized delta rule over the step's tokens: per head a memory ``S [dk, dv]``; with the decay
    ``w = exp(-decay_coef sigmoid(zw + w0))`` and the removal rate ``a = sigmoid(za + ab)`` per key channel and the
    unit key ``u = k / sqrt(sum k^2 + key_eps)``, ``S_t = diag(w_t) S_(t-1) - (a_t u_t) (u_t^T S_(t-1)) + k_t v_t^T``
    (both terms read the old memory) and ``o_t = S_t^T r_t``.  ``r, k [T, H, dk]``, ``v [T, H, dv]`` (row-strided
    views allowed), ``zw`` fp32 ``[T, H*dk]``, ``za [T, H*dk]`` (any float dtype), ``w0``, ``ab`` fp32 ``[H*dk]``.
    Returns fp32 ``[T, H, dv]`` and updates the state pool ``S [slots, H, dk, dv]`` in place at ``state_slots[seq]``
    (a sequence with ``start == 0`` begins from zeros).  ``plan`` (:func:`gla_chunk_plan` of the row offsets)
    lets long portions run chunk-parallel."""
    if use_native(r):
        nat = native_hybrid()
        if plan is None and cu_host is not None:
            plan = gla_chunk_plan(cu_host, r.device)
        if plan is not None and DELTA_CHUNKED and _delta_combine_fits(k.shape[2], v.shape[2]):
            return _delta_scan_chunked(nat, r, k, v, zw, w0, za, ab, decay_coef, key_eps, S, state_slots, start, plan)
        return nat.delta_scan(r, k, v, zw, w0, za, ab, decay_coef, key_eps, S, state_slots, cu, start, None, True, True)
    return ref.delta_scan(r, k, v, zw, w0, za, ab, decay_coef, key_eps, S, state_slots, cu, start)


DELTA_CHUNKED = True  # long portions run chunk-parallel


def _delta_combine_fits(dk: int, dv: int) -> bool:
    """The combine pass holds a head's memory and a chunk's transition product in LDS and tiles them 4 x 4."""
    return dk % 4 == 0 and dv % 4 == 0 and 4 * dk * (dk + dv) <= 65536 and dk * dk <= 48 * 256 and dk * dv <= 8192


def _delta_scan_chunked(nat, r, k, v, zw, w0, za, ab, decay_coef, key_eps, S, state_slots, start, plan):
    """The same recurrence with the chunks of a portion side by side.  The memory is linear in its past: a token
    maps it by ``A_t = diag(w_t) - (a_t u_t) u_t^T`` and adds ``k_t v_t^T``, so over a chunk with transition product
    ``P = A_n ... A_1`` and own contribution ``S_loc`` (the chunk run from zeros), ``S_end = P S_begin + S_loc``.  Three
    passes: (1) every chunk from zeros and, in further waves of the same launch, from the identity without the
    ``k v^T`` term, all at once, no outputs, giving ``(S_loc, P^T)``; (2) the memory at every chunk's first token, chunk
    after chunk, and the sequence's new carried memory; (3) every chunk again from its true memory, all at once,
    writing outputs token by token."""
    pcu_d, base_d, ident, zeros, ones, Pn = plan
    H, dk, dv = r.shape[1], r.shape[2], v.shape[2]
    f32 = dict(dtype=torch.float32, device=r.device)
    loc, prod = torch.empty(Pn, H, dk, dv, **f32), torch.empty(Pn, H, dk, dk, **f32)
    nat.delta_scan(r, k, v, zw, w0, za, ab, decay_coef, key_eps, loc, ident, pcu_d, zeros, prod, False, True)
    init = torch.empty_like(loc)
    nat.delta_chunk_combine(S, state_slots, start, base_d, loc, prod, init)
    return nat.delta_scan(r, k, v, zw, w0, za, ab, decay_coef, key_eps, init, ident, pcu_d, ones, None, True, False)


def tanh_act(x):
    """Elementwise ``tanh`` (computed in fp32) -> x's dtype."""
    if use_native(x):
        return native_hybrid().tanh_act(x.contiguous())
    return ref.tanh_act(x)


def softcap_(x, cap: float):
    """``x <- cap tanh(x / cap)`` in place on an fp32 tensor."""
    if use_native(x):
        native_hybrid().softcap_(x, cap)
        return x
    return ref.softcap_(x, cap)



def gated_add_f32_(out, y, g):
    """``out += y * sigmoid(g)`` in place on the fp32 ``out [T, W]``; ``y [T, W]`` in any float dtype, ``g [T, 1]``
    one gate logit per row (row-strided views allowed)."""
    if use_native(out):
        native_hybrid().gated_add_f32_(out, y, g)
        return out
    return ref.gated_add_f32_(out, y, g)
