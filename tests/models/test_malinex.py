"""Malinex through the serving engine against the plain whole-sequence implementation in
``tests/oracles/malinex_plain.py``: every mechanism alone, whole prompts against token-by-token decoding,
portions down to two tokens, unequal batches, reused pages and state slots, far keys and the edges of
pages, key tiles, scan chunks and temperature steps, the first tokens of a sequence, long decoding, other
sizes, and greedy generation through the scheduler.

Each test runs on the CPU path and, marked ``gpu``, on the HIP kernels: fp32 with a tight bound at every
position; bf16 with loose bounds on the median and on nine positions in ten and a sanity bound on the rest (the norm that
follows every sublayer brings a near-zero result to unit size, so in these tiny models single positions
react strongly to bf16 rounding: a read-out of one stored token is the sign of a dot product)."""

import math
import random

import pytest
import torch

from tests.models import malinex_util as U
from tests.oracles import malinex_plain as plain

DEVICES = [("cpu", torch.float32, 2e-4),
           pytest.param(("cuda", torch.float32, 2e-4), marks=pytest.mark.gpu),
           pytest.param(("cuda", torch.bfloat16, 0.1), marks=pytest.mark.gpu)]


@pytest.fixture(params=DEVICES, ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def dev(request):
    return request.param


def tokens(n, vocab, seed):
    r = random.Random(seed)
    return [r.randrange(vocab) for _ in range(n)]


def check(tmp_path, dev, cfg, requests, steps, seed=0, blocks=64, block_size=4, W=None, max_seqs=4, bf16_tol=None,
          bf16_dense=False):
    """``bf16_dense``: the bf16 run replaces routed experts by dense feed-forwards (an expert near-tie that
    flips under bf16 rounding changes all later positions through the recurrent state; routed experts in
    bf16 are covered by the one-layer tests)."""
    device, dtype, tol = dev
    if bf16_tol is not None and dtype == torch.bfloat16:
        tol = bf16_tol
    if bf16_dense and dtype == torch.bfloat16:
        cfg = U.without_experts(cfg)
    W = {k: v.bfloat16().float() for k, v in (W if W is not None else U.random_weights(cfg, seed)).items()}
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W), device, dtype, blocks, block_size, max_seqs)
    free0 = eng.kv.num_free_blocks
    got = U.run_schedule(eng, requests, steps)
    assert eng.kv.num_free_blocks == free0 and (eng.kv_cache.slots is None or eng.kv_cache.slots.num_free == max_seqs)
    errs = {rid: U.rel_errs(got[rid], plain.forward(cfg, W, toks).float()) for rid, toks in requests.items()}
    if dtype == torch.bfloat16:  # over all positions of the test: the median, nine in ten, and a sanity bound on the rest
        per = torch.cat(list(errs.values()))
        assert float(per.median()) < tol / 2 and float(per.quantile(0.9)) < 2 * tol and float(per.max()) < 1.0, per
    else:
        for rid, per in errs.items():
            assert float(per.max()) < tol, f"{rid}: {per.max()} at {int(per.argmax())}"
    eng.close()


def whole(requests):
    return [[(rid, len(t))] for rid, t in requests.items()]


FULL = [(U.gla(), U.dense()), (U.att(), U.moe()), (U.gla(heads=2, dim=4, vdim=7, tau=9.0, rank=3), U.moe(shared=0)),
        (U.att(heads=2, kv_heads=1, dim=6, vdim=10, coef=None), None), (U.gla(), None), (U.att(), U.dense(12))]
SHARE = {4: 0, 5: 1}


# ------------------------------------------------------------------ each mechanism alone
def test_gla_alone(tmp_path, dev):
    cfg = U.config([(U.gla(), None)])
    r = {"a": tokens(23, 50, 1)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("sizes", [dict(heads=1, dim=1, vdim=1, tau=1.0, rank=1), dict(heads=2, dim=20, vdim=70, tau=2.5, rank=4),
                                   dict(heads=1, dim=130, vdim=9, tau=30.0, rank=2), dict(heads=5, dim=17, vdim=3, tau=12.0, rank=7)])
def test_gla_sizes(tmp_path, dev, sizes):
    # one channel; more value columns than a wave has lanes; more key channels than a lane's first tier; odd sizes
    cfg = U.config([(U.gla(**sizes), None)])
    r = {"a": tokens(19, 50, 2)}
    # (a head of one value column normalises to a sign: loose in bf16)
    check(tmp_path, dev, cfg, r, [[("a", 7)], [("a", 1)], [("a", 11)]], bf16_tol=0.5 if sizes["vdim"] == 1 else None)


def test_gla_slow_and_fast_decay(tmp_path, dev):
    # half of the key channels nearly keep their memory (decay ~ 1), the others lose it within a token or two:
    # a decay applied to the value columns, to the wrong head, or with the wrong power shows
    cfg = U.config([(U.gla(heads=2, dim=6, vdim=5, tau=2.0), None)])
    W = U.random_weights(cfg, 3)
    b = torch.full((12,), 9.0)
    b[::2] = -6.0
    W["l0.mix.a2.b"] = b
    r = {"a": tokens(40, 50, 3)}
    check(tmp_path, dev, cfg, r, [[("a", 13)], [("a", 27)]])


def test_attention_alone(tmp_path, dev):
    cfg = U.config([(U.att(), None)])
    r = {"a": tokens(23, 50, 4)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("sizes", [dict(heads=3, kv_heads=3, dim=10, vdim=4), dict(heads=6, kv_heads=1, dim=4, vdim=8, coef=None),
                                   dict(heads=1, kv_heads=1, dim=2, vdim=2, every=1, coef=1.5), dict(heads=4, kv_heads=2, dim=8, vdim=16, scale=0.9, every=7)])
def test_attention_sizes(tmp_path, dev, sizes):
    # as many kv heads as heads, one kv head, one head, no temperature, a temperature step at every position,
    # a scale that is not dim^-1/2, key and value sizes that differ
    cfg = U.config([(U.att(**sizes), None)])
    r = {"a": tokens(26, 50, 5)}
    check(tmp_path, dev, cfg, r, [[("a", 9)], [("a", 1)], [("a", 16)]])


def test_distance_penalty_and_head_bias_take_effect(tmp_path, dev):
    # the heads' penalties and biases differ widely: one left out, swapped, or put on the wrong head shows
    cfg = U.config([(U.att(heads=4, kv_heads=2), None)])
    W = U.random_weights(cfg, 6)
    W["l0.mix.r1"] = torch.tensor([0.0, 3.0, 0.5, 1.5])
    W["l0.mix.r2"] = torch.tensor([2.0, 0.05, 8.0, 1.0])
    W["l0.mix.pb"] = torch.tensor([-4.0, 3.0, 0.0, -1.0])
    r = {"a": tokens(33, 50, 6)}
    check(tmp_path, dev, cfg, r, [[("a", 20)]] + [[("a", 1)]] * 13)


def test_query_temperature_steps(tmp_path, dev):
    # a large coefficient and a period of 4: the factor changes where (p + 1) / 4 crosses an integer
    cfg = U.config([(U.att(coef=2.0, every=4, scale=0.6), None)])
    r = {"a": tokens(18, 50, 7)}
    check(tmp_path, dev, cfg, r, [[("a", 3)], [("a", 1)], [("a", 4)], [("a", 7)], [("a", 1)], [("a", 2)]])


def test_dense_feed_forward(tmp_path, dev):
    cfg = U.config([(U.att(heads=1, kv_heads=1), U.dense(33))])
    r = {"a": tokens(30, 50, 8)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("f", [dict(experts=5, top=1, ff=7, shared=9), dict(experts=4, top=4, ff=6, shared=0), dict(experts=9, top=3, ff=5, shared=4)])
def test_routed_feed_forward(tmp_path, dev, f):
    cfg = U.config([(U.gla(), U.moe(**f))])
    r = {"a": tokens(30, 50, 9)}
    check(tmp_path, dev, cfg, r, whole(r), bf16_tol=0.25)


@pytest.mark.parametrize("form", ["dense", "batched", "segments"])
def test_expert_forms(tmp_path, dev, form, monkeypatch):
    # steps of few rows run all experts on all rows (unchosen ones weighted by zero); longer ones sort token copies by
    # expert and run the segments as one batch padded to the largest, or, if routing is unbalanced, one by one;
    # here every step is forced into one form
    from llmctl.models.moe import BiasedSoftmaxMoE

    if form == "batched" and dev[0] == "cuda":
        pytest.skip("the batched-segment form is switched off on GPUs: a 2048-token step through it ended in a GPU "
                    "memory fault whose cause is not found")
    monkeypatch.setattr(BiasedSoftmaxMoE, "_dense", lambda self, T: form == "dense")
    monkeypatch.setattr(BiasedSoftmaxMoE, "_batched", lambda self, N, C: form == "batched")
    cfg = U.config([(U.gla(), U.moe(experts=7, top=3, ff=9, shared=5)), (U.att(), U.moe(experts=3, top=1, ff=16, shared=0))])
    r = {"a": tokens(70, 50, 40), "b": tokens(6, 50, 41)}
    check(tmp_path, dev, cfg, r, [[("a", 1)], [("a", 66), ("b", 2)], [("a", 3), ("b", 4)]], bf16_tol=0.25)


def test_selection_bias_chooses_but_does_not_weigh(tmp_path, dev):
    # a bias far larger than any score: the two experts it favours are always chosen, whatever their scores,
    # and are weighted by their scores alone
    cfg = U.config([(U.gla(), U.moe(experts=6, top=2, shared=0))])
    W = U.random_weights(cfg, 10)
    W["l0.mlp.correction"] = torch.tensor([0.0, 5.0, -3.0, 0.0, 4.0, 0.0])
    r = {"a": tokens(21, 50, 10)}
    check(tmp_path, dev, cfg, r, whole(r))
    idx, w = plain.route(W, "l0.mlp.", cfg["layers"][0]["mlp"], torch.randn(8, 20, dtype=torch.float64))
    assert sorted(set(idx.flatten().tolist())) == [1, 4] and torch.allclose(w.sum(-1), torch.ones(8, dtype=torch.float64))


def test_gated_residual_nearly_shut_and_wide_open(tmp_path, dev):
    cfg = U.config([(U.gla(), U.dense()), (U.att(), U.dense())])
    W = U.random_weights(cfg, 11)
    b = torch.full((20,), 6.0)
    b[:10] = -6.0
    W["l0.rg1.b"], W["l1.rg2.b"] = b, b.flip(0)
    r = {"a": tokens(16, 50, 11)}
    check(tmp_path, dev, cfg, r, whole(r))


def test_layers_that_share_weights_keep_their_own_cache(tmp_path, dev):
    cfg = U.config(FULL, share=SHARE)
    r = {"a": tokens(21, 50, 12)}
    check(tmp_path, dev, cfg, r, [[("a", 8)], [("a", 1)], [("a", 12)]], bf16_dense=True)


def test_stream_after_every_layer(tmp_path, dev):
    from llmctl.serve.scheduler import PrefillChunk

    device, dtype, _ = dev
    cfg = U.config(FULL, share=SHARE)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 13).items()}
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W), device, dtype)
    toks = tokens(11, 50, 13)
    seq = eng.open_sequence(toks, request_id="a")
    trail = []
    eng.forward_portions([PrefillChunk(seq, 0, len(toks))], [[len(toks) - 1]], trail=trail)
    want = []
    plain.forward(cfg, W, toks, trail=want)
    assert len(trail) == len(want) == 6
    for got, w in zip(trail, want):
        assert float((got.double().cpu() - w).abs().max() / w.abs().max()) < (1e-4 if dtype == torch.float32 else 0.08)
    eng.close()


def test_positions_and_logit_scale(tmp_path, dev):
    # no layers at all: embedding plus position vector, final norm, head, scale
    cfg = U.config([], logit_scale=1.0)
    r = {"a": tokens(9, 50, 14)}
    check(tmp_path, dev, cfg, r, [[("a", 4)], [("a", 1)], [("a", 4)]])
    cfg = U.config([(U.gla(), None)], logit_scale=3.5)
    check(tmp_path, dev, cfg, r, whole(r))


def test_position_beyond_the_table_is_refused(tmp_path):
    cfg = U.config([(U.gla(), None)], max_positions=6)
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", U.clean(cfg), U.random_weights(cfg, 1)), "cpu")
    with pytest.raises(ValueError):
        U.run_schedule(eng, {"a": tokens(7, 50, 1)}, [[("a", 7)]])
    eng.close()


# ------------------------------------------------------------------ schedules
def test_all_layers_whole_prompts(tmp_path, dev):
    cfg = U.config(FULL, share=SHARE)
    r = {"a": tokens(37, 50, 15), "b": tokens(1, 50, 16), "c": tokens(2, 50, 17)}
    check(tmp_path, dev, cfg, r, whole(r), bf16_dense=True)


def test_prefill_against_token_by_token(tmp_path, dev):
    cfg = U.config(FULL, share=SHARE)
    r = {"a": tokens(26, 50, 18)}
    check(tmp_path, dev, cfg, r, [[("a", 1)]] * 26, bf16_dense=True)


@pytest.mark.parametrize("sizes", [[2] * 12, [5, 2, 7, 3, 1, 6], [1, 23], [13, 2, 2, 2, 2, 1, 1, 1]])
def test_portions(tmp_path, dev, sizes):
    cfg = U.config(FULL, share=SHARE)
    r = {"a": tokens(24, 50, 19)}
    check(tmp_path, dev, cfg, r, [[("a", n)] for n in sizes], bf16_dense=True)


def test_unequal_batch_against_each_alone(tmp_path, dev):
    cfg = U.config(FULL, share=SHARE)
    r = {"a": tokens(30, 50, 20), "b": tokens(9, 50, 21), "c": tokens(17, 50, 22), "d": tokens(3, 50, 23)}
    steps = [[("a", 11), ("b", 2)], [("a", 1), ("b", 5), ("c", 9)], [("c", 1), ("a", 1), ("d", 3), ("b", 1)],
             [("a", 7), ("b", 1), ("c", 1)], [("c", 6), ("a", 1)], [("a", 9)]]
    check(tmp_path, dev, cfg, r, steps, bf16_dense=True)


def test_pages_and_slots_used_again(tmp_path, dev):
    # a pool of 12 pages of 4 tokens and 2 state slots serves five requests one after another and
    # interleaved; what a finished request left in its pages and slot must not leak into the next
    cfg = U.config(FULL, share=SHARE)
    r = {k: tokens(n, 50, 24 + i) for i, (k, n) in enumerate([("a", 22), ("b", 18), ("c", 21), ("d", 9), ("e", 20)])}
    steps = [[("a", 22)], [("b", 10)], [("b", 8), ("c", 5)], [("c", 16)], [("d", 4), ("e", 3)], [("d", 1), ("e", 1)],
             [("d", 4), ("e", 16)]]
    check(tmp_path, dev, cfg, r, steps, blocks=12, block_size=4, max_seqs=2, bf16_dense=True)


def test_first_tokens_one_by_one_in_a_used_slot(tmp_path, dev):
    # the second request starts token by token in the slot and pages the first one left behind: its memory
    # must start from zeros, not from the old owner's
    cfg = U.config(FULL, share=SHARE)
    r = {"a": tokens(12, 50, 30), "b": tokens(8, 50, 31)}
    steps = [[("a", 12)]] + [[("b", 1)]] * 3 + [[("b", 2)], [("b", 3)]]
    check(tmp_path, dev, cfg, r, steps, blocks=8, block_size=4, max_seqs=1, bf16_dense=True)


def test_long_decoding(tmp_path, dev):
    # decoded tokens pass two 64-key tiles, many pages and several temperature steps
    cfg = U.config([(U.gla(), U.dense()), (U.att(every=32), None), (U.gla(), None), (U.att(every=32), U.dense())], share={2: 0, 3: 1})
    r = {"a": tokens(140, 50, 32)}
    check(tmp_path, dev, cfg, r, [[("a", 6)]] + [[("a", 1)]] * 134, block_size=8)


def test_long_portions_in_one_step(tmp_path, dev):
    # portions longer than four scan chunks and two query blocks; the second step goes on from the first one's
    # memory and rows, beside a short request
    cfg = U.config([(U.gla(heads=2, dim=16, vdim=24), U.dense()), (U.att(heads=4, kv_heads=2, dim=16, vdim=16, every=100), None)],
                   width=32, max_positions=700)
    r = {"a": tokens(650, 50, 33), "b": tokens(150, 50, 34), "c": tokens(5, 50, 35)}
    check(tmp_path, dev, cfg, r, [[("a", 330), ("b", 70)], [("a", 320), ("b", 80), ("c", 5)]], blocks=60, block_size=16)


# ------------------------------------------------------------------ far keys, edges of pages and key tiles
def _attention_case(device, dtype, bs, L, j0, form, mfma=True, H=4, G=2, dk=8, dv=8):
    """Key row j0 matches every query of every head and the heads' biases are very negative, so every other
    key weighs next to nothing: the output at position i is row j0's value (times its weight) when j0 <= i
    and next to nothing before.  Pages lie in a shuffled order."""
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(5)
    rs = dv + dk
    nb = (L + bs - 1) // bs + 3
    perm = torch.randperm(nb, generator=g)
    rows = torch.randn(L, G, rs, generator=g) * 0.1
    u = torch.ones(dk) / dk ** 0.5
    rows[j0, :, dv:] = 30.0 * u
    rows[j0, :, :dv] = torch.randn(G, dv, generator=g)
    cache = torch.zeros(nb, bs, G * rs)
    bt = torch.zeros(1, nb, dtype=torch.int32)
    for p in range(L):
        bt[0, p // bs] = perm[p // bs]
        cache[perm[p // bs], p % bs] = rows[p].reshape(-1)
    q = (u * 2.0 + torch.randn(L, H, dk, generator=g) * 0.05)
    r1 = torch.tensor([0.0, 0.7, 0.2, 1.1]).repeat(H // 4 + 1)[:H]
    r2 = torch.tensor([1.0, 0.3, 4.0, 0.01]).repeat(H // 4 + 1)[:H]
    pb = torch.tensor([-12.0, -9.0, -14.0, -10.0]).repeat(H // 4 + 1)[:H]
    scale = 0.5
    cache, q = cache.to(dtype), q.to(dtype)
    w = plain.sigmoid_weights(q.double(), rows.to(dtype).double().repeat_interleave(H // G, 1)[:, :, dv:], scale, r1, r2, pb)
    want = torch.einsum("hij,jhd->ihd", w, rows.to(dtype).double().repeat_interleave(H // G, 1)[:, :, :dv])
    d = torch.device(device)
    kw = dict(groups=G, koff=dv, sig_bias=pb.to(d), dist_a=r1.to(d), dist_b=r2.to(d))
    if form == "prefill":
        cut = L // 3  # the portion starts in the middle of a page
        got = hybrid.latent_attention_prefill(q[cut:].contiguous().to(d), cache.to(d), bt.to(d), torch.tensor([0, L - cut], dtype=torch.int32).to(d),
                                              torch.tensor([L], dtype=torch.int32).to(d), hybrid.NO_LIMIT, None, scale, dv, L - cut,
                                              mfma=mfma, **kw)
        want = want[cut:]
    else:
        n = min(L, 24)  # the last n positions, each decoded alone, as one batch of n sequences
        ctx = torch.arange(L - n + 1, L + 1, dtype=torch.int32)
        got = hybrid.latent_attention_decode(q[L - n:].contiguous().to(d), cache.to(d), bt.expand(n, nb).contiguous().to(d), ctx.to(d),
                                             hybrid.NO_LIMIT, None, scale, dv, mfma=mfma, max_ctx=L, **kw)
        want = want[L - n:]
    return got.double().cpu(), want


@pytest.mark.parametrize("form", ["prefill", "decode"])
@pytest.mark.parametrize("bs,L,j0", [(4, 20, 15), (4, 20, 16), (8, 40, 31), (8, 40, 32), (16, 200, 63), (16, 200, 64), (16, 200, 191),
                                     (16, 200, 192), (16, 200, 195), (16, 420, 0), (16, 420, 3), (16, 420, 411), (16, 700, 1), (16, 700, 600)])
def test_far_keys_and_edges(dev, form, bs, L, j0):
    # the standing-out key lies far back, at the first positions, on either side of a page's and of a 64-key
    # tile's border, and on either side of the first decoded or prompt position that may see it
    device, dtype, _ = dev
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    for mfma in ([True, False] if (device == "cuda" and dtype == torch.bfloat16) else [True]):
        got, want = _attention_case(device, dtype, bs, L, j0, form, mfma)
        assert float(want.abs().max()) > 0.3  # the key is seen by some position
        assert float((got - want).abs().max()) < tol, (mfma, float((got - want).abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv", [(8, 4, 56, 40), (4, 4, 64, 32), (6, 1, 128, 128), (3, 3, 24, 40), (12, 4, 64, 64), (2, 1, 160, 136), (16, 16, 8, 8)])
def test_sigmoid_attention_kernels_gpu(H, G, dk, dv):
    # the matrix-core and the generic kernels on other head counts and sizes, prompt and decode forms
    for dtype, tol in ((torch.bfloat16, 3e-2), (torch.float32, 1e-4)):
        for form in ("prefill", "decode"):
            for mfma in (True, False):
                got, want = _attention_case("cuda", dtype, 16, 300, 170, form, mfma, H=H, G=G, dk=dk, dv=dv)
                assert float((got - want).abs().max()) < tol, (dtype, form, mfma)


def _memory_case(device, dtype, T, dk, dv, H, cuts, far, chunked):
    """One key channel per head keeps its memory (decay ~ 1) and holds what token ``far`` wrote; the other
    channels forget within a few tokens.  The last tokens ask for that channel.  Runs the op over the
    portions ``cuts`` with the memory carried in a two-slot pool whose slots hold another sequence's junk."""
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(7)
    q, k = torch.randn(T, H, dk, generator=g) * 0.3, torch.randn(T, H, dk, generator=g) * 0.3
    v = torch.randn(T, H, dv, generator=g)
    z = torch.randn(T, H * dk, generator=g) - 1.0
    zb = torch.randn(H * dk, generator=g) * 0.2
    keep = [(3 * h) % dk for h in range(H)]
    for h, c in enumerate(keep):
        z[:, h * dk + c] = 14.0
        k[:, h, c] = 0.0
        k[far, h, c] = 6.0
        q[T - 3:, h, c] = 5.0
    tau = 3.0
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    alpha = torch.sigmoid(z.double() + zb.double()).pow(1.0 / tau).view(T, H, dk)
    want, S_end = plain.decayed_memory(q.double() * 0.7, k.double(), v.double(), alpha)
    d = torch.device(device)
    S = torch.randn(2, H, dk, dv, generator=g).to(d)  # junk of an earlier owner
    outs, at = [], 0
    for n in cuts:
        cu = [0, n]
        o = hybrid.gla_scan(q[at:at + n].to(d), k[at:at + n].to(d), v[at:at + n].to(d), z[at:at + n].to(d), zb.to(d), tau, 0.7, S,
                            torch.tensor([1], dtype=torch.int32).to(d), torch.tensor(cu, dtype=torch.int32).to(d),
                            torch.tensor([at], dtype=torch.int32).to(d), cu_host=cu if chunked else None)
        outs.append(o.double().cpu())
        at += n
    assert at == T
    return torch.cat(outs), want, S[1].double().cpu(), S_end, keep


@pytest.mark.parametrize("T,cuts,far", [(40, [40], 2), (300, [300], 1), (300, [7, 1, 1, 290, 1], 5), (700, [257, 443], 3), (130, [64, 64, 2], 63)])
def test_memory_survives_and_forgets(dev, T, cuts, far):
    device, dtype, _ = dev
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    H, dk, dv = 3, 10, 12
    for chunked in ([False, True] if device == "cuda" else [False]):
        got, want, S, S_end, keep = _memory_case(device, dtype, T, dk, dv, H, cuts, far, chunked)
        scale = float(want.abs().max())
        assert float((got - want).abs().max()) / scale < tol, chunked
        assert float((S - S_end).abs().max()) / float(S_end.abs().max()) < tol, chunked
        # the kept channel still holds token ``far``'s value after T tokens; the last outputs are made of it
        assert float(want[T - 1].abs().max()) > 10.0 * float(want[T - 20].abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dk,dv", [(3, 5), (16, 64), (20, 100), (44, 72), (64, 128), (70, 33), (128, 64), (130, 70), (200, 64), (256, 16)])
def test_gla_scan_kernel_tiers_gpu(dk, dv):
    # every register tier of the scan, token by token and chunk-parallel, value sizes beside the 64-lane tile
    for dtype, tol in ((torch.float32, 2e-4), (torch.bfloat16, 3e-2)):
        for chunked in (False, True):
            got, want, S, S_end, _ = _memory_case("cuda", dtype, 280, dk, dv, 2, [150, 1, 129], 4, chunked)
            assert float((got - want).abs().max()) / float(want.abs().max()) < tol, (dtype, chunked)
            assert float((S - S_end).abs().max()) / float(S_end.abs().max()) < tol, (dtype, chunked)


# ------------------------------------------------------------------ the small passes against their formulas
def _devices_dtypes():
    out = [("cpu", torch.float32)]
    if torch.cuda.is_available():
        out += [("cuda", torch.float32), ("cuda", torch.bfloat16)]
    return out


@pytest.mark.parametrize("W", [7, 200, 1000, 2500])
def test_gated_norm_add_norm(W):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(W)
    for device, dtype in _devices_dtypes():
        for ydt in {torch.float32, dtype}:
            x, y, r = torch.randn(5, W, generator=g), torch.randn(5, W + 3, generator=g).to(ydt), torch.randn(5, 2 * W, generator=g).to(dtype)
            wp, wn = torch.randn(W, generator=g), torch.randn(W, generator=g)
            gate = y[:, 3:].double() * torch.sigmoid(r[:, W:].double())
            x2 = x.double() + plain.rms_unit(gate, 1e-5) * wp.double()
            h_want = plain.rms_unit(x2, 1e-5) * wn.double()
            xd = x.clone().to(device)
            h = hybrid.gated_norm_add_norm_f32_(xd, y.to(device)[:, 3:], r.to(device)[:, W:], wp.to(device), wn.to(device), 1e-5, dtype)
            assert h.dtype == dtype
            assert float((xd.double().cpu() - x2).abs().max()) < 1e-4
            assert float((h.double().cpu() - h_want).abs().max()) < (1e-4 if dtype == torch.float32 else 5e-2)
            xd = x.clone().to(device)
            assert hybrid.gated_norm_add_norm_f32_(xd, y.to(device)[:, 3:], r.to(device)[:, W:], wp.to(device), None, 1e-5, dtype) is None
            assert float((xd.double().cpu() - x2).abs().max()) < 1e-4


@pytest.mark.parametrize("E,top", [(4, 1), (6, 2), (16, 4), (5, 5), (70, 8)])
def test_bias_topk_router(E, top):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(E)
    z, b = torch.randn(37, E, generator=g) * 2.0, torch.randn(E, generator=g) * 0.3
    s = torch.softmax(z.double(), -1)
    idx = (s + b.double()).topk(top, -1).indices
    w = s.gather(1, idx)
    w = w / (w.sum(-1, keepdim=True) + 1e-20)
    for device, _ in _devices_dtypes():
        gi, gw = hybrid.bias_topk_router(z.to(device), b.to(device), top)
        assert torch.equal(gi.cpu().sort(-1).values, idx.sort(-1).values)
        dense = torch.zeros(37, E, dtype=torch.float64).scatter_(1, gi.cpu(), gw.double().cpu())
        assert float((dense - torch.zeros(37, E, dtype=torch.float64).scatter_(1, idx, w)).abs().max()) < 1e-5


@pytest.mark.parametrize("F,pad", [(5, 0), (96, 3), (128, 64), (1000, 8)])
def test_activations_on_a_column_range(F, pad):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(F)
    for device, dtype in _devices_dtypes():
        x = (torch.randn(9, F + pad, generator=g) * 2.0).to(dtype)
        xd = x.double()[:, :F]
        for kind, want in (("relu2", plain.relu2(xd)), ("gelu", plain.gelu_erf(xd))):
            got = hybrid.act_any(x.to(device)[:, :F], kind)
            assert got.shape == (9, F) and got.dtype == dtype
            tol = 1e-5 if dtype == torch.float32 else 2e-2
            assert float(((got.double().cpu() - want).abs() / (1.0 + want.abs())).max()) < tol


@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 8, 6), (8, 4, 64, 64), (3, 1, 5, 7), (2, 2, 160, 16)])
def test_whole_projection_norm_and_cache_rows(H, G, dk, dv):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(H * dk)
    T, bs = 11, 4
    for device, dtype in _devices_dtypes():
        z = torch.randn(T, (H + G) * dk + G * dv + H + 5, generator=g).to(dtype)
        wq, wk = torch.randn(H * dk, generator=g), torch.randn(G * dk, generator=g)
        pos = torch.tensor([0, 1, 2, 3, 4, 5, 6, 7, 50, 51, 300], dtype=torch.int32)
        slots = torch.randperm(6 * bs, generator=g)[:T]
        zd = z.double()
        temp = 1.0 + 0.4 * torch.log(torch.floor((pos.double() + 1.0) / 3.0) + 1.0)
        q_want = (plain.norm(zd[:, :H * dk], wq, 1e-5) * temp[:, None]).view(T, H, dk)
        k_want = plain.norm(zd[:, H * dk:(H + G) * dk], wk, 1e-5).view(T, G, dk)
        v_want = zd[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv)
        cache = torch.zeros(6, bs, G * (dv + dk), dtype=dtype, device=device)
        q = hybrid.qk_fullnorm_prep(z.to(device), H, G, dk, dv, wq.to(device), wk.to(device), 1e-5, pos.to(device), 0.4, 3, cache, slots.to(device))
        tol = 1e-5 if dtype == torch.float32 else 3e-2
        rows = cache.view(-1, G, dv + dk)[slots.to(device)].double().cpu()
        assert float((q.double().cpu() - q_want).abs().max()) < tol * float(q_want.abs().max())
        assert float((rows[:, :, dv:] - k_want).abs().max()) < tol * float(k_want.abs().max())
        assert float((rows[:, :, :dv] - v_want).abs().max()) < tol * 4
        untouched = torch.ones(6 * bs, dtype=torch.bool)
        untouched[slots] = False
        assert float(cache.view(-1, G * (dv + dk))[untouched.to(device)].abs().max()) == 0.0


# ------------------------------------------------------------------ the framework's own entry points
def test_greedy_generation_through_the_scheduler(tmp_path, dev):
    from llmctl.serve.scheduler import SamplingParams

    device, dtype, _ = dev
    cfg = U.config(FULL, share=SHARE)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 50).items()}
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W)
    eng = U.engine(path, device, dtype, blocks=40, block_size=4, max_seqs=3, scheduler="dynamic")
    prompts = [tokens(9, 50, 51), tokens(2, 50, 52), tokens(14, 50, 53), tokens(5, 50, 54), tokens(1, 50, 55)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    slack = 1e-3 if dtype == torch.float32 else 0.2
    for s in seqs:
        assert len(s.output_ids) == 12
        logits = plain.forward(cfg, W, s.all_ids[:-1])
        for k, tok in enumerate(s.output_ids):
            row = logits[len(s.prompt_ids) - 1 + k]
            assert row[tok] >= row.max() - slack * float(row.std()), (s.request_id, k)
    assert eng.kv.num_free_blocks == 40 and eng.kv_cache.slots.num_free == 3
    eng.close()


def test_generation_with_preemption(tmp_path):
    # too few pages for all requests: the newest is preempted, loses its pages and state slot, and is
    # recomputed; greedy outputs stay those of an engine with room for all
    from llmctl.serve.scheduler import SamplingParams

    cfg = U.config(FULL, share=SHARE)
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), U.random_weights(cfg, 60))
    prompts = [tokens(6, 50, 61 + i) for i in range(4)]
    p = SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True)
    tight = U.engine(path, "cpu", blocks=10, block_size=4, max_seqs=4).generate(prompts, p)
    roomy = U.engine(path, "cpu", blocks=64, block_size=4, max_seqs=1).generate(prompts, p)
    assert sum(s.preemptions for s in tight) > 0
    assert [s.output_ids for s in tight] == [s.output_ids for s in roomy]


def test_checkpoint_names_round_trip(tmp_path):
    from llmctl.models import get_model_config
    from llmctl.models.malinex import MalinexConfig, MalinexLM, load_malinex

    cfg = U.config(FULL, share=SHARE)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 70).items()}
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W)
    m = load_malinex(tmp_path / "ck", MalinexConfig.from_file(tmp_path / "ck" / "config.json"), dtype=torch.float32)
    assert len(m.blocks) == 4 and len(m.cache_kinds()) == 6  # four weight sets, six cache entries
    back = m.export_named()
    assert set(back) == set(W)
    for k in W:
        assert torch.equal(back[k].float(), W[k]), k
    c = MalinexConfig.from_dict(U.clean(cfg))
    assert MalinexConfig.from_dict(c.to_dict()).to_dict() == c.to_dict()
    t = get_model_config("malinex-w64-l6-h4-g2-e4")
    assert t.architecture == "Malinex" and t.layers == 6 and t.is_moe
    assert sum(p.numel() for p in MalinexLM(t, dtype=torch.float32).parameters()) == t.num_parameters()
    bad = U.clean(U.config([(U.gla(), None)] * 3, share={1: 0}))
    bad["layers"][2] = dict(bad["layers"][1], weights_of=1)  # names a layer that has no weights of its own
    with pytest.raises(ValueError):
        MalinexConfig.from_dict(bad)
    assert path


def test_trace_replay_command(tmp_path):
    # the replay command end to end on a written checkpoint: two requests, a shared step, logits files
    import json
    import subprocess
    import sys

    import numpy as np

    cfg = U.config(FULL, share=SHARE)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 80).items()}
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W)
    a, b = tokens(10, 50, 81), tokens(5, 50, 82)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:7], "want": []}, {"id": "b", "tokens": b[:4], "want": [3]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[4:], "want": [0]}, {"id": "a", "tokens": a[7:], "want": [2]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, "-m", "llmctl.serve.trace_replay", "--model", path, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "64", "--device", "cpu", "--block-size", "4"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = plain.forward(cfg, W, a), plain.forward(cfg, W, b)
    want = {0: la[[0, 5]], 1: lb[[3]], 2: torch.stack([lb[4], la[9]])}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, 50))
        assert U.rel_err(got, w.float()) < 2e-4
