"""Pamazen through the serving engine against the plain whole-sequence implementation in
``tests/oracles/pamazen_plain.py``: every mechanism alone, whole prompts against token-by-token decoding,
portions down to two tokens, unequal batches, reused pages and state slots, far keys and the edges of pages,
key tiles, windows and kept first tokens, the first tokens of a sequence, long decoding, other sizes, and greedy
generation through the scheduler.

Each test runs on the CPU path and, marked ``gpu``, on the HIP kernels: fp32 with a tight bound at every
position; bf16 with loose bounds on the median and on nine positions in ten and a sanity bound on the rest.  Multi-layer
schedules in bf16 use routers that choose every expert (an expert near-tie that flips under bf16 rounding
changes all later positions through the memory); routed choice in bf16 is covered by the one-layer tests."""

import math
import random

import pytest
import torch

from tests.models import pamazen_util as U
from tests.oracles import pamazen_plain as plain

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
          bf16_all=False):
    device, dtype, tol = dev
    if bf16_tol is not None and dtype == torch.bfloat16:
        tol = bf16_tol
    if bf16_all and dtype == torch.bfloat16:
        cfg = U.without_choice(cfg)
    W = {k: v.bfloat16().float() for k, v in (W if W is not None else U.random_weights(cfg, seed)).items()}
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W), device, dtype, blocks, block_size, max_seqs)
    free0 = eng.kv.num_free_blocks
    got = U.run_schedule(eng, requests, steps)
    assert eng.kv.num_free_blocks == free0 and (eng.kv_cache.slots is None or eng.kv_cache.slots.num_free == max_seqs)
    errs = {rid: U.rel_errs(got[rid], plain.forward(cfg, W, toks)[0].float()) for rid, toks in requests.items()}
    if dtype == torch.bfloat16:
        per = torch.cat(list(errs.values()))
        assert float(per.median()) < tol / 2 and float(per.quantile(0.9)) < 2 * tol and float(per.max()) < 1.0, per
    else:
        for rid, per in errs.items():
            assert float(per.max()) < tol, f"{rid}: {per.max()} at {int(per.argmax())}"
    eng.close()


def whole(requests):
    return [[(rid, len(t))] for rid, t in requests.items()]


def left_only(**kw):
    return U.par(ls=1.0, rs=0.0, **kw)


def right_only(**kw):
    return U.par(ls=0.0, rs=1.0, **kw)


FULL = [(U.att(), U.moe()), (U.par(), U.moe(experts=4, top=1, identity=0, groups=1, shared=0)),
        (U.att(heads=2, kv_heads=2, dim=10, vdim=6, rot_dims=10, factor=None), None),
        (U.att(heads=3, kv_heads=3, dim=4, vdim=4, v_mix=False, rot_dims=2), U.moe(experts=5, top=3, identity=1, groups=3, keep=2, ff=6)),
        (U.par(heads=2, kv_heads=2, dim=8, window=20, keep=0, cap=0.0, rheads=1, rdim=7, rank=2), None), (U.att(), U.moe())]


# ------------------------------------------------------------------ each mechanism alone
def test_rotary_attention_alone(tmp_path, dev):
    cfg = U.config([(U.att(), None)], streams=0, mult=1.0, cap=0.0)
    r = {"a": tokens(23, 50, 1)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("sizes", [dict(heads=3, kv_heads=3, dim=10, vdim=4, rot_dims=10), dict(heads=6, kv_heads=1, dim=4, vdim=8, rot_dims=2, factor=None),
                                   dict(heads=1, kv_heads=1, dim=2, vdim=1, rot_dims=2, factor=4.0), dict(heads=4, kv_heads=2, dim=8, vdim=16, scale=0.9, rot_dims=0),
                                   dict(heads=2, kv_heads=2, dim=7, vdim=5, rot_dims=6, base=7.0)])
def test_rotary_attention_sizes(tmp_path, dev, sizes):
    # as many kv heads as heads, one kv head, one head, rotary on all / part / none of the head, no frequency scaling,
    # a scale that is not dim^-1/2, key and value sizes that differ, an odd head size
    cfg = U.config([(U.att(**sizes), None)], streams=2)
    r = {"a": tokens(26, 50, 2)}
    check(tmp_path, dev, cfg, r, [[("a", 9)], [("a", 1)], [("a", 16)]])


def test_denominator_holds_one_more_unit(tmp_path, dev):
    # tiny scores: every weight is close to 1 / (visible keys + 1), so the first positions lose half or a third of
    # their value mass; a plain softmax, or a sink per key head, shows at once
    cfg = U.config([(U.att(scale=1e-3), None)], streams=0)
    r = {"a": tokens(6, 50, 3)}
    check(tmp_path, dev, cfg, r, [[("a", 2)], [("a", 1)], [("a", 3)]])


def test_values_mix_with_the_first_mixing_layer(tmp_path, dev):
    # four attention layers; the second does not mix; the others' factors differ widely (0, 1.5, -0.5): values taken
    # from the previous layer, from a layer that does not take part, or a forgotten first-layer exemption show
    cfg = U.config([(U.att(), None), (U.att(v_mix=False), None), (U.att(), None), (U.att(), None)], streams=2)
    W = U.random_weights(cfg, 4)
    W["l0.mix.vmix"], W["l1.mix.vmix"] = torch.tensor(0.9), torch.tensor(0.8)  # both unused
    W["l2.mix.vmix"], W["l3.mix.vmix"] = torch.tensor(1.5), torch.tensor(-0.5)
    r = {"a": tokens(21, 50, 4), "b": tokens(5, 50, 5)}
    check(tmp_path, dev, cfg, r, [[("a", 12), ("b", 3)], [("a", 1), ("b", 1)], [("a", 8), ("b", 1)]], W=W)


def test_windowed_attention_alone(tmp_path, dev):
    cfg = U.config([(left_only(), None)])
    r = {"a": tokens(31, 50, 6)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("sizes", [dict(heads=3, kv_heads=3, dim=10, window=1, keep=0), dict(heads=6, kv_heads=1, dim=4, window=3, keep=5, cap=0.0),
                                   dict(heads=1, kv_heads=1, dim=1, window=4, keep=1), dict(heads=4, kv_heads=2, dim=16, window=100, keep=3, cap=0.7, scale=0.9),
                                   dict(heads=2, kv_heads=1, dim=9, window=6, keep=40, cap=50.0)])
def test_windowed_attention_sizes(tmp_path, dev, sizes):
    # a window of one key, more kept tokens than the window is long, no cap, a cap that bites everywhere, a window and a
    # kept range longer than the sequence, one channel per head
    cfg = U.config([(left_only(**sizes), None)], streams=2)
    r = {"a": tokens(29, 50, 7)}
    check(tmp_path, dev, cfg, r, [[("a", 11)], [("a", 1)], [("a", 1)], [("a", 16)]], bf16_tol=0.5 if sizes["dim"] == 1 else None)


def test_sinks_differ_between_heads(tmp_path, dev):
    # one head's sink swallows nearly everything, another's is negligible
    cfg = U.config([(left_only(heads=4, kv_heads=2, window=9), None)])
    W = U.random_weights(cfg, 8)
    W["l0.mix.left.sink"] = torch.tensor([6.0, -8.0, 0.0, 2.5])
    r = {"a": tokens(20, 50, 8)}
    check(tmp_path, dev, cfg, r, [[("a", 13)]] + [[("a", 1)]] * 7, W=W)


def test_delta_rule_alone(tmp_path, dev):
    cfg = U.config([(right_only(), None)])
    r = {"a": tokens(27, 50, 9)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("sizes", [dict(rheads=1, rdim=1, rank=1), dict(rheads=2, rdim=20, rank=3), dict(rheads=1, rdim=70, rank=2), dict(rheads=5, rdim=17, rank=7)])
def test_delta_rule_sizes(tmp_path, dev, sizes):
    # one channel; more channels than a wave has lanes; odd sizes; ranks of the decay projection
    cfg = U.config([(right_only(**sizes), None)], streams=1)
    r = {"a": tokens(19, 50, 10)}
    check(tmp_path, dev, cfg, r, [[("a", 7)], [("a", 1)], [("a", 11)]], bf16_tol=0.5 if sizes["rdim"] == 1 else None)


def test_removal_and_decay_take_effect(tmp_path, dev):
    # half of the channels remove all of the old memory along the key (a ~ 1) and decay fast, the others remove nothing
    # (a ~ 0) and barely decay: a removal applied after the write, read from the new memory, or mixed up with the decay shows
    cfg = U.config([(right_only(rheads=2, rdim=6), None)])
    W = U.random_weights(cfg, 11)
    b = torch.full((12,), 9.0)
    b[::2] = -9.0
    W["l0.mix.right.a.b"] = b
    W["l0.mix.right.w0"] = -b
    r = {"a": tokens(40, 50, 11)}
    check(tmp_path, dev, cfg, r, [[("a", 13)], [("a", 27)]], W=W)


def test_both_mixers_side_by_side(tmp_path, dev):
    cfg = U.config([(U.par(ls=-0.4, rs=2.0), None)])
    r = {"a": tokens(25, 50, 12)}
    check(tmp_path, dev, cfg, r, [[("a", 10)], [("a", 1)], [("a", 14)]])


@pytest.mark.parametrize("f", [dict(experts=5, top=1, ff=7, shared=9, identity=0, groups=1), dict(experts=4, top=4, ff=6, shared=0, identity=0, groups=2, keep=2),
                               dict(experts=6, top=3, ff=5, shared=4, identity=3, groups=3, keep=1), dict(experts=2, top=2, ff=8, shared=3, identity=6, groups=4, keep=2),
                               dict(experts=7, top=2, ff=5, shared=0, identity=1, groups=1)])
def test_routed_feed_forward(tmp_path, dev, f):
    # no groups, groups that all stay, identity experts that fill whole groups, one expert per token, no shared expert
    cfg = U.config([(U.att(heads=1, kv_heads=1), U.moe(**f))], streams=2)
    r = {"a": tokens(40, 50, 13), "b": tokens(3, 50, 14)}
    check(tmp_path, dev, cfg, r, [[("a", 40), ("b", 2)], [("b", 1)]], bf16_tol=0.3)


def test_correction_decides_the_choice_not_the_weights(tmp_path, dev):
    # a large correction on two experts of one group and a negative one elsewhere: those two are always chosen (also
    # where all choice scores of a kept group are negative), yet their weights are their small scores
    f = U.moe(experts=6, top=2, identity=2, groups=2, keep=1)
    cfg = U.config([(U.att(heads=1, kv_heads=1), f)])
    W = U.random_weights(cfg, 15)
    W["l0.mlp.correction"] = torch.tensor([-3.0, -3.0, -3.0, -3.0, -6.0, -6.5, -1.0, -1.5])
    r = {"a": tokens(30, 50, 15)}
    check(tmp_path, dev, cfg, r, whole(r), W=W)
    picks = plain.route(torch.randn(9, 20, dtype=torch.float64), {k: v.double() for k, v in W.items()}, "l0.mlp.", f["router"])
    assert all(sorted(ids) == [6, 7] for ids, _ in picks)  # two identity experts of the second group


@pytest.mark.parametrize("streams", [0, 1, 2, 5, 8])
def test_hyper_connections(tmp_path, dev, streams):
    # no stream tensors at all (the plain residual sum), one stream with its own coefficients, several
    cfg = U.config([(U.att(), U.moe()), (U.par(), None)], streams=streams, mult=0.8)
    r = {"a": tokens(17, 50, 16)}
    check(tmp_path, dev, cfg, r, [[("a", 8)], [("a", 1)], [("a", 8)]], bf16_all=True)


def test_stream_after_every_layer(tmp_path):
    cfg = U.config(FULL)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 17).items()}
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W), "cpu")
    toks = tokens(15, 50, 17)
    seq = eng.open_sequence(toks)
    from llmctl.serve.scheduler import PrefillChunk

    trail = []
    eng.forward_portions([PrefillChunk(seq, 0, len(toks))], [[0]], trail=trail)
    want = plain.forward(cfg, W, toks)[1]
    assert len(trail) == len(want) == len(FULL)
    for a, b in zip(trail, want):
        assert float((a.double() - b).abs().max()) < 1e-3 * float(b.abs().max())


def test_no_layers_and_no_caps(tmp_path, dev):
    cfg = U.config([], cap=0.0)
    r = {"a": tokens(5, 50, 18)}
    check(tmp_path, dev, cfg, r, whole(r))
    cfg = U.config([(U.att(), None)], cap=0.5)  # a logit cap that bites
    check(tmp_path / "b", dev, cfg, r, whole(r))


# ------------------------------------------------------------------ schedules
def test_prefill_against_token_by_token(tmp_path, dev):
    cfg = U.config(FULL)
    r = {"a": tokens(26, 50, 20)}
    check(tmp_path, dev, cfg, r, [[("a", 1)]] * 26, bf16_all=True)


def test_portions_of_several_sizes(tmp_path, dev):
    cfg = U.config(FULL)
    r = {"a": tokens(61, 50, 21)}
    check(tmp_path, dev, cfg, r, [[("a", n)] for n in (2, 17, 3, 2, 30, 1, 1, 5)], bf16_all=True)


def test_unequal_batches(tmp_path, dev):
    cfg = U.config(FULL)
    r = {"a": tokens(40, 50, 22), "b": tokens(7, 50, 23), "c": tokens(19, 50, 24), "d": tokens(2, 50, 25)}
    steps = [[("a", 11), ("b", 2)], [("a", 1), ("b", 4), ("c", 9)], [("c", 1), ("a", 20), ("b", 1), ("d", 2)], [("a", 8), ("c", 9)]]
    check(tmp_path, dev, cfg, r, steps, bf16_all=True)


def test_pages_and_slots_used_again(tmp_path, dev):
    # 12 pages of 4 tokens and 2 state slots for five requests: every later request runs in pages and a slot that hold
    # an earlier one's rows and memory
    cfg = U.config(FULL)
    r = {k: tokens(n, 50, 30 + i) for i, (k, n) in enumerate([("a", 22), ("b", 18), ("c", 20), ("d", 9), ("e", 23)])}
    steps = [[("a", 10), ("b", 18)], [("a", 12), ("c", 3)], [("c", 17), ("d", 1)], [("d", 1)], [("d", 7), ("e", 2)], [("e", 21)]]
    check(tmp_path, dev, cfg, r, steps, blocks=12, max_seqs=2, bf16_all=True)


def test_token_by_token_start_in_a_used_slot(tmp_path, dev):
    cfg = U.config([(U.par(), None), (U.att(), None)])
    r = {"a": tokens(30, 50, 36), "b": tokens(12, 50, 37)}
    check(tmp_path, dev, cfg, r, [[("a", 30)]] + [[("b", 1)]] * 12, blocks=10, max_seqs=1)


def test_long_decoding_over_window_and_tile_borders(tmp_path, dev):
    # 150 decoded tokens after a short prompt: the window (37) and the kept tokens pass over decoded tokens, contexts
    # cross 64-key tiles and many pages
    cfg = U.config([(U.par(window=37, keep=3, heads=2, kv_heads=1, dim=8), None), (U.att(), U.moe())], streams=2)
    r = {"a": tokens(156, 50, 38)}
    check(tmp_path, dev, cfg, r, [[("a", 6)]] + [[("a", 1)]] * 150, blocks=48, bf16_all=True)


def test_long_portions(tmp_path, dev):
    # 650-token portions (chunk-parallel scan, several query blocks) continued in a second and a third step
    cfg = U.config([(U.par(window=70, keep=5, rheads=2, rdim=6), None), (U.att(), None)], streams=2)
    r = {"a": tokens(700, 50, 39), "b": tokens(300, 50, 40)}
    check(tmp_path, dev, cfg, r, [[("a", 650), ("b", 10)], [("a", 49), ("b", 290)], [("a", 1)]], blocks=260)


def test_heads_that_fit_the_matrix_cores(tmp_path, dev):
    # head sizes in multiples of 8 (the bf16 runs take the matrix-core attention form), a prompt over several 64-key
    # tiles, a window of 70 keys with 3 kept ones, then decoding, beside a short request
    cfg = U.config([(U.att(heads=4, kv_heads=2, dim=32, vdim=16, rot_dims=16), None),
                    (U.par(heads=4, kv_heads=1, dim=24, window=70, keep=3, rheads=2, rdim=16), None),
                    (U.att(heads=4, kv_heads=2, dim=32, vdim=16, rot_dims=32, factor=None), None)], width=64, streams=4)
    r = {"a": tokens(230, 50, 41), "b": tokens(9, 50, 42)}
    check(tmp_path, dev, cfg, r, [[("a", 200), ("b", 4)]] + [[("a", 1), ("b", 1)]] * 5 + [[("a", 25)]], blocks=80)


# ------------------------------------------------------------------ far keys and edges, at op level
def _window_case(device, dtype, bs, L, j0, form, mfma, window, keep, cap=4.0, H=4, G=2, dk=16):
    """One key (position j0) stands out for the last queries; they see it if it lies in their window or among the kept
    first tokens.  Values are the keys' own sub-rows [v | k].  Returns (got, want) for the last ``n`` positions."""
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(1000 * L + j0)
    q = torch.randn(L, H, dk, generator=g) * 0.3
    k = torch.randn(L, G, dk, generator=g) * 0.3
    v = torch.randn(L, G, dk, generator=g)
    v[j0] += 9.0
    dirn = torch.randn(dk, generator=g)
    dirn /= dirn.norm()
    k[j0] = dirn * 4.0
    n = min(L, 70)
    q[L - n:] += dirn * 3.0
    sink = torch.randn(H, generator=g)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    scale = 1.1
    rep = H // G
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(rep, 1)) * scale
    if cap:
        s = cap * torch.tanh(s / cap)
    i = torch.arange(L)
    d = i[:, None] - i[None, :]
    vis = ((d >= 0) & ((d < window) | (i[None, :] < keep)))[None]
    want = torch.einsum("hij,jhd->ihd", plain.softmax_with_extra(s, vis, sink.double()), v.double().repeat_interleave(rep, 1))
    dev_ = torch.device(device)
    nb = (L + bs - 1) // bs
    perm = torch.randperm(nb + 3, generator=g)[:nb]  # pages lie anywhere in the pool
    cache = torch.zeros(nb + 3, bs, G * 2 * dk, dtype=dtype)
    rows = torch.cat([v, k], -1).reshape(L, G * 2 * dk)
    for p in range(L):
        cache[perm[p // bs], p % bs] = rows[p]
    cache, bt = cache.to(dev_), perm.to(torch.int32).view(1, nb).to(dev_)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev_)
    kw = dict(groups=G, koff=dk, softcap=cap, keep_first=keep)
    if form == "prefill":
        got = hybrid.latent_attention_prefill(q[L - n:].contiguous().to(dev_), cache, bt, i32([0, n]), i32([L]), window, sink.to(dev_), scale, dk, n,
                                              mfma=mfma, **kw)
        want = want[L - n:]
    else:
        m = min(n, 8)
        got = torch.cat([hybrid.latent_attention_decode(q[p:p + 1].contiguous().to(dev_), cache, bt, i32([p + 1]), window, sink.to(dev_), scale, dk,
                                                        mfma=mfma, max_ctx=p + 1, **kw) for p in range(L - m, L)])
        want = want[L - m:]
    return got.double().cpu(), want


@pytest.mark.parametrize("form", ["prefill", "decode"])
@pytest.mark.parametrize("bs,L,j0,window,keep", [(4, 60, 51, 9, 0), (4, 60, 52, 9, 0), (8, 200, 2, 30, 3), (8, 200, 3, 30, 3), (16, 200, 63, 137, 2),
                                                 (16, 200, 64, 137, 2), (16, 420, 0, 50, 1), (16, 420, 5, 50, 6), (16, 420, 6, 50, 6), (16, 700, 66, 100, 70),
                                                 (16, 700, 599, 100, 70), (16, 700, 600, 100, 70), (16, 700, 150, 1 << 30, 0), (16, 330, 127, 203, 128),
                                                 (16, 330, 128, 203, 128)])
def test_far_keys_window_edges_and_kept_tokens(dev, form, bs, L, j0, window, keep):
    # the standing-out key lies far back, among the kept first tokens or just past them, just inside or just outside the
    # last queries' windows, on either side of page and 64-key-tile borders
    device, dtype, _ = dev
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for mfma in ([True, False] if (device == "cuda" and dtype == torch.bfloat16) else [True]):
        got, want = _window_case(device, dtype, bs, L, j0, form, mfma, window, keep)
        err = float((got - want).abs().max()) / max(1.0, float(want.abs().max()))  # (the standing-out value is ~9)
        assert err < tol, (mfma, err)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk", [(8, 4, 56), (4, 4, 64), (6, 1, 128), (3, 3, 24), (12, 4, 64), (2, 1, 160), (16, 16, 8), (5, 5, 20)])
def test_capped_windowed_attention_kernels_gpu(H, G, dk):
    # the matrix-core and the generic kernels on other head counts and sizes, prompt and decode forms
    for dtype, tol in ((torch.bfloat16, 4e-2), (torch.float32, 1e-4)):
        for form in ("prefill", "decode"):
            for mfma in (True, False):
                got, want = _window_case("cuda", dtype, 16, 300, 2, form, mfma, 90, 4, H=H, G=G, dk=dk)
                assert float((got - want).abs().max()) / max(1.0, float(want.abs().max())) < tol, (dtype, form, mfma)


def _memory_case(device, dtype, T, dk, dv, H, cuts, far, chunked):
    """One key channel per head neither decays nor is removed and holds what token ``far`` wrote; the other channels
    forget within a few tokens.  The last tokens ask for that channel.  Runs the op over the portions ``cuts`` with
    the memory carried in a two-slot pool whose slots hold another sequence's junk."""
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(7)
    r, k = torch.randn(T, H, dk, generator=g) * 0.3, torch.randn(T, H, dk, generator=g) * 0.5
    v = torch.randn(T, H, dv, generator=g)
    zw, za = torch.randn(T, H * dk, generator=g) + 2.0, torch.randn(T, H * dk, generator=g)
    w0, ab = torch.randn(H * dk, generator=g) * 0.2, torch.randn(H * dk, generator=g) * 0.2
    keep = [(3 * h) % dk for h in range(H)]
    for h, c in enumerate(keep):
        zw[:, h * dk + c] = -30.0  # decay ~ 1
        za[:, h * dk + c] = -30.0  # nothing removed
        k[:, h, c] = 0.0
        k[far, h, c] = 6.0
        r[T - 3:, h, c] = 5.0
    coef, keps = math.exp(-0.5), 1e-6
    r, k, v, za = r.to(dtype), k.to(dtype), v.to(dtype), za.to(dtype)
    w = torch.exp(-coef * torch.sigmoid(zw.double() + w0.double())).view(T, H, dk)
    a = torch.sigmoid(za.double() + ab.double()).view(T, H, dk)
    kd = k.double()
    u = kd / torch.sqrt((kd * kd).sum(-1, keepdim=True) + keps)
    Sd = torch.zeros(H, dk, dv, dtype=torch.float64)
    want = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        uS = torch.einsum("hk,hkv->hv", u[t], Sd)
        Sd = w[t][:, :, None] * Sd - (a[t] * u[t])[:, :, None] * uS[:, None, :] + kd[t][:, :, None] * v[t].double()[:, None, :]
        want[t] = torch.einsum("hkv,hk->hv", Sd, r[t].double())
    d = torch.device(device)
    S = torch.randn(2, H, dk, dv, generator=g).to(d)  # junk of an earlier owner
    outs, at = [], 0
    for n in cuts:
        cu = [0, n]
        o = hybrid.delta_scan(r[at:at + n].to(d), k[at:at + n].to(d), v[at:at + n].to(d), zw[at:at + n].to(d), w0.to(d), za[at:at + n].to(d),
                              ab.to(d), coef, keps, S, torch.tensor([1], dtype=torch.int32).to(d), torch.tensor(cu, dtype=torch.int32).to(d),
                              torch.tensor([at], dtype=torch.int32).to(d), cu_host=cu if chunked else None)
        outs.append(o.double().cpu())
        at += n
    assert at == T
    return torch.cat(outs), want, S[1].double().cpu(), Sd, keep


@pytest.mark.parametrize("T,cuts,far", [(40, [40], 2), (300, [300], 1), (300, [7, 1, 1, 290, 1], 5), (700, [257, 443], 3), (130, [64, 64, 2], 63)])
def test_memory_survives_and_forgets(dev, T, cuts, far):
    device, dtype, _ = dev
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    H, dk, dv = 3, 12, 20
    for chunked in ([False, True] if device == "cuda" else [False]):
        got, want, S, S_end, keep = _memory_case(device, dtype, T, dk, dv, H, cuts, far, chunked)
        scale = float(want.abs().max())
        assert float((got - want).abs().max()) / scale < tol, chunked
        assert float((S - S_end).abs().max()) / float(S_end.abs().max()) < tol, chunked
        # the kept channel still holds token ``far``'s value after T tokens; the last outputs are made of it
        assert float(want[T - 1].abs().max()) > 5.0 * float(want[T - 20].abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dk,dv", [(3, 5), (16, 64), (20, 100), (44, 72), (64, 128), (64, 64), (70, 33), (128, 64), (130, 70), (200, 40), (256, 16)])
def test_delta_scan_kernel_tiers_gpu(dk, dv):
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


@pytest.mark.parametrize("W,S", [(7, 1), (200, 4), (1000, 3), (2500, 2), (64, 8)])
def test_stream_pass(W, S):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(W)
    for device, dtype in _devices_dtypes():
        for ydt in {torch.float32, dtype}:
            X = torch.randn(5, S, W, generator=g)
            y1, y2 = torch.randn(5, W + 3, generator=g).to(ydt), torch.randn(5, 2 * W, generator=g).to(ydt)
            mix, co, ci = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
            gw = torch.tensor([1.3])
            y = 0.6 * y1[:, 3:].double() - 1.7 * y2[:, W:].double()
            X2 = torch.einsum("st,nsw->ntw", mix.double(), X.double()) + 0.3 * co.double()[None, :, None] * y[:, None, :]
            h_want = plain.rms_unit(torch.einsum("t,ntw->nw", ci.double(), X2), 1e-5) * 1.3
            Xd = X.clone().to(device)
            h = hybrid.hc_update_norm_(Xd, y1.to(device)[:, 3:], 0.6, y2.to(device)[:, W:], -1.7, mix.to(device), co.to(device), 0.3,
                                       ci.to(device), gw.to(device), 1e-5, dtype)
            assert h.dtype == dtype
            assert float((Xd.double().cpu() - X2).abs().max()) < 1e-4
            assert float((h.double().cpu() - h_want).abs().max()) < (1e-4 if dtype == torch.float32 else 5e-2)
            Xd = X.clone().to(device)
            assert hybrid.hc_update_norm_(Xd, y1.to(device)[:, 3:], 0.6, y2.to(device)[:, W:], -1.7, mix.to(device), co.to(device), 0.3,
                                          None, None, 1e-5, dtype) is None
            assert float((Xd.double().cpu() - X2).abs().max()) < 1e-4
        table = torch.randn(11, W, generator=g).to(dtype)
        ids = torch.tensor([3, 0, 10, 3])
        ci = torch.randn(S, generator=g)
        X, h = hybrid.hc_embed_norm(ids.to(device), table.to(device), S, ci.to(device), torch.tensor([0.7]).to(device), 1e-5, dtype)
        e = table.double()[ids]
        assert X.shape == (4, S, W) and float((X.double().cpu() - e[:, None, :]).abs().max()) == 0.0
        assert float((h.double().cpu() - plain.rms_unit(e * ci.double().sum(), 1e-5) * 0.7).abs().max()) < (1e-4 if dtype == torch.float32 else 5e-2)


@pytest.mark.parametrize("E,top,groups,keep", [(4, 1, 1, 1), (6, 2, 3, 2), (16, 4, 2, 1), (12, 5, 4, 3), (70, 8, 7, 2), (8, 2, 8, 3)])
def test_grouped_softmax_router(E, top, groups, keep):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(E)
    z, b = torch.randn(37, E, generator=g) * 2.0, torch.randn(E, generator=g) * 0.3 - 0.2
    Wd = {"r.router": torch.eye(E, dtype=torch.float64), "r.correction": b.double()}
    picks = plain.route(z.double(), Wd, "r.", {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}})
    want = torch.zeros(37, E, dtype=torch.float64)
    for t, (ids, ws) in enumerate(picks):
        want[t, ids] = torch.tensor(ws, dtype=torch.float64)
    for device, _ in _devices_dtypes():
        gi, gw = hybrid.bias_topk_router(z.to(device), b.to(device), top, groups, keep, False)
        dense = torch.zeros(37, E, dtype=torch.float64).scatter_(1, gi.cpu(), gw.double().cpu())
        assert torch.equal(dense > 0, want > 0)
        assert float((dense - want).abs().max()) < 1e-5


@pytest.mark.parametrize("H,G,dk,dv,rot", [(4, 2, 8, 6, 4), (8, 4, 64, 64, 32), (3, 1, 5, 7, 4), (2, 2, 160, 16, 0), (4, 2, 80, 40, 80)])
def test_query_key_value_preparation(H, G, dk, dv, rot):
    # no norms, rotary on neighbour pairs of the first entries with scaled frequencies, the value mix, cache rows
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(H * dk)
    bs = 4
    for device, dtype in _devices_dtypes():
        for T in (11, 300):
            z = torch.randn(T, (H + G) * dk + G * dv + 5, generator=g).to(dtype)
            vf = torch.randn(T, G * dv + 2, generator=g).to(dtype)[:, 2:]
            lam = torch.tensor([0.35])
            pos = torch.randint(0, 3000, (T,), generator=g).to(torch.int32)
            slots = torch.randperm(T + 2 * bs, generator=g)[:T]
            freq = torch.tensor([50.0 ** (-2.0 * i / max(rot, 1)) / 3.0 for i in range(rot // 2)], dtype=torch.float32)
            zd = z.double()

            def turn(x):
                return plain.rotate_pairs_at(x, pos.double(), 50.0, rot, 3.0) if rot else x

            q_want = turn(zd[:, :H * dk].view(T, H, dk))
            k_want = turn(zd[:, H * dk:(H + G) * dk].view(T, G, dk))
            v_want = 0.65 * zd[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv) + 0.35 * vf.double().view(T, G, dv)
            cache = torch.zeros((T + 2 * bs + bs - 1) // bs, bs, G * (dv + dk), dtype=dtype, device=device)
            q = hybrid.attn_qkv_prep(z.to(device), H, G, dk, dv, None, None, 1e-5, pos.to(device), freq.to(device), rot, True, 1.0, None, cache,
                                     slots.to(device), v_first=vf.to(device), v_lambda=lam.to(device))
            tol = 2e-3 if dtype == torch.float32 else 3e-2  # fp32: angles of positions in the thousands
            rows = cache.view(-1, G, dv + dk)[slots.to(device)].double().cpu()
            assert float((q.double().cpu() - q_want).abs().max()) < tol * float(q_want.abs().max())
            assert float((rows[:, :, dv:] - k_want).abs().max()) < tol * float(k_want.abs().max())
            assert float((rows[:, :, :dv] - v_want).abs().max()) < tol * 4


@pytest.mark.parametrize("H,G,dk", [(4, 2, 8), (6, 3, 64), (3, 1, 5)])
def test_values_that_are_the_keys(H, G, dk):
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(H + dk)
    bs = 4
    for device, dtype in _devices_dtypes():
        for T in (9, 280):
            z = torch.randn(T, (H + G) * dk + 6, generator=g).to(dtype)
            wq, wk = torch.randn(dk, generator=g), torch.randn(dk, generator=g)
            pos = torch.arange(T, dtype=torch.int32)
            slots = torch.randperm(T + bs, generator=g)[:T]
            zd = z.double()
            kraw = zd[:, H * dk:(H + G) * dk].view(T, G, dk)
            cache = torch.zeros((T + 2 * bs - 1) // bs, bs, G * 2 * dk, dtype=dtype, device=device)
            q = hybrid.attn_qkv_prep(z.to(device), H, G, dk, dk, wq.to(device), wk.to(device), 1e-5, pos.to(device),
                                     torch.zeros(0, device=device), 0, True, 1.0, None, cache, slots.to(device), v_from_k=True)
            tol = 1e-5 if dtype == torch.float32 else 3e-2
            rows = cache.view(-1, G, 2 * dk)[slots.to(device)].double().cpu()
            assert float((q.double().cpu() - plain.rms_unit(zd[:, :H * dk].view(T, H, dk), 1e-5) * wq.double()).abs().max()) < tol * 4
            assert float((rows[:, :, dk:] - plain.rms_unit(kraw, 1e-5) * wk.double()).abs().max()) < tol * 4
            assert float((rows[:, :, :dk] - kraw).abs().max()) < tol * 4


# ------------------------------------------------------------------ the framework's own entry points
def test_greedy_generation_through_the_scheduler(tmp_path, dev):
    from llmctl.serve.scheduler import SamplingParams

    device, dtype, _ = dev
    cfg = U.config(FULL)
    if dtype == torch.bfloat16:
        cfg = U.without_choice(cfg)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 50).items()}
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W)
    eng = U.engine(path, device, dtype, blocks=40, block_size=4, max_seqs=3, scheduler="dynamic")
    prompts = [tokens(9, 50, 51), tokens(2, 50, 52), tokens(14, 50, 53), tokens(5, 50, 54), tokens(1, 50, 55)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    slack = 1e-3 if dtype == torch.float32 else 0.2
    for s in seqs:
        assert len(s.output_ids) == 12
        logits = plain.forward(cfg, W, s.all_ids[:-1])[0]
        for k, tok in enumerate(s.output_ids):
            row = logits[len(s.prompt_ids) - 1 + k]
            assert row[tok] >= row.max() - slack * float(row.std()), (s.request_id, k)
    assert eng.kv.num_free_blocks == 40 and eng.kv_cache.slots.num_free == 3
    eng.close()


def test_generation_with_preemption(tmp_path):
    # too few pages for all requests: the newest is preempted, loses its pages and state slot, and is recomputed;
    # greedy outputs stay those of an engine with room for all
    from llmctl.serve.scheduler import SamplingParams

    cfg = U.config(FULL)
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), U.random_weights(cfg, 60))
    prompts = [tokens(6, 50, 61 + i) for i in range(4)]
    p = SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True)
    tight = U.engine(path, "cpu", blocks=10, block_size=4, max_seqs=4).generate(prompts, p)
    roomy = U.engine(path, "cpu", blocks=64, block_size=4, max_seqs=1).generate(prompts, p)
    assert sum(s.preemptions for s in tight) > 0
    assert [s.output_ids for s in tight] == [s.output_ids for s in roomy]


def test_checkpoint_names_round_trip(tmp_path):
    from llmctl.models import get_model_config
    from llmctl.models.pamazen import PamazenConfig, PamazenLM, load_pamazen

    cfg = U.config(FULL)
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 70).items()}
    path = U.write_checkpoint(tmp_path / "ck", U.clean(cfg), W)
    m = load_pamazen(tmp_path / "ck", PamazenConfig.from_file(tmp_path / "ck" / "config.json"), dtype=torch.float32)
    kinds = [k for k, _ in m.cache_kinds()]
    assert kinds == ["latent", "rows+state", "latent", "latent", "rows+state", "latent"]
    back = m.export_named()
    assert set(back) == set(W)
    for k in W:
        assert torch.equal(back[k].float(), W[k]), k
    c = PamazenConfig.from_dict(U.clean(cfg))
    assert PamazenConfig.from_dict(c.to_dict()).to_dict() == c.to_dict()
    t = get_model_config("pamazen-w64-l6-h4-g2-e4")
    assert t.architecture == "Pamazen" and t.layers == 6 and t.is_moe
    assert sum(p.numel() for p in PamazenLM(t, dtype=torch.float32).parameters()) == t.num_parameters()
    bad = U.clean(U.config([(U.att(vdim=6), None), (U.att(vdim=8), None)]))  # values of unlike sizes cannot be mixed
    with pytest.raises(ValueError):
        PamazenConfig.from_dict(bad)
    assert path


def test_trace_replay_command(tmp_path):
    # the replay command end to end on a written checkpoint: two requests, a shared step, logits files
    import json
    import subprocess
    import sys

    import numpy as np

    cfg = U.config(FULL)
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
    la, lb = plain.forward(cfg, W, a)[0], plain.forward(cfg, W, b)[0]
    want = {0: la[[0, 5]], 1: lb[[3]], 2: torch.stack([lb[4], la[9]])}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, 50))
        assert U.rel_err(got, w.float()) < 2e-4
