"""Dumalix through the serving engine against the plain whole-sequence implementation in
``tests/oracles/dumalix_plain.py``: every mechanism alone, whole prompts against token-by-token decoding,
portions down to two tokens, unequal batches, reused pages and state slots, chunk edges and far keys,
the first tokens of a sequence, long decoding, other sizes, and greedy generation through the scheduler.

Each test runs on the CPU path and, marked ``gpu``, on the HIP kernels (fp32 with a tight bound, bf16
with a loose one)."""

import math
import random

import pytest
import torch

from tests.models import dumalix_util as U
from tests.oracles import dumalix_plain as plain

DEVICES = [("cpu", torch.float32, 2e-4),
           pytest.param(("cuda", torch.float32, 2e-4), marks=pytest.mark.gpu),
           pytest.param(("cuda", torch.bfloat16, 0.12), marks=pytest.mark.gpu)]


@pytest.fixture(params=DEVICES, ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def dev(request):
    return request.param


def tokens(n, vocab, seed):
    r = random.Random(seed)
    return [r.randrange(vocab) for _ in range(n)]


def check(tmp_path, dev, cfg, requests, steps, seed=0, blocks=64, block_size=4, W=None, max_seqs=4, bf16_tol=None):
    device, dtype, tol = dev
    if bf16_tol is not None and dtype == torch.bfloat16:
        tol = bf16_tol
    W = {k: v.bfloat16().float() for k, v in (W if W is not None else U.random_weights(cfg, seed)).items()}
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", cfg, W), device, dtype, blocks, block_size, max_seqs)
    free0 = eng.kv.num_free_blocks
    got = U.run_schedule(eng, requests, steps)
    assert eng.kv.num_free_blocks == free0 and (eng.kv_cache.slots is None or eng.kv_cache.slots.num_free == max_seqs)
    for rid, toks in requests.items():
        want = plain.forward(cfg, W, toks)
        err = U.rel_err(got[rid], want.float())
        assert err < tol, f"{rid}: {err}"
    eng.close()


def whole(requests):
    return [[(rid, len(t))] for rid, t in requests.items()]


# ------------------------------------------------------------------ each mechanism alone
def test_attention_alone(tmp_path, dev):
    cfg = U.config([(U.att(), None)], taps=0)
    r = {"a": tokens(23, 50, 1)}
    check(tmp_path, dev, cfg, r, whole(r))


def test_attention_plain_causal_no_convolution_partial_rotary(tmp_path, dev):
    cfg = U.config([(U.att(heads=3, kv_heads=3, dim=10, vdim=4, conv=0, chunk=None, rot_dims=6, scaling=None), None)], taps=0)
    r = {"a": tokens(17, 50, 2)}
    check(tmp_path, dev, cfg, r, whole(r))


def test_attention_one_kv_head_chunk_of_one(tmp_path, dev):
    # a chunk of one position sees only the token itself and the sink
    cfg = U.config([(U.att(heads=2, kv_heads=1, dim=4, vdim=8, conv=2, chunk=1), None)], taps=0)
    r = {"a": tokens(9, 50, 3)}
    check(tmp_path, dev, cfg, r, whole(r))


def test_sink_and_temperature_take_effect(tmp_path, dev):
    # a large sink swallows most of the softmax mass and the heads' temperatures differ widely:
    # a sink that is left out, scaled or counted per key, or a temperature on the wrong head, shows
    cfg = U.config([(U.att(heads=4, kv_heads=2, chunk=9), None)], taps=0)
    W = U.random_weights(cfg, 4)
    W["l0.mix.sink"] = torch.tensor([5.0, -2.0, 3.0, 0.5])
    W["l0.mix.temp"] = torch.tensor([0.25, 4.0, 1.0, 2.5])
    r = {"a": tokens(21, 50, 4)}
    check(tmp_path, dev, cfg, r, whole(r), W=W)


def test_latent_attention_alone(tmp_path, dev):
    cfg = U.config([(U.lat(), None)], taps=0)
    r = {"a": tokens(25, 50, 5)}
    check(tmp_path, dev, cfg, r, whole(r))


def test_latent_attention_one_head_no_scaling(tmp_path, dev):
    cfg = U.config([(U.lat(heads=1, dim=3, rot_dim=2, vdim=7, kv_rank=5, scaling=None), None)], taps=0)
    r = {"a": tokens(12, 50, 6)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("sizes", [dict(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=40), dict(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=64),
                                   dict(heads=1, dim=2, rot_dim=2, vdim=2, kv_rank=9)])
def test_latent_attention_whole_prompts_on_expanded_keys(tmp_path, dev, sizes, monkeypatch):
    # whole prompts attend per-head keys and values expanded from the latents (a wide latent makes that the
    # cheaper product); the second request runs in portions, which attend the cached rows, in the same steps
    from llmctl.models.mixers import LatentAttention

    monkeypatch.setattr(LatentAttention, "EXPAND_MIN_TOKENS", 1)
    cfg = U.config([(U.lat(**sizes), U.ff()), (U.lat(**sizes), None)], taps=2)
    r = {"a": tokens(70, 50, 40), "b": tokens(33, 50, 41), "c": tokens(21, 50, 42)}
    check(tmp_path, dev, cfg, r, [[("a", 70), ("b", 20)], [("b", 13)], [("c", 21)]], blocks=40)


def test_feed_forward_alone(tmp_path, dev):
    # the mixer sees one position only, so the clamped feed-forward carries the test; the limit is low
    # enough that both clamps bite
    cfg = U.config([(U.att(heads=1, kv_heads=1, conv=0, chunk=1), U.ff(16, limit=0.6))], taps=0)
    r = {"a": tokens(30, 50, 7)}
    check(tmp_path, dev, cfg, r, whole(r))


@pytest.mark.parametrize("taps", [2, 4, 5])
def test_input_convolution(tmp_path, dev, taps):
    cfg = U.config([(U.lat(), U.ff())], taps=taps)
    r = {"a": tokens(14, 50, 8)}
    check(tmp_path, dev, cfg, r, [[("a", 3)], [("a", 1)], [("a", 2)], [("a", 8)]])


@pytest.mark.parametrize("loop", [(0, 1, 2), (1, 3, 3), (0, 3, 1), (2, 3, 2), (1, 1, 4)])
def test_loop(tmp_path, dev, loop):
    cfg = U.config([(U.lat(), U.ff()), (U.att(), U.ff()), (U.lat(heads=2), None)], loop=loop)
    r = {"a": tokens(13, 50, 9)}
    check(tmp_path, dev, cfg, r, [[("a", 9)], [("a", 1)], [("a", 1)], [("a", 2)]])


def test_stream_after_every_run(tmp_path, dev):
    device, dtype, tol = dev
    cfg = U.config([(U.lat(), U.ff()), (U.att(), U.ff())], loop=(0, 2, 2))
    W = U.random_weights(cfg, 10)
    eng = U.engine(U.write_checkpoint(tmp_path / "ck", cfg, W), device, dtype)
    from llmctl.serve.scheduler import PrefillChunk

    toks = tokens(11, 50, 10)
    seq = eng.open_sequence(toks)
    trail = []
    eng.forward_portions([PrefillChunk(seq, 0, len(toks))], [[0]], trail=trail)
    want = []
    plain.forward(cfg, W, toks, want)
    assert len(trail) == len(want) == 4
    for g, w in zip(trail, want):
        assert float((g.double().cpu() - w).abs().max() / w.abs().max()) < (1e-4 if dtype == torch.float32 else 4e-2)
    eng.close()


def test_yarn_frequencies():
    from llmctl.models.mixers import rotary_frequencies

    for base, dims, sc in [(20000.0, 24, {"factor": 6.0, "original": 4096, "fast": 16.0, "slow": 2.0}),
                           (50.0, 8, U.YARN), (500000.0, 64, {"factor": 2.0, "original": 100, "fast": 8.0, "slow": 2.0}),
                           (100.0, 6, None), (3.0, 4, {"factor": 5.0, "original": 4, "fast": 1.0, "slow": 1.0})]:
        f, amp = rotary_frequencies(base, dims, sc)
        wf, wamp = plain.yarn_frequencies(base, dims, sc)
        assert torch.allclose(f.double(), wf, rtol=1e-6, atol=0) and abs(amp - wamp) < 1e-12


# ------------------------------------------------------------------ the whole design, other sizes
FULL = [(U.lat(), U.ff()), (U.att(), U.ff(9, 2.0)), (U.lat(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=6), None),
        (U.att(heads=2, kv_heads=2, dim=6, vdim=10, conv=4, chunk=5, rot_dims=4), U.ff(7, 0.8))]


def test_all_layers_whole_prompts(tmp_path, dev):
    cfg = U.config(FULL, loop=(1, 3, 2))
    r = {"a": tokens(31, 50, 11), "b": tokens(1, 50, 12), "c": tokens(2, 50, 13)}
    check(tmp_path, dev, cfg, r, whole(r))


def test_layers_of_different_sizes(tmp_path, dev):
    # no two layers alike; widths that are no multiple of 8 take the generic kernels in bf16, the
    # others the matrix-core form; value width above one accumulator tier
    cfg = U.config([(U.att(heads=6, kv_heads=2, dim=16, vdim=24, conv=2, chunk=11), U.ff(10)),
                    (U.lat(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=136), None),
                    (U.att(heads=3, kv_heads=1, dim=5, vdim=6, conv=5, chunk=4, rot_dims=2), U.ff(5, 3.0)),
                    (U.lat(heads=5, dim=2, rot_dim=6, vdim=9, kv_rank=7), U.ff(33))], width=28, vocab=33, taps=2, loop=(1, 2, 2))
    r = {"a": tokens(26, 33, 14)}
    # bf16: the generic and the matrix-core kernels are both ~0.1 off here (a 136-wide latent query rounded
    # to bf16 under sharp softmaxes); the fp32 run carries the comparison
    check(tmp_path, dev, cfg, r, [[("a", 20)]] + [[("a", 1)]] * 6, bf16_tol=0.2)


# ------------------------------------------------------------------ decode, portions, batches
def test_prefill_against_token_by_token(tmp_path, dev):
    cfg = U.config(FULL, loop=(0, 2, 2))
    r = {"a": tokens(19, 50, 15)}
    check(tmp_path, dev, cfg, r, [[("a", 1)]] * 19)


@pytest.mark.parametrize("sizes", [[2] * 12, [5, 2, 7, 3, 1, 6], [1, 23], [13, 2, 2, 2, 2, 1, 1, 1]])
def test_portions(tmp_path, dev, sizes):
    cfg = U.config(FULL, taps=4, loop=(1, 3, 2))
    r = {"a": tokens(sum(sizes), 50, 16)}
    check(tmp_path, dev, cfg, r, [[("a", s)] for s in sizes])


def test_unequal_batch_against_each_alone(tmp_path, dev):
    cfg = U.config(FULL, loop=(1, 2, 3))
    r = {"a": tokens(30, 50, 17), "b": tokens(9, 50, 18), "c": tokens(17, 50, 19), "d": tokens(3, 50, 20)}
    steps = [[("a", 11), ("b", 2)], [("a", 1), ("b", 5), ("c", 9)], [("c", 1), ("a", 1), ("d", 3), ("b", 1)],
             [("a", 7), ("b", 1), ("c", 1)], [("c", 6), ("a", 1)], [("a", 9)]]
    check(tmp_path, dev, cfg, r, steps)


def test_pages_and_slots_used_again(tmp_path, dev):
    # a pool of 12 pages of 4 tokens and 2 state slots serves five requests one after another and
    # interleaved; what a finished request left in its pages and slot must not leak into the next
    cfg = U.config(FULL, loop=(1, 3, 2))
    r = {k: tokens(n, 50, 21 + i) for i, (k, n) in enumerate([("a", 22), ("b", 18), ("c", 21), ("d", 9), ("e", 20)])}
    steps = [[("a", 22)], [("b", 10)], [("b", 8), ("c", 5)], [("c", 16)], [("d", 4), ("e", 3)], [("d", 1), ("e", 1)],
             [("d", 4), ("e", 16)]]
    check(tmp_path, dev, cfg, r, steps, blocks=12, block_size=4, max_seqs=2)


def test_first_tokens_one_by_one_in_a_used_slot(tmp_path, dev):
    # the second request starts token by token in the slot and pages the first one left behind: its
    # convolutions must see zeros before position 0, not the old owner's last inputs
    cfg = U.config(FULL, taps=5)
    r = {"a": tokens(12, 50, 30), "b": tokens(8, 50, 31)}
    steps = [[("a", 12)]] + [[("b", 1)]] * 3 + [[("b", 2)], [("b", 3)]]
    check(tmp_path, dev, cfg, r, steps, blocks=8, block_size=4, max_seqs=1)


def test_long_decoding(tmp_path, dev):
    # decoded tokens pass several chunk borders of both attention layers
    cfg = U.config(FULL, loop=(1, 3, 2))
    r = {"a": tokens(140, 50, 32)}
    check(tmp_path, dev, cfg, r, [[("a", 6)]] + [[("a", 1)]] * 134, block_size=8)


def test_long_portions_in_one_step(tmp_path, dev):
    # more than one 64-key tile and more than one 128-row query block per sequence
    cfg = U.config([(U.att(heads=4, kv_heads=2, dim=16, vdim=16, chunk=100), U.ff()), (U.lat(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=24), None)],
                   width=32)
    r = {"a": tokens(300, 50, 33), "b": tokens(150, 50, 34)}
    check(tmp_path, dev, cfg, r, [[("a", 200), ("b", 70)], [("a", 100), ("b", 80)]], blocks=40, block_size=16)


# ------------------------------------------------------------------ chunk edges, page borders, far keys
def _edge_case(device, dtype, chunk, bs, L, j0, form, mfma=True, H=4, G=2, dk=8, dv=8):
    """Key row j0 matches every query of every head (its score stands far above the rest); the values are
    cached unturned here, so the output at position i is row j0's value exactly when j0 <= i and both lie
    in one chunk, and the plain softmax otherwise."""
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
    hs = 1.0 + 0.3 * torch.randn(H, generator=g).clamp(-2, 2)
    sink = torch.randn(H, generator=g)
    scale = 1.0
    cache, q = cache.to(dtype), q.to(dtype)
    # plain: full scores, explicit mask
    qf, rf = q.double(), rows.to(dtype).double().repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", qf, rf[:, :, dv:]) * scale * hs.double().view(H, 1, 1)
    i, j = torch.arange(L)[:, None], torch.arange(L)[None, :]
    pr = plain.softmax_with_extra(s, (j <= i) & (i // chunk == j // chunk), sink.double())
    want = torch.einsum("hij,jhd->ihd", pr, rf[:, :, :dv])
    d = torch.device(device)
    kw = dict(groups=G, koff=dv, chunk=chunk, hscale=hs.to(d))
    if form == "prefill":
        cut = L // 3  # the portion starts in the middle of pages and chunks
        got = hybrid.latent_attention_prefill(q[cut:].contiguous().to(d), cache.to(d), bt.to(d), torch.tensor([0, L - cut], dtype=torch.int32).to(d),
                                              torch.tensor([L], dtype=torch.int32).to(d), hybrid.NO_LIMIT, sink.to(d), scale, dv, L - cut,
                                              mfma=mfma, **kw)
        want = want[cut:]
    else:
        n = min(L, 24)  # the last n positions, each decoded alone, as one batch of n sequences
        ctx = torch.arange(L - n + 1, L + 1, dtype=torch.int32)
        got = hybrid.latent_attention_decode(q[L - n:].contiguous().to(d), cache.to(d), bt.expand(n, nb).contiguous().to(d), ctx.to(d),
                                             hybrid.NO_LIMIT, sink.to(d), scale, dv, mfma=mfma, max_ctx=L, **kw)
        want = want[L - n:]
    return got.double().cpu(), want


@pytest.mark.parametrize("form", ["prefill", "decode"])
@pytest.mark.parametrize("chunk,bs,L,j0", [(5, 4, 20, 14), (5, 4, 20, 15), (8, 8, 40, 31), (8, 8, 40, 32), (70, 16, 200, 139),
                                           (70, 16, 200, 140), (64, 16, 200, 191), (64, 16, 200, 192), (136, 16, 420, 407), (136, 16, 420, 408),
                                           (1000, 16, 700, 3), (300, 16, 700, 600)])
def test_chunk_edges_and_far_keys(dev, form, chunk, bs, L, j0):
    device, dtype, _ = dev
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    for mfma in ([True, False] if (device == "cuda" and dtype == torch.bfloat16) else [True]):
        got, want = _edge_case(device, dtype, chunk, bs, L, j0, form, mfma)
        assert float((got - want).abs().max()) < tol, (mfma, float((got - want).abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv,chunk", [(8, 4, 56, 40, 210), (4, 4, 64, 32, 33), (6, 1, 128, 128, 1000), (3, 3, 24, 40, 64),
                                            (2, 1, 7, 10, 50), (16, 2, 16, 264, 90)])
def test_grouped_attention_kernels_gpu(H, G, dk, dv, chunk):
    # random rows, every kernel form against full scores with an explicit mask
    for dtype, tol in ((torch.float32, 1e-4), (torch.bfloat16, 3e-2)):
        for form in ("prefill", "decode"):
            for mfma in (True, False):
                got, want = _edge_case("cuda", dtype, chunk, 16, 333, 250, form, mfma, H=H, G=G, dk=dk, dv=dv)
                assert float((got - want).abs().max()) < tol, (dtype, form, mfma)


@pytest.mark.gpu
@pytest.mark.parametrize("T", [20, 300])
@pytest.mark.parametrize("H,G,dk,dv,rot_dims", [(6, 2, 32, 48, 32), (4, 4, 128, 64, 96), (3, 1, 10, 6, 4), (40, 8, 16, 16, 16), (2, 1, 160, 136, 160)])
def test_qkv_preparation_kernels_gpu(T, H, G, dk, dv, rot_dims):
    # both kernel forms (few rows: a wave per head; many rows: a lane per pair) against the plain functions
    from llmctl.models.mixers import rotary_frequencies
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(11)
    d = torch.device("cuda")
    z = torch.randn(T, (H + G) * dk + G * dv, generator=g)
    qn, kn = 1.0 + 0.2 * torch.randn(dk, generator=g), 1.0 + 0.2 * torch.randn(dk, generator=g)
    pos = torch.randint(0, 3000, (T,), generator=g, dtype=torch.int32)
    slots = torch.randperm(T + 7, generator=g)[:T]
    freq, amp = rotary_frequencies(3000.0, rot_dims, {"factor": 5.0, "original": 64, "fast": 8.0, "slow": 1.0})
    vfreq, _ = rotary_frequencies(3000.0, dv, None)
    # angles as the kernels form them: the fp32 product of position and frequency (at positions in the
    # thousands its rounding, ~1e-4 rad, is far above the bound that the comparison can then keep)
    ang = (pos.float()[:, None, None] * freq[None, None, :]).double()
    vang = (pos.float()[:, None, None] * vfreq[None, None, :]).double()

    def expect(zz):
        zz = zz.double()
        turn = lambda x: torch.cat([plain.turn_pairs(x[..., :rot_dims], ang, amp), x[..., rot_dims:]], -1)
        return (turn(plain.norm_plain(zz[:, :H * dk].view(T, H, dk), qn, 1e-5)),
                turn(plain.norm_plain(zz[:, H * dk:(H + G) * dk].view(T, G, dk), kn, 1e-5)),
                plain.turn_pairs(zz[:, (H + G) * dk:].view(T, G, dv), vang))

    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        zt = z.to(dtype)
        q2, k2, v2 = expect(zt)
        cache = torch.zeros(T + 7, 1, G * (dv + dk), dtype=dtype, device=d)
        got_q = hybrid.attn_qkv_prep(zt.to(d), H, G, dk, dv, qn.to(d), kn.to(d), 1e-5, pos.to(d), freq.to(d), rot_dims, True, amp,
                                     vfreq.to(d), cache, slots.to(d))
        rows = cache.view(T + 7, G, dv + dk)[slots.to(d)].double().cpu()
        assert float((got_q.double().cpu() - q2).abs().max()) < tol * 4
        assert float((rows[:, :, dv:] - k2).abs().max()) < tol * 4
        assert float((rows[:, :, :dv] - v2).abs().max()) < tol * 4


def test_output_turn_back():
    # ofreq turns the head outputs' neighbour pairs by minus the query's position
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(7)
    L, H, dk, dv, bs = 9, 2, 4, 6, 4
    rows = torch.randn(L, 1, dv + dk, generator=g)
    cache = torch.zeros(4, bs, dv + dk)
    cache.view(-1, dv + dk)[:L] = rows[:, 0]
    bt = torch.arange(4, dtype=torch.int32)[None]
    q = torch.randn(L, H, dk, generator=g)
    fr = torch.tensor([1.0, 0.3, 0.05])
    a = (torch.tensor([0, L], dtype=torch.int32), torch.tensor([L], dtype=torch.int32))
    base = hybrid.latent_attention_prefill(q, cache, bt, *a, hybrid.NO_LIMIT, None, 0.5, dv, L, koff=dv)
    got = hybrid.latent_attention_prefill(q, cache, bt, *a, hybrid.NO_LIMIT, None, 0.5, dv, L, koff=dv, ofreq=fr)
    ang = -torch.arange(L, dtype=torch.float64)[:, None, None] * fr.double()
    assert torch.allclose(got.double(), plain.turn_pairs(base.double(), ang), atol=1e-5)


# ------------------------------------------------------------------ the convolution and its state
def _conv_case(device, dtype, C, taps, portions, residual, hint=True):
    """Two sequences in portions against the whole-sequence shifted sum; the slots start dirty."""
    from llmctl.ops import hybrid

    g = torch.Generator().manual_seed(3)
    d = torch.device(device)
    lens = [sum(p[0] for p in portions), sum(p[1] for p in portions)]
    u = [torch.randn(n, C, generator=g).to(dtype) for n in lens]
    w = torch.randn(C, taps, generator=g)
    state = torch.randn(3, taps - 1, C, generator=g).to(d)
    at, outs = [0, 0], [[], []]
    for pa, pb in portions:
        seqs = [(s, n) for s, n in ((0, pa), (1, pb)) if n]
        rows = torch.cat([u[s][at[s]:at[s] + n] for s, n in seqs])
        cu = torch.tensor([0] + list(torch.tensor([n for _, n in seqs]).cumsum(0)), dtype=torch.int32)
        seq_of = torch.repeat_interleave(torch.arange(len(seqs), dtype=torch.int32), torch.tensor([n for _, n in seqs]))
        start = torch.tensor([at[s] for s, _ in seqs], dtype=torch.int32)
        slot = torch.tensor([2 - s for s, _ in seqs], dtype=torch.int32)
        y = hybrid.causal_conv(rows.to(d), w.t().contiguous().to(d), state, seq_of.to(d), cu.to(d), start.to(d), slot.to(d), residual,
                               max_len=max(pa, pb) if hint else 0).cpu()
        o = 0
        for s, n in seqs:
            outs[s].append(y[o:o + n])
            o += n
            at[s] += n
    for s in range(2):
        want = plain.causal_conv(u[s].double(), w) + (u[s].double() if residual else 0.0)
        assert torch.allclose(torch.cat(outs[s]).double(), want, atol=1e-5 if dtype == torch.float32 else 5e-2)


@pytest.mark.parametrize("taps,portions", [(4, [(7, 1), (1, 1), (2, 1), (1, 5), (3, 0), (0, 2)]), (2, [(1, 3), (1, 1), (4, 1)]),
                                           (6, [(2, 1), (2, 1), (1, 1), (9, 2)]), (1, [(3, 2), (1, 1)])])
def test_causal_conv_state(dev, taps, portions):
    device, dtype, _ = dev
    _conv_case(device, dtype, 37, taps, portions, residual=False)
    _conv_case(device, dtype, 304, taps, portions, residual=True)  # channel counts that allow 16-byte accesses
    _conv_case(device, dtype, 64, taps, portions, residual=False, hint=False)  # no length hint: never the one-launch form


# ------------------------------------------------------------------ the framework's own entry point
def test_greedy_generation_through_the_scheduler(tmp_path, dev):
    from llmctl.serve.scheduler import SamplingParams

    device, dtype, _ = dev
    cfg = U.config(FULL, loop=(1, 3, 2))
    W = U.random_weights(cfg, 50)
    path = U.write_checkpoint(tmp_path / "ck", cfg, W)
    eng = U.engine(path, device, dtype, blocks=40, block_size=4, max_seqs=3, scheduler="dynamic")
    prompts = [tokens(9, 50, 51), tokens(2, 50, 52), tokens(14, 50, 53), tokens(5, 50, 54), tokens(1, 50, 55)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    slack = 1e-3 if dtype == torch.float32 else 0.15
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

    cfg = U.config(FULL, loop=(1, 3, 2))
    path = U.write_checkpoint(tmp_path / "ck", cfg, U.random_weights(cfg, 60))
    prompts = [tokens(6, 50, 61 + i) for i in range(4)]
    p = SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True)
    tight = U.engine(path, "cpu", blocks=10, block_size=4, max_seqs=4).generate(prompts, p)
    roomy = U.engine(path, "cpu", blocks=64, block_size=4, max_seqs=1).generate(prompts, p)
    assert sum(s.preemptions for s in tight) > 0
    assert [s.output_ids for s in tight] == [s.output_ids for s in roomy]


def test_checkpoint_names_round_trip(tmp_path):
    from llmctl.models import get_model_config
    from llmctl.models.dumalix import DumalixConfig, DumalixLM

    cfg = U.config(FULL, loop=(1, 3, 2))
    W = U.random_weights(cfg, 70)
    m = DumalixLM(DumalixConfig.from_dict(cfg), dtype=torch.float32)
    m.load_named(W)
    back = m.export_named()
    assert set(back) == set(W)
    for k in W:
        assert torch.equal(back[k], W[k]), k
    assert DumalixConfig.from_dict(DumalixConfig.from_dict(cfg).to_dict()).to_dict() == DumalixConfig.from_dict(cfg).to_dict()
    t = get_model_config("dumalix-w64-l4-h4-g2")
    assert t.architecture == "Dumalix" and t.layers == 4 and len(t.runs()) == 4


def test_trace_replay_command(tmp_path):
    # the replay command end to end on a written checkpoint: two requests, a shared step, logits files
    import json
    import subprocess
    import sys

    import numpy as np

    cfg = U.config(FULL, loop=(1, 3, 2))
    W = {k: v.bfloat16().float() for k, v in U.random_weights(cfg, 80).items()}
    path = U.write_checkpoint(tmp_path / "ck", cfg, W)
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
