"""sr_batch_append_tokens: a decode loop that appends the sampled token to every row's history each step
(RecentTokens.Add, ContinuousBatchingEngine.cs:650, 1280) must sample exactly what the CPU oracle samples from the
histories as they stand -- whether a row is updated in place or makes the call rebuild the batch -- and exactly what a
batch uploaded afresh with the longer histories samples."""
import dataclasses

import numpy as np
import pytest

from opentail.stingray_amd import SamplerContext, SamplingParams, pack_allow_mask
from tests.helpers import hooks_lib, oracle_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _rows(rng, vocab):
    """Every kind of row the update distinguishes."""
    def hist(n):
        return rng.integers(-2, vocab + 2, n).tolist()  # a few ids outside the vocabulary

    P = SamplingParams
    return [
        # SampleTopK, penalties that only lower: updated in place
        P(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1, RepeatLastN=64, PreviousTokens=hist(64)),
        P(Temperature=1.0, TopK=8, RepetitionPenalty=1.3, RepeatLastN=5, PreviousTokens=hist(3)),       # window fills up
        P(Temperature=0.7, TopK=100, MinP=0.02, PresencePenalty=0.4, FrequencyPenalty=0.3, PreviousTokens=hist(200)),
        P(Temperature=1.2, TopK=5, RepetitionPenalty=1.5, RepeatLastN=0, PresencePenalty=0.2, PreviousTokens=hist(10)),
        P(Temperature=0.9, TopK=3, RepetitionPenalty=1.2, RepeatLastN=-1, PreviousTokens=hist(1)),
        # greedy with penalties: in place
        P(Temperature=0.0, RepetitionPenalty=1.4, RepeatLastN=8, FrequencyPenalty=0.5, PreviousTokens=hist(12)),
        # full-vocabulary rows with penalties: in place
        P(Temperature=0.7, TopP=0.9, MinP=0.05, FrequencyPenalty=0.5, PresencePenalty=0.3, PreviousTokens=hist(50)),
        P(Temperature=1.0, RepetitionPenalty=1.1, RepeatLastN=4, PreviousTokens=hist(6)),
        # no penalties at all: the history is never read
        P(Temperature=0.8, TopK=20, TopP=0.9, PreviousTokens=hist(5)),
        P(Temperature=0.0, PreviousTokens=None),
        # rows whose first history token makes the call rebuild the batch (once): empty history with penalties
        P(Temperature=0.8, TopK=10, RepetitionPenalty=1.2, PreviousTokens=None),
        P(Temperature=0.0, PresencePenalty=1.0, PreviousTokens=[]),
        # penalties that may raise a logit (edits sorted by id, over-selection by the history length, which grows with
        # every token) and logit bias (edits sorted by id): in place, the edits behind a new id move up
        P(Temperature=0.9, TopK=12, RepetitionPenalty=0.8, PresencePenalty=-0.3, PreviousTokens=hist(7)),
        P(Temperature=1.0, TopP=0.8, PresencePenalty=0.5, LogitBias={3: 2.0, 11: -1.0}, PreviousTokens=hist(4)),
        P(Temperature=0.7, TopK=300, TopP=0.9, FrequencyPenalty=-0.2, RepeatLastN=16, RepetitionPenalty=1.3,
          PreviousTokens=hist(90)),
        P(Temperature=0.8, MinP=0.01, RepetitionPenalty=1.2, RepeatLastN=10,
          LogitBias={i * 37 % 2000: (i % 5) - 2.0 for i in range(40)}, PreviousTokens=hist(30)),
    ]


def _peaked_logits(rng, rows, vocab, hot):
    """The same few tokens carry the mass at every step, so that sampled tokens come back and the penalties decide."""
    lg = rng.normal(0.0, 1.0, (rows, vocab)).astype(np.float32)
    lg[:, hot] += rng.uniform(4.0, 7.0, (rows, len(hot))).astype(np.float32)
    return lg


def _rebuilds(ctx, batch):
    import ctypes as C

    return int(hooks_lib().sr_debug_append_rebuilds(batch.h))


@pytest.mark.parametrize("vocab,dtype_bf16,pad,in_place_only",
                         [(5000, False, 0, True), (2311, False, 3, True), (70001, True, 0, True),
                          (5000, False, 0, False), (40003, True, 1, False)])
def test_decode_loop_with_appended_tokens_matches_oracle_and_fresh_upload(ctx, vocab, dtype_bf16, pad, in_place_only):
    import torch

    rng = np.random.default_rng(vocab + pad)
    params = _rows(rng, vocab)
    if in_place_only:
        params = params[:10]  # without the rows that make every call rebuild the batch
    rows = len(params)
    hists = [list(p.PreviousTokens or []) for p in params]
    u0 = rng.random(rows)
    inc = ctx.new_batch().upload(params, vocab, u0)
    steps = 45  # more new ids than an edit range has room for: rows run out of room and are rebuilt
    hot = rng.choice(vocab, 24, replace=False)
    for step in range(steps):
        lg = _peaked_logits(rng, rows, vocab, hot)
        if dtype_bf16:
            lg = (lg.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)  # exactly representable in bf16
            wide = np.zeros((rows, vocab + pad), dtype=np.float32)
            wide[:, :vocab] = lg
            dev = torch.from_numpy(wide).cuda().to(torch.bfloat16)[:, :vocab]
        else:
            wide = np.zeros((rows, vocab + pad), dtype=np.float32)
            wide[:, :vocab] = lg
            dev = torch.from_numpy(wide).cuda()[:, :vocab]
        u = u0 if step == 0 else u_next
        now = [dataclasses.replace(p, PreviousTokens=list(h)) for p, h in zip(params, hists)]
        want = oracle_tokens(lg, now, u)

        toks = torch.full((rows,), -9, dtype=torch.int32, device="cuda")
        ctx.sample_launch(inc, dev, toks)
        ctx.synchronize()
        got = toks.cpu().numpy()
        assert got.tolist() == want.tolist(), f"step {step}: appended batch differs from the oracle"

        fresh = ctx.new_batch().upload(now, vocab, u)
        toks2 = torch.full((rows,), -9, dtype=torch.int32, device="cuda")
        ctx.sample_launch(fresh, dev, toks2)
        ctx.synchronize()
        assert toks2.cpu().numpy().tolist() == want.tolist(), f"step {step}: fresh upload differs from the oracle"
        fresh.close()

        # the engine appends what it sampled; every seventh step two rows sit out (finished sequences), and now and
        # then a row gets an id outside the vocabulary
        app = got.astype(np.int32).copy()
        if step % 7 == 3:
            app[[1, 6]] = -1
        if step % 11 == 5:
            app[2] = vocab + 5
        u_next = rng.random(rows)
        if step % 2 == 0:
            inc.append_tokens(app, u_next)
        else:  # uniforms handed over separately
            inc.append_tokens(app)
            inc.set_uniforms(u_next)
        for r in range(rows):
            if app[r] >= 0:
                hists[r].append(int(app[r]))
    n_rebuilt, n_moved = _rebuilds(ctx, inc), int(hooks_lib().sr_debug_append_moves(inc.h))
    # a row that runs out of room moves to the end of the edit array; only a row's first history token (or a change of
    # path) rebuilds the batch
    assert n_rebuilt <= (0 if in_place_only else 4), (n_rebuilt, n_moved)
    inc.close()


def test_append_before_the_first_launch_and_new_ids_every_step(ctx):
    """Tokens appended before any launch (no scan masks exist yet) and a run of ids the history has not seen."""
    import torch

    vocab = 4096
    rng = np.random.default_rng(5)
    params = [SamplingParams(Temperature=0.8, TopK=30, RepetitionPenalty=1.3, RepeatLastN=16, FrequencyPenalty=0.2,
                             PreviousTokens=rng.integers(0, vocab, 20).tolist()) for _ in range(6)]
    hists = [list(p.PreviousTokens) for p in params]
    u = rng.random(6)
    b = ctx.new_batch().upload(params, vocab, u)
    for step in range(40):
        app = rng.integers(0, vocab, 6).astype(np.int32)  # mostly unseen ids
        b.append_tokens(app)
        for r in range(6):
            hists[r].append(int(app[r]))
        if step % 4 != 3:
            continue
        lg = rng.normal(0, 2.0, (6, vocab)).astype(np.float32)
        for r in range(6):
            lg[r, hists[r][-8:]] += 6.0  # the recent history carries the mass: the penalties decide
        now = [dataclasses.replace(p, PreviousTokens=list(h)) for p, h in zip(params, hists)]
        toks = torch.full((6,), -9, dtype=torch.int32, device="cuda")
        ctx.sample_launch(b, torch.from_numpy(lg).cuda(), toks)
        ctx.synchronize()
        assert toks.cpu().numpy().tolist() == oracle_tokens(lg, now, u).tolist(), f"step {step}"
    # 40 unseen ids per row, room for 32: every row has moved to the end of the edit array once, none rebuilt the batch
    assert _rebuilds(ctx, b) == 0 and int(hooks_lib().sr_debug_append_moves(b.h)) >= 6
    b.close()


def test_append_is_refused_for_a_batch_with_allow_masks(ctx):
    vocab = 300
    params = [SamplingParams(Temperature=0.8, TopK=5, PreviousTokens=[1, 2])]
    allow = np.ones((1, vocab), dtype=bool)
    b = ctx.new_batch().upload(params, vocab, [0.5], pack_allow_mask(allow))
    with pytest.raises(NotImplementedError):
        b.append_tokens([3])
    b.close()


def test_histories_that_outgrow_the_pinned_staging_memory_of_their_batch(ctx):
    """A long run of appended tokens that are new to their rows: the edit lists grow past what the batch's pinned
    staging memory was sized for, so that an upload sends part of its pieces packed and part straight from the host
    arrays.  The pieces must reach the device in the order they were made (the row descriptors are sent twice)."""
    import torch

    rng = np.random.default_rng(99)
    rows, V, steps = 96, 30_011, 130
    logits = rng.normal(0, 1.5, (rows, V)).astype(np.float32)
    dev = torch.from_numpy(logits).cuda()
    params = []
    for r in range(rows):
        hist = rng.integers(0, V, 24).tolist()
        if r % 4 == 0:
            params.append(SamplingParams(Temperature=0.0, RepetitionPenalty=1.15, PresencePenalty=0.2, PreviousTokens=hist))
        else:
            params.append(SamplingParams(Temperature=0.9, TopK=int(rng.integers(1, 400)), TopP=0.95, RepetitionPenalty=1.1,
                                         FrequencyPenalty=0.1, PresencePenalty=0.1, PreviousTokens=hist))
    u = rng.random(rows)
    batch = ctx.new_batch().upload(params, V, u)
    toks = torch.empty(rows, dtype=torch.int32, device="cuda")
    for step in range(steps):
        new = rng.integers(0, V, rows).astype(np.int32)
        for r, p in enumerate(params):
            p.PreviousTokens = list(p.PreviousTokens) + [int(new[r])]
        u = rng.random(rows)
        batch.append_tokens(new, u)
        ctx.sample_launch(batch, dev, toks)
        if step % 13 == 0 or step == steps - 1:
            ctx.synchronize()
            torch.cuda.synchronize()
            assert np.array_equal(toks.cpu().numpy(), oracle_tokens(logits, params, u)), step
    # rows move to the end of the edit array as they run out of room, until the device array (made for four times what
    # the upload needed) is full and the batch is rebuilt, which packs it again
    assert _rebuilds(ctx, batch) >= 1 and int(hooks_lib().sr_debug_append_moves(batch.h)) >= rows
    batch.close()
