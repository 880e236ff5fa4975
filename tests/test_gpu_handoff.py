"""The selection kernel finishes every row inside its one launch.  The reference has no failure mode here -- SampleTopK
always returns a token (Sampler.cs:216-357, :251-255) -- so neither may the launch: rows whose candidates overflow the
kernel's lists (thousands of equal logits at the cut) are selected exactly from the logits themselves, batches of more
rows than the device has compute units are worked off by the same workers, and the counters of one launch never reach
a later one.  The exact fallback is also forced for every row from the host (a poll limit of zero for the one bounded
wait of the kernel; every kernel exits normally): the results must not change."""
import ctypes as C

import numpy as np
import pytest

from opentail.stingray_amd import SamplerContext, SamplingParams, pack_allow_mask, synthetic
from tests.helpers import hooks_lib, oracle_tokens

pytestmark = pytest.mark.gpu
UNSUPPORTED = np.uint32(1 << 31)


@pytest.fixture()
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _launch(ctx, batch, dev, rows):
    import torch

    toks = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    flags = torch.zeros(rows, dtype=torch.int32, device="cuda")
    ctx.sample_launch(batch, dev, toks, flags)
    ctx.synchronize()
    torch.cuda.synchronize()
    return toks.cpu().numpy(), flags.cpu().numpy().view(np.uint32)


def _mixed_rows(rng, rows, vocab):
    """Greedy, greedy with penalties, top-k with lowering and with raising penalties, masks, ties."""
    logits = (rng.normal(0, 1.5, (rows, vocab))).astype(np.float32)
    logits[:, ::97] = np.round(logits[:, ::97] * 2) / 2          # exact ties
    logits[1] = 0.25                                              # a constant row
    params = []
    for r in range(rows):
        hist = rng.integers(-2, vocab + 2, int(rng.integers(0, 80))).tolist()
        kind = r % 5
        if kind == 0:
            p = SamplingParams(Temperature=0.0)
        elif kind == 1:
            p = SamplingParams(Temperature=0.0, RepetitionPenalty=1.3, PresencePenalty=0.5, PreviousTokens=hist)
        elif kind == 2:
            p = SamplingParams(Temperature=0.8, TopK=int(rng.integers(1, 900)), TopP=0.95, MinP=0.01,
                               RepetitionPenalty=1.1, FrequencyPenalty=0.1, PreviousTokens=hist)
        elif kind == 3:
            p = SamplingParams(Temperature=1.1, TopK=int(rng.integers(1, 60)), RepetitionPenalty=0.8,
                               PresencePenalty=-0.2, PreviousTokens=hist)
        else:
            p = SamplingParams(Temperature=0.6, TopK=int(rng.integers(1, 300)), TopP=float(rng.uniform(0.5, 1.0)))
        params.append(p)
    allowed = np.ones((rows, vocab), dtype=bool)
    active = np.zeros(rows, dtype=np.uint8)
    for r in range(0, rows, 3):
        allowed[r] = synthetic.run_mask(rng, vocab, float(rng.choice([0.002, 0.05, 0.5])))
        active[r] = 1
    return logits, params, pack_allow_mask(allowed), active


@pytest.mark.parametrize("vocab", [9_001, 151_936])
def test_rows_selected_from_the_logits_alone_give_the_same_tokens_and_launches_do_not_disturb_each_other(ctx, vocab):
    rng = np.random.default_rng(vocab)
    rows = 40
    logits, params, mask, active = _mixed_rows(rng, rows, vocab)
    dev = _cuda(logits)
    u = rng.random(rows)
    want = oracle_tokens(logits, params, u, mask, active)
    batch = ctx.new_batch().upload(params, vocab, u, mask, active)
    got, flags = _launch(ctx, batch, dev, rows)
    assert np.array_equal(got, want)
    # no tail waits for its row's other chunks: every row by the exact fallback, while the chunks still count themselves in
    ctx._check(hooks_lib().sr_debug_set_spin_limit(ctx.h, 0))
    for _ in range(3):
        got, flags = _launch(ctx, batch, dev, rows)
        assert np.array_equal(got, want), np.nonzero(got != want)[0]
        assert not np.any(flags & UNSUPPORTED)
    # back to waiting: the counters of the launches before must not be seen
    ctx._check(hooks_lib().sr_debug_set_spin_limit(ctx.h, 1 << 22))
    for _ in range(3):
        u = rng.random(rows)
        batch.set_uniforms(u)
        got, flags = _launch(ctx, batch, dev, rows)
        assert np.array_equal(got, oracle_tokens(logits, params, u, mask, active))
        assert not np.any(flags & UNSUPPORTED)
    batch.close()


def test_plateaus_of_thousands_of_equal_logits_at_the_cut_are_finished_inside_the_launch(ctx):
    rng = np.random.default_rng(75)
    V, rows = 60_000, 8
    logits = rng.normal(0, 1.0, (rows, V)).astype(np.float32)
    for i, width in enumerate([5_000, 9_000, 12_000, 30_000, 59_000]):
        where = rng.permutation(V)
        logits[i, where[:width]] = np.float32(4.0)
        logits[i, where[width:width + 300]] = (4.0 + rng.random(300) * 3).astype(np.float32)
    params = [SamplingParams(Temperature=float(t), TopK=int(k), TopP=float(p), MinP=float(m), RepetitionPenalty=1.15,
                             PreviousTokens=rng.integers(0, V, 100).tolist())
              for t, k, p, m in [(0.8, 1000, 0.98, 0.0), (1.0, 1900, 1.0, 0.0), (1.0, 1900, 1.0, 0.0), (0.7, 600, 0.9, 0.001),
                                 (0.9, 1500, 1.0, 0.0), (0.9, 40, 0.95, 0.02), (1.2, 700, 1.0, 0.0), (0.6, 5, 0.9, 0.0)]]
    dev = _cuda(logits)
    for _ in range(3):
        u = rng.random(rows)
        batch = ctx.new_batch().upload(params, V, u)
        got, flags = _launch(ctx, batch, dev, rows)   # the asynchronous launch alone, no second call
        batch.close()
        assert not np.any(flags & UNSUPPORTED)
        assert np.array_equal(got, oracle_tokens(logits, params, u))


def test_a_batch_of_more_rows_than_the_device_has_compute_units(ctx):
    # more workers than fit the device at once: the surplus starts as slots fall free
    rng = np.random.default_rng(5)
    rows, V = 700, 12_345
    logits = rng.normal(0, 2.0, (rows, V)).astype(np.float32)
    params = [SamplingParams(Temperature=0.0) if r % 7 == 0 else
              SamplingParams(Temperature=0.9, TopK=int(rng.integers(1, 200)), TopP=0.9) for r in range(rows)]
    u = rng.random(rows)
    dev = _cuda(logits)
    batch = ctx.new_batch().upload(params, V, u)
    want = oracle_tokens(logits, params, u)
    for _ in range(2):
        got, flags = _launch(ctx, batch, dev, rows)
        assert np.array_equal(got, want)
    batch.close()
