"""GPU parity, through the C ABI: SampleTopK (Sampler.cs:216-357) for rows whose top_k (plus history) is beyond what
the selection kernel's row tail sorts -- they take two device-wide sorts instead.  Token ids must be bit-exact."""
import numpy as np
import pytest

from opentail.stingray_amd import SamplerContext, SamplingParams, pack_allow_mask
from tests.helpers import oracle_tokens

pytestmark = pytest.mark.gpu
NEG_INF = np.float32("-inf")
OUT_TOPK, OUT_DEGENERATE, OUT_UNSUPPORTED = 2, 8, 1 << 31


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a, dtype=None):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.view(dtype)
    return t.cuda()


def _check(ctx, logits, params, uniforms, device_tensor=None, allow_mask=None, mask_active=None):
    dev = _cuda(logits) if device_tensor is None else device_tensor
    got, flags = ctx.sample_batch(dev, params, uniforms, allow_mask, mask_active, return_flags=True)
    want = oracle_tokens(logits, params, uniforms, allow_mask, mask_active)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"rows {bad[:8]} differ: gpu {got[bad[:8]]} oracle {want[bad[:8]]} flags {flags[bad[:8]]}"
    assert not np.any(flags & OUT_UNSUPPORTED)
    return flags


def test_top_k_beyond_the_row_tail_without_penalties(ctx):
    rng = np.random.default_rng(71)
    V = 40_000
    ks = [2049, 2500, 3000, 5000, 20_000, V - 1, 2048, 64]
    logits = rng.normal(0, 2.5, (len(ks), V)).astype(np.float32)
    logits[:, :40] += np.linspace(9, 3, 40, dtype=np.float32)
    params = [SamplingParams(Temperature=float(rng.choice([0.6, 1.0, 1.5])), TopK=k,
                             TopP=float(rng.choice([1.0, 0.95, 0.6])), MinP=float(rng.choice([0.0, 1e-4, 0.02])))
              for k in ks]
    for _ in range(4):
        flags = _check(ctx, logits, params, rng.random(len(ks)))
        assert np.all(flags & OUT_TOPK)
    # draws at both ends of the unit interval
    _check(ctx, logits, params, np.zeros(len(ks)))
    _check(ctx, logits, params, np.full(len(ks), 1.0 - 2.0 ** -53))


def test_long_histories_with_lowering_and_raising_penalties(ctx):
    rng = np.random.default_rng(72)
    V, rows = 30_000, 10
    logits = rng.normal(0, 2.0, (rows, V)).astype(np.float32)
    head = np.argsort(-logits, axis=1)
    params = []
    for i in range(rows):
        k = [1800, 40, 1500, 2200, 500, 3000, 64, 1000, 2048, 10][i]
        n_hist = [600, 2600, 700, 100, 3000, 3000, 5000, 1200, 1, 2100][i]
        near = head[i, rng.integers(0, k + n_hist, n_hist // 2)]           # many land among the candidates
        hist = np.concatenate([near, rng.integers(-5, V + 5, n_hist - n_hist // 2)])
        rng.shuffle(hist)
        raising = i % 2 == 1
        params.append(SamplingParams(
            Temperature=float(rng.uniform(0.6, 1.4)), TopK=k, TopP=float(rng.choice([1.0, 0.9])),
            MinP=float(rng.choice([0.0, 0.01])),
            RepetitionPenalty=float(rng.choice([0.8, 1.25]) if raising else rng.choice([1.0, 1.3])),
            PresencePenalty=float(rng.choice([-0.6, 0.3]) if raising else rng.choice([0.0, 0.5])),
            FrequencyPenalty=float(rng.choice([-0.2, 0.1]) if raising else rng.choice([0.0, 0.2])),
            RepeatLastN=int(rng.choice([0, 64, 1000])), PreviousTokens=hist.tolist()))
    for _ in range(3):
        _check(ctx, logits, params, rng.random(rows))


def test_ties_masks_and_rows_with_fewer_allowed_ids_than_k(ctx):
    rng = np.random.default_rng(73)
    V, rows = 6_000, 8
    logits = (rng.integers(-20, 20, (rows, V)) / 4.0).astype(np.float32)     # coarse grid: long runs of equal values
    allowed = rng.random((rows, V)) < np.array([0.9, 0.5, 0.3, 0.05, 0.9, 0.01, 0.5, 0.0])[:, None]
    allowed[7] = False                                                        # nothing allowed: index 0
    mask = pack_allow_mask(allowed)
    active = np.array([1, 1, 1, 1, 0, 1, 1, 1], dtype=np.uint8)
    masked = np.where(allowed | (active[:, None] == 0), logits, NEG_INF).astype(np.float32)
    params = []
    for i in range(rows):
        hist = rng.integers(0, V, int(rng.integers(0, 400))).tolist()
        params.append(SamplingParams(Temperature=float(rng.choice([0.5, 1.0])), TopK=int(rng.choice([2100, 4000, V - 1])),
                                     TopP=float(rng.choice([1.0, 0.8])), MinP=float(rng.choice([0.0, 0.001])),
                                     RepetitionPenalty=float(rng.choice([1.0, 1.2])), PreviousTokens=hist))
    for _ in range(3):
        u = rng.random(rows)
        dev = _cuda(logits)
        got, flags = ctx.sample_batch(dev, params, u, mask, active, return_flags=True)
        want = oracle_tokens(masked, params, u)
        assert np.array_equal(got, want), (got, want)
        assert flags[7] & OUT_DEGENERATE and got[7] == 0


def test_bf16_rows_and_a_batch_that_mixes_every_path(ctx):
    import torch

    rng = np.random.default_rng(74)
    V, rows = 50_000, 12
    f32 = rng.normal(0, 3.0, (rows, V)).astype(np.float32)
    bf = (f32.view(np.uint32) >> 16).astype(np.uint16)                        # truncation: exact bf16 values
    logits = (bf.astype(np.uint32) << 16).view(np.float32)
    params = []
    for i in range(rows):
        kind = i % 4
        hist = rng.integers(0, V, 300).tolist()
        if kind == 0:    # wide
            p = SamplingParams(Temperature=0.9, TopK=int(rng.choice([2300, 7000])), TopP=0.97, RepetitionPenalty=1.1,
                               PreviousTokens=hist)
        elif kind == 1:  # selection kernel
            p = SamplingParams(Temperature=0.8, TopK=50, TopP=0.9, MinP=0.02, RepetitionPenalty=1.1, PreviousTokens=hist)
        elif kind == 2:  # greedy
            p = SamplingParams(Temperature=0.0, RepetitionPenalty=1.2, PreviousTokens=hist)
        else:            # full vocabulary
            p = SamplingParams(Temperature=1.0, TopK=0, TopP=0.9)
        params.append(p)
    dev = _cuda(bf.view(np.int16), torch.bfloat16)
    for _ in range(3):
        _check(ctx, logits, params, rng.random(rows), device_tensor=dev)


def test_resampling_named_rows_agrees_with_the_selection_kernel_and_long_plateaus_at_the_cut(ctx):
    import torch

    rng = np.random.default_rng(75)
    V, rows = 60_000, 6
    logits = rng.normal(0, 1.0, (rows, V)).astype(np.float32)
    # rows 0-2: a plateau of 5,000 to 30,000 equal logits right at the top-k cut, a few hundred larger values above it
    for i, width in enumerate([5_000, 12_000, 30_000]):
        where = rng.permutation(V)
        logits[i, where[:width]] = np.float32(4.0)
        logits[i, where[width:width + 300]] = (4.0 + rng.random(300) * 3).astype(np.float32)
    params = [SamplingParams(Temperature=float(t), TopK=int(k), TopP=float(p), MinP=float(m), RepetitionPenalty=1.15,
                             PreviousTokens=rng.integers(0, V, 100).tolist())
              for t, k, p, m in [(0.8, 1000, 0.98, 0.0), (1.0, 2000, 1.0, 0.0), (0.7, 600, 0.9, 0.001),
                                 (0.9, 40, 0.95, 0.02), (1.2, 700, 1.0, 0.0), (0.6, 5, 0.9, 0.0)]]
    dev = _cuda(logits)
    for _ in range(3):
        u = rng.random(rows)
        _check(ctx, logits, params, u, device_tensor=dev)      # sample_batch: overflowing rows are redone by itself
        # every row once more through the sort path, named explicitly
        batch = ctx.new_batch().upload(params, V, u)
        toks = torch.full((rows,), -5, dtype=torch.int32, device="cuda")
        flags = torch.zeros(rows, dtype=torch.int32, device="cuda")
        ctx.resample_rows_launch(batch, dev, np.arange(rows), toks, flags)
        ctx.synchronize()
        torch.cuda.synchronize()
        batch.close()
        assert np.array_equal(toks.cpu().numpy(), oracle_tokens(logits, params, u))
        assert np.all(flags.cpu().numpy().view(np.uint32) & OUT_TOPK)
