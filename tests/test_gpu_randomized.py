"""Randomized GPU parity through the C ABI: seeded random batches (row widths from 2 to 70,000, every filter
combination, history penalties, logit bias, allow-masks, -inf entries, ties, bf16 and unaligned rows) through every
entry point of the path, each result compared with the CPU oracle: token ids and distributions bit for bit."""
import numpy as np
import pytest

from oracle import binding as orc
from opentail.stingray_amd import SamplerContext, SamplingParams, pack_allow_mask
from tests.helpers import oracle_tokens, to_oracle

pytestmark = pytest.mark.gpu
NEG = np.float32("-inf")


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _strided(a, pad, dtype=None):
    """The rows of `a` inside a wider device tensor: row stride = a.shape[1] + pad elements."""
    import torch

    wide = np.zeros((a.shape[0], a.shape[1] + pad), dtype=a.dtype)
    wide[:, :a.shape[1]] = a
    t = torch.from_numpy(wide)
    if dtype is not None:
        t = t.view(dtype)
    return t.cuda()[:, :a.shape[1]]


def _params(rng, n, spec=False):
    hist = rng.integers(-3, n + 3, int(rng.choice([0, 3, 40, 300]))).tolist()
    bias = None
    if rng.random() < 0.2:
        bias = {int(k): float(v) for k, v in zip(rng.integers(-2, n + 2, 3), rng.normal(0, 3, 3))}
    return SamplingParams(
        Temperature=float(rng.choice([0.0, 0.3, 0.8, 1.0, 1.6])),
        TopK=int(rng.choice([0, 0, 1, 2, 7, 50, 900, 2500, n, n + 5])),
        TopP=float(rng.choice([1.0, 0.95, 0.7, 0.2])), MinP=float(rng.choice([0.0, 1e-4, 0.05, 0.4])),
        RepetitionPenalty=float(rng.choice([1.0, 1.2, 0.8])), PresencePenalty=float(rng.choice([0.0, 0.5, -0.5])),
        FrequencyPenalty=float(rng.choice([0.0, 0.2, -0.1])), RepeatLastN=int(rng.choice([0, 5, 64])),
        PreviousTokens=hist, LogitBias=bias,
        SpecDraftPMin=float(rng.choice([0.0, 0.0, 0.05, 0.5])) if spec else 0.0)


def _logits(rng, rows, n):
    kind = rng.integers(0, 4)
    if kind == 0:    # half-integer steps: many exact ties
        lg = (rng.integers(-14, 14, (rows, n)) / 2.0).astype(np.float32)
    elif kind == 1:
        lg = rng.normal(0, rng.choice([0.3, 2.0, 6.0]), (rows, n)).astype(np.float32)
    elif kind == 2:  # quarter steps
        lg = np.round(rng.normal(0, 2, (rows, n)) * 4).astype(np.float32) / 4
    else:            # bf16-representable values
        lg = (rng.normal(0, 2, (rows, n)).astype(np.float32).view(np.uint32) & 0xffff0000).view(np.float32)
    if rng.random() < 0.3:
        lg[rng.random((rows, n)) < 0.2] = NEG
    return lg


def _width(rng, top):
    return int(rng.choice([rng.integers(2, 40), rng.integers(40, 3000), rng.integers(3000, top)]))


def _mask(rng, rows, n):
    if rng.random() >= 0.3:
        return None, None
    return pack_allow_mask(rng.random((rows, n)) < rng.choice([0.02, 0.5, 0.95])), (rng.random(rows) < 0.7).astype(np.uint8)


def _same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint32), np.ascontiguousarray(b).view(np.uint32))


@pytest.mark.parametrize("seed", [6, 8])
def test_random_batches_tokens_and_distributions(ctx, seed):
    import torch

    rng = np.random.default_rng(seed)
    for trial in range(500):
        rows, n = int(rng.integers(1, 10)), _width(rng, 70000)
        lg = _logits(rng, rows, n)
        params = [_params(rng, n) for _ in range(rows)]
        mask, act = _mask(rng, rows, n)
        u = rng.random(rows)
        pad = int(rng.integers(0, 8)) if trial % 3 == 0 else 0
        if trial % 6 == 3:
            bf = (lg.view(np.uint32) >> 16).astype(np.uint16)
            lg = (bf.astype(np.uint32) << 16).view(np.float32)             # what the bf16 tensor holds
            dev = _strided(bf.view(np.int16), pad, torch.bfloat16)
        else:
            dev = _strided(lg, pad)
        got = ctx.sample_batch(dev, params, u, mask, act)
        assert np.array_equal(got, oracle_tokens(lg, params, u, mask, act)), (seed, trial, rows, n, str(dev.dtype), pad)
        if trial % 4 == 0:
            d = ctx.build_distribution(dev, params, None, mask, act).cpu().numpy()
            for r, p in enumerate(params):
                row = orc.apply_allow_mask(lg[r], mask[r]) if (mask is not None and act[r]) else lg[r]
                assert _same_bits(d[r], orc.build_filtered_distribution(row, to_oracle(p))), (seed, trial, r, n, p)
        if trial % 4 == 2:
            toks, d = ctx.sample_with_distribution(dev, params, u)
            d = d.cpu().numpy()
            for r, p in enumerate(params):
                wt, wd = orc.sample_with_distribution(lg[r], to_oracle(p), orc.Rng(replay=[u[r]]))
                assert toks[r] == wt and _same_bits(d[r], wd), (seed, trial, r, n, p)


def test_random_batches_with_a_worker_per_row(ctx):
    # 136 .. 256 rows: the launch in which every worker streams its own row, keeps the chunk results in registers and
    # takes one share of the bound per wave and row.  Row widths of one to four chunks, rows of ties, of negative
    # logits only, with whole chunks masked out, top-k from 1 to 2,000 (beyond the kernel's lists: the wide path),
    # histories that lower and that raise, allow-masks; fp32 and bf16.
    import torch

    from opentail.stingray_amd import synthetic

    rng = np.random.default_rng(77)
    for trial in range(60):
        rows = int(rng.integers(136, 257))
        n = int(rng.choice([rng.integers(600, 3000), rng.integers(3000, 40000), rng.integers(40000, 160000)]))
        kind = rng.integers(0, 5)
        if kind == 0:
            lg = (rng.integers(-14, 14, (rows, n)) / 2.0).astype(np.float32)
        elif kind == 1:
            lg = rng.normal(0, rng.choice([0.3, 2.0, 6.0]), (rows, n)).astype(np.float32)
        elif kind == 2:
            lg = np.round(rng.normal(0, 2, (rows, n)) * 4).astype(np.float32) / 4
        elif kind == 3:
            lg = synthetic.zipf_head_logits(rng, rows, n)
        else:
            lg = -np.abs(rng.normal(0, 3, (rows, n))).astype(np.float32) - 5.0
        if rng.random() < 0.3:
            lg[rng.random((rows, n)) < 0.2] = NEG
        if rng.random() < 0.3:
            lg[:, : n // 2] = NEG
        params = []
        for _ in range(rows):
            hist = rng.integers(0, n, int(rng.choice([0, 3, 40, 400]))).tolist()
            params.append(SamplingParams(
                Temperature=float(rng.choice([0.0, 0.3, 0.8, 1.0, 1.6])),
                TopK=int(rng.choice([1, 2, 7, 40, 64, 65, 300, 900, 1000, 2000])),
                TopP=float(rng.choice([1.0, 0.95, 0.7, 0.2])), MinP=float(rng.choice([0.0, 1e-4, 0.05, 0.4])),
                RepetitionPenalty=float(rng.choice([1.0, 1.2, 1.2, 0.8])),
                PresencePenalty=float(rng.choice([0.0, 0.5, 0.5, -0.5])),
                FrequencyPenalty=float(rng.choice([0.0, 0.2, 0.2, -0.1])), RepeatLastN=int(rng.choice([0, 5, 64])),
                PreviousTokens=hist))
        mask, act = _mask(rng, rows, n)
        u = rng.random(rows)
        if trial % 3 == 1:
            bits = synthetic.to_bf16_bits(lg)
            lg = synthetic.bf16_bits_to_f32(bits)
            dev = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
        else:
            dev = torch.from_numpy(lg).cuda()
        got = ctx.sample_batch(dev, params, u, mask, act)
        want = oracle_tokens(lg, params, u, mask, act)
        assert np.array_equal(got, want), (trial, rows, n, int(kind), str(dev.dtype), np.nonzero(got != want)[0][:4])


def test_random_speculative_verification_rows(ctx):
    import torch

    rng = np.random.default_rng(1003)
    for trial in range(150):
        rows, L, n = int(rng.integers(1, 6)), int(rng.integers(1, 5)), _width(rng, 20000)
        params = [_params(rng, n, True) for _ in range(rows)]
        draft = _logits(rng, rows * L, n).reshape(rows, L, n)
        target = np.empty((rows, L + 1, n), dtype=np.float32)
        target[:, :L] = draft + rng.normal(0, rng.choice([0.0, 0.2, 1.0]), (rows, L, n)).astype(np.float32)
        target[:, L] = _logits(rng, rows, n)
        filtered = rng.random() < 0.5       # the drafter's own filters shape q, or q is the plain softmax
        q = np.empty((rows, L, n), dtype=np.float32)
        toks = np.empty((rows, L), dtype=np.int32)
        for r in range(rows):
            for i in range(L):
                pp = params[r] if (filtered and params[r].Temperature > 0) else SamplingParams()
                toks[r, i], q[r, i] = orc.sample_with_distribution(draft[r, i], to_oracle(pp), orc.Rng(replay=[rng.random()]))
        u = rng.random((rows, L + 1))
        if rng.random() < 0.2:
            u[rng.integers(0, rows), rng.integers(0, L + 1)] = 0.0
        acc, out = ctx.spec_verify(torch.from_numpy(target).cuda(), torch.from_numpy(q).cuda(),
                                   torch.from_numpy(toks).cuda(), params, u)
        for r in range(rows):
            wa, wt = orc.spec_verify_row(target[r], q[r], toks[r], to_oracle(params[r]), orc.Rng(replay=u[r]))
            assert acc[r] == wa and list(out[r][:wa + 1]) == list(wt) and np.all(out[r][wa + 1:] == -1), \
                (trial, r, n, L, params[r], filtered)


def test_random_draws_residuals_and_mtp_rows(ctx):
    import torch

    rng = np.random.default_rng(1004)
    for trial in range(300):
        rows, n = int(rng.integers(1, 8)), _width(rng, 70000)
        z = _logits(rng, rows, n).astype(np.float64)
        z[~np.isfinite(z)] = -50
        p = np.exp(z - z.max(1, keepdims=True))
        p = (p / p.sum(1, keepdims=True)).astype(np.float32)
        z2 = z + rng.normal(0, rng.choice([0.0, 0.5, 2.0]), (rows, n))
        q = np.exp(z2 - z2.max(1, keepdims=True))
        q = (q / q.sum(1, keepdims=True)).astype(np.float32)
        if rng.random() < 0.3:
            p[rng.random((rows, n)) < 0.5] = 0.0
        u = rng.random(rows)
        if rng.random() < 0.2:
            u[0] = 0.0
        pd, qd = torch.from_numpy(p).cuda(), torch.from_numpy(q).cuda()
        got = ctx.sample_from_probs(pd, u)
        for r in range(rows):
            assert got[r] == orc.sample_from_probs(p[r], orc.Rng(replay=[u[r]])), (trial, r, n)
        got = ctx.resample_residual(pd, qd, u)
        for r in range(rows):
            assert got[r] == orc.resample_residual(p[r], q[r], orc.Rng(replay=[u[r]])), (trial, r, n)
        # MtpDecoder.AcceptDraft on random rows
        lg = _logits(rng, rows, n)
        lg[:, 0] = np.where(np.isfinite(lg).any(1), lg[:, 0], 0.0)
        am = np.array([orc.greedy(lg[r]) for r in range(rows)])
        draft = np.where(rng.random(rows) < 0.5, am, rng.integers(0, n, rows)).astype(np.int32)
        p_min = float(rng.choice([1.0, 0.5, 0.2, 0.001]))
        g_am, g_ok, g_pr = ctx.mtp_verify(torch.from_numpy(lg).cuda(), torch.from_numpy(draft).cuda(), p_min)
        for r in range(rows):
            ok, pr = orc.mtp_accept_draft(int(draft[r]), int(am[r]), lg[r], p_min)
            assert g_am[r] == am[r] and bool(g_ok[r]) == ok and abs(g_pr[r] - pr) <= 1e-5 * max(pr, 1e-30), (trial, r, n)
