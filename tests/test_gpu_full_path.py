"""GPU parity of the full-vocabulary path through the C ABI: the exact left-to-right running sum, the slow
path of Sampler.Sample, BuildFilteredDistribution, SampleWithDistribution, SampleFromProbs,
ResampleResidual, speculative verification and the MTP accept test, against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as orc
from opentail.stingray_amd import Sampler, SamplerContext, SamplingParams, pack_allow_mask, synthetic
from tests.helpers import DotnetRandom, ReplayRandom, hooks_lib, oracle_tokens, to_oracle

pytestmark = pytest.mark.gpu
NEG_INF = np.float32("-inf")


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _gpu_seq_sum(ctx, x, s0=0.0, target=float("nan")):
    import torch

    xd = _cuda(np.asarray(x, dtype=np.float32))
    s = torch.zeros(1, dtype=torch.float32, device="cuda")
    idx = torch.zeros(1, dtype=torch.int32, device="cuda")
    ctx._check(hooks_lib().sr_selftest_seqsum(ctx.h, C.c_void_p(xd.data_ptr()), len(x), s0, target,
                                        C.c_void_p(s.data_ptr()), C.c_void_p(idx.data_ptr())))
    ctx.synchronize()
    return np.float32(s.cpu().numpy()[0]), int(idx.cpu().numpy()[0])


def test_exact_running_sum_matches_the_left_to_right_loop(ctx):
    rng = np.random.default_rng(4)
    cases = []
    # softmax-like terms spanning many binades, in index order
    for n in (1, 5, 16, 17, 1000, 16384, 16385, 50000, 151936):
        z = rng.normal(0, 2.5, n)
        cases.append(np.exp(z - z.max()).astype(np.float32))
    # exact ties: terms that are exactly half an ulp of the running sum, with odd and even states
    t = np.full(4000, 2.0 ** -24, dtype=np.float32)
    cases.append(np.concatenate([[1.0], t]).astype(np.float32))
    cases.append(np.concatenate([[1.0 + 2.0 ** -23], t]).astype(np.float32))
    cases.append(np.concatenate([[1.0], np.tile([2.0 ** -24, 2.0 ** -23, 3 * 2.0 ** -25], 3000)]).astype(np.float32))
    # subnormals, zeros, a late large term, all-zero
    cases.append((rng.random(30000) * 1e-44).astype(np.float32))
    cases.append(np.concatenate([np.zeros(500), rng.random(20000) * 1e-39, [3.5], rng.random(9000)]).astype(np.float32))
    cases.append(np.zeros(20000, dtype=np.float32))
    # many binade crossings inside one tile
    cases.append((2.0 ** np.arange(-60, 40, 0.01)).astype(np.float32))
    cases.append(rng.random(100000).astype(np.float32))
    for x in cases:
        want, _ = orc.seq_sum(x)
        got, _ = _gpu_seq_sum(ctx, x)
        assert got.tobytes() == want.tobytes(), (len(x), got, want)
        # search: first index whose running sum reaches the target
        for frac in (0.0, 1e-9, 0.3, 0.77, 0.999999, 1.5):
            tgt = np.float32(frac * float(want))
            ws, wi = orc.seq_sum(x, 0.0, float(tgt))
            gs, gi = _gpu_seq_sum(ctx, x, 0.0, float(tgt))
            assert gi == wi, (len(x), frac, gi, wi)
    # a non-zero start
    x = cases[3]
    assert _gpu_seq_sum(ctx, x, 0.75)[0].tobytes() == orc.seq_sum(x, 0.75)[0].tobytes()


def test_sums_prepared_by_the_whole_device_do_not_depend_on_the_predictions(ctx):
    """The records of a row's segments are made for binades that approximate sums predict; the walk checks every
    record against the exact running sum and adds from the terms where one does not fit.  With predictions that are
    right, half, double and nothing of the truth, on rows that are ragged, misaligned, flat, peaked and sparse, the sum
    and the searches must be those of the left-to-right loop."""
    import torch

    rng = np.random.default_rng(11)
    rows = []
    for n in (1, 15, 1024, 1025, 4096, 5000, 40000, 151936, 262144):
        z = rng.normal(0, 2.5, n)
        rows.append(np.exp(z - z.max()).astype(np.float32))
    rows.append(rng.random(70001).astype(np.float32))                                    # flat: one binade for long
    big = np.exp(rng.normal(0, 1.0, 60000)).astype(np.float32)
    big[[100, 20000, 20001, 59999]] = [3.0e4, 7.0e5, 9.0e5, 2.0e7]                       # jumps over several binades
    rows.append(big)
    sparse = np.zeros(90000, dtype=np.float32)
    sparse[rng.integers(0, 90000, 300)] = rng.random(300).astype(np.float32)             # a residual-like row
    rows.append(sparse)
    rows.append(np.zeros(3000, dtype=np.float32))
    rows.append(np.concatenate([[1.0], np.full(50000, 2.0 ** -24)]).astype(np.float32))   # every add half way
    s = torch.zeros(2, dtype=torch.float32, device="cuda")
    idx = torch.zeros(2, dtype=torch.int32, device="cuda")
    H = hooks_lib()
    for x in rows:
        for shift in (0, 1):                                                             # rows that start off a 16-byte boundary
            buf = _cuda(np.concatenate([np.zeros(shift, np.float32), x]))
            ptr = buf.data_ptr() + 4 * shift
            want, _ = orc.seq_sum(x)
            for skew in (1.0, 0.5, 2.0, 0.0, 1.0 + 1e-4):
                for frac in (float("nan"), 0.0, 1e-9, 0.31, 0.77, 0.999999, 1.5):
                    tgt = np.float32(frac * float(want)) if frac == frac else np.float32("nan")
                    ctx._check(H.sr_selftest_segsum(ctx.h, C.c_void_p(ptr), len(x), skew, float(tgt),
                                                    C.c_void_p(s.data_ptr()), C.c_void_p(idx.data_ptr())))
                    ctx.synchronize()
                    gs, gi = s.cpu().numpy(), idx.cpu().numpy()
                    assert gs[0].tobytes() == want.tobytes(), (len(x), shift, skew, gs[0], want)
                    if frac == frac:
                        ws, wi = orc.seq_sum(x, 0.0, float(tgt))
                        assert gi[0] == wi and gi[1] == wi, (len(x), shift, skew, frac, gi, wi)
                        if wi >= 0:  # (the walk that searches hands back the running sum at the term it stops at)
                            at = orc.seq_sum(x[: wi + 1])[0]
                            assert gs[1].tobytes() == at.tobytes(), (len(x), skew, frac, gs[1], at)


def _check_rows(ctx, logits, params, uniforms, allow_mask=None, mask_active=None):
    got, flags = ctx.sample_batch(_cuda(logits), params, uniforms, allow_mask, mask_active, return_flags=True)
    want = oracle_tokens(logits, params, uniforms, allow_mask, mask_active)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"rows {bad[:8]} differ: gpu {got[bad[:8]]} oracle {want[bad[:8]]} flags {flags[bad[:8]]}"
    return flags


def _check_distribution(ctx, logits, params, allow_mask=None, mask_active=None):
    got = ctx.build_distribution(_cuda(logits), params, None, allow_mask, mask_active).cpu().numpy()
    for r, p in enumerate(params):
        row = logits[r]
        if allow_mask is not None and (mask_active is None or mask_active[r]):
            row = orc.apply_allow_mask(row, allow_mask[r])
        want = orc.build_filtered_distribution(row, to_oracle(p))
        assert np.array_equal(got[r] > 0, want > 0), f"row {r}: support differs"
        nz = want > 0
        assert np.allclose(got[r][nz], want[nz], rtol=1e-5, atol=0), f"row {r}"
        # the arithmetic is the reference's, so the bits agree as well
        assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32)), f"row {r}: bits differ"


def test_slow_path_small_rows_every_stage(ctx):
    rng = np.random.default_rng(31)
    for trial in range(25):
        rows = int(rng.integers(1, 7))
        n = int(rng.integers(1, 900))
        logits = (rng.integers(-14, 14, (rows, n)) / 2.0).astype(np.float32)
        logits[rng.random((rows, n)) < 0.15] = NEG_INF
        params = []
        for _ in range(rows):
            hist = rng.integers(-3, n + 3, int(rng.integers(0, 12))).tolist()
            bias = {int(rng.integers(-2, n + 2)): float(rng.normal(0, 3)) for _ in range(int(rng.integers(0, 4)))}
            params.append(SamplingParams(
                Temperature=float(rng.choice([0.0, 0.5, 1.0, 1.7])), TopK=int(rng.choice([0, 0, 3, n + 5])),
                TopP=float(rng.choice([1.0, 0.9, 0.5])), MinP=float(rng.choice([0.0, 0.05, 0.3])),
                RepetitionPenalty=float(rng.choice([1.0, 1.3, 0.8])), PresencePenalty=float(rng.choice([0.0, 0.4, -0.3])),
                FrequencyPenalty=float(rng.choice([0.0, 0.25])), RepeatLastN=int(rng.choice([0, 3, 64])),
                PreviousTokens=hist, LogitBias=bias or None))
        u = rng.random(rows)
        _check_rows(ctx, logits, params, u)
        _check_distribution(ctx, logits, params)


def test_reference_known_answers_slow_path():
    # SamplerTests.cs: logit bias, BuildFilteredDistribution, SampleWithDistribution, ResampleResidual
    r = DotnetRandom(42)
    assert 0 not in {Sampler.Sample([10, 1, 1, 1], SamplingParams(LogitBias={0: -100.0}), r) for _ in range(100)}
    r = DotnetRandom(42)
    assert {Sampler.Sample([0, 0, 0, 0], SamplingParams(LogitBias={2: 100.0}), r) for _ in range(100)} == {2}
    assert 0 <= Sampler.Sample([1, 2, 3], SamplingParams(LogitBias={999: 100.0, -1: 100.0}), DotnetRandom(42)) <= 2
    assert Sampler.Sample([10, 9.8], SamplingParams(Temperature=0.0, PresencePenalty=1.0, PreviousTokens=[0])) == 1
    probs = Sampler.BuildFilteredDistribution([1.0, 2.0, 3.0, 0.0], SamplingParams()).cpu().numpy()
    e = np.exp(np.array([1.0, 2.0, 3.0, 0.0]) - 3.0)
    assert np.allclose(probs, e / e.sum(), atol=5e-6) and abs(probs.sum() - 1) < 5e-6
    probs = Sampler.BuildFilteredDistribution([1, 9, 3, 2], SamplingParams(Temperature=0.0)).cpu().numpy()
    assert probs[1] == 1.0 and probs[0] + probs[2] + probs[3] == 0.0
    probs = Sampler.BuildFilteredDistribution([5, 4, 3, 2, 1], SamplingParams(TopK=2)).cpu().numpy()
    assert probs[0] > 0 and probs[1] > 0 and probs[2:].sum() == 0 and abs(probs.sum() - 1) < 5e-6
    with pytest.raises(ValueError):
        Sampler.BuildFilteredDistribution([1, 2, 3], SamplingParams(), probs_len=4)
    tok, probs = Sampler.SampleWithDistribution([0, 12, 0, 0], SamplingParams(Temperature=0.1), DotnetRandom(7))
    assert tok == 1 and probs[1] > 0.99
    r = DotnetRandom(3)
    for _ in range(50):
        assert Sampler.ResampleResidual([0, .5, .5, 0], [0, 1.0, 0, 0], r) == 2
    assert 0 <= Sampler.ResampleResidual([.25] * 4, [.25] * 4, DotnetRandom(5)) < 4
    with pytest.raises(ValueError):
        Sampler.ResampleResidual([0.0] * 4, [0.0] * 3, DotnetRandom(1))
    with pytest.raises(TypeError):
        Sampler.SampleFromProbs([0.5, 0.5], None)
    # draw quirks: u == 0 -> index 0 even when probs[0] == 0; rounding fallback -> last index
    assert Sampler.SampleFromProbs([0.0, 1.0], ReplayRandom([0.0])) == 0
    assert Sampler.SampleFromProbs([0.25, 0.25, 0.25], ReplayRandom([0.99])) == 2
    # fully masked row -> uniform over all tokens
    assert Sampler.Sample([NEG_INF] * 4, SamplingParams(), ReplayRandom([0.6])) == 2


def test_config2_shape(ctx):
    w = synthetic.config2(rows=8)
    flags = _check_rows(ctx, w.logits, w.params, w.uniforms)
    assert np.all(flags & 4)
    _check_distribution(ctx, w.logits[:2], w.params[:2])


def test_config4_shape_masks_and_large_nuclei(ctx):
    w = synthetic.config4(rows=12)
    _check_rows(ctx, w.logits, w.params, w.uniforms, w.allow_mask, w.mask_active)
    sampled = [i for i in range(12) if w.params[i].Temperature > 0][:3]
    _check_distribution(ctx, w.logits[sampled], [w.params[i] for i in sampled], w.allow_mask[sampled],
                        w.mask_active[sampled])


def test_top_k_above_the_kernel_limit_goes_down_the_slow_path_of_the_oracle_too(ctx):
    # TopK >= vocab disables top-k in the reference (Sampler.cs:38,71); huge LogitBias rows keep ties at the k-th value
    rng = np.random.default_rng(2)
    logits = rng.normal(0, 1.5, (3, 5000)).astype(np.float32)
    logits[1, 100:140] = 3.25   # ties at the k-th value survive ApplyTopK
    params = [SamplingParams(TopK=5000), SamplingParams(TopK=20, LogitBias={-1: 0.0}, TopP=0.9),
              SamplingParams(TopK=7, LogitBias={5: 2.0}, MinP=0.01, Temperature=0.7)]
    _check_rows(ctx, logits, params, rng.random(3))
    _check_distribution(ctx, logits, params)


def test_sample_from_probs_and_resample_residual_rows(ctx):
    rng = np.random.default_rng(9)
    V = 40_000
    z = rng.normal(0, 2, (6, V))
    p = (np.exp(z) / np.exp(z).sum(1, keepdims=True)).astype(np.float32)
    z2 = z + rng.normal(0, 0.5, (6, V))
    q = (np.exp(z2) / np.exp(z2).sum(1, keepdims=True)).astype(np.float32)
    q[4] = p[4]                      # empty residual -> falls back to sampling p
    u = rng.random(6)
    u[5] = 0.0
    got = ctx.sample_from_probs(_cuda(p), u)
    for r in range(6):
        assert got[r] == orc.sample_from_probs(p[r], orc.Rng(replay=[u[r]]))
    got = ctx.resample_residual(_cuda(p), _cuda(q), u)
    for r in range(6):
        assert got[r] == orc.resample_residual(p[r], q[r], orc.Rng(replay=[u[r]])), r


def _spec_case(rows, L, V, params, seed, filtered_q):
    rng = np.random.default_rng(seed)
    draft = synthetic.zipf_head_logits(rng, rows * L, V).reshape(rows, L, V)
    target = np.empty((rows, L + 1, V), dtype=np.float32)
    target[:, :L] = draft + rng.normal(0, 0.5, (rows, L, V)).astype(np.float32)
    target[:, L] = synthetic.zipf_head_logits(rng, rows, V)
    q = np.empty((rows, L, V), dtype=np.float32)
    toks = np.empty((rows, L), dtype=np.int32)
    for r in range(rows):
        for i in range(L):
            t, d = orc.sample_with_distribution(draft[r, i], to_oracle(params[r] if filtered_q else SamplingParams()),
                                                orc.Rng(replay=[rng.random()]))
            q[r, i], toks[r, i] = d, t
    return target, q, toks, rng.random((rows, L + 1))


def _check_spec(ctx, target, q, toks, params, u):
    acc, out = ctx.spec_verify(_cuda(target), _cuda(q), _cuda(toks), params, u)
    for r in range(target.shape[0]):
        wa, wt = orc.spec_verify_row(target[r], q[r], toks[r], to_oracle(params[r]), orc.Rng(replay=u[r]))
        assert acc[r] == wa, (r, acc[r], wa)
        assert list(out[r][: wa + 1]) == list(wt), (r, out[r], wt)
        assert np.all(out[r][wa + 1:] == -1)


def test_speculative_verification_rows(ctx):
    V, L = 20_000, 4
    # unfiltered p and q (the benchmark's choice), the CLI defaults, and the looser p-min accept
    p1 = [SamplingParams() for _ in range(6)]
    _check_spec(ctx, *_spec_case(6, L, V, p1, 1, False)[:3], p1, _spec_case(6, L, V, p1, 1, False)[3])
    p2 = [SamplingParams(Temperature=0.7, TopK=40, TopP=0.95, MinP=0.05) for _ in range(6)]
    t, q, k, u = _spec_case(6, L, V, p2, 2, True)
    _check_spec(ctx, t, q, k, p2, u)
    p3 = [SamplingParams(Temperature=0.8, SpecDraftPMin=0.05) for _ in range(4)] + [SamplingParams(Temperature=0.0)]
    t, q, k, u = _spec_case(5, L, V, p3, 3, True)
    _check_spec(ctx, t, q, k, p3, u)


def test_corrections_drawn_at_both_ends_of_the_residual(ctx):
    # The residual row of a row's first rejected position is written ahead of the verifier and read back by it.  Rows
    # whose lengths leave the distributions at any alignment; a first uniform just below 1 (rejected unless the ratio is
    # 1) or 0 (accepted wherever p > 0), so that rejections fall on the first and on later positions; corrections drawn
    # with a uniform of 0 (the first positive residual), of the smallest positive double and of nearly 1 (the last
    # entries of the running sum).
    for V, seed in ((20_000, 11), (20_001, 12), (20_003, 13)):
        rows, L = 8, 3
        params = [SamplingParams() if r % 2 == 0 else SamplingParams(Temperature=0.8, TopK=60, TopP=0.9) for r in range(rows)]
        t, q, k, u = _spec_case(rows, L, V, params, seed, True)
        for first, corr in ((0.99999994, 0.0), (0.99999994, 0.99999994), (0.99999994, 5e-324), (0.0, 0.99999994), (0.3, 0.0)):
            uu = u.copy()
            uu[:, 0] = first
            uu[:, 1:] = np.where(np.arange(rows)[:, None] % 3 == 0, corr, uu[:, 1:])  # every third row: all later draws
            uu[1::3, 1] = corr                                                       # the others: the draw behind position 0
            _check_spec(ctx, t, q, k, params, uu)


def test_verification_after_tokens_were_appended_to_the_batch(ctx):
    # The verifier copies the batch's row descriptors on the device: rows with penalties whose histories grew by
    # sr_batch_append_tokens (in place, no new upload) must be verified with the histories as they are now.
    import torch

    V, L, rows = 20_000, 3, 6
    rng = np.random.default_rng(515)
    hist = [rng.integers(0, V, 40).tolist() for _ in range(rows)]
    def params_of(h):
        return [SamplingParams(Temperature=0.9, TopP=0.95, FrequencyPenalty=0.4, PresencePenalty=0.2, RepetitionPenalty=1.1,
                               PreviousTokens=list(h[r])) for r in range(rows)]
    t, q, k, u = _spec_case(rows, L, V, params_of(hist), 21, True)
    batch = ctx.new_batch().upload(params_of(hist), V, u)
    for step in range(3):
        new = rng.integers(0, V, rows)
        for r in range(rows):
            hist[r].append(int(new[r]))
        u = rng.random((rows, L + 1))
        batch.append_tokens(new, u)
    acc = torch.zeros(rows, dtype=torch.int32, device="cuda")
    out = torch.zeros((rows, L + 1), dtype=torch.int32, device="cuda")
    ctx.spec_verify_launch(batch, _cuda(t), _cuda(q), _cuda(k), acc, out)
    ctx.synchronize()
    acc, out = acc.cpu().numpy(), out.cpu().numpy()
    now = params_of(hist)
    for r in range(rows):
        wa, wt = orc.spec_verify_row(t[r], q[r], k[r], to_oracle(now[r]), orc.Rng(replay=u[r]))
        assert acc[r] == wa and list(out[r][: wa + 1]) == list(wt), (r, acc[r], wa, out[r], wt)
    batch.close()


def test_drafts_from_prompt_lookup_take_the_p_min_rule_whatever_p_min_is(ctx):
    # usedPld (SpeculativeDecoder.cs:488-501, 538-552): no draft distributions exist; accept iff px >= SpecDraftPMin or the
    # draft is the argmax, a rejection draws from p.  Rows of both kinds in one launch; then lookup rows alone with no q.
    V, L = 20_000, 5
    kinds = [SamplingParams(SpecDraftFromLookup=True),
             SamplingParams(Temperature=0.7, TopK=40, TopP=0.95, SpecDraftFromLookup=True),
             SamplingParams(Temperature=0.8, SpecDraftPMin=0.05, SpecDraftFromLookup=True),
             SamplingParams(Temperature=0.0, SpecDraftFromLookup=True),
             SamplingParams(Temperature=0.9, TopP=0.9)]
    params = [kinds[r % len(kinds)] for r in range(10)]
    t, q, k, u = _spec_case(10, L, V, params, 5, True)
    rng = np.random.default_rng(6)
    for r in range(10):                                           # lookup drafts: a mix of likely and arbitrary continuations
        if params[r].SpecDraftFromLookup:
            q[r] = np.nan                                         # must not be read
            for i in range(L):
                k[r, i] = int(np.argmax(t[r, i])) if rng.random() < 0.6 else int(rng.integers(0, V))
    _check_spec(ctx, t, q, k, params, u)
    only = [p for p in params if p.SpecDraftFromLookup]
    idx = [r for r, p in enumerate(params) if p.SpecDraftFromLookup]
    acc, out = ctx.spec_verify(_cuda(t[idx]), None, _cuda(k[idx]), only, u[idx])
    for j, r in enumerate(idx):
        wa, wt = orc.spec_verify_row(t[r], q[r], k[r], to_oracle(params[r]), orc.Rng(replay=u[r]))
        assert acc[j] == wa and list(out[j][: wa + 1]) == list(wt), r
    with pytest.raises(TypeError):                                # a row under the ratio test needs q (a null argument)
        ctx.spec_verify(_cuda(t), None, _cuda(k), params, u)


def test_draft_ids_outside_the_vocabulary_end_their_row(ctx):
    # SpeculativeDecoder.cs:536 indexes pDist[x_i]: an id outside the vocabulary throws there.  The device never
    # dereferences it: the row ends at that position with -1 in place of the correction token.
    V, L = 5_000, 4
    params = [SamplingParams() for _ in range(4)]
    t, q, k, u = _spec_case(4, L, V, params, 9, False)
    u[:, :L] = 0.0            # every in-range draft is accepted (u < a for any a > 0)
    k[0, 2] = V               # one past the end
    k[1, 0] = -1
    k[2, 3] = 2 ** 31 - 1
    acc, out = ctx.spec_verify(_cuda(t), _cuda(q), _cuda(k), params, u)
    for r in range(4):
        wa, wt = orc.spec_verify_row(t[r], q[r], k[r], to_oracle(params[r]), orc.Rng(replay=u[r]))
        assert acc[r] == wa and list(out[r][: wa + 1]) == list(wt), (r, acc[r], wa, out[r], wt)
    assert (acc[0], out[0][2]) == (2, -1) and (acc[1], out[1][0]) == (0, -1) and (acc[2], out[2][3]) == (3, -1)
    assert acc[3] == L and out[3][L] >= 0


def test_reference_distribution_preservation_invariant(ctx):
    # SpeculativeSamplingTests.cs:21-50 at a GPU-sized batch: with fixed target/draft rows the emitted
    # histogram of (accepted drafts + correction) follows softmax(target) regardless of the draft.
    P_T = np.array([0.2, 2.5, 0.1, 1.0, 0.3, 1.8, 0.0, 0.5], dtype=np.float32)
    Q_D = np.array([2.0, 0.1, 1.5, 0.2, 1.0, 0.0, 2.2, 0.3], dtype=np.float32)
    rows, L = 4096, 3
    rng = DotnetRandom(12345)
    p = SamplingParams()
    q1 = orc.build_filtered_distribution(Q_D, to_oracle(p))
    qc = np.cumsum(q1)
    toks = np.searchsorted(qc, [rng.NextDouble() for _ in range(rows * L)]).clip(0, 7).astype(np.int32).reshape(rows, L)
    target = np.tile(P_T, (rows, L + 1, 1))
    q = np.tile(q1, (rows, L, 1))
    u = np.array([rng.NextDouble() for _ in range(rows * (L + 1))]).reshape(rows, L + 1)
    acc, out = ctx.spec_verify(_cuda(target), _cuda(q), _cuda(toks), [p] * rows, u)
    # first emitted token of every step is distributed as softmax(target)
    first = np.array([out[r][0] for r in range(rows)])
    e = np.exp(P_T - P_T.max())
    assert np.abs(np.bincount(first, minlength=8) / rows - e / e.sum()).max() < 0.03
    assert 0.01 < acc.mean() / L < 0.99


def test_mtp_accept_draft(ctx):
    import torch

    rng = np.random.default_rng(6)
    V = 50_000
    logits = rng.normal(0, 2, (8, V)).astype(np.float32)
    am = logits.argmax(1)
    draft = np.array([am[0], 5, am[2], 7, 11, am[5], 13, 17], dtype=np.int32)
    logits[3, 7] = logits[3].max() - 0.2     # high-probability non-argmax draft
    for p_min in (1.0, 0.2, 0.001):
        g_am, g_ok, g_pr = ctx.mtp_verify(_cuda(logits), torch.from_numpy(draft).cuda(), p_min)
        for r in range(8):
            ok, pr = orc.mtp_accept_draft(int(draft[r]), int(am[r]), logits[r], p_min)
            assert g_am[r] == am[r] and bool(g_ok[r]) == ok
            assert abs(g_pr[r] - pr) <= 1e-5 * max(pr, 1e-30)


def test_nucleus_finished_from_the_list_of_its_members(ctx):
    # Rows whose nucleus closes inside the kernel are normalised and drawn from the list of their members, not
    # by passes over the row: vocabulary lengths around multiples of 8 (the overlapped tail of the eight-lane
    # sum), members inside that tail, a uniform of exactly 0 (index 0 wins whatever it holds) and one just below 1.
    rng = np.random.default_rng(37)
    for n in (8, 9, 15, 16, 17, 23, 1000, 1001, 1007, 4099):
        rows = 6
        logits = rng.normal(0, 2.0, (rows, n)).astype(np.float32)
        logits[:, n - 1] += 6.0                               # a member in the last, ragged vector
        logits[1, 0] = NEG_INF                                # index 0 outside the nucleus
        logits[2, : n // 2] = NEG_INF
        params = [SamplingParams(Temperature=float(t), TopK=0, TopP=float(p), MinP=float(mp))
                  for t, p, mp in zip([1.0, 0.7, 1.3, 1.0, 0.9, 2.0], [0.9, 0.5, 0.95, 0.999, 0.3, 0.97],
                                      [0.0, 0.0, 0.05, 0.0, 0.02, 0.0])]
        for u in ([0.0] * rows, [0.99999994] * rows, rng.random(rows).tolist()):
            _check_rows(ctx, logits, params, u)
        _check_distribution(ctx, logits, params)


def test_nuclei_of_tens_of_thousands_of_members_take_the_device_wide_sort(ctx):
    # Flat rows: the top-p nucleus does not close among the 4,096 largest probabilities, so the survivors are sorted
    # device-wide (stable: equal probabilities in index order) and cut by the exact search.  Distributions must agree
    # bit for bit -- the support is what the cut decides -- and so must the draws.
    rng = np.random.default_rng(77)
    V = 40_000
    logits = np.stack([
        rng.normal(0, 0.5, V),                               # ~ 80 % of the vocabulary inside a 0.95 nucleus
        np.round(rng.normal(0, 0.7, V) * 8) / 8,             # a coarse grid: thousands of equal probabilities at the cut
        rng.normal(0, 0.3, V),
        rng.normal(0, 3.0, V),                               # a sharp row in the same batch: closes inside the kernel
    ]).astype(np.float32)
    params = [SamplingParams(Temperature=1.0, TopP=0.95), SamplingParams(Temperature=0.8, TopP=0.9),
              SamplingParams(Temperature=1.3, TopP=0.5), SamplingParams(Temperature=1.0, TopP=0.95)]
    _check_distribution(ctx, logits, params)
    for _ in range(4):
        _check_rows(ctx, logits, params, rng.random(4))
    # greedy rows in the same batch of distributions: their (empty) sort segments lie between the others'
    mixed = [SamplingParams(Temperature=0.0), params[0], SamplingParams(Temperature=0.0, TopP=0.5), params[1]]
    _check_distribution(ctx, logits[[3, 0, 2, 1]], mixed)
    # the same under dense allow-masks and next to rows of the other paths
    allowed = rng.random((4, V)) < np.array([0.6, 0.9, 0.5, 1.0])[:, None]
    mask = pack_allow_mask(allowed)
    active = np.ones(4, dtype=np.uint8)
    _check_distribution(ctx, logits, params, mask, active)
    _check_rows(ctx, logits, params, rng.random(4), mask, active)


def test_rows_that_only_top_p_cuts_at_every_size_of_nucleus(ctx):
    # A sampled row with top-p alone is cut without being rewritten: a histogram of its exponentials bounds the slabs
    # that are sorted, the members come from reads of the row in index order.  Nuclei that close in the first slab,
    # that take several slabs (their members then pass through the kernel a block at a time), that are larger than the
    # walk goes (device-wide sort), equal probabilities at the cut (the first ones by index stay), under allow-masks,
    # with uniforms at both ends of the range (a draw near 1 lands among the last members).
    rng = np.random.default_rng(4242)
    V = synthetic.QWEN_VOCAB
    logits = np.stack([
        rng.normal(0, 3.0, V),                               # sharp: a few hundred members
        rng.normal(0, 1.6, V),                               # some thousands
        rng.normal(0, 1.2, V),                               # several slabs
        np.round(rng.normal(0, 1.2, V) * 4) / 4,             # ... with hundreds of equal probabilities at the cut
        np.round(rng.normal(0, 2.5, V) * 2) / 2,             # equal probabilities at a cut inside the first slab
        rng.normal(0, 0.4, V),                               # most of the vocabulary: beyond the walk
    ]).astype(np.float32)
    params = [SamplingParams(Temperature=1.0, TopP=0.95), SamplingParams(Temperature=1.0, TopP=0.9),
              SamplingParams(Temperature=1.0, TopP=0.9), SamplingParams(Temperature=0.9, TopP=0.8),
              SamplingParams(Temperature=1.1, TopP=0.7), SamplingParams(Temperature=1.0, TopP=0.95)]
    rows = len(params)
    for u in ([0.99999994] * rows, [0.0] * rows, [0.9995] * rows, rng.random(rows).tolist(), rng.random(rows).tolist()):
        _check_rows(ctx, logits, params, u)
    # the same rows as distributions (written rows: the walk by slabs of the general way, its first slab ended by the
    # bound on its mass)
    _check_distribution(ctx, logits, params)
    allowed = rng.random((rows, V)) < np.array([0.5, 0.3, 0.9, 0.7, 0.2, 0.8])[:, None]
    mask = pack_allow_mask(allowed)
    active = np.ones(rows, dtype=np.uint8)
    for u in ([0.99999994] * rows, rng.random(rows).tolist()):
        _check_rows(ctx, logits, params, u, mask, active)
    # shorter rows, lengths off the multiples of 4 and 8
    for n in (4097, 20_001, 65_539):
        sub = np.ascontiguousarray(logits[:, :n])
        for u in ([0.99999994] * rows, rng.random(rows).tolist()):
            _check_rows(ctx, sub, params, u)


def test_top_p_rows_in_a_batch_of_more_rows_than_compute_units(ctx):
    """With a compute unit per row the row kernel walks a nucleus in slabs of 8,192 entries, with more rows (two
    workgroups share a compute unit's shared memory) in slabs of 4,096: the same rows both ways."""
    rng = np.random.default_rng(4243)
    V = 65_536
    kinds = np.stack([rng.normal(0, 3.0, V), rng.normal(0, 1.6, V), rng.normal(0, 1.2, V), rng.normal(0, 1.0, V),
                      np.round(rng.normal(0, 1.2, V) * 4) / 4, rng.normal(0, 0.4, V)]).astype(np.float32)
    p6 = [SamplingParams(Temperature=1.0, TopP=0.95), SamplingParams(Temperature=1.0, TopP=0.9),
          SamplingParams(Temperature=1.0, TopP=0.9), SamplingParams(Temperature=1.0, TopP=0.93),
          SamplingParams(Temperature=0.9, TopP=0.8), SamplingParams(Temperature=1.0, TopP=0.95)]
    u6 = rng.random(6)
    few = _check_rows(ctx, kinds, p6, u6)
    reps = 44                                             # 264 rows: more than the device has compute units
    logits = np.tile(kinds, (reps, 1))
    params = p6 * reps
    u = np.tile(u6, reps)
    got = ctx.sample_batch(_cuda(logits), params, u)
    want = oracle_tokens(kinds, p6, u6)
    assert np.array_equal(got, np.tile(want, reps))
    assert few is not None


def test_final_normalize_of_long_rows_at_ragged_lengths(ctx):
    # The eight-lane sum of a long row is taken by one wave per lane over blocks of 8,192 entries; lengths that leave
    # one to seven entries for the overlapped last vector, a last block that is nearly empty or nearly full, rows
    # that top-k cuts to a few entries and rows that keep half of theirs.  The distributions must agree bit for bit.
    rng = np.random.default_rng(909)
    for n in (16_384, 16_385, 16_391, 24_575, 24_577, 65_539, 151_937):
        logits = rng.normal(0, 2.0, (4, n)).astype(np.float32)
        params = [SamplingParams(Temperature=1.0, TopK=40), SamplingParams(Temperature=0.8, TopK=3000),
                  SamplingParams(Temperature=1.2, TopK=5000, TopP=0.99),
                  SamplingParams(Temperature=1.0, TopK=n // 2 if n < 30_000 else 1000, MinP=1e-6)]
        _check_distribution(ctx, logits, params)
        _check_rows(ctx, logits, params, rng.random(4))


def test_top_p_over_thousands_of_equal_logits(ctx):
    # Logits on a grid (as bf16 gives them) put thousands of entries on one probability.  The walk through the nucleus
    # takes such a value as a run of equal terms -- no order among them is needed for the running sum -- and if the cut
    # falls inside the run, the members are its first entries by index.  Rows: a coarse grid (one value per crowded
    # position of the histogram), a cluster of three values so close that they share a position, bf16-rounded logits
    # at a high temperature; uniforms at both ends, and the same under allow-masks.
    rng = np.random.default_rng(2024)
    V = synthetic.QWEN_VOCAB
    grid = np.round(rng.normal(0, 1.0, V) * 8) / 8
    cluster = rng.normal(0, 2.0, V)
    pick = rng.random(V) < 0.6
    cluster[pick] = rng.choice(np.array([1.0, 1.002, 1.004]), size=int(pick.sum()))
    bf = synthetic.bf16_bits_to_f32(synthetic.to_bf16_bits(rng.normal(0, 1.5, (1, V)).astype(np.float32)))[0]
    logits = np.stack([grid, cluster, cluster, bf, grid]).astype(np.float32)
    params = [SamplingParams(Temperature=1.0, TopP=0.9), SamplingParams(Temperature=1.0, TopP=0.6),
              SamplingParams(Temperature=0.8, TopP=0.95), SamplingParams(Temperature=1.3, TopP=0.9),
              SamplingParams(Temperature=2.0, TopP=0.5)]
    rows = len(params)
    for u in ([0.99999994] * rows, [0.0] * rows, rng.random(rows).tolist(), rng.random(rows).tolist()):
        _check_rows(ctx, logits, params, u)
    allowed = rng.random((rows, V)) < np.array([0.5, 0.9, 0.3, 0.8, 0.7])[:, None]
    mask = pack_allow_mask(allowed)
    active = np.ones(rows, dtype=np.uint8)
    for u in ([0.99999994] * rows, rng.random(rows).tolist()):
        _check_rows(ctx, logits, params, u, mask, active)


def _strided(a, pad, dtype=None):
    """The rows of `a` inside a wider device tensor: row stride = a.shape[1] + pad elements."""
    import torch

    wide = np.zeros((a.shape[0], a.shape[1] + pad), dtype=a.dtype)
    wide[:, :a.shape[1]] = a
    t = torch.from_numpy(wide)
    if dtype is not None:
        t = t.view(dtype)
    return t.cuda()[:, :a.shape[1]]


def test_bf16_and_unaligned_rows_on_the_full_path(ctx):
    import torch

    rng = np.random.default_rng(78)
    # (rows of 4,096 entries and more that start on 16-byte boundaries have their sums prepared by the whole device, in
    # segments of 1,024: 40,968 and 50,004 end in a ragged segment, 50,004 is aligned as fp32 only, 8,200 + 8 by its padding)
    for V, pad in [(10_007, 3), (4_096, 0), (33_001, 6), (40_968, 0), (50_004, 0), (8_200, 8)]:
        rows = 8
        f32 = rng.normal(0, 2.0, (rows, V)).astype(np.float32)
        bf = (f32.view(np.uint32) >> 16).astype(np.uint16)
        exact = (bf.astype(np.uint32) << 16).view(np.float32)             # what the bf16 tensor holds
        allowed = rng.random((rows, V)) < 0.7
        mask = pack_allow_mask(allowed)
        active = np.array([0, 1, 0, 1, 0, 0, 1, 0], dtype=np.uint8)
        hist = rng.integers(0, V, 200).tolist()
        params = [SamplingParams(Temperature=0.9, TopP=0.9),                                   # nothing edits the row
                  SamplingParams(Temperature=1.0, TopP=0.95, MinP=0.001),
                  SamplingParams(Temperature=0.7, LogitBias={5: 3.0, V - 1: -2.0, 17: 1.5}, TopK=50, TopP=0.9),
                  SamplingParams(Temperature=1.2, RepetitionPenalty=1.3, FrequencyPenalty=0.2, PreviousTokens=hist),
                  SamplingParams(Temperature=0.0, LogitBias={3: 100.0}),                        # greedy ignores the bias
                  SamplingParams(Temperature=1.0),
                  SamplingParams(Temperature=0.8, MinP=0.02, PresencePenalty=0.5, PreviousTokens=hist[:40]),   # min-p alone, edits
                  SamplingParams(Temperature=0.6, TopP=0.97, FrequencyPenalty=0.3, PreviousTokens=hist[:90])]  # top-p alone, edits
        for logits, dev in [(exact, _strided(bf.view(np.int16), pad, torch.bfloat16)), (f32, _strided(f32, pad))]:
            for _ in range(2):
                u = rng.random(rows)
                got, flags = ctx.sample_batch(dev, params, u, mask, active, return_flags=True)
                assert np.array_equal(got, oracle_tokens(logits, params, u, mask, active)), (V, pad, dev.dtype)
            got = ctx.build_distribution(dev, params, None, mask, active).cpu().numpy()
            for r, p in enumerate(params):
                row = orc.apply_allow_mask(logits[r], mask[r]) if active[r] else logits[r]
                want = orc.build_filtered_distribution(row, to_oracle(p))
                assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32)), (V, pad, dev.dtype, r)


def test_rows_without_a_finite_logit_and_rows_with_a_nan(ctx):
    # Softmax falls back to the uniform distribution when the maximum is -inf or NaN (Sampler.cs:452-458)
    rng = np.random.default_rng(79)
    V = 3_000
    logits = rng.normal(0, 1.0, (4, V)).astype(np.float32)
    logits[0, :] = NEG_INF
    logits[1, 1234] = np.float32("nan")
    allowed = np.ones((4, V), dtype=bool)
    allowed[2, :] = False                                                 # a dead mask: every id forbidden
    mask = pack_allow_mask(allowed)
    active = np.array([0, 0, 1, 0], dtype=np.uint8)
    params = [SamplingParams(Temperature=1.0, TopP=0.9), SamplingParams(Temperature=0.8),
              SamplingParams(Temperature=1.0, MinP=0.1), SamplingParams(Temperature=1.0, TopP=0.9)]
    for _ in range(4):
        u = rng.random(4)
        got, flags = ctx.sample_batch(_cuda(logits), params, u, mask, active, return_flags=True)
        assert np.array_equal(got, oracle_tokens(logits, params, u, mask, active)), (got, flags)
        assert np.all(flags[:3] & 8) and not flags[3] & 8
    _check_distribution(ctx, logits, params, mask, active)


def test_sample_with_distribution_rows(ctx):
    rng = np.random.default_rng(80)
    V, rows = 20_000, 5
    logits = rng.normal(0, 2.0, (rows, V)).astype(np.float32)
    params = [SamplingParams(Temperature=1.0), SamplingParams(Temperature=0.7, TopK=40, TopP=0.9),
              SamplingParams(Temperature=0.0), SamplingParams(Temperature=1.1, MinP=0.02),
              SamplingParams(Temperature=0.9, TopP=0.8, RepetitionPenalty=1.2, PreviousTokens=rng.integers(0, V, 64).tolist())]
    u = rng.random(rows)
    toks, probs = ctx.sample_with_distribution(_cuda(logits), params, u)
    probs = probs.cpu().numpy()
    for r, p in enumerate(params):
        t, d = orc.sample_with_distribution(logits[r], to_oracle(p), orc.Rng(replay=[u[r]]))
        assert toks[r] == t, r
        assert np.array_equal(probs[r].view(np.uint32), np.asarray(d, dtype=np.float32).view(np.uint32)), r


def test_min_p_rows_with_few_and_with_thousands_of_survivors(ctx):
    # min-p survivors are listed while the row is read: rows with up to 1,024 of them are finished from the list
    # (sampled rows are then not written at all), rows with more take the passes over the row
    rng = np.random.default_rng(81)
    V = 50_000
    logits = rng.normal(0, 1.5, (6, V)).astype(np.float32)
    params = [SamplingParams(Temperature=1.0, MinP=0.05), SamplingParams(Temperature=0.8, MinP=0.05, TopP=0.9),
              SamplingParams(Temperature=1.0, MinP=1e-3), SamplingParams(Temperature=1.2, MinP=1e-3, TopP=0.95),
              SamplingParams(Temperature=1.0, MinP=1e-5, TopP=0.9), SamplingParams(Temperature=1.5, MinP=1e-6)]
    _check_distribution(ctx, logits, params)
    for _ in range(4):
        _check_rows(ctx, logits, params, rng.random(6))
    toks, probs = ctx.sample_with_distribution(_cuda(logits), params, np.full(6, 0.999999))
    for r, p in enumerate(params):
        t, d = orc.sample_with_distribution(logits[r], to_oracle(p), orc.Rng(replay=[0.999999]))
        assert toks[r] == t and np.array_equal(probs[r].cpu().numpy().view(np.uint32), np.asarray(d, np.float32).view(np.uint32)), r


def test_rows_with_more_edited_ids_than_the_table_holds_keep_an_adjusted_copy(ctx):
    """A full-vocabulary row whose history touches thousands of distinct ids is not read from the logits by the two
    passes over the device but from its adjusted copy -- also where those passes run over segments (long rows on
    16-byte boundaries): tokens and distributions against the oracle, fp32 and bf16."""
    import torch

    rng = np.random.default_rng(123)
    V = 20_480
    f32 = rng.normal(0, 2.0, (4, V)).astype(np.float32)
    bf = (f32.view(np.uint32) >> 16).astype(np.uint16)
    exact = (bf.astype(np.uint32) << 16).view(np.float32)
    long_hist = rng.permutation(V)[:5000].tolist() + rng.integers(0, V, 3000).tolist()
    params = [SamplingParams(Temperature=0.9, TopP=0.9, RepetitionPenalty=1.2, FrequencyPenalty=0.1, RepeatLastN=0, PreviousTokens=long_hist),
              SamplingParams(Temperature=1.1, MinP=0.01, PresencePenalty=0.4, RepeatLastN=0, PreviousTokens=long_hist[:4000]),
              SamplingParams(Temperature=0.7, TopP=0.95, PreviousTokens=long_hist[:10]),
              SamplingParams(Temperature=0.0, RepetitionPenalty=1.3, RepeatLastN=0, PreviousTokens=long_hist)]
    for logits, dev in [(f32, _cuda(f32)), (exact, torch.from_numpy(bf.view(np.int16)).view(torch.bfloat16).cuda())]:
        for _ in range(3):
            u = rng.random(4)
            got = ctx.sample_batch(dev, params, u)
            assert np.array_equal(got, oracle_tokens(logits, params, u)), str(dev.dtype)
        got = ctx.build_distribution(dev, params).cpu().numpy()
        for r, p in enumerate(params):
            want = orc.build_filtered_distribution(logits[r], to_oracle(p))
            assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32)), (str(dev.dtype), r)


def test_what_a_launch_leaves_for_the_next_one_on_the_same_context(ctx):
    """The rows' scalars on the device (the maximum, the factors that a verifier applies, the list of entries that a
    min-p cut watches) live with the context and are not cleared between launches; a launch whose rows have no edits
    runs no kernel before the passes over the logits.  Launches of every kind in a row, each of them with larger and
    with smaller logits than the one before and with other numbers of rows: every one against the oracle."""
    rng = np.random.default_rng(3131)
    V = 24_000
    hist = rng.integers(0, V, 40).tolist()
    with_edits = [SamplingParams(Temperature=0.9, TopP=0.9, RepetitionPenalty=1.3, PreviousTokens=hist),
                  SamplingParams(Temperature=1.0, MinP=0.02, PresencePenalty=0.5, PreviousTokens=hist),
                  SamplingParams(Temperature=0.0, FrequencyPenalty=0.4, PreviousTokens=hist),
                  SamplingParams(Temperature=1.1, LogitBias={7: 3.0, 9: -2.0})]
    plain = [SamplingParams(Temperature=1.0, MinP=0.01), SamplingParams(Temperature=0.8, TopP=0.9), SamplingParams(),
             SamplingParams(Temperature=1.3, MinP=0.001, TopP=0.95), SamplingParams(Temperature=0.0),
             SamplingParams(Temperature=1.0, MinP=0.05)]
    spec_params = [SamplingParams() for _ in range(3)]  # (rows that no filter touches: their factors go to the verifier)
    t, q, k, us = _spec_case(3, 2, V, spec_params, 77, False)
    for it, shift in enumerate((0.0, 30.0, -30.0, 5.0, -80.0, 0.0)):
        big = (rng.normal(0, 2.0, (6, V)) + shift).astype(np.float32)
        _check_rows(ctx, big[:4], with_edits, rng.random(4))
        _check_rows(ctx, (big - 2 * shift).astype(np.float32), plain, rng.random(6))
        if it % 2 == 0:
            _check_spec(ctx, t + np.float32(shift), q, k, spec_params, us)
        _check_distribution(ctx, big[:2], plain[:2])
        _check_rows(ctx, big[1:3], plain[3:5], rng.random(2))
        _check_rows(ctx, big, plain, rng.random(6))


def test_workgroups_that_stop_waiting_for_their_row_leave_their_segments_to_the_last_one(ctx):
    """The pass over long rows keeps a wave's segments in registers between the row maximum and expf(x - max); the
    workgroups of a row wait for each other in between.  The wait is bounded: with a limit of 0 polls every workgroup
    stops waiting, marks its segments and leaves them to the row's last workgroup, with 1 to 3 polls some do.  Tokens,
    distributions and verification results must not change: rows with edits applied on the fly and rows that keep an
    adjusted copy, allow-masks, bf16, rows for the histogram of a top-p cut and for the list of a min-p cut, launches
    with one and with two segments a wave."""
    import torch

    rng = np.random.default_rng(5150)
    V = 40_968
    hist = rng.integers(0, V, 60).tolist()
    long_hist = rng.permutation(V)[:3000].tolist()
    base = [SamplingParams(Temperature=0.9, TopP=0.9, RepetitionPenalty=1.2, PreviousTokens=hist),
            SamplingParams(Temperature=1.0, MinP=0.02, PresencePenalty=0.4, PreviousTokens=hist),
            SamplingParams(Temperature=0.8, TopP=0.95),
            SamplingParams(Temperature=1.1, MinP=0.01, TopP=0.9, FrequencyPenalty=0.2, RepeatLastN=0, PreviousTokens=long_hist),
            SamplingParams(Temperature=0.0, RepetitionPenalty=1.3, PreviousTokens=hist),
            SamplingParams(), SamplingParams(Temperature=1.4, TopK=30_000)]
    few = rng.normal(0, 2.0, (len(base), V)).astype(np.float32)
    few[2] *= 2.0
    many_rows = 56                                  # x 41 segments: two segments a wave
    many = rng.normal(0, 2.0, (many_rows, V)).astype(np.float32)
    many_params = [base[i % len(base)] for i in range(many_rows)]
    allowed = rng.random((len(base), V)) < 0.6
    mask, active = pack_allow_mask(allowed), np.ones(len(base), dtype=np.uint8)
    bf_bits = synthetic.to_bf16_bits(few)
    bf_exact = synthetic.bf16_bits_to_f32(bf_bits)
    bf_dev = torch.from_numpy(bf_bits.view(np.int16)).view(torch.bfloat16).cuda()
    spec_params = [SamplingParams(), SamplingParams(Temperature=0.8, TopP=0.9), SamplingParams()]
    t, q, k, us = _spec_case(3, 2, 20_000, spec_params, 41, True)
    H = hooks_lib()
    try:
        for polls in (0, 1, 2, 3, 1 << 15):
            ctx._check(H.sr_debug_set_row_wait_limit(ctx.h, polls))
            for _ in range(2):
                _check_rows(ctx, few, base, rng.random(len(base)))
                u = rng.random(many_rows)
                assert np.array_equal(ctx.sample_batch(_cuda(many), many_params, u), oracle_tokens(many, many_params, u)), polls
            _check_rows(ctx, few, base, rng.random(len(base)), mask, active)
            _check_distribution(ctx, few, base)
            u = rng.random(len(base))
            assert np.array_equal(ctx.sample_batch(bf_dev, base, u), oracle_tokens(bf_exact, base, u)), polls
            _check_spec(ctx, t, q, k, spec_params, us)
    finally:
        ctx._check(H.sr_debug_set_row_wait_limit(ctx.h, 1 << 15))


def test_edits_crowded_into_a_few_segments_of_a_long_row(ctx):
    """The pass over long rows applies the edits of a sampled row where it loads the row: a workgroup lists the edits
    that fall into its segments (room for 256) and goes through the row's whole edit list when there are more.  Rows
    whose history and bias ids crowd into the first 3,000 ids, into one segment, and at the very end of the row."""
    rng = np.random.default_rng(606)
    V = 45_000  # (a ragged last segment)
    logits = rng.normal(0, 2.0, (5, V)).astype(np.float32)
    low = rng.permutation(3000)[:900].tolist()
    one_seg = (2048 + rng.permutation(1024)[:700]).tolist()
    tail = (V - 1 - rng.permutation(900)[:500]).tolist()
    params = [SamplingParams(Temperature=0.9, TopP=0.9, RepetitionPenalty=1.3, RepeatLastN=0, PreviousTokens=low + low[:50]),
              SamplingParams(Temperature=1.0, MinP=0.01, PresencePenalty=0.6, FrequencyPenalty=0.2, RepeatLastN=0, PreviousTokens=one_seg),
              SamplingParams(Temperature=0.8, TopP=0.95, LogitBias={int(i): float(b) for i, b in zip(tail[:300], rng.normal(0, 2, 300))},
                             PresencePenalty=0.3, RepeatLastN=0, PreviousTokens=tail),
              SamplingParams(Temperature=1.1, RepetitionPenalty=0.8, RepeatLastN=0, PreviousTokens=low[:400] + tail[:400]),
              SamplingParams(Temperature=0.7, LogitBias={int(i): 4.0 for i in one_seg[:280]})]
    for p in params:
        for i in (p.PreviousTokens or [])[:8]:
            logits[params.index(p), i] += 6.0  # some of the edited ids carry mass: the edits decide
    for _ in range(3):
        _check_rows(ctx, logits, params, rng.random(5))
    _check_distribution(ctx, logits, params)
    bits = synthetic.to_bf16_bits(logits)
    import torch

    dev = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).cuda()
    exact = synthetic.bf16_bits_to_f32(bits)
    u = rng.random(5)
    assert np.array_equal(ctx.sample_batch(dev, params, u), oracle_tokens(exact, params, u))
