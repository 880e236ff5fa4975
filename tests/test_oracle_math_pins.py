"""Pins on the oracle that the reference's own tests leave open, chosen so that a plausible slip
(a dropped term, a wrong sign or index, a swapped operand, a wrong tie rule) fails one of them:
brute force on small rows, closed forms in exact/double arithmetic, invariants."""
import ctypes
import ctypes.util
import math

import numpy as np
import pytest

from oracle import binding as orc
from oracle.binding import Params, Rng

NEG_INF = np.float32("-inf")
f32 = np.float32


def test_expf_equals_host_libm_on_a_dense_sample():
    # (An exhaustive sweep of all 3.26e9 floats in [-inf, 89) was run once while the oracle was written
    # and matched bit for bit; this keeps a 400k-point guard in the suite.)
    libm = ctypes.CDLL(ctypes.util.find_library("m"))
    libm.expf.argtypes = [ctypes.c_float]
    libm.expf.restype = ctypes.c_float
    rng = np.random.default_rng(7)
    xs = np.concatenate([
        -rng.exponential(8.0, 200000), rng.uniform(-104.5, 0, 150000), rng.uniform(0, 88.9, 50000),
        [0.0, -0.0, -87.5, -88.0, -103.0, -103.97, -104.0, -1e-10, -1e-38, 88.7, 88.73],
    ]).astype(np.float32)
    for x in xs:
        a, b = f32(orc.expf(x)), f32(libm.expf(ctypes.c_float(x)))
        assert a.tobytes() == b.tobytes(), (x, a, b)
    assert orc.expf(NEG_INF) == 0.0 and orc.expf(0.0) == 1.0
    assert math.isnan(orc.expf(float("nan")))


def test_tp_sum_lane_shape_is_the_documented_one():
    rng = np.random.default_rng(3)
    for n in [0, 1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 100, 1001]:
        x = (rng.random(n).astype(np.float32) * f32(1e3)).astype(np.float32)
        if n < 4:
            s = f32(0)
            for v in x:
                s = f32(s + v)
        else:
            w = 8 if n >= 8 else 4
            acc = x[:w].copy()
            i = w
            while i <= n - w:
                acc = (acc + x[i:i + w]).astype(np.float32)
                i += w
            if i != n:
                rem = n - i
                last = x[n - w:].copy()
                last[: w - rem] = 0
                acc = (acc + last).astype(np.float32)
            pair = lambda a: f32(f32(a[0] + a[1]) + f32(a[2] + a[3]))
            s = pair(acc) if w == 4 else f32(pair(acc[:4]) + pair(acc[4:]))
        assert f32(orc.tp_sum(x)).tobytes() == f32(s).tobytes(), n
    # and it is a sum: exact on small integers in any order
    assert orc.tp_sum(np.arange(1, 101)) == 5050.0


def test_argmax_matrix_from_the_device_argmax_parity_suite():
    # tests/OpenTail.Stingray.Tests.Cuda/CudaGpuArgmaxParityTests.cs:56-124 (sizes scaled to CPU time)
    for n in [1, 2, 3, 255, 256, 257, 1000, 65536, 152064]:
        r = Rng(seed=1234 + n)
        a = np.array([r.next_double() * 20 - 10 for _ in range(min(n, 3000))], dtype=np.float32)
        a = np.resize(a, n)
        assert orc.greedy(a) == int(np.argmax(a))
        for pos in (0, n // 2, n - 1):
            b = a.copy()
            b[pos] = 1000.0 + pos
            assert orc.greedy(b) == pos
    a = np.full(5000, -1, dtype=np.float32)
    a[700] = a[300] = 5
    assert orc.greedy(a) == 300                       # tie -> lower index
    assert orc.greedy(np.full(8192, 3.5, np.float32)) == 0
    assert orc.greedy(np.full(16, NEG_INF, np.float32)) == 0
    assert orc.greedy([]) == 0


def _brute_top_k_sample(logits, p: Params, u):
    """Independent statement of the fast path for history-free rows: full sort by (value desc, index
    asc), softmax over the first k in fp32 sequential order, cuts, draw."""
    logits = np.asarray(logits, dtype=np.float32)
    order = sorted(range(len(logits)), key=lambda i: (-float(logits[i]), i))
    order = [i for i in order if logits[i] != NEG_INF][: p.top_k]
    if not order:
        return int(np.argmax(logits)) if len(logits) else 0
    inv_t = f32(1) if p.temperature == 1.0 else f32(1) / f32(p.temperature)
    mx = f32(logits[order[0]] * inv_t)
    e = [f32(orc.expf(f32(f32(logits[i] * inv_t) - mx))) for i in order]
    e += [f32(0)] * (p.top_k - len(order))
    s = f32(0)
    for v in e:
        s = f32(s + v)
    inv = f32(1) / s if s > 0 else f32(0)
    pr = [f32(v * inv) for v in e]
    cnt = p.top_k
    if p.min_p > 0:
        thr = f32(f32(p.min_p) * pr[0])
        for t in range(cnt):
            if pr[t] < thr:
                cnt = t
                break
    if 0 < p.top_p < 1:
        c = f32(0)
        for t in range(cnt):
            c = f32(c + pr[t])
            if c >= f32(p.top_p):
                cnt = t + 1
                break
    ks = f32(0)
    for t in range(cnt):
        ks = f32(ks + pr[t])
    r = f32(f32(u) * ks)
    c = f32(0)
    for t in range(cnt):
        c = f32(c + pr[t])
        if r <= c and t < len(order):
            return order[t]
    return order[0]


def test_fast_path_equals_brute_force_with_ties_and_masks():
    rng = np.random.default_rng(11)
    for trial in range(300):
        n = int(rng.integers(2, 200))
        # coarse grid => many exact ties, so the (value desc, index asc) rule is exercised
        logits = (rng.integers(-12, 12, n) / 2.0).astype(np.float32)
        logits[rng.random(n) < 0.2] = NEG_INF
        p = Params(temperature=float(rng.choice([0.5, 1.0, 1.7])), top_k=int(rng.integers(1, n)),
                   top_p=float(rng.choice([1.0, 0.9, 0.5])), min_p=float(rng.choice([0.0, 0.05, 0.3])))
        for u in (0.0, float(rng.random()), 0.9999999):
            assert orc.sample_u(logits, p, u) == _brute_top_k_sample(logits, p, u), (trial, u)


def test_slow_path_closed_forms_small_rows():
    # softmax / min-p / top-p / draw on a row small enough to do by hand in double precision
    logits = np.array([2.0, 1.0, 0.0, -1.0, 3.0, NEG_INF], dtype=np.float32)
    z = np.exp(np.array([2.0, 1.0, 0.0, -1.0, 3.0]) - 3.0)
    sm = z / z.sum()                                   # [.2336 .0859 .0316 .0116 .6364]
    probs = orc.build_filtered_distribution(logits, Params())
    assert np.allclose(probs[:5], sm, rtol=1e-5) and probs[5] == 0.0
    # temperature 0.5 doubles the logits
    z2 = np.exp(2 * (np.array([2.0, 1.0, 0.0, -1.0, 3.0]) - 3.0))
    probs = orc.build_filtered_distribution(logits, Params(temperature=0.5))
    assert np.allclose(probs[:5], z2 / z2.sum(), rtol=1e-5)
    # min-p 0.2 keeps p >= 0.2*0.636 = 0.127 -> tokens {0, 4}
    probs = orc.build_filtered_distribution(logits, Params(min_p=0.2))
    assert set(np.nonzero(probs)[0]) == {0, 4} and np.allclose(probs[[0, 4]], sm[[0, 4]] / sm[[0, 4]].sum(), rtol=1e-5)
    # top-p 0.9: sorted .636,.234 (cum .870),.0859 (cum .956 >= .9) -> keep {4,0,1}
    probs = orc.build_filtered_distribution(logits, Params(top_p=0.9))
    assert set(np.nonzero(probs)[0]) == {0, 1, 4} and abs(probs.sum() - 1) < 1e-6
    # top-p exactly reached by the first token is kept alone
    probs = orc.build_filtered_distribution(logits, Params(top_p=0.6))
    assert set(np.nonzero(probs)[0]) == {4}
    # draw: cumulative in INDEX order, r <= cum
    cum = np.cumsum(sm)
    p = Params()
    assert orc.sample_u(logits, p, 0.0) == 0           # r = 0 <= cum[0]
    assert orc.sample_u(logits, p, float(cum[0]) - 1e-4) == 0
    assert orc.sample_u(logits, p, float(cum[0]) + 1e-4) == 1
    assert orc.sample_u(logits, p, float(cum[3]) + 1e-4) == 4
    assert orc.sample_u(logits, p, 0.99999994) in (4, 5)


def test_draw_quirks():
    # u == 0 returns index 0 even when probs[0] == 0 (Sampler.cs:568-572 with r <= cumSum)
    assert orc.sample_from_probs([0.0, 1.0], Rng(replay=[0.0])) == 0
    # rounding fallback: last index
    assert orc.sample_from_probs([0.25, 0.25, 0.25], Rng(replay=[0.99])) == 2
    # fully masked row -> uniform over ALL tokens (Sampler.cs:452-458)
    probs = orc.build_filtered_distribution([NEG_INF] * 4, Params())
    assert np.all(probs == 0.25)
    assert orc.sample_u([NEG_INF] * 4, Params(), 0.6) == 2


def test_history_penalties_hand_arithmetic():
    logits = np.array([4.0, -2.0, 1.0, 0.5], dtype=np.float32)
    # window = last 2 entries [1, 0]; token 0 appears 3x overall, once in window
    hist = [0, 0, 1, 0]
    p = Params(repetition_penalty=2.0, repeat_last_n=2, presence_penalty=0.25, frequency_penalty=0.5,
               previous_tokens=hist, logit_bias={-1: 0.0})
    # rep: tok0 4/2 = 2; tok1 -2*2 = -4.  pres/freq over whole history: tok0 -(0.25+1.5) = 0.25; tok1 -(0.25+0.5) = -4.75
    adj = np.array([0.25, -4.75, 1.0, 0.5])
    z = np.exp(adj - adj.max())
    probs = orc.build_filtered_distribution(logits, p)
    assert np.allclose(probs, z / z.sum(), rtol=1e-5)
    # repeat_last_n = 0 means the whole history: tok0 4/2/2/2 = .5 -> .5-1.75 = -1.25
    p0 = Params(repetition_penalty=2.0, repeat_last_n=0, presence_penalty=0.25, frequency_penalty=0.5,
                previous_tokens=hist)
    adj0 = np.array([-1.25, -4.75, 1.0, 0.5])
    z0 = np.exp(adj0 - adj0.max())
    assert np.allclose(orc.build_filtered_distribution(logits, p0), z0 / z0.sum(), rtol=1e-5)
    # out-of-range history ids are ignored
    p1 = Params(repetition_penalty=2.0, presence_penalty=1.0, previous_tokens=[99, -5])
    assert np.allclose(orc.build_filtered_distribution(logits, p1), orc.build_filtered_distribution(logits, Params()))
    # fast path uses pow(rep, occWindow) once, then presence/frequency over the whole history
    pf = Params(top_k=2, repetition_penalty=2.0, repeat_last_n=2, presence_penalty=0.25,
                frequency_penalty=0.5, previous_tokens=hist)
    # sel = 2+4 = 4 (=V): vals -> tok0 4/2-1.75=.25, tok1 -4.75, tok2 1, tok3 .5 -> top2 = {2, 3}
    seen = {orc.sample_u(logits, pf, u) for u in np.linspace(0, 0.999, 50)}
    assert seen == {2, 3}


def test_slow_path_top_k_keeps_ties_at_the_kth_value():
    # ApplyTopK zeroes probs < kth only, so every value equal to the k-th survives (Sampler.cs:481-487)
    probs = orc.build_filtered_distribution([3.0, 1.0, 1.0, 1.0, 0.0], Params(top_k=2))
    assert set(np.nonzero(probs)[0]) == {0, 1, 2, 3}


def test_spec_accept_rule_closed_forms():
    V = 4
    tl = np.log(np.array([[.1, .2, .3, .4], [.25, .25, .25, .25]], dtype=np.float64)).astype(np.float32)
    p = Params()
    # q == p -> accept ratio 1 -> always accepted, bonus drawn from row 1
    q = orc.build_filtered_distribution(tl[0], p)[None, :]
    acc, toks = orc.spec_verify_row(tl, q, [2], p, Rng(replay=[0.999999, 0.6]))
    assert acc == 1 and list(toks) == [2, 2]          # bonus: uniform row, r=.6 -> index 2
    # q concentrated on the draft token: a = p[x]/1 = .3; u=.29 accepts, u=.31 rejects
    q1 = np.array([[0, 0, 1.0, 0]], dtype=np.float32)
    acc, _ = orc.spec_verify_row(tl, q1, [2], p, Rng(replay=[0.29, 0.5]))
    assert acc == 1
    r = Rng(replay=[0.31, 0.5])
    acc, toks = orc.spec_verify_row(tl, q1, [2], p, r)
    # residual = p with token 2 removed: [.1,.2,0,.4], target=.5*.7=.35 -> cum .1,.3,.7 -> token 3
    assert acc == 0 and list(toks) == [3] and r.draws == 2
    # qx == 0: accept iff px > 0
    q0 = np.array([[1.0, 0, 0, 0]], dtype=np.float32)
    acc, _ = orc.spec_verify_row(tl, q0, [2], p, Rng(replay=[0.999999, 0.5]))
    assert acc == 1
    # p-min mode: accept iff px >= pmin or draft == argmax
    pm = Params(spec_draft_p_min=0.35)
    assert orc.spec_verify_row(tl, q1, [2], pm, Rng(replay=[0.5]))[0] == 0   # .3 < .35, argmax is 3
    assert orc.spec_verify_row(tl, q1, [3], pm, Rng(replay=[0.5]))[0] == 1
    assert V == 4
    # drafts from prompt lookup (usedPld, SpeculativeDecoder.cs:538-552): the p-min rule and a draw from p itself, also
    # with the default SpecDraftPMin = 1 that selects the ratio test otherwise; q is never read, one draw on a rejection
    pl = Params(draft_from_lookup=True)
    qbad = np.full((1, 4), np.nan, dtype=np.float32)
    r = Rng(replay=[0.55, 0.9])
    acc, toks = orc.spec_verify_row(tl, qbad, [2], pl, r)           # .3 < 1 and the argmax is 3: rejected,
    assert acc == 0 and list(toks) == [2] and r.draws == 1          # p: cum .1,.3,.6 -> u=.55 -> token 2 (not removed)
    r = Rng(replay=[0.6])
    acc, toks = orc.spec_verify_row(tl, qbad, [3], pl, r)           # the argmax is accepted; bonus from the uniform row
    assert acc == 1 and list(toks) == [3, 2] and r.draws == 1
    pl2 = Params(draft_from_lookup=True, spec_draft_p_min=0.25)
    assert orc.spec_verify_row(tl, qbad, [2], pl2, Rng(replay=[0.5]))[0] == 1   # .3 >= .25
    assert orc.spec_verify_row(tl, qbad, [1], pl2, Rng(replay=[0.5]))[0] == 0   # .2 < .25, not the argmax
    # a draft id outside the vocabulary: pDist[x_i] throws in the managed loop (SpeculativeDecoder.cs:536); the
    # restatement ends the row there with -1 and draws nothing
    for bad in (-1, 4, 2 ** 31 - 1):
        r = Rng(replay=[0.1, 0.1])
        acc, toks = orc.spec_verify_row(tl, q1, [bad], p, r)
        assert acc == 0 and list(toks) == [-1] and r.draws == 0


def test_mtp_accept_draft_closed_form():
    # MtpDecoder.cs:562-596; the pMin < 1 branch has no reference test: pinned by the closed form
    logits = np.array([1.0, 3.0, 2.0, -1.0], dtype=np.float32)
    z = np.exp(logits.astype(np.float64) - 3.0)
    for idx in range(4):
        assert abs(orc.softmax_prob_at(logits, idx) - z[idx] / z.sum()) < 1e-7
    assert orc.mtp_accept_draft(1, 1, logits, 1.0) == (True, 0.0)
    assert orc.mtp_accept_draft(2, 1, logits, 1.0) == (False, 0.0)
    ok, pr = orc.mtp_accept_draft(2, 1, logits, 0.2)
    assert ok and abs(pr - z[2] / z.sum()) < 1e-7
    assert not orc.mtp_accept_draft(0, 1, logits, 0.2)[0]


def test_allow_mask_bits():
    logits = np.arange(70, dtype=np.float32)
    words = np.zeros(3, dtype=np.uint32)
    for i in (0, 31, 32, 69):
        words[i >> 5] |= np.uint32(1) << np.uint32(i & 31)
    out = orc.apply_allow_mask(logits, words)
    assert [i for i in range(70) if out[i] != NEG_INF] == [0, 31, 32, 69]
    assert out[69] == 69.0


def test_sample_batch_is_the_row_loop():
    rng = np.random.default_rng(5)
    B, V = 6, 300
    logits = rng.normal(0, 1.5, (B, V)).astype(np.float32)
    params = [Params(temperature=0.8, top_k=int(k), top_p=0.9) for k in (0, 1, 5, 40, 299, 300)]
    us = rng.random(B)
    out = orc.sample_batch(logits, params, us)
    for r in range(B):
        assert out[r] == orc.sample_u(logits[r], params[r], us[r])
