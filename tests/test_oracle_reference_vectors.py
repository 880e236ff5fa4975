"""The oracle against every known-answer test the reference holds for this path.

Each test names the reference test it restates (tests/OpenTail.Stingray.Tests.ForwardPass.Fast/
SamplerTests.cs and SpeculativeSamplingTests.cs).  Seeds are replayed through the oracle's
restatement of System.Random(seed), so the statistical assertions run on the same streams.
"""
import math

import numpy as np
import pytest

from oracle import binding as orc
from oracle.binding import Params, Rng

NEG_INF = float("-inf")


# ── System.Random anchors ─────────────────────────────────────────────────────────────────────
def test_dotnet_random_anchors():
    # Widely published first outputs of new Random(seed).Next() (seeded compat generator).
    assert Rng(seed=42).next() == 1434747710
    assert Rng(seed=0).next() == 1559595546
    assert Rng(seed=1).next() == 534011718


def test_dotnet_random_range_and_determinism():
    a, b = Rng(seed=999), Rng(seed=999)
    xs = [a.next_double() for _ in range(1000)]
    assert xs == [b.next_double() for _ in range(1000)]
    assert all(0.0 <= x < 1.0 for x in xs)
    assert 0.45 < sum(xs) / len(xs) < 0.55


# ── SamplerTests.cs:8-34 ──────────────────────────────────────────────────────────────────────
def test_greedy_returns_argmax():
    assert orc.greedy([1, 5, 3, 2]) == 1
    assert orc.greedy([10, 1, 2, 3]) == 0
    assert orc.greedy([1, 2, 3, 100]) == 3


def test_sample_temperature_zero_is_greedy():
    r = Rng(seed=1)
    assert orc.sample([1, 5, 3, 2], Params(temperature=0.0), r) == 1
    assert r.draws == 0  # greedy consumes no random number


# ── SamplerTests.cs:37-147 (statistical, same seeds) ─────────────────────────────────────────
def test_very_low_temperature_peaks_at_max():
    rng = Rng(seed=42)
    p = Params(temperature=0.001)
    picks = sum(orc.sample([1, 10, 2, 3], p, rng) == 1 for _ in range(100))
    assert picks >= 99


def test_high_temperature_more_uniform():
    rng = Rng(seed=42)
    p = Params(temperature=100.0)
    counts = [0] * 4
    for _ in range(10000):
        counts[orc.sample([0, 0, 0, 10], p, rng)] += 1
    assert all(1500 <= c <= 3500 for c in counts)


def test_top_k_restricts_to_k_tokens():
    rng = Rng(seed=42)
    p = Params(temperature=1.0, top_k=2)
    seen = {orc.sample(list(range(1, 11)), p, rng) for _ in range(1000)}
    assert seen <= {8, 9}


def test_top_p_restricts_to_nucleus():
    rng = Rng(seed=42)
    p = Params(temperature=1.0, top_p=0.5)
    counts = [0] * 10
    for _ in range(100):
        counts[orc.sample([0] * 9 + [20], p, rng)] += 1
    assert counts[9] >= 95


def test_min_p_filters_low_prob_tokens():
    rng = Rng(seed=42)
    p = Params(temperature=1.0, min_p=0.1)
    seen = {orc.sample([0] * 9 + [50], p, rng) for _ in range(100)}
    assert 9 in seen and len(seen) <= 2


def test_returned_token_in_valid_range_and_uniform_logits_all_sampled():
    rng = Rng(seed=42)
    p = Params(temperature=1.0)
    assert all(0 <= orc.sample([1, 2, 3, 4, 5], p, rng) <= 4 for _ in range(100))
    rng = Rng(seed=42)
    assert len({orc.sample([0, 0, 0, 0], p, rng) for _ in range(10000)}) == 4


# ── SamplerTests.cs:152-209 (logit bias) ─────────────────────────────────────────────────────
def test_logit_bias():
    rng = Rng(seed=42)
    p = Params(temperature=1.0, logit_bias={0: -100.0})
    assert 0 not in {orc.sample([10, 1, 1, 1], p, rng) for _ in range(200)}
    rng = Rng(seed=42)
    p = Params(temperature=1.0, logit_bias={2: 100.0})
    assert {orc.sample([0, 0, 0, 0], p, rng) for _ in range(200)} <= {2}
    rng = Rng(seed=42)
    p = Params(temperature=1.0, logit_bias={999: 100.0, -1: 100.0})
    assert 0 <= orc.sample([1, 2, 3], p, rng) <= 2


# ── SamplerTests.cs:211-255 (fast path vs forced slow path) ──────────────────────────────────
def _random_logits(vocab, seed):
    rng = Rng(seed=seed)
    return np.array([np.float32(rng.next_double() * 12 - 6) for _ in range(vocab)], dtype=np.float32)


def _reachable(logits, p, seed, trials):
    rng = Rng(seed=seed)
    return {orc.sample(logits, p, rng) for _ in range(trials)}


@pytest.mark.parametrize("seed", [1, 7, 99])
def test_fast_path_matches_slow_path_reachable_set(seed):
    logits = _random_logits(96, seed)
    base = dict(temperature=0.8, top_k=16, top_p=0.9, min_p=0.02, repetition_penalty=1.3,
                previous_tokens=[3, 3, 10, 25])
    fast = _reachable(logits, Params(**base), 1234, 4000)
    slow = _reachable(logits, Params(**base, logit_bias={-1: 0.0}), 1234, 4000)
    assert sorted(fast) == sorted(slow)


# ── SamplerTests.cs:258-294 ──────────────────────────────────────────────────────────────────
def test_penalty_demotes_token_out_of_top_k():
    p = Params(temperature=1.0, top_k=2, repetition_penalty=4.0, previous_tokens=[1])
    reach = _reachable([10, 8, 7, 1, 0], p, 5, 500)
    assert 1 not in reach and reach <= {0, 2} and 2 in reach


def test_penalty_duplicate_occurrences_compound():
    logits = [9, 8, 6.5, 1]
    once = Params(temperature=1.0, top_k=2, repetition_penalty=1.2, previous_tokens=[1])
    thrice = Params(temperature=1.0, top_k=2, repetition_penalty=1.2, previous_tokens=[1, 1, 1])
    r1 = _reachable(logits, once, 9, 500)
    r3 = _reachable(logits, thrice, 9, 500)
    assert 1 in r1 and 1 not in r3 and 2 in r3


# ── SamplerTests.cs:297-325 ──────────────────────────────────────────────────────────────────
def test_presence_and_frequency_apply_in_logit_space():
    logits = [10, 9.8, 0]
    pres = Params(temperature=1.0, top_k=1, presence_penalty=1.0, previous_tokens=[0])
    freq = Params(temperature=1.0, top_k=1, frequency_penalty=0.6, previous_tokens=[0, 0])
    for u in (0.0, 0.25, 0.999999):  # holds for every uniform
        assert orc.sample_u(logits, pres, u) == 1
        assert orc.sample_u(logits, freq, u) == 1
    assert orc.sample(logits, pres, Rng(seed=1)) == 1


def test_greedy_honours_presence_penalty():
    p = Params(temperature=0.0, presence_penalty=1.0, previous_tokens=[0])
    assert orc.sample([10, 9.8], p, Rng(seed=1)) == 1


# ── SamplerTests.cs:328-361 ──────────────────────────────────────────────────────────────────
def test_neg_inf_logits_never_sampled():
    logits = [2, NEG_INF, 5, NEG_INF, 1, 3]
    p = Params(temperature=1.0, top_k=5, top_p=0.95)
    rng = Rng(seed=3)
    for _ in range(1000):
        tok = orc.sample(logits, p, rng)
        assert 0 <= tok < 6 and logits[tok] != NEG_INF


def test_all_neg_inf_falls_back_to_valid_token():
    p = Params(temperature=1.0, top_k=2, top_p=0.9)
    r = Rng(seed=1)
    assert orc.sample([NEG_INF] * 3, p, r) == 0
    assert r.draws == 0  # degenerate fallback is Greedy: no draw


def test_top_k_then_top_p_nucleus_after_top_k():
    p = Params(temperature=1.0, top_k=3, top_p=0.5)
    assert _reachable([6, 3, 2.5, 0, 0, 0, 0, 0], p, 2, 500) <= {0}


# ── SamplerTests.cs:366-413 ──────────────────────────────────────────────────────────────────
def test_build_filtered_distribution_no_filters_matches_softmax():
    logits = [1.0, 2.0, 3.0, 0.0]
    probs = orc.build_filtered_distribution(logits, Params(temperature=1.0))
    e = [math.exp(x - 3.0) for x in logits]
    for i in range(4):
        assert abs(e[i] / sum(e) - probs[i]) < 5e-6
    assert abs(float(probs.sum()) - 1.0) < 5e-6


def test_build_filtered_distribution_temp_zero_one_hot():
    probs = orc.build_filtered_distribution([1, 9, 3, 2], Params(temperature=0.0))
    assert probs[1] == 1.0 and probs[0] + probs[2] + probs[3] == 0.0


def test_build_filtered_distribution_top_k():
    probs = orc.build_filtered_distribution([5, 4, 3, 2, 1], Params(temperature=1.0, top_k=2))
    assert probs[0] > 0 and probs[1] > 0 and probs[2] + probs[3] + probs[4] == 0.0
    assert abs(float(probs.sum()) - 1.0) < 5e-6
    # closed form: softmax over the two survivors
    assert abs(probs[0] - 1 / (1 + math.exp(-1))) < 1e-6


def test_build_filtered_distribution_length_mismatch_is_an_error():
    with pytest.raises(ValueError):
        orc.build_filtered_distribution([1, 2, 3], Params(), n_probs=4)


def test_sample_with_distribution_fills_probs_and_returns_token():
    tok, probs = orc.sample_with_distribution([0, 12, 0, 0], Params(temperature=0.1), Rng(seed=7))
    assert tok == 1 and probs[1] > 0.99 and abs(float(probs.sum()) - 1.0) < 5e-6


# ── SamplerTests.cs:416-442 ──────────────────────────────────────────────────────────────────
def test_resample_residual():
    rng = Rng(seed=3)
    for _ in range(200):
        assert orc.resample_residual([0, .5, .5, 0], [0, 1.0, 0, 0], rng) == 2
    tok = orc.resample_residual([.25] * 4, [.25] * 4, Rng(seed=5))
    assert 0 <= tok < 4
    with pytest.raises(ValueError):
        orc.resample_residual([0] * 4, [0] * 3, Rng(seed=1))


# ── SpeculativeSamplingTests.cs ──────────────────────────────────────────────────────────────
P_TARGET = [0.2, 2.5, 0.1, 1.0, 0.3, 1.8, 0.0, 0.5]
Q_DRAFT = [2.0, 0.1, 1.5, 0.2, 1.0, 0.0, 2.2, 0.3]


def _run_sampled_spec(seed, n, p, lookahead=4):
    """SpeculativeDecoder.Initialize + Decode with position-independent fixed-distribution passes
    (SpeculativeSamplingTests.cs:119-148): one certain token, lookahead-1 drafts per step."""
    rng = Rng(seed=seed)
    saved, _ = orc.sample_with_distribution(P_TARGET, p, rng)  # SpeculativeDecoder.cs:264
    emitted, acc_total, prop_total = [], 0, 0
    target_rows = np.tile(np.asarray(P_TARGET, dtype=np.float32), (lookahead, 1))
    while len(emitted) < n:
        drafts, qd = [], []
        for _ in range(lookahead - 1):  # SpeculativeDecoder.cs:509-513
            t, q = orc.sample_with_distribution(Q_DRAFT, p, rng)
            drafts.append(t)
            qd.append(q)
        acc, toks = orc.spec_verify_row(target_rows, np.stack(qd), drafts, p, rng)
        emitted.append(saved)
        emitted.extend(int(t) for t in toks[:acc])
        saved = int(toks[acc])
        acc_total += acc
        prop_total += lookahead - 1
    return emitted[:n], acc_total / prop_total


def test_sampled_spec_preserves_target_distribution():
    n = 40000
    emitted, rate = _run_sampled_spec(12345, n, Params(temperature=1.0))
    counts = np.bincount(emitted, minlength=8) / n
    e = np.exp(np.asarray(P_TARGET) - max(P_TARGET))
    assert np.abs(counts - e / e.sum()).max() < 0.02
    assert 0.01 < rate < 0.99


def test_sampled_spec_pmin_looser_accept_valid_tokens():
    emitted, _ = _run_sampled_spec(7, 500, Params(temperature=1.0, spec_draft_p_min=0.05))
    assert len(emitted) == 500 and all(0 <= t < 8 for t in emitted)


def test_sampled_spec_seed_determinism():
    p = Params(temperature=1.0)
    assert _run_sampled_spec(999, 200, p)[0] == _run_sampled_spec(999, 200, p)[0]
    assert _run_sampled_spec(1, 200, p)[0] != _run_sampled_spec(2, 200, p)[0]
