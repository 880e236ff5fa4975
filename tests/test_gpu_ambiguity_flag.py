"""SR_OUT_AMBIGUOUS: the row's token is still the one the documented conventions give, but it rests on something the
managed runtime leaves open -- the draw or a cut lies within a few ulp of a boundary of the running sum (the lane
order of TensorPrimitives.Sum, Sampler.cs:555, and the last bit of MathF.Exp can move such a sum by an ulp or two), or
a top-p cut splits a run of equal probabilities (the unstable sort of Sampler.cs:533).  A managed caller re-runs such a
row on the CPU.  Tested here: draws placed exactly on a boundary are flagged (the boundary is found by bisecting the
oracle's own answer in u), draws in the middle of a token's interval are not, cuts inside runs of equal
probabilities are, and a random batch flags few rows."""
import numpy as np
import pytest

from opentail.stingray_amd import SR_OUT_AMBIGUOUS, SamplerContext, SamplingParams, synthetic
from oracle import binding as orc
from tests.helpers import oracle_tokens, to_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _boundaries(row, p, n_want, rng):
    """Pairs (u_lo, u_hi) of adjacent doubles between which the oracle's token changes, and mid-interval u's."""
    op = to_oracle(p)
    on, mid = [], []
    for _ in range(200):
        a, b = sorted(rng.random(2))
        ta, tb = orc.sample_u(row, op, a), orc.sample_u(row, op, b)
        if ta == tb:
            continue
        for _ in range(80):                       # bisect down to neighbouring doubles
            m = 0.5 * (a + b)
            if m == a or m == b:
                break
            if orc.sample_u(row, op, m) == ta:
                a = m
            else:
                b, tb = m, orc.sample_u(row, op, m)
        on.extend([a, b])
        if len(on) >= n_want:
            break
    # a u whose token's interval in u is wide, taken at the interval's middle
    for _ in range(400):
        u = rng.random()
        t = orc.sample_u(row, op, u)
        d = 1e-4
        if orc.sample_u(row, op, max(u - d, 0.0)) == t and orc.sample_u(row, op, min(u + d, 1.0 - 1e-12)) == t:
            mid.append(u)
        if len(mid) >= n_want:
            break
    return on, mid


@pytest.mark.parametrize("kind", ["topk", "full_top_p", "full_min_p", "full_plain"])
def test_draws_on_a_boundary_are_flagged_and_draws_inside_an_interval_are_not(ctx, kind):
    rng = np.random.default_rng({"topk": 1, "full_top_p": 2, "full_min_p": 3, "full_plain": 4}[kind])
    V = 3_000
    row = rng.normal(0, 1.5, V).astype(np.float32)
    row[rng.integers(0, V, 8)] += np.linspace(6, 2, 8).astype(np.float32)
    p = {"topk": SamplingParams(Temperature=0.9, TopK=50, TopP=0.97),
         "full_top_p": SamplingParams(Temperature=0.8, TopP=0.9),
         "full_min_p": SamplingParams(Temperature=1.1, MinP=0.01),
         "full_plain": SamplingParams(Temperature=1.3)}[kind]
    on, mid = _boundaries(row, p, 12, rng)
    assert len(on) >= 8 and len(mid) >= 8
    us = np.array(on + mid)
    logits = np.tile(row, (len(us), 1))
    got, flags = ctx.sample_batch(_cuda(logits), [p] * len(us), us, return_flags=True)
    assert np.array_equal(got, oracle_tokens(logits, [p] * len(us), us))
    amb = (flags & SR_OUT_AMBIGUOUS) != 0
    assert amb[: len(on)].all(), (kind, np.nonzero(~amb[: len(on)])[0])
    assert not amb[len(on):].any(), (kind, np.nonzero(amb[len(on):])[0])


def test_a_top_p_cut_inside_a_run_of_equal_probabilities_is_flagged(ctx):
    V = 4_096
    rng = np.random.default_rng(9)
    flat = np.full(V, -4.0, dtype=np.float32)
    flat[:64] = 1.0                                   # 64 equal logits carry nearly all the mass; top-p cuts among them
    sharp = rng.normal(0, 1.0, V).astype(np.float32)
    sharp[7] = 9.0                                    # one token far above: the cut is nowhere near a tie
    params = [SamplingParams(Temperature=1.0, TopP=0.5), SamplingParams(Temperature=1.0, TopP=0.5)]
    logits = np.stack([flat, sharp])
    u = np.array([0.3, 0.3])
    got, flags = ctx.sample_batch(_cuda(logits), params, u, return_flags=True)
    assert np.array_equal(got, oracle_tokens(logits, params, u))
    assert flags[0] & SR_OUT_AMBIGUOUS and not flags[1] & SR_OUT_AMBIGUOUS


def test_a_random_batch_flags_few_rows(ctx):
    w = synthetic.config3(rows=256, bf16=False, full_chain=True)
    got, flags = ctx.sample_batch(_cuda(w.logits), w.params, w.uniforms, return_flags=True)
    assert np.array_equal(got, oracle_tokens(w.logits, w.params, w.uniforms))
    assert int(((flags & SR_OUT_AMBIGUOUS) != 0).sum()) <= 2
    w2 = synthetic.config2()
    got, flags = ctx.sample_batch(_cuda(w2.logits), w2.params, w2.uniforms, return_flags=True)
    assert int(((flags & SR_OUT_AMBIGUOUS) != 0).sum()) <= 1
