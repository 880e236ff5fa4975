"""The seam in the engine (IBatchedForwardPass.cs:105-117, ContinuousBatchingEngine.cs:580-650) as a tested component:
`DeviceSamplingGate` + `RocmBatchSampler` driven by the reference's own scripted fixtures and held answers
(ContinuousBatchingConstraintTests.cs:170-231, 309-337), then by random decode runs against the reference's path
(full logits on the host, the CPU oracle sampling) with sequences joining and leaving, forced tokens, rows without a
finite logit, and the per-sequence count of NextDouble() draws."""
import numpy as np
import pytest

from opentail.stingray_amd import SamplingParams
from opentail.stingray_amd.engine_seam import PeekableRandom, RocmBatchSampler, SingleSequenceGate, MaskCache, VerifyGate
from tests.engine_harness import (FORCE_Y, PREFER_X, VOCAB, AndTokenConstraint, FakeBatchedForwardPass, MiniBatcher,
                                  Request, ScriptedConstraint, canned_row)
from tests.helpers import DotnetRandom, to_oracle
from oracle import binding as orc

pytestmark = pytest.mark.gpu


@pytest.fixture()
def sampler():
    s = RocmBatchSampler(0)
    yield s
    s.Dispose()


def _engine(sampler, max_batch, row_fn=canned_row, vocab=VOCAB):
    fwd = FakeBatchedForwardPass(row_fn, sampler)
    return fwd, MiniBatcher(fwd, max_batch, sampler, vocab)


def test_constrained_sequence_is_masked_while_constraining(sampler):
    # ContinuousBatchingConstraintTests.cs:170-191
    fwd, eng = _engine(sampler, 1)
    scripted = ScriptedConstraint(engage_after=1, forced_len=3)
    req = Request("prompt", SamplingParams(Temperature=0.0), 6, constraint=scripted)
    eng.run([req])
    assert req.text == "XYYYXX"
    assert scripted.ResetCount == 1
    assert scripted.AcceptCount >= 6
    assert scripted.FilterCount == 3                 # asked for its mask on exactly the 3 constrained steps
    assert fwd.SampleCalls == 3 and fwd.FullLogitsCalls == 0 and fwd.ArgmaxCalls > 0   # no logits row came to the host


def test_no_constraint_is_unaffected(sampler):
    # :193-208
    fwd, eng = _engine(sampler, 1)
    req = Request("prompt", SamplingParams(Temperature=0.0), 6)
    eng.run([req])
    assert req.text == "XXXXXX"
    assert fwd.ArgmaxCalls > 0 and fwd.FullLogitsCalls == 0 and fwd.SampleCalls == 0
    assert eng.BatchedArgmaxSteps == fwd.ArgmaxCalls and eng.BatchedFullLogitsSteps == 0


def test_history_penalty_bypasses_the_raw_argmax_and_changes_the_greedy_choice(sampler):
    # :210-232: X = 2 with a one-point presence penalty loses to Y = 1.5 on the second token
    fwd, eng = _engine(sampler, 1)
    req = Request("prompt", SamplingParams(Temperature=0.0, PresencePenalty=1.0), 2)
    eng.run([req])
    assert req.text == "XY"
    assert fwd.ArgmaxCalls == 0 and eng.BatchedArgmaxSteps == 0
    assert fwd.SampleCalls > 0 and fwd.FullLogitsCalls == 0          # the device sampler stands where the full logits stood


def test_constrained_and_unconstrained_coexist_with_per_sequence_masking(sampler):
    # :309-337
    fwd, eng = _engine(sampler, 2)
    a = Request("alpha", SamplingParams(Temperature=0.0), 12, constraint=ScriptedConstraint(engage_after=5, forced_len=3))
    b = Request("beta", SamplingParams(Temperature=0.0), 12)
    eng.run([a, b])
    assert a.text == "XXXXXYYYXXXX"
    assert b.text == "XXXXXXXXXXXX"
    assert fwd.MaxBatchWidth == 2
    assert fwd.SampleCalls > 0 and fwd.FullLogitsCalls == 0


def _random_rows(vocab, seed):
    def row_fn(seq_id, position):
        g = np.random.default_rng((seed, seq_id, position))
        x = g.normal(0.0, 1.5, vocab).astype(np.float32)
        top = g.integers(0, vocab, 12)
        x[top] += (12.0 / np.arange(1, 13) ** 1.1).astype(np.float32)
        return x
    return row_fn


def _mixed_requests(rng, n, vocab, max_tokens):
    reqs = []
    for i in range(n):
        kind = i % 7
        c = None
        if kind == 0:
            sp = SamplingParams(Temperature=0.0)
        elif kind == 1:
            sp = SamplingParams(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1)
        elif kind == 2:
            sp = SamplingParams(Temperature=0.7, TopP=0.9, MinP=0.05, FrequencyPenalty=0.5, PresencePenalty=0.3)
        elif kind == 3:
            sp = SamplingParams(Temperature=0.0, RepetitionPenalty=1.3, PresencePenalty=0.4)
        elif kind == 4:
            sp = SamplingParams(Temperature=1.1, TopK=int(rng.integers(1, 300)))
            c = ScriptedConstraint(engage_after=int(rng.integers(1, 5)), forced_len=int(rng.integers(1, 6)), allow=int(rng.integers(0, vocab)))
        elif kind == 5:
            sp = SamplingParams(Temperature=0.6, TopP=0.95)
            c = AndTokenConstraint([_SetConstraint(rng, vocab, 2, 9), _SetConstraint(rng, vocab, 4, 6),
                                    ScriptedConstraint(3, 2, allow=int(rng.integers(0, vocab)))])
        else:
            sp = SamplingParams(Temperature=0.9, TopK=50, RepetitionPenalty=0.9, PresencePenalty=-0.2)   # penalties that raise
        reqs.append(dict(prompt="p" * int(rng.integers(1, 9)), sp=sp, max_new_tokens=int(rng.integers(2, max_tokens)),
                         constraint=c, rng_seed=int(rng.integers(0, 1 << 30)), arrive_at_step=int(rng.integers(0, 14))))
    return reqs


class _SetConstraint:
    """Constraining for a window of accepted tokens; allows a random set of the vocabulary (a grammar state's class)."""

    def __init__(self, rng, vocab, engage_after, forced_len):
        self.engage_after, self.forced_len = engage_after, forced_len
        self.allowed = rng.random(vocab) < 0.3
        self.AcceptCount = 0
        self._m = np.empty(vocab, dtype=np.float32)

    @property
    def IsConstraining(self):
        return self.engage_after <= self.AcceptCount < self.engage_after + self.forced_len

    def Filter(self, logits):
        self._m[:] = np.where(self.allowed, logits, -np.inf)
        return self._m

    def Accept(self, token):
        self.AcceptCount += 1

    def Reset(self):
        self.AcceptCount = 0


@pytest.mark.parametrize("vocab,seed", [(5_003, 1), (49_152, 2)])
def test_random_decode_runs_match_the_reference_path_token_for_token(sampler, vocab, seed):
    row_fn = _random_rows(vocab, seed)

    def build():
        g = np.random.default_rng(seed)          # same draws -> same requests, fresh constraint objects
        return [Request(**s) for s in _mixed_requests(g, 14, vocab, 22)]

    ref_reqs, dev_reqs = build(), build()
    ref_fwd = FakeBatchedForwardPass(row_fn, None)
    MiniBatcher(ref_fwd, 6, None, vocab).run(ref_reqs)
    fwd, eng = _engine(sampler, 6, row_fn, vocab)
    eng.run(dev_reqs)
    for i, (r, d) in enumerate(zip(ref_reqs, dev_reqs)):
        assert r.done and d.done
        assert d.out == r.out, (i, r.sp)
        assert d.draws == r.draws, (i, r.sp, d.draws, r.draws)
    assert fwd.FullLogitsCalls == 0 and fwd.SampleCalls > 0
    assert sampler.appends > 0 and sampler.uploads > 0          # steady steps append, a change of rows uploads
    assert fwd.MaxBatchWidth >= 3


def test_a_forced_token_falls_back_for_the_step_and_the_history_is_uploaded_again(sampler):
    vocab = 4_099
    row_fn = _random_rows(vocab, 7)

    def build():
        return [Request("ab", SamplingParams(Temperature=0.8, TopK=30, RepetitionPenalty=1.2, FrequencyPenalty=0.3), 14, rng_seed=5),
                Request("abc", SamplingParams(Temperature=0.7, TopP=0.9, PresencePenalty=0.5), 14, rng_seed=6, forced_close_at=4),
                Request("a", SamplingParams(Temperature=1.0, TopK=8), 14, rng_seed=7)]

    ref_reqs, dev_reqs = build(), build()
    MiniBatcher(FakeBatchedForwardPass(row_fn, None), 3, None, vocab).run(ref_reqs)
    fwd, eng = _engine(sampler, 3, row_fn, vocab)
    eng.run(dev_reqs)
    for r, d in zip(ref_reqs, dev_reqs):
        assert d.out == r.out and d.draws == r.draws
    assert ord("Z") in dev_reqs[1].out
    assert fwd.FullLogitsCalls == 1                  # exactly the step with the forced token took the host path
    assert sampler.uploads >= 2                      # ... and the step after it uploaded the histories again
    assert eng.BatchedDeviceSampleSteps > 8


def test_a_row_without_a_finite_logit_consumes_no_uniform(sampler):
    # SampleTopK on an all -inf row falls back to Greedy and draws nothing (Sampler.cs:251-255): afterwards the
    # sequence's generator must stand where the reference's stands
    vocab = 2_048
    base = _random_rows(vocab, 11)

    def row_fn(seq_id, position):
        if seq_id == 0 and position in (3, 4):
            return np.full(vocab, -np.inf, dtype=np.float32)
        return base(seq_id, position)

    def build():
        return [Request("a", SamplingParams(Temperature=0.9, TopK=20), 10, rng_seed=42),
                Request("a", SamplingParams(Temperature=0.9, TopP=0.9), 10, rng_seed=43)]

    ref_reqs, dev_reqs = build(), build()
    MiniBatcher(FakeBatchedForwardPass(row_fn, None), 2, None, vocab).run(ref_reqs)
    fwd, eng = _engine(sampler, 2, row_fn, vocab)
    eng.run(dev_reqs)
    for r, d in zip(ref_reqs, dev_reqs):
        assert d.out == r.out and d.draws == r.draws
    assert ref_reqs[0].draws == 9 and ref_reqs[1].draws == 11      # 11 samples each (the last one dropped); two drew nothing


def test_single_sequence_gate_follows_the_single_user_loop(sampler):
    # InferenceEngine.cs:1200-1254: recentTokens starts empty, every token (the first included) is sampled in the loop
    vocab = 10_007
    row_fn = _random_rows(vocab, 21)
    import torch

    class Fwd:
        SupportsGpuSampling = True

        def ForwardSample(self, token, position, inputs, same):
            dev = torch.from_numpy(row_fn(0, position)).cuda().reshape(1, -1)
            toks = torch.empty(1, dtype=torch.int32, device="cuda")
            flags = torch.zeros(1, dtype=torch.int32, device="cuda")
            sampler.Sample(dev, toks, inputs, same, flags)
            sampler.ctx.synchronize()
            return int(toks.cpu()[0]), int(flags.cpu().numpy().view(np.uint32)[0])

    sp = SamplingParams(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1, PresencePenalty=0.2)
    gate = SingleSequenceGate(sampler, MaskCache(sampler, vocab))
    rng = PeekableRandom(DotnetRandom(9))
    ref_rng = orc.Rng(seed=9)
    recent, ref_recent, tok = [], [], 1
    constraint = ScriptedConstraint(engage_after=2, forced_len=3, allow=77)
    ref_constraint = ScriptedConstraint(engage_after=2, forced_len=3, allow=77)
    for step in range(24):
        got = gate.TrySample(Fwd(), tok, step, sp, recent, constraint, rng, False, step)
        row = row_fn(0, step)
        if ref_constraint.IsConstraining:
            row = ref_constraint.Filter(row)
        q = SamplingParams(**{k: getattr(sp, k) for k in sp.__dataclass_fields__})
        q.PreviousTokens = list(ref_recent) if ref_recent else None
        want = int(orc.sample(row, to_oracle(q), ref_rng))
        assert got == want, step
        for c in (constraint, ref_constraint):
            c.Accept(got)
        recent.append(got)
        ref_recent.append(want)
        tok = got
    assert rng.draws == ref_rng.draws == 24
    assert sampler.appends >= 20


def test_verify_gate_accepts_and_draws_like_the_managed_loop(sampler):
    # SpeculativeDecoder.cs:526-559 for one sequence: accepted length, tokens and the number of NextDouble() draws
    import torch

    vocab, k = 8_192, 5
    g = np.random.default_rng(3)
    gate = VerifyGate(sampler.ctx)
    for trial in range(6):
        draft_logits = g.normal(0, 1.5, (k, vocab)).astype(np.float32)
        target = np.concatenate([draft_logits + g.normal(0, 0.5, (k, vocab)).astype(np.float32),
                                 g.normal(0, 1.5, (1, vocab)).astype(np.float32)])
        sp = SamplingParams(Temperature=0.0 if trial == 4 else 0.9, TopK=40 if trial % 2 else 0, TopP=0.95,
                            SpecDraftPMin=0.3 if trial == 5 else 1.0)
        q = np.stack([orc.build_filtered_distribution(draft_logits[i], to_oracle(sp)) for i in range(k)])
        dg = orc.Rng(seed=100 + trial)
        drafts = np.array([orc.sample_from_probs(q[i], dg) for i in range(k)], dtype=np.int32)
        ref_rng = orc.Rng(seed=trial)
        want_acc, want_toks = orc.spec_verify_row(target, q, drafts, to_oracle(sp), ref_rng)
        rng = PeekableRandom(DotnetRandom(trial))
        acc, toks = gate.BatchVerifySample(torch.from_numpy(target).cuda(), torch.from_numpy(q).cuda(),
                                           torch.from_numpy(drafts).cuda(), sp, rng)
        assert acc == want_acc and toks == want_toks.tolist(), trial
        assert rng.draws == ref_rng.draws, (trial, rng.draws, ref_rng.draws)
        assert rng.NextDouble() == ref_rng.next_double()          # ... and both generators stand at the same place
