"""The batcher restated in tests/engine_harness.py, on the reference's own path (full logits on the host, the CPU
oracle as Sampler.Greedy | Sampler.Sample), must give the answers the reference's wiring tests hold
(tests/OpenTail.Stingray.Tests.ForwardPass.Fast/ContinuousBatchingConstraintTests.cs:170-231, 309-337): the GPU tests
of the seam compare the device engine with this one."""
from opentail.stingray_amd import SamplingParams
from tests.engine_harness import FakeBatchedForwardPass, MiniBatcher, Request, ScriptedConstraint


def _run(reqs, max_batch):
    fwd = FakeBatchedForwardPass()
    eng = MiniBatcher(fwd, max_batch, None)
    eng.run(reqs)
    return fwd, eng


def test_constrained_sequence_is_masked_while_constraining():
    scripted = ScriptedConstraint(engage_after=1, forced_len=3)
    req = Request("prompt", SamplingParams(Temperature=0.0), 6, constraint=scripted)
    fwd, _ = _run([req], 1)
    assert req.text == "XYYYXX"
    assert scripted.ResetCount == 1 and scripted.AcceptCount >= 6 and scripted.FilterCount == 3


def test_no_constraint_takes_the_argmax_path_only():
    req = Request("prompt", SamplingParams(Temperature=0.0), 6)
    fwd, eng = _run([req], 1)
    assert req.text == "XXXXXX"
    assert fwd.ArgmaxCalls > 0 and fwd.FullLogitsCalls == 0
    assert eng.BatchedArgmaxSteps == fwd.ArgmaxCalls and eng.BatchedFullLogitsSteps == 0


def test_history_penalty_forces_the_full_logits_path_and_changes_the_greedy_choice():
    req = Request("prompt", SamplingParams(Temperature=0.0, PresencePenalty=1.0), 2)
    fwd, eng = _run([req], 1)
    assert req.text == "XY"
    assert fwd.ArgmaxCalls == 0 and fwd.FullLogitsCalls > 0
    assert eng.BatchedArgmaxSteps == 0 and eng.BatchedFullLogitsSteps > 0


def test_per_sequence_masking_in_one_batch():
    a = Request("alpha", SamplingParams(Temperature=0.0), 12, constraint=ScriptedConstraint(engage_after=5, forced_len=3))
    b = Request("beta", SamplingParams(Temperature=0.0), 12)
    fwd, _ = _run([a, b], 2)
    assert a.text == "XXXXXYYYXXXX" and b.text == "XXXXXXXXXXXX"
    assert fwd.MaxBatchWidth == 2 and fwd.FullLogitsCalls > 0
