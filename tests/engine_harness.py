"""A small batcher for the tests of the engine seam: the decode loop of the reference restated
(src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs:560-740 BatcherLoop, :1194-1281 ActivateSeq) with the
scripted fixtures of its own wiring tests (tests/OpenTail.Stingray.Tests.ForwardPass.Fast/
ContinuousBatchingConstraintTests.cs:29-158: a canned forward pass, a scripted constraint, a one-byte tokenizer).

Two ways through one loop:

* ``device=None``: the reference's path.  Full logits come back to the host, the constraint filters them, the CPU
  oracle samples (``Sampler.Greedy | Sampler.Sample``, :635-647).
* ``device=RocmBatchSampler``: steps that are not all-greedy go through ``DeviceSamplingGate.TrySample``; logits stay
  on the device, tokens come back.

Only what the sampling seam touches is restated: admission, the all-greedy gate, the per-row sampling, Accept /
RecentTokens.Add, the MaxNewTokens cut.  Prefill chunking, caches, reasoning state, streaming decoders are not.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional

import numpy as np

from opentail.stingray_amd import SamplingParams
from opentail.stingray_amd.engine_seam import (DeviceSamplingGate, MaskCache, PeekableRandom, RocmBatchSampler,
                                               StepScratch)
from oracle import binding as orc
from tests.helpers import to_oracle

VOCAB = 128
PREFER_X = ord("X")
FORCE_Y = ord("Y")


class ScriptedConstraint:
    """ContinuousBatchingConstraintTests.cs:66-88: constraining once `engage_after` tokens were accepted, for
    `forced_len` tokens; masks every logit except 'Y'."""

    def __init__(self, engage_after: int, forced_len: int, allow: int = FORCE_Y, always_dead: bool = False):
        self.engage_after, self.forced_len, self.allow, self.always_dead = engage_after, forced_len, allow, always_dead
        self.AcceptCount = self.FilterCount = self.ResetCount = 0
        self._masked: Optional[np.ndarray] = None

    @property
    def IsConstraining(self) -> bool:
        return self.engage_after <= self.AcceptCount < self.engage_after + self.forced_len

    def Filter(self, logits: np.ndarray) -> np.ndarray:
        self.FilterCount += 1
        if self._masked is None:
            self._masked = np.empty(len(logits), dtype=np.float32)
        m = self._masked
        if len(m) != len(logits) or self.always_dead:
            return logits                                   # dead state: the same span comes back
        m[:] = -np.inf
        m[self.allow] = logits[self.allow]
        return m

    def Accept(self, token: int) -> None:
        self.AcceptCount += 1

    def Reset(self) -> None:
        self.AcceptCount = 0
        self.ResetCount += 1


class AndTokenConstraint:
    """src/OpenTail.Stingray.Core/Grammar/AndTokenConstraint.cs:25-97."""

    def __init__(self, inner):
        if len(inner) < 2:
            raise ValueError("at least two inner constraints are required")
        self.Inner = list(inner)
        self._masked: Optional[np.ndarray] = None

    @property
    def IsConstraining(self) -> bool:
        return any(c.IsConstraining for c in self.Inner)

    def Filter(self, logits: np.ndarray) -> np.ndarray:
        live = [c for c in self.Inner if c.IsConstraining]
        if not live:
            return logits
        if len(live) == 1:
            return live[0].Filter(logits)
        if self._masked is None:
            self._masked = np.empty(len(logits), dtype=np.float32)
        masked = self._masked
        if len(masked) != len(logits):
            return logits
        masked[:] = logits
        for c in live:
            view = c.Filter(logits)
            if view is logits or len(view) != len(masked):
                continue
            masked[np.isneginf(view)] = -np.inf
        return masked if np.any(~np.isneginf(masked)) else logits

    def Accept(self, token: int) -> None:
        for c in self.Inner:
            c.Accept(token)

    def Reset(self) -> None:
        for c in self.Inner:
            c.Reset()


def canned_row(seq_id: int, position: int) -> np.ndarray:
    """FakeBatchedForwardPass.Row(): zeros, 'X' = 2 on top, 'Y' = 1.5 the runner-up (:108-114)."""
    r = np.zeros(VOCAB, dtype=np.float32)
    r[PREFER_X] = 2.0
    r[FORCE_Y] = 1.5
    return r


class FakeBatchedForwardPass:
    """The canned forward pass (:93-158) with the sampling sibling added.  `row_fn(seq_id, position)` gives a
    sequence's next-token logits; the device copy of a step's rows is made where a real pass would have left them."""

    SupportsBatchedGpuArgmax = True

    def __init__(self, row_fn: Callable[[int, int], np.ndarray] = canned_row, sampler: Optional[RocmBatchSampler] = None):
        self.row_fn = row_fn
        self.sampler = sampler
        self.ArgmaxCalls = self.FullLogitsCalls = self.SampleCalls = 0
        self.MaxBatchWidth = 0

    @property
    def SupportsBatchedGpuSampling(self) -> bool:
        return self.sampler is not None

    def _rows(self, caches, positions) -> np.ndarray:
        self.MaxBatchWidth = max(self.MaxBatchWidth, len(caches))
        return np.stack([self.row_fn(c, p) for c, p in zip(caches, positions)])

    def Prefill(self, seq_id: int, n_prompt: int) -> np.ndarray:
        return self.row_fn(seq_id, n_prompt - 1)

    def BatchForwardMulti(self, tokens, positions, caches) -> np.ndarray:
        self.FullLogitsCalls += 1
        return self._rows(caches, positions)

    def BatchForwardMultiArgmax(self, tokens, positions, caches):
        self.ArgmaxCalls += 1
        rows = self._rows(caches, positions)
        return [(int(orc.greedy(r)), float(r.max())) for r in rows]

    def InvalidateSamplingState(self) -> None:
        if self.sampler is not None:
            self.sampler.InvalidateHistory()

    def BatchForwardMultiSample(self, tokens, positions, caches, inputs, same_rows):
        import torch

        self.SampleCalls += 1
        dev = torch.from_numpy(self._rows(caches, positions)).cuda()       # the LM head's output, resident
        toks = torch.empty(len(caches), dtype=torch.int32, device="cuda")
        flags = torch.zeros(len(caches), dtype=torch.int32, device="cuda")
        self.sampler.Sample(dev, toks, inputs, same_rows, flags)
        self.sampler.ctx.synchronize()
        return toks.cpu().numpy(), flags.cpu().numpy().view(np.uint32)     # rows x 8 bytes: the step's only download


@dataclass
class Request:
    prompt: str
    sp: SamplingParams
    max_new_tokens: int
    constraint: object = None
    rng_seed: int = 0
    arrive_at_step: int = 0                # the engine step before which the request is queued
    forced_close_at: Optional[int] = None  # test hook: the decode step (of this sequence) whose token is forced
    forced_token: int = ord("Z")
    out: List[int] = field(default_factory=list)
    draws: int = 0
    done: bool = False

    @property
    def text(self) -> str:
        return "".join(chr(t) for t in self.out)


class _ActiveSeq:
    def __init__(self, req: Request, seq_id: int, rng):
        self.req, self.Id, self.Rng = req, seq_id, rng
        self.Sp = req.sp
        self.Constraint = req.constraint
        self.CurrentToken = -1
        self.Position = 0
        self.TokenCount = 0
        self.RecentTokens: Optional[List[int]] = None
        self.decode_steps = 0

    @property
    def ForcedClose(self) -> bool:        # stands for the </think> budget overrun (:584-586, :618-622)
        return self.req.forced_close_at is not None and self.decode_steps == self.req.forced_close_at


class MiniBatcher:
    def __init__(self, fwd: FakeBatchedForwardPass, max_batch: int, device: Optional[RocmBatchSampler] = None, vocab: int = VOCAB):
        self.fwd, self.max_batch, self.device, self.vocab = fwd, max_batch, device, vocab
        self.BatchedArgmaxSteps = self.BatchedFullLogitsSteps = self.BatchedDeviceSampleSteps = 0
        self.scratch = StepScratch(masks=MaskCache(device, vocab)) if device is not None else None
        self._next_id = 0

    # `Temperature <= 0 && !HasHistoryPenalty ? Sampler.Greedy(row) : Sampler.Sample(row, spWithHistory, rng)` on a host
    # row (:641-647, :1218-1222): the reference's own sampler (the oracle) in the reference engine, the single-row
    # device path in the device engine (admission samples from prefill logits, which are on the host in both)
    def _host_sample(self, row: np.ndarray, sp: SamplingParams, history, rng) -> int:
        q = SamplingParams(**{k: getattr(sp, k) for k in sp.__dataclass_fields__})
        q.PreviousTokens = list(history) if history else None
        if self.device is not None:
            import torch

            from opentail.stingray_amd import SR_OUT_DEGENERATE, SR_OUT_PATH_TOPK_FAST

            dev = torch.from_numpy(np.ascontiguousarray(row, dtype=np.float32)).cuda().reshape(1, -1)
            sampled = sp.Temperature > 0.0
            tok, flags = self.device.ctx.sample_batch(dev, [q], [rng.Peek() if sampled else 0.0], return_flags=True)
            if sampled and not ((int(flags[0]) & SR_OUT_DEGENERATE) and (int(flags[0]) & SR_OUT_PATH_TOPK_FAST)):
                rng.Commit()
            return int(tok[0])
        if sp.Temperature <= 0.0 and not sp.HasHistoryPenalty:
            return int(orc.greedy(row))
        if sp.Temperature <= 0.0:
            return int(orc.sample(row, to_oracle(q), orc.Rng(replay=[0.0])))
        r = orc.Rng(replay=[rng.Peek()])            # one NextDouble from the sequence's generator, iff the sampler consumes one
        tok = int(orc.sample(row, to_oracle(q), r))
        if r.draws:
            rng.Commit()
        return tok

    def _activate(self, req: Request) -> Optional[_ActiveSeq]:
        from tests.helpers import DotnetRandom

        seq_id = self._next_id
        self._next_id += 1
        seq = _ActiveSeq(req, seq_id, PeekableRandom(DotnetRandom(req.rng_seed)))
        if seq.Constraint is not None:
            seq.Constraint.Reset()
        logits = self.fwd.Prefill(seq_id, len(req.prompt))
        first_logits = seq.Constraint.Filter(logits) if (seq.Constraint is not None and seq.Constraint.IsConstraining) else logits
        first = self._host_sample(first_logits, req.sp, None, seq.Rng)
        if seq.Constraint is not None:
            seq.Constraint.Accept(first)
        seq.CurrentToken = first
        seq.Position = len(req.prompt)
        seq.TokenCount = 1
        seq.RecentTokens = [first] if req.sp.HasHistoryPenalty else None
        req.out.append(first)
        return seq

    def run(self, requests: List[Request], max_steps: int = 10_000) -> None:
        pending = sorted(requests, key=lambda r: r.arrive_at_step)
        active: List[_ActiveSeq] = []
        step = 0
        while (pending or active) and step < max_steps:
            while pending and pending[0].arrive_at_step <= step and len(active) < self.max_batch:
                active.append(self._activate(pending.pop(0)))
            if not active:
                step += 1
                continue
            n = len(active)
            tokens = [s.CurrentToken for s in active]
            positions = [s.Position for s in active]
            caches = [s.Id for s in active]
            all_greedy = self.fwd.SupportsBatchedGpuArgmax and not any(
                s.Sp.Temperature > 0.0 or s.Sp.HasHistoryPenalty or s.ForcedClose
                or (s.Constraint is not None and s.Constraint.IsConstraining) for s in active)
            argmax_batch = logits_batch = device_tokens = None
            if all_greedy:
                argmax_batch = self.fwd.BatchForwardMultiArgmax(tokens, positions, caches)
                self.BatchedArgmaxSteps += 1
                if self.device is not None:
                    self.device.InvalidateHistory()        # the step did not go through the device sampler
            else:
                if self.device is not None:
                    device_tokens = DeviceSamplingGate.TrySample(self.fwd, active, tokens, positions, caches, self.scratch, step)
                if device_tokens is not None:
                    self.BatchedDeviceSampleSteps += 1
                else:
                    logits_batch = self.fwd.BatchForwardMulti(tokens, positions, caches)
                    self.BatchedFullLogitsSteps += 1
            for i in range(n - 1, -1, -1):                 # in reverse, so that removals keep the indices valid (:608)
                seq = active[i]
                if argmax_batch is not None:
                    nxt = argmax_batch[i][0]
                elif device_tokens is not None:
                    nxt = device_tokens[i]
                elif seq.ForcedClose:
                    nxt = seq.req.forced_token
                else:
                    row = logits_batch[i]
                    if seq.Constraint is not None and seq.Constraint.IsConstraining:
                        row = seq.Constraint.Filter(row)
                    nxt = self._host_sample(row, seq.Sp, seq.RecentTokens, seq.Rng)
                if seq.Constraint is not None:
                    seq.Constraint.Accept(nxt)
                if seq.RecentTokens is not None:
                    seq.RecentTokens.append(nxt)
                seq.decode_steps += 1
                if seq.TokenCount >= seq.req.max_new_tokens:     # the sample is dropped at the cut (:652-655)
                    seq.req.done = True
                    seq.req.draws = seq.Rng.draws
                    active.pop(i)
                else:
                    seq.req.out.append(nxt)
                    seq.CurrentToken = nxt
                    seq.Position += 1
                    seq.TokenCount += 1
            step += 1
