"""The seam in the engine, host side: where the reference's decode loops call ``Sampler.Greedy | Sampler.Sample`` on
downloaded logits, a device sampler slots in and only tokens come back.

Three capability siblings, one per existing device-argmax capability of the reference:

* batched decode -- ``SupportsBatchedGpuSampling`` / ``BatchForwardMultiSample`` beside ``SupportsBatchedGpuArgmax`` /
  ``BatchForwardMultiArgmax`` (src/OpenTail.Stingray.Engine/IBatchedForwardPass.cs:105-117), used by
  :class:`DeviceSamplingGate` where the batcher loop gathers its rows
  (src/OpenTail.Stingray.Engine/ContinuousBatchingEngine.cs:580-650);
* single sequence -- ``SupportsGpuSampling`` / ``ForwardSample`` beside ``SupportsGpuArgmax`` / ``ForwardArgmax``
  (src/OpenTail.Stingray.Core/IForwardPass.cs:25-42), used by :class:`SingleSequenceGate`
  (src/OpenTail.Stingray.Engine/InferenceEngine.cs:1200-1254);
* verification -- ``SupportsBatchVerifySample`` / ``BatchVerifySample`` and ``BatchVerifyAccept`` beside
  ``SupportsBatchVerifyArgmax`` / ``BatchVerifyArgmax`` (IForwardPass.cs:257-283), used by
  :class:`VerifyGate` (SpeculativeDecoder.cs:526-559, MtpDecoder.cs:439-468).

The classes are the line-for-line twins of ``managed/RocmBatchSampler.cs`` and ``managed/EngineSeam.cs``; this file is
the executable one (no .NET SDK where this library is built).  Everything that samples runs in the native library.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import (SR_OUT_DEGENERATE, SR_OUT_PATH_TOPK_FAST, SamplerContext, SamplingParams, pack_allow_mask)

__all__ = ["BatchedSamplingInputs", "RocmBatchSampler", "MaskCache", "PeekableRandom", "DeviceSamplingGate",
           "SingleSequenceGate", "VerifyGate", "StepScratch"]


class PeekableRandom:
    """A sequence's ``Random`` as the gates need it: upcoming ``NextDouble()`` values can be looked at before it is
    known how many of them the sampler will consume.  ``Sampler.Sample`` draws exactly once per sampled call -- except
    that ``SampleTopK`` on a row without a finite logit falls back to ``Greedy`` and draws nothing
    (Sampler.cs:251-255); the accept loop of StepSampled draws once per verified position up to the first rejection
    and once more for the correction (SpeculativeDecoder.cs:530-559).  The device needs the uniforms before it knows;
    values it turns out not to have needed stay pending, and the sequence's next draws return them in order, so the
    stream of values the sequence consumes stays the reference's."""

    def __init__(self, rng):
        self._rng = rng
        self._pending: List[float] = []
        self.draws = 0                      # values consumed, as the reference's Random would count them

    def Peek(self, i: int = 0) -> float:
        while len(self._pending) <= i:
            self._pending.append(float(self._rng.NextDouble()))
        return self._pending[i]

    def Commit(self, n: int = 1) -> None:
        assert n <= len(self._pending)
        del self._pending[:n]
        self.draws += n

    def NextDouble(self) -> float:
        v = self.Peek()
        self.Commit()
        return v


@dataclass
class BatchedSamplingInputs:
    """What one decode step hands over per row (the inputs the hot loop gathers, ContinuousBatchingEngine.cs:609-650)."""

    Params: Sequence[SamplingParams]             # seq.Sp; PreviousTokens is ignored, Histories is used
    Histories: Sequence[Optional[List[int]]]     # seq.RecentTokens (None without a history penalty, :1280)
    MaskIds: Sequence[int]                       # registered mask of the constraint's state, -1 = none / dead state
    Uniforms: Sequence[float]                    # one NextDouble() per row with Temperature > 0, else 0
    PreviousTokens: Optional[Sequence[int]] = None   # the token sampled in the previous step (joins the history)


class RocmBatchSampler:
    """One instance per engine, kept across decode steps (twin of managed/RocmBatchSampler.cs).  Stands where the
    per-row ``Sampler.Greedy | Sampler.Sample`` calls of the batcher loop stand
    (ContinuousBatchingEngine.cs:609-650) and gives the same tokens; the logits never leave the device."""

    def __init__(self, device: int = 0, ctx: Optional[SamplerContext] = None):
        self.ctx = ctx if ctx is not None else SamplerContext(device)
        self._own_ctx = ctx is None
        self._batch = self.ctx.new_batch()
        self._rows = -1
        self._vocab = -1
        # the library's copy of the histories is what the engine's RecentTokens are: true after a step that went
        # through Sample, false after any step that did not (the engine sampled on the host, or skipped the rows)
        self._history_valid = False
        self.uploads = 0
        self.appends = 0

    def BindToCurrentThread(self) -> None:       # IThreadAffineBackend.cs:9-21, ContinuousBatchingEngine.cs:495-500
        self.ctx._check(self.ctx.L.sr_bind_thread(self.ctx.h))

    def RegisterMask(self, words: np.ndarray, vocab: int) -> int:
        return self.ctx.register_mask(words, vocab)

    def ReleaseMask(self, mask_id: int) -> None:
        self.ctx.release_mask(mask_id)

    def MaskAnd(self, ids: Sequence[int]) -> int:
        return self.ctx.mask_and(ids)

    @staticmethod
    def PackMask(masked: np.ndarray) -> np.ndarray:
        """The masked row a Filter call returned -> allow-bits (allowed iff not negative infinity)."""
        return pack_allow_mask(~np.isneginf(np.asarray(masked, dtype=np.float32)))

    def InvalidateHistory(self) -> None:
        """A decode step did not go through Sample: the next one uploads, whatever the caller says about its rows."""
        self._history_valid = False

    def Sample(self, logits_dev, tokens_dev, inputs: BatchedSamplingInputs, same_rows_as_last_step: bool, flags_dev=None) -> None:
        """One step: enqueues the sampling of the rows of ``logits_dev`` ([rows, vocab] on the device) into
        ``tokens_dev``.  First step, changed rows or an invalidated history: pack and upload; else append the previous
        tokens, the mask ids and the uniforms (sr_batch_append_tokens_masks).  Nothing here waits for the device."""
        rows, vocab = logits_dev.shape
        prev = inputs.PreviousTokens
        if (same_rows_as_last_step and self._history_valid and rows == self._rows and vocab == self._vocab
                and prev is not None and len(prev) == rows):
            self._batch.append_tokens(np.asarray(prev, dtype=np.int32), np.asarray(inputs.Uniforms, dtype=np.float64),
                                      mask_ids=np.asarray(inputs.MaskIds, dtype=np.int32))
            self.appends += 1
        else:
            params = []
            for p, h in zip(inputs.Params, inputs.Histories):
                q = SamplingParams(**{k: getattr(p, k) for k in p.__dataclass_fields__})
                q.PreviousTokens = list(h) if h else None     # `sp with { PreviousTokens = seq.RecentTokens }` (:640-642)
                params.append(q)
            self._batch.upload(params, vocab, np.asarray(inputs.Uniforms, dtype=np.float64),
                               mask_ids=np.asarray(inputs.MaskIds, dtype=np.int32))
            self._rows, self._vocab = rows, vocab
            self.uploads += 1
        self.ctx.sample_launch(self._batch, logits_dev, tokens_dev, flags_dev)
        self._history_valid = True

    def Dispose(self) -> None:
        self._batch.close()
        if self._own_ctx:
            self.ctx.close()


class MaskCache:
    """Mask ids of constraint states.  A constraint that can name its state (``MaskStateKey``: an automaton state, a
    trie node) is asked once per state; any other ``ITokenConstraint`` is asked through ``Filter`` on a row of zeros
    -- one call per constrained step, as the loop makes today (ContinuousBatchingEngine.cs:635-637), but on a host
    row that never held logits -- and the packed answer is looked up by content.  ``Filter`` returning its input is
    the dead state: no mask (ITokenConstraint.cs:36-41).  A constraint that exposes its inner constraints
    (``Inner``, as AndTokenConstraint has them) is combined on the device from its inners' ids (sr_mask_and,
    AndTokenConstraint.cs:44-86)."""

    def __init__(self, sampler: RocmBatchSampler, vocab: int):
        self.sampler = sampler
        self.vocab = vocab
        self._probe = np.zeros(vocab, dtype=np.float32)
        self._by_key: Dict[object, int] = {}
        self._by_content: Dict[bytes, int] = {}
        self._by_tuple: Dict[Tuple[int, ...], int] = {}

    def MaskIdOf(self, c) -> int:
        inner = getattr(c, "Inner", None)
        if inner is not None:
            live = [x for x in inner if x.IsConstraining]
            if len(live) == 0:
                return -1
            if len(live) == 1:
                return self.MaskIdOf(live[0])
            ids = tuple(self.MaskIdOf(x) for x in live)
            if ids not in self._by_tuple:
                self._by_tuple[ids] = self.sampler.MaskAnd(ids)
            return self._by_tuple[ids]
        key = getattr(c, "MaskStateKey", None)
        if key is not None and (id(c), key) in self._by_key:
            return self._by_key[(id(c), key)]
        view = c.Filter(self._probe)
        if view is self._probe or len(view) != self.vocab:
            mid = -1
        else:
            words = RocmBatchSampler.PackMask(view)
            h = words.tobytes()
            if h not in self._by_content:
                self._by_content[h] = self.sampler.RegisterMask(words, self.vocab)
            mid = self._by_content[h]
        if key is not None:
            self._by_key[(id(c), key)] = mid
        return mid


@dataclass
class StepScratch:
    """The per-step arrays of the gate (kept by the engine, sized for its batch) and what the gate remembers between
    steps: which sequences the library's batch holds and at which engine step it last sampled them."""

    masks: MaskCache
    last_ids: List[int] = field(default_factory=list)
    last_step: int = -2


class DeviceSamplingGate:
    """Goes in BatcherLoop after the all-greedy gate (ContinuousBatchingEngine.cs:580-606): called where the loop falls
    back to BatchForwardMulti (full logits) because some row is sampled, has history penalties or is constraining."""

    @staticmethod
    def TrySample(fwd, active, tokens, positions, caches, scratch: StepScratch, step_no: int):
        """Returns the tokens of every row, or None when the step must take the full-logits path (the forward pass
        cannot sample; a row's token is forced, :618-622).  Nothing is consumed -- no Filter call, no uniform -- when
        it returns None.  ``step_no`` counts the engine's decode steps: rows are appended to only when the previous
        step sampled the same sequences here."""
        if not getattr(fwd, "SupportsBatchedGpuSampling", False):
            return None
        n = len(active)
        # first pass: decisions only
        for s in active:
            if s.ForcedClose:
                fwd.InvalidateSamplingState()
                return None
        # second pass: masks of the constraints' states; one Filter call per constrained row at most
        mask_ids = [scratch.masks.MaskIdOf(s.Constraint) if (s.Constraint is not None and s.Constraint.IsConstraining) else -1
                    for s in active]
        # third pass: the step is committed to the device; look at one uniform per sampled row (none for greedy rows:
        # Sampler.Sample consumes none there, Sampler.cs:19-22)
        uniforms = [s.Rng.Peek() if s.Sp.Temperature > 0.0 else 0.0 for s in active]
        ids = [s.Id for s in active]
        same_rows = ids == scratch.last_ids and step_no == scratch.last_step + 1
        inputs = BatchedSamplingInputs(
            Params=[s.Sp for s in active], Histories=[s.RecentTokens for s in active], MaskIds=mask_ids, Uniforms=uniforms,
            # the token fed to this forward step is the one the previous step sampled: it joined RecentTokens (:650)
            PreviousTokens=[int(t) if s.RecentTokens is not None else -1 for t, s in zip(tokens, active)] if same_rows else None)
        out, flags = fwd.BatchForwardMultiSample(tokens, positions, caches, inputs, same_rows)
        for s, f in zip(active, flags):
            if s.Sp.Temperature > 0.0 and not ((int(f) & SR_OUT_DEGENERATE) and (int(f) & SR_OUT_PATH_TOPK_FAST)):
                s.Rng.Commit()
        scratch.last_ids = ids
        scratch.last_step = step_no
        return [int(t) for t in out]


class SingleSequenceGate:
    """The single-user decode loop's sibling (InferenceEngine.cs:1200-1254): one row, the same sampler object."""

    def __init__(self, sampler: RocmBatchSampler, masks: MaskCache):
        self.sampler = sampler
        self.masks = masks
        self._last_step = -2

    def TrySample(self, fwd, token: int, position: int, sp: SamplingParams, recent_tokens, constraint, rng: PeekableRandom,
                  forced_close: bool, step_no: int):
        if not getattr(fwd, "SupportsGpuSampling", False) or forced_close:
            self.sampler.InvalidateHistory()
            return None
        mid = self.masks.MaskIdOf(constraint) if (constraint is not None and constraint.IsConstraining) else -1
        u = rng.Peek() if sp.Temperature > 0.0 else 0.0
        same = step_no == self._last_step + 1
        inputs = BatchedSamplingInputs(Params=[sp], Histories=[recent_tokens], MaskIds=[mid], Uniforms=[u],
                                       PreviousTokens=[token if recent_tokens is not None else -1] if same else None)
        tok, flag = fwd.ForwardSample(token, position, inputs, same)
        if sp.Temperature > 0.0 and not ((int(flag) & SR_OUT_DEGENERATE) and (int(flag) & SR_OUT_PATH_TOPK_FAST)):
            rng.Commit()
        self._last_step = step_no
        return int(tok)


class VerifyGate:
    """Verification on the device with the distributions resident there.

    ``BatchVerifySample`` is StepSampled's accept loop (SpeculativeDecoder.cs:526-559) over the k+1 target rows of one
    step and the k draft distributions that ``SampleWithDistribution`` left on the device (:509-513): accepted length
    and tokens come back instead of (k+1) x vocab logits.  ``BatchVerifyAccept`` is MtpDecoder's accept test
    (MtpDecoder.cs:439-468 with AcceptDraft :562-596) for pMin < 1, where ``BatchVerifyArgmax`` alone is not enough."""

    def __init__(self, ctx: SamplerContext):
        self.ctx = ctx

    def BatchVerifySample(self, target_logits_dev, draft_probs_dev, draft_tokens_dev, sp: SamplingParams, rng: PeekableRandom,
                          used_lookup: bool = False):
        """target [k+1, V], q [k, V] (None for prompt-lookup drafts), draft tokens [k] -- device tensors of one sequence.
        Consumes from ``rng`` what the managed loop draws: under the ratio test one NextDouble per verified position up
        to and including the first rejection; then one for the correction token, or for the bonus token when
        Temperature > 0.  Returns (accepted, tokens[accepted + 1])."""
        k = int(draft_tokens_dev.shape[0])
        uniforms = np.array([rng.Peek(i) for i in range(k + 1)], dtype=np.float64)
        q = SamplingParams(**{f: getattr(sp, f) for f in sp.__dataclass_fields__})
        q.SpecDraftFromLookup = bool(used_lookup)
        acc, toks = self.ctx.spec_verify(target_logits_dev[None], None if draft_probs_dev is None else draft_probs_dev[None],
                                         draft_tokens_dev[None], [q], uniforms[None])
        a = int(acc[0])
        ratio_test = not (0.0 < sp.SpecDraftPMin < 1.0) and not used_lookup      # SpeculativeDecoder.cs:538, 549
        rejected = a < k
        rng.Commit((min(a + 1, k) if ratio_test else 0) + (1 if (rejected or sp.Temperature > 0.0) else 0))
        return a, [int(t) for t in toks[0, : a + 1]]

    def BatchVerifyAccept(self, logits_dev, draft_tokens_dev, p_min: float):
        """Per verified position: (argmax, accept, probability of the draft where the softmax was needed)."""
        return self.ctx.mtp_verify(logits_dev, draft_tokens_dev, p_min)
