"""Shared test plumbing: SamplingParams -> oracle parameters, oracle row loops."""
from __future__ import annotations

import numpy as np

from oracle import binding as orc
from opentail.stingray_amd import SamplingParams


def to_oracle(p: SamplingParams) -> orc.Params:
    return orc.Params(temperature=p.Temperature, top_k=p.TopK, top_p=p.TopP, min_p=p.MinP,
                      repetition_penalty=p.RepetitionPenalty, repeat_last_n=p.RepeatLastN,
                      presence_penalty=p.PresencePenalty, frequency_penalty=p.FrequencyPenalty,
                      previous_tokens=p.PreviousTokens, logit_bias=p.LogitBias,
                      spec_draft_p_min=p.SpecDraftPMin, draft_from_lookup=p.SpecDraftFromLookup)


def oracle_tokens(logits: np.ndarray, params, uniforms, allow_mask=None, mask_active=None) -> np.ndarray:
    return orc.sample_batch(np.ascontiguousarray(logits, dtype=np.float32), [to_oracle(p) for p in params],
                            np.asarray(uniforms, dtype=np.float64).reshape(len(params), -1)[:, 0].copy(),
                            allow_mask, mask_active)


_hooks = None


def hooks_lib():
    """libstingray_sampler_hooks.so: the library once more with the test and measurement hooks of
    include/stingray_sampler_test.h compiled in (the product library exports none of them).  Its hooks are called on
    contexts and batches of the product library -- both are built from the same sources, so a hook that sets a field of a
    context or launches a routine on its stream works on either's."""
    global _hooks
    if _hooks is None:
        import ctypes as C
        import os

        import opentail.stingray_amd as sa

        sa.load_library()  # (the product library, and with it torch's HIP runtime, first)
        path = sa.lib_path().replace("libstingray_sampler.so", "libstingray_sampler_hooks.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python -m opentail.stingray_amd.build --hooks`")
        H = C.CDLL(path)
        vp = C.c_void_p
        H.sr_selftest_expf.argtypes = [vp, vp, vp, C.c_int64]
        H.sr_selftest_seqsum.argtypes = [vp, vp, C.c_int32, C.c_float, C.c_float, vp, vp]
        H.sr_selftest_segsum.argtypes = [vp, vp, C.c_int32, C.c_double, C.c_float, vp, vp]
        H.sr_debug_append_rebuilds.argtypes = [vp]
        H.sr_debug_append_moves.argtypes = [vp]
        H.sr_debug_set_spin_limit.argtypes = [vp, C.c_uint32]
        H.sr_debug_set_row_wait_limit.argtypes = [vp, C.c_uint32]
        _hooks = H
    return _hooks


class ReplayRandom:
    """Stands in for System.Random: hands out the given NextDouble() values and counts the draws."""

    def __init__(self, values):
        self.values = list(values)
        self.draws = 0

    def NextDouble(self) -> float:
        v = self.values[self.draws] if self.draws < len(self.values) else 0.0
        self.draws += 1
        return v


class DotnetRandom:
    """System.Random(seed) through the oracle's restatement of the runtime's generator."""

    def __init__(self, seed: int):
        self._r = orc.Rng(seed=seed)

    def NextDouble(self) -> float:
        return self._r.next_double()

    @property
    def draws(self) -> int:
        return self._r.draws
