"""ctypes view of the CPU oracle (oracle/stingray_oracle.c).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg, never by the product package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libstingray_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds). Returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class CParams(C.Structure):
    _fields_ = [
        ("temperature", C.c_float),
        ("top_k", C.c_int32),
        ("top_p", C.c_float),
        ("min_p", C.c_float),
        ("repetition_penalty", C.c_float),
        ("repeat_last_n", C.c_int32),
        ("presence_penalty", C.c_float),
        ("frequency_penalty", C.c_float),
        ("prev", C.POINTER(C.c_int32)),
        ("n_prev", C.c_int32),
        ("bias_ids", C.POINTER(C.c_int32)),
        ("bias_vals", C.POINTER(C.c_float)),
        ("n_bias", C.c_int32),
        ("spec_draft_p_min", C.c_float),
        ("draft_from_lookup", C.c_int32),
    ]


class CRng(C.Structure):
    _fields_ = [
        ("replay", C.POINTER(C.c_double)),
        ("replay_len", C.c_int64),
        ("pos", C.c_int64),
        ("seed_array", C.c_int32 * 56),
        ("inext", C.c_int32),
        ("inextp", C.c_int32),
    ]


@dataclass
class Params:
    """Mirror of the reference's SamplingParams fields the sampler reads (Sampler.cs:648-813)."""

    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    repeat_last_n: int = 64
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    previous_tokens: Optional[Sequence[int]] = None
    logit_bias: Optional[dict] = None
    spec_draft_p_min: float = 1.0
    draft_from_lookup: bool = False
    _keep: list = field(default_factory=list, repr=False)

    def to_c(self) -> CParams:
        cp = CParams()
        cp.temperature = self.temperature
        cp.top_k = self.top_k
        cp.top_p = self.top_p
        cp.min_p = self.min_p
        cp.repetition_penalty = self.repetition_penalty
        cp.repeat_last_n = self.repeat_last_n
        cp.presence_penalty = self.presence_penalty
        cp.frequency_penalty = self.frequency_penalty
        cp.spec_draft_p_min = self.spec_draft_p_min
        cp.draft_from_lookup = 1 if self.draft_from_lookup else 0
        self._keep = []
        if self.previous_tokens is not None and len(self.previous_tokens) > 0:
            prev = np.ascontiguousarray(np.asarray(self.previous_tokens, dtype=np.int32))
            self._keep.append(prev)
            cp.prev = prev.ctypes.data_as(C.POINTER(C.c_int32))
            cp.n_prev = len(prev)
        if self.logit_bias:
            ids = np.ascontiguousarray(np.asarray(list(self.logit_bias.keys()), dtype=np.int32))
            vals = np.ascontiguousarray(np.asarray(list(self.logit_bias.values()), dtype=np.float32))
            self._keep += [ids, vals]
            cp.bias_ids = ids.ctypes.data_as(C.POINTER(C.c_int32))
            cp.bias_vals = vals.ctypes.data_as(C.POINTER(C.c_float))
            cp.n_bias = len(ids)
        return cp


class Rng:
    """Either a seeded .NET-compatible Random or a replayed list of NextDouble() values."""

    def __init__(self, seed: Optional[int] = None, replay: Optional[Sequence[float]] = None):
        self._lib = lib()
        self.c = CRng()
        self._replay = None
        if replay is not None:
            self._replay = np.ascontiguousarray(np.asarray(replay, dtype=np.float64))
            self._lib.oracle_rng_replay(C.byref(self.c), self._replay.ctypes.data_as(C.POINTER(C.c_double)),
                                        len(self._replay))
        else:
            self._lib.oracle_dotnet_random_init(C.byref(self.c), int(seed if seed is not None else 0))

    def next(self) -> int:
        return self._lib.oracle_dotnet_random_next(C.byref(self.c))

    def next_double(self) -> float:
        return self._lib.oracle_rng_next_double(C.byref(self.c))

    @property
    def draws(self) -> int:
        return int(self.c.pos)


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(_LIB_PATH)
    fp = C.POINTER(C.c_float)
    ip = C.POINTER(C.c_int32)
    pp = C.POINTER(CParams)
    rp = C.POINTER(CRng)
    L.oracle_rng_replay.argtypes = [rp, C.POINTER(C.c_double), C.c_int64]
    L.oracle_dotnet_random_init.argtypes = [rp, C.c_int32]
    L.oracle_dotnet_random_next.argtypes = [rp]
    L.oracle_dotnet_random_next.restype = C.c_int32
    L.oracle_rng_next_double.argtypes = [rp]
    L.oracle_rng_next_double.restype = C.c_double
    L.oracle_expf.argtypes = [C.c_float]
    L.oracle_expf.restype = C.c_float
    L.oracle_tp_max.argtypes = [fp, C.c_int32]
    L.oracle_tp_max.restype = C.c_float
    L.oracle_tp_sum.argtypes = [fp, C.c_int32]
    L.oracle_tp_sum.restype = C.c_float
    L.oracle_tp_index_of_max.argtypes = [fp, C.c_int32]
    L.oracle_tp_index_of_max.restype = C.c_int32
    L.oracle_greedy.argtypes = [fp, C.c_int32]
    L.oracle_greedy.restype = C.c_int32
    L.oracle_sample.argtypes = [fp, C.c_int32, pp, rp]
    L.oracle_sample.restype = C.c_int32
    L.oracle_build_filtered_distribution.argtypes = [fp, C.c_int32, pp, fp, C.c_int32]
    L.oracle_build_filtered_distribution.restype = C.c_int32
    L.oracle_sample_with_distribution.argtypes = [fp, C.c_int32, pp, fp, rp]
    L.oracle_sample_with_distribution.restype = C.c_int32
    L.oracle_sample_from_probs.argtypes = [fp, C.c_int32, rp]
    L.oracle_sample_from_probs.restype = C.c_int32
    L.oracle_resample_residual.argtypes = [fp, C.c_int32, fp, C.c_int32, rp]
    L.oracle_resample_residual.restype = C.c_int32
    L.oracle_apply_allow_mask.argtypes = [fp, C.POINTER(C.c_uint32), C.c_int32, fp]
    L.oracle_spec_verify_row.argtypes = [fp, fp, ip, C.c_int32, C.c_int32, pp, rp, fp, ip]
    L.oracle_spec_verify_row.restype = C.c_int32
    L.oracle_softmax_prob_at.argtypes = [fp, C.c_int32, C.c_int32]
    L.oracle_softmax_prob_at.restype = C.c_float
    L.oracle_mtp_accept_draft.argtypes = [C.c_int32, C.c_int32, fp, C.c_int32, C.c_float, fp]
    L.oracle_mtp_accept_draft.restype = C.c_int32
    L.oracle_sample_batch.argtypes = [fp, C.c_int64, C.c_int32, C.c_int32, pp, C.POINTER(C.c_uint32),
                                      C.c_int64, C.POINTER(C.c_uint8), C.POINTER(C.c_double), fp, ip]
    L.oracle_seq_sum.argtypes = [fp, C.c_int64, C.c_float, C.c_float, C.POINTER(C.c_int64)]
    L.oracle_seq_sum.restype = C.c_float
    _lib = L
    return L


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _fp(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def seq_sum(x, s0: float = 0.0, target: float = float("inf")):
    """(left-to-right fp32 sum, first index whose running sum >= target or -1)"""
    a = _f32(x)
    at = C.c_int64(-1)
    s = lib().oracle_seq_sum(_fp(a), len(a), s0, target, C.byref(at))
    return np.float32(s), int(at.value)


def expf(x: float) -> float:
    return float(lib().oracle_expf(np.float32(x)))


def tp_sum(x) -> float:
    a = _f32(x)
    return float(lib().oracle_tp_sum(_fp(a), len(a)))


def greedy(logits) -> int:
    a = _f32(logits)
    return lib().oracle_greedy(_fp(a), len(a))


def sample(logits, p: Params, rng: Rng) -> int:
    a = _f32(logits)
    cp = p.to_c()
    return lib().oracle_sample(_fp(a), len(a), C.byref(cp), C.byref(rng.c))


def sample_u(logits, p: Params, u: float) -> int:
    """Sample with the single NextDouble() value u."""
    return sample(logits, p, Rng(replay=[u]))


def build_filtered_distribution(logits, p: Params, n_probs: Optional[int] = None) -> np.ndarray:
    a = _f32(logits)
    n = len(a) if n_probs is None else n_probs
    out = np.zeros(n, dtype=np.float32)
    cp = p.to_c()
    rc = lib().oracle_build_filtered_distribution(_fp(a), len(a), C.byref(cp), _fp(out), n)
    if rc != 0:
        raise ValueError("probs length must equal logits length")
    return out


def sample_with_distribution(logits, p: Params, rng: Rng):
    a = _f32(logits)
    out = np.zeros(len(a), dtype=np.float32)
    cp = p.to_c()
    tok = lib().oracle_sample_with_distribution(_fp(a), len(a), C.byref(cp), _fp(out), C.byref(rng.c))
    return tok, out


def sample_from_probs(probs, rng: Rng) -> int:
    a = _f32(probs)
    return lib().oracle_sample_from_probs(_fp(a), len(a), C.byref(rng.c))


def resample_residual(p, q, rng: Rng) -> int:
    a, b = _f32(p), _f32(q)
    rc = lib().oracle_resample_residual(_fp(a), len(a), _fp(b), len(b), C.byref(rng.c))
    if rc < 0:
        raise ValueError("p and q must have equal length")
    return rc


def apply_allow_mask(logits, mask_words) -> np.ndarray:
    a = _f32(logits)
    m = np.ascontiguousarray(np.asarray(mask_words, dtype=np.uint32))
    out = np.empty_like(a)
    lib().oracle_apply_allow_mask(_fp(a), m.ctypes.data_as(C.POINTER(C.c_uint32)), len(a), _fp(out))
    return out


def spec_verify_row(target_logits, draft_probs, draft_tokens, p: Params, rng: Rng):
    """target_logits [(L+1), V], draft_probs [L, V], draft_tokens [L] -> (accepted, tokens[accepted+1])."""
    t = _f32(target_logits)
    q = _f32(draft_probs)
    d = np.ascontiguousarray(np.asarray(draft_tokens, dtype=np.int32))
    L = len(d)
    V = t.shape[-1]
    assert t.shape == (L + 1, V) and (L == 0 or q.shape == (L, V))
    scratch = np.empty(V, dtype=np.float32)
    out = np.full(L + 1, -1, dtype=np.int32)
    cp = p.to_c()
    acc = lib().oracle_spec_verify_row(_fp(t), _fp(q), d.ctypes.data_as(C.POINTER(C.c_int32)), L, V,
                                       C.byref(cp), C.byref(rng.c), _fp(scratch),
                                       out.ctypes.data_as(C.POINTER(C.c_int32)))
    return acc, out[: acc + 1].copy()


def softmax_prob_at(logits, idx: int) -> float:
    a = _f32(logits)
    return float(lib().oracle_softmax_prob_at(_fp(a), len(a), idx))


def mtp_accept_draft(draft: int, target: int, logits, p_min: float):
    a = _f32(logits)
    prob = C.c_float(0)
    ok = lib().oracle_mtp_accept_draft(draft, target, _fp(a), len(a), p_min, C.byref(prob))
    return bool(ok), float(prob.value)


def sample_batch(logits: np.ndarray, params: Sequence[Params], uniforms, allow_mask=None, mask_active=None) -> np.ndarray:
    """Rows in order on one thread (the reference's batcher loop). logits [B, V] fp32."""
    a = _f32(logits)
    B, V = a.shape
    arr = (CParams * B)()
    for i, p in enumerate(params):
        arr[i] = p.to_c()
    u = np.ascontiguousarray(np.asarray(uniforms, dtype=np.float64))
    out = np.empty(B, dtype=np.int32)
    scratch = np.empty(V, dtype=np.float32)
    mptr = None
    aptr = None
    stride = 0
    if allow_mask is not None:
        m = np.ascontiguousarray(np.asarray(allow_mask, dtype=np.uint32))
        stride = m.shape[1]
        mptr = m.ctypes.data_as(C.POINTER(C.c_uint32))
        if mask_active is not None:
            act = np.ascontiguousarray(np.asarray(mask_active, dtype=np.uint8))
            aptr = act.ctypes.data_as(C.POINTER(C.c_uint8))
    lib().oracle_sample_batch(_fp(a), V, B, V, arr, mptr, stride, aptr,
                              u.ctypes.data_as(C.POINTER(C.c_double)), _fp(scratch),
                              out.ctypes.data_as(C.POINTER(C.c_int32)))
    return out
