"""Seeded synthetic workloads: the five benchmark configurations of the sampling path.

Generator: numpy Philox, seed 0x57170000 + configuration number.  Logits are N(0, 1.5^2) with the 20
largest entries of each row boosted by 12 * rank^-1.1 (a Zipf(1.1) head of at most +12).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import SamplingParams, pack_allow_mask

SEED_BASE = 0x57170000
QWEN_VOCAB = 151_936
SMOL_VOCAB = 49_152
GEMMA_VOCAB = 262_144


def _rng(config: int, stream: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(key=SEED_BASE + config, counter=[stream, 0, 0, 0]))


def zipf_head_logits(rng: np.random.Generator, rows: int, vocab: int, sigma: float = 1.5, head: int = 20,
                     boost: float = 12.0, s: float = 1.1) -> np.ndarray:
    x = rng.standard_normal((rows, vocab), dtype=np.float32) * np.float32(sigma)
    h = min(head, vocab)
    if h > 0:
        top = np.argpartition(-x, h - 1, axis=1)[:, :h]
        order = np.argsort(-np.take_along_axis(x, top, axis=1), axis=1, kind="stable")
        top = np.take_along_axis(top, order, axis=1)
        add = (boost * np.arange(1, h + 1, dtype=np.float64) ** (-s)).astype(np.float32)
        np.put_along_axis(x, top, np.take_along_axis(x, top, axis=1) + add[None, :], axis=1)
    return x


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (round to nearest even), returned as uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


@dataclass
class Workload:
    name: str
    logits: np.ndarray                       # fp32 [rows, vocab] (for bf16 configs: the exact upcast)
    params: List[SamplingParams]
    uniforms: np.ndarray                     # float64 [rows] or [rows, n]
    logits_bf16: Optional[np.ndarray] = None  # uint16 bits when the tensor is stored as bf16
    allow_mask: Optional[np.ndarray] = None   # uint32 [rows, ceil(vocab/32)]
    mask_active: Optional[np.ndarray] = None
    extra: dict = field(default_factory=dict)

    @property
    def rows(self) -> int:
        return self.logits.shape[0]

    @property
    def vocab(self) -> int:
        return self.logits.shape[1]


def config1(steps: int = 1, vocab: int = SMOL_VOCAB) -> Workload:
    """Single sequence, vocab 49,152; T .8, top-k 40, top-p .95, repetition 1.1 over a 64-token history
    drawn uniformly from the vocab.  `steps` independent rows stand for successive decode steps."""
    rng = _rng(1)
    logits = zipf_head_logits(rng, steps, vocab)
    hist = rng.integers(0, vocab, size=(steps, 64))
    params = [SamplingParams(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1, RepeatLastN=64,
                             PreviousTokens=hist[i].tolist()) for i in range(steps)]
    return Workload("c1", logits, params, rng.random(steps))


def _zipf_history(rng: np.random.Generator, vocab: int, n: int, s: float = 1.1) -> np.ndarray:
    perm_head = rng.permutation(vocab)[:4096]
    w = np.arange(1, len(perm_head) + 1, dtype=np.float64) ** (-s)
    return perm_head[rng.choice(len(perm_head), size=n, p=w / w.sum())]


def config2(rows: int = 64, vocab: int = QWEN_VOCAB, hist_len: int = 512) -> Workload:
    """T .7, top-p .9, min-p .05, frequency .5, presence .3 over 512-token Zipf histories."""
    rng = _rng(2)
    logits = zipf_head_logits(rng, rows, vocab)
    params = [SamplingParams(Temperature=0.7, TopP=0.9, MinP=0.05, FrequencyPenalty=0.5, PresencePenalty=0.3,
                             PreviousTokens=_zipf_history(rng, vocab, hist_len).tolist()) for _ in range(rows)]
    return Workload("c2", logits, params, rng.random(rows))


def config3(rows: int = 256, vocab: int = QWEN_VOCAB, bf16: bool = True, full_chain: bool = False,
            hist_len: int = 64) -> Workload:
    """Heterogeneous rows: top-k U{1..1000}, top-p U[.5,1], T U[.3,1.5], 10% greedy.
    bf16=True stores the logits as bf16 (the configuration as written); bf16=False is the fp32 variant.
    full_chain=True adds min-p .05 and repetition 1.1 / presence .1 / frequency .1 over a 64-token
    history to every sampled row (penalties, top-k, top-p, min-p all active)."""
    rng = _rng(3)
    logits = zipf_head_logits(rng, rows, vocab)
    bits = None
    if bf16:
        bits = to_bf16_bits(logits)
        logits = bf16_bits_to_f32(bits)
    k = rng.integers(1, 1001, size=rows)
    p = rng.uniform(0.5, 1.0, size=rows)
    t = rng.uniform(0.3, 1.5, size=rows)
    greedy = rng.random(rows) < 0.10
    hist = rng.integers(0, vocab, size=(rows, hist_len))
    # make part of each history hit the head of the row so the penalties act on live candidates
    head = np.argsort(-logits, axis=1)[:, :hist_len // 4]
    hist[:, : hist_len // 4] = head
    params = []
    for i in range(rows):
        sp = SamplingParams(Temperature=0.0 if greedy[i] else float(np.float32(t[i])), TopK=int(k[i]),
                            TopP=float(np.float32(p[i])))
        if full_chain:
            sp.MinP = 0.05
            sp.RepetitionPenalty = 1.1
            sp.PresencePenalty = 0.1
            sp.FrequencyPenalty = 0.1
            sp.PreviousTokens = hist[i].tolist()
        params.append(sp)
    name = "c3" + ("_bf16" if bf16 else "_fp32") + ("_full" if full_chain else "")
    return Workload(name, logits, params, rng.random(rows), logits_bf16=bits)


def run_mask(rng: np.random.Generator, vocab: int, density: float) -> np.ndarray:
    """Allowed ids in contiguous runs of length U{1..64} until density * vocab bits are set."""
    allowed = np.zeros(vocab, dtype=bool)
    target = max(1, int(round(density * vocab)))
    while int(allowed.sum()) < target:
        n = int(rng.integers(1, 65))
        s = int(rng.integers(0, vocab))
        allowed[s:s + n] = True
    return allowed


def config4(rows: int = 32, vocab: int = QWEN_VOCAB) -> Workload:
    """Constrained decoding: allow-mask density log-uniform in [0.05%, 50%], mask applied before
    T .6 / top-p .95; rows alternate greedy / sampled."""
    rng = _rng(4)
    logits = zipf_head_logits(rng, rows, vocab)
    dens = np.exp(rng.uniform(np.log(5e-4), np.log(0.5), size=rows))
    allowed = np.stack([run_mask(rng, vocab, float(d)) for d in dens])
    params = [SamplingParams(Temperature=0.0) if i % 2 == 0 else SamplingParams(Temperature=0.6, TopP=0.95)
              for i in range(rows)]
    return Workload("c4", logits, params, rng.random(rows), allow_mask=pack_allow_mask(allowed),
                    mask_active=np.ones(rows, dtype=np.uint8), extra={"density": dens})


def config5(rows: int = 16, n_draft: int = 8, vocab: int = GEMMA_VOCAB) -> Workload:
    """Speculative verification: target = draft + N(0, .5^2); q = softmax(draft) (T=1, no filters);
    draft tokens drawn from q with seeded uniforms; n_draft + 1 uniforms per row.
    logits holds the TARGET rows [rows * (n_draft + 1), vocab]; extra has draft_logits / draft_tokens."""
    rng = _rng(5)
    draft = zipf_head_logits(rng, rows * n_draft, vocab)
    target = np.empty((rows, n_draft + 1, vocab), dtype=np.float32)
    noise = rng.standard_normal((rows, n_draft, vocab), dtype=np.float32) * np.float32(0.5)
    target[:, :n_draft] = draft.reshape(rows, n_draft, vocab) + noise
    target[:, n_draft] = zipf_head_logits(rng, rows, vocab)
    params = [SamplingParams(Temperature=1.0) for _ in range(rows)]
    return Workload("c5", target.reshape(rows * (n_draft + 1), vocab), params, rng.random((rows, n_draft + 1)),
                    extra={"draft_logits": draft, "n_draft": n_draft, "draft_uniforms": rng.random(rows * n_draft)})
