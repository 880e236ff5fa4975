"""Registered allow-masks: the masks of a grammar's states are uploaded once (JsonToolArgumentConstraint.ComputeMask,
JsonToolArgumentConstraint.cs:434-478, computes one per automaton state) and batches name them by id; a constrained
decode loop then advances histories and masks in place (ContinuousBatchingEngine.cs:635-650: Filter -> Sample ->
Accept -> RecentTokens.Add).  Every step is compared with the oracle on the explicitly masked rows and with a batch
uploaded afresh; the device-side packer with the host one (ITokenConstraint.cs:31-42: allowed iff not -inf)."""
import ctypes as C

import numpy as np
import pytest

from opentail.stingray_amd import SamplerContext, SamplingParams, pack_allow_mask, synthetic
from tests.helpers import hooks_lib, oracle_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _launch(ctx, batch, dev, rows):
    import torch

    toks = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    ctx.sample_launch(batch, dev, toks)
    ctx.synchronize()
    torch.cuda.synchronize()
    return toks.cpu().numpy()


def _states(rng, vocab, n):
    dens = np.exp(rng.uniform(np.log(5e-4), np.log(0.5), size=n))
    allowed = np.stack([synthetic.run_mask(rng, vocab, float(d)) for d in dens])
    return allowed, pack_allow_mask(allowed)


def _mixed_params(rng, rows, vocab, hist_len):
    params = []
    for r in range(rows):
        hist = rng.integers(0, vocab, hist_len).tolist()
        kind = r % 8
        if kind == 6:                                                                  # penalties that raise: literal set
            p = SamplingParams(Temperature=0.9, TopK=int(rng.integers(1, 80)), TopP=0.95, RepetitionPenalty=0.85,
                               PresencePenalty=-0.2, PreviousTokens=hist)
        elif kind == 7:                                                                # logit bias: full path, sorted edits
            p = SamplingParams(Temperature=0.8, TopP=0.9, FrequencyPenalty=0.3,
                               LogitBias={int(i): float(rng.normal(0, 2)) for i in rng.integers(0, vocab, 6)},
                               PreviousTokens=hist)
        elif kind == 0:
            p = SamplingParams(Temperature=0.0)                                        # Greedy(masked)
        elif kind == 1:
            p = SamplingParams(Temperature=0.6, TopP=0.95)                             # full path
        elif kind == 2:
            p = SamplingParams(Temperature=0.0, RepetitionPenalty=1.2, PresencePenalty=0.3, PreviousTokens=hist)
        elif kind == 3:
            p = SamplingParams(Temperature=0.8, TopK=int(rng.integers(1, 200)), TopP=0.9, RepetitionPenalty=1.1,
                               FrequencyPenalty=0.2, PreviousTokens=hist)              # selection kernel, history
        elif kind == 4:
            p = SamplingParams(Temperature=0.7, TopP=0.9, MinP=0.02, FrequencyPenalty=0.4, PresencePenalty=0.2,
                               PreviousTokens=hist)                                    # full path, history
        else:
            p = SamplingParams(Temperature=1.0, TopK=int(rng.integers(1, 60)))         # selection kernel
        params.append(p)
    return params


def test_the_device_packer_gives_the_host_packers_bits(ctx):
    import torch

    rng = np.random.default_rng(11)
    for vocab in (1, 31, 64, 65, 4_097, 151_936):
        rows = 5
        x = rng.normal(0, 1, (rows, vocab + 3)).astype(np.float32)
        x[rng.random(x.shape) < 0.6] = -np.inf
        x[0, :] = -np.inf
        if vocab > 40:
            x[1, 3:] = 1.0
        dev = torch.from_numpy(x).cuda()[:, 3:]                           # odd row starts and stride
        got = ctx.pack_allow_mask_launch(dev).cpu().numpy().view(np.uint32)
        want = pack_allow_mask(x[:, 3:] != -np.inf)
        assert np.array_equal(got, want), vocab
        bits = (x[:, 3:].copy().view(np.uint32) >> 16).astype(np.uint16)   # bf16: -inf stays -inf, nothing else becomes it
        devb = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
        gotb = ctx.pack_allow_mask_launch(devb).cpu().numpy().view(np.uint32)
        assert np.array_equal(gotb, pack_allow_mask(bits != 0xff80)), vocab


def test_register_release_and_the_errors(ctx):
    rng = np.random.default_rng(3)
    V = 5_000
    _, words = _states(rng, V, 3)
    ids = [ctx.register_mask(words[i], V) for i in range(3)]
    assert sorted(ids) == [0, 1, 2]
    ctx.release_mask(ids[1])
    assert ctx.register_mask(words[1], V) == ids[1]                       # a freed id is used again
    with pytest.raises(ValueError):
        ctx.release_mask(77)
    with pytest.raises(ValueError):
        ctx.register_mask(words[0][:100], 3_000)                          # another vocabulary while masks are held
    batch = ctx.new_batch()
    with pytest.raises(ValueError):
        batch.upload([SamplingParams(Temperature=0.0)], V, None, mask_ids=[9])       # not registered
    plain = ctx.new_batch().upload([SamplingParams(Temperature=0.0)], V, None)
    with pytest.raises(NotImplementedError):
        plain.append_tokens([1], None, mask_ids=[0])                      # not a batch of mask ids
    for i in ids:
        ctx.release_mask(i)
    assert ctx.register_mask(np.full(100, 0xffffffff, np.uint32), 3_000) == 0        # empty registry: a new vocabulary


@pytest.mark.parametrize("vocab,rows,steps", [(151_936, 32, 6), (20_011, 24, 40)])
def test_constrained_decode_loop_over_registered_states(ctx, vocab, rows, steps):
    import torch

    rng = np.random.default_rng(vocab + rows)
    n_states = 40 if vocab < 100_000 else 7                               # 40: the registry grows past its first 16 slots
    allowed, words = _states(rng, vocab, n_states)
    dev_words = _cuda(words.view(np.int32))
    ids = []
    for s in range(n_states):                                             # from host memory and from device memory
        ids.append(ctx.register_mask(words[s], vocab) if s % 2 == 0 else ctx.register_mask(dev_words[s], vocab))
    logits = synthetic.zipf_head_logits(rng, rows, vocab) if hasattr(synthetic, "zipf_head_logits") else \
        rng.normal(0, 1.5, (rows, vocab)).astype(np.float32)
    dev = _cuda(logits)
    params = _mixed_params(rng, rows, vocab, 24)
    state = rng.integers(-1, n_states, rows)                              # -1: the row is not constrained right now
    u = rng.random(rows)
    batch = ctx.new_batch().upload(params, vocab, u, mask_ids=[ids[s] if s >= 0 else -1 for s in state])

    def masks_of(state):
        m = np.zeros((rows, words.shape[1]), dtype=np.uint32)
        act = np.zeros(rows, dtype=np.uint8)
        for r, s in enumerate(state):
            if s >= 0:
                m[r] = words[s]
                act[r] = 1
        return m, act

    for step in range(steps):
        m, act = masks_of(state)
        got = _launch(ctx, batch, dev, rows)
        want = oracle_tokens(logits, params, u, m, act)
        assert np.array_equal(got, want), (step, np.nonzero(got != want)[0])
        if step % 5 == 0:                                                 # ... and what a fresh upload of the same inputs gives
            fresh = ctx.new_batch().upload(params, vocab, u, m, act)
            assert np.array_equal(_launch(ctx, fresh, dev, rows), want)
            fresh.close()
        # the sampled token joins the row's history (where it has one), every constraint moves to its next state
        for r, p in enumerate(params):
            if p.PreviousTokens is not None:
                p.PreviousTokens = list(p.PreviousTokens) + [int(got[r])]
        tokens = np.array([int(got[r]) if params[r].PreviousTokens is not None else -1 for r in range(rows)], dtype=np.int32)
        stay = rng.random(rows) < 0.3
        state = np.where(stay, state, rng.integers(-1, n_states, rows))
        u = rng.random(rows)
        batch.append_tokens(tokens, u, mask_ids=[ids[s] if s >= 0 else -1 for s in state])
    # the steps were taken in place: only a row that ran out of room for new history ids rebuilds the batch
    assert int(hooks_lib().sr_debug_append_rebuilds(batch.h)) <= steps // 8
    batch.close()
    for i in ids:
        ctx.release_mask(i)


def _allowed_on_device(ctx, mask_id, vocab):
    """Which tokens a registered mask lets through, asked of the sampler itself: row t prefers token t by a wide margin,
    so Greedy(masked row t) == t exactly when t is allowed (the probe of ForcedToolCallConstraintTests.AllowedMask and
    AndTokenConstraintTests.Allowed, through the device)."""
    import torch

    logits = np.zeros((vocab, vocab), dtype=np.float32)
    logits[np.arange(vocab), np.arange(vocab)] = 50.0
    dev = _cuda(logits)
    params = [SamplingParams(Temperature=0.0) for _ in range(vocab)]
    batch = ctx.new_batch().upload(params, vocab, None, mask_ids=[mask_id] * vocab)
    got = _launch(ctx, batch, dev, vocab)
    batch.close()
    return got == np.arange(vocab)


def _one_hot_words(vocab, allow):
    a = np.zeros(vocab, dtype=bool)
    a[list(allow)] = True
    return pack_allow_mask(a)


def test_mask_and_follows_the_and_constraint(ctx):
    """AndTokenConstraintTests.cs: shared token survives, an empty intersection falls back unmasked, dead inners are
    skipped, four inners all contribute (AndTokenConstraint.cs:44-86)."""
    V = 8
    ids = {t: ctx.register_mask(_one_hot_words(V, [t]), V) for t in (0, 1, 2, 3, 4)}
    both = ctx.register_mask(_one_hot_words(V, [2, 4, 5]), V)
    # OverlappingWindows_SharedAllowedToken_Survives
    m = ctx.mask_and([ids[4], ids[4]])
    assert m >= 0 and _allowed_on_device(ctx, m, V).tolist() == [t == 4 for t in range(V)]
    # OverlappingWindows_EmptyIntersection_FallsBackUnmasked / CombineParams_FourSurvivors: no mask at all
    assert ctx.mask_and([ids[2], ids[3]]) == -1
    assert ctx.mask_and([ids[0], ids[1], ids[2], ids[3]]) == -1
    # a dead inner (its Filter returned the input: id -1) is skipped, the others still intersect
    m2 = ctx.mask_and([-1, both, ids[2], -1])
    assert m2 >= 0 and _allowed_on_device(ctx, m2, V).tolist() == [t == 2 for t in range(V)]
    # nothing constraining: no mask; a single survivor: a copy of it
    assert ctx.mask_and([-1, -1]) == -1 and ctx.mask_and([]) == -1
    m3 = ctx.mask_and([both])
    assert m3 not in (both, -1) and _allowed_on_device(ctx, m3, V).tolist() == [t in (2, 4, 5) for t in range(V)]
    with pytest.raises(ValueError):
        ctx.mask_and([ids[0], 99])
    # a wide vocabulary with bits set beyond it: they never count as "a token is left"
    V2_words = np.full((151_936 + 31) // 32, 0, dtype=np.uint32)
    for i in list(ids.values()) + [both, m, m2, m3]:
        ctx.release_mask(i)
    a = V2_words.copy(); a[-1] = 0xffffffff; a[5] = 1 << 7
    b = V2_words.copy(); b[-1] = 0xffff0000; b[5] = 1 << 9
    ia, ib = ctx.register_mask(a, 151_936 - 17), ctx.register_mask(b, 151_936 - 17)
    assert ctx.mask_and([ia, ib]) == -1          # word 4747 overlaps only in bits >= 15, beyond vocab 151,919
    ctx.release_mask(ia)
    ctx.release_mask(ib)


def test_forced_marker_and_trie_masks_through_the_registry(ctx):
    """ForcedToolCallConstraintTests.cs (only the marker is samplable before it), ConstrainedChoiceSamplingTests.cs
    Test16 (:365-378: only token 10 stays legal) and Test2 (:41-64: the illegal top logit 99 loses to token 10)."""
    V = 32
    forced = ctx.register_mask(_one_hot_words(V, [1]), V)
    allowed = _allowed_on_device(ctx, forced, V)
    assert allowed[1] and allowed.sum() == 1
    ctx.release_mask(forced)
    V = 100
    yes = ctx.register_mask(_one_hot_words(V, [10]), V)      # children of the trie's root for AllowedChoices = ["YES"]
    allowed = _allowed_on_device(ctx, yes, V)
    assert allowed[10] and not allowed[0] and not allowed[99] and allowed.sum() == 1
    logits = np.zeros((2, V), dtype=np.float32)
    logits[:, 99] = 9.0                                          # MockHighestLogitForwardPass(99)
    params = [SamplingParams(Temperature=0.0), SamplingParams(Temperature=0.8, TopK=40, TopP=0.95)]
    batch = ctx.new_batch().upload(params, V, [0.0, 0.77], mask_ids=[yes, yes])
    assert _launch(ctx, batch, _cuda(logits), 2).tolist() == [10, 10]
    batch.close()
    ctx.release_mask(yes)
