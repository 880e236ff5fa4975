"""GPU parity, through the C ABI: device expf, row argmax, greedy rows and the top-k-first path
(Sampler.cs:216-357) against the CPU oracle.  Token ids must be bit-exact."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as orc
from opentail.stingray_amd import Sampler, SamplerContext, SamplingParams, pack_allow_mask, synthetic
from tests.helpers import DotnetRandom, ReplayRandom, hooks_lib, oracle_tokens

pytestmark = pytest.mark.gpu
NEG_INF = np.float32("-inf")


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a, dtype=None):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.view(dtype)
    return t.cuda()


def test_device_expf_is_bit_identical_to_the_oracle(ctx):
    import torch

    rng = np.random.default_rng(1)
    xs = np.concatenate([
        -rng.exponential(6.0, 1_500_000), rng.uniform(-104.5, 0.0, 400_000), rng.uniform(0.0, 88.9, 100_000),
        [0.0, -0.0, -87.9, -88.0, -103.0, -103.97, -103.98, -104.0, -1e-10, -1e-38, 88.7, 88.73, -np.inf, np.inf],
    ]).astype(np.float32)
    x = _cuda(xs)
    y = torch.empty_like(x)
    ctx._check(hooks_lib().sr_selftest_expf(ctx.h, C.c_void_p(x.data_ptr()), C.c_void_p(y.data_ptr()), xs.size))
    ctx.synchronize()
    got = y.cpu().numpy()
    lib = orc.lib()
    want = np.array([lib.oracle_expf(C.c_float(v)) for v in xs[:300_000]], dtype=np.float32)
    assert np.array_equal(got[:300_000].view(np.uint32), want.view(np.uint32))
    tail = np.array([lib.oracle_expf(C.c_float(v)) for v in xs[-200_000:]], dtype=np.float32)
    assert np.array_equal(got[-200_000:].view(np.uint32), tail.view(np.uint32))


def test_argmax_matrix(ctx):
    # CudaGpuArgmaxParityTests.cs:56-124: sizes across block boundaries and real vocabularies, maximum
    # at {0, n/2, n-1}, tie -> lower index, all-equal -> 0, all-negative; value returned bit-identical.
    for n in [1, 2, 3, 255, 256, 257, 1000, 65536, 152064, 262144]:
        r = np.random.default_rng(1234 + n)
        a = (r.random(n) * 20 - 10).astype(np.float32)
        rows = [a]
        for pos in (0, n // 2, n - 1):
            b = a.copy()
            b[pos] = 1000.0 + pos
            rows.append(b)
        m = np.stack(rows)
        idx, val = ctx.argmax_rows(_cuda(m))
        for i, row in enumerate(m):
            assert idx[i] == orc.greedy(row)
            assert val[i].tobytes() == row[idx[i]].tobytes()
    a = np.full(5000, -1, dtype=np.float32)
    a[700] = a[300] = 5
    assert ctx.argmax_rows(_cuda(a[None]))[0][0] == 300
    assert ctx.argmax_rows(_cuda(np.full((1, 8192), 3.5, np.float32)))[0][0] == 0
    neg = (-np.random.default_rng(99).random(4096) * 50 - 1).astype(np.float32)
    assert ctx.argmax_rows(_cuda(neg[None]))[0][0] == orc.greedy(neg)
    assert ctx.argmax_rows(_cuda(np.full((1, 64), NEG_INF, np.float32)))[0][0] == 0


def test_argmax_rows_batched_with_ties_and_bf16(ctx):
    import torch

    # CudaGpuArgmaxParityTests.cs:145-173
    for vocab in (1024, 152064):
        for rows in (1, 2, 4, 8):
            r = np.random.default_rng(555 + rows * 31 + vocab)
            flat = (r.random((rows, vocab)) * 10 - 5).astype(np.float32)
            for i in range(rows):
                pos = (i * 37) % vocab
                flat[i, pos] = 50.0 + i
                flat[i, (pos + 50) % vocab] = 50.0 + i
            idx, val = ctx.argmax_rows(_cuda(flat))
            for i in range(rows):
                assert idx[i] == orc.greedy(flat[i]) and val[i] == flat[i, idx[i]]
    bits = synthetic.to_bf16_bits(np.random.default_rng(3).normal(0, 2, (5, 3001)).astype(np.float32))
    up = synthetic.bf16_bits_to_f32(bits)
    idx, val = ctx.argmax_rows(_cuda(bits.view(np.int16), torch.bfloat16))
    for i in range(5):
        assert idx[i] == orc.greedy(up[i]) and val[i] == up[i, idx[i]]


def test_reference_known_answers_through_the_sampler_mirror():
    # SamplerTests.cs restated against the GPU path (any-uniform answers).
    assert Sampler.Greedy([1, 5, 3, 2]) == 1 and Sampler.Greedy([10, 1, 2, 3]) == 0 and Sampler.Greedy([1, 2, 3, 100]) == 3
    assert Sampler.Greedy([]) == 0
    rng = ReplayRandom([0.3])
    assert Sampler.Sample([1, 5, 3, 2], SamplingParams(Temperature=0.0), rng) == 1 and rng.draws == 0
    logits = [10, 9.8, 0]
    pres = SamplingParams(TopK=1, PresencePenalty=1.0, PreviousTokens=[0])
    freq = SamplingParams(TopK=1, FrequencyPenalty=0.6, PreviousTokens=[0, 0])
    for u in (0.0, 0.4, 0.999999):
        assert Sampler.Sample(logits, pres, ReplayRandom([u])) == 1
        assert Sampler.Sample(logits, freq, ReplayRandom([u])) == 1
    # top-k 2 -> only {8, 9}; masks never sampled; all -inf -> index 0 with no draw
    r = DotnetRandom(42)
    seen = {Sampler.Sample(list(range(1, 11)), SamplingParams(TopK=2), r) for _ in range(200)}
    assert seen <= {8, 9} and len(seen) == 2
    masked = [2, NEG_INF, 5, NEG_INF, 1, 3]
    r = DotnetRandom(3)
    for _ in range(200):
        assert masked[Sampler.Sample(masked, SamplingParams(TopK=5, TopP=0.95), r)] != NEG_INF
    rr = ReplayRandom([0.5])
    assert Sampler.Sample([NEG_INF] * 3, SamplingParams(TopK=2, TopP=0.9), rr) == 0
    r = DotnetRandom(2)
    assert {Sampler.Sample([6, 3, 2.5, 0, 0, 0, 0, 0], SamplingParams(TopK=3, TopP=0.5), r) for _ in range(100)} == {0}
    # penalty over-selection (SamplerTests.cs:258-294)
    p = SamplingParams(TopK=2, RepetitionPenalty=4.0, PreviousTokens=[1])
    r = DotnetRandom(5)
    reach = {Sampler.Sample([10, 8, 7, 1, 0], p, r) for _ in range(300)}
    assert 1 not in reach and reach <= {0, 2} and 2 in reach


def _check_rows(ctx, logits_f32, params, uniforms, device_tensor, allow_mask=None, mask_active=None):
    got, flags = ctx.sample_batch(device_tensor, params, uniforms, allow_mask, mask_active, return_flags=True)
    want = oracle_tokens(logits_f32, params, uniforms, allow_mask, mask_active)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"rows {bad[:8]} differ: gpu {got[bad[:8]]} oracle {want[bad[:8]]} flags {flags[bad[:8]]}"
    return flags


def test_small_rows_with_ties_masks_and_every_cut(ctx):
    rng = np.random.default_rng(21)
    for trial in range(40):
        rows = int(rng.integers(1, 9))
        n = int(rng.integers(2, 700))
        logits = (rng.integers(-14, 14, (rows, n)) / 2.0).astype(np.float32)   # coarse grid: many ties
        logits[rng.random((rows, n)) < 0.15] = NEG_INF
        params = []
        for _ in range(rows):
            hist = rng.integers(-3, n + 3, int(rng.integers(0, 12))).tolist()
            params.append(SamplingParams(
                Temperature=float(rng.choice([0.0, 0.5, 1.0, 1.7])), TopK=int(rng.integers(1, n)),
                TopP=float(rng.choice([1.0, 0.9, 0.5])), MinP=float(rng.choice([0.0, 0.05, 0.3])),
                RepetitionPenalty=float(rng.choice([1.0, 1.3])), PresencePenalty=float(rng.choice([0.0, 0.4])),
                FrequencyPenalty=float(rng.choice([0.0, 0.25])), RepeatLastN=int(rng.choice([0, 3, 64])),
                PreviousTokens=hist))
        _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits))


def test_constant_and_quantised_rows(ctx):
    # all-equal rows make every element tie with the threshold: lowest indices must win
    V = 50_000
    logits = np.zeros((3, V), dtype=np.float32)
    logits[1] = 2.5
    logits[2, ::7] = 1.0
    params = [SamplingParams(TopK=50, TopP=0.9), SamplingParams(Temperature=0.0), SamplingParams(TopK=300, Temperature=0.7)]
    for u in (0.0, 0.37, 0.93):
        _check_rows(ctx, logits, params, [u, u, u], _cuda(logits))


def test_config1_shape_many_steps(ctx):
    w = synthetic.config1(steps=200)
    flags = _check_rows(ctx, w.logits, w.params, w.uniforms, _cuda(w.logits))
    assert np.all(flags & 2)   # every row took the top-k-first path


def test_config3_shape_fp32_and_bf16(ctx):
    import torch

    w = synthetic.config3(rows=48, bf16=True)
    _check_rows(ctx, w.logits, w.params, w.uniforms, _cuda(w.logits_bf16.view(np.int16), torch.bfloat16))
    w = synthetic.config3(rows=48, bf16=False)
    _check_rows(ctx, w.logits, w.params, w.uniforms, _cuda(w.logits))


def test_config3_full_chain_with_penalties(ctx):
    w = synthetic.config3(rows=48, bf16=False, full_chain=True)
    _check_rows(ctx, w.logits, w.params, w.uniforms, _cuda(w.logits))


@pytest.mark.parametrize("rows,vocab,kmax", [(120, 20_011, 1000), (150, 20_011, 1000), (200, 151_936, 1000), (256, 20_011, 1000),
                                             (300, 20_011, 1000), (520, 9_973, 1000),
                                             (3, 49_152, 50), (120, 20_011, 64), (150, 20_011, 30), (256, 151_936, 64), (300, 20_011, 8)])
def test_every_shape_of_the_launch_gives_the_oracles_tokens(ctx, rows, vocab, kmax):
    # The host picks the launch's shape from the number of rows: rows dealt out chunk by chunk over all workers (few
    # rows), one worker per row that keeps the chunk results in its registers (from about half the compute units'
    # number of rows up to one row per compute unit), one worker per row that writes them out (more rows).  Rows of
    # every kind in each: greedy with and without penalties, top-k 1 .. 1000 with top-p / min-p, histories that lower
    # and that raise, coarse values (ties at every cut), rows with a handful of finite logits.  A batch whose rows all
    # ask for at most 64 entries (kmax) takes the launches that carry the steps for short lists.
    import torch

    rng = np.random.default_rng(rows * 7 + vocab)
    logits = synthetic.zipf_head_logits(rng, rows, vocab)
    logits[1::5] = np.round(logits[1::5] * 4) / 4                      # quantised rows: ties
    logits[2::17, :] = NEG_INF
    for r in range(2, rows, 17):
        logits[r, rng.integers(0, vocab, 5)] = rng.normal(0, 1, 5).astype(np.float32)
    params = []
    for r in range(rows):
        hist = rng.integers(0, vocab, int(rng.integers(1, 70))).tolist()
        kind = r % 6
        k = int(rng.integers(1, min(kmax + 1, vocab)))
        if kind == 0:
            p = SamplingParams(Temperature=0.0)
        elif kind == 1:
            p = SamplingParams(Temperature=0.0, RepetitionPenalty=1.3, FrequencyPenalty=0.2, PreviousTokens=hist)
        elif kind == 2:
            p = SamplingParams(Temperature=float(rng.uniform(0.3, 1.5)), TopK=k, TopP=float(rng.uniform(0.5, 1.0)))
        elif kind == 3:
            p = SamplingParams(Temperature=float(rng.uniform(0.3, 1.5)), TopK=k, TopP=0.9, MinP=0.02, RepetitionPenalty=1.1,
                               PresencePenalty=0.3, FrequencyPenalty=0.1, PreviousTokens=hist)
        elif kind == 4:
            p = SamplingParams(Temperature=0.8, TopK=min(k, 200), RepetitionPenalty=0.8, PresencePenalty=-0.2,
                               PreviousTokens=hist if kmax > 64 else hist[:3])  # penalties that raise: the literal over-selection
        else:
            p = SamplingParams(Temperature=1.0, TopK=k, MinP=0.1)
        params.append(p)
    u = rng.random(rows)
    flags = _check_rows(ctx, logits, params, u, _cuda(logits))
    assert np.all(flags & 3)                                          # greedy or top-k-first: the selection kernel
    bits = synthetic.to_bf16_bits(logits)
    _check_rows(ctx, synthetic.bf16_bits_to_f32(bits), params, u, _cuda(bits.view(np.int16), torch.bfloat16))


def test_top_k_under_an_allow_mask_and_unaligned_rows(ctx):
    import torch

    rng = np.random.default_rng(8)
    V = 30_011                                            # odd vocabulary: rows are not 16-byte aligned
    logits = rng.normal(0, 1.5, (6, V)).astype(np.float32)
    allowed = np.stack([synthetic.run_mask(rng, V, d) for d in (0.001, 0.01, 0.1, 0.5, 0.9, 0.0005)])
    params = [SamplingParams(Temperature=0.9, TopK=int(k), TopP=0.95) for k in (1, 5, 40, 400, 1000, 64)]
    params[2].Temperature = 0.0
    mask = pack_allow_mask(allowed)
    active = np.array([1, 1, 1, 1, 0, 1], dtype=np.uint8)
    _check_rows(ctx, logits, params, rng.random(6), _cuda(logits), mask, active)
    # a strided view: row stride larger than the vocabulary
    big = torch.zeros((6, V + 37), dtype=torch.float32, device="cuda")
    big[:, :V] = _cuda(logits)
    _check_rows(ctx, logits, params, rng.random(6), big[:, :V], mask, active)


def test_round_trip_properties_at_full_size(ctx):
    # size-independent properties at the benchmark shape: every token is inside its row's top-k set and,
    # for greedy rows, is the row argmax; re-running with the same uniforms is deterministic.
    import torch

    w = synthetic.config3(rows=256, bf16=False)
    x = _cuda(w.logits)
    t1 = ctx.sample_batch(x, w.params, w.uniforms)
    t2 = ctx.sample_batch(x, w.params, w.uniforms)
    assert np.array_equal(t1, t2)
    kth = torch.topk(x, 1000, dim=1).values.cpu().numpy()
    am, _ = ctx.argmax_rows(x)
    for i, p in enumerate(w.params):
        if p.Temperature <= 0:
            assert t1[i] == am[i]
        else:
            assert w.logits[i, t1[i]] >= kth[i, p.TopK - 1]


def test_penalties_that_raise_a_logit_keep_the_reference_over_selection(ctx):
    # Sampler.cs:224-225 only ever looks at the raw top-(k + history length): a history token outside that
    # set is not considered even when a negative penalty would lift it to the top.
    logits = np.array([[10, 9, 8, 1, 0, -1, -2, -3]], dtype=np.float32)
    p = SamplingParams(TopK=1, PresencePenalty=-20.0, PreviousTokens=[3])
    for u in (0.0, 0.5, 0.99):
        assert _check_rows(ctx, logits, [p], [u], _cuda(logits))[0] & 2
    rng = np.random.default_rng(31)
    V, rows = 40_000, 16
    logits = rng.normal(0, 2.0, (rows, V)).astype(np.float32)
    head = np.argsort(-logits, axis=1)
    params = []
    for i, k in enumerate([1, 5, 40, 64, 65, 200, 700, 1500, 3, 64, 65, 300, 33, 1, 900, 128]):
        n_hist = int(rng.integers(20, 300))
        hist = np.concatenate([head[i, rng.integers(0, 2 * k + 50, n_hist // 2)], rng.integers(0, V, n_hist - n_hist // 2)])
        rng.shuffle(hist)
        params.append(SamplingParams(
            Temperature=float(rng.choice([0.0, 0.7, 1.2])) if i % 5 == 4 else float(rng.uniform(0.6, 1.3)), TopK=k,
            TopP=float(rng.choice([1.0, 0.9])), MinP=float(rng.choice([0.0, 0.02])),
            RepetitionPenalty=float(rng.choice([0.7, 1.0, 1.3])), PresencePenalty=float(rng.choice([-0.8, 0.0, 0.5])),
            FrequencyPenalty=float(rng.choice([-0.3, 0.0, 0.2])), RepeatLastN=int(rng.choice([0, 16, 64])),
            PreviousTokens=hist.tolist()))
    for _ in range(3):
        _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits))


def test_large_values_concentrated_in_few_lanes(ctx):
    # the per-wave bound comes from lane-group maxima: put every large value into 16 lanes of a wave so the bound
    # is loose and the exact per-wave selection has to take over
    rng = np.random.default_rng(32)
    V, rows = 40_000, 8
    logits = rng.normal(0, 1.0, (rows, V)).astype(np.float32)
    e = np.arange(V)
    hot = ((e // 4) % 512) < 16
    logits[:, hot] += 40.0 + rng.random((rows, int(hot.sum()))).astype(np.float32)
    params = [SamplingParams(Temperature=float(t), TopK=int(k), TopP=0.97)
              for t, k in zip([1.0, 0.8, 1.3, 0.0, 1.0, 0.9, 1.1, 1.0], [64, 64, 40, 1, 7, 64, 33, 200])]
    params[1].PreviousTokens = np.nonzero(hot)[0][:120].tolist()
    params[1].RepetitionPenalty = 1.2
    _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits))


def test_large_values_concentrated_in_few_lanes_with_a_worker_per_row(ctx):
    # The same with enough rows for the launch in which every worker keeps its row's results and takes one share of
    # the bound per wave and row, from one value per lane and chunk: the large values of a row lie in sixteen lanes of
    # one wave, in one lane, or in one lane's vectors of one group, so that a lane counts once for many of them and
    # the wave's share falls far below the row's k-th largest (the exact selection has to take over), for top-k of
    # every size, greedy rows and rows with a history.  fp32 and bf16.
    import torch

    rng = np.random.default_rng(36)
    V, rows = 40_000, 150
    logits = rng.normal(0, 1.0, (rows, V)).astype(np.float32)
    e = np.arange(V)
    vec = e // 4
    kinds = [(vec % 512) < 16, (vec % 512) == 77, ((vec % 512) == 300) & ((vec // 512) % 4 == 1), (vec % 512) >= 448]
    params = []
    for r in range(rows):
        hot = kinds[r % 4]
        logits[r, hot] += 40.0 + rng.random(int(hot.sum())).astype(np.float32)
        k = int(rng.choice([1, 2, 7, 40, 64, 65, 200, 500, 1000]))
        if r % 11 == 0:
            params.append(SamplingParams(Temperature=0.0))
        elif r % 11 == 1:
            params.append(SamplingParams(Temperature=0.9, TopK=k, TopP=0.97, RepetitionPenalty=1.2, FrequencyPenalty=0.1,
                                         PreviousTokens=np.nonzero(hot)[0][:100].tolist()))
        else:
            params.append(SamplingParams(Temperature=float(rng.uniform(0.5, 1.4)), TopK=k, TopP=float(rng.choice([1.0, 0.97])),
                                         MinP=float(rng.choice([0.0, 0.01]))))
    u = rng.random(rows)
    _check_rows(ctx, logits, params, u, _cuda(logits))
    bits = synthetic.to_bf16_bits(logits)
    _check_rows(ctx, synthetic.bf16_bits_to_f32(bits), params, u, _cuda(bits.view(np.int16), torch.bfloat16))


def test_flat_rows_with_a_history(ctx):
    # every logit equal: the candidates all tie, the lowest indices win, and the penalised history ids drop out
    V = 50_000
    rng = np.random.default_rng(33)
    logits = np.zeros((3, V), dtype=np.float32)
    logits[2] = 1.25
    hist = rng.integers(0, 3000, 300).tolist()
    params = [SamplingParams(Temperature=1.0, TopK=1200, TopP=0.999, RepetitionPenalty=1.2, PreviousTokens=hist),
              SamplingParams(Temperature=1.5, TopK=60, PresencePenalty=0.5, PreviousTokens=hist),
              SamplingParams(Temperature=0.0, FrequencyPenalty=0.25, PreviousTokens=list(range(0, 40)))]
    for u in (0.0, 0.31, 0.77, 0.9999):
        _check_rows(ctx, logits, params, [u, u, u], _cuda(logits))


def test_history_on_unaligned_rows_and_bf16(ctx):
    import torch

    rng = np.random.default_rng(34)
    V, rows = 30_011, 6                                   # odd vocabulary: every row starts at another offset
    logits = rng.normal(0, 1.5, (rows, V)).astype(np.float32)
    head = np.argsort(-logits, axis=1)
    params = []
    for i, k in enumerate([1, 20, 64, 65, 400, 1000]):
        hist = np.concatenate([head[i, :30], rng.integers(0, V, 100)]).tolist()
        params.append(SamplingParams(Temperature=0.9 if i != 2 else 0.0, TopK=k, TopP=0.95, RepetitionPenalty=1.15,
                                     FrequencyPenalty=0.1, PreviousTokens=hist))
    allowed = np.stack([synthetic.run_mask(rng, V, d) for d in (0.5, 0.9, 0.3, 0.01, 0.8, 0.6)])
    mask = pack_allow_mask(allowed)
    _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits))
    _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits), mask, np.array([1, 0, 1, 1, 1, 0], dtype=np.uint8))
    bits = synthetic.to_bf16_bits(logits)
    up = synthetic.bf16_bits_to_f32(bits)
    _check_rows(ctx, up, params, rng.random(rows), _cuda(bits.view(np.int16), torch.bfloat16))
    w = synthetic.config3(rows=32, bf16=True, full_chain=True)
    _check_rows(ctx, w.logits, w.params, w.uniforms, _cuda(w.logits_bf16.view(np.int16), torch.bfloat16))


def test_vocabularies_of_more_than_four_chunks_per_row(ctx):
    # beyond 155,648 fp32 (327,680 bf16) elements a row takes more than four chunk workgroups and the row tail
    # works from the group maxima alone: histories, masks, boosts, greedy rows, ties
    import torch

    rng = np.random.default_rng(35)
    V, rows = 262_144, 8
    logits = rng.normal(0, 1.5, (rows, V)).astype(np.float32)
    logits[6] = np.round(logits[6] * 2) / 2               # heavily tied
    logits[7] = 0.5                                       # flat
    head = np.argsort(-logits, axis=1)
    ks = [1, 40, 64, 500, 1000, 1, 300, 50]
    params = []
    for i, k in enumerate(ks):
        hist = np.concatenate([head[i, :20], rng.integers(0, V, 44)]).tolist()
        params.append(SamplingParams(Temperature=0.0 if i == 5 else float(rng.uniform(0.6, 1.4)), TopK=k,
                                     TopP=float(rng.choice([1.0, 0.9])), MinP=float(rng.choice([0.0, 0.02])),
                                     RepetitionPenalty=1.1, PresencePenalty=0.1 if i != 3 else -0.4,
                                     PreviousTokens=hist if i != 0 else []))
    allowed = np.stack([synthetic.run_mask(rng, V, d) for d in (0.5, 0.9, 0.3, 0.6, 0.8, 0.6, 0.7, 0.2)])
    mask = pack_allow_mask(allowed)
    for _ in range(2):
        _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits))
    _check_rows(ctx, logits, params, rng.random(rows), _cuda(logits), mask, np.array([1, 0, 1, 1, 1, 1, 0, 1], dtype=np.uint8))
    Vb = 400_003                                          # bf16, unaligned rows, 10 chunks
    lb = rng.normal(0, 1.5, (4, Vb)).astype(np.float32)
    bits = synthetic.to_bf16_bits(lb)
    up = synthetic.bf16_bits_to_f32(bits)
    hb = np.argsort(-up, axis=1)
    pb = [SamplingParams(Temperature=0.9 if i != 1 else 0.0, TopK=k, TopP=0.95, RepetitionPenalty=1.2,
                         PreviousTokens=hb[i, :25].tolist() + rng.integers(0, Vb, 30).tolist())
          for i, k in enumerate([5, 1, 200, 900])]
    _check_rows(ctx, up, pb, rng.random(4), _cuda(bits.view(np.int16), torch.bfloat16))


def test_decode_loop_that_uploads_the_batch_again_every_step_without_waiting(ctx):
    # Each step's parameters (the histories grow by the sampled token) are uploaded through the same batch object
    # right behind the previous step's launch; nothing is waited for until the end.
    import torch

    rng = np.random.default_rng(91)
    rows, V, steps = 24, 20_000, 20
    logits = [rng.normal(0, 2.0, (rows, V)).astype(np.float32) for _ in range(3)]
    dev = [_cuda(x) for x in logits]
    hist = [rng.integers(0, V, int(rng.integers(0, 30))).tolist() for _ in range(rows)]
    base = [SamplingParams(Temperature=float(rng.choice([0.0, 0.7, 1.0])), TopK=int(rng.choice([1, 20, 200])),
                           TopP=float(rng.choice([1.0, 0.9])), MinP=float(rng.choice([0.0, 0.02])),
                           RepetitionPenalty=float(rng.choice([1.0, 1.3])), PresencePenalty=float(rng.choice([0.0, 0.4])),
                           RepeatLastN=int(rng.choice([0, 8, 64]))) for _ in range(rows)]
    uniforms = rng.random((steps, rows))
    # the whole sequence from the oracle first
    want, per_step_params = [], []
    for s in range(steps):
        ps = [SamplingParams(**{**p.__dict__, "PreviousTokens": list(hist[r])}) for r, p in enumerate(base)]
        per_step_params.append(ps)
        t = oracle_tokens(logits[s % 3], ps, uniforms[s])
        want.append(t)
        for r in range(rows):
            hist[r].append(int(t[r]))
    batch = ctx.new_batch()
    outs = [torch.full((rows,), -9, dtype=torch.int32, device="cuda") for _ in range(steps)]
    for s in range(steps):
        batch.upload(per_step_params[s], V, uniforms[s])
        ctx.sample_launch(batch, dev[s % 3], outs[s])
    ctx.synchronize()
    torch.cuda.synchronize()
    batch.close()
    for s in range(steps):
        assert np.array_equal(outs[s].cpu().numpy(), want[s]), f"step {s}"


def test_launches_are_ordered_behind_torch_work_on_the_default_stream(ctx):
    # torch's default stream has the handle 0; the context must still run on that stream, not on a stream of its
    # own that nothing orders behind the kernels producing the logits.  The logits arrive behind some milliseconds
    # of queued work and are sampled without a wait in between.
    import torch

    rng = np.random.default_rng(77)
    rows, n = 8, 5000
    lg = rng.normal(0, 3, (rows, n)).astype(np.float32)
    params = [SamplingParams(Temperature=0.0) for _ in range(rows // 2)] + \
             [SamplingParams(Temperature=0.7, TopK=40) for _ in range(rows - rows // 2)]
    u = rng.random(rows)
    want = oracle_tokens(lg, params, u)
    src = _cuda(lg)
    junk = torch.zeros(1 << 27, dtype=torch.float32, device="cuda")
    for attempt in range(3):
        dev = torch.zeros((rows, n), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        for _ in range(30):
            junk.add_(1.0)
        dev.copy_(src)
        got = ctx.sample_batch(dev, params, u)
        assert np.array_equal(got, want), attempt
        probs = ctx.build_distribution(dev, params[rows // 2:] + params[:rows // 2])
        assert float(probs.sum()) == pytest.approx(rows, rel=1e-4)


def test_bf16_rows_of_few_distinct_values_draw_the_right_index_inside_a_run(ctx):
    """bf16 rows that no penalty touches are ranked by value only (one bin per distinct value) and the draw's entry is
    picked from its run of equal values by index at the end: rows of 12 to 200 distinct values, so that the top-k cut,
    the top-p cut and the draw all fall inside runs of dozens of equal logits; also 160 rows (one worker per row with
    its results in registers), masks, and -0 beside +0."""
    import torch

    rng = np.random.default_rng(77)
    V = 60_000
    for rows, n_vals in ((40, 12), (40, 200), (160, 60)):
        levels = np.sort(rng.normal(0, 2.0, n_vals)).astype(np.float32)
        # few entries at the top levels, many below: a run at the cut holds dozens of entries
        pick = np.minimum((rng.exponential(0.12, (rows, V)) * n_vals).astype(np.int64), n_vals - 1)
        logits = levels[n_vals - 1 - pick]
        if n_vals == 12:
            logits[0, :5000] = np.float32(-0.0)
            logits[0, 5000:9000] = np.float32(0.0)
        bits = synthetic.to_bf16_bits(logits)
        up = synthetic.bf16_bits_to_f32(bits)
        params = [SamplingParams(Temperature=float(rng.uniform(0.5, 1.6)), TopK=int(rng.integers(1, 1000)),
                                 TopP=float(rng.choice([1.0, 0.9, 0.6])), MinP=float(rng.choice([0.0, 0.0, 0.02])))
                  for _ in range(rows)]
        allowed = rng.random((rows, V)) < 0.7
        mask = pack_allow_mask(allowed)
        active = (np.arange(rows) % 3 == 0).astype(np.uint8)
        for rep in range(3):
            u = rng.random(rows)
            _check_rows(ctx, up, params, u, _cuda(bits.view(np.int16), torch.bfloat16), mask, active)
