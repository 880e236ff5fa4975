"""The five benchmark configurations at their full shapes, through the C ABI, every row against the CPU oracle:
token ids, accepted lengths and distributions bit for bit.

  1  one sequence, vocabulary 49,152, 1,000 decode steps: SampleTopK (Sampler.cs:216-357) with a repetition penalty
     over the last 64 tokens; the sampled token joins the history each step (sr_batch_append_tokens, the
     RecentTokens.Add of ContinuousBatchingEngine.cs:650)
  2  64 x 151,936, full-vocabulary path with frequency / presence penalties over 512-token histories
  3  256 x 151,936 as bf16 and as fp32 with the full chain (penalties, top-k, top-p, min-p)
  4  32 x 151,936 under allow-masks, half of the rows greedy
  5  16 rows x 8 drafts x 262,144: the draft distributions and tokens are produced on the device
     (SampleWithDistribution, SpeculativeDecoder.cs:509-513) and handed to the verification
     (SpeculativeDecoder.cs:530-559) without leaving it
"""
import dataclasses

import numpy as np
import pytest

from oracle import binding as orc
from opentail.stingray_amd import SamplerContext, SamplingParams, synthetic
from tests.helpers import oracle_tokens, to_oracle

pytestmark = pytest.mark.gpu


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


def _check_all_rows(ctx, w, dev):
    got, flags = ctx.sample_batch(dev, w.params, w.uniforms, w.allow_mask, w.mask_active, return_flags=True)
    want = oracle_tokens(w.logits, w.params, w.uniforms, w.allow_mask, w.mask_active)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"{w.name}: rows {bad[:8]} differ: gpu {got[bad[:8]]} oracle {want[bad[:8]]} flags {flags[bad[:8]]}"
    return flags


def test_config1_thousand_decode_steps_with_the_sampled_token_appended(ctx):
    import torch

    steps = 1000
    w = synthetic.config1(steps=steps)
    p0 = w.params[0]
    hist = list(p0.PreviousTokens)
    batch = ctx.new_batch().upload([p0], w.vocab, [w.uniforms[0]])
    dev = _cuda(w.logits)
    tok = torch.empty(1, dtype=torch.int32, device="cuda")
    flags = torch.zeros(1, dtype=torch.int32, device="cuda")
    for s in range(steps):
        ctx.sample_launch(batch, dev[s:s + 1], tok, flags)
        ctx.synchronize()
        got = int(tok.cpu().numpy()[0])
        now = dataclasses.replace(p0, PreviousTokens=list(hist))
        want = int(oracle_tokens(w.logits[s:s + 1], [now], [w.uniforms[s]])[0])
        assert got == want, (s, got, want, int(flags.cpu().numpy()[0]))
        hist.append(got)
        if s + 1 < steps:
            batch.append_tokens([got], [w.uniforms[s + 1]])
    batch.close()
    assert len(hist) == 64 + steps


def test_config2_all_64_rows(ctx):
    w = synthetic.config2()
    assert w.rows == 64 and w.vocab == synthetic.QWEN_VOCAB
    flags = _check_all_rows(ctx, w, _cuda(w.logits))
    assert np.all(flags & 4)  # the full-vocabulary path


def test_config3_all_256_rows_bf16(ctx):
    import torch

    w = synthetic.config3(rows=256, bf16=True)
    _check_all_rows(ctx, w, _cuda(w.logits_bf16.view(np.int16), torch.bfloat16))


def test_config3_all_256_rows_fp32_full_chain(ctx):
    w = synthetic.config3(rows=256, bf16=False, full_chain=True)
    flags = _check_all_rows(ctx, w, _cuda(w.logits))
    assert not np.any(flags >> 31)


def test_config4_all_32_rows_under_allow_masks(ctx):
    w = synthetic.config4()
    assert w.rows == 32
    _check_all_rows(ctx, w, _cuda(w.logits))


def test_config5_draft_on_the_device_then_verification(ctx):
    import torch

    w = synthetic.config5()
    L, V = w.extra["n_draft"], w.vocab
    rows = len(w.params)
    assert (rows, L, V) == (16, 8, synthetic.GEMMA_VOCAB)
    draft = _cuda(w.extra["draft_logits"])                      # [rows * L, V]
    q = torch.empty((rows * L, V), dtype=torch.float32, device="cuda")
    toks = torch.empty(rows * L, dtype=torch.int32, device="cuda")
    dbatch = ctx.new_batch().upload([SamplingParams()] * (rows * L), V, w.extra["draft_uniforms"])
    ctx.sample_with_distribution_launch(dbatch, draft, q, toks)  # q and the draft tokens stay on the device
    target = _cuda(w.logits.reshape(rows, L + 1, V))
    vbatch = ctx.new_batch().upload(w.params, V, w.uniforms, uniforms_per_row=L + 1)
    acc = torch.empty(rows, dtype=torch.int32, device="cuda")
    out = torch.empty((rows, L + 1), dtype=torch.int32, device="cuda")
    ctx.spec_verify_launch(vbatch, target, q.view(rows, L, V), toks.view(rows, L), acc, out)
    ctx.synchronize()
    dbatch.close()
    vbatch.close()
    del draft
    acc_h, out_h = acc.cpu().numpy(), out.cpu().numpy()
    q_h, toks_h = q.cpu().numpy().reshape(rows, L, V), toks.cpu().numpy().reshape(rows, L)
    # the draft side: distribution and token of every (row, position) against the oracle
    du = np.asarray(w.extra["draft_uniforms"], dtype=np.float64)
    dl = w.extra["draft_logits"]
    for i in range(rows * L):
        t, d = orc.sample_with_distribution(dl[i], to_oracle(SamplingParams()), orc.Rng(replay=[du[i]]))
        assert t == toks_h.reshape(-1)[i], (i, t, toks_h.reshape(-1)[i])
        assert np.array_equal(d.view(np.uint32), q_h.reshape(rows * L, V)[i].view(np.uint32)), f"draft row {i}: bits differ"
    # the verification
    tl = w.logits.reshape(rows, L + 1, V)
    for r in range(rows):
        wa, wt = orc.spec_verify_row(tl[r], q_h[r], toks_h[r], to_oracle(w.params[r]), orc.Rng(replay=w.uniforms[r]))
        assert acc_h[r] == wa, (r, acc_h[r], wa)
        assert list(out_h[r][: wa + 1]) == list(wt), (r, out_h[r], wt)
        assert np.all(out_h[r][wa + 1:] == -1)
    assert 0 < acc_h.mean() < L  # both outcomes occur: rejections with residual resampling and accepted drafts
