"""GPU box, through the C ABI: what the entry points refuse, with which status and text, and that a context goes on
working afterwards.  The statuses stand for the exceptions of the managed sampler (ArgumentException,
ArgumentNullException: Sampler.cs:121-123, 197, 589-592)."""
import ctypes as C

import numpy as np
import pytest

import opentail.stingray_amd as sa
from opentail.stingray_amd import SamplerContext, SamplingParams
from tests.helpers import oracle_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _cuda(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_refused_calls_report_status_and_text_and_leave_the_context_usable(ctx):
    import torch

    rng = np.random.default_rng(3)
    V = 4_000
    logits = rng.normal(0, 2, (3, V)).astype(np.float32)
    dev = _cuda(logits)
    params = [SamplingParams(Temperature=0.8, TopK=20), SamplingParams(Temperature=0.0), SamplingParams(Temperature=1.0, TopP=0.9)]
    toks = torch.empty(3, dtype=torch.int32, device="cuda")
    L, h = ctx.L, ctx.h
    p = lambda t: C.c_void_p(t.data_ptr())

    # a sampled row without a uniform: ArgumentNullException(rng)
    b = ctx.new_batch().upload(params, V, None)
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_ERR_NULL_ARGUMENT
    assert b"uniform" in L.sr_last_error(h)
    b.close()
    b = ctx.new_batch().upload(params, V, rng.random(3))
    # null tensors, an unknown element type, a row stride shorter than the vocabulary
    assert L.sr_sample_launch(h, b.h, None, sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_ERR_NULL_ARGUMENT
    assert L.sr_sample_launch(h, b.h, p(dev), 7, V, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V - 1, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    assert L.sr_last_error(h) != b""
    # probs shorter than the logits: the ArgumentException of BuildFilteredDistribution
    probs = torch.empty((3, V), dtype=torch.float32, device="cuda")
    assert L.sr_build_distribution_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(probs), V, V - 5) == sa.SR_ERR_INVALID_ARGUMENT
    assert b"must equal logits length" in L.sr_last_error(h)
    # rows that are not SampleTopK rows cannot be named for the sort path; neither can rows outside the batch
    rows = (C.c_int32 * 1)(1)
    assert L.sr_resample_rows_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, rows, 1, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    rows = (C.c_int32 * 1)(3)
    assert L.sr_resample_rows_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, rows, 1, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    # ResampleResidual with different lengths, SampleFromProbs without a generator
    u = (C.c_double * 3)(0.1, 0.2, 0.3)
    assert L.sr_resample_residual_launch(h, p(probs), V, V, p(probs), V - 1, V, 3, u, p(toks)) == sa.SR_ERR_INVALID_ARGUMENT
    assert b"equal length" in L.sr_last_error(h)
    assert L.sr_sample_from_probs_launch(h, p(probs), 3, V, V, None, p(toks)) == sa.SR_ERR_NULL_ARGUMENT
    # a mask stride shorter than the vocabulary needs
    words = np.zeros((3, V // 32 - 1), dtype=np.uint32)
    with pytest.raises(ValueError):
        ctx.new_batch().upload(params, V, rng.random(3), words)
    b.close()
    # nothing above has broken the context
    u3 = rng.random(3)
    assert np.array_equal(ctx.sample_batch(dev, params, u3), oracle_tokens(logits, params, u3))


def test_empty_batches_and_a_single_token_vocabulary(ctx):
    import torch

    empty = torch.empty((0, 100), dtype=torch.float32, device="cuda")
    assert ctx.sample_batch(empty, [], []).size == 0
    one = _cuda(np.array([[0.5], [-2.0]], dtype=np.float32))
    params = [SamplingParams(Temperature=1.0, TopP=0.5), SamplingParams(Temperature=0.7, TopK=1)]
    assert ctx.sample_batch(one, params, [0.3, 0.9]).tolist() == [0, 0]


def test_a_batch_that_names_a_released_or_restarted_mask_is_refused_before_any_launch(ctx):
    """Only status codes are looked at: a launch with a stale id would read outside the pool of masks."""
    import torch

    rng = np.random.default_rng(5)
    V = 3_001
    L, h = ctx.L, ctx.h
    p = lambda t: C.c_void_p(t.data_ptr())
    dev = _cuda(rng.normal(0, 1, (2, V)).astype(np.float32))
    toks = torch.empty(2, dtype=torch.int32, device="cuda")
    probs = torch.empty((2, V), dtype=torch.float32, device="cuda")
    words = rng.integers(1, 2**32, (2, (V + 31) // 32), dtype=np.uint64).astype(np.uint32)
    ids = [ctx.register_mask(words[i], V) for i in range(2)]
    params = [SamplingParams(Temperature=0.8, TopK=20), SamplingParams(Temperature=0.9, TopP=0.9)]
    b = ctx.new_batch().upload(params, V, rng.random(2), mask_ids=ids)
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_OK
    ctx.synchronize()
    # released, and registered again with other bits: the id is the same, the mask is not
    ctx.release_mask(ids[1])
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    assert b"released" in L.sr_last_error(h)
    assert ctx.register_mask(words[0], V) == ids[1]
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    assert L.sr_build_distribution_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(probs), V, V) == sa.SR_ERR_INVALID_ARGUMENT
    # naming the id again (the caller states which mask the row has now) makes the batch good again
    b.append_tokens([-1, -1], rng.random(2), mask_ids=ids)
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_OK
    ctx.synchronize()
    # every mask released and one registered for another vocabulary: the pool starts again, the old batch is stale for good
    for i in ids:
        ctx.release_mask(i)
    other = ctx.register_mask(np.full(40, 0xffffffff, np.uint32), 1_000)
    assert L.sr_sample_launch(h, b.h, p(dev), sa.SR_DTYPE_F32, V, p(toks), None) == sa.SR_ERR_INVALID_ARGUMENT
    t = np.array([-1, -1], dtype=np.int32)
    m = np.array([0, 0], dtype=np.int32)
    assert L.sr_batch_append_tokens_masks(b.h, t.ctypes.data_as(C.POINTER(C.c_int32)), None,
                                          m.ctypes.data_as(C.POINTER(C.c_int32))) == sa.SR_ERR_INVALID_ARGUMENT
    ctx.release_mask(other)
    b.close()
