"""sr_argmax_rows_launch_noalloc -- the row argmax (Sampler.Greedy, Sampler.cs:442-446) for callers that cannot
allocate device memory -- gives bit for bit what sr_argmax_rows_launch gives, call after call on the scratch that
all calls on a GPU share: a second call with a smaller input right after a larger one, odd row starts that take
the element-wise loads, bf16, and the size limit reported as an error."""
import ctypes as C

import numpy as np
import pytest

import opentail.stingray_amd as sa
from opentail.stingray_amd import SamplerContext
from oracle import binding as orc

pytestmark = pytest.mark.gpu
MAX_ROWS = 16384


@pytest.fixture()
def ctx():
    c = SamplerContext(0)
    yield c
    c.close()


def _both(ctx, dev):
    """(idx, val) from the allocating entry point and from the one that allocates nothing."""
    import torch

    rows = dev.shape[0]
    outs = []
    for noalloc in (False, True):
        idx = torch.full((rows,), -3, dtype=torch.int32, device="cuda")
        val = torch.full((rows,), 7.0, dtype=torch.float32, device="cuda")
        outs.append(ctx.argmax_rows(dev, out=(idx, val), noalloc=noalloc))
    return outs


def _logits(rng, rows, vocab):
    m = rng.normal(0, 2, (rows, vocab)).astype(np.float32)
    m[:, ::53] = np.round(m[:, ::53])                    # ties
    if rows > 2 and vocab > 10:
        m[1, :] = -1.5                                   # a constant row: index 0
        m[2, vocab // 2] = np.nan                        # a NaN wins outright
    return m


def test_two_calls_in_a_row_the_second_smaller_match_the_allocating_entry_point(ctx):
    import torch

    rng = np.random.default_rng(2024)
    big = _logits(rng, 96, 151_936)       # rows split over several workgroups: slots and counters in use
    small = _logits(rng, 5, 40_000)       # fewer rows, fewer chunks: must not see what the first call left
    for m in (big, small, big[:7], small[:1]):
        dev = torch.from_numpy(m).cuda()
        (i0, v0), (i1, v1) = _both(ctx, dev)
        assert np.array_equal(i0, i1) and np.array_equal(v0.view(np.uint32), v1.view(np.uint32))
        want = np.array([orc.greedy(r) for r in m])
        assert np.array_equal(i1, want)
    # the same call twice more: the scratch is left as it was found
    dev = torch.from_numpy(big).cuda()
    a = ctx.argmax_rows(dev, noalloc=True)
    b = ctx.argmax_rows(dev, noalloc=True)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


def test_rows_that_do_not_start_on_16_bytes_bf16_and_single_chunk_rows(ctx):
    import torch

    rng = np.random.default_rng(7)
    wide = torch.from_numpy(_logits(rng, 9, 50_001 + 3)).cuda()
    view = wide[:, 3:]                                    # rows start 12 bytes past a 16-byte boundary, odd stride
    (i0, v0), (i1, v1) = _both(ctx, view)
    assert np.array_equal(i0, i1) and np.array_equal(v0.view(np.uint32), v1.view(np.uint32))
    assert np.array_equal(i1, np.array([orc.greedy(r) for r in view.cpu().numpy()]))
    bits = (rng.normal(0, 1, (33, 70_007)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    dev = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
    (i0, v0), (i1, v1) = _both(ctx, dev)
    assert np.array_equal(i0, i1) and np.array_equal(v0.view(np.uint32), v1.view(np.uint32))
    f = (bits.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(i1, np.array([orc.greedy(r) for r in f]))
    many = torch.from_numpy(_logits(rng, 3000, 700)).cuda()   # one chunk per row: no slots at all
    (i0, v0), (i1, v1) = _both(ctx, many)
    assert np.array_equal(i0, i1) and np.array_equal(v0.view(np.uint32), v1.view(np.uint32))
    assert np.array_equal(i1, many.cpu().numpy().argmax(1))


def test_calls_on_a_fresh_context_take_no_device_memory(ctx):
    """Free device memory as the driver reports it (the whole device's, not torch's pool) is the same before and after
    calls of several shapes on a context that has served nothing else."""
    import torch

    rng = np.random.default_rng(11)
    devs = [torch.from_numpy(_logits(rng, r, v)).cuda() for r, v in ((64, 151_936), (7, 40_000), (2000, 700))]
    outs = [(torch.empty(d.shape[0], dtype=torch.int32, device="cuda"), torch.empty(d.shape[0], dtype=torch.float32, device="cuda"))
            for d in devs]
    outs[0][0].cpu()  # (whatever torch sets up for its first download is there before the measurement)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        for d, o in zip(devs, outs):
            ctx.argmax_rows(d, out=o, noalloc=True)
    ctx.synchronize()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0


def test_more_rows_than_the_static_scratch_holds_is_an_error_not_a_fault(ctx):
    import torch

    dev = torch.zeros((MAX_ROWS + 1, 8), dtype=torch.float32, device="cuda")
    idx = torch.zeros(MAX_ROWS + 1, dtype=torch.int32, device="cuda")
    rc = ctx.L.sr_argmax_rows_launch_noalloc(ctx.h, C.c_void_p(dev.data_ptr()), 0, MAX_ROWS + 1, 8, 8,
                                             C.c_void_p(idx.data_ptr()), None)
    assert rc == sa.SR_ERR_INVALID_ARGUMENT
    assert b"static scratch holds" in ctx.L.sr_last_error(ctx.h)
    dev = torch.from_numpy(np.arange(MAX_ROWS * 8, dtype=np.float32).reshape(MAX_ROWS, 8) % 7).cuda()
    got = ctx.argmax_rows(dev, noalloc=True)[0]              # exactly the limit is served
    assert np.array_equal(got, dev.cpu().numpy().argmax(1))
