"""Phase timestamps of the selection kernel, read out of a profiling build of the library.

    python -m opentail.stingray_amd.build --profile
    STINGRAY_SAMPLER_LIB=opentail/stingray_amd/lib/libstingray_sampler_prof.so \\
        python phase_profile.py [full|fp32|bf16] [rows]

The profiling build (-DSR_PROFILE) stamps wall_clock64 (100 MHz) at the phase boundaries of every chunk item and of
every row tail of k_topk_rows; sr_debug_set_profile hands it the array.  This prints, for one launch over the
benchmark's batch: when chunks start and end, what a chunk's phases cost, when row tails start and end, and what the
phases of a tail cost by size of the row's candidate list.  The release library has none of this compiled in.
"""
from __future__ import annotations

import ctypes as C
import sys

import numpy as np

import os

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def main(argv):
    import torch

    from opentail.stingray_amd import SamplerContext, synthetic

    name = argv[1] if len(argv) > 1 else "full"
    rows = int(argv[2]) if len(argv) > 2 else 256
    w = synthetic.config3(rows=rows, bf16=(name == "bf16"), full_chain=(name == "full"))
    stream = torch.cuda.Stream()
    torch.cuda.set_stream(stream)
    ctx = SamplerContext(0)
    if name == "bf16":
        x = torch.from_numpy(w.logits_bf16.view(np.int16)).cuda().view(torch.bfloat16)
    else:
        x = torch.from_numpy(w.logits).cuda()
    batch = ctx.new_batch().upload(w.params, w.vocab, w.uniforms)
    toks = torch.empty(rows, dtype=torch.int32, device="cuda")
    for _ in range(3):
        ctx.sample_launch(batch, x, toks)
    torch.cuda.synchronize()
    # one unit of 16 stamps per chunk item (at most 128 per row) and per row tail
    prof = torch.zeros((rows * 129 + 64, 16), dtype=torch.int64, device="cuda")
    ctx.L.sr_debug_set_profile.argtypes = [C.c_void_p, C.c_void_p]
    rc = ctx.L.sr_debug_set_profile(ctx.h, C.c_void_p(prof.data_ptr()))
    if rc != 0:
        raise SystemExit("this library was not built with --profile (sr_debug_set_profile returned %d)" % rc)
    ctx.sample_launch(batch, x, toks)
    torch.cuda.synchronize()
    p = prof.cpu().numpy().astype(np.float64)

    def us(a):
        return a / 100.0

    chunk = (p[:, 0] > 0) & (p[:, 5] > 0) & (p[:, 15] == 0)
    tail = p[:, 15] > 0
    t0 = p[chunk, 0].min()
    pc, pt = p[chunk], p[tail]
    print("chunk items %d, row tails %d, kernel span %.1f us" % (chunk.sum(), tail.sum(), us(max(pt[:, 15].max(), pc[:, 5].max()) - t0)))
    print("chunks: first start %.1f, last start %.1f; end p50 %.1f p90 %.1f max %.1f" % (
        us(pc[:, 0].min() - t0), us(pc[:, 0].max() - t0), *[us(np.percentile(pc[:, 5], q) - t0) for q in (50, 90, 100)]))
    print("chunk phases, mean us: fold %.2f | stores + bound %.2f | hand-over %.2f | total %.2f" % (
        us(pc[:, 1] - pc[:, 0]).mean(), us(pc[:, 2] - pc[:, 1]).mean(), us(pc[:, 5] - pc[:, 2]).mean(), us(pc[:, 5] - pc[:, 0]).mean()))
    print("tails: work starts min %.1f p50 %.1f max %.1f; ends p50 %.1f p90 %.1f max %.1f" % (
        us(pt[:, 4].min() - t0), us(np.median(pt[:, 4]) - t0), us(pt[:, 4].max() - t0),
        *[us(np.percentile(pt[:, 15], q) - t0) for q in (50, 90, 100)]))
    total = us(pt[:, 15] - pt[:, 4])
    n_c = pt[:, 13]
    phases = [("bound", 4, 1), ("classify", 1, 2), ("gather", 2, 11), ("load", 11, 12), ("history", 12, 5), ("bins", 5, 6),
              ("place", 6, 7), ("rank", 7, 8), ("exp + sum", 8, 9), ("cuts", 9, 10), ("draw", 10, 15)]
    for lo, hi in [(0, 1), (2, 100), (101, 400), (401, 800), (801, 8192)]:
        m = (n_c >= lo) & (n_c <= hi)
        if not m.any():
            continue
        parts = []
        for nm, a_, b_ in phases:
            ok = m & (pt[:, a_] > 0) & (pt[:, b_] > 0)
            if ok.any():
                parts.append("%s %.1f" % (nm, us(pt[ok, b_] - pt[ok, a_]).mean()))
        print("tails with %4d..%4d candidates: n %3d, start %.1f, end %.1f, total %.1f us | %s" % (
            lo, hi, m.sum(), us(pt[m, 4] - t0).mean(), us(pt[m, 15] - t0).mean(), total[m].mean(), ", ".join(parts)))
    print("the longest tails:")
    for i in np.argsort(-total)[:6]:
        parts = ["%s %.1f" % (nm, us(pt[i, b_] - pt[i, a_])) for nm, a_, b_ in phases if pt[i, a_] > 0 and pt[i, b_] > 0]
        print("  candidates %5d, start %.1f, end %.1f, total %.1f us | %s" % (
            n_c[i], us(pt[i, 4] - t0), us(pt[i, 15] - t0), total[i], ", ".join(parts)))
    print("time (us)  chunks running  tails running")
    for b0 in np.arange(0, us(pt[:, 15].max() - t0) + 5, 5.0):
        ac = ((us(pc[:, 0] - t0) < b0 + 5) & (us(pc[:, 5] - t0) > b0)).sum()
        at = ((us(pt[:, 4] - t0) < b0 + 5) & (us(pt[:, 15] - t0) > b0)).sum()
        print("%8.0f %14d %14d" % (b0, ac, at))
    batch.close()
    ctx.close()


if __name__ == "__main__":
    main(sys.argv)
