#!/usr/bin/env python3
"""Benchmark of the MI355X token-sampling path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One "step" = one batched sampling call (sr_sample_launch / sr_spec_verify_launch) over a batch of
seeded synthetic logits that are already resident in HBM.  Distinct logits buffers are rotated, enough of them to
exceed the 256 MB Infinity Cache (4 x 155.6 MB for the headline; 8 for c2, 16 for c4; c1 is measured warm and the line
says so), so every step streams cold data.  Prints ONE JSON line.
The default run times c3_fp32_full for K steps and then, in short windows of their own, the other
configurations (c1, c2, c3_bf16, c4, c5): their figures are the "per_config" object of the same line.
Every measured launch is checked against the CPU oracle outside the timed regions, every row of it.

Workloads (opentail/stingray_amd/synthetic.py):
  c3_fp32_full  (default) batch 256 x vocab 151,936 fp32, heterogeneous top-k U{1..1000} / top-p / T,
                10% greedy rows, plus min-p and repetition/presence/frequency penalties over a 64-token
                history: the "full chain" the throughput target is quoted on.
  c3_bf16       the same rows stored as bf16, no penalties (configuration 3 as written)
  c3_fp32       fp32, no penalties
  c1            batch 1 x vocab 49,152 (us/step is the figure of interest)
  c2, c4        full-vocabulary path (batch 64 / batch 32 with allow-masks)
  c5            speculative verification, batch 16 x 8 drafts x vocab 262,144 (sr_spec_verify_launch)
  argmax        Sampler.Greedy per row of 256 x 151,936 fp32 (sr_argmax_rows_launch)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak


def make_workload(name: str, rows: int = 256):
    from opentail.stingray_amd import synthetic

    if name == "c3_fp32_full":
        return synthetic.config3(rows=rows, bf16=False, full_chain=True)
    if name == "c3_fp32":
        return synthetic.config3(rows=rows, bf16=False)
    if name == "c3_bf16":
        return synthetic.config3(rows=rows, bf16=True)
    if name == "c1":
        return synthetic.config1(steps=1)
    if name == "c2":
        return synthetic.config2()
    if name == "c4":
        return synthetic.config4()
    if name == "c5":
        return synthetic.config5()
    raise SystemExit(f"unknown workload {name}")


def host_description() -> dict:
    """CPU model and core count of the box the baseline runs on, and whether a .NET runtime is there."""
    import shutil

    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    dotnet = shutil.which("dotnet")
    return {"cpu_model": model, "nproc": os.cpu_count(), "dotnet": dotnet,
            "note": ("dotnet found at %s, but the managed shim is not built here" % dotnet) if dotnet else
                    "no .NET runtime on this box: the C restatement of the reference sampler is the baseline"}


def cpu_baseline(w, budget_s: float):
    """The CPU oracle (a C restatement of the reference sampler) on one core, rows in order, same inputs.  A step is
    the whole batch.  At least 10 warm-up steps (fewer only when they alone would take longer than the budget), then
    the median of at least 5 timed steps, as many as the budget allows."""
    from oracle import binding as orc
    from tests.helpers import to_oracle

    params = [to_oracle(p) for p in w.params]
    u = np.asarray(w.uniforms, dtype=np.float64).reshape(w.rows, -1)[:, 0].copy()

    def one_step():
        t0 = time.perf_counter()
        orc.sample_batch(w.logits, params, u, w.allow_mask, w.mask_active)
        return time.perf_counter() - t0

    first = one_step()
    n_warm = 10 if first * 10 <= budget_s else max(1, int(budget_s / max(first, 1e-9)) // 2)
    for _ in range(n_warm - 1):
        one_step()
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_all < budget_s and len(times) < 2000):
        times.append(one_step())
    med = float(np.median(times))
    return w.rows / med, n_warm, len(times), med


def prime_events(torch, stream):
    """Warm-up of the event machinery.  The first timing event that a process records on a stream has been seen to
    slow the launches queued behind it down (220 us instead of 53 us per launch for that first window only, in any
    process but the first on a machine), so a pair is recorded and resolved before the warm-up steps."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    e1.record(stream)
    torch.cuda.synchronize()
    e0.elapsed_time(e1)


def bench_spec(args, w, ctx, stream) -> dict:
    """Speculative verification: target logits [rows, L+1, V], draft distributions [rows, L, V] and draft
    tokens resident; two distinct input sets are rotated (2 x 285 MB exceeds the Infinity Cache)."""
    import torch

    from opentail.stingray_amd import SamplingParams
    from oracle import binding as orc
    from tests.helpers import to_oracle

    L = w.extra["n_draft"]
    rows = len(w.params)
    V = w.vocab
    sets = []
    for k in range(2):
        draft = torch.from_numpy(np.roll(w.extra["draft_logits"], k * 3, axis=0)).cuda()
        q = ctx.build_distribution(draft, [SamplingParams()] * (rows * L))          # q = softmax(draft)
        toks = torch.from_numpy(ctx.sample_from_probs(q, w.extra["draft_uniforms"])).cuda().reshape(rows, L)
        target = torch.from_numpy(np.roll(w.logits.reshape(rows, L + 1, V), k, axis=0)).cuda()
        batch = ctx.new_batch().upload(w.params, V, w.uniforms, uniforms_per_row=L + 1)
        acc = torch.empty(rows, dtype=torch.int32, device="cuda")
        out = torch.empty((rows, L + 1), dtype=torch.int32, device="cuda")
        sets.append((target, q.reshape(rows, L, V), toks.contiguous(), batch, acc, out))
    import ctypes as C

    def step(i):
        t, q, k, b, acc, out = sets[i % 2]
        ctx._check(ctx.L.sr_spec_verify_launch(ctx.h, b.h, C.c_void_p(t.data_ptr()), C.c_void_p(q.data_ptr()),
                                               C.c_void_p(k.data_ptr()), L, C.c_void_p(acc.data_ptr()),
                                               C.c_void_p(out.data_ptr())))

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    if args.copy_probe:
        probe = torch.empty_like(sets[0][0])
        for _ in range(3):
            probe.copy_(sets[0][0])   # reads and writes rows * (L + 1) * V * 4 bytes
        torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        step(i)
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_us = ev0.elapsed_time(ev1) * 1e3 / args.steps

    t, q, k, b, acc, out = sets[0]
    acc_h, out_h = acc.cpu().numpy(), out.cpu().numpy()
    parity = None
    if not args.no_parity:
        n_chk = rows
        tn, qn, kn = t[:n_chk].cpu().numpy(), q[:n_chk].cpu().numpy(), k[:n_chk].cpu().numpy()
        bad = 0
        for r in range(n_chk):
            wa, wt = orc.spec_verify_row(tn[r], qn[r], kn[r], to_oracle(w.params[r]), orc.Rng(replay=w.uniforms[r]))
            bad += int(wa != acc_h[r] or list(wt) != list(out_h[r][: wa + 1]))
        parity = {"rows_checked": n_chk, "mismatches": bad}
    cpu = None
    if args.cpu_seconds > 0:
        tn, qn, kn = t[:4].cpu().numpy(), q[:4].cpu().numpy(), k[:4].cpu().numpy()
        c0 = time.perf_counter()
        done = 0
        while time.perf_counter() - c0 < args.cpu_seconds and done < 64:
            r = done % 4
            orc.spec_verify_row(tn[r], qn[r], kn[r], to_oracle(w.params[r]), orc.Rng(replay=w.uniforms[r]))
            done += 1
        el = time.perf_counter() - c0
        cpu = {"value": done / el, "unit": "rows/s", "cores": 1, "kind": "port",
               "sample": f"{done} row verifications (8 drafts each) of the same workload on one thread, {el:.1f} s"}
    # the target logits of the L verified positions once, one draft distribution per row (the position of the first
    # rejection) and the gathers of q at the draft tokens
    alg_bytes = rows * L * V * 4 + rows * V * 4 + rows * L * 4
    bytes_with_bonus = rows * (L + 1) * V * 4 + rows * V * 4 + rows * L * 8   # ... the bonus position counted for every row
    bytes_everything = rows * (L + 1) * V * 4 + rows * L * V * 4              # ... every input tensor in full
    achieved = alg_bytes / (dev_us * 1e-6) / 1e9
    emitted = float((acc_h + 1).mean())
    out_j = {
        "metric": f"verified rows/sec at B={rows}x{L} drafts x {V} vocab", "value": rows * args.steps / wall,
        "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3 / args.steps,
        "us_per_step_device": dev_us, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (target = draft + N(0, .5^2), q = softmax(draft), 2 rotated resident sets)",
        "config": {"workload": "c5", "rows": rows, "n_draft": L, "vocab": V, "mean_tokens_emitted_per_row": emitted},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": committed_traffic("c5"),
                     "traffic_source": "profiles/traffic_c5.json.txt: rocprofv3 --pmc runs of this command, whole step, committed; not measured by this run",
                     "algorithmic_bytes_per_launch": alg_bytes,
                     "bytes_with_bonus_position_for_every_row": bytes_with_bonus, "bytes_reading_every_input": bytes_everything,
                     "kernel": "k_full_softmax_seg", "kernel_us": dev_us},
        "cpu_baseline": cpu, "parity": parity,
    }
    for _, _, _, b, _, _ in sets:
        b.close()
    return out_j


def committed_traffic(workload):
    """HBM bytes per step from the committed counter summary of this workload (profiles/traffic_<workload>.json.txt), or None."""
    try:
        return json.load(open(os.path.join(ROOT, "profiles", f"traffic_{workload}.json.txt"))).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def bench_argmax(args, ctx, stream) -> dict:
    """Row argmax (sr_argmax_rows_launch) of 256 x 151,936 fp32 logits, four rotated resident buffers."""
    import torch

    from opentail.stingray_amd import synthetic

    w = synthetic.config3(rows=256, bf16=False)
    rows, vocab = w.rows, w.vocab
    bufs = [torch.from_numpy(np.roll(w.logits, (i * 7) % rows, axis=0)).cuda() for i in range(4)]
    idx = torch.empty(rows, dtype=torch.int32, device="cuda")
    val = torch.empty(rows, dtype=torch.float32, device="cuda")
    import ctypes as C

    def step(i):
        t = bufs[i % 4]
        ctx._check(ctx.L.sr_argmax_rows_launch(ctx.h, C.c_void_p(t.data_ptr()), 0, rows, vocab, vocab,
                                               C.c_void_p(idx.data_ptr()), C.c_void_p(val.data_ptr())))

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        step(i)
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_us = ev0.elapsed_time(ev1) * 1e3 / args.steps
    parity = None
    if not args.no_parity:
        from oracle import binding as orc

        last = np.roll(w.logits, (((args.steps - 1) % 4) * 7) % rows, axis=0)
        want = np.array([orc.greedy(r) for r in last])
        parity = {"rows_checked": rows, "mismatches": int((idx.cpu().numpy() != want).sum())}
    alg_bytes = rows * vocab * 4 + rows * 8
    achieved = alg_bytes / (dev_us * 1e-6) / 1e9
    return {
        "metric": f"greedy rows/sec at B={rows}x{vocab} vocab", "value": rows * args.steps / wall, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3 / args.steps,
        "us_per_step_device": dev_us, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded Gaussian + Zipf-head logits, 4 rotated resident buffers)",
        "config": {"workload": "argmax", "rows": rows, "vocab": vocab},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_launch": alg_bytes,
                     "kernel": "k_argmax_rows", "kernel_us": dev_us},
        "cpu_baseline": None, "parity": parity,
    }


def run_workload(args, ctx, stream) -> dict:
    """One workload (args.workload) for args.steps timed steps; the result as the dict that main() prints."""
    import torch

    if args.workload == "argmax":
        return bench_argmax(args, ctx, stream)
    w = make_workload(args.workload, getattr(args, "rows", 256))
    rows, vocab = w.rows, w.vocab
    if args.workload == "c5":
        return bench_spec(args, w, ctx, stream)

    # distinct resident logits buffers (row-rotated copies of the seeded tensor) + their batches: four, or as many as
    # it takes to exceed the 256 MB Infinity Cache (16 at most: a smaller workload is measured warm and says so)
    elem = 2 if w.logits_bf16 is not None else 4
    buf_bytes = rows * vocab * elem
    n_buf = int(min(16, max(4, -(-300_000_000 // buf_bytes))))
    cold = n_buf * buf_bytes > 268_435_456
    bufs, batches, host_logits = [], [], []
    for i in range(n_buf):
        sh = (i * 7) % rows if rows > 1 else 0
        lg = np.roll(w.logits, sh, axis=0)
        host_logits.append(lg)
        if w.logits_bf16 is not None:
            t = torch.from_numpy(np.roll(w.logits_bf16, sh, axis=0).view(np.int16)).view(torch.bfloat16).cuda()
        else:
            t = torch.from_numpy(lg).cuda()
        bufs.append(t)
        batches.append(ctx.new_batch().upload(w.params, vocab, w.uniforms, w.allow_mask, w.mask_active))
    toks = [torch.full((rows,), -7, dtype=torch.int32, device="cuda") for _ in range(n_buf)]
    flags = [torch.zeros(rows, dtype=torch.int32, device="cuda") for _ in range(n_buf)]

    def step(i):
        b = i % n_buf
        ctx.sample_launch(batches[b], bufs[b], toks[b], flags[b])

    # every rotated buffer is launched once before the timed steps whatever --warmup says: a batch builds its scan masks
    # at its first launch (they depend on where the logits lie), and that is set-up, not a step
    for i in range(max(args.warmup, n_buf)):
        step(i)
    torch.cuda.synchronize()
    if args.copy_probe:
        probe = torch.empty_like(bufs[0])
        for _ in range(3):
            probe.copy_(bufs[0])   # reads and writes bufs[0].numel() * element_size bytes
        torch.cuda.synchronize()

    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        step(i)
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = ev0.elapsed_time(ev1)
    ms_per_step = wall * 1e3 / args.steps
    kern_us = dev_ms * 1e3 / args.steps  # device time per launch from HIP events on the launch stream

    # the same K steps once more, reported beside the timed region (not used for `value`): a steady-state check
    ev2 = torch.cuda.Event(enable_timing=True)
    ev3 = torch.cuda.Event(enable_timing=True)
    ev2.record(stream)
    for i in range(args.steps):
        step(i)
    ev3.record(stream)
    torch.cuda.synchronize()
    kern_us_again = ev2.elapsed_time(ev3) * 1e3 / args.steps

    # a decode step that also uploads its batch again (histories change every step): host packing + copies + launch
    step_with_upload_us = None
    extra_legs = args.workload.startswith("c3") and not args.short and not os.environ.get("SR_BENCH_NO_UPLOAD_LEG")
    if extra_legs:
        n_up = max(100, args.steps // 4)
        for i in range(3):
            batches[i % n_buf].reupload()
            step(i)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(n_up):
            batches[i % n_buf].reupload()
            step(i)
        torch.cuda.synchronize()
        step_with_upload_us = (time.perf_counter() - t1) * 1e6 / n_up

    # a decode step that appends the sampled token to every history instead (sr_batch_append_tokens; random ids stand
    # in for the sampled ones, so most are new to their history and every 16th step or so a row runs out of room and
    # the batch is rebuilt).  Batches and outputs of their own: the measured ones stay as they are for the parity check.
    step_with_append_us = None
    if extra_legs:
        n_up = max(100, args.steps // 4)
        ab = [ctx.new_batch().upload(w.params, vocab, w.uniforms, w.allow_mask, w.mask_active) for _ in range(n_buf)]
        atok = torch.empty(rows, dtype=torch.int32, device="cuda")
        rng = np.random.default_rng(7)
        ids = rng.integers(0, vocab, (n_up + 3, rows)).astype(np.int32)
        un = rng.random((n_up + 3, rows))
        for i in range(3):
            ab[i % n_buf].append_tokens(ids[i], un[i])
            ctx.sample_launch(ab[i % n_buf], bufs[i % n_buf], atok)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(n_up):
            ab[i % n_buf].append_tokens(ids[i + 3], un[i + 3])
            ctx.sample_launch(ab[i % n_buf], bufs[i % n_buf], atok)
        torch.cuda.synchronize()
        step_with_append_us = (time.perf_counter() - t1) * 1e6 / n_up
        for b_ in ab:
            b_.close()

    # parity of the measured outputs against the oracle (outside the timed region)
    parity = None
    if not args.no_parity:
        from tests.helpers import oracle_tokens

        n_chk = rows  # every row of the measured launch
        got = toks[0].cpu().numpy()[:n_chk]
        want = oracle_tokens(host_logits[0][:n_chk], w.params[:n_chk], np.asarray(w.uniforms)[:n_chk],
                             None if w.allow_mask is None else w.allow_mask[:n_chk],
                             None if w.mask_active is None else w.mask_active[:n_chk])
        parity = {"rows_checked": int(n_chk), "mismatches": int((got != want).sum())}
    unsupported = int(sum(int((f.cpu().numpy().view(np.uint32) >> 31).sum()) for f in flags))
    # rows whose token rests on a convention the managed runtime leaves open (SR_OUT_AMBIGUOUS, bit 4), over the
    # buffers the run touched
    used = flags[: min(n_buf, args.steps + args.warmup)]
    ambiguous = int(sum(int(((f.cpu().numpy().view(np.uint32) >> 4) & 1).sum()) for f in used))

    alg_bytes = rows * vocab * elem + (0 if w.allow_mask is None else w.allow_mask.nbytes) + rows * 8
    achieved = alg_bytes / (kern_us * 1e-6) / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", f"traffic_{args.workload}.json.txt")
    if os.path.exists(tpath) and rows == 256:
        try:
            traffic = json.load(open(tpath)).get("hbm_bytes_per_launch")
        except Exception:
            traffic = None

    cpu = None
    if args.cpu_seconds > 0:
        tps, n_warm, n_rep, med = cpu_baseline(w, args.cpu_seconds)
        host = host_description()
        cpu = {"value": tps, "unit": "tokens/s", "cores": 1, "kind": "port", "us_per_step": med * 1e6,
               "cpu_model": host["cpu_model"], "nproc": host["nproc"],
               "sample": f"one step = the {rows} rows of the same workload ({args.workload}), rows in order on one thread of "
                         f"{host['nproc']}; {n_warm} warm-up steps, median of {n_rep} timed steps; {host['note']}"}

    out = {
        "metric": "sampled tokens/sec at B=256x152k vocab" if rows == 256 else f"sampled tokens/sec at B={rows}x{vocab} vocab",
        "value": rows * args.steps / wall,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "us_per_step_device": kern_us,
        "us_per_step_device_second_window": kern_us_again,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if elem == 4 else "bf16->f32",
        "data": f"synthetic (seeded Gaussian + Zipf-head logits, {n_buf} rotated resident buffers = "
                f"{n_buf * buf_bytes / 1e6:.0f} MB: {'cold reads' if cold else 'WARM: fits the 256 MB Infinity Cache'})",
        "config": {"workload": args.workload, "rows": rows, "vocab": vocab,
                   "chain": "penalties+top-k+top-p+min-p" if args.workload == "c3_fp32_full" else args.workload},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "frac_with_token_append": (None if step_with_append_us is None else
                                                alg_bytes / (step_with_append_us * 1e-6) / 1e9 / HBM_PEAK_GBS),
                     "traffic": traffic,
                     "traffic_source": None if traffic is None else
                     f"profiles/{os.path.basename(tpath)}: rocprofv3 --pmc runs of this command, committed; not measured by this run",
                     "algorithmic_bytes_per_launch": alg_bytes,
                     "kernel": "k_topk_rows" if args.workload.startswith(("c1", "c3")) else ("k_full_softmax_seg" if args.workload == "c2" else "k_full_row"),
                     "kernel_us": kern_us},
        "cpu_baseline": cpu,
        "parity": parity,
        "rows_unsupported": unsupported,
        "rows_flagged_ambiguous": {"rows": ambiguous, "of": rows * len(used)},
        "us_per_step_with_batch_upload": step_with_upload_us,
        "us_per_step_with_token_append": step_with_append_us,
    }
    for b_ in batches:
        b_.close()
    return out


# The other configurations of the benchmark, each for a short window of its own inside the default run:
# (workload, timed steps, warm-up steps, seconds of CPU baseline; c4's steps are two whole turns of its sixteen buffers,
# whose steps differ by the largest nucleus in them)
PER_CONFIG = [("c1", 400, 40, 1.5), ("c2", 60, 6, 1.5), ("c3_bf16", 200, 20, 1.5), ("c4", 32, 4, 1.5), ("c5", 20, 3, 1.5)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="c3_fp32_full")
    ap.add_argument("--rows", type=int, default=256, help="batch rows of the c3_* workloads (the benchmark's point is 256)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU-baseline time budget (0 = skip)")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--no-prime", action="store_true", help="skip the event warm-up (prime_events): for looking at it")
    ap.add_argument("--no-per-config", action="store_true",
                    help="the default workload alone, without the short windows of the other configurations")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain device copy of one logits buffer (known size) so that a counter run\n"
                         "under rocprofv3 --pmc has a reference dispatch to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    args.short = False
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on one GPU (rows shard across GPUs without any exchange); "
                         "run with --gpus 1")

    import torch

    from opentail.stingray_amd import SamplerContext
    from oracle import binding as orc  # noqa: F401  (checker + CPU baseline only; loaded before the timed regions)

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU: the sampler has no CPU path")
    torch.cuda.set_device(0)
    stream = torch.cuda.Stream()            # a real (non-null) stream shared by torch and the library,
    torch.cuda.set_stream(stream)           # so HIP events recorded here bracket the sampler's kernels
    ctx = SamplerContext(0)
    if not args.no_prime:
        prime_events(torch, stream)
    # no collector pauses inside the timed loops (as timeit does): a full collection of this process takes tens of
    # milliseconds, which is hundreds of steps
    import gc
    gc.collect()
    gc.disable()

    out = run_workload(args, ctx, stream)
    if args.workload == "c3_fp32_full" and not args.no_per_config and not args.copy_probe:
        per = {}
        for name, steps, warmup, cpu_s in PER_CONFIG:
            gc.collect()
            torch.cuda.empty_cache()
            sub = argparse.Namespace(**vars(args))
            sub.workload, sub.steps, sub.warmup, sub.short = name, steps, warmup, True
            sub.cpu_seconds = min(cpu_s, args.cpu_seconds)
            r = run_workload(sub, ctx, stream)
            per[name] = {
                "us_per_step": r["us_per_step_device"], "steps": steps, "value": r["value"], "unit": r["unit"],
                "frac": r["roofline"]["frac"], "achieved_gbs": r["roofline"]["achieved"], "kernel": r["roofline"]["kernel"],
                "algorithmic_bytes_per_launch": r["roofline"]["algorithmic_bytes_per_launch"],
                "cpu_baseline": None if r["cpu_baseline"] is None else
                {k: r["cpu_baseline"][k] for k in ("value", "unit", "cores", "kind")},
                "parity": r["parity"], "config": r["config"],
            }
        out["per_config"] = per
        # the headline kernel at other batch sizes (same row width and chain): the curve around the benchmark's point
        sweep = {}
        for n_rows in (64, 128, 192, 320, 512):
            gc.collect()
            torch.cuda.empty_cache()
            sub = argparse.Namespace(**vars(args))
            sub.workload, sub.steps, sub.warmup, sub.short, sub.rows, sub.cpu_seconds = "c3_fp32_full", 200, 20, True, n_rows, 0.0
            r = run_workload(sub, ctx, stream)
            sweep[str(n_rows)] = {"us_per_step": r["us_per_step_device"], "frac": r["roofline"]["frac"], "value": r["value"],
                                  "parity": r["parity"]}
        out["rows_sweep_c3_fp32_full"] = sweep
    print(json.dumps(out))


if __name__ == "__main__":
    main()
