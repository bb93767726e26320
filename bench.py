#!/usr/bin/env python3
"""bench.py -- reduce+codec throughput of one 25 MiB DDP bucket on one MI355X.

A "step" is one pass of the hot path over one bucket: the fused
bf16-decode + reduce + average fold of configuration C2 (butterfly schedule,
3 virtual ranks, 6,553,600 fp32 gradients per rank, bf16 wire, x 1/3) -- every
virtual rank folds its own chunk of the bucket from its own fp32 data and the
two peers' bf16 wire chunks, all resident in HBM, in ONE launch.

Algorithmic bytes per step (what `value` and `roofline.achieved` are computed
from): per bucket element 4 B own fp32 read + 2 x 2 B bf16 peer reads + 4 B fp32
write = 12 B  ->  78,643,200 B.

The K timed steps are recorded into one HIP graph and replayed with a single
submission (the warm-up replays the same graph, i.e. max(W, K) untimed steps).
Two brackets around exactly K steps each:
  * `value` / `ms_per_step`: the wall clock around one replay, queue drained and
    device synchronised on both sides -- it includes what the host pays to submit
    a graph, which does not shrink with K;
  * `roofline`: HIP events on the reduce queue around one replay that is enqueued
    directly behind the warm-up replay, so that the start event is stamped when
    the warm-up ends and the timed launches are already queued behind it.  (With
    a drained queue in front, the start event is stamped at once and the device
    then idles while the host submits the replay: some 10 us that are the host's,
    not the kernel's, and that weigh 0.5 us per step at K = 20 and 0.05 at K = 200.)
Steps rotate over several distinct copies of the workload (> 512 MiB in total) so
the 256 MiB Infinity Cache cannot serve the reads ("cold", the headline); the
same loop over one copy is reported as "warm".

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
CAL_BYTES = 64 << 20   # size of the calibration copy
# HBM bytes one C2 fold launch moves, from rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by the
# calibration copy (profiles/c2_fold_hbm_traffic_pmc.txt): 1.006 x the algorithmic bytes.
C2_MEASURED_TRAFFIC_BYTES = 79_070_677


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=8, help="distinct workload copies the cold loop rotates over")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="headline only (used when profiling)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--timeline", action="store_true",
                    help="instead of the JSON line, print where the time of one C2 launch goes: every block's "
                         "start and end stamps from the measurement build (python -m mccl_amd.build --bench)")
    ap.add_argument("--host-phases", action="store_true",
                    help="instead of the JSON line, print where the host's time goes for a C2 bucket through the "
                         "c10d surface (three native rank threads), phase by phase")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the path; this build runs on a single GPU "
              "(--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    if args.host_phases:
        host_phase_report()
        return

    import numpy as np
    import torch
    from mccl_amd.build import ensure_built, BENCH_LIB_PATH
    ensure_built()
    if args.timeline:
        if not os.path.exists(BENCH_LIB_PATH):
            print("bench.py --timeline needs the measurement build: python -m mccl_amd.build --bench",
                  file=sys.stderr)
            sys.exit(2)
        os.environ["MCCLX_LIBRARY"] = BENCH_LIB_PATH
    from mccl_amd import _lib as L
    from mccl_amd import kernels as K
    from mccl_amd import harness as H
    from mccl_amd import workloads as W

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    q = K.ReduceQueue(0)
    cfg = W.C2
    world, numel = cfg["world"], cfg["numel"]
    chunks = H.chunkize(numel, 1, world)
    scale = 1.0 / world
    bytes_per_step = numel * 12

    # ---- workload: `sets` copies of (3 fp32 rank tensors + their bf16 wire copies)
    host0 = [W.c2_input(r) for r in range(world)]
    tensors, wires = [], []
    for s in range(args.sets):
        ts = [torch.from_numpy(host0[r]).cuda() if s == 0 else
              torch.from_numpy(W.c2_input(r, variant=s)).cuda() for r in range(world)]
        ws = [K.encode_bf16(t, queue=q) for t in ts]
        tensors.append(ts)
        wires.append(ws)
    q.drain()

    # A plain copy of known size (64 MiB in, 64 MiB out), 5 launches: the reference
    # dispatches the memory counters (FETCH_SIZE / WRITE_SIZE) are scaled by.
    cal = torch.empty(2 * CAL_BYTES, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    for _ in range(5):
        q.copy(cal.data_ptr() + CAL_BYTES, cal.data_ptr(), CAL_BYTES)
    q.drain()

    plan = K.make_plan(L.BF16, world, io=L.IO_OWN_FIRST_F32, op=L.SUM, scale_mode=L.SCALE_VIEW, scale=scale)

    # Results go to buffers of their own, so that every step of every replay folds the
    # seeded payload (folding in place would feed step n+8 the result of step n).  The
    # in-place form the scheduler issues moves the same bytes; it is timed as an extra.
    results = [[torch.empty_like(t) for t in ts] for ts in tensors]

    def step_segs(s, with_wire_out=False, out_tensors=None):
        segs = []
        for R, (start, cnt, _, _) in enumerate(chunks):
            own = tensors[s][R].data_ptr() + start * 4
            out = own if out_tensors is None else out_tensors[R].data_ptr() + start * 4
            peers = [wires[s][p].data_ptr() + start * 2 for p in range(world) if p != R]
            wire_out = wires[s][R].data_ptr() + start * 2 if with_wire_out else 0
            segs.append(K.make_seg(out, wire_out, [own] + peers, cnt))
        return segs

    # ---- parity of exactly this launch against the CPU oracle (set 0, out of place)
    from oracle import oracle as orc
    outs = [torch.zeros_like(t) for t in tensors[0]]
    q.fold(plan, step_segs(0, out_tensors=outs))
    q.drain()
    wire_host = [orc.encode_bf16(x) for x in host0]
    parity = True
    for R, (start, cnt, _, _) in enumerate(chunks):
        peers = [np.ascontiguousarray(wire_host[p][start:start + cnt]) for p in range(world) if p != R]
        want = orc.wire_fold_chunk(np.ascontiguousarray(host0[R][start:start + cnt]), peers,
                                   scale_by=scale, threads=min(16, orc.max_threads()))
        got = outs[R][start:start + cnt].cpu().numpy()
        parity &= bool(np.array_equal(got.view(np.uint32), want.view(np.uint32)))
    del outs

    # ---- timed loops, each recorded into one graph
    def record(n_steps, seg_fn, qu):
        qu.graph_begin()
        for i in range(n_steps):
            seg_fn(i)
        return qu.graph_end()

    def timed_replays(qu, graph, reps=5):
        """Median device time (ms) of one replay of `graph`: HIP events on the reduce queue around a
        replay enqueued directly behind an untimed replay of the same graph."""
        ts = []
        for _ in range(reps):
            qu.graph_launch(graph)
            qu.timer_begin()
            qu.graph_launch(graph)
            ts.append(qu.timer_end())
        return sorted(ts)[reps // 2]

    # Marks in a kernel trace: a copy of n x 4 KiB (a grid of n x 256 threads of the plain copy kernel)
    # in front of and behind the headline's timed replays, so that a profile of this program can
    # tell them from the warm-up around them.
    mark_buf = torch.zeros(2 * 16 * 4096, dtype=torch.uint8, device="cuda")

    def mark(n):
        q.copy(mark_buf.data_ptr() + 16 * 4096, mark_buf.data_ptr(), n * 4096)

    single_bracket = {}

    def measure(seg_fn, steps, warmup, wall=False, queue=None, reps=5, marks=None):
        """W untimed warm-up steps, then exactly `steps` timed steps; returns (device ms, wall ms or None).
        `seg_fn(i)` issues step i.  Device time: two graphs are recorded, one of the W warm-up steps
        alone and one of the W warm-up steps followed by the `steps` timed ones (W = `warmup`, but at
        least 10: the first launches behind a graph boundary run slower than the rest).  Each is
        replayed between a pair of HIP events on the reduce queue; the difference of the two times
        is the time of steps W+1 .. W+steps: the launches and the gaps between them, with the warm-up
        and whatever a pair of events and a graph replay add to a bracket (8-11 us, whatever the
        length of the graph; 0.5 us per step if left inside a bracket of 20 steps) taken out.
        Medians of `reps` replays.  The data stays cold: every replay walks all rotating copies again.
        Wall time (`wall=True`): a replay of a graph of the same K steps, bracketed by a drain
        and a device synchronisation on both sides."""
        qu = queue or q
        torch.cuda.synchronize()  # inputs made by torch ops are complete before the queue reads them
        w = max(warmup, min(10, steps))
        g_warm = record(w, seg_fn, qu)
        g_all = record(w + steps, seg_fn, qu)
        # the first replay of a fresh graph is slower still, and a device that has been idle takes
        # some tens of milliseconds of work to reach its steady clocks: 50 ms of untimed replays
        t_ready = time.perf_counter() + 0.05
        while time.perf_counter() < t_ready:
            for _ in range(4):
                qu.graph_launch(g_all)
            qu.drain()
        if marks:
            mark(marks[0])
        ms_all = timed_replays(qu, g_all, reps)
        if marks:
            mark(marks[1])
        ms_dev = ms_all - timed_replays(qu, g_warm, reps)
        qu.graph_destroy(g_warm)
        qu.graph_destroy(g_all)
        ms_wall = None
        if wall:
            gk = record(steps, lambda i: seg_fn(w + i), qu)
            # the same K steps in ONE pair of events (a replay behind an untimed replay): what the
            # subtraction above takes out stays in, 7-11 us per bracket
            single_bracket["ms"] = timed_replays(qu, gk, reps)
            qu.graph_launch(gk)
            qu.drain()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            qu.graph_launch(gk)
            qu.drain()
            torch.cuda.synchronize()
            ms_wall = (time.perf_counter() - t0) * 1e3
            qu.graph_destroy(gk)
        return ms_dev, ms_wall

    cold = lambda i: q.fold(plan, step_segs(i % args.sets, out_tensors=results[i % args.sets]))
    warm = lambda i: q.fold(plan, step_segs(0, out_tensors=results[0]))
    if args.timeline:
        timeline_report(args, q, K, L, torch, np, plan, step_segs, results, measure, bytes_per_step)
        return
    cold_dev, cold_wall = measure(cold, args.steps, args.warmup, wall=True, reps=9, marks=(1, 2))
    warm_dev, _ = measure(warm, args.steps, args.warmup, reps=9, marks=(3, 4))

    gbs = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9
    kernel_us = cold_dev / args.steps * 1e3
    achieved = gbs(bytes_per_step, cold_dev / args.steps)
    value = gbs(bytes_per_step * args.steps, cold_wall)

    result = {
        "metric": "reduce+codec GB/s per 25 MB bucket and % of HBM peak, 1 MI355X vs host CPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(cold_wall / args.steps, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "C2: butterfly schedule, 3 virtual ranks, 6,553,600 fp32 grads (25 MiB) per rank, "
                               "bf16 RNE wire, fused decode+accumulate+x(1/3), peers HBM-resident, "
                               f"cold (rotating {args.sets} copies)",
                   "algorithmic_bytes_per_step": bytes_per_step, "parity_vs_oracle_bit_exact": parity},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": C2_MEASURED_TRAFFIC_BYTES,
                     "kernel": "fold_few_hold_kernel<bf16, own-first fp32, k=3; 4 packets per lane, 512-lane blocks>", "kernel_us": round(kernel_us, 2),
                     "method": "HIP events on the reduce queue; time of a graph of W warm-up + K timed launches minus time of a graph "
                               "of the W warm-up launches alone (W >= 10), medians of 9 replays each, behind 50 ms of untimed replays",
                     "kernel_us_single_bracket": round(single_bracket["ms"] / args.steps * 1e3, 2),
                     "frac_single_bracket": round(gbs(bytes_per_step, single_bracket["ms"] / args.steps) / HBM_PEAK_GBS, 4)},
    }
    lat_ticks, bpt, measured = q.hold_model()
    extra = {"hold_gate": {"latency_ticks": lat_ticks, "bytes_per_tick": bpt, "measured_on_this_device": measured,
                           "ticks_for_this_launch": lat_ticks + (numel * 8) // bpt},
             "warm_GBps": round(gbs(bytes_per_step, warm_dev / args.steps), 1),
             "warm_kernel_us": round(warm_dev / args.steps * 1e3, 2),
             "pct_of_hbm_peak_cold": round(100 * achieved / HBM_PEAK_GBS, 2)}
    # the same launches in single brackets: events around graph replays of 10-160 steps.  A straight
    # line through (steps, microseconds) has the launch period as its slope and what a graph replay
    # and the two events add to a bracket as its intercept
    extra["c2_fold_single_brackets"] = graph_bracket_fit(q, cold, record, np)

    if not args.no_extras:
        try:
            extra.update(extras(args, q, K, H, L, W, torch, np, tensors, wires, chunks, plan, step_segs,
                                measure, gbs, results))
        except Exception as e:  # extras never take the headline down
            extra["extras_error"] = f"{type(e).__name__}: {e}"

    # ---- CPU baseline: the same job in reference-shaped passes on the host cores
    if not args.no_cpu:
        threads = min(16, orc.max_threads())
        own = [np.ascontiguousarray(host0[R][s:s + c]) for R, (s, c, _, _) in enumerate(chunks)]
        prs = [[np.ascontiguousarray(wire_host[p][s:s + c]) for p in range(world) if p != R]
               for R, (s, c, _, _) in enumerate(chunks)]

        def cpu_pass(th):
            t0 = time.perf_counter()
            for R in range(world):
                orc.wire_fold_chunk(own[R], prs[R], scale_by=scale, threads=th)
            return time.perf_counter() - t0

        def best_of(th, budget):
            cpu_pass(th)
            best, spent, reps = 1e9, 0.0, 0
            while spent < budget and reps < 200:
                dt = cpu_pass(th)
                best, spent, reps = min(best, dt), spent + dt, reps + 1
            return best, reps

        b_all, reps_all = best_of(threads, args.cpu_seconds * 0.6)
        b_one, reps_one = best_of(1, args.cpu_seconds * 0.4)
        result["cpu_baseline"] = {
            "value": round(bytes_per_step / b_all / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"the same C2 bucket (3 chunks, 78,643,200 algorithmic bytes) as reference-shaped passes "
                      f"(encode, 2 binary bf16 reduces, scale, decode); best of {reps_all} passes, OpenMP",
            "single_thread_GBps": round(bytes_per_step / b_one / 1e9, 2), "host_cpus": os.cpu_count(),
            "cpu_model": cpu_model()}
    result["extra"] = extra
    print(json.dumps(result))


def graph_bracket_fit(q, seg_fn, record, np):
    ks, tot = (10, 20, 40, 80, 160), []
    for k in ks:
        g = record(k, seg_fn, q)
        ts = []
        for _ in range(5):
            q.graph_launch(g)
            q.graph_launch(g)
            q.timer_begin()
            q.graph_launch(g)
            ts.append(q.timer_end() * 1e3)
        q.graph_destroy(g)
        tot.append(sorted(ts)[2])
    slope, icpt = np.linalg.lstsq(np.vstack([ks, np.ones(len(ks))]).T, np.array(tot), rcond=None)[0]
    return {"us_per_step_by_steps": {str(k): round(t / k, 2) for k, t in zip(ks, tot)},
            "fit_us_per_step": round(float(slope), 2), "fit_us_per_bracket": round(float(icpt), 1)}


def host_phase_report():
    """Host cost of a C2 bucket through ProcessGroupMCCL, by phase (MCCL_PHASE_STATS=1): eight buckets
    back to back per round, three ranks as native threads, synchronous and event-based completion."""
    os.environ["MCCL_PHASE_STATS"] = "1"
    os.environ.update({"MCCL_ALLREDUCE_ALGO": "butterfly", "MCCL_WIRE_DTYPE": "bf16"})
    import torch
    from mccl_amd import _C as CX, workloads as W
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    numel, nb, rounds = W.C2["numel"], 8, 6
    for mode in ("synchronous", "event-based"):
        if mode == "event-based":
            os.environ["MCCL_ALLREDUCE_ASYNC"] = "1"
        else:
            os.environ.pop("MCCL_ALLREDUCE_ASYNC", None)
        CX._allreduce_rate(3, numel, nb, 2)   # first rounds: kernels loaded, graphs recorded
        CX._phase_stats(True)
        us = CX._allreduce_rate(3, numel, nb, rounds)
        st = CX._phase_stats(True)
        print(f"{mode} completion: best round, us per bucket, by rank: {[round(x, 1) for x in us]}")
        print(f"  {'phase':15s} {'calls':>6s} {'mean us':>9s} {'us per bucket, all 3 ranks together':>38s}")
        for k, (calls, tot) in st.items():
            if calls:
                print(f"  {k:15s} {calls:6d} {tot / calls:9.2f} {tot / (nb * rounds):38.2f}")


def cpu_model() -> str:
    """The host CPU as /proc/cpuinfo names it; a virtualised box may only say "AMD EPYC",
    so the family / model numbers and the clock go with it."""
    want = {"model name": None, "cpu family": None, "model": None, "cpu mhz": None}
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, val = line.partition(":")
                key = key.strip().lower()
                if key in want and want[key] is None:
                    want[key] = val.strip()
                if all(v is not None for v in want.values()):
                    break
    except OSError:
        pass
    if want["model name"] is None:
        return "unknown"
    extra = []
    if want["cpu family"] and want["model"]:
        extra.append(f"family {want['cpu family']} model {want['model']}")
    if want["cpu mhz"]:
        extra.append(f"{float(want['cpu mhz']):.0f} MHz")
    return want["model name"] + (f" ({', '.join(extra)})" if extra else "")


def timeline_report(args, q, K, L, torch, np, plan, step_segs, results, measure, bytes_per_step):
    """Where the time of one C2 launch goes.  The instrumented build stamps every block
    (start, arguments fetched, last store issued; 100 MHz wall clock) into a device
    buffer; 16 consecutive cold launches are recorded into one graph, replayed, and
    their stamps reduced to: the launch-to-launch period, the span from the first block's
    start to the last block's end, the gap between launches, and the ramp and drain
    inside the span."""
    import ctypes as C
    lib = L.lib()
    set_tl = lib.mcclx_tune_timeline
    set_tl.restype, set_tl.argtypes = None, [C.c_void_p, C.c_uint64, C.c_uint64]
    slots, per_slot, rec_words = 16, 4096, 4          # a record is 4 x 8 bytes
    cus = q.compute_units
    out = []
    pr = out.append
    pr("C2 fused fold -- timeline of one launch from per-block time stamps, MI355X (gfx950)")
    pr("")
    pr("Command: python -m mccl_amd.build --bench   (here, once)   then on the GPU box:   python bench.py --timeline")
    pr("Every block of the fold <bf16, own-first fp32, k=3> records wall_clock64() (100 MHz, 10 ns ticks) at its first")
    pr("instruction, at a second point, and after its last store was issued.  16 consecutive launches (cold = rotating 8")
    pr("copies of the workload, 944 MB + 629 MB of results) are recorded into one HIP graph; figures are means over")
    pr("launches 3..15 of its 4th replay.  All times in microseconds.")
    lat_ticks, bpt, measured = q.hold_model()
    pr("  hold form  (the default for this launch): 1020 blocks of 512 threads, ONE generation; every lane issues the loads")
    pr("             of its four packets at once, keeps the results in registers and stores them when the gate opens")
    pr(f"             ({lat_ticks} ticks + bytes read / {bpt:,} per tick after its block started; the rate was "
       f"{'measured on this device' if measured else 'taken from the built-in default'}).")
    pr("             Second stamp: the block has its data.")
    pr("  plain form (mcclx_set_hold(ctx, 0); every launch too large for one generation): 3201 blocks, one per 8 KiB tile of")
    pr("             a chunk, loads then stores.  Second stamp: the block has its kernel arguments.")

    def capture(seg_fn, label, hold=False):
        buf = torch.zeros(slots * per_slot * rec_words, dtype=torch.int64, device="cuda")
        torch.cuda.synchronize()
        set_tl(buf.data_ptr(), slots, per_slot)
        q.graph_begin()
        for i in range(slots):
            seg_fn(i)
        g = q.graph_end()
        set_tl(None, 0, 0)
        for _ in range(4):
            q.graph_launch(g)
            q.drain()
        q.graph_destroy(g)
        rec = buf.cpu().numpy().reshape(slots, per_slot, rec_words)
        launches = []
        for i in range(slots):
            r = rec[i]
            r = r[r[:, 2] != 0]
            t0, ta, t1 = r[:, 0].astype(np.int64), r[:, 1].astype(np.int64), r[:, 2].astype(np.int64)
            xcc = ((r[:, 3].view(np.uint64) >> np.uint64(32)) & np.uint64(15)).astype(np.int64)
            launches.append((t0, ta, t1, xcc))
        tick = 0.01
        rows = []
        for i in range(2, slots - 1):
            t0, ta, t1, xcc = launches[i]
            n0 = launches[i + 1][0]
            s0, e1 = t0.min(), t1.max()
            st = np.sort(t0)
            en = np.sort(t1)
            fill_n = min(len(st), 4 * cus) - 1
            per_x = [t1[xcc == x].max() - s0 for x in range(8) if (xcc == x).any()]
            rows.append(dict(
                blocks=len(t0), period=(n0.min() - s0) * tick, span=(e1 - s0) * tick, gap=(n0.min() - e1) * tick,
                fill=(st[fill_n] - s0) * tick, args=float((ta - t0).mean()) * tick, first_end=(en[0] - s0) * tick,
                life=float((t1 - t0).mean()) * tick, last_start=(st[-1] - s0) * tick,
                last90=(e1 - en[int(0.9 * len(en))]) * tick, xcd_spread=(max(per_x) - min(per_x)) * tick))
        m = {k: float(np.mean([r[k] for r in rows])) for k in rows[0]}
        pr("")
        pr(f"[{label}]")
        pr(f"  blocks per launch                                   {int(m['blocks'])}")
        pr(f"  period: first block start -> next launch's first    {m['period']:6.2f}   = {bytes_per_step / m['period'] / 1e3:6.0f} GB/s algorithmic")
        pr(f"  span:   first block start -> last block's end       {m['span']:6.2f}")
        pr(f"  gap:    last block's end -> next launch's first     {m['gap']:6.2f}   (store acknowledgements, end-of-kernel release, dispatch of the next)")
        pr(f"  inside the span:")
        t0, ta, t1, xcc = launches[8]
        s0 = t0.min()
        if hold:
            data = [(np.sort(l[1])[[0, len(l[1]) // 2, -1]] - l[0].min()) * tick for l in launches[2:slots - 1]]
            d0, d50, d100 = (float(np.mean([d[j] for d in data])) for j in range(3))
            pr(f"    all {int(m['blocks'])} blocks started after                     {m['last_start']:6.2f}")
            pr(f"    first / median / last block has its data after    {d0:6.2f} / {d50:.2f} / {d100:.2f}   (the launch's reads are through)")
            pr(f"    first block past its gate, first store issued     {m['first_end']:6.2f}   (nothing has been written before this)")
            pr(f"    last store issued (the span)                      {m['span']:6.2f}")
            pr(f"    spread of the 8 XCDs' finishing times             {m['xcd_spread']:6.2f}")
            m.update(data_first=d0, data_last=d100)
            pr(f"  launch 9 of the 16, per microsecond since its first block started:")
            pr(f"    t       started   have their data   stores issued")
            for b in range(0, int((t1.max() - s0) * tick) + 1):
                lo, hi = s0 + b * 100, s0 + (b + 1) * 100
                pr(f"    {b:2d}-{b + 1:<2d}   {int(((t0 >= lo) & (t0 < hi)).sum()):6d}  {int(((ta >= lo) & (ta < hi)).sum()):10d}  {int(((t1 >= lo) & (t1 < hi)).sum()):14d}")
            return m
        pr(f"    {4 * cus} blocks (all wave slots) started after        {m['fill']:6.2f}")
        pr(f"    a block waits for its kernel arguments            {m['args']:6.2f}   (mean)")
        pr(f"    first block has its data and ends after           {m['first_end']:6.2f}   (nothing has been written before this)")
        pr(f"    mean block lifetime, start -> last store issued   {m['life']:6.2f}")
        pr(f"    last block starts at                              {m['last_start']:6.2f}")
        pr(f"    the last 10 % of block ends take                  {m['last90']:6.2f}   (a tenth of the span would be {0.1 * m['span']:.2f})")
        pr(f"    spread of the 8 XCDs' finishing times             {m['xcd_spread']:6.2f}")
        # one launch in 1 us bins
        pr(f"  launch 9 of the 16, per microsecond since its first block started:")
        pr(f"    t       started   ended   resident   GB/s by block ends")
        per_block = bytes_per_step / len(t0)
        for b in range(0, int((t1.max() - s0) * tick) + 1):
            lo, hi = s0 + b * 100, s0 + (b + 1) * 100
            st_n = int(((t0 >= lo) & (t0 < hi)).sum())
            en_n = int(((t1 >= lo) & (t1 < hi)).sum())
            res = int(((t0 < hi) & (t1 >= hi)).sum())
            pr(f"    {b:2d}-{b + 1:<2d}   {st_n:6d}  {en_n:6d}   {res:6d}     {en_n * per_block / 1e-6 / 1e9:7.0f}")
        return m

    sets = args.sets
    cold_fn = lambda i: q.fold(plan, step_segs(i % sets, out_tensors=results[i % sets]))
    warm_fn = lambda i: q.fold(plan, step_segs(0, out_tensors=results[0]))
    held = capture(cold_fn, "hold form, cold: rotating copies, reads from HBM", hold=True)
    capture(warm_fn, "hold form, warm: one copy, resident in the 256 MiB Infinity Cache", hold=True)
    q.set_hold(False)
    cold = capture(cold_fn, "plain form, cold")
    capture(warm_fn, "plain form, warm")

    # the same launches without the stamps, and what bounds them: one-directional streams of the same footprint
    gbs = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9
    steps = args.steps
    ms, _ = measure(cold_fn, steps, args.warmup)
    plain_us = ms / steps * 1e3
    q.set_hold(True)
    ms, _ = measure(cold_fn, steps, args.warmup)
    fold_us = ms / steps * 1e3
    fp = bytes_per_step
    probe = torch.randint(0, 256, (8 * fp,), dtype=torch.uint8, device="cuda")
    lines = []
    for nbytes, write, name in ((fp, False, "read only,  78,643,200 B"), (fp, True, "write only, 78,643,200 B"),
                                (fp * 2 // 3, False, "read only,  52,428,800 B (the fold's reads)"),
                                (fp // 3, True, "write only, 26,214,400 B (the fold's writes)")):
        ms, _ = measure(lambda i, nbytes=nbytes, write=write: q.probe_stream(probe.data_ptr() + (i % 8) * fp, nbytes, write),
                        steps, args.warmup)
        lines.append((name, ms / steps * 1e3, gbs(nbytes, ms / steps)))
    ms, _ = measure(lambda i: q.copy(probe.data_ptr() + (i % 8) * fp, probe.data_ptr() + (i % 8) * fp + fp // 2, fp // 2),
                    steps, args.warmup)
    lines.append(("plain copy, 39,321,600 B in + 39,321,600 B out", ms / steps * 1e3, gbs(fp, ms / steps)))
    ms, _ = measure(lambda i: q.probe_stream(probe.data_ptr(), 16 * 256, False), steps, args.warmup)
    empty_us = ms / steps * 1e3
    pr("")
    pr(f"[the same launches without stamps, {steps} timed steps behind {max(args.warmup, min(10, steps))} warm-up steps in one graph, HIP events, the warm-up graph's time subtracted; cold]")
    pr(f"  C2 fold (52.4 MB read + 26.2 MB written), hold form {fold_us:6.2f} us per launch = {gbs(fp, fold_us * 1e-3):6.0f} GB/s = {gbs(fp, fold_us * 1e-3) / 80:5.1f} % of 8 TB/s")
    pr(f"  the same, plain form                                {plain_us:6.2f} us per launch = {gbs(fp, plain_us * 1e-3):6.0f} GB/s = {gbs(fp, plain_us * 1e-3) / 80:5.1f} % of 8 TB/s")
    for name, us, g in lines:
        pr(f"  {name:<50s}  {us:6.2f} us per launch = {g:6.0f} GB/s")
    pr(f"  one-block launch (4 KiB read), back to back         {empty_us:6.2f} us per launch: what two dependent launches cost with no work in them")
    pr("")
    pr("Reading: a launch's period = gap + span. The gap (last store issued -> first block of the next launch running) is")
    pr("spent on store acknowledgements, the end-of-kernel cache release and the dispatch of the dependent launch; the span")
    pr("opens with one memory latency in which no byte has arrived and closes with a drain in which the queues empty.")
    pr(f"Plain form, cold: {cold['gap']:.2f} gap + {cold['first_end']:.2f} until the first block has data leave "
       f"{cold['period'] - cold['gap'] - cold['first_end']:.2f} us in which {fp / 1e6:.1f} MB move: "
       f"{fp / (cold['period'] - cold['gap'] - cold['first_end']) / 1e3:.0f} GB/s while data flows, reads and writes mixed.")
    rd, wr = fp * 2 / 3, fp / 3
    pr(f"Hold form, cold: the same {held['gap']:.2f} gap and {held['data_first']:.2f} first round trip; then the reads alone, "
       f"{rd / 1e6:.1f} MB in {held['data_last'] - held['data_first']:.2f} us = {rd / (held['data_last'] - held['data_first']) / 1e3:.0f} GB/s,")
    pr(f"then the writes alone, {wr / 1e6:.1f} MB between the first store ({held['first_end']:.2f}) and the last ({held['span']:.2f}) "
       f"= {wr / (held['span'] - held['first_end']) / 1e3:.0f} GB/s by issue: each direction near what the one-directional launches above reach.")
    print("\n".join(out))


def backend_extras(torch, W):
    """The same work through the c10d surface: N ranks as N threads of this process, each with
    its own ProcessGroupMCCL.  (a) eight C2 buckets per rank, back to back, synchronous (the
    reference's behaviour) and with event-based completion; (b) the C3 ring with MCCL_WIRE=host,
    every chunk crossing the byte transport in pinned host memory."""
    import datetime
    import threading
    import time
    import torch.distributed as dist
    from mccl_amd import _C as CX
    out = {}
    saved = {k: os.environ.get(k) for k in ("MCCL_ALLREDUCE_ASYNC", "MCCL_ALLREDUCE_ALGO", "MCCL_WIRE_DTYPE", "MCCL_WIRE")}

    def run(world, body):
        store = dist.HashStore()
        res, errs = [None] * world, [None] * world

        def go(r):
            try:
                torch.cuda.set_device(0)
                pg = CX._create_process_group_mccl(store, r, world, datetime.timedelta(seconds=120))
                res[r] = body(r, pg)
            except BaseException as e:  # noqa: BLE001
                errs[r] = e
        ts = [threading.Thread(target=go, args=(r,)) for r in range(world)]
        [t.start() for t in ts]
        [t.join() for t in ts]
        for e in errs:
            if e is not None:
                raise e
        return res

    try:
        os.environ.update({"MCCL_ALLREDUCE_ALGO": "butterfly", "MCCL_WIRE_DTYPE": "bf16"})
        os.environ.pop("MCCL_WIRE", None)
        nb, numel = 8, W.C2["numel"]
        for mode in ("sync", "async"):
            if mode == "async":
                os.environ["MCCL_ALLREDUCE_ASYNC"] = "1"
            else:
                os.environ.pop("MCCL_ALLREDUCE_ASYNC", None)

            def buckets(r, pg):
                ts = [torch.randn(numel, device="cuda") * 1e-3 for _ in range(nb)]
                opt = dist.AllreduceOptions()
                opt.reduceOp = dist.ReduceOp.AVG
                best = 1e9
                for rep in range(4):          # the first round records, later rounds replay (sync) or coalesce (async)
                    torch.cuda.synchronize()
                    pg.barrier().wait()
                    before = CX._async_stats(pg)
                    t0 = time.perf_counter()
                    works = [pg.allreduce([t], opt) for t in ts]
                    for w in works:
                        w.wait()
                    torch.cuda.current_stream().synchronize()
                    best = min(best, time.perf_counter() - t0)
                    after = CX._async_stats(pg)
                return best, after[0] - before[0]
            res = run(3, buckets)
            out[f"c2_backend_{mode}_us_per_bucket"] = round(max(b for b, _ in res) / nb * 1e6, 1)
            if mode == "async":
                out["c2_backend_async_launches_for_8_buckets"] = int(res[0][1])
            # the same with the ranks as native threads: what the interpreter lock shared by
            # three Python rank threads adds to the figure above
            out[f"c2_backend_{mode}_native_ranks_us_per_bucket"] = round(max(CX._allreduce_rate(3, numel, nb, 4)), 1)
        # small buckets, event-based, native rank threads: 16 buckets of 1 MiB back to back, with the
        # default gathering of small buckets into one launch and without it
        os.environ["MCCL_ALLREDUCE_ASYNC"] = "1"
        saved_cb = os.environ.get("MCCL_COALESCE_BELOW")
        try:
            small = {}
            for name, below in (("gathered", None), ("one_launch_each", "0")):
                if below is None:
                    os.environ.pop("MCCL_COALESCE_BELOW", None)
                else:
                    os.environ["MCCL_COALESCE_BELOW"] = below
                small[name] = round(max(CX._allreduce_rate(3, (1 << 20) // 4, 16, 6)), 1)
            out["backend_async_native_ranks_16_buckets_of_1MiB_us_per_bucket"] = small
        finally:
            if saved_cb is None:
                os.environ.pop("MCCL_COALESCE_BELOW", None)
            else:
                os.environ["MCCL_COALESCE_BELOW"] = saved_cb
        os.environ.pop("MCCL_ALLREDUCE_ASYNC", None)

        os.environ.update({"MCCL_ALLREDUCE_ALGO": "ring", "MCCL_WIRE": "host"})
        n3 = W.C3["numel"]

        def c3(r, pg):
            t = torch.randn(n3, device="cuda") * 1e-4
            torch.cuda.synchronize()
            # the first two calls allocate and first touch this rank's pinned buffers (two send
            # buffers used in turn, two receive buffers): some 300 and 160 ms; from the third on
            # the call costs what the wire and the device work cost
            best, walls = None, []
            for rep in range(5):
                pg.barrier().wait()
                t0 = time.perf_counter()
                pg.allreduce([t]).wait()
                wall = time.perf_counter() - t0
                walls.append(wall)
                st = CX._wire_stats(pg)
                if rep >= 2 and (best is None or wall < best[2]):
                    best = (st[4], st[2], wall, [round(x, 2) for x in st[6:11]])
            return best + (walls[0],)
        res = run(4, c3)
        out["c3_backend_host_wire_fold_ms_per_rank"] = [round(r[0], 2) for r in res]
        out["c3_backend_host_wire_fold_PCIe_GBps_best_rank"] = round(max(r[1] / r[0] / 1e6 for r in res), 1)
        out["c3_backend_host_wire_allreduce_wall_ms"] = round(max(r[2] for r in res) * 1e3, 1)
        out["c3_backend_host_wire_first_call_wall_ms"] = round(max(r[4] for r in res) * 1e3, 1)
        # host milliseconds of the slowest rank's legs: wire form (encode into pinned memory), reduce-scatter
        # leg of the wire (one memcpy per message: the delivery), fold, allgather leg, casts on arrival
        out["c3_backend_host_wire_legs_ms"] = max(res, key=lambda r: r[2])[3]
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    return out


def extras(args, q, K, H, L, W, torch, np, tensors, wires, chunks, plan, step_segs, measure, gbs, results):
    """Secondary measurements: the other legs of C2 and the other configurations."""
    out = {}
    world, numel = 3, W.C2["numel"]
    sets = len(tensors)
    steps, warm = max(20, args.steps // 4), 5

    # what a plain copy kernel reaches at the same footprint (39.3 MB in, 39.3 MB out per launch,
    # cold-rotated) and at 1 GiB: the practical ceiling next to the published 8 TB/s
    # (filled with random bytes: a copy of zero-filled buffers runs about 5 % faster on this part)
    half = numel * 6
    pool = torch.randint(0, 256, (16 * half,), dtype=torch.uint8, device="cuda")
    ms, _ = measure(lambda i: q.copy(pool.data_ptr() + (2 * (i % 8) + 1) * half, pool.data_ptr() + 2 * (i % 8) * half, half),
                    steps, warm)
    out["plain_copy_same_footprint_GBps"] = round(gbs(2 * half, ms / steps), 1)
    del pool
    big = torch.randint(0, 256, (4 << 30,), dtype=torch.uint8, device="cuda")
    ms, _ = measure(lambda i: q.copy(big.data_ptr() + (2 * (i % 2) + 1) * (1 << 30), big.data_ptr() + 2 * (i % 2) * (1 << 30), 1 << 30),
                    10, 2)
    out["plain_copy_1GiB_GBps"] = round(gbs(2 << 30, ms / 10), 1)
    del big

    # one-directional ceilings at the bucket launch's own footprint (78,643,200 B, cold-rotated): a
    # launch that only reads that many bytes and one that only writes them
    fp = numel * 12
    if L.bench_lib() is not None:  # the probe launch is the measurement build's (python -m mccl_amd.build --bench)
        probe = torch.randint(0, 256, (8 * fp,), dtype=torch.uint8, device="cuda")
        for write, name in ((False, "read_only"), (True, "write_only")):
            ms, _ = measure(lambda i, write=write: q.probe_stream(probe.data_ptr() + (i % 8) * fp, fp, write), steps, warm)
            out[f"{name}_same_footprint_us"] = round(ms / steps * 1e3, 2)
            out[f"{name}_same_footprint_GBps"] = round(gbs(fp, ms / steps), 1)
        del probe
    else:
        out["read_only_same_footprint_us"] = out["write_only_same_footprint_us"] = None

    # the gate of the hold form: the rate measured on this device when the library started, against
    # gates a few per cent earlier and later (each on a context of its own, made with the override)
    lat_ticks, bpt, measured = q.hold_model()
    sweep = {}
    saved = os.environ.get("MCCLX_HOLD_BYTES_PER_TICK")
    try:
        for pct in (-6, -3, 0, 3, 6):
            os.environ["MCCLX_HOLD_BYTES_PER_TICK"] = str(int(bpt * (1 - pct / 100.0)))
            qq = K.ReduceQueue(0)
            try:
                ms, _ = measure(lambda i: qq.fold(plan, step_segs(i % sets, out_tensors=results[i % sets])), steps, warm,
                                queue=qq)
            finally:
                qq.close()
            sweep[f"{pct:+d}%"] = round(ms / steps * 1e3, 2)
    finally:
        if saved is None:
            os.environ.pop("MCCLX_HOLD_BYTES_PER_TICK", None)
        else:
            os.environ["MCCLX_HOLD_BYTES_PER_TICK"] = saved
    out["c2_fold_us_by_gate_shift"] = sweep  # "+3%": the gate 3 % later than the one the library uses

    # the headline launch in the plain form (one block per tile, loads then stores, reads and writes
    # mixed on the memory bus) instead of the hold form (all loads, then all stores) it takes by default
    q.set_hold(False)
    ms, _ = measure(lambda i: q.fold(plan, step_segs(i % sets, out_tensors=results[i % sets])), steps, warm)
    q.set_hold(True)
    out["c2_fold_plain_form_us"] = round(ms / steps * 1e3, 2)
    out["c2_fold_plain_form_GBps"] = round(gbs(fp, ms / steps), 1)

    # the fold as the scheduler issues it: result written in place over the owner's fp32 chunk
    ms, _ = measure(lambda i: q.fold(plan, step_segs(i % sets)), steps, warm)
    out["c2_fold_in_place_us"] = round(ms / steps * 1e3, 2)
    out["c2_fold_in_place_GBps"] = round(gbs(numel * 12, ms / steps), 1)

    # C2 with the bf16 wire copy for the allgather leg also written (14 B/elem)
    ms, _ = measure(lambda i: q.fold(plan, step_segs(i % sets, with_wire_out=True)), steps, warm)
    out["c2_fold_with_wire_out_GBps"] = round(gbs(numel * 14, ms / steps), 1)

    # the same fold with four buckets in ONE launch (the batched entry point): the fixed cost of a
    # launch (about 2 us of ramp-up and drain) is paid once per 100 MiB instead of once per 25 MiB
    nb = min(4, sets)
    ms, _ = measure(lambda i: q.fold(plan, [s for b in range(nb) for s in step_segs((nb * i + b) % sets)]),
                    max(10, steps // nb), warm)
    out["c2_fold_4_buckets_per_launch_GBps"] = round(gbs(nb * numel * 12, ms / max(10, steps // nb)), 1)

    # NOT the headline: consecutive buckets on TWO reduce queues (two contexts, two streams), so that
    # one launch's ramp-up fills the other's drain and the gap between dependent launches is hidden.
    # Out-of-place results as in the headline; wall clock around both graphs, best of 5.  Launches
    # that overlap do not have the memory system to themselves: the hold form (reads, then writes)
    # is switched off on both queues, as the process group does when it runs two queues.
    q2 = K.ReduceQueue(0)
    try:
        q.set_hold(False)
        q2.set_hold(False)
        per_q = max(50, steps // 2)
        graphs = []
        for qi, qq in enumerate((q, q2)):
            qq.graph_begin()
            for i in range(per_q):
                s_ = (2 * i + qi) % sets
                qq.fold(plan, step_segs(s_, out_tensors=results[s_]))
            graphs.append(qq.graph_end())
        best = None
        for _ in range(5):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            q.graph_launch(graphs[0])
            q2.graph_launch(graphs[1])
            q.drain()
            q2.drain()
            dt = time.perf_counter() - t0
            best = dt if best is None or dt < best else best
        q.graph_destroy(graphs[0])
        q2.graph_destroy(graphs[1])
        out["c2_fold_overlapped_on_two_queues_us_per_bucket"] = round(best / (2 * per_q) * 1e6, 2)
        out["c2_fold_overlapped_on_two_queues_GBps"] = round(numel * 12 / (best / (2 * per_q)) / 1e9, 1)
    finally:
        q.set_hold(True)
        del q2

    # C2 with the peers' bf16 chunks left where a NIC or a host transport puts them: pinned host
    # memory, read by the kernel through its device alias (4 B/elem cross PCIe, 8 B/elem stay in HBM)
    pin = []
    try:
        alias = []
        for p in range(world):
            hptr, dptr = q.host_alloc(numel * 2)
            pin.append(hptr)
            alias.append(dptr)
            q.copy(dptr, wires[0][p].data_ptr(), numel * 2)
        q.drain()
        psegs = []
        for R, (start, cnt, _, _) in enumerate(chunks):
            own = tensors[0][R].data_ptr() + start * 4
            psegs.append(K.make_seg(own, 0, [own] + [alias[p] + start * 2 for p in range(world) if p != R], cnt))
        ms, _ = measure(lambda i: q.fold(plan, psegs), 10, 2)
        out["c2_fold_peers_in_pinned_host_us"] = round(ms / 10 * 1e3, 1)
        out["c2_fold_peers_in_pinned_host_PCIe_GBps"] = round(gbs(numel * 4, ms / 10), 1)
        out["c2_fold_peers_in_pinned_host_GBps"] = round(gbs(numel * 12, ms / 10), 1)
    finally:
        for hptr in pin:
            q.host_free(hptr)

    # the same fused fold over other bucket sizes (3 ranks, bf16 wire, x 1/3; cold: copies rotate
    # over >= 600 MB): where the fixed cost of a launch stops mattering
    sweep = {}
    for mib in (1, 4, 16, 64, 256):
        n = mib * (1 << 20) // 4
        ncopies = max(2, min(256, (640 << 20) // (n * 12)))
        ch = H.chunkize(n, 1, world)
        bufs = [([torch.randn(n, device="cuda") * 1e-3 for _ in range(world)],
                 [(torch.randn(n, device="cuda") * 1e-3).to(torch.bfloat16) for _ in range(world)]) for _ in range(ncopies)]

        def sz_step(i, bufs=bufs, ch=ch, ncopies=ncopies):
            ts, ws = bufs[i % ncopies]
            q.fold(plan, [K.make_seg(ts[R].data_ptr() + 4 * st, 0,
                                     [ts[R].data_ptr() + 4 * st] + [ws[p].data_ptr() + 2 * st for p in range(world) if p != R], c)
                          for R, (st, c, _, _) in enumerate(ch)])
        reps = max(10, min(200, (16 << 30) // (n * 12)))
        ms, _ = measure(sz_step, reps, 5)
        sweep[f"{mib}MiB"] = {"us": round(ms / reps * 1e3, 2), "GBps": round(gbs(n * 12, ms / reps), 1)}
        if mib == 1:
            # four 1 MiB buckets in ONE launch (12 segments by value): what the event-based path
            # issues for small buckets that gather while a launch is in flight
            def four(i, bufs=bufs, ch=ch, ncopies=ncopies):
                segs = []
                for b in range(4):
                    ts, ws = bufs[(4 * i + b) % ncopies]
                    segs += [K.make_seg(ts[R].data_ptr() + 4 * st, 0,
                                        [ts[R].data_ptr() + 4 * st] + [ws[p].data_ptr() + 2 * st for p in range(world) if p != R], c)
                             for R, (st, c, _, _) in enumerate(ch)]
                q.fold(plan, segs)
            ms, _ = measure(four, reps, 5)
            sweep["4x1MiB_in_one_launch"] = {"us": round(ms / reps * 1e3, 2), "us_per_bucket": round(ms / reps * 1e3 / 4, 2),
                                             "GBps": round(gbs(4 * n * 12, ms / reps), 1)}
        del bufs
    out["fold_by_bucket_size"] = sweep

    # encode leg: 3 ranks x (4 B read + 2 B write) per element
    def enc(i):
        s = i % sets
        q.fold(K.make_plan(L.BF16, 1, io=L.IO_OWN_FIRST_F32),
               [K.make_seg(0, wires[s][r].data_ptr(), [tensors[s][r].data_ptr()], numel) for r in range(world)])
    ms, _ = measure(enc, steps, warm)
    out["c2_encode_GBps"] = round(gbs(world * numel * 6, ms / steps), 1)
    # its ceilings: the plain copy kernel over the same footprint (118 MB per launch, cold) and the
    # same encode on a tensor large enough for the fixed cost of a launch not to matter (64 Mi elements)
    half = world * numel * 3
    pool = torch.randint(0, 256, (8 * half,), dtype=torch.uint8, device="cuda")
    ms, _ = measure(lambda i: q.copy(pool.data_ptr() + (2 * (i % 4) + 1) * half, pool.data_ptr() + 2 * (i % 4) * half, half),
                    steps, warm)
    out["c2_encode_footprint_plain_copy_GBps"] = round(gbs(2 * half, ms / steps), 1)
    del pool
    nbig = 64 << 20
    src = [torch.randn(nbig, device="cuda") * 1e-3 for _ in range(2)]
    dst = [torch.empty(nbig, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    ms, _ = measure(lambda i: q.fold(K.make_plan(L.BF16, 1, io=L.IO_OWN_FIRST_F32),
                                     [K.make_seg(0, dst[i % 2].data_ptr(), [src[i % 2].data_ptr()], nbig)]), 10, 2)
    out["encode_64Mi_elements_GBps"] = round(gbs(nbig * 6, ms / 10), 1)
    del src, dst

    # whole allreduce of the bucket for all 3 virtual ranks: fused vs the reference's launch sequence
    ws = H.Workspace(q, 3 * (numel * 2 + 256) + 3 * (2 * ((numel + 2) // 3) * 2 + 256))
    for mode, name in ((L.REPLAY_DIRECT, "direct"), (L.REPLAY_FUSED, "fused"), (L.REPLAY_STEPWISE, "stepwise")):
        def rep(i, mode=mode):
            H.allreduce_replay(tensors[i % sets], "avg", L.ALGO_BUTTERFLY, wire_bf16=True, mode=mode,
                               queue=q, workspace=ws, sync=False)
        q.drain()
        # cross-stream waits cannot be recorded: time these eagerly
        for i in range(warm):
            rep(i)
        q.drain()
        q.timer_begin()
        for i in range(steps):
            rep(i)
        ms = q.timer_end()
        out[f"c2_allreduce_{name}_us_per_bucket"] = round(ms / steps * 1e3, 1)
    # the fused schedules again, their launches recorded into a graph (no host launch cost between
    # them): FUSED = encode + a fold over bf16 copies (the shape across GPUs), DIRECT = ONE fold that
    # reads the three fp32 tensors and stores the result into all three (ranks sharing one GPU:
    # 12 B read + 12 B written per element)
    import ctypes as C
    for mode, name in ((L.REPLAY_FUSED, "fused"), (L.REPLAY_DIRECT, "direct")):
        reps = []
        for s in range(sets):
            r = L.Replay()
            r.world, r.algo, r.op, r.dtype = world, L.ALGO_BUTTERFLY, L.AVG, L.F32
            r.wire_bf16, r.mode, r.acc, r.reserved, r.numel = 1, mode, L.ACC_STEP, 0, numel
            ptrs = (C.c_void_p * world)(*[t.data_ptr() for t in tensors[s]])
            r.tensors, r.workspace, r.workspace_bytes = ptrs, ws.ptr, ws.nbytes
            reps.append((r, ptrs))
        ms, _ = measure(lambda i: L.check(L.lib().mcclx_allreduce_replay(q.handle, C.byref(reps[i % sets][0]))), steps, warm)
        out[f"c2_allreduce_{name}_in_graph_us_per_bucket"] = round(ms / steps * 1e3, 1)
    out["c2_allreduce_direct_in_graph_GBps"] = round(gbs(world * numel * 8, ms / steps), 1)
    ws.free()
    # its ceiling: the plain copy kernel over the same footprint (78.6 MB in, 78.6 MB out, cold)
    half = world * numel * 4
    pool = torch.randint(0, 256, (8 * half,), dtype=torch.uint8, device="cuda")
    ms, _ = measure(lambda i: q.copy(pool.data_ptr() + (2 * (i % 4) + 1) * half, pool.data_ptr() + 2 * (i % 4) * half, half),
                    steps, warm)
    out["c2_allreduce_direct_footprint_plain_copy_us"] = round(ms / steps * 1e3, 1)
    out["c2_allreduce_direct_footprint_plain_copy_GBps"] = round(gbs(2 * half, ms / steps), 1)
    del pool

    # C1: ring, 2 ranks, 1 Mi fp32, SUM: one k=2 fold per chunk
    x = [torch.randn(W.C1["numel"], device="cuda") for _ in range(2 * 8)]
    c1 = H.chunkize(W.C1["numel"], 1, 2)

    def c1_step(i):
        a, b = x[2 * (i % 8)], x[2 * (i % 8) + 1]
        segs = []
        for ch, (s, c, _, _) in enumerate(c1):
            owner = (a, b)[(ch - 1) % 2]
            first, last = (a, b)[ch], (a, b)[(ch + 1) % 2]
            segs.append(K.make_seg(owner.data_ptr() + 4 * s, 0, [first.data_ptr() + 4 * s, last.data_ptr() + 4 * s], c))
        q.fold(K.make_plan(L.F32, 2), segs)
    ms, _ = measure(c1_step, steps, warm)
    out["c1_ring_fold_us"] = round(ms / steps * 1e3, 2)
    out["c1_ring_fold_GBps"] = round(gbs(12_582_912, ms / steps), 1)
    del x

    # C4: 4096 x 64 KiB messages x 3 ranks, one persistent table launch
    n4, m4 = W.C4["numel"], W.C4["messages"]
    r4 = [torch.rand(n4 * m4, device="cuda") * 2 - 1 for _ in range(3)]
    segs4 = [K.make_seg(r4[0].data_ptr() + 4 * n4 * m, 0, [t.data_ptr() + 4 * n4 * m for t in r4], n4)
             for m in range(m4)]
    p4 = K.make_plan(L.F32, 3, topo=L.TOPO_BINOMIAL)
    ms, _ = measure(lambda i: q.fold(p4, segs4), 10, 2)
    out["c4_tree_batched_us_total"] = round(ms / 10 * 1e3, 1)
    out["c4_tree_batched_ns_per_message"] = round(ms / 10 * 1e6 / m4, 1)
    out["c4_tree_batched_GBps"] = round(gbs(4 * 65536 * m4, ms / 10), 1)
    # the whole tree allreduce of the 4096 messages as ONE list replay: one fold launch for all
    # messages, which also stores every result into ranks 1 and 2 (3 reads + 3 writes per element)
    reps4 = (L.Replay * m4)()
    keep4 = []
    for m in range(m4):
        r = reps4[m]
        r.world, r.algo, r.op, r.dtype = 3, L.ALGO_TREE, L.SUM, L.F32
        r.wire_bf16, r.mode, r.acc, r.reserved, r.numel = 0, L.REPLAY_FUSED, L.ACC_STEP, 0, n4
        ptrs = (C.c_void_p * 3)(*[t.data_ptr() + 4 * n4 * m for t in r4])
        keep4.append(ptrs)
        r.tensors, r.workspace, r.workspace_bytes = ptrs, None, 0
    ms, _ = measure(lambda i: L.check(L.lib().mcclx_allreduce_replay_many(q.handle, reps4, m4)), 10, 2)
    out["c4_tree_allreduce_4096_messages_us_total"] = round(ms / 10 * 1e3, 1)
    out["c4_tree_allreduce_4096_messages_GBps"] = round(gbs((3 + 3) * 65536 * m4, ms / 10), 1)
    del r4, segs4, reps4, keep4

    # C3: ring, 4 ranks, 110,000,002 fp32, bf16 wire, own operand last; peers in HBM, then in pinned host memory
    n3 = W.C3["numel"]
    c3 = H.chunkize(n3, 1, 4)
    t3 = [torch.randn(n3, device="cuda") * 1e-4 for _ in range(4)]
    w3 = [K.encode_bf16(t, queue=q) for t in t3]
    q.drain()
    p3 = K.make_plan(L.BF16, 4, io=L.IO_OWN_LAST_F32)

    def c3_segs(wire_ptr):
        segs = []
        for ch, (s, c, _, _) in enumerate(c3):
            o = (ch - 1) % 4
            ins = [wire_ptr[(ch + j) % 4] + 2 * s for j in range(3)] + [t3[o].data_ptr() + 4 * s]
            segs.append(K.make_seg(t3[o].data_ptr() + 4 * s, 0, ins, c))
        return segs
    hbm_segs = c3_segs([w.data_ptr() for w in w3])
    ms, _ = measure(lambda i: q.fold(p3, hbm_segs), 10, 2)
    out["c3_ring_fold_hbm_us"] = round(ms / 10 * 1e3, 1)
    out["c3_ring_fold_hbm_GBps"] = round(gbs(n3 * 14, ms / 10), 1)
    host_bufs = []
    try:
        dev_ptrs = []
        for w in w3:
            hptr, dptr = q.host_alloc(n3 * 2)
            host_bufs.append(hptr)
            dev_ptrs.append(dptr)
            q.copy(dptr, w.data_ptr(), n3 * 2)
        q.drain()
        pin_segs = c3_segs(dev_ptrs)
        ms, _ = measure(lambda i: q.fold(p3, pin_segs), 3, 1)
        out["c3_ring_fold_pinned_host_ms"] = round(ms / 3, 2)
        out["c3_ring_fold_pinned_host_PCIe_GBps"] = round(gbs(n3 * 6, ms / 3), 1)
    finally:
        for hptr in host_bufs:
            q.host_free(hptr)
    del t3, w3

    del hbm_segs
    torch.cuda.empty_cache()
    try:
        out.update(backend_extras(torch, W))
    except Exception as e:
        out["backend_extras_error"] = f"{type(e).__name__}: {e}"

    # C5: reduce_scatter (8-input bf16 fold per rank, per-step rounding) and the allgather copy
    n5, w5 = W.C5["numel"], 8
    ch5 = n5 // w5
    i5 = [(torch.randn(n5, device="cuda") * 1e-2).to(torch.bfloat16) for _ in range(w5)]
    o5 = [torch.empty(ch5, dtype=torch.bfloat16, device="cuda") for _ in range(w5)]
    for acc, name in ((L.ACC_STEP, "ref_exact"), (L.ACC_F32, "f32acc")):
        p5 = K.make_plan(L.BF16, w5, acc=acc)
        segs5 = [K.make_seg(o5[r].data_ptr(), 0,
                            [i5[r].data_ptr() + 2 * ch5 * r] + [i5[p].data_ptr() + 2 * ch5 * r for p in range(w5) if p != r],
                            ch5) for r in range(w5)]
        ms, _ = measure(lambda i: q.fold(p5, segs5), 5, 1)
        out[f"c5_reduce_scatter_{name}_us"] = round(ms / 5 * 1e3, 1)
        out[f"c5_reduce_scatter_{name}_GBps"] = round(gbs(9 * ch5 * 2 * w5, ms / 5), 1)
    g5 = torch.empty(n5, dtype=torch.bfloat16, device="cuda")
    ms, _ = measure(lambda i: q.copy_batched([(g5.data_ptr() + 2 * ch5 * p, o5[p].data_ptr(), 2 * ch5) for p in range(w5)]), 5, 1)
    out["c5_allgather_copy_one_rank_GBps"] = round(gbs(2 * n5 * 2, ms / 5), 1)
    return out


if __name__ == "__main__":
    main()
