#!/usr/bin/env python3
"""Stage throughput on one MI355X: one pipeline rank's microbatch loop
(forward, backward, fp32 gradient accumulation, residual stash/restore) in the
order the schedule's task table dictates, with synthetic boundary tensors.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3]

A step is one full pass over the rank's row of the task table (all
microbatches).  Prints one JSON line: the metric, its configuration, the roofline of the
dominant kernel (timed live with HIP events) and a CPU baseline.
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

from jaxpp_amd import runtime as rt            # noqa: E402
from jaxpp_amd import schedules as S           # noqa: E402
from jaxpp_amd.model import workloads          # noqa: E402
from jaxpp_amd.plan import make_rank_plan      # noqa: E402
from jaxpp_amd.rank_loop import RankLoop       # noqa: E402
from jaxpp_amd.types import TaskType           # noqa: E402

MFMA_BF16_PEAK = 2.5e15     # dense bf16 FLOP/s, MI355X
HBM_PEAK = 8.0e12           # B/s


def synthetic_pool(n_elems: int, std: float, seed: int) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rt.to_bf16_bits(rng.standard_normal(n_elems, dtype=np.float32) * np.float32(std))


class Workbench:
    """Device state of one workload: executor, parameters, boundary tensors.

    Synthetic inputs: every parameter matrix and every boundary tensor is a buffer of its own,
    filled from windows - at per-tensor offsets - of one N(0, 0.02^2) pool of 2^26 values
    (weights) and one N(0, 1) pool (boundary activations and cotangents), norm gains one,
    biases zero.  Generating 1.7e9 to 1.2e10 independent normals per workload on the host would
    take minutes per run; the kernels see the same value distribution, no tensor aliases
    another, and no work is skipped.  (The parity tests draw every tensor from its own seed.)"""

    def __init__(self, wl, fused=True, two_streams=False, wgrad_group=0):
        self.wl = wl
        spec = wl.layer
        sched = getattr(S, wl.schedule)(**wl.schedule_kwargs)
        self.plan = make_rank_plan(sched, wl.n_mubatches, wl.rank)
        self.ex = rt.StageExecutor(spec, self.plan.n_chunks, wl.layers_per_stage,
                                   self.plan.max_live, self.plan.split_backward, fused,
                                   two_streams, wgrad_group)
        lib = rt.load()
        # parameters: slices of one N(0, 0.02^2) pool at per-tensor offsets;
        # norm gains one, biases zero
        pool_n = 1 << 26
        wpool = rt.DeviceBuffer.from_numpy(synthetic_pool(pool_n, 0.02, 0))
        ones = rt.DeviceBuffer.from_numpy(rt.to_bf16_bits(np.ones(16384, np.float32)))
        import ctypes as C
        k = 0
        for c in range(self.plan.n_chunks):
            for li in range(wl.layers_per_stage):
                for name, rows, cols in self.ex.params:
                    dst = self.ex._ptr(lib.jpp_stage_param_ptr, c, li, name)
                    n = rows * cols
                    if rows > 1:
                        done = 0
                        while done < n:
                            k += 1
                            off = (k * 7919 * 4096) % (pool_n // 2)
                            take = min(n - done, pool_n - off)
                            rt.check(lib.jpp_memcpy_d2d_async(dst + 2 * done, wpool.ptr + 2 * off,
                                                              2 * take, None))
                            done += take
                    elif name.endswith("_g"):
                        rt.check(lib.jpp_memcpy_d2d_async(dst, ones.ptr, 2 * n, None))
        rt.sync()
        # boundary tensors ~N(0,1): one per (chunk, microbatch) and direction
        act = spec.tokens * spec.hidden
        bpool_n = act + (1 << 22)
        bpool = rt.DeviceBuffer.from_numpy(synthetic_pool(bpool_n, 1.0, 1))
        self.x_in, self.dy_in = {}, {}
        j = 0
        for c in range(self.plan.n_chunks):
            for m in range(wl.n_mubatches):
                for store in (self.x_in, self.dy_in):
                    j += 1
                    buf = rt.DeviceBuffer(act * 2)
                    off = (j * 104729 * 8) % (1 << 22)
                    rt.check(lib.jpp_memcpy_d2d_async(buf.ptr, bpool.ptr + 2 * off, act * 2, None))
                    store[c, m] = buf
        self.out = [rt.DeviceBuffer(act * 2), rt.DeviceBuffer(act * 2)]
        self.loop = RankLoop(self.ex, self.plan, overlap_fused=two_streams)
        rt.sync()
        self._keep = (wpool, ones, bpool)

    def close(self):
        """Frees the executor and every buffer (the next workload needs the memory)."""
        self.ex.close()
        self.x_in, self.dy_in, self.out, self._keep, self.loop = {}, {}, [], (), None

    def step(self, stream=None):
        ex = self.ex
        ex.zero_grads(stream)                 # `Add.state`: accumulators start from zero

        def io(pt, lane):
            m = pt.task.mubatch_idx
            src = self.x_in if pt.exec_kind is TaskType.FWD else self.dy_in
            return src[pt.chunk, m].ptr, self.out[lane].ptr

        self.loop.run(io, stream=stream)
        ex.join(stream)                       # the step ends when the last weight gradient has landed

    def step_flops(self) -> float:
        wl = self.wl
        return 3.0 * wl.layer.fwd_flops() * wl.layers_per_stage * self.plan.n_chunks * wl.n_mubatches


# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# of this script (the counters scaled by what they read for copy kernels of known size), keyed by
# (workload, kernel class, microbatches per weight-gradient launch): a launch over four
# microbatches reads four operand pairs and the accumulator once
MEASURED_TRAFFIC = {("cfg3", "gemm_tn_accf32_256x256w8_multi", 4): 1.2677e10,  # a layer per launch
                    ("cfg3", "gemm_tn_accf32_256x256w8", 4): 2.879e9,
                    ("cfg3", "gemm_tn_accf32_256x256w8", 1): 1.005e9}  # one weight per launch


def dominant_gemm_class(wl) -> str:
    # weight-gradient GEMM with the fp32 accumulate epilogue: a third of the
    # FLOPs and the longest kernel per call
    # (narrow layers: 128x128 tiles, at most two per CU, so the 3-stage variant)
    big = wl.layer.hidden >= 4096
    return "gemm_tn_accf32_256x256w8" if big else "gemm_tn_accf32_128x128w8s3"


def measured_dominant_class(wb, wl) -> str:
    """The weight-gradient class that takes the most time in one (untimed) step with every
    class probed: which launches the stage uses - per weight, or a layer's weight gradients as
    one grid - follows from the shapes, so it is read off rather than restated here."""
    with rt.probe("*") as pr:
        wb.step()
        rt.sync()
    for prefix in ("gemm_tn_accf32", "gemm_tn_", "gemm_"):   # (no fused accumulate: the bf16 form)
        acc = {k: v[1] for k, v in pr.classes.items() if k.startswith(prefix)}
        if acc:
            return max(acc, key=acc.get)
    return dominant_gemm_class(wl)


def default_wgrad_group(wl, two_streams: bool) -> int:
    """How many consecutive microbatches share one weight-gradient product per weight (the
    fp32 accumulator is then read and written once per group).  Measured on MI355X, A/B on one
    box: Llama-8B-shaped stage 1397-1402 ms/step ungrouped, 1393-1395 in pairs, 1373-1379 in
    fours (73 GB); 70B-shaped 4579-4584 / 4545-4552 / 4543-4554 ms (197 / 215 / 251 GB), so
    pairs there.  The Mixtral-shaped stage 2671-2699 ms ungrouped, 2615-2627 in pairs (206 /
    236 GB; the experts' grouped contraction takes the pairs' own row groups): pairs, fours do
    not fit.  BERT-large-shaped stage: a layer's four weight gradients are 192 tiles, three
    quarters of one round of the 256 CUs; four microbatches' are three full rounds - 52.5 ms
    ungrouped, 51.5 in pairs, 51.0 in fours on one stream, 52.0 / 52.0 / 51.0 with the weight
    gradients on a second stream."""
    if wl.dtype != "bf16":
        return 1
    if wl.layer.family == "mixtral" or wl.layer.hidden >= 8192:
        return 2
    return 4


def cpu_baseline(wl, budget_layers: int = 1):
    """The numpy oracle on the host cores: one microbatch through
    `budget_layers` layer(s), forward + backward-input + backward-weight +
    accumulate, scaled to the whole row (layers x chunks x microbatches)."""
    from oracle import layers as L
    from oracle import stage as O
    from jaxpp_amd.model import boundary_tensor, init_layer_params
    spec = wl.layer
    cfg = L.LayerCfg(**spec.as_dict())
    nm = L.Numerics.f32()
    params = [init_layer_params(spec, 0, li) for li in range(budget_layers)]
    shape = (spec.tokens, spec.hidden)
    x = boundary_tensor("x", 0, 0, shape)
    dy = boundary_tensor("dy", 0, 0, shape)
    ro = O.RankOracle(cfg, {0: params}, nm)
    t0 = time.perf_counter()
    ro.fwd(0, 0, x)
    ro.bwd(0, 0, dy)
    dt = time.perf_counter() - t0
    n_chunks = len([s for s in range(wl.schedule_kwargs["num_stages"])
                    if getattr(S, wl.schedule)(**wl.schedule_kwargs).get_mpmd_idx(s) == wl.rank])
    scale = wl.layers_per_stage * n_chunks * wl.n_mubatches / budget_layers
    try:
        import threadpoolctl
        threads = max((p.get("num_threads", 1) for p in threadpoolctl.threadpool_info()),
                      default=1)
    except Exception:
        threads = os.cpu_count() or 1
    return {"value": wl.tokens_per_step / (dt * scale), "unit": "tokens/s", "cores": int(threads),
            "kind": "port",
            "sample": (f"numpy fp32 oracle, 1 microbatch x {budget_layers} layer "
                       f"fwd+bwd_i+bwd_w+accumulate = {dt:.2f} s, extrapolated x{scale:g}")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg3", choices=["cfg2", "cfg3", "cfg4", "cfg5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-side-runs", action="store_true",
                    help="leave out the short extra measurements the default line carries: the "
                         "same row with one weight-gradient product per microbatch "
                         "(`ungrouped`) and, for the default workload, three steps each of "
                         "cfg2 / cfg4 / cfg5 (`other_workloads`)")
    ap.add_argument("--n-mubatches", type=int, default=None,
                    help="override the workload's microbatch count (shorter runs under "
                         "rocprofv3 --pmc, which serialises every dispatch; not the headline)")
    ap.add_argument("--unfused-accumulate", action="store_true",
                    help="bf16 weight gradient + separate fp32 accumulate pass")
    ap.add_argument("--two-streams", choices=["on", "off"], default="off",
                    help="weight gradients on the stage's second stream and the forward of a "
                         "fused entry beside its backward.  Measured: 52.0 ms against 52.5 at "
                         "cfg2 with ungrouped weight gradients, no difference with groups of "
                         "four (51.0); -1%% at cfg3, -2%% at cfg5, and per-kernel timings then "
                         "include the other stream's kernels")
    ap.add_argument("--wgrad-group", type=int, default=None,
                    help="weight gradients of this many consecutive microbatches as one product "
                         "per weight (1: per microbatch; default: see default_wgrad_group)")
    ap.add_argument("--probe", default=None, help="kernel class to time (default: dominant GEMM)")
    ap.add_argument("--graph", choices=["auto", "on", "off"], default="auto", nargs="?", const="on",
                    help="record the step into a HIP graph after the warm-up and time replays "
                         "of it (no host launch work in the timed region); the per-kernel probe "
                         "cannot see inside a replay, so `roofline` then comes from one more "
                         "eager step after the timed ones.  auto: for narrow layers (hidden < "
                         "2048: thousands of small launches per step, +3 %%), not for wide ones "
                         "(the GPU is busy 99.8 %% of an eager step)")
    ap.add_argument("--kernel-table", action="store_true",
                    help="instead of the one-line result, time every kernel class of the step "
                         "with HIP events (jpp_probe_begin(\"*\")) over the timed steps and print "
                         "one JSON object with a row per class: launches per step, average "
                         "duration, share of the kernel time, and the algorithmic rate against "
                         "the roofline that bounds the class (TFLOP/s of 2.5 PFLOP/s for the "
                         "matrix-core kernels, GB/s of 8 TB/s for the others).  Two events per "
                         "launch slow the step by a few per cent: the table is for shares and "
                         "rates, the headline figure comes from the default run.")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="instead of the workload, print what the matrix cores sustain on a "
                         "register-only MFMA loop (zero and random operands, both tile shapes)")
    ap.add_argument("--lds-read-rates", action="store_true",
                    help="instead of the workload, print what the fragment reads of the GEMM "
                         "and attention kernels cost in LDS cycles per wave-level read, address "
                         "pattern by pattern (8 waves reading in a loop), with the operand "
                         "slabs' chunk swizzle of the tree and with the one used before it")
    ap.add_argument("--after-loop", action="store_true",
                    help="also time the step behind the loop - Adam over the stage's f32 "
                         "gradient accumulators, rewriting the bf16 parameters - and report it "
                         "as `after_loop` (not part of `value`; needs 12 more bytes per "
                         "parameter on the device)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build executes one pipeline rank on one GPU; --gpus > 1 is not "
              "supported (the other ranks' boundary tensors are synthetic).", file=sys.stderr)
        sys.exit(2)
    rt.require_gpu()
    if args.mfma_ceiling:
        print(json.dumps({"mfma_sustained_tflops": {
            "32x32x16_zero_operands": rt.mfma_rate(32, False, 200000),
            "32x32x16_random_operands": rt.mfma_rate(32, True, 200000),
            "16x16x32_zero_operands": rt.mfma_rate(16, False, 100000),
            "16x16x32_random_operands": rt.mfma_rate(16, True, 100000)},
            "published_peak_tflops": MFMA_BF16_PEAK / 1e12}))
        return
    if args.lds_read_rates:
        print(json.dumps(lds_read_rates()))
        return
    wl = workloads()[args.workload]
    if args.n_mubatches:
        import dataclasses
        wl = dataclasses.replace(wl, n_mubatches=args.n_mubatches)
    two = args.two_streams == "on"
    group = args.wgrad_group if args.wgrad_group is not None else default_wgrad_group(wl, two)
    if args.unfused_accumulate:
        group = 1
    use_graph = args.graph == "on" or (args.graph == "auto" and wl.layer.hidden < 2048)
    wb = Workbench(wl, fused=not args.unfused_accumulate, two_streams=two, wgrad_group=group)
    if args.kernel_table:
        print(json.dumps(kernel_table(wb, wl, args.steps, args.warmup, two, group)))
        return

    cls = args.probe or measured_dominant_class(wb, wl)
    ms, pr = timed_steps(wb, args.steps, args.warmup, use_graph, cls)
    tokens = wl.tokens_per_step
    flops = wb.step_flops()
    spec = wl.layer
    rec = {
        "metric": "stage_tokens_per_sec_fwd_bwd",
        "value": tokens / (ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": (f"{wl.name}: {spec.family} stage, rank {wl.rank} of {wl.schedule}"
                         f"{wl.schedule_kwargs}, {self_desc(wl, wb)}; every parameter and "
                         "boundary tensor is a buffer of its own filled from windows, at "
                         "per-tensor offsets, of one N(0, 0.02^2) pool (weights) and one "
                         "N(0, 1) pool (activations, cotangents) of 2^26 values"),
            "tokens_per_step": tokens, "n_mubatches": wl.n_mubatches,
            "layers": wl.layers_per_stage * wb.plan.n_chunks,
            # the schedule's own figure: forwards whose backward has not run
            "peak_live_microbatches": wb.plan.max_live,
            # what the run holds: with weight gradients in groups, a microbatch whose weight
            # gradients wait for its group keeps its residual slot beyond the schedule's
            # release point (n_chunks * (wgrad_group - 1) slots more)
            "residual_slots": wb.plan.max_live + wb.plan.n_chunks * (max(group, 1) - 1),
            "fused_wgrad_accumulate": not args.unfused_accumulate,
            "two_streams": two, "hip_graph": bool(use_graph),
            "wgrad_group": group,
            "wgrad_group_meaning": ("weight gradients of this many consecutive microbatches run "
                                    "as one product per weight: the fp32 accumulator is read "
                                    "and written once per group and the additions inside an "
                                    "element are reassociated (equal to the per-microbatch "
                                    "run to fp32 rounding, not bit for bit); 1 = the "
                                    "reference's one accumulate per microbatch"),
            "schedule_task_fusion": not S.schedule_task_fusion_disabled(),
            "device_bytes": wb.ex.nbytes,
        },
        "algorithmic_flops_per_step": flops,
        "mfma_peak_frac": flops / (ms * 1e-3) / MFMA_BF16_PEAK,
    }
    if pr.launches:
        avg_ms = pr.total_ms / pr.launches
        hbm = pr.flops == 0
        ach = (pr.bytes if hbm else pr.flops) / (pr.total_ms * 1e-3)
        rec["roofline"] = {
            "kernel": cls, "bound": "hbm" if hbm else "mfma",
            "achieved": ach / (1e9 if hbm else 1e12),
            "peak": (HBM_PEAK / 1e9) if hbm else (MFMA_BF16_PEAK / 1e12),
            "unit": "GB/s" if hbm else "TFLOP/s",
            "frac": ach / (HBM_PEAK if hbm else MFMA_BF16_PEAK),
            "traffic": MEASURED_TRAFFIC.get((wl.name, cls, max(group, 1))),
            "launches": pr.launches, "avg_launch_ms": avg_ms,
            "algorithmic_per_launch": (pr.bytes if hbm else pr.flops) / pr.launches,
        }
    if args.after_loop:
        rec["after_loop"] = after_loop(wb, wl, args.steps)
    wb.close()
    del wb
    if group > 1 and not args.no_side_runs:
        # the same row with one weight-gradient product per microbatch (the reference's
        # lifetimes and accumulate order), a few steps
        rec["ungrouped"] = side_run(wl, args.workload, wgrad_group=1)
    if not args.no_side_runs and args.workload == "cfg3" and not args.n_mubatches:
        # the other single-GPU configurations, a few steps each, so that one run records them
        rec["other_workloads"] = {name: side_run(workloads()[name], name)
                                  for name in ("cfg2", "cfg4", "cfg5")}
    if not args.no_cpu_baseline:
        # a sample of 10-20 s on the host: about 1.2e13 FLOP at the ~1 TFLOP/s its BLAS reaches
        layers = int(round(1.2e13 / (3.0 * wl.layer.fwd_flops())))
        rec["cpu_baseline"] = cpu_baseline(wl, max(1, min(wl.layers_per_stage, layers)))
    print(json.dumps(rec))


def timed_steps(wb, steps: int, warmup: int, use_graph: bool, cls: str | None):
    """`warmup` untimed steps, then `steps` timed ones between two HIP events; returns
    (ms per step, the probe of kernel class `cls`).

    The host enqueues a step in a fraction of the time the GPU takes to run it.  It is kept at
    most two steps ahead (the queue never drains, so the timing is unaffected): tools that
    keep a record per dispatch in flight, rocprofv3 among them, do not survive a backlog of
    100 000 launches."""
    ends = []

    def paced_step():
        if len(ends) >= 2:
            ends.pop(0).sync()
        wb.step()
        ev = rt.Event()
        ev.record()
        ends.append(ev)

    for _ in range(warmup):
        paced_step()
    rt.sync()
    start, stop = rt.Event(), rt.Event()
    if use_graph:
        stream = rt.Stream()
        if not warmup:
            wb.step(stream.ptr)               # first launches configure their kernels
            stream.sync()
        wb.ex.quiesce()
        graph = rt.Graph(stream)
        with graph:
            wb.step(stream.ptr)
        graph.launch()                        # one untimed replay
        stream.sync()
        start.record(stream.ptr)
        for _ in range(steps):
            graph.launch()
        stop.record(stream.ptr)
        stop.sync()
        with rt.probe(cls or "-") as pr:
            wb.step()
            rt.sync()
    else:
        with rt.probe(cls or "-") as pr:
            start.record()
            for _ in range(steps):
                paced_step()
            stop.record()
            stop.sync()
    rt.sync()
    return start.elapsed_ms(stop) / steps, pr


def side_run(wl, name: str, wgrad_group: int | None = None, steps: int = 3, warmup: int = 1) -> dict:
    """A short measurement of another workload (or of this one in another mode) with the
    settings the bench would choose for it; the executor is freed afterwards."""
    import gc
    gc.collect()
    two = False
    group = wgrad_group if wgrad_group is not None else default_wgrad_group(wl, two)
    wb = Workbench(wl, fused=True, two_streams=two, wgrad_group=group)
    ms, _ = timed_steps(wb, steps, warmup, use_graph=wl.layer.hidden < 2048, cls=None)
    flops = wb.step_flops()
    out = {"ms_per_step": ms, "tokens_per_s": wl.tokens_per_step / (ms * 1e-3),
           "mfma_peak_frac": flops / (ms * 1e-3) / MFMA_BF16_PEAK, "steps": steps,
           "wgrad_group": group, "two_streams": two, "hip_graph": wl.layer.hidden < 2048,
           "device_bytes": wb.ex.nbytes}
    wb.close()
    del wb
    gc.collect()
    return out


def lds_read_rates() -> dict:
    """Cycles per wave-level LDS read for the address patterns of the kernels' fragment reads.
    The patterns restate the address arithmetic of csrc/common.h (slab_off, DmaTile::frag16,
    slab_frag, slab_frag_tr, mc_swz) for lane l of a wave; every pattern is measured at several
    fragment positions and the worst is reported."""
    def swz_tree(row):
        h = (row >> 1) & 7
        return h ^ ((h & 1) * 6)

    def swz_before(row):
        return (row ^ (row >> 3)) & 7

    def mc_swz(k):
        return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1)

    def worst(transposing, patterns):
        return max(rt.lds_read_rate([f(l) for l in range(64)], transposing) for f in patterns)

    out = {"unit": "shader clocks per wave-level read, 8 waves reading",
           "ds_read_b128, lane l at 16 l (no conflicts: 256 B per clock)":
               rt.lds_read_rate([16 * l for l in range(64)], False),
           "ds_read_b64_tr_b16, lane l at 8 l":
               rt.lds_read_rate([8 * l for l in range(64)], True)}
    for name, swz in (("swizzle of the tree", swz_tree), ("swizzle before", swz_before),
                      ("no swizzle", lambda row: 0)):
        def slab_off(row, chunk, swz=swz):
            return row * 128 + ((chunk ^ swz(row)) << 4)

        def frag16(row0, k32):
            return lambda l: slab_off(row0 + (l & 15), k32 * 4 + (l >> 4))

        def frag32(row0, ks):
            return lambda l: slab_off(row0 + (l & 31), ks * 2 + (l >> 5))

        def frag_tr(col0, st, hi):
            def f(l):
                g, s = l >> 4, l & 15
                n = col0 + ((g & 1) << 4) + ((s & 3) << 2)
                k = st * 16 + ((g >> 1) << 2) + (s >> 2) + 8 * hi
                return (n >> 6) * 8192 + ((n & 7) << 1) + slab_off(k, (n & 63) >> 3)
            return f

        out[name] = {
            "GEMM, K-contiguous operand, 16-row fragment (ds_read_b128)":
                worst(False, [frag16(r, k) for r in (0, 16, 48, 240) for k in (0, 1)]),
            "attention, 32-row fragment (ds_read_b128)":
                worst(False, [frag32(r, k) for r in (0, 32) for k in (0, 3)]),
            "attention, transposed fragment (ds_read_b64_tr_b16)":
                worst(True, [frag_tr(c, st, hi) for c in (0, 32, 96) for st in (0, 3)
                             for hi in (0, 1)]),
        }

    def mc_frag(rows, row0, k32, hi):
        def f(l):
            g, s = l >> 4, l & 15
            n = row0 + ((s & 3) << 2)
            k = k32 * 32 + (g << 3) + (s >> 2) + 4 * hi
            return k * (rows * 2) + (((n >> 3) ^ mc_swz(k)) << 4) + ((n & 7) << 1)
        return f

    out["GEMM, operand with the contraction index slow, 256 rows (ds_read_b64_tr_b16)"] = worst(
        True, [mc_frag(256, r, k, hi) for r in (0, 16, 112, 240) for k in (0, 1) for hi in (0, 1)])
    return out


def kernel_table(wb, wl, steps: int, warmup: int, two: bool, group: int) -> dict:
    for _ in range(warmup):
        wb.step()
    rt.sync()
    start, stop = rt.Event(), rt.Event()
    with rt.probe("*") as pr:
        start.record()
        for _ in range(steps):
            wb.step()
            rt.sync()                      # keeps the number of events in flight small
        stop.record()
        stop.sync()
    ms = start.elapsed_ms(stop) / steps
    total = sum(v[1] for v in pr.classes.values())
    rows = []
    for name, (n, t, fl, by) in sorted(pr.classes.items(), key=lambda kv: -kv[1][1]):
        hbm = fl == 0
        rate = (by if hbm else fl) / (t * 1e-3) if t else 0.0
        rows.append({"class": name, "launches_per_step": n / steps, "avg_us": t / n * 1e3,
                     "ms_per_step": t / steps, "share": t / total, "bound": "hbm" if hbm else "mfma",
                     "achieved": rate / (1e9 if hbm else 1e12), "unit": "GB/s" if hbm else "TFLOP/s",
                     "frac": rate / (HBM_PEAK if hbm else MFMA_BF16_PEAK)})
    return {"workload": wl.name, "two_streams": two, "wgrad_group": group, "steps": steps,
            "ms_per_step_probed": ms, "kernel_ms_per_step": total / steps, "classes": rows}


def after_loop(wb, wl, steps: int) -> dict:
    """Adam on the accumulators the timed steps left behind, `steps` times; HBM-bound: 34
    algorithmic bytes per parameter (reads gradient, m, v, f32 weight; writes m, v, weight,
    the bf16 parameter and the cleared gradient)."""
    wb.ex.optimizer_init()
    wb.ex.adam_step(1, grad_scale=1.0 / wl.n_mubatches)    # warm-up
    rt.sync()
    start, stop = rt.Event(), rt.Event()
    with rt.probe("adam") as pr:
        start.record()
        for i in range(steps):
            wb.ex.adam_step(2 + i, grad_scale=1.0 / wl.n_mubatches)
        stop.record()
        stop.sync()
    ms = start.elapsed_ms(stop) / steps
    ach = pr.bytes / (pr.total_ms * 1e-3)
    return {"kernel": "adam", "ms": ms, "bound": "hbm", "achieved": ach / 1e9,
            "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": ach / HBM_PEAK,
            "launches": pr.launches, "avg_launch_ms": pr.total_ms / pr.launches,
            "algorithmic_per_launch": pr.bytes / pr.launches}


def self_desc(wl, wb) -> str:
    s = wl.layer
    return (f"{wl.layers_per_stage} layers x {wb.plan.n_chunks} chunk(s), hidden {s.hidden}, "
            f"heads {s.n_heads}/{s.kvh}, ffn {s.ffn}, seq {s.seq}, microbatch {s.batch}, "
            f"{wl.n_mubatches} microbatches")


if __name__ == "__main__":
    main()
