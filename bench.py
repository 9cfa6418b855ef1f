#!/usr/bin/env python3
"""Headline benchmark: train samples/sec (forward + backward + SGD) of the binary
Tree-LSTM (hidden 512, embedding 300, batch 64, sentence-shaped random trees) through
the batched F-over-G path on one MI355X, with the roofline fraction of the dominant
kernel (the FP32-MFMA gate GEMM) and a CPU baseline (the CPU restatement of the
reference's semantics -- the reference ships no CPU kernels) timed on this host.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3|C2|C4|C5]

A step = host scheduling of a fresh batch structure (a pool of 16 pre-generated seeded
batches is cycled, so graph parsing is inside the timed region, as in the reference's
GraphStatement::Run) + forward rounds + loss head + backward rounds + deferred weight
gradients + SGD.  Vertex inputs and labels are resident in HBM before timing starts;
the graph placeholder is a host tensor by contract.
Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
FP32_MFMA_PEAK_TF = 157.3  # MI355X dense FP32 matrix
# (workload, kernel class) -> HBM bytes per dispatch, from profiles/bench_<workload>_hbm_traffic_pmc.txt
PMC_TRAFFIC_BYTES = {("C3", "gemm"): 82.05e6, ("C3", "round"): 98.59e6, ("C1", "gemm"): 3.35e6, ("C1", "round"): 0.96e6,
                     ("C2", "gemm"): 17.11e6, ("C2", "round"): 4.05e6, ("C4", "gemm"): 299.6e6, ("C4", "round"): 10.55e6,
                     ("C5", "gemm"): 918.6e6, ("C5", "round"): 125.4e6}
# a constant taken from the profile named, not a counter read during this run
PMC_TRAFFIC_SOURCE = {k: f"profiles/bench_{k[0]}_hbm_traffic_pmc.txt (two rocprofv3 --pmc runs of this command, FETCH_SIZE and "
                         "WRITE_SIZE per dispatch of the class; a constant copied from there, not read in this run)"
                      for k in PMC_TRAFFIC_BYTES}


def model_kwargs(w):
    if w["model"] == "treefc":
        return dict(loss="root_sq", act=1, use_bias=True, use_x=True)
    return dict(loss="softmax")


def make_pool(name, n_batches):
    from cavs_amd import synth

    base = synth.make_workload(name)
    pool = [base]
    for i in range(1, n_batches):
        w = synth.make_workload(name, seed=base["seed"] + 7919 * i)
        w["params"] = base["params"]
        pool.append(w)
    return pool


def cpu_baseline(w, budget_s=12.0):
    """Times the CPU checker on this host on a bounded sample of the same workload."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import pyoracle

    threads = min(16, len(os.sched_getaffinity(0)))
    kw = model_kwargs(w)
    args = dict(H=w["H"], E=w["E"], V=w["V"], Cc=w["C"], threads=threads, **kw)
    t0 = time.perf_counter()
    steps = 0
    while True:
        pyoracle.model_step(w["model"], w["graph"], w["x"], w["labels"], w["params"], **args)
        steps += 1
        el = time.perf_counter() - t0
        if el > budget_s or steps >= 400 or el + el / steps > 1.5 * budget_s:
            break
    # the same on one thread (a bounded sample: two steps)
    t1 = time.perf_counter()
    for _ in range(2):
        pyoracle.model_step(w["model"], w["graph"], w["x"], w["labels"], w["params"], **dict(args, threads=1))
    el1 = time.perf_counter() - t1
    # configuration C1, the reference's own CPU-runnable case: the chain LSTM (V=1000, E=H=128, T=20, B=16) on the
    # reference's CPU path -- its serial scheduler (cavs/midend/graph_scheduler.cc:83-167), one
    # forward+backward step, single thread
    from cavs_amd import synth

    c1 = synth.make_workload("C1")
    c1_args = dict(H=c1["H"], E=c1["E"], V=c1["V"], Cc=c1["C"], threads=1, batching=False)
    pyoracle.model_step(c1["model"], c1["graph"], c1["x"], c1["labels"], c1["params"], **c1_args)  # warm
    t2 = time.perf_counter()
    n1 = 0
    while n1 < 3 or (time.perf_counter() - t2 < 2.0 and n1 < 50):
        pyoracle.model_step(c1["model"], c1["graph"], c1["x"], c1["labels"], c1["params"], **c1_args)
        n1 += 1
    el2 = time.perf_counter() - t2
    c1_entry = dict(value=round(c1["B"] * n1 / el2, 3), unit="samples/s", cores=1, kind="port", ms_per_step=round(1e3 * el2 / n1, 3),
                    sample=f"{n1} forward+backward steps of the C1 batch (B={c1['B']}, N={c1['N']}) on the serial scheduler "
                           f"(one vertex per round, no batching) in {el2:.1f} s on one thread")
    return dict(value=round(w["B"] * steps / el, 3), unit="samples/s", cores=threads, kind="port", C1=c1_entry,
                host=dict(nproc=os.cpu_count(), affinity=len(os.sched_getaffinity(0)), omp_threads=threads),
                sample=f"{steps} full fwd+bwd step(s) of the {w['name']} batch (B={w['B']}, N={w['N']}) "
                       f"in {el:.1f} s with {threads} OpenMP threads; CPU restatement of the reference's "
                       "semantics (the reference has no CPU kernels)",
                single_thread=dict(value=round(w["B"] * 2 / el1, 3), unit="samples/s", cores=1,
                                   sample=f"2 steps of the same batch in {el1:.1f} s"))


def front_end_modes(pool, steps=60, warmup=30, only=None):
    """The same training step through the reference's own API (Sym / GraphSupport / Session::Run with
    host feeds, one device synchronisation per Run, loss head and optimizer as ordinary ops), in the
    ways the session can execute F: lowered onto the hand-written round kernels, lowered onto kernels
    generated for it (its shape recognised, not its identity), op by op with the fusion pass's
    generated kernels, and plain op by op -- the reference's execution model on this GPU.  For a
    Tree-LSTM workload also a vertex function no hand-written kernel covers (a forget-gate matrix per
    child, same sizes) and one whose products come in two stages (a child-sum tree GRU, which runs
    as a chain of two generated cells): lowered onto generated kernels against op by op with the
    fusion pass."""
    import torch

    from cavs_amd import apps, session, synth

    w = pool[0]
    B, maxlen = w["graph"].shape
    H = w["H"]
    out = {}
    cases = [("lowered", w["model"], session.OPT_BATCHING, 1), ("lowered_generated", w["model"], session.OPT_BATCHING, 2),
             ("op_by_op_fusion", w["model"], session.OPT_BATCHING | session.OPT_FUSION, 0), ("op_by_op", w["model"], session.OPT_BATCHING, 0)]
    if w["model"] == "treelstm":
        cases += [("fourth_function_lowered_generated", "treelstm2", session.OPT_BATCHING, 1),
                  ("fourth_function_op_by_op_fusion", "treelstm2", session.OPT_BATCHING | session.OPT_FUSION, 0),
                  ("two_stage_function_lowered_generated", "treegru", session.OPT_BATCHING, 1),
                  ("two_stage_function_op_by_op_fusion", "treegru", session.OPT_BATCHING | session.OPT_FUSION, 0)]
    for name, model, opt, lowered in cases:
        if only and name != only:
            continue
        app = apps.App(model, B=B, maxlen=maxlen, H=H, E=w["E"], V=w["V"], C_=w["C"], opt=opt, lr=1e-3, allow_fused=lowered)
        params = dict(w["params"])
        if model == "treefc":  # (the reference's Tree-FC app has the one weight matrix)
            params = {"W": params["W"]}
        if model == "treelstm2":  # [U_iou | U_fl | U_fr]
            params["U"] = np.concatenate([np.ravel(params["U"]), synth.SplitMix64(9).bulk_uniform(H * H, -0.1, 0.1)]).astype(np.float32)
        if model == "treegru":  # three gates instead of four, one state block
            rng = synth.SplitMix64(10)
            params.update({k: rng.bulk_uniform(app.var_size(k), -0.1, 0.1) for k in ("W", "U", "Bv")})
        app.set_params(params)
        # untimed: at least `warmup` steps and 150 ms of continuous work (steady clocks, as in measure())
        # the same pool of batch structures as the headline measurement, cycled the same way
        done, t0 = 0, time.perf_counter()
        while done < warmup or time.perf_counter() - t0 < 0.15:
            q = pool[done % len(pool)]
            app.step(q["graph"], q["x"], q["labels"], fetch=False)
            done += 1
        n = steps if not lowered else 5 * steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            q = pool[i % len(pool)]
            app.step(q["graph"], q["x"], q["labels"], fetch=False)
        torch.cuda.synchronize()
        ms = 1e3 * (time.perf_counter() - t0) / n
        out[name] = {"ms_per_step": round(ms, 4), "value": round(B / ms * 1e3, 1), "unit": "samples/s", "steps": n,
                     "generated_kernels": app.generated_kernels, "vertex_function": model,
                     "runs_on": ("operators", "hand-written round kernels", "generated round kernels")[app.fused_kind]}
        app.close()
    return out


class StepClock:
    """One event on the session's stream after every timed step: the intervals between
    consecutive events are the device's time per step in the steady state of the pipeline
    (the host runs ahead), whose median is reported next to the mean of the timed region."""

    def __init__(self, stream, n):
        import ctypes as C

        from cavs_amd import hip

        self.hip, self.stream, self.C = hip, stream, C
        self.events = []
        for _ in range(n + 1):
            e = C.c_void_p()
            hip.call("cavs_event_create", C.byref(e))
            self.events.append(e)
        self.k = 0

    def tick(self):
        self.hip.call("cavs_event_record", self.events[self.k], self.stream)
        self.k += 1

    def intervals_ms(self):
        out, ms = [], self.C.c_float()
        for a, b in zip(self.events[: self.k - 1], self.events[1: self.k]):
            self.hip.call("cavs_event_elapsed_ms", self.C.byref(ms), a, b)
            out.append(ms.value)
        return out

    def close(self):
        for e in self.events:
            self.hip.call("cavs_event_destroy", e)


def measure(a, workload, steps, warmup, n_pool, schedule="host", plan_cache=0, profile=True, graph_replay=False):
    """Times `steps` training steps of one workload and returns the fields of the JSON line.
    schedule / plan_cache / graph_replay: who builds the round schedule, whether plans are cached, and whether
    a cached plan's launches are replayed from a recorded graph
    (cavs_session_config); profile=False skips the per-kernel-class pass."""
    import torch

    from cavs_amd import session

    pool = make_pool(workload, n_pool)
    w0 = pool[0]
    kw = model_kwargs(w0)
    s = session.Session(w0["model"], H=w0["H"], E=w0["E"], V=w0["V"], C_=w0["C"], pairing=a.pairing,
                        opt=session.OPT_BATCHING, fused_round_rows=a.fused_round_rows, schedule=schedule,
                        plan_cache=plan_cache, tail_rows=a.tail_rows, graph_replay=graph_replay, head_chunks=a.head_chunks, **kw)
    s.set_params(w0["params"])
    feeds = []
    for w in pool:  # inputs resident in HBM before the timed region
        if a.host_feeds:
            feeds.append((w["graph"], np.ascontiguousarray(w["x"]), w["labels"]))
        else:
            feeds.append((w["graph"], torch.from_numpy(np.ascontiguousarray(w["x"])).cuda(),
                          torch.from_numpy(w["labels"]).cuda()))
    torch.cuda.synchronize()

    def run(k0, k):
        for i in range(k0, k0 + k):
            g, x, lab = feeds[i % len(feeds)]
            s.step(g, x, lab, backward=True, lr=a.lr)

    # untimed, before the W warm-up steps: the device takes ~60 ms of this kind of work to reach its
    # steady clocks, whatever W the caller picked
    # (continuous work: a synchronisation every few steps lets it idle and the ramp never happens)
    settle = 0
    if a.settle_ms > 0:
        t_probe = time.perf_counter()
        run(0, 10)
        s.sync()
        per_step = max((time.perf_counter() - t_probe) / 10, 1e-5)
        settle = 10 + min(5000, int(a.settle_ms * 1e-3 / per_step))
        run(10, settle - 10)
    run(0, warmup)
    clock = StepClock(s.stream, steps)
    parse_ms = []
    s.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    clock.tick()
    for i in range(warmup, warmup + steps):
        g, x, lab = feeds[i % len(feeds)]
        s.step(g, x, lab, backward=True, lr=a.lr)
        clock.tick()
        parse_ms.append(s.timing("GraphParsing"))
    s.sync()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / steps
    median_ms = float(np.median(clock.intervals_ms()))
    clock.close()
    # host side of the last timed step (the profiled pass below slows the host down)
    host_ms = {k: round(s.timing(k), 4) for k in ("GraphParsing", "HostSchedule", "HostWait", "HostStep")}
    host_ms["GraphParsing_median"] = round(float(np.median(parse_ms)), 4)
    value = w0["B"] * steps / elapsed
    if not profile:
        out = {"value": round(value, 2), "unit": "samples/s", "steps": steps, "ms_per_step": round(ms_per_step, 4),
               "median_ms_per_step": round(median_ms, 4), "GraphParsing_ms": host_ms["GraphParsing_median"],
               "HostSchedule_ms": host_ms["HostSchedule"], "plan_hits": s.counter("plan_hits"),
               "plan_misses": s.counter("plan_misses")}
        if graph_replay:
            out["graph_replays"] = s.counter("graph_replays")
        s.close()
        del feeds
        torch.cuda.empty_cache()
        return out, w0

    head_chunks = s.counter("head_chunks")  # (of the last timed step; the pass below runs the head in one piece)
    # Roofline of the dominant kernel: the same steps again with the kernels of every entry point
    # stamping a start and a stop event themselves (the interval a kernel trace reports) on the
    # session's own stream; kept out of the throughput figure above.
    s.profile(True)
    flops = hinted = rflops = gbytes = sbytes = 0.0
    for i in range(warmup, warmup + steps):
        g, x, lab = feeds[i % len(feeds)]
        s.step(g, x, lab, backward=True, lr=a.lr)
        flops += s.counter("gemm_flops")
        hinted += s.counter("gemm_flops_hinted")
        rflops += s.counter("round_flops")
        gbytes += s.counter("gather_bytes")
        sbytes += s.counter("scatter_bytes")
    gemm_ms, gemm_n = s.profile_read("gemm")
    gat_ms, gat_n = s.profile_read("gather")
    sca_ms, sca_n = s.profile_read("scatter")
    gates_ms, gates_n = s.profile_read("gates")
    round_ms, round_n = s.profile_read("round")
    other_ms, other_n = s.profile_read("other")
    s.profile(False)
    # the two MFMA-bound kernel classes; the roofline entry describes whichever takes more device time
    mfma = {
        "gemm": dict(ms=gemm_ms, n=gemm_n, flops=flops,
                     kernel="sgemm_mfma_kernel / sgemm_skinny_kernel (x*W, weight-gradient and head GEMMs of a step"
                            "; also the recurrent products of rounds too large for the fused kernels)"),
        "round": dict(ms=round_ms, n=round_n, flops=rflops,
                      kernel={"treelstm": "treelstm_round_fwd_kernel / treelstm_round_bwd_children_kernel / treelstm_tail_fwd_kernel / "
                                          "treelstm_tail_bwd_kernel (the rounds near the roots: one launch per direction)",
                              "lstm": "lstm_round_fwd_kernel / round_bwd_children_kernel",
                              "treefc": "treefc_round_fwd_kernel / round_bwd_children_kernel"}[w0["model"]] +
                             " (one launch per round: gather + recurrent products + gates + scatter)"),
    }
    for v in mfma.values():
        v["tf"] = v["flops"] / (v["ms"] * 1e-3) / 1e12 if v["ms"] else 0.0
    dom_name, dom = max(mfma.items(), key=lambda kv: kv[1]["ms"])
    # HBM bytes per dispatch of that class from the two rocprofv3 --pmc runs (FETCH_SIZE scaled by the
    # factor a plain copy of known size gives, plus WRITE_SIZE) summarised under profiles/; measured
    # for the default workload only
    traffic = PMC_TRAFFIC_BYTES.get((workload, dom_name)) if a.pairing == "reference" else None
    rounds = s.counter("rounds")
    launches = s.counter("launches")

    def hbm(nbytes, ms, n):
        return {"bound": "hbm", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 2) if ms else None, "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "avg_launch_us": round(1e3 * ms / max(n, 1), 3), "launches_per_step": round(n / steps, 1)}

    out = {
        "value": round(value, 2), "unit": "samples/s", "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "median_ms_per_step": round(median_ms, 4),
        "config": {"workload": f"{workload}: {w0['model']} V={w0['V']} E={w0['E']} H={w0['H']} B={w0['B']} "
                               f"N~{w0['N']} vertices/batch, {len(pool)} seeded batches cycled",
                   "step": "schedule+fwd+loss+bwd+sgd", "pairing": a.pairing,
                   "feeds": "pageable host memory, copied every step" if a.host_feeds else "resident in HBM",
                   "rounds_last_batch": rounds, "launches_last_batch": launches, "loss_head_chunks": head_chunks,
                   "untimed_settle_steps": settle},
        "roofline": {"bound": "mfma", "achieved": round(dom["tf"], 3), "peak": FP32_MFMA_PEAK_TF,
                     "unit": "TFLOP/s", "frac": round(dom["tf"] / FP32_MFMA_PEAK_TF, 5), "traffic": traffic,
                     "traffic_source": PMC_TRAFFIC_SOURCE.get((workload, dom_name)) if traffic else None,
                     "kernel": dom["kernel"],
                     "avg_launch_us": round(1e3 * dom["ms"] / dom["n"], 3) if dom["n"] else None,
                     "flops_per_launch": round(dom["flops"] / dom["n"], 1) if dom["n"] else None},
        "kernels": {
            **{k: {"bound": "mfma", "achieved": round(v["tf"], 3), "peak": FP32_MFMA_PEAK_TF, "unit": "TFLOP/s",
                   "frac": round(v["tf"] / FP32_MFMA_PEAK_TF, 4),
                   "avg_launch_us": round(1e3 * v["ms"] / max(v["n"], 1), 3), "launches_per_step": round(v["n"] / steps, 1)}
               for k, v in mfma.items()},
            # of the GEMM class's flops (2*M*N*K of the reference's products): the share that multiplies blocks
            # known to be zero or unused (forget-gate columns of the leaves) and is skipped tile by tile
            "gemm_flops_hinted_frac": round(hinted / flops, 4) if flops else 0.0,
            # separate gather / scatter launches only (rounds that run fused move their rows inside the round kernel)
            "gather": hbm(gbytes, gat_ms, gat_n), "scatter": hbm(sbytes, sca_ms, sca_n),
            "gates": {"avg_launch_us": round(1e3 * gates_ms / max(gates_n, 1), 3)},
            "device_ms_per_step": {"gemm": round(gemm_ms / steps, 4), "round": round(round_ms / steps, 4),
                                   "gather": round(gat_ms / steps, 4), "scatter": round(sca_ms / steps, 4),
                                   "gates": round(gates_ms / steps, 4), "other": round(other_ms / steps, 4)},
        },
        "timers_ms": {**host_ms, "RNNForward": round(s.timing("RNNForward"), 4),
                      "RNNBackward": round(s.timing("RNNBackward"), 4)},
    }
    s.close()
    del feeds
    torch.cuda.empty_cache()
    return out, w0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the device needs about a hundred steps (60 ms) of this workload to reach its steady clocks:
    # 20 warm-up steps read 0.62 ms per step, 100 and more 0.575
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=150)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed steps run for this long before the warm-up steps (clock ramp); 0 to skip")
    ap.add_argument("--workload", default="C3")
    ap.add_argument("--pool", type=int, default=16)
    ap.add_argument("--lr", type=float, default=1e-3)
    ap.add_argument("--pairing", default="reference", choices=["reference", "rowid"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-front-end", action="store_true",
                    help="skip the 'front_end' field (the step through Session::Run in its three execution modes)")
    ap.add_argument("--front-end-case", default="",
                    help="run only this entry of 'front_end' (e.g. fourth_function_lowered_generated) and print it: the command "
                         "behind the kernel statistics of the generated round kernels")
    ap.add_argument("--front-end-steps", type=int, default=60, help="timed steps of an op-by-op front-end case (a lowered one runs five times as many)")
    ap.add_argument("--no-schedule-modes", action="store_true",
                    help="skip 'schedule_modes' (the step with the schedule built on the host / on the GPU / from the plan cache)")
    ap.add_argument("--host-feeds", action="store_true",
                    help="feed x and labels from pageable host memory every step (PCIe-inclusive rate; not the headline value)")
    ap.add_argument("--fused-round-rows", type=int, default=0,
                    help="rounds of at most this many vertices run as fused launches (0: default limit, -1: never)")
    ap.add_argument("--tail-rows", type=int, default=0,
                    help="Tree-LSTM, H = 512: rounds whose rows can be dealt to eight groups with at most this many rows each run "
                         "inside one launch per direction (0: default limit, -1: one launch per round)")
    ap.add_argument("--head-chunks", type=int, default=0,
                    help="the loss head of a wide classifier (C4): 0 = in two chunks beside the backward rounds, 2..4 = in that many, negative = in one piece between the two passes")
    ap.add_argument("--also", default="C1,C2,C4,C5",
                    help="further workloads measured with few steps and reported under 'also' (C5 is the large "
                         "Tree-LSTM configuration, where rounds are GEMM-sized); 'none' to skip")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs the F-over-G path on one GPU; instance graphs shard by sample "
                 "across GPUs, one all-reduce of the weight gradients per step, but no multi-GPU path is built -- run with --gpus 1")

    import torch

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    if a.front_end_case:
        print(json.dumps({"front_end": front_end_modes(make_pool(a.workload, a.pool), steps=a.front_end_steps, warmup=min(30, a.front_end_steps), only=a.front_end_case)}))
        return
    res, w0 = measure(a, a.workload, a.steps, a.warmup, a.pool)
    out = {
        "metric": "train samples/sec (fwd+bwd) Tree-LSTM h=512 bs=64; % HBM/MFMA peak",
        "value": res["value"], "unit": res["unit"], "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": res["ms_per_step"], "median_ms_per_step": res["median_ms_per_step"],
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": res["config"], "roofline": res["roofline"], "kernels": res["kernels"], "timers_ms": res["timers_ms"],
    }
    # (before the other configurations: for a while after C5's 30 ms steps the device runs this small
    # workload about 15 % slower)
    if not a.no_front_end and w0["model"] in ("treelstm", "lstm"):
        out["front_end"] = front_end_modes(make_pool(a.workload, a.pool))
        # the same step as a user of the reference's API gets it: Session::Run with host feeds
        out["session_run"] = dict(out["front_end"]["lowered"], path="Sym / GraphSupport / Session::Run, vertex function "
                                  "lowered onto the fused round kernels, host feeds, optimizer as an op of the main scope")
    if not a.no_schedule_modes:
        # who builds the round schedule and the index lists: the host scheduler (the headline above),
        # the GPU (cavs_schedule_arena), or the plan cache replaying a structure seen before
        modes = {}
        for name, sched, cache, replay in (("host", "host", 0, False), ("device", "device", 0, False), ("cached", "host", a.pool, False),
                                           ("cached_replay", "host", a.pool, True)):
            modes[name], _ = measure(a, a.workload, a.steps, a.warmup, a.pool, schedule=sched, plan_cache=cache, profile=False,
                                     graph_replay=replay)
        out["schedule_modes"] = modes
        out["timers_ms"]["GraphParsing_by_mode"] = {k: v["GraphParsing_ms"] for k, v in modes.items()}
    if a.also.lower() != "none":
        out["also"] = {}
        for name in a.also.split(","):
            if name == a.workload:
                continue
            big = name == "C5"
            steps, warm, npool = (20, 5, 2) if big else (100, 50, 4)
            also, _ = measure(a, name, steps, warm, npool)
            out["also"][name] = {k: also[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step", "median_ms_per_step",
                                                      "config", "roofline", "kernels")}
            if not a.no_schedule_modes:  # the same steps with the lists built on the GPU
                dev, _ = measure(a, name, steps, warm, npool, schedule="device", profile=False)
                hit, _ = measure(a, name, steps, warm, npool, plan_cache=npool, profile=False)
                rep, _ = measure(a, name, steps, warm, npool, plan_cache=npool, profile=False, graph_replay=True)
                keys = ("value", "ms_per_step", "median_ms_per_step", "GraphParsing_ms")
                out["also"][name]["schedule_modes"] = {
                    "host": {k: also[k] for k in ("value", "ms_per_step", "median_ms_per_step")},
                    "device": {k: dev[k] for k in keys}, "cached": {k: hit[k] for k in keys},
                    "cached_replay": {k: rep[k] for k in keys}}
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w0)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
