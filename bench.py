#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.  Prints ONE JSON line.

Headline (BASELINE config 2): row-wise fp16 ops on X[16384,4096] ~ N(0,1) — reduce-sum over
the last axis, softmax, RMSNorm (weight ~ U(0.5,1.5), eps 1e-6), fp32 accumulation — planned
by the Planner and executed inside ONE persistent loop kernel (Model -> plan JSON ->
Executor).  The plan holds four X tensors (4 x 128 MiB, with outputs of their own) and walks
them in turn, so nothing of an X is left in the 256 MB Infinity Cache when its turn comes
again.  Within a turn the three ops read the same X one after the other, and the second and
third read may be served by that cache (the plan keeps X cacheable for them on purpose).  A
"step" is one plan iteration: the three ops over each of the four X tensors (12 ops, 2.68 GB
of algorithmic bytes).

`value` is the whole-job throughput of the timed run of the resident loop kernel (host clock
around run() + wait(), inputs already in HBM) in algorithmic GB/s: the kernel is loaded for 30 ms
untimed first (the chip leaves its idle clocks over tens of milliseconds), then come the W
warm-up steps and exactly K timed ones.  `roofline` prices the
loop kernel itself against 8 TB/s: the same plan launched in one-shot mode (the kernel runs
its iterations and returns) under HIP events on the stream it is launched on, which is the
dispatch `rocprofv3 --kernel-trace` reports.  `roofline.frac` counts algorithmic bytes and so
includes the cache-served re-reads; `roofline.frac_hbm_only` is the same plan with every op
streaming its input from HBM (ARKMI_ROW_CACHED_INPUT=0), and `roofline.per_op` times each of
the three ops alone over the four rotating X tensors, where no byte is read twice.

`configs` holds the other BASELINE configurations (C1 GEMM, C3 SwiGLU FFN, C4 decode GEMV at
batch 1 and 8, C5 decoder layer), each with the same kind of block: a HIP-event-timed one-shot
launch of its loop kernel priced against its roofline, the resident loop kernel and the same
ops as separate kernels beside it, and the CPU oracle timed on a bounded sample.  `machine`
holds what this GPU sustains on an MFMA-only loop and on plain streams, beside the datasheet
peaks used as denominators.

Inputs come from the counter-based generator in ark_amd/prng.py (seed = hash of configuration
and tensor name), drawn on the GPU; the CPU baseline reads the same rounded bits back.
"""
import argparse
import json
import os
import re
import sys
import time

ROWS, COLS = 16384, 4096
ALGO_BYTES = {
    # bytes one launch cannot avoid: reads + writes
    "reduce_sum": ROWS * COLS * 2 + ROWS * 2,
    "softmax": 2 * ROWS * COLS * 2,
    "rmsnorm": 2 * ROWS * COLS * 2 + COLS * 4,
}
HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0
NBUF = 4
ROOT = os.path.dirname(os.path.abspath(__file__))


def profiled_traffic_bytes_per_step():
    """Bytes one step moves between the L2s and the fabric (Infinity Cache hits included; HBM
    sees less), as measured by rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on the one-shot
    loop-kernel dispatch: read from the committed profile summary (not measured in this run).
    None when the summary is missing."""
    path = os.path.join(ROOT, "profiles", "loop_kernel_rows_c2_pmc.txt")
    try:
        with open(path) as f:
            m = re.search(r"^(?:fabric|hbm)_bytes_per_step:\s*(\d+)", f.read(), re.M)
        return (int(m.group(1)), "profiles/loop_kernel_rows_c2_pmc.txt") if m else (None, None)
    except OSError:
        return None, None


class Inputs:
    """Seeded inputs drawn on the GPU, rounded once to the storage type."""

    def __init__(self, torch, prng, config):
        self.torch, self.prng, self.config = torch, prng, config

    def normal(self, name, shape, dtype, std=1.0):
        return self.prng.normal(self.prng.seed_of(self.config, name), tuple(shape), 0.0, std, device="cuda").to(dtype)

    def uniform(self, name, shape, dtype, lo, hi):
        return self.prng.uniform(self.prng.seed_of(self.config, name), tuple(shape), lo, hi, device="cuda").to(dtype)


def _resident_us(torch, Executor, plan, iters, feeds):
    """us per iteration in the resident loop kernel (host clock around run() + wait()): untimed
    batches of `iters` iterations for 30 ms, then the median of five timed batches."""
    ex = Executor(plan, device_id=0).compile()
    for t, v in feeds:
        ex.tensor_write_device(t, v)
    torch.cuda.synchronize()
    ex.launch()
    # untimed load first: the chip leaves its idle clocks over tens of milliseconds, and a batch
    # timed while they still rise reads up to 10 % slow (one batch here, then as many as 30 ms take)
    t0 = time.perf_counter()
    ex.run(iters)
    ex.wait()
    first = time.perf_counter() - t0
    for _ in range(min(50, int(0.03 / max(first, 1e-6)))):
        ex.run(iters)
        ex.wait()
    batches = []
    for _ in range(5):
        t0 = time.perf_counter()
        ex.run(iters)
        ex.wait()
        batches.append((time.perf_counter() - t0) / iters * 1e6)
    info = ex.info()
    ex.stop()
    del ex
    return sorted(batches)[2], info


def _oneshot_and_separate_us(torch, Executor, plan, iters, feeds):
    """(us per iteration of a one-shot launch of the loop kernel, us per iteration with every op
    launched as a kernel of its own), both under HIP events on the executor's stream."""
    side = torch.cuda.Stream()
    ex = Executor(plan, device_id=0, stream=side.cuda_stream, loop_mode=False).compile()
    for t, v in feeds:
        ex.tensor_write_device(t, v)
    torch.cuda.synchronize()
    one, sep = [], []
    with torch.cuda.stream(side):
        ex.launch()
        ex.run(iters)
        ex.wait()
        for _ in range(3):
            s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s_.record()
            ex.run(iters)
            e_.record()
            ex.wait()
            torch.cuda.synchronize()
            one.append(s_.elapsed_time(e_) / iters * 1e3)
        ex.stop()
        ex.run_separate(iters)
        torch.cuda.synchronize()
        for _ in range(3):
            s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s_.record()
            ex.run_separate(iters)
            e_.record()
            torch.cuda.synchronize()
            sep.append(s_.elapsed_time(e_) / iters * 1e3)
    del ex
    return sorted(one)[1], sorted(sep)[1]


def _block(workload, bound, work, one_us, loop_us, sep_us, info, cpu):
    """One configuration's result: `work` is flop (bound mfma) or bytes (bound hbm) per iteration."""
    if bound == "mfma":
        achieved, peak, unit = work / one_us / 1e6, MFMA_PEAK_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, unit = work / one_us / 1e3, HBM_PEAK_GBPS, "GB/s"
    out = {"workload": workload,
           "roofline": {"bound": bound, "kernel": f"arkmi_loop_kernel<{info['kernel_families']}> (one-shot launch)",
                        "achieved": round(achieved, 1), "peak": peak, "unit": unit,
                        "frac": round(achieved / peak, 4), "traffic": None,
                        "us_per_iteration": round(one_us, 1)},
           "resident_loop_kernel_us": round(loop_us, 1), "separate_kernels_us": round(sep_us, 1),
           "loop_faster_than_separate": bool(loop_us < sep_us)}
    if cpu is not None:
        out["cpu_baseline"] = cpu
    return out


def _timed_cpu(fn, unit_work, unit, sample, min_seconds=2.0):
    """Runs fn() until min_seconds have passed; work per call in `unit`-compatible quantity."""
    from oracle import ark_oracle as O
    fn()  # thread pool start-up outside the clock
    n, t0 = 0, time.perf_counter()
    while True:
        fn()
        n += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds:
            break
    return {"value": round(unit_work * n / dt / 1e9, 3), "unit": unit, "cores": O.num_threads(), "kind": "port",
            "sample": f"{sample}; {n} passes in {dt:.1f} s"}


def config_c1(torch, Model, Executor, inp, cpu):
    a = inp.uniform("A", (4096, 4096), torch.float16, -1.0, 1.0)
    b = inp.uniform("B", (4096, 4096), torch.float16, -1.0, 1.0)
    m = Model()
    ta, tb = m.tensor([4096, 4096], "fp16"), m.tensor([4096, 4096], "fp16")
    m.matmul(ta, tb)
    plan, feeds = m.plan(device_id=0), [(ta, a), (tb, b)]
    loop_us, info = _resident_us(torch, Executor, plan, 20, feeds)
    one_us, sep_us = _oneshot_and_separate_us(torch, Executor, plan, 20, feeds)
    base = None
    if cpu:
        from oracle import ark_oracle as O
        an, bn = a[:48].cpu().numpy(), b.cpu().numpy()
        base = _timed_cpu(lambda: O.matmul(an, bn, "fp16"), 2.0 * 48 * 4096 * 4096, "GFLOP/s",
                          "oracle matmul on 48 of the 4096 rows of A against all of B")
    return _block("C1 fp16 GEMM C[4096,4096] = A . B, A, B ~ U[-1,1), fp32 accumulate", "mfma", 2.0 * 4096 ** 3,
                  one_us, loop_us, sep_us, info, base)


def config_c3(torch, Model, Executor, llama, inp, cpu):
    fl = 3 * 2.0 * 8192 * 4096 * 11008
    out = {}
    for fused in (False, True):
        m = Model()
        tx = m.tensor([8192, 4096], "bf16")
        ff = llama.FeedForward(m, 4096, 11008, "bf16")
        ff.forward(tx, fused=fused)
        vals = {"x": inp.normal("x", tx.shape, torch.bfloat16)}
        feeds = [(tx, vals["x"])]
        for name, t in ff.params().items():
            vals[name] = inp.normal(name, t.shape, torch.bfloat16, 0.02)
            feeds.append((t, vals[name]))
        plan = m.plan(device_id=0)
        loop_us, info = _resident_us(torch, Executor, plan, 10, feeds)
        one_us, sep_us = _oneshot_and_separate_us(torch, Executor, plan, 10, feeds)
        base = None
        if cpu and fused:
            from oracle import ark_oracle as O
            xn = vals["x"][:16].view(torch.int16).cpu().numpy().view("uint16")
            w1, w2, w3 = (vals[k].view(torch.int16).cpu().numpy().view("uint16") for k in ("w1", "w2", "w3"))

            def ffn():
                g = O.matmul(xn, w1, "bf16", trans_b=True)
                u = O.matmul(xn, w3, "bf16", trans_b=True)
                h = O.binary(O.binary(g, O.unary(g, "sigmoid", "bf16"), "mul", "bf16"), u, "mul", "bf16")
                return O.matmul(h, w2, "bf16", trans_b=True)
            base = _timed_cpu(ffn, 3 * 2.0 * 16 * 4096 * 11008, "GFLOP/s",
                              "oracle FFN (reference composition) on 16 of the 8192 rows of x")
        del feeds, vals
        key = "fused_ops" if fused else "reference_composition"
        out[key] = _block("C3 SwiGLU FFN x[8192,4096] bf16 -> 11008 -> 4096, one loop kernel ("
                          + ("SwiGLU as one GEMM pass" if fused else "the reference's op-by-op composition") + ")",
                          "mfma", fl, one_us, loop_us, sep_us, info, base)
    return out


def config_c4(torch, Model, Executor, inp, cpu):
    """Decode GEMV.  The headline block of a batch size walks TWO sets of the four matrices in turn
    (810 MB, more than L2 and Infinity Cache hold), so every token step streams its 404.75 MB from
    HBM; `one_weight_set` is the same token step over a single set, of which the 256 MB cache can
    keep a part from one iteration to the next."""
    shapes = [("W_qkv", 4096, 12288), ("W_o", 4096, 4096), ("W_gate_up", 4096, 22016), ("W_down", 11008, 4096)]
    wbytes = float(sum(k * n * 2 for _, k, n in shapes))
    out = {}
    for bsz in (1, 8):
        blocks = {}
        for sets in (2, 1):
            m = Model()
            feeds, vals = [], []
            for rep in range(sets):
                for name, k, n in shapes:
                    tx, tw = m.tensor([bsz, k], "bf16"), m.tensor([k, n], "bf16")
                    m.matmul(tx, tw)
                    x = inp.normal(f"x_{name}_b{bsz}", tx.shape, torch.bfloat16)
                    w = inp.normal(name if rep == 0 else f"{name}_set{rep}", tw.shape, torch.bfloat16, 0.02)
                    feeds += [(tx, x), (tw, w)]
                    if rep == 0:
                        vals.append((x, w))
            plan = m.plan(device_id=0)
            loop_us, info = _resident_us(torch, Executor, plan, 50, feeds)
            one_us, sep_us = _oneshot_and_separate_us(torch, Executor, plan, 50, feeds)
            base = None
            if cpu and sets == 2:
                from oracle import ark_oracle as O
                host = [(x.view(torch.int16).cpu().numpy().view("uint16"), w.view(torch.int16).cpu().numpy().view("uint16"))
                        for x, w in vals]
                base = _timed_cpu(lambda: [O.matmul(x, w, "bf16") for x, w in host], wbytes, "GB/s",
                                  f"oracle matmul of one token step (four matrices, batch {bsz})")
            del feeds, vals
            # per token step: a plan iteration is `sets` token steps
            blocks[sets] = _block(f"C4 decode GEMV, batch {bsz}: x[B,4096] . W_qkv[4096,12288], W_o[4096,4096], "
                                  "W_gate/up[4096,22016], x[B,11008] . W_down[11008,4096], bf16, one plan; "
                                  + ("two weight sets in turn (every token step streams from HBM); per token step"
                                     if sets == 2 else "one weight set, reused every iteration"),
                                  "hbm", wbytes, one_us / sets, loop_us / sets, sep_us / sets, info, base)
        blocks[2]["one_weight_set"] = {k: blocks[1][k] for k in ("roofline", "resident_loop_kernel_us", "separate_kernels_us")}
        out[f"batch{bsz}"] = blocks[2]
    return out


def config_c5(torch, np, Model, Executor, llama, inp, cpu):
    names = {False: "reference_composition", True: "fused_ops", "attention": "fused_ops_attention_op",
             "side_by_side": "fused_ops_attention_op_qk_side_by_side"}
    out = {}
    num_cu = torch.cuda.get_device_properties(0).multi_processor_count
    for fused in (False, True, "attention", "side_by_side"):
        # "side_by_side": the attention-op plan with the query and key projections on full-size tiles
        # on the two halves of the processors at the same time (one kernel per op cannot do that)
        key, pair_on = fused, None
        if fused == "side_by_side":
            fused, pair_on = "attention", num_cu
        m = Model()
        blk = llama.TransformerBlock(m, 4096, 32, 11008, "bf16")
        tx = m.tensor([1, 2048, 4096], "bf16")
        tf = m.tensor([1, 2048, 1, 128], "bf16")
        tm = m.tensor([1, 1, 2048, 2048], "bf16")
        blk.forward(tx, tf, tm, fused=bool(fused), causal=(fused == "attention"), pair_on=pair_on)
        vals = {"x": inp.normal("hidden", tx.shape, torch.bfloat16)}
        feeds = [(tx, vals["x"]),
                 (tf, torch.from_numpy(llama.precompute_freqs_cis(128, 2048)).cuda().bfloat16()),
                 (tm, torch.from_numpy(llama.causal_mask(2048, -np.inf)).cuda().bfloat16())]
        if fused == "attention":
            feeds.pop()  # the attention op applies the causal mask itself: no mask tensor in the plan
        for name, t in blk.params().items():
            vals[name] = (torch.ones(*t.shape, device="cuda") if name.endswith("_norm")
                          else inp.normal(name, t.shape, torch.bfloat16, 0.02))
            feeds.append((t, vals[name]))
        plan = m.plan(device_id=0)
        loop_us, info = _resident_us(torch, Executor, plan, 10, feeds)
        one_us, sep_us = _oneshot_and_separate_us(torch, Executor, plan, 10, feeds)
        counters = None
        if fused == "attention" and pair_on is None:
            # the same plan with its grid barriers replaced by dependency counters (off by default)
            os.environ["ARKMI_DEP_COUNTERS"] = "1"
            try:
                dep_us, dep_info = _resident_us(torch, Executor, plan, 10, feeds)
            finally:
                del os.environ["ARKMI_DEP_COUNTERS"]
            counters = {"resident_loop_kernel_us": round(dep_us, 1), "barriers_counted": dep_info["barriers_counted"]}
        # full (unskipped) attention counts 897.7 GFLOP; the attention op skips the masked key blocks
        fl = 863.3e9 if fused == "attention" else 897.7e9
        base = None
        if cpu and fused == "attention" and pair_on is None:
            from oracle import ark_oracle as O
            host = {k: v.view(torch.int16).cpu().numpy().view("uint16") for k, v in vals.items() if v.dtype == torch.bfloat16}
            xs = host["x"][0, :16]

            def projections():
                q = O.matmul(xs, host["attention.wq"], "bf16", trans_b=True)
                o = O.matmul(q, host["attention.wo"], "bf16", trans_b=True)
                g = O.matmul(o, host["feed_forward.w1"], "bf16", trans_b=True)
                u = O.matmul(o, host["feed_forward.w3"], "bf16", trans_b=True)
                h = O.binary(O.binary(g, O.unary(g, "sigmoid", "bf16"), "mul", "bf16"), u, "mul", "bf16")
                return O.matmul(h, host["feed_forward.w2"], "bf16", trans_b=True)
            base = _timed_cpu(projections, 2.0 * 16 * (2 * 4096 * 4096 + 3 * 4096 * 11008), "GFLOP/s",
                              "oracle Q and output projections and the SwiGLU FFN on 16 of the 2048 positions "
                              "(the K/V projections and the attention itself are left out of the CPU sample)")
        del feeds, vals
        out[names[key]] = _block(
            "C5 Llama-2-7B decoder layer, seq 2048, d 4096, 32 heads x 128, SwiGLU 11008, bf16, RoPE 10000, causal ("
            + {False: "the reference's op-by-op composition", True: "fused ops, matmul/softmax attention",
               "attention": "fused ops, attention as one op; flop count with masked key blocks skipped",
               "side_by_side": "fused ops, attention as one op, query and key projections side by side on "
                               "256x256 tiles; flop count with masked key blocks skipped"}[key] + ")",
            "mfma", fl, one_us, loop_us, sep_us, info, base)
        if counters:
            out[names[key]]["with_dependency_counters"] = counters
    return out


def timeline(torch, np, Model, Executor, llama, prng, which):
    """Per-step workgroup clocks of one configuration's plan in the loop kernel (text, for the
    profile summaries): every workgroup reads the clock when it enters a step, so a step's
    duration per workgroup and the spread of the entry times show where workgroups wait."""
    import json as _json
    import os as _os
    from ark_amd import plan_schedule
    inp = Inputs(torch, prng, which.upper())
    cases = []
    if which == "c4":
        for bsz in (1, 8):
            m = Model()
            feeds = []
            for name, k, n in [("W_qkv", 4096, 12288), ("W_o", 4096, 4096), ("W_gate_up", 4096, 22016), ("W_down", 11008, 4096)]:
                tx, tw = m.tensor([bsz, k], "bf16"), m.tensor([k, n], "bf16")
                m.matmul(tx, tw)
                feeds += [(tx, inp.normal(f"x_{name}_b{bsz}", tx.shape, torch.bfloat16)),
                          (tw, inp.normal(name, tw.shape, torch.bfloat16, 0.02))]
            cases.append((f"C4 batch {bsz}", m.plan(device_id=0), feeds, {}))
    else:
        m = Model()
        blk = llama.TransformerBlock(m, 4096, 32, 11008, "bf16")
        tx, tf, tm = m.tensor([1, 2048, 4096], "bf16"), m.tensor([1, 2048, 1, 128], "bf16"), m.tensor([1, 1, 2048, 2048], "bf16")
        blk.forward(tx, tf, tm, fused=True, causal=True)
        feeds = [(tx, inp.normal("hidden", tx.shape, torch.bfloat16)),
                 (tf, torch.from_numpy(llama.precompute_freqs_cis(128, 2048)).cuda().bfloat16())]
        for name, t in blk.params().items():
            feeds.append((t, torch.ones(*t.shape, device="cuda") if name.endswith("_norm")
                          else inp.normal(name, t.shape, torch.bfloat16, 0.02)))
        plan = m.plan(device_id=0)
        cases.append(("C5 fused ops with the attention op, grid barriers", plan, feeds, {}))
        cases.append(("C5 fused ops with the attention op, dependency counters", plan, feeds, {"ARKMI_DEP_COUNTERS": "1"}))
        # the same layer with the query and key projections side by side (same parameter tensors
        # by name, so the same seeded values)
        m2 = Model()
        blk2 = llama.TransformerBlock(m2, 4096, 32, 11008, "bf16")
        tx2, tf2, tm2 = m2.tensor([1, 2048, 4096], "bf16"), m2.tensor([1, 2048, 1, 128], "bf16"), m2.tensor([1, 1, 2048, 2048], "bf16")
        blk2.forward(tx2, tf2, tm2, fused=True, causal=True, pair_on=torch.cuda.get_device_properties(0).multi_processor_count)
        by_name = {name: v for (name, _), (_, v) in zip(blk.params().items(), feeds[2:])}
        feeds2 = [(tx2, feeds[0][1]), (tf2, feeds[1][1])] + [(t, by_name[name]) for name, t in blk2.params().items()]
        cases.append(("C5 fused ops with the attention op, query and key projections side by side", m2.plan(device_id=0), feeds2, {}))
    for title, plan, feeds, env in cases:
        names = {ti["Id"]: "+".join(o["Type"] for o in ti["Ops"]) for ti in _json.loads(plan)["TaskInfos"]}
        sched = [(names[st["Args"][-1]] if st["Kind"] == "TaskSeq" else "B") for st in plan_schedule(plan)["Steps"]]
        _os.environ.update(env)
        try:
            ex = Executor(plan, device_id=0, trace=True).compile()
        finally:
            for k in env:
                del _os.environ[k]
        for t, x in feeds:
            ex.tensor_write_device(t, x)
        torch.cuda.synchronize()
        ex.launch()
        ex.run(10)
        ex.wait()
        t0 = time.perf_counter()
        ex.run(20)
        ex.wait()
        us = (time.perf_counter() - t0) / 20 * 1e6
        info = ex.info()
        clk, _ = ex.read_step_clocks()
        ex.stop()
        clk = np.array(clk)
        base, d = clk[:, 0].min(), np.diff(clk, axis=1)
        print(f"{title}: {us:.1f} us per iteration with the clocks on; "
              + ", ".join(f"{k} {info[k]}" for k in ("barriers_elided", "barriers_local", "barriers_counted",
                                                      "iteration_sync", "gemv_chains", "kernel_families")))
        print("  schedule: " + " | ".join(sched))
        print("  us, over the workgroups:   time in the step min / median / max      step entered first / last")
        for i in range(d.shape[1]):
            print(f"  step {i:2d} {sched[i][:22]:22s} {d[:, i].min():8.2f} {np.median(d[:, i]):8.2f} {d[:, i].max():8.2f}"
                  f"      {clk[:, i].min() - base:9.2f} {clk[:, i].max() - base:9.2f}")
        print(f"  end of the body reached first / last {clk[:, -1].min() - base:9.2f} {clk[:, -1].max() - base:9.2f}")
        if which == "c4":
            # by XCD (workgroups go to the XCDs round robin): does one of them stream more slowly?
            tot = clk[:, -1] - clk[:, 0]
            print("  time in the body by XCD (workgroup index mod 8), median: "
                  + "  ".join(f"{np.median(tot[x::8]):.1f}" for x in range(8)))
        del ex


def machine_probes(torch, prng):
    """What this GPU sustains: an MFMA-only loop (random and zero operands) and plain streams."""
    import ctypes
    from ark_amd._lib import lib, check
    L = lib()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.zeros(16, device="cuda", dtype=torch.float32)
    out = {"datasheet": {"mfma_dense_fp16_bf16_TFLOPs": MFMA_PEAK_TFLOPS, "hbm_GBps": HBM_PEAK_GBPS}}

    def timed(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s_.record()
        for _ in range(reps):
            fn()
        e_.record()
        torch.cuda.synchronize()
        return s_.elapsed_time(e_) / reps * 1e-3

    for label, data in (("random_U(-1,1)", prng.uniform(11, (1 << 20,), -1.0, 1.0, device="cuda").half()),
                        ("zeros", torch.zeros(1 << 20, device="cuda", dtype=torch.float16))):
        flops = ctypes.c_double()

        def run():
            check(L.arkmi_probe_mfma(ctypes.c_void_p(data.data_ptr()), ctypes.c_size_t(data.numel() * 2), ctypes.c_int(4000),
                                     ctypes.c_void_p(sink.data_ptr()), ctypes.byref(flops), st))
        sec = timed(run)
        out[f"mfma_only_loop_TFLOPs_{label}"] = round(flops.value / sec / 1e12, 1)
    nbytes = 1 << 28
    src = torch.empty(nbytes, device="cuda", dtype=torch.uint8).random_()
    dst = torch.empty_like(src)

    def copy():
        check(L.arkmi_probe_stream(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), ctypes.c_size_t(nbytes),
                                   ctypes.c_void_p(sink.data_ptr()), st))

    def read():
        check(L.arkmi_probe_stream(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(0), ctypes.c_size_t(nbytes),
                                   ctypes.c_void_p(sink.data_ptr()), st))
    out["stream_copy_GBps_read_plus_write"] = round(2 * nbytes / timed(copy, 10) / 1e9, 1)
    out["stream_read_GBps"] = round(nbytes / timed(read, 10) / 1e9, 1)
    return out


def other_configs(torch, np, Model, Executor, llama, prng, cpu, only=None):
    want = lambda c: only is None or only == c
    out = {}
    if want("c1"):
        out["C1_gemm_fp16_4096"] = config_c1(torch, Model, Executor, Inputs(torch, prng, "C1"), cpu)
    if want("c3"):
        out["C3_ffn_bf16"] = config_c3(torch, Model, Executor, llama, Inputs(torch, prng, "C3"), cpu)
    if want("c4"):
        out["C4_decode_gemv_bf16"] = config_c4(torch, Model, Executor, Inputs(torch, prng, "C4"), cpu)
    if want("c5"):
        out["C5_llama7b_layer_seq2048_bf16"] = config_c5(torch, np, Model, Executor, llama, Inputs(torch, prng, "C5"), cpu)
    return out


def _rows_oneshot_ms(torch, Executor, plan, feeds, steps, launches=10, env=None):
    """Average duration (ms) of a one-shot launch of `steps` iterations of a row-op plan, under
    HIP events on the stream the kernel is launched on.  `env` is set while the plan compiles
    (compile() reads the ARKMI_* switches)."""
    side = torch.cuda.Stream()
    old = {k: os.environ.get(k) for k in (env or {})}
    os.environ.update(env or {})
    try:
        ex = Executor(plan, device_id=0, stream=side.cuda_stream, name="bench-oneshot", loop_mode=False).compile()
    finally:
        for k, v in old.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v
    for t, x in feeds:
        ex.tensor_write_device(t, x)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    with torch.cuda.stream(side):
        ex.launch()
        ex.run(steps)
        ex.wait()
        for s_, e_ in ev:
            s_.record()
            ex.run(steps)
            e_.record()
        ex.wait()
    torch.cuda.synchronize()
    ms = sum(s_.elapsed_time(e_) for s_, e_ in ev) / launches
    ex.stop()
    del ex
    return ms


def cpu_baseline_c2(x_np, w_np, min_seconds=8.0):
    """The oracle (a port of the reference's host baselines) timed on this machine's cores:
    passes over one X until `min_seconds` have gone by."""
    from oracle import ark_oracle as O
    O.lib()
    O.reduce(x_np[:256], -1, "sum", "fp16")  # thread pool start-up outside the clock
    passes = 0
    t0 = time.perf_counter()
    while True:
        O.reduce(x_np, -1, "sum", "fp16")
        O.softmax(x_np, "fp16")
        O.rmsnorm(x_np, w_np, "fp16", eps=1e-6)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds:
            break
    total = sum(ALGO_BYTES.values()) * passes
    return {"value": round(total / dt / 1e9, 3), "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
            "sample": f"{passes} passes of reduce_sum+softmax+rmsnorm over one X[16384,4096] fp16 "
                      f"(a quarter of a step) in {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=12)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the other configurations (C1, C3, C4, C5)")
    ap.add_argument("--only", choices=["c1", "c3", "c4", "c5"], default=None,
                    help="run only this configuration and print its block (for profiling one configuration)")
    ap.add_argument("--timeline", action="store_true",
                    help="with --only c4 or c5: print the per-step workgroup clocks of the plan instead (text)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path "
              "(--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import ark_amd
    from ark_amd import Model, Executor, llama, prng

    torch.cuda.set_device(0)
    info = ark_amd.device_info(0)
    cpu = not args.no_cpu_baseline

    if args.timeline:
        if args.only not in ("c4", "c5"):
            print("--timeline needs --only c4 or --only c5", file=sys.stderr)
            sys.exit(2)
        timeline(torch, np, Model, Executor, llama, prng, args.only)
        return
    if args.only:
        print(json.dumps({"only": args.only,
                          "configs": other_configs(torch, np, Model, Executor, llama, prng, cpu, only=args.only)}))
        return

    inp = Inputs(torch, prng, "C2")
    xs = [inp.normal(f"X{i}", (ROWS, COLS), torch.float16) for i in range(NBUF)]
    w = inp.uniform("rmsnorm_weight", (COLS,), torch.float32, 0.5, 1.5)

    # ---- the workload as a model, planned and run in the loop kernel -------------
    m = Model()
    tx = [m.tensor([ROWS, COLS], "fp16") for _ in range(NBUF)]
    tw = m.tensor([COLS], "fp32")
    outs = []
    for t in tx:
        outs.append((m.reduce_sum(t, -1), m.softmax(t), m.rmsnorm(t, tw, 1e-6)))
    plan = m.plan(device_id=0)
    ex = Executor(plan, device_id=0, name="bench").compile()
    for t, x in zip(tx, xs):
        ex.tensor_write_device(t, x)
    ex.tensor_write_device(tw, w)
    torch.cuda.synchronize()

    steps, warm = max(1, args.steps), max(0, args.warmup)
    # The machine probes (a few hundred milliseconds of MFMA and streaming load) run first: the
    # chip leaves its idle clocks over tens of milliseconds of load, longer than the warm-up steps
    # last, and the timed steps should see the clocks every later measurement of this run sees.
    machine = machine_probes(torch, prng)
    # The loop kernel stays resident between run() calls, so a device-wide synchronize inside
    # the timed region would wait for it to leave; Executor.wait() is the completion point.
    ex.launch()
    # Untimed load on this kernel as well, 30 ms of it in batches of the timed size: between the
    # probes and the first command the chip has idled through the kernel's launch, and the `value`
    # leg is meant to read the rate the resident kernel sustains, not the first milliseconds of a
    # clock ramp (the same is done for every other resident figure of this file).  Then the W
    # warm-up steps of the contract, then exactly K timed steps.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < 0.03:
        ex.run(steps)
        ex.wait()
    if warm:
        ex.run(warm)
        ex.wait()
    t0 = time.perf_counter()
    ex.run(steps)
    ex.wait()
    dt = time.perf_counter() - t0
    ex.stop()
    torch.cuda.synchronize()
    ms_per_step = dt / steps * 1e3
    step_bytes = sum(ALGO_BYTES.values()) * NBUF
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # spot check of the loop kernel's results on a few rows (full parity lives in tests/)
    got = torch.empty(ROWS, COLS, device="cuda", dtype=torch.float16)
    ex.tensor_read_device(outs[1][1], got)
    ref = torch.softmax(xs[1][:64].float(), -1)
    assert float((got[:64].float() - ref).abs().max()) < 1e-3, "loop-kernel softmax disagrees"
    kernel_families = ex.info()["kernel_families"]
    del ex

    # ---- roofline of the loop kernel: one-shot launches under HIP events ------------
    # The executor launches on a torch stream (default priority), so torch's events, recorded
    # on that stream, bracket the kernel.
    feeds = list(zip(tx, xs)) + [(tw, w)]
    launch_ms = _rows_oneshot_ms(torch, Executor, plan, feeds, steps)
    launch_bytes = step_bytes * steps
    achieved = launch_bytes / (launch_ms * 1e-3) / 1e9
    # the same plan with every op streaming X from HBM: no byte of the count is a cache hit
    hbm_ms = _rows_oneshot_ms(torch, Executor, plan, feeds, steps, env={"ARKMI_ROW_CACHED_INPUT": "0"})
    hbm_only = launch_bytes / (hbm_ms * 1e-3) / 1e9
    # each op alone over the four rotating X tensors (plans of four ops; nothing is read twice)
    per_op = {}
    for name in ("reduce_sum", "softmax", "rmsnorm"):
        mo = Model()
        txo = [mo.tensor([ROWS, COLS], "fp16") for _ in range(NBUF)]
        two = mo.tensor([COLS], "fp32")
        for t in txo:
            if name == "reduce_sum":
                mo.reduce_sum(t, -1)
            elif name == "softmax":
                mo.softmax(t)
            else:
                mo.rmsnorm(t, two, 1e-6)
        fo = list(zip(txo, xs)) + ([(two, w)] if name == "rmsnorm" else [])
        ms = _rows_oneshot_ms(torch, Executor, mo.plan(device_id=0), fo, steps, launches=5)
        gbps = ALGO_BYTES[name] * NBUF * steps / (ms * 1e-3) / 1e9
        per_op[name] = {"us_per_X": round(ms * 1e3 / steps / NBUF, 2), "achieved": round(gbps, 1),
                        "frac": round(gbps / HBM_PEAK_GBPS, 4)}

    traffic_per_step, traffic_src = profiled_traffic_bytes_per_step()
    roofline = {"bound": "hbm",
                "kernel": f"arkmi_loop_kernel<{kernel_families}> (one-shot launch of {steps} plan iterations = steps)",
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "frac_note": "algorithmic bytes; the second and third read of an X within a step may be served by "
                             "the Infinity Cache",
                "achieved_hbm_only": round(hbm_only, 1), "frac_hbm_only": round(hbm_only / HBM_PEAK_GBPS, 4),
                "hbm_only_note": "the same plan and launch with ARKMI_ROW_CACHED_INPUT=0: every op streams X from HBM",
                "per_op": per_op,
                "traffic": traffic_per_step * steps if traffic_per_step else None,
                "traffic_source": (f"{traffic_src} (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE per step x steps: bytes "
                                   "between the L2s and the fabric, Infinity Cache hits included; not measured in "
                                   "this run)") if traffic_per_step else None,
                "launch_ms": round(launch_ms, 4), "launch_algorithmic_bytes": launch_bytes,
                "us_per_step_in_launch": round(launch_ms * 1e3 / steps, 2)}

    out = {
        "metric": "GEMV/reduce HBM GB/s vs roofline (row ops reduce_sum+softmax+rmsnorm in one loop kernel; "
                  "algorithmic bytes per second through L2 and fabric: the three ops of an X re-read the same "
                  "128 MiB, which the Infinity Cache may serve)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": warm, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 (f32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "C2 row ops: X[16384,4096] fp16 ~N(0,1), reduce_sum + softmax + "
                               "RMSNorm(w~U(0.5,1.5), eps=1e-6), fp32 accumulate, one persistent loop "
                               "kernel; a step = the three ops over each of 4 rotating X tensors",
                   "device": info["gcn_arch"], "num_cu": info["num_cu"]},
        "roofline": roofline,
        "machine": machine,
    }
    if not args.no_extra:
        out["configs"] = other_configs(torch, np, Model, Executor, llama, prng, cpu)
    if cpu:
        out["cpu_baseline"] = cpu_baseline_c2(xs[0].cpu().numpy(), w.cpu().numpy())
    print(json.dumps(out))


if __name__ == "__main__":
    main()
