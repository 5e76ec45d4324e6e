#!/usr/bin/env python3
"""Benchmark of the device path on one MI355X.

A step is one pass of the hot path (every kernel of the lowered program, to EX) over one batch of
synthetic input that is already resident in HBM; the timed steps are queued back to back on the
device's stream (`adhip_program_enqueue`) between two waits (`adhip_program_sync`).  The headline workload is
BASELINE.json configs[1]: fused element-wise + broadcast, forward and backward, 8192x8192 f32.
The other configs are measured too (shorter) and reported under "extra".

Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "autodiff-ir-rust_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense FP32 matrix, published
# Bytes per launch between the L2 caches and the memory fabric, from rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by a plain
# copy kernel of known size (the summaries under profiles/ give the runs).  These counters sit in front of the 256 MiB
# last-level cache, so they bound HBM traffic from above.  Valid for the full-size workloads only.
TRAFFIC_BYTES = {
    # 2 x 393277.1 KiB fetched + 1081785.4 KiB written (the 4 outputs and two [512][8192] partial column-sum buffers)
    "fused_elw": {"elw_colsum": int((2 * 393277.1 + 1081785.4) * 1024)},
    # the one pass of configs[2] (dx with row and column sums riding along): 2 x 131353.0 KiB fetched + 278577.4 KiB
    # written (dx, the [512][4096] partial column sums, one run sum per row and 256 columns)
    "reductions": {"elw_colsum": int((2 * 131353.0 + 278577.4) * 1024)},
    # the stand-alone reductions (profiles/reductions_forward_and_row_chains.hbm_traffic_pmc.txt), by kernel kind and
    # tensors per launch: fetched x 2 + written (the column reduction writes a row of partial sums per 64 rows)
    "reductions_forward": {("reduce_row", 1): int((2 * 131085.5 + 512.0) * 1024), ("reduce_col", 1): int((2 * 131088.5 + 4096.0) * 1024),
                           ("reduce_row", 3): int((2 * 393230.0 + 1536.4) * 1024), ("reduce_col", 3): int((2 * 393233.5 + 12288.0) * 1024)},
    # gather stage of configs[4] (one tiled element-wise launch): 2 x 73777.4 KiB fetched + 294912.0 KiB written
    "manip_loop": {"gather_stage": int((2 * 73777.4 + 294912.0) * 1024)},
}


SPIN_UP_SECONDS = 0.25


def spin_up(prog, seconds=SPIN_UP_SECONDS):
    """Untimed runs until `seconds` have passed: a GPU that has been idle needs some tens of milliseconds of load
    before its clocks settle (the first 25 launches of the headline kernel measure 5-7 % slower than the rest)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            prog.enqueue()
        prog.sync()


def timed_runs(prog, steps, warmup, spin=True):
    """`steps` runs queued back to back on the device's stream, bracketed by a wait on both sides."""
    if spin:
        spin_up(prog)
    for _ in range(warmup):
        prog.run()
    prog.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        prog.enqueue()
    prog.sync()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps


def profile(prog, runs):
    """Per-kernel average durations from HIP events recorded on the stream the kernels run on."""
    prog.set_profiling(True)
    before = {i: (s.launches, s.total_ms) for i, s in enumerate(prog.kernel_stats())}
    for _ in range(runs):
        prog.run()
    prog.set_profiling(False)
    out = []
    for i, s in enumerate(prog.kernel_stats()):
        l0, ms0 = before[i]
        n = s.launches - l0
        if n:
            out.append({"kernel": s.name, "launches_per_run": n / runs, "avg_ms": (s.total_ms - ms0) / n,
                        "bytes": s.bytes_per_launch, "flops": s.flops_per_launch})
    return out


def hbm_roofline(kernel, algorithmic_bytes, traffic=None, note=None):
    """Roofline block of one HBM-bound launch site: algorithmic bytes over its average duration."""
    achieved = algorithmic_bytes / (kernel["avg_ms"] * 1e-3) / 1e9
    out = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
           "traffic": traffic, "kernel": kernel["kernel"], "avg_ms": kernel["avg_ms"], "algorithmic_bytes": algorithmic_bytes}
    if note:
        out["note"] = note
    return out


def compile_resident(dev, workload):
    proc, deps = workload.finish()
    prog = dev.compile(proc, deps)
    prog.upload()
    return prog


def cpu_baseline_fused_elw(rows, cols):
    """The oracle (a CPU restatement of the reference's per-kernel algorithms: one operation at a
    time, every intermediate stored) on a bounded sample of the headline workload."""
    from adhip import workloads as W
    from oracle.interp import OracleDevice, c_kernels
    wl = W.fused_elw(OracleDevice(), rows, cols, seed=0)
    t0 = time.perf_counter()
    wl.run()
    dt = time.perf_counter() - t0
    out = {"value": wl.algorithmic_bytes / dt / 1e9, "unit": "GB/s", "cores": int(c_kernels().ref_num_threads()),
           "kind": "port", "sample": f"fused_elw forward+backward on {rows}x{cols} f32 ({rows}/8192 of the rows), "
           f"{dt:.2f} s wall; rate on the same {wl.algorithmic_bytes:.0f} bytes as the GPU figure (the port itself stores "
           f"every intermediate, as the reference does)", "seconds": dt}
    # the other two rooflines, on bounded samples: configs[2] whole, and one 2048^3 product of configs[3]'s kind
    import numpy as np
    from oracle.interp import ref_dot
    wl3 = W.reductions(OracleDevice(), 16384, 4096, seed=0)
    t0 = time.perf_counter()
    wl3.run()
    dt3 = time.perf_counter() - t0
    a = np.ones((2048, 2048), dtype=np.float32)
    t0 = time.perf_counter()
    ref_dot(a, a)
    dtd = time.perf_counter() - t0
    out["other"] = {"reductions_GBps": wl3.algorithmic_bytes / dt3 / 1e9, "reductions_seconds": dt3,
                    "matmul_GFLOPs": 2.0 * 2048 ** 3 / dtd / 1e9, "matmul_sample": "one 2048x2048x2048 f32 product, "
                    "one output element per work-item, sequential k", "matmul_seconds": dtd}
    return out


def measure_mlp(dev, iters):
    """BASELINE.json configs[3]: `iters` training steps inside one resident program run."""
    from adhip import workloads as W
    wl4 = W.mlp_train(dev, 4096, (4096, 4096, 4096, 1024), iters, seed=0)
    p4 = compile_resident(dev, wl4)
    p4.run()      # warm-up: compiles nothing new, touches every buffer once
    p4.upload()   # a run consumes the loop counter; restore the initial state (not timed)
    t0 = time.perf_counter()
    p4.run()
    dt4 = time.perf_counter() - t0
    k4 = profile_once(p4)
    for k in k4:
        k["launches_per_run"] = k.pop("launches")
    dot_ms = sum(k["avg_ms"] * k["launches_per_run"] for k in k4 if k["kernel"].startswith("dot"))
    dot_fl = sum(k["flops"] * k["launches_per_run"] for k in k4 if k["kernel"].startswith("dot"))
    p4.close()
    tf = dot_fl / (dot_ms * 1e-3) / 1e12 if dot_ms else None
    out = {"steps_per_s": iters / dt4, "ms_per_train_step": dt4 * 1e3 / iters, "matmul_TFLOPs": tf,
           "matmul_frac_of_fp32_mfma_peak": tf / FP32_MFMA_PEAK_TFLOPS if tf else None,
           "flops_per_train_step": wl4.flops / iters}
    if tf:
        # all matrix-product launches of the run together: flops over the sum of their durations
        out["roofline"] = {"bound": "mfma", "achieved": tf, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                           "frac": tf / FP32_MFMA_PEAK_TFLOPS, "traffic": None, "kernel": "dot_mfma (all launches)",
                           "avg_ms": dot_ms / sum(k["launches_per_run"] for k in k4 if k["kernel"].startswith("dot"))}
    return out


MFMA_FP32_PEAK_TFLOPS = 157.3


def measure_attention(dev, seq=2048, d_model=1024, heads=8):
    """Multi-head attention forward (inference), [seq, d_model] activations: the fused attention kernel's rate against
    the FP32 matrix-core peak, and the same program lowered without the fusion beside it."""
    from adhip import workloads as W
    out = {}
    for mode in ("fused", "unfused"):
        if mode == "unfused":
            os.environ["ADHIP_FUSE_ATTENTION"] = "0"
        try:
            wl = W.attention_forward(dev, seq, d_model, heads, seed=0)
            prog = compile_resident(dev, wl)
        finally:
            os.environ.pop("ADHIP_FUSE_ATTENTION", None)
        ms = timed_runs(prog, 10, 3)
        ks = profile(prog, 3)
        entry = {"ms_per_step": ms, "launches_per_step": sum(k["launches_per_run"] for k in ks),
                 "matmul_TFLOPs_whole_step": wl.flops / (ms * 1e-3) / 1e12}
        if mode == "fused":
            for k in ks:
                if k["kernel"].startswith("attention"):
                    tf = wl.attention_flops / (k["avg_ms"] * 1e-3) / 1e12
                    entry["roofline"] = {"kernel": k["kernel"], "bound": "mfma", "achieved": tf, "peak": MFMA_FP32_PEAK_TFLOPS,
                                         "unit": "TFLOP/s", "frac": tf / MFMA_FP32_PEAK_TFLOPS, "traffic": None,
                                         "avg_ms": k["avg_ms"],
                                         "flops_per_launch": wl.attention_flops,
                                         "note": "2 * 2 * seq^2 * head_width flops per head (the two products; the "
                                                 "softmax arithmetic is not counted), all heads in one launch"}
        out[mode] = entry
        prog.close()
    out["config"] = {"seq": seq, "d_model": d_model, "heads": heads}
    return out


def measure_reductions_forward(dev, rows=16384, cols=4096):
    """The stand-alone reduction kernels at HBM size (what a forward-only `x.pow(2).sum(1)` / `x.sum(0)` runs: in the
    forward + backward step of configs[2] the sums ride on the element-wise pass instead).  Three programs: configs[2]
    without its backward pass; row sums of three different 256 MiB tensors; column sums of the same three.  With three
    tensors in turn no launch finds its operand in the 256 MiB last-level cache."""
    import numpy as np
    from adhip import autodiff
    from adhip import workloads as W
    n = rows * cols
    out = {"config": {"rows": rows, "cols": cols, "bytes_per_tensor": 4 * n}}

    def counted_traffic(k, tensors):
        # counter figures exist for the default size only
        return TRAFFIC_BYTES["reductions_forward"].get((k["kernel"].split(":")[0], tensors)) if (rows, cols) == (16384, 4096) else None
    wl = W.reductions(dev, rows, cols, seed=0, backward=False)
    p = compile_resident(dev, wl)
    ms = timed_runs(p, 10, 2)
    ks = profile(p, 5)
    # algorithmic bytes of a reduction launch: its operand read once (what it writes -- a vector, or the partial sums
    # of a two-stage reduction -- is not priced; `bytes` in the kernel list is what the launch moves, partials included)
    out["configs2_forward"] = {"ms_per_step": ms, "kernels": ks,
                               "roofline": [hbm_roofline(k, 4.0 * n, counted_traffic(k, 1), note="x read once by this launch") for k in ks if k["bytes"] > 2.0 * n]}
    p.close()
    rng = np.random.default_rng(0)
    data = [rng.standard_normal(n, dtype=np.float32) for _ in range(3)]
    for name, dim in (("row_sums", 1), ("column_sums", 0)):
        autodiff.set_device(dev)
        outs = {}
        for i, d in enumerate(data):
            s = autodiff.tensor(d, [rows, cols]).sum(dim)
            s.forward()
            s.val().keep()
            outs[f"s{i}"] = s.val()
        wls = W.Workload(name, outs, {}, algorithmic_bytes=3 * 4.0 * (n + (rows if dim else cols)))
        p = compile_resident(dev, wls)
        ms = timed_runs(p, 10, 2)
        ks = profile(p, 5)
        big = [k for k in ks if k["bytes"] > 2.0 * n]
        tensors = sum(round(k["bytes"] / (4.0 * n)) * k["launches_per_run"] for k in big)
        entry = {"ms_per_step": ms, "GBps_whole_step": wls.algorithmic_bytes / (ms * 1e-3) / 1e9, "kernels": ks, "tensors_per_step": tensors,
                 "roofline": [hbm_roofline(k, round(k["bytes"] / (4.0 * n)) * 4.0 * n, counted_traffic(k, round(k["bytes"] / (4.0 * n))), note=f"{round(k['bytes'] / (4.0 * n))} tensor(s) of {4 * n} bytes read once per launch; "
                                           "three tensors in turn, so none is found in the last-level cache") for k in big]}
        out[name] = entry
        p.close()
    return out


def measure_last_layer_products(dev):
    """The three products of configs[3]'s last layer (4096 -> 1024, batch 4096) on their own, without epilogues:
    y = x W (A rows contiguous), dW = x^T dy (A columns contiguous), dx = dy W^T (both along k).  With
    ADHIP_DOT_PLAN=<bm>,<bn>,<splits> in the environment the library launches them with that tile and that many ranges
    of k instead of its own choice, which is how alternative tiles are timed."""
    import numpy as np
    from adhip import ir as IR
    rng = np.random.default_rng(0)
    x = rng.standard_normal(4096 * 4096).astype(np.float32)
    w = rng.standard_normal(4096 * 1024).astype(np.float32)
    dy = rng.standard_normal(4096 * 1024).astype(np.float32)
    cmds = [IR.CreateMat(x, [4096, 4096], "x"), IR.CreateMat(w, [4096, 1024], "w"), IR.CreateMat(dy, [4096, 1024], "dy"),
            IR.DotProduct(a="x", b="w", res="y"),
            IR.Permute(a="x", p=[1, 0], res="xt"), IR.DotProduct(a="xt", b="dy", res="dw"),
            IR.Permute(a="w", p=[1, 0], res="wt"), IR.DotProduct(a="dy", b="wt", res="dx"), IR.EX()]
    prog = dev.compile(IR.IRProcedure("main", cmds), {"y", "dw", "dx"})
    prog.upload()
    ms = timed_runs(prog, 10, 2)
    ks = profile(prog, 5)
    prog.close()
    for k in ks:
        if k["flops"] > 1e9:
            k["TFLOPs"] = k["flops"] / (k["avg_ms"] * 1e-3) / 1e12
            k["frac_of_fp32_mfma_peak"] = k["TFLOPs"] / FP32_MFMA_PEAK_TFLOPS
    return {"plan": os.environ.get("ADHIP_DOT_PLAN", "library's choice"), "ms_per_step": ms, "kernels": ks}


def measure_encoder(dev, kernels=False):
    """One transformer encoder layer, forward + backward, [2048, 1024] activations, 8 heads, feed-forward width 4096;
    `kernels`: also the per-launch-site list (each with its rate by the bytes or flops the lowering prices it at)."""
    from adhip import workloads as W
    wl6 = W.encoder_layer(dev, 2048, 1024, 8, 4096, seed=0)
    p6 = compile_resident(dev, wl6)
    ms6 = timed_runs(p6, 5, 2)
    k6 = profile(p6, 2)
    dot6 = sum(k["avg_ms"] * k["launches_per_run"] for k in k6 if k["kernel"].startswith("dot"))
    all6 = sum(k["avg_ms"] * k["launches_per_run"] for k in k6)
    out = {"ms_per_step": ms6, "matmul_flops_per_step": wl6.flops,
           "matmul_TFLOPs_whole_step": wl6.flops / (ms6 * 1e-3) / 1e12,
           "matmul_kernels_ms": dot6, "other_kernels_ms": all6 - dot6,
           "launches_per_step": sum(k["launches_per_run"] for k in k6)}
    if kernels:
        for k in k6:
            if k["kernel"].startswith("dot") and k.get("flops"):
                k["TFLOPs"] = k["flops"] / (k["avg_ms"] * 1e-3) / 1e12
            elif k["bytes"]:
                k["GBps"] = k["bytes"] / (k["avg_ms"] * 1e-3) / 1e9
        out["kernels"] = sorted(k6, key=lambda k: -k["avg_ms"] * k["launches_per_run"])
    p6.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--skip-extra", action="store_true", help="measure only the headline workload")
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--mlp-iters", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=["all", "copy", "streammix", "mlp", "reductions", "reductions_forward", "manip", "attention", "last_layer_products", "encoder"],
                    help="'copy': only a plain 8192x8192 f32 copy kernel (256 MiB read + 256 MiB written per launch), "
                         "the known-size reference that hardware byte counters are scaled by; "
                         "'streammix': only a bare 3-reads + 4-writes kernel over 8192x8192 f32 (the stream mix of the "
                         "headline pass with trivial arithmetic and no column sums: what the memory system gives that mix); "
                         "'reductions': only configs[2]; 'reductions_forward': only the stand-alone row and column reduction "
                         "kernels on 256 MiB tensors; 'last_layer_products': the three 4096x1024x4096-shaped products of "
                         "configs[3]'s last layer on their own (honours ADHIP_DOT_PLAN); 'mlp': only configs[3]; 'manip': only configs[4] (one run: its "
                         "loop consumes its counter); 'attention': only multi-head attention forward; 'encoder': only the encoder "
                         "layer, with its per-kernel list")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the device path is single-device (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    from adhip import HipDevice
    from adhip import workloads as W

    dev = HipDevice(0)
    rows = cols = 8192
    if args.workload == "copy":
        import numpy as np
        from adhip import autodiff
        autodiff.set_device(dev)
        src = autodiff.tensor(np.zeros(rows * cols, dtype=np.float32), [rows, cols])
        dst = src.contigious()
        dst.forward()
        dst.val().keep()
        wlc = W.Workload("copy", {"dst": dst.val()}, {}, algorithmic_bytes=8.0 * rows * cols)
        pc = compile_resident(dev, wlc)
        msc = timed_runs(pc, args.steps, args.warmup)
        print(json.dumps({"metric": "plain copy", "value": wlc.algorithmic_bytes / (msc * 1e-3) / 1e9, "unit": "GB/s",
                          "ms_per_step": msc, "bytes_read": 4.0 * rows * cols, "bytes_written": 4.0 * rows * cols,
                          "kernels": profile(pc, 3)}))
        return
    if args.workload == "streammix":
        import numpy as np
        from adhip import autodiff
        autodiff.set_device(dev)
        rng = np.random.default_rng(0)
        a, b, c = (autodiff.tensor(rng.uniform(-1.0, 1.0, size=rows * cols).astype(np.float32), [rows, cols]) for _ in range(3))
        outs = {}
        for name, t in (("o0", a + b), ("o1", b + c), ("o2", a + c), ("o3", a * b)):
            t.forward()
            t.val().keep()
            outs[name] = t.val()
        wlm = W.Workload("streammix", outs, {}, algorithmic_bytes=7 * 4.0 * rows * cols)
        pm = compile_resident(dev, wlm)
        msm = timed_runs(pm, args.steps, args.warmup)
        ks = profile(pm, 5)
        print(json.dumps({"metric": "bare 3-read + 4-write stream mix, f32 [8192,8192]", "value": wlm.algorithmic_bytes / (msm * 1e-3) / 1e9,
                          "unit": "GB/s", "ms_per_step": msm, "frac_of_hbm_peak": wlm.algorithmic_bytes / (msm * 1e-3) / 1e9 / HBM_PEAK_GBS,
                          "kernels": ks}))
        return
    if args.workload == "reductions":
        wl3 = W.reductions(dev, 16384, 4096, seed=0)
        p3 = compile_resident(dev, wl3)
        ms3 = timed_runs(p3, args.steps, args.warmup)
        print(json.dumps({"metric": "reductions forward + backward, f32 [16384,4096]", "value": wl3.algorithmic_bytes / (ms3 * 1e-3) / 1e9,
                          "unit": "GB/s", "ms_per_step": ms3, "algorithmic_bytes": wl3.algorithmic_bytes, "kernels": profile(p3, 3)}))
        return
    if args.workload == "last_layer_products":
        print(json.dumps(dict(measure_last_layer_products(dev), metric="products of the 4096 -> 1024 layer, fp32")))
        return
    if args.workload == "reductions_forward":
        print(json.dumps(dict(measure_reductions_forward(dev), metric="stand-alone reductions, f32 [16384,4096]")))
        return
    if args.workload == "manip":
        wl5 = W.manip_loop(dev)
        p5 = compile_resident(dev, wl5)
        t0 = time.perf_counter()
        p5.run()
        ms5 = (time.perf_counter() - t0) * 1e3
        k5 = profile_once(p5)
        spin_up(p5)
        print(json.dumps({"metric": "tensor manipulation + data-dependent loop, one run", "value": ms5, "unit": "ms",
                          "kernels": k5, "stage_after_spin_up": profile(p5, 5)}))
        return
    if args.workload == "attention":
        print(json.dumps(dict(measure_attention(dev), metric="multi-head attention forward, fp32")))
        return
    if args.workload == "encoder":
        print(json.dumps(dict(measure_encoder(dev, kernels=True), metric="transformer encoder layer forward + backward, fp32")))
        return
    if args.workload == "mlp":
        print(json.dumps(dict(measure_mlp(dev, args.mlp_iters), metric="fp32 MLP train steps/s")))
        return
    wl = W.fused_elw(dev, rows, cols, seed=0)
    prog = compile_resident(dev, wl)
    # five timed loops of exactly `steps` steps each; the reported step time is the median loop's, the others say how
    # far one 6 ms sample can be off
    loops = sorted(timed_runs(prog, args.steps, args.warmup if i == 0 else 0, spin=(i == 0)) for i in range(5))
    ms = loops[len(loops) // 2]
    value = wl.algorithmic_bytes / (ms * 1e-3) / 1e9
    kstats = profile(prog, 5)
    dom = max(kstats, key=lambda k: k["avg_ms"] * k["launches_per_run"])
    n = rows * cols
    # algorithmic bytes of the dominant launch: a, b, c, bias read once; y, da, db, dc written once
    dom_alg = 4.0 * (7 * n + cols) if dom["kernel"].startswith("elw") else dom["bytes"]
    roofline = hbm_roofline(dom, dom_alg, TRAFFIC_BYTES["fused_elw"]["elw_colsum"] if dom["kernel"].startswith("elw_colsum") else None)
    roofline["traffic_source"] = ("hardware counters of a separate rocprofv3 --pmc run of this workload (summary: "
                                  "profiles/fused_elw_8192x8192.hbm_traffic_pmc.txt); a constant of this script, not read in this run")
    prog.close()

    extra = {"fused_elw_kernels": kstats}
    if not args.skip_extra:
        # config 1: README MLP, a latency case: complete adhip_execute calls (parse, lower, upload, run, read back)
        wl1 = W.readme_mlp(dev, seed=0)
        proc1, deps1 = wl1.finish()
        dev.execute(proc1, deps1)  # first call compiles the kernels
        dev.execute(proc1, deps1)  # second call captures the launch run into a graph (about 3 ms, once)
        t0 = time.perf_counter()
        for _ in range(20):
            dev.execute(proc1, deps1)
        us_exec = (time.perf_counter() - t0) / 20 * 1e6
        # the same call without the Python serialiser in front of it: the C ABI on a stream that is already in wire format
        from adhip import ir as IR
        blob1, keepalive1 = IR.serialize(proc1)
        dev.execute_serialized(blob1, deps1)
        t0 = time.perf_counter()
        for _ in range(50):
            dev.execute_serialized(blob1, deps1)
        us_abi = (time.perf_counter() - t0) / 50 * 1e6
        del keepalive1
        p1 = dev.compile(proc1, deps1)
        p1.upload()
        p1.run()
        t0 = time.perf_counter()
        for _ in range(50):
            p1.run()
        us_run = (time.perf_counter() - t0) / 50 * 1e6
        extra["readme_mlp"] = {"us_per_execute_call": us_exec, "us_per_adhip_execute": us_abi, "us_per_resident_run": us_run,
                               "kernels_per_run": sum(1 for s_ in p1.kernel_stats())}
        p1.close()
        # config 3: reductions
        wl3 = W.reductions(dev, 16384, 4096, seed=0)
        p3 = compile_resident(dev, wl3)
        ms3 = timed_runs(p3, max(5, args.steps // 2), 2)
        k3 = profile(p3, 3)
        n3 = 16384 * 4096
        extra["reductions"] = {"ms_per_step": ms3, "GBps": wl3.algorithmic_bytes / (ms3 * 1e-3) / 1e9,
                               "frac_of_hbm_peak": wl3.algorithmic_bytes / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                               "algorithmic_bytes": wl3.algorithmic_bytes,
                               "accounting": "bytes the lowered step moves: one pass reads x and writes dx; the row sums "
                                             "(x*x).sum(1) and the column sums x.sum(0) ride along with it",
                               "kernels": k3, "roofline": []}
        for k in k3:
            if k["kernel"].startswith("elw_colsum:"):
                # x read once, dx written once, the row and column sums
                extra["reductions"]["roofline"].append(hbm_roofline(k, 4.0 * (2 * n3 + 4096 + 16384), TRAFFIC_BYTES["reductions"]["elw_colsum"]))
        p3.close()
        extra["reductions_forward"] = measure_reductions_forward(dev)
        # config 5: tensor manipulation + data-dependent loop
        wl5 = W.manip_loop(dev)
        p5 = compile_resident(dev, wl5)
        t0 = time.perf_counter()
        p5.run()
        ms5 = (time.perf_counter() - t0) * 1e3
        k5 = profile_once(p5)
        for k in k5:
            # r is 151 MB and is rewritten every iteration: it stays in the 256 MiB last-level cache, so the loop
            # kernels' rates are cache rates, not HBM rates
            k["GBps"] = k["bytes"] / (k["avg_ms"] * 1e-3) / 1e9
            # (that includes the row reduction launched once right behind the gather stage, which wrote r)
            k["memory"] = "HBM" if k["launches"] == 1 and not k["kernel"].startswith("reduce") else "LLC-resident"
        # The gather stage again, the way every other kernel here is timed (clocks settled, several launches): the
        # run above follows an upload, during which the compute units idle.  Runs of the resident program repeat the
        # stage on the same inputs; the loop after it finds its counter at the limit and does not iterate.
        spin_up(p5)
        stage = [k for k in profile(p5, 5) if k["bytes"] > 1e8 and not k["kernel"].startswith("reduce")]
        extra["manip_loop"] = {"ms_total": ms5, "kernels": k5,
                               "gather_stage": {"algorithmic_bytes": 150994944 + 301989888, "note": "the gathered regions of p and q read "
                                                "once (151 MB), r and the kept copy of the gathered tensor written (151 MB each); "
                                                "ms: average of 5 launches after the clocks have settled (ms_first_run: the "
                                                "single launch right after the upload)",
                                                "traffic": TRAFFIC_BYTES["manip_loop"]["gather_stage"],
                                                "moved_bytes": sum(k["bytes"] for k in stage),
                                                "ms": sum(k["avg_ms"] for k in stage),
                                                "ms_first_run": sum(k["avg_ms"] for k in k5 if k["launches"] == 1 and k["bytes"] > 1e8 and not k["kernel"].startswith("reduce"))}}
        p5.close()
        # config 4: dense MLP training
        extra["mlp_train"] = measure_mlp(dev, args.mlp_iters)
        # beyond BASELINE.json's configs: one transformer encoder layer (the caller side's attention modules),
        # forward + backward, [2048, 1024] activations, 8 heads, feed-forward width 4096
        extra["encoder_layer"] = measure_encoder(dev)
        extra["attention_forward"] = measure_attention(dev)

    cpu = None
    if not args.skip_cpu:
        cpu = cpu_baseline_fused_elw(8192, 8192)

    line = {
        "metric": "fused-ELW & reduce GB/s (% HBM peak); fp32 MLP train steps/s, 1 MI355X",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "ms_per_step_of_each_timed_loop": loops, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "spin_up_seconds": SPIN_UP_SECONDS,
        "data": "synthetic",
        "config": {"workload": "configs[1]: fused element-wise + broadcast, forward + backward, a,b,c f32 [8192,8192], bias [8192]",
                   "algorithmic_bytes_per_step": wl.algorithmic_bytes,
                   "accounting": "a, b, c, bias read once; y, da, db, dc, dbias, L written once (forward and backward are one pass)",
                   "frac_of_hbm_peak": value / HBM_PEAK_GBS,
                   "unfused_accounting_bytes": wl.unfused_bytes,
                   "unfused_accounting_note": "forward and backward priced as separate sweeps; divided by the fused step's time "
                                              "this is not a bandwidth and is not reported as one"},
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(line))


def profile_once(prog):
    """Re-upload the inputs and profile one complete run (for programs whose run is not idempotent)."""
    before = {i: (s.launches, s.total_ms) for i, s in enumerate(prog.kernel_stats())}
    prog.set_profiling(True)
    prog.upload()
    prog.run()
    prog.set_profiling(False)
    out = []
    for i, s in enumerate(prog.kernel_stats()):
        n = s.launches - before[i][0]
        if n:
            out.append({"kernel": s.name, "launches": n, "avg_ms": (s.total_ms - before[i][1]) / n,
                        "bytes": s.bytes_per_launch, "flops": s.flops_per_launch})
    return out


if __name__ == "__main__":
    main()
