#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one decode token's worth of Q4_K projections of a Llama-3-8B-shaped model through the
C ABI — q, k, v, o, gate, up, down, output head: 8 matvecs in the CPU reference's arithmetic, the
activation vector of each of the 5 stages quantized once per 256 (quant_q8k) and shared by the
projections that read it, all reading weights from HBM (the step's 418 MB exceed the 256 MB last-level cache and the weight sets rotate).
Prints ONE JSON line: whole-step GB/s of algorithmic bytes, the roofline of the dominant kernel
(timed per launch with events on the launching stream), the CPU oracle timed on the host cores,
and secondary figures (prefill GEMM, MoE, verify) under "extra".
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
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
Q4_K = 12

# Llama-3-8B projection set: name -> (N = out, K = in)
SHAPES = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
          ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336), ("head", 128256, 4096)]
# stage input -> projections that read it
STAGES = [("x_attn", 4096, ["q", "k", "v"]), ("x_o", 4096, ["o"]), ("x_ffn", 4096, ["gate", "up"]),
          ("x_down", 14336, ["down"]), ("x_head", 4096, ["head"])]


# HBM bytes per launch of the head matvec (128256 x 4096 Q4_K) from hardware counters: FETCH_SIZE
# 144 328 KiB x 2.000 (the factor the same counter needs to read a 512 MiB copy correctly) +
# WRITE_SIZE 502 KiB.  Algorithmic bytes of the launch: 296 031 232.
HEAD_TRAFFIC_BYTES = 296_088_772


def algorithmic_bytes(n: int, k: int) -> int:
    """Weight bytes + activation vector + output vector of one Q4_K matvec."""
    return n * (k // 256) * 144 + 4 * k + 4 * n


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--copies", type=int, default=2, help="rotating weight sets")
    ap.add_argument("--eager", action="store_true", help="issue every launch from the host instead of replaying a recorded step")
    ap.add_argument("--per-projection", action="store_true",
                    help="one launch per projection instead of grouped q/k/v and gate/up launches")
    ap.add_argument("--fused-quant", action="store_true",
                    help="quantize x inside every matvec launch (8 launches per step) instead of once per "
                         "stage in a launch of its own (5 + 8 launches); measured slower")
    ap.add_argument("--split-quant", action="store_true",
                    help="always quantize in a launch of its own (5 + 5 launches) instead of one ojh_mm_multi call per stage")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary measurements")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has one GPU and nothing here uses a "
              "second (no collectives, no sharding). Run with --gpus 1.", file=sys.stderr)
        return 2

    pkg = entry.load_package()
    synth = pkg.synth
    gpu = pkg.HipGpu(0)
    caps = gpu.caps()

    # ---- weights: `copies` sets of the 8 projections, resident in HBM before timing
    t0 = time.time()
    host = {name: synth.q4k_weights(n, k, "bench", "q4k", name) for name, n, k in SHAPES}
    dims = {name: (n, k) for name, n, k in SHAPES}
    sets = [{name: gpu.lin(Q4_K, *dims[name], host[name]) for name, _, _ in SHAPES} for _ in range(args.copies)]
    xs = {st: gpu.upload(synth.normal_f32(k, "bench", st)) for st, k, _ in STAGES}
    xq = {st: gpu.alloc_bytes(k) for st, k, _ in STAGES}
    xsc = {st: gpu.alloc(k // 256) for st, k, _ in STAGES}
    ys = {name: gpu.alloc(n) for name, n, _ in SHAPES}
    setup_s = time.time() - t0

    step_bytes = sum(algorithmic_bytes(n, k) for _, n, k in SHAPES)
    dom = "head"  # the launch that dominates the step: 295.5 MB of its 418 MB

    def one(st: str, lin, y) -> None:
        """One projection alone: from the stage's separately quantized vector, or (--fused-quant) from the f32 vector
        through the single-tensor launch that quantizes it itself."""
        if (not args.fused_quant):
            gpu.mm_q8k(xq[st], xsc[st], lin, y)
        else:
            gpu.mm(xs[st], lin, y, 1, act_mode=pkg.ACT_Q8K)

    grouped = not args.fused_quant and not args.per_projection
    staged = grouped and not args.split_quant

    def step(i: int) -> None:
        w = sets[i % args.copies]
        for st, k, names in STAGES:
            if staged:
                # one call per stage from the f32 vector: the library folds the quantizer into the launch where that is
                # faster (the small q/k/v stage) and otherwise issues a quantizer launch and one grouped launch
                gpu.mm_multi(xs[st], [w[n] for n in names], [ys[n] for n in names])
                continue
            if (not args.fused_quant):
                gpu.quant_q8k(xs[st], 1, k, xq[st], xsc[st])
            if grouped and len(names) > 1:
                # q/k/v and gate/up read the same vector: one launch over the separate tensors
                gpu.mm_q8k_multi(xq[st], xsc[st], [w[n] for n in names], [ys[n] for n in names])
                continue
            for name in names:
                one(st, w[name], ys[name])

    # The launches of a step are recorded once per weight set and replayed with one host call,
    # so the host's per-call cost (here: Python) stays out of the device timeline.
    for i in range(args.copies):
        step(i)
    gpu.submit()
    graphs = []
    if not args.eager:
        for i in range(args.copies):
            gpu.capture_begin()
            step(i)
            graphs.append(gpu.capture_end())

    def run_step(i: int) -> None:
        if graphs:
            graphs[i % args.copies].launch()
        else:
            step(i)

    for i in range(args.warmup):
        run_step(i)
    gpu.submit()
    # ... and about 10 ms more of untimed steps, whatever --warmup says: after the uploads above the part needs
    # milliseconds to bring its clocks back up, and steady-state decode is what the metric means
    gpu.timer_start()
    run_step(0)
    one_ms = max(gpu.timer_stop(), 1e-3)
    preroll_steps = min(2000, int(10.0 / one_ms))
    for i in range(preroll_steps):
        run_step(i)
    preroll_ms = preroll_steps * one_ms     # (no synchronisation here: the timed steps follow on the stream at once)

    # ---- timed region: exactly `steps` steps, events on the launching stream + host clock
    t_host = time.perf_counter()
    gpu.timer_start()
    for i in range(args.steps):
        run_step(i)
    ms_total = gpu.timer_stop()
    gpu.submit()
    host_ms = (time.perf_counter() - t_host) * 1e3
    ms_per_step = ms_total / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- roofline leg: the dominant kernel alone (the head's launch, its own entry point),
    # back to back over the rotating sets, events on the launching stream
    dn, dk = dims[dom]
    dom_bytes = algorithmic_bytes(dn, dk)
    dom_reps = max(args.steps, 20)
    for st, k, _ in STAGES:  # the split form reads these
        gpu.quant_q8k(xs[st], 1, k, xq[st], xsc[st])
    for i in range(3):
        one("x_head", sets[i % args.copies][dom], ys[dom])
    gpu.timer_start()
    for i in range(dom_reps):
        one("x_head", sets[i % args.copies][dom], ys[dom])
    dom_avg_ms = gpu.timer_stop() / dom_reps
    achieved = dom_bytes / (dom_avg_ms * 1e-3) / 1e9

    # ---- calibration launches: a plain copy and a plain read of known size (512 MiB each way),
    # the yardstick for hardware counters and for what this chip's HBM delivers to any kernel
    gpu.ensure_family("glue")
    cal_n16 = (512 << 20) // 16
    cal_src, cal_dst = gpu.alloc_bytes(cal_n16 * 16), gpu.alloc_bytes(cal_n16 * 16)
    gpu.memset0(cal_src)
    cgrid, cblock = gpu.launch_shape("stream_copy_u32x4", 0, cal_n16, 0)
    cal = {}
    for kname, moved in (("stream_copy_u32x4", 2 * cal_n16 * 16), ("stream_read_u32x4", cal_n16 * 16)):
        us = _time(gpu, lambda i: gpu.dispatch(gpu.begin(), kname, [(cal_src, 0), (cal_dst, 0)], [cal_n16], cgrid, cblock), 5, 2)
        cal[kname] = {"bytes_moved": moved, "us": round(us, 1), "gbs": round(moved / us / 1e3, 1)}
    del cal_src, cal_dst
    # ... and what the matrix pipe sustains on this part (it is power-limited: the figure depends on the operands):
    # one workgroup of four waves per CU, 16 independent 32x32x16 f16 MFMAs per trip, operands constant / N(0,1),
    # held in registers / read back from LDS per group of 16 as the prefill tile does / with the copies, LDS writes and
    # vector-ALU work a dequantizing 256x256x64 tile step adds (the ceiling any such tile can reach on this part)
    mf_iters = 1024
    mgrid, mblock = gpu.launch_shape("calib_mfma_f16", 0, 0, 0)
    mf_flops = mgrid[0] * 4 * mf_iters * 64 * 2 * 32 * 32 * 16
    mf_out = gpu.alloc(mgrid[0] * 256)
    n_ops = 8 * 256 * 8 + (4 << 20) // 2      # a workgroup's fragments, then the 4 MB window mode 2 copies from
    ops_const = np.full(n_ops, 1.0, np.float16)
    ops_rand = synth.normal_f32(n_ops, "bench", "mfma_calibration").astype(np.float16)
    for tag, ops in (("constant", ops_const), ("normal", ops_rand)):
        src = gpu.upload_bytes(ops)
        for mode, where in ((0, "registers"), (1, "lds"), (2, "lds_tile_step_mix")):
            us = _time(gpu, lambda i: gpu.dispatch(gpu.begin(), "calib_mfma_f16", [(src, 0), (mf_out, 0)], [mf_iters, mode],
                                                    mgrid, mblock), 5, 2)
            cal[f"mfma_f16_{tag}_{where}"] = {"flops": mf_flops, "us": round(us, 1), "tflops": round(mf_flops / us / 1e6, 1),
                                              "mfma_frac": round(mf_flops / us / 1e6 / 2500.0, 4)}
        del src
    # ... and the int8 matrix instruction of the CPU-arithmetic prefill tile, v_mfma_i32_16x16x64_i8, the same way
    i8_ops = mgrid[0] * 4 * mf_iters * 64 * 2 * 16 * 16 * 64
    for tag, ops in (("constant", np.full(8 * 256 * 16, 1, np.int8)),
                     ("normal", (synth.normal_f32(8 * 256 * 16, "bench", "mfma_i8_calibration") * 60).clip(-127, 127).astype(np.int8))):
        src = gpu.upload_bytes(ops)
        for mode, where in ((0, "registers"), (1, "lds")):
            us = _time(gpu, lambda i: gpu.dispatch(gpu.begin(), "calib_mfma_i8", [(src, 0), (mf_out, 0)], [mf_iters, mode],
                                                    mgrid, mblock), 5, 2)
            cal[f"mfma_i8_{tag}_{where}"] = {"ops": i8_ops, "us": round(us, 1), "tops": round(i8_ops / us / 1e6, 1),
                                             "int8_mfma_frac": round(i8_ops / us / 1e6 / 5000.0, 4)}
        del src
    del mf_out

    # ---- per-shape latency (each shape alone, back to back), for the record, twice: streaming from HBM — as many
    # copies of the shape as it takes to exceed the 256 MB Infinity Cache, visited in turn — and cache-resident (two
    # copies).  The launches are recorded once and replayed from the library, like the step: issued one by one from
    # Python the short ones would show the interpreter's call rate, not the kernel.  The stage's quantized vector is
    # prepared beforehand: these are the matvec launches alone.
    per_shape = {}
    reps = 60
    mall = 256 << 20
    for name, n, k in SHAPES:
        st = next(s for s, _, names in STAGES if name in names)
        b = algorithmic_bytes(n, k)
        wbytes = n * (k // 256) * 144
        ncold = max(2, mall // wbytes + 2)
        extra_lins = [gpu.lin(Q4_K, n, k, host[name]) for _ in range(max(0, ncold - args.copies))]
        pool = [sets[i][name] for i in range(args.copies)] + extra_lins
        entry_ = {"n": n, "k": k}
        for tag, lins in (("hbm", pool[:ncold]), ("cache", pool[:2])):
            gpu.capture_begin()
            for i in range(reps):
                one(st, lins[i % len(lins)], ys[name])
            chain = gpu.capture_end()
            gpu.timer_start()
            chain.launch()
            chain_ms = max(gpu.timer_stop(), 1e-3)
            for _ in range(min(200, int(10.0 / chain_ms))):     # about 10 ms of untimed replays: clocks back up
                chain.launch()
            gpu.timer_start()
            chain.launch()
            us = gpu.timer_stop() / reps * 1e3
            del chain
            if tag == "hbm":
                entry_.update({"us": round(us, 2), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4),
                               "copies": len(lins)})
            else:
                entry_.update({"cache_resident_us": round(us, 2), "cache_resident_gbs": round(b / us / 1e3, 1)})
        per_shape[name] = entry_
        for l in extra_lins:
            l.free()

    result = {
        "metric": "Q4_K decode GEMV GB/s (% HBM peak); prefill dequant-GEMM TFLOPS, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preroll_ms": round(preroll_ms, 2),
        "preroll_steps": preroll_steps,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 x u4 dots (quant_q8k activations), f32 scale algebra",
        "data": "synthetic",
        "config": {"workload": "Q4_K decode GEMV over the Llama-3-8B projection set, batch 1 "
                               "(q,k,v,o 4096; gate,up 14336x4096; down 4096x14336; head 128256x4096), "
                               "f32 activations N(0,1) quantized once per stage, weights in HBM",
                   "bytes_per_step": step_bytes, "weight_sets": args.copies,
                   "launches_per_step": "one ojh_mm_multi call per stage: q/k/v in 1 launch with the quantizer folded in "
                                        "(gemv_fq8k_q4k_x4_r2), the other four stages quantize_q8k + one gemv_q8k_q4k* launch "
                                        "(gate/up grouped over separate tensors): 9 launches" if staged else
                                        "5 quantize_q8k + 5 gemv_q8k_q4k* (q/k/v and gate/up each one grouped "
                                        "launch over separate tensors)" if grouped else
                                        "5 quantize_q8k + 8 gemv_q8k_q4k*" if (not args.fused_quant) else
                                        "8 gemv_fq8k_q4k* (activation quantizer folded into each launch)",
                   "submission": "eager, one host call per launch" if args.eager else
                                 "recorded step replayed from the library (%s)" % os.environ.get("OJAS_HIP_REPLAY", "list")},
        "hbm_frac": round(value / HBM_PEAK_GBS, 4),
        "host_ms_per_step": round(host_ms / args.steps, 5),
        "roofline": {"bound": "hbm", "kernel": "gemv_q8k_q4k_wide" if (not args.fused_quant) else "gemv_fq8k_q4k_wide", "launch": f"head {dn}x{dk}",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": HEAD_TRAFFIC_BYTES if (dom == "head" and not args.fused_quant) else None,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by the "
                                       "same counters over stream_copy_u32x4 (x2.000 / x1.000); a recorded "
                                       "figure, not re-measured by this run",
                     "bytes_per_launch": dom_bytes, "avg_launch_us": round(dom_avg_ms * 1e3, 2)},
        "per_shape": per_shape,
        "calibration": cal,
        "device": {"name": gpu.name(), "cus": caps.compute_units, "clock_mhz": caps.clock_mhz},
        "setup_s": round(setup_s, 1),
    }

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(host, dims)
    if not args.no_extra:
        graphs.clear()
        chain = chain_leg(gpu, pkg, sets, dims, step_bytes)
        lin_q = sets[0]["gate"], sets[0]["down"], sets[0]["head"]
        result["extra"] = extras(gpu, pkg, lin_q)
        result["extra"]["decode_chain_dependent"] = chain
    print(json.dumps(result))
    gpu.close()
    return 0


def _time(gpu, fn, reps: int, warm: int = 3) -> float:
    """Average microseconds per call of `fn(i)` over `reps` calls, events on the launching stream.  Untimed calls come
    first until about 10 ms of them have run: after the idle time a leg's setup leaves, the part needs that long to
    bring its clocks back up (the same launches measure up to 10 % slower right after a pause)."""
    for i in range(warm):
        fn(i)
    gpu.timer_start()
    fn(0)
    one_ms = max(gpu.timer_stop(), 1e-3)
    for i in range(min(2000, int(10.0 / one_ms))):
        fn(i)
    gpu.timer_start()
    for i in range(reps):
        fn(i)
    return gpu.timer_stop() / reps * 1e3


def chain_leg(gpu, pkg, sets, dims, step_bytes) -> dict:
    """The same eight projections as a chain in which every stage reads what the one before it wrote (x -> q,k,v;
    q -> o; rmsnorm(o) -> gate,up; silu(gate) * up -> down; rmsnorm(down) -> head), once as ONE launch
    (ojh_decode_chain) and once as the separate launches that compute the same bits."""
    R, synth = pkg.runtime, pkg.synth
    d, nff = dims["q"][1], dims["gate"][0]
    x0 = gpu.upload(synth.normal_f32(d, "bench", "chain_x0"))
    gamma = gpu.upload(np.ones(d, np.float32))
    y = {n: gpu.alloc(dims[n][0]) for n in dims}
    xq, xs, act = gpu.alloc_bytes(d), gpu.alloc(d // 256), gpu.alloc(nff)
    eps = 1e-5

    def stages(w):
        return [dict(x=x0, ws=[w["q"], w["k"], w["v"]], ys=[y["q"], y["k"], y["v"]]),
                dict(x=y["q"], ws=[w["o"]], ys=[y["o"]]),
                dict(x=y["o"], x2=gamma, prologue=R.CHAIN_X_RMSNORM, eps=eps, ws=[w["gate"], w["up"]], ys=[y["gate"], y["up"]]),
                dict(x=y["gate"], x2=y["up"], prologue=R.CHAIN_X_SILU_MUL, ws=[w["down"]], ys=[y["down"]]),
                dict(x=y["down"], x2=gamma, prologue=R.CHAIN_X_RMSNORM, eps=eps, ws=[w["head"]], ys=[y["head"]])]

    def separate(w):
        gpu.mm_multi(x0, [w["q"], w["k"], w["v"]], [y["q"], y["k"], y["v"]])
        gpu.mm_multi(y["q"], [w["o"]], [y["o"]])
        gpu.rmsnorm_quant_q8k(y["o"], gamma, eps, 1, d, xq, xs)
        gpu.ffn_gu_q8k(xq, xs, w["gate"], w["up"], act)
        gpu.mm_multi(act, [w["down"]], [y["down"]])
        gpu.rmsnorm_quant_q8k(y["down"], gamma, eps, 1, d, xq, xs)
        gpu.mm_q8k_multi(xq, xs, [w["head"]], [y["head"]])

    out = {}
    for tag, fn in (("one_launch", lambda w: gpu.decode_chain(stages(w))), ("separate_launches", separate)):
        fn(sets[0])
        gpu.submit()
        recorded = []
        for w in sets:
            gpu.capture_begin()
            fn(w)
            recorded.append(gpu.capture_end())
        us = _time(gpu, lambda i: recorded[i % len(recorded)].launch(), 200, 10)
        out[tag] = {"us": round(us, 2), "gbs": round(step_bytes / us / 1e3, 1), "hbm_frac": round(step_bytes / us / 8e6, 4)}
        del recorded
    # where the single launch spends its time: per stage, when its first quantizer workgroup had its input (= the rows
    # it depends on were done) and when it had published it, microseconds after the first stage's quantizer started
    tb = gpu.alloc_bytes(8 * 3 * 8)
    gpu.chain_trace(tb)
    gpu.decode_chain(stages(sets[0]))
    gpu.submit()
    gpu.chain_trace(None)
    t = gpu.read(tb, 24, np.uint64).reshape(8, 3).astype(np.float64) / 100.0
    out["one_launch"]["stage_input_arrived_published_us"] = [[round(float(t[s, 1] - t[0, 0]), 2), round(float(t[s, 2] - t[0, 0]), 2)]
                                                             for s in range(5)]
    out["what"] = ("every stage reads the previous stage's output; separate = ojh_mm_multi / ojh_rmsnorm_quant_q8k / "
                   "ojh_ffn_gu_q8k (gate, up and SiLU in one launch) / ojh_mm_q8k_multi, 8 launches; one_launch = "
                   "ojh_decode_chain, bit-identical to them (gate and up stored as well)")
    return out


def extras(gpu, pkg, lin_q) -> dict:
    """Secondary configurations: prefill GEMM, Q8_0 matvec, MoE grouped FFN, Q6_K head verify."""
    synth = pkg.synth
    out = {}
    # ---- prefill dequant-GEMM, Q4_K gate/up (14336x4096) and down (4096x14336), f16 MFMA tile
    gemm = {}
    for name, lin in zip(("gate_up_14336x4096", "down_4096x14336"), lin_q):
        n, k = lin.n, lin.k
        for m in (128, 512, 2048):
            xb = gpu.upload_bytes(synth.to_bf16_bits(synth.normal_f32(m * k, "bench", "gemm_x", m, k)))
            y = gpu.alloc(m * n)
            us = _time(gpu, lambda i: gpu.mm(xb, lin, y, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT), 20, 5)
            tf = 2.0 * m * n * k / us / 1e6
            gemm[f"{name}_M{m}"] = {"us": round(us, 1), "tflops": round(tf, 1), "mfma_frac": round(tf / 2500.0, 4)}
    out["prefill_gemm_q4k"] = {"activations": "bf16 N(0,1), converted to f16 into the tile", "accumulate": "f32",
                               "tile": "v_mfma_f32_32x32x16_f16, weights dequantized straight into the B registers: 256 tokens x 256 rows per workgroup where that fills the chip (M = 2048), 128 x 256 below (gate/up M = 512), 128 x 64 with K split over the workgroup's waves where 256-row tiles are too few (M = 128, down M = 512); "
                                       "weights = binary16 fma(qa, q, qb), the bits of the reference's gemm_mm_q4l",
                               "peak_tflops": 2500.0, "timed": "conversion + zero fill (split-K) + tile", **gemm}
    # ---- the same contraction over Q6_K, Q5_K and Q8_0 weights (the other formats the path names), bf16 in
    for ty, tag, gen in ((pkg.Q6_K, "q6k", synth.q6k_weights), (pkg.Q5_K, "q5k", synth.q5k_weights), (pkg.Q8_0, "q8_0", synth.q80_weights)):
        fam = {}
        for name, (n, k) in (("gate_up_14336x4096", (14336, 4096)), ("down_4096x14336", (4096, 14336))):
            lin = gpu.lin(ty, n, k, gen(n, k, "bench", tag, name))
            for m in (128, 512, 2048):
                xb = gpu.upload_bytes(synth.to_bf16_bits(synth.normal_f32(m * k, "bench", "gemm_x", m, k)))
                y = gpu.alloc(m * n)
                us = _time(gpu, lambda i: gpu.mm(xb, lin, y, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT), 20, 5)
                tf = 2.0 * m * n * k / us / 1e6
                fam[f"{name}_M{m}"] = {"us": round(us, 1), "tflops": round(tf, 1), "mfma_frac": round(tf / 2500.0, 4)}
                del xb, y
            lin.free()
        out[f"prefill_gemm_{tag}"] = {"activations": "bf16 N(0,1), converted to f16 into the tile", "accumulate": "f32",
                                      "peak_tflops": 2500.0, "timed": "conversion + zero fill (split-K) + tile", **fam}
    # ---- the same two matrices in the CPU path's arithmetic (quant_q8k activations, int8 MFMA), f32 in
    i8 = {}
    for name, lin in zip(("gate_up_14336x4096", "down_4096x14336"), lin_q):
        n, k = lin.n, lin.k
        for m in (8, 16, 64, 128, 512, 2048):
            xf = gpu.upload(synth.normal_f32(m * k, "bench", "i8_x", m, k))
            y = gpu.alloc(m * n)
            us = _time(gpu, lambda i: gpu.mm(xf, lin, y, m, act_mode=pkg.ACT_Q8K), 20, 5)
            i8[f"{name}_M{m}"] = {"us": round(us, 1), "tops": round(2.0 * m * n * k / us / 1e6, 1),
                                  "int8_mfma_frac": round(2.0 * m * n * k / us / 1e6 / 5000.0, 4),
                                  "weight_gbs": round(n * (k // 256) * 144 / us / 1e3, 1)}
    out["verify_prefill_q4k_int8"] = {"arithmetic": "quant_q8k activations, int8 x u4 dots on the int8 matrix cores, the CPU "
                                                    "reference's scale algebra (results within 2e-5 of matvec_kq)",
                                      "peak_tops": 5000.0,
                                      "timed": "quantizer + the tile: from 33 tokens (17 where K >= 2 N: down) quantize_q8k_sides + gemm_q8k_q4k_xt{,64} "
                                               "(128-token tiles, scales folded into int8 planes, v_mfma_i32_16x16x64_i8; where the "
                                               "64-row tiles alone leave CUs idle or singly occupied — down up to M = 512 — gemm_q8k_q4k_xt64_sr: K slices "
                                               "summed in slice order by the last to finish); below, "
                                               "gemm_q8k_q4k_mf (down at M = 8: gemm_q8k_q4k_mk)", **i8}
    # ---- the same arithmetic over Q6_K and Q5_K rows (a Q4_K_M / Q5_K_M file mixes them in), f32 in
    for ty, tag, gen in ((pkg.Q6_K, "q6k", synth.q6k_weights), (pkg.Q5_K, "q5k", synth.q5k_weights)):
        fam = {}
        for name, (n, k) in (("gate_up_14336x4096", (14336, 4096)), ("down_4096x14336", (4096, 14336))):
            lin = gpu.lin(ty, n, k, gen(n, k, "bench", tag, name))
            for m in (64, 128, 512):
                xf = gpu.upload(synth.normal_f32(m * k, "bench", "i8_x", m, k))
                y = gpu.alloc(m * n)
                us = _time(gpu, lambda i: gpu.mm(xf, lin, y, m, act_mode=pkg.ACT_Q8K), 20, 5)
                fam[f"{name}_M{m}"] = {"us": round(us, 1), "tops": round(2.0 * m * n * k / us / 1e6, 1),
                                       "int8_mfma_frac": round(2.0 * m * n * k / us / 1e6 / 5000.0, 4)}
                del xf, y
            lin.free()
        out[f"verify_prefill_{tag}_int8"] = {"arithmetic": "quant_q8k activations, integer dots per scale group on the int8 matrix cores "
                                                           f"(v_mfma_i32_32x32x16_i8 per 16 weights of Q6_K, 32x32x32 per 32 of Q5_K), the scale "
                                                           "a 24-bit multiply-add per result: dot_q6k / dot_q5k within 2e-5 of peak",
                                             "peak_tops": 5000.0, "timed": f"quantize_q8k + gemm_q8k_{tag}_gs{{,_sr}}", **fam}
    # ---- speculative verify on the Q4_K output head of the decode step, bf16 activations
    head4 = lin_q[2]
    v4 = {}
    for m in (2, 4, 8, 16):
        xb = gpu.upload_bytes(synth.to_bf16_bits(synth.normal_f32(m * head4.k, "bench", "ver4_x", m)))
        y = gpu.alloc(m * head4.n)
        us = _time(gpu, lambda i: gpu.mm(xb, head4, y, m, x_dtype=pkg.X_BF16), 10, 2)
        b = head4.n * (head4.k // 256) * 144 + m * (2 * head4.k + 4 * head4.n)
        v4[f"M{m}"] = {"us": round(us, 1), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
        del y
    out["verify_q4k_head_128256x4096"] = {"activations": "bf16, quantized per 256 (quant_q8k)",
                                          "kernels": "gemm_q8k_q4k_ml (int8 MFMA, rows copied through LDS)",
                                          "timed": "quantize_q8k_bf16 + the kernel", **v4}
    # ---- config 0: Q8_0 matvec 4096x4096, f32 activations (dot_q80 contract)
    n = k = 4096
    wq8 = [gpu.lin(pkg.Q8_0, n, k, synth.q80_weights(n, k, "bench", "q80")) for _ in range(16)]
    x, y = gpu.upload(synth.normal_f32(k, "bench", "q80x")), gpu.alloc(n)
    us = _time(gpu, lambda i: gpu.mm(x, wq8[i % 16], y), 64, 16)
    b = n * (k // 32) * 34 + 4 * k + 4 * n
    out["q80_gemv_4096x4096"] = {"us": round(us, 2), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
    # the same matrix on the reference GPU decode path's arithmetic: activations quantized per 32, integer dots
    us = _time(gpu, lambda i: gpu.mm(x, wq8[i % 16], y, act_mode=pkg.ACT_Q8_1), 64, 16)
    out["q80_dp4a_gemv_4096x4096"] = {"timed": "quantize_q8_1 + gemv_q80_dp4a", "us": round(us, 2), "gbs": round(b / us / 1e3, 1),
                                      "hbm_frac": round(b / us / 8e6, 4)}
    del wq8
    # the same contract on a tall matrix (rows staged through LDS, activations in registers)
    n = 128256
    wq8 = [gpu.lin(pkg.Q8_0, n, k, synth.q80_weights(n, k, "bench", "q80_head")) for _ in range(2)]
    y = gpu.alloc(n)
    us = _time(gpu, lambda i: gpu.mm(x, wq8[i % 2], y), 20, 3)
    b = n * (k // 32) * 34 + 4 * k + 4 * n
    out["q80_gemv_128256x4096"] = {"us": round(us, 2), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
    del wq8
    # ---- row-int8 weights (K int8 + one f32 scale per row), f32 activations: the reference GPU decoder's `gemv_q8` by name
    gpu.ensure_family("gemv_q8")
    rq = {}
    rng8 = np.random.default_rng(synth.seed_of("bench", "gemv_q8"))
    for name, (n, copies, reps) in (("4096x4096", (4096, 20, 64)), ("128256x4096", (128256, 2, 20))):
        ws = [gpu.upload_bytes(rng8.integers(-127, 128, n * k, dtype=np.int8).view(np.uint8)) for _ in range(copies)]
        sc, y = gpu.upload(np.full(n, 0.01, np.float32)), gpu.alloc(n)
        g, blk = gpu.launch_shape("gemv_q8", k, n)
        us = _time(gpu, lambda i: gpu.dispatch(None, "gemv_q8", [(x, 0), (ws[i % copies], 0), (y, 0), (sc, 0)], [k, n], g, blk), reps, 5)
        b = n * k + 4 * k + 8 * n
        rq[name] = {"us": round(us, 2), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
        del ws
    out["rowq8_gemv_q8"] = {"what": "y[n] = scale[n] * sum_k w[n][k] x[k], w int8 rows streamed from HBM (rotating copies)", **rq}
    # ---- the CPU models' row-int8 matmul (per-token int8 activations, integer dots): 1 .. 8 tokens stream the rows
    # against tokens staged in LDS, batches run on the int8 matrix instruction; the quantizer's launch is in the time
    rm = {}
    n, copies = 14336, 4
    ws = [gpu.upload_bytes(rng8.integers(-127, 128, n * k, dtype=np.int8).view(np.uint8)) for _ in range(copies)]
    sc = gpu.upload(np.full(n, 0.01, np.float32))
    for m in (1, 8, 64, 512, 2048):
        xm, ym = gpu.upload(synth.normal_f32(m * k, "bench", "rowq8x", m)), gpu.alloc(m * n)
        us = _time(gpu, lambda i: gpu.matmul_q8(xm, ws[i % copies], sc, ym, n, k, m), 16, 3)
        b = n * k + 4 * m * k + 4 * m * n + 8 * n
        rm["M%d" % m] = {"us": round(us, 2), "gbs": round(b / us / 1e3, 1), "int8_tops": round(2.0 * m * n * k / us / 1e6, 1),
                         "mfma_frac": round(2.0 * m * n * k / us / 1e6 / 5000.0, 4)}
        del xm, ym
    del ws
    out["rowq8_matmul_14336x4096"] = {"what": "ojh_matmul_q8: quant_rows_i8 + matmul_q8row_{dec,mt_sr,mt,mt128}; int8 rows streamed from HBM (rotating copies)", **rm}
    n = 128256
    # ---- the other block formats on f32 activations (the reference GPU path's contract): a tall head, one token
    fr = {}
    for ty, tag in ((pkg.IQ4_XS, "iq4xs"), (pkg.IQ4_NL, "iq4nl"), (pkg.Q3_K, "q3k"), (pkg.Q2_K, "q2k"), (pkg.Q5_0, "q50"),
                    (pkg.IQ3_S, "iq3s"), (pkg.IQ2_XXS, "iq2xxs")):
        wf = [gpu.lin(ty, n, k, synth.weights(ty, n, k, "bench", tag, "head")) for _ in range(2)]
        us = _time(gpu, lambda i: gpu.mm(x, wf[i % 2], y, act_mode=pkg.ACT_FLOAT), 20, 3)
        b = pkg.row_bytes(ty, k) * n + 4 * k + 4 * n
        fr[tag] = {"us": round(us, 2), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
        del wf
    out["float_rows_gemv_128256x4096"] = {"activations": "f32", "kernels": "gemv_nat_<fmt>_px", **fr}
    # ---- the same formats against a batch (f32 in, OJH_ACT_AUTO): the f16 tile through the formats' own loaders, or the
    # decode pass into f16 scratch + the plain-f16 tile for those without one
    fb = {}
    nb, kb = 14336, 4096
    for ty, tag in ((pkg.IQ4_XS, "iq4xs"), (pkg.Q4_0, "q40"), (pkg.Q5_1, "q51"), (pkg.MXFP4, "mxfp4"), (pkg.Q3_K, "q3k"),
                    (pkg.IQ3_S, "iq3s")):
        wf = [gpu.lin(ty, nb, kb, synth.weights(ty, nb, kb, "bench", tag, "batch")) for _ in range(2)]
        for m in (16, 128, 512):
            xb, yb = gpu.upload(synth.normal_f32(m * kb, "bench", "xb", m)), gpu.alloc(m * nb)
            us = _time(gpu, lambda i: gpu.mm(xb, wf[i % 2], yb, m), 10, 2)
            fb[f"{tag}_M{m}"] = {"us": round(us, 1), "mfma_frac": round(2.0 * m * nb * kb / us / 1e6 / 2500.0, 4)}
        del wf
    out["float_rows_batch_14336x4096"] = {"activations": "f32 -> f16", "kernels": "gemm_mm_<fmt>{,_m128}{,_sk} (IQ4_NL / IQ4_XS, Q4_0 .. Q5_1, MXFP4, Q2_K; Q3_K up to 128 tokens) or dequant_<fmt>_f16 + gemm_mm_f16_m128{,_sk} (Q3_K beyond, the grid codebooks)", **fb}
    # IQ2_XXS as the CPU path multiplies it: int8 activations per 256, integer dots (dot_iq2xxs_q8k)
    wf = [gpu.lin(pkg.IQ2_XXS, n, k, synth.weights(pkg.IQ2_XXS, n, k, "bench", "iq2xxs", "head")) for _ in range(2)]
    us = _time(gpu, lambda i: gpu.mm(x, wf[i % 2], y), 20, 3)
    b = pkg.row_bytes(pkg.IQ2_XXS, k) * n + 4 * k + 4 * n
    out["iq2xxs_q8k_gemv_128256x4096"] = {"timed": "quantize_q8k + gemv_q8k_iq2xxs_wide", "us": round(us, 2),
                                          "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
    del wf
    # ---- one FFN block of a decode layer with the fused epilogues: rmsnorm+quantize, gate/up+SiLU,
    # quantize, down accumulated onto the residual (4 launches, recorded and replayed)
    d, nff = 4096, 14336
    blocks = []
    for c in range(4):
        blocks.append((gpu.lin(pkg.Q4_K, nff, d, synth.q4k_weights(nff, d, "bench", "ffn_g", c)),
                       gpu.lin(pkg.Q4_K, nff, d, synth.q4k_weights(nff, d, "bench", "ffn_u", c)),
                       gpu.lin(pkg.Q4_K, d, nff, synth.q4k_weights(d, nff, "bench", "ffn_d", c))))
    xr = gpu.upload(synth.normal_f32(d, "bench", "ffn_x"))
    gm = gpu.upload(np.ones(d, np.float32))
    xq_, xs_ = gpu.alloc_bytes(d), gpu.alloc(d // 256)
    aq_, as__ = gpu.alloc_bytes(nff), gpu.alloc(nff // 256)
    act_ = gpu.alloc(nff)
    graphs = []
    for g_, u_, d_ in blocks:
        gpu.capture_begin()
        gpu.rmsnorm_quant_q8k(xr, gm, 1e-5, 1, d, xq_, xs_)
        gpu.ffn_gu_q8k(xq_, xs_, g_, u_, act_)
        gpu.quant_q8k(act_, 1, nff, aq_, as__)
        gpu.mm_q8k(aq_, as__, d_, xr, accum=True)
        graphs.append(gpu.capture_end())
    us = _time(gpu, lambda i: graphs[i % 4].launch(), 40, 8)
    b = 3 * nff * (d // 256) * 144
    out["ffn_block_q4k_14336x4096"] = {"launches": "rmsnorm_q8k, ffn_gu_q8k_q4k, quantize_q8k, gemv_q8k_q4k_accum",
                                       "us": round(us, 2), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4)}
    del blocks, graphs
    # ---- MoE: 128 experts, top-8, hidden 2048, expert FFN 768, Q4_K; tokens 1 / 16 / 256
    E, ksel, d, nff = 128, 8, 2048, 768
    gate = gpu.lin(pkg.Q4_K, E * nff, d, synth.q4k_weights(E * nff, d, "bench", "moe_gate"))
    up = gpu.lin(pkg.Q4_K, E * nff, d, synth.q4k_weights(E * nff, d, "bench", "moe_up"))
    down = gpu.lin(pkg.Q4_K, E * d, nff, synth.q4k_weights(E * d, nff, "bench", "moe_down"))
    moe = {}
    for T in (1, 16, 256):
        lg = gpu.upload(synth.normal_f32(T * E, "bench", "moe_lg", T))
        xt, yt = gpu.upload(synth.normal_f32(T * d, "bench", "moe_x", T)), gpu.alloc(T * d)
        idx, wgt = gpu.alloc_bytes(T * ksel * 4), gpu.alloc(T * ksel)

        def layer(i):
            gpu.moe_ffn_routed(xt, T, d, nff, E, ksel, lg, idx, wgt, gate, up, down, yt)
        us = _time(gpu, layer, 20, 3)
        distinct = len(np.unique(gpu.read(idx, T * ksel, np.uint32)))
        b = distinct * 3 * nff * (d // 256) * 144 + T * d * 8
        fl = 2.0 * T * ksel * 3 * nff * d
        moe[f"T{T}"] = {"us": round(us, 1), "distinct_experts": distinct, "gbs": round(b / us / 1e3, 1),
                        "tflops": round(fl / us / 1e6, 2)}
    out["moe_ffn_q4k_128x_top8"] = {"timed": "router + expert FFN, ojh_moe_ffn_routed (T <= 2: gate/up, the router inside it, and down launches addressed by assignment; above: router, quantize + group in one launch, gate/up, quantize, down, combine; T = 256 on int8 MFMA, moe_{gu,down}_q4k_mt, 32 assignments per staged pass)", **moe}
    del gate, up, down
    # the same layer with finer expert tensors in a prefill batch: Q6_K down (int8 matrix tile per expert from 10
    # assignments per expert) and all-Q8_0 experts (grouped f16 matrix tile from 4 per expert)
    mixed = {}
    gate = gpu.lin(pkg.Q4_K, E * nff, d, synth.q4k_weights(E * nff, d, "bench", "moe_gate"))
    up = gpu.lin(pkg.Q4_K, E * nff, d, synth.q4k_weights(E * nff, d, "bench", "moe_up"))
    down6 = gpu.lin(pkg.Q6_K, E * d, nff, synth.q6k_weights(E * d, nff, "bench", "moe_down6"))
    g8 = gpu.lin(pkg.Q8_0, E * nff, d, synth.q80_weights(E * nff, d, "bench", "moe_gate8"))
    u8 = gpu.lin(pkg.Q8_0, E * nff, d, synth.q80_weights(E * nff, d, "bench", "moe_up8"))
    d8 = gpu.lin(pkg.Q8_0, E * d, nff, synth.q80_weights(E * d, nff, "bench", "moe_down8"))
    # (IQ4_XS gate / up with IQ4_NL down, the mix the reference's streamed models ship in: the grouped tile's own loaders)
    gx = gpu.lin(pkg.IQ4_XS, E * nff, d, synth.weights(pkg.IQ4_XS, E * nff, d, "bench", "moe_gatex"))
    ux = gpu.lin(pkg.IQ4_XS, E * nff, d, synth.weights(pkg.IQ4_XS, E * nff, d, "bench", "moe_upx"))
    dn = gpu.lin(pkg.IQ4_NL, E * d, nff, synth.weights(pkg.IQ4_NL, E * d, nff, "bench", "moe_downn"))
    for T in (256, 1024):
        lg = gpu.upload(synth.normal_f32(T * E, "bench", "moe_lg", T))
        xt, yt = gpu.upload(synth.normal_f32(T * d, "bench", "moe_x", T)), gpu.alloc(T * d)
        idx, wgt = gpu.alloc_bytes(T * ksel * 4), gpu.alloc(T * ksel)
        fl = 2.0 * T * ksel * 3 * nff * d
        for tag, (a, b_, c) in (("q4k_gate_up_q6k_down", (gate, up, down6)), ("q8_0", (g8, u8, d8)),
                                ("iq4xs_gate_up_iq4nl_down", (gx, ux, dn))):
            us = _time(gpu, lambda i: gpu.moe_ffn_routed(xt, T, d, nff, E, ksel, lg, idx, wgt, a, b_, c, yt), 10, 2)
            mixed[f"{tag}_T{T}"] = {"us": round(us, 1), "tflops": round(fl / us / 1e6, 2)}
    out["moe_ffn_other_formats_128x_top8"] = {"timed": "router + expert FFN, ojh_moe_ffn_routed", **mixed}
    del gate, up, down6, g8, u8, d8
    # ---- speculative verify on a Q6_K output head 151936 x 4096, bf16 activations
    n, k = 151936, 4096
    head = gpu.lin(pkg.Q6_K, n, k, synth.q6k_weights(n, k, "bench", "q6k_head"))
    ver = {}
    for m in (1, 2, 4, 8, 16):
        xb = gpu.upload_bytes(synth.to_bf16_bits(synth.normal_f32(m * k, "bench", "ver_x", m)))
        y = gpu.alloc(m * n)
        us = _time(gpu, lambda i: gpu.mm(xb, head, y, m, x_dtype=pkg.X_BF16), 10, 2)
        b = n * (k // 256) * 210 + m * (2 * k + 4 * n)
        ver[f"M{m}"] = {"us": round(us, 1), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 8e6, 4),
                        "tflops": round(2.0 * m * n * k / us / 1e6, 2)}
    out["verify_q6k_head_151936x4096"] = {"activations": "bf16, quantized per 256 (quant_q8k)",
                                          "kernels": "M1 gemv_q8k_q6k_px, M2-16 gemv_q8k_q6k_ml (int8 MFMA, rows copied through LDS)",
                                          "timed": "quantize_q8k_bf16 + the kernel", **ver}
    return out


def cpu_baseline(host, dims) -> dict:
    """The CPU oracle's `matvec_kq` (restatement of crates/ojas-cpu/src/cpu_math.rs:1145-1189)
    timed on this machine's host cores over a bounded sample of the same workload."""
    orc = entry.load_oracle()
    threads = min(os.cpu_count() or 1, 16)
    sample = ["q", "gate", "down"]
    x = {4096: np.random.default_rng(1).standard_normal(4096).astype(np.float32),
         14336: np.random.default_rng(2).standard_normal(14336).astype(np.float32)}
    total_b, total_s, reps = 0, 0.0, 0
    t_end = time.time() + 12.0
    for name in sample:  # warm the page cache / thread start-up
        n, k = dims[name]
        orc.matvec_kq(host[name], Q4_K, n, k, x[k], threads)
    while time.time() < t_end and reps < 40:
        for name in sample:
            n, k = dims[name]
            t = time.perf_counter()
            orc.matvec_kq(host[name], Q4_K, n, k, x[k], threads)
            total_s += time.perf_counter() - t
            total_b += algorithmic_bytes(n, k)
        reps += 1
    t = time.perf_counter()
    n, k = dims["q"]
    orc.matvec_kq(host["q"], Q4_K, n, k, x[k], 1)
    one_thread_gbs = algorithmic_bytes(n, k) / (time.perf_counter() - t) / 1e9
    return {"value": round(total_b / total_s / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{reps} passes over the q (4096x4096), gate (14336x4096) and down (4096x14336) "
                      f"Q4_K matvecs, C restatement of matvec_kq, 8-row work stealing",
            "one_thread_gbs": round(one_thread_gbs, 2)}


if __name__ == "__main__":
    sys.exit(main())
