#!/usr/bin/env python3
"""Benchmark of the weight-only quantized linear path on one MI355X.

One "step" is one weight_only_linear call at M=1 on the headline shape
(int4, group 128, K=4096, N=11008, bf16 activations): the bandwidth-bound
decode GEMV.  The timed region holds exactly --steps such calls, captured into
one HIP graph so the host's launch rate does not enter, rotating over enough
distinct copies of the packed weight that neither L2 nor the 256 MB Infinity
Cache can serve a repeat.  A second region times the compute-bound prefill
GEMM (M=2048, int8 per-channel, K=4096, N=12288) and is reported under
"prefill".  The CPU baseline (oracle quantize + dequantize + fp32 matmul on the
host cores) is timed on rank 0 on the same arrays.

Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TF = 2500.0   # MI355X dense bf16 MFMA, published
MFMA_INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA, published

DECODE = dict(M=1, K=4096, N=11008, bits=4, group_size=128, dtype="bfloat16")
PREFILL = dict(M=2048, K=4096, N=12288, bits=8, group_size=-1, dtype="bfloat16")


def _load_traffic():
    """HBM bytes per launch measured with rocprofv3 --pmc (see profiles/)."""
    p = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(p):
        with open(p) as f:
            return json.load(f)
    return {}


def _quantize(torch, Q, w, bits, group_size):
    algo = "weight_only_int8" if bits == 8 else "weight_only_int4"
    return Q.weight_quantize(w, algo=algo, group_size=group_size)


def _time_graph(torch, fn, steps, warmup):
    """Run fn(i) warmup times eagerly, then capture steps calls into one graph
    and time its replay with events on the launching stream.  The graph is
    replayed untimed first (graph upload), as often as it takes to cover the
    warm-up count in graph form too: the clocks need a few milliseconds of
    load to settle, and eager launches of a 6 us kernel do not load the GPU."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(steps):
            fn(warmup + i)
    torch.cuda.synchronize()
    for _ in range(max(1, -(-warmup // steps))):
        g.replay()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / 1e3  # seconds for `steps` launches


def _time_eager(torch, fn, steps, warmup):
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(warmup + i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / 1e3


def cpu_baseline(np, torch, H, w_bits, x_bits, cfg, budget_s=25.0):
    """Oracle quantize (single thread, like the reference's CPU kernel) +
    dequantize to fp32 + fp32 matmul (torch CPU BLAS, all cores), on a bounded
    sample: the first N_s output columns of the decode weight."""
    O = H.O
    dt = H.BF16 if cfg["dtype"] == "bfloat16" else H.F16
    K, N, bits, g = cfg["K"], cfg["N"], cfg["bits"], cfg["group_size"]
    n_s = min(N, 2048)
    wb = np.ascontiguousarray(w_bits[:, :n_s])
    t0 = time.perf_counter()
    codes, scale = O.weight_quantize(wb, dt, bits, g)
    t_q = time.perf_counter() - t0
    reps = 0
    t_dq = t_mm = 0.0
    x32 = torch.from_numpy(H.bits_to_f32(x_bits, dt))
    cores = torch.get_num_threads()
    t_start = time.perf_counter()
    while reps < 3 or (time.perf_counter() - t_start < min(budget_s, 10.0) and reps < 50):
        t0 = time.perf_counter()
        w32, _ = O.dequantize(codes, scale, dt, bits, g)
        t1 = time.perf_counter()
        y = x32 @ torch.from_numpy(w32)
        t2 = time.perf_counter()
        t_dq += t1 - t0
        t_mm += t2 - t1
        reps += 1
    t_dq /= reps
    t_mm /= reps
    wbytes = K * n_s * bits / 8
    return {
        "value": round(wbytes / (t_dq + t_mm) / 1e9, 4),
        "unit": "GB/s",
        "cores": int(cores),
        "kind": "port",
        "sample": "first %d of %d output columns of the decode weight (K=%d, int%d, group %d), M=1; "
                  "per call: dequantize %.2f ms (1 thread) + fp32 matmul %.2f ms (%d threads); "
                  "one-time quantize %.1f ms (1 thread); %d repetitions"
                  % (n_s, N, K, bits, g, t_dq * 1e3, t_mm * 1e3, cores, t_q * 1e3, reps),
    }, (codes, scale, n_s)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--prefill-steps", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-llm-int8", action="store_true", help="skip the llm_int8_linear timing")
    ap.add_argument("--eager", action="store_true", help="time eager launches instead of a graph")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 256 MiB device copies (a known-size kernel to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings with)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path has no collectives); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import helpers as H
    from paddle_amd.nn import quant as Q

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------- decode (the headline metric) ----------------
    c = DECODE
    dt = H.BF16
    w_bits = H.make_weight(c["K"], c["N"], dt, seed=1234)
    x_bits = H.make_act(c["M"], c["K"], dt, seed=1235)
    w = H.bits_to_torch(w_bits, dt, dev)
    x = H.bits_to_torch(x_bits, dt, dev)
    codes, scale = _quantize(torch, Q, w, c["bits"], c["group_size"])
    wbytes = c["K"] * c["N"] * c["bits"] // 8
    sbytes = scale.numel() * 2
    total_bytes = wbytes + sbytes + 2 * (c["M"] * c["K"] + c["M"] * c["N"])
    ncopies = max(2, -(-768 * 1024 * 1024 // wbytes))  # > 3x the Infinity Cache
    copies = [codes.clone() for _ in range(ncopies)]
    scales = [scale.clone() for _ in range(ncopies)]
    wd = "int8" if c["bits"] == 8 else "int4"

    def decode_step(i):
        j = i % ncopies
        return Q.weight_only_linear(x, copies[j], None, scales[j], wd, None, c["group_size"])

    timer = _time_eager if args.eager else _time_graph
    t_dec = timer(torch, decode_step, args.steps, args.warmup)
    dec_s = t_dec / args.steps
    dec_gbs = wbytes / dec_s / 1e9

    # parity gate on the measured configuration
    y = decode_step(0)
    torch.cuda.synchronize()

    # the floor of this launch shape on this machine: the same weight copies read
    # by a kernel of the decode kernel's shape that computes nothing
    from paddle_amd import _lib
    floor_out = torch.empty(c["N"] // 16 * 8, dtype=torch.int32, device=dev)

    def floor_step(i):
        _lib.check(_lib.lib.wol_read_floor(copies[i % ncopies].data_ptr(), c["K"], c["N"], c["bits"],
                                           floor_out.data_ptr(), torch.cuda.current_stream().cuda_stream))

    floor_s = timer(torch, floor_step, args.steps, args.warmup) / args.steps

    # ---------------- prefill ----------------
    p = PREFILL
    pw_bits = H.make_weight(p["K"], p["N"], dt, seed=1236)
    px = H.bits_to_torch(H.make_act(p["M"], p["K"], dt, seed=1237), dt, dev)
    pcodes, pscale = _quantize(torch, Q, H.bits_to_torch(pw_bits, dt, dev), p["bits"], p["group_size"])

    def prefill_step(i):
        return Q.weight_only_linear(px, pcodes, None, pscale, "int8", None, p["group_size"])

    t_pre = timer(torch, prefill_step, args.prefill_steps, args.warmup)
    pre_s = t_pre / args.prefill_steps
    flops = 2.0 * p["M"] * p["K"] * p["N"]
    pre_tf = flops / pre_s / 1e12

    # ---------------- llm_int8_linear on the prefill shape ----------------
    # the sibling op on the same weight (algo="llm.int8"): activations N(0,1)
    # with eight columns scaled x12, so that the outlier branch runs
    llm = None
    if not args.no_llm_int8:
        lw, lscale = Q.weight_quantize(H.bits_to_torch(pw_bits, dt, dev), algo="llm.int8")
        lx = px.clone()
        lx[:, 100:3700:450] *= 12.0

        def llm_step(i):
            return Q.llm_int8_linear(lx, lw, None, lscale, 6.0)

        llm_s = timer(torch, llm_step, args.prefill_steps, args.warmup) / args.prefill_steps
        llm_tops = flops / llm_s / 1e12
        llm = {
            "workload": "llm_int8_linear M=2048, K=4096 N=12288, bf16 x with 8 outlier columns, threshold 6.0; "
                        "all stages of one call (row ranges, activation codes, int8 GEMM with the merge)",
            "value": round(llm_tops, 2),
            "unit": "TOP/s",
            "ms_per_step": round(llm_s * 1e3, 4),
            "steps": args.prefill_steps,
            "roofline": {"bound": "mfma", "achieved": round(llm_tops, 2), "peak": MFMA_INT8_PEAK_TOPS,
                         "unit": "TOP/s", "frac": round(llm_tops / MFMA_INT8_PEAK_TOPS, 4),
                         "traffic": _load_traffic().get("llm_int8_gemm_bytes_per_launch"),
                         "kernel": "wol::llm_gemm_kernel<1, 2, 4, 4, 2, 128, 2, false> (256x256 tiles on 8192 columns) "
                                   "+ <1, 2, 4, 2, 2, 128, 3, false> (128x256 tiles on the rest), "
                                   "v_mfma_i32_32x32x32_i8"},
        }

    # ---------------- CPU baseline + parity of the decode output ----------------
    cpu = None
    parity = {}
    if not args.no_cpu_baseline:
        cpu, (ocodes, oscale, n_s) = cpu_baseline(np, torch, H, w_bits, x_bits, c)
        O = H.O
        o32, oT = O.linear(x_bits, ocodes, oscale, None, dt, c["bits"], c["group_size"])
        got = H.bits_to_f32(H.torch_to_bits(y), dt)[:, :n_s]
        parity["decode_rel_l2_vs_oracle"] = H.rel_l2(got, H.bits_to_f32(oT, dt))
        gs = H.torch_to_bits(scale)[:, :n_s]
        parity["scales_bit_exact"] = bool(np.array_equal(gs, oscale))

    traffic = _load_traffic()
    out = {
        "metric": "weight-only linear GB/s on weight bytes at M=1 (decode GEMV)",
        "value": round(dec_gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dec_s * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "decode GEMV M=1, int4 group_size=128, K=4096 N=11008, bf16 x, no bias; "
                        "%d rotating weight copies; %s" % (ncopies, "eager launches" if args.eager else "one HIP graph of all steps"),
            "prefill_workload": "GEMM M=2048, int8 per-channel, K=4096 N=12288, bf16 x",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(dec_gbs, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dec_gbs / HBM_PEAK_GBS, 4),
            "traffic": traffic.get("decode_bytes_per_launch"),
            "kernel": "wol::stream_kernel<1, 4, 1, 1, 8, 1, 1, true>",
            "algorithmic_bytes_per_launch": wbytes,
            "total_bytes_per_launch": total_bytes,
            "read_floor": {
                "what": "wol_read_floor: the same weight copies read by a kernel of the same launch shape "
                        "that computes nothing (no scales, activations, MFMAs or output)",
                "ms_per_step": round(floor_s * 1e3, 6),
                "GB/s": round(wbytes / floor_s / 1e9, 1),
                "decode_over_floor": round(dec_s / floor_s, 3),
            },
        },
        "prefill": {
            "value": round(pre_tf, 2),
            "unit": "TFLOP/s",
            "ms_per_step": round(pre_s * 1e3, 4),
            "steps": args.prefill_steps,
            "roofline": {
                "bound": "mfma",
                "achieved": round(pre_tf, 2),
                "peak": MFMA_BF16_PEAK_TF,
                "unit": "TFLOP/s",
                "frac": round(pre_tf / MFMA_BF16_PEAK_TF, 4),
                "traffic": traffic.get("prefill_bytes_per_launch"),
                "kernel": "wol::gemm_dma_kernel<1, 8, 0, false, 2, 4, 4, 2, 3> (256x256 tiles on the columns that fill whole rounds of the 256 CUs) + <1, 8, 0, false, 2, 4, 4, 1, 3> (256x128 tiles on the rest)",
            },
        },
        "llm_int8": llm,
        "cpu_baseline": cpu,
        "parity": parity,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
