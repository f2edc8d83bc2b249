#!/usr/bin/env python3
"""Benchmark of the weight-only quantized linear path on one MI355X.

One "step" is one weight_only_linear call at M=1 on the headline shape
(int4, group 128, K=4096, N=11008, bf16 activations): the bandwidth-bound
decode GEMV.  --steps such calls are captured into one HIP graph, so the
host's launch rate does not enter, rotating over enough distinct copies of the
packed weight that neither L2 nor the 256 MB Infinity Cache can serve a
repeat.  Whatever --steps/--warmup say, the graph is replayed untimed until at
least 400 launches and 50 ms of load have run (the clocks need that to
settle), then replayed REPLAYS times, each replay between its own pair of
events on the launching stream; ms_per_step is the MEDIAN replay divided by
--steps (the minimum is reported beside it).

Beside the headline the line carries
  prefill    the compute-bound GEMM (M=2048, int8 per-channel, K=4096,
             N=12288) with an in-run ceiling: a register-only MFMA loop;
  configs    one entry per configuration of BASELINE.json and row count, the
             last one the 32-layer decoder stack as a sequence (decode steps
             at M=8, one prefill chunk at M=1024);
  llm_int8   the sibling op on the prefill shape;
  cpu_baseline  the CPU oracle (quantize, dequantize) + fp32 BLAS matmul on
             the host cores, on a bounded sample;
  parity     the measured outputs against the oracle.  A parity failure makes
             the run exit non-zero: no throughput is published for wrong results.

Prints ONE JSON line.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TF = 2500.0   # MI355X dense bf16 MFMA, published
MFMA_INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA, published
REPLAYS = 7                  # timed replays of every graph (median and minimum are reported)

DECODE = dict(M=1, K=4096, N=11008, bits=4, group_size=128, dtype="bfloat16")
PREFILL = dict(M=2048, K=4096, N=12288, bits=8, group_size=-1, dtype="bfloat16")
REL_L2_BAR = 1e-3


def _load_traffic():
    """HBM bytes per launch measured with rocprofv3 --pmc (see profiles/)."""
    p = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(p):
        with open(p) as f:
            return json.load(f)
    return {}


def _quantize(Q, w, bits, group_size):
    algo = "weight_only_int8" if bits == 8 else "weight_only_int4"
    return Q.weight_quantize(w, algo=algo, group_size=group_size)


EAGER = False  # --eager: every leg launches eagerly (for counter collection, which needs plain dispatches)


def time_graph(torch, fn, launches, warm_launches=400, warm_ms=50.0, replays=REPLAYS, eager=False, whole=None):
    """fn(i) enqueues launch i on the current stream.  Captures `launches`
    calls into one HIP graph, replays it untimed until both warm-up thresholds
    are met, then times `replays` replays one by one (events on the current
    stream).  Returns (median, minimum) seconds per replay.  whole: a callable
    that enqueues all `launches` launches itself (it may fork onto other
    streams and must join back into the current one)."""
    def all_launches():
        if whole is not None:
            whole()
        else:
            for i in range(launches):
                fn(i)

    for i in range(3):
        fn(i)
    torch.cuda.synchronize()
    if eager or EAGER:
        run = all_launches
    else:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            all_launches()
        run = g.replay
    torch.cuda.synchronize()
    done, batch = 0, 1
    t0 = time.perf_counter()
    while True:
        tb = time.perf_counter()
        for _ in range(batch):
            run()
        torch.cuda.synchronize()
        done += launches * batch
        now = time.perf_counter()
        if done >= warm_launches and (now - t0) * 1e3 >= warm_ms:
            break
        # replays go out in batches of about 5 ms so that the GPU stays loaded between host synchronisations
        batch = int(min(256, max(1, 5e-3 / max((now - tb) / batch, 1e-6))))
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(replays)]
    torch.cuda.synchronize()
    for e0, e1 in ev:
        e0.record()
        run()
        e1.record()
    torch.cuda.synchronize()
    ts = [e0.elapsed_time(e1) / 1e3 for e0, e1 in ev]
    return statistics.median(ts), min(ts)


def _plan(_lib, M, K, N, bits, g):
    """The kernel path wol_linear takes for a problem, as the library describes it."""
    import ctypes

    if not hasattr(_lib.lib, "wol_linear_plan"):
        return None
    buf = ctypes.create_string_buffer(256)
    ws = _lib.lib.wol_linear_workspace(M, K, N, bits, g)
    if _lib.lib.wol_linear_plan(M, K, N, bits, g, ws, buf, 256) != 0:
        return None
    return buf.value.decode()


def _device_weight(torch, K, N, tdtype, seed, dev, outlier_cols=0.0):
    """W ~ N(0, 0.02) generated on the device (the configurations' weights are
    too many for the host generator), optionally with a fraction of the columns
    scaled x20, cast to T."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    w = torch.randn((K, N), generator=gen, device=dev, dtype=torch.float32) * 0.02
    if outlier_cols > 0:
        n = int(-(-outlier_cols * N // 1))
        cols = torch.randperm(N, generator=gen, device=dev)[:n]
        w[:, cols] *= 20.0
    return w.to(tdtype)


def bench_configs(torch, Q, _lib, dev, quick):
    """One entry per BASELINE configuration and row count."""
    bf16, f16 = torch.bfloat16, torch.float16
    cases = [
        ("c1", 4096, 4096, 8, -1, bf16, (1,), 0.0, False),
        ("c2", 4096, 11008, 4, -1, bf16, (1, 4, 16), 0.0, True),
        ("c2", 11008, 4096, 4, -1, bf16, (1, 4, 16), 0.0, True),
        ("north-star decode", 4096, 11008, 4, 128, bf16, (1,), 0.0, False),
        ("c3", 8192, 28672, 4, 128, f16, (1, 8, 32, 64), 0.01, False),
        ("c4", 4096, 12288, 8, -1, bf16, (512, 2048, 8192), 0.0, False),
    ]
    out = []
    for ci, (name, K, N, bits, g, tdt, Ms, outl, with_bias) in enumerate(cases):
        w = _device_weight(torch, K, N, tdt, 2000 + ci, dev, outl)
        codes, scale = _quantize(Q, w, bits, g)
        del w
        wbytes = K * N * bits // 8
        ncopies = max(2, -(-640 * 1024 * 1024 // wbytes))
        copies = [codes.clone() for _ in range(ncopies)]
        scales = [scale.clone() for _ in range(ncopies)]
        bias = (torch.randn(N, device=dev) * 0.01).to(tdt) if with_bias else None
        wd = "int8" if bits == 8 else "int4"
        for M in Ms:
            x = torch.randn((M, K), device=dev, dtype=torch.float32).to(tdt)

            def step(i, x=x):
                j = i % ncopies
                return Q.weight_only_linear(x, copies[j], bias, scales[j], wd, None, g)

            flops = 2.0 * M * K * N
            est_us = max(wbytes / 4e6, flops / 1.0e9)  # rough: 4 TB/s, 1 PFLOP/s
            launches = int(min(200, max(10, 2000.0 / est_us)))
            if quick:
                launches = min(launches, 20)
            med, mn = time_graph(torch, step, launches, warm_launches=2 * launches,
                                 warm_ms=10.0 if quick else 30.0, replays=5)
            us, us_min = med / launches * 1e6, mn / launches * 1e6
            e = {"config": name, "M": M, "K": K, "N": N, "weights": "int%d" % bits, "group_size": g,
                 "dtype": "bf16" if tdt == bf16 else "f16", "bias": with_bias,
                 "us": round(us, 3), "us_min": round(us_min, 3), "launches_per_replay": launches,
                 "weight_copies": ncopies}
            if M <= 64:
                gbs = wbytes / us / 1e3
                e.update({"bound": "hbm", "achieved": round(gbs, 1), "unit": "GB/s",
                          "frac": round(gbs / HBM_PEAK_GBS, 4)})
            else:
                tf = flops / us / 1e6
                e.update({"bound": "mfma", "achieved": round(tf, 1), "unit": "TFLOP/s",
                          "frac": round(tf / MFMA_BF16_PEAK_TF, 4)})
            e["path"] = _plan(_lib, M, K, N, bits, g)
            out.append(e)
            del x
        del copies, scales, codes, scale
        torch.cuda.empty_cache()
    return out


def bench_decoder_stack(torch, Q, _lib, dev, quick):
    """BASELINE configuration 5 as the sequence it describes: the four linears
    of 32 LLaMA-7B decoder layers (int8, group 64, every layer its own random
    weights), run back to back as decode steps at batch 8 and as one prefill
    chunk of 1024 tokens.  Attention, norms and the rest of the model are not
    part of this path; every linear reads a fixed random input of its width."""
    layers = 8 if quick else 32
    shapes = [("qkv", 4096, 12288), ("o", 4096, 4096), ("gate_up", 4096, 22016), ("down", 11008, 4096)]
    g, bf16 = 64, torch.bfloat16
    weights = []
    for layer in range(layers):
        for i, (_, K, N) in enumerate(shapes):
            w = _device_weight(torch, K, N, bf16, 1234 + layer * 4 + i, dev)
            weights.append((K, N) + tuple(_quantize(Q, w, 8, g)))
            del w
    wbytes = sum(K * N for K, N, _, _ in weights)
    res = {"layers": layers, "linears_per_layer": [s[0] for s in shapes], "weights": "int8", "group_size": g,
           "dtype": "bf16", "weight_bytes_per_step": wbytes}
    for tag, M, reps in (("decode_M8", 8, 4), ("prefill_M1024", 1024, 1)):
        xs = {K: torch.randn((M, K), device=dev, dtype=torch.float32).to(bf16) for K in (4096, 11008)}

        def step(_i, xs=xs):
            for K, N, codes, scale in weights:
                Q.weight_only_linear(xs[K], codes, None, scale, "int8", None, g)

        med, mn = time_graph(torch, step, reps, warm_launches=2 * reps, warm_ms=20.0, replays=5)
        ms, ms_min = med / reps * 1e3, mn / reps * 1e3
        flops = 2.0 * M * wbytes
        r = {"M": M, "ms_per_step": round(ms, 4), "ms_per_step_min": round(ms_min, 4),
             "launches_per_step": len(weights)}
        if M <= 64:
            ideal = wbytes / (HBM_PEAK_GBS * 1e9) * 1e3
            r.update({"bound": "hbm", "achieved": round(wbytes / ms / 1e6, 1), "unit": "GB/s",
                      "ideal_ms": round(ideal, 4), "frac": round(ideal / ms, 4)})
        else:
            ideal = flops / (MFMA_BF16_PEAK_TF * 1e12) * 1e3
            r.update({"bound": "mfma", "achieved": round(flops / ms / 1e9, 1), "unit": "TFLOP/s",
                      "ideal_ms": round(ideal, 4), "frac": round(ideal / ms, 4)})
        r["paths"] = {s[0]: _plan(_lib, M, s[1], s[2], 8, g) for s in shapes}
        res[tag] = r
    return res


def bench_linear_grad(torch, np, Q, _lib, H, dev, quick, failures):
    """weight_only_linear_grad on the prefill weight shape (int8 per-channel,
    K = N = 4096, bf16): wol_linear_grad (scale preparation, out_grad
    preparation and the MFMA product, three launches) beside the reference's
    composition (weight_dequantize to T, then the library GEMM; torch.matmul
    stands in for phi::MatmulKernel, both call hipBLASLt).  The composition is
    only timed for comparison; a sample of the kernel's result is checked
    against the oracle."""
    K = N = 4096
    bits, g, bf16, dt = 8, -1, torch.bfloat16, H.BF16
    w = _device_weight(torch, K, N, bf16, 77, dev)
    codes, scale = _quantize(Q, w, bits, g)
    del w
    rows = []
    for M in ((2048,) if quick else (512, 2048, 8192)):
        go = torch.randn((M, N), device=dev, dtype=torch.float32).to(bf16)
        out = torch.empty((M, K), device=dev, dtype=bf16)
        wsb = _lib.lib.wol_linear_grad_workspace(M, K, N, bits, g)
        ws = torch.empty(wsb, dtype=torch.uint8, device=dev)

        def step(_i):
            _lib.check(_lib.lib.wol_linear_grad(go.data_ptr(), codes.data_ptr(), scale.data_ptr(), _lib.DTYPE_BF16, M, K,
                                                N, bits, g, out.data_ptr(), ws.data_ptr(), wsb,
                                                torch.cuda.current_stream().cuda_stream))

        def comp(_i):
            wdq = Q.weight_dequantize(codes, scale, algo="weight_only_int8", out_dtype="bfloat16", group_size=g)
            return torch.matmul(go, wdq.t())

        n = 10
        med, mn = time_graph(torch, step, n, warm_launches=40, warm_ms=30.0, replays=5)
        cmed, _ = time_graph(torch, comp, n, warm_launches=40, warm_ms=30.0, replays=5)
        us, cus = med / n * 1e6, cmed / n * 1e6
        tf = 2.0 * M * K * N / (med / n) / 1e12
        step(0)
        torch.cuda.synchronize()
        r_s = 4  # rows checked against the oracle (scalar code)
        rows.append({"M": M, "us": round(us, 2), "us_min": round(mn / n * 1e6, 2), "achieved": round(tf, 1),
                     "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TF, 4),
                     "dequantize_plus_library_gemm_us": round(cus, 2), "speed_vs_composition": round(cus / us, 3),
                     "path": _plan_grad(_lib, M, K, N)})
        if M == 2048:
            gq = H.torch_to_bits(go[:r_s])
            sample = (gq, H.torch_to_bits(out[:r_s]))
    # the oracle needs canonical codes: quantise the same weight on the CPU
    w_bits = H.torch_to_bits(_device_weight(torch, K, N, bf16, 77, dev))
    oq, os_ = H.O.weight_quantize(w_bits, dt, bits, g)
    _, wantT = H.O.linear_grad(sample[0], oq, os_, dt, bits, g)
    err = H.rel_l2(H.bits_to_f32(sample[1], dt), H.bits_to_f32(wantT, dt))
    if err > REL_L2_BAR:
        failures.append("linear_grad output differs from the oracle")
    return {"workload": "x_grad = out_grad [M, 4096] . dequant(W)[4096, 4096]^T, int8 per-channel, bf16",
            "arithmetic": "fp16 MFMA operands, code*scale rounded once to 11 bits, fp32 sums",
            "rows": rows, "rel_l2_vs_oracle": err, "parity_sample": "first 4 rows of the M=2048 result"}


def bench_fused_swiglu(torch, Q, dev, quick):
    """weight_only_linear_fused(act="swiglu") on a gate|up projection of Llama-2-7B's
    size (K = 4096, N = 2 x 11008) beside the plain linear on the same weight:
    the swiglu is formed inside the decode kernels and the GEMM epilogue, so the
    fused call should cost what the linear costs and save the separate
    [M, N] -> [M, N/2] pass and its round trip through memory."""
    K, N = 4096, 22016
    bf16 = torch.bfloat16
    w = _device_weight(torch, K, N, bf16, 700, dev)
    rows = []
    for bits, g in ((4, 128),) if quick else ((4, 128), (8, -1), (8, 64)):
        codes, scale = _quantize(Q, w, bits, g)
        ncp = max(2, -(-640 * 1024 * 1024 // codes.numel()))
        cps = [codes.clone() for _ in range(ncp)]
        wd = "int8" if bits == 8 else "int4"
        for M in (1, 16, 2048):
            gen = torch.Generator(device=dev)
            gen.manual_seed(M)
            x = torch.randn((M, K), generator=gen, device=dev, dtype=torch.float32).to(bf16)
            n = 4 if M > 64 else 100
            plain, _ = time_graph(torch, lambda i: Q.weight_only_linear(x, cps[i % ncp], None, scale, wd, None, g), n,
                                  warm_launches=2 * n, warm_ms=20.0, replays=5)
            fused, _ = time_graph(torch, lambda i: Q.weight_only_linear_fused(x, cps[i % ncp], None, scale, wd, g,
                                                                             act="swiglu"), n,
                                  warm_launches=2 * n, warm_ms=20.0, replays=5)
            rows.append({"weights": "int%d g%d" % (bits, g), "M": M, "linear_us": round(plain / n * 1e6, 2),
                         "fused_swiglu_us": round(fused / n * 1e6, 2), "fused_over_linear": round(fused / plain, 4)})
        del cps
    return {"workload": "gate|up projection K=4096 N=22016, bf16: weight_only_linear against "
                        "weight_only_linear_fused(act=swiglu, out [M, 11008])", "rows": rows}


def bench_prefill_phases(torch, np, Q, _lib, dev):
    """wol_prefill_phases: the prefill GEMM's 256 x 256 launch on an instantiation
    that reads the cycle counter around its waits.  Per k tile and wavefront,
    averaged over all wavefronts of the launch: cycles between the barriers
    (MFMAs and what is issued among them), waiting for the wavefront's own tile
    loads, waiting at the barrier; and the prologue and epilogue of a tile."""
    K = 4096
    bf16 = torch.bfloat16
    rows = []
    for M, N in ((2048, 8192), (8192, 8192)):
        w = _device_weight(torch, K, N, bf16, 900, dev)
        codes, scale = _quantize(Q, w, 8, -1)
        del w
        gen = torch.Generator(device=dev)
        gen.manual_seed(M)
        x = torch.randn((M, K), generator=gen, device=dev, dtype=torch.float32).to(bf16)
        out = torch.empty((M, N), dtype=bf16, device=dev)
        wgs = (M // 256) * (N // 256)
        ph = torch.zeros(wgs * 64, dtype=torch.int64, device=dev)

        def stamped(_i):
            _lib.check(_lib.lib.wol_prefill_phases(x.data_ptr(), codes.data_ptr(), scale.data_ptr(), M, K, N,
                                                   out.data_ptr(), ph.data_ptr(), ph.numel() * 8, torch.cuda.current_stream().cuda_stream))

        t_st, _ = time_graph(torch, stamped, 4, warm_launches=8, warm_ms=30.0, replays=5)
        t_pl, _ = time_graph(torch, lambda i: Q.weight_only_linear(x, codes, None, scale, "int8"), 4, warm_launches=8,
                             warm_ms=30.0, replays=5)
        torch.cuda.synchronize()
        c = ph.cpu().numpy().reshape(wgs * 8, 8).astype(np.float64)
        tiles = float(c[0, 7])
        mean = c.mean(axis=0)
        tiles_per_cu = max(1.0, wgs / 256.0)
        rows.append({
            "M": M, "K": K, "N": N, "workgroups": wgs, "k_tiles": int(tiles),
            "stamped_us": round(t_st / 4 * 1e6, 1), "product_us": round(t_pl / 4 * 1e6, 1),
            "counter_ghz": round(mean[6] * tiles_per_cu / (t_st / 4) / 1e9, 3),
            "cycles_per_k_tile": {"between_barriers": round(mean[1] / tiles, 1), "wait_own_loads": round(mean[2] / tiles, 1),
                                  "wait_barrier": round(mean[3] / tiles, 1),
                                  "mfma_issue_at_full_rate": 2048},
            "cycles_per_tile": {"prologue": round(mean[0], 0), "last_tile_tail": round(mean[4], 0),
                                "epilogue": round(mean[5], 0), "total": round(mean[6], 0)},
            "share_of_total": {"between_barriers": round(mean[1] / mean[6], 4), "wait_own_loads": round(mean[2] / mean[6], 4),
                               "wait_barrier": round(mean[3] / mean[6], 4), "prologue": round(mean[0] / mean[6], 4),
                               "epilogue": round((mean[4] + mean[5]) / mean[6], 4)},
            "slowest_wavefront_wait_barrier_share": round(float((c[:, 3] / c[:, 6]).min()), 4),
            # wavefronts 0-3 of a workgroup are the first on their SIMDs, 4-7 the second
            "by_wavefront_of_simd": {
                name: {"between_barriers": round(float(g[:, 1].mean()) / tiles, 1),
                       "wait_barrier": round(float(g[:, 3].mean()) / tiles, 1)}
                for name, g in (("first", c.reshape(wgs, 8, 8)[:, :4].reshape(-1, 8)),
                                ("second", c.reshape(wgs, 8, 8)[:, 4:].reshape(-1, 8)))},
        })
    return {"what": "wol_prefill_phases: per-wavefront cycle stamps in the 256 x 256 tile of the prefill GEMM "
                    "(int8 per-channel, bf16); 2048 cycles per k tile is what two wavefronts per SIMD need to issue "
                    "their 2 x 32 MFMAs of 32 cycles back to back", "rows": rows}


def bench_decode_phases(torch, np, Q, _lib, dev, c, x, copies, scales, steps):
    """wol_decode_phases: the headline decode kernel on an instantiation that reads
    the clocks as it goes, launched as the headline figure launches the product
    kernel (`steps` launches in one graph, each on the next copy of the weights,
    the copies together several times the Infinity Cache).  Four consecutive
    launches in the middle of the graph stamp into phases of their own, so that
    the device's constant-rate clock (100 MHz) places every wavefront of theirs
    on one time line: how long after a launch's first wavefront its last one
    enters, how long after it the last one ends (the span in which the weights
    are read), and how long the device then takes until the next launch's first
    wavefront starts.  The shader-cycle stamps split a wavefront's life into
    its phases."""
    K, N, g = c["K"], c["N"], c["group_size"]
    out = torch.empty((1, N), dtype=torch.bfloat16, device=dev)
    wgs, L = N // 16, 4
    first = max(0, steps // 2 - L // 2)
    ph = [torch.zeros(wgs * 64, dtype=torch.int64, device=dev) for _ in range(L + 1)]  # the last one takes all other launches'

    def stamped(i):
        j = i % len(copies)
        p_ = ph[i - first] if first <= i < first + L else ph[L]
        _lib.check(_lib.lib.wol_decode_phases(x.data_ptr(), copies[j].data_ptr(), scales[j].data_ptr(), K, N, g, out.data_ptr(),
                                              p_.data_ptr(), p_.numel() * 8, torch.cuda.current_stream().cuda_stream))

    t_st, _ = time_graph(torch, stamped, steps, warm_launches=400)
    torch.cuda.synchronize()
    cs = [p_.cpu().numpy().reshape(wgs * 8, 8).astype(np.float64) for p_ in ph[:L]]
    tick_us = 0.01
    enter = [float((c_[:, 0].max() - c_[:, 0].min()) * tick_us) for c_ in cs]
    span = [float((c_[:, 1].max() - c_[:, 0].min()) * tick_us) for c_ in cs]
    gap = [float((cs[i + 1][:, 0].min() - cs[i][:, 1].max()) * tick_us) for i in range(L - 1)]
    period = [float((cs[i + 1][:, 0].min() - cs[i][:, 0].min()) * tick_us) for i in range(L - 1)]
    allc = np.concatenate(cs)
    mean = allc.mean(axis=0)
    bytes_read = K * N // 2  # the codes alone, as the headline figure counts
    span_us = statistics.median(span)
    names = ("arguments", "issue_loads", "wait_loads", "compute", "wait_barrier", "epilogue")
    life = allc[:, 2:8].sum(axis=1)
    ghz = float(life.mean() / ((allc[:, 1] - allc[:, 0]) * tick_us).mean() / 1e3)
    # when a wavefront's last load has landed, on the launch's own time line
    landed = [(c_[:, 0] - c_[:, 0].min()) * tick_us + c_[:, 2:5].sum(axis=1) / (ghz * 1e3) for c_ in cs]
    return {
        "what": "wol_decode_phases: clock stamps per wavefront of the headline decode kernel (bf16, int4 group %d, "
                "M=1, K=%d, N=%d); %d launches in one graph on %d weight copies, %d consecutive ones stamped into phases "
                "of their own" % (g, K, N, steps, len(copies), L),
        "workgroups": wgs, "stamped_us": round(t_st / steps * 1e6, 3),
        "last_wavefront_enters_after_us": round(statistics.median(enter), 2),
        "first_entry_to_last_end_us": round(span_us, 2),
        "last_end_to_next_launch_first_entry_us": round(statistics.median(gap), 2),
        "first_entry_to_next_first_entry_us": round(statistics.median(period), 2),
        "hbm_frac_within_span": round(bytes_read / (span_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
        "wavefront_life_us": round(float(((allc[:, 1] - allc[:, 0]) * tick_us).mean()), 2),
        "shader_clock_ghz": round(ghz, 3),
        "loads_landed_after_us": {"first_wavefront": round(statistics.median(float(l.min()) for l in landed), 2),
                                  "median_wavefront": round(statistics.median(float(np.median(l)) for l in landed), 2),
                                  "last_wavefront": round(statistics.median(float(l.max()) for l in landed), 2)},
        # workgroups in the order they were dealt out, 256 (one per CU) to a round: when a round's workgroups have their data
        "last_load_landed_by_round_of_256_us": [
            round(statistics.median(float(l.reshape(wgs, 8).max(axis=1)[r0:r0 + 256].mean()) for l in landed), 2)
            for r0 in range(0, wgs, 256)],
        "cycles": {n: round(float(mean[2 + i]), 0) for i, n in enumerate(names)},
        "share_of_life": {n: round(float(mean[2 + i] / life.mean()), 4) for i, n in enumerate(names)},
    }


def bench_decode_rounds(torch, Q, _lib, dev, c, steps):
    """The headline decode call and the pure read of the same bytes over the number
    of strips (K, bits and group size of the headline; N from one workgroup per CU
    to five): a launch costs a fixed part plus a part per round of 256 workgroups."""
    K, g, bits = c["K"], c["group_size"], c["bits"]
    wd = "int8" if bits == 8 else "int4"
    rows = []
    for N in (4096, 8192, 10240, 11008, 12288, 14336, 16384, 20480):
        codes, scale = _quantize(Q, _device_weight(torch, K, N, torch.bfloat16, 950, dev), bits, g)
        wbytes = K * N * bits // 8
        ncopies = max(2, -(-768 * 1024 * 1024 // wbytes))
        copies = [codes.clone() for _ in range(ncopies)]
        scales = [scale.clone() for _ in range(ncopies)]
        x = torch.randn((1, K), device=dev, dtype=torch.float32).to(torch.bfloat16)
        floor_out = torch.empty(N // 16 * 8, dtype=torch.int32, device=dev)

        def call(i):
            return Q.weight_only_linear(x, copies[i % ncopies], None, scales[i % ncopies], wd, None, g)

        def floor(i):
            _lib.check(_lib.lib.wol_read_floor(copies[i % ncopies].data_ptr(), K, N, bits, floor_out.data_ptr(),
                                               torch.cuda.current_stream().cuda_stream))

        t_c, _ = time_graph(torch, call, steps, warm_launches=400)
        t_f, _ = time_graph(torch, floor, steps, warm_launches=400)
        rows.append({"N": N, "strips": N // 16, "rounds_of_256": round(N / 16 / 256, 2),
                     "linear_us": round(t_c / steps * 1e6, 3), "read_floor_us": round(t_f / steps * 1e6, 3)})
        del copies, scales
        torch.cuda.empty_cache()
    return {"what": "wol_linear (M=1, int%d g%d, K=%d, bf16) and wol_read_floor over N: one workgroup per 16-column strip, "
                    "256 CUs" % (bits, g, K), "rows": rows}


def bench_moe_ffn(torch, np, Q, H, dev, quick, failures):
    """moe_ffn on weight-only int8 experts of Mixtral-8x7B's size (8 experts,
    hidden 4096, fc1 width 2 x 14336 for swiglu, bf16): a prefill-like call
    (4096 rows in expert order, 512 per expert; MFMA-bound) and a decode-like
    one (128 rows, 16 per expert; bound by the 1.4 GB of expert weights every
    call streams).  Two rows of one expert are checked against the oracle (the
    oracle's linear, swiglu on its rounded output, the oracle's linear)."""
    E, hidden, inter = 8, 4096, 28672
    bf16, dt = torch.bfloat16, H.BF16
    q1, s1, q2, s2 = [], [], [], []
    for e in range(E):
        c, s = _quantize(Q, _device_weight(torch, hidden, inter, bf16, 500 + e, dev), 8, -1)
        q1.append(c); s1.append(s)
        c, s = _quantize(Q, _device_weight(torch, inter // 2, hidden, bf16, 600 + e, dev), 8, -1)
        q2.append(c); s2.append(s)
    q1, s1, q2, s2 = torch.stack(q1), torch.stack(s1), torch.stack(q2), torch.stack(s2)
    wbytes = E * (hidden * inter + inter // 2 * hidden)
    rows_out = []
    sample = None
    for rows in ((4096,) if quick else (4096, 128)):
        gen = torch.Generator(device=dev)
        gen.manual_seed(rows)
        x = torch.randn((rows, hidden), generator=gen, device=dev, dtype=torch.float32).to(bf16)
        cum = torch.arange(1, E + 1, device=dev, dtype=torch.int64) * (rows // E)
        holder = {}

        def step(_i):
            holder["out"] = Q.moe_ffn(x, cum, q1, q2, None, s1, s2, "weight_only_int8")

        n = 2 if rows >= 1024 else 4
        med, mn = time_graph(torch, step, n, warm_launches=8, warm_ms=30.0, replays=5)
        t = med / n
        flops = 2.0 * rows * hidden * inter + 2.0 * rows * (inter // 2) * hidden
        entry = {"rows": rows, "rows_per_expert": rows // E, "ms": round(t * 1e3, 4), "ms_min": round(mn / n * 1e3, 4)}
        if rows >= 1024:
            tf = flops / t / 1e12
            entry.update({"bound": "mfma", "achieved": round(tf, 1), "unit": "TFLOP/s",
                          "frac": round(tf / MFMA_BF16_PEAK_TF, 4)})
        else:
            gbs = wbytes / t / 1e9
            entry.update({"bound": "hbm", "achieved": round(gbs, 1), "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4)})
        rows_out.append(entry)
        if rows == 4096:
            step(0)
            torch.cuda.synchronize()
            e_s, r0 = 3, 3 * (rows // E)  # two rows of expert 3
            sample = (H.torch_to_bits(x[r0:r0 + 2]), H.torch_to_bits(holder["out"][r0:r0 + 2]), e_s)
    xb, got, e_s = sample
    O = H.O
    c1, sc1 = O.weight_quantize(H.torch_to_bits(_device_weight(torch, hidden, inter, bf16, 500 + e_s, dev)), dt, 8, -1)
    c2, sc2 = O.weight_quantize(H.torch_to_bits(_device_weight(torch, inter // 2, hidden, bf16, 600 + e_s, dev)), dt, 8, -1)
    _, fc1 = O.linear(xb, c1, sc1, None, dt, 8, -1)
    _, act = O.activation(H.bits_to_f32(fc1, dt), O.ACT_SWIGLU, dt)
    _, want = O.linear(act, c2, sc2, None, dt, 8, -1)
    err = H.rel_l2(H.bits_to_f32(got, dt), H.bits_to_f32(want, dt))
    if err > REL_L2_BAR:
        failures.append("moe_ffn output differs from the oracle")
    return {"workload": "moe_ffn, 8 experts, hidden 4096, fc1 width 28672 (swiglu to 14336), int8 per-channel, bf16; "
                        "rows in expert order, the same number per expert",
            "launches_per_call": "tile table, grouped GEMM, swiglu pass, grouped GEMM",
            "weight_bytes": wbytes, "rows": rows_out, "rel_l2_vs_oracle": err,
            "parity_sample": "two rows of expert 3 of the 4096-row call"}


def _plan_grad(_lib, M, K, N):
    import ctypes
    buf = ctypes.create_string_buffer(256)
    if _lib.lib.wol_linear_grad_plan(M, K, N, buf, 256) != 0:
        return None
    return buf.value.decode()


def cpu_decode_baseline(np, torch, H, w_bits, x_bits, cfg, budget_s=10.0):
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
    while reps < 3 or (time.perf_counter() - t_start < budget_s and reps < 400):
        t0 = time.perf_counter()
        w32, _ = O.dequantize(codes, scale, dt, bits, g)
        t1 = time.perf_counter()
        _ = x32 @ torch.from_numpy(w32)
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
        "sample": "first %d of %d columns of the decode weight, M=1, %d repetitions" % (n_s, N, reps),
        "sample_columns": n_s,
        "repetitions": reps,
        "dequantize_ms": round(t_dq * 1e3, 3),
        "dequantize_cores": 1,
        "matmul_ms": round(t_mm * 1e3, 3),
        "matmul_cores": int(cores),
        "quantize_ms": round(t_q * 1e3, 2),
        "quantize_cores": 1,
        "quantize_gbs": round(K * n_s * 2 / t_q / 1e9, 4),
        "stages": "per call: oracle dequantize (1 thread) + fp32 matmul (torch CPU BLAS, all threads); quantize_ms is the "
                  "one-time oracle weight_quantize of the same sample (1 thread), quantize_gbs on its bf16 weight read",
    }, (codes, scale, n_s)


def cpu_prefill_baseline(np, torch, H, pw_bits, px_bits, cfg, n_s=1024):
    """The same three stages on the prefill shape, first n_s output columns."""
    O = H.O
    dt = H.BF16
    K, M, bits, g = cfg["K"], cfg["M"], cfg["bits"], cfg["group_size"]
    wb = np.ascontiguousarray(pw_bits[:, :n_s])
    t0 = time.perf_counter()
    codes, scale = O.weight_quantize(wb, dt, bits, g)
    t_q = time.perf_counter() - t0
    x32 = torch.from_numpy(H.bits_to_f32(px_bits, dt))
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        w32, _ = O.dequantize(codes, scale, dt, bits, g)
        y = x32 @ torch.from_numpy(w32)
        ts.append(time.perf_counter() - t0)
    t = statistics.median(ts)
    return {"value": round(2.0 * M * K * n_s / t / 1e12, 4), "unit": "TFLOP/s", "cores": int(torch.get_num_threads()),
            "kind": "port", "ms": round(t * 1e3, 2), "quantize_ms": round(t_q * 1e3, 2), "sample_columns": n_s,
            "sample": "first %d of %d columns, M=%d: dequantize (1 thread) + fp32 matmul (all threads)"
                      % (n_s, cfg["N"], M)}, (codes, scale, y.numpy())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--prefill-steps", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU timing (parity still runs)")
    ap.add_argument("--no-llm-int8", action="store_true", help="skip the llm_int8_linear timing")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration table")
    ap.add_argument("--no-ladder", action="store_true", help="skip the wol_mfma_probe ladder")
    ap.add_argument("--no-decode-rounds", action="store_true",
                    help="skip the decode call over the number of strips (it launches the headline kernel on other grids)")
    ap.add_argument("--quick", action="store_true", help="shorter per-configuration runs, 8 decoder layers")
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
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

    if args.copy_calibration:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    failures = []
    global EAGER
    EAGER = args.eager

    # ---------------- decode (the headline metric) ----------------
    c = DECODE
    dt = H.BF16
    w_bits = H.make_weight(c["K"], c["N"], dt, seed=1234)
    x_bits = H.make_act(c["M"], c["K"], dt, seed=1235)
    w = H.bits_to_torch(w_bits, dt, dev)
    x = H.bits_to_torch(x_bits, dt, dev)
    codes, scale = _quantize(Q, w, c["bits"], c["group_size"])
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

    dec_med, dec_min = time_graph(torch, decode_step, args.steps, warm_launches=max(400, args.warmup),
                                  eager=args.eager)
    dec_s = dec_med / args.steps
    dec_gbs = wbytes / dec_s / 1e9
    y = decode_step(0)
    torch.cuda.synchronize()

    # the floor of this launch shape on this machine: the same weight copies read
    # by a kernel of the decode kernel's shape that computes nothing
    floor_out = torch.empty(c["N"] // 16 * 8, dtype=torch.int32, device=dev)

    def floor_step(i):
        _lib.check(_lib.lib.wol_read_floor(copies[i % ncopies].data_ptr(), c["K"], c["N"], c["bits"],
                                           floor_out.data_ptr(), stream()))

    floor_med, _ = time_graph(torch, floor_step, args.steps, warm_launches=max(400, args.warmup), eager=args.eager)
    floor_s = floor_med / args.steps

    # Independent decode GEMVs with no edge between them: --steps calls dealt
    # round-robin to four streams that fork from and join the launching stream
    # inside the same graph, so up to four launches are in flight at a time
    # (independent projections of one input: q/k/v or gate/up kept as separate
    # weights, the experts of a mixture).  Every call still reads its own
    # weight copy from HBM once; what overlaps is one call's launch and drain
    # with another's stream.
    n_par = 4
    par_steps = max(args.steps, 400)  # the fork and join of a replay cost as much as several calls: many calls per replay
    par_streams = [torch.cuda.Stream(device=dev) for _ in range(n_par - 1)]
    par_x = [x.clone() for _ in range(n_par)]

    def par_call(i, s):
        j = i % ncopies
        with torch.cuda.stream(s):
            return Q.weight_only_linear(par_x[i % n_par], copies[j], None, scales[j], wd, None, c["group_size"])

    def par_whole():
        cur = torch.cuda.current_stream()
        fork = torch.cuda.Event()
        fork.record(cur)
        for s in par_streams:
            s.wait_event(fork)
        for i in range(par_steps):
            par_call(i, cur if i % n_par == 0 else par_streams[i % n_par - 1])
        for s in par_streams:
            e = torch.cuda.Event()
            e.record(s)
            cur.wait_event(e)

    par_med, par_min = time_graph(torch, decode_step, par_steps, warm_launches=max(400, args.warmup),
                                  eager=args.eager, whole=par_whole)
    par_s = par_med / par_steps

    # ---------------- prefill ----------------
    p = PREFILL
    pw_bits = H.make_weight(p["K"], p["N"], dt, seed=1236)
    px_bits = H.make_act(p["M"], p["K"], dt, seed=1237)
    px = H.bits_to_torch(px_bits, dt, dev)
    pcodes, pscale = _quantize(Q, H.bits_to_torch(pw_bits, dt, dev), p["bits"], p["group_size"])
    pcopies = [(pcodes.clone(), pscale.clone()) for _ in range(6)]  # 300 MB: past the Infinity Cache

    def prefill_step(i):
        cw, cs = pcopies[i % len(pcopies)]
        return Q.weight_only_linear(px, cw, None, cs, "int8", None, p["group_size"])

    pre_med, pre_min = time_graph(torch, prefill_step, args.prefill_steps, warm_launches=40, eager=args.eager)
    pre_s = pre_med / args.prefill_steps
    flops = 2.0 * p["M"] * p["K"] * p["N"]
    pre_tf = flops / pre_s / 1e12
    py = prefill_step(0)
    torch.cuda.synchronize()

    # the ceiling of the matrix pipes on this machine: nothing but MFMAs on random operands
    ops = torch.randn(8 * 64 * 8, device=dev).to(torch.bfloat16)
    ceil_wgs, ceil_iters = 1024, 2000
    ceil_out = torch.empty(ceil_wgs * 512, dtype=torch.float32, device=dev)

    def ceil_step(_i):
        _lib.check(_lib.lib.wol_mfma_ceiling(ops.data_ptr(), ceil_wgs, ceil_iters, ceil_out.data_ptr(), stream()))

    ceil_med, _ = time_graph(torch, ceil_step, 4, warm_launches=8, warm_ms=30.0, replays=5, eager=args.eager)
    ceil_tf = ceil_wgs * 8.0 * ceil_iters * 8 * 2 * 32 * 32 * 16 / (ceil_med / 4) / 1e12

    # the prefill tile's inner loop with its ingredients switched on one at a time (wol_mfma_probe)
    ladder = None
    if not args.no_ladder:
        probe_ops = torch.randn(12 * 1024 * 1024 + 65536, device=dev).to(torch.bfloat16)  # > WOL_MFMA_PROBE_OPERAND_BYTES
        names = ["mfma_only", "plus_dequant", "plus_a_reads", "plus_dequant_and_a_reads", "plus_barrier",
                 "plus_barrier_and_tile_loads", "mfma_barrier_and_tile_loads", "mfma16x16x32_only",
                 "mfma16x16x32_dequant_a_reads_barrier"]
        p_wgs, p_iters = 1024, 400
        p_out = torch.empty(p_wgs * 512, dtype=torch.float32, device=dev)
        ladder = {}
        for v, nm in enumerate(names):
            def probe_step(_i, v=v):
                _lib.check(_lib.lib.wol_mfma_probe(v, probe_ops.data_ptr(), probe_ops.numel() * 2, p_wgs, p_iters,
                                                   p_out.data_ptr(), stream()))

            med, _ = time_graph(torch, probe_step, 4, warm_launches=8, warm_ms=20.0, replays=5, eager=args.eager)
            ladder[nm] = round(p_wgs * 8.0 * p_iters * 1048576 / (med / 4) / 1e12, 1)
        del probe_ops

    # ---------------- llm_int8_linear on the prefill shape ----------------
    # the sibling op on the same weight (algo="llm.int8"): activations N(0,1)
    # with eight columns scaled x12, so that the outlier branch runs
    llm = None
    lx = ly = None
    if not args.no_llm_int8:
        lw, lscale = Q.weight_quantize(H.bits_to_torch(pw_bits, dt, dev), algo="llm.int8")
        lx = px.clone()
        lx[:, 100:3700:450] *= 12.0

        def llm_step(i):
            return Q.llm_int8_linear(lx, lw, None, lscale, 6.0)

        llm_med, llm_min = time_graph(torch, llm_step, args.prefill_steps, warm_launches=40, eager=args.eager)
        llm_s = llm_med / args.prefill_steps
        llm_tops = flops / llm_s / 1e12
        ly = llm_step(0)
        torch.cuda.synchronize()
        llm = {
            "workload": "llm_int8_linear M=2048, K=4096 N=12288, bf16 x with 8 outlier columns, threshold 6.0; "
                        "all stages of one call (row ranges, activation codes, int8 GEMM with the merge)",
            "value": round(llm_tops, 2),
            "unit": "TOP/s",
            "ms_per_step": round(llm_s * 1e3, 4),
            "ms_per_step_min": round(llm_min / args.prefill_steps * 1e3, 4),
            "steps": args.prefill_steps,
            "roofline": {"bound": "mfma", "achieved": round(llm_tops, 2), "peak": MFMA_INT8_PEAK_TOPS,
                         "unit": "TOP/s", "frac": round(llm_tops / MFMA_INT8_PEAK_TOPS, 4),
                         "traffic": _load_traffic().get("llm_int8_gemm_bytes_per_launch"),
                         "kernel": "wol::llm_gemm_kernel<1, 2, 4, 4, 2, 128, 2, false> (256x256 tiles on 8192 columns) "
                                   "+ <1, 2, 4, 2, 2, 128, 3, false> (128x256 tiles on the rest), "
                                   "v_mfma_i32_32x32x32_i8"},
        }

    # ---------------- every BASELINE configuration ----------------
    configs = stack = grad = moe = fused = phases = dphases = drounds = None
    if not args.no_configs:
        if c["K"] == 4096 and c["bits"] == 4 and c["group_size"] in (64, 128) and not args.eager and args.steps >= 8:
            dphases = bench_decode_phases(torch, np, Q, _lib, dev, c, x, copies, scales, args.steps)
        del copies, scales
        torch.cuda.empty_cache()
        configs = bench_configs(torch, Q, _lib, dev, args.quick)
        stack = bench_decoder_stack(torch, Q, _lib, dev, args.quick)
        grad = bench_linear_grad(torch, np, Q, _lib, H, dev, args.quick, failures)
        torch.cuda.empty_cache()
        moe = bench_moe_ffn(torch, np, Q, H, dev, args.quick, failures)
        torch.cuda.empty_cache()
        fused = bench_fused_swiglu(torch, Q, dev, args.quick)
        torch.cuda.empty_cache()
        phases = bench_prefill_phases(torch, np, Q, _lib, dev)
        torch.cuda.empty_cache()
        if not args.quick and not args.eager and not args.no_decode_rounds:
            drounds = bench_decode_rounds(torch, Q, _lib, dev, c, max(args.steps, 100))

    # ---------------- parity of what was measured, against the oracle ----------------
    O = H.O
    parity = {}
    cpu = None
    if args.no_cpu_baseline:
        n_s = 512
        ocodes, oscale = O.weight_quantize(np.ascontiguousarray(w_bits[:, :n_s]), dt, c["bits"], c["group_size"])
    else:
        cpu, (ocodes, oscale, n_s) = cpu_decode_baseline(np, torch, H, w_bits, x_bits, c)
    _, oT = O.linear(x_bits, ocodes, oscale, None, dt, c["bits"], c["group_size"])
    got = H.bits_to_f32(H.torch_to_bits(y), dt)[:, :n_s]
    parity["decode_rel_l2_vs_oracle"] = H.rel_l2(got, H.bits_to_f32(oT, dt))
    parity["scales_bit_exact"] = bool(np.array_equal(H.torch_to_bits(scale)[:, :n_s], oscale))
    if parity["decode_rel_l2_vs_oracle"] > REL_L2_BAR:
        failures.append("decode output differs from the oracle")
    if not parity["scales_bit_exact"]:
        failures.append("decode scales differ from the oracle")

    # prefill: the first rows and columns of the measured output
    rows, cols = 64, 256
    pq, ps = O.weight_quantize(np.ascontiguousarray(pw_bits[:, :cols]), dt, p["bits"], p["group_size"])
    _, pT = O.linear(px_bits[:rows], pq, ps, None, dt, p["bits"], p["group_size"])
    got = H.bits_to_f32(H.torch_to_bits(py[:rows, :cols]), dt)
    parity["prefill_rel_l2_vs_oracle"] = H.rel_l2(got, H.bits_to_f32(pT, dt))
    parity["prefill_sample"] = "first %d rows x %d columns" % (rows, cols)
    if parity["prefill_rel_l2_vs_oracle"] > REL_L2_BAR:
        failures.append("prefill output differs from the oracle")
    if not args.no_cpu_baseline:
        pcpu, _ = cpu_prefill_baseline(np, torch, H, pw_bits, px_bits, p)
        cpu["prefill"] = pcpu
        cpu["prefill_tflops"] = pcpu["value"]
        cpu["prefill_ms"] = pcpu["ms"]
        cpu["prefill_quantize_ms"] = pcpu["quantize_ms"]
        cpu["prefill_sample_columns"] = pcpu["sample_columns"]

    # llm_int8_linear: all rows (the outlier columns depend on every row), the first columns
    if ly is not None:
        cols = 64
        lq, ls = O.weight_quantize_llm_int8(np.ascontiguousarray(pw_bits[:, :cols]), dt)
        ref = O.llm_int8_linear(H.torch_to_bits(lx), np.ascontiguousarray(lq.T), None, ls, 6.0, dt)
        same = np.array_equal(ref["out"], H.torch_to_bits(ly[:, :cols]))
        parity["llm_int8_bit_exact_vs_oracle"] = bool(same)
        parity["llm_int8_sample"] = "all rows x first %d columns" % cols
        if not same:
            failures.append("llm_int8_linear output differs from the oracle")

    traffic = _load_traffic()
    out = {
        "metric": "weight-only linear GB/s on weight bytes at M=1 (decode GEMV)",
        "value": round(dec_gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dec_s * 1e3, 6),
        "ms_per_step_min": round(dec_min / args.steps * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "timing": "one HIP graph of --steps launches, replayed untimed until >= 400 launches and >= 50 ms have run, "
                  "then %d timed replays (events on the launching stream); ms_per_step = median replay / steps"
                  % REPLAYS if not args.eager else "eager launches",
        "config": {
            "workload": "decode GEMV M=1, int4 group_size=128, K=4096 N=11008, bf16 x, no bias; "
                        "%d rotating weight copies" % ncopies,
            "prefill_workload": "GEMM M=2048, int8 per-channel, K=4096 N=12288, bf16 x, 6 rotating weight copies",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(dec_gbs, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dec_gbs / HBM_PEAK_GBS, 4),
            "traffic": traffic.get("decode_bytes_per_launch"),
            "traffic_source": "profiles/traffic.json (rocprofv3 --pmc runs of this command, not measured in this run)",
            "kernel": _plan(_lib, c["M"], c["K"], c["N"], c["bits"], c["group_size"]) or "wol::stream_kernel",
            "algorithmic_bytes_per_launch": wbytes,
            "total_bytes_per_launch": total_bytes,
            # the M=2048 half of the metric and the two in-run bounds, as plain numbers
            "prefill_tflops": round(pre_tf, 2),
            "prefill_frac": round(pre_tf / MFMA_BF16_PEAK_TF, 4),
            "prefill_ms_per_step": round(pre_s * 1e3, 4),
            "prefill_peak_tflops": MFMA_BF16_PEAK_TF,
            "mfma_ceiling_tflops": round(ceil_tf, 1),
            "read_floor_gbs": round(wbytes / floor_s / 1e9, 1),
            "read_floor_ms_per_step": round(floor_s * 1e3, 6),
            # the same decode call, four independent calls in flight (no edge between them in the graph)
            "decode_4_in_flight_gbs": round(wbytes / par_s / 1e9, 1),
            "decode_4_in_flight_frac": round(wbytes / par_s / 1e9 / HBM_PEAK_GBS, 4),
            "decode_4_in_flight_ms_per_step": round(par_s * 1e3, 6),
            "decode_4_in_flight_steps_per_replay": par_steps,
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
            "ms_per_step_min": round(pre_min / args.prefill_steps * 1e3, 4),
            "steps": args.prefill_steps,
            "roofline": {
                "bound": "mfma",
                "achieved": round(pre_tf, 2),
                "peak": MFMA_BF16_PEAK_TF,
                "unit": "TFLOP/s",
                "frac": round(pre_tf / MFMA_BF16_PEAK_TF, 4),
                "traffic": traffic.get("prefill_bytes_per_launch"),
                "kernel": _plan(_lib, p["M"], p["K"], p["N"], p["bits"], p["group_size"]) or "wol::gemm_dma_kernel",
                "mfma_ceiling": {
                    "what": "wol_mfma_ceiling: v_mfma_f32_32x32x16_bf16 on random operands held in registers, "
                            "8 independent accumulator blocks per wavefront, 8 wavefronts per CU, no memory traffic",
                    "TFLOP/s": round(ceil_tf, 1),
                    "frac_of_peak": round(ceil_tf / MFMA_BF16_PEAK_TF, 4),
                    "prefill_over_ceiling": round(pre_tf / ceil_tf, 4),
                },
                "inner_loop_ladder_tflops": ladder,
            },
        },
        "configs": configs,
        "decoder_stack": stack,
        "linear_grad": grad,
        "moe_ffn": moe,
        "fused_swiglu": fused,
        "prefill_phases": phases,
        "decode_phases": dphases,
        "decode_rounds": drounds,
        "llm_int8": llm,
        "cpu_baseline": cpu,
        "parity": parity,
    }
    # every per-configuration fraction of its roofline once more as plain numbers of `roofline`
    flat = out["roofline"]
    for e in configs or []:
        tag = "north_star" if e["config"].startswith("north") else e["config"]
        flat["%s_K%d_N%d_M%d_frac" % (tag, e["K"], e["N"], e["M"])] = e["frac"]
    if stack:
        flat["c5_decode_M8_frac"] = stack["decode_M8"]["frac"]
        flat["c5_prefill_M1024_frac"] = stack["prefill_M1024"]["frac"]
    if grad:
        for r in grad["rows"]:
            flat["linear_grad_M%d_vs_composition" % r["M"]] = r["speed_vs_composition"]
    if moe:
        for r in moe["rows"]:
            flat["moe_ffn_rows%d_frac" % r["rows"]] = r["frac"]
    if fused:
        for r in fused["rows"]:
            flat["fused_swiglu_%s_M%d_over_linear" % (r["weights"].replace(" ", "_"), r["M"])] = r["fused_over_linear"]
    if phases:
        for r in phases["rows"]:
            for k, v in r["share_of_total"].items():
                flat["prefill_phase_M%d_%s_share" % (r["M"], k)] = v
    if dphases:
        for k in ("first_entry_to_last_end_us", "last_end_to_next_launch_first_entry_us", "hbm_frac_within_span"):
            flat["decode_phase_" + k] = dphases[k]
    if drounds:
        for r_ in drounds["rows"]:
            flat["decode_rounds_strips%d_linear_us" % r_["strips"]] = r_["linear_us"]
            flat["decode_rounds_strips%d_read_floor_us" % r_["strips"]] = r_["read_floor_us"]
    if llm:
        flat["llm_int8_frac"] = llm["roofline"]["frac"]
    for nm, tf in (ladder or {}).items():
        flat["ladder_%s_tflops" % nm] = tf
    print(json.dumps(out))
    if failures:
        print("bench.py: PARITY FAILURE: " + "; ".join(failures), file=sys.stderr)
        sys.exit(4)


if __name__ == "__main__":
    main()
