#!/usr/bin/env python3
"""Benchmark of the W4A16 linear hot path on one MI355X.

Workload (the headline decode configuration): the six W4A16 linears of one
OPT-6.7B decoder layer -- q/k/v/out 4096x4096, fc1 4096->16384, fc2 16384->4096 --
int4 weights in layout L1, group size 128, fp16 activations, M = 1 token.  One
"step" is one pass over the six linears of one layer, launched back to back on one
HIP stream through the C ABI (sq_w4a16_gemm).  Successive steps walk a pool of
distinct layers (> 256 MB in total), so every launch streams its weights from HBM
rather than from the Infinity Cache.

The metric is achieved GB/s: algorithmic bytes of a step
    sum over linears of  N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2   (= 107 102 208 B at M = 1)
divided by the time of a step, inputs already resident in HBM.

Also printed on the same JSON line:
  roofline      algorithmic bytes per launch / average launch duration of the decode
                kernel (HIP events on the launch stream over the timed region) against
                the 8 TB/s HBM peak
  cpu_baseline  the CPU restatement of the same path (oracle/) timed on this box's
                host cores on one step
  prefill       TFLOP/s of the M = 2048 linears (second half of the metric)
  decode_batch  GB/s of the same six linears at M = 4, 8, 16, 32

`--m`, `--group` and `--shapes` select other points of the same workload family.
"""
import argparse
import ctypes
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(REPO, "sparse-quant_amd"), os.path.join(REPO, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
MFMA_FP16_PEAK_TFLOPS = 2500.0
OPT67_LAYER = [("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096), ("out_proj", 4096, 4096),
               ("fc1", 16384, 4096), ("fc2", 4096, 16384)]  # (name, N, K)


def algorithmic_bytes(m, n, k, g):
    return n * k // 2 + (k // g) * n * 4 + m * k * 2 + m * n * 2


def make_linear(n, k, g, dev, gen):
    import torch
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=gen)
    z = torch.randint(0, 16, (n, k // g), device=dev, generator=gen).half() + 64
    s = (torch.randn((n, k // g), device=dev, generator=gen).abs() * 0.02 + 1e-3).half()
    zs = torch.stack([z, s], dim=-1).reshape(n, 2 * (k // g)).contiguous()
    return w, zs


def cpu_baseline(m, g, shapes):
    """One step of the same workload through the oracle's C restatement (all host cores)."""
    import numpy as np
    import w4a16_oracle as orc
    so = os.path.join(REPO, "oracle", "build", "libw4a16_oracle.so")
    total_bytes = sum(algorithmic_bytes(m, n, k, g) for _, n, k in shapes)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    data = []
    for idx, (_, n, k) in enumerate(shapes):
        d = orc.synth_linear(n, k, g, seed=idx)
        data.append((n, k, d["w_l1"], d["zs_l1"], orc.synth_x(m, k, seed=100 + idx)))
    if os.path.exists(so):
        lib = ctypes.CDLL(so)
        vp = ctypes.c_void_p

        def step():
            for n, k, w, zs, x in data:
                y = np.empty((m, n), dtype=np.float32)
                lib.sq_oracle_gemm_l1(vp(x.ctypes.data), vp(w.ctypes.data), vp(zs.ctypes.data), vp(y.ctypes.data),
                                      m, n, k, g)
        kind_note = "C restatement (oracle/w4a16_oracle.c, OpenMP)"
    else:
        threads = 1

        def step():
            for n, k, w, zs, x in data:
                orc.gemm_l1(x, w, zs, g)
        kind_note = "numpy restatement (oracle/w4a16_oracle.py)"
    step()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[1]
    return {"value": round(total_bytes / t / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "one step (six linears of one OPT-6.7B layer, M=%d, g=%d), median of 3, %s, %.1f ms per step"
                      % (m, g, kind_note, t * 1e3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--m", type=int, default=1, help="tokens per launch (decode batch)")
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--layers", type=int, default=8, help="distinct layers in the rotating weight pool")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the M=2048 TFLOP/s leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the fused-QKV, LUT-attention and end-to-end OPT-6.7B legs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch plain device copies of 256 MiB (reads 256 MiB, writes 256 MiB): the known-size "
                         "kernel that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    from sqamd import capi
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    lib = capi.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)
    m, g = args.m, args.group
    shapes = OPT67_LAYER

    pool = [[make_linear(n, k, g, dev, gen) for _, n, k in shapes] for _ in range(args.layers)]
    xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in {k for _, _, k in shapes}}
    ys = {n: torch.empty((m, n), dtype=torch.float16, device=dev) for n in {n for _, n, _ in shapes}}
    bytes_per_step = sum(algorithmic_bytes(m, n, k, g) for _, n, k in shapes)
    launches_per_step = len(shapes)

    stream = torch.cuda.Stream(device=dev)
    vp = ctypes.c_void_p
    st = vp(stream.cuda_stream)
    calls = []
    for layer in pool:
        row = []
        for (w, zs), (_, n, k) in zip(layer, shapes):
            row.append((vp(xs[k].data_ptr()), vp(w.data_ptr()), vp(zs.data_ptr()), vp(ys[n].data_ptr()), m, n, k, g,
                        capi.SQ_LAYOUT_L1, st))
        calls.append(row)
    gemm = lib.sq_w4a16_gemm

    def run_layer(i):
        for a in calls[i % len(calls)]:
            rc = gemm(*a)
            if rc != 0:
                raise RuntimeError("sq_w4a16_gemm failed: " + capi.strerror(rc))

    with torch.cuda.stream(stream):
        for i in range(len(calls)):
            run_layer(i)
        stream.synchronize()
        graph = None
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(len(calls)):
                    run_layer(i)
        per_replay = len(calls)

        def run_steps(count):
            if graph is None:
                for i in range(count):
                    run_layer(i)
                return count
            reps = (count + per_replay - 1) // per_replay
            for _ in range(reps):
                graph.replay()
            return reps * per_replay

        run_steps(args.warmup)
        stream.synchronize()
        steps = args.steps if graph is None else ((args.steps + per_replay - 1) // per_replay) * per_replay
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        done = run_steps(steps)
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        assert done == steps
        # The same step with the arithmetic taken away: sq_read_probe streams each weight with the GEMV's
        # own grid and access pattern and only folds the bits.  What it needs per step is the floor that
        # six dependent launches of these sizes leave to any kernel on this part.
        probe_out = torch.zeros(4096, dtype=torch.int32, device=dev)
        probe = capi.probes().sq_read_probe
        floor_us = None
        if m == 1 and not args.no_graph:
            def probe_layer(i):
                for a in calls[i % len(calls)]:
                    rc = probe(a[1], a[2], vp(probe_out.data_ptr()), a[5], a[6], a[7], st)
                    if rc != 0:
                        raise RuntimeError("sq_read_probe failed: " + capi.strerror(rc))
            for i in range(len(calls)):
                probe_layer(i)
            stream.synchronize()
            pgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(pgraph, stream=stream):
                for i in range(len(calls)):
                    probe_layer(i)
            reps = max(1, steps // per_replay)
            for _ in range(max(1, reps // 10)):
                pgraph.replay()
            p0 = torch.cuda.Event(enable_timing=True)
            p1 = torch.cuda.Event(enable_timing=True)
            p0.record(stream)
            for _ in range(reps):
                pgraph.replay()
            p1.record(stream)
            stream.synchronize()
            floor_us = p0.elapsed_time(p1) * 1e3 / (reps * per_replay)
    wall_ms = (t1 - t0) * 1e3
    gpu_ms = e0.elapsed_time(e1)
    ms_per_step = wall_ms / steps
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    launch_us = gpu_ms * 1e3 / (steps * launches_per_step)
    achieved = (bytes_per_step / launches_per_step) / (launch_us * 1e-6) / 1e9

    traffic = None
    tfile = os.path.join(REPO, "profiles", "gemv_decode_traffic.json")
    if os.path.exists(tfile) and m == 1 and g == 128:
        try:
            traffic = json.load(open(tfile)).get("hbm_bytes_per_launch")
        except Exception:
            traffic = None

    out = {
        "metric": "W4A16 linear GB/s at M=1 (OPT-6.7B decoder-layer linears, cold weights)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights x fp16 activations, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "OPT-6.7B decoder-layer linears (q,k,v,out 4096x4096; fc1 4096->16384; fc2 "
                               "16384->4096), W4A16 group %d, M=%d, one step = six launches, %d-layer rotating "
                               "weight pool (%.0f MB)" % (g, m, args.layers, args.layers * bytes_per_step / 1e6),
                   "launch": "hip-graph replay" if graph is not None else "eager", "bytes_per_step": bytes_per_step},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "kernel": "sq::gemv2_kernel (decode GEMV)", "avg_launch_us": round(launch_us, 3),
                     "bytes_per_launch": bytes_per_step // launches_per_step},
    }

    if floor_us is not None:
        out["read_only_floor"] = {
            "what": "the same six launches per step through sq_read_probe (weights and zeros_scales streamed with "
                    "the GEMV's grid and access pattern, no arithmetic, no activations, no output)",
            "us_per_step": round(floor_us, 2), "gbs": round(bytes_per_step / floor_us / 1e3, 1),
            "frac_of_hbm_peak": round(bytes_per_step / floor_us / 1e3 / HBM_PEAK_GBS, 4),
            "value_over_floor": round(floor_us / (ms_per_step * 1e3), 4)}

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration"] = {"kernel": "torch elementwise copy", "bytes_read": 256 << 20, "bytes_written": 256 << 20,
                              "launches": 5}
    if not args.no_prefill:
        out["prefill"] = prefill_leg(torch, capi, pool[0], shapes, g, dev, gen, stream)
    if not args.no_extras:
        # Additional, separately labelled legs; none of them feeds `value`.
        try:
            out["decode_batch"] = decode_batch_leg(torch, capi, pool, shapes, g, dev, gen, stream)
            out["fused_qkv"] = fused_qkv_leg(torch, capi, m, g, dev, gen, stream, args.layers, bytes_per_step)
            out["attention"] = attention_leg(torch, capi, dev)
            out["decode_attention"] = decode_attention_leg(torch, capi, dev)
            from sqamd import opt_decode
            out["e2e_opt67"] = opt_decode.run_e2e(batch=8, prompt=512, new_tokens=128)
        except Exception as exc:  # an extra leg must never hide the headline line
            out["extras_error"] = repr(exc)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(m, g, shapes)
    print(json.dumps(out))


def prefill_leg(torch, capi, layer, shapes, g, dev, gen, stream, m=2048, reps=10):
    """TFLOP/s of the M=2048 linears of the same layer (the prefill configuration).

    Reported beside each figure: the library's dense fp16 GEMM (torch.matmul, no int4 work at all) on
    the same shape in the same run, and the shader clock the chip sustains while the kernel runs
    (a one-wave probe on a second stream).  Matrix-heavy kernels run power-limited on this part, so the
    fraction of the nominal-clock peak is bounded well below 1 for any kernel; the dense figure shows
    where that bound sits for these shapes."""
    res = {}
    flops_total, time_total, dense_time_total = 0.0, 0.0, 0.0
    side = torch.cuda.Stream(device=dev)

    def timed(fn):
        for _ in range(3):
            fn()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        stream.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    def clock_under(fn, us):
        n = max(8, int(3000.0 / us))           # about 3 ms of load on either side of the probe
        for _ in range(n):
            fn()
        with torch.cuda.stream(side):
            ticks = capi.clock_probe(spins=200000, stream=side)
        for _ in range(2 * n):
            fn()
        torch.cuda.synchronize()
        c, r = int(ticks[0].item()), int(ticks[1].item())
        return round(c / (r / 100.0)) if r else None

    with torch.cuda.stream(stream):
        for (w, zs), (name, n, k) in list(zip(layer, shapes))[3:]:
            x = torch.randn((m, k), device=dev, generator=gen).half()
            y = torch.empty((m, n), dtype=torch.float16, device=dev)
            wd = torch.randn((k, n), device=dev, generator=gen).half()
            run = lambda: capi.gemm(x, w, zs, n, k, g, out=y, stream=stream)
            dense = lambda: torch.matmul(x, wd, out=y)
            us = timed(run)
            us_dense = timed(dense)
            fl = 2.0 * m * n * k
            res[name] = {"us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                         "shader_mhz_under_load": clock_under(run, us),
                         "dense_fp16_library_us": round(us_dense, 1),
                         "dense_fp16_library_tflops": round(fl / us_dense / 1e6, 1),
                         "dense_fp16_library_shader_mhz": clock_under(dense, us_dense)}
            flops_total += fl
            time_total += us
            dense_time_total += us_dense
            del wd
    tf = flops_total / time_total / 1e6
    tfd = flops_total / dense_time_total / 1e6
    # the other two token counts of the same configuration, aggregate only
    other = {}
    with torch.cuda.stream(stream):
        for m2 in (512, 4096):
            fl2, t2 = 0.0, 0.0
            for (w, zs), (name, n, k) in list(zip(layer, shapes))[3:]:
                x = torch.randn((m2, k), device=dev, generator=gen).half()
                y = torch.empty((m2, n), dtype=torch.float16, device=dev)
                ws = capi.workspace(m2, n, k, dev, stream)  # the extension passes one for up to 1024 tokens
                t2 += timed(lambda: capi.gemm_ws(x, w, zs, n, k, g, out=y, stream=stream, ws=ws))
                fl2 += 2.0 * m2 * n * k
            other["m%d" % m2] = {"tflops": round(fl2 / t2 / 1e6, 1),
                                 "frac_of_fp16_mfma_peak": round(fl2 / t2 / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4)}
    # What the matrix pipes sustain under the power limit: a loop of nothing but independent
    # v_mfma_f32_32x32x16_f16 on all CUs (one wave per SIMD), on N(0,1) operands and on zeros.
    roof = {}
    with torch.cuda.stream(stream):
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        iters = 20000
        for name, data in (("normal_operands", torch.randn(5120, device=dev, generator=gen).half()),
                           ("zero_operands", torch.zeros(5120, device=dev, dtype=torch.float16))):
            us = timed(lambda: capi.mfma_probe(data, cus, iters, stream=stream))
            ticks = capi.mfma_probe(data, cus, iters, stream=stream)
            torch.cuda.synchronize()
            roof[name] = {"tflops": round(cus * 4 * iters * 16 * 32768.0 / us / 1e6, 1),
                          "shader_mhz": round(float(ticks.double().median().item()) / us),
                          "cycles_per_mfma": round(float(ticks.double().median().item()) / (iters * 16), 2)}
    return {"m": m, "other_token_counts": other, "tflops": round(tf, 1), "frac_of_fp16_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4),
            "dense_fp16_library_tflops": round(tfd, 1), "vs_dense_fp16_library": round(tf / tfd, 3),
            "nominal_shader_mhz": 2400, "mfma_only_loop": roof,
            "frac_of_mfma_only_loop": round(tf / roof["normal_operands"]["tflops"], 4), "per_linear": res}


def decode_batch_leg(torch, capi, pool, shapes, g, dev, gen, stream):
    """GB/s of the same six linears at decode batches M = 4, 8, 16, 32 (the other batch sizes of the decode configuration), through
    the product dispatch with its workspace (sq_w4a16_gemm_ws), HIP-graph replay over the rotating pool."""
    res = {}
    for m in (4, 8, 16, 32):
        xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in {k for _, _, k in shapes}}
        ys = {n: torch.empty((m, n), dtype=torch.float16, device=dev) for n in {n for _, n, _ in shapes}}
        bytes_per_step = sum(algorithmic_bytes(m, n, k, g) for _, n, k in shapes)
        with torch.cuda.stream(stream):
            ws = capi.workspace(m, 16384, 16384, dev, stream)

            def run(i):
                for (w, zs), (_, n, k) in zip(pool[i % len(pool)], shapes):
                    capi.gemm_ws(xs[k], w, zs, n, k, g, out=ys[n], stream=stream, ws=ws)
            for i in range(len(pool)):
                run(i)
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(len(pool)):
                    run(i)
            for _ in range(5):
                graph.replay()
            reps = 60
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                graph.replay()
            e1.record(stream)
            stream.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * len(pool))
        res["m%d" % m] = {"us_per_step": round(us, 2), "gbs": round(bytes_per_step / us / 1e3, 1),
                          "frac_of_hbm_peak": round(bytes_per_step / us / 1e3 / HBM_PEAK_GBS, 4)}
    return res


def fused_qkv_leg(torch, capi, m, g, dev, gen, stream, layers, bytes_per_step):
    """The same step with q/k/v served by ONE launch on the row-concatenated weight [12288, 4096]
    (possible because layout L1 is row-major in N); four launches per step instead of six."""
    shapes = [("qkv_proj", 12288, 4096), ("out_proj", 4096, 4096), ("fc1", 16384, 4096), ("fc2", 4096, 16384)]
    pool = [[make_linear(n, k, g, dev, gen) for _, n, k in shapes] for _ in range(layers)]
    xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in (4096, 16384)}
    ys = {n: torch.empty((m, n), dtype=torch.float16, device=dev) for n in (12288, 4096, 16384)}
    steps = 2000
    with torch.cuda.stream(stream):
        def run(i):
            for (w, zs), (_, n, k) in zip(pool[i % layers], shapes):
                capi.gemm(xs[k], w, zs, n, k, g, out=ys[n], stream=stream)
        for i in range(layers):
            run(i)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(layers):
                run(i)
        for _ in range(10):
            graph.replay()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps // layers):
            graph.replay()
        e1.record(stream)
        stream.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (steps // layers * layers)
    return {"us_per_step": round(us, 2), "gbs": round(bytes_per_step / us / 1e3, 1), "launches_per_step": 4}


def attention_leg(torch, capi, dev):
    """LUT block-sparse attention at the BERT-large shape: batch 8, 16 heads, head dim 64, 64x64 blocks,
    ~25 % density with the diagonal block kept, non-causal; flops = 4 * kept blocks * 64 * 64 * D."""
    from sqamd.lut_layout import layout2lut_single_density, synth_layout
    res = {}
    for s in (512, 4096):
        z, h, d = 8, 16, 64
        lay = synth_layout(h, s // 64, 0.25, False, seed=1)
        lut = layout2lut_single_density(lay[None])[0].to(dev)
        kept = int(lay.sum().item()) * z
        q = torch.randn((z, h, s, d), device=dev).half()
        k = torch.randn_like(q)
        v = torch.randn_like(q)
        for _ in range(3):
            capi.lut_attention(q, k, v, lut, d ** -0.5, False)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            capi.lut_attention(q, k, v, lut, d ** -0.5, False)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / 20
        tf = 4.0 * kept * 64 * 64 * d / us / 1e6
        res["seq%d" % s] = {"us": round(us, 1), "tflops": round(tf, 1),
                            "frac_of_fp16_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4)}
    return res


def decode_attention_leg(torch, capi, dev, pool=8, reps=20):
    """Dense decode attention of the end-to-end configuration: batch 8, 32 heads, head dim 128, 640 cache
    rows (639 valid + the appended one), fp16; algorithmic bytes = K and V rows read once; caches rotate
    through a pool larger than the last-level cache; HIP-graph replay.  torch's SDPA on the same tensors
    (which also needs two copy launches for the append, not timed) is shown beside it."""
    b, h, d, rows = 8, 32, 128, 640
    qs = [torch.randn((b, h, 1, d), device=dev).half() for _ in range(pool)]
    kcs = [torch.randn((b, h, rows, d), device=dev).half() for _ in range(pool)]
    vcs = [torch.randn((b, h, rows, d), device=dev).half() for _ in range(pool)]
    pos = torch.tensor([rows - 1], device=dev)
    scale = d ** -0.5

    def ours():
        for i in range(pool):
            capi.decode_attention(qs[i], kcs[i], vcs[i], pos, scale, k_new=qs[i], v_new=qs[i])

    def sdpa():
        for i in range(pool):
            torch.nn.functional.scaled_dot_product_attention(qs[i], kcs[i], vcs[i])

    res = {"shape": "B=8 H=32 D=128 rows=640", "bytes": 2 * b * h * rows * d * 2}
    for name, fn in (("kernel", ours), ("torch_sdpa", sdpa)):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * pool)
        res[name] = {"us": round(us, 2), "gbs": round(res["bytes"] / us / 1e3, 1),
                     "frac_of_hbm_peak": round(res["bytes"] / us / 1e3 / HBM_PEAK_GBS, 4)}
    return res


if __name__ == "__main__":
    main()
