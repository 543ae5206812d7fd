#!/usr/bin/env python3
"""Benchmark of the W4A16 linear hot path on one MI355X.

Workload (the headline decode configuration): the six W4A16 linears of one
OPT-6.7B decoder layer -- q/k/v/out 4096x4096, fc1 4096->16384, fc2 16384->4096 --
int4 weights in layout L1, group size 128, fp16 activations, M = 1 token.  One
"step" is one pass over the six linears of one layer on one HIP stream through the
C ABI: sq_w4a16_gemv_sequence with the layer's data flow (q, k and v share a launch;
out_proj, fc1 and fc2 get one each: four launches), or with --per-linear one
sq_w4a16_gemm per linear (six launches).  Successive steps walk a pool of distinct
layers (> 256 MB in total), so every launch streams its weights from HBM rather than
from the Infinity Cache.

The metric is achieved GB/s: algorithmic bytes of a step
    sum over linears of  N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2   (= 107 102 208 B at M = 1)
divided by the time of a step, inputs already resident in HBM.

Also printed on the same JSON line:
  parity        every leg's kernels are checked against the CPU oracle on sampled rows before they
                are timed (gate: max|Y - Y_ref| <= 1e-2 * max|Y_ref|, dequant bit-exact); a failed
                gate ends the run with an error instead of a number
  roofline      algorithmic bytes per launch / average launch duration of the decode
                kernel (HIP events on the launch stream over the timed region) against
                the 8 TB/s HBM peak
  long_window   the same step timed over 3200 steps whatever --steps says (the driver's --steps may
                be as low as 20, i.e. under a millisecond)
  cpu_baseline  the reference CPU path (torch dequant to fp32 + matmul, timed separately) on this
                box's host cores on one step, with the C restatement of the oracle as a second figure
  config1       the single q_proj-shaped linear with group size 64 at M = 1 and 16
  prefill       TFLOP/s of the M = 2048 linears, OPT and Llama-MLP shapes (second half of the metric)
  decode_batch  GB/s of the same six linears at M = 4, 8, 16, 32
  sequence      the same six linears through sq_w4a16_gemv_sequence

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


def decode_kernel_source_sha16():
    """First 16 hex digits of the SHA-256 over the sources of the single-token decode kernel."""
    import hashlib
    h = hashlib.sha256()
    for name in ("sq_gemv2.hip", "sq_common.h"):
        with open(os.path.join(REPO, "sparse-quant_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def algorithmic_bytes(m, n, k, g):
    return n * k // 2 + (k // g) * n * 4 + m * k * 2 + m * n * 2


def make_linear(n, k, g, dev, gen):
    import torch
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=gen)
    z = torch.randint(0, 16, (n, k // g), device=dev, generator=gen).half() + 64
    s = (torch.randn((n, k // g), device=dev, generator=gen).abs() * 0.02 + 1e-3).half()
    zs = torch.stack([z, s], dim=-1).reshape(n, 2 * (k // g)).contiguous()
    return w, zs


PARITY_GATE = 1e-2


class ParityError(RuntimeError):
    pass


def parity_linear(torch, w, zs, n, k, g, x, y, seed=0, rows=64, tokens=32):
    """max|Y - Y_ref| / max|Y_ref| of a GPU result against the CPU oracle on sampled output rows (and,
    with many tokens, sampled token rows): the oracle dequantises those rows of the weight and forms
    the fp32 product.  Outside every timed region."""
    import numpy as np
    import w4a16_oracle as orc
    rng = np.random.default_rng(seed)
    ridx = np.sort(rng.choice(n, size=min(rows, n), replace=False))
    m = x.shape[0]
    tidx = np.arange(m) if m <= tokens else np.sort(rng.choice(m, size=tokens, replace=False))
    # Whole tensors come to the host and are sampled there, so that the check does not depend on the ordering
    # of index uploads and device-side gathers (a run under rocprofv3 --pmc once sampled non-finite data that way).
    torch.cuda.synchronize()
    w_hat = orc.dequant_l1(w.cpu().numpy()[ridx], zs.cpu().numpy()[ridx], g)
    y_ref = orc.gemm_ref(x.cpu().numpy()[tidx], w_hat)
    got = y.float().cpu().numpy()[tidx][:, ridx]
    if not np.all(np.isfinite(got)) or not np.all(np.isfinite(y_ref)):
        raise ParityError("parity gate: non-finite data (sampled result %d, activations %d, dequantised weight rows %d "
                          "of %d x %d non-finite)" % (np.sum(~np.isfinite(got)), np.sum(~np.isfinite(x.cpu().numpy())),
                                                      np.sum(~np.isfinite(w_hat)), n, k))
    return float(np.max(np.abs(got - y_ref)) / np.max(np.abs(y_ref)))


def parity_dequant(torch, capi, w, zs, n, k, g, seed=0, rows=64):
    """Bit-exactness of the dequant kernel on sampled rows of a weight."""
    import numpy as np
    import w4a16_oracle as orc
    rng = np.random.default_rng(seed)
    ridx = np.sort(rng.choice(n, size=min(rows, n), replace=False))
    torch.cuda.synchronize()
    want = orc.dequant_l1(w.cpu().numpy()[ridx], zs.cpu().numpy()[ridx], g)
    got = capi.dequant(w, zs, n, k, g).cpu().numpy()[ridx]
    return bool(np.array_equal(got.view(np.int16), want.view(np.int16)))


def gate(err, what):
    if not err <= PARITY_GATE:
        raise ParityError("parity gate failed for %s: max rel err %.3e > %.0e" % (what, err, PARITY_GATE))
    return err


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_reference_torch(m, g, shapes, reps=3):
    """The reference's CPU path on the host cores: W = (q.float() - z.float()) * s.float() ("dequant"), then
    Y = X.float() @ W.t() ("matmul"), timed separately, median of `reps`, one step = the six linears."""
    import torch
    gen = torch.Generator()
    gen.manual_seed(0)
    data = []
    for _, n, k in shapes:
        q = torch.randint(0, 16, (n, k), dtype=torch.uint8, generator=gen)
        z = torch.randint(0, 16, (n, k // g), dtype=torch.uint8, generator=gen)
        s = (torch.randn((n, k // g), generator=gen).abs() * 0.02 + 1e-3).half()
        x = torch.randn((m, k), generator=gen).half()
        data.append((q, z, s, x))
    deq_t, mm_t = [], []
    for _ in range(reps + 1):
        td = tm = 0.0
        for q, z, s, x in data:
            t0 = time.perf_counter()
            w = (q.float() - z.float().repeat_interleave(g, 1)) * s.float().repeat_interleave(g, 1)
            t1 = time.perf_counter()
            y = x.float() @ w.t()
            t2 = time.perf_counter()
            td += t1 - t0
            tm += t2 - t1
            del w, y
        deq_t.append(td)
        mm_t.append(tm)
    med = lambda v: sorted(v[1:])[len(v[1:]) // 2]  # the first repetition warms the allocator
    return med(deq_t), med(mm_t), torch.get_num_threads()


def cpu_baseline(m, g, shapes):
    """One step of the same workload on the host: the reference's torch recipe (dequant to fp32 + matmul) and,
    as a second figure, the oracle's C restatement (all host cores)."""
    total_bytes = sum(algorithmic_bytes(m, n, k, g) for _, n, k in shapes)
    total_flops = sum(2.0 * m * n * k for _, n, k in shapes)
    deq_s, mm_s, threads = cpu_reference_torch(m, g, shapes)
    port = cpu_baseline_c_port(m, g, shapes)
    t = deq_s + mm_s
    return {"value": round(total_bytes / t / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "one step (six linears of one OPT-6.7B layer, M=%d, g=%d), median of 3: torch dequant to fp32 "
                      "%.1f ms + torch matmul %.1f ms = %.1f ms per step (the reference's CPU recipe restated with "
                      "torch ops on the host)" % (m, g, deq_s * 1e3, mm_s * 1e3, t * 1e3),
            "dequant_ms": round(deq_s * 1e3, 2), "matmul_ms": round(mm_s * 1e3, 2),
            "gflops": round(total_flops / t / 1e9, 3), "cpu_model": cpu_model(), "os_cpu_count": os.cpu_count(),
            "torch_threads": threads, "c_port": port}


def cpu_baseline_c_port(m, g, shapes):
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
    return {"value": round(total_bytes / t / 1e9, 3), "unit": "GB/s", "cores": threads,
            "sample": "one step, median of 3, %s, %.1f ms per step" % (kind_note, t * 1e3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--m", type=int, default=1, help="tokens per launch (decode batch)")
    ap.add_argument("--group", type=int, default=128)
    ap.add_argument("--layers", type=int, default=8, help="distinct layers in the rotating weight pool")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--per-linear", action="store_true",
                    help="headline through one sq_w4a16_gemm call per linear (six launches per step) instead of "
                         "sq_w4a16_gemv_sequence")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the M=2048 TFLOP/s leg")
    ap.add_argument("--prefill-other-tokens", default="64,128,256,512,1024,4096",
                    help="token counts the prefill leg also measures (comma separated; a counter run names fewer)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the fused-QKV, LUT-attention and end-to-end OPT-6.7B legs")
    ap.add_argument("--prefill-shape", default=None,
                    help="run ONLY one linear of the prefill leg at --m tokens (out_proj, fc1, fc2, llama_mlp_up or "
                         "llama_mlp_down) and print its own JSON line: under rocprofv3 --kernel-trace --stats every "
                         "kernel row of such a run is one shape")
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
    if args.prefill_shape is not None:
        print(json.dumps(prefill_one_shape(torch, capi, args.prefill_shape, m, g, dev, gen)))
        return

    pool = [[make_linear(n, k, g, dev, gen) for _, n, k in shapes] for _ in range(args.layers)]
    xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in {k for _, _, k in shapes}}
    ys = [torch.empty((m, n), dtype=torch.float16, device=dev) for _, n, _ in shapes]  # one output per linear
    bytes_per_step = sum(algorithmic_bytes(m, n, k, g) for _, n, k in shapes)
    # The step goes through sq_w4a16_gemv_sequence with the data flow of the decoder layer: q, k and v do not depend
    # on each other (one launch for the three), out_proj, fc1 and fc2 each consume an earlier output (a launch
    # each): four launches per step.  With more than 4 tokens, or --per-linear, one sq_w4a16_gemm per linear.
    use_sequence = (m <= 4) and not args.per_linear
    depends = [False, False, False, True, True, True]
    launches_per_step = 4 if use_sequence else len(shapes)

    stream = torch.cuda.Stream(device=dev)
    vp = ctypes.c_void_p
    st = vp(stream.cuda_stream)
    calls = []
    for layer in pool:
        row = []
        for idx, ((w, zs), (_, n, k)) in enumerate(zip(layer, shapes)):
            row.append((vp(xs[k].data_ptr()), vp(w.data_ptr()), vp(zs.data_ptr()), vp(ys[idx].data_ptr()), m, n, k, g,
                        capi.SQ_LAYOUT_L1, st))
        calls.append(row)
    gemm = lib.sq_w4a16_gemm
    seqs = None
    if use_sequence:
        seqs = [capi.LinearSequence([dict(x=xs[k], w=w, zs=zs, y=ys[idx], n=n, k=k, group_size=g, depends=depends[idx])
                                     for idx, ((w, zs), (_, n, k)) in enumerate(zip(layer, shapes))], m, dev,
                                    workspace=False) for layer in pool]

    def run_layer(i):
        if seqs is not None:
            seqs[i % len(seqs)].run(stream=stream)
            return
        for a in calls[i % len(calls)]:
            rc = gemm(*a)
            if rc != 0:
                raise RuntimeError("sq_w4a16_gemm failed: " + capi.strerror(rc))

    torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
    with torch.cuda.stream(stream):
        for i in range(len(calls)):
            run_layer(i)
        stream.synchronize()
        # Parity gate, outside every timed region: every linear of the first layer against the CPU oracle on
        # sampled output rows, and the dequant kernel bit for bit on two of the weights.
        parity_err, deq_exact = 0.0, True
        for li in (0, len(calls) - 1):
            for y in ys:
                y.fill_(float("nan"))
            run_layer(li)
            stream.synchronize()
            for idx, ((w, zs), (name, n, k)) in enumerate(zip(pool[li], shapes)):
                parity_err = max(parity_err, gate(parity_linear(torch, w, zs, n, k, g, xs[k], ys[idx], seed=idx),
                                                  "%s at M=%d" % (name, m)))
        for idx in (0, len(shapes) - 2):
            w, zs = pool[0][idx]
            deq_exact = deq_exact and parity_dequant(torch, capi, w, zs, shapes[idx][1], shapes[idx][2], g, seed=idx)
        if not deq_exact:
            raise ParityError("parity gate failed: dequant is not bit-exact")
        per_replay = len(calls)
        graphs = {}

        unit = 64  # steps per replayed graph: eight passes over the pool, so that gaps between graph launches are rare

        def graph_of(count):
            """A captured graph of `count` consecutive steps (cycling through the layers of the pool)."""
            if count not in graphs:
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=stream):
                    for i in range(count):
                        run_layer(i)
                graphs[count] = gr
            return graphs[count]

        def run_steps(count):
            """Exactly `count` steps: whole passes over the pool plus one shorter graph for the rest."""
            if args.no_graph:
                for i in range(count):
                    run_layer(i)
                return
            full, rest = divmod(count, unit)
            for _ in range(full):
                graphs[unit].replay()
            if rest:
                graphs[rest].replay()

        if not args.no_graph:
            graph_of(unit)
            for c in {args.steps % unit, args.warmup % unit} - {0}:
                graph_of(c)
        graph = graphs.get(unit)
        steps = args.steps
        run_steps(args.warmup)
        stream.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        # The timed region is the GPU time of exactly `steps` steps between two events on the launch stream.  It is
        # queued directly behind a longer untimed-for-the-headline window of the same steps (3200 of them, with
        # events of its own: `long_window`), without a host synchronisation in between: the host has then
        # submitted the timed steps before the first event fires and the chip is at its working clocks, which
        # matters when --steps is small (20 steps are about 0.6 ms, less than the host needs to submit them
        # after an idle period).
        long_window = None
        t0 = time.perf_counter()
        if graph is not None:
            reps_long = 50
            l0 = torch.cuda.Event(enable_timing=True)
            l1 = torch.cuda.Event(enable_timing=True)
            l0.record(stream)
            for _ in range(reps_long):
                graph.replay()
            l1.record(stream)
        e0.record(stream)
        run_steps(steps)
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if graph is not None:
            us_long = l0.elapsed_time(l1) * 1e3 / (reps_long * unit)
            long_window = {"steps": reps_long * unit, "us_per_step": round(us_long, 3),
                           "gbs": round(bytes_per_step / us_long / 1e3, 1),
                           "frac_of_hbm_peak": round(bytes_per_step / us_long / 1e3 / HBM_PEAK_GBS, 4)}
        # The same step with one sq_w4a16_gemm launch per linear (six launches), for comparison.
        per_linear = None
        if seqs is not None and graph is not None:
            def six(i):
                for a in calls[i]:
                    rc = gemm(*a)
                    if rc != 0:
                        raise RuntimeError("sq_w4a16_gemm failed: " + capi.strerror(rc))
            for i in range(len(calls)):
                six(i)
            stream.synchronize()
            g6 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g6, stream=stream):
                for i in range(len(calls)):
                    six(i)
            for _ in range(20):
                g6.replay()
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record(stream)
            for _ in range(200):
                g6.replay()
            s1.record(stream)
            stream.synchronize()
            us6 = s0.elapsed_time(s1) * 1e3 / (200 * per_replay)
            per_linear = {"launches_per_step": 6, "us_per_step": round(us6, 3), "gbs": round(bytes_per_step / us6 / 1e3, 1),
                          "frac_of_hbm_peak": round(bytes_per_step / us6 / 1e3 / HBM_PEAK_GBS, 4)}
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
            reps = max(50, steps // per_replay)
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
    wall_ms = (t1 - t0) * 1e3  # host wall clock over the long window and the timed steps: reported, not used
    gpu_ms = e0.elapsed_time(e1)
    ms_per_step = gpu_ms / steps
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    launch_us = gpu_ms * 1e3 / (steps * launches_per_step)
    achieved = (bytes_per_step / launches_per_step) / (launch_us * 1e-6) / 1e9

    # HBM traffic per launch comes from a counter run of this command (rocprofv3 --pmc cannot run inside the timed
    # process); the stored figure is used only while the decode kernel's source is the one it was measured on.
    traffic, traffic_note = None, "no stored counter run"
    tfile = os.path.join(REPO, "profiles", "gemv_decode_traffic.json")
    if os.path.exists(tfile) and m == 1 and g == 128 and use_sequence:
        try:
            stored = json.load(open(tfile))
            if stored.get("decode_kernel_source_sha16") == decode_kernel_source_sha16():
                traffic = stored.get("hbm_bytes_per_launch")
                traffic_note = ("stored from profiles/gemv_decode_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                "of this command, scaled by a 256 MiB copy; same decode kernel source), not measured in "
                                "this run")
            else:
                traffic_note = ("profiles/gemv_decode_traffic.json was measured on another version of the decode "
                                "kernel's source: not reported")
        except Exception:
            traffic = None

    out = {
        "metric": "W4A16 linear GB/s at M=1 (OPT-6.7B decoder-layer linears, cold weights)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "timed_region": "HIP events on the launch stream around exactly `steps` "
        "steps, queued behind the 3200 steps of long_window (host wall clock over both: %.3f ms)" % wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights x fp16 activations, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "OPT-6.7B decoder-layer linears (q,k,v,out 4096x4096; fc1 4096->16384; fc2 "
                               "16384->4096), W4A16 group %d, M=%d, one step = the six linears through %s, %d-layer "
                               "rotating weight pool (%.0f MB)"
                               % (g, m, "sq_w4a16_gemv_sequence with the layer's data flow (q, k, v in one launch; out_proj, "
                                        "fc1, fc2 a launch each: four launches)" if use_sequence else
                                  "one sq_w4a16_gemm each (six launches)", args.layers, args.layers * bytes_per_step / 1e6),
                   "launch": "hip-graph replay" if graph is not None else "eager", "bytes_per_step": bytes_per_step},
        "parity": {"max_rel_err": round(parity_err, 6), "gate": PARITY_GATE, "dequant_bit_exact": deq_exact,
                   "checked": "every linear of two layers of the pool against the CPU oracle on 64 sampled output rows "
                              "(fp32 reference of the dequantised rows), dequant kernel bit for bit on 64 rows of two "
                              "weights; every other leg below carries its own parity_max_rel_err, checked the same way "
                              "before it is timed"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_note,
                     "kernel": "sq::gemv2_kernel / sq::gemv2_group_kernel (decode GEMV)",
                     "launches_per_step": launches_per_step, "avg_launch_us": round(launch_us, 3),
                     "bytes_per_launch": bytes_per_step // launches_per_step},
    }

    if long_window is not None:
        out["long_window"] = long_window
    if per_linear is not None:
        out["per_linear_launches"] = per_linear
    if floor_us is not None:
        out["read_only_floor"] = {
            "what": "six launches per step (one per linear) through sq_read_probe (weights and zeros_scales streamed "
                    "with the single-linear GEMV's grid and access pattern, no arithmetic, no activations, no output)",
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
        other_tokens = tuple(int(t) for t in args.prefill_other_tokens.split(",") if t.strip())
        out["prefill"] = prefill_leg(torch, capi, pool[0], shapes, g, dev, gen, stream, other_tokens=other_tokens)
    if not args.no_extras:
        # Additional, separately labelled legs; none of them feeds `value`.
        try:
            out["decode_batch"] = decode_batch_leg(torch, capi, pool, shapes, g, dev, gen, stream)
            out["config1"] = config1_leg(torch, capi, dev, gen, stream)
            out["layernorm_fused"] = ln_fused_leg(torch, capi, pool, shapes, g, dev, gen, stream)
            out["gated_mlp"] = gated_mlp_leg(torch, capi, g, dev, gen, stream)
            if m <= 4:
                out["sequence"] = sequence_leg(torch, capi, pool, shapes, m, g, dev, gen, stream, bytes_per_step)
            out["fused_qkv"] = fused_qkv_leg(torch, capi, m, g, dev, gen, stream, args.layers, bytes_per_step)
            out["attention"] = attention_leg(torch, capi, dev)
            out["decode_attention"] = decode_attention_leg(torch, capi, dev)
            from sqamd import opt_decode
            out["e2e_opt67"] = opt_decode.run_e2e(batch=8, prompt=512, new_tokens=128)
            # The end-to-end harness draws smaller scales than BASELINE's so that 32 random layers stay finite.
            # What that changes is bounded here: two layers (which BASELINE's scales survive) with either
            # distribution, same kernels, same bytes.
            pair = {}
            for label, kw in (("baseline_scales", dict(scale_std=0.02, scale_min=1e-3)), ("harness_scales", {})):
                r = opt_decode.run_e2e(batch=8, prompt=512, new_tokens=33, layers=2, lut_density=None, **kw)
                pair[label] = {"decode_ms_per_step": r["decode_ms_per_step"], "prefill_ms": r["prefill_ms"],
                               "logits_finite": r["logits_finite"], "weights": r["weights"]}
            pair["decode_ratio"] = round(pair["baseline_scales"]["decode_ms_per_step"] /
                                         pair["harness_scales"]["decode_ms_per_step"], 4)
            out["e2e_opt67"]["two_layers_either_scale_distribution"] = pair
            out["kernel_picker"] = picker_leg(torch, capi, g, dev, gen, stream)  # last: it records choices
        except ParityError:
            raise
        except Exception as exc:  # an extra leg must never hide the headline line
            out["extras_error"] = repr(exc)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(m, g, shapes)
    print(json.dumps(out))


PREFILL_SHAPES = {"out_proj": (4096, 4096), "fc1": (16384, 4096), "fc2": (4096, 16384),
                  "llama_mlp_up": (11008, 4096), "llama_mlp_down": (4096, 11008)}  # name -> (N, K)


def prefill_one_shape(torch, capi, name, m, g, dev, gen):
    """One linear of the prefill leg by itself: parity gate, 20 ms of warm-up, then a window of about 40 ms timed
    with HIP events on the launch stream.  Nothing else runs, so a kernel trace of the process has one row per
    kernel and that row is this shape."""
    n, k = PREFILL_SHAPES[name]
    w, zs = make_linear(n, k, g, dev, gen)
    x = torch.randn((m, k), device=dev, generator=gen).half()
    y = torch.empty((m, n), dtype=torch.float16, device=dev)
    stream = torch.cuda.Stream(device=dev)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        run = lambda: capi.gemm(x, w, zs, n, k, g, out=y, stream=stream)
        run()
        stream.synchronize()
        err = gate(parity_linear(torch, w, zs, n, k, g, x, y, seed=n + k), "%s at M=%d" % (name, m))

        def window(count):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(count):
                run()
            e1.record(stream)
            stream.synchronize()
            return e0.elapsed_time(e1) * 1e3 / count
        est = max(window(3), 1.0)
        window(max(3, min(2000, int(20000.0 / est))))
        launches = max(10, min(4000, int(40000.0 / est)))
        us = window(launches)
    fl = 2.0 * m * n * k
    return {"prefill_shape": name, "m": m, "n": n, "k": k, "group": g, "flops_per_launch": fl, "timed_launches": launches,
            "us": round(us, 2), "tflops": round(fl / us / 1e6, 1),
            "frac_of_fp16_mfma_peak": round(fl / us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4), "parity_max_rel_err": round(err, 6)}


def prefill_leg(torch, capi, layer, shapes, g, dev, gen, stream, m=2048, reps=10, other_tokens=(512, 4096)):
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
        # A first estimate from a few launches, then a warm-up of about 20 ms and a timed window of about 40 ms
        # (at least `reps` launches): after an idle gap the clocks take milliseconds to settle, and a window of a
        # few launches reads up to 20 % low.
        def window(n):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(n):
                fn()
            e1.record(stream)
            stream.synchronize()
            return e0.elapsed_time(e1) * 1e3 / n
        est = max(window(3), 1.0)
        window(max(3, min(2000, int(20000.0 / est))))
        return window(max(reps, min(4000, int(40000.0 / est))))

    def clock_under(fn, us):
        n = max(8, int(3000.0 / us))           # about 3 ms of load on either side of the probe
        for _ in range(n):
            fn()
        torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
        with torch.cuda.stream(side):
            ticks = capi.clock_probe(spins=200000, stream=side)
        for _ in range(2 * n):
            fn()
        torch.cuda.synchronize()
        c, r = int(ticks[0].item()), int(ticks[1].item())
        return round(c / (r / 100.0)) if r else None

    # q/k/v/out share one shape: out_proj stands for the four; then fc1, fc2 and the Llama-2-7B MLP shapes
    work = [(w, zs, name, n, k) for (w, zs), (name, n, k) in list(zip(layer, shapes))[3:]]
    for name, n, k in (("llama_mlp_up", 11008, 4096), ("llama_mlp_down", 4096, 11008)):
        w, zs = make_linear(n, k, g, dev, gen)
        work.append((w, zs, name, n, k))
    opt_names = {name for _, _, name, _, _ in work[:3]}
    worst = 0.0
    torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
    with torch.cuda.stream(stream):
        for w, zs, name, n, k in work:
            x = torch.randn((m, k), device=dev, generator=gen).half()
            y = torch.empty((m, n), dtype=torch.float16, device=dev)
            wd = torch.randn((k, n), device=dev, generator=gen).half()
            run = lambda: capi.gemm(x, w, zs, n, k, g, out=y, stream=stream)
            dense = lambda: torch.matmul(x, wd, out=y)
            run()
            stream.synchronize()
            err = gate(parity_linear(torch, w, zs, n, k, g, x, y, seed=n + k), "%s at M=%d" % (name, m))
            worst = max(worst, err)
            us = timed(run)
            us_dense = timed(dense)
            fl = 2.0 * m * n * k
            res[name] = {"us": round(us, 1), "tflops": round(fl / us / 1e6, 1), "parity_max_rel_err": round(err, 6),
                         "shader_mhz_under_load": clock_under(run, us),
                         "dense_fp16_library_us": round(us_dense, 1),
                         "dense_fp16_library_tflops": round(fl / us_dense / 1e6, 1),
                         "dense_fp16_library_shader_mhz": clock_under(dense, us_dense)}
            if name in opt_names:  # the aggregate stays the OPT-6.7B set, comparable from run to run
                flops_total += fl
                time_total += us
                dense_time_total += us_dense
            del wd
    tf = flops_total / time_total / 1e6
    tfd = flops_total / dense_time_total / 1e6
    # other token counts of the same configuration (64..1024: the range between decode and prefill), aggregate
    # and per-linear time
    other = {}
    torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
    with torch.cuda.stream(stream):
        for m2 in other_tokens:
            fl2, t2 = 0.0, 0.0
            per = {}
            for w, zs, name, n, k in work:
                x = torch.randn((m2, k), device=dev, generator=gen).half()
                y = torch.empty((m2, n), dtype=torch.float16, device=dev)
                ws = capi.workspace(m2, n, k, dev, stream)  # the extension passes one for up to 1024 tokens
                capi.gemm_ws(x, w, zs, n, k, g, out=y, stream=stream, ws=ws)
                stream.synchronize()
                err = gate(parity_linear(torch, w, zs, n, k, g, x, y, seed=m2 + n), "%s at M=%d" % (name, m2))
                worst = max(worst, err)
                us2 = timed(lambda: capi.gemm_ws(x, w, zs, n, k, g, out=y, stream=stream, ws=ws))
                per[name] = {"us": round(us2, 1), "tflops": round(2.0 * m2 * n * k / us2 / 1e6, 1)}
                if name in opt_names:
                    t2 += us2
                    fl2 += 2.0 * m2 * n * k
            other["m%d" % m2] = {"tflops": round(fl2 / t2 / 1e6, 1),
                                 "frac_of_fp16_mfma_peak": round(fl2 / t2 / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4),
                                 "per_linear": per}
    # What the matrix pipes sustain under the power limit: a loop of nothing but independent
    # v_mfma_f32_32x32x16_f16 on all CUs (one wave per SIMD), on N(0,1) operands and on zeros.
    roof = {}
    torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
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
    return {"m": m, "aggregate_over": "out_proj (4096x4096), fc1, fc2; the Llama MLP shapes are listed per linear",
            "parity_max_rel_err": round(worst, 6),
            "other_token_counts": other, "tflops": round(tf, 1), "frac_of_fp16_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4),
            "dense_fp16_library_tflops": round(tfd, 1), "vs_dense_fp16_library": round(tf / tfd, 3),
            "nominal_shader_mhz": 2400, "mfma_only_loop": roof,
            "frac_of_mfma_only_loop": round(tf / roof["normal_operands"]["tflops"], 4), "per_linear": res}


def decode_batch_leg(torch, capi, pool, shapes, g, dev, gen, stream):
    """GB/s of the same six linears at decode batches M = 4, 8, 16, 32 (the other batch sizes of the decode configuration),
    through sq_w4a16_gemv_sequence like the headline (q, k, v in one launch, the others a launch each, split-K
    workspace for 5..32 tokens); HIP-graph replay over the rotating pool."""
    res = {}
    for m in (4, 8, 16, 32):
        xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in {k for _, _, k in shapes}}
        ys = {n: torch.empty((m, n), dtype=torch.float16, device=dev) for n in {n for _, n, _ in shapes}}
        bytes_per_step = sum(algorithmic_bytes(m, n, k, g) for _, n, k in shapes)
        torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
        with torch.cuda.stream(stream):
            ws = capi.workspace(m, 16384, 16384, dev, stream)
            seqs = None
            if m <= 32:
                yl = [torch.empty((m, n), dtype=torch.float16, device=dev) for _, n, _ in shapes]
                dep = [False, False, False, True, True, True]
                seqs = [capi.LinearSequence([dict(x=xs[k], w=w, zs=zs, y=yl[i], n=n, k=k, group_size=g, depends=dep[i])
                                             for i, ((w, zs), (_, n, k)) in enumerate(zip(layer, shapes))], m, dev,
                                            workspace=False) for layer in pool]
                for sq in seqs:  # one shared split-K workspace (the calls are ordered on one stream)
                    sq.ws = ws

            def run(i):
                if seqs is not None:
                    seqs[i % len(pool)].run(stream=stream)
                    return
                for (w, zs), (_, n, k) in zip(pool[i % len(pool)], shapes):
                    capi.gemm_ws(xs[k], w, zs, n, k, g, out=ys[n], stream=stream, ws=ws)
            for i in range(len(pool)):
                run(i)
            stream.synchronize()
            worst = 0.0
            if seqs is not None:
                seqs[0].run(stream=stream)
                stream.synchronize()
            for idx, ((w, zs), (name, n, k)) in enumerate(zip(pool[0], shapes)):
                if seqs is not None:
                    ytmp = yl[idx]
                else:
                    if idx in (1, 2):
                        continue  # same shape and kernel as q_proj
                    ytmp = torch.empty((m, n), dtype=torch.float16, device=dev)
                    capi.gemm_ws(xs[k], w, zs, n, k, g, out=ytmp, stream=stream, ws=ws)
                    stream.synchronize()
                worst = max(worst, gate(parity_linear(torch, w, zs, n, k, g, xs[k], ytmp, seed=idx + m),
                                        "%s at M=%d" % (name, m)))
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(len(pool)):
                    run(i)
            for _ in range(60):  # about 20 ms: the clocks have settled when the timed window starts
                graph.replay()
            reps = 120
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                graph.replay()
            e1.record(stream)
            stream.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * len(pool))
        res["m%d" % m] = {"us_per_step": round(us, 2), "gbs": round(bytes_per_step / us / 1e3, 1),
                          "frac_of_hbm_peak": round(bytes_per_step / us / 1e3 / HBM_PEAK_GBS, 4),
                          "launches_per_step": 4 if seqs is not None else 6, "parity_max_rel_err": round(worst, 6)}
    return res


def config1_leg(torch, capi, dev, gen, stream, g=64, n=4096, k=4096, copies=32):
    """The single q_proj-shaped linear with group size 64 (4096 x 4096) at M = 1 and M = 16, cold weights
    (32 copies = 302 MB rotating), HIP-graph replay, product dispatch with workspace."""
    pool = [make_linear(n, k, g, dev, gen) for _ in range(copies)]
    res = {"shape": "N=4096 K=4096 group 64", "pool_mb": round(copies * algorithmic_bytes(1, n, k, g) / 1e6)}
    for m in (1, 16):
        x = torch.randn((m, k), device=dev, generator=gen).half()
        y = torch.empty((m, n), dtype=torch.float16, device=dev)
        nbytes = algorithmic_bytes(m, n, k, g)
        torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
        with torch.cuda.stream(stream):
            ws = capi.workspace(m, n, k, dev, stream)
            run = lambda: [capi.gemm_ws(x, w, zs, n, k, g, out=y, stream=stream, ws=ws) for w, zs in pool]
            run()
            stream.synchronize()
            err = gate(parity_linear(torch, pool[-1][0], pool[-1][1], n, k, g, x, y, seed=m), "config 1 at M=%d" % m)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                run()
            for _ in range(5):
                graph.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(50):
                graph.replay()
            e1.record(stream)
            stream.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (50 * copies)
        res["m%d" % m] = {"us": round(us, 3), "gbs": round(nbytes / us / 1e3, 1),
                          "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                          "parity_max_rel_err": round(err, 6)}
    return res


def ln_fused_leg(torch, capi, pool, shapes, g, dev, gen, stream, m=8):
    """LayerNorm + fc1 at M = 8 (the shape of the end-to-end decode step): sq_layernorm followed by the linear (two
    launches) against sq_w4a16_gemm_ln_fused (the normalisation inside the linear's kernel), cold weights, HIP-graph
    replay; parity of the fused call against the oracle's LayerNorm (rounded to fp16) and product on sampled rows."""
    import numpy as np
    import w4a16_oracle as orc
    idx = [i for i, (name, _, _) in enumerate(shapes) if name == "fc1"][0]
    _, n, k = shapes[idx]
    x = (torch.randn((m, k), device=dev, generator=gen) * 1.5 + 0.2).half()
    gamma = (torch.randn(k, device=dev, generator=gen) * 0.2 + 1.0).half()
    beta = (torch.randn(k, device=dev, generator=gen) * 0.2).half()
    h = torch.empty_like(x)
    y = torch.empty((m, n), dtype=torch.float16, device=dev)
    torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
    res = {"shape": "LayerNorm(8 x 4096) -> fc1 4096 -> 16384, group %d" % g}
    with torch.cuda.stream(stream):
        ws = capi.workspace(m, n, k, dev, stream)

        def two():
            for layer in pool:
                capi.layernorm(x, gamma, beta, 1e-5, out=h, stream=stream)
                capi.gemm_ws(h, layer[idx][0], layer[idx][1], n, k, g, out=y, stream=stream, ws=ws)

        def fused():
            for layer in pool:
                capi.gemm_ln_fused(x, gamma, beta, 1e-5, layer[idx][0], layer[idx][1], n, k, g, out=y, stream=stream, ws=ws)

        fused()
        stream.synchronize()
        w, zs = pool[-1][idx]
        ridx = np.sort(np.random.default_rng(5).choice(n, size=64, replace=False))
        hn = orc.layernorm_ref(x.cpu().numpy(), gamma.cpu().numpy(), beta.cpu().numpy(), 1e-5).astype(np.float16)
        ref = orc.gemm_ref(hn, orc.dequant_l1(w.cpu().numpy()[ridx], zs.cpu().numpy()[ridx], g))
        got = y.float().cpu().numpy()[:, ridx]
        err = gate(float(np.max(np.abs(got - ref)) / np.max(np.abs(ref))) if np.all(np.isfinite(got)) else float("inf"),
                   "LayerNorm inside fc1 at M=%d" % m)
        res["parity_max_rel_err"] = round(err, 6)
        for name, fn in (("layernorm_then_linear", two), ("layernorm_inside_linear", fused)):
            fn()
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                fn()
            for _ in range(5):
                graph.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(50):
                graph.replay()
            e1.record(stream)
            stream.synchronize()
            res[name] = {"us": round(e0.elapsed_time(e1) * 1e3 / (50 * len(pool)), 2),
                         "launches": 2 if fn is two else 1}
    return res


def gated_mlp_leg(torch, capi, g, dev, gen, stream, n=11008, k=4096, tokens=(1, 8, 2048), copies=8):
    """Front half of a Llama-7B MLP, silu(x W_gate^T) * (x W_up^T) with both weights 11008 x 4096: sq_w4a16_gemm_silu_dot
    (two launches, SiLU and product in the second one's store) against two plain linears followed by torch's silu and
    multiply (four launches), cold weights (rotating pool), HIP-graph replay; parity against the oracle's float64
    formula on sampled output rows."""
    import numpy as np
    import w4a16_oracle as orc
    pool = [(make_linear(n, k, g, dev, gen), make_linear(n, k, g, dev, gen)) for _ in range(copies)]
    res = {"shape": "gate, up %d x %d, group %d" % (n, k, g), "pool_mb": round(copies * 2 * n * k / 2 / 1e6)}
    for m in tokens:
        x = torch.randn((m, k), device=dev, generator=gen).half()
        y = torch.empty((m, n), dtype=torch.float16, device=dev)
        a = torch.empty((m, n), dtype=torch.float16, device=dev)
        b = torch.empty((m, n), dtype=torch.float16, device=dev)
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            ws = capi.workspace(m, n, k, dev, stream) if 2 < m <= 1024 else None

            def fused():
                for (wg, zg), (wu, zu) in pool:
                    capi.gemm_silu_dot(x, wg, zg, wu, zu, n, k, g, out=y, stream=stream, ws=ws, up_out=b)

            def unfused():
                for (wg, zg), (wu, zu) in pool:
                    capi.gemm_ws(x, wg, zg, n, k, g, out=a, stream=stream, ws=ws)
                    capi.gemm_ws(x, wu, zu, n, k, g, out=b, stream=stream, ws=ws)
                    torch.mul(torch.nn.functional.silu(a), b, out=y)

            fused()
            stream.synchronize()
            (wg, zg), (wu, zu) = pool[-1]
            rng = np.random.default_rng(m)
            ridx = np.sort(rng.choice(n, size=64, replace=False))
            tidx = np.arange(m) if m <= 32 else np.sort(rng.choice(m, size=32, replace=False))
            want = orc.silu_dot_ref(x.cpu().numpy()[tidx], orc.dequant_l1(wg.cpu().numpy()[ridx], zg.cpu().numpy()[ridx], g),
                                    orc.dequant_l1(wu.cpu().numpy()[ridx], zu.cpu().numpy()[ridx], g))
            got = y.float().cpu().numpy()[tidx][:, ridx]
            err = gate(float(np.max(np.abs(got - want)) / np.max(np.abs(want))) if np.all(np.isfinite(got)) else float("inf"),
                       "gated MLP at M=%d" % m)
            entry = {"parity_max_rel_err": round(err, 6)}
            for name, fn in (("silu_dot_in_the_store", fused), ("two_linears_then_torch", unfused)):
                fn()
                stream.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    fn()
                reps = 20 if m <= 64 else 3
                for _ in range(reps):
                    graph.replay()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(2 * reps):
                    graph.replay()
                e1.record(stream)
                stream.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / (2 * reps * copies)
                entry[name] = {"us": round(us, 2), "launches": 2 if fn is fused else 4}
                if m >= 512:
                    entry[name]["tflops"] = round(4.0 * m * n * k / us * 1e-6, 1)
                else:
                    entry[name]["gbs"] = round(2 * algorithmic_bytes(m, n, k, g) / us * 1e-3, 1)
            res["m%d" % m] = entry
    return res


def sequence_leg(torch, capi, pool, shapes, m, g, dev, gen, stream, bytes_per_step):
    """The same six linears through sq_w4a16_gemv_sequence with the decoder layer's data flow as real buffers (q, k
    and v read x; out_proj reads q's output, fc1 out_proj's, fc2 fc1's): in the default mode (a new launch at every
    dependent linear), as ONE persistent launch (outputs travel between workgroups as tagged words, no grid
    barrier), and six independent linears in one persistent launch.  x is N(0, 1) / 64 so that four random
    linears in a row stay inside fp16."""
    x0 = (torch.randn((m, 4096), device=dev, generator=gen) / 64).half()
    x16 = (torch.randn((m, 16384), device=dev, generator=gen) / 64).half()
    ys = [torch.empty((m, n), dtype=torch.float16, device=dev) for _, n, _ in shapes]
    chained = [x0, x0, x0, ys[0], ys[3], ys[4]]
    loose = [x0, x0, x0, x0, x0, x16]
    res = {}
    for label, dep, mode in (("layer_dependencies_auto", "000111", capi.SQ_SEQ_AUTO),
                             ("layer_dependencies_one_launch", "000111", capi.SQ_SEQ_ONE_LAUNCH),
                             ("independent_one_launch", "000000", capi.SQ_SEQ_ONE_LAUNCH)):
        xin = chained if dep != "000000" else loose
        seqs = [capi.LinearSequence([dict(x=xin[i], w=w, zs=zs, y=ys[i], n=n, k=k, group_size=g, depends=dep[i] == "1")
                                     for i, ((w, zs), (_, n, k)) in enumerate(zip(layer, shapes))], m, dev, mode=mode)
                for layer in pool]
        torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
        with torch.cuda.stream(stream):
            for y in ys:
                y.fill_(float("nan"))
            seqs[0].run(stream=stream)
            stream.synchronize()
            worst = 0.0
            for i, ((w, zs), (name, n, k)) in enumerate(zip(pool[0], shapes)):
                worst = max(worst, gate(parity_linear(torch, w, zs, n, k, g, xin[i], ys[i], seed=i), "sequence " + name))
            for sq in seqs:
                sq.run(stream=stream)
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for sq in seqs:
                    sq.run(stream=stream)
            for _ in range(10):
                graph.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(200):
                graph.replay()
            e1.record(stream)
            stream.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (200 * len(pool))
        res[label] = {"depends": dep, "us_per_step": round(us, 2), "gbs": round(bytes_per_step / us / 1e3, 1),
                      "frac_of_hbm_peak": round(bytes_per_step / us / 1e3 / HBM_PEAK_GBS, 4),
                      "parity_max_rel_err": round(worst, 6), "wait_timeouts": sum(sq.error_flag() for sq in seqs)}
    return res


def picker_leg(torch, capi, g, dev, gen, stream):
    """The measured kernel picker (sq_w4a16_autotune) on shapes the built-in rules were swept on and on shapes they
    were not: per shape and token count the launch time of the built-in choice, of the fastest candidate, and that
    candidate's kernel word (0 = the built-in choice stands).  Weights rotate through a pool beyond the last-level
    cache.  The recorded choices are dropped again at the end."""
    res = {}
    shapes = (("opt_fc1", 16384, 4096), ("opt_fc2", 4096, 16384), ("llama13b_up", 13824, 5120),
              ("llama13b_down", 5120, 13824), ("n1024_k8192", 1024, 8192))
    try:
        for name, n, k in shapes:
            copies = max(2, int(600e6 / (n * k / 2)))
            w = torch.randint(0, 256, (copies, n, k // 2), dtype=torch.uint8, device=dev, generator=gen)
            z = torch.randint(0, 16, (copies, n, k // g), device=dev, generator=gen).half() + 64
            sc = (torch.randn((copies, n, k // g), device=dev, generator=gen).abs() * 0.02 + 1e-3).half()
            zs = torch.stack([z, sc], dim=-1).reshape(copies, n, 2 * (k // g)).contiguous()
            per = {}
            for m in (1, 8, 32, 128, 1024):
                x = torch.randn((m, k), device=dev, generator=gen).half()
                y = torch.empty((m, n), dtype=torch.float16, device=dev)
                ws = capi.workspace(m, n, k, dev, stream)
                torch.cuda.synchronize()
                with torch.cuda.stream(stream):
                    word, t_best, t_auto = capi.autotune(x, w, zs, n, k, g, ws=ws, reps=max(copies, 20), out=y, stream=stream)
                    # the product path now takes the recorded choice: check it like every other leg
                    capi.gemm_ws(x, w[0], zs[0], n, k, g, out=y, stream=stream, ws=ws)
                    stream.synchronize()
                    err = gate(parity_linear(torch, w[0], zs[0], n, k, g, x, y, seed=m), "picker %s at M=%d" % (name, m))
                per["m%d" % m] = {"builtin_us": round(t_auto, 2), "best_us": round(t_best, 2),
                                  "best_kernel_word": "0x%x" % word, "gain": round(t_auto / t_best, 3),
                                  "parity_max_rel_err": round(err, 6)}
            res[name] = per
            del w, z, sc, zs
    finally:
        res["choices_recorded"] = capi.autotune_clear()
    return res


def fused_qkv_leg(torch, capi, m, g, dev, gen, stream, layers, bytes_per_step):
    """The same step with q/k/v served by ONE launch on the row-concatenated weight [12288, 4096]
    (possible because layout L1 is row-major in N); four launches per step instead of six."""
    shapes = [("qkv_proj", 12288, 4096), ("out_proj", 4096, 4096), ("fc1", 16384, 4096), ("fc2", 4096, 16384)]
    pool = [[make_linear(n, k, g, dev, gen) for _, n, k in shapes] for _ in range(layers)]
    xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in (4096, 16384)}
    ys = {n: torch.empty((m, n), dtype=torch.float16, device=dev) for n in (12288, 4096, 16384)}
    steps = 2000
    torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
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
            out = capi.lut_attention(q, k, v, lut, d ** -0.5, False)
        torch.cuda.synchronize()
        import numpy as np
        import lut_attention_oracle as att
        worst = 0.0
        for zi, hi in ((0, 0), (z - 1, h - 1)):  # the float64 oracle on two (batch, head) pairs
            sl = (slice(zi, zi + 1), slice(hi, hi + 1))
            ref = att.attention_ref(q[sl].cpu().numpy(), k[sl].cpu().numpy(), v[sl].cpu().numpy(),
                                    lut[hi:hi + 1].cpu().numpy(), d ** -0.5, False)
            err = float(np.max(np.abs(out[sl].float().cpu().numpy() - ref)) / np.max(np.abs(ref)))
            worst = max(worst, gate(err, "LUT attention S=%d" % s))
        # the oracle above left the GPU idle for seconds: about 20 ms of warm-up, then a window of about 40 ms
        def window(n):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                capi.lut_attention(q, k, v, lut, d ** -0.5, False)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / n
        est = max(window(3), 1.0)
        window(max(3, min(2000, int(20000.0 / est))))
        us = window(max(20, min(4000, int(40000.0 / est))))
        tf = 4.0 * kept * 64 * 64 * d / us / 1e6
        res["seq%d" % s] = {"us": round(us, 1), "tflops": round(tf, 1),
                            "frac_of_fp16_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4),
                            "parity_max_rel_err": round(worst, 6)}
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

    import numpy as np
    import lut_attention_oracle as att
    kc0, vc0 = kcs[0].clone(), vcs[0].clone()
    got = capi.decode_attention(qs[0], kc0, vc0, pos, scale, k_new=qs[0], v_new=qs[0])
    torch.cuda.synchronize()
    ref = att.decode_attention_ref(qs[0][:2, :, 0].cpu().numpy(), kc0[:2].cpu().numpy(), vc0[:2].cpu().numpy(), scale)
    err = float(np.max(np.abs(got.view(b, h, d)[:2].float().cpu().numpy() - ref)) / max(1.0, np.max(np.abs(ref))))
    if not err <= 2e-3:
        raise ParityError("parity gate failed for decode attention: %.3e" % err)
    res = {"shape": "B=8 H=32 D=128 rows=640", "bytes": 2 * b * h * rows * d * 2, "parity_max_err": round(err, 6)}
    for name, fn in (("kernel", ours), ("torch_sdpa", sdpa)):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                fn()
        for _ in range(5 * reps):  # about 15 ms of warm-up after the idle gap of the parity check
            graph.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10 * reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (10 * reps * pool)
        res[name] = {"us": round(us, 2), "gbs": round(res["bytes"] / us / 1e3, 1),
                     "frac_of_hbm_peak": round(res["bytes"] / us / 1e3 / HBM_PEAK_GBS, 4)}
    return res


if __name__ == "__main__":
    main()
