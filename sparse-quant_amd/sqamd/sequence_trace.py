"""Where a sequence of decode linears spends its time inside the persistent kernel.

Runs the six W4A16 linears of an OPT-6.7B decoder layer (group 128, cold weights from a rotating
pool) through the time-stamping instantiation of the sequence kernel (sq_sequence_trace in
libsq_probes.so) and prints, per stage, when the workgroups reached it (microseconds since the first
workgroup started; minimum / median / maximum over the workgroups).

    python -m sqamd.sequence_trace [M] [depends]

`depends` is a string of six 0/1 flags, one per linear (q, k, v, out_proj, fc1, fc2): 1 = the linear
consumes an earlier output, so a grid barrier precedes it.  "000111" is the data flow of the decoder
layer, "000000" six independent linears.  Also prints the wall-clock time of the same sequence and of
one launch per linear (HIP-graph replay), for comparison.
"""
import sys

import torch

from . import capi

SHAPES = [("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096), ("out_proj", 4096, 4096),
          ("fc1", 16384, 4096), ("fc2", 4096, 16384)]


def main(m=1, dep="000111", g=128, layers=8):
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)

    def make(n, k):
        w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=gen)
        z = torch.randint(0, 16, (n, k // g), device=dev, generator=gen).half() + 64
        s = (torch.randn((n, k // g), device=dev, generator=gen).abs() * 0.02 + 1e-3).half()
        return w, torch.stack([z, s], dim=-1).reshape(n, 2 * (k // g)).contiguous()

    pool = [[make(n, k) for _, n, k in SHAPES] for _ in range(layers)]
    xs = {k: torch.randn((m, k), device=dev, generator=gen).half() for k in (4096, 16384)}
    ys = [torch.empty((m, n), dtype=torch.float16, device=dev) for _, n, _ in SHAPES]

    def linears(layer):
        return [dict(x=xs[k], w=w, zs=zs, y=ys[i], n=n, k=k, group_size=g, depends=int(dep[i] == "1"))
                for i, ((w, zs), (_, n, k)) in enumerate(zip(layer, SHAPES))]

    trace = None
    for _ in range(3):
        for layer in pool:
            trace = capi.sequence_trace(linears(layer), m, g)
    torch.cuda.synchronize()
    t = trace.cpu().double()
    t0 = t[:, 0].min()

    def row(name, col):
        v = (t[:, col] - t0) / 100.0
        print("%-34s %7.2f %7.2f %7.2f" % (name, v.min(), v.median(), v.max()))

    print("M = %d, depends = %s, %d workgroups; us since the first workgroup started: min / median / max" % (m, dep, t.shape[0]))
    row("workgroup starts", 0)
    row("first activations staged", 1)
    for l, (name, _, _) in enumerate(SHAPES):
        row("%s: weights consumed (wave 0)" % name, 2 + 4 * l)
        row("%s: Y stored" % name, 3 + 4 * l)
        if l + 1 < len(SHAPES):
            if dep[l + 1] == "1":
                row("%s: grid barrier passed" % name, 4 + 4 * l)
            row("%s: next activations staged" % name, 5 + 4 * l)
    row("streaming wave 0 leaves", 60)
    row("control waves leave", 61)

    # wall clock of the same work, HIP-graph replay over the pool
    stream = torch.cuda.Stream()

    def timed(fn, reps=200):
        torch.cuda.synchronize()  # tensors made on the default stream are complete before this stream reads them
        with torch.cuda.stream(stream):
            fn()
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                fn()
            for _ in range(20):
                graph.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                graph.replay()
            e1.record(stream)
            stream.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * layers)

    for label, mode in (("one persistent launch, grid barriers", capi.SQ_SEQ_ONE_LAUNCH),
                        ("a new launch at every dependent linear", capi.SQ_SEQ_AUTO)):
        seqs = [capi.LinearSequence(linears(layer), m, dev, mode=mode) for layer in pool]
        print("%-44s %6.2f us per step" % (label, timed(lambda: [s.run(stream=stream) for s in seqs])))

    def single():
        for layer in pool:
            for l in linears(layer):
                capi.gemm(l["x"], l["w"], l["zs"], l["n"], l["k"], g, out=l["y"], stream=stream)
    print("%-44s %6.2f us per step" % ("one launch per linear (sq_w4a16_gemm)", timed(single)))


if __name__ == "__main__":
    main(int(sys.argv[1]) if len(sys.argv) > 1 else 1, sys.argv[2] if len(sys.argv) > 2 else "000111")
