#!/usr/bin/env python3
"""Benchmark of the fused non-GEMM kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (BASELINE.json configs[4], the largest that fits one GPU):
the non-GEMM chain of one GPT-NeoX-20B-shaped layer, bf16, batch 4, sequence
2048, hidden 6144, 64 heads.  One step = eight launches through the C ABI,
    ln_fwd, ln_bwd                  [8192, 6144]
    softmax_causal_fwd, _bwd        [256, 2048, 2048], scale 1/sqrt(96)
    bias_gelu_fwd, _bwd             [8192, 24576]
    bias_dropout_add_fwd, _bwd      [8192, 6144], p = 0.1
every buffer resident in HBM and pre-allocated; each stage has its own
synthetic input (the GEMMs between the stages are not part of the path).  The
four 2 GB tensors of the softmax stage are laid out as the Python binding lays
them out for a user of FusedScaleMaskSoftmax: the scores and the incoming
gradient are plain torch allocations, the probabilities and the input gradient
come from the binding's own allocation helper (`_C.empty_staggered`), which
keeps them off the 2 MiB phase of the operands; the kernel table holds the
same backward launch on four plain allocations for comparison.
`value` = algorithmic bytes of a step (10 537.7 MB) / wall time per step.

Prints ONE JSON line.  Beside the contract's keys it carries
  roofline      the dominant launch of the step (causal softmax backward,
                4 296.0 MB), timed with events on the launch stream inside the
                timed region; `traffic` is read from the rocprofv3 counter
                summary under profiles/,
  cpu_baseline  the same chain through the reference's unfused torch path
                (oracle/torch_path.py) on the host cores, on a bounded sample,
  kernels       a compact table (cols / rows) of achieved GB/s and fraction of
                the 8 TB/s HBM peak for every fused kernel of BASELINE.json's
                five configurations, with mean / median / minimum times, the
                time per launch inside a captured HIP graph for the backward
                kernels that end in a second (finalize) launch, and plain
                copies of matching sizes,
  cpu_path      the reference's unfused torch path, forward + backward, per
                configuration on bounded samples, with the GPU rate of the
                same fused forward + backward pair (the metric's own unit:
                gpu_GBps and gpu_frac of the peak) and their ratio,
  modules       forward + backward through the oslo_amd.torch.nn modules and
                functions with autograd (output allocation, saved tensors and
                the binding's checks included), next to the C-ABI pair of the
                kernel table and their ratio.
"""
import argparse
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
METRIC = "achieved HBM GB/s (% of MI355X peak) per fused fwd+bwd kernel; speedup vs CPU path"
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "bench_all_kernels_hbm_traffic.txt")

F32, F16, BF16 = 0, 1, 2


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--table-iters", type=int, default=200, help="launches per kernel in the per-kernel table (0 = skip)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph-column", action="store_true", help="skip the captured-graph timings of the table")
    ap.add_argument("--no-modules", action="store_true", help="skip the module-API rows")
    ap.add_argument("--finalize-ab", action="store_true",
                    help="only the A/B of the column-sum finalize launch (serial against a second stream or a "
                         "graph branch): prints its own JSON line and exits")
    ap.add_argument("--tune-ab", metavar="KEY=V1,V2,...",
                    help="print the kernel table once per value of one launch knob (oslo_tune; 0 = the default) "
                         "and exit: the A/B behind a default, from committed code")
    ap.add_argument("--only", default="", help="with --tune-ab: keep the rows whose kernel name contains this")
    ap.add_argument("--tune-fixed", default="", metavar="KEY=V[,KEY=V]",
                    help="with --tune-ab: other knobs held at a value in every column")
    ap.add_argument("--traffic-optional", action="store_true",
                    help="report roofline.traffic as null when the counter summary has no row for the roofline "
                         "kernel (for the profiling runs that produce that summary); without it a missing row "
                         "is an error")
    return ap.parse_args()


class Lib:
    """Raw C-ABI calls on pre-allocated tensors (no allocation per call)."""

    def __init__(self, torch, _C):
        self.torch = torch
        self.lib = _C.load_library()
        self._C = _C

    def stream(self):
        return self.torch.cuda.current_stream().cuda_stream

    def ok(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.oslo_hip_last_error().decode())

    def ws(self, op, n1, n2, device):
        nbytes = int(self.lib.oslo_workspace_bytes(op, n1, n2))
        return self.torch.empty(max(nbytes, 16), dtype=self.torch.uint8, device=device), nbytes


def p(t):
    return None if t is None else t.data_ptr()


WARM_MS = 30.0  # launches before a timed region: the clocks of an idle GPU take this long to settle
BATCHES = 10    # event pairs per table row: mean over all launches, median and minimum over the batches


def time_launches(torch, fn, iters, nsets):
    """Times fn(i % nsets) with events on the current stream: `iters` launches
    in BATCHES batches, each between one pair of events.  Returns (mean,
    median of the batch means, smallest batch mean) in ms per launch."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    # warm-up: every buffer set is touched, and the GPU is kept busy for WARM_MS
    n = max(3, nsets)
    spent = 0.0
    while spent < WARM_MS:
        e0.record()
        for i in range(n):
            fn(i % nsets)
        e1.record()
        torch.cuda.synchronize()
        spent += e0.elapsed_time(e1)
        n = min(4 * n, 400)
    per = max(1, iters // BATCHES)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(BATCHES)]
    k = 0
    for a, b in evs:
        a.record()
        for _ in range(per):
            fn(k % nsets)
            k += 1
        b.record()
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) / per for a, b in evs)
    return sum(times) / len(times), times[len(times) // 2], times[0]


def time_in_graph(torch, fn, nsets, launches=24, replays=8):
    """ms per launch of fn inside a captured HIP graph (the dependent launches
    of one call follow each other without host dispatch); None if capture fails."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            for i in range(nsets):
                fn(i)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(launches):
                    fn(i % nsets)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (replays * launches)
    except Exception as exc:  # noqa: BLE001 - a timing column, never fatal
        sys.stderr.write("bench.py: graph timing skipped (%s)\n" % (exc,))
        return None


def time_queued(torch, fn, nsets, blocker, calls=16, repeats=6):
    """ms per call of fn when the host runs ahead of the GPU, the regime of a
    training step whose GEMMs keep the GPU busy while Python prepares the next
    launches: `blocker()` first puts a few ms of work on the stream, then
    `calls` calls of fn are enqueued behind it and timed by events on the
    stream.  The events bracket GPU time only as long as the host has enqueued
    every call before the GPU reaches it, which the blocker's length ensures
    (16 calls x ~0.12 ms of Python against >= 4 ms of blocker)."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    for i in range(max(3, nsets)):
        fn(i % nsets)
    torch.cuda.synchronize()
    times = []
    k = 0
    for _ in range(repeats):
        blocker()
        e0.record()
        for _ in range(calls):
            fn(k % nsets)
            k += 1
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / calls)
    times.sort()
    return times[len(times) // 2]


def norm_buffers(torch, dev, n1, n2, nsets, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    sets = []
    for _ in range(nsets):
        s = {
            "x": torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16),
            "dy": torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16),
            "y": torch.empty(n1, n2, device=dev, dtype=torch.bfloat16),
            "dx": torch.empty(n1, n2, device=dev, dtype=torch.bfloat16),
            "mean": torch.empty(n1, device=dev, dtype=torch.float32),
            "invvar": torch.empty(n1, device=dev, dtype=torch.float32),
        }
        sets.append(s)
    gamma = (1 + 0.02 * torch.randn(n2, generator=g, device=dev)).to(torch.bfloat16)
    beta = (0.02 * torch.randn(n2, generator=g, device=dev)).to(torch.bfloat16)
    dgamma = torch.empty_like(gamma)
    dbeta = torch.empty_like(beta)
    return sets, gamma, beta, dgamma, dbeta


def make_norm_calls(L, dev, n1, n2, nsets, seed=0):
    torch = L.torch
    lib = L.lib
    sets, gamma, beta, dgamma, dbeta = norm_buffers(torch, dev, n1, n2, nsets, seed)
    ws_ln, ws_ln_bytes = L.ws(L._C.OSLO_OP_LN_BWD, n1, n2, dev)
    ws_rms, ws_rms_bytes = L.ws(L._C.OSLO_OP_RMS_BWD, n1, n2, dev)
    keep = (sets, gamma, beta, dgamma, dbeta, ws_ln, ws_rms)

    def ln_fwd(i):
        s = sets[i]
        L.ok(lib.oslo_ln_fwd(p(s["x"]), p(gamma), p(beta), p(s["y"]), p(s["mean"]), p(s["invvar"]),
                             n1, n2, 1e-5, BF16, BF16, L.stream()))

    def ln_bwd(i):
        s = sets[i]
        L.ok(lib.oslo_ln_bwd(p(s["dy"]), p(s["x"]), p(s["mean"]), p(s["invvar"]), p(gamma), p(s["dx"]),
                             p(dgamma), p(dbeta), p(ws_ln), ws_ln_bytes, n1, n2, BF16, BF16, L.stream()))

    def rms_fwd(i):
        s = sets[i]
        L.ok(lib.oslo_rms_fwd(p(s["x"]), p(gamma), p(s["y"]), p(s["invvar"]), n1, n2, 1e-5, BF16, BF16,
                              L.stream()))

    def rms_bwd(i):
        s = sets[i]
        L.ok(lib.oslo_rms_bwd(p(s["dy"]), p(s["x"]), p(s["invvar"]), p(gamma), p(s["dx"]), p(dgamma),
                              p(ws_rms), ws_rms_bytes, n1, n2, BF16, BF16, L.stream()))

    return {"ln_fwd": ln_fwd, "ln_bwd": ln_bwd, "rms_fwd": rms_fwd, "rms_bwd": rms_bwd, "_keep": keep}


# ---------------------------------------------------------------------------
# the headline step: BASELINE.json configs[4]
# ---------------------------------------------------------------------------
# the step's largest launch: one wave (64 threads) per softmax row
ROOF_KERNEL, ROOF_BLOCKS, ROOF_WG = "softmax_bwd_kernel", 256 * 2048, 64

CHAIN = {
    "tokens": 8192, "hidden": 6144, "attn_batches": 256, "seq": 2048, "ffn": 24576,
    "scale": 1.0 / math.sqrt(96.0), "p": 0.1,
}


def softmax_set(L, dev, shape, dtype, policy=True):
    """The four tensors of a softmax forward + backward pair (x, y, dy, dx) laid
    out as the product path lays them out: x and dy are what torch hands the
    binding (plain allocations), y and dx are what the binding allocates, by
    `_C.empty_staggered` on phases 1 and 2 of a 2 MiB period.  The causal
    softmax backward streams three 2 GB tensors at identical offsets; when all
    of them start on the same 2 MiB phase their requests meet in the same
    memory channels and the kernel runs 1.5-4 % slower (687-699 us against
    701-736 us, depending on the box).  `policy=False` gives four plain
    allocations."""
    torch = L.torch
    mk = L._C.empty_staggered
    return [mk(shape, dtype, dev, k if policy else 0) for k in (0, 1, 0, 2)]


def chain_bytes():
    """Algorithmic bytes of each launch of the step (bf16: 2 bytes per element)."""
    c = CHAIN
    t_ln = c["tokens"] * c["hidden"] * 2
    t_sm = c["attn_batches"] * c["seq"] * c["seq"] * 2
    t_ff = c["tokens"] * c["ffn"] * 2
    f = (c["seq"] + 1) / (2.0 * c["seq"])
    return [
        ("ln_fwd", 2 * t_ln), ("ln_bwd", 3 * t_ln),
        ("softmax_causal_fwd", (1 + f) * t_sm), ("softmax_causal_bwd", (1 + 2 * f) * t_sm),
        ("bias_gelu_fwd", 2 * t_ff), ("bias_gelu_bwd", 3 * t_ff),
        ("bias_dropout_add_fwd", 3 * t_ln), ("bias_dropout_add_bwd", 2 * t_ln),
    ]


def make_chain(L, dev):
    """Pre-allocates every buffer of the step and returns its eight launches in
    order (the order of the reference's layer: LayerNorm, attention softmax,
    feed-forward activation, output dropout + residual), each as fn()."""
    torch = L.torch
    lib = L.lib
    c = CHAIN
    n1, h, ab, s, ff = c["tokens"], c["hidden"], c["attn_batches"], c["seq"], c["ffn"]
    g = torch.Generator(device=dev).manual_seed(0)
    bf = torch.bfloat16

    def rnd(*shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(*shape, generator=g, device=dev)).to(bf)

    ln = {"x": rnd(n1, h), "dy": rnd(n1, h), "y": torch.empty(n1, h, device=dev, dtype=bf),
          "dx": torch.empty(n1, h, device=dev, dtype=bf), "mean": torch.empty(n1, device=dev),
          "invvar": torch.empty(n1, device=dev), "gamma": rnd(h, std=0.02, mean=1.0), "beta": rnd(h, std=0.02)}
    ln["dgamma"], ln["dbeta"] = torch.empty_like(ln["gamma"]), torch.empty_like(ln["beta"])
    ws_ln, ws_ln_b = L.ws(L._C.OSLO_OP_LN_BWD, n1, h, dev)
    sm = dict(zip(("x", "y", "dy", "dx"), softmax_set(L, dev, (ab, s, s), bf)))
    sm["x"].normal_(generator=g)
    sm["dy"].normal_(generator=g)
    ge = {"x": rnd(n1, ff), "g": rnd(n1, ff), "bias": rnd(ff, std=0.02)}
    ge["y"], ge["dx"], ge["dbias"] = torch.empty_like(ge["x"]), torch.empty_like(ge["x"]), torch.empty_like(ge["bias"])
    ws_ge, ws_ge_b = L.ws(L._C.OSLO_OP_BIAS_GELU_BWD, n1, ff, dev)
    bd = {"x": rnd(n1, h), "res": rnd(n1, h), "g": rnd(n1, h), "bias": rnd(h, std=0.02)}
    bd["out"], bd["dx"], bd["dbias"] = torch.empty_like(bd["x"]), torch.empty_like(bd["x"]), torch.empty_like(bd["bias"])
    ws_bd, ws_bd_b = L.ws(L._C.OSLO_OP_BIAS_DROPOUT_ADD_BWD, n1, h, dev)
    keep = (ln, sm, ge, bd, ws_ln, ws_ge, ws_bd)
    st = L.stream

    calls = [
        lambda: L.ok(lib.oslo_ln_fwd(p(ln["x"]), p(ln["gamma"]), p(ln["beta"]), p(ln["y"]), p(ln["mean"]),
                                     p(ln["invvar"]), n1, h, 1e-5, BF16, BF16, st())),
        lambda: L.ok(lib.oslo_ln_bwd(p(ln["dy"]), p(ln["x"]), p(ln["mean"]), p(ln["invvar"]), p(ln["gamma"]),
                                     p(ln["dx"]), p(ln["dgamma"]), p(ln["dbeta"]), p(ws_ln), ws_ln_b, n1, h,
                                     BF16, BF16, st())),
        lambda: L.ok(lib.oslo_softmax_causal_fwd(p(sm["x"]), p(sm["y"]), ab, s, s, c["scale"], BF16, st())),
        lambda: L.ok(lib.oslo_softmax_causal_bwd(p(sm["dy"]), p(sm["y"]), p(sm["dx"]), ab, s, s, c["scale"], BF16,
                                                 st())),
        lambda: L.ok(lib.oslo_bias_gelu_fwd(p(ge["x"]), p(ge["bias"]), p(ge["y"]), n1, ff, BF16, st())),
        lambda: L.ok(lib.oslo_bias_gelu_bwd(p(ge["g"]), p(ge["x"]), p(ge["bias"]), p(ge["dx"]), p(ge["dbias"]),
                                            p(ws_ge), ws_ge_b, n1, ff, BF16, st())),
        lambda: L.ok(lib.oslo_bias_dropout_add_fwd(p(bd["x"]), p(bd["bias"]), p(bd["res"]), p(bd["out"]), None, n1, h,
                                                   c["p"], 1234, 0, BF16, st())),
        lambda: L.ok(lib.oslo_bias_dropout_add_bwd(p(bd["g"]), p(bd["dx"]), p(bd["dbias"]), p(ws_bd), ws_bd_b, n1, h,
                                                   c["p"], 1234, 0, BF16, st())),
    ]
    return calls, keep


def traffic_from_profile(kernel, blocks, wg):
    """HBM bytes per launch of `kernel` at launch shape blocks x wg, from the
    committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary (columns: kernel,
    template, blocks, wg, FETCH KiB, WRITE KiB, read MB, write MB)."""
    try:
        text = open(TRAFFIC_SUMMARY).read()
    except OSError as exc:
        raise RuntimeError("bench.py: counter summary %s is missing (%s)" % (TRAFFIC_SUMMARY, exc))
    for line in text.splitlines():
        f = line.split()
        if len(f) >= 8 and f[0] == kernel and f[-6] == str(blocks) and f[-5] == str(wg):
            try:
                return (float(f[-2]) + float(f[-1])) * 1e6
            except ValueError:
                continue
    raise RuntimeError("bench.py: no row for %s at %d x %d in %s" % (kernel, blocks, wg, TRAFFIC_SUMMARY))


TABLE_COLS = ["kernel", "cfg", "MB", "us", "us_med", "us_min", "GBps", "frac", "graph_us", "note"]


def table_row(name, cfg, nbytes, t, graph_ms=None, note=""):
    mean, med, mn = t
    gbps = nbytes / (mean * 1e-3) / 1e9
    return [name, cfg, round(nbytes / 1e6, 1), round(mean * 1e3, 2), round(med * 1e3, 2), round(mn * 1e3, 2),
            round(gbps, 1), round(gbps / HBM_PEAK_GBPS, 4),
            None if graph_ms is None else round(graph_ms * 1e3, 2), note]


def nsets_for(total_bytes_per_set):
    """Enough rotating sets that consecutive launches cannot hit in the 256 MB cache."""
    return max(1, min(8, math.ceil(1.0e9 / max(total_bytes_per_set, 1))))


def kernel_table(L, dev, iters, graph_column=True):
    """Every fused kernel at the shapes of BASELINE.json's five configurations."""
    torch = L.torch
    lib = L.lib
    rows = []

    def timed(fn, nsets):
        return time_launches(torch, fn, iters, nsets)

    def graphed(fn, nsets):
        return time_in_graph(torch, fn, nsets) if graph_column else None

    # ---- LayerNorm / RMSNorm: cfg2 and cfg5 ----
    for cfg, n1, n2 in (("cfg2", 16384, 4096), ("cfg5", 8192, 6144)):
        T = n1 * n2 * 2
        ns = nsets_for(4 * T)
        calls = make_norm_calls(L, dev, n1, n2, ns, seed=1)
        for name, mult in (("ln_fwd", 2), ("ln_bwd", 3), ("rms_fwd", 2), ("rms_bwd", 3)):
            if cfg == "cfg5" and name.startswith("rms"):
                continue
            if name.endswith("bwd"):
                for i in range(ns):
                    calls[name.replace("bwd", "fwd")](i)
            rows.append(table_row(name, cfg, mult * T, timed(calls[name], ns),
                                  graphed(calls[name], ns) if name.endswith("bwd") else None))
        del calls
        torch.cuda.empty_cache()

    # ---- causal softmax: cfg1 (fp32) and cfg5 (bf16) ----
    for cfg, ab, s, tdt, code, esz, scale in (
        ("cfg1", 48, 512, torch.float32, F32, 4, 0.125),
        ("cfg5", 256, 2048, torch.bfloat16, BF16, 2, 1.0 / math.sqrt(96.0)),
        # short rows (batch 256 x 12 heads at sequence length 128): several
        # rows lie side by side in one wavefront
        ("seq128", 3072, 128, torch.bfloat16, BF16, 2, 0.125),
    ):
        T = ab * s * s * esz
        f = (s + 1) / (2.0 * s)
        ns = nsets_for(4 * T)
        g = torch.Generator(device=dev).manual_seed(2)
        bufs = []
        for _ in range(ns):
            x, y, dy, dx = softmax_set(L, dev, (ab, s, s), tdt)
            x.normal_(generator=g)
            dy.normal_(generator=g)
            bufs.append((x, y, dy, dx))

        def fwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_causal_fwd(p(x), p(y), ab, s, s, scale, code, L.stream()))

        def bwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_causal_bwd(p(dy), p(y), p(dx), ab, s, s, scale, code, L.stream()))

        rows.append(table_row("softmax_causal_fwd", cfg, (1 + f) * T, timed(fwd, ns)))
        rows.append(table_row("softmax_causal_bwd", cfg, (1 + 2 * f) * T, timed(bwd, ns),
                              note="y, dx placed by the binding's allocation policy" if cfg == "cfg5" else ""))
        if cfg == "cfg5":
            # the same launches on four plain torch allocations (all on one 2 MiB phase)
            plain = softmax_set(L, dev, (ab, s, s), tdt, policy=False)
            plain[0].copy_(bufs[0][0])
            plain[2].copy_(bufs[0][2])

            def pfwd(i):
                L.ok(lib.oslo_softmax_causal_fwd(p(plain[0]), p(plain[1]), ab, s, s, scale, code, L.stream()))

            def pbwd(i):
                L.ok(lib.oslo_softmax_causal_bwd(p(plain[2]), p(plain[1]), p(plain[3]), ab, s, s, scale, code,
                                                 L.stream()))

            pfwd(0)
            rows.append(table_row("softmax_causal_fwd", cfg, (1 + f) * T, timed(pfwd, 1), note="plain allocations"))
            rows.append(table_row("softmax_causal_bwd", cfg, (1 + 2 * f) * T, timed(pbwd, 1), note="plain allocations"))
            del plain

        # softmax with the attention dropout (p = 0.1) fused in: the same
        # compulsory bytes (backward reads the logits instead of the
        # probabilities; the row statistics are 8 bytes a row)
        stats = torch.empty(ab * s, 2, device=dev, dtype=torch.float32)

        def dfwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_causal_dropout_fwd(p(x), p(y), p(stats), ab, s, s, scale, 0.1, 1234, 0, code, L.stream()))

        def dbwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_causal_dropout_bwd(p(dy), p(x), p(stats), p(dx), ab, s, s, scale, 0.1, 1234, 0, code, L.stream()))

        rows.append(table_row("softmax_causal_dropout_fwd", cfg, (1 + f) * T, timed(dfwd, ns), note="p=0.1"))
        rows.append(table_row("softmax_causal_dropout_bwd", cfg, (1 + 2 * f) * T, timed(dbwd, ns), note="p=0.1"))
        del bufs, stats
        torch.cuda.empty_cache()

    # ---- padding-masked softmax: cfg3 ----
    b, h, s = 16, 16, 1024
    T = b * h * s * s * 2
    g = torch.Generator(device=dev).manual_seed(3)
    valid = torch.randint(256, 1025, (b,), generator=torch.Generator().manual_seed(3))
    r = float(valid.double().mean()) / s
    mask = (torch.arange(s)[None, :] >= valid[:, None]).view(b, 1, 1, s).to(dev).view(torch.uint8)
    ns = 2
    bufs = []
    for _ in range(ns):
        x = (2 * torch.randn(b, h, s, s, generator=g, device=dev)).to(torch.float16)
        dy = torch.randn(b, h, s, s, generator=g, device=dev).to(torch.float16)
        bufs.append((x, torch.empty_like(x), dy, torch.empty_like(x)))

    def mfwd(i):
        x, y, dy, dx = bufs[i]
        L.ok(lib.oslo_softmax_masked_fwd(p(x), p(mask), p(y), b, h, s, s, b, 1, 0.125, F16, L.stream()))

    def mbwd(i):
        x, y, dy, dx = bufs[i]
        L.ok(lib.oslo_softmax_masked_bwd(p(dy), p(y), p(mask), p(dx), b, h, s, s, b, 1, 0.125, F16, L.stream()))

    t = timed(mfwd, ns)
    rows.append(table_row("softmax_masked_fwd", "cfg3", (r + 1) * T, t,
                          note="valid %.4f, dense-equivalent %.0f GB/s" % (r, 2 * T / (t[0] * 1e-3) / 1e9)))
    t = timed(mbwd, ns)
    rows.append(table_row("softmax_masked_bwd", "cfg3", (2 * r + 1) * T, t,
                          note="valid %.4f, dense-equivalent %.0f GB/s" % (r, 3 * T / (t[0] * 1e-3) / 1e9)))
    # ---- the same configuration with the mask as the reference's models pass it:
    # an additive fp16 term [16, 1, 1, 1024] (modeling_bert.py:298-306).  A fill
    # of -10000 obliges the kernel to read every logit (a row whose keys are all
    # filled is the softmax of the logits): forward 2T, backward 3T.  A fill of
    # -inf hides the key for good: the backward pass skips its loads as with the
    # boolean mask (the forward pass reads every logit either way, see the
    # binding).  And a dense fp16 position bias [1, 16, 1024, 1024]
    # (modeling_t5.py:508-514), read once per batch entry: forward 2T + T/16. ----
    pad = (torch.arange(s)[None, :] >= valid[:, None]).view(b, 1, 1, s).to(dev)
    for fill, tag in ((-10000.0, "-10000"), (float("-inf"), "-inf")):
        term = torch.zeros(b, 1, 1, s, dtype=torch.float16, device=dev).masked_fill_(pad, fill)
        # what the binding passes for a term shared by heads and queries: the logits of a forward
        # pass are always read (waiting for the term costs more than the unread logits save), the
        # backward pass skips hidden chunks (OSLO_SOFTMAX_SKIP_HIDDEN)
        dense = fill == -10000.0

        def bfwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_bias_fwd(p(x), p(term), p(y), b, h, s, s, s, 0, 0, F16, 0, 0.125, F16,
                                           L.stream()))

        def bbwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_bias_bwd(p(dy), p(y), p(term), p(dx), b, h, s, s, s, 0, 0, F16, 2, 0.125,
                                           F16, L.stream()))

        rows.append(table_row("softmax_bias_fwd", "cfg3", 2 * T, timed(bfwd, ns),
                              note="additive [16,1,1,1024] fp16 mask, fill %s" % tag))
        rows.append(table_row("softmax_bias_bwd", "cfg3", (3 if dense else 2 * r + 1) * T, timed(bbwd, ns),
                              note="additive [16,1,1,1024] fp16 mask, fill %s" % tag))
    term = (2 * torch.randn(1, h, s, s, generator=g, device=dev)).to(torch.float16)

    def tfwd(i):
        x, y, dy, dx = bufs[i]
        L.ok(lib.oslo_softmax_bias_fwd(p(x), p(term), p(y), b, h, s, s, 0, s * s, s, F16, 0, 0.125, F16, L.stream()))

    def tbwd(i):
        x, y, dy, dx = bufs[i]
        L.ok(lib.oslo_softmax_bias_bwd(p(dy), p(y), None, p(dx), b, h, s, s, 0, 0, 0, F16, 0, 0.125, F16, L.stream()))

    rows.append(table_row("softmax_bias_fwd", "cfg3", 2 * T + T / b, timed(tfwd, ns),
                          note="position bias [1,16,1024,1024] fp16"))
    rows.append(table_row("softmax_bias_bwd", "cfg3", 3 * T, timed(tbwd, ns),
                          note="position bias [1,16,1024,1024] fp16"))
    del bufs, term
    torch.cuda.empty_cache()

    # ---- causal + key-padding mask in one call, cfg5 shape [4,64,2048,2048]
    # bf16 with valid lengths ~ U[1024, 2048]: reads stop at the diagonal and
    # at the valid length, whichever comes first ----
    b, h, s = 4, 64, 2048
    T = b * h * s * s * 2
    g = torch.Generator(device=dev).manual_seed(6)
    valid = torch.randint(1024, 2049, (b,), generator=torch.Generator().manual_seed(6))
    qi = torch.arange(1, s + 1, dtype=torch.float64)
    r = float(torch.minimum(qi[None, :], valid[:, None].double()).mean()) / s
    mask = (torch.arange(s)[None, :] >= valid[:, None]).view(b, 1, 1, s).to(dev).view(torch.uint8)
    x, y, dy, dx = softmax_set(L, dev, (b, h, s, s), torch.bfloat16)
    x.normal_(generator=g)
    dy.normal_(generator=g)
    sc = 1.0 / math.sqrt(96.0)

    def cmfwd(i):
        L.ok(lib.oslo_softmax_causal_masked_fwd(p(x), p(mask), p(y), b, h, s, s, b, 1, sc, BF16, L.stream()))

    def cmbwd(i):
        L.ok(lib.oslo_softmax_causal_masked_bwd(p(dy), p(y), p(mask), p(dx), b, h, s, s, b, 1, sc, BF16, L.stream()))

    rows.append(table_row("softmax_causal_masked_fwd", "cfg5pad", (r + 1) * T, timed(cmfwd, 1),
                          note="visible %.4f of the square" % r))
    rows.append(table_row("softmax_causal_masked_bwd", "cfg5pad", (2 * r + 1) * T, timed(cmbwd, 1),
                          note="visible %.4f of the square" % r))
    del x, dy, y, dx
    torch.cuda.empty_cache()

    # ---- bias-GeLU: cfg4 and cfg5 ----
    for cfg, n1, n2 in (("cfg4", 16384, 16384), ("cfg5", 8192, 24576)):
        T = n1 * n2 * 2
        ns = nsets_for(4 * T)
        g = torch.Generator(device=dev).manual_seed(4)
        bias = (0.02 * torch.randn(n2, generator=g, device=dev)).to(torch.bfloat16)
        dbias = torch.empty_like(bias)
        ws, wsb = L.ws(L._C.OSLO_OP_BIAS_GELU_BWD, n1, n2, dev)
        bufs = []
        for _ in range(ns):
            x = torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16)
            gg = torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16)
            bufs.append((x, torch.empty_like(x), gg, torch.empty_like(x)))

        def gfwd(i):
            x, y, gg, dx = bufs[i]
            L.ok(lib.oslo_bias_gelu_fwd(p(x), p(bias), p(y), n1, n2, BF16, L.stream()))

        def gbwd(i):
            x, y, gg, dx = bufs[i]
            L.ok(lib.oslo_bias_gelu_bwd(p(gg), p(x), p(bias), p(dx), p(dbias), p(ws), wsb, n1, n2, BF16, L.stream()))

        rows.append(table_row("bias_gelu_fwd", cfg, 2 * T, timed(gfwd, ns)))
        rows.append(table_row("bias_gelu_bwd", cfg, 3 * T, timed(gbwd, ns), graphed(gbwd, ns)))
        del bufs
        torch.cuda.empty_cache()

    # ---- bias-dropout-add: cfg4 (p = 0.1 and p = 0) and cfg5 ----
    for cfg, n1, n2, pdrop in (("cfg4", 16384, 4096, 0.1), ("cfg4", 16384, 4096, 0.0), ("cfg5", 8192, 6144, 0.1)):
        T = n1 * n2 * 2
        ns = nsets_for(5 * T)
        g = torch.Generator(device=dev).manual_seed(5)
        bias = (0.02 * torch.randn(n2, generator=g, device=dev)).to(torch.bfloat16)
        dbias = torch.empty_like(bias)
        ws, wsb = L.ws(L._C.OSLO_OP_BIAS_DROPOUT_ADD_BWD, n1, n2, dev)
        bufs = []
        for _ in range(ns):
            x = torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16)
            res = torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16)
            gg = torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16)
            bufs.append((x, res, torch.empty_like(x), gg, torch.empty_like(x)))

        def dfwd(i):
            x, res, out, gg, dx = bufs[i]
            L.ok(lib.oslo_bias_dropout_add_fwd(p(x), p(bias), p(res), p(out), None, n1, n2, pdrop, 1234, 0, BF16,
                                               L.stream()))

        def dbwd(i):
            x, res, out, gg, dx = bufs[i]
            L.ok(lib.oslo_bias_dropout_add_bwd(p(gg), p(dx), p(dbias), p(ws), wsb, n1, n2, pdrop, 1234, 0, BF16,
                                               L.stream()))

        tag = "p=%.1f" % pdrop
        rows.append(table_row("bias_dropout_add_fwd", cfg, 3 * T, timed(dfwd, ns), note=tag))
        rows.append(table_row("bias_dropout_add_bwd", cfg, 2 * T, timed(dbwd, ns), graphed(dbwd, ns), note=tag))

        # the same op fused into the LayerNorm that follows it (post-LN block):
        # forward reads x, residual and writes h, y (4T instead of 3T + 2T);
        # backward reads dy, h and writes the residual and x gradients (4T
        # instead of 3T + 2T)
        if pdrop > 0:
            gamma = (1 + 0.02 * torch.randn(n2, generator=g, device=dev)).to(torch.bfloat16)
            beta = (0.02 * torch.randn(n2, generator=g, device=dev)).to(torch.bfloat16)
            dgamma, dbeta = torch.empty_like(gamma), torch.empty_like(beta)
            mean = torch.empty(n1, device=dev, dtype=torch.float32)
            invvar = torch.empty(n1, device=dev, dtype=torch.float32)
            ws2, wsb2 = L.ws(L._C.OSLO_OP_BIAS_DROPOUT_ADD_NORM_BWD, n1, n2, dev)
            extra = [(torch.empty_like(b[0]), torch.empty_like(b[0])) for b in bufs]  # h, dres

            def ffwd(i):
                x, res, out, gg, dx = bufs[i]
                L.ok(lib.oslo_bias_dropout_add_norm_fwd(p(x), p(bias), p(res), p(gamma), p(beta), p(extra[i][0]),
                                                        p(out), p(mean), p(invvar), n1, n2, 1e-5, pdrop, 1234, 0, 0,
                                                        BF16, L.stream()))

            def fbwd(i):
                x, res, out, gg, dx = bufs[i]
                L.ok(lib.oslo_bias_dropout_add_norm_bwd(p(gg), None, p(extra[i][0]), p(mean), p(invvar), p(gamma),
                                                        p(extra[i][1]), p(dx), p(dgamma), p(dbeta), p(dbias), p(ws2),
                                                        wsb2, n1, n2, pdrop, 1234, 0, 0, BF16, L.stream()))

            rows.append(table_row("bias_dropout_add_ln_fwd", cfg, 4 * T, timed(ffwd, ns), note=tag))
            for i in range(ns):
                ffwd(i)
            rows.append(table_row("bias_dropout_add_ln_bwd", cfg, 4 * T, timed(fbwd, ns), graphed(fbwd, ns), note=tag))
            del extra
        del bufs
        torch.cuda.empty_cache()

    # ---- multi-tensor Adam (AdamW mode): the parameters of 16 transformer
    # layers of hidden size 2048 (12 tensors a layer, 0.8e9 bytes a state array
    # in fp32); reads g, p, m, v and writes p, m, v: 7 values per element ----
    import ctypes

    shapes = []
    for _ in range(16):
        shapes += [(2048, 6144), (6144,), (2048, 2048), (2048,), (2048, 8192), (8192,), (8192, 2048), (2048,),
                   (2048,), (2048,), (2048,), (2048,)]

    def optimizer_tensors(tdt):
        lists = [[torch.zeros(s, device=dev, dtype=tdt) for s in shapes] for _ in range(4)]
        for t in lists[0]:
            t.normal_()
        n = len(shapes)
        arr = ctypes.c_void_p * n
        tables = [arr(*[t.data_ptr() for t in lst]) for lst in lists]
        sizes = (ctypes.c_int64 * n)(*[t.numel() for t in lists[0]])
        return lists, tables, sizes, n, sum(t.numel() for t in lists[0])

    for tdt, code, esz in ((torch.float32, F32, 4), (torch.bfloat16, BF16, 2)):
        lists, tables, sizes, n, nel = optimizer_tensors(tdt)
        step_no = [0]

        def adam(i):
            step_no[0] += 1
            L.ok(lib.oslo_multi_tensor_adam(tables[0], tables[1], tables[2], tables[3], sizes, n, 1e-3, 0.9, 0.999,
                                            1e-8, step_no[0], 1, 1, 0.01, code, L.stream()))

        dname = "f32" if tdt == torch.float32 else "bf16"
        opt_iters = max(10, iters // 4)
        rows.append(table_row("mt_adam", dname, 7 * nel * esz, time_launches(torch, adam, opt_iters, 1)))
        del lists, tables
        torch.cuda.empty_cache()

    # ---- plain copies with the same load/store path, at the traffic of the
    # short kernels above and at 2 GiB: the practical ceiling at each size ----
    for total_mb in (75.5, 100.8, 201.3, 268.4, 402.7, 830.0, 2147.5):
        nbytes = int(total_mb * 1e6 / 2) // 16 * 16
        ns = nsets_for(2 * nbytes)
        src = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(ns)]
        dst = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(ns)]
        for s_ in src:
            s_.fill_(1)

        def cp(i):
            L.ok(lib.oslo_copy_probe(p(src[i]), p(dst[i]), nbytes, L.stream()))

        rows.append(table_row("copy_probe", "-", 2 * nbytes, timed(cp, ns)))
        del src, dst
        torch.cuda.empty_cache()

    # ---- the other multi-tensor optimizer steps on the tensors of the Adam rows
    # (values moved per element: SGD with momentum and Adagrad read 3 and write 2;
    # NovoGrad reads the gradients once more for their norms; LAMB = parameter
    # norms 1 + stage 1 (reads 4, writes 3) + update norms 1 + stage 2 (reads 2,
    # writes 1)) ----
    for tdt, code, esz in ((torch.float32, F32, 4), (torch.bfloat16, BF16, 2)):
        lists, tables, sizes, n, nel = optimizer_tensors(tdt)
        step_no = [0]
        dname = "f32" if tdt == torch.float32 else "bf16"
        opt_iters = max(10, iters // 4)
        need = int(lib.oslo_multi_tensor_norm_partials(sizes, n, code))
        partials = torch.empty(need, dtype=torch.float32, device=dev)
        norms = torch.ones(n, dtype=torch.float32, device=dev)
        norms2 = torch.ones(n, dtype=torch.float32, device=dev)
        gnorm = torch.ones(1, dtype=torch.float32, device=dev)

        def sgd(i):
            L.ok(lib.oslo_multi_tensor_sgd(tables[0], tables[1], tables[2], None, sizes, n, 0.01, 0.9, 0.0, 1e-3,
                                           0, 0, 0, 1.0, code, code, 0, None, L.stream()))

        def adagrad(i):
            L.ok(lib.oslo_multi_tensor_adagrad(tables[0], tables[1], tables[3], sizes, n, 1e-3, 1e-10, 0, 0.01,
                                               code, L.stream()))

        def l2norm(i):
            L.ok(lib.oslo_multi_tensor_norm(tables[0], sizes, n, code, p(partials), need, p(gnorm), p(norms), 2, 0,
                                            0.0, 0.0, None, 0, L.stream()))

        def novograd(i):
            step_no[0] += 1
            L.ok(lib.oslo_multi_tensor_norm(tables[0], sizes, n, code, p(partials), need, None, p(norms), 2, 1,
                                            0.98, 0.02, None, 0, L.stream()))
            L.ok(lib.oslo_multi_tensor_novograd(tables[0], tables[1], tables[2], sizes, n, p(norms), 1e-3, 0.95, 0.98,
                                                1e-8, step_no[0], 1, 0.01, 1, 1, code, L.stream()))

        def lamb(i):
            step_no[0] += 1
            L.ok(lib.oslo_multi_tensor_norm(tables[1], sizes, n, code, p(partials), need, None, p(norms), 2, 0,
                                            0.0, 0.0, None, 0, L.stream()))
            L.ok(lib.oslo_multi_tensor_lamb_stage1(tables[0], tables[1], tables[2], tables[3], sizes, n, 0.9, 0.999,
                                                   1e-6, step_no[0], 1, 0.01, 1, 1, p(gnorm), 1.0, code, L.stream()))
            L.ok(lib.oslo_multi_tensor_norm(tables[0], sizes, n, code, p(partials), need, None, p(norms2), 2, 0,
                                            0.0, 0.0, None, 0, L.stream()))
            L.ok(lib.oslo_multi_tensor_lamb_stage2(tables[0], tables[1], sizes, n, p(norms), p(norms2), 1e-3, 0.01,
                                                   0, code, L.stream()))

        for name, fn, values in (("mt_sgd", sgd, 5), ("mt_adagrad", adagrad, 5), ("mt_l2norm", l2norm, 1),
                                 ("mt_novograd", novograd, 6), ("mt_lamb", lamb, 12)):
            if fn is lamb:  # stage 1 overwrites the gradients: start every timing from fresh ones
                for t in lists[0]:
                    t.normal_()
            rows.append(table_row(name, dname, values * nel * esz, time_launches(torch, fn, opt_iters, 1)))
        del lists, tables, partials
        torch.cuda.empty_cache()
    return rows


def module_table(L, dev, iters, kernel_rows):
    """Forward + backward through the public modules and functions of
    oslo_amd.torch.nn with autograd -- what a user of the drop-in API runs:
    the binding's checks, the output allocations by torch's caching allocator,
    the saved tensors and the workspace cache are all inside the timed region
    (`out = m(x); out.backward(g)` between events, rotating inputs).  Each row
    carries the rate of the C-ABI pair of the kernel table and the ratio."""
    torch = L.torch
    import oslo_amd.torch.nn as onn
    from oslo_amd.torch.nn.modules.softmax import AttnMaskType

    bf = torch.bfloat16
    rows = []
    # ~5 ms of GPU work for time_queued: copies of a 2 GiB buffer
    blk_src = torch.empty(1 << 31, dtype=torch.uint8, device=dev)
    blk_dst = torch.empty(1 << 31, dtype=torch.uint8, device=dev)

    def blocker():
        for _ in range(8):
            blk_dst.copy_(blk_src, non_blocking=True)

    def abi_rate(names, cfg, note=None, exclude=None):
        sel = [r for r in kernel_rows if r[0] in names and r[1] == cfg and (note is None or r[9] == note)
               and (exclude is None or r[9] != exclude)]
        if len(sel) != len(names):
            return None
        return sum(r[2] for r in sel) / sum(r[3] for r in sel) * 1e3  # MB / us -> GB/s

    def run(name, cfg, nbytes, params, make_inputs, call, nsets, abi):
        g = torch.Generator(device=dev).manual_seed(7)
        sets = [make_inputs(g) for _ in range(nsets)]
        leaves = list(params)

        def fn(i):
            inputs, grad = sets[i]
            for t in leaves:
                t.grad = None
            for t in inputs:
                if t.requires_grad:
                    t.grad = None
            call(*inputs).backward(grad)

        t = time_launches(torch, fn, iters, nsets)
        gbps = nbytes / (t[0] * 1e-3) / 1e9
        # the same eager calls enqueued behind a few ms of other GPU work, so that the
        # host runs ahead: a call costs the host 90-130 us of Python per forward +
        # backward (autograd.Function, ctypes), more than the shorter kernels run, and
        # a loop of nothing but such calls measures Python, not the GPU
        tq = time_queued(torch, fn, nsets, blocker)
        qgbps = nbytes / (tq * 1e-3) / 1e9
        rows.append({
            "module": name, "cfg": cfg, "MB": round(nbytes / 1e6, 1), "us": round(t[0] * 1e3, 2),
            "us_med": round(t[1] * 1e3, 2), "us_min": round(t[2] * 1e3, 2), "GBps": round(gbps, 1),
            "frac": round(gbps / HBM_PEAK_GBPS, 4),
            "queued_us": round(tq * 1e3, 2), "queued_GBps": round(qgbps, 1),
            "queued_frac": round(qgbps / HBM_PEAK_GBPS, 4),
            "c_abi_GBps": None if abi is None else round(abi, 1),
            "ratio_to_c_abi": None if abi is None else round(gbps / abi, 4),
            "queued_ratio_to_c_abi": None if abi is None else round(qgbps / abi, 4),
        })
        del sets
        torch.cuda.empty_cache()

    def act(n1, n2):
        def make(g):
            x = torch.randn(n1, n2, generator=g, device=dev).to(bf).requires_grad_()
            return (x,), torch.randn(n1, n2, generator=g, device=dev).to(bf)
        return make

    # LayerNorm / RMSNorm at cfg2, LayerNorm at cfg5
    for cfg, n1, n2, kinds in (("cfg2", 16384, 4096, ("ln", "rms")), ("cfg5", 8192, 6144, ("ln",))):
        T = n1 * n2 * 2
        for kind in kinds:
            m = (onn.FusedLayerNorm if kind == "ln" else onn.FusedRMSNorm)(n2, eps=1e-5).to(dev).to(bf)
            with torch.no_grad():
                m.weight.normal_(1.0, 0.02)
                if kind == "ln":
                    m.bias.normal_(0.0, 0.02)
            run("FusedLayerNorm" if kind == "ln" else "FusedRMSNorm", cfg, 5 * T, list(m.parameters()), act(n1, n2),
                m, nsets_for(4 * T), abi_rate(("%s_fwd" % kind, "%s_bwd" % kind), cfg))

    # the four stages of cfg5
    c = CHAIN
    n1, hdim, heads, s, ff = c["tokens"], c["hidden"], 64, c["seq"], c["ffn"]
    f = (s + 1) / (2.0 * s)
    T = 4 * heads * s * s * 2
    sm = onn.FusedScaleMaskSoftmax(input_in_bf16=True, attn_mask_type=AttnMaskType.causal, scale=c["scale"])

    def make_scores(g):
        x = torch.empty(4, heads, s, s, device=dev, dtype=bf).normal_(generator=g).requires_grad_()
        return (x,), torch.empty(4, heads, s, s, device=dev, dtype=bf).normal_(generator=g)

    run("FusedScaleMaskSoftmax(causal)", "cfg5", (2 + 3 * f) * T, [], make_scores, lambda x: sm(x, None), 1,
        abi_rate(("softmax_causal_fwd", "softmax_causal_bwd"), "cfg5", exclude="plain allocations"))

    T = n1 * ff * 2
    bias_ff = (0.02 * torch.randn(ff, device=dev)).to(bf).requires_grad_()
    run("fused_bias_gelu", "cfg5", 5 * T, [bias_ff], act(n1, ff), lambda x: onn.fused_bias_gelu(x, bias_ff),
        nsets_for(4 * T), abi_rate(("bias_gelu_fwd", "bias_gelu_bwd"), "cfg5"))

    T = n1 * hdim * 2
    bias_h = (0.02 * torch.randn(hdim, device=dev)).to(bf).requires_grad_()

    def make_bda(g):
        x = torch.randn(n1, hdim, generator=g, device=dev).to(bf).requires_grad_()
        res = torch.randn(n1, hdim, generator=g, device=dev).to(bf)
        return (x, res), torch.randn(n1, hdim, generator=g, device=dev).to(bf)

    run("fused_bias_dropout_add", "cfg5", 5 * T, [bias_h], make_bda,
        lambda x, res: onn.fused_bias_dropout_add(x, bias_h, res, c["p"], True), nsets_for(5 * T),
        abi_rate(("bias_dropout_add_fwd", "bias_dropout_add_bwd"), "cfg5", "p=0.1"))
    return rows


def finalize_ab(L, dev, iters=200):
    """A/B of the second launch of the column-sum backwards (their partial rows
    are reduced by a finalize kernel that cannot start before the main kernel
    has drained): serial on one stream, as the entry points issue it, against
    the finalize on a second stream beside the next call's main kernel, eager
    (events between the streams) and as a parallel branch of a captured graph.
    Uses the measurement knob "colsum_defer" and oslo_colsum_finalize_probe of
    include/oslo_hip_testing.h.  Returns rows for the JSON line."""
    torch = L.torch
    lib = L.lib
    _C = L._C
    main = torch.cuda.current_stream()
    side = torch.cuda.Stream()
    out = []

    def ab(name, nbytes, run_main, finalize, nsets):
        _C.tune("colsum_defer", 0)
        t_serial = time_launches(torch, lambda i: run_main(i, main.cuda_stream, 0), iters, nsets)[0]
        _C.tune("colsum_defer", 1)
        ready = [torch.cuda.Event() for _ in range(2)]
        free = [torch.cuda.Event() for _ in range(2)]
        used = [False, False]

        def deferred(i):
            w = i % 2  # two workspaces: the main kernel of call i + 1 must not overwrite rows finalize(i) reads
            if used[w]:
                main.wait_event(free[w])
            run_main(i % nsets, main.cuda_stream, w)
            ready[w].record(main)
            side.wait_event(ready[w])
            finalize(side.cuda_stream, w)
            free[w].record(side)
            used[w] = True

        t_side = time_launches(torch, deferred, iters, max(2, nsets) * 2)[0]
        torch.cuda.synchronize()

        def graph_time(branch):
            _C.tune("colsum_defer", 1 if branch else 0)
            cap, br = torch.cuda.Stream(), torch.cuda.Stream()
            g = torch.cuda.CUDAGraph()
            cap.wait_stream(main)
            reps = 12
            with torch.cuda.stream(cap):
                with torch.cuda.graph(g, stream=cap):
                    for k in range(reps):
                        run_main(k % nsets, cap.cuda_stream, k % 2)
                        if branch:
                            br.wait_stream(cap)
                            finalize(br.cuda_stream, k % 2)
                            if k % 2 == 1:
                                cap.wait_stream(br)  # both workspaces free again
                    if branch:
                        cap.wait_stream(br)
            main.wait_stream(cap)
            torch.cuda.synchronize()
            for _ in range(3):
                g.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(8):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / (8 * reps)

        tg_serial, tg_branch = graph_time(False), graph_time(True)
        _C.tune("colsum_defer", 0)
        out.append({"kernel": name, "MB": round(nbytes / 1e6, 1),
                    "serial_us": round(t_serial * 1e3, 2), "side_stream_us": round(t_side * 1e3, 2),
                    "graph_serial_us": round(tg_serial * 1e3, 2), "graph_branch_us": round(tg_branch * 1e3, 2)})

    for cfg, n1, n2 in (("cfg5", 8192, 6144), ("cfg2", 16384, 4096)):
        T = n1 * n2 * 2
        ns = nsets_for(4 * T)
        sets, gamma, beta, dgamma, dbeta = norm_buffers(torch, dev, n1, n2, ns, 1)
        wss = [L.ws(_C.OSLO_OP_LN_BWD, n1, n2, dev) for _ in range(2)]
        for s_ in sets:
            L.ok(lib.oslo_ln_fwd(p(s_["x"]), p(gamma), p(beta), p(s_["y"]), p(s_["mean"]), p(s_["invvar"]), n1, n2,
                                 1e-5, BF16, BF16, main.cuda_stream))
        parts = wss[0][1] // (2 * n2 * 4)

        def run_main(i, st, w):
            s_ = sets[i]
            L.ok(lib.oslo_ln_bwd(p(s_["dy"]), p(s_["x"]), p(s_["mean"]), p(s_["invvar"]), p(gamma), p(s_["dx"]),
                                 p(dgamma), p(dbeta), p(wss[w][0]), wss[w][1], n1, n2, BF16, BF16, st))

        def fin(st, w):
            L.ok(lib.oslo_colsum_finalize_probe(p(wss[w][0]), parts, n2, p(dgamma), p(dbeta), None, BF16, st))

        ab("ln_bwd " + cfg, 3 * T, run_main, fin, ns)
        del sets
        torch.cuda.empty_cache()

    n1, n2 = 8192, 6144
    T = n1 * n2 * 2
    ns = nsets_for(5 * T)
    g = torch.Generator(device=dev).manual_seed(5)
    gs = [torch.randn(n1, n2, generator=g, device=dev).to(torch.bfloat16) for _ in range(ns)]
    dxs = [torch.empty_like(t) for t in gs]
    dbias = torch.empty(n2, device=dev, dtype=torch.bfloat16)
    wss = [L.ws(_C.OSLO_OP_BIAS_DROPOUT_ADD_BWD, n1, n2, dev) for _ in range(2)]
    parts = wss[0][1] // (n2 * 4)

    def run_bda(i, st, w):
        L.ok(lib.oslo_bias_dropout_add_bwd(p(gs[i]), p(dxs[i]), p(dbias), p(wss[w][0]), wss[w][1], n1, n2, 0.1, 1234,
                                           0, BF16, st))

    def fin_bda(st, w):
        L.ok(lib.oslo_colsum_finalize_probe(p(wss[w][0]), parts, n2, p(dbias), None, None, BF16, st))

    ab("bias_dropout_add_bwd cfg5", 2 * T, run_bda, fin_bda, ns)
    return out


def cpu_model():
    """Model string of the host CPU with family / model / stepping (a virtual
    machine may shorten the name) and the number of logical CPUs."""
    fields = {}
    try:
        for line in open("/proc/cpuinfo"):
            if ":" in line:
                k, v = line.split(":", 1)
                k = k.strip()
                if k in ("model name", "cpu family", "model", "stepping", "vendor_id") and k not in fields:
                    fields[k] = v.strip()
    except OSError:
        pass
    if not fields:
        return "unknown"
    return "%s (%s family %s model %s stepping %s), %d logical CPUs" % (
        fields.get("model name", "?"), fields.get("vendor_id", "?"), fields.get("cpu family", "?"),
        fields.get("model", "?"), fields.get("stepping", "?"), os.cpu_count() or 0)


def cpu_baseline(budget_s=4.0):
    """The reference's unfused torch path for the chain of the headline step on
    the host cores.  Each stage runs on a bounded sample of its rows (the CPU
    rate does not depend on the row count at these sizes) and its time is
    scaled to the full stage; `value` = the step's algorithmic bytes / the sum
    of the scaled stage times."""
    import torch

    from oracle import torch_path as tp

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    bf = torch.bfloat16
    c = CHAIN

    def rnd(shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(shape, generator=g)).to(bf)

    def timed(fn):
        fn()
        times, spent = [], 0.0
        while len(times) < 3 or (spent < budget_s and len(times) < 200):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
            spent += times[-1]
        measured[0] += spent
        runs.append(len(times))
        times.sort()
        return times[len(times) // 2]

    stages, measured, runs = [], [0.0], []
    # LayerNorm: the whole [8192, 6144] tensor (a smaller sample would stay in the host caches)
    n1, h = c["tokens"], c["hidden"]
    x, dy = rnd((n1, h)).requires_grad_(), rnd((n1, h))
    gamma, beta = rnd((h,), 0.02, 1.0).requires_grad_(), rnd((h,), 0.02).requires_grad_()

    def ln():
        x.grad = gamma.grad = beta.grad = None  # (no copy of an input inside the timed function)
        tp.layer_norm(x, gamma, beta, 1e-5).backward(dy)
    stages.append(("layer_norm", "[8192,6144] (all)", timed(ln), 1.0))
    # causal softmax: 32 of the 256 attention batches
    s = c["seq"]
    xs, ds = rnd((32, s, s)).requires_grad_(), rnd((32, s, s))

    def sm():
        xs.grad = None
        tp.causal_softmax(xs, c["scale"]).backward(ds)
    stages.append(("softmax_causal", "[32,2048,2048] of 256 batches", timed(sm), c["attn_batches"] / 32.0))
    del xs, ds
    # bias-GeLU: 4096 of the 8192 rows
    xg, dg, bg = rnd((4096, c["ffn"])).requires_grad_(), rnd((4096, c["ffn"])), rnd((c["ffn"],), 0.02).requires_grad_()

    def ge():
        xg.grad = bg.grad = None
        tp.bias_gelu(xg, bg).backward(dg)
    stages.append(("bias_gelu", "[4096,24576] of 8192 rows", timed(ge), n1 / 4096.0))
    del xg, dg
    # bias-dropout-add: the whole [8192, 6144] tensor
    xb, rb, db, bb = rnd((n1, h)).requires_grad_(), rnd((n1, h)), rnd((n1, h)), rnd((h,), 0.02).requires_grad_()

    def bd():
        xb.grad = bb.grad = None
        tp.bias_dropout_add(xb, bb, rb, c["p"], True).backward(db)
    stages.append(("bias_dropout_add", "[8192,6144] (all)", timed(bd), 1.0))

    full_s = sum(t * k for _, _, t, k in stages)
    nbytes = sum(b for _, b in chain_bytes())
    return {
        "value": round(nbytes / full_s / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "cpu": cpu_model(),
        "kind": "port",
        "sample": "forward + backward through torch CPU ops and autograd, bf16, median of %d-%d runs per stage "
                  "(%.0f s of timed CPU work per stage at most); " % (min(runs), max(runs), budget_s)
                  + "; ".join("%s %s %.2f s x %g" % (n, smp, t, k) for n, smp, t, k in stages)
                  + "; stage times scaled to the full stage and summed",
        "ms_per_step_scaled": round(full_s * 1e3, 1),
        "cpu_seconds_measured": round(measured[0], 1),
    }


def cpu_path_table(gpu_rows, budget_s=3.0):
    """The reference's unfused torch path, forward + backward, for every
    configuration, on the host cores and on a BOUNDED sample of the rows (the
    CPU rate does not depend on the row count at these sizes); each entry
    carries the GPU rate of the same forward + backward pair from the kernel
    table and their ratio.  At most `budget_s` seconds of timed work per entry."""
    import torch

    from oracle import torch_path as tp

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)

    def rnd(shape, dtype, std=1.0):
        return (std * torch.randn(shape, generator=g)).to(dtype)

    def gpu_rate(names, cfg, note=None):
        rows = [r for r in gpu_rows if r[0] in names and r[1] == cfg and r[9] != "plain allocations"
                and (note is None or r[9] == note)]
        if len(rows) != len(names):
            return None
        return sum(r[2] for r in rows) / sum(r[3] for r in rows) * 1e3

    def timed(fn):
        fn()
        times, spent = [], 0.0
        while len(times) < 3 and spent < budget_s:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
            spent += times[-1]
        times.sort()
        return times[len(times) // 2]

    BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32
    out = []

    def entry(name, cfg, sample, nbytes, fn, gpu):
        t = timed(fn)
        cpu = nbytes / t / 1e9
        out.append({
            "kernel": name, "config": cfg, "sample": sample, "cores": threads,
            "cpu_ms": round(t * 1e3, 1), "cpu_GBps": round(cpu, 2),
            "gpu_GBps": None if gpu is None else round(gpu, 1),
            "gpu_frac": None if gpu is None else round(gpu / HBM_PEAK_GBPS, 4),
            "speedup": None if gpu is None else round(gpu / cpu, 1),
        })

    def causal(cfg, ab, s, dtype, scale, esz):
        x, dy = rnd((ab, s, s), dtype).requires_grad_(), rnd((ab, s, s), dtype)
        f = (s + 1) / (2.0 * s)

        def fn():
            x.grad = None  # (no copy of an input inside the timed function)
            tp.causal_softmax(x, scale).backward(dy)
        entry("softmax_causal fwd+bwd", cfg, "[%d,%d,%d] %s" % (ab, s, s, str(dtype).split(".")[-1]),
              (2 + 3 * f) * ab * s * s * esz, fn,
              gpu_rate(("softmax_causal_fwd", "softmax_causal_bwd"), cfg))

    def norm_ln(cfg, n1, n2):
        x, dy = rnd((n1, n2), BF16).requires_grad_(), rnd((n1, n2), BF16)
        gamma, beta = (rnd((n2,), BF16, 0.02) + 1).requires_grad_(), rnd((n2,), BF16, 0.02).requires_grad_()

        def fn():
            x.grad = gamma.grad = beta.grad = None
            tp.layer_norm(x, gamma, beta, 1e-5).backward(dy)
        entry("layer_norm fwd+bwd", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("ln_fwd", "ln_bwd"), cfg))

    def norm_rms(cfg, n1, n2):
        x, dy = rnd((n1, n2), BF16).requires_grad_(), rnd((n1, n2), BF16)
        gamma = (rnd((n2,), BF16, 0.02) + 1).requires_grad_()

        def fn():
            x.grad = gamma.grad = None
            tp.rms_norm(x, gamma, 1e-5).backward(dy)
        entry("rms_norm fwd+bwd", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("rms_fwd", "rms_bwd"), cfg))

    def gelu(cfg, n1, n2):
        x, dy, b = rnd((n1, n2), BF16).requires_grad_(), rnd((n1, n2), BF16), rnd((n2,), BF16, 0.02).requires_grad_()

        def fn():
            x.grad = b.grad = None
            tp.bias_gelu(x, b).backward(dy)
        entry("bias_gelu fwd+bwd", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("bias_gelu_fwd", "bias_gelu_bwd"), cfg))

    def bda(cfg, n1, n2):
        x, res, dy = rnd((n1, n2), BF16).requires_grad_(), rnd((n1, n2), BF16), rnd((n1, n2), BF16)
        b = rnd((n2,), BF16, 0.02).requires_grad_()

        def fn():
            x.grad = b.grad = None
            tp.bias_dropout_add(x, b, res, 0.1, True).backward(dy)
        entry("bias_dropout_add fwd+bwd (p=0.1)", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("bias_dropout_add_fwd", "bias_dropout_add_bwd"), cfg, "p=0.1"))

    causal("cfg1", 48, 512, F32, 0.125, 4)
    norm_ln("cfg2", 16384, 4096)
    norm_rms("cfg2", 16384, 4096)
    # cfg3: two of the sixteen batch entries
    b_, h, s = 2, 16, 1024
    x, dy = rnd((b_, h, s, s), F16, 2.0).requires_grad_(), rnd((b_, h, s, s), F16)
    valid = torch.tensor([1024, 640])
    pad = torch.arange(s)[None, :] >= valid[:, None]
    r = float(valid.double().mean()) / s

    def masked():
        x.grad = None
        tp.padding_softmax(x, pad, 0.125).backward(dy)
    entry("softmax_masked fwd+bwd", "cfg3", "[2,16,1024,1024] fp16 of batch 16", (2 + 3 * r) * x.numel() * 2,
          masked, gpu_rate(("softmax_masked_fwd", "softmax_masked_bwd"), "cfg3"))
    del x, dy
    gelu("cfg4", 2048, 16384)
    bda("cfg4", 4096, 4096)
    norm_ln("cfg5", 8192, 6144)  # whole: a smaller sample would stay in the host caches
    causal("cfg5", 8, 2048, BF16, 1.0 / math.sqrt(96.0), 2)
    gelu("cfg5", 1024, 24576)
    bda("cfg5", 2048, 6144)
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.stderr.write(
            "bench.py: this build measures one GPU only (the path has no collectives); "
            "run with --gpus 1.\n"
        )
        sys.exit(2)

    import torch

    from oslo_amd.torch import _C

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = Lib(torch, _C)

    if args.finalize_ab:
        print(json.dumps({"finalize_ab": finalize_ab(L, dev, max(20, args.table_iters))}))
        return

    if args.tune_ab:
        key, _, values = args.tune_ab.partition("=")
        fixed = [kv.split("=") for kv in args.tune_fixed.split(",") if kv]
        out = {"knob": key, "fixed": args.tune_fixed, "only": args.only, "iters": max(20, args.table_iters),
               "cols": TABLE_COLS, "values": {}}
        for v in [int(t) for t in values.split(",")]:
            for fk, fv in fixed:
                _C.tune(fk, int(fv))
            _C.tune(key, v)
            try:
                rows = kernel_table(L, dev, out["iters"], graph_column=False)
            finally:
                _C.tune(key, 0)
                for fk, _ in fixed:
                    _C.tune(fk, 0)
            out["values"][str(v)] = [r for r in rows if args.only in r[0]]
        print(json.dumps({"tune_ab": out}))
        return

    # the counter summary must hold the roofline kernel's row: fail before timing anything
    try:
        traffic = traffic_from_profile(ROOF_KERNEL, ROOF_BLOCKS, ROOF_WG)
    except RuntimeError:
        if not args.traffic_optional:
            raise
        traffic = None

    calls, keep = make_chain(L, dev)
    names_bytes = chain_bytes()
    step_bytes = sum(b for _, b in names_bytes)
    roof_idx = 3  # softmax_causal_bwd: the step's largest launch
    roof_bytes = names_bytes[roof_idx][1]

    def step():
        for fn in calls:
            fn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        for k, fn in enumerate(calls):
            if k == roof_idx:
                ev[i][0].record()
                fn()
                ev[i][1].record()
            else:
                fn()
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_per_step = (t1 - t0) * 1e3 / max(args.steps, 1)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    roof_ms = sum(a.elapsed_time(b) for a, b in ev) / max(len(ev), 1)
    achieved = roof_bytes / (roof_ms * 1e-3) / 1e9

    out = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE.json configs[4]: GPT-NeoX-20B-layer-shaped non-GEMM chain fwd+bwd, bf16, batch 4, "
                        "seq 2048, hidden 6144, 64 heads; step = ln_fwd, ln_bwd [8192,6144], softmax_causal_fwd, _bwd "
                        "[256,2048,2048], bias_gelu_fwd, _bwd [8192,24576], bias_dropout_add_fwd, _bwd [8192,6144] p=0.1",
            "io_dtype": "bf16",
            "algorithmic_MB_per_step": round(step_bytes / 1e6, 1),
            "algorithmic_MB_per_launch": {n: round(b / 1e6, 1) for n, b in names_bytes},
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "roofline": {
            "kernel": "oslo_softmax_causal_bwd = softmax_bwd_kernel<bf16, 4 chunks per lane, 1 row per wave, causal> "
                      "(524288 x 64)",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_unit": "HBM bytes per launch: rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy, read "
                            "from profiles/bench_all_kernels_hbm_traffic.txt",
            "algorithmic_MB_per_launch": round(roof_bytes / 1e6, 1),
            "avg_us": round(roof_ms * 1e3, 2),
        },
    }
    del calls, keep
    torch.cuda.empty_cache()

    if args.table_iters > 0:
        rows = kernel_table(L, dev, args.table_iters, graph_column=not args.no_graph_column)
        out["kernels"] = {
            "cols": TABLE_COLS,
            "units": "MB = algorithmic bytes per launch / 1e6; us = mean over %d launches (events on the launch "
                     "stream, %d batches), us_med / us_min = median / smallest batch mean; frac = GBps / 8000; "
                     "graph_us = per launch inside a captured HIP graph; mt_* = multi-tensor optimizer steps over "
                     "192 tensors; copy_probe = a plain copy" % (args.table_iters, BATCHES),
            "rows": rows,
        }
    if args.table_iters > 0 and not args.no_modules:
        out["modules"] = {
            "what": "forward + backward through oslo_amd.torch.nn with autograd (out = m(x); out.backward(g) between "
                    "events on the launch stream, rotating inputs, gradients cleared to None before each call); MB = "
                    "algorithmic bytes of the pair; c_abi_GBps = the same pair through the raw C ABI on pre-allocated "
                    "buffers (kernel table); ratio_to_c_abi = GBps / c_abi_GBps; us / GBps = a loop of nothing but "
                    "these calls (bound by the 90-130 us of Python per call where the kernels are shorter); queued_* "
                    "= the same eager calls enqueued behind ~5 ms of other GPU work, so that the host runs ahead of "
                    "the GPU as it does in a training step (events on the stream bracket the calls' GPU time)",
            "rows": module_table(L, dev, max(20, args.table_iters // 2), rows),
        }
    if not args.no_cpu_baseline:
        cb = cpu_baseline()
        cb["speedup_gpu_over_cpu"] = round(value / cb["value"], 1) if cb["value"] > 0 else None
        out["cpu_baseline"] = cb
        if "kernels" in out:
            out["cpu_path"] = cpu_path_table(out["kernels"]["rows"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
