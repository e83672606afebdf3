#!/usr/bin/env python3
"""Benchmark of the fused non-GEMM kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (BASELINE.json configs[1]): LayerNorm and RMSNorm forward +
backward on a bf16 [16384, 4096] activation.  One step = LN fwd, LN bwd, RMS
fwd, RMS bwd over one batch, called through the C ABI with every buffer
resident in HBM and pre-allocated; buffer sets rotate so the 256 MB Infinity
Cache cannot serve the reads.  `value` = algorithmic bytes of a step (10 T,
T = 134.2 MB) / wall time per step.

Prints ONE JSON line.  Beside the contract's keys it carries
  roofline      the dominant launch (LN backward), timed with events on the
                launch stream inside the timed region,
  cpu_baseline  the reference's unfused torch path (oracle/torch_path.py) on
                the host cores, same workload,
  kernels       achieved GB/s and fraction of the 8 TB/s HBM peak for every
                fused kernel of BASELINE.json's five configurations,
  cpu_path      the reference's unfused torch path, forward + backward, for
                the other four configurations on bounded samples, with the
                GPU rate of the same pair and their ratio.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
METRIC = "achieved HBM GB/s (% of MI355X peak) per fused fwd+bwd kernel; speedup vs CPU path"
# HBM traffic of one LayerNorm-backward call on bf16 [16384, 4096], measured with
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and calibrated against a 1 GiB copy:
# main kernel 270.9 MB read + 142.6 MB written, finalize 8.4 MB read
# (summary: profiles/bench_all_kernels_hbm_traffic.txt).  Algorithmic: 402.7 MB.
LN_BWD_TRAFFIC_BYTES = 421.9e6

F32, F16, BF16 = 0, 1, 2


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--table-iters", type=int, default=200, help="launches per kernel in the per-kernel table (0 = skip)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-reps", type=int, default=15)
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


def time_launches(torch, fn, iters, nsets):
    """Average duration in ms of fn(i % nsets), events on the current stream."""
    # warm-up: every buffer set is touched, 20 launches ahead of a long timed region
    for i in range(max(3, nsets, min(20, iters // 10))):
        fn(i % nsets)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        fn(i % nsets)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


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


def table_row(name, cfg, shape, dtype, nbytes, ms):
    gbps = nbytes / (ms * 1e-3) / 1e9
    return {
        "kernel": name, "config": cfg, "shape": shape, "io_dtype": dtype,
        "algorithmic_MB": round(nbytes / 1e6, 1), "us": round(ms * 1e3, 2),
        "GBps": round(gbps, 1), "frac_of_peak": round(gbps / HBM_PEAK_GBPS, 4),
    }


def nsets_for(total_bytes_per_set):
    """Enough rotating sets that consecutive launches cannot hit in the 256 MB cache."""
    return max(1, min(8, math.ceil(1.0e9 / max(total_bytes_per_set, 1))))


def kernel_table(L, dev, iters):
    """Every fused kernel at the shapes of BASELINE.json's five configurations."""
    torch = L.torch
    lib = L.lib
    rows = []

    def timed(fn, nsets):
        return time_launches(torch, fn, iters, nsets)

    # ---- LayerNorm / RMSNorm: cfg2 and cfg5 ----
    for cfg, n1, n2 in (("cfg2", 16384, 4096), ("cfg5", 8192, 6144)):
        T = n1 * n2 * 2
        ns = nsets_for(4 * T)
        calls = make_norm_calls(L, dev, n1, n2, ns, seed=1)
        for name, mult in (("ln_fwd", 2), ("ln_bwd", 3), ("rms_fwd", 2), ("rms_bwd", 3)):
            if cfg == "cfg5" and name.startswith("rms"):
                continue
            if name.endswith("bwd"):
                calls[name.replace("bwd", "fwd")](0)
                for i in range(ns):
                    calls[name.replace("bwd", "fwd")](i)
            rows.append(table_row(name, cfg, [n1, n2], "bf16", mult * T, timed(calls[name], ns)))
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
            x = torch.randn(ab, s, s, generator=g, device=dev).to(tdt)
            dy = torch.randn(ab, s, s, generator=g, device=dev).to(tdt)
            bufs.append((x, torch.empty_like(x), dy, torch.empty_like(x)))

        def fwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_causal_fwd(p(x), p(y), ab, s, s, scale, code, L.stream()))

        def bwd(i):
            x, y, dy, dx = bufs[i]
            L.ok(lib.oslo_softmax_causal_bwd(p(dy), p(y), p(dx), ab, s, s, scale, code, L.stream()))

        rows.append(table_row("softmax_causal_fwd", cfg, [ab, s, s], str(tdt).split(".")[-1], (1 + f) * T, timed(fwd, ns)))
        rows.append(table_row("softmax_causal_bwd", cfg, [ab, s, s], str(tdt).split(".")[-1], (1 + 2 * f) * T, timed(bwd, ns)))

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

        for name, fn, nbytes in (("softmax_causal_dropout_fwd", dfwd, (1 + f) * T), ("softmax_causal_dropout_bwd", dbwd, (1 + 2 * f) * T)):
            row = table_row(name, cfg, [ab, s, s], str(tdt).split(".")[-1], nbytes, timed(fn, ns))
            row["p"] = 0.1
            rows.append(row)
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

    row = table_row("softmax_masked_fwd", "cfg3", [b, h, s, s], "float16", (r + 1) * T, timed(mfwd, ns))
    row["valid_fraction"] = round(r, 4)
    row["dense_equiv_GBps"] = round(2 * T / (row["us"] * 1e-6) / 1e9, 1)
    rows.append(row)
    row = table_row("softmax_masked_bwd", "cfg3", [b, h, s, s], "float16", (2 * r + 1) * T, timed(mbwd, ns))
    row["valid_fraction"] = round(r, 4)
    row["dense_equiv_GBps"] = round(3 * T / (row["us"] * 1e-6) / 1e9, 1)
    rows.append(row)
    del bufs
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

        rows.append(table_row("bias_gelu_fwd", cfg, [n1, n2], "bf16", 2 * T, timed(gfwd, ns)))
        rows.append(table_row("bias_gelu_bwd", cfg, [n1, n2], "bf16", 3 * T, timed(gbwd, ns)))
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
        r1 = table_row("bias_dropout_add_fwd", cfg, [n1, n2], "bf16", 3 * T, timed(dfwd, ns))
        r2 = table_row("bias_dropout_add_bwd", cfg, [n1, n2], "bf16", 2 * T, timed(dbwd, ns))
        r1["p"] = r2["p"] = pdrop
        rows += [r1, r2]

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

            r3 = table_row("bias_dropout_add_ln_fwd", cfg, [n1, n2], "bf16", 4 * T, timed(ffwd, ns))
            for i in range(ns):
                ffwd(i)
            r4 = table_row("bias_dropout_add_ln_bwd", cfg, [n1, n2], "bf16", 4 * T, timed(fbwd, ns))
            r3["p"] = r4["p"] = pdrop
            rows += [r3, r4]
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
    for tdt, code, esz in ((torch.float32, F32, 4), (torch.bfloat16, BF16, 2)):
        lists = [[torch.zeros(s, device=dev, dtype=tdt) for s in shapes] for _ in range(4)]
        for t in lists[0]:
            t.normal_()
        nel = sum(t.numel() for t in lists[0])
        n = len(shapes)
        arr = ctypes.c_void_p * n
        tables = [arr(*[t.data_ptr() for t in lst]) for lst in lists]
        sizes = (ctypes.c_int64 * n)(*[t.numel() for t in lists[0]])
        step_no = [0]

        def adam(i):
            step_no[0] += 1
            L.ok(lib.oslo_multi_tensor_adam(tables[0], tables[1], tables[2], tables[3], sizes, n, 1e-3, 0.9, 0.999,
                                            1e-8, step_no[0], 1, 1, 0.01, code, L.stream()))

        row = table_row("multi_tensor_adam", "-", [n, nel], str(tdt).split(".")[-1], 7 * nel * esz, timed(adam, 1))
        row["tensors"] = n
        rows.append(row)
        del lists, tables
        torch.cuda.empty_cache()

    # ---- plain copy with the same load/store path: the practical ceiling ----
    nbytes = 1 << 30
    src = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(2)]
    dst = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(2)]
    for s_ in src:
        s_.fill_(1)

    def cp(i):
        L.ok(lib.oslo_copy_probe(p(src[i]), p(dst[i]), nbytes, L.stream()))

    rows.append(table_row("copy_probe", "-", [nbytes], "u8", 2 * nbytes, timed(cp, 2)))
    return rows


def cpu_baseline(n1, n2, reps):
    """The reference's unfused torch path on the host cores, same workload."""
    import torch

    from oracle import torch_path as tp

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(n1, n2, generator=g).to(torch.bfloat16)
    dy = torch.randn(n1, n2, generator=g).to(torch.bfloat16)
    gamma = (1 + 0.02 * torch.randn(n2, generator=g)).to(torch.bfloat16)
    beta = (0.02 * torch.randn(n2, generator=g)).to(torch.bfloat16)

    def step():
        xr = x.clone().requires_grad_()
        w, b = gamma.clone().requires_grad_(), beta.clone().requires_grad_()
        tp.layer_norm(xr, w, b, 1e-5).backward(dy)
        xr = x.clone().requires_grad_()
        w = gamma.clone().requires_grad_()
        tp.rms_norm(xr, w, 1e-5).backward(dy)

    step()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    nbytes = 10 * n1 * n2 * 2
    return {
        "value": round(nbytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": "full workload [%d,%d] bf16, LN+RMS fwd+bwd via torch CPU ops (F.layer_norm, manual_rms_norm, autograd), "
                  "median of %d reps, %.2f s each" % (n1, n2, reps, med),
        "ms_per_step": round(med * 1e3, 1),
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

    def gpu_rate(names, cfg, **match):
        rows = [r for r in gpu_rows if r["kernel"] in names and r["config"] == cfg
                and all(r.get(k) == v for k, v in match.items())]
        if len(rows) != len(names):
            return None
        return sum(r["algorithmic_MB"] for r in rows) / sum(r["us"] for r in rows) * 1e3

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
            "speedup": None if gpu is None else round(gpu / cpu, 1),
        })

    def causal(cfg, ab, s, dtype, scale, esz):
        x, dy = rnd((ab, s, s), dtype), rnd((ab, s, s), dtype)
        f = (s + 1) / (2.0 * s)

        def fn():
            xr = x.clone().requires_grad_()
            tp.causal_softmax(xr, scale).backward(dy)
        entry("softmax_causal fwd+bwd", cfg, "[%d,%d,%d] %s" % (ab, s, s, str(dtype).split(".")[-1]),
              (2 + 3 * f) * ab * s * s * esz, fn,
              gpu_rate(("softmax_causal_fwd", "softmax_causal_bwd"), cfg))

    def norm_ln(cfg, n1, n2):
        x, dy = rnd((n1, n2), BF16), rnd((n1, n2), BF16)
        gamma, beta = rnd((n2,), BF16, 0.02) + 1, rnd((n2,), BF16, 0.02)

        def fn():
            xr = x.clone().requires_grad_()
            w, b = gamma.clone().requires_grad_(), beta.clone().requires_grad_()
            tp.layer_norm(xr, w, b, 1e-5).backward(dy)
        entry("layer_norm fwd+bwd", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("ln_fwd", "ln_bwd"), cfg))

    def gelu(cfg, n1, n2):
        x, dy, b = rnd((n1, n2), BF16), rnd((n1, n2), BF16), rnd((n2,), BF16, 0.02)

        def fn():
            xr, br = x.clone().requires_grad_(), b.clone().requires_grad_()
            tp.bias_gelu(xr, br).backward(dy)
        entry("bias_gelu fwd+bwd", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("bias_gelu_fwd", "bias_gelu_bwd"), cfg))

    def bda(cfg, n1, n2):
        x, res, dy, b = rnd((n1, n2), BF16), rnd((n1, n2), BF16), rnd((n1, n2), BF16), rnd((n2,), BF16, 0.02)

        def fn():
            xr, br = x.clone().requires_grad_(), b.clone().requires_grad_()
            tp.bias_dropout_add(xr, br, res, 0.1, True).backward(dy)
        entry("bias_dropout_add fwd+bwd (p=0.1)", cfg, "[%d,%d] bf16" % (n1, n2), 5 * n1 * n2 * 2, fn,
              gpu_rate(("bias_dropout_add_fwd", "bias_dropout_add_bwd"), cfg, p=0.1))

    causal("cfg1", 48, 512, F32, 0.125, 4)
    # cfg3: two of the sixteen batch entries
    b_, h, s = 2, 16, 1024
    x, dy = rnd((b_, h, s, s), F16, 2.0), rnd((b_, h, s, s), F16)
    valid = torch.tensor([1024, 640])
    pad = torch.arange(s)[None, :] >= valid[:, None]
    r = float(valid.double().mean()) / s

    def masked():
        xr = x.clone().requires_grad_()
        tp.padding_softmax(xr, pad, 0.125).backward(dy)
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

    n1, n2 = 16384, 4096
    T = n1 * n2 * 2
    nsets = 4
    calls = make_norm_calls(L, dev, n1, n2, nsets, seed=0)

    def step(i):
        k = i % nsets
        calls["ln_fwd"](k)
        calls["ln_bwd"](k)
        calls["rms_fwd"](k)
        calls["rms_bwd"](k)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        k = i % nsets
        calls["ln_fwd"](k)
        ev[i][0].record()
        calls["ln_bwd"](k)
        ev[i][1].record()
        calls["rms_fwd"](k)
        calls["rms_bwd"](k)
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    step_bytes = 10 * T
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    bwd_ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
    achieved = 3 * T / (bwd_ms * 1e-3) / 1e9

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
            "workload": "BASELINE.json configs[1]: LayerNorm + RMSNorm fwd+bwd, bf16 [16384,4096], eps 1e-5; "
                        "step = ln_fwd, ln_bwd, rms_fwd, rms_bwd",
            "io_dtype": "bf16",
            "algorithmic_MB_per_step": round(step_bytes / 1e6, 1),
            "rotating_buffer_sets": nsets,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "roofline": {
            "kernel": "oslo_ln_bwd = norm_bwd_reg_kernel + colsum_finalize_kernel",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": LN_BWD_TRAFFIC_BYTES,
            "traffic_unit": "HBM bytes per oslo_ln_bwd call, rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy",
            "algorithmic_MB_per_launch": round(3 * T / 1e6, 1),
            "avg_us": round(bwd_ms * 1e3, 2),
        },
    }
    del calls
    torch.cuda.empty_cache()

    if args.table_iters > 0:
        out["kernels"] = kernel_table(L, dev, args.table_iters)
    if not args.no_cpu_baseline:
        cb = cpu_baseline(n1, n2, args.cpu_reps)
        cb["speedup_gpu_over_cpu"] = round(value / cb["value"], 1) if cb["value"] > 0 else None
        out["cpu_baseline"] = cb
        if "kernels" in out:
            out["cpu_path"] = cpu_path_table(out["kernels"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
