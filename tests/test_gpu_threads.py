"""Concurrent use of the library: several host threads, each on a stream of its
own, call the entry points at the same time.  The library holds no shared
mutable state besides a per-thread error string, and every kernel is
deterministic, so each thread's results must equal, bit for bit, what the same
calls return when run alone.  (The reference enqueues on the current stream and
is called from autograd's worker threads,
oslo/torch/_C/csrc/fused_layer_norm.cu:746, 813.)"""
import threading

import pytest
import torch

from helpers import randn
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def _work(device, seed):
    ln = _C.get_layernorm_kernel()
    sm = _C.get_softmax_kernel()
    ek = _C.get_fused_elementwise_kernel()
    n1, n2 = 192 + 8 * seed, 1024
    x = randn((n1, n2), BF16, seed).to(device)
    dy = randn((n1, n2), BF16, seed + 50).to(device)
    gamma = randn((n2,), BF16, seed + 1, std=0.02, mean=1.0).to(device)
    beta = randn((n2,), BF16, seed + 2, std=0.02).to(device)
    sc = randn((3, 128, 128), BF16, seed + 3).to(device)
    outs = []
    for it in range(8):
        y, mean, invvar = ln.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
        dx, dg, db = ln.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, 1e-5)
        r, rinv = ln.rms_norm_forward_affine(x, (n2,), gamma, 1e-5)
        rdx, rdg = ln.rms_norm_backward_affine(dy, rinv, x, (n2,), gamma, 1e-5)
        act = ek.bias_gelu_forward(y, beta)
        dact, dbias = ek.bias_gelu_backward(dx, y, beta)
        out = ek.bias_dropout_add_forward(act, beta, x, 0.1, seed, it)
        g_in, g_b = ek.bias_dropout_add_backward(dact, 0.1, seed, it)
        p = sm.fused_scaled_upper_triang_masked_softmax_forward(sc, 0.125)
        dp = sm.fused_scaled_upper_triang_masked_softmax_backward(sc.clone(), p, 0.125)
        outs += [y, dx, dg, db, r, rdx, rdg, act, dact, dbias, out, g_in, g_b, p, dp]
        x = (x + 0.01 * dx).contiguous()
    return outs


def test_threads_on_their_own_streams_match_the_serial_results(device):
    nthreads = 4
    want = [_work(device, s) for s in range(nthreads)]
    torch.cuda.synchronize()
    got = [None] * nthreads
    errors = []
    start = threading.Barrier(nthreads)

    def run(i):
        try:
            stream = torch.cuda.Stream(device=device)
            start.wait(timeout=60)
            with torch.cuda.stream(stream):
                got[i] = _work(device, i)
            stream.synchronize()
        except Exception as exc:  # reported by the parent thread
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(nthreads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    assert not errors, errors
    assert all(not t.is_alive() for t in threads)
    torch.cuda.synchronize()
    for i in range(nthreads):
        assert len(got[i]) == len(want[i])
        for k, (a, b) in enumerate(zip(got[i], want[i])):
            assert torch.equal(a, b), "thread %d, output %d differs" % (i, k)


def test_threads_that_share_the_default_stream_match_the_serial_results(device):
    """Two host threads on one stream (autograd's worker thread and the main
    thread are the everyday case): a backward entry point launches a main
    kernel and a finalize kernel that share a workspace, and the binding keeps
    one workspace per stream, so it must hand it out for whole calls only --
    were the launches of two calls to interleave, one call's finalize would
    read the other's partial rows."""
    ln = _C.get_layernorm_kernel()
    ek = _C.get_fused_elementwise_kernel()
    n2 = 1024
    gamma = randn((n2,), BF16, 1, std=0.02, mean=1.0).to(device)
    beta = randn((n2,), BF16, 2, std=0.02).to(device)
    nthreads, iters = 2, 40
    data = []
    for i in range(nthreads):
        n1 = 1024 + 512 * i
        x = randn((n1, n2), BF16, 10 + i).to(device)
        dy = randn((n1, n2), BF16, 20 + i).to(device)
        _, mean, invvar = ln.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
        data.append((x, dy, mean, invvar))

    def work(i):
        x, dy, mean, invvar = data[i]
        outs = []
        for _ in range(iters):
            dx, dg, db = ln.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, 1e-5)
            dact, dbias = ek.bias_gelu_backward(dy, x, beta)
            g_in, g_b = ek.bias_dropout_add_backward(dy, 0.1, 5, 8)
            outs.append((dg, db, dbias, g_b))
        return outs

    want = [work(i)[0] for i in range(nthreads)]
    torch.cuda.synchronize()
    got = [None] * nthreads
    errors = []
    start = threading.Barrier(nthreads)

    def run(i):
        try:
            start.wait(timeout=60)
            got[i] = work(i)        # torch's current stream of a new thread is the default stream
        except Exception as exc:  # reported by the parent thread
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(nthreads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    assert not errors, errors
    assert all(not t.is_alive() for t in threads)
    torch.cuda.synchronize()
    for i in range(nthreads):
        for it, outs in enumerate(got[i]):
            for k, (a, b) in enumerate(zip(outs, want[i])):
                assert torch.equal(a, b), "thread %d, iteration %d, output %d differs" % (i, it, k)


def test_the_error_message_belongs_to_the_calling_thread(device):
    lib = _C.load_library()
    seen = {}

    def failing():
        # a row length of zero is rejected before anything is launched
        rc = lib.oslo_ln_fwd(None, None, None, None, None, None, 4, 0, 1e-5, 0, 0, None)
        seen["rc"] = rc
        seen["own"] = lib.oslo_hip_last_error().decode()

    t = threading.Thread(target=failing)
    # this thread's own last message, whatever it is, must not change
    before = lib.oslo_hip_last_error().decode()
    t.start()
    t.join(timeout=30)
    assert seen["rc"] < 0 and "bad shape" in seen["own"]
    assert lib.oslo_hip_last_error().decode() == before
