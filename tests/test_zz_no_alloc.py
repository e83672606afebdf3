"""oslo_ln_bwd_static, the entry point that allocates nothing: its fp32 partial
rows live in a device array that is part of the library.  Called through the
C ABI and compared with oslo_ln_bwd (caller-owned workspace) on the same
inputs: dx, dgamma and dbeta must be bit-identical (same kernels, same order
of additions), on two calls in a row, the second one on a smaller problem so
that stale partial rows of the first would show.  oslo_ln_bwd itself is
checked against the float64 oracle in test_gpu_norm.py; the first case here
repeats that check for the new entry point.

This file sorts last on purpose: a failure here must not hide other tests."""
import pytest
import torch

from helpers import check, f64, randn
from oracle import closed_form as cf
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16
CODE = {F32: 0, F16: 1, BF16: 2}


def _p(t):
    return None if t is None else t.data_ptr()


def _run_pair(lib, dev, n1, n2, tin, tout, seed, affine=True):
    """Returns ((dx, dgamma, dbeta) of oslo_ln_bwd, the same of oslo_ln_bwd_static, inputs)."""
    x = randn((n1, n2), tin, seed, std=1.3, mean=0.2).to(dev)
    dy = randn((n1, n2), tout, seed + 1).to(dev)
    gamma = randn((n2,), tout, seed + 2, std=0.02, mean=1.0).to(dev) if affine else None
    beta = randn((n2,), tout, seed + 3, std=0.02).to(dev) if affine else None
    y = torch.empty(n1, n2, dtype=tout, device=dev)
    mean = torch.empty(n1, dtype=F32, device=dev)
    invvar = torch.empty(n1, dtype=F32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.oslo_ln_fwd(_p(x), _p(gamma), _p(beta), _p(y), _p(mean), _p(invvar), n1, n2, 1e-5,
                         CODE[tin], CODE[tout], st)
    assert rc == 0, lib.oslo_hip_last_error()

    nbytes = int(lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, n1, n2))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    outs = []
    for static in (False, True):
        dx = torch.full((n1, n2), float("nan"), dtype=tin, device=dev)
        dg = torch.full((n2,), float("nan"), dtype=tout, device=dev) if affine else None
        db = torch.full((n2,), float("nan"), dtype=tout, device=dev) if affine else None
        if static:
            rc = lib.oslo_ln_bwd_static(_p(dy), _p(x), _p(mean), _p(invvar), _p(gamma), _p(dx), _p(dg), _p(db),
                                        n1, n2, CODE[tin], CODE[tout], st)
        else:
            rc = lib.oslo_ln_bwd(_p(dy), _p(x), _p(mean), _p(invvar), _p(gamma), _p(dx), _p(dg), _p(db),
                                 _p(ws), nbytes, n1, n2, CODE[tin], CODE[tout], st)
        assert rc == 0, lib.oslo_hip_last_error()
        outs.append((dx, dg, db))
    torch.cuda.synchronize()
    return outs[0], outs[1], (x, dy, gamma, mean, invvar)


def _same_bits(a, b, what):
    if a is None:
        assert b is None
        return
    assert not torch.isnan(b.float()).any(), what + ": output not written"
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), what + " differs from oslo_ln_bwd"


def test_static_scratch_two_calls_in_a_row(device):
    lib = _C.load_library()
    # first call: many rows (256 partial rows per array), then a smaller
    # problem (fewer rows, shorter rows) that reuses the same scratch array
    for n1, n2, tin, tout in ((2048, 4096, BF16, BF16), (96, 1024, BF16, BF16)):
        ref, got, (x, dy, gamma, mean, invvar) = _run_pair(lib, device, n1, n2, tin, tout, seed=11)
        for a, b, name in zip(ref, got, ("dx", "dgamma", "dbeta")):
            _same_bits(a, b, "[%d,%d] %s" % (n1, n2, name))
        # and against the float64 oracle, to the bar of the other norm tests
        odx, odg, odb = cf.layer_norm_bwd(f64(dy), f64(x), f64(mean), f64(invvar), f64(gamma))
        patol = 1e-5 * (n1 ** 0.5) + 1e-6
        check(got[0], odx, "static dx [%d,%d]" % (n1, n2), atol=4e-6)
        check(got[1], odg, "static dgamma [%d,%d]" % (n1, n2), atol=patol, min_exact=0.97)
        check(got[2], odb, "static dbeta [%d,%d]" % (n1, n2), atol=patol, min_exact=0.97)


@pytest.mark.parametrize("n1,n2,tin,tout,affine", [
    (300, 2048, F32, F32, True),
    (100, 1024, F32, BF16, True),   # mixed dtypes
    (7, 513, BF16, BF16, True),     # scalar path: two-step column sums through the scratch
    (3001, 100, F16, F16, True),
    (64, 768, BF16, BF16, False),   # no parameters: the scratch is not touched
    (1, 8, F32, F32, True),
])
def test_static_scratch_matches_workspace_entry_point(device, n1, n2, tin, tout, affine):
    lib = _C.load_library()
    ref, got, _ = _run_pair(lib, device, n1, n2, tin, tout, seed=5, affine=affine)
    for a, b, name in zip(ref, got, ("dx", "dgamma", "dbeta")):
        _same_bits(a, b, name)


def test_static_scratch_refuses_problems_beyond_its_size(device):
    lib = _C.load_library()
    n1, n2 = 4096, 16384
    need = int(lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, n1, n2))
    assert need > _C.OSLO_LN_BWD_STATIC_SCRATCH_BYTES
    # rejected before anything is launched: the pointers are never touched
    dummy = torch.empty(16, dtype=torch.uint8, device=device)
    p = dummy.data_ptr()
    rc = lib.oslo_ln_bwd_static(p, p, p, p, p, p, p, p, n1, n2, CODE[BF16], CODE[BF16],
                                torch.cuda.current_stream().cuda_stream)
    assert rc == -3
    assert b"static scratch" in lib.oslo_hip_last_error()
    # an empty batch needs no scratch and still defines zero parameter gradients
    dg = torch.full((64,), 1.0, dtype=BF16, device=device)
    db = torch.full((64,), 1.0, dtype=BF16, device=device)
    rc = lib.oslo_ln_bwd_static(None, None, None, None, p, None, dg.data_ptr(), db.data_ptr(), 0, 64,
                                CODE[BF16], CODE[BF16], torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    assert float(dg.float().abs().max()) == 0.0 and float(db.float().abs().max()) == 0.0


def test_static_scratch_allocates_nothing_and_can_be_captured(device):
    """The property the entry point exists for: it can run where device memory
    cannot be allocated.  Under stream capture an allocation by the library
    would fail the capture; here the call is captured (the empty-batch form,
    which clears the parameter gradients with a kernel, included), the graph is
    replayed with new inputs against oslo_ln_bwd, and the device's free memory
    is the same before and after the eager calls."""
    lib = _C.load_library()
    n1, n2 = 512, 1024
    x = randn((n1, n2), BF16, 1, std=1.3, mean=0.2).to(device)
    dy = randn((n1, n2), BF16, 2).to(device)
    gamma = randn((n2,), BF16, 3, std=0.02, mean=1.0).to(device)
    beta = randn((n2,), BF16, 4, std=0.02).to(device)
    y = torch.empty_like(x)
    mean = torch.empty(n1, dtype=F32, device=device)
    invvar = torch.empty(n1, dtype=F32, device=device)
    dx, dg, db = torch.empty_like(x), torch.empty_like(gamma), torch.empty_like(gamma)
    eg, eb = torch.ones(64, dtype=BF16, device=device), torch.ones(64, dtype=BF16, device=device)
    nbytes = int(lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, n1, n2))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device)
    rdx, rdg, rdb = torch.empty_like(x), torch.empty_like(gamma), torch.empty_like(gamma)

    def fwd(st):
        assert lib.oslo_ln_fwd(_p(x), _p(gamma), _p(beta), _p(y), _p(mean), _p(invvar), n1, n2, 1e-5,
                               CODE[BF16], CODE[BF16], st) == 0

    def static(st):
        rc = lib.oslo_ln_bwd_static(_p(dy), _p(x), _p(mean), _p(invvar), _p(gamma), _p(dx), _p(dg), _p(db),
                                    n1, n2, CODE[BF16], CODE[BF16], st)
        assert rc == 0, lib.oslo_hip_last_error()
        rc = lib.oslo_ln_bwd_static(None, None, None, None, _p(gamma), None, _p(eg), _p(eb), 0, 64,
                                    CODE[BF16], CODE[BF16], st)
        assert rc == 0, lib.oslo_hip_last_error()

    # eager: free device memory does not move (the first call has already fetched
    # the array's address; the array itself is part of the loaded code object)
    st = torch.cuda.current_stream().cuda_stream
    fwd(st)
    static(st)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(device)
    for _ in range(5):
        static(st)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(device)
    assert free1 == free0

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        x.copy_(randn((n1, n2), BF16, 30 + rep, std=1.3).to(device))
        dy.copy_(randn((n1, n2), BF16, 40 + rep).to(device))
        eg.fill_(1.0)
        st = torch.cuda.current_stream().cuda_stream
        fwd(st)
        rc = lib.oslo_ln_bwd(_p(dy), _p(x), _p(mean), _p(invvar), _p(gamma), _p(rdx), _p(rdg), _p(rdb),
                             _p(ws), nbytes, n1, n2, CODE[BF16], CODE[BF16], st)
        assert rc == 0, lib.oslo_hip_last_error()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b, name in ((rdx, dx, "dx"), (rdg, dg, "dgamma"), (rdb, db, "dbeta")):
            _same_bits(a, b, "replay %d %s" % (rep, name))
        assert float(eg.float().abs().max()) == 0.0 and float(eb.float().abs().max()) == 0.0
