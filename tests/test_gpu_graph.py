"""The entry points only launch kernels on the stream they are given (no
allocation, no memset node, no synchronisation), so a caller may capture them
in a HIP graph.  The graph is replayed several times, with new inputs and eager
work between the replays, and every replay is compared with the eager result."""
import pytest
import torch

from helpers import randn
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def test_captured_layer_chain_replays(device):
    n1, n2, ab, s = 256, 1024, 6, 256
    ln = _C.get_layernorm_kernel()
    sm = _C.get_softmax_kernel()
    ek = _C.get_fused_elementwise_kernel()
    ad = _C.get_adam_kernel()
    x = randn((n1, n2), BF16, 1).to(device)
    dy = randn((n1, n2), BF16, 2).to(device)
    gamma = randn((n2,), BF16, 3, std=0.1, mean=1.0).to(device)
    beta = randn((n2,), BF16, 4, std=0.1).to(device)
    bias = randn((n2,), BF16, 5, std=0.1).to(device)
    sc = randn((ab, s, s), BF16, 6).to(device)
    dsc = randn((ab, s, s), BF16, 7).to(device)
    params = [randn((n,), torch.float32, 8 + i).to(device) for i, n in enumerate((1000, 4096, 33))]

    def chain(p_list, m_list, v_list):
        y, mean, invvar = ln.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
        dx, dg, db = ln.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, 1e-5)
        act = ek.bias_gelu_forward(y, bias)
        dact, dbias = ek.bias_gelu_backward(dx, y, bias)
        fy, h, fmean, finv = ln.bias_dropout_add_norm_forward(
            False, act, bias, x, (n2,), gamma, beta, 1e-5, 0.1, 99, 8)
        fres, fin, fdg, fdb, fdbias = ln.bias_dropout_add_norm_backward(
            False, dact, dy, h, fmean, finv, (n2,), gamma, 0.1, 99, 8)
        probs, stats = sm.softmax_dropout_forward(sc, None, 0.125, 0.1, 7, 4)
        dsx = sm.softmax_dropout_backward(dsc, sc, stats, None, 0.125, 0.1, 7, 4)
        grads = [t * 0.5 for t in p_list]
        ad.multi_tensor_adam(0, None, [grads, p_list, m_list, v_list], 1e-2, 0.9, 0.999, 1e-8, 3, 1, 1, 0.01)
        return [y, dx, dg, db, act, dact, dbias, fy, fres, fin, fdg, fdb, fdbias, probs, dsx]

    def fresh_state():
        return ([t.clone() for t in params], [torch.zeros_like(t) for t in params],
                [torch.ones_like(t) for t in params])

    # warm up on a side stream, then capture
    gp, gm, gv = fresh_state()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain(*fresh_state())
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = chain(gp, gm, gv)
    for rep in range(3):
        # new inputs in the captured buffers, and eager work between the replays
        x.copy_(randn((n1, n2), BF16, 100 + rep).to(device))
        sc.copy_(randn((ab, s, s), BF16, 200 + rep).to(device))
        state = fresh_state()
        for dst, src in zip(gp + gm + gv, state[0] + state[1] + state[2]):
            dst.copy_(src)
        ep, em, ev = fresh_state()
        want = chain(ep, em, ev)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(outs, want)):
            assert torch.equal(a, b), "output %d differs on replay %d" % (i, rep)
        for a, b in zip(gp + gm + gv, ep + em + ev):
            assert torch.equal(a, b), "optimizer state differs on replay %d" % rep


def test_captured_dropout_draws_a_new_mask_on_every_replay(device):
    """Through the Python layer: during capture the kernels read (seed, offset)
    from device memory, a captured add advances the offset, and backward takes
    the forward's pair; every replay must equal the integer Philox oracle for
    the pair that the state held when the replay started."""
    import numpy as np

    from oracle import philox
    from oslo_amd.torch.nn.modules import functional as F_

    n1, n2, p = 64, 256, 0.25
    x = randn((n1, n2), BF16, 1).to(device)
    b = torch.zeros(n2, dtype=BF16, device=device)
    dy = torch.ones(n1, n2, dtype=BF16, device=device)
    sc = randn((2, 64, 64), BF16, 2).to(device)

    # before any eager call on the device there is no state to read
    F_._graph_rng.clear()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="eager step first"):
        with torch.cuda.graph(graph):
            F_.fused_bias_dropout_add(x, b, None, p, True)

    torch.manual_seed(1234)
    F_.fused_bias_dropout_add(x, b, None, p, True)  # eager: creates the state
    index = device.index if device.index is not None else torch.cuda.current_device()
    state = F_._graph_rng[index][1]

    xg = x.clone().requires_grad_()
    scg = sc.clone().requires_grad_()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up of the autograd machinery
        F_.fused_bias_dropout_add(xg, b, None, p, True).backward(dy)
    torch.cuda.current_stream().wait_stream(side)
    xg.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = F_.fused_bias_dropout_add(xg, b, None, p, True)
        gx, = torch.autograd.grad(out, xg, dy)
        probs = F_.scaled_upper_triang_masked_softmax_dropout(scg, 0.5, p, True)
        gs, = torch.autograd.grad(probs, scg, torch.ones_like(probs))
    masks = []
    for rep in range(3):
        seed, offset = (int(v) for v in state.cpu())
        graph.replay()
        torch.cuda.synchronize()
        keep = philox.keep_mask(n1 * n2, p, seed % 2 ** 64, offset % 2 ** 64).reshape(n1, n2).astype(bool)
        got = (out != 0).cpu().numpy() | (x == 0).cpu().numpy()
        assert np.array_equal(got, keep | (x == 0).cpu().numpy()), "forward mask differs from the oracle"
        # backward used the forward's pair: dx = keep / (1 - p)
        assert np.array_equal((gx != 0).cpu().numpy(), keep)
        # the softmax call was captured second: its pair is 4 further
        keep2 = philox.keep_mask(sc.numel(), p, seed % 2 ** 64, (offset + 4) % 2 ** 64).reshape(sc.shape).astype(bool)
        visible = np.tril(np.ones((64, 64), dtype=bool))[None]
        assert np.array_equal((probs != 0).cpu().numpy(), keep2 & visible)
        assert torch.isfinite(gs).all()
        masks.append(keep)
        assert int(state.cpu()[1]) == offset + 8, "two captured calls advance the offset by 8"
    assert not np.array_equal(masks[0], masks[1]) and not np.array_equal(masks[1], masks[2])
    # the fusion into the norm reads the same state (prologue and epilogue)
    w = torch.ones(n2, dtype=BF16, device=device)
    res = torch.zeros(n1, n2, dtype=BF16, device=device)
    xg2 = x.clone().requires_grad_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y, h = F_.fused_bias_dropout_add_layer_norm(xg2, b, res, w, b, (n2,), 1e-5, p, True,
                                                    return_sum=True)
        gx2, = torch.autograd.grad(y, xg2, dy)
    for rep in range(2):
        seed, offset = (int(v) for v in state.cpu())
        graph.replay()
        torch.cuda.synchronize()
        keep = philox.keep_mask(n1 * n2, p, seed % 2 ** 64, offset % 2 ** 64).reshape(n1, n2).astype(bool)
        assert np.array_equal((h != 0).cpu().numpy() | (x == 0).cpu().numpy(),
                              keep | (x == 0).cpu().numpy())
        assert ((gx2 == 0).cpu().numpy() | keep).all(), "dropped elements get no gradient"
    # p = 0 captures without touching the state
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        same = F_.fused_bias_dropout_add(x, b, None, 0.0, True)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(same, x)


def test_reseeding_keeps_the_state_tensor_that_captured_graphs_hold(device):
    """torch.manual_seed followed by an eager dropout call re-seeds the dropout
    state of the device.  A captured graph holds the address of that state, so
    the new seed must land in the same memory: a replay afterwards draws the
    mask of the new (seed, offset) pair, and the tensor is the one the graph
    was captured with."""
    import numpy as np

    from oracle import philox
    from oslo_amd.torch.nn.modules import functional as F_

    n1, n2, p = 64, 512, 0.25
    x = torch.ones(n1, n2, dtype=BF16, device=device)
    b = torch.zeros(n2, dtype=BF16, device=device)
    torch.manual_seed(11)
    F_.fused_bias_dropout_add(x, b, None, p, True)  # eager: creates (or re-seeds) the state
    index = device.index if device.index is not None else torch.cuda.current_device()
    state = F_._graph_rng[index][1]
    ptr = state.data_ptr()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = F_.fused_bias_dropout_add(x, b, None, p, True)
    graph.replay()
    torch.cuda.synchronize()
    torch.manual_seed(2024)
    F_.fused_bias_dropout_add(x, b, None, p, True)  # eager call after the seed change
    junk = [torch.full((2,), -1, dtype=torch.int64, device=device) for _ in range(64)]  # reuses freed blocks
    assert F_._graph_rng[index][1] is state and state.data_ptr() == ptr
    seed, offset = (int(v) for v in state.cpu())
    assert seed == 2024
    graph.replay()
    torch.cuda.synchronize()
    keep = philox.keep_mask(n1 * n2, p, seed % 2 ** 64, offset % 2 ** 64).reshape(n1, n2).astype(bool)
    assert np.array_equal((out != 0).cpu().numpy(), keep), "replay after re-seeding: mask differs from the oracle"
    assert int(state.cpu()[1]) == offset + 4
    assert all(int(j.cpu()[0]) == -1 for j in junk), "a replay wrote outside the state tensor"


def test_captured_mixed_precision_lamb_step_counts_and_replays(device):
    """FusedMixedPrecisionLamb keeps its step count, learning rate and loss scale
    on the device, so a captured step is a whole optimizer step: every replay
    advances the count and gives what the eager optimizer gives."""
    from oslo_amd.torch.optim import FusedMixedPrecisionLamb

    shapes = [(64, 48), (48,), (1000,)]

    def make():
        ps = [torch.nn.Parameter(randn(s, torch.float32, 20 + i).to(device)) for i, s in enumerate(shapes)]
        for p in ps:
            p.grad = torch.zeros_like(p)
        return ps, FusedMixedPrecisionLamb(ps, lr=0.01, weight_decay=0.01, max_grad_norm=1.0)

    grads = [[randn(s, torch.float32, 40 + 10 * k + i).to(device) for i, s in enumerate(shapes)] for k in range(4)]

    def load(ps, k):
        # the step leaves its update direction in the gradients: refill them every time
        for p, g in zip(ps, grads[k]):
            p.grad.copy_(g)

    eager_ps, eager = make()
    graph_ps, captured = make()
    # first step eagerly on both (it creates the moments), on a side stream as capture wants
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        load(eager_ps, 0)
        eager.step()
        load(graph_ps, 0)
        captured.step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    load(graph_ps, 1)
    with torch.cuda.graph(graph):
        captured.step()
    # (capture does not execute: the step count has not moved yet)
    assert captured.param_groups[0]["step"].item() == 1
    for k in (1, 2, 3):
        load(eager_ps, k)
        eager.step()
        load(graph_ps, k)
        graph.replay()
        scratch = torch.randn(1 << 16, device=device).sum()  # eager work between the replays
        torch.cuda.synchronize()
        assert scratch.isfinite()
        assert captured.param_groups[0]["step"].item() == k + 1 == eager.param_groups[0]["step"].item()
        for a, b in zip(eager_ps, graph_ps):
            assert torch.equal(a, b), "replay %d" % k


def test_two_graphs_do_not_share_a_backward_workspace(device, monkeypatch):
    """A backward entry point writes partial rows to a workspace and reads them
    in a second launch.  A captured call must own its workspace: two graphs
    that capture the same op at the same shape get different ones, deleting the
    first graph leaves the second intact, and the two replayed at the same time
    on two streams give the serial results bit for bit."""
    n1, n2 = 2048, 1024
    ln = _C.get_layernorm_kernel()
    gamma = randn((n2,), BF16, 3, std=0.1, mean=1.0).to(device)
    beta = randn((n2,), BF16, 4, std=0.1).to(device)
    xs = [randn((n1, n2), BF16, 10 + i).to(device) for i in range(2)]
    dys = [randn((n1, n2), BF16, 20 + i).to(device) for i in range(2)]
    stats = [ln.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)[1:] for x in xs]

    seen = []
    real = _C._allocate_workspace

    def allocate(nbytes, index):
        t = real(nbytes, index)
        seen.append((t.data_ptr(), torch.cuda.is_current_stream_capturing()))
        return t

    monkeypatch.setattr(_C._ws_cache, "allocate", allocate)

    def bwd(i):
        mean, invvar = stats[i]
        return ln.layer_norm_backward_affine(dys[i], mean, invvar, xs[i], (n2,), gamma, beta, 1e-5)

    want = [[t.clone() for t in bwd(i)] for i in range(2)]   # eager (warms the cache up, too)
    torch.cuda.synchronize()
    graphs, outs = [], []
    for i in range(2):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            outs.append(bwd(i))
        graphs.append(g)
    captured = [ptr for ptr, capturing in seen if capturing]
    assert len(captured) == 2 and captured[0] != captured[1]
    eager_ptrs = {ptr for ptr, capturing in seen if not capturing}
    assert not eager_ptrs & set(captured)       # nor the cached one
    # both at once on two streams, three times, with eager calls of the same op in between
    streams = [torch.cuda.Stream(device=device) for _ in range(2)]
    for rep in range(3):
        for o in outs:
            for t in o:
                t.zero_()
        torch.cuda.synchronize()
        for g, s in zip(graphs, streams):
            with torch.cuda.stream(s):
                g.replay()
        eager = bwd(rep % 2)                    # shares the device, not the workspace
        torch.cuda.synchronize()
        for i in range(2):
            for k, (a, b) in enumerate(zip(outs[i], want[i])):
                assert torch.equal(a, b), "graph %d, output %d, replay %d" % (i, k, rep)
        for a, b in zip(eager, want[rep % 2]):
            assert torch.equal(a, b)
    # the second graph does not depend on the first one's memory
    keep = [t.clone() for t in want[1]]
    del graphs[0], outs[0]
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    filler = [torch.full((n1, n2), 7.0, dtype=BF16, device=device) for _ in range(8)]  # reuses freed blocks
    graphs[0].replay()
    torch.cuda.synchronize()
    for a, b in zip(outs[0], keep):
        assert torch.equal(a, b)
    del filler
