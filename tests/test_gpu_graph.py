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


def test_dropout_from_the_generator_refuses_capture_with_a_message(device):
    from oslo_amd.torch.nn.modules import functional as F_

    x = randn((8, 64), BF16, 1).to(device)
    b = torch.zeros(64, dtype=BF16, device=device)
    F_.fused_bias_dropout_add(x, b, None, 0.5, True)  # eager: fine
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="cannot be captured"):
        with torch.cuda.graph(graph):
            F_.fused_bias_dropout_add(x, b, None, 0.5, True)
    # p = 0 captures (nothing is drawn)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = F_.fused_bias_dropout_add(x, b, None, 0.0, True)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, x)
