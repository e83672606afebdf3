"""The C ABI refuses what it cannot run, for callers that do not come through
the Python bindings (which make the same checks before they call): a negative
return code, a message from oslo_hip_last_error(), and nothing launched.  The
role of TORCH_CHECK / AT_ASSERTM in the reference's shims
(oslo/torch/_C/csrc/FusedLayerNormBinder.cpp:8-14, 38-93;
FusedScaleMaskSoftmaxBinder.cpp:41-45, 83-86).  Every case changes one argument
of a call that is accepted as it stands."""
import pytest
import torch

from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

BF16, F64 = 2, 3   # dtype codes of include/oslo_hip.h


class Harness:
    def __init__(self, device):
        self.lib = _C.load_library()
        self.st = torch.cuda.current_stream().cuda_stream
        z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt, device=device)
        self.t = z(8, 64)          # activations [8, 64] (also [2, 2, 2, 64] and [4, 2, 64])
        self.u = z(8, 64)
        self.w = z(8, 64)
        self.v = z(8, 64)
        self.vec = z(64)
        self.vec2 = z(64)
        self.vec3 = z(64)
        self.stat = z(8, dt=torch.float32)
        self.stat2 = z(8, dt=torch.float32)
        self.stats = z(8, 2, dt=torch.float32)
        self.mask = z(2, 64, dt=torch.uint8)
        self.ws = z(1 << 20, dt=torch.uint8)

    def refused(self, name, good, changes):
        fn = getattr(self.lib, name)
        assert fn(*good) == 0, "%s: the unchanged call: %s" % (name, self.lib.oslo_hip_last_error())
        for index, value, text in changes:
            args = list(good)
            args[index] = value
            rc = fn(*args)
            msg = self.lib.oslo_hip_last_error()
            msg = msg.decode() if isinstance(msg, bytes) else msg
            assert rc < 0 and text in msg, (name, index, value, rc, msg)
        torch.cuda.synchronize()


def test_norm_entry_points(device):
    h = Harness(device)
    p = lambda t: t.data_ptr()
    x, y, g, b, mean, inv = p(h.t), p(h.u), p(h.vec), p(h.vec2), p(h.stat), p(h.stat2)
    h.refused("oslo_ln_fwd", [x, g, b, y, mean, inv, 8, 64, 1e-5, BF16, BF16, h.st], [
        (6, -1, "bad shape"), (7, 0, "bad shape"), (7, 1 << 32, "too large"), (0, None, "null tensor pointer"),
        (4, None, "null mean pointer"), (2, None, "both be given"), (9, 7, "unknown dtype"),
        (10, 0, "requires the same output type"), (9, F64, "go together")])
    h.refused("oslo_rms_fwd", [x, g, y, inv, 8, 64, 1e-5, BF16, BF16, h.st], [
        (4, -1, "bad shape"), (3, None, "null tensor pointer"), (7, 9, "unknown dtype")])
    ws, nws = p(h.ws), h.ws.numel()
    h.refused("oslo_ln_bwd", [x, x, mean, inv, g, y, g, b, ws, nws, 8, 64, BF16, BF16, h.st], [
        (10, -1, "bad shape"), (11, 1 << 32, "too large"), (0, None, "null tensor pointer"),
        (2, None, "null mean pointer"), (7, None, "both be given"), (9, 16, "workspace of"),
        (8, None, "workspace of")])
    h.refused("oslo_ln_bwd", [x, x, mean, inv, None, y, None, None, None, 0, 8, 64, BF16, BF16, h.st], [
        (6, g, "dgamma requested without gamma")])
    h.refused("oslo_rms_bwd", [x, x, inv, g, y, g, ws, nws, 8, 64, BF16, BF16, h.st], [
        (8, -1, "bad shape"), (4, None, "null tensor pointer"), (7, 16, "workspace of")])
    h.refused("oslo_ln_bwd_static", [x, x, mean, inv, g, y, g, b, 8, 64, BF16, BF16, h.st], [
        (9, 0, "bad shape")])


def test_fused_norm_entry_points(device):
    h = Harness(device)
    p = lambda t: t.data_ptr()
    x, y, hh, g, b, mean, inv = p(h.t), p(h.u), p(h.w), p(h.vec), p(h.vec2), p(h.stat), p(h.stat2)
    h.refused("oslo_bias_dropout_add_norm_fwd",
              [x, b, x, g, b, hh, y, mean, inv, 8, 64, 1e-5, 0.1, 1, 0, 0, BF16, h.st], [
                  (10, 0, "bad shape"), (12, 1.5, "outside [0, 1]"), (6, None, "null tensor pointer"),
                  (7, None, "null mean pointer"), (4, None, "both be given"), (16, 9, "dtype")])
    ws, nws = p(h.ws), h.ws.numel()
    good = [x, x, hh, mean, inv, g, y, p(h.v), g, b, p(h.vec3), ws, nws, 8, 64, 0.1, 1, 0, 0, BF16, h.st]
    h.refused("oslo_bias_dropout_add_norm_bwd", good, [
        (13, -1, "bad shape"), (15, -0.5, "outside [0, 1]"), (9, None, "both be given"),
        (7, None, "needs its own tensor"), (0, None, "null tensor pointer"), (3, None, "null mean pointer"),
        (12, 16, "workspace of")])
    good[5], good[8], good[9] = None, None, None
    h.refused("oslo_bias_dropout_add_norm_bwd", good, [(8, g, "dgamma requested without gamma")])


def test_softmax_entry_points(device):
    h = Harness(device)
    p = lambda t: t.data_ptr()
    x, y, dx, m, st = p(h.t), p(h.u), p(h.w), p(h.mask), p(h.stats)
    h.refused("oslo_softmax_causal_fwd", [x, y, 4, 2, 64, 1.0, BF16, h.st], [
        (2, -1, "bad shape"), (4, 0, "bad shape"), (6, 5, "unknown dtype"), (0, None, "null tensor pointer")])
    h.refused("oslo_softmax_causal_bwd", [x, y, dx, 4, 2, 64, 1.0, BF16, h.st], [
        (3, -1, "bad shape"), (2, None, "null tensor pointer")])
    h.refused("oslo_softmax_masked_fwd", [x, m, y, 2, 2, 2, 64, 2, 1, 1.0, BF16, h.st], [
        (3, -1, "bad shape"), (4, -1, "bad batch/head count"), (7, 3, "does not broadcast"),
        (8, 5, "does not broadcast"), (1, None, "null tensor pointer"),
        (10, 4, "unknown dtype")])
    h.refused("oslo_softmax_masked_bwd", [x, y, m, dx, 2, 2, 2, 64, 2, 1, 1.0, BF16, h.st], [
        (8, 3, "does not broadcast"), (3, None, "null tensor pointer")])
    h.refused("oslo_softmax_causal_masked_fwd", [x, m, y, 2, 2, 2, 64, 2, 1, 1.0, BF16, h.st], [
        (7, 3, "does not broadcast"), (2, None, "null tensor pointer")])
    h.refused("oslo_softmax_causal_dropout_fwd", [x, y, st, 4, 2, 64, 1.0, 0.1, 1, 0, BF16, h.st], [
        (7, 1.5, "outside [0, 1]"), (2, None, "null pointer"), (5, -1, "bad shape")])
    h.refused("oslo_softmax_causal_dropout_bwd", [x, x, st, dx, 4, 2, 64, 1.0, 0.1, 1, 0, BF16, h.st], [
        (8, -0.1, "outside [0, 1]"), (3, None, "null pointer")])
    h.refused("oslo_softmax_masked_dropout_fwd", [x, m, y, st, 2, 2, 2, 64, 2, 1, 1.0, 0.1, 1, 0, BF16, h.st], [
        (11, 2.0, "outside [0, 1]"), (1, None, "null pointer"), (8, 3, "does not broadcast")])
    h.refused("oslo_softmax_masked_dropout_bwd", [x, x, m, st, dx, 2, 2, 2, 64, 2, 1, 1.0, 0.1, 1, 0, BF16, h.st], [
        (3, None, "null pointer"), (9, 3, "does not broadcast")])
    # additive term [2, 1, 1, 64]: strides (64, 0, 0), the logits' dtype
    term = h.vec.new_zeros(2, 64)
    bias = p(term)
    h.refused("oslo_softmax_bias_fwd", [x, bias, y, 2, 2, 2, 64, 64, 0, 0, BF16, 0, 1.0, BF16, h.st], [
        (1, None, "null additive term"), (0, None, "null tensor pointer"), (11, 8, "unknown flag bits"),
        (10, 1, "logits' dtype or float32"), (7, -64, "negative stride"), (3, -1, "bad shape"),
        (4, -1, "bad batch/head count"), (13, 6, "unknown dtype")])
    h.refused("oslo_softmax_bias_bwd", [x, y, bias, dx, 2, 2, 2, 64, 64, 0, 0, BF16, 0, 1.0, BF16, h.st], [
        (3, None, "null tensor pointer"), (12, 4, "unknown flag bits")])
    h.refused("oslo_softmax_bias_dropout_fwd",
              [x, bias, y, st, 2, 2, 2, 64, 64, 0, 0, BF16, 0, 1.0, 0.1, 1, 0, BF16, h.st], [
                  (1, None, "null additive term"), (3, None, "null pointer"), (14, 1.5, "outside [0, 1]")])
    h.refused("oslo_softmax_bias_dropout_bwd",
              [x, x, bias, st, dx, 2, 2, 2, 64, 64, 0, 0, BF16, 0, 1.0, 0.1, 1, 0, BF16, h.st], [
                  (2, None, "null additive term"), (4, None, "null pointer"), (15, 1.5, "outside [0, 1]")])


def test_elementwise_entry_points(device):
    h = Harness(device)
    p = lambda t: t.data_ptr()
    x, y, dx, b = p(h.t), p(h.u), p(h.w), p(h.vec)
    ws, nws = p(h.ws), h.ws.numel()
    h.refused("oslo_bias_gelu_fwd", [x, b, y, 8, 64, BF16, h.st], [
        (3, -1, "bad shape"), (4, 0, "bad shape"), (5, 11, "unknown dtype"), (2, None, "null tensor pointer")])
    h.refused("oslo_bias_gelu_bwd", [x, x, b, dx, b, ws, nws, 8, 64, BF16, h.st], [
        (3, None, "null tensor pointer"), (6, 16, "workspace of"), (5, None, "workspace of"), (7, -2, "bad shape")])
    h.refused("oslo_bias_dropout_add_fwd", [x, b, x, y, None, 8, 64, 0.1, 1, 0, BF16, h.st], [
        (7, 1.5, "not in [0, 1]"), (3, None, "null tensor pointer"), (6, -1, "bad shape")])
    h.refused("oslo_bias_dropout_add_bwd", [x, dx, b, ws, nws, 8, 64, 0.1, 1, 0, BF16, h.st], [
        (7, -1.0, "not in [0, 1]"), (0, None, "null gradient pointer"), (4, 16, "workspace of"),
        (10, 8, "unknown dtype")])
    h.refused("oslo_bias_dropout_add_bwd", [x, dx, None, None, 0, 8, 64, 0.1, 1, 0, BF16, h.st], [
        (1, None, "nothing to compute")])
    h.refused("oslo_philox_mask", [p(h.mask), 128, 0.1, 1, 0, h.st], [
        (1, -1, "bad arguments"), (2, 1.5, "bad arguments"), (0, None, "null output")])
    h.refused("oslo_copy_probe", [x, y, 512, h.st], [(2, 8, "multiple of 16"), (0, x + 2, "multiple of 16")])


def test_workspace_sizes_and_overrides(device):
    lib = _C.load_library()
    msg = lambda: (lib.oslo_hip_last_error().decode() if isinstance(lib.oslo_hip_last_error(), bytes)
                   else lib.oslo_hip_last_error())
    assert lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, 8, 64) > 0
    assert lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, -1, 64) < 0 and "bad shape" in msg()
    assert lib.oslo_workspace_bytes(999, 8, 64) < 0 and "unknown op" in msg()
    assert lib.oslo_tune(None, 1) < 0 and "bad arguments" in msg()
    assert lib.oslo_tune(b"softmax_rows_per_wave", 3) < 0 and "no valid value" in msg()
    assert lib.oslo_tune(b"no_such_knob", 1) < 0 and "unknown key" in msg()


def test_adam_entry_point(device):
    import ctypes

    lib = _C.load_library()
    st = torch.cuda.current_stream().cuda_stream
    t = [torch.zeros(40, device=device) for _ in range(4)]
    table = lambda x: (ctypes.c_void_p * 1)(x.data_ptr())
    sizes = (ctypes.c_int64 * 1)(40)
    good = [table(t[0]), table(t[1]), table(t[2]), table(t[3]), sizes, 1, 1e-3, 0.9, 0.999, 1e-8, 1, 1, 1, 0.0, 0, st]
    assert lib.oslo_multi_tensor_adam(*good) == 0
    bad_sizes, null_table = (ctypes.c_int64 * 1)(-3), (ctypes.c_void_p * 1)(None)
    for index, value, text in [(5, -1, "negative tensor count"), (11, 2, "neither 0"), (14, 9, "unknown dtype"),
                               (0, None, "null table pointer"), (4, bad_sizes, "has size"),
                               (2, null_table, "null pointer")]:
        args = list(good)
        args[index] = value
        assert lib.oslo_multi_tensor_adam(*args) < 0
        m = lib.oslo_hip_last_error()
        assert text in (m.decode() if isinstance(m, bytes) else m), (index, m)
    torch.cuda.synchronize()
