"""Loader and thin bindings for ``liboslo_hip.so`` (the C ABI in ``include/oslo_hip.h``).

Mirrors the role of the reference's ``oslo/torch/_C/__init__.py``: lazily
obtained kernel objects (``get_layernorm_kernel()`` at ``_C/__init__.py:193-206``
there) whose methods have the signatures of the reference's pybind modules
(``FusedLayerNormBinder.cpp:404-424``, ``FusedScaleMaskSoftmaxBinder.cpp:111-127``).
Instead of JIT-compiling CUDA through ``torch.utils.cpp_extension`` the shared
library is built ahead of time by ``hipcc`` for gfx950 and bound with ctypes;
tensors cross the boundary as raw device pointers and every output and
workspace is allocated here, by torch's caching allocator.

A missing or unloadable library raises ``EnvironmentError`` (the reference's
exception type, ``_C/__init__.py:200-204``); there is no fallback for GPU
tensors.
"""
import ctypes
import os
import subprocess
import threading

import torch

_CSRC_DIR = os.path.normpath(
    os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", "csrc")
)
LIBRARY_PATH = os.path.join(_CSRC_DIR, "liboslo_hip.so")

OSLO_OP_LN_BWD = 1
OSLO_OP_RMS_BWD = 2
OSLO_OP_BIAS_GELU_BWD = 3
OSLO_OP_BIAS_DROPOUT_ADD_BWD = 4
OSLO_OP_BIAS_DROPOUT_ADD_NORM_BWD = 5

ABI_VERSION = 1

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
OSLO_DTYPE_F64 = 3  # LayerNorm / RMSNorm only
OSLO_LN_BWD_STATIC_SCRATCH_BYTES = 16 * 1024 * 1024

_lib = None
_lib_lock = threading.Lock()

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_int = ctypes.c_int
_f32 = ctypes.c_float
_f64 = ctypes.c_double

# name -> (restype, argtypes); one entry per declaration in include/oslo_hip.h and
# include/oslo_hip_testing.h
_SIGNATURES = {
    "oslo_hip_last_error": (ctypes.c_char_p, []),
    "oslo_hip_arch": (ctypes.c_char_p, []),
    "oslo_hip_abi_version": (_int, []),
    "oslo_workspace_bytes": (_i64, [_int, _i64, _i64]),
    "oslo_ln_fwd": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _f64, _int, _int, _p]),
    "oslo_ln_bwd": (
        _int,
        [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _p],
    ),
    "oslo_ln_bwd_static": (
        _int,
        [_p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _int, _int, _p],
    ),
    "oslo_rms_fwd": (_int, [_p, _p, _p, _p, _i64, _i64, _f64, _int, _int, _p]),
    "oslo_rms_bwd": (
        _int,
        [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _int, _p],
    ),
    "oslo_softmax_causal_fwd": (_int, [_p, _p, _i64, _i64, _i64, _f32, _int, _p]),
    "oslo_softmax_causal_bwd": (_int, [_p, _p, _p, _i64, _i64, _i64, _f32, _int, _p]),
    "oslo_softmax_masked_fwd": (
        _int,
        [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _int, _p],
    ),
    "oslo_softmax_masked_bwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _int, _p],
    ),
    "oslo_softmax_causal_masked_fwd": (
        _int,
        [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _int, _p],
    ),
    "oslo_softmax_causal_masked_bwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _int, _p],
    ),
    "oslo_softmax_causal_masked_dropout_fwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _u64, _u64,
         _int, _p],
    ),
    "oslo_softmax_causal_masked_dropout_bwd": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _u64,
         _u64, _int, _p],
    ),
    "oslo_softmax_batch_per_block": (_int, [_i64, _i64, _i64, _i64]),
    "oslo_softmax_causal_dropout_fwd": (
        _int,
        [_p, _p, _p, _i64, _i64, _i64, _f32, _f32, _u64, _u64, _int, _p],
    ),
    "oslo_softmax_causal_dropout_bwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _f32, _f32, _u64, _u64, _int, _p],
    ),
    "oslo_softmax_masked_dropout_fwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _u64, _u64,
         _int, _p],
    ),
    "oslo_softmax_masked_dropout_bwd": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _u64,
         _u64, _int, _p],
    ),
    "oslo_softmax_bias_fwd": (
        _int,
        [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _p],
    ),
    "oslo_softmax_bias_bwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _p],
    ),
    "oslo_softmax_bias_dropout_fwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _f32, _f32,
         _u64, _u64, _int, _p],
    ),
    "oslo_softmax_bias_dropout_bwd": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _f32, _f32,
         _u64, _u64, _int, _p],
    ),
    "oslo_bias_gelu_fwd": (_int, [_p, _p, _p, _i64, _i64, _int, _p]),
    "oslo_bias_gelu_bwd": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p]),
    "oslo_bias_dropout_add_fwd": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _i64, _f32, _u64, _u64, _int, _p],
    ),
    "oslo_bias_dropout_add_bwd": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _f32, _u64, _u64, _int, _p],
    ),
    "oslo_bias_dropout_add_norm_fwd": (
        _int,
        [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _f64, _f32, _u64, _u64, _int,
         _int, _p],
    ),
    "oslo_bias_dropout_add_norm_bwd": (
        _int,
        [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _f32, _u64,
         _u64, _int, _int, _p],
    ),
    "oslo_multi_tensor_adam": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _f32, _f32, _f32, _f32, _int, _int, _int, _f32, _int, _p],
    ),
    "oslo_multi_tensor_sgd": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _f32, _f32, _f32, _f32, _int, _int, _int, _f32, _int, _int,
         _int, _p, _p],
    ),
    "oslo_multi_tensor_adagrad": (_int, [_p, _p, _p, _p, _i64, _f32, _f32, _int, _f32, _int, _p]),
    "oslo_multi_tensor_novograd": (
        _int,
        [_p, _p, _p, _p, _i64, _p, _f32, _f32, _f32, _f32, _int, _int, _f32, _int, _int, _int, _p],
    ),
    "oslo_multi_tensor_lamb_stage1": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _f32, _f32, _f32, _int, _int, _f32, _int, _int, _p, _f32,
         _int, _p],
    ),
    "oslo_multi_tensor_lamb_stage2": (
        _int, [_p, _p, _p, _i64, _p, _p, _f32, _f32, _int, _int, _p],
    ),
    "oslo_multi_tensor_norm_partials": (_i64, [_p, _i64, _int]),
    "oslo_multi_tensor_norm": (
        _int, [_p, _p, _i64, _int, _p, _i64, _p, _p, _int, _int, _f32, _f32, _p, _int, _p],
    ),
    "oslo_multi_tensor_lamb_mp_stage1": (
        _int,
        [_p, _p, _p, _p, _p, _i64, _f32, _f32, _f32, _p, _int, _f32, _int, _int, _p, _p, _p, _p,
         _int, _int, _p],
    ),
    "oslo_multi_tensor_lamb_mp_stage2": (
        _int, [_p, _p, _p, _p, _i64, _p, _p, _p, _f32, _int, _p, _int, _int, _p],
    ),
    "oslo_rng_from_device": (_int, [_p]),
    "oslo_philox_mask": (_int, [_p, _i64, _f32, _u64, _u64, _p]),
    "oslo_philox_words": (_int, [_p, _i64, _i64, _u64, _u64, _p]),
    "oslo_copy_probe": (_int, [_p, _p, _i64, _p]),
    "oslo_colsum_finalize_probe": (_int, [_p, _i64, _i64, _p, _p, _p, _int, _p]),
    "oslo_wave_reduce_selftest": (_int, [_p, _p]),
    "oslo_tune": (_int, [ctypes.c_char_p, _int]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def build_library(force=False):
    """Compiles ``liboslo_hip.so`` in place with hipcc (``make`` in ``csrc``)."""
    cmd = ["make", "-C", _CSRC_DIR, "-j8"]
    if force:
        subprocess.run(["make", "-C", _CSRC_DIR, "clean"], check=True,
                       stdout=subprocess.DEVNULL)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise EnvironmentError(
            "Failed compiling the HIP kernels for gfx950 (%s):\n%s"
            % (" ".join(cmd), proc.stdout[-4000:])
        )
    return LIBRARY_PATH


def load_library():
    """Returns the ctypes handle, loading (and if absent, building) the library."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIBRARY_PATH):
            build_library()
        try:
            lib = ctypes.CDLL(LIBRARY_PATH)
            for name, (restype, argtypes) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            if lib.oslo_hip_abi_version() != ABI_VERSION:
                raise OSError(
                    "ABI version %d, expected %d"
                    % (lib.oslo_hip_abi_version(), ABI_VERSION)
                )
        except (OSError, AttributeError) as exc:
            raise EnvironmentError(
                "Failed loading the HIP kernels (%s): %s. Rebuild with "
                "`make -C %s`." % (LIBRARY_PATH, exc, _CSRC_DIR)
            ) from exc
        _lib = lib
    return _lib


def _check(rc, lib):
    if rc != 0:
        raise RuntimeError(lib.oslo_hip_last_error().decode("utf-8", "replace"))


def _ptr(t):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t):
    """Handle of torch's current stream on the tensor's device."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _SameDevice:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_SAME_DEVICE = _SameDevice()


def _device_of(t):
    """Context that makes the tensor's device current; nothing to do (and
    nothing allocated) when it already is."""
    if t.device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device_of(t)


def _dtype_code(t, what, allow_f64=False):
    if allow_f64 and t.dtype == torch.float64:
        return OSLO_DTYPE_F64
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise RuntimeError(
            "%s: dtype %s is not supported by the HIP kernels "
            "(float32, float16 and bfloat16 are%s)"
            % (what, t.dtype, "" if allow_f64 else "; float64 only by the norms")
        ) from None


def _stat_dtype(t):
    # FusedLayerNormBinder.cpp:146-152: the statistics are fp32 for 16-bit
    # inputs and have the input's type otherwise
    return torch.float64 if t.dtype == torch.float64 else torch.float32


def _check_input(t, name):
    # CHECK_INPUT of FusedLayerNormBinder.cpp:8-14
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


# Backward workspaces (fp32 partial rows of the parameter gradients).  A backward
# entry point enqueues two launches, the main kernel that writes the partial rows
# and the finalize kernel that reads them, so a workspace must not be handed to
# another call before both launches of this one are on the stream:
#   * eager calls share one workspace per (device, stream, op), grown on demand;
#     the slot's lock is held from the moment the workspace is picked until the C
#     call has returned.  Calls that share a stream are then ordered on it as
#     whole calls (two host threads on one stream cannot interleave their
#     launches); calls on different streams or devices never share a workspace;
#   * a call under stream capture neither reads nor writes the cache: it gets a
#     workspace of its own, which the graph's private pool then owns.  Two graphs
#     never share partial rows, deleting one graph cannot free memory another one
#     points at, and the cached tensors are never referenced by a graph, so
#     replacing one by a larger one is always safe.
class _WorkspaceSlot:
    __slots__ = ("lock", "tensor")

    def __init__(self):
        self.lock = threading.Lock()
        self.tensor = None


class _WorkspaceLease:
    """``with lease as ws:`` -> ``ws.tensor`` (None when the call needs no
    workspace) and ``ws.nbytes`` for the duration of one C call."""

    __slots__ = ("tensor", "nbytes", "_cache", "_key", "_slot")

    def __init__(self, cache=None, key=None, nbytes=0):
        self.tensor, self.nbytes = None, nbytes
        self._cache, self._key, self._slot = cache, key, None

    def __enter__(self):
        cache = self._cache
        if cache is None or self.nbytes <= 0:
            return self
        if cache.capturing():
            self.tensor = cache.allocate(self.nbytes, self._key[0])
            return self
        slot = cache.slots.get(self._key)
        if slot is None:
            slot = cache.slots.setdefault(self._key, _WorkspaceSlot())
        slot.lock.acquire()
        self._slot = slot
        try:
            ws = slot.tensor
            if ws is None or ws.numel() < self.nbytes:
                # (round up so that a sweep over growing shapes settles quickly)
                size = max(self.nbytes, 16)
                if size > (1 << 16):
                    size = (size + (1 << 20) - 1) & ~((1 << 20) - 1)
                ws = slot.tensor = cache.allocate(size, self._key[0])
            self.tensor = ws
        except BaseException:
            self._slot = None
            slot.lock.release()
            raise
        return self

    def __exit__(self, *exc):
        slot, self._slot = self._slot, None
        if slot is not None:
            slot.lock.release()
        return False


class _WorkspaceCache:
    def __init__(self, allocate, capturing):
        self.slots = {}
        self.allocate = allocate    # (nbytes, device index) -> uint8 tensor
        self.capturing = capturing  # () -> bool: the current stream is being captured

    def lease(self, index, stream, op, nbytes):
        return _WorkspaceLease(self, (index, stream, op), nbytes)


def _allocate_workspace(nbytes, index):
    return torch.empty(nbytes, dtype=torch.uint8, device=torch.device("cuda", index))


_ws_cache = _WorkspaceCache(_allocate_workspace, torch.cuda.is_current_stream_capturing)
_ws_bytes_cache = {}
_NO_WORKSPACE = _WorkspaceLease()


def _workspace(lib, op, n1, n2, device):
    """Lease of the workspace of backward op `op` on an [n1, n2] problem."""
    key = (op, n1, n2)
    nbytes = _ws_bytes_cache.get(key)
    if nbytes is None:
        nbytes = int(lib.oslo_workspace_bytes(op, n1, n2))
        if nbytes < 0:
            _check(nbytes, lib)
        if len(_ws_bytes_cache) < 4096:
            _ws_bytes_cache[key] = nbytes
    index = device.index if device.index is not None else torch.cuda.current_device()
    stream = _raw_stream(index) if _raw_stream is not None else torch.cuda.current_stream(device).cuda_stream
    return _ws_cache.lease(index, stream, op, nbytes)


class device_rng:
    """Within the block, the dropout entry points called on this host thread
    read (seed, offset) from ``state`` -- two 64-bit integers in device memory --
    when their kernels run, and add their ``offset`` argument to it; their
    ``seed`` argument is ignored.  ``state`` None makes the block a no-op.
    Launches captured in a graph then draw a new mask on every replay."""

    def __init__(self, state):
        if state is not None:
            if not (state.is_cuda and state.is_contiguous() and state.numel() == 2
                    and state.element_size() == 8):
                raise RuntimeError("device_rng: two 64-bit integers on the GPU expected")
        self._state = state

    def __enter__(self):
        if self._state is not None:
            lib = load_library()
            _check(lib.oslo_rng_from_device(self._state.data_ptr()), lib)
        return self

    def __exit__(self, *exc):
        if self._state is not None:
            lib = load_library()
            lib.oslo_rng_from_device(None)
        return False


def tune(key, value):
    """Overrides a launch heuristic of the library (0 restores the default)."""
    lib = load_library()
    _check(lib.oslo_tune(key.encode(), int(value)), lib)
    _ws_bytes_cache.clear()  # workspace sizes depend on the launch shapes


# ---------------------------------------------------------------------------
# LayerNorm / RMSNorm
# ---------------------------------------------------------------------------
def _compute_n1_n2(input, normalized_shape):
    # check_args / compute_n1_n2 of FusedLayerNormBinder.cpp:19-36, 59-93
    if len(normalized_shape) == 1 and input.dim() >= 1 and input.shape[-1] == normalized_shape[0]:
        n2 = int(normalized_shape[0])  # the common case, without building tuples
        return (input.numel() // n2 if n2 > 0 else 0), n2
    normalized_shape = tuple(int(s) for s in normalized_shape)
    if len(normalized_shape) < 1:
        raise RuntimeError(
            "Expected normalized_shape to be at least 1-dimensional, i.e., "
            "containing at least one element, but got normalized_shape=%s"
            % (list(normalized_shape),)
        )
    nd = len(normalized_shape)
    if input.dim() < nd or tuple(input.shape[input.dim() - nd:]) != normalized_shape:
        raise RuntimeError(
            "Given normalized_shape=%s, expected input with shape [*, %s], but got "
            "input of size%s"
            % (
                list(normalized_shape),
                ", ".join(str(s) for s in normalized_shape),
                list(input.shape),
            )
        )
    n2 = 1
    for s in normalized_shape:
        n2 *= s
    n1 = input.numel() // n2 if n2 > 0 else 0
    return n1, n2


def _check_param(p, normalized_shape, name):
    if p is not None and tuple(p.shape) != tuple(int(s) for s in normalized_shape):
        raise RuntimeError(
            "%s of shape %s does not match normalized_shape=%s"
            % (name, list(p.shape), list(normalized_shape))
        )


class _LayerNormKernel:
    """The ten functions of the reference's ``oslo_fused_layer_norm`` module."""

    def __init__(self, lib):
        self._lib = lib

    # -- forward ----------------------------------------------------------
    def _forward(self, rms, input, normalized_shape, gamma, beta, eps, out_dtype):
        lib = self._lib
        _check_input(input, "input")
        n1, n2 = _compute_n1_n2(input, normalized_shape)
        if gamma is not None:
            _check_param(gamma, normalized_shape, "gamma")
            _check_param(beta, normalized_shape, "beta")
        din = _dtype_code(input, "input", allow_f64=True)
        output = torch.empty_like(input, dtype=out_dtype)
        dout = _dtype_code(output, "output", allow_f64=True)
        for name, t in (("gamma", gamma), ("beta", beta)):
            if t is not None:
                _check_input(t, name)
                if t.dtype != out_dtype:
                    raise RuntimeError(
                        "%s has dtype %s but the output dtype is %s"
                        % (name, t.dtype, out_dtype)
                    )
        invvar = torch.empty(n1, dtype=_stat_dtype(input), device=input.device)
        with _device_of(input):
            if rms:
                rc = lib.oslo_rms_fwd(
                    _ptr(input), _ptr(gamma), _ptr(output), _ptr(invvar),
                    n1, n2, float(eps), din, dout, _stream(input),
                )
                _check(rc, lib)
                return [output, invvar]
            mean = torch.empty(n1, dtype=_stat_dtype(input), device=input.device)
            rc = lib.oslo_ln_fwd(
                _ptr(input), _ptr(gamma), _ptr(beta), _ptr(output), _ptr(mean),
                _ptr(invvar), n1, n2, float(eps), din, dout, _stream(input),
            )
            _check(rc, lib)
        return [output, mean, invvar]

    def layer_norm_forward(self, input, normalized_shape, eps):
        return self._forward(False, input, normalized_shape, None, None, eps, input.dtype)

    def layer_norm_forward_affine(self, input, normalized_shape, gamma, beta, eps):
        return self._forward(False, input, normalized_shape, gamma, beta, eps, input.dtype)

    def layer_norm_forward_affine_mixed_dtypes(self, input, normalized_shape, gamma, beta, eps):
        return self._forward(False, input, normalized_shape, gamma, beta, eps, gamma.dtype)

    def rms_norm_forward(self, input, normalized_shape, eps):
        return self._forward(True, input, normalized_shape, None, None, eps, input.dtype)

    def rms_norm_forward_affine(self, input, normalized_shape, gamma, eps):
        return self._forward(True, input, normalized_shape, gamma, None, eps, input.dtype)

    def rms_norm_forward_affine_mixed_dtypes(self, input, normalized_shape, gamma, eps):
        return self._forward(True, input, normalized_shape, gamma, None, eps, gamma.dtype)

    # -- backward ---------------------------------------------------------
    def _backward(self, rms, dout, mean, invvar, input, normalized_shape, gamma, beta):
        lib = self._lib
        for name, t in (("dout", dout), ("invvar", invvar), ("input", input)):
            _check_input(t, name)
        if not rms:
            _check_input(mean, "mean")
        n1, n2 = _compute_n1_n2(input, normalized_shape)
        if dout.shape != input.shape:
            raise RuntimeError(
                "dout of size %s does not match input of size %s"
                % (list(dout.shape), list(input.shape))
            )
        din = _dtype_code(input, "input", allow_f64=True)
        dcode = _dtype_code(dout, "dout", allow_f64=True)
        for name, t in (("invvar", invvar), ("mean", mean)):
            if t is not None and t.dtype != _stat_dtype(input):
                raise RuntimeError(
                    "%s has dtype %s, expected %s" % (name, t.dtype, _stat_dtype(input))
                )
            if t is not None and t.numel() != n1:
                raise RuntimeError(
                    "%s has %d elements for %d rows of input" % (name, t.numel(), n1)
                )
        grad_input = torch.empty_like(input)
        grad_gamma = grad_beta = None
        lease = _NO_WORKSPACE
        if gamma is not None:
            _check_input(gamma, "gamma")
            _check_param(gamma, normalized_shape, "gamma")
            if gamma.dtype != dout.dtype:
                raise RuntimeError(
                    "gamma has dtype %s but dout has dtype %s" % (gamma.dtype, dout.dtype)
                )
            grad_gamma = torch.empty_like(gamma)
            if not rms:
                grad_beta = torch.empty_like(beta if beta is not None else gamma)
            lease = _workspace(
                lib, OSLO_OP_RMS_BWD if rms else OSLO_OP_LN_BWD, n1, n2, input.device
            )
        with _device_of(input), lease as ws:
            if rms:
                rc = lib.oslo_rms_bwd(
                    _ptr(dout), _ptr(input), _ptr(invvar), _ptr(gamma), _ptr(grad_input),
                    _ptr(grad_gamma), _ptr(ws.tensor), ws.nbytes, n1, n2, din, dcode,
                    _stream(input),
                )
            else:
                rc = lib.oslo_ln_bwd(
                    _ptr(dout), _ptr(input), _ptr(mean), _ptr(invvar), _ptr(gamma),
                    _ptr(grad_input), _ptr(grad_gamma), _ptr(grad_beta), _ptr(ws.tensor),
                    ws.nbytes, n1, n2, din, dcode, _stream(input),
                )
            _check(rc, lib)
        return grad_input, grad_gamma, grad_beta

    def layer_norm_backward(self, dout, mean, invvar, input, normalized_shape, eps):
        return self._backward(False, dout, mean, invvar, input, normalized_shape, None, None)[0]

    def layer_norm_backward_affine(
        self, dout, mean, invvar, input, normalized_shape, gamma, beta, eps
    ):
        return list(
            self._backward(False, dout, mean, invvar, input, normalized_shape, gamma, beta)
        )

    def rms_norm_backward(self, dout, invvar, input, normalized_shape, eps):
        return self._backward(True, dout, None, invvar, input, normalized_shape, None, None)[0]

    def rms_norm_backward_affine(self, dout, invvar, input, normalized_shape, gamma, eps):
        gi, gg, _ = self._backward(
            True, dout, None, invvar, input, normalized_shape, gamma, None
        )
        return [gi, gg]

    # -- bias-dropout-add fused into the norm (no counterpart in the
    #    reference's module: its models chain FusedBiasDropout, the residual
    #    add and LayerNorm, oslo/transformers/models/bert/modeling_bert.py:
    #    343-346) ----------------------------------------------------------
    def bias_dropout_add_norm_forward(
        self, rms, input, bias, residual, normalized_shape, gamma, beta, eps,
        p, seed, offset, want_h=True,
    ):
        """``h = dropout(input + bias, p) + residual; y = norm(h)``.

        Returns ``[y, h, mean, invvar]`` (``h`` None when ``want_h`` is false,
        ``mean`` None for RMSNorm).  One dtype throughout.
        """
        lib = self._lib
        _check_input(input, "input")
        n1, n2 = _compute_n1_n2(input, normalized_shape)
        for name, t in (("gamma", gamma), ("beta", beta), ("bias", bias)):
            if t is not None:
                _check_input(t, name)
                _check_param(t, normalized_shape, name)
        if residual is not None:
            _check_input(residual, "residual")
            if residual.shape != input.shape:
                raise RuntimeError("residual and input differ in shape")
        for name, t in (("gamma", gamma), ("beta", beta), ("bias", bias), ("residual", residual)):
            if t is not None and t.dtype != input.dtype:
                raise RuntimeError(
                    "%s has dtype %s but input has dtype %s" % (name, t.dtype, input.dtype)
                )
        code = _dtype_code(input, "input")
        y = torch.empty_like(input)
        h = torch.empty_like(input) if want_h else None
        invvar = torch.empty(n1, dtype=torch.float32, device=input.device)
        mean = None if rms else torch.empty(n1, dtype=torch.float32, device=input.device)
        with _device_of(input):
            rc = lib.oslo_bias_dropout_add_norm_fwd(
                _ptr(input), _ptr(bias), _ptr(residual), _ptr(gamma), _ptr(beta), _ptr(h),
                _ptr(y), _ptr(mean), _ptr(invvar), n1, n2, float(eps), float(p),
                int(seed), int(offset), 1 if rms else 0, code, _stream(input),
            )
            _check(rc, lib)
        return [y, h, mean, invvar]

    def bias_dropout_add_norm_backward(
        self, rms, dout, dh_extra, h, mean, invvar, normalized_shape, gamma,
        p, seed, offset, need_bias_grad=True,
    ):
        """Returns ``(grad_residual, grad_input, grad_gamma, grad_beta, grad_bias)``;
        ``grad_input`` is ``grad_residual`` itself when ``p == 0``."""
        lib = self._lib
        for name, t in (("dout", dout), ("h", h), ("invvar", invvar)):
            _check_input(t, name)
        n1, n2 = _compute_n1_n2(h, normalized_shape)
        if dout.shape != h.shape or dout.dtype != h.dtype:
            raise RuntimeError("dout and h differ in shape or dtype")
        if not rms:
            _check_input(mean, "mean")
        for name, t in (("invvar", invvar), ("mean", None if rms else mean)):
            if t is not None and (t.dtype != torch.float32 or t.numel() != n1):
                raise RuntimeError("%s must be float32 with one element per row of h" % name)
        if dh_extra is not None:
            _check_input(dh_extra, "dh_extra")
            if dh_extra.shape != h.shape or dh_extra.dtype != h.dtype:
                raise RuntimeError("dh_extra and h differ in shape or dtype")
        code = _dtype_code(h, "h")
        grad_res = torch.empty_like(h)
        grad_in = torch.empty_like(h) if p > 0.0 else None
        grad_gamma = grad_beta = grad_bias = None
        if gamma is not None:
            _check_input(gamma, "gamma")
            _check_param(gamma, normalized_shape, "gamma")
            if gamma.dtype != h.dtype:
                raise RuntimeError(
                    "gamma has dtype %s but h has dtype %s" % (gamma.dtype, h.dtype)
                )
            grad_gamma = torch.empty_like(gamma)
            if not rms:
                grad_beta = torch.empty_like(gamma)
        if need_bias_grad:
            grad_bias = torch.empty(n2, dtype=h.dtype, device=h.device)
        lease = _NO_WORKSPACE
        if gamma is not None or need_bias_grad:
            lease = _workspace(lib, OSLO_OP_BIAS_DROPOUT_ADD_NORM_BWD, n1, n2, h.device)
        with _device_of(h), lease as ws:
            rc = lib.oslo_bias_dropout_add_norm_bwd(
                _ptr(dout), _ptr(dh_extra), _ptr(h), _ptr(mean), _ptr(invvar), _ptr(gamma),
                _ptr(grad_res), _ptr(grad_in), _ptr(grad_gamma), _ptr(grad_beta),
                _ptr(grad_bias), _ptr(ws.tensor), ws.nbytes, n1, n2, float(p), int(seed),
                int(offset), 1 if rms else 0, code, _stream(h),
            )
            _check(rc, lib)
        if grad_in is None:
            grad_in = grad_res
        if grad_bias is not None:
            grad_bias = grad_bias.view(tuple(int(s) for s in normalized_shape))
        return grad_res, grad_in, grad_gamma, grad_beta, grad_bias


# ---------------------------------------------------------------------------
# scaled masked softmax
# ---------------------------------------------------------------------------
# The softmax backward streams three tensors of gigabytes at identical offsets
# (y, dy -> dx).  torch places large tensors on 2 MiB boundaries; when all three
# start on the same 2 MiB phase their requests meet in the same memory channels
# and the kernel measures 1.5-4 % slower on MI355X than with the starts a little
# over 1 MiB apart.  The tensors this binding allocates for the softmax (the
# probabilities in forward, the input gradient in backward) are therefore placed
# on phase k * (1 MiB + 4 KiB) of their own 2 MiB-rounded allocation, k = 1 for
# forward outputs and k = 2 for backward outputs; operands that torch allocated
# (the scores, the incoming gradient) sit on phase 0.
STAGGER_MIN_BYTES = 64 << 20
STAGGER_STEP = (1 << 20) + 4096
_STAGGER_ROUND = 2 << 20


def empty_staggered(shape, dtype, device, k):
    """An uninitialised contiguous tensor whose first byte lies k * STAGGER_STEP
    (modulo 2 MiB) past a 2 MiB boundary; small tensors and k == 0 are plain
    ``torch.empty``.  Costs 2 MiB of slack per tensor."""
    n = 1
    for d in shape:
        n *= int(d)
    nbytes = n * torch.empty(0, dtype=dtype).element_size()
    if k == 0 or nbytes < STAGGER_MIN_BYTES:
        return torch.empty(tuple(shape), dtype=dtype, device=device)
    base = torch.empty(nbytes + _STAGGER_ROUND, dtype=torch.uint8, device=device)
    off = (k * STAGGER_STEP - base.data_ptr()) % _STAGGER_ROUND
    return base[off:off + nbytes].view(dtype).view(tuple(shape))


def _softmax_out(like, k):
    return empty_staggered(like.shape, like.dtype, like.device, k)


class _SoftmaxKernel:
    """The five functions of ``FusedScaleMaskSoftmaxBinder.cpp:111-127``.

    The reference admits fp16 / bf16 only (``:42-44, 84-86``); fp32 is accepted
    here as well.  ``fused_scaled_masked_softmax_backward`` takes an optional
    ``mask`` (not in the reference signature) that lets the kernel skip loads
    of masked keys.
    """

    def __init__(self, lib):
        self._lib = lib

    @staticmethod
    def _mask_u8(mask, like):
        """The mask as contiguous bytes (non-zero = masked out); it has to live
        on the device of ``like``, since the kernel reads it through a raw pointer."""
        if mask.device != like.device:
            raise RuntimeError(
                "mask is on %s but the softmax operand is on %s" % (mask.device, like.device)
            )
        if mask.dtype == torch.bool:
            return mask.contiguous().view(torch.uint8)
        if mask.dtype == torch.uint8:
            return mask.contiguous()
        return (mask != 0).contiguous().view(torch.uint8)

    def fused_scaled_masked_softmax_forward(self, input, mask, scale_factor, causal=False):
        """``causal=True`` (not in the reference's shim) hides the keys beyond
        the diagonal as well: causal attention on a padded batch."""
        lib = self._lib
        b, np_, sq, sk, mb, msq = self._masked_dims(input, mask)
        _check_input(input, "input")
        m8 = self._mask_u8(mask, input)
        out = _softmax_out(input, 1)
        with _device_of(input):
            fn = lib.oslo_softmax_causal_masked_fwd if causal else lib.oslo_softmax_masked_fwd
            rc = fn(
                _ptr(input), _ptr(m8), _ptr(out), b, np_, sq, sk, mb, msq,
                float(scale_factor), _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return out

    def fused_scaled_masked_softmax_backward(
        self, output_grads, softmax_results, scale_factor, mask=None, inplace=False,
        causal=False,
    ):
        lib = self._lib
        if output_grads.dim() != 4 or softmax_results.dim() != 4:
            raise RuntimeError("expected 4D tensor")
        _check_input(output_grads, "output_grads")
        _check_input(softmax_results, "softmax_results")
        if output_grads.dtype != softmax_results.dtype:
            raise RuntimeError("output_grads and softmax_results differ in dtype")
        if output_grads.shape != softmax_results.shape:
            raise RuntimeError("output_grads and softmax_results differ in shape")
        b, np_, sq, sk = softmax_results.shape
        mb = msq = 1
        m8 = None
        if mask is not None:
            _, _, _, _, mb, msq = self._masked_dims(softmax_results, mask)
            m8 = self._mask_u8(mask, softmax_results)
        # inplace=True overwrites output_grads, as the kernel this shim was
        # written for does
        grad_input = output_grads if inplace else _softmax_out(output_grads, 2)
        with _device_of(output_grads):
            fn = lib.oslo_softmax_causal_masked_bwd if causal else lib.oslo_softmax_masked_bwd
            rc = fn(
                _ptr(output_grads), _ptr(softmax_results), _ptr(m8), _ptr(grad_input),
                b, np_, sq, sk, mb, msq, float(scale_factor),
                _dtype_code(output_grads, "output_grads"), _stream(output_grads),
            )
            _check(rc, lib)
        return grad_input

    def get_batch_per_block(self, query_seq_len, key_seq_len, batches, attn_heads):
        lib = self._lib
        rc = lib.oslo_softmax_batch_per_block(
            int(query_seq_len), int(key_seq_len), int(batches), int(attn_heads)
        )
        if rc < 0:
            _check(rc, lib)
        return int(rc)

    def fused_scaled_upper_triang_masked_softmax_forward(self, input, scale_factor):
        lib = self._lib
        if input.dim() != 3:
            raise RuntimeError("expected 3D tensor")
        _check_input(input, "input")
        ab, sq, sk = input.shape
        out = _softmax_out(input, 1)
        with _device_of(input):
            rc = lib.oslo_softmax_causal_fwd(
                _ptr(input), _ptr(out), ab, sq, sk, float(scale_factor),
                _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return out

    def fused_scaled_upper_triang_masked_softmax_backward(
        self, output_grads, softmax_results, scale_factor, inplace=False
    ):
        lib = self._lib
        if output_grads.dim() != 3 or softmax_results.dim() != 3:
            raise RuntimeError("expected 3D tensor")
        _check_input(output_grads, "output_grads")
        _check_input(softmax_results, "softmax_results")
        if output_grads.dtype != softmax_results.dtype:
            raise RuntimeError("output_grads and softmax_results differ in dtype")
        if output_grads.shape != softmax_results.shape:
            raise RuntimeError("output_grads and softmax_results differ in shape")
        ab, sq, sk = softmax_results.shape
        grad_input = output_grads if inplace else _softmax_out(output_grads, 2)
        with _device_of(output_grads):
            rc = lib.oslo_softmax_causal_bwd(
                _ptr(output_grads), _ptr(softmax_results), _ptr(grad_input), ab, sq, sk,
                float(scale_factor), _dtype_code(output_grads, "output_grads"),
                _stream(output_grads),
            )
            _check(rc, lib)
        return grad_input

    # -- softmax with the attention dropout fused in (no counterpart in the
    #    reference's shim: the models apply nn.Dropout to the probabilities,
    #    oslo/transformers/models/gpt2/modeling_gpt2.py:138-142) -------------
    def _masked_dims(self, input, mask):
        if input.dim() != 4 or mask.dim() != 4:
            raise RuntimeError("expected 4D tensor")
        b, np_, sq, sk = input.shape
        mb, mh, msq, msk = mask.shape
        if mh != 1 or msk != sk or mb not in (1, b) or msq not in (1, sq):
            raise RuntimeError(
                "mask of size %s does not broadcast to [%d, 1, %d, %d]"
                % (list(mask.shape), b, sq, sk)
            )
        return b, np_, sq, sk, mb, msq

    def softmax_dropout_forward(self, input, mask, scale_factor, p, seed, offset, causal=False):
        """``dropout(softmax(mask(scale * input)), p)`` -> ``[out, stats]``.

        ``mask=None`` selects the causal form on a 3-D ``[attn_batches, sq, sk]``
        input, otherwise ``input`` is ``[b, np, sq, sk]`` and ``mask`` a 4-D
        padding mask (with ``causal=True`` the keys beyond the diagonal are
        hidden as well).  ``stats`` (float32 ``[rows, 2]``) and ``input`` are
        what the backward pass needs.
        """
        lib = self._lib
        _check_input(input, "input")
        out = _softmax_out(input, 1)
        rows = input.numel() // input.shape[-1] if input.numel() else 0
        stats = torch.empty((rows, 2), dtype=torch.float32, device=input.device)
        with _device_of(input):
            if mask is None:
                if input.dim() != 3:
                    raise RuntimeError("expected 3D tensor")
                ab, sq, sk = input.shape
                rc = lib.oslo_softmax_causal_dropout_fwd(
                    _ptr(input), _ptr(out), _ptr(stats), ab, sq, sk,
                    float(scale_factor), float(p), int(seed), int(offset),
                    _dtype_code(input, "input"), _stream(input),
                )
            else:
                b, np_, sq, sk, mb, msq = self._masked_dims(input, mask)
                m8 = self._mask_u8(mask, input)
                fn = (lib.oslo_softmax_causal_masked_dropout_fwd if causal
                      else lib.oslo_softmax_masked_dropout_fwd)
                rc = fn(
                    _ptr(input), _ptr(m8), _ptr(out), _ptr(stats), b, np_, sq, sk,
                    mb, msq, float(scale_factor), float(p), int(seed), int(offset),
                    _dtype_code(input, "input"), _stream(input),
                )
            _check(rc, lib)
        return [out, stats]

    def softmax_dropout_backward(
        self, output_grads, input, stats, mask, scale_factor, p, seed, offset,
        inplace=False, causal=False,
    ):
        lib = self._lib
        _check_input(output_grads, "output_grads")
        _check_input(input, "input")
        _check_input(stats, "stats")
        if output_grads.dtype != input.dtype or output_grads.shape != input.shape:
            raise RuntimeError("output_grads and input differ in dtype or shape")
        rows = input.numel() // input.shape[-1] if input.numel() else 0
        if stats.dtype != torch.float32 or stats.numel() != 2 * rows:
            raise RuntimeError("stats must be float32 [rows, 2]")
        grad_input = output_grads if inplace else _softmax_out(output_grads, 2)
        with _device_of(input):
            if mask is None:
                if input.dim() != 3:
                    raise RuntimeError("expected 3D tensor")
                ab, sq, sk = input.shape
                rc = lib.oslo_softmax_causal_dropout_bwd(
                    _ptr(output_grads), _ptr(input), _ptr(stats), _ptr(grad_input),
                    ab, sq, sk, float(scale_factor), float(p), int(seed), int(offset),
                    _dtype_code(input, "input"), _stream(input),
                )
            else:
                b, np_, sq, sk, mb, msq = self._masked_dims(input, mask)
                m8 = self._mask_u8(mask, input)
                fn = (lib.oslo_softmax_causal_masked_dropout_bwd if causal
                      else lib.oslo_softmax_masked_dropout_bwd)
                rc = fn(
                    _ptr(output_grads), _ptr(input), _ptr(m8), _ptr(stats),
                    _ptr(grad_input), b, np_, sq, sk, mb, msq, float(scale_factor),
                    float(p), int(seed), int(offset), _dtype_code(input, "input"),
                    _stream(input),
                )
            _check(rc, lib)
        return grad_input


    # -- softmax with an additive floating-point term (no counterpart in the
    #    reference's shim; its models add the term to the scores with torch,
    #    oslo/transformers/models/bert/modeling_bert.py:298-306) -------------
    @staticmethod
    def _bias_operand(bias, input):
        """The additive term as the kernel addresses it: ``(tensor, stride_b,
        stride_h, stride_q, dtype_code)``.  ``bias`` broadcasts against the 4-D
        ``input``: up to four dimensions, each of the leading three either 1 or
        the full size (expanded views are fine: their stride is 0), the keys
        contiguous; its dtype becomes the input's or float32."""
        if input.dim() != 4:
            raise RuntimeError("expected 4D tensor")
        if not bias.is_floating_point():
            raise RuntimeError("the additive term must be a floating-point tensor")
        if bias.device != input.device:
            raise RuntimeError(
                "the additive term is on %s but the softmax operand is on %s"
                % (bias.device, input.device)
            )
        if bias.dim() > 4:
            raise RuntimeError("the additive term has more than four dimensions")
        while bias.dim() < 4:
            bias = bias.unsqueeze(0)
        b, np_, sq, sk = input.shape
        for d, full in enumerate((b, np_, sq)):
            if bias.size(d) not in (1, full):
                raise RuntimeError(
                    "additive term of size %s does not broadcast to %s"
                    % (list(bias.shape), list(input.shape))
                )
        if bias.size(3) != sk:
            if bias.size(3) != 1:
                raise RuntimeError(
                    "additive term of size %s does not broadcast to %s"
                    % (list(bias.shape), list(input.shape))
                )
            bias = bias.expand(-1, -1, -1, sk).contiguous()
        if bias.dtype != input.dtype and bias.dtype != torch.float32:
            bias = bias.float()
        if sk > 1 and bias.stride(3) != 1:
            bias = bias.contiguous()
        strides = [0 if bias.size(d) == 1 else bias.stride(d) for d in range(3)]
        return bias, strides[0], strides[1], strides[2], _DTYPE_CODE[bias.dtype]

    @staticmethod
    def _bias_flags(causal, skip_hidden, strides, forward):
        if skip_hidden is None:
            # Reading the term first pays in the backward passes when the term is
            # small next to the logits (a mask shared by the heads or by the
            # queries): a hidden chunk saves two loads there.  In the forward
            # pass it does not: the loads of the logits then wait for the term,
            # which costs more than the unread logits save (measured at
            # [16,16,1024,1024] fp16 with 48 % of the keys under -inf: 159 us
            # with the test, 163 us without; with a -10000 mask, which hides
            # nothing, 190-210 us against 163 us).
            skip_hidden = (not forward) and (strides[1] == 0 or strides[2] == 0)
        return (1 if causal else 0) | (2 if skip_hidden else 0)

    def softmax_bias_forward(self, input, bias, scale_factor, causal=False, skip_hidden=None):
        """``softmax(scale * input + bias)`` over the last dimension of the
        ``[b, np, sq, sk]`` input; ``causal`` hides the keys beyond the diagonal
        as well.  ``skip_hidden`` (default: off in the forward passes, on in the
        backward passes when the term is shared by heads or queries) lets the
        kernel leave logits unread whose term is -inf or the lowest finite value."""
        lib = self._lib
        _check_input(input, "input")
        bias, sb, sh, sq_, bcode = self._bias_operand(bias, input)
        b, np_, sq, sk = input.shape
        out = _softmax_out(input, 1)
        flags = self._bias_flags(causal, skip_hidden, (sb, sh, sq_), True)
        with _device_of(input):
            rc = lib.oslo_softmax_bias_fwd(
                _ptr(input), _ptr(bias), _ptr(out), b, np_, sq, sk, sb, sh, sq_, bcode,
                flags, float(scale_factor), _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return out

    def softmax_bias_backward(
        self, output_grads, softmax_results, scale_factor, bias=None, causal=False,
        skip_hidden=None, inplace=False,
    ):
        """``scale * y * (g - sum(g * y))``; ``bias`` (optional) only lets the
        kernel skip loads, as in the forward pass."""
        lib = self._lib
        if output_grads.dim() != 4 or softmax_results.dim() != 4:
            raise RuntimeError("expected 4D tensor")
        _check_input(output_grads, "output_grads")
        _check_input(softmax_results, "softmax_results")
        if output_grads.dtype != softmax_results.dtype:
            raise RuntimeError("output_grads and softmax_results differ in dtype")
        if output_grads.shape != softmax_results.shape:
            raise RuntimeError("output_grads and softmax_results differ in shape")
        b, np_, sq, sk = softmax_results.shape
        sb = sh = sq_ = 0
        bcode = _dtype_code(softmax_results, "softmax_results")
        flags = 1 if causal else 0
        if bias is not None:
            bias, sb, sh, sq_, bcode = self._bias_operand(bias, softmax_results)
            flags = self._bias_flags(causal, skip_hidden, (sb, sh, sq_), False)
            if not flags & 2:
                bias = None
        grad_input = output_grads if inplace else _softmax_out(output_grads, 2)
        with _device_of(output_grads):
            rc = lib.oslo_softmax_bias_bwd(
                _ptr(output_grads), _ptr(softmax_results), _ptr(bias), _ptr(grad_input),
                b, np_, sq, sk, sb, sh, sq_, bcode, flags, float(scale_factor),
                _dtype_code(output_grads, "output_grads"), _stream(output_grads),
            )
            _check(rc, lib)
        return grad_input

    def softmax_bias_dropout_forward(
        self, input, bias, scale_factor, p, seed, offset, causal=False, skip_hidden=None
    ):
        """``dropout(softmax(scale * input + bias), p)`` -> ``[out, stats]``."""
        lib = self._lib
        _check_input(input, "input")
        bias, sb, sh, sq_, bcode = self._bias_operand(bias, input)
        b, np_, sq, sk = input.shape
        out = _softmax_out(input, 1)
        stats = torch.empty((b * np_ * sq, 2), dtype=torch.float32, device=input.device)
        flags = self._bias_flags(causal, skip_hidden, (sb, sh, sq_), True)
        with _device_of(input):
            rc = lib.oslo_softmax_bias_dropout_fwd(
                _ptr(input), _ptr(bias), _ptr(out), _ptr(stats), b, np_, sq, sk, sb, sh, sq_,
                bcode, flags, float(scale_factor), float(p), int(seed), int(offset),
                _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return [out, stats]

    def softmax_bias_dropout_backward(
        self, output_grads, input, bias, stats, scale_factor, p, seed, offset,
        causal=False, skip_hidden=None, inplace=False,
    ):
        lib = self._lib
        _check_input(output_grads, "output_grads")
        _check_input(input, "input")
        _check_input(stats, "stats")
        if output_grads.dtype != input.dtype or output_grads.shape != input.shape:
            raise RuntimeError("output_grads and input differ in dtype or shape")
        bias, sb, sh, sq_, bcode = self._bias_operand(bias, input)
        b, np_, sq, sk = input.shape
        if stats.dtype != torch.float32 or stats.numel() != 2 * b * np_ * sq:
            raise RuntimeError("stats must be float32 [rows, 2]")
        flags = self._bias_flags(causal, skip_hidden, (sb, sh, sq_), False)
        grad_input = output_grads if inplace else _softmax_out(output_grads, 2)
        with _device_of(input):
            rc = lib.oslo_softmax_bias_dropout_bwd(
                _ptr(output_grads), _ptr(input), _ptr(bias), _ptr(stats), _ptr(grad_input),
                b, np_, sq, sk, sb, sh, sq_, bcode, flags, float(scale_factor), float(p),
                int(seed), int(offset), _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return grad_input


# ---------------------------------------------------------------------------
# bias-GeLU and bias-dropout-add (TorchScript in the reference,
# oslo/torch/nn/modules/functional.py:23-50, 295-298; native here)
# ---------------------------------------------------------------------------
def _rows_cols(x, bias):
    cols = x.shape[-1] if x.dim() > 0 else 1
    if bias is not None:
        if bias.dim() != 1 or bias.shape[0] != cols:
            raise RuntimeError(
                "bias of size %s does not match the last dimension of input of size %s"
                % (list(bias.shape), list(x.shape))
            )
    rows = x.numel() // cols if cols > 0 else 0
    return rows, cols


class _FusedElementwiseKernel:
    def __init__(self, lib):
        self._lib = lib

    def bias_gelu_forward(self, input, bias):
        lib = self._lib
        _check_input(input, "input")
        if bias is not None:
            _check_input(bias, "bias")
            if bias.dtype != input.dtype:
                raise RuntimeError("bias and input differ in dtype")
        rows, cols = _rows_cols(input, bias)
        out = torch.empty_like(input)
        with _device_of(input):
            rc = lib.oslo_bias_gelu_fwd(
                _ptr(input), _ptr(bias), _ptr(out), rows, cols,
                _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return out

    def bias_gelu_backward(self, grad_output, input, bias, need_bias_grad=True):
        lib = self._lib
        _check_input(grad_output, "grad_output")
        _check_input(input, "input")
        if grad_output.dtype != input.dtype or grad_output.shape != input.shape:
            raise RuntimeError("grad_output does not match input")
        if bias is not None:
            _check_input(bias, "bias")
            if bias.dtype != input.dtype:
                raise RuntimeError("bias and input differ in dtype")
        rows, cols = _rows_cols(input, bias)
        grad_input = torch.empty_like(input)
        grad_bias = None
        lease = _NO_WORKSPACE
        if bias is not None and need_bias_grad:
            grad_bias = torch.empty_like(bias)
            lease = _workspace(lib, OSLO_OP_BIAS_GELU_BWD, rows, cols, input.device)
        with _device_of(input), lease as ws:
            rc = lib.oslo_bias_gelu_bwd(
                _ptr(grad_output), _ptr(input), _ptr(bias), _ptr(grad_input),
                _ptr(grad_bias), _ptr(ws.tensor), ws.nbytes, rows, cols,
                _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return grad_input, grad_bias

    def bias_dropout_add_forward(
        self, input, bias, residual, p, seed, offset, out=None, return_mask=False
    ):
        lib = self._lib
        _check_input(input, "input")
        for name, t in (("bias", bias), ("residual", residual)):
            if t is not None:
                _check_input(t, name)
                if t.dtype != input.dtype:
                    raise RuntimeError("%s and input differ in dtype" % name)
        if residual is not None and residual.shape != input.shape:
            raise RuntimeError("residual does not match input")
        rows, cols = _rows_cols(input, bias)
        if out is None:
            out = torch.empty_like(input)
        mask = (
            torch.empty(input.shape, dtype=torch.uint8, device=input.device)
            if return_mask
            else None
        )
        with _device_of(input):
            rc = lib.oslo_bias_dropout_add_fwd(
                _ptr(input), _ptr(bias), _ptr(residual), _ptr(out), _ptr(mask),
                rows, cols, float(p), int(seed), int(offset),
                _dtype_code(input, "input"), _stream(input),
            )
            _check(rc, lib)
        return (out, mask) if return_mask else out

    def bias_dropout_add_backward(
        self, grad_output, p, seed, offset, need_input_grad=True, need_bias_grad=True
    ):
        lib = self._lib
        _check_input(grad_output, "grad_output")
        cols = grad_output.shape[-1]
        rows = grad_output.numel() // cols if cols > 0 else 0
        grad_input = torch.empty_like(grad_output) if need_input_grad else None
        grad_bias = None
        lease = _NO_WORKSPACE
        if need_bias_grad:
            grad_bias = torch.empty(cols, dtype=grad_output.dtype, device=grad_output.device)
            lease = _workspace(
                lib, OSLO_OP_BIAS_DROPOUT_ADD_BWD, rows, cols, grad_output.device
            )
        if grad_input is None and grad_bias is None:
            return None, None
        with _device_of(grad_output), lease as ws:
            rc = lib.oslo_bias_dropout_add_bwd(
                _ptr(grad_output), _ptr(grad_input), _ptr(grad_bias), _ptr(ws.tensor), ws.nbytes,
                rows, cols, float(p), int(seed), int(offset),
                _dtype_code(grad_output, "grad_output"), _stream(grad_output),
            )
            _check(rc, lib)
        return grad_input, grad_bias

    def philox_mask(self, n, p, seed, offset, device):
        lib = self._lib
        mask = torch.empty(int(n), dtype=torch.uint8, device=device)
        with torch.cuda.device(mask.device):
            rc = lib.oslo_philox_mask(
                _ptr(mask), int(n), float(p), int(seed), int(offset), _stream(mask)
            )
            _check(rc, lib)
        return mask

    def philox_words(self, ngroups, first_group, seed, offset, device):
        lib = self._lib
        out = torch.empty(int(ngroups) * 4, dtype=torch.int32, device=device)
        with torch.cuda.device(out.device):
            rc = lib.oslo_philox_words(
                _ptr(out), int(ngroups), int(first_group), int(seed), int(offset),
                _stream(out),
            )
            _check(rc, lib)
        return out

    def copy_probe(self, src, dst):
        lib = self._lib
        nbytes = src.numel() * src.element_size()
        with _device_of(src):
            _check(lib.oslo_copy_probe(_ptr(src), _ptr(dst), nbytes, _stream(src)), lib)
        return dst

    def wave_reduce_selftest(self, device):
        lib = self._lib
        out = torch.zeros(4, dtype=torch.float32, device=device)
        with torch.cuda.device(out.device):
            _check(lib.oslo_wave_reduce_selftest(_ptr(out), _stream(out)), lib)
        return out


_layernorm_kernel = None
_softmax_kernel = None
_elementwise_kernel = None


def get_layernorm_kernel():
    global _layernorm_kernel
    if _layernorm_kernel is None:
        _layernorm_kernel = _LayerNormKernel(load_library())
    return _layernorm_kernel


def get_softmax_kernel():
    global _softmax_kernel
    if _softmax_kernel is None:
        _softmax_kernel = _SoftmaxKernel(load_library())
    return _softmax_kernel


# ---------------------------------------------------------------------------
# multi-tensor optimizer steps
# ---------------------------------------------------------------------------
def _tensor_tables(tensor_lists, names, dtypes=None):
    """Checks lists of equally long, pairwise equally sized contiguous GPU
    tensors (the checks of the reference's multi_tensor_apply.cuh:44-72) and
    returns ``(pointer tables, sizes, n, first tensor)``; ``dtypes[k]`` None
    means list k follows the dtype of its first tensor."""
    n = len(tensor_lists[0])
    for lst in tensor_lists:
        if len(lst) != n:
            raise RuntimeError("Size mismatch among tensor lists")
    if n == 0:
        return None, None, 0, None
    ref = tensor_lists[0][0]
    device = ref.device
    counts = [t.numel() for t in tensor_lists[0]]
    for k, lst in enumerate(tensor_lists):
        want = lst[0].dtype if dtypes is None or dtypes[k] is None else dtypes[k]
        # one pass per list; the slow loop below only runs to name the offender
        if all(t.is_cuda and t.dtype == want and t.device == device and t.is_contiguous() for t in lst):
            if k == 0 or [t.numel() for t in lst] == counts:
                continue
        for i, t in enumerate(lst):
            _check_input(t, "%s %d" % (names[k], i))
            if t.dtype != want or t.device != device:
                raise RuntimeError(
                    "A tensor was not the same dtype / on the same device as the first tensor"
                )
            if t.numel() != counts[i]:
                raise RuntimeError("Size mismatch among tensor lists")
    arr = ctypes.c_void_p * n
    sizes = (ctypes.c_int64 * n)(*counts)
    tables = [arr(*[t.data_ptr() for t in lst]) for lst in tensor_lists]
    return tables, sizes, n, ref


class _AdamKernel:
    """``multi_tensor_adam`` of the reference's ``oslo_fused_adam`` module
    (``oslo/torch/_C/csrc/FusedAdamBinder.cpp:12-15``), same argument list."""

    def __init__(self, lib):
        self._lib = lib

    def multi_tensor_adam(
        self, chunk_size, noop_flag, tensor_lists, lr, beta1, beta2, epsilon, step,
        mode, bias_correction, weight_decay,
    ):
        """``tensor_lists`` = ``[grads, params, exp_avgs, exp_avg_sqs]``, updated in
        place.  ``chunk_size`` and ``noop_flag`` are accepted for signature
        compatibility; the reference's kernel does not act on them either
        (``multi_tensor_adam.cu:29-31``)."""
        lib = self._lib
        if len(tensor_lists) != 4:
            raise RuntimeError("tensor_lists must hold [grads, params, exp_avgs, exp_avg_sqs]")
        names = ("grad", "param", "exp_avg", "exp_avg_sq")
        ref_dtype = tensor_lists[1][0].dtype if len(tensor_lists[1]) else None
        tables, sizes, n, ref = _tensor_tables(tensor_lists, names, [ref_dtype] * 4)
        if n == 0:
            return
        code = _dtype_code(ref, "params[0]")
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_adam(
                tables[0], tables[1], tables[2], tables[3], sizes, n, float(lr), float(beta1),
                float(beta2), float(epsilon), int(step), int(mode), int(bias_correction),
                float(weight_decay), code, _stream(ref),
            )
            _check(rc, lib)


def _flag_ptr(noop_flag, ref):
    """Device pointer of the overflow flag (an int32 tensor), or None."""
    if noop_flag is None:
        return None
    if not (noop_flag.is_cuda and noop_flag.dtype == torch.int32 and noop_flag.numel() >= 1):
        raise RuntimeError("noop_flag must be an int32 tensor on the GPU")
    if ref is not None and noop_flag.device != ref.device:
        raise RuntimeError("expected noop flag to be on the same device as tensors")
    return noop_flag.data_ptr()


class _SGDKernel:
    """``multi_tensor_sgd`` of ``oslo/torch/_C/csrc/FusedSGDBinder.cpp``."""

    def __init__(self, lib):
        self._lib = lib

    def multi_tensor_sgd(
        self, chunk_size, noop_flag, tensor_lists, wd, momentum, dampening, lr, nesterov,
        first_run, wd_after_momentum, scale,
    ):
        """``tensor_lists`` = ``[grads, weights, momentum buffers]`` or, with a
        fourth list, additionally 16-bit copies of the updated float32 weights
        (``multi_tensor_sgd.cu:139-201``).  Nothing happens while ``noop_flag``
        is non-zero."""
        lib = self._lib
        if len(tensor_lists) not in (3, 4):
            raise RuntimeError("tensor_lists must hold [grads, weights, momentums(, weight copies)]")
        names = ("grad", "weight", "momentum", "weight copy")
        wdtype = tensor_lists[1][0].dtype if len(tensor_lists[1]) else None
        dts = [None, wdtype, wdtype, None][: len(tensor_lists)]
        tables, sizes, n, ref = _tensor_tables(tensor_lists, names, dts)
        if n == 0:
            return
        copy = len(tensor_lists) == 4
        if copy and tensor_lists[3][0].dtype not in (torch.float16, torch.bfloat16):
            raise RuntimeError("Additional output tensors should always be fp16 (or bf16).")
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_sgd(
                tables[0], tables[1], tables[2], tables[3] if copy else None, sizes, n,
                float(wd), float(momentum), float(dampening), float(lr), int(bool(nesterov)),
                int(bool(first_run)), int(bool(wd_after_momentum)), float(scale),
                _dtype_code(tensor_lists[0][0], "grads[0]"),
                _dtype_code(tensor_lists[1][0], "weights[0]"),
                _dtype_code(tensor_lists[3][0], "copies[0]") if copy else 0,
                _flag_ptr(noop_flag, ref), _stream(ref),
            )
            _check(rc, lib)


class _AdagradKernel:
    """``multi_tensor_adagrad`` of ``oslo/torch/_C/csrc/FusedAdagradBinder.cpp``."""

    def __init__(self, lib):
        self._lib = lib

    def multi_tensor_adagrad(self, chunk_size, noop_flag, tensor_lists, lr, epsilon, mode,
                             weight_decay):
        """``tensor_lists`` = ``[grads, params, sums of squares]``, one dtype."""
        lib = self._lib
        if len(tensor_lists) != 3:
            raise RuntimeError("tensor_lists must hold [grads, params, sums]")
        d = tensor_lists[0][0].dtype if len(tensor_lists[0]) else None
        tables, sizes, n, ref = _tensor_tables(tensor_lists, ("grad", "param", "sum"), [d] * 3)
        if n == 0:
            return
        # (an int32 tensor on the GPU, which multi_tensor_apply.cuh:100 takes the pointer
        #  of; the update itself does not read it, multi_tensor_adagrad.cu:26-80)
        _flag_ptr(noop_flag, ref)
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_adagrad(
                tables[0], tables[1], tables[2], sizes, n, float(lr), float(epsilon), int(mode),
                float(weight_decay), _dtype_code(ref, "grads[0]"), _stream(ref),
            )
            _check(rc, lib)


class _L2NormKernel:
    """``multi_tensor_l2norm`` of ``oslo/torch/_C/csrc/FusedL2NormBinder.cpp``,
    and ``norm_out``, the blend into stored per-tensor norms that the
    reference's NovoGrad step calls internally
    (``multi_tensor_l2norm.cu:323-385``)."""

    def __init__(self, lib):
        self._lib = lib

    def _run(self, tensors, out_global, out_per_tensor, norm_type, blend, alpha, beta, noop_flag,
             skip_if_flag=False):
        lib = self._lib
        tables, sizes, n, ref = _tensor_tables([tensors], ("tensor",))
        code = _dtype_code(ref, "tensors[0]")
        need = int(lib.oslo_multi_tensor_norm_partials(sizes, n, code))
        if need < 0:
            _check(need, lib)
        partials = torch.empty(need, dtype=torch.float32, device=ref.device)
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_norm(
                tables[0], sizes, n, code, _ptr(partials), need, _ptr(out_global),
                _ptr(out_per_tensor), int(norm_type), int(blend), float(alpha), float(beta),
                _flag_ptr(noop_flag, ref), int(bool(skip_if_flag)), _stream(ref),
            )
            _check(rc, lib)

    def multi_tensor_l2norm_mp(self, chunk_size, noop_flag, tensor_lists, per_tensor=False):
        """``multi_tensor_l2norm`` that does nothing while ``noop_flag`` is
        raised: the results then hold whatever their memory held
        (``oslo/torch/_C/csrc/FusedMixedPrecisionL2NormBinder.cpp``,
        ``multi_tensor_l2norm_mp.cu:33-35, 113-115``)."""
        if noop_flag is None:
            raise RuntimeError("multi_tensor_l2norm_mp needs the overflow flag")
        return self.multi_tensor_l2norm(chunk_size, noop_flag, tensor_lists, per_tensor,
                                        _skip_if_flag=True)

    def multi_tensor_l2norm(self, chunk_size, noop_flag, tensor_lists, per_tensor=False,
                            _skip_if_flag=False):
        """Returns ``(norm over all tensors [1], norm of each tensor [n] or an
        empty tensor)``, float32.  A sum that is not finite sets ``noop_flag``."""
        if len(tensor_lists) != 1:
            raise RuntimeError("tensor_lists must hold one list")
        tensors = tensor_lists[0]
        if len(tensors) == 0:
            raise RuntimeError("multi_tensor_l2norm: no tensors")
        dev = tensors[0].device
        ret = torch.empty(1, dtype=torch.float32, device=dev)
        ret_per_tensor = torch.empty(len(tensors) if per_tensor else 0, dtype=torch.float32,
                                     device=dev)
        self._run(tensors, ret, ret_per_tensor if per_tensor else None, 2, 0, 0.0, 0.0, noop_flag,
                  _skip_if_flag)
        return ret, ret_per_tensor

    def multi_tensor_norm_out(self, chunk_size, noop_flag, tensor_lists, out, alpha, beta,
                              norm_type):
        """``out[t] = sqrt(alpha * out[t]**2 + beta * |x_t|_2**2)`` (``norm_type``
        2) or ``alpha * out[t] + beta * max|x_t|`` (``norm_type`` 0), in place."""
        tensors = tensor_lists[0]
        if len(tensors) == 0:
            return
        _check_input(out, "out")
        if out.dtype != torch.float32 or out.numel() != len(tensors):
            raise RuntimeError("out must be float32 with one element per tensor")
        if norm_type not in (0, 2):
            raise RuntimeError("only the L2 norm (2) and the max norm (0) are supported")
        self._run(tensors, None, out, norm_type, 1, alpha, beta, noop_flag)


class _NovogradKernel:
    """``multi_tensor_novograd`` of ``oslo/torch/_C/csrc/FusedNovogradBinder.cpp``."""

    def __init__(self, lib):
        self._lib = lib

    def multi_tensor_novograd(
        self, chunk_size, noop_flag, tensor_lists, grad_norms, lr, beta1, beta2, epsilon, step,
        bias_correction, weight_decay, grad_averaging, moment_mode, norm_type,
    ):
        """``tensor_lists`` = ``[grads, params, exp_avgs]``; ``grad_norms`` holds
        one float32 per tensor and is blended with this step's gradient norms
        first, as in the reference's host function
        (``multi_tensor_novograd.cu:131-136``)."""
        lib = self._lib
        if len(tensor_lists) != 3:
            raise RuntimeError("tensor_lists must hold [grads, params, exp_avgs]")
        d = tensor_lists[0][0].dtype if len(tensor_lists[0]) else None
        tables, sizes, n, ref = _tensor_tables(tensor_lists, ("grad", "param", "exp_avg"), [d] * 3)
        if n == 0:
            return
        get_l2norm_kernel().multi_tensor_norm_out(
            chunk_size, noop_flag, [tensor_lists[0]], grad_norms, beta2, 1.0 - beta2, norm_type
        )
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_novograd(
                tables[0], tables[1], tables[2], sizes, n, _ptr(grad_norms), float(lr),
                float(beta1), float(beta2), float(epsilon), int(step), int(bias_correction),
                float(weight_decay), int(grad_averaging), int(moment_mode),
                _dtype_code(ref, "grads[0]"), _stream(ref),
            )
            _check(rc, lib)


class _LambKernel:
    """``multi_tensor_lamb`` of ``oslo/torch/_C/csrc/FusedLambBinder.cpp``."""

    def __init__(self, lib):
        self._lib = lib

    def multi_tensor_lamb(
        self, chunk_size, noop_flag, tensor_lists, lr, beta1, beta2, epsilon, step,
        bias_correction, weight_decay, grad_averaging, mode, global_grad_norm, max_grad_norm,
        use_nvlamb=False,
    ):
        """``tensor_lists`` = ``[grads, params, exp_avgs, exp_avg_sqs]``, one
        dtype; the gradients are overwritten with the update direction
        (``multi_tensor_lamb.cu:313-317``).  ``global_grad_norm`` is a float32
        tensor with the norm of all gradients."""
        lib = self._lib
        if len(tensor_lists) != 4:
            raise RuntimeError("tensor_lists must hold [grads, params, exp_avgs, exp_avg_sqs]")
        names = ("grad", "param", "exp_avg", "exp_avg_sq")
        d = tensor_lists[0][0].dtype if len(tensor_lists[0]) else None
        tables, sizes, n, ref = _tensor_tables(tensor_lists, names, [d] * 4)
        if n == 0:
            return
        _check_input(global_grad_norm, "global_grad_norm")
        if global_grad_norm.dtype != torch.float32 or global_grad_norm.numel() < 1:
            raise RuntimeError("global_grad_norm must be a float32 tensor")
        code = _dtype_code(ref, "grads[0]")
        norms = get_l2norm_kernel()
        _, param_norms = norms.multi_tensor_l2norm(chunk_size, noop_flag, [tensor_lists[1]], True)
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_lamb_stage1(
                tables[0], tables[1], tables[2], tables[3], sizes, n, float(beta1), float(beta2),
                float(epsilon), int(step), int(bias_correction), float(weight_decay),
                int(grad_averaging), int(mode), _ptr(global_grad_norm), float(max_grad_norm),
                code, _stream(ref),
            )
            _check(rc, lib)
        _, update_norms = norms.multi_tensor_l2norm(chunk_size, noop_flag, [tensor_lists[0]], True)
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_lamb_stage2(
                tables[0], tables[1], sizes, n, _ptr(param_norms), _ptr(update_norms), float(lr),
                float(weight_decay), int(bool(use_nvlamb)), code, _stream(ref),
            )
            _check(rc, lib)


def _device_scalar(t, name, dtype, ref):
    """Pointer of a one-element tensor of ``dtype`` on the device of ``ref``."""
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.numel() >= 1
            and t.device == ref.device):
        raise RuntimeError("%s must be a %s tensor on %s" % (name, dtype, ref.device))
    return t.data_ptr()


class _LambMpKernel:
    """``multi_tensor_lamb_mp`` of
    ``oslo/torch/_C/csrc/FusedMixedPrecisionLambBinder.cpp``."""

    def __init__(self, lib):
        self._lib = lib

    def multi_tensor_lamb_mp(
        self, chunk_size, noop_flag, tensor_lists, lr, beta1, beta2, epsilon, step,
        bias_correction, weight_decay, grad_averaging, mode, global_grad_norm, max_grad_norm,
        use_nvlamb, found_inf, inv_scale,
    ):
        """``tensor_lists`` = ``[grads, params, exp_avgs, exp_avg_sqs]`` of one
        dtype, or with a fifth list ``[grads, float32 master params, float32
        exp_avgs, float32 exp_avg_sqs, model params of the gradients' dtype]``
        (``multi_tensor_lamb_mp.cu:334-337``).  ``lr``, ``step`` (int32),
        ``global_grad_norm``, ``max_grad_norm`` and ``inv_scale`` are one-element
        tensors on the GPU; nothing is updated while ``noop_flag`` is raised.
        ``found_inf`` is accepted as in the reference, whose kernels do not
        read it either."""
        lib = self._lib
        if len(tensor_lists) not in (4, 5):
            raise RuntimeError("tensor_lists must hold 4 or 5 lists")
        names = ("grad", "param", "exp_avg", "exp_avg_sq", "model param")
        gd = tensor_lists[0][0].dtype if len(tensor_lists[0]) else None
        pd = tensor_lists[1][0].dtype if len(tensor_lists[1]) else None
        master = len(tensor_lists) == 5
        dts = [gd, pd, pd, pd] + ([gd] if master else [])
        tables, sizes, n, ref = _tensor_tables(tensor_lists, names, dts)
        if n == 0:
            return
        if master and pd != torch.float32:
            raise RuntimeError("with five lists the parameters and moments are float32 master values")
        if not master and pd != gd:
            raise RuntimeError("with four lists all tensors share one dtype")
        flag = _flag_ptr(noop_flag, ref)
        if flag is None:
            raise RuntimeError("multi_tensor_lamb_mp needs the overflow flag")
        gcode, pcode = _dtype_code(tensor_lists[0][0], "grads[0]"), _dtype_code(tensor_lists[1][0], "params[0]")
        norms = get_l2norm_kernel()
        _, param_norms = norms.multi_tensor_l2norm_mp(chunk_size, noop_flag, [tensor_lists[1]], True)
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_lamb_mp_stage1(
                tables[0], tables[1], tables[2], tables[3], sizes, n, float(beta1), float(beta2),
                float(epsilon), _device_scalar(step, "step", torch.int32, ref), int(bias_correction),
                float(weight_decay), int(grad_averaging), int(mode),
                _device_scalar(global_grad_norm, "global_grad_norm", torch.float32, ref),
                _device_scalar(max_grad_norm, "max_grad_norm", torch.float32, ref),
                _device_scalar(inv_scale, "inv_scale", torch.float32, ref), flag, gcode, pcode,
                _stream(ref),
            )
            _check(rc, lib)
        _, update_norms = norms.multi_tensor_l2norm_mp(chunk_size, noop_flag, [tensor_lists[0]], True)
        with _device_of(ref):
            rc = lib.oslo_multi_tensor_lamb_mp_stage2(
                tables[0], tables[1], tables[4] if master else None, sizes, n, _ptr(param_norms),
                _ptr(update_norms), _device_scalar(lr, "lr", torch.float32, ref),
                float(weight_decay), int(bool(use_nvlamb)), flag, gcode, pcode, _stream(ref),
            )
            _check(rc, lib)


_optimizer_kernels = {}


def _optimizer_kernel(cls):
    kernel = _optimizer_kernels.get(cls)
    if kernel is None:
        kernel = _optimizer_kernels[cls] = cls(load_library())
    return kernel


def get_adam_kernel():
    return _optimizer_kernel(_AdamKernel)


def get_sgd_kernel():
    return _optimizer_kernel(_SGDKernel)


def get_adagrad_kernel():
    return _optimizer_kernel(_AdagradKernel)


def get_novograd_kernel():
    return _optimizer_kernel(_NovogradKernel)


def get_l2norm_kernel():
    return _optimizer_kernel(_L2NormKernel)


def get_lamb_kernel():
    return _optimizer_kernel(_LambKernel)


def get_l2norm_mp_kernel():
    return _optimizer_kernel(_L2NormKernel)


def get_lamb_mp_kernel():
    return _optimizer_kernel(_LambMpKernel)


def get_fused_elementwise_kernel():
    global _elementwise_kernel
    if _elementwise_kernel is None:
        _elementwise_kernel = _FusedElementwiseKernel(load_library())
    return _elementwise_kernel
