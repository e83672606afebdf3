"""The launch-shape overrides of the norm kernels (oslo_tune) change how a row
is split over lanes, waves and workgroups, never the result: every override
runs LayerNorm and RMSNorm forward and backward, plain and fused with
bias-dropout-add, against the float64 oracle with the tolerances of the default
launch shapes."""
import pytest
import torch

from oslo_amd.torch import _C
from test_gpu_norm import test_layer_norm as check_layer_norm
from test_gpu_norm import test_rms_norm as check_rms_norm
from test_gpu_residual_norm import test_fused_vs_oracle as check_fused

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

KEYS = [
    "norm_fwd_vpl", "norm_fwd_waves", "norm_fwd_iters", "norm_bwd_vpl", "norm_bwd_prefetch",
    "norm_bwd_waves", "norm_bwd_blocks_per_cu", "norm_lanes_per_row",
]

OVERRIDES = [
    ("norm_fwd_vpl", 1), ("norm_fwd_vpl", 2), ("norm_fwd_vpl", 3), ("norm_fwd_vpl", 4), ("norm_fwd_vpl", 8),
    ("norm_fwd_waves", 8), ("norm_fwd_waves", 16),
    ("norm_fwd_iters", 1), ("norm_fwd_iters", 4),
    ("norm_bwd_vpl", 1), ("norm_bwd_vpl", 2),
    ("norm_bwd_prefetch", 1), ("norm_bwd_prefetch", 2),
    ("norm_bwd_waves", 4), ("norm_bwd_waves", 8),
    ("norm_bwd_blocks_per_cu", 2),
    ("norm_lanes_per_row", 64), ("norm_lanes_per_row", 32),
]

# (n1, n2, input dtype, output dtype)
SHAPES = [
    (300, 128, BF16, BF16),    # short rows, side by side in a wave by default
    (37, 1024, BF16, BF16),
    (33, 2000, F16, F16),      # 250 chunks: lanes past the end of the row
    (19, 4096, BF16, BF16),
    (9, 6144, F16, F16),
    (5, 16384, BF16, BF16),
    (21, 2048, F32, F32),
    (11, 4096, F32, BF16),
]


@pytest.fixture
def tuned():
    yield
    for key in KEYS:
        _C.tune(key, 0)


@pytest.mark.parametrize("key,value", OVERRIDES)
@pytest.mark.parametrize("n1,n2,tin,tout", SHAPES)
def test_override_keeps_the_result(device, tuned, n1, n2, tin, tout, key, value):
    _C.tune(key, value)
    check_layer_norm(device, n1, n2, tin, tout, True)
    check_rms_norm(device, n1, n2, tin, tout, True)
    if tin == tout:  # the bias-dropout-add prologue / epilogue builds (LayerNorm or RMSNorm by shape)
        check_fused(device, n1, n2, tin, 0.1, n1 % 2 == 0)
