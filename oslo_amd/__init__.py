"""oslo_amd: MI355X (gfx950) kernels for the fused non-GEMM chain of a
transformer layer behind the ``oslo.torch.nn`` API
(``import oslo_amd.torch.nn as onn``)."""
__version__ = "0.1.0"
