"""What the fused optimizers share: the applier, the per-dtype buckets and the
``zero_grad`` of the reference's classes."""
import torch

from oslo_amd.torch.utils.multi_tensor_apply import multi_tensor_applier  # noqa: F401  (re-exported)

KERNEL_DTYPES = (torch.float16, torch.bfloat16, torch.float32)


def checked_params(group, name):
    """The parameters of ``group`` that have a gradient, after the checks every
    fused optimizer makes (dense gradient, GPU tensor, a dtype with a kernel,
    contiguous storage)."""
    for p in group["params"]:
        if p.grad is None:
            continue
        if p.grad.data.is_sparse:
            raise RuntimeError("%s does not support sparse gradients" % name)
        if not p.is_cuda:
            raise RuntimeError("%s is GPU-only: parameter on %s" % (name, p.device))
        if p.dtype not in KERNEL_DTYPES:
            raise RuntimeError("%s only support fp16, bf16 and fp32." % name)
        if not p.data.is_contiguous():
            raise RuntimeError("%s needs contiguous parameters" % name)
        yield p


class ZeroGradMixin:
    """``zero_grad`` that drops the gradients when ``set_grad_none`` is set
    (``oslo/torch/optim/fused_sgd.py:125-131`` and its siblings)."""

    def zero_grad(self, set_to_none=None):
        if self.set_grad_none if set_to_none is None else set_to_none:
            for group in self.param_groups:
                for p in group["params"]:
                    p.grad = None
        else:
            super().zero_grad(set_to_none=False)
