"""FusedAdam: Adam / AdamW with all parameters of a group updated by one (or a
few) multi-tensor kernel launches.

Constructor, defaults and error behaviour follow
``oslo/torch/optim/fused_adam.py:17-184`` of the reference.  Differences: the
parameters may be bfloat16 as well as float16 / float32, and the step count is
kept per parameter group and advances once per ``step()`` (the reference keeps
it in the state of the last parameter it visited and advances it once per
dtype bucket, ``:150-182``, which double-counts a group that mixes dtypes).
"""
import torch

from oslo_amd.torch._C import get_adam_kernel
from oslo_amd.torch.utils.multi_tensor_apply import multi_tensor_applier


class FusedAdam(torch.optim.Optimizer):
    """Implements the Adam algorithm on the GPU.

    Arguments:
        params (iterable): iterable of parameters to optimize or dicts defining
            parameter groups.
        lr (float, optional): learning rate. (default: 1e-3)
        bias_correction (bool, optional): divide the moments by ``1 - beta^step``.
            (default: True)
        betas (Tuple[float, float], optional): coefficients used for computing
            running averages of gradient and its square. (default: (0.9, 0.999))
        eps (float, optional): term added to the denominator to improve
            numerical stability. (default: 1e-8)
        adam_w_mode (boolean, optional): True for decoupled weight decay (AdamW),
            False for L2 regularization. (default: True)
        weight_decay (float, optional): weight decay (default: 0)
        amsgrad (boolean, optional): NOT SUPPORTED.
        set_grad_none (bool, optional): whether ``zero_grad()`` sets the
            gradients to None. (default: True)
    """

    def __init__(
        self,
        params,
        lr=1e-3,
        bias_correction=True,
        betas=(0.9, 0.999),
        eps=1e-8,
        adam_w_mode=True,
        weight_decay=0.0,
        amsgrad=False,
        set_grad_none=True,
    ):
        if amsgrad:
            raise RuntimeError("FusedAdam does not support the AMSGrad variant.")
        defaults = dict(
            lr=lr,
            bias_correction=bias_correction,
            betas=betas,
            eps=eps,
            weight_decay=weight_decay,
        )
        super(FusedAdam, self).__init__(params, defaults)
        self.adam_w_mode = 1 if adam_w_mode else 0
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None
        self.multi_tensor_adam = None

    def zero_grad(self, set_to_none=None):
        if self.set_grad_none if set_to_none is None else set_to_none:
            for group in self.param_groups:
                for p in group["params"]:
                    p.grad = None
        else:
            super(FusedAdam, self).zero_grad(set_to_none=False)

    def step(self, closure=None, grads=None, output_params=None, scale=None, grad_norms=None):
        """Performs a single optimization step.

        Arguments:
            closure (callable, optional): A closure that reevaluates the model
                and returns the loss.

        The remaining arguments are deprecated, and are only retained for
        error-checking purposes.
        """
        if any(p is not None for p in [grads, output_params, scale, grad_norms]):
            raise RuntimeError(
                "FusedAdam has been updated.  Simply initialize it identically to "
                "torch.optim.Adam, and call step() with no arguments."
            )
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        if self.multi_tensor_adam is None:
            self.multi_tensor_adam = get_adam_kernel().multi_tensor_adam

        for group in self.param_groups:
            bias_correction = 1 if group["bias_correction"] else 0
            beta1, beta2 = group["betas"]
            buckets = {}
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.data.is_sparse:
                    raise RuntimeError(
                        "FusedAdam does not support sparse gradients, please consider "
                        "SparseAdam instead"
                    )
                if not p.is_cuda:
                    raise RuntimeError("FusedAdam is GPU-only: parameter on %s" % p.device)
                if p.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                    raise RuntimeError("FusedAdam only support fp16, bf16 and fp32.")
                state = self.state[p]
                if len(state) == 0:
                    state["exp_avg"] = torch.zeros_like(p.data, memory_format=torch.contiguous_format)
                    state["exp_avg_sq"] = torch.zeros_like(p.data, memory_format=torch.contiguous_format)
                if not p.data.is_contiguous():
                    raise RuntimeError("FusedAdam needs contiguous parameters")
                g, pd, m, v = buckets.setdefault((p.dtype, p.device), ([], [], [], []))
                g.append(p.grad.data.contiguous())
                pd.append(p.data)
                m.append(state["exp_avg"])
                v.append(state["exp_avg_sq"])
            if not buckets:
                continue
            group["step"] = group.get("step", 0) + 1
            for lists in buckets.values():
                multi_tensor_applier(
                    self.multi_tensor_adam,
                    self._dummy_overflow_buf,
                    list(lists),
                    group["lr"],
                    beta1,
                    beta2,
                    group["eps"],
                    group["step"],
                    self.adam_w_mode,
                    bias_correction,
                    group["weight_decay"],
                )
        return loss
