"""FusedAdagrad: Adagrad with all parameters of a group updated by one (or a
few) multi-tensor kernel launches.

Constructor, defaults and update rule follow
``oslo/torch/optim/fused_adagrad.py:7-133`` of the reference; bfloat16
parameters are accepted next to float16 / float32.
"""
import torch

from oslo_amd.torch._C import get_adagrad_kernel
from oslo_amd.torch.optim._common import ZeroGradMixin, checked_params, multi_tensor_applier


class FusedAdagrad(ZeroGradMixin, torch.optim.Optimizer):
    """Implements the Adagrad algorithm on the GPU.

    Arguments:
        params (iterable): iterable of parameters to optimize or dicts defining
            parameter groups
        lr (float, optional): learning rate (default: 1e-3)
        eps (float, optional): term added to the denominator to improve
            numerical stability (default: 1e-10)
        weight_decay (float, optional): weight decay (default: 0)
        set_grad_none (bool, optional): ``zero_grad()`` sets the gradients to
            None (default: True)
        adagrad_w_mode (boolean, optional): True for decoupled weight decay,
            False for L2 regularization (default: False)
    """

    def __init__(
        self,
        params,
        lr=1e-3,
        eps=1e-10,
        weight_decay=0.0,
        set_grad_none=True,
        adagrad_w_mode=False,
    ):
        defaults = dict(lr=lr, eps=eps, weight_decay=weight_decay)
        super(FusedAdagrad, self).__init__(params, defaults)
        self.adagrad_w_mode = 1 if adagrad_w_mode else 0
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None
        self.multi_tensor_adagrad = None

    def step(self, closure=None):
        """Performs a single optimization step.

        Arguments:
            closure (callable, optional): A closure that reevaluates the model
                and returns the loss.
        """
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if self.multi_tensor_adagrad is None:
            self.multi_tensor_adagrad = get_adagrad_kernel().multi_tensor_adagrad

        for group in self.param_groups:
            buckets = {}
            for p in checked_params(group, "FusedAdagrad"):
                state = self.state[p]
                if len(state) == 0:
                    # running sum of squared gradients
                    state["sum"] = torch.zeros_like(p.data, memory_format=torch.contiguous_format)
                g, pd, h = buckets.setdefault((p.dtype, p.device), ([], [], []))
                g.append(p.grad.data.contiguous())
                pd.append(p.data)
                h.append(state["sum"])
            for lists in buckets.values():
                multi_tensor_applier(
                    self.multi_tensor_adagrad,
                    self._dummy_overflow_buf,
                    list(lists),
                    group["lr"],
                    group["eps"],
                    self.adagrad_w_mode,
                    group["weight_decay"],
                )
        return loss
