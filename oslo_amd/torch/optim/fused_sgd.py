"""FusedSGD: SGD with momentum, all parameters of a group updated by one (or a
few) multi-tensor kernel launches.

Constructor, defaults and update rule follow ``oslo/torch/optim/fused_sgd.py:8-295``
of the reference (drop-in for ``torch.optim.SGD``: ``v = rho v + g``,
``p = p - lr v``, ``:64-85``).  Differences: bfloat16 parameters are accepted
next to float16 / float32; a parameter that joins a group after the first step
gets its momentum buffer initialised on its own first step (the reference
derives ``first_run`` from the last parameter it looked at, ``:133-149``); the
branch for apex amp's master-weight stash (``:168-245``) has no counterpart, as
apex amp is not part of this package -- the kernel's four-list form (16-bit
model copies of float32 master weights) is reachable through
``oslo_amd.torch._C.get_sgd_kernel()``.
"""
import torch

from oslo_amd.torch._C import get_sgd_kernel
from oslo_amd.torch.optim._common import ZeroGradMixin, checked_params, multi_tensor_applier


class FusedSGD(ZeroGradMixin, torch.optim.Optimizer):
    """Implements stochastic gradient descent (optionally with momentum) on the GPU.

    Args:
        params (iterable): iterable of parameters to optimize or dicts defining
            parameter groups
        lr (float): learning rate
        momentum (float, optional): momentum factor (default: 0)
        weight_decay (float, optional): weight decay (L2 penalty) (default: 0)
        dampening (float, optional): dampening for momentum (default: 0)
        nesterov (bool, optional): enables Nesterov momentum (default: False)
        wd_after_momentum (bool, optional): apply the weight decay after the
            momentum step instead of before (default: False)
        set_grad_none (bool, optional): ``zero_grad()`` sets the gradients to
            None (default: False)
    """

    def __init__(
        self,
        params,
        lr=1e-3,
        momentum=0,
        dampening=0,
        weight_decay=0,
        nesterov=False,
        wd_after_momentum=False,
        materialize_master_grads=True,
        set_grad_none=False,
    ):
        if lr < 0.0:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        if weight_decay < 0.0:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        defaults = dict(
            lr=lr,
            momentum=momentum,
            dampening=dampening,
            weight_decay=weight_decay,
            nesterov=nesterov,
        )
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        super(FusedSGD, self).__init__(params, defaults)
        self.wd_after_momentum = wd_after_momentum
        self.materialize_master_grads = materialize_master_grads
        self.most_recent_scale = 1.0
        self.scale_set_by_backward = False
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None
        self.multi_tensor_sgd = None

    def __setstate__(self, state):
        super(FusedSGD, self).__setstate__(state)
        for group in self.param_groups:
            group.setdefault("nesterov", False)

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
        if self.multi_tensor_sgd is None:
            self.multi_tensor_sgd = get_sgd_kernel().multi_tensor_sgd

        for group in self.param_groups:
            # one launch set per (dtype, device, first run or not)
            buckets = {}
            use_momentum = group["momentum"] != 0
            for p in checked_params(group, "FusedSGD"):
                state = self.state[p]
                first_run = use_momentum and "momentum_buffer" not in state
                if first_run:
                    state["momentum_buffer"] = torch.zeros_like(
                        p.data, memory_format=torch.contiguous_format
                    )
                g, w, m = buckets.setdefault((p.dtype, p.device, first_run), ([], [], []))
                g.append(p.grad.data.contiguous())
                w.append(p.data)
                # without momentum the kernel neither reads nor writes the third
                # list: the weight stands in, and no buffer is allocated (the
                # reference allocates one per parameter regardless, :133-149)
                m.append(state["momentum_buffer"] if use_momentum else p.data)
            for (_, _, first_run), lists in buckets.items():
                multi_tensor_applier(
                    self.multi_tensor_sgd,
                    self._dummy_overflow_buf,
                    list(lists),
                    group["weight_decay"],
                    group["momentum"],
                    group["dampening"],
                    group["lr"],
                    group["nesterov"],
                    first_run,
                    self.wd_after_momentum,
                    1.0 / self.most_recent_scale,
                )
        self.most_recent_scale = 1.0
        self.scale_set_by_backward = False
        return loss
