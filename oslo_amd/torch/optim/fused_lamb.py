"""FusedLamb: LAMB with all parameters of a group updated by a few multi-tensor
launches (``multi_tensor_lamb``, ``oslo/torch/_C/csrc/multi_tensor_lamb.cu``).

The reference's ``oslo/torch/optim/fused_lamb.py`` cannot run against the kernel
module it ships: its ``step`` calls ``fused_lamb_cuda.lamb(...)`` per tensor
(``:168-185``), a function that ``FusedLambBinder.cpp`` does not export (it
exports ``multi_tensor_lamb`` only).  This class therefore drives the kernel the
reference does ship, the way that kernel's host function defines the step
(``multi_tensor_lamb.cu:285-352``): the gradients of all groups are clipped by
their global L2 norm against ``max_grad_norm``, every tensor takes an Adam-style
update direction, and tensors under weight decay (all tensors with
``use_nvlamb``) scale their step by ``|p| / |update|``.  The constructor keeps
the reference's arguments that the kernel has a meaning for (``lr``,
``bias_correction``, ``betas``, ``eps``, ``weight_decay``, ``max_grad_norm``,
``amsgrad``); ``eps_inside_sqrt``, ``max_coeff`` and ``min_coeff`` belong to the
per-tensor kernel the reference lacks and are refused when set.
"""
import torch

from oslo_amd.torch._C import get_l2norm_kernel, get_lamb_kernel
from oslo_amd.torch.optim._common import ZeroGradMixin, checked_params, multi_tensor_applier


class FusedLamb(ZeroGradMixin, torch.optim.Optimizer):
    """Implements the LAMB algorithm on the GPU.

    ``step()`` leaves the update direction in each parameter's ``.grad`` (the
    kernel works in place, ``multi_tensor_lamb.cu:313-317``): read the gradients
    before the step, not after.

    Arguments:
        params (iterable): iterable of parameters to optimize or dicts defining
            parameter groups.
        lr (float, optional): learning rate. (default: 1e-3)
        bias_correction (bool, optional): bias correction (default: True)
        betas (Tuple[float, float], optional): coefficients used for computing
            running averages of gradient and its square. (default: (0.9, 0.999))
        eps (float, optional): term added to the denominator to improve
            numerical stability. (default: 1e-8)
        weight_decay (float, optional): weight decay (default: 0)
        max_grad_norm (float, optional): value used to clip the global gradient
            norm; 0 switches clipping off (default: 0.0)
        amsgrad (boolean, optional): NOT SUPPORTED.
        adam_w_mode (boolean, optional): True for decoupled weight decay, False
            for L2 regularization (default: True)
        grad_averaging (bool, optional): whether to apply (1 - beta1) to the
            gradient in its running average. (default: True)
        use_nvlamb (boolean, optional): apply the adaptive learning rate to
            tensors without weight decay as well (default: False)
        set_grad_none (bool, optional): ``zero_grad()`` sets the gradients to
            None. (default: True)
    """

    def __init__(
        self,
        params,
        lr=1e-3,
        bias_correction=True,
        betas=(0.9, 0.999),
        eps=1e-8,
        eps_inside_sqrt=False,
        weight_decay=0.0,
        max_grad_norm=0.0,
        max_coeff=10.0,
        min_coeff=0.01,
        amsgrad=False,
        adam_w_mode=True,
        grad_averaging=True,
        use_nvlamb=False,
        set_grad_none=True,
    ):
        if amsgrad:
            raise RuntimeError("FusedLamb does not support the AMSGrad variant.")
        if eps_inside_sqrt or max_coeff != 10.0 or min_coeff != 0.01:
            raise RuntimeError(
                "FusedLamb: eps_inside_sqrt, max_coeff and min_coeff have no meaning for the "
                "multi-tensor LAMB kernel (the trust ratio is not clamped)."
            )
        defaults = dict(
            lr=lr,
            bias_correction=bias_correction,
            betas=betas,
            eps=eps,
            weight_decay=weight_decay,
            grad_averaging=grad_averaging,
            max_grad_norm=max_grad_norm,
        )
        super(FusedLamb, self).__init__(params, defaults)
        self.adam_w_mode = 1 if adam_w_mode else 0
        self.use_nvlamb = use_nvlamb
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None
        self.multi_tensor_lamb = None

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
        if self.multi_tensor_lamb is None:
            self.multi_tensor_lamb = get_lamb_kernel().multi_tensor_lamb

        # the norm of all gradients, blended over the dtype buckets
        per_group = []
        by_bucket = {}
        for group in self.param_groups:
            buckets = {}
            for p in checked_params(group, "FusedLamb"):
                state = self.state[p]
                if len(state) == 0:
                    state["exp_avg"] = torch.zeros_like(p.data, memory_format=torch.contiguous_format)
                    state["exp_avg_sq"] = torch.zeros_like(p.data, memory_format=torch.contiguous_format)
                g, pd, m, v = buckets.setdefault((p.dtype, p.device), ([], [], [], []))
                g.append(p.grad.data.contiguous())
                pd.append(p.data)
                m.append(state["exp_avg"])
                v.append(state["exp_avg_sq"])
                by_bucket.setdefault((p.dtype, p.device), []).append(g[-1])
            per_group.append(buckets)
        if not by_bucket:
            return loss
        devices = {key[1] for key in by_bucket}
        if len(devices) != 1:
            raise RuntimeError("FusedLamb needs all parameters on one device")
        norms = [
            get_l2norm_kernel().multi_tensor_l2norm(0, self._dummy_overflow_buf, [grads], False)[0]
            for grads in by_bucket.values()
        ]
        global_grad_norm = norms[0] if len(norms) == 1 else torch.linalg.vector_norm(torch.cat(norms)).view(1)

        for group, buckets in zip(self.param_groups, per_group):
            if not buckets:
                continue
            bias_correction = 1 if group["bias_correction"] else 0
            beta1, beta2 = group["betas"]
            grad_averaging = 1 if group["grad_averaging"] else 0
            group["step"] = group.get("step", 0) + 1
            # the kernel clips when the norm exceeds the threshold; no threshold = none
            max_grad_norm = group["max_grad_norm"] if group["max_grad_norm"] > 0 else float("inf")
            for lists in buckets.values():
                # the kernel overwrites the gradients with the update direction
                multi_tensor_applier(
                    self.multi_tensor_lamb,
                    self._dummy_overflow_buf,
                    list(lists),
                    group["lr"],
                    beta1,
                    beta2,
                    group["eps"],
                    group["step"],
                    bias_correction,
                    group["weight_decay"],
                    grad_averaging,
                    self.adam_w_mode,
                    global_grad_norm,
                    max_grad_norm,
                    self.use_nvlamb,
                )
        return loss
