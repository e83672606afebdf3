"""FusedNovograd: NovoGrad (a first moment per element, a second moment per
tensor) with all parameters of a group updated by a few multi-tensor launches.

Constructor, defaults and update rule follow
``oslo/torch/optim/fused_novograd.py:7-264`` of the reference.  Differences:
bfloat16 parameters are accepted next to float16 / float32; the per-tensor norms
of a group are kept per (dtype, device) bucket under the same
``group["exp_avg_sq"]`` key (the reference keeps a two-element list, float16
then float32, ``:172-226``); the norms of the first step come from the
multi-tensor norm kernel instead of one ``.item()`` per tensor (``:188-204``).
"""
import torch

from oslo_amd.torch._C import get_l2norm_kernel, get_novograd_kernel
from oslo_amd.torch.optim._common import ZeroGradMixin, checked_params, multi_tensor_applier


def _bucket_name(dtype):
    """Key of a dtype's norms in ``group["exp_avg_sq"]``: a plain string, so
    that a state dict holds nothing tied to a device index."""
    return str(dtype).split(".")[-1]


class FusedNovograd(ZeroGradMixin, torch.optim.Optimizer):
    """Implements the NovoGrad algorithm on the GPU.

    Arguments:
        params (iterable): iterable of parameters to optimize or dicts defining
            parameter groups.
        lr (float, optional): learning rate. (default: 1e-3)
        bias_correction (bool, optional): divide the moments by their bias
            corrections. (default: True)
        betas (Tuple[float, float], optional): coefficients used for computing
            running averages of gradient and its norm. (default: (0.9, 0.999))
        eps (float, optional): term added to the denominator to improve
            numerical stability. (default: 1e-8)
        weight_decay (float, optional): weight decay (L2 penalty) (default: 0)
        amsgrad (boolean, optional): NOT SUPPORTED.
        reg_inside_moment (bool, optional): whether to do the regularization
            (norm and L2) inside the momentum calculation instead of on the
            update term only. (default: False)
        grad_averaging (bool, optional): whether to apply (1 - beta1) to the
            gradient in its running average. (default: True)
        norm_type (int, optional): norm calculated for each layer, 2 for the L2
            norm and 0 for the infinity norm. (default: 2)
        init_zero (bool, optional): whether to start the norm at 0 (averaging
            starts on the first step) or at the first step's norm (averaging
            starts on the second step). (default: False)
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
        weight_decay=0.0,
        amsgrad=False,
        reg_inside_moment=False,
        grad_averaging=True,
        norm_type=2,
        init_zero=False,
        set_grad_none=True,
    ):
        if amsgrad:
            raise RuntimeError("FusedNovograd does not support the AMSGrad variant.")
        if norm_type not in (0, 2):
            raise RuntimeError("FusedNovograd only support l2/inf norm now.")
        defaults = dict(
            lr=lr,
            bias_correction=bias_correction,
            betas=betas,
            eps=eps,
            weight_decay=weight_decay,
            grad_averaging=grad_averaging,
            norm_type=norm_type,
            init_zero=init_zero,
        )
        super(FusedNovograd, self).__init__(params, defaults)
        self.moment_mode = 0 if reg_inside_moment else 1
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None
        self.multi_tensor_novograd = None

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
        if self.multi_tensor_novograd is None:
            self.multi_tensor_novograd = get_novograd_kernel().multi_tensor_novograd

        for group in self.param_groups:
            bias_correction = 1 if group["bias_correction"] else 0
            beta1, beta2 = group["betas"]
            grad_averaging = 1 if group["grad_averaging"] else 0
            # one step count per group (fused_novograd.py:147-152)
            group["step"] = group.get("step", 0) + 1

            buckets = {}
            device = None
            for p in checked_params(group, "FusedNovograd"):
                if device is None:
                    device = p.device
                elif p.device != device:
                    raise RuntimeError("FusedNovograd: the parameters of a group must live on one device")
                state = self.state[p]
                if len(state) == 0:
                    state["exp_avg"] = torch.zeros_like(p.data, memory_format=torch.contiguous_format)
                g, pd, m = buckets.setdefault(_bucket_name(p.dtype), ([], [], []))
                g.append(p.grad.data.contiguous())
                pd.append(p.data)
                m.append(state["exp_avg"])

            # one norm per tensor (the norm, not its square, so that both norm
            # types blend the same way), kept per dtype in the parameter group,
            # in the order of the parameters that have a gradient
            norms = group.get("exp_avg_sq")
            if isinstance(norms, (list, tuple)):
                # a state dict of the reference: [norms of the 16-bit tensors,
                # norms of the float32 tensors] (fused_novograd.py:172-226)
                norms = {
                    name: norms[1 if name == "float32" else 0].to(device=device, dtype=torch.float32)
                    for name in buckets
                    if len(norms) > (1 if name == "float32" else 0)
                    and norms[1 if name == "float32" else 0].numel() > 0
                }
            if norms is None:
                norms = {}
            group["exp_avg_sq"] = norms
            for key, (g, pd, m) in buckets.items():
                if key not in norms:
                    if group["init_zero"]:
                        norms[key] = torch.zeros(len(g), dtype=torch.float32, device=device)
                    else:
                        # the first step's own norm: the first blend changes nothing
                        norms[key] = torch.zeros(len(g), dtype=torch.float32, device=device)
                        get_l2norm_kernel().multi_tensor_norm_out(
                            0, None, [g], norms[key], 0.0, 1.0, group["norm_type"]
                        )
                elif norms[key].device != device:
                    norms[key] = norms[key].to(device)
                elif norms[key].numel() != len(g):
                    raise RuntimeError(
                        "FusedNovograd: the set of parameters with gradients changed between steps"
                    )
                multi_tensor_applier(
                    self.multi_tensor_novograd,
                    self._dummy_overflow_buf,
                    [g, pd, m],
                    norms[key],
                    group["lr"],
                    beta1,
                    beta2,
                    group["eps"],
                    group["step"],
                    bias_correction,
                    group["weight_decay"],
                    grad_averaging,
                    self.moment_mode,
                    group["norm_type"],
                )
        return loss
