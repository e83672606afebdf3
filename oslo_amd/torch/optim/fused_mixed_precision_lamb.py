"""FusedMixedPrecisionLamb: LAMB whose whole step stays on the GPU.

Behaviour of ``oslo/torch/optim/fused_mixed_precision_lamb.py`` of the
reference (kernels ``multi_tensor_lamb_mp`` / ``multi_tensor_l2norm_mp``),
written from what that optimizer does rather than from how it is laid out:

* the learning rate and the step count of every parameter group are tensors
  on the parameters' device, so a step reads nothing back to the host and can
  be captured in a graph;
* with ``reduced_precision_dtype`` set, a parameter of that dtype is stepped
  through a float32 master copy with float32 moments (made on the first step:
  a data-parallel wrapper may still broadcast the model after the optimizer
  was built), and the model's parameter is the master rounded to its dtype;
* the loss scale comes from a ``torch.amp.GradScaler``, either passed to
  ``step`` or handed over as the ``found_inf`` / ``grad_scale`` attributes
  torch sets: the gradients are unscaled inside the kernel, the clip threshold
  is compared with the norm of the *scaled* gradients, and while the overflow
  flag is raised nothing changes and the step count stands still;
* the state dict keeps the moments in the dtype they have (float32 next to
  16-bit parameters); loading does not cast them to the parameters' dtype.
"""
import torch

from oslo_amd.torch._C import get_l2norm_mp_kernel, get_lamb_mp_kernel
from oslo_amd.torch.optim._common import KERNEL_DTYPES, multi_tensor_applier

_NAME = "FusedMixedPrecisionLamb"


class FusedMixedPrecisionLamb(torch.optim.Optimizer):
    def __init__(
        self,
        params,
        lr=1e-3,
        step=0,
        bias_correction=True,
        betas=(0.9, 0.999),
        eps=1e-6,
        weight_decay=0.01,
        amsgrad=False,
        adam_w_mode=True,
        grad_averaging=True,
        max_grad_norm=1.0,
        use_nvlamb=False,
        reduced_precision_dtype=None,
    ):
        if amsgrad:
            raise RuntimeError("FusedLAMB does not support the AMSGrad variant.")
        super().__init__(params, {
            "lr": torch.tensor(lr, dtype=torch.float32),
            "step": torch.tensor([step], dtype=torch.int),
            "bias_correction": bias_correction,
            "betas": betas,
            "eps": eps,
            "weight_decay": weight_decay,
            "grad_averaging": grad_averaging,
            "max_grad_norm": max_grad_norm,
        })
        self._device = self.param_groups[0]["params"][0].device
        for group in self.param_groups:
            self._scalars_to_device(group)
        self.adam_w_mode = int(bool(adam_w_mode))
        self.use_nvlamb = use_nvlamb
        self.reduced_precision_dtype = reduced_precision_dtype
        self._step_supports_amp_scaling = True  # GradScaler: do not unscale, hand the scale over
        self._overflow = torch.zeros(1, dtype=torch.int, device=self._device)
        self._masters = {}      # parameter -> float32 master copy
        self._kernels = None

    # -- parameter groups ----------------------------------------------------
    def _scalars_to_device(self, group):
        for name in ("lr", "step"):
            if isinstance(group[name], torch.Tensor):
                # (a copy per group: groups must not share one tensor)
                group[name] = group[name].detach().clone().to(self._device)

    def add_param_group(self, param_group):
        super().add_param_group(param_group)
        if hasattr(self, "_device"):
            self._scalars_to_device(self.param_groups[-1])

    @property
    def param_groups_full_precision(self):
        """The float32 master copies, laid out like ``param_groups`` (None
        where a parameter has none, which is everywhere before the first step)."""
        return [{"params": [self._masters.get(p) for p in g["params"]]} for g in self.param_groups]

    def _wants_master(self, p):
        return self.reduced_precision_dtype is not None and p.dtype == self.reduced_precision_dtype

    # -- state dict ----------------------------------------------------------
    def load_state_dict(self, state_dict):
        """As the base class, except that the moments keep the dtype they were
        saved in: the base class casts floating-point state to its
        parameter's dtype, which would round float32 moments of 16-bit
        parameters."""
        saved_ids = [i for g in state_dict["param_groups"] for i in g["params"]]
        super().load_state_dict(state_dict)
        own = [p for g in self.param_groups for p in g["params"]]
        if len(own) != len(saved_ids):
            return
        for p, i in zip(own, saved_ids):
            saved = state_dict["state"].get(i)
            if not saved:
                continue
            for key, value in saved.items():
                if isinstance(value, torch.Tensor) and value.is_floating_point() \
                        and self.state[p][key].dtype != value.dtype:
                    self.state[p][key] = value.detach().clone().to(p.device)
        for group in self.param_groups:
            self._scalars_to_device(group)

    # -- one step --------------------------------------------------------------
    def _loss_scale(self, grad_scaler):
        """(overflow flag, scale, 1 / scale) as float tensors of one element on
        the device; without a scaler the gradients count as unscaled."""
        dev = self._device
        if grad_scaler is not None:
            found_inf = grad_scaler._check_inf_per_device(self)[dev]
            scale = grad_scaler._get_scale_async()
        else:
            found_inf = getattr(self, "found_inf", None)
            scale = getattr(self, "grad_scale", None) if found_inf is not None else None
        if found_inf is None:
            return torch.zeros(1, device=dev), torch.ones(1, device=dev), torch.ones(1, device=dev)
        found_inf = found_inf.reshape(1).float()
        scale = torch.ones(1, device=dev) if scale is None else scale.reshape(1).float()
        # (the reciprocal in double: float 1/1024 and the like are exact either way,
        #  odd scales are not)
        return found_inf, scale, scale.double().reciprocal().float()

    def _operands(self, group):
        """The tensor lists of one group for the kernel: gradients, the
        weights that are stepped, both moments and, with master copies, the
        model's weights to refresh."""
        with_master = self.reduced_precision_dtype is not None
        grads, weights, avg, avg_sq, model = [], [], [], [], []
        dtype0 = group["params"][0].dtype
        for p in group["params"]:
            if p.dtype != dtype0:
                raise RuntimeError(
                    "Error: Parameters are not of the identical type: {} != {}".format(dtype0, p.dtype))
            if p.grad is None:
                continue
            if p.grad.is_sparse:
                raise RuntimeError("%s does not support sparse gradients" % _NAME)
            if not p.is_cuda or p.dtype not in KERNEL_DTYPES:
                raise RuntimeError("%s needs fp16, bf16 or fp32 parameters on the GPU" % _NAME)
            if not p.grad.is_contiguous():
                # the kernel leaves the update direction in the gradient; a copy would hide it
                raise RuntimeError("%s needs contiguous gradients" % _NAME)
            if with_master and not self._wants_master(p):
                raise RuntimeError(
                    "%s: with reduced_precision_dtype=%s every parameter must have that dtype, got %s"
                    % (_NAME, self.reduced_precision_dtype, p.dtype))
            stepped = p.data
            if with_master:
                stepped = self._masters.get(p)
                if stepped is None:
                    stepped = self._masters[p] = p.detach().clone().float()
                model.append(p.data)
            state = self.state[p]
            if not state:
                for key in ("exp_avg", "exp_avg_sq"):
                    state[key] = torch.zeros_like(stepped, memory_format=torch.contiguous_format)
            grads.append(p.grad.data)
            weights.append(stepped)
            avg.append(state["exp_avg"])
            avg_sq.append(state["exp_avg_sq"])
        lists = [grads, weights, avg, avg_sq]
        if with_master:
            lists.append(model)
        return lists

    @torch.no_grad()
    def step(self, closure=None, grad_scaler=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if self._kernels is None:
            self._kernels = (get_l2norm_mp_kernel().multi_tensor_l2norm_mp,
                             get_lamb_mp_kernel().multi_tensor_lamb_mp)
        l2norm, lamb = self._kernels

        per_group = [self._operands(group) for group in self.param_groups]
        all_grads = [g for lists in per_group for g in lists[0]]
        if not all_grads:
            return loss
        if len({g.dtype for g in all_grads}) != 1:
            raise RuntimeError("%s needs gradients of one dtype" % _NAME)

        found_inf, scale, inv_scale = self._loss_scale(grad_scaler)
        self._overflow.copy_(found_inf)
        # one norm over every gradient of the model, taken of the gradients as they
        # are (still scaled): the clip threshold is scaled to match
        grad_norm = multi_tensor_applier(l2norm, self._overflow, [all_grads], False)[0]
        clip_at = (self.defaults["max_grad_norm"] * scale).float().reshape(1)
        advance = (self._overflow != 1).to(torch.int)  # 0 while the flag is raised

        for group, lists in zip(self.param_groups, per_group):
            group["step"] += advance
            if not lists[0]:
                continue
            beta1, beta2 = group["betas"]
            multi_tensor_applier(
                lamb, self._overflow, lists, group["lr"], beta1, beta2, group["eps"], group["step"],
                int(bool(group["bias_correction"])), group["weight_decay"],
                int(bool(group["grad_averaging"])), self.adam_w_mode, grad_norm, clip_at,
                self.use_nvlamb, found_inf, inv_scale,
            )
        return loss
