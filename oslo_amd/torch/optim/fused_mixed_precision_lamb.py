"""FusedMixedPrecisionLamb: LAMB whose step needs no host synchronisation --
learning rate, step count, clip threshold and loss scale live on the GPU -- and
which can keep float32 master copies of reduced-precision parameters.

Constructor, state and step follow
``oslo/torch/optim/fused_mixed_precision_lamb.py:11-288`` of the reference
(kernels: ``multi_tensor_lamb_mp``, ``multi_tensor_l2norm_mp``).  With
``reduced_precision_dtype`` set, parameters of that dtype get a float32 master
copy and float32 moments on the first step; the kernel updates the master copy
and writes the model's parameter from it.  A ``torch.amp.GradScaler`` passed to
``step`` supplies the overflow flag and the inverse scale; while the flag is
raised the step changes nothing and the step count does not advance.
"""
from collections import defaultdict
from copy import deepcopy
from itertools import chain

import torch

from oslo_amd.torch._C import get_l2norm_mp_kernel, get_lamb_mp_kernel
from oslo_amd.torch.optim._common import KERNEL_DTYPES, multi_tensor_applier


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
        # lr and step are tensors so that they can live on the device
        defaults = dict(
            lr=torch.tensor(lr, dtype=torch.float32),
            step=torch.tensor([step], dtype=torch.int),
            bias_correction=bias_correction,
            betas=betas,
            eps=eps,
            weight_decay=weight_decay,
            grad_averaging=grad_averaging,
            max_grad_norm=max_grad_norm,
        )
        super(FusedMixedPrecisionLamb, self).__init__(params, defaults)
        device = self.param_groups[0]["params"][0].device
        for group in self.param_groups:
            for item in ("lr", "step"):
                group[item] = group[item].to(device=device)
        self.multi_tensor_l2norm = None
        self.multi_tensor_lamb = None
        self._dummy_overflow_buf = torch.tensor([0], dtype=torch.int, device=device)
        self.reduced_precision_dtype = reduced_precision_dtype
        self.param_groups_full_precision = []
        self._step_supports_amp_scaling = True
        self.adam_w_mode = 1 if adam_w_mode else 0
        self.use_nvlamb = use_nvlamb

    def load_state_dict(self, state_dict):
        """Loads the optimizer state without casting it to the parameters'
        dtype: the moments of reduced-precision parameters are float32
        (fused_mixed_precision_lamb.py:65-137 of the reference)."""
        state_dict = deepcopy(state_dict)
        groups = self.param_groups
        saved_groups = state_dict["param_groups"]
        if len(groups) != len(saved_groups):
            raise ValueError("loaded state dict has a different number of parameter groups")
        if any(len(g["params"]) != len(s["params"]) for g, s in zip(groups, saved_groups)):
            raise ValueError(
                "loaded state dict contains a parameter group that doesn't match the size of "
                "optimizer's group"
            )
        id_map = dict(zip(chain.from_iterable(g["params"] for g in saved_groups),
                          chain.from_iterable(g["params"] for g in groups)))
        state = defaultdict(dict)
        for k, v in state_dict["state"].items():
            state[id_map[k] if k in id_map else k] = v
        param_groups = []
        for group, new_group in zip(groups, saved_groups):
            new_group["params"] = group["params"]
            param_groups.append(new_group)
        self.__setstate__({"state": state, "param_groups": param_groups})

    def _setup_full_precision_params(self):
        for group in self.param_groups:
            self.param_groups_full_precision.append({
                "params": [
                    p.clone().detach().to(dtype=torch.float32)
                    if self.reduced_precision_dtype is not None and p.dtype == self.reduced_precision_dtype
                    else None
                    for p in group["params"]
                ],
            })

    def add_param_group(self, param_group):
        # tensor defaults are cloned: two groups must not share one lr / step tensor
        super().add_param_group(param_group)
        for name, default in self.defaults.items():
            if isinstance(default, torch.Tensor):
                self.param_groups[-1][name] = default.clone()

    @torch.no_grad()
    def step(self, closure=None, grad_scaler=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if self.multi_tensor_lamb is None:
            self.multi_tensor_l2norm = get_l2norm_mp_kernel().multi_tensor_l2norm_mp
            self.multi_tensor_lamb = get_lamb_mp_kernel().multi_tensor_lamb_mp
        # the master copies are made on the first step, not in the constructor:
        # a data-parallel wrapper may still synchronise the model's parameters
        # after the optimizer has been built
        if len(self.param_groups_full_precision) == 0:
            self._setup_full_precision_params()

        grad_list = []
        for group in self.param_groups:
            first = group["params"][0]
            for p in group["params"]:
                if p.dtype != first.dtype:
                    raise RuntimeError(
                        "Error: Parameters are not of the identical type: {} != {}".format(first.dtype, p.dtype)
                    )
                if p.grad is None:
                    continue
                if not p.is_cuda or p.dtype not in KERNEL_DTYPES:
                    raise RuntimeError("FusedMixedPrecisionLamb needs fp16, bf16 or fp32 parameters on the GPU")
                grad_list.append(p.grad)
        if not grad_list:
            return loss
        if len({g.dtype for g in grad_list}) != 1:
            raise RuntimeError("FusedMixedPrecisionLamb needs gradients of one dtype")

        device = self.param_groups[0]["params"][0].device
        if grad_scaler is not None:
            found_inf = grad_scaler._check_inf_per_device(self)[device]
            scale = grad_scaler._get_scale_async()
            inv_scale = scale.double().reciprocal().float()
        elif getattr(self, "found_inf", None) is not None:
            # a GradScaler that hands its state over as attributes instead of
            # passing itself (what torch does for steps without a grad_scaler
            # argument); grad_scale None = the gradients are unscaled already
            found_inf = self.found_inf.reshape(1).float()
            given = getattr(self, "grad_scale", None)
            scale = torch.ones((1,), device=device) if given is None else given.reshape(1).float()
            inv_scale = scale.double().reciprocal().float()
        else:
            found_inf = torch.zeros((1,), device=device)
            scale = torch.ones((1,), device=device)
            inv_scale = torch.ones((1,), device=device)
        self._dummy_overflow_buf.copy_(found_inf)
        # the norm is that of the scaled gradients: the threshold is scaled too
        max_grad_norm = (self.defaults["max_grad_norm"] * scale).float().reshape(1)
        grad_norm = multi_tensor_applier(
            self.multi_tensor_l2norm, self._dummy_overflow_buf, [[g.contiguous() for g in grad_list]], False
        )[0]

        for group, group_full in zip(self.param_groups, self.param_groups_full_precision):
            bias_correction = 1 if group["bias_correction"] else 0
            beta1, beta2 = group["betas"]
            grad_averaging = 1 if group["grad_averaging"] else 0
            # one step count per group; it stands still while the flag is raised
            group["step"] += (self._dummy_overflow_buf != 1).to(torch.int)

            master = self.reduced_precision_dtype is not None
            lists = [[], [], [], []] + ([[]] if master else [])
            for p, p_full in zip(group["params"], group_full["params"]):
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("FusedMixedPrecisionLamb does not support sparse gradients")
                state = self.state[p]
                if len(state) == 0:
                    dtype = torch.float32 if master and p.dtype == self.reduced_precision_dtype else p.dtype
                    state["exp_avg"] = torch.zeros_like(p.data, dtype=dtype, memory_format=torch.contiguous_format)
                    state["exp_avg_sq"] = torch.zeros_like(p.data, dtype=dtype, memory_format=torch.contiguous_format)
                if master and p_full is None:
                    raise RuntimeError(
                        "FusedMixedPrecisionLamb: with reduced_precision_dtype=%s every parameter must have "
                        "that dtype, got %s" % (self.reduced_precision_dtype, p.dtype)
                    )
                if not p.grad.is_contiguous():
                    # the kernel leaves the update direction in the gradient; a copy would hide it
                    raise RuntimeError("FusedMixedPrecisionLamb needs contiguous gradients")
                lists[0].append(p.grad.data)
                lists[1].append(p_full.data if master else p.data)
                lists[2].append(state["exp_avg"])
                lists[3].append(state["exp_avg_sq"])
                if master:
                    lists[4].append(p.data)
            if not lists[0]:
                continue
            multi_tensor_applier(
                self.multi_tensor_lamb,
                self._dummy_overflow_buf,
                lists,
                group["lr"],
                beta1,
                beta2,
                group["eps"],
                group["step"],
                bias_correction,
                group["weight_decay"],
                grad_averaging,
                self.adam_w_mode,
                grad_norm,
                max_grad_norm,
                self.use_nvlamb,
                found_inf,
                inv_scale,
            )
        return loss
