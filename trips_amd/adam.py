"""MyAdam: the reference's point-parameter optimiser (src/lib/models/MyAdam.{h,cu}) over the fused HIP kernel.

Same option names as torch::optim::MyAdamOptions (MyAdam.h:28-48): lr, betas, eps, relative_weight_decay,
absolute_weight_decay, weight_clipping_magnitude, adabound. State per parameter: param_steps (one counter per element;
int32 here, the reference keeps int64 — nothing outside the optimiser reads it, and the narrower counter saves 8 of
the 44 bytes an updated element moves), first_moments, second_moments (float32) and current_step
(MyAdam.cu:145-160,188-203). All tensors of
all groups are stepped by ONE kernel launch (the reference launches once per tensor and synchronises).
"""
import torch

from . import abi
from .renderer import get_context


class MyAdam(torch.optim.Optimizer):
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, relative_weight_decay=0.0,
                 absolute_weight_decay=0.0, weight_clipping_magnitude=0.0, adabound=False,
                 param_steps_dtype=torch.int32):
        if param_steps_dtype not in (torch.int32, torch.int64):
            raise ValueError("param_steps_dtype must be torch.int32 or torch.int64 (the reference's state tensor)")
        self.param_steps_dtype = param_steps_dtype
        if lr < 0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if eps < 0:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0 <= betas[0] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 0: {betas[0]}")
        if not 0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 1: {betas[1]}")
        if relative_weight_decay < 0:
            raise ValueError(f"Invalid relative_weight_decay value: {relative_weight_decay}")
        if absolute_weight_decay < 0:
            raise ValueError(f"Invalid absolute_weight_decay value: {absolute_weight_decay}")
        defaults = dict(lr=lr, betas=betas, eps=eps, relative_weight_decay=relative_weight_decay,
                        absolute_weight_decay=absolute_weight_decay,
                        weight_clipping_magnitude=weight_clipping_magnitude, adabound=adabound)
        super().__init__(params, defaults)

    def _state_for(self, p):
        st = self.state[p]
        if len(st) == 0:
            st["param_steps"] = torch.zeros(p.shape, dtype=self.param_steps_dtype, device=p.device)
            st["first_moments"] = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
            st["second_moments"] = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
            st["current_step"] = 0
        return st

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        descs, keep, device = [], [], None
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("Adam does not support sparse gradients")
                if p.dtype not in (torch.float32, torch.float64):
                    raise RuntimeError("MyAdam supports float32 and float64 parameters")
                if not p.is_contiguous():
                    raise RuntimeError("MyAdam needs contiguous parameters")
                st = self._state_for(p)
                st["current_step"] += 1
                lower, upper = 0.0, abi.FLT_MAX
                if group["adabound"]:
                    # AdaBound bounds, MyAdam.cu:213-221
                    lower = 0.1 - 0.1 / ((1 - beta2) * float(st["current_step"]) + 1)
                    upper = 0.1 + 0.1 / ((1 - beta2) * float(st["current_step"]))
                g = p.grad.contiguous()
                keep.append(g)
                t = abi.TripsAdamTensor()
                t.weights = p.data_ptr()
                t.grads = g.data_ptr()
                t.first_moment = st["first_moments"].data_ptr()
                t.second_moment = st["second_moments"].data_ptr()
                t.steps = st["param_steps"].data_ptr()
                t.steps_dtype = abi.TRIPS_STEPS_I32 if st["param_steps"].dtype == torch.int32 else abi.TRIPS_STEPS_I64
                t.n = p.numel()
                t.dtype = abi.TRIPS_DTYPE_F64 if p.dtype == torch.float64 else abi.TRIPS_DTYPE_F32
                t.lr = group["lr"]
                t.beta1, t.beta2, t.eps = beta1, beta2, group["eps"]
                t.relative_weight_decay = group["relative_weight_decay"]
                t.absolute_weight_decay = group["absolute_weight_decay"]
                t.weight_clipping_magnitude = group["weight_clipping_magnitude"]
                t.lower_lr_bound, t.upper_lr_bound = lower, upper
                t.loss_scale = 1.0
                descs.append(t)
                device = p.device
        if descs:
            get_context(device).adam_step(descs)
        return loss

    # point removal / addition (MyAdam.cu:346-415): state follows the last dimension of the parameter
    @torch.no_grad()
    def shrinkInternalState(self, param_group_index, indices_to_keep):
        for p in self.param_groups[param_group_index]["params"]:
            st = self.state.get(p)
            if not st:
                continue
            idx = indices_to_keep.reshape(-1).to(p.device)
            for k in ("first_moments", "second_moments", "param_steps"):
                st[k] = st[k].index_select(st[k].dim() - 1, idx).contiguous()

    @torch.no_grad()
    def appendToInternalState(self, param_group_index, new_size):
        for p in self.param_groups[param_group_index]["params"]:
            st = self.state.get(p)
            if not st:
                continue
            for k in ("first_moments", "second_moments", "param_steps"):
                t = st[k]
                shape = list(t.shape)
                shape[-1] = new_size - t.shape[-1]
                st[k] = torch.cat([t, torch.zeros(shape, dtype=t.dtype, device=t.device)], dim=-1).contiguous()
