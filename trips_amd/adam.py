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


class MyAdamPoints(MyAdam):
    """MyAdam whose state for the four parameter tensors of a point cloud is packed per point.

    `position` [N,4], `point_size` [N] or [N,1], `texture` [C,N] and `confidence` [N] or [1,N] (float32, contiguous;
    NeuralPointCloudCuda.cpp:103-108, NeuralTexture.cpp:53-55) must be among `params`; their options come from their
    parameter groups as usual, and every other parameter is stepped as MyAdam steps it. The four are stepped by one
    kernel over rows of {first moment, second moment, step counter} per point (trips_adam_step_points): the same
    arithmetic per element, bit-identical results, but a point whose gradients are all zero (MyAdam.cu:57-61: not seen
    in this step) is skipped without its state being read, which the per-tensor state arrays cannot offer.
    `packed_state` [N, row] int32 holds the rows; `unpacked_state(p)` gives a parameter's state in MyAdam's own form.
    Point removal / addition (MyAdam.cu:346-415, which select along the LAST dimension of a state tensor and therefore
    fit the descriptors and the confidence): the rows follow the group that holds `texture`."""

    def __init__(self, params, position, point_size, texture, confidence, **options):
        super().__init__(params, **options)
        self._packed = [position, point_size, texture, confidence]
        known = {id(p) for g in self.param_groups for p in g["params"]}
        for p in self._packed:
            if id(p) not in known:
                raise ValueError("position, point_size, texture and confidence must be among the optimised parameters")
            if p.dtype != torch.float32 or not p.is_contiguous():
                raise ValueError("the point parameters must be contiguous float32 tensors")
        self.packed_state = None
        self._zero_grads = {}

    def state_dict(self):
        """MyAdam's state dict plus the rows of the four point parameters (`packed_state`) and their step counts, which
        live outside the per-parameter state."""
        d = super().state_dict()
        d["packed_state"] = None if self.packed_state is None else self.packed_state.clone()
        return d

    def load_state_dict(self, state_dict):
        state_dict = dict(state_dict)
        rows = state_dict.pop("packed_state", None)
        super().load_state_dict(state_dict)
        self.packed_state = None if rows is None else rows.to(self._packed[0].device).contiguous().clone()

    def _geometry(self):
        position, point_size, texture, confidence = self._packed
        n = int(position.shape[0])
        if position.dim() != 2 or position.shape[1] != 4 or texture.dim() != 2 or texture.shape[1] != n \
                or point_size.numel() != n or confidence.numel() != n:
            raise RuntimeError("MyAdamPoints: position [N,4], point_size [N], texture [C,N], confidence [N] expected")
        return n, int(texture.shape[0])

    def _rows(self, n, c, device):
        ctx = get_context(device)
        nbytes, row = ctx.adam_points_state_size(n, c)
        if self.packed_state is None:
            self.packed_state = torch.zeros((n, row // 4), dtype=torch.int32, device=device)
        if tuple(self.packed_state.shape) != (n, row // 4):
            raise RuntimeError("MyAdamPoints: the number of points changed without shrinkInternalState / "
                               "appendToInternalState")
        return self.packed_state

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        packed_ids = {id(p): i for i, p in enumerate(self._packed)}
        descs, keep, device = [], [], None
        packed_descs = [None] * 4
        any_packed_grad = any(p.grad is not None for p in self._packed)
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            for p in group["params"]:
                slot = packed_ids.get(id(p))
                if p.grad is None and (slot is None or not any_packed_grad):
                    continue
                if p.grad is not None and p.grad.is_sparse:
                    raise RuntimeError("Adam does not support sparse gradients")
                if p.dtype not in (torch.float32, torch.float64):
                    raise RuntimeError("MyAdam supports float32 and float64 parameters")
                if not p.is_contiguous():
                    raise RuntimeError("MyAdam needs contiguous parameters")
                if slot is None:
                    st = self._state_for(p)
                else:
                    st = self.state[p]
                    st.setdefault("current_step", 0)
                lower, upper = 0.0, abi.FLT_MAX
                if p.grad is not None:
                    st["current_step"] += 1
                    g = p.grad.contiguous()
                else:
                    # a point parameter without a gradient in this step: zeros leave it and its state as they are
                    g = self._zero_grads.get(id(p))
                    if g is None or g.shape != p.shape:
                        g = self._zero_grads[id(p)] = torch.zeros_like(p)
                if group["adabound"] and st["current_step"] > 0:
                    lower = 0.1 - 0.1 / ((1 - beta2) * float(st["current_step"]) + 1)
                    upper = 0.1 + 0.1 / ((1 - beta2) * float(st["current_step"]))
                keep.append(g)
                t = abi.TripsAdamTensor()
                t.weights = p.data_ptr()
                t.grads = g.data_ptr()
                t.n = p.numel()
                t.dtype = abi.TRIPS_DTYPE_F64 if p.dtype == torch.float64 else abi.TRIPS_DTYPE_F32
                t.lr = group["lr"]
                t.beta1, t.beta2, t.eps = beta1, beta2, group["eps"]
                t.relative_weight_decay = group["relative_weight_decay"]
                t.absolute_weight_decay = group["absolute_weight_decay"]
                t.weight_clipping_magnitude = group["weight_clipping_magnitude"]
                t.lower_lr_bound, t.upper_lr_bound = lower, upper
                t.loss_scale = 1.0
                device = p.device
                if slot is None:
                    t.first_moment = st["first_moments"].data_ptr()
                    t.second_moment = st["second_moments"].data_ptr()
                    t.steps = st["param_steps"].data_ptr()
                    t.steps_dtype = abi.TRIPS_STEPS_I32 if st["param_steps"].dtype == torch.int32 else abi.TRIPS_STEPS_I64
                    descs.append(t)
                else:
                    packed_descs[slot] = t
        if any_packed_grad:
            n, c = self._geometry()
            dev = self._packed[0].device
            get_context(dev).adam_step_points(packed_descs, n, c, self._rows(n, c, dev))
        if descs:
            get_context(device).adam_step(descs)
        return loss

    def unpacked_state(self, p):
        """first_moments, second_moments, param_steps of one of the four point parameters, shaped like it (copies)."""
        slot = [id(q) for q in self._packed].index(id(p))
        n, c = self._geometry()
        if self.packed_state is None:
            z = torch.zeros_like(p)
            return dict(first_moments=z, second_moments=z.clone(), param_steps=torch.zeros(p.shape, dtype=torch.int32, device=p.device))
        first, count = ((0, 4), (4, 1), (5, c), (5 + c, 1))[slot]
        tri = self.packed_state[:, :3 * (6 + c)].reshape(n, 6 + c, 3)[:, first:first + count, :]
        if slot == 2:
            tri = tri.transpose(0, 1)  # [C, N, 3]
        m = tri[..., 0].contiguous().view(torch.float32).reshape(p.shape)
        v = tri[..., 1].contiguous().view(torch.float32).reshape(p.shape)
        s = tri[..., 2].contiguous().reshape(p.shape)
        return dict(first_moments=m, second_moments=v, param_steps=s)

    @torch.no_grad()
    def shrinkInternalState(self, param_group_index, indices_to_keep):
        packed_ids = {id(p) for p in self._packed}
        group = self.param_groups[param_group_index]["params"]
        if any(p is self._packed[2] for p in group) and self.packed_state is not None:
            idx = indices_to_keep.reshape(-1).to(self.packed_state.device)
            self.packed_state = self.packed_state.index_select(0, idx).contiguous()
        others = [p for p in group if id(p) not in packed_ids]
        self._per_tensor_state(others, lambda t: t.index_select(t.dim() - 1, indices_to_keep.reshape(-1).to(t.device)).contiguous())

    @torch.no_grad()
    def appendToInternalState(self, param_group_index, new_size):
        packed_ids = {id(p) for p in self._packed}
        group = self.param_groups[param_group_index]["params"]
        if any(p is self._packed[2] for p in group) and self.packed_state is not None:
            t = self.packed_state
            self.packed_state = torch.cat([t, torch.zeros((new_size - t.shape[0], t.shape[1]), dtype=t.dtype, device=t.device)]).contiguous()
        others = [p for p in group if id(p) not in packed_ids]

        def grow(t):
            shape = list(t.shape)
            shape[-1] = new_size - t.shape[-1]
            return torch.cat([t, torch.zeros(shape, dtype=t.dtype, device=t.device)], dim=-1).contiguous()
        self._per_tensor_state(others, grow)

    def _per_tensor_state(self, params, fn):
        for p in params:
            st = self.state.get(p)
            if not st or "first_moments" not in st:
                continue
            for k in ("first_moments", "second_moments", "param_steps"):
                st[k] = fn(st[k])

