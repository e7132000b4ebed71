"""Base optimizers of the weight-stashing wrapper: ``SGD`` and ``Adam`` whose whole step
is one fused multi-tensor HIP kernel (``pd_sgd_step`` / ``pd_adam_step``).

They keep ``torch.optim``'s object model -- ``param_groups`` with run-time ``lr`` etc.,
per-parameter ``state`` entries named like ``torch.optim.SGD`` / ``torch.optim.Adam``
(``momentum_buffer``; ``step``, ``exp_avg``, ``exp_avg_sq``), ``state_dict()`` /
``load_state_dict()`` -- because the reference relays every unknown attribute of
``OptimizerWithWeightStashing`` to its base optimizer (runtime/optimizer.py:54-56) and
its callers write ``optimizer.param_groups[i]['lr']`` every iteration
(runtime/image_classification/main_with_runtime.py:562-563).

The update reads the parameters from one ring slot and writes them to another, which
is how the stash copy of runtime/optimizer.py:156-159 disappears.
"""
import ctypes

import torch

from . import _cabi
from .arena import WeightArena, staggered_empty


class _FusedOptimizer(torch.optim.Optimizer):
    _state_names = ()

    def __init__(self, params, defaults, arena=None):
        super(_FusedOptimizer, self).__init__(params, defaults)
        self._lib = _cabi.lib()
        masters = [p for g in self.param_groups for p in g["params"]]
        if arena is None:
            arena = WeightArena([], masters, 1)
        self.arena = arena
        self._index = {}
        # mixed precision: the parameters this optimizer updates are fp32 masters outside the ring, entry i of
        # the ring holds the 16-bit model parameter of master i
        self.mixed = arena.fp32_masters is not None
        self._elem = 2 if self.mixed else 4                   # bytes per element of a ring entry
        owners = arena.fp32_masters if self.mixed else [e.tensor for e in arena.entries[:arena.num_master]]
        for e, owner in zip(arena.entries[:arena.num_master], owners):
            self._index[id(owner)] = e
        for p in masters:
            if id(p) not in self._index:
                raise ValueError("parameter is not part of the weight arena")
        self._formats = (_cabi.PD_F32, _cabi.PD_BF16)
        if self.mixed:
            fmt = _cabi.PD_BF16 if arena.half_dtype == torch.bfloat16 else _cabi.PD_F16
            self._formats = (fmt, fmt)
        n = arena.master_bytes // self._elem
        device = arena.buffer.device
        # flat state buffers share the slot layout of the master section
        # (start addresses staggered against the ring's slots, see arena.staggered_empty)
        self._flat_state = []
        for i, _ in enumerate(self._state_names):
            buf = staggered_empty(4 * n, device, 2 + i)[1].view(torch.float32)
            self._flat_state.append(buf.zero_())
        self._descs = (_cabi.TensorDesc * max(1, len(masters)))()
        self.bf16_copy = arena.bf16_image  # per-slot flat bf16 images of the master section, or None

    # -- helpers -----------------------------------------------------------------------
    def _state_view(self, which, p):
        e = self._index[id(p)]
        lo = e.offset // self._elem
        flat = self._flat_state[which][lo:lo + e.numel]
        if e.tensor.is_contiguous():
            return flat.view(e.shape)
        return flat.as_strided(e.shape, e.stride)

    def _grad_owner(self, p):
        """The tensor whose ``.grad`` the step reads: the parameter itself, or in mixed precision the 16-bit
        model parameter behind the master (the kernel widens it: no master gradient is ever materialised)."""
        return self._index[id(p)].tensor if self.mixed else p

    def _grad_for(self, p):
        owner = self._grad_owner(p)
        g = owner.grad
        if g.dtype != owner.dtype or g.device != p.device or g.is_sparse:
            raise TypeError("gradients must be dense %s tensors on the parameter's device" % owner.dtype)
        if g.stride() != (p.stride() if self.mixed else owner.stride()):
            # bring the gradient into the parameter's memory order
            g2 = torch.empty(p.shape, dtype=g.dtype, device=g.device)
            g2.copy_(g)
            g = g2
        return g

    def zero_grad(self, set_to_none=True):
        super(_FusedOptimizer, self).zero_grad(set_to_none=set_to_none)
        if self.mixed:
            # the gradients the step reads live on the model parameters
            for e in self.arena.entries[:self.arena.num_master]:
                if set_to_none:
                    e.tensor.grad = None
                elif e.tensor.grad is not None:
                    e.tensor.grad.zero_()

    def _fill(self, k, p, g, in_slot, out_slot, use_s0, use_s1):
        e = self._index[id(p)]
        d = self._descs[k]
        d.grad = g.data_ptr()
        state_offset = e.offset // self._elem * 4
        d.state0 = self._flat_state[0].data_ptr() + state_offset if use_s0 else None
        d.state1 = self._flat_state[1].data_ptr() + state_offset if use_s1 else None
        if self.mixed:
            # the master is updated in place; its 16-bit image goes into the ring's write slot
            d.p_in = d.p_out = p.data_ptr()
            d.bf16_out = e.views[out_slot].data_ptr()
        else:
            d.p_in = e.views[in_slot].data_ptr()
            d.p_out = e.views[out_slot].data_ptr()
            if self.bf16_copy is not None:
                d.bf16_out = self.bf16_copy[out_slot].data_ptr() + e.offset // 2
            else:
                d.bf16_out = None
        d.n = e.numel

    def load_state_dict(self, state_dict):
        super(_FusedOptimizer, self).load_state_dict(state_dict)
        # re-home loaded state tensors into the flat buffers
        with torch.no_grad():
            for g in self.param_groups:
                for p in g["params"]:
                    st = self.state.get(p)
                    if not st:
                        continue
                    for which, name in enumerate(self._state_names):
                        if name in st and st[name] is not None:
                            view = self._state_view(which, p)
                            view.copy_(st[name])
                            st[name] = view


class SGD(_FusedOptimizer):
    """``torch.optim.SGD`` semantics (the optimizer runtime/sgd.py:17 selects)."""
    _state_names = ("momentum_buffer",)

    def __init__(self, params, lr, momentum=0, dampening=0, weight_decay=0, nesterov=False, arena=None):
        if isinstance(lr, (int, float)) and lr < 0.0:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        if weight_decay < 0.0:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        defaults = dict(lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay,
                        nesterov=nesterov)
        super(SGD, self).__init__(params, defaults, arena)

    @torch.no_grad()
    def step(self, closure=None, in_slot=None, out_slot=None, loss_scale=1.0, update_interval=1.0):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        arena = self.arena
        in_slot = arena.live_slot if in_slot is None else in_slot
        out_slot = in_slot if out_slot is None else out_slot
        stream = _cabi.stream_ptr()
        keep = []
        for group in self.param_groups:
            momentum = group["momentum"]
            for first in (False, True):
                k = 0
                for p in group["params"]:
                    if self._grad_owner(p).grad is None:
                        continue
                    st = self.state[p]
                    is_first = momentum != 0 and st.get("momentum_buffer") is None
                    if is_first != first:
                        continue
                    g = self._grad_for(p)
                    keep.append(g)
                    self._fill(k, p, g, in_slot, out_slot, momentum != 0, False)
                    if is_first:
                        st["momentum_buffer"] = self._state_view(0, p)
                    k += 1
                if k:
                    self._lib.pd_sgd_step_mixed(self._descs, k, float(group["lr"]), float(momentum),
                                                float(group["dampening"]), float(group["weight_decay"]),
                                                int(bool(group["nesterov"])), int(first), float(loss_scale),
                                                float(update_interval), self._formats[0], self._formats[1], stream)
        self._carry_untouched(in_slot, out_slot)
        return loss

    def _carry_untouched(self, in_slot, out_slot):
        """Parameters without a gradient are not updated by torch.optim; when the step
        writes to a different slot their values still have to follow."""
        if in_slot == out_slot:
            return
        for group in self.param_groups:
            for p in group["params"]:
                if self._grad_owner(p).grad is None:
                    e = self._index[id(p)]
                    if self.mixed:          # (a 16-bit entry's size need not be a multiple of 4 bytes)
                        e.views[out_slot].copy_(e.views[in_slot])
                        continue
                    self._lib.pd_copy(ctypes.c_void_p(e.views[out_slot].data_ptr()),
                                      ctypes.c_void_p(e.views[in_slot].data_ptr()), e.nbytes, _cabi.stream_ptr())
                    if self.bf16_copy is not None:
                        views = e.tensor._pd_bf16_views
                        self._lib.pd_cast_f32_to_bf16(ctypes.c_void_p(e.views[out_slot].data_ptr()),
                                                      ctypes.c_void_p(views[out_slot].data_ptr()), e.numel,
                                                      _cabi.stream_ptr())


class Adam(_FusedOptimizer):
    """``torch.optim.Adam`` semantics (the optimizer runtime/adam.py:16 selects).

    ``eps_mode=0`` is the installed torch's formula, ``eps_mode=1`` the PyTorch-1.1 one
    (``denom = sqrt(v) + eps``) the reference's container shipped.
    """
    _state_names = ("exp_avg", "exp_avg_sq")

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False,
                 eps_mode=0, arena=None):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        if amsgrad:
            raise NotImplementedError("amsgrad is not implemented by the fused Adam kernel")
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=False)
        self.eps_mode = int(eps_mode)
        super(Adam, self).__init__(params, defaults, arena)

    @torch.no_grad()
    def step(self, closure=None, in_slot=None, out_slot=None, loss_scale=1.0, update_interval=1.0):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        arena = self.arena
        in_slot = arena.live_slot if in_slot is None else in_slot
        out_slot = in_slot if out_slot is None else out_slot
        stream = _cabi.stream_ptr()
        keep = []
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            by_step = {}
            for p in group["params"]:
                if self._grad_owner(p).grad is None:
                    continue
                st = self.state[p]
                if "step" not in st:
                    st["step"] = torch.tensor(0.0, dtype=torch.float32)
                    st["exp_avg"] = self._state_view(0, p)
                    st["exp_avg_sq"] = self._state_view(1, p)
                    st["exp_avg"].zero_()
                    st["exp_avg_sq"].zero_()
                st["step"] += 1
                by_step.setdefault(int(st["step"].item()), []).append(p)
            for t, plist in by_step.items():
                for k, p in enumerate(plist):
                    g = self._grad_for(p)
                    keep.append(g)
                    self._fill(k, p, g, in_slot, out_slot, True, True)
                self._lib.pd_adam_step_mixed(self._descs, len(plist), float(group["lr"]), float(beta1), float(beta2),
                                             float(group["eps"]), float(group["weight_decay"]), t, self.eps_mode,
                                             float(loss_scale), float(update_interval), self._formats[0],
                                             self._formats[1], stream)
        SGD._carry_untouched(self, in_slot, out_slot)
        return loss


# name -> class, the analogue of getattr(torch.optim, optim_name) at runtime/optimizer.py:40
BASE_OPTIMIZERS = {"SGD": SGD, "Adam": Adam}
