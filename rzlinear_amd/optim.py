"""Fused optimiser steps for RzLinear parameters (``rz_sgd_step`` / ``rz_adam_step``).

The reference leaves the update to ``torch.optim``; these classes apply the same rules
(``torch.optim.SGD``, ``torch.optim.Adam`` / ``AdamW``) with one kernel per parameter and step.
They read the gradient from ``param.main_grad`` when the parameter has one (the fp32 buffer
that ``RzLinear(..., fuse_grad_accumulation=True)`` adds into) and from ``param.grad`` otherwise,
and can keep an fp32 master copy of 16-bit parameters.  Parameters must live on the GPU: there
is no CPU path.
"""
import torch

from . import _lib


def _gradient(p):
    g = getattr(p, "main_grad", None)
    return g if g is not None else p.grad


def _check(p, g):
    if not p.is_cuda:
        raise RuntimeError("rzlinear_amd.optim updates GPU parameters only (no CPU fallback)")
    if not p.is_contiguous() or not g.is_contiguous():
        raise RuntimeError("parameter and gradient must be contiguous")
    if g.shape != p.shape or (g.dtype != p.dtype and g.dtype != torch.float32):
        raise RuntimeError("gradient must have the parameter's shape and its dtype or float32")


class _Fused(torch.optim.Optimizer):
    def _master(self, p, state, group):
        if group["master_weights"] and p.dtype != torch.float32:
            if "master" not in state:
                state["master"] = p.detach().float().clone()
            return state["master"].data_ptr()
        return None

    def zero_grad(self, set_to_none=True):
        """As torch's, and also clears ``main_grad`` buffers (in place: layers keep adding into them)."""
        super().zero_grad(set_to_none=set_to_none)
        for group in self.param_groups:
            for p in group["params"]:
                g = getattr(p, "main_grad", None)
                if g is not None:
                    g.zero_()


class FusedSGD(_Fused):
    """``torch.optim.SGD`` (momentum, dampening, weight_decay, nesterov) in one kernel per parameter."""

    def __init__(self, params, lr=1e-3, momentum=0.0, dampening=0.0, weight_decay=0.0, nesterov=False,
                 master_weights=False, grad_scale=1.0):
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        super().__init__(params, dict(lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay,
                                      nesterov=nesterov, master_weights=master_weights, grad_scale=grad_scale))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = _lib.load()
        for group in self.param_groups:
            for p in group["params"]:
                g = _gradient(p)
                if g is None:
                    continue
                _check(p, g)
                state = self.state[p]
                first = "step" not in state
                state["step"] = state.get("step", 0) + 1
                buf = None
                if group["momentum"] != 0:
                    if "momentum_buffer" not in state:
                        state["momentum_buffer"] = torch.empty(p.shape, dtype=torch.float32, device=p.device)
                    buf = state["momentum_buffer"].data_ptr()
                _lib.check(lib.rz_sgd_step(p.data_ptr(), g.data_ptr(), buf, self._master(p, state, group), p.numel(),
                                           _lib.dtype_code(p), _lib.dtype_code(g), group["lr"], group["momentum"],
                                           group["dampening"], group["weight_decay"], int(group["nesterov"]),
                                           int(first), group["grad_scale"],
                                           torch.cuda.current_stream(p.device).cuda_stream))
        return loss


class FusedAdam(_Fused):
    """``torch.optim.Adam`` (``decoupled_weight_decay=True``: ``AdamW``), amsgrad off, in one kernel per parameter."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0,
                 decoupled_weight_decay=False, master_weights=False, grad_scale=1.0):
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
                                      decoupled_weight_decay=decoupled_weight_decay,
                                      master_weights=master_weights, grad_scale=grad_scale))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = _lib.load()
        for group in self.param_groups:
            for p in group["params"]:
                g = _gradient(p)
                if g is None:
                    continue
                _check(p, g)
                state = self.state[p]
                if "step" not in state:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
                    state["exp_avg_sq"] = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
                state["step"] += 1
                b1, b2 = group["betas"]
                _lib.check(lib.rz_adam_step(p.data_ptr(), g.data_ptr(), state["exp_avg"].data_ptr(),
                                            state["exp_avg_sq"].data_ptr(), self._master(p, state, group), p.numel(),
                                            _lib.dtype_code(p), _lib.dtype_code(g), group["lr"], b1, b2, group["eps"],
                                            group["weight_decay"], int(group["decoupled_weight_decay"]),
                                            state["step"], group["grad_scale"],
                                            torch.cuda.current_stream(p.device).cuda_stream))
        return loss
