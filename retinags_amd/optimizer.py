"""Adam with the update of every tensor of a submodel in one kernel launch (rgs_adam_step,
include/rgs.h).  A torch.optim.Optimizer, so parameter groups, per-group learning rates, the
state dictionary ("step", "exp_avg", "exp_avg_sq" per parameter: what the reference's
densification edits, scene/gaussian_nn_module.py:588-635) and zero_grad work as with
torch.optim.Adam, which the reference uses with eps = 1e-15 (scene/gaussian_nn_module.py:443)."""
from __future__ import annotations

import ctypes as C

import torch

from . import _capi
from ._capi import check, lib


class Adam(torch.optim.Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8):
        if lr < 0 or eps < 0 or not 0 <= betas[0] < 1 or not 0 <= betas[1] < 1:
            raise ValueError("invalid Adam hyper-parameter")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        # tensors that share betas and eps go into one call
        batches = {}
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                if not p.is_cuda:
                    raise RuntimeError("this optimiser updates device tensors only")
                if p.grad.is_sparse or p.dtype != torch.float32 or not p.is_contiguous():
                    raise RuntimeError("parameters must be dense contiguous float32")
                state = self.state[p]
                if len(state) == 0:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state["step"] = int(state["step"]) + 1
                grad = p.grad if p.grad.is_contiguous() else p.grad.contiguous()
                key = (p.device, float(group["betas"][0]), float(group["betas"][1]), float(group["eps"]))
                batches.setdefault(key, []).append((p, grad, state, float(group["lr"])))
        for (device, beta1, beta2, eps), items in batches.items():
            arr = (_capi.AdamTensor * len(items))()
            for k, (p, grad, state, lr) in enumerate(items):
                arr[k] = _capi.AdamTensor(p.data_ptr(), grad.data_ptr(), state["exp_avg"].data_ptr(),
                                          state["exp_avg_sq"].data_ptr(), p.numel(), lr, state["step"])
            check(lib.rgs_adam_step(len(items), arr, beta1, beta2, eps,
                                    C.c_void_p(torch.cuda.current_stream(device).cuda_stream)))
        return loss
