"""RangerLite, the reference's optimizer (model/optimizers/ranger_lite.py:216-808), with its fused
update running as HIP kernels of libnnueft.so instead of CuPy kernels.

Same constructor, parameter-group keys, state keys ("step", "grad_ma", "variance_ma",
"neg_grad_ma", "lookahead_params", "is_swapped") and train()/eval() behaviour, so checkpoints
and the wrapper around it (rangerlite_wrapper.py:44-118) carry over.  Which path a step takes
follows the reference (ranger_lite.py:517-587):

  fused      every parameter with a gradient is a contiguous float32 GPU tensor, no norm loss,
             no legacy mode.  Without weight decay one kernel per tensor does everything; with
             it, a variance kernel per tensor, the global variance norm, then the update kernel.
             On a lookahead merge step the blend happens inside the update kernel.
  torch ops  everything else (CPU tensors, norm loss, legacy mode), as the reference's Python path.

Tensors on the GPU with the library missing raise: there is no silent slow path for them.
"""
import collections.abc
import math

import torch

from . import _native
from .sparse_linear_functions import _stream_ptr


class RangerLite(torch.optim.Optimizer):
    MULTI_TENSOR_BELOW = 1 << 20      # elements; smaller tensors are updated several per launch

    def __init__(self, params, lr=1.0, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-7, pnm_activate=True,
                 pnm_momentum=1.0, lookahead_active=True, lookahead_mergetime=5, lookahead_blending_alpha=0.5,
                 normloss_active=True, normloss_factor=1e-4, use_legacy_scoping_bug=False):
        defaults = dict(lr=lr, weight_decay=weight_decay, betas=betas, eps=eps, pnm_momentum=pnm_momentum,
                        normloss_factor=normloss_factor)
        super().__init__(params, defaults)
        self.lookahead_active = lookahead_active
        self.lookahead_mergetime = lookahead_mergetime
        self.lookahead_alpha = lookahead_blending_alpha
        self.lookahead_step = 0
        self.pnm_active = pnm_activate
        self.normloss_active = normloss_active
        self.eps = eps
        self.param_size = 0
        self.use_legacy_scoping_bug = use_legacy_scoping_bug

    # ------------------------------------------------------------------ state
    def _init_state(self, p):
        state = self.state[p]
        if len(state) == 0:
            state["step"] = 0
            state["grad_ma"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            state["variance_ma"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            if self.lookahead_active:
                state["lookahead_params"] = torch.clone(p.data)
            if self.pnm_active:
                state["neg_grad_ma"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        return state

    def _active(self):
        return [(p, g) for g in self.param_groups for p in g["params"] if p.grad is not None]

    def _fusable(self, active):
        if self.normloss_active or self.use_legacy_scoping_bug:
            return False
        names = ["grad_ma", "variance_ma"] + (["neg_grad_ma"] if self.pnm_active else []) + \
                (["lookahead_params"] if self.lookahead_active else [])
        for p, _ in active:
            g = p.grad
            if g.is_sparse or p.dtype != torch.float32 or p.device.type != "cuda":
                return False
            if not p.is_contiguous() or not g.is_contiguous() or g.dtype != torch.float32:
                return False
            state = self.state[p]
            for name in names:
                t = state.get(name)
                if t is not None and (t.dtype != torch.float32 or t.device != p.device or not t.is_contiguous()):
                    return False
        return True

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None and isinstance(closure, collections.abc.Callable):
            with torch.enable_grad():
                loss = closure()
        active = self._active()
        if not active:
            return loss
        if self._fusable(active):
            self._step_fused(active)
        else:
            self._step_torch()
            if self.lookahead_active:
                self.lookahead_process_step()
        return loss

    @torch.compiler.disable
    def _step_fused(self, active):
        lib = _native.load()     # raises when libnnueft.so is missing
        needs_norm = any(g.get("weight_decay", 0.0) != 0.0 for g in self.param_groups)
        param_size = 0
        for p, _ in active:
            self._init_state(p)["step"] += 1
            param_size += p.numel()

        variance_norm = None
        if needs_norm:
            total = None
            for p, group in active:
                state = self.state[p]
                beta2 = group["betas"][1]
                with torch.cuda.device(p.device):
                    rc = lib.nnueft_ranger_lite_update_variance(p.grad.data_ptr(), state["variance_ma"].data_ptr(),
                                                                p.numel(), beta2, 1.0 - beta2, _stream_ptr(p.device))
                _native.check(rc, "nnueft_ranger_lite_update_variance")
                part = state["variance_ma"].sum() / (1.0 - beta2 ** state["step"])
                total = part if total is None else total + part
            if not self.param_size:
                self.param_size = param_size
            variance_norm = torch.sqrt(total / self.param_size).clamp_min(self.eps).item()

        merge = False
        if self.lookahead_active:
            self.lookahead_step += 1
            if self.lookahead_step >= self.lookahead_mergetime:
                self.lookahead_step = 0
                merge = True

        # tensors below this size share launches (a launch costs a few microseconds whatever the size)
        small = {}
        for p, group in active:
            state = self.state[p]
            beta1, beta2 = group["betas"]
            lr, eps, step = group["lr"], group["eps"], state["step"]
            decay = group.get("weight_decay", 0.0)
            wd_factor = decay * lr / variance_norm if (decay and variance_norm is not None) else 0.0
            bc2 = 1.0 - beta2 ** step
            slow = state["lookahead_params"].data_ptr() if merge else None
            if p.numel() < self.MULTI_TENSOR_BELOW:
                a = _native.RangerArgs()
                a.p, a.grad, a.grad_ma = p.data_ptr(), p.grad.data_ptr(), state["grad_ma"].data_ptr()
                a.variance_ma, a.lookahead_params, a.n = state["variance_ma"].data_ptr(), slow, p.numel()
                a.beta2, a.one_minus_beta2, a.bias_correction2 = beta2, 1.0 - beta2, bc2
                a.eps, a.wd_factor = eps, wd_factor
                a.lookahead_alpha, a.one_minus_lookahead_alpha = self.lookahead_alpha, 1.0 - self.lookahead_alpha
                a.update_variance = 0 if needs_norm else 1
                if self.pnm_active:
                    pnm = group["pnm_momentum"]
                    a.neg_grad_ma = state["neg_grad_ma"].data_ptr()
                    a.beta1, a.one_minus_beta1 = beta1 * beta1, 1.0 - beta1 * beta1
                    a.one_plus_pnm, a.pnm_factor = 1.0 + pnm, pnm
                    a.noise_norm = math.sqrt((1.0 + pnm) ** 2 + pnm ** 2)
                    a.lr_div_bc1 = lr / (1.0 - beta1 ** (((step + 1) // 2) * 2))
                    a.odd_step = step & 1
                else:
                    a.neg_grad_ma = None
                    a.beta1, a.one_minus_beta1 = beta1, 1.0 - beta1
                    a.lr_div_bc1 = lr / (1.0 - beta1 ** step)
                small.setdefault(p.device, []).append(a)
                continue
            with torch.cuda.device(p.device):
                if self.pnm_active:
                    pnm = group["pnm_momentum"]
                    bc1 = 1.0 - beta1 ** (((step + 1) // 2) * 2)
                    rc = lib.nnueft_ranger_lite_update_pnm(
                        p.data_ptr(), p.grad.data_ptr(), state["grad_ma"].data_ptr(), state["neg_grad_ma"].data_ptr(),
                        state["variance_ma"].data_ptr(), p.numel(), beta2, 1.0 - beta2, bc2, beta1 * beta1,
                        1.0 - beta1 * beta1, 1.0 + pnm, pnm, math.sqrt((1.0 + pnm) ** 2 + pnm ** 2), lr / bc1, eps,
                        step, wd_factor, 0 if needs_norm else 1, slow, self.lookahead_alpha, _stream_ptr(p.device))
                    _native.check(rc, "nnueft_ranger_lite_update_pnm")
                else:
                    bc1 = 1.0 - beta1 ** step
                    rc = lib.nnueft_ranger_lite_update_adam(
                        p.data_ptr(), p.grad.data_ptr(), state["grad_ma"].data_ptr(), state["variance_ma"].data_ptr(),
                        p.numel(), beta2, 1.0 - beta2, bc2, beta1, 1.0 - beta1, lr / bc1, eps, wd_factor,
                        0 if needs_norm else 1, slow, self.lookahead_alpha, _stream_ptr(p.device))
                    _native.check(rc, "nnueft_ranger_lite_update_adam")
        for device, records in small.items():
            arr = (_native.RangerArgs * len(records))(*records)
            with torch.cuda.device(device):
                rc = lib.nnueft_ranger_lite_update_multi(arr, len(records), _stream_ptr(device))
            _native.check(rc, "nnueft_ranger_lite_update_multi")

    def _step_torch(self):
        """The reference's Python path (ranger_lite.py:589-735) in torch ops."""
        first = next(p for g in self.param_groups for p in g["params"] if p.grad is not None)
        variance_sum = torch.zeros(1, device=first.device)
        param_size = 0
        last_seen = None
        for group in self.param_groups:
            beta2 = group["betas"][1]
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("Sparse matrix not supported")
                last_seen = p
                param_size += p.numel()
                state = self._init_state(p)
                state["step"] += 1
                v = state["variance_ma"]
                v.mul_(beta2).addcmul_(p.grad, p.grad, value=1 - beta2)
                variance_sum += (v / (1 - beta2 ** state["step"])).sum()
        if not self.param_size:
            self.param_size = param_size
        variance_norm = torch.sqrt(variance_sum / self.param_size).clamp_min(self.eps)

        def shrink(t, decay, lr, normloss_factor):
            if decay:
                t.data.mul_(1 - decay * lr / variance_norm)
            if self.normloss_active:
                unorm = self.unit_norm(t.data)
                t.data.mul_(1 - lr * (2 * normloss_factor * (1 - torch.div(1, unorm + self.eps))))

        for group in self.param_groups:
            decay, lr = group["weight_decay"], group["lr"]
            beta1, beta2 = group["betas"]
            pnm, normloss_factor = group["pnm_momentum"], group["normloss_factor"]
            if self.use_legacy_scoping_bug and last_seen is not None:
                # legacy behaviour: decay and norm loss hit the last tensor the previous loop touched
                shrink(last_seen, decay, lr, normloss_factor)
            for p in group["params"]:
                if self.use_legacy_scoping_bug:
                    last_seen = p
                if p.grad is None:
                    continue
                state = self.state[p]
                if not self.use_legacy_scoping_bug:
                    shrink(p, decay, lr, normloss_factor)
                grad, step = p.grad, state["step"]
                denom = (state["variance_ma"].sqrt() / math.sqrt(1 - beta2 ** step)).add_(group["eps"])
                if self.pnm_active:
                    if step % 2 == 1:
                        pos, neg = state["grad_ma"], state["neg_grad_ma"]
                    else:
                        pos, neg = state["neg_grad_ma"], state["grad_ma"]
                    pos.mul_(beta1 ** 2).add_(grad, alpha=1 - beta1 ** 2)
                    if self.use_legacy_scoping_bug:
                        bc1 = 1 - beta1 ** step
                        noise_norm = math.sqrt((1 + beta2) ** 2 + beta2 ** 2)
                    else:
                        bc1 = 1 - beta1 ** (((step + 1) // 2) * 2)
                        noise_norm = math.sqrt((1 + pnm) ** 2 + pnm ** 2)
                    direction = pos.mul(1 + pnm).add(neg, alpha=-pnm).mul(1 / noise_norm)
                    p.addcdiv_(direction, denom, value=-lr / bc1)
                else:
                    bc1 = 1 - beta1 ** step
                    state["grad_ma"].mul_(beta1).add_(grad, alpha=1 - beta1)
                    p.addcdiv_(state["grad_ma"], denom, value=-lr / bc1)

    def unit_norm(self, x):
        """L2 norm per row / filter / embedding vector (keepdim), or of the whole tensor when 1-D."""
        if x.ndim <= 1:
            return x.norm(p=2.0, keepdim=False)
        return x.norm(dim=tuple(range(1, x.ndim)), keepdim=True, p=2.0)

    # ------------------------------------------------------------------ lookahead
    def lookahead_process_step(self):
        if not self.lookahead_active:
            return
        self.lookahead_step += 1
        if self.lookahead_step < self.lookahead_mergetime:
            return
        self.lookahead_step = 0
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                slow = self.state[p]["lookahead_params"]
                p.data.mul_(self.lookahead_alpha).add_(slow, alpha=1.0 - self.lookahead_alpha)
                slow.copy_(p.data)

    def train(self):
        if self.lookahead_active:
            self.restore_for_training()

    def eval(self):
        if self.lookahead_active:
            self.swap_for_inference()

    def swap_for_inference(self):
        """The slow weights become the parameters (pointer swap); idempotent."""
        if not self.lookahead_active:
            return
        for group in self.param_groups:
            for p in group["params"]:
                state = self.state[p]
                if "lookahead_params" in state and "is_swapped" not in state:
                    p.data, state["lookahead_params"] = state["lookahead_params"], p.data
                    state["is_swapped"] = True

    def restore_for_training(self):
        """The fast weights come back; what eval mode did to the parameters stays as the slow copy."""
        if not self.lookahead_active:
            return
        for group in self.param_groups:
            for p in group["params"]:
                state = self.state[p]
                if "is_swapped" in state:
                    p.data, state["lookahead_params"] = state["lookahead_params"], p.data
                    del state["is_swapped"]
