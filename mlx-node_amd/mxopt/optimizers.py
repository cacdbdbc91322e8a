"""The reference's optimizer API (crates/mlx-core/src/optimizers, packages/core/index.d.cts:38-81,
486-521, 722, 1696-1712, 1855-1872, 2144, 2159) over torch device tensors.

Same class and method names, argument order, defaults and error cases as the reference; every
method is a thin shim over the C ABI in include/mxopt_optimizers.h: it extracts
(pointer, size, dtype) from the tensors, allocates the output tensor the reference would have
returned, and calls the library.  Name-keyed maps are plain dicts.

Output dtype: the reference's optimizers and clip functions return float32 for bf16 input
(MLX promotes against the float32 scalar operands and nothing casts back).  That is the
default here (`out_dtype=None` -> float32); `out_dtype="param"` / `"grad"` asks for one
round-to-nearest-even write-back in the input's own dtype instead.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib as L
from .core import Context, dtype_code

_default_ctx: Optional[Context] = None


def default_context() -> Context:
    global _default_ctx
    if _default_ctx is None or _default_ctx.handle is None:
        _default_ctx = Context()
    return _default_ctx


def _arr(t: Optional[torch.Tensor]) -> L.Array:
    if t is None:
        return L.Array(None, 0, 0)
    if not t.is_cuda:
        raise L.InvalidArg(L.ERR_INVALID_ARG, "mxopt needs device tensors (no CPU path exists)")
    if not t.is_contiguous():
        raise L.InvalidArg(L.ERR_INVALID_ARG, "mxopt needs dense (contiguous) buffers")
    return L.Array(t.data_ptr() if t.numel() else None, t.numel(), dtype_code(t))


def _arrs(ts: Sequence[Optional[torch.Tensor]]):
    a = (L.Array * max(len(ts), 1))()
    for i, t in enumerate(ts):
        a[i] = _arr(t)
    return a


def _opt(x, ctype):
    return None if x is None else C.byref(ctype(x))


def _out_like(t: torch.Tensor, out_dtype) -> torch.Tensor:
    if out_dtype is None or out_dtype == "float32":
        return torch.empty_like(t, dtype=torch.float32)
    if out_dtype in ("param", "grad", "same"):
        return torch.empty_like(t)
    return torch.empty_like(t, dtype=out_dtype)


class _Optimizer:
    """Common part of the four optimizer classes: update_single / update_many / reset."""

    def __init__(self, ctx: Optional[Context]):
        self.ctx = ctx or default_context()
        self.lib = self.ctx.lib
        self.handle = C.c_void_p()

    def __del__(self):
        if getattr(self, "handle", None) and getattr(self.ctx, "handle", None):
            self.lib.mxopt_optimizer_free(self.handle)
        self.handle = None

    def update_single(self, param_name: str, param: torch.Tensor, grad: torch.Tensor,
                      out: Optional[torch.Tensor] = None, out_dtype=None) -> torch.Tensor:
        """updateSingle(paramName, param, grad) -> new parameter array.  `out` may be `param`
        itself for an in-place update."""
        if out is None:
            out = _out_like(param, out_dtype)
        L.check(self.lib.mxopt_optimizer_update_single(self.handle, param_name.encode(), C.byref(_arr(param)),
                                                       C.byref(_arr(grad)), C.byref(_arr(out))), self.ctx.handle)
        return out

    def update_many(self, names: Sequence[str], params: Sequence[torch.Tensor], grads: Sequence[torch.Tensor],
                    outs: Optional[Sequence[torch.Tensor]] = None, out_dtype=None,
                    prep: Optional[L.GradPrep] = None) -> List[torch.Tensor]:
        """The caller's `for name, p in params: opt.update_single(name, p, g)` loop as one launch."""
        if outs is None:
            outs = [_out_like(p, out_dtype) for p in params]
        n = len(names)
        cnames = (C.c_char_p * max(n, 1))(*[s.encode() for s in names])
        L.check(self.lib.mxopt_optimizer_update_many(self.handle, n, cnames, _arrs(params), _arrs(grads), _arrs(outs),
                                                     C.byref(prep) if prep else None), self.ctx.handle)
        return list(outs)

    def update_many_accumulated(self, names: Sequence[str], params: Sequence[torch.Tensor],
                                micro_batches: Sequence[Sequence[torch.Tensor]],
                                outs: Optional[Sequence[torch.Tensor]] = None, prep: Optional[L.GradPrep] = None,
                                max_norm: float = -1.0, clip_mode: int = L.CLIP_ALWAYS_MULTIPLY,
                                norm_out=None) -> List[torch.Tensor]:
        """One optimizer step on the sum of `micro_batches` (added in registers, in order, in float32),
        clipped to `max_norm` by its global norm when max_norm >= 0.  In place unless `outs` is given."""
        if outs is None:
            outs = list(params)
        n, k = len(names), len(micro_batches)
        if any(len(mb) != n for mb in micro_batches):
            raise L.InvalidArg(L.ERR_INVALID_ARG, "every micro-batch needs one gradient per name")
        cnames = (C.c_char_p * max(n, 1))(*[s.encode() for s in names])
        flat = [g for mb in micro_batches for g in mb]
        L.check(self.lib.mxopt_optimizer_update_many_accumulated(
            self.handle, n, cnames, _arrs(params), k, _arrs(flat), _arrs(outs), C.byref(prep) if prep else None,
            max_norm, clip_mode, C.c_void_p(norm_out.ptr) if norm_out is not None else None), self.ctx.handle)
        return list(outs)

    def reset(self) -> None:
        L.check(self.lib.mxopt_optimizer_reset(self.handle), self.ctx.handle)

    @property
    def step(self) -> int:
        return self.lib.mxopt_optimizer_step_count(self.handle)

    def state(self, param_name: str) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        """Copies of (m, v) for a name; None where the optimizer keeps no such state."""
        m, v, n, hv = C.c_void_p(), C.c_void_p(), C.c_uint64(), C.c_int()
        L.check(self.lib.mxopt_optimizer_state(self.handle, param_name.encode(), C.byref(m), C.byref(v), C.byref(n),
                                               C.byref(hv)), self.ctx.handle)

        dev = self.ctx.device
        mo = torch.empty(n.value, dtype=torch.float32, device=dev) if m.value and n.value else None
        vo = torch.empty(n.value, dtype=torch.float32, device=dev) if v.value and n.value else None
        if mo is not None or vo is not None:
            L.check(self.lib.mxopt_optimizer_save_state(self.handle, param_name.encode(),
                                                        mo.data_ptr() if mo is not None else None,
                                                        vo.data_ptr() if vo is not None else None), self.ctx.handle)
        if isinstance(self, SGD) and not hv.value:
            vo = None     # SGD before its first momentum step: no velocity yet
        return mo, vo

    def save_file(self, path: str) -> None:
        """Writes every moment / velocity and the call counter to a safetensors file."""
        L.check(self.lib.mxopt_optimizer_save_file(self.handle, str(path).encode()), self.ctx.handle)

    def load_file(self, path: str) -> None:
        """Replaces this optimizer's state with a checkpoint written by save_file."""
        L.check(self.lib.mxopt_optimizer_load_file(self.handle, str(path).encode()), self.ctx.handle)

    def load_state(self, param_name: str, m: Optional[torch.Tensor], v: Optional[torch.Tensor],
                   step_count: int = 0) -> None:
        n = (m if m is not None else v).numel()
        L.check(self.lib.mxopt_optimizer_load_state(self.handle, param_name.encode(),
                                                    m.data_ptr() if m is not None else None,
                                                    v.data_ptr() if v is not None else None, n, step_count),
                self.ctx.handle)


class Adam(_Optimizer):
    """new Adam(learningRate?, beta1?, beta2?, eps?, biasCorrection?)  (optimizers/adam.rs:41-57)."""

    def __init__(self, learning_rate: Optional[float] = None, beta1: Optional[float] = None,
                 beta2: Optional[float] = None, eps: Optional[float] = None,
                 bias_correction: Optional[bool] = None, ctx: Optional[Context] = None):
        super().__init__(ctx)
        L.check(self.lib.mxopt_adam_new(self.ctx.handle, _opt(learning_rate, C.c_double), _opt(beta1, C.c_double),
                                        _opt(beta2, C.c_double), _opt(eps, C.c_double),
                                        _opt(None if bias_correction is None else int(bias_correction), C.c_int),
                                        C.byref(self.handle)), self.ctx.handle)


class AdamW(_Optimizer):
    """new AdamW(learningRate?, beta1?, beta2?, eps?, weightDecay?, biasCorrection?)  (adamw.rs:43-61)."""

    def __init__(self, learning_rate: Optional[float] = None, beta1: Optional[float] = None,
                 beta2: Optional[float] = None, eps: Optional[float] = None, weight_decay: Optional[float] = None,
                 bias_correction: Optional[bool] = None, ctx: Optional[Context] = None):
        super().__init__(ctx)
        L.check(self.lib.mxopt_adamw_new(self.ctx.handle, _opt(learning_rate, C.c_double), _opt(beta1, C.c_double),
                                         _opt(beta2, C.c_double), _opt(eps, C.c_double),
                                         _opt(weight_decay, C.c_double),
                                         _opt(None if bias_correction is None else int(bias_correction), C.c_int),
                                         C.byref(self.handle)), self.ctx.handle)


class SGD(_Optimizer):
    """new SGD(learningRate, momentum?, weightDecay?, dampening?, nesterov?)  (sgd.rs:40-67); raises
    ValueError (InvalidArg) for Nesterov without momentum or with dampening."""

    def __init__(self, learning_rate: float, momentum: Optional[float] = None, weight_decay: Optional[float] = None,
                 dampening: Optional[float] = None, nesterov: Optional[bool] = None, ctx: Optional[Context] = None):
        super().__init__(ctx)
        L.check(self.lib.mxopt_sgd_new(self.ctx.handle, learning_rate, _opt(momentum, C.c_double),
                                       _opt(weight_decay, C.c_double), _opt(dampening, C.c_double),
                                       _opt(None if nesterov is None else int(nesterov), C.c_int),
                                       C.byref(self.handle)), self.ctx.handle)


class RMSprop(_Optimizer):
    """new RMSprop(learningRate?, alpha?, eps?, weightDecay?)  (rmsprop.rs:36-50)."""

    def __init__(self, learning_rate: Optional[float] = None, alpha: Optional[float] = None,
                 eps: Optional[float] = None, weight_decay: Optional[float] = None, ctx: Optional[Context] = None):
        super().__init__(ctx)
        L.check(self.lib.mxopt_rmsprop_new(self.ctx.handle, _opt(learning_rate, C.c_double), _opt(alpha, C.c_double),
                                           _opt(eps, C.c_double), _opt(weight_decay, C.c_double),
                                           C.byref(self.handle)), self.ctx.handle)


class GradientUtils:
    """optimizers/mod.rs:33-227 (all static, like the reference)."""

    @staticmethod
    def compute_gradient_norm(gradients: Dict[str, torch.Tensor], ctx: Optional[Context] = None) -> float:
        ctx = ctx or default_context()
        gs = list(gradients.values())
        out = C.c_double()
        L.check(ctx.lib.mxopt_compute_gradient_norm(ctx.handle, len(gs), _arrs(gs), C.byref(out)), ctx.handle)
        return out.value

    @staticmethod
    def clip_grad_norm(gradients: Dict[str, torch.Tensor], max_norm: float, out_dtype=None,
                       ctx: Optional[Context] = None) -> Dict[str, torch.Tensor]:
        ctx = ctx or default_context()
        names, gs = list(gradients.keys()), list(gradients.values())
        outs = [_out_like(g, out_dtype) for g in gs]
        L.check(ctx.lib.mxopt_clip_grad_norm(ctx.handle, len(gs), _arrs(gs), max_norm, _arrs(outs), None),
                ctx.handle)
        return dict(zip(names, outs))

    @staticmethod
    def clip_grad_norm_with_norm(gradients: Dict[str, torch.Tensor], max_norm: float, out_dtype=None,
                                 ctx: Optional[Context] = None) -> Tuple[Dict[str, torch.Tensor], float]:
        ctx = ctx or default_context()
        names, gs = list(gradients.keys()), list(gradients.values())
        outs = [_out_like(g, out_dtype) for g in gs]
        norm = C.c_double()
        L.check(ctx.lib.mxopt_clip_grad_norm(ctx.handle, len(gs), _arrs(gs), max_norm, _arrs(outs), C.byref(norm)),
                ctx.handle)
        return dict(zip(names, outs)), norm.value

    @staticmethod
    def clip_grad_value(grad: torch.Tensor, min_val: float, max_val: float, out_dtype=None,
                        ctx: Optional[Context] = None) -> torch.Tensor:
        ctx = ctx or default_context()
        out = _out_like(grad, out_dtype)
        L.check(ctx.lib.mxopt_clip_grad_value(ctx.handle, C.byref(_arr(grad)), min_val, max_val, C.byref(_arr(out))),
                ctx.handle)
        return out

    @staticmethod
    def clip_grad_value_and_norm(gradients: Dict[str, torch.Tensor], clip_value: float, max_norm: Optional[float],
                                 out_dtype=None, ctx: Optional[Context] = None) -> Dict[str, torch.Tensor]:
        ctx = ctx or default_context()
        names, gs = list(gradients.keys()), list(gradients.values())
        outs = [_out_like(g, out_dtype) for g in gs]
        L.check(ctx.lib.mxopt_clip_grad_value_and_norm(ctx.handle, len(gs), _arrs(gs), clip_value,
                                                       _opt(max_norm, C.c_double), _arrs(outs)), ctx.handle)
        return dict(zip(names, outs))


def clip_gradients_by_global_norm(gradients: Sequence[torch.Tensor], max_norm: float, out_dtype=None,
                                  ctx: Optional[Context] = None) -> List[torch.Tensor]:
    """gradients/mod.rs:233-285."""
    ctx = ctx or default_context()
    gs = list(gradients)
    outs = [_out_like(g, out_dtype) for g in gs]
    L.check(ctx.lib.mxopt_clip_gradients_by_global_norm(ctx.handle, len(gs), _arrs(gs), max_norm, _arrs(outs)),
            ctx.handle)
    return outs


def clip_gradients_by_value(gradients: Sequence[torch.Tensor], min_value: float, max_value: float, out_dtype=None,
                            ctx: Optional[Context] = None) -> List[torch.Tensor]:
    """gradients/mod.rs:299-312."""
    ctx = ctx or default_context()
    gs = list(gradients)
    outs = [_out_like(g, out_dtype) for g in gs]
    L.check(ctx.lib.mxopt_clip_gradients_by_value(ctx.handle, len(gs), _arrs(gs), min_value, max_value, _arrs(outs)),
            ctx.handle)
    return outs


def _promote(a: torch.Tensor, b: torch.Tensor) -> torch.dtype:
    return a.dtype if a.dtype == b.dtype else torch.float32


def accumulate_gradients(accumulated_gradients: Dict[str, torch.Tensor], new_gradients: Dict[str, torch.Tensor],
                         ctx: Optional[Context] = None) -> Dict[str, torch.Tensor]:
    """Qwen3Model.accumulateGradients (models/qwen3/model.rs:2217-2243): a new dict; names only in the
    accumulator are carried over, names only in the new gradients are copied."""
    ctx = ctx or default_context()
    names = list(new_gradients.keys())
    new = [new_gradients[k] for k in names]
    acc = [accumulated_gradients.get(k) for k in names]
    outs = [torch.empty_like(g, dtype=_promote(a, g)) if a is not None else torch.empty_like(g)
            for a, g in zip(acc, new)]
    L.check(ctx.lib.mxopt_accumulate_gradients(ctx.handle, len(names), _arrs(acc), _arrs(new), _arrs(outs)),
            ctx.handle)
    result = dict(zip(names, outs))
    for k, a in accumulated_gradients.items():
        if k not in result:
            result[k] = a.clone()
    return result


class GradientAccumulator:
    """The engines' accumulation state (grpo/engine.rs:2632-2666; sft/engine.rs:282-290 with
    `drop_unknown=True`): sums in place into buffers it owns."""

    def __init__(self, drop_unknown: bool = False, dtype: Optional[torch.dtype] = None,
                 ctx: Optional[Context] = None):
        self.ctx = ctx or default_context()
        self.drop_unknown = drop_unknown
        self.dtype = dtype            # None: the gradient's own dtype (reference); float32: widened buffer
        self.accumulated: Optional[Dict[str, torch.Tensor]] = None
        self.micro_step = 0

    def accumulate(self, new_grads: Dict[str, torch.Tensor]) -> None:
        ctx = self.ctx
        if self.accumulated is None:
            self.accumulated = {}
            fresh = list(new_grads.keys())
        else:
            fresh = [] if self.drop_unknown else [k for k in new_grads if k not in self.accumulated]
        known = [k for k in new_grads if k in self.accumulated]
        for k in fresh:
            g = new_grads[k]
            self.accumulated[k] = torch.empty_like(g, dtype=self.dtype or g.dtype)
        names = fresh + known
        if names:
            acc = [None] * len(fresh) + [self.accumulated[k] for k in known]
            outs = [self.accumulated[k] for k in names]
            new = [new_grads[k] for k in names]
            L.check(ctx.lib.mxopt_accumulate_gradients(ctx.handle, len(names), _arrs(acc), _arrs(new), _arrs(outs)),
                    ctx.handle)
        self.micro_step += 1

    def take(self) -> Dict[str, torch.Tensor]:
        out, self.accumulated, self.micro_step = self.accumulated or {}, None, 0
        return out


def apply_gradients(params: Dict[str, torch.Tensor], gradients: Dict[str, torch.Tensor], learning_rate: float,
                    ctx: Optional[Context] = None) -> None:
    """Qwen3Model.applyGradients (models/qwen3/model.rs:2409-2460): plain SGD in the parameter's dtype,
    in place on `params`; parameters without a gradient are untouched; an unknown name raises."""
    ctx = ctx or default_context()
    names = list(gradients.keys())
    for k in names:
        if k not in params:
            raise L.MxoptError(L.ERR_FAILURE, f"Parameter '{k}' not found in model")   # model.rs:2427-2432
    ps = [params[k] for k in names]
    gs = [gradients[k] for k in names]
    L.check(ctx.lib.mxopt_apply_gradients(ctx.handle, len(names), _arrs(ps), _arrs(gs), learning_rate, _arrs(ps)),
            ctx.handle)


class LRScheduler:
    """optimizers/mod.rs:239-292."""

    @staticmethod
    def linear_decay(initial_lr: float, final_lr: float, current_step: int, total_steps: int) -> float:
        return L.load().mxopt_lr_linear_decay(initial_lr, final_lr, current_step, total_steps)

    @staticmethod
    def exponential_decay(initial_lr: float, decay_rate: float, current_step: int, decay_steps: int) -> float:
        return L.load().mxopt_lr_exponential_decay(initial_lr, decay_rate, current_step, decay_steps)

    @staticmethod
    def cosine_annealing(initial_lr: float, min_lr: float, current_step: int, total_steps: int) -> float:
        return L.load().mxopt_lr_cosine_annealing(initial_lr, min_lr, current_step, total_steps)

    @staticmethod
    def step_decay(initial_lr: float, factor: float, current_step: int, step_size: int) -> float:
        return L.load().mxopt_lr_step_decay(initial_lr, factor, current_step, step_size)
