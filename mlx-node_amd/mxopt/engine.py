"""The optimizer side of the reference's training engines (GRPOTrainingEngine,
crates/mlx-core/src/grpo/engine.rs:561-704; SftTrainingEngine, crates/mlx-core/src/sft/engine.rs:215-371,
459-553) over torch device tensors: a thin shim over include/mxopt_engine.h.

Config keyword names and defaults are those of GRPOEngineConfig / SftEngineConfig (None = the
reference's Option::None); getters are those of the engines (step, micro_step, nan_gradient_count,
needs_emergency_save, clear_emergency_save_flag, reset).  Parameters are updated in place.
With defer_accumulation=True the engine keeps no accumulation buffer: it remembers the gradient tensors
of a cycle (this shim keeps them alive) and the applying call adds them in registers.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional

import torch

from . import _lib as L
from .core import Context
from .optimizers import _arr, default_context


class TrainingStopped(L.MxoptError):
    """The engines' "Training stopped: exceeded ... NaN gradient ..." error (GenericFailure)."""


class _EngineOptimizerSide:
    KIND = L.ENGINE_GRPO

    def __init__(self, params: Dict[str, torch.Tensor], cfg: L.EngineConfig, ctx: Optional[Context]):
        self.ctx = ctx or default_context()
        self.lib = self.ctx.lib
        self.defers = bool(cfg.defer_accumulation)
        self._held = []
        self.params = dict(params)
        names = list(self.params)
        cnames = (C.c_char_p * max(len(names), 1))(*[s.encode() for s in names])
        arrs = (L.Array * max(len(names), 1))()
        for i, nm in enumerate(names):
            arrs[i] = _arr(self.params[nm])
        self.handle = C.c_void_p()
        L.check(self.lib.mxopt_engine_new(self.ctx.handle, C.byref(cfg), len(names), cnames, arrs,
                                          C.byref(self.handle)), self.ctx.handle)

    def __del__(self):
        if getattr(self, "handle", None) and getattr(self.ctx, "handle", None):
            self.lib.mxopt_engine_free(self.handle)
        self.handle = None

    def _release_held(self) -> None:
        """The applying call has been enqueued, not finished: tell torch's allocator that the cycle's gradient
        tensors are still in use on the context's stream before dropping the references to them."""
        for tensors in self._held:
            for t in tensors:
                if t.is_cuda:
                    t.record_stream(self.ctx.stream)
        self._held = []

    def _check(self, rc: int) -> None:
        if rc == L.OK:
            return
        msg = self.lib.mxopt_last_error(self.ctx.handle).decode("utf-8", "replace")
        if msg.startswith("Training stopped"):
            raise TrainingStopped(rc, msg)
        if msg.startswith("Parameter '") and msg.endswith("not found in model"):
            raise KeyError(msg)
        L.check(rc, self.ctx.handle)

    def micro_batch(self, gradients: Dict[str, torch.Tensor]) -> L.EngineMetrics:
        """The part of train_step after the backward pass, for one micro-batch of gradients."""
        names = list(gradients)
        cnames = (C.c_char_p * max(len(names), 1))(*[s.encode() for s in names])
        arrs = (L.Array * max(len(names), 1))()
        for i, nm in enumerate(names):
            arrs[i] = _arr(gradients[nm])
        m = L.EngineMetrics()
        if self.defers:   # deferred accumulation reads the cycle's gradients when it is applied: keep them alive
            self._held.append(list(gradients.values()))
        self._check(self.lib.mxopt_engine_micro_batch(self.handle, len(names), cnames, arrs, C.byref(m)))
        if m.gradients_applied or m.micro_step == 0:
            self._release_held()
        return m

    def micro_batch_async(self, gradients: Dict[str, torch.Tensor]) -> None:
        """micro_batch without the host synchronisation (GRPO, plain-SGD apply): the validity flag stays on the
        device; settle() -- or the next call of any kind -- books a skipped micro-batch afterwards."""
        names = list(gradients)
        cnames = (C.c_char_p * max(len(names), 1))(*[s.encode() for s in names])
        arrs = (L.Array * max(len(names), 1))()
        for i, nm in enumerate(names):
            arrs[i] = _arr(gradients[nm])
        # the kernels read the gradients after this returns: they stay alive until the call after next has settled them
        self._async_keep = [getattr(self, "_async_keep", [None, None])[1], list(gradients.values())]
        if self.defers:
            self._held.append(list(gradients.values()))
        self._check(self.lib.mxopt_engine_micro_batch_async(self.handle, len(names), cnames, arrs))

    def settle(self) -> L.EngineMetrics:
        m = L.EngineMetrics()
        self._check(self.lib.mxopt_engine_settle(self.handle, C.byref(m)))
        if self.defers and (m.gradients_applied or m.micro_step == 0):
            self._release_held()
        return m

    def metrics(self) -> L.EngineMetrics:
        m = L.EngineMetrics()
        self._check(self.lib.mxopt_engine_get_metrics(self.handle, C.byref(m)))
        return m

    @property
    def step(self) -> int:
        return self.metrics().step

    @property
    def micro_step(self) -> int:
        return self.metrics().micro_step

    @property
    def nan_gradient_count(self) -> int:
        return self.metrics().nan_gradient_count

    @property
    def needs_emergency_save(self) -> bool:
        return bool(self.metrics().needs_emergency_save)

    def clear_emergency_save_flag(self) -> None:
        self._check(self.lib.mxopt_engine_clear_emergency_save_flag(self.handle))

    def reset(self) -> None:
        self._check(self.lib.mxopt_engine_reset(self.handle))
        self._release_held()

    def save_optimizer_state(self, path) -> None:
        self._check(self.lib.mxopt_engine_save_optimizer_state(self.handle, str(path).encode()))

    def load_optimizer_state(self, path) -> None:
        self._check(self.lib.mxopt_engine_load_optimizer_state(self.handle, str(path).encode()))


def _config(kind, learning_rate, gradient_accumulation_steps, gradient_clip_norm, gradient_clip_value, weight_decay,
            max_nan_gradients, emergency_save_threshold, apply, beta1, beta2, eps, accumulate_in_f32,
            defer_accumulation=False) -> L.EngineConfig:
    cfg = L.EngineConfig()
    L.load().mxopt_engine_config_default(kind, C.byref(cfg))
    if learning_rate is not None:
        cfg.learning_rate = learning_rate
    if gradient_accumulation_steps is not None:
        cfg.gradient_accumulation_steps = gradient_accumulation_steps
    cfg.has_gradient_clip_norm = int(gradient_clip_norm is not None)
    cfg.gradient_clip_norm = gradient_clip_norm or 0.0
    cfg.has_gradient_clip_value = int(gradient_clip_value is not None)
    cfg.gradient_clip_value = gradient_clip_value or 0.0
    if weight_decay is not None:
        cfg.weight_decay = weight_decay
    if max_nan_gradients is not None:
        cfg.max_nan_gradients = max_nan_gradients
    if emergency_save_threshold is not None:
        cfg.emergency_save_threshold = emergency_save_threshold
    cfg.apply = {"sgd": L.ENGINE_APPLY_SGD, "adamw": L.ENGINE_APPLY_ADAMW}[apply]
    cfg.beta1, cfg.beta2, cfg.eps = beta1, beta2, eps
    cfg.accumulate_in_f32 = int(accumulate_in_f32)
    cfg.defer_accumulation = int(defer_accumulation)
    return cfg


class GRPOEngineOptimizerSide(_EngineOptimizerSide):
    """grpo/engine.rs:561-704.  gradient_clip_norm=None: no norm clipping (GRPOEngineConfig::default has
    Some(1.0)); gradient_clip_value=None: 1.0 (engine.rs:636)."""

    def __init__(self, params, learning_rate: Optional[float] = None, gradient_accumulation_steps: Optional[int] = None,
                 gradient_clip_norm: Optional[float] = 1.0, gradient_clip_value: Optional[float] = None,
                 max_nan_gradients: Optional[int] = None, emergency_save_threshold: Optional[int] = None,
                 apply: str = "sgd", weight_decay: float = 0.01, beta1: float = 0.9, beta2: float = 0.999,
                 eps: float = 1e-8, defer_accumulation: bool = False, ctx: Optional[Context] = None):
        super().__init__(params, _config(L.ENGINE_GRPO, learning_rate, gradient_accumulation_steps, gradient_clip_norm,
                                         gradient_clip_value, weight_decay, max_nan_gradients,
                                         emergency_save_threshold, apply, beta1, beta2, eps, True,
                                         defer_accumulation), ctx)


class SFTEngineOptimizerSide(_EngineOptimizerSide):
    """sft/engine.rs:215-371, :459-553.  weight_decay=None: 0 (the config default is Some(0.01))."""

    def __init__(self, params, learning_rate: Optional[float] = None, gradient_accumulation_steps: Optional[int] = None,
                 gradient_clip_norm: Optional[float] = 1.0, gradient_clip_value: Optional[float] = None,
                 weight_decay: Optional[float] = None, max_nan_gradients: Optional[int] = None,
                 emergency_save_threshold: Optional[int] = None, apply: str = "sgd", beta1: float = 0.9,
                 beta2: float = 0.999, eps: float = 1e-8, accumulate_in_f32: bool = False,
                 defer_accumulation: bool = False, ctx: Optional[Context] = None):
        super().__init__(params, _config(L.ENGINE_SFT, learning_rate, gradient_accumulation_steps, gradient_clip_norm,
                                         gradient_clip_value, 0.0 if weight_decay is None else weight_decay,
                                         max_nan_gradients, emergency_save_threshold, apply, beta1, beta2, eps,
                                         accumulate_in_f32, defer_accumulation), ctx)

    def flush_gradients(self) -> bool:
        flushed = C.c_int()
        m = L.EngineMetrics()
        self._check(self.lib.mxopt_engine_flush_gradients(self.handle, C.byref(flushed), C.byref(m)))
        self._held = []
        self.last_metrics = m
        return bool(flushed.value)

    def report_nonfinite_loss(self) -> L.EngineMetrics:
        m = L.EngineMetrics()
        self._check(self.lib.mxopt_engine_report_nonfinite_loss(self.handle, C.byref(m)))
        return m
