"""CPU oracle for the optimizer-step path of mlx-node (TEST INFRASTRUCTURE ONLY).

This module restates, in NumPy float32 and one rounded operation at a time, what
the reference's optimizer path computes.  It exists to check the HIP kernels; it is
never imported by the product package, only by tests, the smoke check and the
CPU-baseline leg of the benchmark.

Conventions shared by every function here
-----------------------------------------
* The reference builds each optimizer as a chain of MLX element-wise ops, and MLX
  rounds to float32 after every op.  Every line below is therefore exactly one
  IEEE float32 operation on arrays (NumPy does not contract a*b+c).
* Every host scalar reaches MLX as ``array(static_cast<float>(value))``
  (crates/mlx-sys/src/mlx.cpp:335-338, 525-547): coefficients are evaluated in
  float64 on the host and only then cast to float32.  ``_f32`` is that cast.
* bfloat16 tensors are carried as ``numpy.uint16`` bit patterns.  A bf16 operand
  combined with a float32 scalar array promotes to float32 (MLX type promotion),
  so the optimizers below up-cast bf16 inputs, compute in float32 and return
  float32, exactly like ``update_single`` which never casts back
  (crates/mlx-core/src/optimizers/adamw.rs:81-142).

What pins each function (see tests/test_oracle_*.py)
----------------------------------------------------
* SGD, SGD+momentum, L2 decay, clip-by-value, gradient norm, clip-by-norm,
  LR schedules, gradient accumulation, apply_gradients: the closed-form
  known-answer values held by the reference's own tests
  (__test__/core/optimizers.test.ts, __test__/trainers/grpo-gradient-accumulation.test.ts,
  __test__/training/basic-training.test.ts).
* Adam/AdamW (bias correction on, one tensor), SGD, RMSprop, clip_grad_norm:
  agreement with torch.optim / torch.nn.utils (a library that is not the
  reference) to ~1e-6 relative, plus float64 brute force on small inputs.
* f32<->bf16 conversion: bit-exact against torch's CPU conversion.
* GradientUtils.clip_grad_value_and_norm (clamp, norm of the clamped values, scale; max_norm=None
  returns the clamped values: optimizers/mod.rs:174-226) and clip_gradients_by_value with a one-sided
  bound through inf (gradients/mod.rs:299-312, mlx.cpp:469-481): closed forms worked by hand in
  tests/test_oracle_kat.py.

PARITY UNPINNED (no reference test, fixture or buildable reference covers it):
* bf16 inputs through any optimizer (promotion to float32 by the scalar multiplies and
  a 16-bit ``square`` of a 16-bit gradient are MLX's documented rules, but no
  reference test runs either);
* the order in which MLX sums squares for the global norm (the oracle uses the
  exact float64 sum, rounded once);
* NaN handling of ``clip`` (NaN is propagated here);
* the per-call ``step`` quirk, Nesterov's stored state and the
  ``(m/(sqrt(v)+eps))*lr`` association are pinned only by reading the source;
* the engines' optimizer-side state machines (GRPOEngineOptimizerSide,
  SFTEngineOptimizerSide: skip-on-NaN counters, emergency flag, step counting,
  flush): no reference test exercises them; their arithmetic is a composition of
  the pinned functions above (the lr/N and accumulate-then-apply identities are
  the reference's own known answers, grpo-gradient-accumulation.test.ts:48-68,134-171),
  their bookkeeping is pinned only by reading the source;
* the ``apply="adamw"`` mode of those two classes has no counterpart in the
  reference at all (it is this build's fused replacement for apply_gradients).
"""
from __future__ import annotations

import math
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np

F32 = np.float32


def _f32(x: float) -> np.float32:
    """float64 host scalar -> float32 MLX scalar (mlx.cpp:335-338, 531-535)."""
    return np.float32(np.float64(x))


# --------------------------------------------------------------------------
# bfloat16 helpers (bit patterns in uint16)
# --------------------------------------------------------------------------

def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    """Exact widening of bf16 bit patterns to float32."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round-to-nearest-even; NaN stays a quiet NaN.

    This is ``astype(bfloat16)`` of the reference (models/qwen3/model.rs:2443-2448).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if np.any(nan):
        quiet = ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16)
        rounded = np.where(nan, quiet, rounded)
    return rounded


def as_f32(x: np.ndarray) -> np.ndarray:
    """Promote an oracle tensor (float32, or bf16 bits as uint16) to float32."""
    x = np.asarray(x)
    if x.dtype == np.uint16:
        return bf16_to_f32(x)
    if x.dtype == np.float16:
        return x.astype(np.float32)
    if x.dtype != np.float32:
        raise TypeError(f"oracle tensors are float32, float16 or uint16(bf16); got {x.dtype}")
    return x


def is_bf16(x: np.ndarray) -> bool:
    return np.asarray(x).dtype == np.uint16


def square_in_dtype_of(x: np.ndarray, xf: np.ndarray) -> np.ndarray:
    """mlx square of the tensor ``x`` (``xf`` = its float32 widening), widened back to float32.

    ``square`` is a unary MLX op and keeps its operand's dtype (crates/mlx-sys/src/mlx.cpp:2016-2020):
    the square of a bf16 / float16 tensor is a bf16 / float16 tensor, and only the scalar multiply that
    follows promotes it.  x*x is exact in float32 for 16-bit x, so one rounding gives that tensor
    (torch's bf16/float16 ``square`` agrees bit for bit: tests/test_oracle_library.py).
    """
    sq = xf * xf
    x = np.asarray(x)
    if x.dtype == np.uint16:
        return bf16_to_f32(f32_to_bf16(sq))
    if x.dtype == np.float16:
        with np.errstate(over="ignore"):
            return sq.astype(np.float16).astype(np.float32)
    return sq


# --------------------------------------------------------------------------
# Optimizers  (crates/mlx-core/src/optimizers/{adam,adamw,sgd,rmsprop}.rs)
# --------------------------------------------------------------------------

class Adam:
    """optimizers/adam.rs:41-153.  ``step`` counts update_single CALLS (adam.rs:73)."""

    def __init__(self, learning_rate: Optional[float] = None, beta1: Optional[float] = None,
                 beta2: Optional[float] = None, eps: Optional[float] = None,
                 bias_correction: Optional[bool] = None):
        self.learning_rate = 1e-3 if learning_rate is None else float(learning_rate)
        self.beta1 = 0.9 if beta1 is None else float(beta1)
        self.beta2 = 0.999 if beta2 is None else float(beta2)
        self.eps = 1e-8 if eps is None else float(eps)
        self.bias_correction = False if bias_correction is None else bool(bias_correction)
        self.step = 0
        self.state: Dict[str, Tuple[np.ndarray, np.ndarray]] = {}

    def _decayed(self, p: np.ndarray) -> np.ndarray:
        return p

    def update_single(self, param_name: str, param: np.ndarray, grad: np.ndarray) -> np.ndarray:
        p = as_f32(param)
        g = as_f32(grad)
        if param_name not in self.state:  # init_state: float32 zeros (adam.rs:148-153)
            self.state[param_name] = (np.zeros(p.shape, F32), np.zeros(p.shape, F32))
        self.step += 1
        m, v = self.state[param_name]

        pd = self._decayed(p)
        beta1_m = m * _f32(self.beta1)
        omb1_g = g * _f32(1.0 - self.beta1)
        new_m = beta1_m + omb1_g
        g_sq = square_in_dtype_of(grad, g)         # mlx square: in the gradient's own dtype
        beta2_v = v * _f32(self.beta2)
        omb2_g2 = g_sq * _f32(1.0 - self.beta2)
        new_v = beta2_v + omb2_g2
        if self.bias_correction:
            t = float(self.step)
            bc1 = 1.0 / (1.0 - math.pow(self.beta1, t))
            bc2 = 1.0 / (1.0 - math.pow(self.beta2, t))
            m_hat = new_m * _f32(bc1)
            v_hat = new_v * _f32(bc2)
        else:
            m_hat, v_hat = new_m, new_v
        sqrt_v = np.sqrt(v_hat)
        denom = sqrt_v + _f32(self.eps)
        with np.errstate(divide="ignore", invalid="ignore"):
            update = m_hat / denom
        lr_update = update * _f32(self.learning_rate)
        new_p = pd - lr_update
        self.state[param_name] = (new_m, new_v)    # UNcorrected moments are stored
        return new_p

    def reset(self) -> None:
        self.state.clear()
        self.step = 0


class AdamW(Adam):
    """optimizers/adamw.rs:43-157: Adam plus the decoupled decay multiply (adamw.rs:83-84)."""

    def __init__(self, learning_rate=None, beta1=None, beta2=None, eps=None,
                 weight_decay: Optional[float] = None, bias_correction=None):
        super().__init__(learning_rate, beta1, beta2, eps, bias_correction)
        self.weight_decay = 0.01 if weight_decay is None else float(weight_decay)

    def _decayed(self, p: np.ndarray) -> np.ndarray:
        return p * _f32(1.0 - self.learning_rate * self.weight_decay)


class SGD:
    """optimizers/sgd.rs:40-159."""

    def __init__(self, learning_rate: float, momentum: Optional[float] = None,
                 weight_decay: Optional[float] = None, dampening: Optional[float] = None,
                 nesterov: Optional[bool] = None):
        momentum = 0.0 if momentum is None else float(momentum)
        dampening = 0.0 if dampening is None else float(dampening)
        nesterov = False if nesterov is None else bool(nesterov)
        if nesterov and (momentum <= 0.0 or dampening != 0.0):     # sgd.rs:51-56
            raise ValueError("Nesterov momentum requires momentum > 0 and dampening = 0")
        self.learning_rate = float(learning_rate)
        self.momentum = momentum
        self.weight_decay = 0.0 if weight_decay is None else float(weight_decay)
        self.dampening = dampening
        self.nesterov = nesterov
        self.state: Dict[str, Optional[np.ndarray]] = {}

    def update_single(self, param_name: str, param: np.ndarray, grad: np.ndarray) -> np.ndarray:
        p = as_f32(param)
        g = as_f32(grad)
        self.state.setdefault(param_name, None)
        if self.weight_decay != 0.0:                                # sgd.rs:86-94
            ge = g + p * _f32(self.weight_decay)
        else:
            ge = g
        if self.momentum != 0.0:
            v = self.state[param_name]
            if v is not None:                                       # sgd.rs:98-106
                new_v = v * _f32(self.momentum) + ge * _f32(1.0 - self.dampening)
            else:                                                   # first call: copy (sgd.rs:107-114)
                new_v = ge * _f32(1.0)
            if self.nesterov:                                       # sgd.rs:117-125
                final = new_v + ge
            else:
                final = new_v
            self.state[param_name] = final                          # sgd.rs:130 stores final_update
            update = final
        else:
            update = ge
        return p - update * _f32(self.learning_rate)                # sgd.rs:139-140

    def reset(self) -> None:
        self.state.clear()


class RMSprop:
    """optimizers/rmsprop.rs:36-127."""

    def __init__(self, learning_rate: Optional[float] = None, alpha: Optional[float] = None,
                 eps: Optional[float] = None, weight_decay: Optional[float] = None):
        self.learning_rate = 1e-2 if learning_rate is None else float(learning_rate)
        self.alpha = 0.99 if alpha is None else float(alpha)
        self.eps = 1e-8 if eps is None else float(eps)
        self.weight_decay = 0.0 if weight_decay is None else float(weight_decay)
        self.state: Dict[str, np.ndarray] = {}

    def update_single(self, param_name: str, param: np.ndarray, grad: np.ndarray) -> np.ndarray:
        p = as_f32(param)
        g = as_f32(grad)
        if param_name not in self.state:
            self.state[param_name] = np.zeros(p.shape, F32)
        v = self.state[param_name]
        if self.weight_decay != 0.0:                                # rmsprop.rs:69-77
            ge = g + p * _f32(self.weight_decay)
            g_sq = ge * ge                                          # of a float32 tensor
        else:
            ge = g
            g_sq = square_in_dtype_of(grad, g)                      # of the gradient as it came (rmsprop.rs:80)
        new_v = v * _f32(self.alpha) + g_sq * _f32(1.0 - self.alpha)  # rmsprop.rs:80-83
        denom = np.sqrt(new_v) + _f32(self.eps)                     # rmsprop.rs:86-88
        with np.errstate(divide="ignore", invalid="ignore"):
            update = ge / denom                                     # rmsprop.rs:91
        new_p = p - update * _f32(self.learning_rate)               # rmsprop.rs:92-93
        self.state[param_name] = new_v
        return new_p

    def reset(self) -> None:
        self.state.clear()


# --------------------------------------------------------------------------
# Gradient utilities  (optimizers/mod.rs:33-227, gradients/mod.rs:233-312)
# --------------------------------------------------------------------------

def exact_sumsq(grads: Iterable[np.ndarray]) -> float:
    """Sum of squares of the stored gradient values, accumulated in float64."""
    total = 0.0
    for g in grads:
        x = as_f32(g).astype(np.float64).ravel()
        total += float(np.dot(x, x))
    return total


def clip_value(grad: np.ndarray, lo: float, hi: float) -> np.ndarray:
    """``clip`` with float32 bounds (mlx.cpp:469-481); a non-finite bound is 'no bound'.
    Returns float32.  NaN elements stay NaN."""
    g = as_f32(grad)
    out = g
    if math.isfinite(lo):
        out = np.where(np.isnan(out), out, np.maximum(out, _f32(lo)))
    if math.isfinite(hi):
        out = np.where(np.isnan(out), out, np.minimum(out, _f32(hi)))
    return out.astype(F32, copy=False)


def norm_scale_c1(sumsq: float, max_norm: float) -> Tuple[np.float32, np.float32]:
    """(norm, scale) of ``GradientUtils::clip_grad_norm`` (optimizers/mod.rs:87-96):
    n = sqrt(S) in float32, scale = min(f32(max) / (n + f32(1e-6)), 1.0f)."""
    n = np.float32(math.sqrt(sumsq))
    with np.errstate(divide="ignore", over="ignore"):
        scale = np.minimum(_f32(max_norm) / (n + _f32(1e-6)), F32(1.0))
    return n, F32(scale)


class GradientUtils:
    """optimizers/mod.rs:33-227."""

    @staticmethod
    def compute_gradient_norm(gradients: Dict[str, np.ndarray]) -> float:
        """optimizers/mod.rs:43-55: float64 sum of squares of the float32 read-back."""
        return math.sqrt(exact_sumsq(gradients.values()))

    @staticmethod
    def clip_grad_norm(gradients: Dict[str, np.ndarray], max_norm: float) -> Dict[str, np.ndarray]:
        """optimizers/mod.rs:67-107.  Every tensor is multiplied by the scale, also when it is 1."""
        if not gradients:
            return {}
        _, scale = norm_scale_c1(exact_sumsq(gradients.values()), max_norm)
        return {k: as_f32(g) * scale for k, g in gradients.items()}

    @staticmethod
    def clip_grad_norm_with_norm(gradients, max_norm):
        """optimizers/mod.rs:116-158: also returns the float32 norm widened to float64."""
        if not gradients:
            return {}, 0.0
        n, scale = norm_scale_c1(exact_sumsq(gradients.values()), max_norm)
        return {k: as_f32(g) * scale for k, g in gradients.items()}, float(n)

    @staticmethod
    def clip_grad_value(grad: np.ndarray, min_val: float, max_val: float) -> np.ndarray:
        """optimizers/mod.rs:164-166."""
        return clip_value(grad, min_val, max_val)

    @staticmethod
    def clip_grad_value_and_norm(gradients, clip_val: float, max_norm: Optional[float]):
        """optimizers/mod.rs:174-226: clamp to +-clip_val, then clip_grad_norm of the clamped values."""
        if not gradients:
            return {}
        clamped = {k: clip_value(g, -clip_val, clip_val) for k, g in gradients.items()}
        if max_norm is None:
            return clamped
        _, scale = norm_scale_c1(exact_sumsq(clamped.values()), max_norm)
        return {k: g * scale for k, g in clamped.items()}


def clip_gradients_by_global_norm(gradients: Sequence[np.ndarray], max_norm: float) -> List[np.ndarray]:
    """gradients/mod.rs:233-285: float64 norm on the host; unchanged copies when n <= max,
    otherwise multiply by f32(max / (n + 1e-6)) evaluated in float64."""
    if not gradients:
        return []
    n = math.sqrt(exact_sumsq(gradients))
    if n <= max_norm:
        return [np.array(g, copy=True) for g in gradients]
    scale = _f32(max_norm / (n + 1e-6))
    return [as_f32(g) * scale for g in gradients]


def clip_gradients_by_value(gradients: Sequence[np.ndarray], lo: float, hi: float) -> List[np.ndarray]:
    """gradients/mod.rs:299-312."""
    return [clip_value(g, lo, hi) for g in gradients]


# --------------------------------------------------------------------------
# Accumulation and plain-SGD apply
# --------------------------------------------------------------------------

def _add_promoted(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """MLX ``add`` of two tensors: result dtype = promote(a, b).  bf16 + bf16 is one
    float32 add rounded to bf16; any float32 operand makes the result float32."""
    s = as_f32(a) + as_f32(b)
    if is_bf16(a) and is_bf16(b):
        return f32_to_bf16(s)
    return s


def accumulate_gradients(accumulated: Dict[str, np.ndarray], new: Dict[str, np.ndarray]) -> Dict[str, np.ndarray]:
    """Qwen3Model::accumulate_gradients, models/qwen3/model.rs:2217-2243 (also the engine's
    variant, grpo/engine.rs:2632-2666, which differs only in when it evaluates)."""
    out: Dict[str, np.ndarray] = {}
    for name, g in new.items():
        if name in accumulated:
            out[name] = _add_promoted(accumulated[name], g)
        else:
            out[name] = np.array(g, copy=True)
    for name, a in accumulated.items():
        if name not in out:
            out[name] = np.array(a, copy=True)
    return out


def accumulate_gradients_sft(accumulated: Optional[Dict[str, np.ndarray]], new: Dict[str, np.ndarray]):
    """sft/engine.rs:282-290: names missing from the accumulator are silently dropped."""
    if accumulated is None:
        return {k: np.array(v, copy=True) for k, v in new.items()}
    out = dict(accumulated)
    for name, g in new.items():
        if name in out:
            out[name] = _add_promoted(out[name], g)
    return out


def accumulate_fp32(acc: Optional[np.ndarray], grad: np.ndarray) -> np.ndarray:
    """Mixed-precision accumulation buffer: acc(float32) + widen(grad); first call = widen.
    (The intent stated at grpo/autograd.rs:317-318; the reference itself sums in grad dtype.)"""
    g = as_f32(grad)
    return g.astype(F32, copy=True) if acc is None else acc + g


def mul_scalar(x: np.ndarray, value: float) -> np.ndarray:
    """``mul_scalar`` (mlx.cpp:531-535): promotes to float32."""
    return as_f32(x) * _f32(value)


def apply_gradients(params: Dict[str, np.ndarray], gradients: Dict[str, np.ndarray],
                    learning_rate: float) -> Dict[str, np.ndarray]:
    """Qwen3Model::apply_gradients, models/qwen3/model.rs:2409-2460: plain SGD in the
    parameter's dtype.  lr is cast to the parameter dtype, lr*g and p-(lr*g) are each one
    rounded op in the promoted dtype, the result is cast back to the parameter dtype."""
    out: Dict[str, np.ndarray] = {}
    for name, g in gradients.items():
        if name not in params:
            raise KeyError(f"Parameter '{name}' not found in model")   # model.rs:2427-2432
        p = params[name]
        lr32 = _f32(learning_rate)
        if is_bf16(p):
            lr_p = bf16_to_f32(f32_to_bf16(np.array([lr32], F32)))[0]
            scaled = lr_p * as_f32(g)
            if is_bf16(g):
                scaled = bf16_to_f32(f32_to_bf16(scaled))              # bf16*bf16 -> bf16
                out[name] = f32_to_bf16(bf16_to_f32(p) - scaled)       # bf16-bf16 -> bf16
            else:
                out[name] = f32_to_bf16(bf16_to_f32(p) - scaled)       # fp32 result cast back
        else:
            out[name] = as_f32(p) - lr32 * as_f32(g)
    return out


# --------------------------------------------------------------------------
# The optimizer side of the training engines (what runs between the backward pass and the
# next forward pass): grpo/engine.rs:561-704 (and :1691-1790), sft/engine.rs:215-371, :459-553
# --------------------------------------------------------------------------

class TrainingStopped(RuntimeError):
    """Error::new(Status::GenericFailure, "Training stopped: exceeded ...") of both engines."""


def _has_invalid(g: np.ndarray) -> bool:
    """grpo/engine.rs:563-569: any NaN or Inf element of the float32 read-back."""
    return not bool(np.isfinite(as_f32(g)).all())


class _EngineState:
    """EngineState (grpo/engine.rs:227-271, sft/engine.rs:114-145), optimizer-side fields only."""

    def __init__(self):
        self.accumulated: Optional[Dict[str, np.ndarray]] = None
        self.micro_step = 0
        self.step = 0
        self.nan_gradient_count = 0
        self.consecutive_nan_count = 0
        self.needs_emergency_save = False


class _EngineBase:
    def __init__(self, params: Dict[str, np.ndarray], learning_rate, gradient_accumulation_steps,
                 gradient_clip_norm, gradient_clip_value, weight_decay, max_nan_gradients,
                 emergency_save_threshold, apply, beta1, beta2, eps):
        self.params = dict(params)
        self.learning_rate = learning_rate
        self.n_acc = 1 if gradient_accumulation_steps is None else int(gradient_accumulation_steps)
        self.clip_norm = gradient_clip_norm
        self.clip_value = gradient_clip_value
        self.weight_decay = weight_decay
        self.max_nan = 100 if max_nan_gradients is None else int(max_nan_gradients)
        self.emergency_threshold = 5 if emergency_save_threshold is None else int(emergency_save_threshold)
        self.apply = apply
        self.adamw = AdamW(learning_rate, beta1, beta2, eps, weight_decay) if apply == "adamw" else None
        self.state = _EngineState()

    # getters of both engines (grpo/engine.rs:2460-2600, sft/engine.rs:590-625)
    @property
    def step(self): return self.state.step
    @property
    def micro_step(self): return self.state.micro_step
    @property
    def nan_gradient_count(self): return self.state.nan_gradient_count
    @property
    def needs_emergency_save(self): return self.state.needs_emergency_save

    def clear_emergency_save_flag(self) -> None:
        self.state.needs_emergency_save = False

    def reset(self) -> None:
        """grpo/engine.rs:2533-2546, sft/engine.rs:671-: *state = EngineState::default().  With this
        build's AdamW apply the moments go too, as after the optimizers' own reset() (adamw.rs:146-150)."""
        self.state = _EngineState()
        if self.adamw is not None:
            self.adamw.reset()

    def _adamw_apply(self, grads: Dict[str, np.ndarray]) -> None:
        """This build's replacement for apply_gradients: AdamW on the prepared gradient, parameter
        written back in its own dtype with one round-to-nearest-even."""
        for name, g in grads.items():
            if name not in self.params:
                raise KeyError(f"Parameter '{name}' not found in model")
            p = self.params[name]
            new_p = self.adamw.update_single(name, p, g)
            self.params[name] = f32_to_bf16(new_p) if is_bf16(p) else new_p


class GRPOEngineOptimizerSide(_EngineBase):
    """GRPOTrainingEngine, everything after the backward pass of one micro-batch
    (grpo/engine.rs:561-704; :1691-1790 is the same arithmetic through clip_grad_value_and_norm).
    ``gradient_clip_norm=None`` means no norm clipping (the config default is Some(1.0));
    ``gradient_clip_value=None`` means 1.0 (engine.rs:636)."""

    def __init__(self, params, learning_rate: Optional[float] = None, gradient_accumulation_steps: Optional[int] = None,
                 gradient_clip_norm: Optional[float] = 1.0, gradient_clip_value: Optional[float] = None,
                 max_nan_gradients: Optional[int] = None, emergency_save_threshold: Optional[int] = None,
                 apply: str = "sgd", weight_decay: float = 0.01, beta1: float = 0.9, beta2: float = 0.999,
                 eps: float = 1e-8):
        super().__init__(params, 1e-6 if learning_rate is None else learning_rate, gradient_accumulation_steps,
                         gradient_clip_norm, 1.0 if gradient_clip_value is None else gradient_clip_value,
                         weight_decay, max_nan_gradients, emergency_save_threshold, apply, beta1, beta2, eps)

    def micro_batch(self, gradients: Dict[str, np.ndarray], norm_sumsq: Optional[float] = None) -> Dict[str, object]:
        """One micro-batch of gradients.  ``norm_sumsq``: use this sum of squares of the clamped
        gradients in place of the exact one (a checker passes the device's own value, which it has
        compared with the exact one, so that the comparison downstream can be bit for bit)."""
        st = self.state
        # Step 1 (engine.rs:561-633): any NaN/Inf anywhere => skip the whole micro-batch
        if any(_has_invalid(g) for g in gradients.values()):
            st.nan_gradient_count += 1
            st.consecutive_nan_count += 1
            if st.nan_gradient_count >= self.max_nan:                          # engine.rs:588-596
                raise TrainingStopped(f"Training stopped: exceeded maximum NaN gradient count "
                                      f"({st.nan_gradient_count}/{self.max_nan})")
            if st.consecutive_nan_count >= self.emergency_threshold:           # engine.rs:599-606
                st.needs_emergency_save = True
            st.step += 1                                                       # engine.rs:608
            return {"step": st.step, "gradients_applied": False, "skipped": True}
        # Step 2 (engine.rs:636-644): clamp; Step 3 (:647-653): clip by global norm of the clamped values
        clamped = {k: clip_value(g, -self.clip_value, self.clip_value) for k, g in gradients.items()}
        if self.clip_norm is not None:
            sumsq = exact_sumsq(clamped.values()) if norm_sumsq is None else norm_sumsq
            _, scale = norm_scale_c1(sumsq, self.clip_norm)
            grads = {k: g * scale for k, g in clamped.items()}
        else:
            grads = clamped
        st.consecutive_nan_count = 0                                           # engine.rs:660
        # engine.rs:2632-2666
        if st.accumulated is None:
            st.accumulated = dict(grads)
        else:
            for name, g in grads.items():
                st.accumulated[name] = _add_promoted(st.accumulated[name], g) if name in st.accumulated else g
        st.micro_step += 1
        applied = False
        if st.micro_step >= self.n_acc:                                        # engine.rs:666-692
            acc, st.accumulated = st.accumulated, None
            if self.apply == "adamw":
                self._adamw_apply({k: mul_scalar(g, 1.0 / self.n_acc) for k, g in acc.items()})
            else:
                self.params.update(apply_gradients(self.params, acc, self.learning_rate / self.n_acc))
            st.micro_step = 0
            applied = True
        st.step += 1                                                           # engine.rs:690, :696
        return {"step": st.step, "gradients_applied": applied, "skipped": False}


class SFTEngineOptimizerSide(_EngineBase):
    """SftTrainingEngine, everything after the backward pass of one micro-batch
    (sft/engine.rs:268-371) plus flush_gradients (:459-553) and the NaN-loss bookkeeping
    (:221-258).  ``gradient_clip_norm=None`` / ``gradient_clip_value=None`` mean "not configured"."""

    def __init__(self, params, learning_rate: Optional[float] = None, gradient_accumulation_steps: Optional[int] = None,
                 gradient_clip_norm: Optional[float] = 1.0, gradient_clip_value: Optional[float] = None,
                 weight_decay: Optional[float] = None, max_nan_gradients: Optional[int] = None,
                 emergency_save_threshold: Optional[int] = None, apply: str = "sgd", beta1: float = 0.9,
                 beta2: float = 0.999, eps: float = 1e-8):
        super().__init__(params, 2e-5 if learning_rate is None else learning_rate, gradient_accumulation_steps,
                         gradient_clip_norm, gradient_clip_value, 0.0 if weight_decay is None else weight_decay,
                         max_nan_gradients, emergency_save_threshold, apply, beta1, beta2, eps)

    def report_nonfinite_loss(self) -> int:
        """sft/engine.rs:221-258: the loss was NaN/Inf, nothing is accumulated."""
        st = self.state
        st.nan_gradient_count += 1
        st.consecutive_nan_count += 1
        if st.consecutive_nan_count >= self.emergency_threshold:
            st.needs_emergency_save = True
        if st.nan_gradient_count >= self.max_nan:
            raise TrainingStopped(f"Training stopped: exceeded {self.max_nan} NaN gradient limit")
        return st.step

    def micro_batch(self, gradients: Dict[str, np.ndarray], norm_sumsq: Optional[float] = None) -> Dict[str, object]:
        st = self.state
        st.consecutive_nan_count = 0                                           # sft/engine.rs:261-267
        st.accumulated = accumulate_gradients_sft(st.accumulated, gradients)   # :282-290
        st.micro_step += 1
        applied = False
        if st.micro_step >= self.n_acc:
            self._apply(self.n_acc, norm_sumsq)
            applied = True
        return {"step": st.step, "gradients_applied": applied, "skipped": False}

    def flush_gradients(self, norm_sumsq: Optional[float] = None) -> bool:
        """sft/engine.rs:459-553: leftover micro-batches are averaged by their actual count."""
        st = self.state
        if st.micro_step == 0 or st.accumulated is None:
            return False
        self._apply(st.micro_step, norm_sumsq)
        return True

    def _apply(self, count: int, norm_sumsq: Optional[float]) -> None:
        st = self.state
        acc, st.accumulated = st.accumulated, None
        averaged = {k: mul_scalar(g, 1.0 / count) for k, g in acc.items()}     # :297-305
        if self.clip_norm is not None:                                         # :308-314
            sumsq = exact_sumsq(averaged.values()) if norm_sumsq is None else norm_sumsq
            _, scale = norm_scale_c1(sumsq, self.clip_norm)
            averaged = {k: g * scale for k, g in averaged.items()}
        if self.clip_value is not None:                                        # :317-329
            averaged = {k: clip_value(g, -self.clip_value, self.clip_value) for k, g in averaged.items()}
        if self.apply == "adamw":
            self._adamw_apply(averaged)                                        # decoupled decay inside AdamW
        else:
            if self.weight_decay > 0.0:                                        # :345-365
                averaged = {k: (g + mul_scalar(self.params[k], self.weight_decay)) if k in self.params else g
                            for k, g in averaged.items()}
            self.params.update(apply_gradients(self.params, averaged, self.learning_rate))
        st.step += 1
        st.micro_step = 0


# --------------------------------------------------------------------------
# Synthetic inputs: the host twin of the library's counter-based generator (its definition is in
# include/mxopt.h at mxopt_fill_synthetic).  Not part of the reference; it lets a checker regenerate
# any slice of any benchmark input without copying it.
# --------------------------------------------------------------------------

_M64 = (1 << 64) - 1
SYNTH_NORMAL, SYNTH_NORMAL_OUTLIERS, SYNTH_UNIFORM, SYNTH_GAUSSIAN, SYNTH_GAUSSIAN_OUTLIERS = 0, 1, 2, 3, 4
_GAUSS_TABLE: Optional[np.ndarray] = None


def gauss_quantile_table() -> np.ndarray:
    """The 32 x 33 float32 quantile table of the Gaussian modes, read from the header the device code
    compiles (mlx-node_amd/csrc/mxopt_gauss_table.h: hexadecimal literals, exact)."""
    global _GAUSS_TABLE
    if _GAUSS_TABLE is None:
        import os
        import re
        path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mlx-node_amd", "csrc",
                            "mxopt_gauss_table.h")
        vals = [float.fromhex(h) for h in re.findall(r"(-?0x[0-9a-f.]+p[+-]\d+)f", open(path).read())]
        _GAUSS_TABLE = np.array(vals, dtype=np.float64).astype(F32).reshape(32, 33)
    return _GAUSS_TABLE


def _gauss_magnitude(u: np.ndarray) -> np.ndarray:
    """|x| for the 32-bit tail code u (see MXOPT_SYNTH_GAUSSIAN in include/mxopt.h): three float32 ops."""
    t = gauss_quantile_table()
    u = np.where(u == 0, 1, u).astype(np.uint64)
    _, e = np.frexp(u.astype(np.float64))            # u in [2^(e-1), 2^e): exact for 32-bit integers
    k = (32 - e).astype(np.int64)                     # leading zeros
    v = (u << k.astype(np.uint64)) & np.uint64(0xFFFFFFFF)
    j = ((v >> np.uint64(26)) & np.uint64(31)).astype(np.int64)
    f = ((v >> np.uint64(10)) & np.uint64(0xFFFF)).astype(F32) * F32(2.0 ** -16)
    t0 = t[k, j]
    d = t[k, j + 1] - t0
    step = d * f
    return t0 + step


def _splitmix_finish(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def synthetic_hash(seed: int, index: np.ndarray) -> np.ndarray:
    idx = np.asarray(index, dtype=np.uint64)
    with np.errstate(over="ignore"):
        return _splitmix_finish(np.uint64(seed & _M64) + (idx + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15))


def synthetic_key(seed: int, config: int = 0, step: int = 0, micro_batch: int = 0, tensor_index: int = 0) -> int:
    z = ((seed ^ config ^ (step << 32) ^ (micro_batch << 48) ^ tensor_index) + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def synthetic(n: int, dtype: str, seed: int, distribution: int = SYNTH_NORMAL, a: float = 1.0, b: float = 0.0,
              first_index: int = 0) -> np.ndarray:
    """Elements first_index .. first_index+n-1 of the stream `seed`; dtype "f32", "bf16" (uint16 bits) or "f16"."""
    idx = np.arange(first_index, first_index + n, dtype=np.uint64)
    z = synthetic_hash(seed, idx)
    if distribution == SYNTH_UNIFORM:
        x = (z >> np.uint64(40)).astype(F32) * _f32((b - a) / 16777216.0)
        x = x + _f32(a)
    elif distribution in (SYNTH_GAUSSIAN, SYNTH_GAUSSIAN_OUTLIERS):
        mag = _gauss_magnitude((z >> np.uint64(31)) & np.uint64(0xFFFFFFFF))
        x = np.where((z >> np.uint64(63)) != 0, -mag, mag).astype(F32)
        x = x * _f32(a)
        if distribution == SYNTH_GAUSSIAN_OUTLIERS:
            hit = synthetic_hash(seed ^ 0xA5A5A5A5A5A5A5A5, idx) % np.uint64(100) == np.uint64(0)
            x = np.where(hit, x * _f32(b), x).astype(F32)
    else:
        m = np.uint64(0xFFFF)
        total = ((z & m) + ((z >> np.uint64(16)) & m) + ((z >> np.uint64(32)) & m) + (z >> np.uint64(48))).astype(np.int64)
        x = (total - 131070).astype(F32) * _f32(a / math.sqrt((65536.0 * 65536.0 - 1.0) / 3.0))
        if distribution == SYNTH_NORMAL_OUTLIERS:
            hit = synthetic_hash(seed ^ 0xA5A5A5A5A5A5A5A5, idx) % np.uint64(100) == np.uint64(0)
            x = np.where(hit, x * _f32(b), x).astype(F32)
    if dtype == "bf16":
        return f32_to_bf16(x)
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16)
    return x.astype(F32, copy=False)


# --------------------------------------------------------------------------
# Learning-rate schedules  (optimizers/mod.rs:239-292) -- host float64 closed forms
# --------------------------------------------------------------------------

def _idiv(a: int, b: int) -> int:
    """Rust i64 division truncates toward zero."""
    q = abs(a) // abs(b)
    return q if (a >= 0) == (b >= 0) else -q


class LRScheduler:
    @staticmethod
    def linear_decay(initial_lr: float, final_lr: float, current_step: int, total_steps: int) -> float:
        if current_step >= total_steps:
            return final_lr
        return initial_lr + (final_lr - initial_lr) * (current_step / total_steps)

    @staticmethod
    def exponential_decay(initial_lr: float, decay_rate: float, current_step: int, decay_steps: int) -> float:
        # integer division of the step counters (optimizers/mod.rs:263)
        return initial_lr * math.pow(decay_rate, float(_idiv(current_step, decay_steps)))

    @staticmethod
    def cosine_annealing(initial_lr: float, min_lr: float, current_step: int, total_steps: int) -> float:
        if current_step >= total_steps:
            return min_lr
        progress = current_step / total_steps
        return min_lr + (initial_lr - min_lr) * 0.5 * (1.0 + math.cos(progress * math.pi))

    @staticmethod
    def step_decay(initial_lr: float, factor: float, current_step: int, step_size: int) -> float:
        return initial_lr * (factor ** _idiv(current_step, step_size))


# --------------------------------------------------------------------------
# Helpers used by parity tests
# --------------------------------------------------------------------------

def ulp_diff_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in float32 units-in-the-last-place (monotone integer mapping)."""
    def key(x):
        i = np.ascontiguousarray(x, dtype=np.float32).view(np.int32).astype(np.int64)
        return np.where(i < 0, np.int64(-(2 ** 31)) - i, i)
    return np.abs(key(a) - key(b))


def ulp_diff_bf16(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    def key(x):
        i = np.asarray(x, dtype=np.uint16).view(np.int16).astype(np.int64)
        return np.where(i < 0, np.int64(-(2 ** 15)) - i, i)
    return np.abs(key(a_bits) - key(b_bits))
