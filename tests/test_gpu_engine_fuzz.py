"""Random call sequences against both engines' optimizer side: micro-batches with all or some of the
names, poisoned micro-batches (GRPO), flushes and NaN-loss reports (SFT), resets -- with and without
an accumulation buffer, plain-SGD and AdamW apply, bf16 and float32, the GRPO call blocking or asynchronous.  After every call parameters
(bit for bit), counters and flags must equal the oracle's.  Derandomised; MXOPT_PROPERTY_EXAMPLES=<n>
draws n fresh random sequences instead."""
import math
import os

import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
SIZES = {"embed": 12289, "ln": 64, "tiny": 7, "w1": 4097, "w2": 1}
SOAK = int(os.environ.get("MXOPT_PROPERTY_EXAMPLES", "0"))
OPS = st.sampled_from(["mb", "mb", "mb", "mb", "partial", "poison", "flush", "nanloss", "reset"])


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


def check_state(dev, ref, dparams, what):
    m, s = dev.metrics(), ref.state
    assert (m.step, m.micro_step, m.nan_gradient_count, m.consecutive_nan_count, bool(m.needs_emergency_save)) == \
           (s.step, s.micro_step, s.nan_gradient_count, s.consecutive_nan_count, s.needs_emergency_save), what
    for k in dparams:
        assert_bit_equal(to_host(dparams[k]), ref.params[k], f"{what}: {k}")


def both(what, dev_call, ref_call, mx):
    """Runs the device call, then the oracle call (which may need the device's result); both must stop
    training, or neither."""
    stopped = [None, None]
    out = None
    try:
        out = dev_call()
    except mx.TrainingStopped as e:
        stopped[0] = str(e)
    try:
        ref_call(out)
    except O.TrainingStopped as e:
        stopped[1] = str(e)
    assert (stopped[0] is None) == (stopped[1] is None), (what, stopped)
    if stopped[0] is not None:
        assert stopped[1] in stopped[0], (what, stopped)
    return out


@settings(max_examples=SOAK or 120, deadline=None, derandomize=not SOAK, database=None,
          suppress_health_check=list(HealthCheck))
@given(kind=st.sampled_from(["grpo", "sft"]), bf16=st.booleans(), apply=st.sampled_from(["sgd", "adamw"]),
       n_acc=st.sampled_from([1, 2, 3, 5, 9]), defer=st.booleans(), acc_f32=st.booleans(),
       clip_norm=st.sampled_from([None, 0.5]), clip_value=st.sampled_from([None, 0.003]),
       wd=st.sampled_from([0.0, 0.01]), ops=st.lists(OPS, min_size=1, max_size=22), seed=st.integers(0, 2 ** 31),
       use_async=st.booleans())
def test_random_engine_sequences(mx, kind, bf16, apply, n_acc, defer, acc_f32, clip_norm, clip_value, wd, ops, seed,
                                 use_async):
    rng = np.random.default_rng(seed)
    if kind == "grpo" and defer:
        apply = "sgd"
    if kind == "sft" and defer:
        acc_f32 = True
    cast = O.f32_to_bf16 if bf16 else (lambda a: a)
    params = {k: cast(rng.normal(0, 0.5, n).astype(F)) for k, n in SIZES.items()}
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.03, gradient_accumulation_steps=n_acc, gradient_clip_norm=clip_norm,
              gradient_clip_value=clip_value, max_nan_gradients=4, emergency_save_threshold=2, apply=apply,
              weight_decay=wd)
    if kind == "grpo":
        dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=defer, **kw)
        ref = O.GRPOEngineOptimizerSide(params, **kw)
    else:
        dev = mx.SFTEngineOptimizerSide(dparams, accumulate_in_f32=acc_f32, defer_accumulation=defer, **kw)
        ref = O.SFTEngineOptimizerSide(params, **kw)
    widen = (lambda g: O.as_f32(g)) if (kind == "sft" and acc_f32) else (lambda g: g)
    cv = 1.0 if (kind == "grpo" and clip_value is None) else clip_value

    for it, op in enumerate(ops):
        what = f"call {it} ({op})"
        if op in ("mb", "partial", "poison"):
            names = list(SIZES)
            if op == "partial" and not defer:
                names = [k for k in names if rng.random() < 0.6] or ["w1"]
            grads = {k: cast(rng.normal(0, 0.004 * (1 + it % 3), SIZES[k]).astype(F)) for k in names}
            poisoned = op == "poison" and kind == "grpo"
            if poisoned:
                k = names[int(rng.integers(0, len(names)))]
                v = O.as_f32(grads[k]).copy()
                v[int(rng.integers(0, v.size))] = [np.nan, np.inf, -np.inf][int(rng.integers(0, 3))]
                grads[k] = cast(v)
            boundary = ref.state.micro_step + 1 >= n_acc

            def ref_call(m, grads=grads, poisoned=poisoned, boundary=boundary):
                g = {k: widen(v) for k, v in grads.items()}
                measured = m is not None and m.norm_measured and clip_norm is not None
                if kind == "grpo":
                    if measured and not poisoned:
                        exact = O.exact_sumsq([O.clip_value(x, -cv, cv) for x in grads.values()])
                        assert abs(m.grad_sumsq - exact) <= 1e-5 * max(exact, 1e-300)
                        return ref.micro_batch(g, norm_sumsq=m.grad_sumsq)
                    return ref.micro_batch(g)
                return ref.micro_batch(g, norm_sumsq=m.grad_sumsq) if (measured and boundary) else ref.micro_batch(g)

            # GRPO with the plain-SGD apply also through the call that does not wait for the validity flag: booked as
            # valid, kernels guarded on the device, put right by settle()
            if use_async and kind == "grpo":
                def dev_call(grads=grads):
                    dev.micro_batch_async({k: to_dev(g) for k, g in grads.items()})
                    return dev.settle()
            else:
                def dev_call(grads=grads):
                    return dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
            m = both(what, dev_call, ref_call, mx)
            if m is not None and kind == "grpo":
                assert bool(m.skipped) == poisoned
        elif op == "flush":
            if kind != "sft":
                continue
            flushed = dev.flush_gradients()
            sumsq = dev.last_metrics.grad_sumsq if (flushed and clip_norm is not None) else None
            assert ref.flush_gradients(norm_sumsq=sumsq) is flushed
        elif op == "nanloss":
            if kind != "sft":
                continue
            both(what, dev.report_nonfinite_loss, lambda _m: ref.report_nonfinite_loss(), mx)
        else:
            dev.reset()
            ref.reset()
        check_state(dev, ref, dparams, what)
