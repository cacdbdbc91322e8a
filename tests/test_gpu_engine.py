"""GPU parity of the engines' optimizer side (include/mxopt_engine.h) against the oracle's restatement
of grpo/engine.rs:561-704 and sft/engine.rs:215-371, 459-553, through the C ABI: parameters bit for
bit after every micro-batch, counters and flags equal, the measured norm within rel 1e-5 of the exact
one (the oracle is then handed the device's sum of squares so that the clip factor is the same scalar)."""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
SIZES = {"embed": 100003, "ln": 64, "tiny": 7, "w1": 3 * 4096, "w2": 4097}


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


def make_params(rng, bf16):
    ps = {k: rng.normal(0, 0.5, n).astype(F) for k, n in SIZES.items()}
    return {k: O.f32_to_bf16(v) for k, v in ps.items()} if bf16 else ps


def make_grads(rng, bf16, std, names=SIZES):
    gs = {k: rng.normal(0, std, SIZES[k]).astype(F) for k in names}
    return {k: O.f32_to_bf16(v) for k, v in gs.items()} if bf16 else gs


def check_state(dev, ref, dparams, what):
    m = dev.metrics()
    st = ref.state
    assert (m.step, m.micro_step, m.nan_gradient_count, m.consecutive_nan_count, bool(m.needs_emergency_save)) == \
           (st.step, st.micro_step, st.nan_gradient_count, st.consecutive_nan_count, st.needs_emergency_save), what
    for k in dparams:
        assert_bit_equal(to_host(dparams[k]), ref.params[k], f"{what}: {k}")


def exact_clamped_sumsq(grads, cv):
    return O.exact_sumsq([O.clip_value(g, -cv, cv) for g in grads.values()])


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("apply", ["sgd", "adamw"])
@pytest.mark.parametrize("n_acc", [1, 3])
def test_grpo_sequence(mx, bf16, apply, n_acc):
    rng = np.random.default_rng(7 + n_acc)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=n_acc, gradient_clip_norm=2.0, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=2, apply=apply, weight_decay=0.01)
    dev = mx.GRPOEngineOptimizerSide(dparams, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    script = ["ok", "ok", "nan", "inf", "ok", "ok", "-inf", "ok", "ok", "ok"]
    for it, kind in enumerate(script):
        grads = make_grads(rng, bf16, 0.01 * (1 + it % 3))
        if kind != "ok":
            bad = {"nan": np.nan, "inf": np.inf, "-inf": -np.inf}[kind]
            v = O.as_f32(grads["w1"]).copy()
            v[4096 + 5] = bad                     # +-Inf would be clamped to a finite bound: the raw value counts
            grads["w1"] = O.f32_to_bf16(v) if bf16 else v
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        if kind == "ok":
            exact = exact_clamped_sumsq(grads, 0.02)
            assert m.norm_measured and abs(m.grad_norm - math.sqrt(exact)) <= 1e-5 * math.sqrt(exact)
            r = ref.micro_batch(grads, norm_sumsq=m.grad_sumsq)
            assert F(m.clip_scale) == O.norm_scale_c1(m.grad_sumsq, 2.0)[1]
        else:
            r = ref.micro_batch(grads)
        assert (bool(m.skipped), bool(m.gradients_applied), m.step) == (r["skipped"], r["gradients_applied"], r["step"])
        check_state(dev, ref, dparams, f"micro-batch {it} ({kind})")
    assert ref.state.nan_gradient_count == 3 and ref.needs_emergency_save
    dev.clear_emergency_save_flag()
    ref.clear_emergency_save_flag()
    dev.reset()
    ref.reset()
    check_state(dev, ref, dparams, "after reset")


def test_grpo_defaults_new_names_and_errors(mx):
    """Default config (lr 1e-6, clamp 1.0, clip 1.0, N 1); a name that shows up only in a later
    micro-batch of a cycle is inserted (engine.rs:2650-2654); unknown names are refused."""
    rng = np.random.default_rng(11)
    params = make_params(rng, True)
    dparams = {k: to_dev(v) for k, v in params.items()}
    dev = mx.GRPOEngineOptimizerSide(dparams, gradient_accumulation_steps=2, learning_rate=0.01)
    ref = O.GRPOEngineOptimizerSide(params, gradient_accumulation_steps=2, learning_rate=0.01)
    for names in (["embed", "w1"], ["embed", "w1", "ln", "tiny"], ["w2"], ["embed", "w2"]):
        grads = make_grads(rng, True, 0.4, names)          # large enough for clamp and clip to act
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        ref.micro_batch(grads, norm_sumsq=m.grad_sumsq)
        assert m.clip_scale < 1.0
        check_state(dev, ref, dparams, str(names))
    before = {k: to_host(v) for k, v in dparams.items()}
    with pytest.raises(KeyError, match="Parameter 'nope' not found in model"):
        dev.micro_batch({"embed": to_dev(np.zeros(SIZES["embed"], F)), "nope": to_dev(np.zeros(3, F))})
    with pytest.raises(ValueError):
        dev.micro_batch({"ln": to_dev(np.zeros(SIZES["ln"] + 1, F))})
    check_state(dev, ref, dparams, "after refused calls")
    for k in dparams:
        assert_bit_equal(to_host(dparams[k]), before[k], k)


def test_grpo_training_stopped(mx):
    params = {"w": np.ones(100, F)}
    dparams = {"w": to_dev(params["w"])}
    dev = mx.GRPOEngineOptimizerSide(dparams, max_nan_gradients=3)
    ref = O.GRPOEngineOptimizerSide(params, max_nan_gradients=3)
    bad = np.zeros(100, F)
    bad[3] = np.nan
    for _ in range(2):
        dev.micro_batch({"w": to_dev(bad)})
        ref.micro_batch({"w": bad})
    with pytest.raises(mx.TrainingStopped, match=r"exceeded maximum NaN gradient count \(3/3\)"):
        dev.micro_batch({"w": to_dev(bad)})
    with pytest.raises(O.TrainingStopped):
        ref.micro_batch({"w": bad})
    check_state(dev, ref, dparams, "after the limit")


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("apply", ["sgd", "adamw"])
@pytest.mark.parametrize("acc_f32", [False, True])
def test_sft_sequence(mx, bf16, apply, acc_f32):
    if acc_f32 and not bf16:
        pytest.skip("float32 gradients already accumulate in float32")
    rng = np.random.default_rng(23)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.02, gradient_accumulation_steps=3, gradient_clip_norm=0.5, gradient_clip_value=0.002,
              weight_decay=0.01, apply=apply)
    dev = mx.SFTEngineOptimizerSide(dparams, accumulate_in_f32=acc_f32, **kw)
    ref = O.SFTEngineOptimizerSide(params, **kw)
    widen = (lambda g: O.as_f32(g)) if acc_f32 else (lambda g: g)   # a float32 buffer = float32 gradients to the oracle
    for it in range(7):                                            # two full cycles + one leftover micro-batch
        names = list(SIZES) if it != 4 else ["embed", "w1"]        # a micro-batch that misses some names
        grads = make_grads(rng, bf16, 0.01, names)
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        boundary = ref.state.micro_step + 1 >= 3
        if boundary:
            assert m.norm_measured and m.gradients_applied
            r = ref.micro_batch({k: widen(g) for k, g in grads.items()}, norm_sumsq=m.grad_sumsq)
        else:
            r = ref.micro_batch({k: widen(g) for k, g in grads.items()})
        assert (bool(m.gradients_applied), m.step) == (r["gradients_applied"], r["step"])
        check_state(dev, ref, dparams, f"micro-batch {it}")
    assert ref.state.micro_step == 1
    assert dev.flush_gradients() is True
    assert ref.flush_gradients(norm_sumsq=dev.last_metrics.grad_sumsq) is True
    check_state(dev, ref, dparams, "after flush")
    assert dev.flush_gradients() is False and ref.flush_gradients() is False
    # NaN-loss bookkeeping
    for _ in range(5):
        dev.report_nonfinite_loss()
        ref.report_nonfinite_loss()
    check_state(dev, ref, dparams, "after NaN losses")
    assert dev.needs_emergency_save


def test_sft_norm_is_of_the_averaged_sum(mx):
    """The fused norm (last accumulation pass) and the separate one (a micro-batch that misses names)
    both describe acc / N."""
    rng = np.random.default_rng(31)
    params = make_params(rng, False)
    for partial_last in (False, True):
        dparams = {k: to_dev(v) for k, v in params.items()}
        dev = mx.SFTEngineOptimizerSide(dparams, gradient_accumulation_steps=2, gradient_clip_norm=1e-3, learning_rate=0.1)
        ref = O.SFTEngineOptimizerSide(params, gradient_accumulation_steps=2, gradient_clip_norm=1e-3, learning_rate=0.1)
        g1 = make_grads(rng, False, 0.01)
        g2 = make_grads(rng, False, 0.01, ["embed", "ln"] if partial_last else SIZES)
        dev.micro_batch({k: to_dev(g) for k, g in g1.items()})
        ref.micro_batch(g1)
        m = dev.micro_batch({k: to_dev(g) for k, g in g2.items()})
        acc = {k: g1[k] + g2[k] if k in g2 else g1[k] for k in g1}
        exact = O.exact_sumsq([a * F(0.5) for a in acc.values()])
        assert abs(m.grad_sumsq - exact) <= 1e-6 * exact
        ref.micro_batch(g2, norm_sumsq=m.grad_sumsq)
        check_state(dev, ref, dparams, f"partial_last={partial_last}")


@pytest.mark.parametrize("kind", ["grpo", "sft"])
@pytest.mark.parametrize("apply", ["sgd", "adamw"])
@pytest.mark.parametrize("bf16", [False, True])
def test_one_micro_batch_per_step(mx, kind, apply, bf16):
    """gradient_accumulation_steps = 1 (both engines' default): the gradient is applied from where it
    lies, no accumulator is involved."""
    rng = np.random.default_rng(41)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    if kind == "grpo":
        kw = dict(learning_rate=0.05, gradient_clip_norm=1.5, gradient_clip_value=0.03, apply=apply, weight_decay=0.02)
        dev, ref = mx.GRPOEngineOptimizerSide(dparams, **kw), O.GRPOEngineOptimizerSide(params, **kw)
    else:
        kw = dict(learning_rate=0.05, gradient_clip_norm=1.5, gradient_clip_value=0.003, apply=apply, weight_decay=0.02)
        dev, ref = mx.SFTEngineOptimizerSide(dparams, **kw), O.SFTEngineOptimizerSide(params, **kw)
    for it in range(4):
        names = list(SIZES) if it != 2 else ["embed", "tiny"]
        grads = make_grads(rng, bf16, 0.02, names)
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        assert m.gradients_applied and m.norm_measured and m.clip_scale < 1.0
        ref.micro_batch(grads, norm_sumsq=m.grad_sumsq)
        check_state(dev, ref, dparams, f"{kind} step {it}")


# ---------------------------------------------------------------------------------------
# defer_accumulation: no accumulation buffer, the micro-batches of a cycle are added in registers by
# the applying call.  The oracle is the unchanged (buffered) engine: every number must be the same.
# ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("n_acc", [1, 3, 4, 6, 8, 9, 11])
def test_grpo_deferred_sequence(mx, bf16, n_acc):
    """More than eight micro-batches in a cycle: the oldest are added into the float32 buffers as the later
    ones arrive (clamped and clipped by their own factors), the last seven stay deferred."""
    rng = np.random.default_rng(107 + n_acc)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=n_acc, gradient_clip_norm=2.0, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=2)
    dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=True, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    script = ["ok", "ok", "nan", "inf", "ok", "ok", "-inf", "ok", "ok", "ok", "ok", "ok", "ok", "ok", "ok"]
    script += ["ok", "nan"] + ["ok"] * 10 if n_acc > 6 else []
    for it, kind in enumerate(script):
        grads = make_grads(rng, bf16, 0.01 * (1 + it % 3))
        if kind != "ok":
            v = O.as_f32(grads["w1"]).copy()
            v[4096 + 5] = {"nan": np.nan, "inf": np.inf, "-inf": -np.inf}[kind]
            grads["w1"] = O.f32_to_bf16(v) if bf16 else v
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        if kind == "ok":
            exact = exact_clamped_sumsq(grads, 0.02)
            assert m.norm_measured and abs(m.grad_norm - math.sqrt(exact)) <= 1e-5 * math.sqrt(exact)
            r = ref.micro_batch(grads, norm_sumsq=m.grad_sumsq)
        else:
            r = ref.micro_batch(grads)
        assert (bool(m.skipped), bool(m.gradients_applied), m.step) == (r["skipped"], r["gradients_applied"], r["step"])
        if m.gradients_applied or n_acc == 1:
            check_state(dev, ref, dparams, f"micro-batch {it} ({kind})")
        else:   # inside a cycle the parameters have not moved on either side; the counters must agree
            st, mm = ref.state, dev.metrics()
            assert (mm.step, mm.micro_step, mm.nan_gradient_count) == (st.step, st.micro_step, st.nan_gradient_count)
    dev.reset()
    ref.reset()
    check_state(dev, ref, dparams, "after reset")


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("apply", ["sgd", "adamw"])
@pytest.mark.parametrize("n_acc", [3, 6, 9, 12])
def test_sft_deferred_sequence(mx, bf16, apply, n_acc):
    rng = np.random.default_rng(123)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.02, gradient_accumulation_steps=n_acc, gradient_clip_norm=0.5, gradient_clip_value=0.002,
              weight_decay=0.01, apply=apply)
    dev = mx.SFTEngineOptimizerSide(dparams, accumulate_in_f32=True, defer_accumulation=True, **kw)
    ref = O.SFTEngineOptimizerSide(params, **kw)
    for it in range(2 * n_acc + 2):                         # two full cycles + two leftover micro-batches
        grads = make_grads(rng, bf16, 0.01)
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        wide = {k: O.as_f32(g) for k, g in grads.items()}    # a float32 sum = float32 gradients to the oracle
        boundary = ref.state.micro_step + 1 >= n_acc
        r = ref.micro_batch(wide, norm_sumsq=m.grad_sumsq) if boundary else ref.micro_batch(wide)
        assert bool(m.norm_measured) == boundary
        assert (bool(m.gradients_applied), m.step) == (r["gradients_applied"], r["step"])
        check_state(dev, ref, dparams, f"micro-batch {it}")
    assert ref.state.micro_step == 2
    assert dev.flush_gradients() is True
    assert ref.flush_gradients(norm_sumsq=dev.last_metrics.grad_sumsq) is True
    check_state(dev, ref, dparams, "after flush")
    assert dev.flush_gradients() is False and ref.flush_gradients() is False


@pytest.mark.parametrize("bf16", [False, True])
def test_sft_deferred_flush_after_the_oldest_micro_batches_were_spilled(mx, bf16):
    """Ten of twelve micro-batches, then flush: three have gone into the float32 buffers, seven are still
    deferred; the average is over the ten."""
    rng = np.random.default_rng(77)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.02, gradient_accumulation_steps=12, gradient_clip_norm=0.5, weight_decay=0.01)
    dev = mx.SFTEngineOptimizerSide(dparams, accumulate_in_f32=True, defer_accumulation=True, **kw)
    ref = O.SFTEngineOptimizerSide(params, **kw)
    for cycle in range(2):                                   # the second cycle reuses the buffers of the first
        for it in range(10):
            grads = make_grads(rng, bf16, 0.01)
            m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
            ref.micro_batch({k: O.as_f32(g) for k, g in grads.items()})
            assert not m.gradients_applied
        assert dev.flush_gradients() is True
        assert ref.flush_gradients(norm_sumsq=dev.last_metrics.grad_sumsq) is True
        check_state(dev, ref, dparams, f"after flush {cycle}")


@pytest.mark.parametrize("kind", ["sft", "grpo"])
@pytest.mark.parametrize("n_acc", [3, 10])
def test_deferred_cycles_with_an_empty_and_a_one_element_tensor(mx, kind, n_acc):
    rng = np.random.default_rng(1)
    params = {"a": np.zeros(0, F), "b": rng.normal(0, 0.1, 5000).astype(F), "c": rng.normal(0, 0.1, 1).astype(F)}
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=n_acc, gradient_clip_norm=0.5)
    if kind == "sft":
        dev = mx.SFTEngineOptimizerSide(dparams, accumulate_in_f32=True, defer_accumulation=True, **kw)
        ref = O.SFTEngineOptimizerSide(params, **kw)
    else:
        dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=True, **kw)
        ref = O.GRPOEngineOptimizerSide(params, **kw)
    for it in range(2 * n_acc):
        grads = {k: rng.normal(0, 0.01, v.size).astype(F) for k, v in params.items()}
        m = dev.micro_batch({k: to_dev(g) for k, g in grads.items()})
        if kind == "grpo" or m.gradients_applied:
            ref.micro_batch(grads, norm_sumsq=m.grad_sumsq)
        else:
            ref.micro_batch(grads)
    check_state(dev, ref, dparams, f"{kind} N={n_acc}")


def test_deferred_mode_refuses_what_it_cannot_hold(mx):
    rng = np.random.default_rng(5)
    params = make_params(rng, False)
    dparams = {k: to_dev(v) for k, v in params.items()}
    with pytest.raises(ValueError, match="adds in float32"):
        mx.SFTEngineOptimizerSide(dparams, gradient_accumulation_steps=2, defer_accumulation=True)
    with pytest.raises(ValueError, match="plain SGD only"):
        mx.GRPOEngineOptimizerSide(dparams, gradient_accumulation_steps=2, apply="adamw", defer_accumulation=True)
    dev = mx.SFTEngineOptimizerSide(dparams, gradient_accumulation_steps=2, accumulate_in_f32=True, defer_accumulation=True)
    dev.micro_batch({k: to_dev(g) for k, g in make_grads(rng, False, 0.01).items()})
    before = {k: to_host(v) for k, v in dparams.items()}
    with pytest.raises(ValueError, match="same gradient names"):
        dev.micro_batch({k: to_dev(g) for k, g in make_grads(rng, False, 0.01, ["embed", "w1"]).items()})
    assert dev.micro_step == 1
    for k in dparams:
        assert_bit_equal(to_host(dparams[k]), before[k], k)
    # the cycle is still open: the complete micro-batch finishes it
    m = dev.micro_batch({k: to_dev(g) for k, g in make_grads(rng, False, 0.01).items()})
    assert m.gradients_applied and dev.micro_step == 0
