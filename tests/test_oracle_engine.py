"""The oracle's restatement of the engines' optimizer side (oracle/mxopt_oracle.py:
GRPOEngineOptimizerSide, SFTEngineOptimizerSide).

Arithmetic: pinned by the reference's own known answers for accumulate-then-apply with lr/N
(__test__/trainers/grpo-gradient-accumulation.test.ts:48-68, 134-171), by the clip known answers
(__test__/core/optimizers.test.ts:281-365) and by closed forms / brute force in float64.
Bookkeeping (NaN counters, emergency flag, step counting, flush): no reference test runs it; the
cases below restate grpo/engine.rs:561-704 and sft/engine.rs:215-371, 459-553 line by line and are
what "pinned only by reading the source" means for these two classes.
"""
import math

import numpy as np
import pytest

import mxopt_oracle as O

F = np.float32


def test_grpo_lr_over_n_known_answer():
    # grpo-gradient-accumulation.test.ts:134-171: param [10, 20], four gradients, lr 0.01, N = 4
    grads = [[1.0, 2.0], [2.0, 3.0], [3.0, 4.0], [4.0, 5.0]]
    e = O.GRPOEngineOptimizerSide({"w": np.array([10.0, 20.0], F)}, learning_rate=0.01, gradient_accumulation_steps=4,
                                  gradient_clip_norm=None, gradient_clip_value=100.0)
    for k, g in enumerate(grads):
        r = e.micro_batch({"w": np.array(g, F)})
        assert r["gradients_applied"] == (k == 3) and r["step"] == k + 1       # step counts micro-batches
    assert abs(e.params["w"][0] - (10.0 - 0.0025 * 10.0)) < 5e-6               # toBeCloseTo(.., 5)
    assert abs(e.params["w"][1] - (20.0 - 0.0025 * 14.0)) < 5e-6
    # :93-131: (lr/N) * sum == lr * mean = [0.4, 0.5] for lr 0.1 and these four gradients
    e = O.GRPOEngineOptimizerSide({"w": np.zeros(2, F)}, learning_rate=0.1, gradient_accumulation_steps=4,
                                  gradient_clip_norm=None, gradient_clip_value=100.0)
    for g in ([1.0, 2.0], [3.0, 4.0], [5.0, 6.0], [7.0, 8.0]):
        e.micro_batch({"w": np.array(g, F)})
    assert np.allclose(-e.params["w"], [0.4, 0.5], atol=5e-7)
    assert e.micro_step == 0 and e.state.accumulated is None


def test_grpo_clamp_then_clip_norm_per_micro_batch():
    # engine.rs:636-653: clamp to +-1 first, the norm is that of the clamped values.
    # g = [3, -4, 0.5] -> clamped [1, -1, 0.5], norm 1.5 -> scale 1/1.5 (optimizers.test.ts:324-351 style)
    e = O.GRPOEngineOptimizerSide({"w": np.zeros(3, F)}, learning_rate=1.0, gradient_accumulation_steps=1)
    e.micro_batch({"w": np.array([3.0, -4.0, 0.5], F)})
    want = -np.array([1.0, -1.0, 0.5]) / 1.5
    assert np.allclose(e.params["w"], want, rtol=2e-6)
    # below the norm limit the gradient passes unchanged (x 1.0)
    e = O.GRPOEngineOptimizerSide({"w": np.zeros(2, F)}, learning_rate=1.0)
    e.micro_batch({"w": np.array([0.3, 0.4], F)})
    assert np.array_equal(e.params["w"], -np.array([0.3, 0.4], F))


def test_grpo_nan_policy():
    p0 = np.array([1.0, 2.0], F)
    e = O.GRPOEngineOptimizerSide({"w": p0}, learning_rate=0.1, gradient_accumulation_steps=2,
                                  max_nan_gradients=8, emergency_save_threshold=3)
    good = {"w": np.array([0.1, 0.2], F)}
    e.micro_batch(good)
    for k, bad in enumerate((np.nan, np.inf, -np.inf)):
        r = e.micro_batch({"w": np.array([0.1, bad], F)})
        assert r["skipped"] and not r["gradients_applied"]
        assert r["step"] == 2 + k                                   # engine.rs:608: a skipped step still counts
        assert e.micro_step == 1                                    # but not as a micro-step
        assert e.needs_emergency_save == (k == 2)                   # third consecutive one
    assert e.nan_gradient_count == 3 and np.array_equal(e.params["w"], p0)
    e.clear_emergency_save_flag()
    r = e.micro_batch(good)                                         # completes the cycle of two
    assert r["gradients_applied"] and e.state.consecutive_nan_count == 0 and not e.needs_emergency_save
    assert not np.array_equal(e.params["w"], p0)
    for _ in range(4):
        e.micro_batch({"w": np.array([np.nan, 0.0], F)})
    assert e.nan_gradient_count == 7
    with pytest.raises(O.TrainingStopped, match=r"maximum NaN gradient count \(8/8\)"):
        e.micro_batch({"w": np.array([np.nan, 0.0], F)})
    assert e.nan_gradient_count == 8                                 # counted before the error (engine.rs:580-596)
    e.reset()
    assert (e.step, e.micro_step, e.nan_gradient_count, e.needs_emergency_save) == (0, 0, 0, False)


def test_grpo_unknown_name_fails_at_apply():
    e = O.GRPOEngineOptimizerSide({"w": np.zeros(2, F)}, gradient_accumulation_steps=1)
    with pytest.raises(KeyError, match="not found in model"):
        e.micro_batch({"nope": np.zeros(2, F)})


def test_grpo_bf16_gradients_accumulate_in_float32():
    rng = np.random.default_rng(1)
    g = [O.f32_to_bf16(rng.normal(0, 0.3, 1000).astype(F)) for _ in range(3)]
    p = O.f32_to_bf16(rng.normal(0, 1, 1000).astype(F))
    e = O.GRPOEngineOptimizerSide({"w": p}, learning_rate=0.3, gradient_accumulation_steps=3)
    for x in g:
        e.micro_batch({"w": x})
    # float64 brute force of the same formula, then one bf16 rounding of the parameter
    acc = np.zeros(1000)
    for x in g:
        c = np.clip(O.bf16_to_f32(x).astype(np.float64), -1, 1)
        acc += c * min(1.0 / (math.sqrt((c * c).sum()) + 1e-6), 1.0)
    lr_bf16 = float(O.bf16_to_f32(O.f32_to_bf16(np.array([0.3 / 3], F)))[0])
    want = O.bf16_to_f32(p).astype(np.float64) - lr_bf16 * acc
    got = O.bf16_to_f32(e.params["w"]).astype(np.float64)
    assert e.params["w"].dtype == np.uint16
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30)       # within one bf16 rounding


def test_sft_average_clip_clamp_decay_closed_form():
    # sft/engine.rs:293-371 with N = 2: avg = [3, 4] -> norm 5 -> x 1/5 -> [0.6, 0.8] -> clamp 0.7 -> [0.6, 0.7]
    # -> + 0.1 * p -> p - lr * that
    p = np.array([1.0, -2.0], F)
    e = O.SFTEngineOptimizerSide({"w": p}, learning_rate=0.5, gradient_accumulation_steps=2, gradient_clip_norm=1.0,
                                 gradient_clip_value=0.7, weight_decay=0.1)
    r = e.micro_batch({"w": np.array([2.0, 3.0], F)})
    assert not r["gradients_applied"] and r["step"] == 0            # SFT counts optimizer steps (:371)
    r = e.micro_batch({"w": np.array([4.0, 5.0], F)})
    assert r["gradients_applied"] and r["step"] == 1
    want = p.astype(np.float64) - 0.5 * (np.array([0.6, 0.7]) + 0.1 * p)
    assert np.allclose(e.params["w"], want, rtol=3e-6)


def test_sft_drops_names_missing_from_the_accumulator_and_flushes_by_actual_count():
    e = O.SFTEngineOptimizerSide({"a": np.zeros(1, F), "b": np.zeros(1, F)}, learning_rate=1.0,
                                 gradient_accumulation_steps=4, gradient_clip_norm=None)
    e.micro_batch({"a": np.array([1.0], F)})
    e.micro_batch({"a": np.array([2.0], F), "b": np.array([5.0], F)})          # "b" is dropped (:283-287)
    e.micro_batch({"a": np.array([3.0], F)})
    assert e.flush_gradients() is True and e.step == 1 and e.micro_step == 0
    assert np.allclose(e.params["a"], [-(1 + 2 + 3) / 3.0]) and e.params["b"][0] == 0.0   # mean over 3, not 4
    assert e.flush_gradients() is False                                          # nothing left (:469-472)


def test_sft_nonfinite_loss_bookkeeping():
    e = O.SFTEngineOptimizerSide({"w": np.zeros(1, F)}, max_nan_gradients=3, emergency_save_threshold=2)
    assert e.report_nonfinite_loss() == 0 and not e.needs_emergency_save
    e.report_nonfinite_loss()
    assert e.needs_emergency_save and e.nan_gradient_count == 2
    e.micro_batch({"w": np.ones(1, F)})                                         # a good step resets the streak
    assert e.state.consecutive_nan_count == 0
    with pytest.raises(O.TrainingStopped, match="exceeded 3 NaN gradient limit"):
        e.report_nonfinite_loss()


def test_adamw_apply_is_adamw_on_the_prepared_gradient():
    rng = np.random.default_rng(2)
    p = rng.normal(0, 1, 64).astype(F)
    gs = [rng.normal(0, 0.01, 64).astype(F) for _ in range(2)]
    e = O.GRPOEngineOptimizerSide({"w": p}, learning_rate=1e-3, gradient_accumulation_steps=2, gradient_clip_norm=None,
                                  apply="adamw", weight_decay=0.01)
    for g in gs:
        e.micro_batch({"w": g})
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    want = ref.update_single("w", p, (gs[0] + gs[1]) * F(0.5))
    assert np.array_equal(e.params["w"], want)
