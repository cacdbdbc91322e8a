"""Pins the CPU oracle against the known-answer values held by the reference's own tests.

Each test names the reference test it restates.  `close(a, b, digits)` is vitest's
`toBeCloseTo`: |a - b| < 10**-digits / 2.
"""
import math

import numpy as np
import pytest

import mxopt_oracle as O

F = np.float32


def arr(*v):
    return np.array(v, dtype=np.float32)


def close(a, b, digits=2):
    return abs(float(a) - float(b)) < (10.0 ** -digits) / 2


# ---- __test__/core/optimizers.test.ts ------------------------------------

def test_adam_default_decreases():  # :7-23
    out = O.Adam().update_single("param1", arr(1, 2, 3), arr(0.1, 0.2, 0.3))
    assert (out < arr(1, 2, 3)).all()


def test_adam_bias_correction_differs():  # :43-65
    a = O.Adam(0.01, 0.9, 0.999, 1e-8, True).update_single("p", arr(1, 1), arr(0.1, 0.1))
    b = O.Adam(0.01, 0.9, 0.999, 1e-8, False).update_single("p", arr(1, 1), arr(0.1, 0.1))
    assert not close(a[0], 1.0) or True
    assert not close(a[0], b[0], 2)
    # closed form of step 1: with correction the step is lr*g/(|g|+eps) = lr;
    # without it is lr*(1-b1)g/(sqrt(1-b2)|g|+eps) = lr*0.1/sqrt(0.001)
    assert close(1.0 - a[0], 0.01, 6)
    assert close(1.0 - b[0], 0.01 * 0.1 / math.sqrt(0.001), 6)


def test_adam_reset():  # :67-87
    adam = O.Adam()
    u1 = adam.update_single("p", arr(1, 2), arr(0.1, 0.2))
    adam.reset()
    u2 = adam.update_single("p", arr(1, 2), arr(0.1, 0.2))
    assert np.array_equal(u1, u2)


def test_adamw_zero_grad_decay():  # :107-130
    p = arr(1, 2, 3)
    w = O.AdamW(0.01, 0.9, 0.999, 1e-8, 0.01).update_single("p", p, arr(0, 0, 0))
    a = O.Adam(0.01, 0.9, 0.999, 1e-8).update_single("p", p, arr(0, 0, 0))
    assert (w < p).all()
    assert np.array_equal(a, p)
    assert np.allclose(w, p * (1 - 0.01 * 0.01), rtol=1e-7)


def test_sgd_basic():  # :151-164
    out = O.SGD(0.1).update_single("p", arr(1, 2, 3), arr(0.1, 0.2, 0.3))
    for o, e in zip(out, (1 - 0.1 * 0.1, 2 - 0.1 * 0.2, 3 - 0.1 * 0.3)):
        assert close(o, e, 5)


def test_sgd_momentum_two_steps():  # :166-188
    sgd = O.SGD(0.1, 0.9)
    u1 = sgd.update_single("p", arr(1, 2), arr(0.1, 0.2))
    u2 = sgd.update_single("p", u1, arr(0.1, 0.2))
    assert close(u2[0], 1.0 - 0.1 * 0.1 - 0.1 * 0.19, 4)
    assert close(u2[1], 2.0 - 0.1 * 0.2 - 0.1 * 0.38, 4)


def test_sgd_weight_decay():  # :190-203
    out = O.SGD(0.1, 0.0, 0.01).update_single("p", arr(1, 2), arr(0, 0))
    assert close(out[0], 1.0 - 0.1 * 0.01 * 1.0, 5)
    assert close(out[1], 2.0 - 0.1 * 0.01 * 2.0, 5)


def test_sgd_nesterov_validation():  # :205-214
    with pytest.raises(ValueError):
        O.SGD(0.1, 0.0, 0.0, 0.0, True)
    with pytest.raises(ValueError):
        O.SGD(0.1, 0.9, 0.0, 0.1, True)
    O.SGD(0.1, 0.9, 0.0, 0.0, True)


def test_rmsprop_decreases_and_alpha():  # :218-277
    out = O.RMSprop(0.01).update_single("p", arr(1, 2, 3), arr(0.1, 0.2, 0.3))
    assert (out < arr(1, 2, 3)).all()
    lo, hi = O.RMSprop(0.01, 0.9), O.RMSprop(0.01, 0.99)
    a = b = arr(1, 1)
    for _ in range(3):
        a = lo.update_single("p", a, arr(0.1, 0.1))
        b = hi.update_single("p", b, arr(0.1, 0.1))
    assert not close(a[0], b[0], 3)


def test_clip_grad_value():  # :281-291
    out = O.GradientUtils.clip_grad_value(arr(-2, -0.5, 0, 0.5, 2), -1.0, 1.0)
    assert np.array_equal(out, arr(-1, -0.5, 0, 0.5, 1))


def test_gradient_norm():  # :293-310
    assert close(O.GradientUtils.compute_gradient_norm({"a": arr(3, 4)}), 5.0, 5)
    assert close(O.GradientUtils.compute_gradient_norm({"a": arr(1, 2), "b": arr(2)}), 3.0, 5)


def test_clip_norm_identity_below_max():  # :312-322
    out = O.GradientUtils.clip_grad_norm({"p": arr(3, 4)}, 10.0)["p"]
    assert np.array_equal(out, arr(3, 4))


def test_clip_norm_half():  # :324-351
    out = O.GradientUtils.clip_grad_norm({"p": arr(3, 4)}, 2.5)["p"]
    assert close(out[0], 1.5, 4) and close(out[1], 2.0, 4)
    out = O.GradientUtils.clip_grad_norm({"a": arr(1, 2), "b": arr(2)}, 1.5)
    assert close(out["a"][0], 0.5, 4) and close(out["a"][1], 1.0, 4) and close(out["b"][0], 1.0, 4)


def test_clip_with_norm():  # :353-365
    out, n = O.GradientUtils.clip_grad_norm_with_norm({"p": arr(3, 4)}, 2.5)
    assert close(n, 5.0, 5)
    assert close(out["p"][0], 1.5, 4) and close(out["p"][1], 2.0, 4)
    assert O.GradientUtils.clip_grad_norm_with_norm({}, 1.0) == ({}, 0.0)


def test_lr_schedules():  # :382-433
    S = O.LRScheduler
    assert close(S.linear_decay(1.0, 0.1, 0, 100), 1.0, 5)
    assert close(S.linear_decay(1.0, 0.1, 50, 100), 0.55, 5)
    assert close(S.linear_decay(1.0, 0.1, 100, 100), 0.1, 5)
    assert close(S.linear_decay(1.0, 0.1, 200, 100), 0.1, 5)
    assert close(S.exponential_decay(1.0, 0.9, 0, 10), 1.0, 5)
    assert close(S.exponential_decay(1.0, 0.9, 10, 10), 0.9, 5)
    assert close(S.exponential_decay(1.0, 0.9, 20, 10), 0.81, 5)
    assert close(S.exponential_decay(1.0, 0.9, 19, 10), 0.9, 5)  # integer division (mod.rs:263)
    assert close(S.cosine_annealing(1.0, 0.1, 0, 100), 1.0, 5)
    assert close(S.cosine_annealing(1.0, 0.1, 50, 100), 0.55, 5)
    assert close(S.cosine_annealing(1.0, 0.1, 100, 100), 0.1, 5)
    d25 = S.cosine_annealing(1.0, 0.1, 0, 100) - S.cosine_annealing(1.0, 0.1, 25, 100)
    d75 = S.cosine_annealing(1.0, 0.1, 75, 100) - S.cosine_annealing(1.0, 0.1, 100, 100)
    assert close(d25, d75, 3)
    for step, want in ((0, 1.0), (9, 1.0), (10, 0.5), (20, 0.25), (30, 0.125)):
        assert close(S.step_decay(1.0, 0.5, step, 10), want, 5)


def test_adam_quadratic_converges():  # :437-455
    adam = O.Adam(0.1)
    x = arr(10.0)
    for _ in range(100):
        x = adam.update_single("x", x, x * F(2.0))
    assert abs(float(x[0])) < 10.0


# ---- __test__/core/optimizers-extended.test.ts ---------------------------

@pytest.mark.parametrize("make", [lambda: O.Adam(0.01), lambda: O.AdamW(0.01), lambda: O.RMSprop(0.01),
                                  lambda: O.SGD(0.01)])
def test_reset_equals_fresh(make):  # :442-477 (toEqual => bit-identical)
    p, g = arr(1, 2, 3), arr(0.1, -0.2, 0.3)
    used = make()
    q = p
    for _ in range(3):
        q = used.update_single("p", q, g)
    used.reset()
    fresh = make()
    assert np.array_equal(used.update_single("p", p, g), fresh.update_single("p", p, g))


def test_first_momentum_step_is_plain_sgd():  # :51-65
    p, g = arr(1, 2), arr(0.5, -0.25)
    assert np.array_equal(O.SGD(0.1, 0.9).update_single("p", p, g), O.SGD(0.1).update_single("p", p, g))


def test_zero_grad_leaves_adam_param():  # :69-84 and parameter-updates.test.ts:290-312
    p = arr(0.5, -1.5, 2.5)
    adam = O.Adam()
    q = p
    for _ in range(5):
        q = adam.update_single("p", q, np.zeros(3, F))
    assert np.array_equal(q, p)


# ---- __test__/trainers/grpo-gradient-accumulation.test.ts ----------------

def test_accumulate_sums():  # :7-29
    out = O.accumulate_gradients({"w": arr(1, 2, 3)}, {"w": arr(0.5, 0.5, 0.5)})
    assert np.array_equal(out["w"], arr(1.5, 2.5, 3.5))


def test_accumulate_empty_copies():  # :31-44
    out = O.accumulate_gradients({}, {"w": arr(1, 2, 3)})
    assert np.array_equal(out["w"], arr(1, 2, 3))


def test_accumulate_n_times_and_lr_over_n():  # :48-68, :134-171
    g = arr(0.25, -0.5, 1.0)
    acc = {}
    for _ in range(4):
        acc = O.accumulate_gradients(acc, {"w": g})
    assert np.array_equal(acc["w"], g * F(4))
    p = {"w": arr(1, 1, 1)}
    a = O.apply_gradients(p, acc, 0.1 / 4)["w"]
    b = O.apply_gradients(p, {"w": g}, 0.1)["w"]
    assert np.allclose(a, b, rtol=0, atol=1e-6)


def test_accumulate_keeps_names_only_in_acc():  # model.rs:2235-2240
    out = O.accumulate_gradients({"a": arr(1), "b": arr(2)}, {"a": arr(1)})
    assert set(out) == {"a", "b"} and out["b"][0] == 2


def test_sft_accumulate_drops_unknown_names():  # sft/engine.rs:283-287
    out = O.accumulate_gradients_sft({"a": arr(1)}, {"a": arr(1), "zzz": arr(5)})
    assert set(out) == {"a"} and out["a"][0] == 2


# ---- __test__/training/basic-training.test.ts:95-128 ---------------------

def test_apply_gradients_closed_form():
    p = {"w": np.full(8, 0.5, F)}
    out = O.apply_gradients(p, {"w": np.full(8, 0.01, F)}, 0.001)["w"]
    assert np.allclose(out, 0.5 - 0.001 * 0.01, rtol=0, atol=1e-7)
    with pytest.raises(KeyError):
        O.apply_gradients(p, {"nope": np.zeros(8, F)}, 0.001)


# ---- behaviours pinned only by reading the source ------------------------

def test_step_counts_calls_not_optimizer_steps():  # adam.rs:73, adamw.rs:77
    adam = O.Adam(0.01, 0.9, 0.999, 1e-8, True)
    adam.update_single("a", arr(1), arr(0.1))
    adam.update_single("b", arr(1), arr(0.1))
    assert adam.step == 2
    # the second tensor sees t=2 although its own moments are at their first update
    b2 = O.Adam(0.01, 0.9, 0.999, 1e-8, True)
    b2.step = 1
    expect = b2.update_single("b", arr(1), arr(0.1))
    c = O.Adam(0.01, 0.9, 0.999, 1e-8, True)
    c.update_single("a", arr(1), arr(0.1))
    assert np.array_equal(c.update_single("b", arr(1), arr(0.1)), expect)


def test_nesterov_stores_lookahead_as_state():  # sgd.rs:117-130
    s = O.SGD(0.1, 0.9, None, None, True)
    g = arr(0.5)
    s.update_single("p", arr(1), g)
    assert s.state["p"][0] == F(1.0)       # first call: v = g, stored u = v + g = 2g
    s.update_single("p", arr(1), g)
    assert s.state["p"][0] == F(1.0) * F(0.9) + F(0.5) + F(0.5)


def test_sgd_first_step_ignores_dampening():  # sgd.rs:107-114
    s = O.SGD(0.1, 0.9, None, 0.5)
    out = s.update_single("p", arr(1), arr(0.5))
    assert out[0] == F(1) - F(0.5) * F(0.1)
    s.update_single("p", out, arr(0.5))
    assert s.state["p"][0] == F(0.5) * F(0.9) + F(0.5) * F(0.5)


def test_vec_clip_returns_unchanged_when_below():  # gradients/mod.rs:258-265
    g = [arr(3, 4)]
    assert np.array_equal(O.clip_gradients_by_global_norm(g, 5.0)[0], g[0])   # n <= max
    out = O.clip_gradients_by_global_norm(g, 2.5)[0]
    assert np.array_equal(out, g[0] * F(2.5 / (5.0 + 1e-6)))
    assert O.clip_gradients_by_global_norm([], 1.0) == []


def test_coefficients_are_f64_then_f32():  # mlx.cpp:531-535 with adamw.rs:88,94
    assert O._f32(1.0 - 0.999) != F(1.0) - F(0.999)
    g = arr(3.0)
    ad = O.Adam()
    ad.update_single("p", arr(0), g)
    assert ad.state["p"][1][0] == (g * g)[0] * O._f32(1.0 - 0.999)


# ---- compositions that no reference test runs: hand-derived closed forms ----

def test_clip_grad_value_and_norm_closed_form():  # optimizers/mod.rs:174-226
    """Clamp to +-clip_value first (:188-192), the norm is taken of the CLAMPED values (:196-205), the factor is
    min(max / (n + 1e-6), 1) in float32 (:207-213) and every clamped tensor is multiplied by it (:219-226).
    [3, -4, 0.5] clamped to +-1 is [1, -1, 0.5]: n = sqrt(2.25) = 1.5, so with max 1 the factor is 1/(1.5+1e-6).
    A factor taken of the raw values would be 1/sqrt(25.25); scaling before clamping would give [0.6, -0.8, 0.1]."""
    g = {"a": arr(3, -4), "b": arr(0.5)}
    out = O.GradientUtils.clip_grad_value_and_norm(g, 1.0, 1.0)
    s = F(1.0) / (F(1.5) + F(1e-6))
    assert np.array_equal(out["a"], arr(1, -1) * s) and np.array_equal(out["b"], arr(0.5) * s)
    assert abs(float(out["a"][0]) - 2.0 / 3.0) < 1e-6
    # norm below the maximum: the factor is min(...) = exactly 1, the clamped values come back unchanged
    out = O.GradientUtils.clip_grad_value_and_norm(g, 1.0, 10.0)
    assert np.array_equal(out["a"], arr(1, -1)) and np.array_equal(out["b"], arr(0.5))
    # max_norm = None (:195, :222-224): the clamped values themselves, no multiply
    out = O.GradientUtils.clip_grad_value_and_norm(g, 2.5, None)
    assert np.array_equal(out["a"], arr(2.5, -2.5)) and np.array_equal(out["b"], arr(0.5))
    assert O.GradientUtils.clip_grad_value_and_norm({}, 1.0, 1.0) == {}   # :179-181
    # the result is float32 whatever the input (clip with float32 bounds promotes bf16)
    out = O.GradientUtils.clip_grad_value_and_norm({"h": O.f32_to_bf16(arr(3, -4, 0.5))}, 1.0, 1.0)
    assert out["h"].dtype == np.float32 and np.array_equal(out["h"], arr(1, -1, 0.5) * s)


def test_clip_gradients_by_value_one_sided_bounds():  # gradients/mod.rs:299-312 over mlx.cpp:469-481
    """Every tensor of the list is clamped on its own; a non-finite bound is 'no bound' on that side
    (std::isfinite, mlx.cpp:473-478), so (-inf, 1) only caps and (0, +inf) only floors."""
    gs = [arr(-5, -0.5, 0.5, 5), arr(7), arr()]
    out = O.clip_gradients_by_value(gs, -1.0, 1.0)
    assert [o.tolist() for o in out] == [[-1, -0.5, 0.5, 1], [1], []]
    out = O.clip_gradients_by_value(gs, -math.inf, 1.0)
    assert [o.tolist() for o in out] == [[-5, -0.5, 0.5, 1], [1], []]
    out = O.clip_gradients_by_value(gs, 0.0, math.inf)
    assert [o.tolist() for o in out] == [[0, 0, 0.5, 5], [7], []]
    out = O.clip_gradients_by_value(gs, math.nan, math.nan)        # neither bound is finite: untouched
    assert [o.tolist() for o in out] == [[-5, -0.5, 0.5, 5], [7], []]
    # the bounds are cast to float32 before the comparison (static_cast<float>, :474, :477): 0.1 is not
    # representable, and a value between float32(0.1) and the float64 0.1 is capped to float32(0.1)
    out = O.clip_gradients_by_value([arr(0.2)], -1.0, 0.1)
    assert out[0][0] == F(0.1) and float(out[0][0]) != 0.1
    assert O.clip_gradients_by_value([], -1.0, 1.0) == []
