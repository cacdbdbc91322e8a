"""The reference's own optimizer tests, restated against the host layer (same classes, methods,
arguments and expectations), followed by parity of that layer with the CPU oracle.

Sections name the reference test file they follow.  `close(a, b, digits)` is vitest's
toBeCloseTo.  Everything runs on the GPU through libmxopt.so.
"""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


def arr(*v):
    """createFloat32Array (__test__/test-utils.ts:15-60)."""
    return to_dev(np.array(v, dtype=F))


def vals(t):
    return to_host(t)


def close(a, b, digits=2):
    return abs(float(a) - float(b)) < (10.0 ** -digits) / 2


# ---- __test__/core/optimizers.test.ts ------------------------------------------------------

def test_adam_default_settings(mx):  # :7-23
    adam = mx.Adam()
    v = vals(adam.update_single("param1", arr(1, 2, 3), arr(0.1, 0.2, 0.3)))
    assert v[0] < 1.0 and v[1] < 2.0 and v[2] < 3.0


def test_adam_separate_state(mx):  # :25-41
    adam = mx.Adam()
    g = arr(0.1, 0.2)
    v1 = vals(adam.update_single("param1", arr(1, 2), g))
    v2 = vals(adam.update_single("param2", arr(3, 4), g))
    assert not close(v1[0], v2[0]) and not close(v1[1], v2[1])


def test_adam_bias_correction(mx):  # :43-65
    with_b = vals(mx.Adam(0.01, 0.9, 0.999, 1e-8, True).update_single("param", arr(1, 1), arr(0.1, 0.1)))
    without = vals(mx.Adam(0.01, 0.9, 0.999, 1e-8, False).update_single("param", arr(1, 1), arr(0.1, 0.1)))
    assert not close(with_b[0], 1.0) and not close(without[0], 1.0)
    assert not close(with_b[0], without[0])


def test_adam_reset(mx):  # :67-87
    adam = mx.Adam()
    p, g = arr(1, 2), arr(0.1, 0.2)
    u1 = vals(adam.update_single("param", p, g))
    adam.reset()
    u2 = vals(adam.update_single("param", p, g))
    assert close(u1[0], u2[0], 5) and close(u1[1], u2[1], 5)


def test_adam_learning_rates(mx):  # :89-104
    lo = vals(mx.Adam(0.001).update_single("param", arr(1, 1), arr(0.1, 0.1)))
    hi = vals(mx.Adam(0.01).update_single("param", arr(1, 1), arr(0.1, 0.1)))
    assert abs(1.0 - hi[0]) > abs(1.0 - lo[0])


def test_adamw_weight_decay(mx):  # :107-148
    p, z = arr(1, 2, 3), arr(0, 0, 0)
    w = vals(mx.AdamW(0.01, 0.9, 0.999, 1e-8, 0.01).update_single("param", p, z))
    a = vals(mx.Adam(0.01, 0.9, 0.999, 1e-8).update_single("param", p, z))
    assert w[0] < 1.0 and w[1] < 2.0 and w[2] < 3.0
    assert close(a[0], 1.0, 5) and close(a[1], 2.0, 5) and close(a[2], 3.0, 5)
    lo = vals(mx.AdamW(0.01, 0.9, 0.999, 1e-8, 0.001).update_single("param", arr(1, 1), arr(0, 0)))
    hi = vals(mx.AdamW(0.01, 0.9, 0.999, 1e-8, 0.1).update_single("param", arr(1, 1), arr(0, 0)))
    assert hi[0] < lo[0]


def test_sgd_basic(mx):  # :151-164
    v = vals(mx.SGD(0.1).update_single("param", arr(1, 2, 3), arr(0.1, 0.2, 0.3)))
    assert close(v[0], 1.0 - 0.1 * 0.1, 5) and close(v[1], 2.0 - 0.1 * 0.2, 5) and close(v[2], 3.0 - 0.1 * 0.3, 5)


def test_sgd_momentum(mx):  # :166-188
    sgd = mx.SGD(0.1, 0.9)
    u1 = sgd.update_single("param", arr(1, 2), arr(0.1, 0.2))
    v2 = vals(sgd.update_single("param", u1, arr(0.1, 0.2)))
    assert close(v2[0], 1.0 - 0.1 * 0.1 - 0.1 * 0.19, 4)
    assert close(v2[1], 2.0 - 0.1 * 0.2 - 0.1 * 0.38, 4)


def test_sgd_weight_decay(mx):  # :190-203
    v = vals(mx.SGD(0.1, 0.0, 0.01).update_single("param", arr(1, 2), arr(0, 0)))
    assert close(v[0], 1.0 - 0.1 * 0.01 * 1.0, 5) and close(v[1], 2.0 - 0.1 * 0.01 * 2.0, 5)


def test_sgd_invalid_nesterov(mx):  # :205-214
    with pytest.raises(ValueError, match="Nesterov"):
        mx.SGD(0.1, 0.0, 0.0, 0.0, True)
    with pytest.raises(ValueError, match="Nesterov"):
        mx.SGD(0.1, 0.9, 0.0, 0.1, True)
    mx.SGD(0.1, 0.9, 0.0, 0.0, True)


def test_rmsprop(mx):  # :217-277
    v = vals(mx.RMSprop(0.01).update_single("param", arr(1, 2, 3), arr(0.1, 0.2, 0.3)))
    assert v[0] < 1.0 and v[1] < 2.0 and v[2] < 3.0
    r = mx.RMSprop(0.01)
    cur = arr(1, 1)
    for _ in range(5):
        cur = r.update_single("param", cur, arr(1.0, 0.1))
    c = vals(cur)
    assert abs(1 - c[0]) > 0 and abs(1 - c[1]) > 0
    lo, hi = mx.RMSprop(0.01, 0.9), mx.RMSprop(0.01, 0.99)
    a = b = arr(1, 1)
    for _ in range(3):
        a = lo.update_single("param", a, arr(0.1, 0.1))
        b = hi.update_single("param", b, arr(0.1, 0.1))
    assert not close(vals(a)[0], vals(b)[0], 3)


def test_gradient_utils(mx):  # :280-379
    GU = mx.GradientUtils
    v = vals(GU.clip_grad_value(arr(-2, -0.5, 0, 0.5, 2), -1.0, 1.0))
    assert [close(a, b, 5) for a, b in zip(v, (-1, -0.5, 0, 0.5, 1))] == [True] * 5
    assert close(GU.compute_gradient_norm({"param1": arr(3, 4)}), 5.0, 5)
    assert close(GU.compute_gradient_norm({"param1": arr(1, 2), "param2": arr(2)}), 3.0, 5)
    v = vals(GU.clip_grad_norm({"param": arr(3, 4)}, 10.0)["param"])
    assert close(v[0], 3.0, 5) and close(v[1], 4.0, 5)
    v = vals(GU.clip_grad_norm({"param": arr(3, 4)}, 2.5)["param"])
    assert close(v[0], 1.5, 4) and close(v[1], 2.0, 4)
    c = GU.clip_grad_norm({"param1": arr(1, 2), "param2": arr(2)}, 1.5)
    assert close(vals(c["param1"])[0], 0.5, 4) and close(vals(c["param1"])[1], 1.0, 4)
    assert close(vals(c["param2"])[0], 1.0, 4)
    clipped, norm = GU.clip_grad_norm_with_norm({"param": arr(3, 4)}, 2.5)
    assert close(norm, 5.0, 5)
    assert close(vals(clipped["param"])[0], 1.5, 4) and close(vals(clipped["param"])[1], 2.0, 4)
    c = GU.clip_grad_norm({"weight": arr(1, 2, 3), "bias": arr(4, 5)}, 100.0)
    assert set(c) == {"weight", "bias"} and c["weight"].shape == (3,) and c["bias"].shape == (2,)
    assert GU.clip_grad_norm({}, 1.0) == {} and GU.clip_grad_norm_with_norm({}, 1.0) == ({}, 0.0)


def test_lr_scheduler(mx):  # :381-434
    S = mx.LRScheduler
    assert close(S.linear_decay(1.0, 0.1, 0, 100), 1.0, 5) and close(S.linear_decay(1.0, 0.1, 50, 100), 0.55, 5)
    assert close(S.linear_decay(1.0, 0.1, 100, 100), 0.1, 5) and close(S.linear_decay(1.0, 0.1, 200, 100), 0.1, 5)
    assert close(S.exponential_decay(1.0, 0.9, 0, 10), 1.0, 5) and close(S.exponential_decay(1.0, 0.9, 10, 10), 0.9, 5)
    assert close(S.exponential_decay(1.0, 0.9, 20, 10), 0.81, 5)
    assert close(S.cosine_annealing(1.0, 0.1, 0, 100), 1.0, 5) and close(S.cosine_annealing(1.0, 0.1, 50, 100), 0.55, 5)
    assert close(S.cosine_annealing(1.0, 0.1, 100, 100), 0.1, 5)
    d25 = S.cosine_annealing(1.0, 0.1, 0, 100) - S.cosine_annealing(1.0, 0.1, 25, 100)
    d75 = S.cosine_annealing(1.0, 0.1, 75, 100) - S.cosine_annealing(1.0, 0.1, 100, 100)
    assert close(d25, d75, 3)
    for step, want in ((0, 1.0), (9, 1.0), (10, 0.5), (20, 0.25), (30, 0.125)):
        assert close(S.step_decay(1.0, 0.5, step, 10), want, 5)
    for args in ((1.0, 0.1, 37, 100), (3e-4, 1e-5, 0, 7), (1.0, 0.5, 99, 10)):   # and the oracle, exactly
        assert S.linear_decay(*args) == O.LRScheduler.linear_decay(*args)
        assert S.cosine_annealing(*args) == O.LRScheduler.cosine_annealing(*args)
        assert S.exponential_decay(*args) == O.LRScheduler.exponential_decay(*args)
        assert abs(S.step_decay(*args) - O.LRScheduler.step_decay(*args)) <= 1e-15


def test_integration_quadratic(mx):  # :436-475
    adam = mx.Adam(0.1)
    x = arr(10.0)
    two = arr(2.0)
    for _ in range(100):
        x = adam.update_single("x", x, x * two)      # gradient = 2x (torch only builds the test input)
    assert abs(vals(x)[0]) < 10.0
    sgd = mx.SGD(0.1, 0.9)
    x = arr(10.0)
    for _ in range(100):
        x = sgd.update_single("x", x, x * two)
    assert abs(vals(x)[0]) < 1.0


# ---- __test__/core/optimizers-extended.test.ts ------------------------------------------------

def test_zero_gradients(mx):  # :68-123
    p = arr(0.5, -1.5, 2.5)
    z = arr(0, 0, 0)
    adam = mx.Adam()
    q = p
    for _ in range(5):
        q = adam.update_single("p", q, z)
    assert np.array_equal(vals(q), vals(p))
    assert np.array_equal(vals(mx.SGD(0.1).update_single("p", p, z)), vals(p))
    assert np.array_equal(vals(mx.RMSprop(0.01).update_single("p", p, z)), vals(p))


def test_extreme_gradients(mx):  # :126-181
    for opt in (mx.Adam(0.01), mx.AdamW(0.01), mx.RMSprop(0.01), mx.SGD(0.01, 0.9)):
        big = vals(opt.update_single("a", arr(1, 1), arr(1e6, -1e6)))
        tiny = vals(opt.update_single("b", arr(1, 1), arr(1e-10, -1e-10)))
        assert np.isfinite(big).all() and np.isfinite(tiny).all()


@pytest.mark.parametrize("make", ["adam", "adamw", "rmsprop", "sgd"])
def test_reset_is_bit_identical_to_fresh(mx, make):  # :442-477 (toEqual)
    mk = {"adam": lambda: mx.Adam(0.01), "adamw": lambda: mx.AdamW(0.01), "rmsprop": lambda: mx.RMSprop(0.01),
          "sgd": lambda: mx.SGD(0.01)}[make]
    p, g = arr(1, 2, 3), arr(0.1, -0.2, 0.3)
    used = mk()
    q = p
    for _ in range(3):
        q = used.update_single("p", q, g)
    used.reset()
    assert np.array_equal(vals(used.update_single("p", p, g)), vals(mk().update_single("p", p, g)))


def test_first_momentum_step_equals_plain_sgd(mx):  # :51-65
    p, g = arr(1, 2), arr(0.5, -0.25)
    assert np.array_equal(vals(mx.SGD(0.1, 0.9).update_single("p", p, g)), vals(mx.SGD(0.1).update_single("p", p, g)))


def test_rosenbrock_converges(mx):  # :214-251 (fewer steps: the point is a long dependent chain)
    import torch
    adam = mx.Adam(0.01)
    xy = arr(-1.0, 1.0)
    for _ in range(300):
        x, y = xy[0], xy[1]
        g = torch.stack([-2 * (1 - x) - 400 * x * (y - x * x), 200 * (y - x * x)])
        xy = adam.update_single("xy", xy, g)
    x, y = vals(xy)
    f = (1 - x) ** 2 + 100 * (y - x * x) ** 2
    assert f < (1 - -1.0) ** 2 + 100 * (1.0 - 1.0) ** 2


# ---- __test__/core/numerical-consistency.test.ts:309-391 ---------------------------------------

def test_two_identical_adam_runs_agree(mx):
    rng = np.random.default_rng(1)
    p0 = rng.normal(0, 1, 1000).astype(F)
    gs = [rng.normal(0, 1, 1000).astype(F) for _ in range(5)]
    outs = []
    for _ in range(2):
        adam = mx.Adam(0.01)
        p = to_dev(p0)
        for g in gs:
            p = adam.update_single("w", p, to_dev(g))
        outs.append(vals(p))
    assert np.array_equal(outs[0], outs[1])


# ---- __test__/trainers/grpo-gradient-accumulation.test.ts ----------------------------------------

def test_accumulate_gradients(mx):
    out = mx.accumulate_gradients({"w": arr(1, 2, 3)}, {"w": arr(0.5, 0.5, 0.5)})      # :7-29
    assert np.array_equal(vals(out["w"]), np.array([1.5, 2.5, 3.5], F))
    out = mx.accumulate_gradients({}, {"w": arr(1, 2, 3)})                                # :31-44
    assert np.array_equal(vals(out["w"]), np.array([1, 2, 3], F))
    g = arr(0.25, -0.5, 1.0)                                                             # :48-68
    acc = {}
    for _ in range(4):
        acc = mx.accumulate_gradients(acc, {"w": g})
    assert np.array_equal(vals(acc["w"]), vals(g) * F(4))
    assert acc["w"].shape == g.shape                                                     # :70-89
    pa, pb = {"w": arr(1, 1, 1)}, {"w": arr(1, 1, 1)}                                    # :134-171
    mx.apply_gradients(pa, acc, 0.1 / 4)
    mx.apply_gradients(pb, {"w": g}, 0.1)
    assert np.allclose(vals(pa["w"]), vals(pb["w"]), rtol=0, atol=1e-6)
    out = mx.accumulate_gradients({"a": arr(1), "b": arr(2)}, {"a": arr(1)})             # model.rs:2235-2240
    assert set(out) == {"a", "b"} and vals(out["b"])[0] == 2 and vals(out["a"])[0] == 2


def test_accumulate_gradients_promotes_mixed_dtypes(mx):
    """models/qwen3/model.rs:2227 is `acc.add(new)`: operands of different dtypes give a float32 sum (MLX
    promote_types), equal 16-bit dtypes stay 16-bit.  Every pairing against the oracle, ragged sizes."""
    import torch
    rng = np.random.default_rng(29)
    for n in (1, 4097, 100003):
        a32, g32 = rng.normal(0, 1e-2, n).astype(F), rng.normal(0, 1e-2, n).astype(F)
        forms = {"f32": lambda x: x, "bf16": O.f32_to_bf16, "f16": lambda x: x.astype(np.float16)}
        for ka, fa in forms.items():
            for kg, fg in forms.items():
                a, g = fa(a32), fg(g32)
                out = mx.accumulate_gradients({"w": to_dev(a)}, {"w": to_dev(g)})["w"]
                s = O.as_f32(a) + O.as_f32(g)
                if ka == kg:
                    want = forms[ka](s) if ka != "f16" else s.astype(np.float16)
                    assert out.dtype == {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[ka]
                else:
                    want = s
                    assert out.dtype == torch.float32, (ka, kg)
                assert_bit_equal(to_host(out), want, f"{ka} + {kg}, n={n}")
    # the C entry point refuses an output that is not the promoted dtype
    ctx = mx.default_context()
    import mxopt.optimizers as MO
    a, g = to_dev(O.f32_to_bf16(a32)), to_dev(g32)
    bad = torch.empty(len(g32), dtype=torch.bfloat16, device="cuda")
    rc = ctx.lib.mxopt_accumulate_gradients(ctx.handle, 1, MO._arrs([a]), MO._arrs([g]), MO._arrs([bad]))
    assert rc == mx._lib.ERR_INVALID_ARG and b"promoted dtype" in ctx.lib.mxopt_last_error(ctx.handle)


def test_a_refused_update_many_leaves_the_call_counter_alone(mx):
    """adam.rs:73 counts update_single calls; an update_many that is refused launches nothing and must not
    shift later bias corrections."""
    ps, gs = rand_lists(31)
    names = [f"p{i}" for i in range(len(ps))]
    opt = mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    opt.update_many(names, dp, dg, outs=dp)
    assert opt.step == len(ps)
    wrong = list(dg)
    wrong[-1] = to_dev(np.zeros(len(gs[-1]) + 1, F))          # the last pair does not match: refused as a whole
    with pytest.raises(ValueError):
        opt.update_many(names, dp, wrong, outs=dp)
    assert opt.step == len(ps)
    opt.update_many(names, dp, dg, outs=dp)
    cur = list(ps)
    for _ in range(2):
        cur = [ref.update_single(nm, p, g) for nm, p, g in zip(names, cur, gs)]
    for i, p in enumerate(dp):
        assert_bit_equal(to_host(p), cur[i], f"p{i} after a refused call in between")


# ---- __test__/training/basic-training.test.ts:95-128 ----------------------------------------------

def test_apply_gradients_closed_form(mx):
    p = {"w": to_dev(np.full(8, 0.5, F)), "frozen": to_dev(np.full(4, 7.0, F))}
    mx.apply_gradients(p, {"w": to_dev(np.full(8, 0.01, F))}, 0.001)
    assert np.allclose(vals(p["w"]), 0.5 - 0.001 * 0.01, rtol=0, atol=1e-7)
    assert np.array_equal(vals(p["frozen"]), np.full(4, 7.0, F))
    with pytest.raises(RuntimeError, match="not found in model"):
        mx.apply_gradients(p, {"nope": arr(0)}, 0.001)


# ---- parity of the host layer with the oracle ------------------------------------------------------

SIZES = [0, 1, 9, 4097, 20011]


def rand_lists(seed, bf16=False):
    rng = np.random.default_rng(seed)
    ps = [rng.normal(0, 0.02, n).astype(F) for n in SIZES]
    gs = [rng.normal(0, 1e-3, n).astype(F) for n in SIZES]
    if bf16:
        ps, gs = [O.f32_to_bf16(p) for p in ps], [O.f32_to_bf16(g) for g in gs]
    return ps, gs


@pytest.mark.parametrize("kind", ["adam", "adamw", "adamw_bias", "sgd_nesterov", "sgd_damp", "rmsprop"])
@pytest.mark.parametrize("bf16", [False, True])
def test_update_single_and_many_match_oracle(mx, kind, bf16):
    """update_single per tensor, and update_many for the list, are the same numbers as the oracle's
    update_single loop -- including the per-call step counter under bias correction."""
    make = {
        "adam": (lambda m: m.Adam(1e-3)),
        "adamw": (lambda m: m.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)),
        "adamw_bias": (lambda m: m.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True)),
        "sgd_nesterov": (lambda m: m.SGD(1e-2, 0.9, 1e-4, None, True)),
        "sgd_damp": (lambda m: m.SGD(1e-2, 0.9, None, 0.25)),
        "rmsprop": (lambda m: m.RMSprop(1e-4, 0.99, 1e-8, 0.01)),
    }[kind]
    ps, gs = rand_lists(5, bf16)
    names = [f"layers.{i}.w" for i in range(len(ps))]
    ref, one, many = make(O), make(mx), make(mx)
    dps, dgs = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    cur_ref = list(ps)
    cur_one = list(dps)
    cur_many = list(dps)
    for it in range(3):
        outs_many = many.update_many(names, cur_many, dgs)
        for i, nm in enumerate(names):
            r = ref.update_single(nm, cur_ref[i], gs[i])
            o = one.update_single(nm, cur_one[i], dgs[i])
            assert_bit_equal(to_host(o), r, f"single {nm} it{it}")
            assert_bit_equal(to_host(outs_many[i]), r, f"many {nm} it{it}")
            cur_ref[i], cur_one[i] = r, o
        cur_many = outs_many
    if kind.startswith("adam"):
        assert one.step == ref.step == many.step == 3 * len(names)
        m, v = one.state(names[3])
        assert_bit_equal(to_host(m), ref.state[names[3]][0], "m")
        assert_bit_equal(to_host(v), ref.state[names[3]][1], "v")
    else:
        assert one.step == 0


def test_in_place_bf16_update_many_with_clip(mx):
    """The production shape: bf16 parameters updated in place, one launch, clip scale from the device."""
    ps, gs = rand_lists(9, bf16=True)
    names = [str(i) for i in range(len(ps))]
    dps, dgs = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    ctx = mx.default_context()
    res = ctx.norm_result()
    ctx.global_norm(ctx.table([mx.TensorSpec(g=g) for g in dgs]), res, max_norm=1e-3)
    scale = F(ctx.read_norm_result(res).scale)
    _, want_scale = O.norm_scale_c1(O.exact_sumsq(gs), 1e-3)
    assert O.ulp_diff_f32(np.array([scale]), np.array([want_scale]))[0] <= 1
    opt = mx.AdamW(5e-6)
    ref = O.AdamW(5e-6)
    cur = list(ps)
    for it in range(2):
        opt.update_many(names, dps, dgs, outs=dps, prep=mx.make_prep(scale=res))
        for i, nm in enumerate(names):
            cur[i] = O.f32_to_bf16(ref.update_single(nm, cur[i], O.as_f32(gs[i]) * scale))
            assert_bit_equal(to_host(dps[i]), cur[i], f"{nm} it{it}")


def test_state_save_load_round_trip(mx):
    ps, gs = rand_lists(11)
    a = mx.AdamW(1e-3, None, None, None, None, True)
    p = to_dev(ps[4])
    g = to_dev(gs[4])
    for _ in range(3):
        p = a.update_single("w", p, g)
    m, v = a.state("w")
    b = mx.AdamW(1e-3, None, None, None, None, True)
    b.load_state("w", m, v, a.step)
    assert b.step == a.step == 3
    assert_bit_equal(to_host(b.update_single("w", p, g)), to_host(a.update_single("w", p, g)), "resumed step")
    s = mx.SGD(0.1, 0.9)
    assert s.state("w") == (None, None)
    s.update_single("w", p, g)
    assert s.state("w")[0] is None and s.state("w")[1] is not None


def test_gradient_utils_match_oracle(mx):
    _, gs = rand_lists(13)
    _, gb = rand_lists(13, bf16=True)
    GU = mx.GradientUtils
    for grads, keep in ((gs, None), (gb, None), (gb, "grad")):
        d = {str(i): to_dev(g) for i, g in enumerate(grads)}
        n_dev = GU.compute_gradient_norm(d)
        n_ref = O.GradientUtils.compute_gradient_norm({k: g for k, g in zip(d, grads)})
        assert abs(n_dev - n_ref) <= 1e-5 * n_ref          # the stated bar; observed ~1e-8
        for max_norm in (n_ref / 3, n_ref * 3):
            clipped, norm = GU.clip_grad_norm_with_norm(d, max_norm, out_dtype=keep)
            assert abs(norm - n_ref) <= 1e-5 * n_ref
            n32, s = O.norm_scale_c1(norm * norm, max_norm)     # the scalar chain, from the device's own norm
            for k, g in zip(d, grads):
                w = O.as_f32(g) * s
                assert_bit_equal(to_host(clipped[k]), O.f32_to_bf16(w) if keep else w, f"clip {k}")
            vec = mx.clip_gradients_by_global_norm(list(d.values()), max_norm, out_dtype=keep)
            if n_ref <= max_norm:     # unchanged copies (gradients/mod.rs:258-265)
                for t, g in zip(vec, grads):
                    assert_bit_equal(to_host(t), O.f32_to_bf16(O.as_f32(g)) if keep else O.as_f32(g), "vec copy")
            else:
                s64 = F(max_norm / (n_dev + 1e-6))
                for t, g in zip(vec, grads):
                    w = O.as_f32(g) * s64
                    got = to_host(t)
                    want = O.f32_to_bf16(w) if keep else w
                    # the device's float64 norm and the oracle's may differ in the last bits
                    if keep:
                        assert (O.ulp_diff_bf16(got, want) <= 1).all()
                    else:
                        assert (O.ulp_diff_f32(got, want) <= 2).all()
        both = GU.clip_grad_value_and_norm(d, 5e-4, None, out_dtype=keep)
        for k, g in zip(d, grads):
            w = O.clip_value(g, -5e-4, 5e-4)
            assert_bit_equal(to_host(both[k]), O.f32_to_bf16(w) if keep else w, f"clamp {k}")
        byv = mx.clip_gradients_by_value(list(d.values()), -1e-4, float("inf"), out_dtype=keep)
        for t, g in zip(byv, grads):
            w = O.clip_value(g, -1e-4, float("inf"))
            assert_bit_equal(to_host(t), O.f32_to_bf16(w) if keep else w, "by value")


def test_engine_accumulator_semantics(mx):
    """grpo/engine.rs:2632-2666 (new names join) vs sft/engine.rs:282-290 (unknown names dropped),
    and the widened float32 buffer."""
    import torch
    _, gb = rand_lists(17, bf16=True)
    g = {str(i): to_dev(x) for i, x in enumerate(gb)}
    grpo = mx.GradientAccumulator()
    grpo.accumulate({k: g[k] for k in ("1", "2")})
    grpo.accumulate(g)
    acc = grpo.take()
    assert set(acc) == set(g) and grpo.micro_step == 0
    assert_bit_equal(to_host(acc["2"]), O.accumulate_gradients({"w": gb[2]}, {"w": gb[2]})["w"], "bf16 sum")
    assert_bit_equal(to_host(acc["3"]), gb[3], "joined later")
    sft = mx.GradientAccumulator(drop_unknown=True)
    sft.accumulate({k: g[k] for k in ("1", "2")})
    sft.accumulate(g)
    assert set(sft.take()) == {"1", "2"}
    wide = mx.GradientAccumulator(dtype=torch.float32)
    for _ in range(3):
        wide.accumulate(g)
    ref = None
    for _ in range(3):
        ref = O.accumulate_fp32(ref, gb[4])
    assert_bit_equal(to_host(wide.take()["4"]), ref, "float32 buffer")


def test_error_cases(mx):
    import torch
    a = mx.Adam()
    with pytest.raises(ValueError):
        a.update_single("w", arr(1, 2), arr(1, 2, 3))
    with pytest.raises(ValueError):
        a.update_single("w", torch.zeros(4, dtype=torch.int32, device="cuda"), arr(1, 2, 3, 4))
    a.update_single("w", arr(1, 2), arr(1, 2))
    with pytest.raises(ValueError, match="elements"):
        a.update_single("w", arr(1, 2, 3), arr(1, 2, 3))        # same name, other size
    with pytest.raises(ValueError):
        a.update_single("v", arr(1, 2), arr(1, 2), out=torch.zeros(2, dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError):
        mx.Adam().update_single("w", torch.zeros(2), torch.zeros(2))   # host tensors: no CPU path


# ---- __test__/core/training-demo-simple.test.ts ------------------------------------------------

def test_demo_quadratic_with_four_optimizers(mx):  # :6-50
    opts = {"adam": mx.Adam(0.1), "adamw": mx.AdamW(0.1, 0.9, 0.999, 1e-8, 0.01), "sgd": mx.SGD(0.1),
            "sgdMomentum": mx.SGD(0.1, 0.9)}
    refs = {"adam": O.Adam(0.1), "adamw": O.AdamW(0.1, 0.9, 0.999, 1e-8, 0.01), "sgd": O.SGD(0.1),
            "sgdMomentum": O.SGD(0.1, 0.9)}
    for name, opt in opts.items():
        params, rp = arr(0.0, 0.0), np.zeros(2, F)
        traj = []
        for _ in range(50):
            v = vals(params)
            grad = np.array([2 * (v[0] - 2), 2 * (v[1] - 3)], F)      # f = (x-2)^2 + (y-3)^2
            params = opt.update_single(f"{name}_params", params, to_dev(grad))
            rp = refs[name].update_single(f"{name}_params", rp, grad)
            assert_bit_equal(vals(params), rp, name)                    # and the whole trajectory is the oracle's
            nv = vals(params)
            traj.append(math.hypot(nv[0] - 2, nv[1] - 3))
        assert traj[-1] < 0.5 and traj[-1] < traj[0], name


def test_demo_learning_rate_schedule(mx):  # :91-140
    rng = np.random.default_rng(0)
    w, b = arr(0.0), arr(0.0)
    losses = []
    for step in range(100):
        lr = mx.LRScheduler.cosine_annealing(0.1, 0.001, step, 100)
        sgd = mx.SGD(lr)
        x = rng.uniform(-1, 1, 10).astype(F)
        y = 2 * x + 1
        diff = x * vals(w)[0] + vals(b)[0] - y
        losses.append(float((diff ** 2).mean()))
        w = sgd.update_single("weight", w, arr(2 * float((x * diff).mean())))
        b = sgd.update_single("bias", b, arr(2 * float(diff.mean())))
    assert abs(vals(w)[0] - 2.0) < 0.5 and abs(vals(b)[0] - 1.0) < 0.5
    assert sum(losses[-10:]) < sum(losses[:10])


def test_demo_gradient_clipping(mx):  # :142-165
    clipped = mx.GradientUtils.clip_grad_value(arr(10.0, -15.0, 20.0), -5.0, 5.0)
    c = vals(clipped)
    assert close(c[0], 5.0) and close(c[1], -5.0) and close(c[2], 5.0)
    u = vals(mx.Adam(0.01).update_single("param", arr(1.0, 2.0, 3.0), clipped))
    assert all(abs(u[i] - [1.0, 2.0, 3.0][i]) < 1.0 for i in range(3))


def test_demo_weight_decay(mx):  # :220-251
    no_wd, wd = mx.Adam(0.01), mx.AdamW(0.01, 0.9, 0.999, 1e-8, 0.1)
    a, b = arr(10.0, 10.0), arr(10.0, 10.0)
    z = arr(0.0, 0.0)
    for _ in range(50):
        a = no_wd.update_single("params", a, z)
        b = wd.update_single("params", b, z)
    va, vb = vals(a), vals(b)
    assert close(va[0], 10.0, 2) and close(va[1], 10.0, 2)
    assert vb[0] < va[0] and vb[1] < va[1]
    assert abs(vb[0] - 10.0 * (1 - 0.01 * 0.1) ** 50) < 1e-4            # closed form of the decoupled decay
