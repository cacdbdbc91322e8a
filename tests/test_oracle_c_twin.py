"""The C twin of the oracle must agree bit for bit with the NumPy oracle (both are one
rounded float32 operation per step), fused and un-fused alike."""
import numpy as np
import pytest

import mxopt_oracle as O
import oracle_c_binding as B

F = np.float32


def _data(n=10007, seed=1):
    rng = np.random.default_rng(seed)
    p = rng.normal(0, 0.02, n).astype(F)
    g = rng.normal(0, 1e-3, n).astype(F)
    g[::97] *= 100
    return p, g


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("adamw,bias", [(True, False), (True, True), (False, False), (False, True)])
@pytest.mark.parametrize("bf16", [False, True])
def test_adam_twin(oracle_c, fused, adamw, bias, bf16):
    p, g = _data()
    if bf16:
        p, g = O.f32_to_bf16(p), O.f32_to_bf16(g)
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    ref = O.AdamW(lr, b1, b2, eps, wd, bias) if adamw else O.Adam(lr, b1, b2, eps, bias)
    m = np.zeros(p.shape, F)
    v = np.zeros(p.shape, F)
    cur_ref, cur = p, p
    for step in range(1, 4):
        cur_ref = ref.update_single("p", cur_ref, g)
        bc1 = 1.0 / (1.0 - b1 ** step) if bias else 1.0
        bc2 = 1.0 / (1.0 - b2 ** step) if bias else 1.0
        args = B.adam_args(lr, b1, b2, eps, wd if adamw else None, bc1, bc2, bias_correction=bias)
        cur = oracle_c.adam(cur, g, m, v, args, fused=fused)
        assert np.array_equal(cur.view(np.uint32), cur_ref.view(np.uint32))
        assert np.array_equal(m.view(np.uint32), ref.state["p"][0].view(np.uint32))
        assert np.array_equal(v.view(np.uint32), ref.state["p"][1].view(np.uint32))


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("mom,damp,wd,nest", [(0.0, 0.0, 0.0, False), (0.9, 0.0, 1e-4, False),
                                              (0.9, 0.25, 0.0, False), (0.9, 0.0, 1e-4, True)])
def test_sgd_twin(oracle_c, fused, mom, damp, wd, nest):
    p, g = _data()
    ref = O.SGD(1e-2, mom, wd, damp, nest)
    v = np.zeros(p.shape, F)
    cur_ref = cur = p
    f = lambda x: float(np.float32(x))
    for step in range(3):
        cur_ref = ref.update_single("p", cur_ref, g)
        args = B.SgdArgs(lr=f(1e-2), momentum=f(mom), one_minus_damp=f(1.0 - damp), wd=f(wd),
                         has_wd=int(wd != 0), has_momentum=int(mom != 0), nesterov=int(nest), first=int(step == 0))
        cur = oracle_c.sgd(cur, g, v, args, fused=fused)
        assert np.array_equal(cur.view(np.uint32), cur_ref.view(np.uint32))
        if mom != 0:
            assert np.array_equal(v.view(np.uint32), ref.state["p"].view(np.uint32))


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_rmsprop_twin(oracle_c, fused, wd):
    p, g = _data()
    ref = O.RMSprop(1e-4, 0.99, 1e-8, wd)
    v = np.zeros(p.shape, F)
    cur_ref = cur = p
    f = lambda x: float(np.float32(x))
    for _ in range(3):
        cur_ref = ref.update_single("p", cur_ref, g)
        args = B.RmspropArgs(lr=f(1e-4), alpha=f(0.99), one_minus_alpha=f(1.0 - 0.99), eps=f(1e-8), wd=f(wd),
                             has_wd=int(wd != 0))
        cur = oracle_c.rmsprop(cur, g, v, args, fused=fused)
        assert np.array_equal(cur.view(np.uint32), cur_ref.view(np.uint32))
        assert np.array_equal(v.view(np.uint32), ref.state["p"].view(np.uint32))


def test_sumsq_bf16_accumulate_scale(oracle_c):
    p, g = _data(50001)
    gb = O.f32_to_bf16(g)
    assert np.array_equal(oracle_c.f32_to_bf16(g), gb)
    for x in (g, gb):
        want = O.exact_sumsq([x])
        assert abs(oracle_c.sumsq(x) - want) <= 1e-12 * want
    acc = np.empty(g.shape, F)
    oracle_c.accumulate_f32(acc, gb, True)
    ref = O.accumulate_fp32(None, gb)
    assert np.array_equal(acc, ref)
    oracle_c.accumulate_f32(acc, gb, False)
    assert np.array_equal(acc, O.accumulate_fp32(ref, gb))
    _, s = O.norm_scale_c1(O.exact_sumsq([gb]), 1e-3)
    assert np.array_equal(oracle_c.scale_f32(gb, float(s)), O.bf16_to_f32(gb) * s)
