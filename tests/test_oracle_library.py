"""Pins the oracle's formulae against routines that are not the reference: torch.optim,
torch.nn.utils.clip_grad_norm_, torch's bf16 conversion, and float64 brute force.

torch fuses and orders the float32 operations differently, so these agree to ~1e-6
relative (they catch a dropped term, a wrong sign, eps inside the square root, coupled vs
decoupled decay ...), not bit for bit.
"""
import math

import numpy as np
import pytest
import torch

import mxopt_oracle as O

F = np.float32


def _run_torch(opt_factory, p0, grads):
    p = torch.nn.Parameter(torch.tensor(p0, dtype=torch.float32))
    opt = opt_factory([p])
    for g in grads:
        p.grad = torch.tensor(g, dtype=torch.float32)
        opt.step()
    return p.detach().numpy()


def _run_oracle(opt, p0, grads):
    p = p0.copy()
    for g in grads:
        p = opt.update_single("p", p, g)
    return p


@pytest.fixture
def data():
    rng = np.random.default_rng(7)
    p0 = rng.normal(0, 0.5, 4096).astype(F)
    grads = [rng.normal(0, 0.1, 4096).astype(F) for _ in range(6)]
    return p0, grads


def test_adam_matches_torch(data):
    p0, grads = data
    want = _run_torch(lambda ps: torch.optim.Adam(ps, lr=1e-2, betas=(0.9, 0.999), eps=1e-8), p0, grads)
    got = _run_oracle(O.Adam(1e-2, 0.9, 0.999, 1e-8, True), p0, grads)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)


def test_adamw_matches_torch(data):
    p0, grads = data
    want = _run_torch(lambda ps: torch.optim.AdamW(ps, lr=1e-2, betas=(0.9, 0.99), eps=1e-8, weight_decay=0.1),
                      p0, grads)
    got = _run_oracle(O.AdamW(1e-2, 0.9, 0.99, 1e-8, 0.1, True), p0, grads)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)
    # eps is OUTSIDE the square root and applied AFTER correcting v: a variant with eps inside fails this
    bad = _run_oracle(O.AdamW(1e-2, 0.9, 0.99, 1e-3, 0.1, True), p0, grads)
    assert np.abs(bad - want).max() > 1e-4


@pytest.mark.parametrize("momentum,damp,wd", [(0.0, 0.0, 0.0), (0.9, 0.0, 1e-4), (0.8, 0.3, 0.01)])
def test_sgd_matches_torch(data, momentum, damp, wd):
    p0, grads = data
    want = _run_torch(lambda ps: torch.optim.SGD(ps, lr=0.05, momentum=momentum, dampening=damp,
                                                 weight_decay=wd), p0, grads)
    got = _run_oracle(O.SGD(0.05, momentum, wd, damp), p0, grads)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_rmsprop_matches_torch(data, wd):
    p0, grads = data
    want = _run_torch(lambda ps: torch.optim.RMSprop(ps, lr=1e-3, alpha=0.99, eps=1e-8, weight_decay=wd),
                      p0, grads)
    got = _run_oracle(O.RMSprop(1e-3, 0.99, 1e-8, wd), p0, grads)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("max_norm", [0.5, 1e6])
def test_clip_grad_norm_matches_torch(max_norm):
    rng = np.random.default_rng(3)
    gs = {f"t{i}": rng.normal(0, 1, n).astype(F) for i, n in enumerate((5, 1000, 77))}
    ps = [torch.nn.Parameter(torch.zeros(len(g))) for g in gs.values()]
    for p, g in zip(ps, gs.values()):
        p.grad = torch.tensor(g)
    total = torch.nn.utils.clip_grad_norm_(ps, max_norm)   # max/(n+1e-6) clamped to 1
    got, n = O.GradientUtils.clip_grad_norm_with_norm(gs, max_norm)
    assert abs(n - float(total)) / float(total) < 1e-6
    for p, k in zip(ps, gs):
        np.testing.assert_allclose(got[k], p.grad.numpy(), rtol=1e-6, atol=0)


def test_bf16_round_trip_matches_torch():
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.normal(0, 1, 100000).astype(F),
                        (rng.normal(0, 1, 1000) * 1e-38).astype(F),          # subnormals
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 3.3895314e38, 1.0039062, 1.0117188],
                                 dtype=F)])
    # every tie pattern: all 65536 upper halves with lower half exactly 0x8000
    ties = ((np.arange(65536, dtype=np.uint32) << 16) | 0x8000).view(F)
    x = np.concatenate([x, ties])
    want = torch.tensor(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.f32_to_bf16(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(O.bf16_to_f32(got[nan])).all()
    back = torch.tensor(want.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(O.bf16_to_f32(want)[~nan], back[~nan])


def test_f64_brute_force_bounds_adamw():
    """The float32 op chain stays within a few ulp of the same formula evaluated in float64."""
    rng = np.random.default_rng(5)
    p = rng.normal(0, 0.02, 2048).astype(F)
    g = rng.normal(0, 1e-3, 2048).astype(F)
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    got = O.AdamW(lr, b1, b2, eps, wd).update_single("p", p, g)
    P, G = p.astype(np.float64), g.astype(np.float64)
    m = (1 - b1) * G
    v = (1 - b2) * G * G
    want = P * (1 - lr * wd) - lr * m / (np.sqrt(v) + eps)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-9)


def test_apply_gradients_bf16_roundings():
    """bf16 params: lr is rounded to bf16, lr*g is rounded to bf16, p - lr*g is rounded to bf16
    (models/qwen3/model.rs:2434-2451).  torch's bf16 CPU arithmetic rounds once per op too."""
    rng = np.random.default_rng(9)
    p = torch.tensor(rng.normal(0, 0.02, 4096).astype(F)).to(torch.bfloat16)
    g = torch.tensor(rng.normal(0, 1e-1, 4096).astype(F)).to(torch.bfloat16)
    lr = torch.tensor(2e-2, dtype=torch.float32).to(torch.bfloat16)
    want = (p - lr * g).view(torch.int16).numpy().view(np.uint16)
    pb = p.view(torch.int16).numpy().view(np.uint16)
    gb = g.view(torch.int16).numpy().view(np.uint16)
    got = O.apply_gradients({"w": pb}, {"w": gb}, 2e-2)["w"]
    assert np.array_equal(got, want)


def test_bf16_accumulate_matches_torch():
    rng = np.random.default_rng(10)
    a = torch.tensor(rng.normal(0, 1, 4096).astype(F)).to(torch.bfloat16)
    b = torch.tensor(rng.normal(0, 1, 4096).astype(F)).to(torch.bfloat16)
    want = (a + b).view(torch.int16).numpy().view(np.uint16)
    ab = a.view(torch.int16).numpy().view(np.uint16)
    bb = b.view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.accumulate_gradients({"w": ab}, {"w": bb})["w"], want)


def test_square_of_a_16bit_gradient_is_a_16bit_tensor_like_torch():
    """mlx square keeps its operand's dtype (crates/mlx-sys/src/mlx.cpp:2016-2020), so Adam's and RMSprop's
    g*g of a bf16 / float16 gradient is rounded to that dtype before the float32 scalar multiply promotes it
    (adamw.rs:92-94, rmsprop.rs:80-82).  torch's CPU square of a bf16 / float16 tensor is the same single
    rounding of the exact product; it pins the rounding model, and the optimizers must show it in v."""
    rng = np.random.default_rng(21)
    x = np.concatenate([rng.normal(0, 1e-3, 4000), rng.normal(0, 30.0, 1000), [0.0, -0.0, 1e-20, 250.0, 6e4]]).astype(F)
    bits = O.f32_to_bf16(x)
    t = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    want = t.square().view(torch.int16).numpy().view(np.uint16)
    got = O.f32_to_bf16(O.square_in_dtype_of(bits, O.bf16_to_f32(bits)))
    assert np.array_equal(got, want)
    assert np.array_equal(O.bf16_to_f32(got), O.square_in_dtype_of(bits, O.bf16_to_f32(bits)))   # already a bf16 value
    h = x.astype(np.float16)
    want16 = torch.from_numpy(h.copy()).square().numpy()
    got16 = O.square_in_dtype_of(h, h.astype(F))
    assert np.array_equal(got16.astype(np.float16).view(np.uint16), want16.view(np.uint16))
    assert np.array_equal(O.square_in_dtype_of(x, x), x * x)                                   # float32: no extra rounding
    # the optimizers: v after one step from zero state is (1 - beta2) * square, square in the gradient's dtype
    g = bits[:4000]
    p = O.f32_to_bf16(rng.normal(0, 0.02, 4000).astype(F))
    opt = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    opt.update_single("w", p, g)
    gf = O.bf16_to_f32(g)
    assert np.array_equal(opt.state["w"][1], O.bf16_to_f32(O.f32_to_bf16(gf * gf)) * F(1.0 - 0.999))
    assert not np.array_equal(opt.state["w"][1], (gf * gf) * F(1.0 - 0.999))                  # the rounding shows
    opt32 = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    opt32.update_single("w", p, gf)                                                           # the same values as float32
    assert np.array_equal(opt32.state["w"][1], (gf * gf) * F(1.0 - 0.999))
    r = O.RMSprop(1e-2, 0.99, 1e-8, 0.0)
    r.update_single("w", p, g)
    assert np.array_equal(r.state["w"], O.bf16_to_f32(O.f32_to_bf16(gf * gf)) * F(1.0 - 0.99))
    rw = O.RMSprop(1e-2, 0.99, 1e-8, 0.1)                                                     # coupled decay promotes first
    rw.update_single("w", p, g)
    ge = gf + O.bf16_to_f32(p) * F(0.1)
    assert np.array_equal(rw.state["w"], (ge * ge) * F(1.0 - 0.99))
