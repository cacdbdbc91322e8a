"""GPU parity: every mxopt kernel, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Bar: bit-exact for float32 outputs and for bf16 write-back (the budget stated
for the path is 2 float32 ulp / 1 bf16 ulp; one rounding per reference op makes 0 reachable);
the global norm against the exact float64 value to rel 1e-5 (observed ~1e-12).
"""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32

# ragged sizes: empty, one element, around the 8-element group and the 4096-element chunk
SIZES = [0, 1, 7, 8, 9, 4095, 4096, 4097, 3 * 4096, 100003, 64, 1024]


@pytest.fixture(scope="module")
def mx():
    import torch
    import mxopt
    assert torch.cuda.is_available()
    return mxopt


@pytest.fixture(scope="module")
def ctx(mx):
    c = mx.Context()
    yield c
    c.close()


def make_lists(seed, sizes=SIZES, bf16=False, outliers=True):
    rng = np.random.default_rng(seed)
    ps, gs = [], []
    for n in sizes:
        p = rng.normal(0, 0.02, n).astype(F)
        g = rng.normal(0, 1e-3, n).astype(F)
        if outliers and n:
            g[rng.random(n) < 0.01] *= 100
        if bf16:
            p, g = O.f32_to_bf16(p), O.f32_to_bf16(g)
        ps.append(p)
        gs.append(g)
    return ps, gs


def device_scale(ctx, res, grads, max_norm):
    """The clip factor the device derived, after checking it against the oracle's (which uses the
    exact float64 norm): the two float32 norms may differ in the last place, never by more."""
    r = ctx.read_norm_result(res)
    n, s = O.norm_scale_c1(O.exact_sumsq(grads), max_norm)
    assert abs(r.norm - float(n)) <= 1e-5 * float(n)
    assert O.ulp_diff_f32(np.array([r.scale], F), np.array([s], F))[0] <= 1
    return F(r.scale)


def out_like(mx, p_dev, out_bf16):
    import torch
    return torch.empty_like(p_dev, dtype=torch.bfloat16 if out_bf16 else torch.float32)


def want_out(ref_f32, out_bf16):
    return O.f32_to_bf16(ref_f32) if out_bf16 else ref_f32


# ---------------------------------------------------------------------------------
# Adam / AdamW
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("adamw", [True, False])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("in_bf16,out_bf16", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("offset", [0, 1])
def test_adam_multi_tensor(mx, ctx, adamw, bias, in_bf16, out_bf16, offset):
    import torch
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    ps, gs = make_lists(11, bf16=in_bf16)
    ref = O.AdamW(lr, b1, b2, eps, wd, bias) if adamw else O.Adam(lr, b1, b2, eps, bias)
    hp = mx.adam_hp(lr, b1, b2, eps, wd if adamw else None)
    names = [f"t{i}" for i in range(len(ps))]
    dp = [to_dev(p, offset) for p in ps]
    dg = [to_dev(g, offset) for g in gs]
    dm = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    dv = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    do = [out_like(mx, p, out_bf16) for p in dp]
    table = ctx.table([mx.TensorSpec(p=p, p_out=o, g=g, m=m, v=v) for p, o, g, m, v in zip(dp, do, dg, dm, dv)])
    assert table.total_elems == sum(SIZES)
    cur = list(ps)
    step = 0
    for it in range(3):
        if bias:  # t counts update_single calls: tensor i of step s sees s*N + i + 1
            bcs = [mx.bias_correction(b1, b2, step + i + 1) for i in range(len(ps))]
            table.set_step_scalars([a for a, _ in bcs], [b for _, b in bcs])
        step += len(ps)
        ctx.adam(table, hp)
        ctx.synchronize()
        for i, name in enumerate(names):
            r = ref.update_single(name, cur[i], gs[i])
            assert_bit_equal(to_host(do[i]), want_out(r, out_bf16), f"param {name} it {it}")
            assert_bit_equal(to_host(dm[i]), ref.state[name][0], f"m {name} it {it}")
            assert_bit_equal(to_host(dv[i]), ref.state[name][1], f"v {name} it {it}")
            # feed the kernel's own output back, as a training loop would
            if in_bf16 and not out_bf16:
                cur[i] = O.f32_to_bf16(r)
                dp[i].copy_(do[i].to(torch.bfloat16))
            else:
                cur[i] = want_out(r, out_bf16)
                dp[i].copy_(do[i])


def test_adam_in_place_and_fp32_grad_for_bf16_param(mx, ctx):
    """bf16 parameter updated in place from a float32 gradient (the accumulation buffer)."""
    import torch
    lr, b1, b2, eps, wd = 5e-6, 0.9, 0.999, 1e-8, 0.01
    ps, _ = make_lists(5, bf16=True)
    _, gs = make_lists(6, bf16=False)
    ref = O.AdamW(lr, b1, b2, eps, wd)
    dp = [to_dev(p) for p in ps]
    dg = [to_dev(g) for g in gs]
    dm = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    dv = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    cur = list(ps)
    for it in range(2):
        ctx.adam(table, mx.adam_hp(lr, b1, b2, eps, wd))
        for i in range(len(ps)):
            cur[i] = O.f32_to_bf16(ref.update_single(str(i), cur[i], gs[i]))
            assert_bit_equal(to_host(dp[i]), cur[i], f"p{i} it{it}")
            assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v{i} it{it}")


@pytest.mark.parametrize("half", ["bf16", "f16"])
def test_square_of_a_16bit_gradient_is_taken_in_its_dtype(mx, ctx, half):
    """adamw.rs:92 / rmsprop.rs:80: mlx square keeps the gradient's dtype.  A 16-bit gradient that reaches the
    optimizer as it came gives a 16-bit square; one that a prep stage touched first (here: x 1.0) is float32
    by then and so is its square.  Both against the oracle, and the two must differ in v."""
    import torch
    rng = np.random.default_rng(31)
    n = 4096 * 3 + 11
    pf, gf = rng.normal(0, 0.02, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
    if half == "bf16":
        p, g = O.f32_to_bf16(pf), O.f32_to_bf16(gf)
    else:
        p, g = pf.astype(np.float16), gf.astype(np.float16)
    g32 = O.as_f32(g)

    def run(launch, prep):
        dp, dg = to_dev(p), to_dev(g)
        do = torch.empty(n, dtype=torch.float32, device="cuda")
        dm, dv = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
        t = ctx.table([mx.TensorSpec(p=dp, p_out=do, g=dg, m=dm, v=dv)])
        launch(t, prep)
        ctx.synchronize()
        return to_host(do), to_host(dv)

    adam = lambda t, prep: ctx.adam(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01), prep)
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    want_p = ref.update_single("w", p, g)
    got_p, got_v = run(adam, None)
    assert_bit_equal(got_v, ref.state["w"][1], "v, square in the gradient's dtype")
    assert_bit_equal(got_p, want_p, "p, square in the gradient's dtype")
    ref32 = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    want_p32 = ref32.update_single("w", p, g32 * F(1.0))
    got_p32, got_v32 = run(adam, mx.make_prep(pre_mul=1.0))
    assert_bit_equal(got_v32, ref32.state["w"][1], "v, gradient scaled first")
    assert_bit_equal(got_p32, want_p32, "p, gradient scaled first")
    assert not np.array_equal(got_v, got_v32)

    for wd in (0.0, 0.1):
        rms = lambda t, prep: ctx.rmsprop(t, mx.rmsprop_hp(1e-2, 0.99, 1e-8, wd), prep)
        r = O.RMSprop(1e-2, 0.99, 1e-8, wd)
        want = r.update_single("w", p, g)
        got_p, got_v = run(rms, None)
        assert_bit_equal(got_v, r.state["w"], f"rmsprop v, wd={wd}")
        assert_bit_equal(got_p, want, f"rmsprop p, wd={wd}")


@pytest.mark.parametrize("persistent,nontemporal,bpc", [(0, 0, 8), (1, 0, 1), (0, 1, 8)])
def test_adam_launch_options_do_not_change_results(mx, persistent, nontemporal, bpc):
    import torch
    c = mx.Context()
    c.set_option("persistent", persistent)
    c.set_option("nontemporal", nontemporal)
    c.set_option("grid_blocks_per_cu", bpc)
    ps, gs = make_lists(3, sizes=[4096 * 37 + 5, 9, 4096])
    ref = O.AdamW()
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    dm = [torch.zeros_like(p) for p in dp]
    dv = [torch.zeros_like(p) for p in dp]
    table = c.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    c.adam(table, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01))
    for i in range(len(ps)):
        assert_bit_equal(to_host(dp[i]), ref.update_single(str(i), ps[i], gs[i]), f"p{i}")
    table.close()
    c.close()


# ---------------------------------------------------------------------------------
# SGD, RMSprop
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("mom,damp,wd,nest", [(0.0, 0.0, 0.0, False), (0.9, 0.0, 1e-4, False),
                                              (0.9, 0.25, 0.0, False), (0.9, 0.0, 1e-4, True)])
@pytest.mark.parametrize("bf16", [False, True])
def test_sgd(mx, ctx, mom, damp, wd, nest, bf16):
    import torch
    ps, gs = make_lists(21, bf16=bf16)
    ref = O.SGD(1e-2, mom, wd, damp, nest)
    hp = mx.sgd_hp(1e-2, mom, wd, damp, nest)
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    do = [torch.empty(len(p), dtype=torch.float32, device="cuda") for p in ps]
    dv = [torch.full((len(p),), float("nan"), dtype=torch.float32, device="cuda") if mom else None for p in ps]
    table = ctx.table([mx.TensorSpec(p=p, p_out=o, g=g, v=v, flags=mx.TF_FIRST)
                       for p, o, g, v in zip(dp, do, dg, dv)])
    for it in range(3):
        if it == 1:
            table.set_step_scalars(flags=[0] * len(ps))
        ctx.sgd(table, hp)
        for i in range(len(ps)):
            r = ref.update_single(str(i), ps[i], gs[i])
            assert_bit_equal(to_host(do[i]), r, f"p{i} it{it}")
            if mom:
                assert_bit_equal(to_host(dv[i]), ref.state[str(i)], f"v{i} it{it}")


def test_sgd_nesterov_validation(mx):
    with pytest.raises(ValueError):
        mx.sgd_hp(0.1, 0.0, 0.0, 0.0, True)
    with pytest.raises(ValueError):
        mx.sgd_hp(0.1, 0.9, 0.0, 0.1, True)
    mx.sgd_hp(0.1, 0.9, 0.0, 0.0, True)


@pytest.mark.parametrize("wd", [0.0, 0.01])
@pytest.mark.parametrize("bf16", [False, True])
def test_rmsprop(mx, ctx, wd, bf16):
    import torch
    ps, gs = make_lists(31, bf16=bf16)
    ref = O.RMSprop(1e-4, 0.99, 1e-8, wd)
    hp = mx.rmsprop_hp(1e-4, 0.99, 1e-8, wd)
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    do = [torch.empty(len(p), dtype=torch.float32, device="cuda") for p in ps]
    dv = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    table = ctx.table([mx.TensorSpec(p=p, p_out=o, g=g, v=v) for p, o, g, v in zip(dp, do, dg, dv)])
    for it in range(3):
        ctx.rmsprop(table, hp)
        for i in range(len(ps)):
            assert_bit_equal(to_host(do[i]), ref.update_single(str(i), ps[i], gs[i]), f"p{i} it{it}")
            assert_bit_equal(to_host(dv[i]), ref.state[str(i)], f"v{i} it{it}")


# ---------------------------------------------------------------------------------
# apply_gradients (plain SGD in the parameter dtype)
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("p_bf16,g_bf16", [(False, False), (True, True), (True, False), (False, True)])
def test_sgd_plain(mx, ctx, p_bf16, g_bf16):
    ps, _ = make_lists(41, bf16=p_bf16)
    _, gs = make_lists(42, bf16=g_bf16)
    want = O.apply_gradients({str(i): p for i, p in enumerate(ps)}, {str(i): g for i, g in enumerate(gs)}, 2e-2)
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g) for p, g in zip(dp, dg)])
    ctx.sgd_plain(table, 2e-2)
    for i in range(len(ps)):
        assert_bit_equal(to_host(dp[i]), want[str(i)], f"p{i}")


def test_sgd_plain_with_l2_decay(mx, ctx):
    """sft/engine.rs:345-365: g + f32(wd)*p (float32), then apply_gradients."""
    ps, gs = make_lists(43, bf16=True)
    wd, lr = 0.01, 2e-5
    want = {}
    for i, (p, g) in enumerate(zip(ps, gs)):
        gd = O.as_f32(g) + O.mul_scalar(p, wd)
        want[str(i)] = O.apply_gradients({"w": p}, {"w": gd}, lr)["w"]
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g) for p, g in zip(dp, dg)])
    ctx.sgd_plain(table, lr, wd)
    for i in range(len(ps)):
        assert_bit_equal(to_host(dp[i]), want[str(i)], f"p{i}")


# ---------------------------------------------------------------------------------
# Global norm, clip scale, transform
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("offset", [0, 3])
def test_global_norm_and_scales(mx, ctx, bf16, offset):
    _, gs = make_lists(51, bf16=bf16, sizes=SIZES + [4096 * 300 + 17])
    dg = [to_dev(g, offset) for g in gs]
    table = ctx.table([mx.TensorSpec(g=g) for g in dg])
    res = ctx.norm_result()
    exact = O.exact_sumsq(gs)
    for max_norm in (1e-3, 1e6):
        ctx.global_norm(table, res, max_norm=max_norm)
        r = ctx.read_norm_result(res)
        assert abs(r.sumsq - exact) <= 1e-6 * exact
        assert abs(r.norm - math.sqrt(exact)) <= 1e-5 * math.sqrt(exact)
        n, s = O.norm_scale_c1(r.sumsq, max_norm)   # scalar chain of optimizers/mod.rs:87-96
        assert F(r.norm_f32) == n and F(r.scale) == s
        assert r.nonfinite == 0
        # Vec API rule (gradients/mod.rs:255-270)
        ctx.global_norm(table, res, max_norm=max_norm, clip_mode=mx.CLIP_IF_ABOVE)
        r2 = ctx.read_norm_result(res)
        want = F(1.0) if r2.norm <= max_norm else F(max_norm / (r2.norm + 1e-6))
        assert F(r2.scale) == want
    ctx.global_norm(table, res)            # no max: scale stays 1
    assert ctx.read_norm_result(res).scale == 1.0


def test_global_norm_is_deterministic_and_flags_nonfinite(mx, ctx):
    _, gs = make_lists(52, sizes=[4096 * 50 + 1, 77])
    gs[0][5] = np.inf
    gs[0][4096 * 3] = np.nan
    gs[1][76] = -np.inf
    dg = [to_dev(g) for g in gs]
    table = ctx.table([mx.TensorSpec(g=g) for g in dg])
    res = ctx.norm_result()
    ctx.global_norm(table, res, max_norm=1.0)
    r = ctx.read_norm_result(res)
    assert r.nonfinite == 1 and math.isnan(r.sumsq) and math.isnan(r.scale)   # a flag, not a count
    gs[0][5] = gs[0][4096 * 3] = 0
    gs[1][76] = 0
    dg = [to_dev(g) for g in gs]
    table = ctx.table([mx.TensorSpec(g=g) for g in dg])
    seen = set()
    for _ in range(5):
        ctx.global_norm(table, res, max_norm=1.0)
        seen.add(ctx.read_norm_result(res).sumsq)
    assert len(seen) == 1


@pytest.mark.parametrize("bf16,keep_dtype", [(False, False), (True, False), (True, True)])
def test_clip_grad_norm_transform(mx, ctx, bf16, keep_dtype):
    """GradientUtils::clip_grad_norm end to end on the device: norm -> scale -> g * scale."""
    import torch
    _, gs = make_lists(53, bf16=bf16)
    dg = [to_dev(g) for g in gs]
    out = [torch.empty(len(g), dtype=torch.bfloat16 if keep_dtype else torch.float32, device="cuda") for g in gs]
    table = ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(dg, out)])
    res = ctx.norm_result()
    max_norm = 1e-2
    ctx.global_norm(table, res, max_norm=max_norm)
    ctx.grad_transform(table, mx.make_prep(scale=res))
    scale = device_scale(ctx, res, gs, max_norm)
    for i in range(len(gs)):
        w = O.as_f32(gs[i]) * scale          # optimizers/mod.rs:98-102
        assert_bit_equal(to_host(out[i]), O.f32_to_bf16(w) if keep_dtype else w, f"g{i}")


def test_clamp_then_norm_then_scale(mx, ctx):
    """clip_grad_value_and_norm (optimizers/mod.rs:174-226): clamp, norm of the clamped, scale."""
    import torch
    _, gs = make_lists(54)
    gs[3][2] = np.nan
    gsd = {str(i): g for i, g in enumerate(gs)}
    clip_v, max_norm = 5e-3, 1e-2
    dg = [to_dev(g) for g in gs]
    out = [torch.empty_like(g) for g in dg]
    table = ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(dg, out)])
    # value clamp alone (clip_grad_value, optimizers/mod.rs:164-166)
    ctx.grad_transform(table, mx.make_prep(clamp_pre=(-clip_v, clip_v)))
    for i, g in enumerate(gs):
        assert_bit_equal(to_host(out[i]), O.clip_value(g, -clip_v, clip_v), f"clamp{i}")
    gs[3][2] = 0.0
    dg[3].copy_(to_dev(gs[3]))
    res = ctx.norm_result()
    prep = mx.make_prep(clamp_pre=(-clip_v, clip_v))
    ctx.global_norm(table, res, prep=prep, max_norm=max_norm)
    ctx.grad_transform(table, mx.make_prep(clamp_pre=(-clip_v, clip_v), scale=res))
    clamped = [O.clip_value(g, -clip_v, clip_v) for g in gs]
    scale = device_scale(ctx, res, clamped, max_norm)
    for i in range(len(gs)):
        assert_bit_equal(to_host(out[i]), clamped[i] * scale, f"g{i}")


# ---------------------------------------------------------------------------------
# Accumulation
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("acc_bf16,g_bf16", [(False, True), (False, False), (True, True)])
def test_accumulate(mx, ctx, acc_bf16, g_bf16):
    import torch
    micro = [make_lists(60 + k, bf16=g_bf16)[1] for k in range(4)]
    n_t = len(micro[0])
    acc = [torch.full((len(g),), float("nan"), dtype=torch.bfloat16 if acc_bf16 else torch.float32, device="cuda")
           for g in micro[0]]
    dg = [to_dev(g) for g in micro[0]]
    table = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, acc)])
    res = ctx.norm_result()
    ref = [None] * n_t
    for k in range(4):
        for i in range(n_t):
            dg[i].copy_(to_dev(micro[k][i]))
            if acc_bf16:   # reference semantics: bf16 + bf16 -> bf16 (model.rs:2227)
                ref[i] = (np.array(micro[k][i], copy=True) if ref[i] is None
                          else O.accumulate_gradients({"w": ref[i]}, {"w": micro[k][i]})["w"])
            else:
                ref[i] = O.accumulate_fp32(ref[i], micro[k][i])
        last = k == 3
        ctx.accumulate(table, first=(k == 0), out=res if last else None, max_norm=1.0)
        for i in range(n_t):
            assert_bit_equal(to_host(acc[i]), ref[i], f"acc{i} micro{k}")
    r = ctx.read_norm_result(res)
    exact = O.exact_sumsq(ref)
    assert abs(r.sumsq - exact) <= 1e-6 * exact
    n, s = O.norm_scale_c1(r.sumsq, 1.0)
    assert F(r.scale) == s and F(r.norm_f32) == n


def test_sft_pipeline_average_clip_clamp_adamw(mx, ctx):
    """accumulate -> x(1/N) -> clip-norm -> clamp, fused into the AdamW kernel's registers, against
    the same sequence of separate oracle ops (sft/engine.rs:282-329 ordering)."""
    import torch
    N, max_norm, clip_v = 4, 1e-3, 2e-4
    ps, _ = make_lists(70, bf16=True)
    micro = [make_lists(71 + k, bf16=True)[1] for k in range(N)]
    n_t = len(ps)
    acc_ref = [None] * n_t
    for k in range(N):
        for i in range(n_t):
            acc_ref[i] = O.accumulate_fp32(acc_ref[i], micro[k][i])
    avg = [O.mul_scalar(a, 1.0 / N) for a in acc_ref]

    dp = [to_dev(p) for p in ps]
    dg = [to_dev(g) for g in micro[0]]
    acc = [torch.empty(len(p), dtype=torch.float32, device="cuda") for p in ps]
    dm = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    dv = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
    t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, acc)])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, m=m, v=v) for p, a, m, v in zip(dp, acc, dm, dv)])
    res = ctx.norm_result()
    inv_n = float(F(1.0 / N))
    for k in range(N):
        for i in range(n_t):
            dg[i].copy_(to_dev(micro[k][i]))
        ctx.accumulate(t_acc, first=(k == 0), out=res if k == N - 1 else None,
                       prep=mx.make_prep(pre_mul=inv_n), max_norm=max_norm)
    ctx.adam(t_upd, mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01),
             mx.make_prep(pre_mul=inv_n, scale=res, clamp_post=(-clip_v, clip_v)))
    scale = device_scale(ctx, res, avg, max_norm)
    final = [O.clip_value(a * scale, -clip_v, clip_v) for a in avg]
    ref = O.AdamW(5e-6, 0.9, 0.999, 1e-8, 0.01)
    for i in range(n_t):
        want = O.f32_to_bf16(ref.update_single(str(i), ps[i], final[i]))
        assert_bit_equal(to_host(dp[i]), want, f"p{i}")
        assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"m{i}")
        assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v{i}")


# ---------------------------------------------------------------------------------
# Error paths (host-side validation; nothing is launched)
# ---------------------------------------------------------------------------------

def test_errors(mx, ctx):
    import torch
    g = torch.zeros(16, device="cuda")
    table = ctx.table([mx.TensorSpec(g=g)])
    with pytest.raises(ValueError, match="NULL pointer"):
        ctx.adam(table, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8))
    with pytest.raises(ValueError):
        ctx.table([mx.TensorSpec(g=torch.zeros(4, dtype=torch.int32, device="cuda"))])
    with pytest.raises(ValueError):
        mx.TensorSpec(p=torch.zeros(4, device="cuda"), g=torch.zeros(5, device="cuda")).to_c()
    with pytest.raises(ValueError):
        ctx.set_option("no_such_option", 1)
    other = mx.Context()
    with pytest.raises(ValueError, match="another context"):
        other.global_norm(table, other.norm_result())
    other.close()
    empty = ctx.table([])
    ctx.global_norm(empty, ctx.norm_result(), max_norm=1.0)   # legal: norm 0, scale 1


# ---------------------------------------------------------------------------------
# Last micro-batch folded into the update; skip-on-non-finite policy
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("g_bf16", [True, False])
def test_pending_micro_batch_equals_accumulate_then_adam(mx, ctx, g_bf16):
    """accumulate_norm_only + adam_with_pending give the numbers of accumulate(+norm) + adam,
    without writing the accumulation buffer a last time."""
    import torch
    ps, _ = make_lists(80, bf16=True)
    micro = [make_lists(81 + k, bf16=g_bf16)[1] for k in range(3)]
    n_t = len(ps)
    hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
    results = []
    for fused in (False, True):
        dp = [to_dev(p) for p in ps]
        dg = [to_dev(g) for g in micro[0]]
        acc = [torch.empty(len(p), dtype=torch.float32, device="cuda") for p in ps]
        dm = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
        dv = [torch.zeros(len(p), dtype=torch.float32, device="cuda") for p in ps]
        t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, acc)])
        res = ctx.norm_result()
        for k in range(3):
            for i in range(n_t):
                dg[i].copy_(to_dev(micro[k][i]))
            last = k == 2
            if last and fused:
                ctx.accumulate_norm_only(t_acc, res, max_norm=1e-3)
            else:
                ctx.accumulate(t_acc, first=(k == 0), out=res if last else None, max_norm=1e-3)
        prep = mx.make_prep(scale=res)
        if fused:
            t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=m, v=v)
                           for p, a, g, m, v in zip(dp, acc, dg, dm, dv)])
            ctx.adam_with_pending(t, hp, prep)
        else:
            t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, m=m, v=v) for p, a, m, v in zip(dp, acc, dm, dv)])
            ctx.adam(t, hp, prep)
        r = ctx.read_norm_result(res)
        results.append((r.sumsq, r.scale, [to_host(x) for x in dp], [to_host(x) for x in dm], [to_host(x) for x in dv]))
    a, b = results
    assert a[0] == b[0] and a[1] == b[1]
    for i in range(n_t):
        assert_bit_equal(b[2][i], a[2][i], f"p{i}")
        assert_bit_equal(b[3][i], a[3][i], f"m{i}")
        assert_bit_equal(b[4][i], a[4][i], f"v{i}")
    # and the un-fused side is the oracle's
    acc_ref = [None] * n_t
    for k in range(3):
        for i in range(n_t):
            acc_ref[i] = O.accumulate_fp32(acc_ref[i], micro[k][i])
    ref = O.AdamW(5e-6, 0.9, 0.999, 1e-8, 0.01)
    for i in range(n_t):
        want = O.f32_to_bf16(ref.update_single(str(i), ps[i], acc_ref[i] * F(a[1])))
        assert_bit_equal(a[2][i], want, f"oracle p{i}")


def test_skip_step_when_a_gradient_is_not_finite(mx, ctx):
    """grpo/engine.rs:561-607: any NaN/Inf gradient => nothing is modified.  The counter comes from
    the norm pass; no host round trip."""
    import torch
    ps, gs = make_lists(90, sizes=[4096 * 3 + 5, 100, 4096])
    for poison in (True, False):
        g2 = [g.copy() for g in gs]
        if poison:
            g2[0][4096 + 17] = np.nan
        dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in g2]
        dm = [torch.zeros_like(p) for p in dp]
        dv = [torch.zeros_like(p) for p in dp]
        out = [torch.full_like(g, 7.0) for g in dg]
        t_g = ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(dg, out)])
        t_u = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
        res = ctx.norm_result()
        ctx.global_norm(t_g, res, max_norm=1.0)
        prep = mx.make_prep(scale=res, skip_if_nonfinite=res)
        ctx.adam(t_u, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01), prep)
        ctx.grad_transform(t_g, prep)
        assert ctx.read_norm_result(res).nonfinite == (1 if poison else 0)
        for i in range(len(ps)):
            changed = not np.array_equal(to_host(dp[i]), ps[i])
            assert changed != poison, f"tensor {i}"
            assert (to_host(dm[i]) == 0).all() == poison
            assert (to_host(out[i]) == 7.0).all() == poison


# ---------------------------------------------------------------------------------
# Tensors whose streams all start the same number of elements off a 16-byte boundary (views into
# packed slabs): a few head elements are peeled and the rest takes the 128-bit path.
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("shift", [1, 2, 3, 5, 7])
def test_common_shift_of_all_streams(mx, ctx, shift):
    import torch
    sizes = [1, 2, shift, shift + 1, 7, 8, 9, 15, 4096, 4096 + shift, 4097 + shift, 2 * 4096 + shift - 1, 50001]
    ps, gs = make_lists(70 + shift, sizes=sizes, bf16=True)
    zeros = [np.zeros(n, F) for n in sizes]
    dp, dg = [to_dev(p, shift) for p in ps], [to_dev(g, shift) for g in gs]
    dm, dv, da = ([to_dev(z, shift) for z in zeros] for _ in range(3))
    for a in da:
        a.fill_(float("nan"))
    res = ctx.norm_result()
    t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, da)])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=m, v=v)
                       for p, a, g, m, v in zip(dp, da, dg, dm, dv)])
    ctx.accumulate(t_acc, first=True)
    ctx.accumulate(t_acc, first=False)
    ctx.accumulate_norm_only(t_acc, res, max_norm=1e-3)
    acc2 = [O.accumulate_fp32(O.accumulate_fp32(None, g), g) for g in gs]
    acc3 = [O.accumulate_fp32(a, g) for a, g in zip(acc2, gs)]
    for i in range(len(sizes)):
        assert_bit_equal(to_host(da[i]), acc2[i], f"acc {i}")
    scale = device_scale(ctx, res, acc3, 1e-3)
    ctx.adam_with_pending(t_upd, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01), mx.make_prep(scale=res))
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    for i in range(len(sizes)):
        want = O.f32_to_bf16(ref.update_single(str(i), ps[i], acc3[i] * scale))
        assert_bit_equal(to_host(dp[i]), want, f"p {i} (n={sizes[i]})")
        assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"m {i}")
        assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v {i}")
    # gradient transform and a separate norm pass over the same views
    out = [to_dev(z, shift) for z in zeros]
    t_g = ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(dg, out)])
    ctx.global_norm(t_g, res, max_norm=1e-3)
    s2 = device_scale(ctx, res, gs, 1e-3)
    ctx.grad_transform(t_g, mx.make_prep(scale=res))
    for i in range(len(sizes)):
        assert_bit_equal(to_host(out[i]), O.bf16_to_f32(gs[i]) * s2, f"scaled g {i}")
    for t in (t_acc, t_upd, t_g):
        t.close()


# ---------------------------------------------------------------------------------
# One table, several dtype combinations: one launch per group, one norm over all of them
# ---------------------------------------------------------------------------------

def test_mixed_dtype_table(mx, ctx):
    import torch
    rng = np.random.default_rng(404)
    sizes = [100003, 4096, 7, 0, 12289, 4097, 64, 9000]
    kinds = ["f32/f32", "bf16/bf16", "bf16/f32", "f32/bf16", "bf16/bf16", "f32/f32", "bf16/f32", "f32/bf16"]
    ps, gs = [], []
    for n, k in zip(sizes, kinds):
        p = rng.normal(0, 0.02, n).astype(F)
        g = rng.normal(0, 1e-3, n).astype(F)
        pk, gk = k.split("/")
        ps.append(O.f32_to_bf16(p) if pk == "bf16" else p)
        gs.append(O.f32_to_bf16(g) if gk == "bf16" else g)
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    dm = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
    dv = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
    res = ctx.norm_result()
    t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    assert t_upd.total_elems == sum(sizes)
    hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    cur = list(ps)
    for it in range(2):
        ctx.global_norm(t_g, res, max_norm=1e-2)
        scale = device_scale(ctx, res, gs, 1e-2)
        ctx.adam(t_upd, hp, mx.make_prep(scale=res))
        for i in range(len(sizes)):
            r = ref.update_single(str(i), cur[i], O.as_f32(gs[i]) * scale)
            cur[i] = O.f32_to_bf16(r) if cur[i].dtype == np.uint16 else r
            assert_bit_equal(to_host(dp[i]), cur[i], f"p{i} ({kinds[i]}) it {it}")
            assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"m{i} it {it}")
            assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v{i} it {it}")
    t_g.close()
    t_upd.close()


# ---------------------------------------------------------------------------------
# A table follows its tensors to new buffers
# ---------------------------------------------------------------------------------

def test_table_retarget(mx, ctx):
    import torch
    hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
    sizes = [5, 4096, 12289, 100003]
    table = None
    for rnd in range(3):
        ps, gs = make_lists(500 + rnd, sizes=sizes, bf16=True)
        dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
        dm = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
        dv = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
        rows = [mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)]
        if table is None:
            table = ctx.table(rows)
            chunks = table.num_chunks
        else:
            table.retarget(rows)
            assert table.num_chunks == chunks
        ctx.adam(table, hp)
        ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
        for i in range(len(sizes)):
            assert_bit_equal(to_host(dp[i]), O.f32_to_bf16(ref.update_single(str(i), ps[i], gs[i])), f"round {rnd} p{i}")
            assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"round {rnd} m{i}")
    # a different layout is refused and leaves the table as it was
    other = [mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)]
    other[1] = mx.TensorSpec(p=dp[1][:100], p_out=dp[1][:100], g=dg[1][:100], m=dm[1][:100], v=dv[1][:100])
    with pytest.raises(ValueError, match="different layout"):
        table.retarget(other)
    shifted = list(rows)
    shifted[2] = mx.TensorSpec(p=dp[2][1:], p_out=dp[2][1:], g=dg[2][1:], m=dm[2][1:], v=dv[2][1:])
    with pytest.raises(ValueError):
        table.retarget(shifted)
    before = [to_host(p) for p in dp]
    ctx.adam(table, hp)
    ref2 = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    ref2.state = ref.state
    for i in range(len(sizes)):
        assert_bit_equal(to_host(dp[i]), O.f32_to_bf16(ref2.update_single(str(i), before[i], gs[i])), f"after refusal p{i}")
    table.close()


# ---------------------------------------------------------------------------------
# Subnormal float32 intermediates (g*g around 1e-40, sqrt and divide of such values) are kept, as a
# CPU float32 op chain keeps them: nothing is flushed to zero.
# ---------------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["adamw", "rmsprop", "sgd"])
def test_subnormal_intermediates(mx, ctx, kind):
    import torch
    rng = np.random.default_rng(77)
    n = 9001
    p = rng.normal(0, 1e-18, n).astype(F)
    g = (rng.normal(0, 1, n) * 10.0 ** rng.uniform(-24, -18, n)).astype(F)     # squares between 1e-48 and 1e-36
    g[:16] = (rng.normal(0, 1, 16) * 1e-41).astype(F)                           # subnormal gradients themselves
    assert (np.abs(g[:16]) < np.finfo(F).tiny).any()
    dp, dg = to_dev(p), to_dev(g)
    dm = torch.zeros(n, dtype=torch.float32, device="cuda")
    dv = torch.zeros(n, dtype=torch.float32, device="cuda")
    do = torch.empty(n, dtype=torch.float32, device="cuda")
    if kind == "adamw":
        ref, run = O.AdamW(1e-3, 0.9, 0.999, 1e-30, 0.01), lambda t: ctx.adam(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-30, 0.01))
        row = mx.TensorSpec(p=dp, p_out=do, g=dg, m=dm, v=dv)
    elif kind == "rmsprop":
        ref, run = O.RMSprop(1e-3, 0.99, 1e-30, 0.0), lambda t: ctx.rmsprop(t, mx.rmsprop_hp(1e-3, 0.99, 1e-30, 0.0))
        row = mx.TensorSpec(p=dp, p_out=do, g=dg, v=dv)
    else:
        ref, run = O.SGD(1e-3, 0.9, 1e-4), lambda t: ctx.sgd(t, mx.sgd_hp(1e-3, 0.9, 1e-4))
        row = mx.TensorSpec(p=dp, p_out=do, g=dg, v=dv, flags=mx.TF_FIRST)
    table = ctx.table([row])
    cur = p
    for it in range(3):
        if kind == "sgd" and it == 1:
            table.set_step_scalars(flags=[0])
        run(table)
        with np.errstate(under="ignore"):
            cur = ref.update_single("w", cur, g)
        assert_bit_equal(to_host(do), cur, f"{kind} it {it}")
        state = ref.state["w"]
        v_ref = state[1] if isinstance(state, tuple) else state
        assert_bit_equal(to_host(dv), v_ref, f"{kind} v it {it}")
        if kind == "adamw":
            assert (np.abs(v_ref[v_ref != 0]) < np.finfo(F).tiny).any()        # the test does reach subnormals
        dp.copy_(do)
    table.close()


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("where", ["full chunk", "last chunk", "head"])
@pytest.mark.parametrize("path", ["norm", "accumulate", "norm_only", "list"])
def test_validity_flag_tells_invalid_elements_from_overflowing_squares(mx, ctx, bf16, where, path):
    """Without a clamp the flag is the engines' per-element test (grpo/engine.rs:563-569): bit 0 says "some
    element is a NaN or an infinity".  A finite 1e20 is a valid gradient whose square leaves float32 range: the
    reference's own sum of squares becomes +Inf there, its clip factor 0 (optimizers/mod.rs:87-96), and the step
    is taken with zeroed gradients -- so the flag reads 2, the factor 0, and a kernel told to skip on the flag
    still runs.  A real infinity reads 1 and the kernel does nothing."""
    import torch
    sizes = [3 * 4096 + 100, 300]
    _, gs = make_lists(90, sizes=sizes, bf16=bf16, outliers=False)
    shift = 1 if where == "head" else 0          # a one-element shift: the vector path runs behind a peeled head
    at = {"full chunk": 4096 + 77, "last chunk": 3 * 4096 + 50, "head": 0}[where]

    def put(value):
        out = [g.copy() for g in gs]
        if bf16:
            out[0][at] = O.f32_to_bf16(np.array([value], F))[0]
        else:
            out[0][at] = value
        return out

    def flag_of(grads):
        shift_g = shift * (7 if bf16 else 3)     # 14 / 12 bytes in: every stream of the row is aligned again one element later
        dg = [to_dev(g, shift_g) for g in grads]
        res = ctx.norm_result()
        if path == "norm":
            t = ctx.table([mx.TensorSpec(g=g) for g in dg])
            ctx.global_norm(t, res, max_norm=1.0)
        elif path == "list":
            dz = [to_dev(np.zeros_like(g), shift_g) for g in grads]
            t = ctx.table([mx.TensorSpec(g=z) for z in dz])
            t.set_pending([dg])
            ctx.norm_with_pending_list(t, res, max_norm=1.0)
        else:
            da = [to_dev(np.zeros(g.size, F), shift * 3) for g in grads]
            t = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, da)])
            if path == "accumulate":
                ctx.accumulate(t, first=False, out=res, max_norm=1.0)
            else:
                ctx.accumulate_norm_only(t, res, max_norm=1.0)
        r = ctx.read_norm_result(res)
        # what a kernel that obeys the flag does afterwards
        dst = [torch.full((g.size,), 7.0, device="cuda") for g in grads]
        tt = ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(dg, dst)])
        ctx.grad_transform(tt, mx.make_prep(scale=res, skip_if_nonfinite=res))
        ran = bool((dst[1] != 7.0).any())
        t.close(); tt.close()
        return r, ran, dst

    r, ran, _ = flag_of(put(0.001))
    assert r.nonfinite == 0 and ran
    r, ran, dst = flag_of(put(1e20))
    assert r.nonfinite == 2 and math.isinf(r.sumsq) and r.scale == 0.0 and ran
    assert float(dst[0].abs().max()) == 0.0 and float(dst[1].abs().max()) == 0.0     # finite gradients times 0
    for bad in (np.inf, -np.inf, np.nan):
        r, ran, _ = flag_of(put(bad))
        assert r.nonfinite == 1 and math.isnan(r.sumsq) and not ran
