"""GPU parity of deferred accumulation: the micro-batch gradients are never summed into a buffer,
the norm pass and the update kernel add them in registers.  The oracle side is the plain sequence
accumulate (float32 buffer, micro-batch by micro-batch) -> clip -> update, so every case checks
that the in-register sum is the buffer's sum, bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
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


def cast(a, kind):
    if kind == "bf16":
        return O.f32_to_bf16(a)
    if kind == "f16":
        return a.astype(np.float16)
    return a.astype(F)


def lists(seed, sizes, kind, sigma):
    rng = np.random.default_rng(seed)
    out = []
    for n in sizes:
        a = rng.normal(0, sigma, n).astype(F)
        if n:
            a[rng.random(n) < 0.01] *= 100
        out.append(cast(a, kind))
    return out


def to_param_dtype(x, kind):
    return cast(x, kind)


def oracle_sum(first, pending):
    acc = [O.accumulate_fp32(None, g) if g.dtype != np.float32 else g.copy() for g in first]
    for stream in pending:
        acc = [O.accumulate_fp32(a, g) for a, g in zip(acc, stream)]
    return acc


def device_scale(ctx, res, grads, max_norm):
    """The clip factor the device derived.  Its norm must agree with the exact float64 one to rel 1e-5,
    and the factor must be exactly what the reference's float32 scalar chain (optimizers/mod.rs:87-96)
    makes of the device's own sum of squares."""
    r = ctx.read_norm_result(res)
    n, _ = O.norm_scale_c1(O.exact_sumsq(grads), max_norm)
    assert abs(r.norm - float(n)) <= 1e-5 * float(n)
    _, s = O.norm_scale_c1(r.sumsq, max_norm)
    assert F(r.scale) == s
    return F(r.scale)


# (parameter dtype, dtype of tensor.g, dtype of the pending streams)
COMBOS = [("bf16", "bf16", "bf16"), ("f32", "f32", "f32"), ("f16", "f16", "f16"), ("bf16", "f32", "bf16"),
          ("f32", "bf16", "bf16"), ("f32", "f32", "f16")]


@pytest.mark.parametrize("combo", COMBOS, ids=lambda c: "-".join(c))
@pytest.mark.parametrize("k", [0, 1, 2, 3, 5, 7])
@pytest.mark.parametrize("layout", ["aligned", "head", "elementwise"])
def test_adamw_over_deferred_micro_batches(mx, ctx, combo, k, layout):
    """layout "head": every stream becomes 16-byte aligned after one element (float32 buffers start 12
    bytes, 16-bit buffers 14 bytes past a boundary), so the vector path runs behind a peeled head;
    "elementwise": all buffers start three elements in, the 16-bit and the float32 ones then disagree
    about the head and the tensor is walked element by element."""
    pk, gk, xk = combo
    seed = 1000 + 10 * k + len(layout)
    if layout == "elementwise" and pk == gk == "f32" and xk != "f32":
        pytest.skip("float32 rows keep the vector path; 16-bit pending streams three elements in are rejected")
    off = {"aligned": {"f32": 0, "bf16": 0, "f16": 0}, "head": {"f32": 3, "bf16": 7, "f16": 7},
           "elementwise": {"f32": 3, "bf16": 3, "f16": 3}}[layout]

    kind_of = {np.dtype(np.float32): "f32", np.dtype(np.uint16): "bf16", np.dtype(np.float16): "f16"}

    def place(a):
        return to_dev(a, off[kind_of[a.dtype]])

    ps = lists(seed, SIZES, pk, 0.02)
    first = lists(seed + 1, SIZES, gk, 1e-3)
    pending = [lists(seed + 2 + j, SIZES, xk, 1e-3) for j in range(k)]
    zeros = [np.zeros(n, F) for n in SIZES]
    dp = [place(p) for p in ps]
    dg = [place(g) for g in first]
    dx = [[place(g) for g in s] for s in pending]
    dm, dv = ([place(z) for z in zeros] for _ in range(2))
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    table.set_pending(dx)
    res = ctx.norm_result()
    max_norm = 1e-2
    ctx.norm_with_pending_list(table, res, max_norm=max_norm)
    acc = oracle_sum(first, pending)
    scale = device_scale(ctx, res, acc, max_norm)
    ctx.adam_with_pending_list(table, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01), mx.make_prep(scale=res))
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    for i, n in enumerate(SIZES):
        want = to_param_dtype(ref.update_single(str(i), ps[i], acc[i] * scale), pk)
        assert_bit_equal(to_host(dp[i]), want, f"p {i} (n={n})")
        assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"m {i}")
        assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v {i}")
    # the gradient streams are inputs only
    for i in range(len(SIZES)):
        assert_bit_equal(to_host(dg[i]), first[i], f"g {i}")
        for j in range(k):
            assert_bit_equal(to_host(dx[j][i]), pending[j][i], f"x{j} {i}")
    table.close()


@pytest.mark.parametrize("which", ["sgd_first", "sgd_later", "sgd_nesterov", "rmsprop"])
@pytest.mark.parametrize("combo", [("bf16", "bf16", "bf16"), ("f32", "f32", "f32"), ("bf16", "f32", "bf16"),
                                   ("f16", "f16", "f16")], ids=lambda c: "-".join(c))
@pytest.mark.parametrize("k", [1, 3, 6])
@pytest.mark.parametrize("layout", ["aligned", "head", "elementwise"])
def test_sgd_and_rmsprop_over_deferred_micro_batches(mx, ctx, which, combo, k, layout):
    """The momentum-SGD and RMSprop kernels on g + x0 + ... with the clip factor taken from the device:
    first step (velocity = gradient), a later step (velocity read), Nesterov, RMSprop with decay."""
    pk, gk, xk = combo
    seed = 3000 + 10 * k + len(layout)
    off = {"aligned": {"f32": 0, "bf16": 0, "f16": 0}, "head": {"f32": 3, "bf16": 7, "f16": 7},
           "elementwise": {"f32": 3, "bf16": 3, "f16": 3}}[layout]
    kind_of = {np.dtype(np.float32): "f32", np.dtype(np.uint16): "bf16", np.dtype(np.float16): "f16"}

    def place(a):
        return to_dev(a, off[kind_of[a.dtype]])

    ps = lists(seed, SIZES, pk, 0.02)
    first = lists(seed + 1, SIZES, gk, 1e-3)
    pending = [lists(seed + 2 + j, SIZES, xk, 1e-3) for j in range(k)]
    v0 = [np.abs(a) for a in lists(seed + 20, SIZES, "f32", 1e-3)]   # RMSprop's average of squares is >= 0
    dp = [place(p) for p in ps]
    dg = [place(g) for g in first]
    dx = [[place(g) for g in s] for s in pending]
    dv = [place(v) for v in v0]
    if which == "rmsprop":
        ref = O.RMSprop(1e-2, 0.95, 1e-8, 1e-3)
        hp, run, flags = mx.rmsprop_hp(1e-2, 0.95, 1e-8, 1e-3), ctx.rmsprop_with_pending_list, 0
    else:
        nesterov = which == "sgd_nesterov"
        args = (0.05, 0.9, 0.0, 0.0, True) if nesterov else (0.05, 0.9, 1e-3, 0.1, False)
        ref = O.SGD(*args)
        hp, run = mx.sgd_hp(*args), ctx.sgd_with_pending_list
        flags = mx.TF_FIRST if which == "sgd_first" else 0
    if flags == 0:
        for i in range(len(SIZES)):
            ref.state[str(i)] = v0[i].copy()
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v, flags=flags) for p, g, v in zip(dp, dg, dv)])
    table.set_pending(dx)
    res = ctx.norm_result()
    ctx.norm_with_pending_list(table, res, max_norm=1e-2)
    acc = oracle_sum(first, pending)
    scale = device_scale(ctx, res, acc, 1e-2)
    run(table, hp, mx.make_prep(scale=res))
    for i, n in enumerate(SIZES):
        want = to_param_dtype(ref.update_single(str(i), ps[i], acc[i] * scale), pk)
        assert_bit_equal(to_host(dp[i]), want, f"p {i} (n={n})")
        assert_bit_equal(to_host(dv[i]), ref.state[str(i)], f"v {i}")
    for i in range(len(SIZES)):
        assert_bit_equal(to_host(dg[i]), first[i], f"g {i}")
        for j in range(k):
            assert_bit_equal(to_host(dx[j][i]), pending[j][i], f"x{j} {i}")
    table.close()


def test_first_is_sum_wants_a_float32_buffer_without_a_clip_factor(mx, ctx):
    ps, gs, xs = lists(1, [4096], "bf16", 0.02), lists(2, [4096], "bf16", 1e-3), lists(3, [4096], "bf16", 1e-3)
    dp, dg, dx = to_dev(ps[0]), to_dev(gs[0]), to_dev(xs[0])
    dsum = to_dev(O.as_f32(gs[0]))
    res = ctx.norm_result()
    t16 = ctx.table([mx.TensorSpec(p=dp, p_out=dp, g=dg)])
    t16.set_pending([[dx]])
    with pytest.raises(mx.InvalidArg, match="is float32"):
        ctx.sgd_plain_with_pending_list_each(t16, 0.1, [None, None], first_is_sum=True)
    t32 = ctx.table([mx.TensorSpec(p=dp, p_out=dp, g=dsum)])
    t32.set_pending([[dx]])
    with pytest.raises(mx.InvalidArg, match="has no clip factor"):
        ctx.sgd_plain_with_pending_list_each(t32, 0.1, [res.scale_ptr, res.scale_ptr], first_is_sum=True)
    with pytest.raises(mx.InvalidArg, match="either every micro-batch"):
        ctx.sgd_plain_with_pending_list_each(t32, 0.1, [res.scale_ptr, None])
    assert_bit_equal(to_host(dp), ps[0], "a refused call changed the parameter")
    # the sum is taken as it is: no clamp, no factor; the pending stream is clamped
    ctx.sgd_plain_with_pending_list_each(t32, 0.1, [None, None], prep=mx.make_prep(clamp_pre=(-1e-3, 1e-3)),
                                         first_is_sum=True)
    total = O.as_f32(gs[0]) + np.clip(O.as_f32(xs[0]), F(-1e-3), F(1e-3))
    want = O.apply_gradients({"p": ps[0]}, {"p": total}, 0.1)["p"]
    assert_bit_equal(to_host(dp), want, "p")
    t16.close()
    t32.close()


def test_first_momentum_step_cannot_be_conditional(mx, ctx):
    """The first SGD-with-momentum step stores the velocity every later step reads; the host cannot know
    whether a device-side conditional update ran, so that combination is refused, and accepted afterwards."""
    names, ps, gs = ["a", "b"], lists(7, [4096, 33], "f32", 0.02), lists(8, [4096, 33], "f32", 1e-3)
    dp, dg = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    res = ctx.norm_result()
    opt = mx.SGD(0.05, 0.9, ctx=ctx)
    with pytest.raises(mx.InvalidArg, match="cannot be conditional"):
        opt.update_many(names, dp, dg, outs=dp, prep=mx.make_prep(skip_if_nonfinite=res))
    for i in range(2):
        assert_bit_equal(to_host(dp[i]), ps[i], "refused call changed a parameter")
    opt.update_many(names, dp, dg, outs=dp)
    opt.update_many_accumulated(names, dp, [dg, dg], prep=mx.make_prep(skip_if_nonfinite=res), max_norm=1.0, norm_out=res)
    ref = O.SGD(0.05, 0.9)
    cur = [ref.update_single(n, p, g) for n, p, g in zip(names, ps, gs)]
    acc = oracle_sum(gs, [gs])
    scale = device_scale(ctx, res, acc, 1.0)
    for i, n in enumerate(names):
        assert_bit_equal(to_host(dp[i]), ref.update_single(n, cur[i], acc[i] * scale), n)


def test_deferred_equals_buffered_path_bit_for_bit(mx, ctx):
    """Four bf16 micro-batches: accumulate x3 + accumulate_norm_only + adam_with_pending (float32 buffer)
    against norm_with_pending_list + adam_with_pending_list (no buffer): same sum of squares (to float64
    rounding), same clip factor, same parameters and moments."""
    import torch
    sizes = [4096 * 5 + 3, 17, 4096, 250001]
    ps = lists(7, sizes, "bf16", 0.02)
    micro = [lists(8 + j, sizes, "bf16", 1e-3) for j in range(4)]
    hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
    out = []
    for deferred in (False, True):
        dp = [to_dev(p) for p in ps]
        dm = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
        dv = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
        dmicro = [[to_dev(g) for g in s] for s in micro]
        res = ctx.norm_result()
        if deferred:
            t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dmicro[0], dm, dv)])
            t.set_pending(dmicro[1:])
            ctx.norm_with_pending_list(t, res, max_norm=1.0e-2)
            ctx.adam_with_pending_list(t, hp, mx.make_prep(scale=res))
        else:
            acc = [torch.empty(n, dtype=torch.float32, device="cuda") for n in sizes]
            for j in range(4):
                t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dmicro[j], acc)])
                if j < 3:
                    ctx.accumulate(t_acc, first=(j == 0))
                else:
                    ctx.accumulate_norm_only(t_acc, res, max_norm=1.0e-2)
            t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=m, v=v)
                           for p, a, g, m, v in zip(dp, acc, dmicro[3], dm, dv)])
            ctx.adam_with_pending(t, hp, mx.make_prep(scale=res))
        r = ctx.read_norm_result(res)
        out.append((r.sumsq, r.scale, [to_host(x) for x in dp], [to_host(x) for x in dm], [to_host(x) for x in dv]))
    a, b = out
    # the two norm passes fold their per-workgroup float64 partials over different grids
    assert abs(a[0] - b[0]) <= 1e-12 * a[0] and a[1] == b[1]
    for i in range(len(sizes)):
        assert_bit_equal(b[2][i], a[2][i], f"p{i}")
        assert_bit_equal(b[3][i], a[3][i], f"m{i}")
        assert_bit_equal(b[4][i], a[4][i], f"v{i}")


@pytest.mark.parametrize("pk,xk", [("bf16", "bf16"), ("f32", "f32"), ("bf16", "f32")])
def test_sft_boundary_over_deferred_micro_batches(mx, ctx, pk, xk):
    """sft/engine.rs:293-371 with the sum formed in registers: average, clip by the norm of the averaged
    sum, clamp, add weight decay, plain SGD."""
    sizes = [5, 4096, 4097, 30011]
    n_micro = 3
    ps = lists(21, sizes, pk, 0.02)
    micro = [lists(22 + j, sizes, xk, 1e-2) for j in range(n_micro)]
    dp = [to_dev(p) for p in ps]
    dmicro = [[to_dev(g) for g in s] for s in micro]
    t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g) for p, g in zip(dp, dmicro[0])])
    t.set_pending(dmicro[1:])
    res = ctx.norm_result()
    lr, wd, max_norm, clip_value = 1e-2, 0.01, 0.5, 0.004
    pre = mx.make_prep(pre_mul=1.0 / n_micro)
    ctx.norm_with_pending_list(t, res, prep=pre, max_norm=max_norm)
    acc = oracle_sum(micro[0], micro[1:])
    avg = [a * F(1.0 / n_micro) for a in acc]
    scale = device_scale(ctx, res, avg, max_norm)
    ctx.sgd_plain_with_pending_list(t, lr, wd, mx.make_prep(pre_mul=1.0 / n_micro, scale=res,
                                                            clamp_post=(-clip_value, clip_value)))
    for i in range(len(sizes)):
        g = O.clip_value(avg[i] * scale, -clip_value, clip_value)
        p32 = O.as_f32(ps[i])
        g = g + F(wd) * p32
        lr_p = O.as_f32(cast(np.array([lr], F), pk))[0]
        want = cast(p32 - lr_p * g, pk)
        assert_bit_equal(to_host(dp[i]), want, f"p {i}")
    t.close()


def test_nonfinite_micro_batch_is_seen_and_skipped(mx, ctx):
    import torch
    sizes = [4096 * 2 + 9, 100]
    ps = lists(31, sizes, "bf16", 0.02)
    micro = [lists(32 + j, sizes, "bf16", 1e-3) for j in range(3)]
    bad = micro[2][0].copy()
    bad[4096 + 5] = 0x7F80   # +Inf as bf16 bits
    micro[2][0] = bad
    dp = [to_dev(p) for p in ps]
    dm = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
    dv = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in sizes]
    dmicro = [[to_dev(g) for g in s] for s in micro]
    t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dmicro[0], dm, dv)])
    t.set_pending(dmicro[1:])
    res = ctx.norm_result()
    ctx.norm_with_pending_list(t, res, max_norm=1.0)
    ctx.adam_with_pending_list(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01),
                               mx.make_prep(scale=res, skip_if_nonfinite=res))
    assert ctx.read_norm_result(res).nonfinite == 1
    for i in range(len(sizes)):
        assert_bit_equal(to_host(dp[i]), ps[i], f"p {i} untouched")
        assert (to_host(dm[i]) == 0).all() and (to_host(dv[i]) == 0).all()
    t.close()


def test_set_pending_rejects_what_the_kernels_cannot_walk(mx, ctx):
    import torch
    n = 5000
    p = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    g = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    m = torch.zeros(n, dtype=torch.float32, device="cuda")
    v = torch.zeros(n, dtype=torch.float32, device="cuda")
    t = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v)])
    slab = torch.zeros(n + 8, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(mx.InvalidArg, match="16-byte phase"):
        t.set_pending([[slab[1:n + 1]]])
    with pytest.raises(mx.InvalidArg, match="k must be"):
        t.set_pending([[g]] * 8)
    with pytest.raises(mx.InvalidArg, match="one tensor per table row"):
        t.set_pending([[g, g]])
    # float32 pending streams next to a bf16 first addend have no kernel
    t.set_pending([[torch.zeros(n, dtype=torch.float32, device="cuda")]])
    with pytest.raises(mx.InvalidArg, match="unsupported dtypes"):
        ctx.adam_with_pending_list(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01))
    # detaching restores the plain behaviour: the list entry point equals mxopt_adam
    t.set_pending([])
    ctx.adam_with_pending_list(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01))
    ctx.synchronize()
    t.close()


OPTIMIZERS = {
    "adamw": (lambda mx, ctx: mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True, ctx=ctx),
              lambda: O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True)),
    "sgd": (lambda mx, ctx: mx.SGD(0.05, 0.9, 1e-3, 0.1, False, ctx=ctx), lambda: O.SGD(0.05, 0.9, 1e-3, 0.1, False)),
    "sgd_nesterov": (lambda mx, ctx: mx.SGD(0.05, 0.9, 0.0, 0.0, True, ctx=ctx), lambda: O.SGD(0.05, 0.9, 0.0, 0.0, True)),
    "sgd_plain": (lambda mx, ctx: mx.SGD(0.05, ctx=ctx), lambda: O.SGD(0.05)),
    "rmsprop": (lambda mx, ctx: mx.RMSprop(1e-2, 0.95, 1e-8, 1e-3, ctx=ctx), lambda: O.RMSprop(1e-2, 0.95, 1e-8, 1e-3)),
}


@pytest.mark.parametrize("which", list(OPTIMIZERS))
@pytest.mark.parametrize("kind", ["bf16", "f32"])
def test_optimizer_object_steps_over_unsummed_micro_batches(mx, ctx, kind, which):
    """update_many_accumulated == accumulate_gradients (float32 buffer) k-1 times, clip_grad_norm,
    then update_single tensor by tensor, including the per-call step count under bias correction;
    two optimizer steps, the second with fresh buffers (table retargeted) and fewer micro-batches."""
    sizes = [3, 4096, 5000, 70001]
    names = [f"layers.{i}.w" for i in range(len(sizes))]
    ps = lists(41, sizes, kind, 0.02)
    opt, ref = OPTIMIZERS[which][0](mx, ctx), OPTIMIZERS[which][1]()
    dp = [to_dev(p) for p in ps]
    res = ctx.norm_result()
    cur = ps
    for step, k in enumerate((4, 2, 7, 11, 9)):    # more than eight: the oldest go through a float32 buffer first
        micro = [lists(50 + 10 * step + j, sizes, kind, 1e-3) for j in range(k)]
        dmicro = [[to_dev(g) for g in mb] for mb in micro]
        opt.update_many_accumulated(names, dp, dmicro, max_norm=1e-2, norm_out=res)
        acc = oracle_sum(micro[0], micro[1:])
        scale = device_scale(ctx, res, acc, 1e-2)
        nxt = []
        for i, name in enumerate(names):
            want = cast(ref.update_single(name, cur[i], acc[i] * scale), kind)
            assert_bit_equal(to_host(dp[i]), want, f"step {step} {name}")
            m, v = opt.state(name)
            if which == "adamw":
                assert_bit_equal(to_host(m), ref.state[name][0], f"m {name}")
                assert_bit_equal(to_host(v), ref.state[name][1], f"v {name}")
            elif which == "sgd_plain":
                assert m is None and v is None
            else:                              # velocity / running average of squares
                assert m is None
                assert_bit_equal(to_host(v), ref.state[name], f"v {name}")
            nxt.append(want)
        cur = nxt
        if which == "adamw":
            assert opt.step == ref.step == (step + 1) * len(names)
    # a refused call leaves the counter alone
    with pytest.raises(mx.InvalidArg, match="at least one micro-batch"):
        opt.update_many_accumulated(names, dp, [])
    opt.update_many_accumulated([], [], [[] for _ in range(10)])   # an empty list is a no-op for any k
    if which == "adamw":
        assert opt.step == 5 * len(names)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("which", ["adamw", "rmsprop"])
def test_lone_16bit_gradient_keeps_its_dtype_in_the_square(mx, ctx, kind, which):
    """One micro-batch, no clip, no stage: the gradient reaches the optimizer as it came, so its square is a
    16-bit tensor (mlx.cpp:2016-2020 through adamw.rs:92 / rmsprop.rs:80).  The deferred kernels with no
    pending stream, update_many_accumulated with one micro-batch, update_many and the table kernel all have to
    agree with update_single of the oracle on that."""
    sizes = [5, 4096, 4099, 70001]
    names = [f"w{i}" for i in range(len(sizes))]
    ps = lists(71, sizes, kind, 0.02)
    gs = [cast(g, kind) for g in lists(72, sizes, "f32", 3e-2)]   # large enough for the 16-bit rounding of g*g to show in v
    make = {"adamw": (lambda: mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, ctx=ctx), lambda: O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)),
            "rmsprop": (lambda: mx.RMSprop(1e-2, 0.95, 1e-8, 0.0, ctx=ctx), lambda: O.RMSprop(1e-2, 0.95, 1e-8, 0.0))}[which]
    ref = make[1]()
    want_p = [cast(ref.update_single(n, p, g), kind) for n, p, g in zip(names, ps, gs)]
    want_v = [ref.state[n][1] if which == "adamw" else ref.state[n] for n in names]
    # the float32 square would give another v: the case has to be able to tell the two apart
    wide = make[1]()
    for n, p, g in zip(names, ps, gs):
        wide.update_single(n, p, O.as_f32(g))
    assert any(not np.array_equal((wide.state[n][1] if which == "adamw" else wide.state[n]), w) for n, w in zip(names, want_v))

    # 1. optimizer object, one un-summed micro-batch
    opt = make[0]()
    dp = [to_dev(p) for p in ps]
    opt.update_many_accumulated(names, dp, [[to_dev(g) for g in gs]])
    for i, n in enumerate(names):
        assert_bit_equal(to_host(dp[i]), want_p[i], f"update_many_accumulated p {n}")
        assert_bit_equal(to_host(opt.state(n)[1]), want_v[i], f"update_many_accumulated v {n}")
    # 2. the same through update_many
    opt2 = make[0]()
    dp2 = [to_dev(p) for p in ps]
    opt2.update_many(names, dp2, [to_dev(g) for g in gs], outs=dp2)
    for i, n in enumerate(names):
        assert_bit_equal(to_host(dp2[i]), want_p[i], f"update_many p {n}")
        assert_bit_equal(to_host(opt2.state(n)[1]), want_v[i], f"update_many v {n}")
    # 3. the bare list kernel with no pending stream against the bare table kernel
    dp3, dg3 = [to_dev(p) for p in ps], [to_dev(g) for g in gs]
    dm3, dv3 = ([to_dev(np.zeros(n, F)) for n in sizes] for _ in range(2))
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp3, dg3, dm3, dv3)])
    table.set_pending([])
    if which == "adamw":
        ctx.adam_with_pending_list(table, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01))
    else:
        ctx.rmsprop_with_pending_list(table, mx.rmsprop_hp(1e-2, 0.95, 1e-8, 0.0))
    for i, n in enumerate(names):
        assert_bit_equal(to_host(dp3[i]), want_p[i], f"list kernel p {n}")
        assert_bit_equal(to_host(dv3[i]), want_v[i], f"list kernel v {n}")
    table.close()
