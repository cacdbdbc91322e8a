"""Property test of the update kernels: random table shapes (ragged sizes around the 8-element group
and the 4096-element chunk, empty tensors), element shifts that are common to all streams or not,
every dtype combination the kernels accept, every optimizer, every stage of the gradient
pre-processing -- always bit for bit against the oracle.  Examples are derandomised: the same cases
run every time.  MXOPT_PROPERTY_EXAMPLES=<n> in the environment turns the file into a soak: n fresh random
cases per test instead of the fixed ones."""
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
SOAK = int(os.environ.get("MXOPT_PROPERTY_EXAMPLES", "0"))


def cases(n):
    return settings(max_examples=SOAK or n, deadline=None, derandomize=not SOAK, database=None,
                    suppress_health_check=list(HealthCheck))


SIZES = st.one_of(st.integers(0, 20), st.integers(4088, 4104), st.integers(8185, 8200), st.integers(21, 30000))
DTYPES = ["f32", "bf16", "f16"]


def cast(x, dt):
    return {"f32": lambda a: a.astype(F), "bf16": O.f32_to_bf16, "f16": lambda a: a.astype(np.float16)}[dt](x)


def round_out(x, dt):
    with np.errstate(over="ignore"):
        return cast(np.asarray(x, F), dt)


def torch_dtype(torch, dt):
    return {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dt]


def prep_oracle(g, pre_mul, clamp_pre, scale, clamp_post):
    x = O.as_f32(g)
    if pre_mul is not None:
        x = x * F(pre_mul)
    if clamp_pre is not None:
        x = O.clip_value(x, -clamp_pre, clamp_pre)
    pre = x
    if scale is not None:
        x = x * F(scale)
    if clamp_post is not None:
        x = O.clip_value(x, -clamp_post, clamp_post)
    return pre, x


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


@cases(200)
@given(sizes=st.lists(SIZES, min_size=1, max_size=5), shift=st.integers(0, 9), common_shift=st.booleans(),
       kind=st.sampled_from(["adam", "adamw", "adamw_bias", "sgd", "sgd_nesterov", "sgd_no_momentum", "rmsprop"]),
       pd=st.sampled_from(DTYPES), gd=st.sampled_from(DTYPES), out_f32=st.booleans(), in_place=st.booleans(),
       pre_mul=st.sampled_from([None, 0.25]), clamp_pre=st.sampled_from([None, 1.5e-3]),
       clip=st.booleans(), clamp_post=st.sampled_from([None, 4e-4]), seed=st.integers(0, 2 ** 31))
def test_update_kernels_match_the_oracle(mx, sizes, shift, common_shift, kind, pd, gd, out_f32, in_place, pre_mul,
                                         clamp_pre, clip, clamp_post, seed):
    import torch
    rng = np.random.default_rng(seed)
    od = "f32" if out_f32 else pd
    in_place = in_place and od == pd
    ctx = mx.default_context()
    ps = [cast(rng.normal(0, 0.05, n).astype(F), pd) for n in sizes]
    state_shift = shift if common_shift else 0
    dp = [to_dev(p, shift) for p in ps]
    do = dp if in_place else [torch.empty(n + 16, dtype=torch_dtype(torch, od), device="cuda")[state_shift:state_shift + n]
                              for n in sizes]
    dm = [to_dev(np.zeros(n, F), state_shift) for n in sizes]
    dv = [to_dev(np.zeros(n, F), state_shift) for n in sizes]
    dg = [torch.empty(n + 16, dtype=torch_dtype(torch, gd), device="cuda")[shift:shift + n] for n in sizes]
    adam = kind.startswith("adam")
    if adam:
        bias = kind == "adamw_bias"
        wd = None if kind == "adam" else 0.02
        hp = mx.adam_hp(3e-3, 0.9, 0.99, 1e-8, wd)
        ref = (O.Adam(3e-3, 0.9, 0.99, 1e-8, bias) if wd is None else O.AdamW(3e-3, 0.9, 0.99, 1e-8, wd, bias))
        rows = [mx.TensorSpec(p=p, p_out=o, g=g, m=m, v=v) for p, o, g, m, v in zip(dp, do, dg, dm, dv)]
    elif kind.startswith("sgd"):
        mom = 0.0 if kind == "sgd_no_momentum" else 0.9
        nest = kind == "sgd_nesterov"
        hp = mx.sgd_hp(2e-2, mom, 1e-3, 0.0, nest)
        ref = O.SGD(2e-2, mom, 1e-3, 0.0, nest)
        rows = [mx.TensorSpec(p=p, p_out=o, g=g, v=(v if mom else None), flags=mx.TF_FIRST)
                for p, o, g, v in zip(dp, do, dg, dv)]
    else:
        hp = mx.rmsprop_hp(1e-3, 0.95, 1e-8, 0.01)
        ref = O.RMSprop(1e-3, 0.95, 1e-8, 0.01)
        rows = [mx.TensorSpec(p=p, p_out=o, g=g, v=v) for p, o, g, v in zip(dp, do, dg, dv)]
    table = ctx.table(rows)
    t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
    res = ctx.norm_result()
    cur = list(ps)
    step = 0
    for it in range(2):
        gs = [cast(rng.normal(0, 1e-3, n).astype(F), gd) for n in sizes]
        for d, g in zip(dg, gs):
            d.copy_(to_dev(g))
        scale = None
        if clip:
            pre_only = mx.make_prep(pre_mul=pre_mul, clamp_pre=(-clamp_pre, clamp_pre) if clamp_pre else None)
            ctx.global_norm(t_g, res, prep=pre_only, max_norm=5e-3)
            r = ctx.read_norm_result(res)
            exact = O.exact_sumsq([prep_oracle(g, pre_mul, clamp_pre, None, None)[0] for g in gs])
            assert abs(r.sumsq - exact) <= 1e-6 * exact + 1e-300
            assert F(r.scale) == O.norm_scale_c1(r.sumsq, 5e-3)[1]
            scale = r.scale
        prep = mx.make_prep(pre_mul=pre_mul, clamp_pre=(-clamp_pre, clamp_pre) if clamp_pre else None,
                            scale=res if clip else None, clamp_post=(-clamp_post, clamp_post) if clamp_post else None)
        if adam and kind == "adamw_bias":
            bcs = [mx.bias_correction(0.9, 0.99, step + i + 1) for i in range(len(sizes))]
            table.set_step_scalars([a for a, _ in bcs], [b for _, b in bcs])
        if kind.startswith("sgd") and it == 1:
            table.set_step_scalars(flags=[0] * len(sizes))
        step += len(sizes)
        if adam:
            ctx.adam(table, hp, prep)
        elif kind.startswith("sgd"):
            ctx.sgd(table, hp, prep)
        else:
            ctx.rmsprop(table, hp, prep)
        for i, n in enumerate(sizes):
            g_eff = prep_oracle(gs[i], pre_mul, clamp_pre, scale, clamp_post)[1]
            if pre_mul is None and clamp_pre is None and scale is None and clamp_post is None:
                g_eff = gs[i]        # untouched: a 16-bit gradient reaches the optimizer (and its square) as 16-bit
            want = round_out(ref.update_single(str(i), cur[i], g_eff), od)
            what = f"{kind} {pd}/{gd}->{od} n={n} shift={shift}/{state_shift} it={it} tensor {i}"
            assert_bit_equal(to_host(do[i]), want, what)
            if in_place:
                cur[i] = want
        ctx.synchronize()
    table.close()
    t_g.close()


@cases(150)
@given(sizes=st.lists(SIZES, min_size=1, max_size=5), shift=st.integers(0, 9), gd=st.sampled_from(DTYPES),
       acc_f32=st.booleans(), pre_mul=st.sampled_from([None, 0.5]), clamp=st.sampled_from([None, 1.2e-3]),
       poison=st.sampled_from([None, "nan", "inf", "-inf"]), seed=st.integers(0, 2 ** 31))
def test_accumulation_and_transform_kernels_match_the_oracle(mx, sizes, shift, gd, acc_f32, pre_mul, clamp, poison, seed):
    """acc = g0; acc += g1 with the norm of the new sum fused; the same sum measured without being
    written (norm-only); acc2 = T(g0) + T(g1) with T = clamp and clip; g_out = T(g).  A NaN/Inf element
    must raise the flag, also when the clamp would hide it, and then nothing may be written."""
    import torch
    rng = np.random.default_rng(seed)
    ad = "f32" if acc_f32 else gd
    ctx = mx.default_context()
    g0 = [cast(rng.normal(0, 1e-3, n).astype(F), gd) for n in sizes]
    g1 = [cast(rng.normal(0, 1e-3, n).astype(F), gd) for n in sizes]
    total = sum(sizes)
    if poison and total:
        i = int(np.argmax(sizes))
        v = O.as_f32(g1[i]).copy()
        v[sizes[i] // 2] = {"nan": np.nan, "inf": np.inf, "-inf": -np.inf}[poison]
        g1[i] = cast(v, gd)
    dg = [torch.empty(n + 16, dtype=torch_dtype(torch, gd), device="cuda")[shift:shift + n] for n in sizes]
    da = [torch.full((n + 16,), float("nan"), dtype=torch_dtype(torch, ad), device="cuda")[shift:shift + n] for n in sizes]
    t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, da)])
    res = ctx.norm_result()
    pre = mx.make_prep(pre_mul=pre_mul, clamp_pre=(-clamp, clamp) if clamp else None)

    def load(gs):
        for d, g in zip(dg, gs):
            d.copy_(to_dev(g))

    def add(a, b):          # promote(acc, g): equal 16-bit dtypes round the sum to that dtype
        s = O.as_f32(a) + O.as_f32(b)
        return round_out(s, ad)

    load(g0)
    ctx.accumulate(t_acc, first=True)
    acc0 = [round_out(O.as_f32(g), ad) for g in g0]
    for i in range(len(sizes)):
        assert_bit_equal(to_host(da[i]), acc0[i], f"first {i}")
    load(g1)
    ctx.accumulate_norm_only(t_acc, res, prep=pre, max_norm=2e-3)
    r_only = ctx.read_norm_result(res)
    for i in range(len(sizes)):
        assert_bit_equal(to_host(da[i]), acc0[i], f"norm-only wrote {i}")
    ctx.accumulate(t_acc, first=False, out=res, prep=pre, max_norm=2e-3)
    r = ctx.read_norm_result(res)
    acc1 = [add(a, g) for a, g in zip(acc0, g1)]
    for i in range(len(sizes)):
        assert_bit_equal(to_host(da[i]), acc1[i], f"sum {i}")
    bad = poison is not None and total > 0
    assert r.nonfinite == int(bad) and r_only.nonfinite == int(bad)
    if not bad:
        exact = O.exact_sumsq([prep_oracle(a, pre_mul, clamp, None, None)[0] for a in acc1])
        assert abs(r.sumsq - exact) <= 1e-6 * exact + 1e-300 and r.sumsq == r_only.sumsq
        assert F(r.scale) == O.norm_scale_c1(r.sumsq, 2e-3)[1]

    # clip-then-accumulate (float32 buffer) and the plain transform, with the skip flag wired in
    db = [torch.full((n + 16,), 7.0, dtype=torch.float32, device="cuda")[shift:shift + n] for n in sizes]
    dt = [torch.full((n + 16,), 7.0, dtype=torch.float32, device="cuda")[shift:shift + n] for n in sizes]
    t_b = ctx.table([mx.TensorSpec(g=g, g_out=b) for g, b in zip(dg, db)])
    t_t = ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(dg, dt)])
    t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
    want_b = None
    for k, gs in enumerate((g0, g1)):
        load(gs)
        ctx.global_norm(t_g, res, prep=pre, max_norm=1e-3)
        rk = ctx.read_norm_result(res)
        full = mx.make_prep(pre_mul=pre_mul, clamp_pre=(-clamp, clamp) if clamp else None, scale=res,
                            skip_if_nonfinite=res)
        ctx.accumulate_transformed(t_b, first=(k == 0), prep=full)
        ctx.grad_transform(t_t, full)
        if k == 1 and bad:
            assert rk.nonfinite == 1
            for i in range(len(sizes)):     # skipped: still what the first micro-batch left
                assert_bit_equal(to_host(db[i]), want_b[i], f"skipped accumulate {i}")
                assert_bit_equal(to_host(dt[i]), want_t[i], f"skipped transform {i}")
            break
        tg = [prep_oracle(g, pre_mul, clamp, rk.scale, None)[1] for g in gs]
        want_b = tg if k == 0 else [a + b for a, b in zip(want_b, tg)]
        want_t = tg
        for i in range(len(sizes)):
            assert_bit_equal(to_host(db[i]), want_b[i], f"transformed accumulate {k} {i}")
            assert_bit_equal(to_host(dt[i]), want_t[i], f"transform {k} {i}")
    for t in (t_acc, t_b, t_t, t_g):
        t.close()


@cases(120)
@given(sizes=st.lists(SIZES, min_size=1, max_size=4), bf16=st.booleans(), max_norm=st.sampled_from([1e-3, 3e-2, 10.0]),
       clip_val=st.sampled_from([2e-4, 1.0]), lr=st.sampled_from([1e-6, 2e-5, 0.3]), seed=st.integers(0, 2 ** 31))
def test_host_layer_utilities_match_the_oracle(mx, sizes, bf16, max_norm, clip_val, lr, seed):
    """GradientUtils, the Vec clip API, accumulate_gradients and apply_gradients over name-keyed maps of
    random shape, against the oracle (clip outputs given the device's norm, everything else bit for bit)."""
    rng = np.random.default_rng(seed)
    dt = "bf16" if bf16 else "f32"
    names = [f"t{i}" for i in range(len(sizes))]
    gs = {k: cast(rng.normal(0, 1e-3, n).astype(F), dt) for k, n in zip(names, sizes)}
    ps = {k: cast(rng.normal(0, 0.5, n).astype(F), dt) for k, n in zip(names, sizes)}
    dg = {k: to_dev(v) for k, v in gs.items()}
    exact = O.GradientUtils.compute_gradient_norm(gs)
    got = mx.GradientUtils.compute_gradient_norm(dg)
    assert abs(got - exact) <= 1e-5 * exact + 1e-30
    # clip by norm (always multiplies) and the Vec API (unchanged when below)
    clipped, n32 = mx.GradientUtils.clip_grad_norm_with_norm(dg, max_norm)
    assert abs(n32 - exact) <= 1e-5 * exact + 1e-30
    _, scale = O.norm_scale_c1(float(n32) ** 2, max_norm)
    for k in names:
        want = O.as_f32(gs[k]) * scale
        assert np.allclose(to_host(clipped[k]), want, rtol=3e-7, atol=0), k
    vec = mx.clip_gradients_by_global_norm([dg[k] for k in names], max_norm)
    want_vec = O.clip_gradients_by_global_norm([gs[k] for k in names], max_norm)
    for k, g, w in zip(names, vec, want_vec):
        assert np.allclose(O.as_f32(to_host(g)), O.as_f32(w), rtol=3e-7, atol=0), k
    # clamp: bit for bit, NaN kept
    for k in names[:2]:
        assert_bit_equal(to_host(mx.GradientUtils.clip_grad_value(dg[k], -clip_val, clip_val)),
                         O.clip_value(gs[k], -clip_val, clip_val), f"clamp {k}")
    # accumulate three times through the map API, with a name that appears late and one that stops
    acc_d, acc_o = {}, {}
    for it in range(3):
        keep = names if it != 1 else names[:-1] or names
        new_o = {k: cast(rng.normal(0, 1e-3, sizes[names.index(k)]).astype(F), dt) for k in keep}
        acc_d = mx.accumulate_gradients(acc_d, {k: to_dev(v) for k, v in new_o.items()})
        acc_o = O.accumulate_gradients(acc_o, new_o)
    assert set(acc_d) == set(acc_o)
    for k in acc_o:
        assert_bit_equal(to_host(acc_d[k]), acc_o[k], f"accumulated {k}")
    # apply: plain SGD in the parameter's dtype, in place
    dp = {k: to_dev(v) for k, v in ps.items()}
    mx.apply_gradients(dp, acc_d, lr)
    want_p = O.apply_gradients(ps, acc_o, lr)
    for k in names:
        assert_bit_equal(to_host(dp[k]), want_p[k], f"applied {k}")


@cases(150)
@given(sizes=st.lists(SIZES, min_size=1, max_size=4), k=st.integers(0, 7), head=st.sampled_from([0, 1, 2, 3, "mixed"]),
       pd=st.sampled_from(DTYPES), xd=st.sampled_from(DTYPES), first_f32=st.booleans(),
       kind=st.sampled_from(["adamw", "sgd_plain", "sgd_plain_each"]), pre_mul=st.sampled_from([None, 0.5]),
       clamp_pre=st.sampled_from([None, 1.5e-3]), clip=st.booleans(), clamp_post=st.sampled_from([None, 4e-4]),
       poison=st.sampled_from([None, "nan", "inf"]), seed=st.integers(0, 2 ** 31))
def test_deferred_accumulation_kernels_match_the_oracle(mx, sizes, k, head, pd, xd, first_f32, kind, pre_mul, clamp_pre,
                                                        clip, clamp_post, poison, seed):
    """g + x0 + ... summed in registers.  "adamw" / "sgd_plain": prep(sum) with the clip factor of the
    sum's norm; "sgd_plain_each": every stream clamped and clipped by its own norm before the add (the
    GRPO order).  The oracle accumulates into a float32 buffer, micro-batch by micro-batch.  head = h:
    every buffer becomes 16-byte aligned after h elements (vector path behind a peeled head); "mixed":
    every buffer starts one element in, so 16-bit and float32 streams disagree (element-wise path)."""
    import torch
    rng = np.random.default_rng(seed)
    ctx = mx.default_context()
    gd = "f32" if first_f32 else xd
    if head == "mixed":
        shift = {"f32": 1, "bf16": 1, "f16": 1}
    else:
        shift = {"f32": (4 - head) % 4, "bf16": (8 - head) % 8, "f16": (8 - head) % 8}
    ps = [cast(rng.normal(0, 0.05, n).astype(F), pd) for n in sizes]
    streams = [[cast(rng.normal(0, 1e-3, n).astype(F), gd if j == 0 else xd) for n in sizes] for j in range(k + 1)]
    if poison and sum(sizes):
        j = int(rng.integers(0, k + 1))
        i = int(rng.choice([t for t, n in enumerate(sizes) if n]))
        a = O.as_f32(streams[j][i]).copy()
        a[int(rng.integers(0, sizes[i]))] = np.nan if poison == "nan" else np.inf
        with np.errstate(over="ignore"):
            streams[j][i] = cast(a, gd if j == 0 else xd)
    dp = [to_dev(p, shift[pd]) for p in ps]
    dstreams = [[to_dev(g, shift[gd if j == 0 else xd]) for g in s] for j, s in enumerate(streams)]
    dm = [to_dev(np.zeros(n, F), shift["f32"]) for n in sizes]
    dv = [to_dev(np.zeros(n, F), shift["f32"]) for n in sizes]
    adam = kind == "adamw"
    rows = [mx.TensorSpec(p=p, p_out=p, g=g, m=m if adam else None, v=v if adam else None)
            for p, g, m, v in zip(dp, dstreams[0], dm, dv)]
    table = ctx.table(rows)
    if head == "mixed" and pd == gd == "f32" and xd != "f32" and k and sum(sizes):
        # the row's own buffers agree (all float32, head 3), a 16-bit pending stream one element in does not
        with pytest.raises(mx.InvalidArg, match="16-byte phase"):
            table.set_pending(dstreams[1:])
        table.close()
        return
    table.set_pending(dstreams[1:])
    max_norm = 1e-2
    lr, wd = 0.05, 0.01

    if kind == "sgd_plain_each":
        # one norm per stream, of the clamped values (grpo/engine.rs:636-653)
        # an even seed with a float32 first stream: that stream is a sum of earlier, already prepared
        # micro-batches and is added untouched
        first_is_sum = gd == "f32" and seed % 2 == 0
        results, scales, bad = [], [], False
        for j in range(k + 1):
            res = ctx.norm_result()
            tj = ctx.table([mx.TensorSpec(g=g) for g in dstreams[j]])
            ctx.global_norm(tj, res, prep=mx.make_prep(clamp_pre=(-clamp_pre, clamp_pre)) if clamp_pre else None,
                            max_norm=max_norm)
            r = ctx.read_norm_result(res)
            bad = bad or bool(r.nonfinite)
            results.append(res)
            scales.append(F(r.scale))
            tj.close()
        if bad:
            table.close()
            return          # the engine drops such a micro-batch before anything is added
        prep = mx.make_prep(clamp_pre=(-clamp_pre, clamp_pre) if clamp_pre else None)
        ptrs = [r.scale_ptr for r in results] if clip else [None] * (k + 1)
        if first_is_sum:
            ptrs[0] = None
        ctx.sgd_plain_with_pending_list_each(table, lr, ptrs, prep=prep, first_is_sum=first_is_sum)
        want_g = []
        for i in range(len(sizes)):
            total = None
            for j in range(k + 1):
                if j == 0 and first_is_sum:
                    t = O.as_f32(streams[0][i])
                else:
                    t = prep_oracle(streams[j][i], None, clamp_pre, scales[j] if clip else None, None)[1]
                total = t if total is None else total + t
            want_g.append(total)
    else:
        res = ctx.norm_result()
        pre = mx.make_prep(pre_mul=pre_mul, clamp_pre=(-clamp_pre, clamp_pre) if clamp_pre else None)
        if clip:
            ctx.norm_with_pending_list(table, res, prep=pre, max_norm=max_norm)
        r = ctx.read_norm_result(res)
        acc = [O.accumulate_fp32(None, g) for g in streams[0]]
        for s in streams[1:]:
            acc = [O.accumulate_fp32(a, g) for a, g in zip(acc, s)]
        if clip:
            with np.errstate(invalid="ignore", over="ignore"):
                pre_vals = [prep_oracle(a, pre_mul, clamp_pre, None, None)[0] for a in acc]
                finite = all(np.isfinite(a).all() for a in acc)
            assert bool(r.nonfinite) == (not finite)
            if not finite:
                table.close()
                return      # the caller skips the step; what a NaN clip factor does to p is not specified
            exact = O.exact_sumsq(pre_vals)
            assert abs(r.sumsq - exact) <= 1e-5 * max(exact, 1e-300)
        scale = F(r.scale) if clip else None
        prep = mx.make_prep(pre_mul=pre_mul, clamp_pre=(-clamp_pre, clamp_pre) if clamp_pre else None,
                            scale=res if clip else None, clamp_post=(-clamp_post, clamp_post) if clamp_post else None)
        if adam:
            ctx.adam_with_pending_list(table, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.02), prep)
        else:
            ctx.sgd_plain_with_pending_list(table, lr, wd, prep)
        with np.errstate(invalid="ignore", over="ignore"):
            want_g = [prep_oracle(a, pre_mul, clamp_pre, scale, clamp_post)[1] for a in acc]
        if adam and k == 0 and not (pre_mul or clamp_pre or clip or clamp_post):
            # a lone gradient with nothing in front of the optimizer reaches it in its own dtype: the square
            # of a 16-bit tensor is a 16-bit tensor (mlx.cpp:2016-2020 through adamw.rs:92)
            want_g = list(streams[0])

    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.02)
    for i, n in enumerate(sizes):
        p32 = O.as_f32(ps[i])
        with np.errstate(invalid="ignore", over="ignore"):
            if adam:
                want = ref.update_single(str(i), ps[i], want_g[i])
            else:
                g = want_g[i] + (F(wd) * p32 if kind == "sgd_plain" else 0)
                lr_eff = lr
                lr_p = O.as_f32(cast(np.array([lr_eff], F), pd))[0]
                want = p32 - lr_p * g
            assert_bit_equal(to_host(dp[i]), round_out(want, pd), f"p {i} (n={n})")
        if adam:
            assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"m {i}")
            assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v {i}")
    table.close()
