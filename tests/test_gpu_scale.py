"""Parity at the full sizes of the benchmark configurations.

* Qwen3-0.6B list, float32 AdamW (config 1): EVERY element of parameters and moments, two steps,
  bit for bit against the C twin of the oracle -- once with the reference's default (no bias
  correction) through the kernel-level table, once bias-corrected through the optimizer object, where
  tensor i of step s must see t = s*N + i + 1 (the reference counts update_single calls).
* Qwen3-1.7B list, bf16 parameters and gradients with 1 % x100 outliers, clip 1.0 (config 2): EVERY
  element, two steps; the inputs are generated on the device by the library's counter-based generator
  and regenerated on the host by the oracle's twin of it, the norm is checked against the exact
  float64 sum.
* Qwen3-4B list, float32 SGD with momentum / RMSprop (config 3): every tensor of at most 1 Mi elements in
  full plus seeded windows (head, tail, interior) of every larger one, bit for bit; with generated inputs,
  EVERY element of every third tensor (1.5 G elements) over two steps of each optimizer.
* 10,000 small bf16 tensors (config 4): EVERY element, three steps, packed back to back so that most
  tensors start at an address that is only 2-byte aligned, and separately allocated.
* Qwen3-8B list, bf16 parameters / float32 moments, 4 micro-batches into a float32 buffer, clip 1.0,
  last micro-batch folded into the update (config 5, ~131 GB resident): seeded windows of every stream
  are read back before and after the step and pushed through the NumPy oracle (bit-exact given the
  device's clip factor); norm as above.  With generated inputs, EVERY element of every sixth tensor
  (1.5 G elements, the embedding among them) of parameters, moments and accumulation buffer against
  the C twin of the oracle.
* The same configuration without its accumulation buffer (deferred accumulation: the four resident
  micro-batches are summed in registers): the same sum of squares and a position-weighted checksum of
  EVERY parameter and moment bit equal to those of the buffered run from identical generated inputs.
"""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
import oracle_c_binding as B
from gpu_util import assert_within_ulps, to_host

F = np.float32


def f32(x):
    return float(np.float32(x))


def carve(torch, sizes, dtype, align=256):
    offs, total = [], 0
    for n in sizes:
        offs.append(total)
        total += (n + align - 1) // align * align
    slab = torch.empty(total, dtype=dtype, device="cuda")
    return slab, offs, [slab[o:o + n] for o, n in zip(offs, sizes)]


def qwen_sizes(model):
    from mxopt.qwen3_shapes import QWEN3, numel, param_list
    plist = param_list(QWEN3[model])
    return [name for name, _ in plist], [numel(s) for _, s in plist]


def window_index(torch, sizes, offs, seed, small=1 << 20, W=16384, interior=3):
    """Flat slab indices: all of every tensor <= `small` elements; head, tail and `interior` seeded
    windows (odd starts, so not group aligned) of every larger one."""
    rng = np.random.default_rng(seed)
    pieces = []
    for o, n in zip(offs, sizes):
        if n <= small:
            pieces.append(np.arange(o, o + n))
            continue
        pieces.append(np.arange(o, o + W))
        pieces.append(np.arange(o + n - W, o + n))
        for s in rng.integers(0, n - W, interior):
            s = int(s) // 8 * 8 + 3
            pieces.append(np.arange(o + s, min(o + s + W, o + n)))
    return torch.from_numpy(np.concatenate(pieces)).cuda()


def device_sumsq_f64(torch, tensors):
    return sum(float(t.double().square().sum()) for t in tensors)


def check_norm(r, ref_sumsq, max_norm=1.0):
    """rel 1e-5 on the norm; the clip factor is the reference's scalar chain applied to the device's sum."""
    assert abs(r.norm - math.sqrt(ref_sumsq)) <= 1e-5 * math.sqrt(ref_sumsq)
    n32, scale = O.norm_scale_c1(r.sumsq, max_norm)
    assert F(r.scale) == scale and F(r.norm_f32) == n32 and r.nonfinite == 0
    return float(scale)


def same_bits(got, want, what):
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, what
    v = np.uint32 if got.dtype == np.float32 else np.uint16
    bad = got.view(v) != want.view(v)
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} differ, first at {int(np.flatnonzero(bad)[0])}"


# ---------------------------------------------------------------------------------------
# config 1
# ---------------------------------------------------------------------------------------

def test_config1_full_list_every_element(oracle_c):
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("0.6B")
    n = sum(sizes)
    assert n == 596_049_920 and len(sizes) == 310
    gen = torch.Generator().manual_seed(0x5EED0001)
    p_h = torch.empty(n).normal_(0, 0.02, generator=gen)
    offs = np.concatenate([[0], np.cumsum(sizes)])
    dp = [p_h[offs[i]:offs[i + 1]].cuda() for i in range(len(sizes))]
    dg = [torch.empty(s, device="cuda") for s in sizes]
    dm = [torch.zeros(s, device="cuda") for s in sizes]
    dv = [torch.zeros(s, device="cuda") for s in sizes]
    ctx = mx.Context()
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
    args = B.adam_args(1e-3, 0.9, 0.999, 1e-8, 0.01)
    p_ref = p_h.numpy()
    m_ref, v_ref = np.zeros(n, F), np.zeros(n, F)
    for step in range(2):
        g_h = torch.empty(n).normal_(0, 1e-3, generator=gen)       # fresh seeded gradients each step
        for i, g in enumerate(dg):
            g.copy_(g_h[offs[i]:offs[i + 1]])
        ctx.adam(table, hp)
        p_ref = oracle_c.adam(p_ref, g_h.numpy(), m_ref, v_ref, args, fused=True)
        for name, dev, ref in (("p", dp, p_ref), ("m", dm, m_ref), ("v", dv, v_ref)):
            got = torch.cat(dev).cpu().numpy()
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), f"{name} differs at step {step}"
    table.close()
    ctx.close()


def test_config1_bias_corrected_per_call_step_count(oracle_c):
    import torch
    import mxopt as mx
    names, sizes = qwen_sizes("0.6B")
    n, nt = sum(sizes), len(sizes)
    gen = torch.Generator().manual_seed(0x5EED0011)
    p_ref = torch.empty(n).normal_(0, 0.02, generator=gen).numpy()
    offs = np.concatenate([[0], np.cumsum(sizes)])
    dp = [torch.from_numpy(p_ref[offs[i]:offs[i + 1]]).cuda() for i in range(nt)]
    dg = [torch.empty(s, device="cuda") for s in sizes]
    ctx = mx.Context()
    opt = mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True, ctx=ctx)
    m_ref, v_ref = np.zeros(n, F), np.zeros(n, F)
    for step in range(2):
        g_h = torch.empty(n).normal_(0, 1e-3, generator=gen)
        for i, g in enumerate(dg):
            g.copy_(g_h[offs[i]:offs[i + 1]])
        opt.update_many(names, dp, dg, outs=dp)                      # in place, one launch
        g_np = g_h.numpy()
        new_p = np.empty(n, F)
        for i in range(nt):
            t = float(step * nt + i + 1)                             # adam.rs:73: one count per call
            a = B.adam_args(1e-3, 0.9, 0.999, 1e-8, 0.01, bc1=1.0 / (1.0 - math.pow(0.9, t)),
                            bc2=1.0 / (1.0 - math.pow(0.999, t)), bias_correction=True)
            s = slice(offs[i], offs[i + 1])
            new_p[s] = oracle_c.adam(p_ref[s], g_np[s], m_ref[s], v_ref[s], a, fused=True)
        p_ref = new_p
        assert opt.step == (step + 1) * nt
        same_bits(torch.cat(dp).cpu().numpy(), p_ref, f"p step {step}")
    for i in (0, 1, 5, nt // 2, nt - 1):                              # moments live inside the object
        m, v = opt.state(names[i])
        same_bits(m.cpu().numpy(), m_ref[offs[i]:offs[i + 1]], f"m {names[i]}")
        same_bits(v.cpu().numpy(), v_ref[offs[i]:offs[i + 1]], f"v {names[i]}")
    del opt
    ctx.close()


# ---------------------------------------------------------------------------------------
# config 2
# ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("tails", ["bell", "gaussian"])
def test_config2_full_size_every_element(oracle_c, tails):
    """Inputs come from the library's counter-based generator on the device and are regenerated on the
    host by the oracle's twin of it: nothing is copied to the device, every one of 1.72 G elements of
    p, m and v is compared after each step.  One step with the four-uniform bell (|x| <= 3.46 sigma), two
    with the Gaussian mode, whose tails reach 6 sigma before the x100 outliers multiply them."""
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("1.7B")
    n, nt = sum(sizes), len(sizes)
    assert n == 1_720_574_976 and nt == 310
    bf = torch.bfloat16
    offs = np.concatenate([[0], np.cumsum(sizes)])
    dp = [torch.empty(s, dtype=bf, device="cuda") for s in sizes]
    dg = [torch.empty(s, dtype=bf, device="cuda") for s in sizes]
    dm = [torch.zeros(s, device="cuda") for s in sizes]
    dv = [torch.zeros(s, device="cuda") for s in sizes]
    ctx = mx.Context()
    SEED, CFG = 0x5EED0001, 2
    PLAIN, SPIKED = ((O.SYNTH_NORMAL, O.SYNTH_NORMAL_OUTLIERS) if tails == "bell"
                     else (O.SYNTH_GAUSSIAN, O.SYNTH_GAUSSIAN_OUTLIERS))
    p_ref = np.empty(n, np.uint16)
    for i in range(nt):
        key = mx.synthetic_key(SEED, CFG, 0, 0, i)
        ctx.fill_synthetic(dp[i], key, PLAIN, 0.02)
        p_ref[offs[i]:offs[i + 1]] = oracle_c.fill_synthetic(sizes[i], "bf16", key, PLAIN, 0.02)
    t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
    res = ctx.norm_result()
    m_ref, v_ref = np.zeros(n, F), np.zeros(n, F)
    g_ref = np.empty(n, np.uint16)
    # a second host trajectory that never sees a device value: the oracle with its OWN clip factor, from the
    # exact float64 sum (optimizers/mod.rs:87-102 -> adamw.rs:84-116)
    own_p, own_m, own_v = p_ref.copy(), np.zeros(n, F), np.zeros(n, F)
    for step in range(2 if tails == "gaussian" else 1):
        for i in range(nt):                     # fresh gradients each step: 1 % of the elements x100
            key = mx.synthetic_key(SEED, CFG, step + 1, 1, i)
            ctx.fill_synthetic(dg[i], key, SPIKED, 1e-3, 100.0)
            g_ref[offs[i]:offs[i + 1]] = oracle_c.fill_synthetic(sizes[i], "bf16", key, SPIKED, 1e-3, 100.0)
        top = float(O.bf16_to_f32(g_ref[:50_000_000]).__abs__().max())
        assert (top > 0.45) if tails == "gaussian" else (top <= 0.347)     # 100 x 4.5 sigma and more, or capped at 100 x 3.46 sigma
        ctx.global_norm(t_g, res, max_norm=1.0)
        ctx.adam(t_upd, hp, mx.make_prep(scale=res))
        r = ctx.read_norm_result(res)
        scale = check_norm(r, oracle_c.sumsq(g_ref))                       # exact float64 sum on the host
        expected = 1e-3 * math.sqrt(n * (0.99 + 0.01 * 1e4))               # ~417: the clip is active
        assert abs(r.norm - expected) < 0.02 * expected and scale < 0.01
        args = B.adam_args(5e-6, 0.9, 0.999, 1e-8, 0.01, scale=scale)
        p_ref = oracle_c.f32_to_bf16(oracle_c.adam(p_ref, g_ref, m_ref, v_ref, args, fused=True))
        same_bits(to_host(torch.cat(dp)), p_ref, f"p step {step}")
        same_bits(torch.cat(dm).cpu().numpy(), m_ref, f"m step {step}")
        same_bits(torch.cat(dv).cpu().numpy(), v_ref, f"v step {step}")
        # end to end, stated tolerance: 2 float32 ulp (rel 1e-6) on the moments, 1 bf16 ulp on the parameters
        _, own_scale = O.norm_scale_c1(oracle_c.sumsq(g_ref), 1.0)
        own_args = B.adam_args(5e-6, 0.9, 0.999, 1e-8, 0.01, scale=float(own_scale))
        own_p = oracle_c.f32_to_bf16(oracle_c.adam(own_p, g_ref, own_m, own_v, own_args, fused=True))
        assert_within_ulps(torch.cat(dm).cpu().numpy(), own_m, 2, 1e-6, f"m step {step}, oracle's own clip factor")
        assert_within_ulps(torch.cat(dv).cpu().numpy(), own_v, 2, 1e-6, f"v step {step}, oracle's own clip factor")
        assert_within_ulps(to_host(torch.cat(dp)), own_p, 1, what=f"p step {step}, oracle's own clip factor")
    t_g.close()
    t_upd.close()
    ctx.close()


# ---------------------------------------------------------------------------------------
# config 3
# ---------------------------------------------------------------------------------------

def test_config3_full_size_sgd_and_rmsprop_windows(oracle_c):
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("4B")
    n = sum(sizes)
    assert n == 4_022_468_096 and len(sizes) == 398
    torch.manual_seed(0x5EED0003)
    p_slab, offs, dp = carve(torch, sizes, torch.float32)
    g_slab, _, dg = carve(torch, sizes, torch.float32)
    v_slab, _, dv = carve(torch, sizes, torch.float32)
    p_slab.normal_(0, 0.02)
    idx = window_index(torch, sizes, offs, seed=3)
    win = lambda slab: to_host(slab[idx])
    ctx = mx.Context()

    # SGD, momentum 0.9, dampening 0, weight decay 1e-4: step 1 takes the velocity-less branch
    v_slab.fill_(float("nan"))                                        # must not be read on the first step
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v, flags=mx.TF_FIRST) for p, g, v in zip(dp, dg, dv)])
    hp = mx.sgd_hp(1e-4, 0.9, 1e-4, 0.0, False)
    p_ref, v_ref = win(p_slab), np.zeros(idx.numel(), F)
    for step in range(3):
        g_slab.normal_(0, 1e-3)
        if step == 1:
            table.set_step_scalars(flags=[0] * len(sizes))
        ctx.sgd(table, hp)
        args = B.SgdArgs(lr=f32(1e-4), momentum=f32(0.9), one_minus_damp=f32(1.0), wd=f32(1e-4), has_wd=1,
                         has_momentum=1, nesterov=0, first=int(step == 0))
        p_ref = oracle_c.sgd(p_ref, win(g_slab), v_ref, args, fused=True)
        same_bits(win(p_slab), p_ref, f"sgd p step {step}")
        same_bits(win(v_slab), v_ref, f"sgd v step {step}")
    table.close()

    # RMSprop, alpha 0.99, eps 1e-8, lr 1e-4
    v_slab.zero_()
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v) for p, g, v in zip(dp, dg, dv)])
    hp = mx.rmsprop_hp(1e-4, 0.99, 1e-8, 0.0)
    p_ref, v_ref = win(p_slab), np.zeros(idx.numel(), F)
    for step in range(2):
        g_slab.normal_(0, 1e-3)
        ctx.rmsprop(table, hp)
        args = B.RmspropArgs(lr=f32(1e-4), alpha=f32(0.99), one_minus_alpha=f32(1.0 - 0.99), eps=f32(1e-8),
                             wd=0.0, has_wd=0)
        p_ref = oracle_c.rmsprop(p_ref, win(g_slab), v_ref, args, fused=True)
        same_bits(win(p_slab), p_ref, f"rmsprop p step {step}")
        same_bits(win(v_slab), v_ref, f"rmsprop v step {step}")
    table.close()
    ctx.close()


def test_config3_every_element_of_every_third_tensor(oracle_c):
    """SGD with momentum and RMSprop on the whole 4B list from generated inputs, two steps each (the
    first SGD step takes the velocity-less branch); every element of every third tensor -- 1.5 G
    elements, the embedding among them -- is recomputed on the host by the C twin from regenerated
    inputs."""
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("4B")
    nt = len(sizes)
    torch.cuda.empty_cache()
    dp = [torch.empty(s, device="cuda") for s in sizes]
    dg = [torch.empty(s, device="cuda") for s in sizes]
    dv = [torch.empty(s, device="cuda") for s in sizes]
    ctx = mx.Context()
    SEED, CFG = 0x5EED0001, 3
    picked = list(range(0, nt, 3))

    def key(stream, step, i):
        return mx.synthetic_key(SEED, CFG, step, stream, i)

    def fill(tensors, stream, step, std):
        for i, t in enumerate(tensors):
            ctx.fill_synthetic(t, key(stream, step, i), mx.SYNTH_NORMAL, std)

    def host(i, stream, step, std):
        return oracle_c.fill_synthetic(sizes[i], "f32", key(stream, step, i), O.SYNTH_NORMAL, std)

    for opt in ("sgd", "rmsprop"):
        fill(dp, 0, 0, 0.02)
        p_ref = {i: host(i, 0, 0, 0.02) for i in picked}
        v_ref = {i: np.zeros(sizes[i], F) for i in picked}
        if opt == "sgd":
            for v in dv:
                v.fill_(float("nan"))                      # must not be read on the first step
            table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v, flags=mx.TF_FIRST) for p, g, v in zip(dp, dg, dv)])
            hp = mx.sgd_hp(1e-4, 0.9, 1e-4, 0.0, False)
        else:
            for v in dv:
                v.zero_()
            table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v) for p, g, v in zip(dp, dg, dv)])
            hp = mx.rmsprop_hp(1e-4, 0.99, 1e-8, 0.0)
        for step in range(2):
            stream = 1 if opt == "sgd" else 2
            fill(dg, stream, step + 1, 1e-3)
            if opt == "sgd":
                if step == 1:
                    table.set_step_scalars(flags=[0] * nt)
                ctx.sgd(table, hp)
                args = B.SgdArgs(lr=f32(1e-4), momentum=f32(0.9), one_minus_damp=f32(1.0), wd=f32(1e-4), has_wd=1,
                                 has_momentum=1, nesterov=0, first=int(step == 0))
            else:
                ctx.rmsprop(table, hp)
                args = B.RmspropArgs(lr=f32(1e-4), alpha=f32(0.99), one_minus_alpha=f32(1.0 - 0.99), eps=f32(1e-8),
                                     wd=0.0, has_wd=0)
            for i in picked:
                g = host(i, stream, step + 1, 1e-3)
                fn = oracle_c.sgd if opt == "sgd" else oracle_c.rmsprop
                p_ref[i] = fn(p_ref[i], g, v_ref[i], args, fused=True)
                same_bits(dp[i].cpu().numpy(), p_ref[i], f"{opt} p of tensor {i}, step {step}")
                same_bits(dv[i].cpu().numpy(), v_ref[i], f"{opt} v of tensor {i}, step {step}")
        table.close()
    assert sum(sizes[i] for i in picked) > 1_300_000_000
    ctx.close()


# ---------------------------------------------------------------------------------------
# config 4
# ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("alloc", ["packed", "separate"])
def test_config4_ten_thousand_small_tensors_every_element(oracle_c, alloc):
    import torch
    import mxopt as mx
    rng = np.random.default_rng(0x5EED0001)
    sizes = np.floor(np.exp(rng.uniform(np.log(64), np.log(65536), 10000))).astype(np.int64).tolist()
    n = int(sum(sizes))
    offs = np.concatenate([[0], np.cumsum(sizes)])
    bf = torch.bfloat16
    torch.manual_seed(0x5EED0004)

    def make(dtype):
        if alloc == "packed":        # back to back: tensor i starts offs[i] elements into the slab
            slab = torch.empty(n, dtype=dtype, device="cuda")
            return [slab[offs[i]:offs[i + 1]] for i in range(len(sizes))]
        return [torch.empty(s, dtype=dtype, device="cuda") for s in sizes]

    dp, dg, dm, dv = make(bf), make(bf), make(torch.float32), make(torch.float32)
    if alloc == "packed":
        assert sum(1 for p in dp if p.data_ptr() % 16) > 8000         # most heads are not 16-byte aligned
    for p, m, v in zip(dp, dm, dv):
        p.uniform_(0.9, 1.1)
        m.zero_()
        v.zero_()
    flat = lambda ts: to_host(torch.cat(ts))
    ctx = mx.Context()
    t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.0)
    res = ctx.norm_result()
    p_ref, m_ref, v_ref = flat(dp), np.zeros(n, F), np.zeros(n, F)
    for step in range(3):
        for g in dg:
            g.normal_(0, 1e-2)
        ctx.global_norm(t_g, res, max_norm=1.0)
        ctx.adam(t_upd, hp, mx.make_prep(scale=res))
        r = ctx.read_norm_result(res)
        g_h = flat(dg)
        scale = check_norm(r, oracle_c.sumsq(g_h))                    # exact float64 sum on the host
        assert scale < 0.02                                           # norm ~ 1e-2 * sqrt(n) ~ 97: clip active
        args = B.adam_args(1e-3, 0.9, 0.999, 1e-8, 0.0, scale=scale)
        p_ref = oracle_c.f32_to_bf16(oracle_c.adam(p_ref, g_h, m_ref, v_ref, args, fused=True))
        same_bits(flat(dp), p_ref, f"p step {step}")
        same_bits(flat(dm), m_ref, f"m step {step}")
        same_bits(flat(dv), v_ref, f"v step {step}")
    t_g.close()
    t_upd.close()
    ctx.close()


# ---------------------------------------------------------------------------------------
# config 5
# ---------------------------------------------------------------------------------------

def test_config5_full_size_windows_and_norm():
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("8B")
    n = sum(sizes)
    assert n == 8_190_735_360 and len(sizes) == 399
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    if free < n * 16 + (8 << 30):
        pytest.skip("needs ~131 GB of free device memory")
    torch.manual_seed(0x5EED0005)
    bf = torch.bfloat16
    p_slab, offs, dp = carve(torch, sizes, bf)
    g_slab, _, dg = carve(torch, sizes, bf)
    a_slab, _, da = carve(torch, sizes, torch.float32)
    m_slab, _, dm = carve(torch, sizes, torch.float32)
    v_slab, _, dv = carve(torch, sizes, torch.float32)
    p_slab.normal_(0, 0.02)
    m_slab.normal_(0, 1e-4)          # non-trivial moments, as in the middle of training
    v_slab.normal_(0, 1e-4).square_()
    a_slab.fill_(float("nan"))       # the first accumulation must overwrite, not add

    # seeded windows in flat slab coordinates: tensor heads, tails, interiors of the largest tensors
    rng = np.random.default_rng(5)
    W = 8192
    starts = set()
    for i in rng.choice(len(sizes), 24, replace=False):
        starts.add(offs[i])
        starts.add(max(offs[i], offs[i] + sizes[i] - W))
    big = int(np.argmax(sizes))
    for s in rng.integers(0, sizes[big] - W, 16):
        starts.add(offs[big] + int(s) // 8 * 8 + 3)     # odd offsets: windows are not group aligned
    idx = torch.from_numpy(np.concatenate([np.arange(s, s + W) for s in sorted(starts)])).cuda()
    # padding between tensors belongs to no tensor: keep only indices that fall inside one
    ends = np.array(offs) + np.array(sizes)
    flat = idx.cpu().numpy()
    owner = np.searchsorted(np.array(offs), flat, side="right") - 1
    keep = flat < ends[owner]
    idx = idx[torch.from_numpy(keep).cuda()]

    def win(slab):
        return to_host(slab[idx])

    p0, m0, v0 = win(p_slab), win(m_slab), win(v_slab)
    ctx = mx.Context()
    t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, da)])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=m, v=v) for p, a, g, m, v in zip(dp, da, dg, dm, dv)])
    res = ctx.norm_result()
    micro = []
    for k in range(4):
        g_slab.normal_(0, 1e-3)
        micro.append(win(g_slab))
        if k < 3:
            ctx.accumulate(t_acc, first=(k == 0))
        else:
            ctx.accumulate_norm_only(t_acc, res, max_norm=1.0)
            # float64 reference of the same quantity by torch, tensor by tensor
            ref_sumsq = 0.0
            for a, g in zip(da, dg):
                ref_sumsq += float((a + g.float()).double().square().sum())
    hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
    ctx.adam_with_pending(t_upd, hp, mx.make_prep(scale=res))
    r = ctx.read_norm_result(res)
    ctx.synchronize()

    # norm: rel 1e-5 against the float64 reduction; the clip factor is the scalar chain of the reference
    assert abs(r.norm - math.sqrt(ref_sumsq)) <= 1e-5 * math.sqrt(ref_sumsq)
    expected_norm = 1e-3 * math.sqrt(4 * n)
    assert abs(r.norm - expected_norm) < 0.01 * expected_norm          # sanity: N(0,1e-6) summed 4 times
    n32, scale = O.norm_scale_c1(r.sumsq, 1.0)
    assert F(r.scale) == scale and F(r.norm_f32) == n32 and r.nonfinite == 0

    # windows through the oracle
    acc = None
    for k in range(4):
        acc = O.accumulate_fp32(acc, micro[k])
    assert np.array_equal(win(a_slab).view(np.uint32), O.accumulate_fp32(O.accumulate_fp32(
        O.accumulate_fp32(None, micro[0]), micro[1]), micro[2]).view(np.uint32)), "accumulation buffer (3 micro-batches)"
    ref = O.AdamW(5e-6, 0.9, 0.999, 1e-8, 0.01)
    ref.state["w"] = (m0.copy(), v0.copy())
    want_p = O.f32_to_bf16(ref.update_single("w", p0, acc * scale))
    assert np.array_equal(win(p_slab), want_p), "parameters"
    assert np.array_equal(win(m_slab).view(np.uint32), ref.state["w"][0].view(np.uint32)), "first moment"
    assert np.array_equal(win(v_slab).view(np.uint32), ref.state["w"][1].view(np.uint32)), "second moment"

    # End to end: the oracle with ITS OWN clip factor, taken from the float64 sum instead of the device's
    # (optimizers/mod.rs:87-102 -> adamw.rs:84-116).  Stated tolerance: 2 float32 ulp (rel 1e-6) on the
    # moments, 1 bf16 ulp on the parameters, norm rel 1e-5 (asserted above).
    _, own_scale = O.norm_scale_c1(ref_sumsq, 1.0)
    own = O.AdamW(5e-6, 0.9, 0.999, 1e-8, 0.01)
    own.state["w"] = (m0.copy(), v0.copy())
    own_p = O.f32_to_bf16(own.update_single("w", p0, acc * own_scale))
    assert_within_ulps(win(m_slab), own.state["w"][0], 2, 1e-6, "first moment, oracle's own clip factor")
    assert_within_ulps(win(v_slab), own.state["w"][1], 2, 1e-6, "second moment, oracle's own clip factor")
    assert_within_ulps(win(p_slab), own_p, 1, what="bf16 parameters, oracle's own clip factor")
    t_acc.close()
    t_upd.close()
    ctx.close()


def test_config5_every_element_of_every_sixth_tensor(oracle_c):
    """The benchmark's default step on the whole 8B list from generated inputs (one gradient buffer,
    refilled for each micro-batch); every element of parameters, moments and accumulation buffer of every
    sixth tensor -- the embedding and 66 others, 1.5 G elements -- is recomputed on the host by the C
    twin of the oracle from regenerated inputs and compared bit for bit."""
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("8B")
    n, nt = sum(sizes), len(sizes)
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    if free < n * 16 + (8 << 30):
        pytest.skip("needs ~131 GB of free device memory")
    bf = torch.bfloat16
    dp = [torch.empty(s, dtype=bf, device="cuda") for s in sizes]
    dg = [torch.empty(s, dtype=bf, device="cuda") for s in sizes]
    da = [torch.empty(s, device="cuda") for s in sizes]
    dm = [torch.empty(s, device="cuda") for s in sizes]
    dv = [torch.empty(s, device="cuda") for s in sizes]
    ctx = mx.Context()
    SEED, CFG = 0x5EED0001, 5
    P, M, V, G = 0, 1, 2, 3          # stream ids inside the key; micro-batch k uses stream G + k

    def spec(stream):
        if stream == P:
            return mx.SYNTH_NORMAL, 0.02, 0.0
        if stream == M:
            return mx.SYNTH_NORMAL, 1e-4, 0.0
        if stream == V:
            return mx.SYNTH_UNIFORM, 0.0, 1e-8
        return mx.SYNTH_NORMAL, 1e-3, 0.0

    def fill(tensors, stream):
        dist, a, b = spec(stream)
        for i, t in enumerate(tensors):
            ctx.fill_synthetic(t, mx.synthetic_key(SEED, CFG, 0, stream, i), dist, a, b)

    def host(i, stream, dtype):
        dist, a, b = spec(stream)
        return oracle_c.fill_synthetic(sizes[i], dtype, mx.synthetic_key(SEED, CFG, 0, stream, i), dist, a, b)

    fill(dp, P); fill(dm, M); fill(dv, V)
    t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(dg, da)])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=m, v=v) for p, a, g, m, v in zip(dp, da, dg, dm, dv)])
    res = ctx.norm_result()
    for k in range(4):
        fill(dg, G + k)
        if k < 3:
            ctx.accumulate(t_acc, first=(k == 0))
        else:
            ctx.accumulate_norm_only(t_acc, res, max_norm=1.0)
    ctx.adam_with_pending(t_upd, mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01), mx.make_prep(scale=res))
    r = ctx.read_norm_result(res)
    expected_norm = 1e-3 * math.sqrt(4 * n)
    assert abs(r.norm - expected_norm) < 0.01 * expected_norm
    n32, scale = O.norm_scale_c1(r.sumsq, 1.0)
    assert F(r.scale) == scale and F(r.norm_f32) == n32 and r.nonfinite == 0

    args = B.adam_args(5e-6, 0.9, 0.999, 1e-8, 0.01, scale=float(scale))
    checked = 0
    for i in range(0, nt, 6):
        p_ref, m_ref, v_ref = host(i, P, "bf16"), host(i, M, "f32"), host(i, V, "f32")
        acc = np.empty(sizes[i], F)
        for k in range(3):
            oracle_c.accumulate_f32(acc, host(i, G + k, "bf16"), k == 0)
        same_bits(da[i].cpu().numpy(), acc, f"accumulation buffer of tensor {i} (three micro-batches)")
        oracle_c.accumulate_f32(acc, host(i, G + 3, "bf16"), False)
        p_new = oracle_c.f32_to_bf16(oracle_c.adam(p_ref, acc, m_ref, v_ref, args, fused=True))
        same_bits(to_host(dp[i]), p_new, f"p of tensor {i}")
        same_bits(dm[i].cpu().numpy(), m_ref, f"m of tensor {i}")
        same_bits(dv[i].cpu().numpy(), v_ref, f"v of tensor {i}")
        checked += sizes[i]
    assert checked > 1_400_000_000
    t_acc.close()
    t_upd.close()
    ctx.close()


def bit_checksums(torch, slab, piece=1 << 26):
    """(sum of the bit patterns, sum of bit pattern x (1 + position mod 65521)) over a whole slab, in
    wrapping int64: a single flipped bit, or two equal values changing places, changes one of them."""
    bits = slab.view(torch.int16 if slab.element_size() == 2 else torch.int32)
    plain = weighted = 0
    for start in range(0, bits.numel(), piece):
        b = bits[start:start + piece].to(torch.int64)
        w = torch.arange(start, start + b.numel(), device=slab.device, dtype=torch.int64).remainder_(65521).add_(1)
        plain = (plain + int(b.sum())) & (2 ** 64 - 1)
        weighted = (weighted + int((b * w).sum())) & (2 ** 64 - 1)
    return plain, weighted


def test_config5_deferred_accumulation_equals_buffered_every_element():
    import torch
    import mxopt as mx
    _, sizes = qwen_sizes("8B")
    n = sum(sizes)
    torch.cuda.empty_cache()      # what earlier tests left in torch's cache is not free memory to the driver
    free, _ = torch.cuda.mem_get_info()
    if free < n * 22 + (12 << 30):
        pytest.skip("needs ~190 GB of free device memory")
    bf = torch.bfloat16
    p_slab, offs, dp = carve(torch, sizes, bf)
    m_slab, _, dm = carve(torch, sizes, torch.float32)
    v_slab, _, dv = carve(torch, sizes, torch.float32)
    micro = [carve(torch, sizes, bf) for _ in range(4)]
    ctx = mx.Context()
    seed = 0x5EED0055

    def generate():
        for i in range(len(sizes)):
            ctx.fill_synthetic(dp[i], mx.synthetic_key(seed, 5, 0, 0, i), mx.SYNTH_NORMAL, 0.02)
            ctx.fill_synthetic(dm[i], mx.synthetic_key(seed, 5, 0, 1, i), mx.SYNTH_NORMAL, 1e-4)
            ctx.fill_synthetic(dv[i], mx.synthetic_key(seed, 5, 0, 2, i), mx.SYNTH_UNIFORM, 0.0, 1e-8)

    for k, (_, _, dg) in enumerate(micro):
        for i in range(len(sizes)):
            ctx.fill_synthetic(dg[i], mx.synthetic_key(seed, 5, 0, 3 + k, i), mx.SYNTH_NORMAL, 1e-3)
    hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
    res = ctx.norm_result()

    # buffered: three accumulation passes, the fourth micro-batch measured and folded into the update
    generate()
    a_slab, _, da = carve(torch, sizes, torch.float32)
    for k in range(4):
        t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(micro[k][2], da)])
        if k < 3:
            ctx.accumulate(t_acc, first=(k == 0))
        else:
            ctx.accumulate_norm_only(t_acc, res, max_norm=1.0)
        ctx.synchronize()
        t_acc.close()
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=m, v=v)
                       for p, a, g, m, v in zip(dp, da, micro[3][2], dm, dv)])
    ctx.adam_with_pending(t_upd, hp, mx.make_prep(scale=res))
    r_buf = ctx.read_norm_result(res)
    t_upd.close()
    del a_slab, da
    sums_buf = [bit_checksums(torch, s) for s in (p_slab, m_slab, v_slab)]

    # deferred: no buffer; the inputs are regenerated, the micro-batches are still where they were
    generate()
    sums_before = [bit_checksums(torch, s) for s in (p_slab, m_slab, v_slab)]
    assert sums_before != sums_buf                       # the update did change every stream
    t_def = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, micro[0][2], dm, dv)])
    t_def.set_pending([mb[2] for mb in micro[1:]])
    ctx.norm_with_pending_list(t_def, res, max_norm=1.0)
    ctx.adam_with_pending_list(t_def, hp, mx.make_prep(scale=res))
    r_def = ctx.read_norm_result(res)
    sums_def = [bit_checksums(torch, s) for s in (p_slab, m_slab, v_slab)]

    assert abs(r_def.sumsq - r_buf.sumsq) <= 1e-12 * r_buf.sumsq and r_def.scale == r_buf.scale and r_def.nonfinite == 0
    expected_norm = 1e-3 * math.sqrt(4 * n)
    assert abs(r_def.norm - expected_norm) < 0.01 * expected_norm
    assert sums_def == sums_buf
    t_def.close()
    ctx.close()
