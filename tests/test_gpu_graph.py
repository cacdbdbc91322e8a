"""The kernel-level entry points are plain launches on the context's stream once the reduction's
partials buffer exists (one warm-up call): a whole step can be captured into a HIP graph and replayed.
Every replay is checked against the oracle, with eager work and synchronisations in between."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
SIZES = [5, 4096, 4097, 3 * 4096 + 11, 100003, 64]


def test_clip_and_adamw_step_replays_from_a_graph():
    import torch
    import mxopt as mx
    rng = np.random.default_rng(123)
    ps = [O.f32_to_bf16(rng.normal(0, 0.02, n).astype(F)) for n in SIZES]
    stream = torch.cuda.Stream()
    ctx = mx.Context(stream=stream)
    dp = [to_dev(p) for p in ps]
    dg = [torch.zeros(n, dtype=torch.bfloat16, device="cuda") for n in SIZES]
    dm = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in SIZES]
    dv = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in SIZES]
    res, res2 = ctx.norm_result(), ctx.norm_result()
    t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
    hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
    prep = mx.make_prep(scale=res, skip_if_nonfinite=res)
    torch.cuda.synchronize()

    ctx.global_norm(t_g, res, max_norm=1e-2)          # warm-up: allocates the partials buffer
    ctx.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        ctx.global_norm(t_g, res, max_norm=1e-2)
        ctx.adam(t_upd, hp, prep)
    torch.cuda.synchronize()
    for i, p in enumerate(ps):                        # capturing runs nothing
        assert_bit_equal(to_host(dp[i]), p, f"p{i} untouched by capture")

    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    cur = list(ps)
    scratch = torch.zeros(1 << 20, device="cuda")
    for it in range(4):
        gs = [O.f32_to_bf16(rng.normal(0, 1e-3 * (it + 1), n).astype(F)) for n in SIZES]
        if it == 2:
            gs[3][77] = 0x7FC0                        # a NaN gradient: this replay must change nothing
        for d, g in zip(dg, gs):
            d.copy_(to_dev(g))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        r = ctx.read_norm_result(res)
        if it == 2:
            assert r.nonfinite == 1
        else:
            n32, scale = O.norm_scale_c1(O.exact_sumsq(gs), 1e-2)
            assert r.nonfinite == 0 and abs(r.norm - float(n32)) <= 1e-5 * float(n32)
            for i in range(len(SIZES)):
                cur[i] = O.f32_to_bf16(ref.update_single(str(i), cur[i], O.bf16_to_f32(gs[i]) * F(r.scale)))
        for i in range(len(SIZES)):
            assert_bit_equal(to_host(dp[i]), cur[i], f"p{i} replay {it}")
            if str(i) in ref.state:
                assert_bit_equal(to_host(dm[i]), ref.state[str(i)][0], f"m{i} replay {it}")
                assert_bit_equal(to_host(dv[i]), ref.state[str(i)][1], f"v{i} replay {it}")
        scratch.add_(1.0)                             # eager work between replays
        ctx.global_norm(t_g, res2)                    # and an eager call into the library itself
        torch.cuda.synchronize()
    for t in (t_g, t_upd):
        t.close()
    ctx.close()


def test_deferred_accumulation_step_replays_from_a_graph():
    """norm over three un-summed micro-batches + AdamW on their sum, captured once; the pending pointers
    were uploaded before the capture (mxopt_table_set_pending copies from host memory)."""
    import torch
    import mxopt as mx
    rng = np.random.default_rng(321)
    ps = [O.f32_to_bf16(rng.normal(0, 0.02, n).astype(F)) for n in SIZES]
    stream = torch.cuda.Stream()
    ctx = mx.Context(stream=stream)
    dp = [to_dev(p) for p in ps]
    dmicro = [[torch.zeros(n, dtype=torch.bfloat16, device="cuda") for n in SIZES] for _ in range(3)]
    dm = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in SIZES]
    dv = [torch.zeros(n, dtype=torch.float32, device="cuda") for n in SIZES]
    res = ctx.norm_result()
    table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dmicro[0], dm, dv)])
    table.set_pending(dmicro[1:])
    hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
    prep = mx.make_prep(scale=res, skip_if_nonfinite=res)
    ctx.norm_with_pending_list(table, res, max_norm=1e-2)     # warm-up: sizes the partials buffer
    ctx.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        ctx.norm_with_pending_list(table, res, max_norm=1e-2)
        ctx.adam_with_pending_list(table, hp, prep)
    torch.cuda.synchronize()

    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    cur = list(ps)
    scratch = torch.zeros(1 << 20, device="cuda")
    for it in range(4):
        micro = [[O.f32_to_bf16(rng.normal(0, 1e-3 * (it + 1), n).astype(F)) for n in SIZES] for _ in range(3)]
        if it == 1:
            micro[2][4][1234] = 0x7F80                # +Inf in the last micro-batch: nothing may change
        for dst, src in zip(dmicro, micro):
            for d, g in zip(dst, src):
                d.copy_(to_dev(g))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        r = ctx.read_norm_result(res)
        if it == 1:
            assert r.nonfinite == 1
        else:
            acc = [O.accumulate_fp32(O.accumulate_fp32(O.accumulate_fp32(None, a), b), c) for a, b, c in zip(*micro)]
            n32, _ = O.norm_scale_c1(O.exact_sumsq(acc), 1e-2)
            assert r.nonfinite == 0 and abs(r.norm - float(n32)) <= 1e-5 * float(n32)
            for i in range(len(SIZES)):
                cur[i] = O.f32_to_bf16(ref.update_single(str(i), cur[i], acc[i] * F(r.scale)))
        for i in range(len(SIZES)):
            assert_bit_equal(to_host(dp[i]), cur[i], f"p{i} replay {it}")
        scratch.add_(1.0)
        torch.cuda.synchronize()
    table.close()
    ctx.close()
