"""mxopt_global_norm_static: the global-norm entry point that allocates nothing (its per-workgroup
partial sums live in a fixed array inside the library's code object).  Checked, through the C ABI,
against mxopt_global_norm on the same inputs, bit for bit, on two calls in a row of which the second
has the smaller input; a fresh context is used so that the allocating entry point has not yet sized
any buffer the static one could be leaning on."""
from __future__ import annotations

import math

import numpy as np
import pytest

from gpu_util import to_dev

pytestmark = pytest.mark.gpu
F = np.float32


def _grads(seed, sizes, bf16):
    rng = np.random.default_rng(seed)
    out = []
    for n in sizes:
        g = rng.normal(0, 1e-2, n).astype(F)
        if bf16:
            g = (g.view(np.uint32) >> 16).astype(np.uint16)
        out.append(g)
    return out


def _fields(r):
    return (np.float64(r.sumsq).tobytes(), np.float64(r.norm).tobytes(), F(r.norm_f32).tobytes(),
            F(r.scale).tobytes(), int(r.nonfinite))


@pytest.mark.parametrize("bf16", [False, True])
def test_static_norm_matches_allocating_norm_twice_in_a_row(bf16):
    import torch
    import mxopt as mx
    assert torch.cuda.is_available()
    big = [4096 * 700 + 13, 1, 0, 4095, 4097, 100003, 4096 * 64]
    small = [4096 * 3 + 5, 77]
    static_ctx, plain_ctx = mx.Context(), mx.Context()
    try:
        for call, sizes in enumerate((big, small)):          # second call: smaller input, stale slots behind it
            gs = _grads(900 + call, sizes, bf16)
            dg = [to_dev(g, 3 if call else 0) for g in gs]
            res_s, res_p = static_ctx.norm_result(), plain_ctx.norm_result()
            t_s = static_ctx.table([mx.TensorSpec(g=g) for g in dg])
            t_p = plain_ctx.table([mx.TensorSpec(g=g) for g in dg])
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            for max_norm, mode in ((1e-3, mx.CLIP_ALWAYS_MULTIPLY), (1e6, mx.CLIP_IF_ABOVE), (-1.0, mx.CLIP_ALWAYS_MULTIPLY)):
                static_ctx.global_norm_static(t_s, res_s, max_norm=max_norm, clip_mode=mode)
                got = static_ctx.read_norm_result(res_s)
                if call == 0 and max_norm == 1e-3:
                    # nothing was allocated on the device by the first static call of a fresh context
                    assert torch.cuda.mem_get_info()[0] == free_before
                plain_ctx.global_norm(t_p, res_p, max_norm=max_norm, clip_mode=mode)
                want = plain_ctx.read_norm_result(res_p)
                assert _fields(got) == _fields(want), (call, max_norm, mode)
            # and the value itself, against the exact float64 sum of the stored gradients
            exact = 0.0
            for g in gs:
                x = (g.astype(np.uint32) << 16).view(F) if bf16 else g
                exact += float(np.sum(x.astype(np.float64) ** 2))
            assert abs(got.sumsq - exact) <= 1e-6 * exact
            assert abs(got.norm - math.sqrt(exact)) <= 1e-5 * math.sqrt(exact)
            # clamp_pre in front of the norm goes through the same path
            prep = mx.make_prep(clamp_pre=(-5e-3, 5e-3))
            static_ctx.global_norm_static(t_s, res_s, prep=prep, max_norm=1e-3)
            plain_ctx.global_norm(t_p, res_p, prep=prep, max_norm=1e-3)
            assert _fields(static_ctx.read_norm_result(res_s)) == _fields(plain_ctx.read_norm_result(res_p))
    finally:
        static_ctx.close()
        plain_ctx.close()


def test_static_norm_flags_nonfinite_and_refuses_oversized_grids():
    import mxopt as mx
    ctx = mx.Context()
    try:
        gs = _grads(77, [4096 * 40 + 9], False)
        gs[0][12345] = np.nan
        table = ctx.table([mx.TensorSpec(g=to_dev(gs[0]))])
        res = ctx.norm_result()
        ctx.global_norm_static(table, res, max_norm=1.0)
        r = ctx.read_norm_result(res)
        assert r.nonfinite == 1 and math.isnan(r.scale)
        # one float64 slot per workgroup: a grid beyond the fixed array's size is refused, not truncated
        big = ctx.table([mx.TensorSpec(g=to_dev(_grads(78, [4096 * 20000], False)[0]))])
        ctx.set_option("grid_blocks_per_cu", 128)          # 256 CUs x 128 > 16384 slots
        with pytest.raises(mx.MxoptError, match="fixed array holds 16384"):
            ctx.global_norm_static(big, res, max_norm=1.0)
        ctx.global_norm(big, res, max_norm=1.0)            # the allocating entry point takes it
        assert ctx.read_norm_result(res).nonfinite == 0
        ctx.set_option("grid_blocks_per_cu", 16)
        ctx.global_norm_static(big, res, max_norm=1.0)     # and so does the static one at the default grid
        assert ctx.read_norm_result(res).nonfinite == 0
    finally:
        ctx.close()
