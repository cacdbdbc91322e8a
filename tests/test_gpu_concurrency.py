"""Two contexts driven from two host threads at once (the header allows one context per thread), and a
context on a side stream ordered only by that stream with the torch kernels that produce its inputs."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32


def test_two_contexts_on_two_threads():
    import torch
    import mxopt as mx
    sizes = [300007, 4096, 65, 120001]
    errors = []

    def worker(seed):
        try:
            torch.cuda.set_device(0)
            rng = np.random.default_rng(seed)
            stream = torch.cuda.Stream()
            ctx = mx.Context(stream=stream)
            ps = [rng.normal(0, 0.02, n).astype(F) for n in sizes]
            dp = [to_dev(p) for p in ps]
            dm = [torch.zeros(n, device="cuda") for n in sizes]
            dv = [torch.zeros(n, device="cuda") for n in sizes]
            dg = [torch.empty(n, device="cuda") for n in sizes]
            torch.cuda.synchronize()
            table = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v) for p, g, m, v in zip(dp, dg, dm, dv)])
            t_g = ctx.table([mx.TensorSpec(g=g) for g in dg])
            res = ctx.norm_result()
            torch.cuda.synchronize()
            hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
            ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
            cur = list(ps)
            for it in range(25):
                gs = [rng.normal(0, 1e-3, n).astype(F) for n in sizes]
                for d, g in zip(dg, gs):
                    d.copy_(torch.from_numpy(g))
                torch.cuda.synchronize()
                ctx.global_norm(t_g, res, max_norm=1e-2)
                ctx.adam(table, hp, mx.make_prep(scale=res))
                r = ctx.read_norm_result(res)
                for i in range(len(sizes)):
                    cur[i] = ref.update_single(str(i), cur[i], gs[i] * F(r.scale))
            for i in range(len(sizes)):
                assert_bit_equal(to_host(dp[i]), cur[i], f"seed {seed} tensor {i}")
            table.close()
            t_g.close()
            ctx.close()
        except BaseException as e:  # noqa: BLE001 - reported to the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(s,)) for s in (1, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]


def test_side_stream_orders_with_its_producers():
    """Inputs are produced by torch kernels on the same side stream, long enough to still be running
    when the library's kernels are enqueued; no host synchronisation in between."""
    import torch
    import mxopt as mx
    n = 1 << 24
    stream = torch.cuda.Stream()
    ctx = mx.Context(stream=stream)
    p = torch.ones(n, device="cuda")
    g = torch.zeros(n, device="cuda")
    out = torch.empty(n, device="cuda")
    table = ctx.table([mx.TensorSpec(p=p, p_out=out, g=g)])
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        for k in range(50):                 # g = 50 after a chain of dependent kernels
            g.add_(1.0)
        ctx.sgd_plain(table, 0.01)          # enqueued behind them on the same stream
        back = out.clone()                  # and a torch consumer behind the library's kernel
    stream.synchronize()
    assert torch.all(back == (1.0 - F(0.01) * F(50.0))).item()
    table.close()
    ctx.close()
