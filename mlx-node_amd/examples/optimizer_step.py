#!/usr/bin/env python3
"""One optimizer step four ways, on a small Qwen3-shaped list, checking that they agree bit for bit:

  1. the reference's call sequence, tensor by tensor: accumulate_gradients per micro-batch,
     GradientUtils.clip_grad_norm, then AdamW.update_single for every parameter
     (what packages/trl's trainers do through optimizers/*.rs today);
  2. the same objects, one launch for the whole list (update_many with the clip fused in);
  3. the kernel level with the last micro-batch folded into the update;
  4. deferred accumulation: the micro-batches are never summed into a buffer.

Run on an MI355X:  python mlx-node_amd/examples/optimizer_step.py
"""
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import mxopt as mx                                    # noqa: E402
from mxopt.qwen3_shapes import QWEN3, numel, param_list  # noqa: E402


def main() -> int:
    ctx = mx.default_context()
    shapes = [(name, max(64, numel(shape) // 4096)) for name, shape in param_list(QWEN3["0.6B"])][:40]
    names = [n for n, _ in shapes]
    bf = torch.bfloat16
    seed = 2024
    max_norm = 0.25                                       # below the gradient norm: the clip is active

    def fresh(stream, dtype, std):
        out = []
        for i, (_, n) in enumerate(shapes):
            t = torch.empty(n, dtype=dtype, device="cuda")
            ctx.fill_synthetic(t, mx.synthetic_key(seed, 0, 0, stream, i), mx.SYNTH_NORMAL, std)
            out.append(t)
        return out

    micro = [fresh(10 + k, bf, 1e-3) for k in range(4)]       # four micro-batches of bf16 gradients
    hyper = dict(learning_rate=5e-6, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01)
    results = {}

    # 1. tensor by tensor, the reference's own sequence (float32 accumulation)
    params = fresh(1, bf, 0.02)
    acc = {}
    for mb in micro:
        acc = mx.accumulate_gradients(acc, {n: g.float() for n, g in zip(names, mb)})
    clipped, norm = mx.GradientUtils.clip_grad_norm_with_norm(acc, max_norm)
    opt = mx.AdamW(**hyper)
    results["update_single loop"] = [opt.update_single(n, p, clipped[n], out_dtype=bf) for n, p in zip(names, params)]

    # 2. one launch: the clip factor stays on the device and is applied inside the update
    params = fresh(1, bf, 0.02)
    res = ctx.norm_result()
    t_norm = ctx.table([mx.TensorSpec(g=acc[n]) for n in names])
    ctx.global_norm(t_norm, res, max_norm=max_norm)
    opt = mx.AdamW(**hyper)
    results["update_many"] = opt.update_many(names, params, [acc[n] for n in names], outs=params,
                                             prep=mx.make_prep(scale=res))

    # 3. kernel level, last micro-batch folded into the update
    params = fresh(1, bf, 0.02)
    buf = [torch.empty(n, dtype=torch.float32, device="cuda") for _, n in shapes]
    m = [torch.zeros_like(b) for b in buf]
    v = [torch.zeros_like(b) for b in buf]
    for k, mb in enumerate(micro):
        t_acc = ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(mb, buf)])
        if k < 3:
            ctx.accumulate(t_acc, first=(k == 0))
        else:
            ctx.accumulate_norm_only(t_acc, res, max_norm=max_norm)
    t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=g, m=mm, v=vv)
                       for p, a, g, mm, vv in zip(params, buf, micro[3], m, v)])
    hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
    ctx.adam_with_pending(t_upd, hp, mx.make_prep(scale=res))
    results["folded kernels"] = params

    # 4. deferred accumulation: no buffer at all
    params = fresh(1, bf, 0.02)
    opt = mx.AdamW(**hyper)
    results["deferred"] = opt.update_many_accumulated(names, params, micro, max_norm=max_norm, norm_out=res)

    ctx.synchronize()
    base = results["update_single loop"]
    ok = True
    for how, ps in results.items():
        same = all(torch.equal(a.view(torch.int16), b.view(torch.int16)) for a, b in zip(base, ps))
        print(f"{how:20s} {'identical' if same else 'DIFFERENT'}")
        ok = ok and same
    print(f"gradient norm {norm:.6g}, clip factor {ctx.read_norm_result(res).scale:.6g}, "
          f"{sum(n for _, n in shapes)} elements in {len(shapes)} tensors")
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
