"""No kernel writes outside its tensors: every buffer lives inside a slab between two guard zones filled with a
sentinel bit pattern; after every entry point has run over ragged sizes and odd element offsets the guards
must be untouched, and input-only streams must be unchanged."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GUARD = 64           # elements on either side
SIZES = [0, 1, 7, 8, 9, 63, 4095, 4096, 4097, 8191, 8200, 12288, 50001]


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


class Guarded:
    """A list of tensors, each a view into its own slab: [guard | offset | payload | guard]."""

    def __init__(self, torch, sizes, dtype, offset, fill):
        self.torch, self.dtype = torch, dtype
        self.int_dtype = torch.int16 if dtype != torch.float32 else torch.int32
        self.sentinel = 0x7FA5 if dtype != torch.float32 else 0x7FA5A5A5      # a NaN with a recognisable payload
        self.slabs, self.views, self.spans = [], [], []
        for n in sizes:
            slab = torch.empty(GUARD + offset + n + GUARD, dtype=dtype, device="cuda")
            slab.view(self.int_dtype).fill_(self.sentinel)
            view = slab[GUARD + offset:GUARD + offset + n]
            if fill == "normal":
                view.copy_(torch.randn(n, device="cuda") * 0.01)
            elif fill == "zero":
                view.zero_()
            self.slabs.append(slab)
            self.views.append(view)
            self.spans.append((GUARD + offset, GUARD + offset + n))
        self.before = None

    def snapshot(self):
        self.before = [s.clone() for s in self.slabs]

    def assert_guards_intact(self, what):
        for i, (slab, (a, b)) in enumerate(zip(self.slabs, self.spans)):
            bits = slab.view(self.int_dtype)
            ok = bool((bits[:a] == self.sentinel).all()) and bool((bits[b:] == self.sentinel).all())
            assert ok, f"{what}: guard zone of tensor {i} ({b - a} elements) was written"

    def assert_unchanged(self, what):
        for i, (slab, old) in enumerate(zip(self.slabs, self.before)):
            assert self.torch.equal(slab.view(self.int_dtype), old.view(self.int_dtype)), f"{what}: input tensor {i} changed"


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("offset", [0, 1, 3, 5])
def test_guard_zones_survive_every_kernel(mx, bf16, offset):
    import torch
    torch.manual_seed(offset + 10 * bf16)
    ctx = mx.default_context()
    dt = torch.bfloat16 if bf16 else torch.float32
    f32 = torch.float32
    p = Guarded(torch, SIZES, dt, offset, "normal")
    g = Guarded(torch, SIZES, dt, offset, "normal")
    g2 = Guarded(torch, SIZES, dt, offset, "normal")
    g3 = Guarded(torch, SIZES, dt, offset, "normal")
    m = Guarded(torch, SIZES, f32, offset, "zero")
    v = Guarded(torch, SIZES, f32, offset, "zero")
    acc = Guarded(torch, SIZES, f32, offset, "zero")
    out = Guarded(torch, SIZES, dt, offset, "zero")
    everything = {"p": p, "g": g, "g2": g2, "g3": g3, "m": m, "v": v, "acc": acc, "out": out}
    res = ctx.norm_result()

    def run(what, call, inputs=("g", "g2", "g3")):
        """`inputs`: the streams this call may only read."""
        for name in inputs:
            everything[name].snapshot()
        call()
        ctx.synchronize()
        for name, buf in everything.items():
            buf.assert_guards_intact(f"{what} [{name}]")
        for name in inputs:
            everything[name].assert_unchanged(f"{what} [{name}]")

    adam_hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
    upd = ctx.table([mx.TensorSpec(p=a, p_out=a, g=b, m=c, v=d) for a, b, c, d in zip(p.views, g.views, m.views, v.views)])
    run("global_norm", lambda: ctx.global_norm(upd, res, max_norm=1.0), inputs=("g", "p", "m", "v"))
    run("adam", lambda: ctx.adam(upd, adam_hp, mx.make_prep(scale=res)))
    run("rmsprop", lambda: ctx.rmsprop(upd, mx.rmsprop_hp(1e-3, 0.99, 1e-8, 0.0)), inputs=("g", "m"))
    run("sgd", lambda: ctx.sgd(upd, mx.sgd_hp(1e-2, 0.9, 1e-4, 0.0, False)), inputs=("g", "m"))
    run("sgd_plain", lambda: ctx.sgd_plain(upd, 1e-2), inputs=("g", "m", "v"))

    tr = ctx.table([mx.TensorSpec(g=a, g_out=b) for a, b in zip(g.views, out.views)])
    run("grad_transform", lambda: ctx.grad_transform(tr, mx.make_prep(clamp_pre=(-0.01, 0.01), scale=res)),
        inputs=("g", "p", "m", "v", "acc"))

    ac = ctx.table([mx.TensorSpec(g=a, g_out=b) for a, b in zip(g.views, acc.views)])
    run("accumulate (first)", lambda: ctx.accumulate(ac, first=True), inputs=("g", "p", "m", "v", "out"))
    run("accumulate", lambda: ctx.accumulate(ac, first=False, out=res, max_norm=1.0), inputs=("g", "p", "m", "v", "out"))
    run("accumulate_transformed", lambda: ctx.accumulate_transformed(ac, first=False, prep=mx.make_prep(clamp_pre=(-0.01, 0.01))),
        inputs=("g", "p", "m", "v", "out"))
    run("accumulate_norm_only", lambda: ctx.accumulate_norm_only(ac, res, max_norm=1.0), inputs=("g", "acc", "p", "m", "v", "out"))

    pend = ctx.table([mx.TensorSpec(p=a, p_out=a, g=b, g_out=c, m=d, v=e)
                      for a, b, c, d, e in zip(p.views, acc.views, g.views, m.views, v.views)])
    run("adam_with_pending", lambda: ctx.adam_with_pending(pend, adam_hp, mx.make_prep(scale=res)), inputs=("g", "acc", "out"))
    run("sgd_plain_with_pending", lambda: ctx.sgd_plain_with_pending(pend, 1e-2, 0.0, mx.make_prep(scale=res), prep_covers_sum=True),
        inputs=("g", "acc", "m", "v", "out"))

    upd.set_pending([g2.views, g3.views])
    run("norm_with_pending_list", lambda: ctx.norm_with_pending_list(upd, res, max_norm=1.0),
        inputs=("g", "g2", "g3", "p", "m", "v", "acc", "out"))
    run("adam_with_pending_list", lambda: ctx.adam_with_pending_list(upd, adam_hp, mx.make_prep(scale=res)),
        inputs=("g", "g2", "g3", "acc", "out"))
    run("sgd_plain_with_pending_list", lambda: ctx.sgd_plain_with_pending_list(upd, 1e-2, 0.0, mx.make_prep(scale=res)),
        inputs=("g", "g2", "g3", "m", "v", "acc", "out"))
    run("sgd_plain_with_pending_list_each",
        lambda: ctx.sgd_plain_with_pending_list_each(upd, 1e-2, [res.scale_ptr] * 3, prep=mx.make_prep(clamp_pre=(-0.01, 0.01))),
        inputs=("g", "g2", "g3", "m", "v", "acc", "out"))

    def fill():
        for i, view in enumerate(out.views):
            ctx.fill_synthetic(view, 1234 + i, mx.SYNTH_NORMAL, 1e-3)
    run("fill_synthetic", fill, inputs=("g", "g2", "g3", "p", "m", "v", "acc"))
    for t in (upd, tr, ac, pend):
        t.close()
