"""Random call sequences against the optimizer objects (state by name, per-call step counting, cached and
retargeted tables, first-step velocity, checkpoints): update_single in and out of place, update_many over
subsets in any order with the same or with moved buffers, update_many_accumulated over 1..12 un-summed
micro-batches with or without clipping, reset, save_file/load_file into a fresh object.  After every call
the parameters must equal the oracle's bit for bit.  Derandomised; MXOPT_PROPERTY_EXAMPLES=<n> draws n
fresh random sequences instead."""
import os

import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
SIZES = {"embed": 12289, "ln": 64, "tiny": 7, "w1": 4097, "w2": 1, "w3": 8192}
SOAK = int(os.environ.get("MXOPT_PROPERTY_EXAMPLES", "0"))
OPS = st.sampled_from(["single", "single_in_place", "many", "many", "many_moved", "accumulated", "accumulated",
                       "reset", "checkpoint"])


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


def make_pair(mx, kind, ctx):
    if kind == "adam":
        return (lambda: mx.Adam(1e-2, 0.9, 0.99, 1e-8, False, ctx=ctx)), O.Adam(1e-2, 0.9, 0.99, 1e-8, False)
    if kind == "adamw":
        return (lambda: mx.AdamW(1e-2, 0.9, 0.99, 1e-8, 0.05, False, ctx=ctx)), O.AdamW(1e-2, 0.9, 0.99, 1e-8, 0.05, False)
    if kind == "adamw_bias":
        return (lambda: mx.AdamW(1e-2, 0.9, 0.99, 1e-8, 0.05, True, ctx=ctx)), O.AdamW(1e-2, 0.9, 0.99, 1e-8, 0.05, True)
    if kind == "sgd":
        return (lambda: mx.SGD(0.05, 0.9, 1e-3, 0.1, False, ctx=ctx)), O.SGD(0.05, 0.9, 1e-3, 0.1, False)
    if kind == "sgd_nesterov":
        return (lambda: mx.SGD(0.05, 0.9, 0.0, 0.0, True, ctx=ctx)), O.SGD(0.05, 0.9, 0.0, 0.0, True)
    return (lambda: mx.RMSprop(1e-2, 0.95, 1e-8, 1e-3, ctx=ctx)), O.RMSprop(1e-2, 0.95, 1e-8, 1e-3)


@settings(max_examples=SOAK or 120, deadline=None, derandomize=not SOAK, database=None,
          suppress_health_check=list(HealthCheck))
@given(kind=st.sampled_from(["adam", "adamw", "adamw_bias", "sgd", "sgd_nesterov", "rmsprop"]), bf16=st.booleans(),
       g_bf16=st.booleans(), ops=st.lists(OPS, min_size=1, max_size=12), seed=st.integers(0, 2 ** 31))
def test_random_optimizer_sequences(mx, tmp_path_factory, kind, bf16, g_bf16, ops, seed):
    import torch
    rng = np.random.default_rng(seed)
    ctx = mx.default_context()
    new_dev, ref = make_pair(mx, kind, ctx)
    dev = new_dev()
    cast_p = O.f32_to_bf16 if bf16 else (lambda a: a.astype(F))
    cast_g = O.f32_to_bf16 if g_bf16 else (lambda a: a.astype(F))
    cur = {k: cast_p(rng.normal(0, 0.5, n).astype(F)) for k, n in SIZES.items()}     # the oracle's parameters
    dparams = {k: to_dev(v) for k, v in cur.items()}
    adam_like = kind.startswith("adam")
    ckpt = str(tmp_path_factory.mktemp("ckpt") / "state.safetensors")

    def grad(k):
        return cast_g(rng.normal(0, 0.01, SIZES[k]).astype(F))

    def ref_step(k, g):
        cur[k] = cast_p(ref.update_single(k, cur[k], g))

    for it, op in enumerate(ops):
        what = f"call {it} ({op})"
        if op in ("single", "single_in_place"):
            k = list(SIZES)[int(rng.integers(0, len(SIZES)))]
            g = grad(k)
            if op == "single_in_place":
                dev.update_single(k, dparams[k], to_dev(g), out=dparams[k])
            else:
                dparams[k] = dev.update_single(k, dparams[k], to_dev(g), out_dtype="param")
            ref_step(k, g)
        elif op in ("many", "many_moved"):
            names = [k for k in SIZES if rng.random() < 0.7] or ["w1"]
            rng.shuffle(names)
            if op == "many_moved":           # the same tensors in other buffers, as a functional host hands them over
                for k in names:
                    dparams[k] = dparams[k].clone()
            gs = {k: grad(k) for k in names}
            dev.update_many(names, [dparams[k] for k in names], [to_dev(gs[k]) for k in names],
                            outs=[dparams[k] for k in names])
            for k in names:
                ref_step(k, gs[k])
        elif op == "accumulated":
            names = [k for k in SIZES if rng.random() < 0.7] or ["embed"]
            n_micro = int(rng.integers(1, 13))
            micro = [{k: grad(k) for k in names} for _ in range(n_micro)]
            clip = bool(rng.integers(0, 2))
            res = ctx.norm_result()
            dev.update_many_accumulated(names, [dparams[k] for k in names],
                                        [[to_dev(mb[k]) for k in names] for mb in micro],
                                        max_norm=0.05 if clip else -1.0, norm_out=res if clip else None)
            acc = {}
            for k in names:
                a = None
                for mb in micro:
                    a = O.accumulate_fp32(a, mb[k])
                acc[k] = a
            if n_micro == 1 and not clip:
                # nothing was added and nothing multiplied: the lone gradient reaches the optimizer in its own
                # dtype, exactly as through update_many (a 16-bit gradient's square is 16-bit, mlx.cpp:2016-2020)
                acc = dict(micro[0])
            if clip:
                r = ctx.read_norm_result(res)
                exact = O.exact_sumsq(acc.values())
                assert abs(r.sumsq - exact) <= 1e-5 * max(exact, 1e-300), what
                scale = O.norm_scale_c1(r.sumsq, 0.05)[1]
                assert F(r.scale) == scale
                acc = {k: a * scale for k, a in acc.items()}
            for k in names:
                ref_step(k, acc[k])
        elif op == "reset":
            dev.reset()
            ref.reset()
        else:                                  # checkpoint: a fresh object continues from the file
            dev.save_file(ckpt)
            dev = new_dev()
            dev.load_file(ckpt)
        if adam_like:
            assert dev.step == ref.step, what
        for k in SIZES:
            assert_bit_equal(to_host(dparams[k]), cur[k], f"{what}: {k}")
