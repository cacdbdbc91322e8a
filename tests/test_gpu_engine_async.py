"""mxopt_engine_micro_batch_async / mxopt_engine_settle: the GRPO engine's micro-batch call without its host
synchronisation.  The validity flag stays on the device, the kernels obey it there, and the host books a
skipped micro-batch when it settles -- parameters, counters and flags must be those of the oracle's blocking
restatement of grpo/engine.rs:561-704 at every point, with NaN/Inf micro-batches at the first, a middle and
the applying position of a cycle."""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host
from test_gpu_engine import SIZES, check_state, exact_clamped_sumsq, make_grads, make_params

F = np.float32
SCRIPT = ["nan", "ok", "ok", "inf", "ok", "ok", "ok", "-inf", "nan", "ok", "ok", "ok", "ok", "nan", "ok", "ok"]


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


def poisoned(rng, bf16, it, kind):
    grads = make_grads(rng, bf16, 0.01 * (1 + it % 3))
    if kind != "ok":
        v = O.as_f32(grads["w1"]).copy()
        v[4096 + 5] = {"nan": np.nan, "inf": np.inf, "-inf": -np.inf}[kind]   # +-Inf would be clamped: the raw value counts
        grads["w1"] = O.f32_to_bf16(v) if bf16 else v
    return grads


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("mode", ["sgd", "sgd-deferred", "adamw"])
@pytest.mark.parametrize("n_acc", [1, 3])
def test_async_settled_after_every_micro_batch(mx, tmp_path, bf16, mode, n_acc):
    """Every call is settled before the next: the speculative bookkeeping, the guarded kernels and the
    roll-back are exercised, and the device's own sum of squares can be handed to the oracle (clip active)."""
    rng = np.random.default_rng(41 + n_acc)
    params = make_params(rng, bf16)
    dparams = {k: to_dev(v) for k, v in params.items()}
    defer = mode == "sgd-deferred"
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=n_acc, gradient_clip_norm=2.0, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=2, apply=mode.split("-")[0], weight_decay=0.01)
    dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=defer, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    applied = 0
    for it, kind in enumerate(SCRIPT):
        grads = poisoned(rng, bf16, it, kind)
        dev.micro_batch_async({k: to_dev(g) for k, g in grads.items()})
        m = dev.settle()
        if kind == "ok":
            exact = exact_clamped_sumsq(grads, 0.02)
            assert m.norm_measured and abs(m.grad_norm - math.sqrt(exact)) <= 1e-5 * math.sqrt(exact)
            r = ref.micro_batch(grads, norm_sumsq=m.grad_sumsq)
        else:
            r = ref.micro_batch(grads)
        assert (bool(m.skipped), bool(m.gradients_applied), m.step) == (r["skipped"], r["gradients_applied"], r["step"]), it
        applied += int(r["gradients_applied"])
        check_state(dev, ref, dparams, f"micro-batch {it} ({kind})")
    assert ref.state.nan_gradient_count == 5
    if mode == "adamw":      # the optimizer object's call counter saw only the updates that took place
        import ctypes as C
        path = tmp_path / "state.safetensors"
        dev.save_optimizer_state(path)
        kind, step, tensors, elements = C.create_string_buffer(32), C.c_int64(), C.c_uint64(), C.c_uint64()
        assert mx.load().mxopt_checkpoint_inspect(str(path).encode(), kind, 32, C.byref(step), C.byref(tensors),
                                                  C.byref(elements)) == 0
        assert step.value == applied * len(params)


@pytest.mark.parametrize("mode", ["sgd", "sgd-deferred", "adamw"])
@pytest.mark.parametrize("n_acc", [2, 4])
def test_async_pipelined_never_settled_in_between(mx, mode, n_acc):
    """No settle between the calls: each call books its predecessor's flag itself.  The clip threshold is out
    of reach (factor exactly 1), so the oracle needs no figure from the device and every call can be left
    unsettled; blocking calls and getters mixed in must settle by themselves."""
    rng = np.random.default_rng(43)
    params = make_params(rng, True)
    dparams = {k: to_dev(v) for k, v in params.items()}
    defer = mode == "sgd-deferred"
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=n_acc, gradient_clip_norm=1e9, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=2, apply=mode.split("-")[0], weight_decay=0.01)
    dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=defer, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    keep = []
    for it, kind in enumerate(SCRIPT + SCRIPT):
        grads = poisoned(rng, True, it, kind)
        dg = {k: to_dev(g) for k, g in grads.items()}
        keep.append(dg)                       # the caller's side of the contract: buffers outlive the kernels
        if it % 7 == 6:
            dev.micro_batch(dg)               # a blocking call in between settles what is pending
        else:
            dev.micro_batch_async(dg)
        ref.micro_batch(grads)
        if it % 5 == 4:
            check_state(dev, ref, dparams, f"after micro-batch {it}")     # the getters settle too
    m = dev.settle()
    assert m.step == ref.state.step
    check_state(dev, ref, dparams, "end")


def test_async_training_stopped_surfaces_when_settled(mx):
    params = {"w": np.ones(100, F)}
    dparams = {"w": to_dev(params["w"])}
    dev = mx.GRPOEngineOptimizerSide(dparams, max_nan_gradients=2)
    ref = O.GRPOEngineOptimizerSide(params, max_nan_gradients=2)
    bad = np.zeros(100, F)
    bad[3] = np.nan
    dbad = to_dev(bad)
    dev.micro_batch_async({"w": dbad})
    ref.micro_batch({"w": bad})
    dev.micro_batch_async({"w": dbad})        # settles the first (a skip), enqueues the second: the limit is reached ...
    with pytest.raises(O.TrainingStopped):
        ref.micro_batch({"w": bad})
    with pytest.raises(mx.TrainingStopped, match=r"exceeded maximum NaN gradient count \(2/2\)"):
        dev.settle()                          # ... and reported by the call that settles it
    check_state(dev, ref, dparams, "after the limit")
    assert_bit_equal(to_host(dparams["w"]), params["w"], "nothing was touched")


def test_async_is_refused_where_nothing_blocks(mx):
    dparams = {"w": to_dev(np.ones(100, F))}
    g = {"w": to_dev(np.zeros(100, F))}
    with pytest.raises(mx.InvalidArg, match="only the GRPO engine reads a flag back"):
        mx.SFTEngineOptimizerSide(dparams).micro_batch_async(g)
    dev = mx.GRPOEngineOptimizerSide(dparams)
    assert dev.settle().step == 0             # nothing pending: a no-op


def _inspect_step(mx, path):
    import ctypes as C
    kind, step, tensors, elements = C.create_string_buffer(32), C.c_int64(), C.c_uint64(), C.c_uint64()
    assert mx.load().mxopt_checkpoint_inspect(str(path).encode(), kind, 32, C.byref(step), C.byref(tensors),
                                              C.byref(elements)) == 0
    return step.value


def test_save_and_load_settle_a_pending_micro_batch_first(mx, tmp_path):
    """AdamW apply, one micro-batch per step.  A NaN micro-batch that is still unsettled has advanced the call
    counter speculatively: a checkpoint written then must hold the counter of the updates that took place, and a
    checkpoint loaded then must not be overwritten by the roll-back that follows."""
    rng = np.random.default_rng(47)
    params = make_params(rng, True)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=1, gradient_clip_norm=1e9, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=2, apply="adamw", weight_decay=0.01)
    dev = mx.GRPOEngineOptimizerSide(dparams, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    n = len(params)
    keep = []

    def call(kind, it):
        grads = poisoned(rng, True, it, kind)
        dg = {k: to_dev(g) for k, g in grads.items()}
        keep.append(dg)
        dev.micro_batch_async(dg)
        ref.micro_batch(grads)

    call("ok", 0)
    first = tmp_path / "first.safetensors"
    dev.save_optimizer_state(first)                   # settles the valid call: one update per parameter
    assert _inspect_step(mx, first) == n
    call("ok", 1)
    call("nan", 2)                                    # unsettled; the counter stands at 3n speculatively
    second = tmp_path / "second.safetensors"
    dev.save_optimizer_state(second)
    assert _inspect_step(mx, second) == 2 * n
    check_state(dev, ref, dparams, "after the save")
    call("inf", 3)                                    # unsettled again
    dev.load_optimizer_state(first)                   # the skip is booked first, then the file's counter stands
    third = tmp_path / "third.safetensors"
    dev.save_optimizer_state(third)
    assert _inspect_step(mx, third) == n
    m = dev.metrics()
    assert (m.step, m.nan_gradient_count) == (ref.state.step, ref.state.nan_gradient_count) == (4, 2)


def test_spill_is_not_undone_by_an_invalid_arrival(mx):
    """Deferred accumulation with more micro-batches than streams, asynchronous calls: the arrival that makes the
    two oldest micro-batches move into the float32 buffers holds a NaN.  The move is made whatever that flag says,
    so the caller may reuse those two buffers straight away, as after a blocking call."""
    import torch
    rng = np.random.default_rng(53)
    params = make_params(rng, True)
    dparams = {k: to_dev(v) for k, v in params.items()}
    n_acc = 11
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=n_acc, gradient_clip_norm=1e9, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=3)
    dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=True, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    script = ["ok"] * (mx.MAX_PENDING + 1) + ["nan"] + ["ok"] * (n_acc - mx.MAX_PENDING - 1)
    sent = []
    for it, kind in enumerate(script):
        grads = poisoned(rng, True, it, kind)
        dg = {k: to_dev(g) for k, g in grads.items()}
        sent.append(dg)
        dev.micro_batch_async(dg)
        ref.micro_batch(grads)
        if kind == "nan":
            torch.cuda.synchronize()
            for old in sent[:2]:                      # "free again after that call"
                for t in old.values():
                    t.fill_(float("nan"))
    m = dev.settle()
    assert m.gradients_applied and m.step == ref.state.step
    check_state(dev, ref, dparams, "end of the cycle")


@pytest.mark.parametrize("kind", ["ok", "nan"])
def test_async_call_that_fails_after_its_flag_was_requested(mx, kind):
    """Deferred accumulation refuses a micro-batch whose names differ from the cycle's -- after the norm pass and
    the flag copy were enqueued.  The bookkeeping goes back to where it was; if the refused micro-batch also held
    a NaN it is booked as the skip the blocking call would have returned before it reached that check."""
    rng = np.random.default_rng(59)
    params = make_params(rng, False)
    dparams = {k: to_dev(v) for k, v in params.items()}
    kw = dict(learning_rate=0.05, gradient_accumulation_steps=3, gradient_clip_norm=1e9, gradient_clip_value=0.02,
              max_nan_gradients=50, emergency_save_threshold=3)
    dev = mx.GRPOEngineOptimizerSide(dparams, defer_accumulation=True, **kw)
    ref = O.GRPOEngineOptimizerSide(params, **kw)
    g0 = make_grads(rng, False, 0.01)
    d0 = {k: to_dev(g) for k, g in g0.items()}
    dev.micro_batch_async(d0)
    ref.micro_batch(g0)
    sub = poisoned(rng, False, 1, kind)
    del sub["ln"]
    dsub = {k: to_dev(g) for k, g in sub.items()}
    with pytest.raises(mx.InvalidArg, match="same gradient names"):
        dev.micro_batch_async(dsub)
    if kind == "nan":
        ref.micro_batch(sub)                          # a skip: the raw values are tested before anything else
    check_state(dev, ref, dparams, "after the refused call")
    for it in (2, 3):                                 # the cycle goes on as if the refused call had not been made
        g = make_grads(rng, False, 0.01)
        dg = {k: to_dev(v) for k, v in g.items()}
        d0[f"keep{it}"] = dg
        dev.micro_batch_async(dg)
        ref.micro_batch(g)
    m = dev.settle()
    assert m.gradients_applied
    check_state(dev, ref, dparams, "end of the cycle")
