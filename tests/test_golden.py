"""Committed golden fixtures (tests/golden/):

* reference_kat.json  -- the known-answer values of the reference's own tests, as data;
* oracle_vectors.npz  -- seeded inputs + the oracle's outputs (tests/golden/make_oracle_vectors.py).

CPU tests check the oracle against both (the second freezes it); GPU tests check the library
against both through the C ABI without importing the oracle at all.
"""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KAT = json.load(open(os.path.join(GOLDEN, "reference_kat.json")))
F = np.float32


def close(a, b, digits):
    return abs(float(a) - float(b)) < (10.0 ** -digits) / 2


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(GOLDEN, "oracle_vectors.npz"))


# ---------------------------------------------------------------------------------------
# The implementation under test, behind one small adapter: the oracle (CPU) or the library (GPU)
# ---------------------------------------------------------------------------------------

class OracleImpl:
    def __init__(self):
        import mxopt_oracle as O
        self.O = O
        self.invalid = ValueError

    def tensor(self, a):
        return np.asarray(a)

    def host(self, t):
        return np.asarray(t)

    def optimizer(self, name, args):
        return getattr(self.O, name)(*args)

    def apply_gradients(self, p, g, lr):
        return self.O.apply_gradients({"w": p}, {"w": g}, lr)["w"]

    def __getattr__(self, name):      # GradientUtils, LRScheduler, accumulate_gradients, clip_gradients_by_*
        return getattr(self.O, name)


class GpuImpl:
    def __init__(self):
        import mxopt
        from gpu_util import to_dev, to_host
        self.mx, self.to_dev, self.to_host = mxopt, to_dev, to_host
        self.invalid = ValueError

    def tensor(self, a):
        return self.to_dev(np.asarray(a))

    def host(self, t):
        return self.to_host(t)

    def optimizer(self, name, args):
        return getattr(self.mx, name)(*args)

    def apply_gradients(self, p, g, lr):
        params = {"w": p.clone()}
        self.mx.apply_gradients(params, {"w": g}, lr)
        return params["w"]

    def __getattr__(self, name):
        return getattr(self.mx, name)


def run_kat(impl):
    for case in KAT["optimizer_steps"]:
        cur = None
        if case["optimizer"] == "apply_gradients":
            st = case["steps"][0]
            cur = impl.apply_gradients(impl.tensor(np.array(st["param"], F)), impl.tensor(np.array(st["grad"], F)),
                                       case["args"][0])
        else:
            opt = impl.optimizer(case["optimizer"], case["args"])
            for st in case["steps"]:
                p = cur if st["param"] == "previous" else impl.tensor(np.array(st["param"], F))
                cur = opt.update_single("param", p, impl.tensor(np.array(st["grad"], F)))
        got = impl.host(cur)
        for g, w in zip(got, case["expected"]):
            assert close(g, w, case["digits"]), (case["source"], got)
    for case in KAT["invalid_constructors"]:
        with pytest.raises(impl.invalid):
            impl.optimizer(case["optimizer"], case["args"])
    for case in KAT["clip_grad_value"]:
        got = impl.host(impl.GradientUtils.clip_grad_value(impl.tensor(np.array(case["grad"], F)), case["min"],
                                                           case["max"]))
        assert all(close(g, w, case["digits"]) for g, w in zip(got, case["expected"])), case["source"]
    for case in KAT["gradient_norm"]:
        d = {k: impl.tensor(np.array(v, F)) for k, v in case["gradients"].items()}
        assert close(impl.GradientUtils.compute_gradient_norm(d), case["expected"], case["digits"]), case["source"]
    for case in KAT["clip_grad_norm"]:
        d = {k: impl.tensor(np.array(v, F)) for k, v in case["gradients"].items()}
        if "expected_norm" in case:
            out, norm = impl.GradientUtils.clip_grad_norm_with_norm(d, case["max_norm"])
            assert close(norm, case["expected_norm"], 5), case["source"]
        else:
            out = impl.GradientUtils.clip_grad_norm(d, case["max_norm"])
        assert set(out) == set(case["expected"])
        for k, want in case["expected"].items():
            assert all(close(g, w, case["digits"]) for g, w in zip(impl.host(out[k]), want)), case["source"]
    for case in KAT["lr_schedules"]:
        fn = getattr(impl.LRScheduler, case["fn"])
        for args, want in case["cases"]:
            assert close(fn(*args), want, case["digits"]), (case["source"], args)
    for case in KAT["accumulate_gradients"]:
        acc = {k: impl.tensor(np.array(v, F)) for k, v in case["accumulated"].items()}
        new = {k: impl.tensor(np.array(v, F)) for k, v in case["new"].items()}
        out = impl.accumulate_gradients(acc, new)
        for k, want in case["expected"].items():
            assert np.array_equal(impl.host(out[k]), np.array(want, F)), case["source"]


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)


def same(got, want, what):
    got, want = np.asarray(got), np.asarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, (what, got.dtype, want.dtype)
    assert np.array_equal(bits(got), bits(want)), what


def widen(a):
    """bf16 bit patterns -> float32 (the Vec clip API hands back the input dtype when it does not clip)."""
    a = np.asarray(a)
    return (a.astype(np.uint32) << np.uint32(16)).view(F) if a.dtype == np.uint16 else a


def round_bf16(x):
    u = np.ascontiguousarray(x, F).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


OPTS = {"adam": ("Adam", (1e-3, 0.9, 0.999, 1e-8, False)), "adam_bias": ("Adam", (1e-2, 0.8, 0.99, 1e-8, True)),
        "adamw": ("AdamW", (1e-3, 0.9, 0.999, 1e-8, 0.01, False)),
        "adamw_bias": ("AdamW", (5e-6, 0.9, 0.999, 1e-8, 0.1, True)), "sgd_plain": ("SGD", (0.1,)),
        "sgd_momentum_wd": ("SGD", (1e-2, 0.9, 1e-4)), "sgd_dampening": ("SGD", (1e-2, 0.9, 0.0, 0.25)),
        "sgd_nesterov": ("SGD", (1e-2, 0.9, 1e-4, 0.0, True)), "rmsprop": ("RMSprop", (1e-4, 0.99, 1e-8, 0.0)),
        "rmsprop_wd": ("RMSprop", (1e-2, 0.9, 1e-6, 0.01))}


def run_vectors(impl, vec, exact_scale):
    for name, (cls, args) in OPTS.items():
        for dt in ("f32", "bf16"):
            tag = f"{name}.{dt}"
            opt = impl.optimizer(cls, args)
            cur = impl.tensor(vec[f"{tag}.param"])
            k = 0
            while f"{tag}.grad{k}" in vec:
                g = impl.tensor(vec[f"{tag}.grad{k}"])
                opt.update_single("other", cur, g)
                new = opt.update_single("w", cur, g)
                want = vec[f"{tag}.out{k}"]
                same(impl.host(new), want, f"{tag} step {k}")
                cur = impl.tensor(round_bf16(want)) if dt == "bf16" else new
                k += 1
            assert k == 2
    for dt in ("f32", "bf16"):
        gs = [vec[f"utils.{dt}.g{i}"] for i in range(4)]
        d = {str(i): impl.tensor(g) for i, g in enumerate(gs)}
        norm = float(vec[f"utils.{dt}.norm"][0])
        assert abs(impl.GradientUtils.compute_gradient_norm(d) - norm) <= 1e-5 * norm
        for label in ("clip", "noclip"):
            max_norm = float(vec[f"utils.{dt}.{label}.max_norm"][0])
            out, n32 = impl.GradientUtils.clip_grad_norm_with_norm(d, max_norm)
            assert abs(n32 - float(vec[f"utils.{dt}.{label}.norm32"][0])) <= 1e-5 * norm
            vecs = impl.clip_gradients_by_global_norm(list(d.values()), max_norm)
            for i in range(4):
                got, want = impl.host(out[str(i)]), vec[f"utils.{dt}.{label}.out{i}"]
                gv, wv = widen(impl.host(vecs[i])), vec[f"utils.{dt}.{label}.vec{i}"]
                if exact_scale:
                    same(got, want, f"clip {dt} {label} {i}")
                    same(gv, wv, f"vec {dt} {label} {i}")
                else:   # the device's norm may differ from the exact one in the last float32 place
                    assert np.allclose(got, want, rtol=3e-7, atol=0) and np.allclose(gv, wv, rtol=3e-7, atol=0)
        both = impl.GradientUtils.clip_grad_value_and_norm(d, 5e-3, norm / 4)
        for i in range(4):
            same(impl.host(impl.GradientUtils.clip_grad_value(d[str(i)], -5e-3, 5e-3)), vec[f"utils.{dt}.value.out{i}"],
                 f"value {dt} {i}")
            assert np.allclose(impl.host(both[str(i)]), vec[f"utils.{dt}.value_and_norm.out{i}"], rtol=3e-7, atol=0)
        acc = {}
        for _ in range(3):
            acc = impl.accumulate_gradients(acc, {"w": d["3"]})
        same(impl.host(acc["w"]), vec[f"utils.{dt}.acc_same_dtype"], f"accumulate {dt}")
        same(impl.host(impl.apply_gradients(impl.tensor(vec[f"utils.{dt}.apply.param"]), d["3"], 2e-2)),
             vec[f"utils.{dt}.apply.out"], f"apply {dt}")


# ---- CPU: the oracle against the fixtures ------------------------------------------------

def test_oracle_against_reference_kat():
    run_kat(OracleImpl())


def test_oracle_is_frozen_by_committed_vectors(vec):
    run_vectors(OracleImpl(), vec, exact_scale=True)


# ---- GPU: the library against the fixtures -----------------------------------------------

@pytest.mark.gpu
def test_library_against_reference_kat():
    run_kat(GpuImpl())


@pytest.mark.gpu
def test_library_against_committed_vectors(vec):
    run_vectors(GpuImpl(), vec, exact_scale=False)


@pytest.mark.gpu
def test_float32_accumulation_buffer_against_committed_vectors(vec):
    import torch
    impl = GpuImpl()
    for dt in ("f32", "bf16"):
        acc = impl.mx.GradientAccumulator(dtype=torch.float32)
        g = impl.tensor(vec[f"utils.{dt}.g3"])
        for _ in range(3):
            acc.accumulate({"w": g})
        same(impl.host(acc.take()["w"]), vec[f"utils.{dt}.acc_f32"], f"f32 accumulate {dt}")


# ---- engines' optimizer side: scripted micro-batch sequences (tests/golden/engine_vectors.npz) ----

@pytest.fixture(scope="module")
def engine_vec():
    return np.load(os.path.join(GOLDEN, "engine_vectors.npz"))


def engine_cases():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_oracle_vectors", os.path.join(GOLDEN, "make_oracle_vectors.py"))
    # only the case table is needed; the generator module imports the oracle, which CPU tests may do
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.ENGINE_CASES, mod.ENGINE_SIZES


# the case table, restated so that the GPU half does not import the generator (and with it the oracle)
ENGINE_CASES = {
    "grpo_sgd": ("GRPOEngineOptimizerSide", dict(learning_rate=0.05, gradient_accumulation_steps=2, gradient_clip_norm=0.5,
                                                gradient_clip_value=0.02, emergency_save_threshold=1),
                 ["abc", "abc", "ab", "nan", "bc", "abc"]),
    "grpo_adamw": ("GRPOEngineOptimizerSide", dict(learning_rate=1e-3, gradient_accumulation_steps=3, gradient_clip_norm=None,
                                                  apply="adamw", weight_decay=0.1),
                   ["abc", "abc", "abc", "abc", "nan", "abc", "abc"]),
    "sft_sgd": ("SFTEngineOptimizerSide", dict(learning_rate=0.02, gradient_accumulation_steps=2, gradient_clip_norm=0.3,
                                              gradient_clip_value=0.004, weight_decay=0.01),
                ["abc", "abc", "ab", "abc", "abc", "flush"]),
    "sft_adamw": ("SFTEngineOptimizerSide", dict(learning_rate=1e-3, gradient_accumulation_steps=2, gradient_clip_norm=1.0,
                                                apply="adamw", weight_decay=0.05),
                  ["abc", "abc", "abc", "flush"]),
}


def test_engine_case_table_matches_the_generator():
    cases, _ = engine_cases()
    assert cases == ENGINE_CASES


def close_params(got, want, exact):
    got, want = np.asarray(got), np.asarray(want)
    assert got.dtype == want.dtype
    if exact:
        return np.array_equal(bits(got), bits(want))
    if got.dtype == np.uint16:      # the device's norm may differ in the last float32 place: <= 1 bf16 ulp
        return np.abs(got.astype(np.int32) - want.astype(np.int32)).max() <= 1
    return np.allclose(got, want, rtol=1e-6, atol=1e-9)


def run_engine_vectors(make_engine, tensor, host, vec, exact):
    for case, (cls, kw, script) in ENGINE_CASES.items():
        for dt in ("f32", "bf16"):
            tag = f"{case}.{dt}"
            params = {k: tensor(vec[f"{tag}.param.{k}"]) for k in "abc"}
            eng, live = make_engine(cls, params, kw)
            for i, what in enumerate(script):
                if what == "flush":
                    applied = eng.flush_gradients()
                else:
                    names = "abc" if what == "nan" else what
                    m = eng.micro_batch({k: tensor(vec[f"{tag}.mb{i}.grad.{k}"]) for k in names})
                    applied = m["gradients_applied"] if isinstance(m, dict) else bool(m.gradients_applied)
                st = vec[f"{tag}.mb{i}.state"]
                assert (eng.step, eng.micro_step, eng.nan_gradient_count, int(eng.needs_emergency_save),
                        int(applied)) == (st[0], st[1], st[2], st[4], st[5]), (tag, i)
                for k in "abc":
                    assert close_params(host(live(eng)[k]), vec[f"{tag}.mb{i}.param.{k}"], exact), (tag, i, k)


def test_oracle_engines_are_frozen_by_committed_vectors(engine_vec):
    import mxopt_oracle as O
    run_engine_vectors(lambda cls, params, kw: (getattr(O, cls)(params, **kw), lambda e: e.params),
                       np.asarray, np.asarray, engine_vec, exact=True)


@pytest.mark.gpu
def test_library_engines_against_committed_vectors(engine_vec):
    impl = GpuImpl()

    def make(cls, params, kw):
        eng = getattr(impl.mx, cls)(params, **kw)
        return eng, lambda e: params          # updated in place

    run_engine_vectors(make, impl.tensor, impl.host, engine_vec, exact=False)
