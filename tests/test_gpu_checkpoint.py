"""Optimizer-state checkpoints (mxopt_optimizer_save_file / load_file): the file is a standard
safetensors file (read back here with the `safetensors` package, a library that is neither this
build nor the reference), and a run resumed from it continues bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
SIZES = {"model.embed": 5003, "layers.0.w": 4096, "odd \"name\"\\x": 7}


@pytest.fixture(scope="module")
def mx():
    import mxopt
    return mxopt


def run_steps(opt, params, rng, steps):
    for _ in range(steps):
        for name in params:
            g = rng.normal(0, 1e-2, params[name].numel()).astype(F)
            opt.update_single(name, params[name], to_dev(g), out=params[name])


@pytest.mark.parametrize("kind", ["adamw_bias", "adam", "sgd", "rmsprop"])
def test_save_resume_is_bit_identical(mx, tmp_path, kind):
    from safetensors import safe_open
    make = {"adamw_bias": lambda: mx.AdamW(1e-2, 0.9, 0.99, 1e-8, 0.01, True), "adam": lambda: mx.Adam(1e-2),
            "sgd": lambda: mx.SGD(1e-2, 0.9, 1e-4), "rmsprop": lambda: mx.RMSprop(1e-3, 0.9)}[kind]
    rng0 = np.random.default_rng(5)
    init = {k: rng0.normal(0, 0.1, n).astype(F) for k, n in SIZES.items()}

    # uninterrupted: 2 + 2 steps
    a = {k: to_dev(v) for k, v in init.items()}
    opt_a = make()
    rng = np.random.default_rng(6)
    run_steps(opt_a, a, rng, 2)
    path = tmp_path / "opt.safetensors"
    opt_a.save_file(path)
    mid = {k: v.clone() for k, v in a.items()}
    run_steps(opt_a, a, rng, 2)

    # the file, read by the safetensors package
    with safe_open(str(path), framework="np") as f:
        meta = f.metadata()
        keys = set(f.keys())
        assert meta["format"] == "mxopt-optimizer-state" and meta["optimizer"] == kind.split("_")[0]
        assert int(meta["step"]) == (2 * len(SIZES) if kind.startswith("adam") else 0)
        want_keys = {f"{k}.v" for k in SIZES} | ({f"{k}.m" for k in SIZES} if kind.startswith("adam") else set())
        assert keys == want_keys
        for k, n in SIZES.items():
            assert f.get_tensor(f"{k}.v").shape == (n,) and f.get_tensor(f"{k}.v").dtype == np.float32

    # resumed: a fresh optimizer, the parameters as they were at the checkpoint, the same 2 further steps
    opt_b = make()
    opt_b.load_file(path)
    assert opt_b.step == (opt_a.step - 2 * len(SIZES) if kind.startswith("adam") else 0)
    b = {k: v.clone() for k, v in mid.items()}
    rng_b = np.random.default_rng(6)
    # replay the generator to where the checkpoint was taken
    for _ in range(2):
        for name in SIZES:
            rng_b.normal(0, 1e-2, SIZES[name])
    run_steps(opt_b, b, rng_b, 2)
    for k in SIZES:
        assert_bit_equal(to_host(b[k]), to_host(a[k]), f"{kind}: {k}")
        ma, va = opt_a.state(k)
        mb, vb = opt_b.state(k)
        assert_bit_equal(to_host(vb), to_host(va), f"{kind}: v of {k}")
        if ma is not None:
            assert_bit_equal(to_host(mb), to_host(ma), f"{kind}: m of {k}")


def test_reads_a_file_written_by_the_safetensors_package(mx, tmp_path):
    from safetensors.numpy import save_file
    rng = np.random.default_rng(9)
    m = rng.normal(0, 1e-3, 1000).astype(F)
    v = (rng.normal(0, 1e-3, 1000).astype(F)) ** 2
    path = tmp_path / "external.safetensors"
    save_file({"w.m": m, "w.v": v}, str(path), metadata={"format": "mxopt-optimizer-state", "optimizer": "adamw",
                                                          "step": "41"})
    opt = mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
    opt.load_file(path)
    assert opt.step == 41
    p = rng.normal(0, 1, 1000).astype(F)
    g = rng.normal(0, 1e-2, 1000).astype(F)
    got = opt.update_single("w", to_dev(p), to_dev(g))
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
    ref.state["w"] = (m.copy(), v.copy())
    ref.step = 41
    assert_bit_equal(to_host(got), ref.update_single("w", p, g), "first step after loading")


def test_refusals(mx, tmp_path):
    opt = mx.AdamW()
    opt.update_single("w", to_dev(np.ones(10, F)), to_dev(np.ones(10, F)))
    path = tmp_path / "a.safetensors"
    opt.save_file(path)
    with pytest.raises(ValueError, match="checkpoint is for optimizer 'adamw'"):
        mx.SGD(0.1, 0.9).load_file(path)
    with pytest.raises(mx.MxoptError, match="cannot open"):
        opt.load_file(tmp_path / "missing.safetensors")
    data = path.read_bytes()
    (tmp_path / "cut.safetensors").write_bytes(data[:-8])
    with pytest.raises(mx.MxoptError, match="outside the file|truncated"):
        mx.AdamW().load_file(tmp_path / "cut.safetensors")
    (tmp_path / "junk.safetensors").write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{not json.......")
    with pytest.raises(mx.MxoptError):
        mx.AdamW().load_file(tmp_path / "junk.safetensors")
    from safetensors.numpy import save_file
    save_file({"w": np.ones(3, F)}, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="not an optimizer-state checkpoint"):
        mx.AdamW().load_file(tmp_path / "model.safetensors")
    # a failed load leaves an empty optimizer, not a half-filled one
    fresh = mx.AdamW()
    with pytest.raises(mx.MxoptError):
        fresh.load_file(tmp_path / "cut.safetensors")
    assert fresh.state("w") == (None, None)


def test_engine_with_adamw_resumes_from_its_optimizer_state(mx, tmp_path):
    rng = np.random.default_rng(12)
    init = {k: O.f32_to_bf16(rng.normal(0, 0.1, n).astype(F)) for k, n in SIZES.items()}
    grads = [{k: O.f32_to_bf16(rng.normal(0, 1e-2, n).astype(F)) for k, n in SIZES.items()} for _ in range(4)]
    kw = dict(learning_rate=1e-2, gradient_accumulation_steps=1, apply="adamw", weight_decay=0.01)
    a = {k: to_dev(v) for k, v in init.items()}
    ea = mx.GRPOEngineOptimizerSide(a, **kw)
    for g in grads[:2]:
        ea.micro_batch({k: to_dev(v) for k, v in g.items()})
    ea.save_optimizer_state(tmp_path / "engine.safetensors")
    b = {k: v.clone() for k, v in a.items()}
    for g in grads[2:]:
        ea.micro_batch({k: to_dev(v) for k, v in g.items()})
    eb = mx.GRPOEngineOptimizerSide(b, **kw)
    eb.load_optimizer_state(tmp_path / "engine.safetensors")
    for g in grads[2:]:
        eb.micro_batch({k: to_dev(v) for k, v in g.items()})
    for k in SIZES:
        assert_bit_equal(to_host(b[k]), to_host(a[k]), k)
    with pytest.raises(ValueError, match="plain SGD"):
        mx.GRPOEngineOptimizerSide(b).save_optimizer_state(tmp_path / "none.safetensors")
