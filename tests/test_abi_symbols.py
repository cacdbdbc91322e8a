"""CPU-only checks of the drop-in boundary: the shared library loads without a GPU, exports every
function the public headers declare, the ctypes structs have the C layout, and the host-only
entry points (hyper-parameter casts, LR schedules, constructor validation) behave like the
reference.  No kernel is launched here."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "mlx-node_amd"))

import mxopt_oracle as O

HEADERS = [os.path.join(ROOT, "include", h) for h in ("mxopt.h", "mxopt_optimizers.h", "mxopt_engine.h", "mxopt_diagnostics.h")]


@pytest.fixture(scope="module")
def L():
    from mxopt import _lib
    _lib.load()
    return _lib


def declared_functions():
    names = []
    for h in HEADERS:
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names += re.findall(r"\b(mxopt_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_every_declared_symbol_is_exported_and_bound(L):
    lib = L.load()
    names = declared_functions()
    assert len(names) > 40
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/ but not exported by libmxopt.so"
        assert n in L.SIGNATURES, f"{n} has no ctypes signature"
    assert set(L.SIGNATURES) <= set(names)


def test_ctypes_structs_match_c_layout(L, tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "mxopt_engine.h"
#include "mxopt_diagnostics.h"
#define S(T) printf(#T " %zu\n", sizeof(T))
#define F(T, f) printf(#T "." #f " %zu\n", offsetof(T, f))
#define V(name) printf("=" #name " %ld\n", (long)(name))
int main(void) {
  S(mxopt_tensor); F(mxopt_tensor, n); F(mxopt_tensor, p_dtype); F(mxopt_tensor, flags); F(mxopt_tensor, bc2);
  S(mxopt_norm_result); F(mxopt_norm_result, norm_f32); F(mxopt_norm_result, scale); F(mxopt_norm_result, nonfinite);
  S(mxopt_grad_prep); F(mxopt_grad_prep, d_scale); F(mxopt_grad_prep, post_hi);
  S(mxopt_adam_hp); F(mxopt_adam_hp, decoupled_decay);
  S(mxopt_sgd_hp); F(mxopt_sgd_hp, nesterov);
  S(mxopt_rmsprop_hp); F(mxopt_rmsprop_hp, has_weight_decay);
  S(mxopt_array); F(mxopt_array, dtype);
  S(mxopt_engine_config); F(mxopt_engine_config, gradient_clip_norm); F(mxopt_engine_config, max_nan_gradients);
  F(mxopt_engine_config, apply); F(mxopt_engine_config, eps); F(mxopt_engine_config, accumulate_in_f32); F(mxopt_engine_config, defer_accumulation);
  S(mxopt_engine_metrics); F(mxopt_engine_metrics, nan_gradient_count); F(mxopt_engine_metrics, clip_scale);
  F(mxopt_engine_metrics, grad_norm);
  V(MXOPT_OK); V(MXOPT_ERR_INVALID_ARG); V(MXOPT_ERR_FAILURE); V(MXOPT_ERR_HIP); V(MXOPT_ERR_OOM);
  V(MXOPT_TF_FIRST); V(MXOPT_CHUNK_ELEMS); V(MXOPT_MAX_PENDING); V(MXOPT_CLIP_ALWAYS_MULTIPLY); V(MXOPT_CLIP_IF_ABOVE);
  V(MXOPT_SYNTH_NORMAL); V(MXOPT_SYNTH_NORMAL_OUTLIERS); V(MXOPT_SYNTH_UNIFORM);
  V(MXOPT_ENGINE_GRPO); V(MXOPT_ENGINE_SFT); V(MXOPT_ENGINE_APPLY_SGD); V(MXOPT_ENGINE_APPLY_ADAMW);
  V(MXOPT_F32); V(MXOPT_F16); V(MXOPT_BF16);
  V(MXOPT_PROBE_READ); V(MXOPT_PROBE_WRITE); V(MXOPT_PROBE_COPY); V(MXOPT_PROBE_MIX43); V(MXOPT_PROBE_STREAMING);
  V(MXOPT_HBM_INTERLEAVED); V(MXOPT_HBM_ONE_REGION);
  return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    want = dict(line.rsplit(" ", 1) for line in subprocess.check_output([str(exe)], text=True).splitlines())
    py = {"mxopt_tensor": L.Tensor, "mxopt_norm_result": L.NormResult, "mxopt_grad_prep": L.GradPrep,
          "mxopt_adam_hp": L.AdamHp, "mxopt_sgd_hp": L.SgdHp, "mxopt_rmsprop_hp": L.RmspropHp, "mxopt_array": L.Array,
          "mxopt_engine_config": L.EngineConfig, "mxopt_engine_metrics": L.EngineMetrics}
    for key, val in want.items():
        if key.startswith("="):     # a constant: the ctypes module carries it without the MXOPT_ prefix
            assert getattr(L, key[len("=MXOPT_"):]) == int(val), key
        elif "." in key:
            t, f = key.split(".")
            assert getattr(py[t], f).offset == int(val), key
        else:
            assert C.sizeof(py[key]) == int(val), key


def test_hyper_parameters_are_f64_then_f32(L):
    """Coefficients cross the boundary as static_cast<float>(float64 expression) (mlx.cpp:531-535)."""
    lib = L.load()
    hp = L.AdamHp()
    lib.mxopt_adam_hp_from_f64(1e-3, 0.9, 0.999, 1e-8, 0.01, 1, C.byref(hp))
    f = lambda x: float(np.float32(np.float64(x)))
    assert hp.one_minus_beta2 == f(1.0 - 0.999) != float(np.float32(1.0) - np.float32(0.999))
    assert hp.one_minus_beta1 == f(1.0 - 0.9) and hp.decay == f(1.0 - 1e-3 * 0.01) and hp.eps == f(1e-8)
    assert hp.decoupled_decay == 1
    a, b = C.c_float(), C.c_float()
    for t in (1, 2, 7, 311, 100000):
        lib.mxopt_bias_correction(0.9, 0.999, t, C.byref(a), C.byref(b))
        assert a.value == f(1.0 / (1.0 - 0.9 ** t)) and b.value == f(1.0 / (1.0 - 0.999 ** t))
    s = L.SgdHp()
    assert lib.mxopt_sgd_hp_from_f64(0.1, 0.9, 1e-4, 0.25, 0, C.byref(s)) == 0
    assert s.one_minus_dampening == f(1.0 - 0.25) and s.has_momentum == 1 and s.has_weight_decay == 1
    assert lib.mxopt_sgd_hp_from_f64(0.1, 0.0, 0.0, 0.0, 1, C.byref(s)) == L.ERR_INVALID_ARG
    assert b"Nesterov" in lib.mxopt_last_error(None)


def test_lr_schedules_equal_the_oracle(L):
    lib = L.load()
    for args in ((1.0, 0.1, 0, 100), (1.0, 0.1, 50, 100), (1.0, 0.1, 250, 100), (3e-4, 1e-6, 19, 10), (2.0, 0.5, 9, 10)):
        assert lib.mxopt_lr_linear_decay(*args) == O.LRScheduler.linear_decay(*args)
        assert lib.mxopt_lr_cosine_annealing(*args) == O.LRScheduler.cosine_annealing(*args)
        assert lib.mxopt_lr_exponential_decay(*args) == O.LRScheduler.exponential_decay(*args)
        assert abs(lib.mxopt_lr_step_decay(*args) - O.LRScheduler.step_decay(*args)) <= 1e-15


def test_no_gpu_means_a_loud_error_not_a_fallback(L):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    import mxopt
    with pytest.raises(mxopt.MxoptError, match="no CPU path"):
        mxopt.Context()
    handle = C.c_void_p()
    assert L.load().mxopt_create(0, None, C.byref(handle)) != 0     # the C ABI refuses as well
    assert handle.value is None


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "mlx-node_amd")
    for dirpath, _, files in os.walk(pkg):
        for fn in files:
            if fn.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, fn), errors="replace").read()
                assert "oracle" not in text.lower(), f"{fn} mentions the oracle"


def test_tensor_layout_head_and_chunk_count(L):
    """Host logic of the table builder: the common head that aligns every stream, the chunk count,
    and the per-element fallback when the streams disagree (pointers are never dereferenced)."""
    lib = L.load()
    BASE = 0x7f0000000000

    def layout(n, p=None, g=None, m=None, v=None, p_dt=L.BF16, g_dt=L.BF16):
        t = L.Tensor(p=p, p_out=p, g=g, g_out=None, m=m, v=v, n=n, p_dtype=p_dt, p_out_dtype=p_dt, g_dtype=g_dt,
                     g_out_dtype=0, flags=0, bc1=1.0, bc2=1.0)
        head, vec, nc = C.c_uint32(), C.c_int(), C.c_uint64()
        assert lib.mxopt_tensor_layout(C.byref(t), C.byref(head), C.byref(vec), C.byref(nc)) == 0
        return head.value, vec.value, nc.value

    assert layout(4096, p=BASE, g=BASE + 4096 * 2, m=BASE + 65536, v=BASE + 131072) == (0, 1, 1)
    assert layout(4097, p=BASE, g=BASE) == (0, 1, 2)
    assert layout(0, p=BASE + 2, g=BASE + 2) == (7, 1, 0)
    # the same element offset k into packed bf16 and float32 slabs: head = (8 - k) % 8
    for k in range(1, 16):
        h = (8 - k) % 8
        got = layout(10000, p=BASE + 2 * k, g=BASE + (1 << 20) + 2 * k, m=BASE + (2 << 20) + 4 * k,
                     v=BASE + (3 << 20) + 4 * k)
        assert got == (h, 1, (10000 - h + 4095) // 4096), (k, got)
    # float32 only: the smallest head is k-dependent modulo 4
    assert layout(100, p=BASE + 4, g=BASE + 20, p_dt=L.F32, g_dt=L.F32) == (3, 1, 1)
    # fewer elements than the head: one entry, all of it head
    assert layout(3, p=BASE + 2, g=BASE + 2) == (7, 1, 1)
    assert layout(7 + 4096, p=BASE + 2, g=BASE + 2) == (7, 1, 1)
    assert layout(7 + 4097, p=BASE + 2, g=BASE + 2) == (7, 1, 2)
    # streams that disagree: bf16 p one element in, float32 m on a boundary
    assert layout(5000, p=BASE + 2, g=BASE + 2, m=BASE + 65536, v=BASE + 131072) == (0, 0, 2)
    assert lib.mxopt_tensor_layout(None, None, None, None) == 1


def test_engine_config_defaults_are_the_reference_defaults(L):
    """GRPOEngineConfig::default (grpo/engine.rs:114-141) and SftEngineConfig::default (sft/engine.rs:50-66)."""
    lib = L.load()
    g, s = L.EngineConfig(), L.EngineConfig()
    lib.mxopt_engine_config_default(L.ENGINE_GRPO, C.byref(g))
    lib.mxopt_engine_config_default(L.ENGINE_SFT, C.byref(s))
    assert (g.learning_rate, g.gradient_accumulation_steps, g.has_gradient_clip_norm, g.gradient_clip_norm,
            g.has_gradient_clip_value, g.gradient_clip_value, g.max_nan_gradients, g.emergency_save_threshold,
            g.apply) == (1e-6, 1, 1, 1.0, 1, 1.0, 100, 5, L.ENGINE_APPLY_SGD)
    assert (s.learning_rate, s.gradient_accumulation_steps, s.has_gradient_clip_norm, s.gradient_clip_norm,
            s.has_gradient_clip_value, s.weight_decay, s.max_nan_gradients, s.emergency_save_threshold,
            s.apply) == (2e-5, 1, 1, 1.0, 0, 0.01, 100, 5, L.ENGINE_APPLY_SGD)
    # entry points refuse a null engine without touching a device
    assert lib.mxopt_engine_micro_batch(None, 0, None, None, None) == 1
    assert lib.mxopt_engine_reset(None) == 1 and lib.mxopt_optimizer_save_file(None, b"/tmp/x") == 1
