#!/usr/bin/env python3
"""Writes tests/golden/oracle_vectors.npz: small seeded inputs and the CPU oracle's outputs for
every optimizer and utility of the path, float32 and bf16 (bf16 as uint16 bit patterns), and
tests/golden/engine_vectors.npz: scripted micro-batch sequences through the oracle's restatement
of the two training engines' optimizer side (parameters and counters after every micro-batch).

The vectors freeze the oracle (a later edit that changes a result fails tests/test_golden.py)
and let the GPU tests check the HIP path against committed data without importing the oracle.
The reference itself cannot be run (Rust + MLX are absent), so these are the oracle's numbers,
pinned by tests/test_oracle_kat.py and tests/test_oracle_library.py; re-run after a deliberate
oracle change:  python tests/golden/make_oracle_vectors.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "oracle"))
import mxopt_oracle as O  # noqa: E402

F = np.float32
N = 261          # not a multiple of the 8-element vector group
STEPS = 2

CASES = {
    # name: (factory taking the module, constructor args)
    "adam": ("Adam", (1e-3, 0.9, 0.999, 1e-8, False)),
    "adam_bias": ("Adam", (1e-2, 0.8, 0.99, 1e-8, True)),
    "adamw": ("AdamW", (1e-3, 0.9, 0.999, 1e-8, 0.01, False)),
    "adamw_bias": ("AdamW", (5e-6, 0.9, 0.999, 1e-8, 0.1, True)),
    "sgd_plain": ("SGD", (0.1,)),
    "sgd_momentum_wd": ("SGD", (1e-2, 0.9, 1e-4)),
    "sgd_dampening": ("SGD", (1e-2, 0.9, 0.0, 0.25)),
    "sgd_nesterov": ("SGD", (1e-2, 0.9, 1e-4, 0.0, True)),
    "rmsprop": ("RMSprop", (1e-4, 0.99, 1e-8, 0.0)),
    "rmsprop_wd": ("RMSprop", (1e-2, 0.9, 1e-6, 0.01)),
}


def inputs(seed, bf16):
    rng = np.random.default_rng(seed)
    p = rng.normal(0, 0.02, N).astype(F)
    gs = []
    for _ in range(STEPS):
        g = rng.normal(0, 1e-3, N).astype(F)
        g[rng.random(N) < 0.02] *= 100
        gs.append(g)
    if bf16:
        p, gs = O.f32_to_bf16(p), [O.f32_to_bf16(g) for g in gs]
    return p, gs


def main():
    out = {}
    for ci, (name, (cls, args)) in enumerate(sorted(CASES.items())):
        for bf16 in (False, True):
            tag = f"{name}.{'bf16' if bf16 else 'f32'}"
            p, gs = inputs(1000 + ci, bf16)
            out[f"{tag}.param"] = p
            opt = getattr(O, cls)(*args)
            cur = p
            for k, g in enumerate(gs):
                out[f"{tag}.grad{k}"] = g
                # two tensors share the optimizer so that the per-call step counter matters
                opt.update_single("other", cur, g)
                new = opt.update_single("w", cur, g)
                out[f"{tag}.out{k}"] = new                       # float32, as the reference returns
                st = opt.state["w"]
                if isinstance(st, tuple):
                    out[f"{tag}.m{k}"], out[f"{tag}.v{k}"] = st
                elif st is not None:
                    out[f"{tag}.v{k}"] = st
                cur = O.f32_to_bf16(new) if bf16 else new
    # gradient utilities on a ragged list
    rng = np.random.default_rng(77)
    sizes = [1, 9, 100, N]
    for bf16 in (False, True):
        tag = "bf16" if bf16 else "f32"
        gs = [rng.normal(0, 1e-2, n).astype(F) for n in sizes]
        if bf16:
            gs = [O.f32_to_bf16(g) for g in gs]
        d = {str(i): g for i, g in enumerate(gs)}
        norm = O.GradientUtils.compute_gradient_norm(d)
        out[f"utils.{tag}.norm"] = np.array([norm])
        for i, g in enumerate(gs):
            out[f"utils.{tag}.g{i}"] = g
        for label, max_norm in (("clip", norm / 4), ("noclip", norm * 4)):
            clipped, n32 = O.GradientUtils.clip_grad_norm_with_norm(d, max_norm)
            vec = O.clip_gradients_by_global_norm(gs, max_norm)
            out[f"utils.{tag}.{label}.max_norm"] = np.array([max_norm])
            out[f"utils.{tag}.{label}.norm32"] = np.array([n32])
            for i in range(len(gs)):
                out[f"utils.{tag}.{label}.out{i}"] = clipped[str(i)]
                out[f"utils.{tag}.{label}.vec{i}"] = O.as_f32(vec[i])
        both = O.GradientUtils.clip_grad_value_and_norm(d, 5e-3, norm / 4)
        for i in range(len(gs)):
            out[f"utils.{tag}.value.out{i}"] = O.clip_value(gs[i], -5e-3, 5e-3)
            out[f"utils.{tag}.value_and_norm.out{i}"] = both[str(i)]
        acc = None
        acc16 = {}
        for k in range(3):
            acc = O.accumulate_fp32(acc, gs[3])
            acc16 = O.accumulate_gradients(acc16, {"w": gs[3]})
        out[f"utils.{tag}.acc_f32"] = acc
        out[f"utils.{tag}.acc_same_dtype"] = acc16["w"]
        p = O.f32_to_bf16(rng.normal(0, 0.02, N).astype(F)) if bf16 else rng.normal(0, 0.02, N).astype(F)
        out[f"utils.{tag}.apply.param"] = p
        out[f"utils.{tag}.apply.out"] = O.apply_gradients({"w": p}, {"w": gs[3]}, 2e-2)["w"]
    np.savez_compressed(os.path.join(HERE, "oracle_vectors.npz"), **out)
    print(f"wrote {len(out)} arrays")
    eng = engine_vectors()
    np.savez_compressed(os.path.join(HERE, "engine_vectors.npz"), **eng)
    print(f"wrote {len(eng)} engine arrays")


ENGINE_SIZES = {"a": 261, "b": 70, "c": 517}
ENGINE_CASES = {
    # name: (oracle class, keyword arguments, script: which names each micro-batch carries / "nan" / "flush")
    "grpo_sgd": ("GRPOEngineOptimizerSide",
                 dict(learning_rate=0.05, gradient_accumulation_steps=2, gradient_clip_norm=0.5,
                      gradient_clip_value=0.02, emergency_save_threshold=1),
                 ["abc", "abc", "ab", "nan", "bc", "abc"]),
    "grpo_adamw": ("GRPOEngineOptimizerSide",
                   dict(learning_rate=1e-3, gradient_accumulation_steps=3, gradient_clip_norm=None, apply="adamw",
                        weight_decay=0.1),
                   ["abc", "abc", "abc", "abc", "nan", "abc", "abc"]),
    "sft_sgd": ("SFTEngineOptimizerSide",
                dict(learning_rate=0.02, gradient_accumulation_steps=2, gradient_clip_norm=0.3,
                     gradient_clip_value=0.004, weight_decay=0.01),
                ["abc", "abc", "ab", "abc", "abc", "flush"]),
    "sft_adamw": ("SFTEngineOptimizerSide",
                  dict(learning_rate=1e-3, gradient_accumulation_steps=2, gradient_clip_norm=1.0, apply="adamw",
                       weight_decay=0.05),
                  ["abc", "abc", "abc", "flush"]),
}


def engine_vectors():
    out = {}
    for case, (cls, kw, script) in ENGINE_CASES.items():
        for bf16 in (False, True):
            tag = f"{case}.{'bf16' if bf16 else 'f32'}"
            rng = np.random.default_rng(sum(map(ord, tag)))
            cast = O.f32_to_bf16 if bf16 else (lambda x: x)
            params = {k: cast(rng.normal(0, 0.5, n).astype(F)) for k, n in ENGINE_SIZES.items()}
            for k, v in params.items():
                out[f"{tag}.param.{k}"] = v
            eng = getattr(O, cls)(params, **kw)
            for i, what in enumerate(script):
                if what == "flush":
                    applied = eng.flush_gradients()
                else:
                    names = "abc" if what == "nan" else what
                    grads = {k: rng.normal(0, 0.01, ENGINE_SIZES[k]).astype(F) for k in names}
                    if what == "nan":
                        grads["b"][7] = np.inf
                    grads = {k: cast(g) for k, g in grads.items()}
                    for k, g in grads.items():
                        out[f"{tag}.mb{i}.grad.{k}"] = g
                    applied = eng.micro_batch(grads)["gradients_applied"]
                st = eng.state
                out[f"{tag}.mb{i}.state"] = np.array([st.step, st.micro_step, st.nan_gradient_count,
                                                      st.consecutive_nan_count, int(st.needs_emergency_save),
                                                      int(applied)], np.int64)
                for k in ENGINE_SIZES:
                    out[f"{tag}.mb{i}.param.{k}"] = eng.params[k]
    return out


if __name__ == "__main__":
    main()
