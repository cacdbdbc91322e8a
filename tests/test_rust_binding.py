"""The generated Rust declarations (mlx-node_amd/bindings/mxopt_sys.rs) are in step with the headers: the
committed file is what the generator writes today, every function the headers declare is there with the
same number of parameters as its ctypes signature, and every struct has the fields of its ctypes twin in
the same order.  (Nothing compiles Rust here; this keeps the file honest against the C side.)"""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEN = os.path.join(ROOT, "mlx-node_amd", "bindings", "gen_rust_sys.py")
RS = os.path.join(ROOT, "mlx-node_amd", "bindings", "mxopt_sys.rs")
sys.path.insert(0, os.path.join(ROOT, "mlx-node_amd"))


def test_committed_file_is_up_to_date():
    r = subprocess.run([sys.executable, GEN, "--check"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr


def test_functions_and_structs_match_the_ctypes_side():
    from mxopt import _lib as L
    text = open(RS).read()
    fns = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (mxopt_\w+)\((.*?)\)(?: -> [^;]+)?;", text)}
    # the diagnostics header (probes, data generator, the pool scan on synthetic rates) gets no Rust declarations
    diag = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "mxopt_diagnostics.h")).read(), flags=re.S)
    diagnostics = set(re.findall(r"\b(mxopt_[a-z0-9_]+)\s*\(", diag))
    assert diagnostics and diagnostics < set(L.SIGNATURES)
    assert set(fns) == set(L.SIGNATURES) - diagnostics, set(fns) ^ (set(L.SIGNATURES) - diagnostics)
    for name, params in fns.items():
        n_rust = 0 if not params.strip() else len(params.split(", "))
        assert n_rust == len(L.SIGNATURES[name][1]), name
    twins = {"mxopt_tensor": L.Tensor, "mxopt_norm_result": L.NormResult, "mxopt_grad_prep": L.GradPrep,
             "mxopt_adam_hp": L.AdamHp, "mxopt_sgd_hp": L.SgdHp, "mxopt_rmsprop_hp": L.RmspropHp,
             "mxopt_array": L.Array, "mxopt_engine_config": L.EngineConfig, "mxopt_engine_metrics": L.EngineMetrics}
    for name, ct in twins.items():
        body = re.search(r"pub struct %s \{(.*?)\n\}" % name, text, flags=re.S).group(1)
        fields = [f.replace("r#", "") for f in re.findall(r"pub (\S+):", body)]
        assert fields == [f[0] for f in ct._fields_], name


def test_pointer_types_are_translated_with_their_constness():
    sys.path.insert(0, os.path.dirname(GEN))
    import gen_rust_sys as G
    opaque, structs = {"mxopt_ctx"}, {"mxopt_array"}
    cases = {"const char* const*": "*const *const c_char", "const float* const*": "*const *const f32",
             "mxopt_ctx**": "*mut *mut mxopt_ctx", "const mxopt_ctx*": "*const mxopt_ctx", "void*": "*mut c_void",
             "const void* const*": "*const *const c_void", "float**": "*mut *mut f32", "uint64_t": "u64",
             "const mxopt_array*": "*const mxopt_array", "unsigned long long": "u64", "size_t": "usize",
             "const double*": "*const f64", "int64_t*": "*mut i64", "char*": "*mut c_char"}
    for c, want in cases.items():
        assert G.rust_type(c, opaque, structs) == want, c
