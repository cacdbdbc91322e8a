"""ctypes binding of oracle/mxopt_oracle.c (TEST INFRASTRUCTURE ONLY: imported by tests,
the smoke check and the benchmark's CPU-baseline leg, never by the product package)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")

DT_F32, DT_BF16 = 0, 3


class AdamArgs(C.Structure):
    _fields_ = [(n, C.c_float) for n in
                ("lr", "beta1", "beta2", "omb1", "omb2", "eps", "decay", "bc1", "bc2")] + [
        ("decoupled_decay", C.c_int), ("has_scale", C.c_int), ("scale", C.c_float),
        ("bias_correction", C.c_int)]


class SgdArgs(C.Structure):
    _fields_ = [("lr", C.c_float), ("momentum", C.c_float), ("one_minus_damp", C.c_float),
                ("wd", C.c_float), ("has_wd", C.c_int), ("has_momentum", C.c_int),
                ("nesterov", C.c_int), ("first", C.c_int)]


class RmspropArgs(C.Structure):
    _fields_ = [("lr", C.c_float), ("alpha", C.c_float), ("one_minus_alpha", C.c_float),
                ("eps", C.c_float), ("wd", C.c_float), ("has_wd", C.c_int)]


def build(force: bool = False) -> str:
    src = os.path.join(HERE, "mxopt_oracle.c")
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return LIB


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _dt(a: np.ndarray) -> int:
    if a.dtype == np.float32:
        return DT_F32
    if a.dtype == np.uint16:
        return DT_BF16
    raise TypeError(a.dtype)


class OracleC:
    def __init__(self, lib):
        self.lib = lib
        lib.oracle_sumsq.restype = C.c_double
        lib.oracle_sumsq.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        lib.oracle_num_threads.restype = C.c_int
        for name in ("oracle_adam_unfused", "oracle_adam_fused"):
            f = getattr(lib, name)
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p,
                          C.c_void_p, C.c_size_t, C.POINTER(AdamArgs)]
        lib.oracle_adam_unfused.restype = C.c_int
        lib.oracle_adam_fused.restype = None
        for name, T in (("oracle_sgd_unfused", SgdArgs), ("oracle_sgd_fused", SgdArgs),
                        ("oracle_rmsprop_unfused", RmspropArgs), ("oracle_rmsprop_fused", RmspropArgs)):
            f = getattr(lib, name)
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(T)]
            f.restype = C.c_int if name.endswith("unfused") else None
        lib.oracle_accumulate_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_int]
        lib.oracle_accumulate_f32.restype = None
        lib.oracle_scale_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_float]
        lib.oracle_scale_f32.restype = None
        lib.oracle_fill_synthetic.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_uint64, C.c_uint64, C.c_int,
                                              C.c_double, C.c_double]
        lib.oracle_fill_synthetic.restype = None
        lib.oracle_f32_to_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        lib.oracle_bf16_to_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]

    def num_threads(self) -> int:
        return self.lib.oracle_num_threads()

    def sumsq(self, g: np.ndarray) -> float:
        return self.lib.oracle_sumsq(_ptr(g), _dt(g), g.size)

    def f32_to_bf16(self, x: np.ndarray) -> np.ndarray:
        out = np.empty(x.shape, np.uint16)
        self.lib.oracle_f32_to_bf16(_ptr(x), _ptr(out), x.size)
        return out

    def fill_synthetic(self, n: int, dtype: str, seed: int, distribution: int = 0, a: float = 1.0, b: float = 0.0,
                       first_index: int = 0) -> np.ndarray:
        out = np.empty(n, np.uint16 if dtype == "bf16" else np.float32)
        self.lib.oracle_fill_synthetic(_ptr(out), DT_BF16 if dtype == "bf16" else DT_F32, n, seed & (2 ** 64 - 1),
                                       first_index, distribution, a, b)
        return out

    def adam(self, p, g, m, v, args: AdamArgs, fused: bool = True) -> np.ndarray:
        """Updates m and v in place, returns the new float32 parameter."""
        out = np.empty(p.shape, np.float32)
        f = self.lib.oracle_adam_fused if fused else self.lib.oracle_adam_unfused
        rc = f(_ptr(out), _ptr(p), _dt(p), _ptr(g), _dt(g), _ptr(m), _ptr(v), p.size, C.byref(args))
        if rc:
            raise MemoryError("oracle_adam_unfused")
        return out

    def sgd(self, p, g, v, args: SgdArgs, fused: bool = True) -> np.ndarray:
        out = np.empty(p.shape, np.float32)
        f = self.lib.oracle_sgd_fused if fused else self.lib.oracle_sgd_unfused
        rc = f(_ptr(out), _ptr(p), _ptr(g), _ptr(v), p.size, C.byref(args))
        if rc:
            raise MemoryError("oracle_sgd_unfused")
        return out

    def rmsprop(self, p, g, v, args: RmspropArgs, fused: bool = True) -> np.ndarray:
        out = np.empty(p.shape, np.float32)
        f = self.lib.oracle_rmsprop_fused if fused else self.lib.oracle_rmsprop_unfused
        rc = f(_ptr(out), _ptr(p), _ptr(g), _ptr(v), p.size, C.byref(args))
        if rc:
            raise MemoryError("oracle_rmsprop_unfused")
        return out

    def accumulate_f32(self, acc: np.ndarray, g: np.ndarray, first: bool) -> None:
        self.lib.oracle_accumulate_f32(_ptr(acc), _ptr(g), _dt(g), g.size, int(first))

    def scale_f32(self, g: np.ndarray, scale: float) -> np.ndarray:
        out = np.empty(g.shape, np.float32)
        self.lib.oracle_scale_f32(_ptr(out), _ptr(g), _dt(g), g.size, C.c_float(scale))
        return out


def adam_args(lr, beta1, beta2, eps, wd=None, bc1=1.0, bc2=1.0, scale=None, bias_correction=False) -> AdamArgs:
    """float64 hyper-parameters -> the float32 coefficients the reference would hand to MLX."""
    f = lambda x: float(np.float32(np.float64(x)))
    return AdamArgs(lr=f(lr), beta1=f(beta1), beta2=f(beta2), omb1=f(1.0 - beta1), omb2=f(1.0 - beta2),
                    eps=f(eps), decay=f(1.0 - lr * wd) if wd is not None else 1.0, bc1=f(bc1), bc2=f(bc2),
                    decoupled_decay=int(wd is not None), has_scale=int(scale is not None),
                    scale=float(scale) if scale is not None else 1.0, bias_correction=int(bias_correction))


def load() -> OracleC:
    return OracleC(C.CDLL(build()))
