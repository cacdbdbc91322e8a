"""ctypes view of include/mxopt.h.  Loading fails loudly when the HIP library has not been
built: there is no CPU fallback in this package."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(HERE), "libmxopt.so")

F32, I32, F16, BF16, U32 = 0, 1, 2, 3, 4
OK, ERR_INVALID_ARG, ERR_FAILURE, ERR_HIP, ERR_OOM = 0, 1, 2, 3, 4
TF_FIRST = 0x1
SYNTH_NORMAL, SYNTH_NORMAL_OUTLIERS, SYNTH_UNIFORM, SYNTH_GAUSSIAN, SYNTH_GAUSSIAN_OUTLIERS = 0, 1, 2, 3, 4
CLIP_ALWAYS_MULTIPLY, CLIP_IF_ABOVE = 0, 1
CHUNK_ELEMS = 4096
MAX_PENDING = 7


class MxoptError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"mxopt error {code}: {message}")
        self.code = code
        self.message = message


class InvalidArg(MxoptError, ValueError):
    """napi Status::InvalidArg."""


class Tensor(C.Structure):
    _fields_ = [("p", C.c_void_p), ("p_out", C.c_void_p), ("g", C.c_void_p), ("g_out", C.c_void_p),
                ("m", C.c_void_p), ("v", C.c_void_p), ("n", C.c_uint64),
                ("p_dtype", C.c_uint8), ("p_out_dtype", C.c_uint8), ("g_dtype", C.c_uint8), ("g_out_dtype", C.c_uint8),
                ("flags", C.c_uint32), ("bc1", C.c_float), ("bc2", C.c_float)]


class NormResult(C.Structure):
    _fields_ = [("sumsq", C.c_double), ("norm", C.c_double), ("norm_f32", C.c_float), ("scale", C.c_float),
                ("nonfinite", C.c_uint64)]


class GradPrep(C.Structure):
    _fields_ = [("has_pre_mul", C.c_int), ("pre_mul", C.c_float),
                ("has_clamp_pre", C.c_int), ("pre_lo", C.c_float), ("pre_hi", C.c_float),
                ("d_scale", C.c_void_p),
                ("has_clamp_post", C.c_int), ("post_lo", C.c_float), ("post_hi", C.c_float),
                ("d_skip_if_nonzero", C.c_void_p)]


class AdamHp(C.Structure):
    _fields_ = [("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("one_minus_beta1", C.c_float),
                ("one_minus_beta2", C.c_float), ("eps", C.c_float), ("decay", C.c_float),
                ("decoupled_decay", C.c_int)]


class SgdHp(C.Structure):
    _fields_ = [("lr", C.c_float), ("momentum", C.c_float), ("one_minus_dampening", C.c_float),
                ("weight_decay", C.c_float), ("has_weight_decay", C.c_int), ("has_momentum", C.c_int),
                ("nesterov", C.c_int)]


HBM_MAX_REGIONS = 8
PROBE_READ, PROBE_WRITE, PROBE_COPY, PROBE_MIX43 = 0, 1, 2, 3
PROBE_STREAMING = 0x100


class HbmPoolInfo(C.Structure):
    _fields_ = [("capacity_bytes", C.c_uint64), ("used_bytes", C.c_uint64), ("chunk_bytes", C.c_uint64),
                ("regions", C.c_int32), ("reserved_", C.c_int32),
                ("region_free_bytes", C.c_uint64 * HBM_MAX_REGIONS),
                ("region_arena_bytes", C.c_uint64 * HBM_MAX_REGIONS),
                ("probe_same_region_gbps", C.c_double), ("probe_cross_region_gbps", C.c_double),
                ("setup_seconds", C.c_double), ("create_seconds", C.c_double), ("scan_seconds", C.c_double),
                ("probes", C.c_int32), ("reserved2_", C.c_int32), ("interleaved_bytes", C.c_uint64),
                ("arena_probe_gbps", C.c_double)]


class HbmPoolOptions(C.Structure):
    _fields_ = [("capacity_bytes", C.c_size_t), ("chunk_bytes", C.c_size_t), ("max_regions", C.c_int),
                ("reserved_", C.c_int), ("max_take_bytes", C.c_size_t), ("slab_bytes", C.c_size_t)]


class HbmScanReport(C.Structure):
    _fields_ = [("regions", C.c_int32), ("probes", C.c_int32), ("same_region_gbps", C.c_double),
                ("cross_region_gbps", C.c_double)]


class HbmArenaReport(C.Structure):
    _fields_ = [("real_regions", C.c_int32), ("active_regions", C.c_int32), ("interleaved_chunks", C.c_int32),
                ("reserved_", C.c_int32)]


SLAB_PROBE_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_double))
HBM_INTERLEAVED, HBM_ONE_REGION = 0, 1


class RmspropHp(C.Structure):
    _fields_ = [("lr", C.c_float), ("alpha", C.c_float), ("one_minus_alpha", C.c_float), ("eps", C.c_float),
                ("weight_decay", C.c_float), ("has_weight_decay", C.c_int)]


# name -> (restype, argtypes); every symbol declared in include/mxopt.h
SIGNATURES = {
    "mxopt_create": (C.c_int, [C.c_int, C.c_void_p, C.POINTER(C.c_void_p)]),
    "mxopt_destroy": (None, [C.c_void_p]),
    "mxopt_last_error": (C.c_char_p, [C.c_void_p]),
    "mxopt_synchronize": (C.c_int, [C.c_void_p]),
    "mxopt_set_option": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int64]),
    "mxopt_get_option": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_int64)]),
    "mxopt_table_build": (C.c_int, [C.c_void_p, C.POINTER(Tensor), C.c_size_t, C.POINTER(C.c_void_p)]),
    "mxopt_table_set_step_scalars": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float),
                                               C.POINTER(C.c_uint32)]),
    "mxopt_table_destroy": (None, [C.c_void_p]),
    "mxopt_table_total_elems": (C.c_uint64, [C.c_void_p]),
    "mxopt_table_num_chunks": (C.c_uint64, [C.c_void_p]),
    "mxopt_table_num_tensors": (C.c_uint64, [C.c_void_p]),
    "mxopt_table_retarget": (C.c_int, [C.c_void_p, C.POINTER(Tensor), C.c_size_t]),
    "mxopt_tensor_layout": (C.c_int, [C.POINTER(Tensor), C.POINTER(C.c_uint32), C.POINTER(C.c_int),
                                      C.POINTER(C.c_uint64)]),
    "mxopt_adam_hp_from_f64": (None, [C.c_double, C.c_double, C.c_double, C.c_double, C.c_double, C.c_int,
                                      C.POINTER(AdamHp)]),
    "mxopt_bias_correction": (None, [C.c_double, C.c_double, C.c_int64, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "mxopt_sgd_hp_from_f64": (C.c_int, [C.c_double, C.c_double, C.c_double, C.c_double, C.c_int, C.POINTER(SgdHp)]),
    "mxopt_rmsprop_hp_from_f64": (None, [C.c_double, C.c_double, C.c_double, C.c_double, C.POINTER(RmspropHp)]),
    "mxopt_adam": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(AdamHp), C.POINTER(GradPrep)]),
    "mxopt_hbm_spread_begin": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_void_p)]),
    "mxopt_hbm_spread_end": (C.c_int, [C.c_void_p]),
    "mxopt_hbm_pool_create": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.POINTER(C.c_void_p)]),
    "mxopt_hbm_pool_create_ex": (C.c_int, [C.c_void_p, C.POINTER(HbmPoolOptions), C.POINTER(C.c_void_p)]),
    "mxopt_hbm_pool_destroy": (C.c_int, [C.c_void_p]),
    "mxopt_hbm_pool_alloc_kind": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_void_p)]),
    "mxopt_hbm_pool_set_hook_kind": (C.c_int, [C.c_int]),
    "mxopt_hbm_classify_regions": (C.c_int, [C.c_int, SLAB_PROBE_FN, C.c_void_p, C.POINTER(C.c_int),
                                             C.POINTER(HbmScanReport)]),
    "mxopt_hbm_plan_arena": (C.c_int, [C.c_int, C.POINTER(C.c_int), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                       C.POINTER(C.c_int), C.POINTER(HbmArenaReport)]),
    "mxopt_hbm_pool_alloc": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "mxopt_hbm_pool_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "mxopt_hbm_pool_owns": (C.c_int, [C.c_void_p, C.c_void_p]),
    "mxopt_hbm_pool_get_info": (C.c_int, [C.c_void_p, C.POINTER(HbmPoolInfo)]),
    "mxopt_set_state_pool": (C.c_int, [C.c_void_p, C.c_void_p]),
    "mxopt_hbm_pool_set_hook_target": (C.c_int, [C.c_void_p]),
    "mxopt_hbm_pool_hook_alloc": (C.c_void_p, [C.c_ssize_t, C.c_int, C.c_void_p]),
    "mxopt_hbm_pool_hook_free": (None, [C.c_void_p, C.c_ssize_t, C.c_int, C.c_void_p]),
    "mxopt_probe_stream": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64]),
    "mxopt_probe_list": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint64]),
    "mxopt_table_set_pending": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.c_int]),
    "mxopt_norm_with_pending_list": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(GradPrep), C.c_double, C.c_int,
                                               C.c_void_p]),
    "mxopt_adam_with_pending_list": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(AdamHp), C.POINTER(GradPrep)]),
    "mxopt_sgd_with_pending_list": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(SgdHp), C.POINTER(GradPrep)]),
    "mxopt_rmsprop_with_pending_list": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(RmspropHp), C.POINTER(GradPrep)]),
    "mxopt_sgd_plain_with_pending_list": (C.c_int, [C.c_void_p, C.c_void_p, C.c_double, C.c_double,
                                                    C.POINTER(GradPrep)]),
    "mxopt_sgd_plain_with_pending_list_each": (C.c_int, [C.c_void_p, C.c_void_p, C.c_double, C.c_double,
                                                         C.POINTER(GradPrep), C.POINTER(C.c_void_p), C.c_int]),
    "mxopt_adam_with_pending": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(AdamHp), C.POINTER(GradPrep)]),
    "mxopt_sgd": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(SgdHp), C.POINTER(GradPrep)]),
    "mxopt_rmsprop": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(RmspropHp), C.POINTER(GradPrep)]),
    "mxopt_sgd_plain": (C.c_int, [C.c_void_p, C.c_void_p, C.c_double, C.c_double, C.POINTER(GradPrep)]),
    "mxopt_sgd_plain_with_pending": (C.c_int, [C.c_void_p, C.c_void_p, C.c_double, C.c_double, C.POINTER(GradPrep),
                                               C.c_int]),
    "mxopt_global_norm": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(GradPrep), C.c_double, C.c_int,
                                    C.c_void_p]),
    "mxopt_global_norm_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(GradPrep), C.c_double, C.c_int,
                                           C.c_void_p]),
    "mxopt_grad_transform": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(GradPrep)]),
    "mxopt_accumulate_transformed": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(GradPrep)]),
    "mxopt_accumulate": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(GradPrep), C.c_double, C.c_int,
                                   C.c_void_p]),
    "mxopt_accumulate_norm_only": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(GradPrep), C.c_double, C.c_int,
                                             C.c_void_p]),
    "mxopt_fill_synthetic": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_uint64, C.c_uint64, C.c_int,
                                       C.c_double, C.c_double]),
    "mxopt_synthetic_key": (C.c_uint64, [C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64]),
    "mxopt_read_norm_result": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(NormResult)]),
    "mxopt_version": (C.c_char_p, []),
}


class Array(C.Structure):
    """mxopt_array (include/mxopt_optimizers.h)."""
    _fields_ = [("data", C.c_void_p), ("n", C.c_uint64), ("dtype", C.c_int32)]


_PD = C.POINTER(C.c_double)
_PI = C.POINTER(C.c_int)
_PA = C.POINTER(Array)

# every symbol declared in include/mxopt_optimizers.h
SIGNATURES.update({
    "mxopt_adam_new": (C.c_int, [C.c_void_p, _PD, _PD, _PD, _PD, _PI, C.POINTER(C.c_void_p)]),
    "mxopt_adamw_new": (C.c_int, [C.c_void_p, _PD, _PD, _PD, _PD, _PD, _PI, C.POINTER(C.c_void_p)]),
    "mxopt_sgd_new": (C.c_int, [C.c_void_p, C.c_double, _PD, _PD, _PD, _PI, C.POINTER(C.c_void_p)]),
    "mxopt_rmsprop_new": (C.c_int, [C.c_void_p, _PD, _PD, _PD, _PD, C.POINTER(C.c_void_p)]),
    "mxopt_optimizer_free": (None, [C.c_void_p]),
    "mxopt_optimizer_update_single": (C.c_int, [C.c_void_p, C.c_char_p, _PA, _PA, _PA]),
    "mxopt_optimizer_update_many": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_char_p), _PA, _PA, _PA,
                                              C.POINTER(GradPrep)]),
    "mxopt_optimizer_update_many_accumulated": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_char_p), _PA, C.c_size_t,
                                                          _PA, _PA, C.POINTER(GradPrep), C.c_double, C.c_int,
                                                          C.c_void_p]),
    "mxopt_optimizer_reset": (C.c_int, [C.c_void_p]),
    "mxopt_optimizer_step_count": (C.c_int64, [C.c_void_p]),
    "mxopt_optimizer_state": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                        C.POINTER(C.c_uint64), _PI]),
    "mxopt_optimizer_save_state": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p]),
    "mxopt_optimizer_load_state": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_uint64,
                                             C.c_int64]),
    "mxopt_optimizer_save_file": (C.c_int, [C.c_void_p, C.c_char_p]),
    "mxopt_optimizer_load_file": (C.c_int, [C.c_void_p, C.c_char_p]),
    "mxopt_checkpoint_inspect": (C.c_int, [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_int64),
                                           C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "mxopt_compute_gradient_norm": (C.c_int, [C.c_void_p, C.c_size_t, _PA, _PD]),
    "mxopt_clip_grad_norm": (C.c_int, [C.c_void_p, C.c_size_t, _PA, C.c_double, _PA, _PD]),
    "mxopt_clip_grad_value": (C.c_int, [C.c_void_p, _PA, C.c_double, C.c_double, _PA]),
    "mxopt_clip_grad_value_and_norm": (C.c_int, [C.c_void_p, C.c_size_t, _PA, C.c_double, _PD, _PA]),
    "mxopt_clip_gradients_by_global_norm": (C.c_int, [C.c_void_p, C.c_size_t, _PA, C.c_double, _PA]),
    "mxopt_clip_gradients_by_value": (C.c_int, [C.c_void_p, C.c_size_t, _PA, C.c_double, C.c_double, _PA]),
    "mxopt_accumulate_gradients": (C.c_int, [C.c_void_p, C.c_size_t, _PA, _PA, _PA]),
    "mxopt_apply_gradients": (C.c_int, [C.c_void_p, C.c_size_t, _PA, _PA, C.c_double, _PA]),
    "mxopt_lr_linear_decay": (C.c_double, [C.c_double, C.c_double, C.c_int64, C.c_int64]),
    "mxopt_lr_exponential_decay": (C.c_double, [C.c_double, C.c_double, C.c_int64, C.c_int64]),
    "mxopt_lr_cosine_annealing": (C.c_double, [C.c_double, C.c_double, C.c_int64, C.c_int64]),
    "mxopt_lr_step_decay": (C.c_double, [C.c_double, C.c_double, C.c_int64, C.c_int64]),
})

_lib = None



class EngineConfig(C.Structure):
    """mxopt_engine_config (include/mxopt_engine.h)."""
    _fields_ = [("kind", C.c_int32), ("gradient_accumulation_steps", C.c_int32), ("learning_rate", C.c_double),
                ("has_gradient_clip_norm", C.c_int32), ("gradient_clip_norm", C.c_double),
                ("has_gradient_clip_value", C.c_int32), ("gradient_clip_value", C.c_double),
                ("weight_decay", C.c_double), ("max_nan_gradients", C.c_int64),
                ("emergency_save_threshold", C.c_int32), ("apply", C.c_int32),
                ("beta1", C.c_double), ("beta2", C.c_double), ("eps", C.c_double),
                ("accumulate_in_f32", C.c_int32), ("defer_accumulation", C.c_int32)]


class EngineMetrics(C.Structure):
    """mxopt_engine_metrics (include/mxopt_engine.h)."""
    _fields_ = [("step", C.c_int64), ("micro_step", C.c_int32), ("gradients_applied", C.c_int32),
                ("skipped", C.c_int32), ("needs_emergency_save", C.c_int32), ("consecutive_nan_count", C.c_uint32),
                ("nan_gradient_count", C.c_uint64), ("norm_measured", C.c_int32), ("clip_scale", C.c_float),
                ("grad_sumsq", C.c_double), ("grad_norm", C.c_double)]


ENGINE_GRPO, ENGINE_SFT = 0, 1
ENGINE_APPLY_SGD, ENGINE_APPLY_ADAMW = 0, 1
_PM = C.POINTER(EngineMetrics)

# every symbol declared in include/mxopt_engine.h
SIGNATURES.update({
    "mxopt_engine_config_default": (None, [C.c_int32, C.POINTER(EngineConfig)]),
    "mxopt_engine_new": (C.c_int, [C.c_void_p, C.POINTER(EngineConfig), C.c_size_t, C.POINTER(C.c_char_p), _PA,
                                   C.POINTER(C.c_void_p)]),
    "mxopt_engine_free": (None, [C.c_void_p]),
    "mxopt_engine_micro_batch": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_char_p), _PA, _PM]),
    "mxopt_engine_micro_batch_async": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_char_p), _PA]),
    "mxopt_engine_settle": (C.c_int, [C.c_void_p, _PM]),
    "mxopt_engine_flush_gradients": (C.c_int, [C.c_void_p, _PI, _PM]),
    "mxopt_engine_report_nonfinite_loss": (C.c_int, [C.c_void_p, _PM]),
    "mxopt_engine_get_metrics": (C.c_int, [C.c_void_p, _PM]),
    "mxopt_engine_clear_emergency_save_flag": (C.c_int, [C.c_void_p]),
    "mxopt_engine_reset": (C.c_int, [C.c_void_p]),
    "mxopt_engine_save_optimizer_state": (C.c_int, [C.c_void_p, C.c_char_p]),
    "mxopt_engine_load_optimizer_state": (C.c_int, [C.c_void_p, C.c_char_p]),
})

def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `python mlx-node_amd/build.py` "
                              "(there is no CPU fallback)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc: int, ctx=None) -> None:
    if rc == OK:
        return
    msg = load().mxopt_last_error(ctx).decode("utf-8", "replace")
    raise (InvalidArg if rc == ERR_INVALID_ARG else MxoptError)(rc, msg)
