"""mxopt: MI355X-native optimizer step (Adam/AdamW, SGD, RMSprop, global-norm clipping,
gradient accumulation) behind the mlx-node optimizer API.  All computation runs in
libmxopt.so (hand-written HIP for gfx950); importing fails if the library is not built."""
from ._lib import (BF16, CLIP_ALWAYS_MULTIPLY, CLIP_IF_ABOVE, F16, F32, HBM_INTERLEAVED, HBM_ONE_REGION, MAX_PENDING, PROBE_COPY, PROBE_STREAMING, PROBE_MIX43, PROBE_READ,
                   PROBE_WRITE, SYNTH_GAUSSIAN, SYNTH_GAUSSIAN_OUTLIERS, SYNTH_NORMAL, SYNTH_NORMAL_OUTLIERS, SYNTH_UNIFORM, TF_FIRST, InvalidArg, MxoptError, load)
from .core import (Context, HbmPool, NormResultBuffer, Table, TensorSpec, adam_hp, bias_correction, classify_regions,
                   make_prep, plan_arena, rmsprop_hp, sgd_hp, synthetic_key)
from .optimizers import (SGD, Adam, AdamW, GradientAccumulator, GradientUtils, LRScheduler, RMSprop,
                         accumulate_gradients, apply_gradients, clip_gradients_by_global_norm,
                         clip_gradients_by_value, default_context)
from .engine import GRPOEngineOptimizerSide, SFTEngineOptimizerSide, TrainingStopped

load()
