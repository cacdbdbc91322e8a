"""Thin object wrappers over the C ABI for callers that hold torch tensors.

torch is used for device memory and streams only; every computation goes through
libmxopt.so.  Tensors handed to a Table must stay alive (and keep their storage) for as
long as the table is used: the table stores raw device pointers.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from . import _lib as L

_DTYPES = {torch.float32: L.F32, torch.float16: L.F16, torch.bfloat16: L.BF16}


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise L.InvalidArg(L.ERR_INVALID_ARG, f"unsupported dtype {t.dtype}") from None


def _dev_ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    if not t.is_cuda:
        raise L.InvalidArg(L.ERR_INVALID_ARG, "mxopt needs device tensors (no CPU path exists)")
    if not t.is_contiguous():
        raise L.InvalidArg(L.ERR_INVALID_ARG, "mxopt needs dense (contiguous) buffers")
    return t.data_ptr() if t.numel() else None


@dataclass
class TensorSpec:
    """One row of a table, as torch tensors (any may be None when the kernel does not use it)."""
    p: Optional[torch.Tensor] = None
    p_out: Optional[torch.Tensor] = None
    g: Optional[torch.Tensor] = None
    g_out: Optional[torch.Tensor] = None
    m: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    bc1: float = 1.0
    bc2: float = 1.0
    flags: int = 0

    def numel(self) -> int:
        ns = {t.numel() for t in (self.p, self.p_out, self.g, self.g_out, self.m, self.v) if t is not None}
        if len(ns) != 1:
            raise L.InvalidArg(L.ERR_INVALID_ARG, f"tensors of one table row differ in size: {sorted(ns)}")
        return ns.pop()

    def to_c(self) -> L.Tensor:
        for name in ("m", "v"):
            t = getattr(self, name)
            if t is not None and t.dtype != torch.float32:
                raise L.InvalidArg(L.ERR_INVALID_ARG, f"{name} must be float32")
        c = L.Tensor()
        c.p, c.p_out, c.g, c.g_out = _dev_ptr(self.p), _dev_ptr(self.p_out), _dev_ptr(self.g), _dev_ptr(self.g_out)
        c.m, c.v = _dev_ptr(self.m), _dev_ptr(self.v)
        c.n = self.numel()
        c.p_dtype = dtype_code(self.p) if self.p is not None else 0
        c.p_out_dtype = dtype_code(self.p_out) if self.p_out is not None else 0
        c.g_dtype = dtype_code(self.g) if self.g is not None else 0
        c.g_out_dtype = dtype_code(self.g_out) if self.g_out is not None else 0
        c.flags, c.bc1, c.bc2 = self.flags, self.bc1, self.bc2
        return c


def make_prep(pre_mul: Optional[float] = None, clamp_pre: Optional[Sequence[float]] = None,
              scale: Optional["NormResultBuffer"] = None, clamp_post: Optional[Sequence[float]] = None,
              skip_if_nonfinite: Optional["NormResultBuffer"] = None) -> Optional[L.GradPrep]:
    if pre_mul is None and clamp_pre is None and scale is None and clamp_post is None and skip_if_nonfinite is None:
        return None
    p = L.GradPrep()
    if pre_mul is not None:
        p.has_pre_mul, p.pre_mul = 1, pre_mul
    if clamp_pre is not None:
        p.has_clamp_pre, p.pre_lo, p.pre_hi = 1, clamp_pre[0], clamp_pre[1]
    if scale is not None:
        p.d_scale = scale.scale_ptr
    if clamp_post is not None:
        p.has_clamp_post, p.post_lo, p.post_hi = 1, clamp_post[0], clamp_post[1]
    if skip_if_nonfinite is not None:
        p.d_skip_if_nonzero = skip_if_nonfinite.nonfinite_ptr
    return p


class NormResultBuffer:
    """Device memory for one mxopt_norm_result."""

    def __init__(self, device):
        self.buf = torch.zeros(C.sizeof(L.NormResult), dtype=torch.uint8, device=device)
        self.buf[L.NormResult.scale.offset:L.NormResult.scale.offset + 4] = torch.tensor(
            [0, 0, 0x80, 0x3F], dtype=torch.uint8, device=device)  # scale = 1.0f

    @property
    def ptr(self) -> int:
        return self.buf.data_ptr()

    @property
    def scale_ptr(self) -> int:
        return self.buf.data_ptr() + L.NormResult.scale.offset

    @property
    def nonfinite_ptr(self) -> int:
        return self.buf.data_ptr() + L.NormResult.nonfinite.offset


class Context:
    def __init__(self, device: Optional[torch.device] = None, stream: Optional[torch.cuda.Stream] = None):
        self.lib = L.load()
        if not torch.cuda.is_available():
            raise L.MxoptError(L.ERR_FAILURE, "no GPU visible: mxopt has no CPU path")
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.device = torch.device("cuda", index)
        # torch's current stream, so that mxopt kernels order with the torch ops that made the inputs
        self.stream = torch.cuda.current_stream(self.device) if stream is None else stream
        handle = C.c_void_p()
        L.check(self.lib.mxopt_create(index, C.c_void_p(self.stream.cuda_stream), C.byref(handle)))
        self.handle = handle

    def close(self) -> None:
        if getattr(self, "handle", None):
            self.lib.mxopt_destroy(self.handle)
            self.handle = None

    __del__ = close

    def set_option(self, name: str, value: int) -> None:
        L.check(self.lib.mxopt_set_option(self.handle, name.encode(), value), self.handle)

    def get_option(self, name: str) -> int:
        v = C.c_int64()
        L.check(self.lib.mxopt_get_option(self.handle, name.encode(), C.byref(v)), self.handle)
        return v.value

    def synchronize(self) -> None:
        L.check(self.lib.mxopt_synchronize(self.handle), self.handle)

    def table(self, rows: Sequence[TensorSpec]) -> "Table":
        return Table(self, rows)

    def norm_result(self) -> NormResultBuffer:
        return NormResultBuffer(self.device)

    def read_norm_result(self, buf: NormResultBuffer) -> L.NormResult:
        out = L.NormResult()
        L.check(self.lib.mxopt_read_norm_result(self.handle, C.c_void_p(buf.ptr), C.byref(out)), self.handle)
        return out

    # ---- kernels ----
    def adam(self, table: "Table", hp: L.AdamHp, prep: Optional[L.GradPrep] = None) -> None:
        L.check(self.lib.mxopt_adam(self.handle, table.handle, C.byref(hp), C.byref(prep) if prep else None),
                self.handle)

    def adam_with_pending(self, table: "Table", hp: L.AdamHp, prep: Optional[L.GradPrep] = None) -> None:
        L.check(self.lib.mxopt_adam_with_pending(self.handle, table.handle, C.byref(hp),
                                                 C.byref(prep) if prep else None), self.handle)

    def sgd(self, table: "Table", hp: L.SgdHp, prep: Optional[L.GradPrep] = None) -> None:
        L.check(self.lib.mxopt_sgd(self.handle, table.handle, C.byref(hp), C.byref(prep) if prep else None),
                self.handle)

    def rmsprop(self, table: "Table", hp: L.RmspropHp, prep: Optional[L.GradPrep] = None) -> None:
        L.check(self.lib.mxopt_rmsprop(self.handle, table.handle, C.byref(hp), C.byref(prep) if prep else None),
                self.handle)

    def sgd_plain(self, table: "Table", learning_rate: float, weight_decay: float = 0.0,
                  prep: Optional[L.GradPrep] = None) -> None:
        L.check(self.lib.mxopt_sgd_plain(self.handle, table.handle, learning_rate, weight_decay,
                                         C.byref(prep) if prep else None), self.handle)

    def global_norm(self, table: "Table", out: NormResultBuffer, which: int = 0,
                    prep: Optional[L.GradPrep] = None, max_norm: float = -1.0,
                    clip_mode: int = L.CLIP_ALWAYS_MULTIPLY) -> None:
        L.check(self.lib.mxopt_global_norm(self.handle, table.handle, which, C.byref(prep) if prep else None,
                                           max_norm, clip_mode, C.c_void_p(out.ptr)), self.handle)

    def global_norm_static(self, table: "Table", out: NormResultBuffer, which: int = 0,
                           prep: Optional[L.GradPrep] = None, max_norm: float = -1.0,
                           clip_mode: int = L.CLIP_ALWAYS_MULTIPLY) -> None:
        """global_norm with its partial sums in the library's fixed device array: allocates nothing."""
        L.check(self.lib.mxopt_global_norm_static(self.handle, table.handle, which,
                                                  C.byref(prep) if prep else None, max_norm, clip_mode,
                                                  C.c_void_p(out.ptr)), self.handle)

    def grad_transform(self, table: "Table", prep: Optional[L.GradPrep]) -> None:
        L.check(self.lib.mxopt_grad_transform(self.handle, table.handle, C.byref(prep) if prep else None),
                self.handle)

    def accumulate(self, table: "Table", first: bool, out: Optional[NormResultBuffer] = None,
                   prep: Optional[L.GradPrep] = None, max_norm: float = -1.0,
                   clip_mode: int = L.CLIP_ALWAYS_MULTIPLY) -> None:
        L.check(self.lib.mxopt_accumulate(self.handle, table.handle, int(first), C.byref(prep) if prep else None,
                                          max_norm, clip_mode, C.c_void_p(out.ptr) if out else None), self.handle)


def _sgd_plain_with_pending(self, table: "Table", learning_rate: float, weight_decay: float = 0.0,
                            prep: Optional[L.GradPrep] = None, prep_covers_sum: bool = False) -> None:
    L.check(self.lib.mxopt_sgd_plain_with_pending(self.handle, table.handle, learning_rate, weight_decay,
                                                  C.byref(prep) if prep else None, int(prep_covers_sum)),
            self.handle)


def _fill_synthetic(self, t: torch.Tensor, seed: int, distribution: int = L.SYNTH_NORMAL, a: float = 1.0,
                    b: float = 0.0, first_index: int = 0) -> None:
    """Deterministic synthetic data into `t` (see mxopt_fill_synthetic): reproducible on the host."""
    if not t.is_contiguous():
        raise L.InvalidArg(L.ERR_INVALID_ARG, "mxopt needs dense (contiguous) buffers")
    L.check(self.lib.mxopt_fill_synthetic(self.handle, _dev_ptr(t), t.numel(), dtype_code(t), seed & (2 ** 64 - 1),
                                          first_index, distribution, a, b), self.handle)


def synthetic_key(seed: int, config: int = 0, step: int = 0, micro_batch: int = 0, tensor_index: int = 0) -> int:
    return L.load().mxopt_synthetic_key(seed & (2 ** 64 - 1), config, step, micro_batch, tensor_index)


def _accumulate_transformed(self, table: "Table", first: bool, prep: Optional[L.GradPrep] = None) -> None:
    L.check(self.lib.mxopt_accumulate_transformed(self.handle, table.handle, int(first),
                                                  C.byref(prep) if prep else None), self.handle)


def _accumulate_norm_only(self, table: "Table", out: NormResultBuffer, prep: Optional[L.GradPrep] = None,
                          max_norm: float = -1.0, clip_mode: int = L.CLIP_ALWAYS_MULTIPLY) -> None:
    L.check(self.lib.mxopt_accumulate_norm_only(self.handle, table.handle, C.byref(prep) if prep else None,
                                                max_norm, clip_mode, C.c_void_p(out.ptr)), self.handle)


def _norm_with_pending_list(self, table: "Table", out: NormResultBuffer, prep: Optional[L.GradPrep] = None,
                            max_norm: float = -1.0, clip_mode: int = L.CLIP_ALWAYS_MULTIPLY) -> None:
    L.check(self.lib.mxopt_norm_with_pending_list(self.handle, table.handle, C.byref(prep) if prep else None,
                                                  max_norm, clip_mode, C.c_void_p(out.ptr)), self.handle)


def _adam_with_pending_list(self, table: "Table", hp: L.AdamHp, prep: Optional[L.GradPrep] = None) -> None:
    L.check(self.lib.mxopt_adam_with_pending_list(self.handle, table.handle, C.byref(hp),
                                                  C.byref(prep) if prep else None), self.handle)


def _sgd_with_pending_list(self, table: "Table", hp: L.SgdHp, prep: Optional[L.GradPrep] = None) -> None:
    L.check(self.lib.mxopt_sgd_with_pending_list(self.handle, table.handle, C.byref(hp),
                                                 C.byref(prep) if prep else None), self.handle)


def _rmsprop_with_pending_list(self, table: "Table", hp: L.RmspropHp, prep: Optional[L.GradPrep] = None) -> None:
    L.check(self.lib.mxopt_rmsprop_with_pending_list(self.handle, table.handle, C.byref(hp),
                                                     C.byref(prep) if prep else None), self.handle)


def _sgd_plain_with_pending_list(self, table: "Table", learning_rate: float, weight_decay: float = 0.0,
                                 prep: Optional[L.GradPrep] = None) -> None:
    L.check(self.lib.mxopt_sgd_plain_with_pending_list(self.handle, table.handle, learning_rate, weight_decay,
                                                       C.byref(prep) if prep else None), self.handle)


def _sgd_plain_with_pending_list_each(self, table: "Table", learning_rate: float, scales: Sequence[Optional[int]],
                                      weight_decay: float = 0.0, prep: Optional[L.GradPrep] = None,
                                      first_is_sum: bool = False) -> None:
    """scales: one device address of a float per stream (tensor.g first), or None for all of them.
    first_is_sum: tensor.g is a float32 sum of already prepared micro-batches (scales[0] is None then)."""
    arr = (C.c_void_p * max(len(scales), 1))(*scales)
    L.check(self.lib.mxopt_sgd_plain_with_pending_list_each(self.handle, table.handle, learning_rate, weight_decay,
                                                            C.byref(prep) if prep else None, arr,
                                                            int(first_is_sum)), self.handle)


Context.sgd_plain_with_pending_list_each = _sgd_plain_with_pending_list_each
class _HbmSpread:
    """with ctx.hbm_spread(): allocate the long-lived buffers here (see mxopt_hbm_spread_begin)."""

    def __init__(self, ctx: "Context", block_bytes: int, keep_one_in: int):
        self.ctx, self.block_bytes, self.keep_one_in = ctx, block_bytes, keep_one_in
        self.handle = C.c_void_p()

    def __enter__(self):
        torch.cuda.empty_cache()     # what torch caches is not free memory to the driver
        L.check(self.ctx.lib.mxopt_hbm_spread_begin(self.ctx.handle, self.block_bytes, self.keep_one_in,
                                                    C.byref(self.handle)), self.ctx.handle)
        return self

    def __exit__(self, *exc):
        if self.handle:
            L.check(self.ctx.lib.mxopt_hbm_spread_end(self.handle), self.ctx.handle)
            self.handle = C.c_void_p()
        return False


class HbmPool:
    """Region-interleaved device memory (mxopt_hbm_pool_create).  `torch_pool()` makes torch allocate from
    it: `with torch.cuda.use_mem_pool(pool.torch_pool()): p = torch.empty(...)`."""

    MAX_REGIONS = L.HBM_MAX_REGIONS
    _torch_allocator = None   # one per process: torch keeps the function pointers

    def __init__(self, ctx: "Context", capacity_bytes: int, chunk_bytes: int = 0, max_regions: int = 0,
                 max_take_bytes: int = 0, slab_bytes: int = 0):
        self.ctx = ctx
        self.handle = C.c_void_p()
        torch.cuda.empty_cache()     # what torch caches is not free memory to the driver
        opts = L.HbmPoolOptions(capacity_bytes=capacity_bytes, chunk_bytes=chunk_bytes, max_regions=max_regions,
                                max_take_bytes=max_take_bytes, slab_bytes=slab_bytes)
        L.check(ctx.lib.mxopt_hbm_pool_create_ex(ctx.handle, C.byref(opts), C.byref(self.handle)), ctx.handle)

    def info(self) -> L.HbmPoolInfo:
        out = L.HbmPoolInfo()
        L.check(self.ctx.lib.mxopt_hbm_pool_get_info(self.handle, C.byref(out)), self.ctx.handle)
        return out

    def alloc(self, nbytes: int, kind: int = L.HBM_INTERLEAVED) -> int:
        p = C.c_void_p()
        L.check(self.ctx.lib.mxopt_hbm_pool_alloc_kind(self.handle, nbytes, kind, C.byref(p)), self.ctx.handle)
        return p.value

    @staticmethod
    def hook_kind(kind: int) -> None:
        """What torch's allocations through torch_pool() get from now on: HBM_INTERLEAVED or HBM_ONE_REGION."""
        L.check(L.load().mxopt_hbm_pool_set_hook_kind(kind))

    def free(self, ptr: int) -> None:
        L.check(self.ctx.lib.mxopt_hbm_pool_free(self.handle, C.c_void_p(ptr)), self.ctx.handle)

    def owns(self, ptr: int) -> bool:
        return bool(self.ctx.lib.mxopt_hbm_pool_owns(self.handle, C.c_void_p(ptr)))

    def use_for_state(self) -> None:
        """Moments and accumulation buffers of objects created on this context from now on live here."""
        L.check(self.ctx.lib.mxopt_set_state_pool(self.ctx.handle, self.handle), self.ctx.handle)

    def torch_pool(self):
        """A new torch.cuda.MemPool whose segments come from this pool (and from hipMalloc once it is full).
        Dropping the MemPool and its tensors hands the segments back."""
        L.check(self.ctx.lib.mxopt_hbm_pool_set_hook_target(self.handle), self.ctx.handle)
        if HbmPool._torch_allocator is None:
            HbmPool._torch_allocator = torch.cuda.memory.CUDAPluggableAllocator(
                L.LIB_PATH, "mxopt_hbm_pool_hook_alloc", "mxopt_hbm_pool_hook_free")
        return torch.cuda.MemPool(HbmPool._torch_allocator.allocator())

    def close(self) -> None:
        """Raises while anything allocated from the pool is alive (torch tensors and MemPools included)."""
        if self.handle:
            torch.cuda.empty_cache()     # segments torch only caches go back through the free hook
            L.check(self.ctx.lib.mxopt_hbm_pool_destroy(self.handle), self.ctx.handle)
            self.handle = C.c_void_p()


def _hbm_pool(self, capacity_bytes: int, chunk_bytes: int = 0, max_regions: int = 0, max_take_bytes: int = 0,
              slab_bytes: int = 0) -> HbmPool:
    return HbmPool(self, capacity_bytes, chunk_bytes, max_regions, max_take_bytes, slab_bytes)


def classify_regions(n_slabs: int, probe):
    """mxopt_hbm_classify_regions on a Python callable probe(ref_slab, slab) -> GB/s: (regions per slab, report)."""
    def thunk(_user, ref, slab, out):
        out[0] = float(probe(ref, slab))
        return 0
    fn = L.SLAB_PROBE_FN(thunk)
    regions = (C.c_int * max(n_slabs, 1))()
    report = L.HbmScanReport()
    L.check(L.load().mxopt_hbm_classify_regions(n_slabs, fn, None, regions, C.byref(report)))
    return list(regions[:n_slabs]), report


def plan_arena(slab_region, regions: int, chunks_per_slab: int, total_chunks: int, want_chunks: int, max_regions: int = 0):
    """mxopt_hbm_plan_arena: (physical chunk of every arena chunk, report)."""
    n = len(slab_region)
    sr = (C.c_int * max(n, 1))(*slab_region)
    order = (C.c_int * max(want_chunks, 1))()
    report = L.HbmArenaReport()
    L.check(L.load().mxopt_hbm_plan_arena(n, sr, regions, chunks_per_slab, total_chunks, want_chunks, max_regions, order,
                                          C.byref(report)))
    return list(order[:want_chunks]), report


def _probe_stream(self, kind: int, a, b=None, c=None, d=None) -> None:
    """One launch of a bare streaming probe over float32 tensors of equal size (mxopt_probe_stream)."""
    ptr = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    L.check(self.lib.mxopt_probe_stream(self.handle, kind, ptr(a), ptr(b), ptr(c), ptr(d), a.numel()), self.handle)


def _hbm_spread(self, block_bytes: int = 0, keep_one_in: int = 0) -> _HbmSpread:
    return _HbmSpread(self, block_bytes, keep_one_in)


Context.hbm_spread = _hbm_spread
Context.hbm_pool = _hbm_pool
def _probe_list(self, p, m, v, grads, streaming: bool = False) -> None:
    """One launch of the bare byte mix of the update over un-summed 16-bit micro-batches (mxopt_probe_list);
    streaming: the 2-byte streams with streaming-hint loads and stores, as the list kernels access them."""
    arr = (C.c_void_p * len(grads))(*[_dev_ptr(g) for g in grads])
    k = len(grads) | (L.PROBE_STREAMING if streaming else 0)
    L.check(self.lib.mxopt_probe_list(self.handle, C.c_void_p(_dev_ptr(p)), C.c_void_p(_dev_ptr(m)),
                                      C.c_void_p(_dev_ptr(v)), arr, k, p.numel()), self.handle)


Context.probe_stream = _probe_stream
Context.probe_list = _probe_list
Context.accumulate_norm_only = _accumulate_norm_only
Context.norm_with_pending_list = _norm_with_pending_list
Context.adam_with_pending_list = _adam_with_pending_list
Context.sgd_plain_with_pending_list = _sgd_plain_with_pending_list
Context.sgd_with_pending_list = _sgd_with_pending_list
Context.rmsprop_with_pending_list = _rmsprop_with_pending_list
Context.accumulate_transformed = _accumulate_transformed
Context.fill_synthetic = _fill_synthetic
Context.sgd_plain_with_pending = _sgd_plain_with_pending


class Table:
    def __init__(self, ctx: Context, rows: Sequence[TensorSpec]):
        self.ctx = ctx
        self.rows: List[TensorSpec] = list(rows)   # keeps the tensors alive
        n = len(self.rows)
        arr = (L.Tensor * max(n, 1))()
        for i, r in enumerate(self.rows):
            arr[i] = r.to_c()
        handle = C.c_void_p()
        L.check(ctx.lib.mxopt_table_build(ctx.handle, arr, n, C.byref(handle)), ctx.handle)
        self.handle = handle

    def close(self) -> None:
        if getattr(self, "handle", None) and getattr(self.ctx, "handle", None):
            self.ctx.lib.mxopt_table_destroy(self.handle)
        self.handle = None

    __del__ = close

    def retarget(self, rows: Sequence[TensorSpec]) -> None:
        """Same tensors in new buffers: swaps the pointers, keeps the chunk list."""
        rows = list(rows)
        arr = (L.Tensor * max(len(rows), 1))()
        for i, r in enumerate(rows):
            arr[i] = r.to_c()
        L.check(self.ctx.lib.mxopt_table_retarget(self.handle, arr, len(rows)), self.ctx.handle)
        self.rows = rows

    def set_pending(self, streams: Sequence[Sequence[torch.Tensor]]) -> None:
        """Deferred accumulation: streams[j][i] is pending gradient j of row i (all of one dtype)."""
        streams = [list(s) for s in streams]
        k, n = len(streams), len(self.rows)
        if k == 0:
            L.check(self.ctx.lib.mxopt_table_set_pending(self.handle, 0, None, 0), self.ctx.handle)
            self.pending = []
            return
        if any(len(s) != n for s in streams):
            raise L.InvalidArg(L.ERR_INVALID_ARG, "every pending stream needs one tensor per table row")
        flat = [t for s in streams for t in s]
        if any(not t.is_contiguous() for t in flat):
            raise L.InvalidArg(L.ERR_INVALID_ARG, "mxopt needs dense (contiguous) buffers")
        if any(t.dtype != flat[0].dtype for t in flat):
            raise L.InvalidArg(L.ERR_INVALID_ARG, "pending streams must share one dtype")
        arr = (C.c_void_p * max(len(flat), 1))(*[_dev_ptr(t) for t in flat])
        code = dtype_code(flat[0]) if flat else 0
        L.check(self.ctx.lib.mxopt_table_set_pending(self.handle, k, arr, code), self.ctx.handle)
        self.pending = streams   # keeps the tensors alive

    @property
    def total_elems(self) -> int:
        return self.ctx.lib.mxopt_table_total_elems(self.handle)

    @property
    def num_chunks(self) -> int:
        return self.ctx.lib.mxopt_table_num_chunks(self.handle)

    def set_step_scalars(self, bc1: Optional[Sequence[float]] = None, bc2: Optional[Sequence[float]] = None,
                         flags: Optional[Sequence[int]] = None) -> None:
        n = len(self.rows)
        a = (C.c_float * n)(*bc1) if bc1 is not None else None
        b = (C.c_float * n)(*bc2) if bc2 is not None else None
        f = (C.c_uint32 * n)(*flags) if flags is not None else None
        L.check(self.ctx.lib.mxopt_table_set_step_scalars(self.handle, a, b, f), self.ctx.handle)


def adam_hp(lr: float, beta1: float, beta2: float, eps: float, weight_decay: Optional[float] = None) -> L.AdamHp:
    """weight_decay None = Adam, a number = AdamW."""
    hp = L.AdamHp()
    L.load().mxopt_adam_hp_from_f64(lr, beta1, beta2, eps, 0.0 if weight_decay is None else weight_decay,
                                    int(weight_decay is not None), C.byref(hp))
    return hp


def bias_correction(beta1: float, beta2: float, t: int):
    a, b = C.c_float(), C.c_float()
    L.load().mxopt_bias_correction(beta1, beta2, t, C.byref(a), C.byref(b))
    return a.value, b.value


def sgd_hp(lr: float, momentum: float = 0.0, weight_decay: float = 0.0, dampening: float = 0.0,
           nesterov: bool = False) -> L.SgdHp:
    hp = L.SgdHp()
    L.check(L.load().mxopt_sgd_hp_from_f64(lr, momentum, weight_decay, dampening, int(nesterov), C.byref(hp)))
    return hp


def rmsprop_hp(lr: float, alpha: float, eps: float, weight_decay: float = 0.0) -> L.RmspropHp:
    hp = L.RmspropHp()
    L.load().mxopt_rmsprop_hp_from_f64(lr, alpha, eps, weight_decay, C.byref(hp))
    return hp
