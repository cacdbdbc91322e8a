#!/usr/bin/env python3
"""Benchmark of the optimizer-step hot path on one MI355X.

Default workload (the one the headline metric is quoted on): Qwen3-8B-shaped training step --
4 micro-batch bf16 gradients accumulated into a float32 buffer, global-norm clip at 1.0, AdamW
with bf16 parameters updated in place and float32 moments; everything resident in HBM (~131 GB
+ 3 more micro-gradient buffers).  By default the 4th micro-batch is only measured (its norm
contribution) and then folded into the update kernel, which saves the accumulation buffer's
last write: 6 + 10 + 10 + 6 + 26 = 58 B/elem/step instead of 6 + 3*10 + 24 = 60 (--fold-last 0).

Prints ONE JSON line.  `value` = optimizer steps/s over the timed region (inputs resident
before it starts).  `roofline` describes the dominant kernel (the AdamW update): algorithmic
bytes per launch / its average duration measured with events on the launch stream.
`cpu_baseline` times the CPU restatement of the reference's un-fused op chain (oracle/) on a
bounded sample of the same workload and scales it to the full parameter list.
`deferred_accumulation` (default workload only, when four micro-batch buffers fit) is the same step on
the same buffers with the micro-batches added in registers instead of into the float32 buffer.
Every buffer comes from a region-interleaved arena (mxopt_hbm_pool_create, `config.placement`) unless
--placement plain or spread is given.  The default run also measures the four bare streaming probes on
memory from the same arena (`roofline.measured_ceiling`) and, after config 5's buffers are released,
BASELINE's configs 1 - 4 for a few steps each (`other_configs`).
"""
from __future__ import annotations

import argparse
import contextlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "mlx-node_amd"))

HBM_PEAK_GBPS = 8000.0

# HBM bytes per element per launch of the dominant kernel from an EARLIER rocprofv3 run, not from this
# one (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for this library's plain
# copy kernel).  Printed as roofline.traffic with roofline.traffic_source naming the file; null once the
# kernel sources no longer hash to what that file records.
# (workload, fold_last) -> bytes per element
TRAFFIC_PROFILE = "profiles/hbm_traffic_pmc_cfg5_and_copy.txt"
TRAFFIC_KERNEL_SOURCES = ["mxopt_kernels.hip", "mxopt_kernels_common.h", "mxopt_device.h", "mxopt_list_kernels.h",
                          "mxopt_list_kernels.hip"]
MEASURED_TRAFFIC_B_PER_ELEM = {("cfg5", 1): 25.91, ("cfg5-deferred", 1): 27.89}
PROBE_PROFILE = "profiles/probe_streams_pool_and_plain.txt"
OTHER_CONFIGS = ["cfg1", "cfg2", "cfg3-sgd", "cfg3-rmsprop", "cfg4", "cfg4-flat"]
# steps each configuration states for itself
OTHER_CONFIG_STEPS = {"cfg1": 10, "cfg2": 20, "cfg3-sgd": 20, "cfg3-rmsprop": 20, "cfg4": 100, "cfg4-flat": 100}


def traffic_profile_is_current():
    """True while the kernel sources are the ones the counters were taken on."""
    import hashlib
    import re
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
        h = hashlib.sha256()
        for f in TRAFFIC_KERNEL_SOURCES:
            h.update(open(os.path.join(ROOT, "mlx-node_amd", "csrc", f), "rb").read())
    except OSError:
        return False
    m = re.search(r"kernel-sources-sha256: ([0-9a-f]{64})", text)
    return bool(m) and m.group(1) == h.hexdigest()


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg5",
                    choices=["cfg1", "cfg1-update-single", "cfg1-update-many", "cfg2", "cfg3-sgd", "cfg3-rmsprop",
                             "cfg3-sgd-deferred", "cfg3-rmsprop-deferred",
                             "cfg4", "cfg4-flat", "cfg5", "cfg5-deferred", "copy", "probes", "grpo-engine", "sft-engine"])
    ap.add_argument("--cpu-sample", type=int, default=512 * 1024 * 1024,
                    help="elements of the CPU-baseline sample (0 = skip the CPU leg)")
    ap.add_argument("--scale", type=float, default=1.0,
                    help="shrink every tensor's first dimension (for quick runs; invalid as a result)")
    ap.add_argument("--option", action="append", default=[], help="mxopt option name=value")
    ap.add_argument("--alloc", default="tensor", choices=["tensor", "slab", "packed"],
                    help="tensor: one device allocation per tensor and stream; slab: one allocation per stream, "
                         "tensors are 512-byte aligned views into it")
    ap.add_argument("--placement", default="pool", choices=["pool", "state-pool", "spread", "plain"],
                    help="pool: every buffer comes from a region-interleaved arena (mxopt_hbm_pool_create); state-pool: "
                         "only what the library itself would own (moments, accumulation buffers) comes from the arena, "
                         "parameters and gradients lie wherever the host's allocator (here torch's) put them -- what a "
                         "drop-in host sees after mxopt_set_state_pool; spread: the buffers are allocated inside "
                         "mxopt_hbm_spread_begin/end (their physical pages interleaved with released memory, a matter of "
                         "luck); plain: wherever the driver puts them")
    ap.add_argument("--placements", type=int, default=-1,
                    help="1: the default workload is also measured with --placement plain (in a child process started "
                         "before this one touches the GPU: the first allocations of a fresh process) and with "
                         "--placement state-pool, and config.placement carries the three AdamW rates; default: only "
                         "for cfg5 at full scale on the arena")
    ap.add_argument("--plain-leg", default="first", choices=["first", "last"],
                    help="--placements: when the child process with --placement plain runs.  first (default): before this "
                         "process touches the GPU; on a fresh box the child's are then the first allocations of a fresh "
                         "process, one compact physical run in one region, the worst case (5.37 TB/s in every run); this "
                         "process then waits --settle-s before it looks at the device.  last: after this process has given "
                         "all its memory back; the child then gets pieces from all over the device, which is what a host "
                         "sees on a GPU other processes have used (5.5 - 6.05 TB/s measured)")
    ap.add_argument("--verify", type=int, default=-1,
                    help="1: after the timed steps, seeded windows of parameters and moments are recomputed on the host "
                         "by the C twin of the oracle for exactly the steps that ran and compared bit for bit "
                         "(`verified` in the line); default: cfg5 only")
    ap.add_argument("--pool-regions", type=int, default=2, help="--placement pool: regions to alternate between (0 = all found)")
    ap.add_argument("--pool-gib", type=float, default=0.0,
                    help="--placement pool: size of the arena in GiB (0 = all free memory but a margin, less what the "
                         "state-pool leg keeps in plain memory)")
    ap.add_argument("--settle-s", type=float, default=-1.0,
                    help="seconds to wait after device memory went back to the driver (an arena smaller than the free "
                         "memory; a child process that has exited) before anything is measured or probed: for about 3 s "
                         "after a release of tens of GB every kernel runs 0.7 %% slower (75.44 against 74.92 ms per step "
                         "with 80 GiB released, fresh machines, twice each; 74.94 after 3 s).  -1: 4 s after the arena, "
                         "8 s after a child that held the whole workload")
    ap.add_argument("--pool-chunk-mb", type=int, default=0, help="--placement pool: chunk size (0 = the library's 64)")
    ap.add_argument("--pool-slab-mb", type=int, default=0, help="--placement pool: unit of the region scan, 512 ... 4096 (0 = the library's 1024)")
    ap.add_argument("--grads-one-region", type=int, default=0,
                    help="--placement pool: 1 = gradient buffers (read only in every kernel) come from the part of the "
                         "arena behind the alternation, i.e. from one region")
    ap.add_argument("--others", type=int, default=-1,
                    help="1: after the main workload, run BASELINE's configs 1-4 for a few steps each and report them as "
                         "other_configs; default: only when the workload is cfg5 at full scale")
    ap.add_argument("--others-steps", type=int, default=0,
                    help="timed steps of each of the other configurations (0 = what the configuration states: 10, 20, 20, 100)")
    ap.add_argument("--ceiling", type=int, default=1, help="0: skip the bare probes (roofline.measured_ceiling)")
    ap.add_argument("--variants", type=int, default=1,
                    help="cfg5: 0 = skip the same step done the other ways (deferred accumulation, the other --fold-last)")
    ap.add_argument("--spread-block-mb", type=int, default=0, help="--placement spread: block size (0 = the library's 64)")
    ap.add_argument("--spread-keep", type=int, default=0, help="--placement spread: every n-th block is kept (0 = 3)")
    ap.add_argument("--micro", type=int, default=4,
                    help="cfg5-deferred and the engine workloads: micro-batches per optimizer step (deferred: up to 8)")
    ap.add_argument("--defer", type=int, default=0,
                    help="engine workloads: 1 = defer_accumulation (four resident micro-batches, no accumulation "
                         "buffer, summed in registers by the applying call)")
    ap.add_argument("--async-engine", type=int, default=0,
                    help="grpo-engine: 1 = mxopt_engine_micro_batch_async (no read-back per micro-batch; settled once per step)")
    ap.add_argument("--fold-last", type=int, default=1,
                    help="cfg5: 1 = the last micro-batch is measured (norm) but folded into the update instead of "
                         "being written to the accumulation buffer; 0 = four plain accumulation passes")
    return ap.parse_args()


# ----------------------------------------------------------------------------------------
# workloads
# ----------------------------------------------------------------------------------------

def tensor_sizes(args):
    from mxopt.qwen3_shapes import QWEN3, numel, param_list
    model = {"cfg1": "0.6B", "cfg1-update-single": "0.6B", "cfg1-update-many": "0.6B", "cfg2": "1.7B", "cfg3-sgd": "4B", "cfg3-rmsprop": "4B", "cfg3-sgd-deferred": "4B", "cfg3-rmsprop-deferred": "4B", "cfg5": "8B", "cfg5-deferred": "8B", "grpo-engine": "8B", "sft-engine": "8B"}.get(args.workload)
    if model:
        sizes = []
        for _, shape in param_list(QWEN3[model]):
            if args.scale != 1.0 and len(shape) == 2:
                shape = (max(1, int(shape[0] * args.scale)), shape[1])
            sizes.append(numel(shape))
        return sizes, f"qwen3-{model.lower()}"
    if args.workload == "copy":
        return [int((1 << 30) * args.scale)], "one-flat-f32-tensor"
    if args.workload == "probes":
        return [max(4096, int((1 << 30) * args.scale) // 4096 * 4096)], "four-flat-f32-streams"
    import numpy as np
    rng = np.random.default_rng(0x5EED0001)
    sizes = np.floor(np.exp(rng.uniform(np.log(64), np.log(65536), 10000))).astype(np.int64).tolist()
    if args.workload == "cfg4-flat":
        return [int(sum(sizes))], "one-flat-tensor-of-cfg4-size"
    return sizes, "10000-small-tensors"


class Workload:
    """Holds device buffers + tables and knows how to run one step and what it costs."""

    def __init__(self, args, torch, mx, ctx, pool=None):
        self.args, self.torch, self.mx = args, torch, mx
        self.ctx, self.pool = ctx, pool
        self.sizes, self.list_name = tensor_sizes(args)
        self.n = int(sum(self.sizes))
        self.kernel_events = {}     # kernel name -> list of (start, end) events
        self.res = self.ctx.norm_result()
        self.mem_pool = pool.torch_pool() if pool is not None else None   # torch allocates from the arena through it
        # state-pool: only moments and accumulation buffers (what the library's own objects allocate through
        # mxopt_set_state_pool) come from the arena; parameters and gradients are the host's and lie in plain memory
        self.arena_kinds = (() if pool is None else ("state",) if args.placement == "state-pool"
                            else ("param", "grad", "state"))
        if args.placement == "spread":
            window = self.ctx.hbm_spread(args.spread_block_mb << 20, args.spread_keep)
        else:
            window = contextlib.nullcontext()
        with window:
            getattr(self, "_setup_" + args.workload.replace("-", "_"))()
            torch.cuda.synchronize()

    @contextlib.contextmanager
    def _window(self, kind):
        """Where buffers of this kind ("param", "grad", "state") are allocated."""
        if kind not in self.arena_kinds:
            yield
            return
        # gradient buffers are only ever read: with --grads-one-region they come from the part of the arena that
        # lies behind the alternation (one region at a time), where read-only passes run a few per cent faster
        one_region = kind == "grad" and getattr(self.args, "grads_one_region", 0)
        if one_region:
            self.mx.HbmPool.hook_kind(self.mx.HBM_ONE_REGION)
        try:
            with self.torch.cuda.use_mem_pool(self.mem_pool):
                yield
        finally:
            if one_region:
                self.mx.HbmPool.hook_kind(self.mx.HBM_INTERLEAVED)

    def free_bytes(self, kind="state"):
        """Device memory this workload may still take for buffers of that kind."""
        if kind in self.arena_kinds:
            i = self.pool.info()
            return i.capacity_bytes - i.used_bytes
        return self.torch.cuda.mem_get_info()[0]

    def close(self):
        """Gives the buffers back (to the arena, or to the driver)."""
        self.torch.cuda.synchronize()
        for k in list(vars(self)):
            if k not in ("args", "torch", "mx", "ctx", "pool", "n", "sizes", "list_name"):
                delattr(self, k)
        import gc
        gc.collect()
        self.torch.cuda.empty_cache()

    # -- helpers
    SEED = 0x5EED0001
    CONFIG_ID = {"cfg1": 1, "cfg1-update-single": 1, "cfg1-update-many": 1, "cfg2": 2, "cfg3-sgd": 3, "cfg3-rmsprop": 3,
                 "cfg3-sgd-deferred": 3, "cfg3-rmsprop-deferred": 3,
                 "cfg4": 4, "cfg4-flat": 4, "cfg5": 5, "cfg5-deferred": 5, "copy": 6, "grpo-engine": 7, "sft-engine": 8,
                 "probes": 9}

    def _fill(self, views, stream_id, dist, a, b=0.0):
        """Counter-based synthetic data (mxopt_fill_synthetic): every element is a function of
        (seed, configuration, stream, tensor, index), so a host program can regenerate any slice."""
        cfg = self.CONFIG_ID[self.args.workload]
        for i, v in enumerate(views):
            self.ctx.fill_synthetic(v, self.mx.synthetic_key(self.SEED, cfg, 0, stream_id, i), dist, a, b)

    # one list of tensors per stream, either separately allocated or carved out of one slab
    def _carve(self, dtype, kind):
        t = self.torch
        mode = getattr(self.args, "alloc", "tensor")
        with self._window(kind):
            if mode == "tensor":
                return None, [t.empty(n, dtype=dtype, device="cuda") for n in self.sizes]
            offs, total = [], 0
            for n in self.sizes:
                offs.append(total)
                # slab: 512 B (bf16) / 1 KiB (f32) alignment; packed: back to back, natural alignment only
                total += (n + 255) // 256 * 256 if mode == "slab" else n
            slab = t.empty(max(total, 1), dtype=dtype, device="cuda")
            return slab, [slab[o:o + n] for o, n in zip(offs, self.sizes)]

    def _randn_list(self, dtype, std, outliers=False, kind="grad"):
        """A list of tensors with bell-shaped values of standard deviation `std` (optionally 1 % x100)."""
        _, views = self._carve(dtype, kind)
        self._next_stream = getattr(self, "_next_stream", 0) + 1
        mx = self.mx
        dist = mx.SYNTH_GAUSSIAN_OUTLIERS if outliers else mx.SYNTH_GAUSSIAN
        self._fill(views, self._next_stream, dist, std, 100.0)
        # what a host program needs to regenerate any slice of this stream: (stream id, distribution, a, b)
        self.stream_specs = getattr(self, "stream_specs", {})
        self.stream_specs[self._next_stream] = (dist, std, 100.0)
        return views

    def _zeros_list(self, kind="state"):
        slab, views = self._carve(self.torch.float32, kind)
        if slab is not None:
            slab.zero_()
        else:
            for v in views:
                v.zero_()
        return views

    def _empty_list(self, dtype, kind="state"):
        return self._carve(dtype, kind)[1]

    def _timed(self, name, fn):
        s = self.torch.cuda.Event(enable_timing=True)
        e = self.torch.cuda.Event(enable_timing=True)
        s.record(self.ctx.stream)
        fn()
        e.record(self.ctx.stream)
        self.kernel_events.setdefault(name, []).append((s, e))

    def kernel_ms(self, name):
        ev = self.kernel_events.get(name, [])
        return [s.elapsed_time(e) for s, e in ev]

    # -- cfg5: 4x accumulate (bf16 -> f32), clip 1.0, AdamW bf16 p / f32 m,v
    def _setup_cfg5(self):
        t, mx = self.torch, self.mx
        bf = t.bfloat16
        self.n_micro = 4
        if "grad" in self.arena_kinds or not self.arena_kinds:    # everything from one place
            n_gbuf = 4 if self.free_bytes("grad") > self.n * (2 + 8 + 4) + 4 * self.n * 2 + (3 << 30) else 1
        else:                                                     # parameters and gradients in plain memory
            n_gbuf = 4 if self.free_bytes("grad") > self.n * 2 + 4 * self.n * 2 + (3 << 30) else 1
        self.p = self._randn_list(bf, 0.02, kind="param")
        self.m = self._zeros_list()
        self.v = self._zeros_list()
        self.acc = self._empty_list(t.float32)
        self.g = [self._randn_list(bf, 1e-3) for _ in range(n_gbuf)]
        self.t_acc = [self.ctx.table([mx.TensorSpec(g=g, g_out=a) for g, a in zip(gk, self.acc)]) for gk in self.g]
        self.t_upd = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, m=m, v=v)
                                     for p, a, m, v in zip(self.p, self.acc, self.m, self.v)])
        self.hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
        self.prep = mx.make_prep(scale=self.res)
        self.dtype = "f32"
        self.storage = "bf16 parameters and gradients, float32 accumulation buffer and moments"
        self.fold_last = bool(self.args.fold_last)
        # folded: the update reads the accumulation buffer AND the last micro-batch (24 + 2 B/elem); the last
        # accumulation pass only measures the norm (6 B/elem): 6 + 10 + 10 + 6 + 26 = 58 B/elem/step.
        # unfolded: four plain accumulation passes, 6 + 3 * 10 + 24 = 60 B/elem/step
        last = self.g[(self.n_micro - 1) % n_gbuf]
        self.t_upd_pending = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=a, g_out=gl, m=m, v=v)
                                             for p, a, gl, m, v in zip(self.p, self.acc, last, self.m, self.v)])
        if self.fold_last:
            self.bytes_per_elem = {"accumulate_first": 6, "accumulate": 10, "accumulate_norm_only": 6, "adamw": 26}
            self.step_bytes_per_elem = 6 + 10 * 2 + 6 + 26
        else:
            self.bytes_per_elem = {"accumulate_first": 6, "accumulate": 10, "accumulate_sumsq": 10, "adamw": 24}
            self.step_bytes_per_elem = 6 + 10 * 3 + 24
        self.dominant = "adamw"
        self.note = f"{n_gbuf} resident micro-gradient buffer(s); fold_last={int(self.fold_last)}"
        if n_gbuf == self.n_micro:
            # the same buffers without the accumulation buffer: reported beside the headline figure
            self.t_deferred = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v)
                                              for p, g, m, v in zip(self.p, self.g[0], self.m, self.v)])
            self.t_deferred.set_pending(self.g[1:])

    def deferred_variant(self, steps):
        """Config 5 with the micro-batches summed in registers (no accumulation buffer), same buffers."""
        if not hasattr(self, "t_deferred"):
            return None
        t, c = self.torch, self.ctx

        def one():
            c.norm_with_pending_list(self.t_deferred, self.res, max_norm=1.0)
            c.adam_with_pending_list(self.t_deferred, self.hp, self.prep)
        one()
        t.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one()
        t.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        self.deferred_steps_done = steps + 1
        return {"value": round(1.0 / dt, 4), "unit": "steps/s", "ms_per_step": round(dt * 1e3, 4),
                "bytes_per_elem_per_step": 36, "step_hbm_gbps": round(36 * self.n / dt / 1e9, 1),
                "note": "same buffers and result; the four resident micro-batches are added in registers by the norm "
                        "pass (8 B/elem) and by AdamW (28 B/elem) instead of being accumulated into the float32 buffer"}

    def _step_cfg5(self, fold_last=None):
        c = self.ctx
        fold_last = self.fold_last if fold_last is None else fold_last
        for k in range(self.n_micro):
            tab = self.t_acc[k % len(self.t_acc)]
            last = k == self.n_micro - 1
            if last and fold_last:
                self._timed("accumulate_norm_only", lambda: c.accumulate_norm_only(tab, self.res, max_norm=1.0))
                continue
            name = "accumulate_first" if k == 0 else ("accumulate_sumsq" if last else "accumulate")
            self._timed(name, lambda: c.accumulate(tab, first=(k == 0), out=self.res if last else None,
                                                   max_norm=1.0))
        if fold_last:
            self._timed("adamw", lambda: c.adam_with_pending(self.t_upd_pending, self.hp, self.prep))
        else:
            self._timed("adamw", lambda: c.adam(self.t_upd, self.hp, self.prep))

    def other_fold_variant(self, steps):
        """Config 5 on the same buffers with the other --fold-last setting (same result, 60 instead of 58 B/elem
        or the reverse)."""
        t = self.torch
        fold = not self.fold_last
        bpe = 58 if fold else 60
        self._step_cfg5(fold)
        t.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            self._step_cfg5(fold)
        t.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        self.other_fold_steps_done = steps + 1
        return {"fold_last": int(fold), "value": round(1.0 / dt, 4), "unit": "steps/s", "ms_per_step": round(dt * 1e3, 4),
                "bytes_per_elem_per_step": bpe, "step_hbm_gbps": round(bpe * self.n / dt / 1e9, 1),
                "note": ("four plain accumulation passes (6 + 3 x 10 B/elem), the last carrying the sum of squares, and "
                         "AdamW from the buffer alone (24 B/elem): the step as counted at 60 B/elem") if not fold else
                        "the last micro-batch only measured (6 B/elem) and added again inside AdamW (26 B/elem)"}

    # -- cfg5 without its accumulation buffer: the four micro-batches stay resident and are summed in
    #    registers, in arrival order, by the norm pass (8 B/elem) and by the update (18 + 10 B/elem)
    def _setup_cfg5_deferred(self):
        t, mx = self.torch, self.mx
        bf = t.bfloat16
        self.n_micro = self.args.micro
        self.p = self._randn_list(bf, 0.02, kind="param")
        self.m = self._zeros_list()
        self.v = self._zeros_list()
        self.g = [self._randn_list(bf, 1e-3) for _ in range(self.n_micro)]
        self.t_upd = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v)
                                     for p, g, m, v in zip(self.p, self.g[0], self.m, self.v)])
        self.t_upd.set_pending(self.g[1:])
        self.hp = mx.adam_hp(5e-6, 0.9, 0.999, 1e-8, 0.01)
        self.prep = mx.make_prep(scale=self.res)
        self.dtype = "f32"
        self.storage = "bf16 parameters and gradients, float32 moments, no accumulation buffer"
        self.bytes_per_elem = {"norm_of_sum": 2 * self.n_micro, "adamw": 2 * self.n_micro + 10 + 10}
        self.step_bytes_per_elem = sum(self.bytes_per_elem.values())
        self.dominant = "adamw"
        self.note = (f"{self.n_micro} resident micro-batches summed in registers (float32, arrival order) by the norm "
                     "pass and by AdamW")

    def _step_cfg5_deferred(self):
        c = self.ctx
        self._timed("norm_of_sum", lambda: c.norm_with_pending_list(self.t_upd, self.res, max_norm=1.0))
        self._timed("adamw", lambda: c.adam_with_pending_list(self.t_upd, self.hp, self.prep))

    # -- cfg1: fp32 AdamW
    def _setup_cfg1(self):
        t, mx = self.torch, self.mx
        self.p = self._randn_list(t.float32, 0.02, kind="param")
        self.g = self._randn_list(t.float32, 1e-3)
        self.m = self._zeros_list()
        self.v = self._zeros_list()
        self.t_upd = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v)
                                     for p, g, m, v in zip(self.p, self.g, self.m, self.v)])
        self.hp = mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01)
        self.dtype = "f32"
        self.bytes_per_elem = {"adamw": 28}
        self.step_bytes_per_elem = 28
        self.dominant = "adamw"
        self.note = ""

    def _step_cfg1(self):
        self._timed("adamw", lambda: self.ctx.adam(self.t_upd, self.hp))

    # -- cfg1 through the optimizer object, as the reference's callers use it: one updateSingle per tensor
    #    returning a new array (310 launches per step), or the same loop as one update_many call in place
    def _setup_cfg1_update_single(self):
        from mxopt.qwen3_shapes import QWEN3, param_list
        self._setup_cfg1()
        self.names = [name for name, _ in param_list(QWEN3["0.6B"])]
        self.opt = self.mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, ctx=self.ctx)
        self.bytes_per_elem = {"adamw_object": 28}
        self.dominant = "adamw_object"
        self.note = "AdamW object through ctypes: " + self.args.workload.split("-", 1)[1]

    _setup_cfg1_update_many = _setup_cfg1_update_single

    def _step_cfg1_update_single(self):
        def loop():
            self.p = [self.opt.update_single(nm, p, g) for nm, p, g in zip(self.names, self.p, self.g)]
        self._timed("adamw_object", loop)

    def _step_cfg1_update_many(self):
        self._timed("adamw_object", lambda: self.opt.update_many(self.names, self.p, self.g, outs=self.p))

    # -- cfg2 / cfg4: bf16 p,g + f32 m,v AdamW with a separate norm pass
    def _setup_cfg2(self, lr=5e-6, wd=0.01, gstd=1e-3, uniform_p=False):
        t, mx = self.torch, self.mx
        bf = t.bfloat16
        if uniform_p:
            self.p = self._carve(bf, "param")[1]
            self._fill(self.p, 100, mx.SYNTH_UNIFORM, 0.9, 1.1)
        else:
            self.p = self._randn_list(bf, 0.02, kind="param")
        self.g = self._randn_list(bf, gstd, outliers=self.args.workload == "cfg2")   # cfg2: 1 % of the elements x100
        self.m = self._zeros_list()
        self.v = self._zeros_list()
        self.t_g = self.ctx.table([mx.TensorSpec(g=g) for g in self.g])
        self.t_upd = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v)
                                     for p, g, m, v in zip(self.p, self.g, self.m, self.v)])
        self.hp = mx.adam_hp(lr, 0.9, 0.999, 1e-8, wd)
        self.prep = mx.make_prep(scale=self.res)
        self.dtype = "f32"
        self.storage = "bf16 parameters and gradients, float32 moments"
        self.bytes_per_elem = {"global_norm": 2, "adamw": 22}
        self.step_bytes_per_elem = 24
        self.dominant = "adamw"
        self.note = ""

    def _step_cfg2(self):
        self._timed("global_norm", lambda: self.ctx.global_norm(self.t_g, self.res, max_norm=1.0))
        self._timed("adamw", lambda: self.ctx.adam(self.t_upd, self.hp, self.prep))

    def _setup_cfg4(self):
        self._setup_cfg2(lr=1e-3, wd=0.0, gstd=1e-2, uniform_p=True)
        self.graph_variant = self._graph_variant   # config 4 exists to show launch overhead: also timed from a HIP graph

    def _graph_variant(self, steps):
        """The same step (norm pass, its one-workgroup second pass, AdamW) on a side stream, eager and replayed
        from a HIP graph: three launches whose gaps are a measurable part of a 0.4 ms step."""
        t, mx = self.torch, self.mx
        s = t.cuda.Stream()
        ctx = mx.Context(stream=s)
        res = ctx.norm_result()
        t_g = ctx.table([mx.TensorSpec(g=g) for g in self.g])
        t_upd = ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, m=m, v=v)
                           for p, g, m, v in zip(self.p, self.g, self.m, self.v)])
        prep = mx.make_prep(scale=res)

        def one():
            ctx.global_norm(t_g, res, max_norm=1.0)
            ctx.adam(t_upd, self.hp, prep)
        t.cuda.synchronize()
        with t.cuda.stream(s):
            one()                                   # warm-up: the partial-sum buffer exists before the capture
            s.synchronize()
            graph = t.cuda.CUDAGraph()
            with t.cuda.graph(graph, stream=s):
                one()
            out = {}
            for name, fn in (("eager_ms_per_step", one), ("graph_ms_per_step", graph.replay)):
                for _ in range(3):
                    fn()
                s.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    fn()
                s.synchronize()
                out[name] = round((time.perf_counter() - t0) * 1e3 / steps, 4)
        out["graph_step_hbm_gbps"] = round(self.step_bytes_per_elem * self.n / (out["graph_ms_per_step"] * 1e-3) / 1e9, 1)
        out["what"] = "mxopt_global_norm + mxopt_adam captured once on a side stream and replayed; same buffers"
        del graph
        t_g.close(); t_upd.close(); ctx.close()
        return out

    _step_cfg4 = _step_cfg2
    _setup_cfg4_flat = _setup_cfg4
    _step_cfg4_flat = _step_cfg2

    # -- cfg3: fp32 SGD / RMSprop
    def _setup_cfg3(self):
        t, mx = self.torch, self.mx
        self.p = self._randn_list(t.float32, 0.02, kind="param")
        self.g = self._randn_list(t.float32, 1e-3)
        self.v = self._zeros_list()
        self.t_upd = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v)
                                     for p, g, v in zip(self.p, self.g, self.v)])
        self.dtype = "f32"
        self.step_bytes_per_elem = 20
        self.note = ""

    def _setup_cfg3_sgd(self):
        self._setup_cfg3()
        self.hp = self.mx.sgd_hp(1e-4, 0.9, 1e-4, 0.0, False)
        self.bytes_per_elem = {"sgd": 20}
        self.dominant = "sgd"

    def _step_cfg3_sgd(self):
        self._timed("sgd", lambda: self.ctx.sgd(self.t_upd, self.hp))

    def _setup_cfg3_rmsprop(self):
        self._setup_cfg3()
        self.hp = self.mx.rmsprop_hp(1e-4, 0.99, 1e-8, 0.0)
        self.bytes_per_elem = {"rmsprop": 20}
        self.dominant = "rmsprop"

    def _step_cfg3_rmsprop(self):
        self._timed("rmsprop", lambda: self.ctx.rmsprop(self.t_upd, self.hp))

    # -- cfg3's optimizers over --micro un-summed float32 micro-batches (deferred accumulation): the norm of the sum
    #    (4k B/elem, read only) and the update over k + 2 read and 2 write streams (4k + 16 B/elem)
    def _setup_cfg3_deferred(self, which):
        t, mx = self.torch, self.mx
        k = self.n_micro = self.args.micro
        self.p = self._randn_list(t.float32, 0.02, kind="param")
        self.g = [self._randn_list(t.float32, 1e-3) for _ in range(k)]
        self.v = self._zeros_list()
        self.t_upd = self.ctx.table([mx.TensorSpec(p=p, p_out=p, g=g, v=v) for p, g, v in zip(self.p, self.g[0], self.v)])
        self.t_upd.set_pending(self.g[1:])
        self.prep = mx.make_prep(scale=self.res)
        self.hp = mx.sgd_hp(1e-4, 0.9, 1e-4, 0.0, False) if which == "sgd" else mx.rmsprop_hp(1e-4, 0.99, 1e-8, 0.0)
        self.dtype = "f32"
        self.bytes_per_elem = {"norm_of_sum": 4 * k, which: 4 * k + 16}
        self.step_bytes_per_elem = 8 * k + 16
        self.dominant = which
        self.note = f"{k} resident float32 micro-batches summed in registers by the norm pass and by the update; clip 1.0"

    def _setup_cfg3_sgd_deferred(self):
        self._setup_cfg3_deferred("sgd")

    def _setup_cfg3_rmsprop_deferred(self):
        self._setup_cfg3_deferred("rmsprop")

    def _step_cfg3_sgd_deferred(self):
        c = self.ctx
        self._timed("norm_of_sum", lambda: c.norm_with_pending_list(self.t_upd, self.res, max_norm=1.0))
        self._timed("sgd", lambda: c.sgd_with_pending_list(self.t_upd, self.hp, self.prep))

    def _step_cfg3_rmsprop_deferred(self):
        c = self.ctx
        self._timed("norm_of_sum", lambda: c.norm_with_pending_list(self.t_upd, self.res, max_norm=1.0))
        self._timed("rmsprop", lambda: c.rmsprop_with_pending_list(self.t_upd, self.hp, self.prep))

    # -- the engines' optimizer side (include/mxopt_engine.h) on the 8B list: 4 micro-batches of bf16
    #    gradients per optimizer step, bf16 parameters updated in place by the reference's plain SGD
    def _setup_engine(self, kind):
        from mxopt.qwen3_shapes import QWEN3, param_list
        t, mx = self.torch, self.mx
        bf = t.bfloat16
        self.names = [name for name, _ in param_list(QWEN3["8B"])]
        self.p = self._randn_list(bf, 0.02, kind="param")
        self.g = self._randn_list(bf, 1e-3)
        params = dict(zip(self.names, self.p))
        self.n_micro = N = self.args.micro
        defer = bool(self.args.defer)
        # deferred accumulation reads every micro-batch of the cycle at the end: they must all be resident
        self.micro = [dict(zip(self.names, self.g))]
        # (with more than eight in a cycle the engine adds the oldest into its float32 buffers as later ones
        # arrive; the synthetic buffers are never rewritten, so eight of them used in turn stand for any number)
        for _ in range(min(self.n_micro, mx.MAX_PENDING + 1) - 1 if defer else 0):
            self.micro.append(dict(zip(self.names, self._randn_list(bf, 1e-3))))
        if kind == "grpo":   # clamp 1.0 + clip 1.0 per micro-batch, float32 accumulation, p -= lr/N * acc
            self.engine = mx.GRPOEngineOptimizerSide(params, learning_rate=1e-6, gradient_accumulation_steps=N,
                                                     defer_accumulation=defer, ctx=self.ctx)
            if defer:
                self.bytes_per_elem = {"micro_batch_first": 2, "micro_batch": 2, "micro_batch_apply": 2 + N * 2 + 4}
                self.note = ("per micro-batch: validity+norm of clamp(g) (2 B), 32-byte read-back; the last call adds "
                             "sum_j clip_j(clamp(g_j)) in registers and applies lr/N (12 B)")
            else:
                self.bytes_per_elem = {"micro_batch_first": 2 + 6, "micro_batch": 2 + 10, "micro_batch_apply": 2 + 10}
                self.note = "per micro-batch: validity+norm of clamp(g) (2 B), acc += clip(clamp(g)) (6/10 B), 32-byte read-back"
        else:                # acc += g in float32, last pass carries the norm of acc/N; p -= lr*(clip(acc/N) + wd*p)
            self.engine = mx.SFTEngineOptimizerSide(params, learning_rate=2e-5, gradient_accumulation_steps=N,
                                                    weight_decay=0.01, accumulate_in_f32=True,
                                                    defer_accumulation=defer, ctx=self.ctx)
            if defer:
                self.bytes_per_elem = {"micro_batch_apply": N * 2 + N * 2 + 4}
                self.note = ("micro-batches 1-3 only leave their addresses; the last call takes the norm of sum/N "
                             "(8 B, read only) and updates from the same four streams (12 B)")
            else:
                self.bytes_per_elem = {"micro_batch_first": 6, "micro_batch": 10, "micro_batch_apply": 6 + 10}
                self.note = "float32 accumulation buffer; last micro-batch: norm of (acc+g)/N read-only, then folded into the update"
        if N == 1:   # one micro-batch per step: norm of g (2 B), update straight from g (6 B), either engine
            self.bytes_per_elem = {"micro_batch_apply": 2 + 6}
        elif N == 2:
            self.bytes_per_elem.pop("micro_batch", None)
        self.step_bytes_per_elem = (self.bytes_per_elem.get("micro_batch_first", 0) +
                                    (N - 2) * self.bytes_per_elem.get("micro_batch", 0) +
                                    self.bytes_per_elem["micro_batch_apply"])
        if defer and N > mx.MAX_PENDING + 1:
            # the ninth micro-batch moves the two oldest into the float32 buffers (6 + 10 B), every later one
            # one more (10 B); the applying call reads that buffer and seven deferred streams
            spill = 6 + 10 * (N - mx.MAX_PENDING - 1)
            norms = 2 * N if kind == "grpo" else 4 + 2 * mx.MAX_PENDING
            apply = 4 + 2 * mx.MAX_PENDING + 4
            # the applying call first makes room for its own micro-batch (10 B), like every call after the eighth
            self.bytes_per_elem = {"micro_batch_apply": 10 + apply + (2 if kind == "grpo" else norms)}
            self.step_bytes_per_elem = spill + norms + apply
            self.note += "; more than eight micro-batches: the oldest are added into float32 buffers as later ones arrive"
        self.dominant = "micro_batch_apply"
        self.dtype = "f32"
        self.storage = ("bf16 parameters and gradients, no accumulation buffer" if defer
                        else "bf16 parameters and gradients, float32 accumulation buffer")

    def _setup_grpo_engine(self):
        self._setup_engine("grpo")

    def _setup_sft_engine(self):
        self._setup_engine("sft")

    def _step_grpo_engine(self):
        use_async = bool(getattr(self.args, "async_engine", 0)) and self.args.workload == "grpo-engine"
        for k in range(self.n_micro):
            name = "micro_batch_apply" if k == self.n_micro - 1 else ("micro_batch_first" if k == 0 else "micro_batch")
            call = self.engine.micro_batch_async if use_async else self.engine.micro_batch
            self._timed(name, lambda: call(self.micro[k % len(self.micro)]))

    _step_sft_engine = _step_grpo_engine

    # -- copy: g_out = g (float32, no pre-processing): the plain copy that calibrates HBM counters
    def _setup_copy(self):
        t, mx = self.torch, self.mx
        self.g = self._randn_list(t.float32, 1.0)
        with self._window("grad"):
            self.o = [t.empty_like(g) for g in self.g]
        self.t_copy = self.ctx.table([mx.TensorSpec(g=g, g_out=o) for g, o in zip(self.g, self.o)])
        self.dtype = "f32"
        self.bytes_per_elem = {"copy": 8}
        self.step_bytes_per_elem = 8
        self.dominant = "copy"
        self.note = "mxopt_grad_transform with no stage enabled"

    def _step_copy(self):
        self._timed("copy", lambda: self.ctx.grad_transform(self.t_copy, None))

    # -- probes: the bare streaming kernels (mxopt_probe_stream), one launch each per step: the measured
    #    ceilings of a read-only, a write-only, a copy and a 4-read/3-write pass on this memory
    def _setup_probes(self):
        t = self.torch
        with self._window("param"):
            self.streams = [t.zeros(self.n, dtype=t.float32, device="cuda") for _ in range(5)]
        # the deferred update's mix: four 2-byte gradient streams and a 2-byte parameter (halves of two of the
        # buffers, viewed as bf16), two 4-byte moments
        halves = [h for s in (self.streams[1], self.streams[4]) for h in s.view(t.bfloat16).chunk(2)]
        self.list_streams = (self.streams[0].view(t.bfloat16)[:self.n], self.streams[2], self.streams[3], halves)
        self.dtype = "u32"
        self.bytes_per_elem = {"probe_read": 4, "probe_write": 4, "probe_copy": 8, "probe_mix43": 28, "probe_list4": 28,
                               "probe_write_streaming": 4, "probe_copy_streaming": 8, "probe_mix43_streaming": 28,
                               "probe_list4_streaming": 28}
        self.step_bytes_per_elem = 140
        self.dominant = "probe_mix43"
        self.note = "bare kernels: no table, no tails, no arithmetic; mix43 = float32 AdamW's four read and three write streams"

    def _step_probes(self):
        c, mx, s = self.ctx, self.mx, self.streams
        self._timed("probe_read", lambda: c.probe_stream(mx.PROBE_READ, s[0]))
        self._timed("probe_write", lambda: c.probe_stream(mx.PROBE_WRITE, s[1]))
        self._timed("probe_copy", lambda: c.probe_stream(mx.PROBE_COPY, s[0], s[1]))
        self._timed("probe_mix43", lambda: c.probe_stream(mx.PROBE_MIX43, *s[:4]))
        p16, m, v, gs = self.list_streams
        self._timed("probe_list4", lambda: c.probe_list(p16, m, v, gs))
        # the same streams the way the update kernels access them by default: streaming-hint loads and stores
        nt = mx.PROBE_STREAMING
        self._timed("probe_write_streaming", lambda: c.probe_stream(mx.PROBE_WRITE | nt, s[1]))
        self._timed("probe_copy_streaming", lambda: c.probe_stream(mx.PROBE_COPY | nt, s[0], s[1]))
        self._timed("probe_mix43_streaming", lambda: c.probe_stream(mx.PROBE_MIX43 | nt, *s[:4]))
        self._timed("probe_list4_streaming", lambda: c.probe_list(p16, m, v, gs, streaming=True))

    def step(self):
        getattr(self, "_step_" + self.args.workload.replace("-", "_"))()
        self.steps_done = getattr(self, "steps_done", 0) + 1


# ----------------------------------------------------------------------------------------
# Self-check of the timed configuration (outside the timed region; the oracle is the checker only)
# ----------------------------------------------------------------------------------------

def verify_cfg5(wl, segments, window=256 * 1024, n_large=12):
    """Recomputes, on the host, seeded windows of config 5's parameters and moments for exactly the optimizer
    steps that ran on the device, and compares them bit for bit with what the device holds now.

    The inputs are regenerated from the generator's host twin (no device value is read for them), pushed through
    the C twin of the oracle -- four float32 accumulations in arrival order, AdamW on the clipped sum, bf16
    write-back -- once per step.  `segments` is [(steps, clip factor)]: the factor is the device's own (checked
    here against the reference's float32 scalar chain on the device's sum of squares, and the norm against a
    float64 reduction by torch over the device buffers at rel 1e-5).  Windows: every tensor of at most 64 Ki
    elements in full, and head, tail and an odd interior offset of `n_large` large tensors spread over the list
    (the largest among them)."""
    import math
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import mxopt_oracle as O
    import oracle_c_binding as B
    torch, mx = wl.torch, wl.mx
    oc = B.load()
    t0 = time.perf_counter()
    sizes, cfg = wl.sizes, wl.CONFIG_ID[wl.args.workload]
    n_gbuf = len(wl.g)

    def host(stream, i, dtype, off, length):
        dist, a, b = wl.stream_specs[stream]
        return oc.fill_synthetic(length, dtype, mx.synthetic_key(wl.SEED, cfg, 0, stream, i), dist, a, b, first_index=off)

    def bits(t):
        t = t.cpu().contiguous()
        return (t.view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.bfloat16
                else t.numpy().view(np.uint32))

    large = [i for i, n in enumerate(sizes) if n > 65536]
    picked = sorted(set([large[(len(large) - 1) * k // (n_large - 1)] for k in range(n_large)] +
                        [max(range(len(sizes)), key=lambda i: sizes[i])]))
    windows = [(i, 0, n) for i, n in enumerate(sizes) if 0 < n <= 65536]
    for i in picked:
        n, w = sizes[i], min(window, sizes[i])
        mid = (n // 2) | 1                       # an odd element offset: not 16-byte aligned in any stream
        for off in sorted({0, min(mid, n - w), n - w}):
            windows.append((i, off, w))

    # the norm the device took, against an independent float64 reduction of the same device buffers
    total_t = torch.zeros((), dtype=torch.float64, device="cuda")
    piece = 1 << 26
    for i, n in enumerate(sizes):
        for s in range(0, n, piece):
            e = min(n, s + piece)
            x = wl.g[0][i][s:e].float()
            for k in range(1, wl.n_micro):
                x += wl.g[k % n_gbuf][i][s:e].float()
            total_t += x.double().square_().sum()
    total = float(total_t)
    norm_rel = 0.0
    factor_ok = True
    for _, scale, sumsq in segments:
        norm_rel = max(norm_rel, abs(math.sqrt(sumsq) - math.sqrt(total)) / math.sqrt(total))
        _, want = O.norm_scale_c1(sumsq, 1.0)
        factor_ok = factor_ok and np.float32(scale) == want

    elements = mismatches = 0
    first_bad = None
    for i, off, w in windows:
        p = host(1, i, "bf16", off, w)
        gs = [host(2 + (k % n_gbuf), i, "bf16", off, w) for k in range(wl.n_micro)]
        m, v = np.zeros(w, np.float32), np.zeros(w, np.float32)
        acc = np.empty(w, np.float32)
        for k, g in enumerate(gs):
            oc.accumulate_f32(acc, g, k == 0)
        for steps, scale, _ in segments:
            args = B.adam_args(5e-6, 0.9, 0.999, 1e-8, 0.01, scale=float(scale))
            for _ in range(steps):
                p = oc.f32_to_bf16(oc.adam(p, acc, m, v, args, fused=True))
        for name, want, got in (("p", p, bits(wl.p[i][off:off + w])), ("m", m.view(np.uint32), bits(wl.m[i][off:off + w])),
                                ("v", v.view(np.uint32), bits(wl.v[i][off:off + w]))):
            bad = int(np.count_nonzero(want.view(got.dtype) != got))
            mismatches += bad
            if bad and first_bad is None:
                first_bad = f"{name} of tensor {i} at offset {off}"
        elements += 3 * w
    ok = mismatches == 0 and factor_ok and norm_rel <= 1e-5
    out = {"windows": len(windows), "elements": elements, "bit_exact": mismatches == 0,
           "optimizer_steps_checked": sum(s for s, _, _ in segments),
           "clip_factor_is_reference_chain_on_device_sum": bool(factor_ok),
           "norm_rel_err_vs_torch_float64": float(f"{norm_rel:.3g}"), "ok": bool(ok),
           "seconds": round(time.perf_counter() - t0, 2),
           "what": "p, m, v windows recomputed by the C twin of the oracle from regenerated inputs for every step "
                   "this process ran (warm-up, timed, and the deferred variant's), compared bit for bit"}
    if first_bad:
        out["first_mismatch"] = first_bad
    return out


# ----------------------------------------------------------------------------------------
# CPU baseline: the oracle's C twin (un-fused op chain) on a bounded sample
# ----------------------------------------------------------------------------------------

def cpu_baseline(args, n_total):
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle_c_binding as B
    import mxopt
    oc = B.load()
    S = int(min(args.cpu_sample, n_total))
    w = args.workload
    f32 = np.float32
    cfg = Workload.CONFIG_ID[w]
    GAUSS, GAUSS_OUT, UNIFORM = mxopt.SYNTH_GAUSSIAN, mxopt.SYNTH_GAUSSIAN_OUTLIERS, mxopt.SYNTH_UNIFORM

    def gen(stream, dtype, dist, a, b=100.0):
        """The first S elements of stream `stream` as the device workload holds them, tensor after tensor
        (the library generator's host twin; same keys as Workload._fill)."""
        sizes, _ = tensor_sizes(args)
        out = np.empty(S, np.uint16 if dtype == "bf16" else f32)
        pos = 0
        for i, n in enumerate(sizes):
            if pos >= S:
                break
            take = min(n, S - pos)
            out[pos:pos + take] = oc.fill_synthetic(take, dtype, mxopt.synthetic_key(Workload.SEED, cfg, 0, stream, i), dist, a, b)
            pos += take
        return out

    m, v = np.zeros(S, f32), np.zeros(S, f32)

    def timeit(fn, reps=2):
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        return best

    fused_s = None
    if w in ("cfg5", "cfg5-deferred", "cfg2", "cfg4", "cfg4-flat"):
        five = w in ("cfg5", "cfg5-deferred")
        if w in ("cfg4", "cfg4-flat"):
            p = gen(100, "bf16", UNIFORM, 0.9, 1.1)
            gs = [gen(1, "bf16", GAUSS, 1e-2)]
        else:
            p = gen(1, "bf16", GAUSS, 0.02)
            gs = ([gen(2 + k, "bf16", GAUSS, 1e-3) for k in range(4)] if five
                  else [gen(2, "bf16", GAUSS_OUT, 1e-3)])
        acc = np.empty(S, f32)
        lr, wd = (5e-6, 0.01) if w not in ("cfg4", "cfg4-flat") else (1e-3, 0.0)

        def step(fused):
            src = gs[0]
            if five:
                for k in range(4):
                    oc.accumulate_f32(acc, gs[k], k == 0)
                src = acc
            sumsq = oc.sumsq(src)
            scale = float(min(np.float32(1.0) / (np.float32(np.sqrt(sumsq)) + np.float32(1e-6)), np.float32(1.0)))
            a = B.adam_args(lr, 0.9, 0.999, 1e-8, wd, scale=scale)
            out = oc.adam(p, src, m, v, a, fused=fused)
            oc.f32_to_bf16(out)     # parameters are kept in bf16
        what = ("4x accumulate + sumsq + scale + AdamW as 13 separate float32 passes (adamw.rs:84-116) + bf16 cast"
                if five else "sumsq + scale + AdamW as 13 separate float32 passes + bf16 cast")
        t_unfused = timeit(lambda: step(False))
        fused_s = timeit(lambda: step(True))
    elif w.startswith("cfg1"):
        p32, g32 = gen(1, "f32", GAUSS, 0.02), gen(2, "f32", GAUSS, 1e-3)
        a = B.adam_args(1e-3, 0.9, 0.999, 1e-8, 0.01)
        t_unfused = timeit(lambda: oc.adam(p32, g32, m, v, a, fused=False))
        fused_s = timeit(lambda: oc.adam(p32, g32, m, v, a, fused=True))
        what = "AdamW as 13 separate float32 passes (adamw.rs:84-116)"
    elif w.startswith("cfg3-sgd"):
        p32, g32 = gen(1, "f32", GAUSS, 0.02), gen(2, "f32", GAUSS, 1e-3)
        fl = lambda x: float(np.float32(x))
        a = B.SgdArgs(lr=fl(1e-4), momentum=fl(0.9), one_minus_damp=1.0, wd=fl(1e-4), has_wd=1, has_momentum=1,
                      nesterov=0, first=0)
        t_unfused = timeit(lambda: oc.sgd(p32, g32, v, a, fused=False))
        fused_s = timeit(lambda: oc.sgd(p32, g32, v, a, fused=True))
        what = "SGD+momentum+L2 as 7 separate float32 passes (sgd.rs:86-140)"
    else:
        p32, g32 = gen(1, "f32", GAUSS, 0.02), gen(2, "f32", GAUSS, 1e-3)
        fl = lambda x: float(np.float32(x))
        a = B.RmspropArgs(lr=fl(1e-4), alpha=fl(0.99), one_minus_alpha=fl(1.0 - 0.99), eps=fl(1e-8), wd=0.0, has_wd=0)
        t_unfused = timeit(lambda: oc.rmsprop(p32, g32, v, a, fused=False))
        fused_s = timeit(lambda: oc.rmsprop(p32, g32, v, a, fused=True))
        what = "RMSprop as 9 separate float32 passes (rmsprop.rs:69-93)"

    scale_up = n_total / S
    return {
        "value": 1.0 / (t_unfused * scale_up), "unit": "steps/s", "cores": oc.num_threads(), "kind": "port",
        "sample": f"the first {S} of {n_total} elements of the workload's own streams (the library generator's host "
                  f"twin regenerates what the device holds: same seed, keys and distributions), one flat tensor, best "
                  f"of 2; {what}; scaled per element to the full list (sample step {t_unfused * 1e3:.1f} ms)",
        "fused_single_pass_value": (1.0 / (fused_s * scale_up)) if fused_s else None,
    }


# ----------------------------------------------------------------------------------------

def cpu_baseline_cfg1_full():
    """BASELINE's config 1 on the host in full: the Qwen3-0.6B list (310 tensors, 596 M elements), inputs from the
    library's synthetic generator (the host twin regenerates what the device would hold), one AdamW step as the
    reference runs it: per tensor, 13 separate float32 passes."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle_c_binding as B
    from mxopt.qwen3_shapes import QWEN3, numel, param_list
    import mxopt
    oc = B.load()
    sizes = [numel(shape) for _, shape in param_list(QWEN3["0.6B"])]
    key = lambda stream, i: mxopt.synthetic_key(Workload.SEED, 1, 0, stream, i)
    ps = [oc.fill_synthetic(n, "f32", key(1, i), 3, 0.02) for i, n in enumerate(sizes)]      # 3 = MXOPT_SYNTH_GAUSSIAN
    gs = [oc.fill_synthetic(n, "f32", key(2, i), 3, 1e-3) for i, n in enumerate(sizes)]
    ms = [np.zeros(n, np.float32) for n in sizes]
    vs = [np.zeros(n, np.float32) for n in sizes]
    a = B.adam_args(1e-3, 0.9, 0.999, 1e-8, 0.01)
    best = {}
    for fused in (False, True):
        best[fused] = float("inf")
        for _ in range(2):
            t0 = time.perf_counter()
            for p, g, m, v in zip(ps, gs, ms, vs):
                oc.adam(p, g, m, v, a, fused=fused)
            best[fused] = min(best[fused], time.perf_counter() - t0)
    return {"value": round(1.0 / best[False], 4), "unit": "steps/s", "cores": oc.num_threads(), "kind": "port",
            "sample": f"the whole list ({len(sizes)} tensors, {sum(sizes)} elements), synthetic inputs of the library's "
                      "generator regenerated on the host, best of 2; AdamW as 13 separate float32 passes per tensor "
                      "(adamw.rs:84-116)",
            "fused_single_pass_value": round(1.0 / best[True], 4)}


def measure(wl, steps, warmup):
    """Warm-up, then `steps` timed steps bracketed by device synchronisation; per-kernel times from events."""
    torch = wl.torch
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    wl.kernel_events.clear()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    for i in range(steps):
        marks[i].record(wl.ctx.stream)
        wl.step()
    marks[-1].record(wl.ctx.stream)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    step_ms = sorted(a.elapsed_time(b) for a, b in zip(marks[:-1], marks[1:]))
    n = wl.n
    kernels = {}
    for name, bpe in wl.bytes_per_elem.items():
        ms = wl.kernel_ms(name)
        if not ms:
            continue
        avg = sum(ms) / len(ms)
        kernels[name] = {"avg_ms": round(avg, 4), "min_ms": round(min(ms), 4), "launches": len(ms),
                         "bytes_per_elem": bpe, "gbps": round(bpe * n / (avg * 1e-3) / 1e9, 1)}
    return {"elapsed": elapsed, "steps": steps, "ms_per_step": elapsed * 1e3 / steps, "steps_per_s": steps / elapsed,
            "step_ms_sorted": step_ms, "kernels": kernels,
            "step_gbps": wl.step_bytes_per_elem * n / (elapsed / steps) / 1e9}


def with_workload(args, name):
    import copy
    a = copy.copy(args)
    a.workload = name
    return a


def measured_ceiling(args, torch, mx, ctx, pool):
    """The four bare probes on 4 x 4 GiB of the same kind of memory the workload used."""
    wl = Workload(with_workload(args, "probes"), torch, mx, ctx, pool)
    r = measure(wl, 5, 2)
    wl.close()
    k = r["kernels"]
    return {"mix43_gbps": k["probe_mix43"]["gbps"], "copy_gbps": k["probe_copy"]["gbps"],
            "read_gbps": k["probe_read"]["gbps"], "write_gbps": k["probe_write"]["gbps"],
            "list4_gbps": k["probe_list4"]["gbps"],
            "streaming": {"mix43_gbps": k["probe_mix43_streaming"]["gbps"], "copy_gbps": k["probe_copy_streaming"]["gbps"],
                          "write_gbps": k["probe_write_streaming"]["gbps"], "list4_gbps": k["probe_list4_streaming"]["gbps"]},
            "what": "bare kernels (no table, no arithmetic) over 4 GiB per float32 stream from the same "
                    "allocator, measured in this run; mix43 = 4 read + 3 write streams in place; list4 = the deferred "
                    "update's mix: four 2-byte gradient streams and a 2-byte parameter, two 4-byte moments, 28 B/elem; "
                    "streaming = the same with streaming-hint loads and stores, the update kernels' default "
                    "(the read probe always streams)",
            "profile": PROBE_PROFILE}


def child_leg(args, placement, steps=5, warmup=2):
    """The same workload in a child process with another placement; returns what its line says about the step and
    the dominant kernel.  Run before this process touches the GPU, the child's allocations are the first of a
    fresh process: one compact physical run, which is what `plain` means on a freshly started host."""
    import subprocess
    cmd = [sys.executable, os.path.abspath(__file__), "--workload", args.workload, "--placement", placement,
           "--steps", str(steps), "--warmup", str(warmup), "--cpu-sample", "0", "--others", "0", "--placements", "0",
           "--verify", "0", "--ceiling", "0", "--variants", "0", "--fold-last", str(args.fold_last),
           "--scale", str(args.scale), "--alloc", args.alloc, "--micro", str(args.micro)]
    try:
        proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        line = [l for l in proc.stdout.splitlines() if l.startswith("{")][-1]
        d = json.loads(line)
        k = d["kernels"][d["roofline"]["kernel"]]
        return {"ms_per_step": d["ms_per_step"], "dominant_kernel_gbps": k["gbps"], "dominant_kernel_ms": k["avg_ms"],
                "step_hbm_gbps": d["step_hbm_gbps"], "steps": steps}
    except Exception as e:  # the leg is a side figure: its failure must not take the headline with it
        return {"error": f"{type(e).__name__}: {e}"[:300]}


def leg_summary(r, wl, steps):
    d = r["kernels"][wl.dominant]
    return {"ms_per_step": round(r["ms_per_step"], 4), "dominant_kernel_gbps": d["gbps"], "dominant_kernel_ms": d["avg_ms"],
            "step_hbm_gbps": round(r["step_gbps"], 1), "steps": steps}


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)")
    full_default = args.workload == "cfg5" and args.scale == 1.0
    three_placements = args.placement == "pool" and (args.placements == 1 or (args.placements == -1 and full_default))
    # first: before anything here touches the GPU, so that on a fresh box the child's are the first allocations
    plain_leg = child_leg(args, "plain") if three_placements and args.plain_leg == "first" else None
    if plain_leg is not None:
        time.sleep(8.0 if args.settle_s < 0 else args.settle_s)   # the child's memory is on its way back to the driver

    import torch
    import mxopt

    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X: mxopt has no CPU path")
    torch.cuda.set_device(0)

    ctx = mxopt.Context()
    for opt in args.option:
        k, v = opt.split("=")
        ctx.set_option(k, int(v))
    pool = None
    placement = "plain"
    sizes, _ = tensor_sizes(args)
    if args.placement in ("pool", "state-pool"):
        # the arena takes the free memory but for a margin left to torch's own scratch and the runtime -- and, when
        # the state-pool leg follows (or is the placement asked for), for the parameters and gradients that leg
        # keeps in plain memory
        free = torch.cuda.mem_get_info()[0]
        host_side = 0
        if three_placements or args.placement == "state-pool":
            host_side = sum(sizes) * 2 * 5 + (4 << 30) if args.workload == "cfg5" else free // 2
        try:
            want = int(args.pool_gib * 2**30) if args.pool_gib > 0 else free - (8 << 30) - host_side
            pool = ctx.hbm_pool(want, args.pool_chunk_mb << 20, args.pool_regions,
                                slab_bytes=args.pool_slab_mb << 20)
        except mxopt.MxoptError as e:
            # e.g. another process holds most of the device: measure in plain memory and say so in the line
            print(f"bench.py: no region-interleaved arena ({e}); buffers come from plain device memory", file=sys.stderr)
            placement = {"kind": "plain", "arena_refused": str(e)}
    if pool is not None:
        gave_back = free - pool.info().capacity_bytes > (16 << 30)
        settle = args.settle_s if args.settle_s >= 0 else (4.0 if gave_back else 0.0)
        if settle > 0:
            time.sleep(settle)
    if pool is not None:
        pool.use_for_state()
        i = pool.info()
        placement = {"kind": "mxopt_hbm_pool" if args.placement == "pool" else
                             "moments and accumulation buffers from mxopt_hbm_pool (mxopt_set_state_pool); parameters and "
                             "gradients in plain device memory",
                     "chunk_mib": i.chunk_bytes >> 20, "regions_found": i.regions,
                     "regions_used": min(args.pool_regions, i.regions) if args.pool_regions else i.regions,
                     "arena_gib": round(i.capacity_bytes / 2**30, 1),
                     "interleaved_gib": round(i.interleaved_bytes / 2**30, 1),
                     "gradients": "one region (behind the alternation)" if args.grads_one_region else "interleaved",
                     "region_free_gib": [round(x / 2**30, 1) for x in i.region_free_bytes[:i.regions]],
                     "probe_same_region_gbps": round(i.probe_same_region_gbps, 1),
                     "probe_cross_region_gbps": round(i.probe_cross_region_gbps, 1),
                     "probe_on_arena_gbps": round(i.arena_probe_gbps, 1),
                     "setup_s": round(i.setup_seconds, 2), "scan_s": round(i.scan_seconds, 2), "probes": i.probes}
    elif args.placement == "spread":
        placement = (f"buffers allocated between mxopt_hbm_spread_begin and _end ({args.spread_block_mb or 64} MiB "
                     f"blocks, one in {args.spread_keep or 3} kept meanwhile)")

    wl = Workload(args, torch, mxopt, ctx, pool)
    r = measure(wl, args.steps, args.warmup)
    n = wl.n
    kernels = r["kernels"]
    step_ms = r["step_ms_sorted"]
    dom = kernels[wl.dominant]
    key = (args.workload, int(args.fold_last))
    have_traffic = key in MEASURED_TRAFFIC_B_PER_ELEM and args.micro == 4 and traffic_profile_is_current()
    roofline = {"bound": "hbm", "achieved": dom["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(dom["gbps"] / HBM_PEAK_GBPS, 4),
                "traffic": round(MEASURED_TRAFFIC_B_PER_ELEM[key] * n) if have_traffic else None,
                "traffic_source": (TRAFFIC_PROFILE + " (rocprofv3 FETCH_SIZE + WRITE_SIZE of an earlier run of this "
                                   "kernel, scaled per element; not counted in this run)") if have_traffic else None,
                "kernel": wl.dominant, "algorithmic_bytes_per_launch": dom["bytes_per_elem"] * n,
                "avg_launch_ms": dom["avg_ms"]}

    # config 5 only: the same buffers stepped two other ways (every one a full optimizer step with the same
    # result), then the self-check over all steps this process made
    deferred = unfolded = verified = None
    if args.workload == "cfg5":
        segments = []

        def book(steps):
            h = ctx.read_norm_result(wl.res)
            segments.append((steps, h.scale, h.sumsq))
        book(wl.steps_done)
        if args.variants:
            deferred = wl.deferred_variant(args.steps)
            if deferred:
                book(wl.deferred_steps_done)
            unfolded = wl.other_fold_variant(args.steps)
            book(wl.other_fold_steps_done)
        if args.verify == 1 or (args.verify == -1 and args.scale == 1.0):
            verified = verify_cfg5(wl, segments)
    config = {"workload": f"{args.workload}: {wl.list_name}", "tensors": len(wl.sizes), "elements": n,
              "bytes_per_elem_per_step": wl.step_bytes_per_elem,
              "storage": getattr(wl, "storage", "float32 everywhere"),
              "note": "; ".join(x for x in (wl.note,
                                            "the gradient buffers are generated once and reused by every step (their values do "
                                            "not change the traffic)",
                                            "'normal' inputs come from the generator's Gaussian mode (quantile table, tails to "
                                            "6.3 sigma)") if x),
              "scale": args.scale, "alloc": args.alloc, "placement": placement}
    dtype = wl.dtype
    main_leg = leg_summary(r, wl, args.steps)
    wl.close()

    if args.ceiling and args.workload not in ("probes", "copy"):
        roofline["measured_ceiling"] = measured_ceiling(args, torch, mxopt, ctx, pool)
        mc = roofline["measured_ceiling"]
        roofline["frac_of_measured_ceiling"] = round(dom["gbps"] / max(mc["mix43_gbps"], mc["streaming"]["mix43_gbps"]), 4)

    if three_placements and pool is not None:
        # what a drop-in host sees: its own allocator keeps parameters and gradients, the library's pool only
        # moments and accumulation buffers
        a = with_workload(args, args.workload)
        a.placement = "state-pool"
        w3 = Workload(a, torch, mxopt, ctx, pool)
        state_pool_leg = leg_summary(measure(w3, 5, 2), w3, 5)
        w3.close()
        # that leg's parameters and gradients (80 GB of plain memory) have just gone back to the driver
        time.sleep(4.0 if args.settle_s < 0 else args.settle_s)
        placement["plain_leg_ran"] = args.plain_leg
        legs = placement["legs"] = {
            "arena (every buffer from the pool; the headline)": main_leg,
            "state_pool (moments and accumulation buffers from the pool, parameters and gradients from torch's allocator)":
                state_pool_leg,
            "plain (torch's allocator for everything; a child process)": plain_leg}
        placement["adamw_gbps"] = {"arena": main_leg["dominant_kernel_gbps"],
                                   "state_pool": state_pool_leg["dominant_kernel_gbps"],
                                   "plain": (plain_leg or {}).get("dominant_kernel_gbps")}

    others = None
    if args.others == 1 or (args.others == -1 and full_default):
        others = {}
        for name in OTHER_CONFIGS:
            a = with_workload(args, name)
            a.placement = "pool" if pool is not None else "plain"
            steps2 = args.others_steps or OTHER_CONFIG_STEPS[name]
            w2 = Workload(a, torch, mxopt, ctx, pool)
            r2 = measure(w2, steps2, 2)
            d2 = r2["kernels"][w2.dominant]
            others[name] = {"list": w2.list_name, "tensors": len(w2.sizes), "elements": w2.n,
                            "steps": steps2, "steps_per_s": round(r2["steps_per_s"], 3),
                            "ms_per_step": round(r2["ms_per_step"], 4),
                            "bytes_per_elem_per_step": w2.step_bytes_per_elem,
                            "step_hbm_gbps": round(r2["step_gbps"], 1),
                            "dominant_kernel": w2.dominant, "dominant_kernel_ms": d2["avg_ms"],
                            "dominant_kernel_gbps": d2["gbps"], "frac": round(d2["gbps"] / HBM_PEAK_GBPS, 4),
                            "kernels": r2["kernels"]}
            if hasattr(w2, "graph_variant"):
                others[name]["hip_graph"] = w2.graph_variant(steps2)
            w2.close()
        if args.cpu_sample > 0:
            others["cfg1"]["cpu_baseline"] = cpu_baseline_cfg1_full()

    if three_placements and pool is not None and args.plain_leg == "last":
        # everything this process held goes back to the driver first; the child then allocates as any host would
        # that starts on a device other processes have used
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        try:
            pool.close()
            pool = None
        except mxopt.MxoptError as e:      # something still lives in the arena: the child gets what is left
            placement["arena_not_released"] = str(e)
        torch.cuda.empty_cache()
        plain_leg = child_leg(args, "plain")
        placement["legs"]["plain (torch's allocator for everything; a child process)"] = plain_leg
        placement["adamw_gbps"]["plain"] = plain_leg.get("dominant_kernel_gbps")

    no_cpu_leg = ("copy", "probes", "grpo-engine", "sft-engine")
    cpu = cpu_baseline(args, n) if args.cpu_sample > 0 and args.workload not in no_cpu_leg else None

    out = {
        "metric": "optimizer steps/s + achieved HBM GB/s (% of 8 TB/s), AdamW on Qwen3-8B shapes",
        "value": round(r["steps_per_s"], 4), "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["ms_per_step"], 4), "ms_per_step_median": round(step_ms[len(step_ms) // 2], 4),
        "ms_per_step_min": round(step_ms[0], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic (counter-based generator of the library, seed 0x5EED0001; reproducible on the host)",
        "config": config,
        "elements_per_s": round(n * r["steps_per_s"], 1),
        "step_hbm_gbps": round(r["step_gbps"], 1), "step_hbm_frac": round(r["step_gbps"] / HBM_PEAK_GBPS, 4),
        "kernels": kernels,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if verified:
        out["verified"] = verified
    if unfolded:
        out["other_fold"] = unfolded
    if deferred:
        out["deferred_accumulation"] = deferred
    if others:
        out["other_configs"] = others
    print(json.dumps(out))
    if verified and not verified["ok"]:
        sys.exit("bench.py: the timed configuration failed its own check (see `verified` in the line above)")


if __name__ == "__main__":
    main()
