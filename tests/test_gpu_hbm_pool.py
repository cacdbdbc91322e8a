"""mxopt_hbm_pool_*: the region-interleaved arena, its allocator, the hooks a host allocator plugs in, the
optimizer state taken from it -- and the bare streaming probes (mxopt_probe_stream), whose data movement
is checked element by element.  Results never depend on where a buffer lies."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mxopt_oracle as O
from gpu_util import assert_bit_equal, to_dev, to_host

F = np.float32
GiB = 1 << 30


@pytest.fixture(scope="module")
def mx():
    import torch
    import mxopt
    assert torch.cuda.is_available()
    return mxopt


@pytest.fixture(scope="module")
def ctx(mx):
    c = mx.Context()
    yield c
    c.close()


@pytest.fixture(scope="module")
def pool(mx, ctx):
    import torch
    torch.cuda.empty_cache()
    free0 = torch.cuda.mem_get_info()[0]
    p = ctx.hbm_pool(6 * GiB)
    # what the arena does not hold went back to the driver before create returned
    assert torch.cuda.mem_get_info()[0] > free0 - 7 * GiB
    yield p
    p.close()
    assert torch.cuda.mem_get_info()[0] > free0 - GiB


def test_pool_finds_regions_and_interleaves(mx, pool):
    i = pool.info()
    assert i.capacity_bytes == 6 * GiB and i.chunk_bytes == 64 << 20 and i.used_bytes == 0
    assert 1 <= i.regions <= mx.HbmPool.MAX_REGIONS
    assert sum(i.region_arena_bytes) == i.capacity_bytes
    if i.regions >= 2:     # a device with most of its memory free: the arena is split evenly
        assert i.probe_cross_region_gbps > 1.07 * i.probe_same_region_gbps
        share = [b for b in i.region_arena_bytes[:i.regions]]
        assert max(share) - min(share) <= i.chunk_bytes
    assert i.probes > 0 and 0 < i.scan_seconds <= i.setup_seconds < 30


def test_pool_limited_to_two_regions(mx, ctx, pool):
    """max_regions = 2: the arena alternates between the two regions with the most free memory only."""
    small = ctx.hbm_pool(3 * GiB, 0, 2)
    try:
        i = small.info()
        assert i.capacity_bytes == 3 * GiB and i.regions >= 1
        assert sum(i.region_arena_bytes) == i.capacity_bytes
        if i.regions >= 2:
            assert i.probe_cross_region_gbps > 1.07 * i.probe_same_region_gbps
            assert abs(i.region_arena_bytes[0] - i.region_arena_bytes[1]) <= i.chunk_bytes
            assert sum(i.region_arena_bytes[2:]) == 0
        a = small.alloc(3 * GiB)
        assert small.owns(a) and not pool.owns(a)
        with pytest.raises(mx.InvalidArg, match=r"1 allocation\(s\), 3072 MiB, are still live"):
            small.close()                     # unmapping under a live allocation is refused
        assert small.owns(a)
        small.free(a)
    finally:
        small.close()


def test_pool_allocator_first_fit_coalesces_and_refuses(mx, ctx, pool):
    a = pool.alloc(1000)
    b = pool.alloc(3 * GiB)
    c = pool.alloc(1)
    assert a % 512 == 0 and b == a + 1024 and c == b + 3 * GiB and pool.owns(a) and pool.owns(c)
    assert pool.info().used_bytes == 1024 + 3 * GiB + 512
    with pytest.raises(mx.MxoptError, match="no free range"):
        pool.alloc(4 * GiB)
    pool.free(b)
    b2 = pool.alloc(2 * GiB)                  # first fit: the hole b left
    assert b2 == b
    pool.free(a)
    pool.free(b2)
    pool.free(c)
    assert pool.info().used_bytes == 0
    whole = pool.alloc(6 * GiB)               # everything coalesced again
    pool.free(whole)
    with pytest.raises(mx.InvalidArg, match="not a live allocation"):
        pool.free(whole)
    assert not pool.owns(0) and not pool.owns(whole + 6 * GiB)
    with pytest.raises(mx.InvalidArg, match="power of two"):
        ctx.hbm_pool(GiB, 3 << 20)
    with pytest.raises(mx.InvalidArg, match="capacity_bytes is 0"):
        ctx.hbm_pool(0)
    with pytest.raises(mx.MxoptError, match="MiB free"):
        ctx.hbm_pool(4000 * GiB)


def test_results_do_not_depend_on_the_arena(mx, ctx, pool):
    """AdamW on tensors torch allocated from the arena (the plug-in allocator hooks) against the oracle."""
    import torch
    rng = np.random.default_rng(11)
    n = (1 << 20) + 77
    p, g = rng.normal(0, 0.02, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
    mem = pool.torch_pool()
    with torch.cuda.use_mem_pool(mem):
        dp, dg = torch.empty(n, device="cuda"), torch.empty(n, device="cuda")
        dm, dv = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    assert all(pool.owns(t.data_ptr()) for t in (dp, dg, dm, dv))
    dp.copy_(torch.from_numpy(p))
    dg.copy_(torch.from_numpy(g))
    t = ctx.table([mx.TensorSpec(p=dp, p_out=dp, g=dg, m=dm, v=dv)])
    ref = O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01)
    want = p
    for _ in range(2):
        ctx.adam(t, mx.adam_hp(1e-3, 0.9, 0.999, 1e-8, 0.01))
        want = ref.update_single("w", want, g)
    assert_bit_equal(to_host(dp), want, "parameters in arena memory")
    t.close()
    used = pool.info().used_bytes
    assert used > 0
    del dp, dg, dm, dv, mem, t      # the table kept its tensors alive
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    assert pool.info().used_bytes == 0        # torch handed its segments back through the free hook


def test_optimizer_state_comes_from_the_pool(mx, ctx, pool):
    rng = np.random.default_rng(12)
    n = 300_000
    p, g = rng.normal(0, 0.02, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
    pool.use_for_state()
    try:
        opt = mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, ctx=ctx)
        out = opt.update_single("w", to_dev(p), to_dev(g))
        m, v, cnt, hv = C.c_void_p(), C.c_void_p(), C.c_uint64(), C.c_int()
        mx.load().mxopt_optimizer_state(opt.handle, b"w", C.byref(m), C.byref(v), C.byref(cnt), C.byref(hv))
        assert pool.owns(m.value) and pool.owns(v.value) and cnt.value == n
        assert pool.info().used_bytes >= 2 * 4 * n
        assert_bit_equal(to_host(out), O.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01).update_single("w", p, g), "AdamW, pooled state")
        ctx.lib.mxopt_set_state_pool(ctx.handle, None)
        del opt                               # detached meanwhile: the moments still find their way back
        assert pool.info().used_bytes == 0
    finally:
        ctx.lib.mxopt_set_state_pool(ctx.handle, None)
    opt = mx.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, ctx=ctx)   # detached again: state from the driver
    opt.update_single("w", to_dev(p), to_dev(g))
    assert pool.info().used_bytes == 0
    del opt


@pytest.mark.parametrize("streaming", [0, 1])
def test_probes_move_the_bytes_they_claim(mx, ctx, streaming):
    """Both forms of every probe (plain accesses; MXOPT_PROBE_STREAMING: streaming-hint loads and stores)."""
    import torch
    flag = mx.PROBE_STREAMING if streaming else 0
    n = 4096 * 37
    rng = np.random.default_rng(13)
    host = [rng.integers(0, 2**31 - 1, n, dtype=np.int64).astype(np.int32) for _ in range(4)]
    a, b, c, d = [torch.from_numpy(h.copy()).cuda().view(torch.float32) for h in host]
    before = [t.clone() for t in (a, b, c, d)]
    ctx.probe_stream(mx.PROBE_READ | flag, a)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int32), before[0].view(torch.int32))
    ctx.probe_stream(mx.PROBE_COPY | flag, a, b)
    torch.cuda.synchronize()
    assert torch.equal(b.view(torch.int32), a.view(torch.int32))
    a0, g0, c0, d0 = [t.view(torch.int32).cpu().numpy().astype(np.uint32) for t in (a, b, c, d)]
    ctx.probe_stream(mx.PROBE_MIX43 | flag, a, b, c, d)
    torch.cuda.synchronize()
    got = [t.view(torch.int32).cpu().numpy().astype(np.uint32) for t in (a, b, c, d)]
    assert np.array_equal(got[0], a0 ^ g0) and np.array_equal(got[1], g0)
    assert np.array_equal(got[2], c0 + g0) and np.array_equal(got[3], d0 ^ (g0 >> 1))
    ctx.probe_stream(mx.PROBE_WRITE | flag, a)
    torch.cuda.synchronize()
    w = a.view(torch.int32).cpu().numpy()
    assert np.array_equal(w, np.repeat(np.arange(n // 4096, dtype=np.int32), 4096))   # every element written, by its tile
    with pytest.raises(mx.InvalidArg, match="multiple of 4096"):
        ctx.probe_stream(mx.PROBE_READ, a[:1000])
    with pytest.raises(mx.InvalidArg, match="non-NULL"):
        ctx.probe_stream(mx.PROBE_COPY, a)
    with pytest.raises(mx.InvalidArg, match="unknown kind"):
        ctx.probe_stream(9 | flag, a)


@pytest.mark.parametrize("k,streaming", [(1, False), (4, False), (4, True), (8, True)])
def test_list_probe_moves_the_bytes_it_claims(mx, ctx, k, streaming):
    """mxopt_probe_list: per 4096-element tile and lane, two 16-byte pieces of every 2-byte stream and four of every
    4-byte stream; s = the word-wise sum of the gradient pieces, p ^= s, m += s, v ^= s >> 1 (both 16-byte halves of a
    moment group get the s of their parameter piece)."""
    import torch
    tiles = 9
    n = 4096 * tiles
    rng = np.random.default_rng(k + 100 * streaming)
    words = lambda count: rng.integers(0, 2**32, count, dtype=np.uint64).astype(np.uint32)
    g_h = [words(n // 2) for _ in range(k)]                  # 2 bytes per element
    p_h, m_h, v_h = words(n // 2), words(n), words(n)
    dev = lambda h: torch.from_numpy(h.view(np.int32).copy()).cuda()
    gs, p, m, v = [dev(h).view(torch.bfloat16) for h in g_h], dev(p_h).view(torch.bfloat16), dev(m_h).view(torch.float32), dev(v_h).view(torch.float32)
    ctx.probe_list(p, m, v, gs, streaming=streaming)
    torch.cuda.synchronize()
    back = lambda t: t.view(torch.int32).cpu().numpy().view(np.uint32)
    S = np.zeros((tiles, 2, 256, 4), np.uint32)
    for h in g_h:
        S = S + h.reshape(tiles, 2, 256, 4)
    assert np.array_equal(back(p).reshape(tiles, 2, 256, 4), p_h.reshape(tiles, 2, 256, 4) ^ S)
    assert np.array_equal(back(m).reshape(tiles, 2, 2, 256, 4), m_h.reshape(tiles, 2, 2, 256, 4) + S[:, :, None])
    assert np.array_equal(back(v).reshape(tiles, 2, 2, 256, 4), v_h.reshape(tiles, 2, 2, 256, 4) ^ (S >> 1)[:, :, None])
    for g, h in zip(gs, g_h):
        assert np.array_equal(back(g), h)                   # read only
    with pytest.raises(mx.InvalidArg, match="1 to 8"):
        ctx.probe_list(p, m, v, gs * 9)


def test_one_region_kind_without_such_a_part_changes_nothing(mx, pool):
    """The module's 6 GiB pool alternates over its whole length (or found one region: then nothing is interleaved):
    MXOPT_HBM_ONE_REGION allocations are served like any other."""
    i = pool.info()
    assert i.interleaved_bytes in (0, i.capacity_bytes)
    a = pool.alloc(GiB, mx.HBM_ONE_REGION)
    assert pool.owns(a)
    pool.free(a)
    with pytest.raises(mx.InvalidArg, match="unknown kind"):
        pool.alloc(GiB, 5)
