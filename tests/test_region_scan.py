"""The memory pool's region scan on synthetic rate maps (CPU only: the classifier is a pure function behind
mxopt_hbm_classify_regions / mxopt_hbm_plan_arena, the same code mxopt_hbm_pool_create runs on measured rates).

Model of the device: every slab is 16 chunks, every chunk lies in one region; the 4-read/3-write probe with two
streams in slab a and two in slab b runs at `SAME` GB/s when all their chunks share a region, at `CROSS` when none do,
and in between in proportion to the chance that a chunk of a and a chunk of b share one (a slab that straddles a
region boundary).  SAME and CROSS are the levels measured on MI355X."""
import numpy as np
import pytest

import mxopt

SAME, CROSS = 5350.0, 6150.0
CHUNKS = 16


def device(layout, noise=0.0, seed=0):
    """layout: per slab either a region number or a list of (region, chunks) for a straddler.
    Returns (probe(ref, slab) -> GB/s, fractions)."""
    regions = 1 + max(r for s in layout for r, _ in ([(s, CHUNKS)] if isinstance(s, int) else s))
    frac = np.zeros((len(layout), regions))
    for i, s in enumerate(layout):
        for r, c in ([(s, CHUNKS)] if isinstance(s, int) else s):
            frac[i, r] += c / CHUNKS
    rng = np.random.default_rng(seed)
    calls = []

    def probe(ref, slab):
        calls.append((ref, slab))
        overlap = float(frac[ref] @ frac[slab])
        rate = CROSS - (CROSS - SAME) * overlap
        return rate * (1.0 + noise * (2.0 * rng.random() - 1.0))
    return probe, frac, calls


def same_partition(got, truth, pure):
    """The classification equals the truth up to the names of the regions, on the slabs that lie in one region."""
    pairs = {(got[i], truth[i]) for i in pure}
    return len({g for g, _ in pairs}) == len(pairs) == len({t for _, t in pairs})


def check(layout, noise=0.0, seed=0, want_regions=None, max_probe_share=0.75):
    probe, frac, calls = device(layout, noise, seed)
    got, report = mxopt.classify_regions(len(layout), probe)
    pure = [i for i, s in enumerate(layout) if isinstance(s, int)]
    truth = [s if isinstance(s, int) else -1 for s in layout]
    assert same_partition(got, truth, pure), (got, truth)
    if want_regions is not None:
        assert len({got[i] for i in pure}) == want_regions
    assert report.probes == len(calls)
    # the coarse scan probes a fraction of the slabs per region found, not all of them against everything
    assert report.probes <= max_probe_share * len(layout) * max(report.regions, 1)
    return got, report


def test_fresh_device_three_regions_in_physical_order():
    layout = [0] * 78 + [1] * 96 + [2] * 96 + [0] * 0
    got, report = check(layout, want_regions=3)
    assert report.regions == 3 and abs(report.same_region_gbps - SAME) < 1 and abs(report.cross_region_gbps - CROSS) < 1
    assert report.probes < 200


def test_one_region_only():
    got, report = check([0] * 40, want_regions=1, max_probe_share=1.0)   # three references, a quarter of the slabs each
    assert set(got) == {0} and report.regions == 1 and report.cross_region_gbps == 0.0
    assert abs(report.same_region_gbps - SAME) < 1


def test_two_regions():
    check([0] * 30 + [1] * 50, want_regions=2)


def test_boundary_slabs_that_straddle_two_regions():
    layout = [0] * 20 + [[(0, 9), (1, 7)]] + [1] * 30 + [[(1, 4), (2, 12)]] + [2] * 25
    got, _ = check(layout, want_regions=3)
    # a straddler goes with one of its two regions
    assert got[20] in (got[0], got[21]) and got[51] in (got[50], got[52])


def test_reference_slab_that_straddles():
    """Slab 0, the first reference, lies half in each region: every rate against it is the same intermediate value.
    The scan has to notice (one class only) and take another reference instead of calling everything one region."""
    layout = [[(0, 8), (1, 8)]] + [0] * 30 + [1] * 30
    check(layout, want_regions=2, max_probe_share=1.5)


def test_fragmented_creation_order():
    """After other processes came and went, creation order is no longer physical order: regions come in runs of a
    few slabs (the shortest seen on a real device were three), with straddlers where runs meet."""
    rng = np.random.default_rng(5)
    layout, region = [], 0
    while len(layout) < 280:
        run = int(rng.integers(3, 40))
        layout += [region] * run
        nxt = int(rng.choice([r for r in range(3) if r != region]))
        if rng.random() < 0.5:
            k = int(rng.integers(1, CHUNKS))
            layout.append([(region, k), (nxt, CHUNKS - k)])
        region = nxt
    check(layout[:280], want_regions=3, max_probe_share=1.0)


@pytest.mark.parametrize("seed", range(8))
def test_noise_of_five_percent(seed):
    """+-5 % on every measurement (the device shows +-1.5 %): the classes are 14 % apart and must still come out
    right, and one region must not be split in two by the noise."""
    check([0] * 60 + [1] * 70 + [2] * 50, noise=0.05, seed=seed, want_regions=3, max_probe_share=1.0)
    got, report = check([0] * 64, noise=0.05, seed=seed, want_regions=1, max_probe_share=1.5)
    assert report.regions == 1


def test_fewer_than_four_slabs_are_one_region_without_a_probe():
    for n in (0, 1, 3):
        probe, _, calls = device([0, 1, 2][:n] if n else [0])
        got, report = mxopt.classify_regions(n, probe)
        assert got == [0] * n and report.regions == 1 and not calls


def test_more_groups_than_the_bookkeeping_has_slots():
    layout = [r for r in range(10) for _ in range(8)]      # ten "regions" of eight slabs
    probe, _, _ = device(layout)
    got, report = mxopt.classify_regions(len(layout), probe)
    assert report.regions == 8 and max(got) == 7
    for r in range(7):                                      # the first seven come out exactly, the rest is lumped
        assert len({got[i] for i in range(8 * r, 8 * r + 8)}) == 1
    assert len({got[i] for i in range(56, 80)}) == 1


def test_a_failing_probe_is_handed_back():
    import ctypes as C
    L = mxopt._lib if hasattr(mxopt, "_lib") else __import__("mxopt._lib", fromlist=["x"])
    fn = L.SLAB_PROBE_FN(lambda user, ref, slab, out: 7)
    regions = (C.c_int * 16)()
    assert L.load().mxopt_hbm_classify_regions(16, fn, None, regions, None) == 7


# ---- the arena's chunk order -------------------------------------------------------------

def region_of_chunk(slab_region, per_slab):
    return lambda chunk: slab_region[min(chunk // per_slab, len(slab_region) - 1)]


def test_arena_alternates_between_the_two_largest_regions_then_uses_the_rest():
    slab_region = [0] * 78 + [1] * 96 + [2] * 96
    per, total = 16, 270 * 16
    order, rep = mxopt.plan_arena(slab_region, 3, per, total, total, max_regions=2)
    where = region_of_chunk(slab_region, per)
    assert sorted(order) == list(range(total))              # every chunk exactly once
    assert rep.real_regions == 3 and rep.active_regions == 2
    assert rep.interleaved_chunks == 2 * 96 * 16
    inter = [where(c) for c in order[:rep.interleaved_chunks]]
    assert set(inter) == {1, 2} and all(a != b for a, b in zip(inter, inter[1:]))
    assert {where(c) for c in order[rep.interleaved_chunks:]} == {0}     # what lies behind: one region


def test_arena_over_all_regions_and_leftover_groups():
    # a fourth group of two slabs is a leftover of the scan (under a tenth of the chunks): served last, not counted
    slab_region = [0] * 40 + [3] * 2 + [1] * 40 + [2] * 38
    per, total = 4, 120 * 4
    where = region_of_chunk(slab_region, per)
    order, rep = mxopt.plan_arena(slab_region, 4, per, total, 400, max_regions=0)
    assert rep.real_regions == 3 and rep.active_regions == 3 and rep.interleaved_chunks == 400
    head = [where(c) for c in order]
    assert all(len({head[i], head[i + 1], head[i + 2]}) == 3 for i in range(0, len(head) - 2, 3))
    assert len(set(order)) == len(order) == 400
    # the whole device: three regions alternate until the smallest is used up (3 x 152 chunks), the two larger ones go
    # on alternating (2 x 8), and the leftover group comes last
    order, rep = mxopt.plan_arena(slab_region, 4, per, total, total, max_regions=0)
    assert sorted(order) == list(range(total)) and rep.interleaved_chunks == 3 * 152 + 16
    tail = [where(c) for c in order[rep.interleaved_chunks:]]
    assert tail == [3] * 8
    mid = [where(c) for c in order[3 * 152:3 * 152 + 16]]
    assert set(mid) == {0, 1} and all(a != b for a, b in zip(mid, mid[1:]))


def test_arena_with_one_region_has_nothing_interleaved():
    order, rep = mxopt.plan_arena([0] * 10, 1, 16, 160, 100, max_regions=2)
    assert order == list(range(100)) and rep.active_regions == 1 and rep.interleaved_chunks == 0


def test_arena_refuses_more_chunks_than_there_are():
    with pytest.raises(mxopt.MxoptError):
        mxopt.plan_arena([0] * 4, 1, 16, 64, 65)
