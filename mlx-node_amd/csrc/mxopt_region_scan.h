// Which groups of physical memory chunks ("slabs") share a memory region, decided from probe rates alone.
//
// Host code without a single HIP call: the pool hands in a function that times the 4-read/3-write
// probe with two streams in a reference slab and two in a slab under test, and the tests hand in
// synthetic rate maps.  A pair in one region answers slowly, a pair in two regions quickly; the
// classifier only ever compares rates measured against the same reference.
#pragma once

#include <stddef.h>

#include <functional>
#include <string>
#include <vector>

namespace mxopt {

// Every constant of the scan, with the measurement it comes from (MI355X, 1 GiB slabs, 512 MiB streams).
struct ScanLimits {
  // Two clusters of rates are "one region and another" when their means differ by at least this factor.
  // Measured: 5.26 - 5.42 TB/s inside one region, 6.03 - 6.16 across two: the class means are a factor 1.15
  // apart.  One class under +-5 % of uniform noise splits into clusters at most 1.053 apart (plus sampling
  // error), and a reference that straddles a boundary 3 : 1 shows the two regions only 1.07 apart -- such a
  // reference is better replaced than trusted -- so 1.10 stands between the cases.
  double class_ratio = 1.10;
  // ... and when the slowest member of the fast cluster is at least this factor above the fastest member
  // of the slow one (noise of +-5 % on both classes still leaves 1.04).
  double class_gap = 1.015;
  // Coarse scan: every stride-th slab in creation order is probed, the ones in between only where two probed
  // neighbours disagree.  On a fresh device creation order is physical order and a region is a run of
  // ~96 slabs; after other processes came and went the shortest runs seen were 3 slabs.
  size_t coarse_stride = 4;
  // A reference slab that straddles two regions makes every other slab look fast; when a scan shows one class
  // only, another reference (a quarter further into the list each time) is tried this many times before the
  // remaining slabs are taken to share one region.
  int reference_attempts = 3;
  // Fewer slabs than this are boundary leftovers, not a region of their own: they join the last region found.
  size_t min_region_slabs = 4;
  // Groups beyond this many are lumped into the last one (the arena's bookkeeping has this many slots).
  int max_regions = 8;
};

// rate of the probe, in GB/s, with streams p, g in `ref_slab` and m, v in `slab`; non-zero = error code
using SlabProbe = std::function<int(int ref_slab, int slab, double* gbps)>;

struct ScanResult {
  std::vector<int> slab_region;  // region index of every slab, in order of discovery
  int regions = 1;
  double same_region_gbps = 0.0;   // level of the slow class in the scan that first showed both (0: never seen)
  double cross_region_gbps = 0.0;  // level of the fast class there
  int probes = 0;
  std::string trace;               // one line per scan: the reference, the threshold and every rate (for MXOPT_LOG=debug)
};

// Classifies `nslab` slabs.  Returns 0, or the first non-zero code a probe returned.
int classify_slabs(size_t nslab, const SlabProbe& probe, const ScanLimits& limits, ScanResult* out);

// The arena's chunk order: consecutive arena chunks alternate between the `max_regions` (0 = all) largest
// real regions for as long as each has chunks, then the remaining chunks follow region by region.
struct ArenaPlan {
  std::vector<size_t> order;        // physical chunk index of arena chunk 0, 1, ...
  int real_regions = 1;             // regions holding at least a tenth of all chunks (smaller groups are scan leftovers)
  int active = 1;                   // regions that take part in the alternation
  std::vector<int> rank;            // region indices, most chunks first
  std::vector<size_t> region_chunks;  // chunks of each region (indexed like rank)
  std::vector<size_t> region_used;    // ... and how many of them the arena took
  size_t interleaved_chunks = 0;    // arena chunks [0, this) alternate; the rest lie in one region at a time
};
// chunk i belongs to slab i / chunks_per_slab (chunks beyond the last whole slab to the last slab's region).
ArenaPlan plan_arena(const std::vector<int>& slab_region, int regions, size_t chunks_per_slab, size_t total_chunks,
                     size_t want_chunks, int max_regions);

}  // namespace mxopt
