// Region classification of physical memory slabs from probe rates, and the arena's chunk order.
// Pure host code (no HIP): see mxopt_region_scan.h.
#include "mxopt_region_scan.h"

#include <algorithm>
#include <cmath>
#include <cstdio>

namespace mxopt {

namespace {

// The rates of one scan (all against one reference), split into a slow and a fast class if they form two.
struct Split {
  bool two = false;
  double threshold = 0.0;  // geometric middle of the gap between the classes
  double slow = 0.0, fast = 0.0;  // class means (slow == fast == overall mean when there is one class)
};

Split split_classes(std::vector<double> r, const ScanLimits& lim) {
  Split s;
  std::sort(r.begin(), r.end());
  const size_t n = r.size();
  double total = 0.0;
  for (double x : r) total += x;
  s.slow = s.fast = n ? total / (double)n : 0.0;
  if (n < 2 || r.front() <= 0.0) return s;
  // the widest relative gap between neighbours that also separates two clusters far enough apart
  double below = 0.0, best_gap = 0.0;
  for (size_t k = 1; k < n; ++k) {
    below += r[k - 1];
    const double gap = r[k] / r[k - 1];
    const double mean_lo = below / (double)k, mean_hi = (total - below) / (double)(n - k);
    if (gap >= lim.class_gap && mean_hi >= mean_lo * lim.class_ratio && gap > best_gap) {
      best_gap = gap;
      s.two = true;
      s.threshold = std::sqrt(r[k] * r[k - 1]);
      s.slow = mean_lo;
      s.fast = mean_hi;
    }
  }
  return s;
}

}  // namespace

int classify_slabs(size_t nslab, const SlabProbe& probe, const ScanLimits& lim, ScanResult* out) {
  out->slab_region.assign(nslab, 0);
  out->regions = 1;
  out->same_region_gbps = out->cross_region_gbps = 0.0;
  out->probes = 0;
  out->trace.clear();
  if (nslab < lim.min_region_slabs) return 0;

  std::vector<int> todo(nslab);
  for (size_t i = 0; i < nslab; ++i) todo[i] = (int)i;
  std::vector<double> rate(nslab, 0.0);
  double abs_thr = 0.0;  // once a scan has shown both classes, every later scan is judged by its threshold
  int region = 0, attempts = 0;
  const size_t stride = std::max<size_t>(lim.coarse_stride, 1);

  while (!todo.empty() && region < lim.max_regions) {
    if (todo.size() < lim.min_region_slabs) {  // a few boundary slabs are no region of their own
      for (int x : todo) out->slab_region[x] = std::max(region - 1, 0);
      todo.clear();
      break;
    }
    // The reference must lie inside one region: first the first slab of the list, after a scan that showed
    // one class only, one a quarter further in.
    const size_t ref_pos = std::min(todo.size() - 1, todo.size() * (size_t)attempts / 4);
    const int ref = todo[ref_pos];
    std::vector<int> others;
    others.reserve(todo.size() - 1);
    for (size_t i = 0; i < todo.size(); ++i)
      if (i != ref_pos) others.push_back(todo[i]);
    std::vector<char> probed(others.size(), 0);
    auto scan = [&](size_t k) -> int {
      if (probed[k]) return 0;
      const int rc = probe(ref, others[k], &rate[others[k]]);
      if (rc) return rc;
      probed[k] = 1;
      ++out->probes;
      return 0;
    };
    for (size_t k = 0; k < others.size(); k += stride)
      if (int rc = scan(k)) return rc;
    if (int rc = scan(others.size() - 1)) return rc;

    std::vector<double> seen;
    for (size_t k = 0; k < others.size(); ++k)
      if (probed[k]) seen.push_back(rate[others[k]]);
    Split sp = split_classes(seen, lim);
    if (abs_thr > 0.0) {  // the classes are known: two of them are present iff rates fall on both sides
      const bool any_slow = std::any_of(seen.begin(), seen.end(), [&](double x) { return x < abs_thr; });
      const bool any_fast = std::any_of(seen.begin(), seen.end(), [&](double x) { return x >= abs_thr; });
      sp.two = any_slow && any_fast;
      sp.threshold = abs_thr;
    }
    auto trace_line = [&](const char* verdict, double thr) {
      char head[160];
      std::snprintf(head, sizeof head, "scan %d: reference slab %d, threshold %.0f, %s:", region, ref, thr, verdict);
      out->trace += head;
      for (size_t k = 0; k < others.size(); ++k)
        if (probed[k]) {
          char item[48];
          std::snprintf(item, sizeof item, " %d=%.0f", others[k], rate[others[k]]);
          out->trace += item;
        }
      out->trace += "\n";
    };

    if (!sp.two) {
      const double level = sp.slow;
      // One class only.  Fast against everything (known threshold) means the reference straddles a boundary;
      // with no threshold yet it may be either, so other references get their turn first.
      const bool straddler = abs_thr > 0.0 ? level >= abs_thr : attempts + 1 < lim.reference_attempts;
      if (straddler && attempts < lim.reference_attempts) {
        trace_line("one class, another reference is tried", abs_thr);
        if (abs_thr > 0.0) {  // a boundary slab: lumped with its predecessors
          out->slab_region[ref] = std::max(region - 1, 0);
          todo.erase(todo.begin() + (ptrdiff_t)ref_pos);
        }
        ++attempts;
        continue;
      }
      trace_line("one class: the rest shares the reference's region", abs_thr);
      for (int x : todo) out->slab_region[x] = region;
      if (abs_thr == 0.0) out->same_region_gbps = level;
      ++region;
      todo.clear();
      break;
    }

    const double thr = sp.threshold;
    for (size_t k = 0; k + 1 < others.size();) {  // refine between probed neighbours that disagree
      size_t k2 = k + 1;
      while (!probed[k2]) ++k2;
      if ((rate[others[k]] < thr) != (rate[others[k2]] < thr))
        for (size_t q = k + 1; q < k2; ++q)
          if (int rc = scan(q)) return rc;
      k = k2;
    }
    trace_line("two classes", thr);
    if (abs_thr == 0.0) {
      abs_thr = thr;
      out->same_region_gbps = sp.slow;
      out->cross_region_gbps = sp.fast;
    }
    std::vector<int> rest;
    bool same = true;
    for (size_t k = 0; k < others.size(); ++k) {
      if (probed[k]) same = rate[others[k]] < thr;  // slabs between two agreeing neighbours inherit
      if (same) out->slab_region[others[k]] = region;
      else rest.push_back(others[k]);
    }
    out->slab_region[ref] = region;
    ++region;
    attempts = 0;
    todo.swap(rest);
  }
  out->regions = std::max(region, 1);
  for (int s : todo) out->slab_region[s] = out->regions - 1;  // more groups than max_regions: lumped together
  return 0;
}

ArenaPlan plan_arena(const std::vector<int>& slab_region, int regions, size_t chunks_per_slab, size_t total_chunks,
                     size_t want_chunks, int max_regions) {
  ArenaPlan plan;
  regions = std::max(regions, 1);
  const size_t nslab = slab_region.size();
  std::vector<std::vector<size_t>> by_region((size_t)regions);
  for (size_t i = 0; i < total_chunks; ++i) {
    const size_t slab = chunks_per_slab ? i / chunks_per_slab : 0;
    int r = slab < nslab ? slab_region[slab] : (nslab ? slab_region[nslab - 1] : 0);
    r = std::min(std::max(r, 0), regions - 1);
    by_region[(size_t)r].push_back(i);
  }
  // Regions by free memory, largest first.  Groups holding under a tenth of the chunks are leftovers of the
  // scan (slabs whose chunks straddle regions when the free memory was fragmented): they serve last and are
  // not counted.
  plan.rank.resize((size_t)regions);
  for (int r = 0; r < regions; ++r) plan.rank[(size_t)r] = r;
  std::stable_sort(plan.rank.begin(), plan.rank.end(),
                   [&](int a, int c) { return by_region[(size_t)a].size() > by_region[(size_t)c].size(); });
  int real = 0;
  for (int k = 0; k < regions; ++k)
    if (by_region[(size_t)plan.rank[(size_t)k]].size() * 10 >= total_chunks) ++real;
  plan.real_regions = std::max(real, 1);
  plan.active = max_regions > 0 ? std::min(max_regions, plan.real_regions) : plan.real_regions;
  std::vector<size_t> next((size_t)regions, 0);
  plan.order.reserve(want_chunks);
  for (int lo_rank = 0; lo_rank < regions && plan.order.size() < want_chunks;) {
    const int hi_rank = lo_rank == 0 ? plan.active : regions;  // first the alternation, then whatever is left
    // A round that takes chunks from at least two regions still alternates; from the first round that finds
    // only one region with chunks left, consecutive arena chunks share a region.
    bool alternating = lo_rank == 0 && hi_rank > 1;
    while (plan.order.size() < want_chunks) {
      int contributors = 0;
      for (int k = lo_rank; k < hi_rank && plan.order.size() < want_chunks; ++k) {
        const size_t r = (size_t)plan.rank[(size_t)k];
        if (next[r] < by_region[r].size()) {
          plan.order.push_back(by_region[r][next[r]++]);
          ++contributors;
        }
      }
      if (contributors == 0) break;
      const bool cut_short = plan.order.size() == want_chunks;  // the round ended because the arena is complete
      if (contributors < 2 && !cut_short) alternating = false;
      if (alternating) plan.interleaved_chunks = plan.order.size();
    }
    lo_rank = hi_rank;
  }
  plan.region_chunks.resize((size_t)regions);
  plan.region_used.resize((size_t)regions);
  for (int k = 0; k < regions; ++k) {
    plan.region_chunks[(size_t)k] = by_region[(size_t)plan.rank[(size_t)k]].size();
    plan.region_used[(size_t)k] = next[(size_t)plan.rank[(size_t)k]];
  }
  return plan;
}

}  // namespace mxopt
