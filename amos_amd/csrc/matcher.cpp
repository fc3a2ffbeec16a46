// Matcher and mapping enumeration of the mapper (host C++).
//
// The reference does the same in three steps: an expression-structure walk in lock step
// (include/tvm/auto_tensorize/matcher.h:62-290), an index match over all injective
// assignments of intrinsic to target iteration variables (src/auto_tensorize/matcher.cc:174-310)
// and, in Python, the enumeration of unified subsets of the match points
// (python/tvm/auto_tensorize/tensorization_phases/compute_transform.py:115-207).  Here index
// expressions arrive already in affine form, so the index match is linear algebra on small
// integer rows instead of symbolic simplification.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <map>
#include <set>
#include <vector>

#include "amos_mi355x.h"
#include "mapper.h"

namespace amos {

namespace {

struct LoadView {
  int ndim;
  const int64_t* rows;  // ndim rows of (n_iters + 2)
};

std::vector<LoadView> loads_of(const amos_compute_t* c) {
  std::vector<LoadView> out;
  const int64_t* p = c->coeffs;
  for (int l = 0; l < c->n_loads; ++l) {
    out.push_back({c->load_ndim[l], p});
    p += (int64_t)c->load_ndim[l] * (c->n_iters + 2);
  }
  return out;
}

// does the assignment (intrinsic var a -> target var assign[a]) satisfy one pair of loads?
bool load_matches(const amos_compute_t* tgt, const amos_compute_t* itr, const LoadView& lt,
                  const LoadView& li, const std::vector<int>& assign) {
  const int nt = tgt->n_iters, ni = itr->n_iters;
  const int wt = nt + 2, wi = ni + 2;
  std::vector<char> used(lt.ndim, 0);
  // a mapped variable may not occur in an opaque (non-affine) target index
  for (int d = 0; d < lt.ndim; ++d) {
    const int64_t* row = lt.rows + (int64_t)d * wt;
    if (row[nt + 1]) continue;
    for (int a = 0; a < ni; ++a)
      if (row[assign[a]] != 0) return false;
  }
  for (int di = 0; di < li.ndim; ++di) {
    const int64_t* irow = li.rows + (int64_t)di * wi;
    if (!irow[ni + 1]) return false;
    bool any = false;
    for (int a = 0; a < ni; ++a) any |= irow[a] != 0;
    if (!any) continue;  // a constant intrinsic index constrains nothing
    int found = -1;
    for (int dt = 0; dt < lt.ndim && found < 0; ++dt) {
      if (used[dt]) continue;
      const int64_t* trow = lt.rows + (int64_t)dt * wt;
      if (!trow[nt + 1]) continue;
      // restricted to mapped variables, the target row must be a positive multiple of the
      // intrinsic row: trow[assign[a]] * q == irow[a] * p for one ratio p/q > 0
      int64_t p = 0, q = 0;
      bool ok = true;
      for (int a = 0; a < ni && ok; ++a) {
        const int64_t tv = trow[assign[a]], iv = irow[a];
        if ((tv == 0) != (iv == 0)) { ok = false; break; }
        if (iv == 0) continue;
        if ((tv > 0) != (iv > 0)) { ok = false; break; }
        if (p == 0) { p = tv; q = iv; }
        else if (tv * q != iv * p) ok = false;
      }
      if (ok && p != 0) found = dt;
    }
    if (found < 0) return false;
    used[found] = 1;
  }
  // every other target dimension must be constant in the mapped variables
  for (int dt = 0; dt < lt.ndim; ++dt) {
    if (used[dt]) continue;
    const int64_t* trow = lt.rows + (int64_t)dt * wt;
    for (int a = 0; a < ni; ++a)
      if (trow[assign[a]] != 0) return false;
  }
  return true;
}

}  // namespace

}  // namespace amos

using namespace amos;

extern "C" {

int amos_match(const amos_compute_t* target, const amos_compute_t* intrin, int32_t* points,
               int32_t max_points) {
  if (!target || !intrin || (!points && max_points > 0))
    return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  if (target->n_iters <= 0 || intrin->n_iters <= 0 || intrin->n_iters > 8 || target->n_iters > 64)
    return set_error(AMOS_ERR_BAD_ARG, "iteration variable count out of range");
  // 1. bodies line up node by node (kinds and dtypes), loads in the same places
  if (target->n_tokens != intrin->n_tokens || target->n_loads != intrin->n_loads) return 0;
  if (memcmp(target->tokens, intrin->tokens, sizeof(int32_t) * target->n_tokens) != 0) return 0;
  const std::vector<LoadView> lt = loads_of(target), li = loads_of(intrin);
  // 2. all injective, kind-preserving assignments, in combination-then-permutation order of
  //    the target variables
  const int nt = target->n_iters, ni = intrin->n_iters;
  std::vector<int> assign(ni, -1);
  std::vector<char> taken(nt, 0);
  int count = 0;
  // depth-first over intrinsic variables
  struct Frame { int a; int next; };
  std::vector<Frame> stack;
  stack.push_back({0, 0});
  while (!stack.empty()) {
    Frame& f = stack.back();
    if (f.a == ni) {
      bool ok = true;
      for (size_t l = 0; l < lt.size() && ok; ++l) ok = load_matches(target, intrin, lt[l], li[l], assign);
      if (ok) {
        if (count < max_points)
          for (int a = 0; a < ni; ++a) points[(int64_t)count * ni + a] = assign[a];
        ++count;
      }
      stack.pop_back();
      continue;
    }
    if (assign[f.a] >= 0) { taken[assign[f.a]] = 0; assign[f.a] = -1; }
    int t = f.next;
    while (t < nt && (taken[t] || target->iter_kinds[t] != intrin->iter_kinds[f.a])) ++t;
    if (t == nt) { stack.pop_back(); continue; }
    f.next = t + 1;
    assign[f.a] = t;
    taken[t] = 1;
    stack.push_back({f.a + 1, 0});
  }
  return count;
}

int amos_enumerate_mappings(int32_t n_points, int32_t n_axes, const int32_t* points,
                            const int64_t* target_extents, const int64_t* intrin_extents,
                            uint8_t* bits, uint8_t* feasible, int32_t max_mappings) {
  if (n_points <= 0 || n_axes <= 0 || !points || !target_extents || !intrin_extents || !bits || !feasible)
    return set_error(AMOS_ERR_BAD_ARG, "bad argument to amos_enumerate_mappings");
  if (n_points > 62) return set_error(AMOS_ERR_UNSUPPORTED, "more than 62 match points");
  std::vector<std::vector<uint8_t>> candidates;
  if (n_points <= 15) {
    for (uint32_t v = 1; v < (1u << n_points); ++v) {
      std::vector<uint8_t> b(n_points);
      for (int i = 0; i < n_points; ++i) b[i] = (v >> (n_points - 1 - i)) & 1;  // first point = MSB
      candidates.push_back(b);
    }
  } else {
    for (int i = 0; i < n_points; ++i) {
      bool equal = true;
      for (int a = 0; a < n_axes; ++a)
        equal &= target_extents[points[(int64_t)i * n_axes + a]] == intrin_extents[a];
      if (equal) {
        std::vector<uint8_t> b(n_points, 0);
        b[i] = 1;
        candidates.push_back(b);
      }
    }
    if (candidates.empty())
      for (int i = 0; i < n_points; ++i) {
        std::vector<uint8_t> b(n_points, 0);
        b[i] = 1;
        candidates.push_back(b);
      }
    candidates.push_back(std::vector<uint8_t>(n_points, 1));
  }
  std::set<std::vector<std::vector<int>>> visited;
  int count = 0;
  for (const auto& b : candidates) {
    std::vector<std::vector<int>> key(n_axes);
    for (int a = 0; a < n_axes; ++a) {
      std::set<int> s;
      for (int i = 0; i < n_points; ++i)
        if (b[i]) s.insert(points[(int64_t)i * n_axes + a]);
      key[a].assign(s.begin(), s.end());
    }
    if (!visited.insert(key).second) continue;
    if (count < max_mappings) {
      memcpy(bits + (int64_t)count * n_points, b.data(), n_points);
      bool ok = true;
      for (int a = 0; a < n_axes; ++a) {
        if (intrin_extents[a] <= 1) continue;
        int64_t fused = 1;
        for (int id : key[a]) fused *= target_extents[id];
        ok &= fused >= intrin_extents[a];
      }
      feasible[count] = ok ? 1 : 0;
    }
    ++count;
  }
  return count;
}

}  // extern "C"
