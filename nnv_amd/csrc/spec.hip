// LP-free part of the specification check (utils/verify_specification.m:36-80): the output sets
// are mapped through the stacked half-space matrices with the skinny GEMM, the rows of the result
// are bounded over the predicate box by the estimateRanges kernels, and the three-way verdict per
// (set, half-space) is formed on the host from R x count doubles.  The dense constraint matrix is
// never touched here.
#include <algorithm>
#include <cmath>
#include <memory>
#include <vector>

#include "internal.h"

using namespace nnvhip;

namespace {

constexpr double kSpecMargin = 1e-9;  // relative to max(|lo|, |hi|, |g|) of the row

struct FcGuard {
  nnvhip_fc* fc = nullptr;
  ~FcGuard() {
    if (fc) nnvhip_fc_destroy(fc);
  }
};

struct StarsGuard {
  std::vector<nnvhip_star*> v;
  ~StarsGuard() {
    for (auto* s : v)
      if (s) nnvhip_star_release(s);
  }
};

int check_sets(nnvhip_ctx* c, int64_t count, nnvhip_star* const* sets, int64_t N) {
  if (!sets || count <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  for (int64_t i = 0; i < count; ++i) {
    if (!sets[i] || sets[i]->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle %lld", (long long)i);
    if (sets[i]->N != N) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension between halfspace and star set");
  }
  return NNVHIP_OK;
}

}  // namespace

extern "C" {

int nnvhip_halfspace_check(nnvhip_ctx* c, int64_t count, nnvhip_star* const* sets, int64_t n_hs, const int64_t* row_ptr,
                           const double* G, const double* g, int64_t N, int32_t* verdict, double* lo, double* hi) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  NNV_TRY(nnvhip::enter_ctx(c));
  if (!row_ptr || !G || !g || n_hs <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (row_ptr[0] != 0) NNV_FAIL(NNVHIP_ERR_ARG, "row_ptr must start at 0");
  for (int64_t h = 0; h < n_hs; ++h)
    if (row_ptr[h + 1] <= row_ptr[h])
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension between Halfspace matrix and halfspace vector");
  const int64_t R = row_ptr[n_hs];
  NNV_TRY(check_sets(c, count, sets, N));

  FcGuard map;
  NNV_TRY(nnvhip_fc_create(c, G, nullptr, R, N, &map.fc));
  StarsGuard mapped;
  mapped.v.assign(count, nullptr);
  NNV_TRY(nnvhip_affine_fc(c, map.fc, count, sets, mapped.v.data()));
  std::vector<double> lo_h((size_t)(R * count)), hi_h((size_t)(R * count));
  NNV_TRY(nnvhip_estimate_ranges_batch(c, count, mapped.v.data(), lo_h.data(), hi_h.data()));

  for (int64_t s = 0; s < count; ++s) {
    const double* l = lo_h.data() + s * R;
    const double* u = hi_h.data() + s * R;
    for (int64_t h = 0; h < n_hs; ++h) {
      bool disjoint = false, inside = true;
      for (int64_t r = row_ptr[h]; r < row_ptr[h + 1]; ++r) {
        // "disjoint" is the verdict a caller reports as robust, and the bounds carry rounding of the order of
        // the row's scale: a pair is only called disjoint with a margin beyond that; a pair inside the margin
        // stays undecided and goes to the LP, as the reference decides every pair
        const double scale = std::max(std::max(std::fabs(l[r]), std::fabs(u[r])), std::fabs(g[r]));
        disjoint = disjoint || l[r] - g[r] > kSpecMargin * scale;
        inside = inside && u[r] <= g[r];
      }
      if (verdict) verdict[s + count * h] = disjoint ? NNVHIP_HS_DISJOINT : inside ? NNVHIP_HS_INSIDE : NNVHIP_HS_UNDECIDED;
    }
  }
  if (lo) std::copy(lo_h.begin(), lo_h.end(), lo);
  if (hi) std::copy(hi_h.begin(), hi_h.end(), hi);
  return NNVHIP_OK;
}

int nnvhip_halfspace_rows(nnvhip_ctx* c, nnvhip_star* s, int64_t R, const double* G, const double* g, int64_t N,
                          double* C1, double* d1) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  NNV_TRY(nnvhip::enter_ctx(c));
  if (!G || !g || R <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  NNV_TRY(check_sets(c, 1, &s, N));
  FcGuard map;
  NNV_TRY(nnvhip_fc_create(c, G, nullptr, R, N, &map.fc));
  StarsGuard mapped;
  mapped.v.assign(1, nullptr);
  NNV_TRY(nnvhip_affine_fc(c, map.fc, 1, &s, mapped.v.data()));
  const int64_t n = s->n;
  std::vector<double> Y((size_t)(R * (n + 1)));
  NNV_TRY(nnvhip_star_fetch_V(mapped.v[0], Y.data()));
  if (C1) std::copy(Y.begin() + R, Y.end(), C1);  // G * V(:, 2:n+1)
  if (d1)
    for (int64_t r = 0; r < R; ++r) d1[r] = g[r] - Y[(size_t)r];  // g - G * V(:, 1)
  return NNVHIP_OK;
}

}  // extern "C"
