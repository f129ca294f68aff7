// The other layer entry points: convolution (implicit GEMM, filter stamps, generator windows), the ReLU step's
// C entry points and the layer loop of NN.reach in one call.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>

#include "internal.h"

using namespace nnvhip;

extern "C" {

int nnvhip_affine_conv2d(nnvhip_ctx* c, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t count,
                         nnvhip_star* const* in, nnvhip_star** out) {
  CHECK_CTX(c);
  if (!cv || cv->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid layer handle");
  NNV_TRY(check_set_array(c, count, in, out));
  if (H <= 0 || W <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "The input is not an ImageStar object");
  for (int64_t i = 0; i < count; ++i) {
    if (in[i]->N % (H * W) != 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension in the ImageStar and the original Star set");
    int64_t ch = in[i]->N / (H * W);
    if (ch != cv->Cin)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Input set contains %lld channels while the convolutional layers has %lld channels",
               (long long)ch, (long long)cv->Cin);
  }
  int64_t Ho = 0, Wo = 0;
  NNV_TRY(nnvhip_conv2d_output_size(cv, H, W, &Ho, &Wo));
  int64_t Nout = Ho * Wo * cv->Cout;
  if (Nout >= (int64_t(1) << 31) || in[0]->N >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "image too large");
  std::vector<nnvhip_star*> outs;
  bool contig = false;
  int64_t cols = 0;
  NNV_TRY(c->begin_op());
  int st = make_affine_outputs(c, count, in, Nout, &outs, &contig, &cols);
  // generator images that are scaled unit vectors (box ImageStars, columns appended by a ReLU) turn
  // into stamps of the filter; the implicit GEMM runs over the leading dense images only
  std::vector<ConvStampSet> stamps((size_t)count);
  auto mask_on_load = [&](const nnvhip_star* s) {
    return !c->no_conv_mask && s->cls != nullptr && conv2d_can_mask(cv, H, W, Ho, Wo, s->ld);
  };
  bool any_stamps = false;
  int64_t max_m = 0;
  // Windows of the generator images (internal.h, nnvhip_star::box).  The output's come from the input's windows and
  // from the pixels of its unit-vector columns (without either an image counts as full); where the input's dense
  // images have small windows the implicit GEMM computes inside the output windows only.
  const bool track_boxes = !c->no_conv_boxes && H < 32768 && W < 32768 && Ho < 32768 && Wo < 32768;
  struct Plan {
    int64_t nc = 0, dense = 0, m = 0;
    bool in_ok = false;      // the input's windows describe its dense images
    bool out_boxes = false;  // the output gets windows
    bool compact = false;    // the dense images are computed inside their windows only
    int dense_eh = 0, dense_ew = 0;
  };
  std::vector<Plan> plan((size_t)count);
  for (int64_t i = 0; i < count; ++i) {
    Plan& pl = plan[i];
    pl.nc = in[i]->n + 1;
    pl.dense = (!c->dense_affine && in[i]->oh_from > 0 && in[i]->oh_from < pl.nc) ? in[i]->oh_from : pl.nc;
    pl.m = pl.nc - pl.dense;
    if (!track_boxes) continue;
    pl.in_ok = in[i]->box != nullptr && in[i]->box_H == H && in[i]->box_W == W && in[i]->box_cols >= pl.dense;
    pl.out_boxes = pl.in_ok || (pl.m > 0 && pl.dense == 1);
    if (pl.in_ok && pl.dense > 1) {
      pl.dense_eh = (int)conv_box_extent(cv, 0, in[i]->box_eh, Ho);
      pl.dense_ew = (int)conv_box_extent(cv, 1, in[i]->box_ew, Wo);
      // (any table will do for the question; the real one is made below)
      pl.compact = conv2d_in_windows(cv, H, W, Ho, Wo, in[i]->ld, pl.dense, in[i]->box, pl.dense_eh, pl.dense_ew);
    }
  }
  {
    // The implicit GEMM reads whole images: pending row resets are run first, and sets whose unit-vector
    // columns take part in the contraction get those written out.  (A pending reset alone is applied by the
    // kernel as it loads, from one bit per row, where that fits; images that are in memory inside their windows
    // only are fine for the kernel that stays inside the windows.)
    std::vector<nnvhip_star*> full, prefix;
    for (int64_t i = 0; i < count; ++i) {
      const ColSource& cs = in[i]->cs;
      if (plan[i].dense > in[i]->stored_cols())
        full.push_back(in[i]);
      else if (cs.pending || cs.zero_to > 1 || cs.delta_pending() || (cs.win_pending() && !plan[i].compact) ||
               (in[i]->rows_pending && !mask_on_load(in[i])))
        prefix.push_back(in[i]);
    }
    if (st == NNVHIP_OK && !full.empty()) st = ensure_dense_batch(c, (int64_t)full.size(), full.data());
    if (st == NNVHIP_OK && !prefix.empty()) st = ensure_dense_batch(c, (int64_t)prefix.size(), prefix.data(), false);
  }
  // range sums of the stamped columns, left on the output handles: one buffer for the call
  for (int64_t i = 0; i < count; ++i) {
    any_stamps = any_stamps || plan[i].m > 0;
    max_m = std::max<int64_t>(max_m, plan[i].m);
  }
  const int64_t sch = any_stamps && st == NNVHIP_OK ? conv_stamp_chunks(cv, outs[0]->ld, count, max_m) : 0;
  BufRef sums;
  if (sch > 0) st = c->alloc(sizeof(double) * 4 * outs[0]->ld * sch * count, &sums);
  std::vector<char> stamped((size_t)count, 0);
  for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
    const Plan& pl = plan[i];
    nnvhip_star* o = outs[i];
    const ColBox* ob = nullptr;
    if (pl.out_boxes) {
      st = c->alloc(sizeof(ColBox) * (size_t)pl.nc, &o->box_buf);
      if (st != NNVHIP_OK) break;
      ColBox* tab = o->box_buf->as<ColBox>();
      st = launch_conv_boxes(c, cv, H, W, Ho, Wo, pl.in_ok ? in[i]->box : nullptr, pl.dense, in[i]->oh_idx, pl.m, tab);
      if (st != NNVHIP_OK) break;
      int64_t eh = pl.dense > 1 ? pl.dense_eh : 0, ew = pl.dense > 1 ? pl.dense_ew : 0;
      if (pl.m > 0) {
        eh = std::max(eh, conv_box_extent(cv, 0, 1, Ho));
        ew = std::max(ew, conv_box_extent(cv, 1, 1, Wo));
      }
      ob = tab;
      o->box = tab;
      o->box_cols = pl.nc;
      o->box_H = (int32_t)Ho;
      o->box_W = (int32_t)Wo;
      o->box_eh = (int32_t)eh;
      o->box_ew = (int32_t)ew;
    }
    // Images with windows are written inside them only; the zeros around them wait for a reader of whole
    // columns (ColSource::win_*).  Not when the caller wants every column in memory.
    const bool lazy = ob != nullptr && !c->eager_cols;
    const int64_t win_from = lazy ? (pl.compact ? 1 : pl.dense) : 0;
    const int64_t win_to = lazy ? (pl.m > 0 ? pl.nc : (pl.compact ? pl.dense : 0)) : 0;
    if (win_to > win_from) {
      o->cs.win_box_buf = o->box_buf;
      o->cs.win_box = ob;
      o->cs.win_from = win_from;
      o->cs.win_to = win_to;
      o->cs.win_rows = Nout;
      o->cs.win_H = (int32_t)Ho;
      o->cs.win_W = (int32_t)Wo;
      if (c->poison_pending)  // debugging aid: NaNs where nothing will be written
        NNV_HIP_TRY(hipMemsetAsync(o->V + win_from * o->ld, 0xff, sizeof(double) * o->ld * (win_to - win_from), c->stream));
    }
    stamps[i].idx = in[i]->oh_idx;
    stamps[i].scale = in[i]->oh_scale;
    stamps[i].out = o->V + pl.dense * o->ld;
    stamps[i].plb = o->plb + (pl.dense - 1);
    stamps[i].pub = o->pub + (pl.dense - 1);
    stamps[i].part = sums ? sums->as<double>() + 4 * outs[0]->ld * sch * i : nullptr;
    stamps[i].m = (int32_t)pl.m;
    if (pl.m > 0 && in[i]->oh_inv == nullptr && conv_stamps_by_pixel(cv)) {
      // (kept on the input: its columns do not change, and an input set is usually mapped again)
      st = launch_pixel_columns(c, in[i]->oh_idx, pl.m, in[i]->N, &in[i]->oh_inv_buf);
      if (st != NNVHIP_OK) break;
      in[i]->oh_inv = in[i]->oh_inv_buf->as<int32_t>();
    }
    stamps[i].pixel_col = in[i]->oh_inv;
    stamps[i].win_only = (lazy && pl.m > 0) ? 1 : 0;
    bool done = false;
    st = launch_conv2d(c, cv, H, W, Ho, Wo, in[i]->V, in[i]->ld, o->V, o->ld, pl.dense,
                       in[i]->rows_pending ? in[i]->cls : nullptr, pl.compact ? ob : nullptr, pl.dense_eh, pl.dense_ew,
                       pl.compact ? in[i]->box : nullptr, pl.compact && lazy, in[i]->rows_pending ? in[i]->keep_bits : nullptr,
                       sch == 1 ? &stamps[i] : nullptr, &done);
    stamped[(size_t)i] = done ? 1 : 0;
    // (launch_conv2d zeroes the padding rows of the columns it writes; the stamp kernel only writes them when
    // it writes whole columns)
    if (st == NNVHIP_OK && stamps[i].win_only && o->ld != Nout) st = launch_zero_pad_rows(c, stamps[i].out, o->ld, Nout, pl.m);
  }
  if (st == NNVHIP_OK && any_stamps) {
    // the stamp pass also leaves the range sums of its columns on the output handles; sets whose stamps went into
    // their convolution's launch are done
    std::vector<ConvStampSet> rest = stamps;
    bool any_left = false;
    for (int64_t i = 0; i < count; ++i) {
      if (stamped[(size_t)i]) rest[(size_t)i].m = 0;
      any_left = any_left || rest[(size_t)i].m > 0;
    }
    if (any_left) st = launch_conv_stamps(c, cv, H, W, Ho, Wo, outs[0]->ld, count, rest.data(), sch);
    for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
      if (stamps[i].m > 0) {
        outs[i]->rng_buf = sums;
        outs[i]->rng_part = stamps[i].part;
        outs[i]->rng_chunks = sch;
        outs[i]->rng_first_col = (in[i]->n + 1) - stamps[i].m;
      }
  }
  if (st == NNVHIP_OK) st = c->end_op();
  if (st != NNVHIP_OK) {
    release_all(outs);
    return st;
  }
  for (int64_t i = 0; i < count; ++i) out[i] = outs[i];
  return NNVHIP_OK;
}

int nnvhip_relu_relax(nnvhip_ctx* c, int order, double relax_factor, int64_t count, nnvhip_star* const* in,
                      nnvhip_star** out) {
  CHECK_CTX(c);
  NNV_TRY(check_set_array(c, count, in, out));
  if (order != NNVHIP_ORDER_INDEX && order != NNVHIP_ORDER_AREA && order != NNVHIP_ORDER_RANGE)
    NNV_FAIL(NNVHIP_ERR_METHOD, "This reachability method does not exist");
  if (!(relax_factor >= 0.0 && relax_factor <= 1.0)) NNV_FAIL(NNVHIP_ERR_RELAX_FACTOR, "Invalid relax factor");
  if (relax_factor != 1.0)
    NNV_FAIL(NNVHIP_ERR_RELAX_FACTOR, "relaxFactor < 1 needs the LP-based range optimisation, which this library does not provide");
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N != in[0]->N) NNV_FAIL(NNVHIP_ERR_SHAPE, "sets of one array must have the same dimension");
  NNV_TRY(c->begin_op());
  NNV_TRY(relu_relax(c, order, count, in, out));
  return c->end_op();
}

int nnvhip_reach_layers(nnvhip_ctx* c, int64_t n_layers, const int32_t* kind, const void* const* layer, const int64_t* hw,
                        int order, double relax_factor, int64_t count, nnvhip_star* const* in, nnvhip_star** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (n_layers < 0 || count <= 0 || !in || (n_layers > 0 && (!kind || !layer || !out))) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  nnvhip_star* const* cur = in;
  int st = NNVHIP_OK;
  int64_t done = 0;
  if (n_layers > 0 && relax_factor == 1.0) {
    // small fully connected networks: the whole loop below as one launch
    NNV_TRY(nnvhip::enter_ctx(c));
    bool taken = false;
    for (int64_t t = 0; t < n_layers * count; ++t) out[t] = nullptr;
    st = reach_small_chain(c, n_layers, kind, layer, order, count, in, out, &taken);
    if (taken) {
      if (st != NNVHIP_OK)
        for (int64_t t = 0; t < n_layers * count; ++t) {
          nnvhip_star_release(out[t]);
          out[t] = nullptr;
        }
      return st;
    }
  }
  for (int64_t l = 0; l < n_layers && st == NNVHIP_OK; ++l) {
    nnvhip_star** dst = out + l * count;
    // the set that is handed back is written in full by the layer that produces it
    const bool eager = l == n_layers - 1 && !c->eager_cols;
    if (eager) c->eager_cols = true;
    switch (kind[l]) {
      case NNVHIP_LAYER_FC:
        st = nnvhip_affine_fc(c, static_cast<const nnvhip_fc*>(layer[l]), count, cur, dst);
        break;
      case NNVHIP_LAYER_CONV2D:
        if (!hw) {
          set_error("null argument");
          st = NNVHIP_ERR_ARG;
        } else {
          st = nnvhip_affine_conv2d(c, static_cast<const nnvhip_conv2d*>(layer[l]), hw[2 * l], hw[2 * l + 1], count, cur, dst);
        }
        break;
      case NNVHIP_LAYER_RELU:
        st = nnvhip_relu_relax(c, order, relax_factor, count, cur, dst);
        break;
      default:
        set_error("unknown layer kind %d", (int)kind[l]);
        st = NNVHIP_ERR_ARG;
    }
    if (eager) c->eager_cols = false;
    if (st == NNVHIP_OK) {
      cur = dst;
      done = l + 1;
    }
  }
  if (st != NNVHIP_OK) {
    for (int64_t t = 0; t < done * count; ++t) {
      nnvhip_star_release(out[t]);
      out[t] = nullptr;
    }
  }
  return st;
}

int nnvhip_relu_apply_lists(nnvhip_ctx* c, nnvhip_star* in, int64_t n_reset, const int32_t* reset_rows, int64_t m,
                            const int32_t* index, const double* lb, const double* ub, nnvhip_star** out) {
  CHECK_CTX(c);
  if (!in || in->ctx != c || !out) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle");
  if (n_reset < 0 || m < 0 || (n_reset > 0 && !reset_rows) || (m > 0 && (!index || !lb || !ub)))
    NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  const int64_t N = in->N;
  // per-row bounds that make the classification reproduce the two lists: a reset row looks inactive
  // (ub = 0), a listed neuron carries its own (lb, ub), every other row looks active; the keys put the
  // new predicates in the order of the list
  std::vector<double> rows((size_t)(3 * N));
  double* L = rows.data();
  double* U = L + N;
  double* K = U + N;
  std::vector<char> seen((size_t)N, 0);
  for (int64_t r = 0; r < N; ++r) {
    L[r] = 0.0;
    U[r] = 1.0;
    K[r] = 0.0;
  }
  for (int64_t t = 0; t < n_reset; ++t) {
    const int64_t r = reset_rows[t];
    if (r < 0 || r >= N) NNV_FAIL(NNVHIP_ERR_ARG, "Invalid index");
    if (seen[r]) NNV_FAIL(NNVHIP_ERR_ARG, "row %lld is listed twice", (long long)r);
    seen[r] = 1;
    L[r] = -1.0;
    U[r] = 0.0;
  }
  for (int64_t t = 0; t < m; ++t) {
    const int64_t r = index[t];
    if (r < 0 || r >= N) NNV_FAIL(NNVHIP_ERR_ARG, "Invalid index");
    if (seen[r]) NNV_FAIL(NNVHIP_ERR_ARG, "row %lld is listed twice", (long long)r);
    if (!(lb[t] < 0.0 && ub[t] > 0.0)) NNV_FAIL(NNVHIP_ERR_ARG, "neuron %lld: the triangle relaxation needs lb < 0 < ub", (long long)r);
    seen[r] = 1;
    L[r] = lb[t];
    U[r] = ub[t];
    K[r] = (double)(m - t);
  }
  NNV_TRY(c->begin_op());
  BufRef dev;
  NNV_TRY(c->upload(rows.data(), sizeof(double) * 3 * N, &dev));
  ReluGiven g{dev->as<double>(), dev->as<double>() + N, dev->as<double>() + 2 * N};
  NNV_TRY(relu_relax(c, kOrderGiven, 1, &in, out, &g));
  return c->end_op();
}

}  // extern "C"
