// Set handles: constructors (Star(V, C, d, lb, ub), Star(lb, ub) for arrays of boxes, the reduceMem box), reference
// counting, property reads and the estimateRanges entry points.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>

#include "internal.h"

using namespace nnvhip;

extern "C" {

/* ------------------------------------------------------------------------------------------ */
/* sets                                                                                        */
/* ------------------------------------------------------------------------------------------ */

// Uploads a host column-major rows x cols matrix into a zero-padded device matrix with leading
// dimension ld.
static int upload_matrix(nnvhip_ctx* c, const double* host, int64_t rows, int64_t cols, int64_t ld,
                         double* dev) {
  if (rows == 0 || cols == 0) return NNVHIP_OK;
  if (ld != rows) NNV_HIP_TRY(hipMemsetAsync(dev, 0, sizeof(double) * ld * cols, c->stream));
  NNV_HIP_TRY(hipMemcpy2DAsync(dev, sizeof(double) * ld, host, sizeof(double) * rows, sizeof(double) * rows,
                               cols, hipMemcpyHostToDevice, c->stream));
  c->h2d_bytes += (int64_t)sizeof(double) * rows * cols;
  // the source is pageable caller memory: finish before returning
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_star_create(nnvhip_ctx* c, int64_t N, int64_t n, const double* V, const double* pred_lb,
                       const double* pred_ub, const double* C, const double* d, int64_t p,
                       nnvhip_star** out) {
  CHECK_CTX(c);
  if (!out || !V) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (N <= 0 || n < 0 || p < 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "invalid set size N=%lld n=%lld p=%lld", (long long)N, (long long)n, (long long)p);
  if ((pred_lb == nullptr) != (pred_ub == nullptr))
    NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistency between number of predicate variables and predicate lower- or upper-bounds vector");
  if (p > 0 && (!C || !d)) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistency between constraint matrix and constraint vector");
  nnvhip_star* s = new_star(c);
  std::unique_ptr<nnvhip_star, int (*)(nnvhip_star*)> guard(s, nnvhip_star_release);
  s->N = N;
  s->n = n;
  s->ld = round_up(N, kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * s->ld * (n + 1), &s->Vbuf));
  s->V = s->Vbuf->as<double>();
  NNV_TRY(upload_matrix(c, V, N, n + 1, s->ld, s->V));
  int64_t npad = round_up(std::max<int64_t>(n, 1), kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * 2 * npad, &s->pbuf));
  s->plb = s->pbuf->as<double>();
  s->pub = s->plb + npad;
  if (n > 0) {
    std::vector<double> tmp(2 * npad, 0.0);
    for (int64_t i = 0; i < n; ++i) {
      tmp[i] = pred_lb ? pred_lb[i] : -1.0;  // default of Star.estimateRanges, set/Star.m:1091-1096
      tmp[npad + i] = pred_ub ? pred_ub[i] : 1.0;
    }
    NNV_HIP_TRY(hipMemcpyAsync(s->plb, tmp.data(), sizeof(double) * 2 * npad, hipMemcpyHostToDevice, c->stream));
    c->h2d_bytes += (int64_t)sizeof(double) * 2 * npad;
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  auto base = make_ref<ConsNode>();
  base->p_total = p;
  base->n_total = n;
  if (p > 0 && n > 0) {
    base->ldc = round_up(p, kLdAlign);
    NNV_TRY(c->alloc(sizeof(double) * base->ldc * n, &base->C0));
    NNV_TRY(upload_matrix(c, C, p, n, base->ldc, base->C0->as<double>()));
  }
  if (p > 0) {
    NNV_TRY(c->alloc(sizeof(double) * p, &base->d0));
    NNV_HIP_TRY(hipMemcpyAsync(base->d0->ptr, d, sizeof(double) * p, hipMemcpyHostToDevice, c->stream));
    c->h2d_bytes += (int64_t)sizeof(double) * p;
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  s->cons = base;
  *out = guard.release();
  return NNVHIP_OK;
}

__global__ void box_fill_kernel(double* __restrict__ V, int64_t ld, int N, const double* __restrict__ center,
                                const double* __restrict__ vec, const int32_t* __restrict__ gen_dim,
                                const int64_t* __restrict__ col_off, const int64_t* __restrict__ gen_off) {
  // one block column per (set, column); rows across threads.  Column 0 is the centre; column
  // 1+g holds vec(dim_g) at row dim_g and zeros elsewhere (diag(vec) with empty columns removed).
  int set = blockIdx.z;
  int64_t ncols = col_off[set + 1] - col_off[set];
  for (int64_t j = blockIdx.y; j < ncols; j += gridDim.y) {
    double* col = V + (col_off[set] + j) * ld;
    int dim = j == 0 ? -1 : gen_dim[gen_off[set] + j - 1];
    // two rows per thread, one 16-byte store (ld is even and every column starts on a 16-byte boundary)
    for (int r = 2 * (blockIdx.x * blockDim.x + threadIdx.x); r < ld; r += 2 * gridDim.x * blockDim.x) {
      double v[2] = {0.0, 0.0};
#pragma unroll
      for (int e = 0; e < 2; ++e)
        if (r + e < N) {
          if (j == 0) v[e] = center[(int64_t)set * N + r + e];
          else if (r + e == dim) v[e] = vec[(int64_t)set * N + r + e];
        }
      *reinterpret_cast<double2*>(col + r) = make_double2(v[0], v[1]);
    }
  }
}

// info[2s] = offset of set s in the bounds buffer, info[2s+1] = its padded predicate count
__global__ void fill_pm_one_kernel(double* __restrict__ bounds, const int64_t* __restrict__ info) {
  const int64_t off = info[2 * blockIdx.y], n = info[2 * blockIdx.y + 1];
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i < n) {
    bounds[off + i] = -1.0;
    bounds[off + n + i] = 1.0;
  }
}

int nnvhip_star_from_box(nnvhip_ctx* c, int64_t N, int64_t count, const double* lb, const double* ub,
                         nnvhip_star** out) {
  CHECK_CTX(c);
  if (!lb || !ub || !out) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (N <= 0 || count <= 0 || count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimensions between lb and ub");
  // Box constructor arithmetic on the host (set/Box.m:35-45): it decides the column count.
  std::vector<double> center(N * count), vec(N * count);
  std::vector<int32_t> gen_dim;
  std::vector<int64_t> col_off(count + 1, 0), gen_off(count + 1, 0);
  std::vector<char> neg_scale((size_t)count, 0);
  // Sets with the same half-widths, bit for bit (the boxes of a regular partition), share one scale vector and one
  // index list on the device: layers downstream recognise by the pointers that such sets gather the same scaled
  // weight columns.  shape_of[s] = the first set with set s's half-widths (among the first few distinct shapes).
  std::vector<int64_t> shape_of((size_t)count);
  std::vector<int64_t> shapes;
  std::vector<uint64_t> shape_hash;
  for (int64_t s = 0; s < count; ++s) {
    int64_t n = 0;
    uint64_t hash = 0x9E3779B97F4A7C15ull;  // of the half-widths' bit patterns: vectors are compared only when it matches
    for (int64_t i = 0; i < N; ++i) {
      double l = lb[s * N + i], u = ub[s * N + i];
      center[s * N + i] = 0.5 * (l + u);
      double v = 0.5 * (u - l);
      vec[s * N + i] = v;
      uint64_t bits;
      memcpy(&bits, &v, sizeof bits);
      hash = (hash ^ bits) * 0x100000001B3ull;
      hash ^= hash >> 29;
      if (v < 0.0) neg_scale[s] = 1;
      // zero columns are deleted only when the generator matrix has more than one element
      if (v != 0.0 || N == 1) {
        gen_dim.push_back((int32_t)i);
        ++n;
      }
    }
    gen_off[s + 1] = gen_off[s] + n;
    col_off[s + 1] = col_off[s] + n + 1;
    shape_of[s] = s;
    for (size_t k = 0; k < shapes.size(); ++k)
      if (shape_hash[k] == hash && memcmp(&vec[shapes[k] * N], &vec[s * N], sizeof(double) * N) == 0) {
        shape_of[s] = shapes[k];
        break;
      }
    if (shape_of[s] == s && shapes.size() < 16) {
      shapes.push_back(s);
      shape_hash.push_back(hash);
    }
  }
  int64_t ld = round_up(N, kLdAlign);
  int64_t total_cols = col_off[count];
  BufRef arena, dcenter, dvec, dgen, dcol, dgoff;
  NNV_TRY(c->alloc(sizeof(double) * ld * total_cols, &arena));
  NNV_TRY(c->upload(center.data(), sizeof(double) * center.size(), &dcenter));
  NNV_TRY(c->upload(vec.data(), sizeof(double) * vec.size(), &dvec));
  if (gen_dim.empty()) gen_dim.push_back(0);
  NNV_TRY(c->upload(gen_dim.data(), sizeof(int32_t) * gen_dim.size(), &dgen));
  NNV_TRY(c->upload(col_off.data(), sizeof(int64_t) * col_off.size(), &dcol));
  NNV_TRY(c->upload(gen_off.data(), sizeof(int64_t) * gen_off.size(), &dgoff));
  int64_t max_cols = 0;
  for (int64_t s = 0; s < count; ++s) max_cols = std::max(max_cols, col_off[s + 1] - col_off[s]);
  dim3 grid((unsigned)std::min<int64_t>(ceil_div(ld, 512), 64), (unsigned)std::min<int64_t>(max_cols, 4096),
            (unsigned)count);
  hipLaunchKernelGGL(box_fill_kernel, grid, dim3(256), 0, c->stream, arena->as<double>(), ld, (int)N,
                     dcenter->as<double>(), dvec->as<double>(), dgen->as<int32_t>(), dcol->as<int64_t>(),
                     dgoff->as<int64_t>());
  NNV_HIP_TRY(hipGetLastError());
  // predicate bounds -1/+1 for all sets in one buffer
  int64_t npad_total = 0;
  std::vector<int64_t> poff(count);
  for (int64_t s = 0; s < count; ++s) {
    poff[s] = npad_total;
    npad_total += 2 * round_up(std::max<int64_t>(gen_off[s + 1] - gen_off[s], 1), kLdAlign);
  }
  BufRef pb;
  NNV_TRY(c->alloc(sizeof(double) * npad_total, &pb));
  for (int64_t s = 0; s < count; ++s) {
    nnvhip_star* st = new_star(c);
    st->N = N;
    st->n = gen_off[s + 1] - gen_off[s];
    st->ld = ld;
    st->Vbuf = arena;
    st->V = arena->as<double>() + col_off[s] * ld;
    st->pbuf = pb;
    int64_t npad = round_up(std::max<int64_t>(st->n, 1), kLdAlign);
    st->plb = pb->as<double>() + poff[shape_of[s]];  // (the same -1 / +1 for every set of the shape)
    st->pub = st->plb + npad;
    // C = zeros(1, n), d = 0 (set/Star.m:226-227): a base node with one all-zero row
    auto base = make_ref<ConsNode>();
    base->p_total = 1;
    base->n_total = st->n;
    st->cons = base;  // C0/d0 left null = all zeros
    st->has_zono = true;  // Z = Zono(center, gens), set/Star.m:230-236
    if (st->n > 0) {  // every generator column is vec(dim) * e_dim
      st->oh_from = 1;
      st->oh_idx_buf = dgen;
      st->oh_idx = dgen->as<int32_t>() + gen_off[shape_of[s]];
      st->oh_scale_buf = dvec;
      st->oh_scale = dvec->as<double>() + shape_of[s] * N;
      st->oh_scale_neg = neg_scale[s] != 0;
    }
    out[s] = st;
  }
  // one launch fills every set's bounds: lb half gets -1, ub half +1
  {
    std::vector<int64_t> pinfo((size_t)(2 * count));
    int64_t max_npad = 0;
    for (int64_t s = 0; s < count; ++s) {
      pinfo[2 * s] = poff[s];
      pinfo[2 * s + 1] = round_up(std::max<int64_t>(out[s]->n, 1), kLdAlign);
      max_npad = std::max(max_npad, pinfo[2 * s + 1]);
    }
    BufRef dinfo;
    NNV_TRY(c->upload(pinfo.data(), sizeof(int64_t) * pinfo.size(), &dinfo));
    hipLaunchKernelGGL(fill_pm_one_kernel, dim3((unsigned)ceil_div(max_npad, 256), (unsigned)count), dim3(256), 0, c->stream,
                       pb->as<double>(), dinfo->as<int64_t>());
  }
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

// Columns of the set the reduceMem suffix of the ReLU layer builds: column 0 the centre, column 1 + g the value
// val[g] on every channel of pixel pix[g] (rows pix[g] + k * HW), every other entry zero.
__global__ void rebox_fill_kernel(double* __restrict__ V, int64_t ld, int N, int HW, int64_t ncols, int ngen,
                                  const double* __restrict__ center, const int32_t* __restrict__ pix,
                                  const double* __restrict__ val) {
  for (int64_t j = blockIdx.y; j < ncols; j += gridDim.y) {
    double* col = V + j * ld;
    const int p = (j >= 1 && j - 1 < ngen) ? pix[j - 1] : -1;
    const double pv = p >= 0 ? val[j - 1] : 0.0;
    for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < ld; r += gridDim.x * blockDim.x) {
      double v = 0.0;
      if (r < N) {
        if (j == 0) v = center[r];
        else if (p >= 0 && r % HW == p) v = pv;
      }
      col[r] = v;
    }
  }
}

int nnvhip_relu_reduce_mem(nnvhip_ctx* c, nnvhip_star* in, int64_t H, int64_t W, int64_t C, nnvhip_star** out, double* im_lb,
                           double* im_ub) {
  CHECK_CTX(c);
  if (!in || in->ctx != c || !out) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle");
  if (H <= 0 || W <= 0 || C <= 0 || H * W * C != in->N)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension in the ImageStar and the original Star set");
  const int64_t N = in->N, HW = H * W;
  // [l, u] = images(i).estimateRanges
  NNV_TRY(compute_ranges(c, 1, &in));
  std::vector<double> l((size_t)N), u((size_t)N);
  NNV_HIP_TRY(hipMemcpyAsync(l.data(), in->lb, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipMemcpyAsync(u.data(), in->ub, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  // center = 0.5*(u+l); v = 0.5*(u-l); n = numel(find(l-u)); one generator per pixel (i1 outer, i2 inner) whose
  // first-channel half-width is non-zero
  std::vector<double> center((size_t)N), val;
  std::vector<int32_t> pix;
  int64_t n = 0;
  for (int64_t i = 0; i < N; ++i) {
    center[i] = 0.5 * (u[i] + l[i]);
    if (l[i] - u[i] != 0.0) ++n;
  }
  for (int64_t i1 = 0; i1 < H; ++i1)
    for (int64_t i2 = 0; i2 < W; ++i2) {
      const double bv = 0.5 * (u[i1 + i2 * H] - l[i1 + i2 * H]);
      if (bv != 0.0) {
        pix.push_back((int32_t)(i1 + i2 * H));
        val.push_back(bv);
      }
    }
  if ((int64_t)pix.size() > n) NNV_FAIL(NNVHIP_ERR_SHAPE, "Index exceeds the number of array elements");  // (cannot happen: C >= 1)
  nnvhip_star* s = new_star(c);
  std::unique_ptr<nnvhip_star, int (*)(nnvhip_star*)> guard(s, nnvhip_star_release);
  s->N = N;
  s->n = n;
  s->ld = round_up(N, kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * s->ld * (n + 1), &s->Vbuf));
  s->V = s->Vbuf->as<double>();
  BufRef dcen, dpix, dval;
  NNV_TRY(c->upload(center.data(), sizeof(double) * N, &dcen));
  const int ngen = (int)pix.size();
  if (pix.empty()) {  // (something to upload)
    pix.push_back(0);
    val.push_back(0.0);
  }
  NNV_TRY(c->upload(pix.data(), sizeof(int32_t) * pix.size(), &dpix));
  NNV_TRY(c->upload(val.data(), sizeof(double) * val.size(), &dval));
  dim3 grid((unsigned)std::min<int64_t>(ceil_div(s->ld, 256), 64), (unsigned)std::min<int64_t>(n + 1, 4096));
  hipLaunchKernelGGL(rebox_fill_kernel, grid, dim3(256), 0, c->stream, s->V, s->ld, (int)N, (int)HW, n + 1, ngen,
                     dcen->as<double>(), dpix->as<int32_t>(), dval->as<double>());
  NNV_HIP_TRY(hipGetLastError());
  // predicate bounds -1 / +1; C = zeros(1, n), d = 0
  const int64_t npad = round_up(std::max<int64_t>(n, 1), kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * 2 * npad, &s->pbuf));
  s->plb = s->pbuf->as<double>();
  s->pub = s->plb + npad;
  {
    const int64_t pinfo[2] = {0, npad};
    BufRef dinfo;
    NNV_TRY(c->upload(pinfo, sizeof(pinfo), &dinfo));
    hipLaunchKernelGGL(fill_pm_one_kernel, dim3((unsigned)ceil_div(npad, 256), 1), dim3(256), 0, c->stream, s->plb, dinfo->as<int64_t>());
    NNV_HIP_TRY(hipGetLastError());
  }
  auto base = make_ref<ConsNode>();
  base->p_total = 1;
  base->n_total = n;
  s->cons = base;
  if (C == 1 && ngen == n && n > 0) {  // a plain box star: every generator is val * e_pix
    std::vector<double> scale((size_t)N, 0.0);
    bool neg = false;
    for (size_t g = 0; g < (size_t)ngen; ++g) {
      scale[pix[g]] = val[g];
      neg = neg || val[g] < 0.0;
    }
    BufRef dscale;
    NNV_TRY(c->upload(scale.data(), sizeof(double) * N, &dscale));
    s->oh_from = 1;
    s->oh_idx_buf = dpix;
    s->oh_idx = dpix->as<int32_t>();
    s->oh_scale_buf = dscale;
    s->oh_scale = dscale->as<double>();
    s->oh_scale_neg = neg;
  }
  if (im_lb) memcpy(im_lb, l.data(), sizeof(double) * N);
  if (im_ub) memcpy(im_ub, u.data(), sizeof(double) * N);
  *out = guard.release();
  return NNVHIP_OK;
}

int nnvhip_star_retain(nnvhip_star* s) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  s->refs.fetch_add(1);
  return NNVHIP_OK;
}

int nnvhip_star_release(nnvhip_star* s) {
  if (!s) return NNVHIP_OK;
  if (s->refs.fetch_sub(1) == 1) {
    delete_star(s);
  }
  return NNVHIP_OK;
}

int nnvhip_star_release_array(int64_t count, nnvhip_star* const* sets) {
  if (count < 0 || (count > 0 && !sets)) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  // a large array is let go later, where the host waits for the device anyway (nnvhip_ctx::deferred)
  const bool later = count >= 256;
  for (int64_t i = 0; i < count; ++i) {
    if (later && sets[i] != nullptr)
      sets[i]->ctx->deferred.push_back(sets[i]);
    else
      nnvhip_star_release(sets[i]);
  }
  return NNVHIP_OK;
}

int nnvhip_star_dims(const nnvhip_star* s, int64_t* N, int64_t* n, int64_t* p) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  if (N) *N = s->N;
  if (n) *n = s->n;
  if (p) *p = s->cons ? s->cons->p_total : 0;
  return NNVHIP_OK;
}

int nnvhip_star_has_zono(const nnvhip_star* s, int32_t* flag) {
  if (!s || !flag) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  *flag = s->has_zono ? 1 : 0;
  return NNVHIP_OK;
}

int nnvhip_star_has_user_constraints(const nnvhip_star* s, int32_t* flag) {
  if (!s || !flag) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  const ConsNode* nd = s->cons.get();
  while (nd && nd->prev) nd = nd->prev.get();
  *flag = (nd && nd->C0) ? 1 : 0;  // the base node holds dense rows only when a caller handed some in
  return NNVHIP_OK;
}

int nnvhip_star_fetch_V(const nnvhip_star* s, double* V) {
  if (!s || !V) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  nnvhip_ctx* c = s->ctx;
  NNV_TRY(nnvhip::enter_ctx(c));
  NNV_TRY(ensure_dense(c, const_cast<nnvhip_star*>(s)));  // implicit columns are written out on first read
  NNV_HIP_TRY(hipMemcpy2DAsync(V, sizeof(double) * s->N, s->V, sizeof(double) * s->ld, sizeof(double) * s->N,
                               s->n + 1, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_star_fetch_rows(const nnvhip_star* s, int64_t R, const int32_t* rows, double* out) {
  if (!s || (R > 0 && (!rows || !out)) || R < 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (R == 0) return NNVHIP_OK;
  nnvhip_ctx* c = s->ctx;
  for (int64_t t = 0; t < R; ++t)
    if (rows[t] < 0 || rows[t] >= s->N) NNV_FAIL(NNVHIP_ERR_ARG, "Invalid index");
  NNV_TRY(nnvhip::enter_ctx(c));
  NNV_TRY(ensure_dense(c, const_cast<nnvhip_star*>(s)));
  // gather on the device into an Rp x (n+1) matrix (Rp = R rounded up to whole K-tiles, the packing
  // kernel's granularity), one contiguous copy, then drop the padding rows on the host
  const int64_t Rp = round_up(R, kLdAlign), nc = s->n + 1;
  std::vector<int32_t> list((size_t)Rp, -1);
  std::copy(rows, rows + R, list.begin());
  BufRef dlist, packed;
  NNV_TRY(c->upload(list.data(), sizeof(int32_t) * Rp, &dlist));
  NNV_TRY(c->alloc(sizeof(double) * Rp * nc, &packed));
  PackSet ps{s->V, dlist->as<int32_t>(), packed->as<double>(), s->ld, (int32_t)Rp, (int32_t)nc};
  NNV_TRY(launch_pack_rows(c, 1, &ps));
  std::vector<double> tmp((size_t)(Rp * nc));
  NNV_HIP_TRY(hipMemcpyAsync(tmp.data(), packed->ptr, sizeof(double) * Rp * nc, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  for (int64_t j = 0; j < nc; ++j) memcpy(out + j * R, tmp.data() + j * Rp, sizeof(double) * R);
  return NNVHIP_OK;
}

int nnvhip_star_fetch_pred_bounds(const nnvhip_star* s, double* lb, double* ub) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  nnvhip_ctx* c = s->ctx;
  NNV_TRY(nnvhip::enter_ctx(c));
  if (s->n > 0) {
    if (lb) NNV_HIP_TRY(hipMemcpyAsync(lb, s->plb, sizeof(double) * s->n, hipMemcpyDeviceToHost, c->stream));
    if (ub) NNV_HIP_TRY(hipMemcpyAsync(ub, s->pub, sizeof(double) * s->n, hipMemcpyDeviceToHost, c->stream));
  }
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_star_fetch_constraints(const nnvhip_star* s, double* C, double* d) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  NNV_TRY(nnvhip::enter_ctx(s->ctx));
  return materialize_constraints(s, C, d);
}

int nnvhip_star_relu_counts(const nnvhip_star* s, int64_t* n_inactive, int64_t* n_crossing) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  if (s->n_crossing < 0) NNV_FAIL(NNVHIP_ERR_ARG, "set was not produced by the ReLU step");
  if (n_inactive) *n_inactive = s->n_inactive;
  if (n_crossing) *n_crossing = s->n_crossing;
  return NNVHIP_OK;
}

int nnvhip_star_fetch_crossing(const nnvhip_star* s, int32_t* index, double* lb, double* ub) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  if (s->n_crossing < 0) NNV_FAIL(NNVHIP_ERR_ARG, "set was not produced by the ReLU step");
  nnvhip_ctx* c = s->ctx;
  NNV_TRY(nnvhip::enter_ctx(c));
  const ConsNode* node = s->cons.get();
  int64_t m = s->n_crossing;
  if (m > 0) {
    if (index) NNV_HIP_TRY(hipMemcpyAsync(index, node->index->as<int32_t>() + node->index_off, sizeof(int32_t) * m, hipMemcpyDeviceToHost, c->stream));
    const double* lbub = node->lbub->as<double>() + node->lbub_off;
    if (lb) NNV_HIP_TRY(hipMemcpyAsync(lb, lbub, sizeof(double) * m, hipMemcpyDeviceToHost, c->stream));
    if (ub) NNV_HIP_TRY(hipMemcpyAsync(ub, lbub + node->ld_lbub, sizeof(double) * m, hipMemcpyDeviceToHost, c->stream));
  }
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_estimate_ranges(nnvhip_ctx* c, nnvhip_star* s, double* lb, double* ub) {
  return nnvhip_estimate_ranges_batch(c, 1, &s, lb, ub);
}

int nnvhip_estimate_ranges_static(nnvhip_ctx* c, const nnvhip_star* s, double* lb_dev, double* ub_dev) {
  CHECK_CTX(c);
  if (!s || s->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle");
  if (!lb_dev && !ub_dev) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  return ranges_into_static(c, s, lb_dev, ub_dev);
}

int nnvhip_estimate_ranges_batch(nnvhip_ctx* c, int64_t count, nnvhip_star* const* s, double* lb, double* ub) {
  CHECK_CTX(c);
  if (!s || count <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  for (int64_t i = 0; i < count; ++i) {
    if (!s[i] || s[i]->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle %lld", (long long)i);
    if (s[i]->N != s[0]->N) NNV_FAIL(NNVHIP_ERR_SHAPE, "sets of one array must have the same dimension");
  }
  NNV_TRY(c->begin_op());
  NNV_TRY(compute_ranges(c, count, s));
  NNV_TRY(c->end_op());
  if (lb || ub) {
    int64_t N = s[0]->N;
    // ranges computed by one call sit at a fixed stride in one buffer
    const int64_t stride = count > 1 ? s[1]->lb - s[0]->lb : 0;
    bool regular = count > 1 && stride >= N;
    for (int64_t i = 1; i < count && regular; ++i)
      regular = s[i]->rbuf == s[0]->rbuf && s[i]->lb == s[0]->lb + i * stride && s[i]->ub == s[0]->ub + i * stride;
    if (regular && stride <= 4 * N + 64) {
      // one contiguous copy of the whole range buffer, unpacked on the host (strided 2-D copies of
      // short rows are issued row by row by the runtime)
      const int64_t off_ub = s[0]->ub - s[0]->lb;
      std::vector<double> tmp((size_t)(stride * (count - 1) + std::max<int64_t>(N, off_ub + N)));
      NNV_HIP_TRY(hipMemcpyAsync(tmp.data(), s[0]->lb, sizeof(double) * tmp.size(), hipMemcpyDeviceToHost, c->stream));
      NNV_HIP_TRY(hipStreamSynchronize(c->stream));
      for (int64_t i = 0; i < count; ++i) {
        if (lb) std::copy(tmp.begin() + i * stride, tmp.begin() + i * stride + N, lb + i * N);
        if (ub) std::copy(tmp.begin() + i * stride + off_ub, tmp.begin() + i * stride + off_ub + N, ub + i * N);
      }
      return NNVHIP_OK;
    } else {
      for (int64_t i = 0; i < count; ++i) {
        if (lb) NNV_HIP_TRY(hipMemcpyAsync(lb + i * N, s[i]->lb, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
        if (ub) NNV_HIP_TRY(hipMemcpyAsync(ub + i * N, s[i]->ub, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
      }
    }
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  return NNVHIP_OK;
}

}  // extern "C"
