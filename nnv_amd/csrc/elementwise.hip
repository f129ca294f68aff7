// Affine layers that act row by row or through small fixed windows; all are single passes over
// the generator matrix (HBM bound):
//   * per-row affine programs: BatchNormalizationLayer (nn/layers/BatchNormalizationLayer.m:247-351),
//     ImageInputLayer normalisation (nn/layers/ImageInputLayer.m:121-166), ImageStar.affineMap
//     (set/ImageStar.m:431-460) -- the steps are applied in the reference's order so results
//     round the same way;
//   * AveragePooling2DLayer (nn/layers/AveragePooling2DLayer.m:229-247, 424-436; the arithmetic is
//     MatConvNet's vl_nnpool 'avg': mean over the part of the window inside the image);
//   * row permutations: the C-style FlattenLayer variants (nn/layers/FlattenLayer.m:118-170).
// Geometry of every kernel: a lane owns two adjacent rows, the eight waves of a block interleave
// columns; grid = (row blocks, column chunks, sets).
#include <algorithm>
#include <memory>
#include <vector>

#include "internal.h"

struct nnvhip_rowmap {
  nnvhip_ctx* ctx = nullptr;
  int64_t N = 0, ld = 0;
  int32_t n_steps = 0;
  int32_t op[8] = {0}, scope[8] = {0};
  nnvhip::BufRef params;  // ld x n_steps, zero padded rows
};

struct nnvhip_avgpool2d {
  nnvhip_ctx* ctx = nullptr;
  int64_t pool[2] = {1, 1}, stride[2] = {1, 1}, pad[4] = {0, 0, 0, 0};
};

namespace nnvhip {

constexpr int kEwWaves = 8;
constexpr int kEwRows = 128;  // rows per wave: 64 lanes x 2
constexpr int kMaxSteps = 8;

struct SetDesc {
  const double* in;
  double* out;
  int32_t ncols;
  int32_t pad_;
};

struct RowmapArgs {
  const double* params;
  int64_t ld;      // leading dimension of in, out and params
  int32_t n_steps;
  int32_t cols_per_chunk;
  int32_t op[kMaxSteps];
  int32_t scope[kMaxSteps];
};

__device__ __forceinline__ double apply_op(int op, double v, double p) {
  switch (op) {
    case NNVHIP_OP_ADD: return __dadd_rn(v, p);
    case NNVHIP_OP_SUB: return __dsub_rn(v, p);
    case NNVHIP_OP_MUL: return __dmul_rn(v, p);
    default: return __ddiv_rn(v, p);
  }
}

__global__ __launch_bounds__(64 * kEwWaves) void rowmap_kernel(const SetDesc* __restrict__ table, SetDesc one,
                                                               RowmapArgs a) {
  const SetDesc d = table ? table[blockIdx.z] : one;
  const int j0 = blockIdx.y * a.cols_per_chunk;
  if (j0 >= d.ncols) return;
  const int j1 = min(d.ncols, j0 + a.cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r0 = (int64_t)blockIdx.x * kEwRows + 2 * lane;
  if (r0 >= a.ld) return;
  double2 p[kMaxSteps];
#pragma unroll
  for (int s = 0; s < kMaxSteps; ++s)
    if (s < a.n_steps) p[s] = *reinterpret_cast<const double2*>(a.params + (int64_t)s * a.ld + r0);
  for (int jb = j0 + 4 * wave; jb < j1; jb += 4 * kEwWaves) {
    double2 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (jb + u < j1) v[u] = *reinterpret_cast<const double2*>(d.in + r0 + (int64_t)(jb + u) * a.ld);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = jb + u;
      if (j >= j1) break;
      double2 x = v[u];
#pragma unroll
      for (int s = 0; s < kMaxSteps; ++s) {
        if (s >= a.n_steps) break;
        if (a.scope[s] == NNVHIP_SCOPE_ALL || j == 0) {
          x.x = apply_op(a.op[s], x.x, p[s].x);
          x.y = apply_op(a.op[s], x.y, p[s].y);
        }
      }
      *reinterpret_cast<double2*>(d.out + r0 + (int64_t)j * a.ld) = x;
    }
  }
}

struct PoolArgs {
  int64_t ldin, ldout;
  int32_t H, W, C, Ho, Wo;
  int32_t ph, pw, sh, sw, pt, pl;
  int32_t cols_per_chunk;
};

// One thread per output row (ho fastest, then wo, then channel); the waves of a block interleave
// columns.  Sum order: window columns outer, window rows inner, then one multiplication by
// 1 / (number of window cells inside the image).
__global__ __launch_bounds__(64 * kEwWaves) void avgpool_kernel(const SetDesc* __restrict__ table, SetDesc one,
                                                                PoolArgs a) {
  const SetDesc d = table ? table[blockIdx.z] : one;
  const int j0 = blockIdx.y * a.cols_per_chunk;
  if (j0 >= d.ncols) return;
  const int j1 = min(d.ncols, j0 + a.cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r = (int64_t)blockIdx.x * 64 + lane;
  if (r >= a.ldout) return;
  const int64_t Nout = (int64_t)a.Ho * a.Wo * a.C;
  const bool real = r < Nout;
  int y1 = 0, y2 = 0, x1 = 0, x2 = 0;
  int64_t base = 0;
  double scale = 0.0;
  if (real) {
    const int ho = (int)(r % a.Ho);
    const int wo = (int)((r / a.Ho) % a.Wo);
    const int c = (int)(r / ((int64_t)a.Ho * a.Wo));
    y1 = ho * a.sh - a.pt;
    x1 = wo * a.sw - a.pl;
    y2 = min(y1 + a.ph, a.H);
    x2 = min(x1 + a.pw, a.W);
    y1 = max(y1, 0);
    x1 = max(x1, 0);
    base = (int64_t)c * a.H * a.W;
    scale = 1.0 / (double)((y2 - y1) * (x2 - x1));
  }
  // each wave takes 4 consecutive columns per step: four independent sums keep more loads in flight
  for (int jb = j0 + 4 * wave; jb < j1; jb += 4 * kEwWaves) {
    const int nu = min(4, j1 - jb);
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    if (real) {
      const double* col = d.in + (int64_t)jb * a.ldin + base;
      if (nu == 4) {
        for (int x = x1; x < x2; ++x)
          for (int y = y1; y < y2; ++y) {
            const double* p = col + y + (int64_t)x * a.H;
            const double v0 = p[0], v1 = p[a.ldin], v2 = p[2 * a.ldin], v3 = p[3 * a.ldin];
            acc[0] = __dadd_rn(acc[0], v0);
            acc[1] = __dadd_rn(acc[1], v1);
            acc[2] = __dadd_rn(acc[2], v2);
            acc[3] = __dadd_rn(acc[3], v3);
          }
      } else {
        for (int u = 0; u < nu; ++u)
          for (int x = x1; x < x2; ++x)
            for (int y = y1; y < y2; ++y) acc[u] = __dadd_rn(acc[u], col[y + (int64_t)x * a.H + (int64_t)u * a.ldin]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] = __dmul_rn(acc[u], scale);
    }
    for (int u = 0; u < nu; ++u) d.out[r + (int64_t)(jb + u) * a.ldout] = acc[u];  // padding rows stay zero
  }
}

struct PermArgs {
  const int32_t* src_row;  // ldout entries; -1 = padding row (written as zero)
  int64_t ldin, ldout;
  int32_t cols_per_chunk;
};

__global__ __launch_bounds__(64 * kEwWaves) void permute_rows_kernel(const SetDesc* __restrict__ table, SetDesc one,
                                                                     PermArgs a) {
  const SetDesc d = table ? table[blockIdx.z] : one;
  const int j0 = blockIdx.y * a.cols_per_chunk;
  if (j0 >= d.ncols) return;
  const int j1 = min(d.ncols, j0 + a.cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r0 = (int64_t)blockIdx.x * kEwRows + 2 * lane;
  if (r0 >= a.ldout) return;
  const int2 src = *reinterpret_cast<const int2*>(a.src_row + r0);
  for (int jb = j0 + 4 * wave; jb < j1; jb += 4 * kEwWaves) {
    double2 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      v[u] = make_double2(0.0, 0.0);
      if (jb + u < j1) {
        const double* col = d.in + (int64_t)(jb + u) * a.ldin;
        if (src.x >= 0) v[u].x = col[src.x];
        if (src.y >= 0) v[u].y = col[src.y];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (jb + u < j1) *reinterpret_cast<double2*>(d.out + r0 + (int64_t)(jb + u) * a.ldout) = v[u];
  }
}

// Short columns (N <= kPermLdsRows): a block stages whole columns in LDS with coalesced loads and
// gathers from there, so global memory sees only contiguous traffic.  Grid: (1, column chunks, sets).
constexpr int kPermLdsRows = 4096;
constexpr int kPermCols = 2;  // columns staged per step

__global__ __launch_bounds__(64 * kEwWaves) void permute_rows_lds_kernel(const SetDesc* __restrict__ table, SetDesc one,
                                                                         PermArgs a, int n_rows) {
  const SetDesc d = table ? table[blockIdx.z] : one;
  const int j0 = blockIdx.y * a.cols_per_chunk;
  if (j0 >= d.ncols) return;
  const int j1 = min(d.ncols, j0 + a.cols_per_chunk);
  __shared__ double stage[kPermCols][kPermLdsRows];
  const int tid = threadIdx.x;
  for (int jb = j0; jb < j1; jb += kPermCols) {
#pragma unroll
    for (int u = 0; u < kPermCols; ++u)
      if (jb + u < j1)
        for (int r = tid; r < n_rows; r += 64 * kEwWaves) stage[u][r] = d.in[r + (int64_t)(jb + u) * a.ldin];
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kPermCols; ++u)
      if (jb + u < j1)
        for (int64_t r = tid; r < a.ldout; r += 64 * kEwWaves) {
          const int src = a.src_row[r];
          d.out[r + (int64_t)(jb + u) * a.ldout] = src >= 0 ? stage[u][src] : 0.0;
        }
    __syncthreads();
  }
}

// Common launch plumbing: output handles, descriptor table, grid with a few thousand blocks.
template <class Launch>
static int run_row_layer(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, nnvhip_star** out, int64_t Nout,
                         int64_t rows_per_block, int min_cols_per_chunk, Launch launch) {
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  for (int64_t i = 0; i < count; ++i) {
    if (in[i]->N != in[0]->N || in[i]->ld != in[0]->ld)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "sets of one array must have the same dimension");
  }
  NNV_TRY(ensure_dense_batch(c, count, in));  // these passes read every column
  std::vector<nnvhip_star*> outs;
  bool contig = false;
  int64_t cols = 0;
  NNV_TRY(c->begin_op());
  int st = make_affine_outputs(c, count, in, Nout, &outs, &contig, &cols);
  if (st == NNVHIP_OK) {
    std::vector<SetDesc> descs((size_t)count);
    int64_t max_cols = 0;
    for (int64_t i = 0; i < count; ++i) {
      descs[i].in = in[i]->V;
      descs[i].out = outs[i]->V;
      descs[i].ncols = (int32_t)(in[i]->n + 1);
      descs[i].pad_ = 0;
      max_cols = std::max<int64_t>(max_cols, in[i]->n + 1);
    }
    const SetDesc* table = nullptr;
    BufRef tab;
    if (count > 1) {
      st = c->upload_table(descs.data(), sizeof(SetDesc) * descs.size(), &tab);
      if (st == NNVHIP_OK) table = tab->as<SetDesc>();
    }
    if (st == NNVHIP_OK) {
      const int64_t ldout = outs[0]->ld;
      const int64_t row_blocks = ceil_div(ldout, rows_per_block);
      int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(8192, row_blocks * count),
                                                               ceil_div(max_cols, min_cols_per_chunk)));
      const int64_t cpc = ceil_div(max_cols, chunks);
      chunks = ceil_div(max_cols, cpc);
      double bytes = 0.0;  // algorithmic: every input element read once, every output element written once
      for (int64_t i = 0; i < count; ++i) bytes += 8.0 * (double)(in[i]->N + Nout) * (double)(in[i]->n + 1);
      st = c->kernel_timer_begin(c->kernel_timing);
      launch(dim3((unsigned)row_blocks, (unsigned)chunks, (unsigned)count), table, descs[0], (int32_t)cpc, outs[0]->ld);
      if (st == NNVHIP_OK) st = c->kernel_timer_end(c->kernel_timing, 4, bytes);
      if (hipGetLastError() != hipSuccess) {
        set_error("kernel launch failed");
        st = NNVHIP_ERR_HIP;
      }
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

}  // namespace nnvhip

using namespace nnvhip;

extern "C" {

int nnvhip_rowmap_create(nnvhip_ctx* c, int64_t N, int32_t n_steps, const int32_t* op, const int32_t* scope,
                         const double* params, nnvhip_rowmap** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  NNV_TRY(nnvhip::enter_ctx(c));
  if (!op || !scope || !params || !out) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (N <= 0 || n_steps <= 0 || n_steps > kMaxSteps) NNV_FAIL(NNVHIP_ERR_SHAPE, "a row map has 1 to 8 steps");
  std::unique_ptr<nnvhip_rowmap> m(new nnvhip_rowmap());
  m->ctx = c;
  m->N = N;
  m->ld = round_up(N, kLdAlign);
  m->n_steps = n_steps;
  for (int s = 0; s < n_steps; ++s) {
    if (op[s] < NNVHIP_OP_ADD || op[s] > NNVHIP_OP_DIV || (scope[s] != NNVHIP_SCOPE_CENTRE && scope[s] != NNVHIP_SCOPE_ALL))
      NNV_FAIL(NNVHIP_ERR_ARG, "invalid step %d", s);
    m->op[s] = op[s];
    m->scope[s] = scope[s];
  }
  // padding rows get the neutral operand of their step so that they stay exactly zero
  std::vector<double> host((size_t)(m->ld * n_steps));
  for (int s = 0; s < n_steps; ++s) {
    const double neutral = (op[s] == NNVHIP_OP_MUL || op[s] == NNVHIP_OP_DIV) ? 1.0 : 0.0;
    for (int64_t r = 0; r < m->ld; ++r) host[(size_t)(s * m->ld + r)] = r < N ? params[s * N + r] : neutral;
  }
  NNV_TRY(c->alloc(sizeof(double) * host.size(), &m->params));
  NNV_HIP_TRY(hipMemcpyAsync(m->params->ptr, host.data(), sizeof(double) * host.size(), hipMemcpyHostToDevice, c->stream));
  c->h2d_bytes += (int64_t)(sizeof(double) * host.size());
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  *out = m.release();
  return NNVHIP_OK;
}

int nnvhip_rowmap_destroy(nnvhip_rowmap* m) {
  delete m;
  return NNVHIP_OK;
}

int nnvhip_affine_rowmap(nnvhip_ctx* c, const nnvhip_rowmap* m, int64_t count, nnvhip_star* const* in,
                         nnvhip_star** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  NNV_TRY(nnvhip::enter_ctx(c));
  if (!m || m->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid layer handle");
  NNV_TRY(check_set_array(c, count, in, out));
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N != m->N)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent number of channels between scale array and the ImageStar");
  RowmapArgs a{};
  a.params = m->params->as<double>();
  a.ld = m->ld;
  a.n_steps = m->n_steps;
  for (int s = 0; s < kMaxSteps; ++s) {
    a.op[s] = m->op[s];
    a.scope[s] = m->scope[s];
  }
  return run_row_layer(c, count, in, out, m->N, kEwRows, 4 * kEwWaves,
                       [&](dim3 grid, const SetDesc* table, const SetDesc& one, int32_t cpc, int64_t) {
                         a.cols_per_chunk = cpc;
                         NNV_LAUNCH(c, c->kernel_timing, rowmap_kernel, grid, dim3(64 * kEwWaves), 0, table, one, a);
                       });
}

int nnvhip_avgpool2d_create(nnvhip_ctx* c, const int64_t pool[2], const int64_t stride[2], const int64_t padding[4],
                            nnvhip_avgpool2d** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (!pool || !stride || !padding || !out) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (pool[0] < 1 || pool[1] < 1) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid pool size");
  if (stride[0] < 1 || stride[1] < 1) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid stride");
  for (int i = 0; i < 4; ++i)
    if (padding[i] < 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalide padding size");
  // a window that lies entirely in the padding would have no cell to average
  if (padding[0] >= pool[0] || padding[1] >= pool[0] || padding[2] >= pool[1] || padding[3] >= pool[1])
    NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalide padding size");
  nnvhip_avgpool2d* p = new nnvhip_avgpool2d();
  p->ctx = c;
  for (int i = 0; i < 2; ++i) {
    p->pool[i] = pool[i];
    p->stride[i] = stride[i];
  }
  for (int i = 0; i < 4; ++i) p->pad[i] = padding[i];
  *out = p;
  return NNVHIP_OK;
}

int nnvhip_avgpool2d_destroy(nnvhip_avgpool2d* p) {
  delete p;
  return NNVHIP_OK;
}

int nnvhip_avgpool2d_output_size(const nnvhip_avgpool2d* p, int64_t H, int64_t W, int64_t* Ho, int64_t* Wo) {
  if (!p || !Ho || !Wo) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  // (InputSize + padding - FilterSize)/Stride + 1, rounded down (AveragePooling2DLayer.m:396-418)
  const int64_t h = H + p->pad[0] + p->pad[1] - p->pool[0];
  const int64_t w = W + p->pad[2] + p->pad[3] - p->pool[1];
  if (h < 0 || w < 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid pool size");
  *Ho = h / p->stride[0] + 1;
  *Wo = w / p->stride[1] + 1;
  return NNVHIP_OK;
}

int nnvhip_affine_avgpool2d(nnvhip_ctx* c, const nnvhip_avgpool2d* p, int64_t H, int64_t W, int64_t count,
                            nnvhip_star* const* in, nnvhip_star** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  NNV_TRY(nnvhip::enter_ctx(c));
  if (!p || p->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid layer handle");
  NNV_TRY(check_set_array(c, count, in, out));
  if (H <= 0 || W <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "The input is not an ImageStar object");
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N % (H * W) != 0)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension in the ImageStar and the original Star set");
  const int64_t C = in[0]->N / (H * W);
  int64_t Ho = 0, Wo = 0;
  NNV_TRY(nnvhip_avgpool2d_output_size(p, H, W, &Ho, &Wo));
  if (in[0]->N >= (int64_t(1) << 31) || Ho * Wo * C >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "image too large");
  PoolArgs a{};
  a.ldin = in[0]->ld;
  a.H = (int32_t)H;
  a.W = (int32_t)W;
  a.C = (int32_t)C;
  a.Ho = (int32_t)Ho;
  a.Wo = (int32_t)Wo;
  a.ph = (int32_t)p->pool[0];
  a.pw = (int32_t)p->pool[1];
  a.sh = (int32_t)p->stride[0];
  a.sw = (int32_t)p->stride[1];
  a.pt = (int32_t)p->pad[0];
  a.pl = (int32_t)p->pad[2];
  return run_row_layer(c, count, in, out, Ho * Wo * C, 64, 4 * kEwWaves,
                       [&](dim3 grid, const SetDesc* table, const SetDesc& one, int32_t cpc, int64_t ldout) {
                         a.cols_per_chunk = cpc;
                         a.ldout = ldout;
                         NNV_LAUNCH(c, c->kernel_timing, avgpool_kernel, grid, dim3(64 * kEwWaves), 0, table, one, a);
                       });
}

int nnvhip_permute_rows(nnvhip_ctx* c, int64_t N, const int32_t* src_row, int64_t count, nnvhip_star* const* in,
                        nnvhip_star** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  NNV_TRY(nnvhip::enter_ctx(c));
  if (!src_row) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  NNV_TRY(check_set_array(c, count, in, out));
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N != N) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension in the ImageStar and the original Star set");
  if (N >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "image too large");
  const int64_t ld = round_up(N, kLdAlign);
  std::vector<int32_t> host((size_t)ld, -1);
  std::vector<char> seen((size_t)N, 0);
  for (int64_t r = 0; r < N; ++r) {
    if (src_row[r] < 0 || src_row[r] >= N || seen[(size_t)src_row[r]]) NNV_FAIL(NNVHIP_ERR_ARG, "not a permutation");
    seen[(size_t)src_row[r]] = 1;
    host[(size_t)r] = src_row[r];
  }
  BufRef perm;
  NNV_TRY(c->upload(host.data(), sizeof(int32_t) * host.size(), &perm));
  PermArgs a{};
  a.src_row = perm->as<int32_t>();
  a.ldin = in[0]->ld;
  if (ld <= kPermLdsRows)
    return run_row_layer(c, count, in, out, N, int64_t(1) << 30, 4 * kPermCols,
                         [&](dim3 grid, const SetDesc* table, const SetDesc& one, int32_t cpc, int64_t ldout) {
                           a.cols_per_chunk = cpc;
                           a.ldout = ldout;
                           NNV_LAUNCH(c, c->kernel_timing, permute_rows_lds_kernel, grid, dim3(64 * kEwWaves), 0, table, one,
                                              a, (int)N);
                         });
  return run_row_layer(c, count, in, out, N, kEwRows, 4 * kEwWaves,
                       [&](dim3 grid, const SetDesc* table, const SetDesc& one, int32_t cpc, int64_t ldout) {
                         a.cols_per_chunk = cpc;
                         a.ldout = ldout;
                         NNV_LAUNCH(c, c->kernel_timing, permute_rows_kernel, grid, dim3(64 * kEwWaves), 0, table, one, a);
                       });
}

}  // extern "C"
