// Star.estimateRanges (set/Star.m:1078-1106) as one coalesced pass over V.
//
// V is column-major, so consecutive lanes own consecutive rows: every wave reads 1 KiB lines down a
// column (two rows per lane).  The eight waves of a block interleave the columns of the block's
// column chunk, eight loads in flight per wave; partial sums of the chunks are combined in a fixed order by a second tiny kernel,
// so results are bit-reproducible from run to run (no floating-point atomics).
#include <algorithm>
#include <cstdlib>

#include "internal.h"

#include <mutex>

namespace nnvhip {

struct RangeDesc {
  const double* V;    // N x (n+1), column 0 = centre
  const double* plb;  // n
  const double* pub;  // n
  double* part;       // [chunks][4][ld] partial sums (unused when chunks == 1 and chunks2 == 0)
  const double* part2;  // further chunks2 chunks left by the producer of the trailing columns, or null
  const double* part3;  // sums of gathered columns from the matrix product: [xmin1; xmax2], [xmax1; xmin2] (2*ld each), or null
  int32_t chunks2;
  int32_t chunks2_at;   // the first chunks2_at of those chunks are read at *part2_at instead (another set's, which are the same)
  const double* const* part2_at;
  int32_t cchunks;      // > 0: the centre is the sum of cchunks vectors at cpart (ld apart) plus cbias (or
  const double* cpart;  // null), written to cout before it enters lb / ub
  const double* cbias;
  double* cout;
  double* lb;         // ld
  double* ub;         // ld
  int64_t ld;
  int32_t n;
  int32_t chunks;
  int32_t cols_per_chunk;
  int32_t row_waves;  // waves of a block laid along rows (1, 2, 4 or 8); the others interleave columns
  // windows of the generator images (column j is zero, and possibly not in memory, outside box[j]: images of
  // bH x bW positions per channel), or null: a row outside a column's window is not loaded
  const ColBox* box;
  int32_t bH, bW;
  // not null: the kernel that combines the partial sums also counts, per block of its rows, the neurons a ReLU step
  // will find crossing (lb < 0 < ub), inactive (ub <= 0) and kept among the first nrows rows: three numbers per block
  int32_t* blk3;
  int32_t nrows;
};

constexpr int kRowsPerWave = 128;  // 64 lanes x 2 rows
constexpr int kRangeWaves = 8;     // waves per block

template <int U, int OCC>
__global__ __launch_bounds__(64 * kRangeWaves, OCC) void ranges_partial_kernel(const RangeDesc* __restrict__ table,
                                                                               RangeDesc one) {
  const RangeDesc d = table ? table[blockIdx.z] : one;
  const int chunk = blockIdx.y;
  if (chunk >= d.chunks) return;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wrow = wave % d.row_waves;
  const int wcol = wave / d.row_waves;
  const int col_waves = kRangeWaves / d.row_waves;
  const int64_t r0 = ((int64_t)blockIdx.x * d.row_waves + wrow) * kRowsPerWave + 2 * lane;
  const bool active = r0 < d.ld;
  // generator columns are 1..n; chunk c owns [1 + c*cpc, min(n, (c+1)*cpc) + 1)
  const int j0 = 1 + chunk * d.cols_per_chunk;
  const int j1 = min(d.n, (chunk + 1) * d.cols_per_chunk) + 1;
  double2 xmin1 = {0, 0}, xmin2 = {0, 0}, xmax1 = {0, 0}, xmax2 = {0, 0};
  if (active) {
    const double* col = d.V + r0;
    // each wave takes U consecutive columns per step; the U loads are issued before any is used
#pragma unroll 1
    for (int jb = j0 + U * wcol; jb < j1; jb += U * col_waves) {
      double2 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        v[u] = make_double2(0.0, 0.0);
        if (jb + u < j1) v[u] = *reinterpret_cast<const double2*>(col + (int64_t)(jb + u) * d.ld);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int j = jb + u;
        if (j >= j1) break;
        const double pl = d.plb[j - 1];
        const double pu = d.pub[j - 1];
        const double px = fmax(v[u].x, 0.0), nx = fmin(v[u].x, 0.0);
        const double py = fmax(v[u].y, 0.0), ny = fmin(v[u].y, 0.0);
        xmin1.x = fma(px, pl, xmin1.x);
        xmin1.y = fma(py, pl, xmin1.y);
        xmax1.x = fma(px, pu, xmax1.x);
        xmax1.y = fma(py, pu, xmax1.y);
        xmin2.x = fma(nx, pu, xmin2.x);
        xmin2.y = fma(ny, pu, xmin2.y);
        xmax2.x = fma(nx, pl, xmax2.x);
        xmax2.y = fma(ny, pl, xmax2.y);
      }
    }
  }
  // waves that share rows (same wrow) are combined in wave order by the wcol == 0 wave
  __shared__ double2 red[kRangeWaves][4][64];
  if (wcol > 0) {
    red[wave][0][lane] = xmin1;
    red[wave][1][lane] = xmin2;
    red[wave][2][lane] = xmax1;
    red[wave][3][lane] = xmax2;
  }
  __syncthreads();
  if (wcol == 0 && active) {
    for (int w = 1; w < col_waves; ++w) {
      const int src = w * d.row_waves + wrow;
      xmin1.x += red[src][0][lane].x;
      xmin1.y += red[src][0][lane].y;
      xmin2.x += red[src][1][lane].x;
      xmin2.y += red[src][1][lane].y;
      xmax1.x += red[src][2][lane].x;
      xmax1.y += red[src][2][lane].y;
      xmax2.x += red[src][3][lane].x;
      xmax2.y += red[src][3][lane].y;
    }
    if (d.chunks == 1 && d.chunks2 == 0 && d.part3 == nullptr) {
      // lb = (c + xmin1) + xmin2, the reference's left-to-right order
      const double2 c = *reinterpret_cast<const double2*>(d.V + r0);
      *reinterpret_cast<double2*>(d.lb + r0) = make_double2((c.x + xmin1.x) + xmin2.x, (c.y + xmin1.y) + xmin2.y);
      *reinterpret_cast<double2*>(d.ub + r0) = make_double2((c.x + xmax1.x) + xmax2.x, (c.y + xmax1.y) + xmax2.y);
    } else {
      double* p = d.part + ((int64_t)chunk * 4) * d.ld + r0;
      *reinterpret_cast<double2*>(p) = xmin1;
      *reinterpret_cast<double2*>(p + d.ld) = xmin2;
      *reinterpret_cast<double2*>(p + 2 * d.ld) = xmax1;
      *reinterpret_cast<double2*>(p + 3 * d.ld) = xmax2;
    }
  }
}

// The same sums for a set whose generator images come with windows (RangeDesc::box), read inside the windows only:
// the images may not even be in memory outside them.  A lane owns PW consecutive image positions (PW = 2 where the
// image has an even number of positions: 16-byte loads) of 4 / PW channels, a block 64 * PW positions, so that one
// window test serves several loads.  Columns are dealt to the eight waves, added up and combined exactly as in
// ranges_partial_kernel with row_waves = 1 (wave w takes the columns j0 + 8w + 64k ... + 7 in order; wave 0 then
// adds the other waves' sums in wave order): skipping the exact zeros outside a window (whole columns whose
// window misses the block included) leaves every sum as it is, so both kernels give the same bits.
constexpr int kTake = 4;  // columns whose loads a wave has in flight together
template <int PW>
__global__ __launch_bounds__(512, 4) void ranges_window_kernel(const RangeDesc* __restrict__ table, RangeDesc one, int nposb, int C) {
  constexpr int CG = 4 / PW;  // channels of a block
  const RangeDesc d = table ? table[blockIdx.z] : one;
  const int chunk = blockIdx.y;
  if (chunk >= d.chunks) return;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pb = blockIdx.x % nposb, cg = blockIdx.x / nposb;
  const int P = d.bH * d.bW;
  const int p = (pb * 64 + lane) * PW;  // first of the lane's positions
  bool pvalid[PW];
  int w[PW], h[PW];
#pragma unroll
  for (int e = 0; e < PW; ++e) {
    pvalid[e] = p + e < P;
    w[e] = (p + e) / d.bH;
    h[e] = (p + e) - w[e] * d.bH;
  }
  const int c0 = cg * CG;
  const int nc = min(CG, C - c0);
  const int j0 = 1 + chunk * d.cols_per_chunk;
  const int j1 = min(d.n, (chunk + 1) * d.cols_per_chunk) + 1;
  double s[CG][4][PW];
#pragma unroll
  for (int cc = 0; cc < CG; ++cc)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int e = 0; e < PW; ++e) s[cc][a][e] = 0.0;
  // the image positions of the block: a window that misses all of them is skipped by the whole block (what it
  // would add are exact zeros)
  const int pfirst = pb * 64 * PW, plast = min(P - 1, pfirst + 64 * PW - 1);
  const int wlo = pfirst / d.bH, whi = plast / d.bH;
  const int hlo = wlo == whi ? pfirst - wlo * d.bH : 0, hhi = wlo == whi ? plast - wlo * d.bH : d.bH - 1;
  // Most windows miss the positions of a block altogether.  A wave therefore first looks at the windows of 64
  // of its columns at a time (one per lane) and queues the ones that reach the block, in ascending order; the
  // queue is worked off kTake columns at a time, so that the loads of a step are all wanted.
  __shared__ int queue[8][64 + kTake];
  int* const qw = queue[wave];
  int qn = 0;
  auto take = [&](int first, int cnt) {
    // up to kTake queued columns: window tests first, then all their loads in flight together, then the sums
    // column by column
    bool in[kTake][PW];
    double pl[kTake], pu[kTake];
    int col_j[kTake];
#pragma unroll
    for (int u = 0; u < kTake; ++u) {
#pragma unroll
      for (int e = 0; e < PW; ++e) in[u][e] = false;
      pl[u] = pu[u] = 0.0;
      col_j[u] = 0;
      if (u < cnt) {
        const int j = __builtin_amdgcn_readfirstlane(qw[first + u]);
        col_j[u] = j;
        const ColBox b = d.box[j];
#pragma unroll
        for (int e = 0; e < PW; ++e) in[u][e] = pvalid[e] && h[e] >= b.h0 && h[e] <= b.h1 && w[e] >= b.w0 && w[e] <= b.w1;
        pl[u] = d.plb[j - 1];
        pu[u] = d.pub[j - 1];
      }
    }
    double v[kTake][CG][PW];
#pragma unroll
    for (int u = 0; u < kTake; ++u) {
      // (a block-uniform address plus the lane's position: one offset register serves every load)
      const double* col = d.V + (int64_t)col_j[u] * d.ld + (int64_t)P * c0;
#pragma unroll
      for (int cc = 0; cc < CG; ++cc) {
        const double* src = col + (int64_t)P * cc;
        if constexpr (PW == 2) {
          // both positions in one load; what lies outside the window may never have been written
          double2 t = make_double2(0.0, 0.0);
          if ((in[u][0] || in[u][1]) && cc < nc) t = *reinterpret_cast<const double2*>(src + (unsigned)p);
          v[u][cc][0] = in[u][0] ? t.x : 0.0;
          v[u][cc][1] = in[u][1] ? t.y : 0.0;
        } else {
          v[u][cc][0] = (in[u][0] && cc < nc) ? src[(unsigned)p] : 0.0;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kTake; ++u) {
      if (u >= cnt) break;  // (uniform)
#pragma unroll
      for (int cc = 0; cc < CG; ++cc)
#pragma unroll
        for (int e = 0; e < PW; ++e) {
          const double px = fmax(v[u][cc][e], 0.0), nx = fmin(v[u][cc][e], 0.0);
          s[cc][0][e] = fma(px, pl[u], s[cc][0][e]);  // xmin1
          s[cc][1][e] = fma(nx, pu[u], s[cc][1][e]);  // xmin2
          s[cc][2][e] = fma(px, pu[u], s[cc][2][e]);  // xmax1
          s[cc][3][e] = fma(nx, pl[u], s[cc][3][e]);  // xmax2
        }
    }
  };
  // the wave's columns in its order: entry e is column j0 + 8 * wave + 64 * (e / 8) + e % 8
#pragma unroll 1
  for (int e0 = 0; j0 + 8 * wave + 8 * e0 < j1; e0 += 64) {
    const int e = e0 + lane;
    const int j = j0 + 8 * wave + 64 * (e >> 3) + (e & 7);
    bool hit = false;
    if (j < j1) {
      const ColBox b = d.box[j];
      hit = b.w1 >= wlo && b.w0 <= whi && b.h1 >= hlo && b.h0 <= hhi;
    }
    const unsigned long long mask = __ballot(hit);
    if (hit) qw[qn + __popcll(mask & ((1ull << lane) - 1ull))] = j;
    qn += __popcll(mask);
    __builtin_amdgcn_wave_barrier();
    int qh = 0;
    for (; qn - qh >= kTake; qh += kTake) take(qh, kTake);
    if (qh > 0) {  // the (fewer than kTake) columns left over move to the front
      const int rem = qn - qh;
      int keep = 0;
      if (lane < rem) keep = qw[qh + lane];
      __builtin_amdgcn_wave_barrier();
      if (lane < rem) qw[lane] = keep;
      __builtin_amdgcn_wave_barrier();
      qn = rem;
    }
  }
  if (qn > 0) take(0, qn);
  __shared__ double red[8][4][64 * PW];
  const bool direct = d.chunks == 1 && d.chunks2 == 0 && d.part3 == nullptr;
#pragma unroll
  for (int cc = 0; cc < CG; ++cc) {
    if (cc < nc) {  // (uniform over the block)
      if (wave > 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int e = 0; e < PW; ++e) red[wave][a][lane * PW + e] = s[cc][a][e];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int e = 0; e < PW; ++e) {
          if (!pvalid[e]) continue;
          double t[4];
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            t[a] = s[cc][a][e];
            for (int w2 = 1; w2 < 8; ++w2) t[a] += red[w2][a][lane * PW + e];
          }
          const int64_t r = p + e + (int64_t)P * (c0 + cc);
          if (direct) {
            const double c = d.V[r];
            d.lb[r] = (c + t[0]) + t[1];
            d.ub[r] = (c + t[2]) + t[3];
          } else {
            double* q = d.part + ((int64_t)chunk * 4) * d.ld + r;
            q[0] = t[0];
            q[d.ld] = t[1];
            q[2 * d.ld] = t[2];
            q[3 * d.ld] = t[3];
          }
        }
      }
      __syncthreads();
    }
  }
  // the padding rows behind the image: no generator reaches them
  if (blockIdx.x == 0 && wave == 0) {
    const int64_t r = (int64_t)P * C + lane;
    if (r < d.ld) {
      if (direct) {
        d.lb[r] = d.ub[r] = d.V[r];
      } else {
        double* q = d.part + ((int64_t)chunk * 4) * d.ld + r;
        q[0] = q[d.ld] = q[2 * d.ld] = q[3 * d.ld] = 0.0;
      }
    }
  }
}

// R consecutive rows (R = 1 or 2) from 8 * R-byte aligned memory
template <int R>
__device__ __forceinline__ void load_rows(const double* __restrict__ p, double (&v)[R]) {
  if constexpr (R == 2) {
    const double2 t = *reinterpret_cast<const double2*>(p);
    v[0] = t.x;
    v[1] = t.y;
  } else {
    v[0] = p[0];
  }
}

// Combines the chunk partials in chunk order.  64 * R rows per block (every lane owns R consecutive rows: with
// R = 2 the partials are read 16 bytes at a time, which is what an array of many sets wants; a single set gets
// more blocks out of R = 1); the four sums of a row are handled by four different waves so that the dependent
// add chains are short.
template <int R>
__global__ __launch_bounds__(320) void ranges_final_kernel(const RangeDesc* __restrict__ table, RangeDesc one) {
  const RangeDesc d = table ? table[blockIdx.z] : one;
  const int lane = threadIdx.x & 63;
  const int q = threadIdx.x >> 6;
  const int64_t r = ((int64_t)blockIdx.x * 64 + lane) * R;
  // the classes of the block's rows for the ReLU step that follows (RangeDesc::blk3), by the wave that has lb / ub
  auto count_classes = [&](const double (&l)[R], const double (&u)[R]) {
    int nc = 0, ni = 0, nk = 0;
#pragma unroll
    for (int e = 0; e < R; ++e) {
      const bool valid = r + e < d.nrows;
      const bool inactive = valid && (u[e] <= 0.0);
      const bool crossing = valid && (l[e] < 0.0) && (u[e] > 0.0);
      nc += __popcll(__ballot(crossing));
      ni += __popcll(__ballot(inactive));
      nk += __popcll(__ballot(valid && !inactive && !crossing));
    }
    if (lane == 0) {
      d.blk3[3 * blockIdx.x] = nc;
      d.blk3[3 * blockIdx.x + 1] = ni;
      d.blk3[3 * blockIdx.x + 2] = nk;
    }
  };
  if (d.chunks == 1 && d.chunks2 == 0 && d.part3 == nullptr && d.cols_per_chunk != 0) {  // the column pass wrote lb/ub itself
    if (d.blk3 != nullptr && q == 0) {
      double l[R], u[R];
#pragma unroll
      for (int e = 0; e < R; ++e) {
        l[e] = r + e < d.ld ? d.lb[r + e] : 0.0;
        u[e] = r + e < d.ld ? d.ub[r + e] : 0.0;
      }
      count_classes(l, u);
    }
    return;
  }
  __shared__ double sums[4][64 * R];
  __shared__ double cen[64 * R];
  if (q == 4) {  // a wave of its own (the launch that has a centre to form brings five)
    if (d.cchunks > 0 && r < d.ld) {
#pragma unroll
      for (int e = 0; e < R; ++e) {
        double c0 = 0.0;
        for (int c = 0; c < d.cchunks; c += 32) {
          double v[32];
#pragma unroll
          for (int u = 0; u < 32; ++u) v[u] = c + u < d.cchunks ? d.cpart[(int64_t)(c + u) * d.ld + r + e] : 0.0;
#pragma unroll
          for (int u = 0; u < 32; ++u)
            if (c + u < d.cchunks) c0 += v[u];
        }
        if (d.cbias != nullptr) c0 = c0 + d.cbias[r + e];
        d.cout[r + e] = c0;
        cen[lane * R + e] = c0;
      }
    }
    __syncthreads();
    return;
  }
  double s[R];
#pragma unroll
  for (int e = 0; e < R; ++e) s[e] = 0.0;
  if (r < d.ld) {
    // the partial sums were written by other CUs moments ago: every load is a trip to memory, so as many
    // as possible are in flight at once; the additions stay in chunk order
    const double* p = d.part + (int64_t)q * d.ld + r;
    int c = 0;
    if (d.chunks <= 8) {  // the common case after a fused GEMM epilogue: one short batch
      double v[8][R];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
#pragma unroll
        for (int e = 0; e < R; ++e) v[u][e] = 0.0;
        if (u < d.chunks) load_rows<R>(p + (int64_t)u * 4 * d.ld, v[u]);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (u < d.chunks) {
#pragma unroll
          for (int e = 0; e < R; ++e) s[e] += v[u][e];
        }
      c = d.chunks;
    }
    constexpr int kBatch = 32 / R;
    for (; c < d.chunks; c += kBatch) {
      double v[kBatch][R];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
#pragma unroll
        for (int e = 0; e < R; ++e) v[u][e] = 0.0;
        if (c + u < d.chunks) load_rows<R>(p + (int64_t)(c + u) * 4 * d.ld, v[u]);
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (c + u < d.chunks) {
#pragma unroll
          for (int e = 0; e < R; ++e) s[e] += v[u][e];
        }
    }
    if (d.chunks2 > 0) {
      const double* p2 = d.part2 + (int64_t)q * d.ld + r;
      const double* p2at = d.chunks2_at > 0 ? *d.part2_at + (int64_t)q * d.ld + r : p2;
      for (int c2 = 0; c2 < d.chunks2; c2 += 8) {
        double v[8][R];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
          for (int e = 0; e < R; ++e) v[u][e] = 0.0;
          if (c2 + u < d.chunks2) load_rows<R>((c2 + u < d.chunks2_at ? p2at : p2) + (int64_t)(c2 + u) * 4 * d.ld, v[u]);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (c2 + u < d.chunks2) {
#pragma unroll
            for (int e = 0; e < R; ++e) s[e] += v[u][e];
          }
      }
    }
    // xmin1, xmin2, xmax1, xmax2 sit in blocks 0, 3, 2, 1 of the product's two columns
    if (d.part3 != nullptr) {
      double v[R];
      load_rows<R>(d.part3 + (int64_t)((4 - q) & 3) * d.ld + r, v);
#pragma unroll
      for (int e = 0; e < R; ++e) s[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < R; ++e) sums[q][lane * R + e] = s[e];
  __syncthreads();
  if (q == 0) {
    double l[R], u[R];
#pragma unroll
    for (int e = 0; e < R; ++e) l[e] = u[e] = 0.0;
    if (r < d.ld) {
#pragma unroll
      for (int e = 0; e < R; ++e) {
        const double c0 = d.cchunks > 0 ? cen[lane * R + e] : d.V[r + e];
        l[e] = (c0 + sums[0][lane * R + e]) + sums[1][lane * R + e];
        u[e] = (c0 + sums[2][lane * R + e]) + sums[3][lane * R + e];
        d.lb[r + e] = l[e];
        d.ub[r + e] = u[e];
      }
    }
    if (d.blk3 != nullptr) count_classes(l, u);
  }
}


// ---- W * (block of scaled unit vectors) -------------------------------------------------------
// Column j of the block is scale * e_r, so the product column is W(:, r) * scale: a gather of W's
// columns.  0 + w*scale reproduces what the dense accumulation (starting from +0) leaves, bit for bit.
// Same geometry as the range pass, and with part != null it also leaves that pass's four partial
// sums for its columns.
struct GatherArgs {
  const double* W;
  int64_t ldw, ldout;
  int32_t cols_per_chunk;
  int32_t with_sums;  // every chunk of the grid leaves range sums in the set's `part` (if it has one)
  int64_t Mp;         // rows of W (a multiple of 16): the bias has that many entries
  // XCD-aware block order (xcd_row_blocks > 0; the grid is then one-dimensional): workgroups are dealt to the eight
  // XCDs round-robin, and every block of a 128-row slice of W goes to the same XCD (row block mod 8), sets and
  // column chunks in turn, so that the slice stays in that XCD's L2 while all sets gather from it.
  int32_t xcd_row_blocks, xcd_chunks, xcd_count;
};

// CENTRE: the variant that also forms the centre's product (GatherSet::cin); kept apart because its extra
// registers would cost the plain pass a resident block per CU.
template <bool CENTRE>
__global__ __launch_bounds__(64 * kRangeWaves) void gather_columns_kernel(const GatherSet* __restrict__ table, GatherSet one,
                                                                         GatherArgs a) {
  int row_block = blockIdx.x, chunk = blockIdx.y, set = blockIdx.z, nchunks = gridDim.y;
  if (a.xcd_row_blocks > 0) {
    const unsigned xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const unsigned per_rb = (unsigned)a.xcd_chunks * (unsigned)a.xcd_count;
    row_block = (int)((slot / per_rb) * 8u + xcd);
    if (row_block >= a.xcd_row_blocks) return;
    const unsigned rem = slot % per_rb;
    set = (int)(rem / (unsigned)a.xcd_chunks);
    chunk = (int)(rem % (unsigned)a.xcd_chunks);
    nchunks = a.xcd_chunks;
  }
  const GatherSet d = table ? table[set] : one;
  const int j0 = chunk * a.cols_per_chunk;
  double* part = a.with_sums ? d.part : nullptr;
  if (j0 >= d.m && part == nullptr && d.nfill == 0 && d.red == nullptr) return;
  // a set whose columns stay unwritten and whose sums come from elsewhere has no column work here
  const bool no_cols = d.lazy && part == nullptr && !(CENTRE && d.cin != nullptr);
  const int j1 = no_cols ? j0 : min(d.m, j0 + a.cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r0 = (int64_t)row_block * kRowsPerWave + 2 * lane;
  const bool active = r0 < a.ldout;
  // The centre column came out of a split-K product: the first chunk's blocks sum its partial vectors in
  // split order and add the bias, as the reduction kernel would have.
  if (d.red != nullptr && chunk == 0 && wave == 0 && active && r0 < a.Mp) {
    double2 s = make_double2(0.0, 0.0);
    for (int k = 0; k < d.red_k; ++k) {
      const double2 p = *reinterpret_cast<const double2*>(d.red + (int64_t)k * a.Mp + r0);
      s.x += p.x;
      s.y += p.y;
    }
    if (d.bias != nullptr) {
      s.x = s.x + d.bias[r0];
      s.y = s.y + d.bias[r0 + 1];
    }
    *reinterpret_cast<double2*>(d.centre + r0) = s;
  }
  // A contraction over no rows at all leaves +0 everywhere and the bias on the centre: this chunk's share
  // of those columns is written here instead of by a GEMM launch (they add nothing to the range sums).
  if (d.nfill > 0 && active) {
    const int nf = d.lazy ? 1 : d.nfill;  // unwritten columns: only the centre is stored
    const int fpc = (nf + nchunks - 1) / nchunks;
    const int f1 = min(nf, (chunk + 1) * fpc);
    for (int j = chunk * fpc + wave; j < f1; j += kRangeWaves) {
      double2 o = make_double2(0.0, 0.0);
      if (j == 0 && d.bias != nullptr && r0 < a.Mp) {
        o.x = __dadd_rn(0.0, d.bias[r0]);
        o.y = __dadd_rn(0.0, d.bias[r0 + 1]);
      }
      if (j == 0 || !d.lazy) *reinterpret_cast<double2*>(d.fill + r0 + (int64_t)j * a.ldout) = o;
    }
  }
  double2 xmin1 = {0, 0}, xmin2 = {0, 0}, xmax1 = {0, 0}, xmax2 = {0, 0}, cacc = {0, 0};
  if (active) {
    for (int jb = j0 + 4 * wave; jb < j1; jb += 4 * kRangeWaves) {
      double2 v[4];
      double sc[4], cj[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        v[u] = make_double2(0.0, 0.0);
        sc[u] = 1.0;
        cj[u] = 0.0;
        if (jb + u < j1) {
          const int src = d.idx[jb + u];
          if (d.scale != nullptr) sc[u] = d.scale[src];
          if (CENTRE && d.cin != nullptr) cj[u] = d.cin[src];
          v[u] = *reinterpret_cast<const double2*>(a.W + r0 + (int64_t)src * a.ldw);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jb + u;
        if (j >= j1) break;
        if (CENTRE && d.cin != nullptr) {  // the centre's product rides along
          cacc.x = fma(v[u].x, cj[u], cacc.x);
          cacc.y = fma(v[u].y, cj[u], cacc.y);
        }
        double2 o;
        o.x = __dadd_rn(0.0, __dmul_rn(v[u].x, sc[u]));
        o.y = __dadd_rn(0.0, __dmul_rn(v[u].y, sc[u]));
        if (!d.lazy) {  // (streaming store: nothing here reads the column again)
          typedef double dd2 __attribute__((ext_vector_type(2)));
          __builtin_nontemporal_store(dd2{o.x, o.y}, reinterpret_cast<dd2*>(d.out + r0 + (int64_t)j * a.ldout));
        }
        if (part != nullptr) {
          const double pl = d.plb[j], pu = d.pub[j];
          const double px = fmax(o.x, 0.0), nx = fmin(o.x, 0.0);
          const double py = fmax(o.y, 0.0), ny = fmin(o.y, 0.0);
          xmin1.x = fma(px, pl, xmin1.x);
          xmin1.y = fma(py, pl, xmin1.y);
          xmax1.x = fma(px, pu, xmax1.x);
          xmax1.y = fma(py, pu, xmax1.y);
          xmin2.x = fma(nx, pu, xmin2.x);
          xmin2.y = fma(ny, pu, xmin2.y);
          xmax2.x = fma(nx, pl, xmax2.x);
          xmax2.y = fma(ny, pl, xmax2.y);
        }
      }
    }
  }
  if (part == nullptr) return;
  __shared__ double2 red[kRangeWaves - 1][CENTRE ? 5 : 4][64];  // (wave 0 keeps its own in registers)
  if (wave > 0) {
    red[wave - 1][0][lane] = xmin1;
    red[wave - 1][1][lane] = xmin2;
    red[wave - 1][2][lane] = xmax1;
    red[wave - 1][3][lane] = xmax2;
    if (CENTRE) red[wave - 1][4][lane] = cacc;
  }
  __syncthreads();
  if (wave == 0 && active) {
    for (int w = 0; w < kRangeWaves - 1; ++w) {
      if (CENTRE) {
        cacc.x += red[w][4][lane].x;
        cacc.y += red[w][4][lane].y;
      }
      xmin1.x += red[w][0][lane].x;
      xmin1.y += red[w][0][lane].y;
      xmin2.x += red[w][1][lane].x;
      xmin2.y += red[w][1][lane].y;
      xmax1.x += red[w][2][lane].x;
      xmax1.y += red[w][2][lane].y;
      xmax2.x += red[w][3][lane].x;
      xmax2.y += red[w][3][lane].y;
    }
    double* p = part + ((int64_t)chunk * 4) * a.ldout + r0;
    *reinterpret_cast<double2*>(p) = xmin1;
    *reinterpret_cast<double2*>(p + a.ldout) = xmin2;
    *reinterpret_cast<double2*>(p + 2 * a.ldout) = xmax1;
    *reinterpret_cast<double2*>(p + 3 * a.ldout) = xmax2;
    if (CENTRE && d.cin != nullptr) *reinterpret_cast<double2*>(d.cpart + (int64_t)chunk * a.ldout + r0) = cacc;
  }
}

// The same pass for outputs of at most 32 rows (the last layer of a classifier): with one lane per two rows only
// 8 or 16 lanes of a wave would have rows, so a wave takes 64 / HL columns at once instead (HL = ldout / 2 lanes
// per column; a wave writes 1 KiB of consecutive columns per step).  Columns and, with part != null, their four
// range sums, and filled leading columns; nothing else (no split-K centre, no centre product, no unwritten columns).
template <int HL>
__global__ __launch_bounds__(256) void gather_skinny_kernel(const GatherSet* __restrict__ table, GatherSet one, GatherArgs a) {
  constexpr int CPW = 64 / HL;  // columns per wave and step
  typedef double dd2 __attribute__((ext_vector_type(2)));  // (streaming stores: nothing here reads a column again)
  const GatherSet d = table ? table[blockIdx.z] : one;
  const int chunk = blockIdx.y;
  const int j0 = chunk * a.cols_per_chunk;
  double* part = a.with_sums ? d.part : nullptr;
  if (j0 >= d.m && part == nullptr && d.nfill == 0) return;
  const int j1 = min(d.m, j0 + a.cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r0 = 2 * (lane % HL), cs = lane / HL;
  // leading columns a contraction over no rows would have left: the bias on the centre, +0 elsewhere
  if (d.nfill > 0) {
    const int fpc = (d.nfill + (int)gridDim.y - 1) / (int)gridDim.y;
    const int f1 = min(d.nfill, (chunk + 1) * fpc);
    for (int j = chunk * fpc + wave * CPW + cs; j < f1; j += 4 * CPW) {
      double2 o = make_double2(0.0, 0.0);
      if (j == 0 && d.bias != nullptr && r0 < a.Mp) {
        o.x = __dadd_rn(0.0, d.bias[r0]);
        o.y = __dadd_rn(0.0, d.bias[r0 + 1]);
      }
      __builtin_nontemporal_store(dd2{o.x, o.y}, reinterpret_cast<dd2*>(d.fill + r0 + (int64_t)j * a.ldout));
    }
  }
  double2 xmin1 = {0, 0}, xmin2 = {0, 0}, xmax1 = {0, 0}, xmax2 = {0, 0};
  for (int jb = j0 + wave * CPW + cs; jb < j1; jb += 4 * 4 * CPW) {
    double2 v[4];
    double sc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = jb + u * 4 * CPW;
      v[u] = make_double2(0.0, 0.0);
      sc[u] = 1.0;
      if (j < j1) {
        const int src = d.idx[j];
        if (d.scale != nullptr) sc[u] = d.scale[src];
        v[u] = *reinterpret_cast<const double2*>(a.W + r0 + (int64_t)src * a.ldw);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = jb + u * 4 * CPW;
      if (j >= j1) break;
      double2 o;
      o.x = __dadd_rn(0.0, __dmul_rn(v[u].x, sc[u]));
      o.y = __dadd_rn(0.0, __dmul_rn(v[u].y, sc[u]));
      __builtin_nontemporal_store(dd2{o.x, o.y}, reinterpret_cast<dd2*>(d.out + r0 + (int64_t)j * a.ldout));
      if (part != nullptr) {
        const double pl = d.plb[j], pu = d.pub[j];
        const double px = fmax(o.x, 0.0), nx = fmin(o.x, 0.0);
        const double py = fmax(o.y, 0.0), ny = fmin(o.y, 0.0);
        xmin1.x = fma(px, pl, xmin1.x);
        xmin1.y = fma(py, pl, xmin1.y);
        xmax1.x = fma(px, pu, xmax1.x);
        xmax1.y = fma(py, pu, xmax1.y);
        xmin2.x = fma(nx, pu, xmin2.x);
        xmin2.y = fma(ny, pu, xmin2.y);
        xmax2.x = fma(nx, pl, xmax2.x);
        xmax2.y = fma(ny, pl, xmax2.y);
      }
    }
  }
  if (part == nullptr) return;
  // the column slots of a wave are added pairwise (always the same tree), the waves then in wave order
  double2* acc[4] = {&xmin1, &xmin2, &xmax1, &xmax2};
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int mask = HL; mask < 64; mask *= 2) {
      acc[k]->x += __shfl_xor(acc[k]->x, mask);
      acc[k]->y += __shfl_xor(acc[k]->y, mask);
    }
  __shared__ double2 red[3][4][HL];
  if (wave > 0 && cs == 0) {
#pragma unroll
    for (int k = 0; k < 4; ++k) red[wave - 1][k][lane] = *acc[k];
  }
  __syncthreads();
  if (wave == 0 && cs == 0) {
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[k]->x += red[w][k][lane].x;
        acc[k]->y += red[w][k][lane].y;
      }
    double* q = part + ((int64_t)chunk * 4) * a.ldout + r0;
#pragma unroll
    for (int k = 0; k < 4; ++k) *reinterpret_cast<double2*>(q + k * a.ldout) = *acc[k];
  }
}

// Column chunks of a gather over `count` sets with at most max_m one-hot columns each.
int64_t gather_chunks_batch(int64_t ldout, int64_t count, int64_t max_m) {
  if (max_m <= 0) return 0;
  const int64_t row_blocks = ceil_div(ldout, kRowsPerWave);
  return std::max<int64_t>(1, std::min<int64_t>(ceil_div(8192, row_blocks * count), ceil_div(max_m, 4 * kRangeWaves)));
}

// Column chunks of the gather for one set of m one-hot columns: enough blocks to cover the chip.
int64_t gather_chunks(int64_t Mp, int64_t m) {
  if (m <= 0) return 0;
  const int64_t row_blocks = ceil_div(Mp, kRowsPerWave);
  return std::max<int64_t>(1, std::min<int64_t>(ceil_div(1024, row_blocks), ceil_div(m, 4 * kRangeWaves)));
}

int launch_gather_columns(nnvhip_ctx* ctx, const double* W, int64_t ldw, int64_t Mp, int64_t ldout, int64_t count,
                          const GatherSet* sets, int64_t chunks) {
  if (count <= 0) return NNVHIP_OK;
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  const bool with_sums = chunks > 0;
  // columns the launch has work for (a set that neither writes its columns nor wants their sums has none)
  int64_t max_m = 0, max_fill = 0;
  for (int64_t i = 0; i < count; ++i) {
    const bool idle = sets[i].lazy && !(with_sums && sets[i].part != nullptr) && sets[i].cin == nullptr;
    max_m = std::max<int64_t>(max_m, idle ? 0 : sets[i].m);
    max_fill = std::max<int64_t>(max_fill, sets[i].lazy ? std::min<int32_t>(sets[i].nfill, 1) : sets[i].nfill);
  }
  bool any_red = false;
  for (int64_t i = 0; i < count; ++i) any_red = any_red || sets[i].red != nullptr;
  if (max_m == 0 && max_fill == 0 && !any_red) return NNVHIP_OK;
  const int64_t row_blocks = ceil_div(ldout, kRowsPerWave);
  if (!with_sums) chunks = std::max<int64_t>(1, gather_chunks_batch(ldout, count, std::max(max_m, max_fill)));
  GatherArgs a{};
  a.W = W;
  a.ldw = ldw;
  a.ldout = ldout;
  a.Mp = Mp;
  a.with_sums = with_sums ? 1 : 0;
  a.cols_per_chunk = (int32_t)ceil_div(std::max<int64_t>(max_m, 1), chunks);
  const GatherSet* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(ctx->upload_table(sets, sizeof(GatherSet) * count, &tab));
    table = tab->as<GatherSet>();
  }
  // algorithmic HBM bytes: every output column that is written, once; W read once (its columns are
  // re-read from cache); the range sums of a set whose columns stay unwritten
  double bytes = 8.0 * (double)Mp * (double)ldw;
  for (int64_t i = 0; i < count; ++i)
    bytes += sets[i].lazy ? 8.0 * (double)Mp * (sets[i].nfill > 0 ? 1.0 : 0.0) + (with_sums && sets[i].part ? 32.0 * (double)ldout * (double)chunks : 0.0)
                          : 8.0 * (double)Mp * (double)(sets[i].m + sets[i].nfill);
  NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
  bool centre = false;
  for (int64_t i = 0; i < count; ++i) centre = centre || sets[i].cin != nullptr;
  // a skinny output whose columns are all written and that asks for nothing but columns and their sums
  bool skinny = (ldout == 16 || ldout == 32) && !centre && !any_red;
  for (int64_t i = 0; i < count && skinny; ++i) skinny = !sets[i].lazy;
  if (skinny) {
    const dim3 grid(1, (unsigned)chunks, (unsigned)count);
    if (ldout == 16)
      NNV_LAUNCH(ctx, ctx->kernel_timing, gather_skinny_kernel<8>, grid, dim3(256), 0, table, sets[0], a);
    else
      NNV_LAUNCH(ctx, ctx->kernel_timing, gather_skinny_kernel<16>, grid, dim3(256), 0, table, sets[0], a);
  } else {
    // large launches over arrays: blocks ordered so that a row slice of W is served from one XCD's L2
    dim3 grid((unsigned)row_blocks, (unsigned)chunks, (unsigned)count);
    const int64_t xcd_blocks = 8 * ceil_div(row_blocks, 8) * chunks * count;
    if (count >= 8 && row_blocks >= 8 && row_blocks * chunks * count >= 4096 && xcd_blocks < (int64_t(1) << 31) &&
        xcd_blocks * 4 <= row_blocks * chunks * count * 5) {
      a.xcd_row_blocks = (int32_t)row_blocks;
      a.xcd_chunks = (int32_t)chunks;
      a.xcd_count = (int32_t)count;
      grid = dim3((unsigned)xcd_blocks, 1, 1);
    }
    if (centre)
      NNV_LAUNCH(ctx, ctx->kernel_timing, gather_columns_kernel<true>, grid, dim3(64 * kRangeWaves), 0, table, sets[0], a);
    else
      NNV_LAUNCH(ctx, ctx->kernel_timing, gather_columns_kernel<false>, grid, dim3(64 * kRangeWaves), 0, table, sets[0], a);
  }
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 5, bytes));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

// ---- lb / ub of a fully connected layer's output straight from the weights (one set) -----------------
// The generator columns the layer gathers are W(:, r) * sc_r, one per input row r that carries a unit
// vector, so their four range sums are signed dot products of a row of W with one vector:
//   box star (bounds -1 / +1, sc >= 0):   S+ = sum_r max(W_ir, 0) * sc_r,  S- = sum_r min(W_ir, 0) * sc_r,
//                                          xmin1 = -S+, xmin2 = S-, xmax1 = S+, xmax2 = -S-
//   ReLU output (bounds 0 / ub_r, sc = 1): the same with sc_r = ub_r for crossing neurons (0 otherwise),
//                                          xmin1 = xmax2 = 0, xmin2 = S-, xmax1 = S+.
// One block owns 8 output rows and walks over all input rows: 8 lanes read 64 contiguous bytes of a column
// of W, the eight lane groups and the sixteen waves take different columns, and the block ends with the
// finished lb / ub of its rows (plus the partial sums the GEMM over the other columns left, plus the centre:
// taken from memory, formed along the way as W * c + b, or just b).  No partial sums leave the kernel and no
// reduction kernel follows.
struct RowSumArgs {
  const double* W;
  int64_t ldw;
  int32_t Mp, K;
  int32_t mode;         // 0: box star (scale), 1: ReLU output (cls, pre_ub)
  int32_t centre_mode;  // 0: the centre is in memory; 1: W * cin + bias, written; 2: 0 + bias, written
  const double* scale;
  const int32_t* cls;
  const double* pre_ub;
  const double* cin;
  const double* bias;
  double* centre;
  const double* part;  // [chunks][4][ld] from the GEMM epilogue, or null
  int32_t chunks;
  int32_t pad_;
  int64_t ld;
  double* lb;
  double* ub;
};

constexpr int kRowSumRows = 8;  // output rows per block

__global__ __launch_bounds__(1024) void fc_rowsum_kernel(RowSumArgs a) {
  __shared__ double red[16][3][kRowSumRows];
  __shared__ double skey[4 * kRowSumRows];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rl = lane & 7, cs = lane >> 3;
  const int row = blockIdx.x * kRowSumRows + rl;
  const double* wrow = a.W + row;
  const bool with_centre = a.centre_mode == 1;
  double sp = 0.0, sn = 0.0, cacc = 0.0;
  // 128 input rows per step (16 waves x 8 lane groups, 8 lanes = 64 contiguous bytes of a column of W);
  // eight steps' loads -- none depends on another -- are issued before any is used
  for (int r0 = wave * 8 + cs; r0 < a.K; r0 += 8 * 128) {
    double w[8], b[8], cj[8];
    int cl[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int r = r0 + u * 128;
      w[u] = 0.0;
      b[u] = 0.0;
      cj[u] = 0.0;
      cl[u] = -1;
      if (r < a.K) {
        w[u] = wrow[(int64_t)r * a.ldw];
        if (a.mode == 0) {
          b[u] = a.scale[r];
          cl[u] = 0;
        } else {
          b[u] = a.pre_ub[r];
          cl[u] = a.cls[r];
        }
        if (with_centre) cj[u] = a.cin[r];
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const double bu = cl[u] >= 0 ? b[u] : 0.0;  // ReLU output: only crossing neurons carry a column
      sp = fma(fmax(w[u], 0.0), bu, sp);
      sn = fma(fmin(w[u], 0.0), bu, sn);
      cacc = fma(w[u], cj[u], cacc);
    }
  }
  // the eight lane groups, then the sixteen waves, in a fixed order
#pragma unroll
  for (int off = 8; off < 64; off <<= 1) {
    sp += __shfl_xor(sp, off);
    sn += __shfl_xor(sn, off);
    cacc += __shfl_xor(cacc, off);
  }
  if (cs == 0) {
    red[wave][0][rl] = sp;
    red[wave][1][rl] = sn;
    red[wave][2][rl] = cacc;
  }
  __syncthreads();
  if (tid < 3 * kRowSumRows) {
    const int which = tid / kRowSumRows, r8 = tid % kRowSumRows;
    double t = 0.0;
#pragma unroll
    for (int w2 = 0; w2 < 16; ++w2) t += red[w2][which][r8];
    red[0][which][r8] = t;  // (the thread's own slot: read before it is written)
  }
  __syncthreads();
  if (tid < 4 * kRowSumRows) {  // sum q of a row: the GEMM tiles' chunks in order, then the gathered columns' term
    const int q = tid / kRowSumRows, r8 = tid % kRowSumRows;
    const int orow = blockIdx.x * kRowSumRows + r8;
    double x = 0.0;
    if (a.part != nullptr) {
      // (sixteen loads in flight at a time, added in chunk order: one at a time they cost a trip to memory each)
      for (int c = 0; c < a.chunks; c += 16) {
        double v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = c + u < a.chunks ? a.part[((int64_t)(c + u) * 4 + q) * a.ld + orow] : 0.0;
#pragma unroll
        for (int u = 0; u < 16; ++u)
          if (c + u < a.chunks) x += v[u];
      }
    }
    const double Sp = red[0][0][r8], Sn = red[0][1][r8];
    double term;
    if (a.mode == 0) term = q == 0 ? -Sp : q == 1 ? Sn : q == 2 ? Sp : -Sn;
    else term = q == 1 ? Sn : q == 2 ? Sp : 0.0;
    x += term;
    skey[tid] = x;
  }
  __syncthreads();
  if (tid < kRowSumRows) {
    const int orow = blockIdx.x * kRowSumRows + tid;
    double c0;
    if (a.centre_mode == 0) {
      c0 = a.centre[orow];
    } else {
      c0 = a.centre_mode == 1 ? red[0][2][tid] : 0.0;
      if (a.bias != nullptr) c0 = c0 + a.bias[orow];
      a.centre[orow] = c0;
    }
    // lb = (c + xmin1) + xmin2, the reference's left-to-right order (set/Star.m:1098-1104)
    a.lb[orow] = (c0 + skey[tid]) + skey[kRowSumRows + tid];
    a.ub[orow] = (c0 + skey[2 * kRowSumRows + tid]) + skey[3 * kRowSumRows + tid];
  }
}

int launch_fc_rowsum(nnvhip_ctx* ctx, const nnvhip_fc* fc, nnvhip_star* out, int mode, const double* scale, const int32_t* cls,
                     const double* pre_ub, int centre_mode, const double* cin, const double* part, int64_t chunks) {
  BufRef rb;
  NNV_TRY(ctx->alloc(sizeof(double) * 2 * out->ld, &rb));
  RowSumArgs a{};
  a.W = fc->W->as<double>();
  a.ldw = fc->Mp;
  a.Mp = (int32_t)fc->Mp;
  a.K = (int32_t)fc->K;
  a.mode = mode;
  a.centre_mode = centre_mode;
  a.scale = scale;
  a.cls = cls;
  a.pre_ub = pre_ub;
  a.cin = cin;
  a.bias = fc->bias ? fc->bias->as<double>() : nullptr;
  a.centre = out->V;
  a.part = part;
  a.chunks = (int32_t)chunks;
  a.ld = out->ld;
  a.lb = rb->as<double>();
  a.ub = a.lb + out->ld;
  const int64_t row_blocks = fc->Mp / kRowSumRows;
  // algorithmic bytes: W once, the finished ranges (timed with the gather passes it stands in for)
  const double bytes = 8.0 * (double)fc->Mp * (double)fc->K + 16.0 * (double)fc->Mp;
  NNV_LAUNCH(ctx, ctx->kernel_timing, fc_rowsum_kernel, dim3((unsigned)row_blocks), dim3(1024), 0, a);
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 5, bytes));
  NNV_HIP_TRY(hipGetLastError());
  out->rbuf = rb;
  out->lb = a.lb;
  out->ub = a.ub;
  return NNVHIP_OK;
}

// ---- range sums of gathered columns as one matrix product --------------------------------------------
__global__ __launch_bounds__(256) void split_sign_kernel(const double* __restrict__ W, double* __restrict__ Wpn, int64_t Mp,
                                                          int64_t Kp) {
  const int64_t total = Mp * Kp;
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = t % Mp, c = t / Mp;
    const double w = W[t];
    Wpn[r + c * 2 * Mp] = fmax(w, 0.0);
    Wpn[Mp + r + c * 2 * Mp] = fmin(w, 0.0);
  }
}

// Columns 2i and 2i+1 of X (Kp rows): a = scatter(sc * plb), b = scatter(sc * pub) of set i.
__global__ __launch_bounds__(256) void sum_vectors_kernel(const GatherSet* __restrict__ table, double* __restrict__ X, int Kp) {
  const GatherSet d = table[blockIdx.x];
  double* xa = X + (int64_t)2 * blockIdx.x * Kp;
  double* xb = xa + Kp;
  for (int k = threadIdx.x; k < Kp; k += 256) {
    xa[k] = 0.0;
    xb[k] = 0.0;
  }
  __syncthreads();
  for (int j = threadIdx.x; j < d.m; j += 256) {
    const int r = d.idx[j];
    const double sc = d.scale != nullptr ? d.scale[r] : 1.0;
    xa[r] = __dmul_rn(sc, d.plb[j]);
    xb[r] = __dmul_rn(sc, d.pub[j]);
  }
}

static int ensure_split_weights(nnvhip_ctx* ctx, const nnvhip_fc* fc) {
  if (fc->Wpn) return NNVHIP_OK;
  const int64_t Mp = fc->Mp, Kp = fc->Kp;
  BufRef w;
  NNV_TRY(ctx->alloc(sizeof(double) * 2 * Mp * Kp, &w));
  hipLaunchKernelGGL(split_sign_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(Mp * Kp, 256), 4096)), dim3(256), 0, ctx->stream,
                     fc->W->as<double>(), w->as<double>(), Mp, Kp);
  NNV_HIP_TRY(hipGetLastError());
  fc->Wpn = w;
  return NNVHIP_OK;
}

// [W+; W-] * (the odd columns of X) into the odd column pairs of *out, whose even ones ([xmin1; xmax2], products with
// a zero vector) are +0: what the product leaves when every gathered column has lower predicate bound zero.
// (zeroed: the caller's own kernel has already filled the even column pairs of *out, which it allocated)
static int range_sums_upper_half(nnvhip_ctx* ctx, const nnvhip_fc* fc, int64_t nu, const BufRef& X, BufRef* out, bool zeroed = false) {
  const int64_t Mp = fc->Mp, Kp = fc->Kp;
  if (!zeroed) {
    NNV_TRY(ctx->alloc(sizeof(double) * 2 * Mp * 2 * nu, out));
    NNV_HIP_TRY(hipMemsetAsync((*out)->ptr, 0, sizeof(double) * 2 * Mp * 2 * nu, ctx->stream));
  }
  std::vector<int32_t> odd((size_t)nu);
  for (int64_t k = 0; k < nu; ++k) odd[(size_t)k] = (int32_t)(2 * k + 1);
  BufRef cmap;
  NNV_TRY(ctx->upload_table(odd.data(), sizeof(int32_t) * odd.size(), &cmap));
  GemmRows rows;
  rows.colmap = cmap->as<int32_t>();
  if (Kp <= 2048) rows.tile_hint = 64;
  return launch_gemm(ctx, fc->Wpn->as<double>(), 2 * Mp, X->as<double>(), Kp, (*out)->as<double>(), 2 * Mp, 2 * Mp, nu, Kp, nullptr,
                     nullptr, &rows);
}

// Column 2i+1 of X (Kp rows): ub where the neuron crosses, zero elsewhere (column 2i is not read).  And column pair
// 2i of the product to come (2 * Mp2 entries, Mp2 = the product's rows), which no tile of it writes: +0.
__global__ __launch_bounds__(256) void crossing_ub_vectors_kernel(const AheadSet* __restrict__ table, double* __restrict__ X, int Kp, int N,
                                                                  double* __restrict__ prod, int64_t Mp2) {
  const AheadSet d = table[blockIdx.x];
  double* xb = X + ((int64_t)2 * blockIdx.x + 1) * Kp;
  for (int r = threadIdx.x; r < Kp; r += 256) xb[r] = (r < N && d.cls[r] >= 0) ? d.ub[r] : 0.0;
  double2* z = reinterpret_cast<double2*>(prod + (int64_t)2 * blockIdx.x * Mp2);  // (Mp2 is even, the buffer 256-byte aligned)
  for (int64_t r = threadIdx.x; r < Mp2 / 2; r += 256) z[r] = make_double2(0.0, 0.0);
}

int launch_range_sums_mm_ahead(nnvhip_ctx* ctx, const nnvhip_fc* fc, int64_t count, const AheadSet* sets, int64_t N, BufRef* out) {
  const int64_t Kp = fc->Kp;
  if (count >= (int64_t(1) << 30) || N > Kp) NNV_FAIL(NNVHIP_ERR_ARG, "internal: range sums ahead of their layer out of range");
  NNV_TRY(ensure_split_weights(ctx, fc));
  BufRef X, tab;
  NNV_TRY(ctx->alloc(sizeof(double) * Kp * 2 * count, &X));
  NNV_TRY(ctx->alloc(sizeof(double) * 2 * fc->Mp * 2 * count, out));
  NNV_TRY(ctx->upload_table(sets, sizeof(AheadSet) * count, &tab));
  hipLaunchKernelGGL(crossing_ub_vectors_kernel, dim3((unsigned)count), dim3(256), 0, ctx->stream, tab->as<AheadSet>(), X->as<double>(),
                     (int)Kp, (int)N, (*out)->as<double>(), 2 * fc->Mp);
  NNV_HIP_TRY(hipGetLastError());
  return range_sums_upper_half(ctx, fc, count, X, out, true);
}

int launch_range_sums_mm(nnvhip_ctx* ctx, const nnvhip_fc* fc, int64_t count, const GatherSet* sets, BufRef* out,
                         std::vector<int64_t>* slot, bool plb_zero) {
  const int64_t Mp = fc->Mp, Kp = fc->Kp;
  NNV_TRY(ensure_split_weights(ctx, fc));
  // Sets that gather the same columns with the same scales under the same bounds (the boxes of one shape,
  // nnvhip_star_from_box) have the same sums: one pair of columns serves them all.  Only runs of a few distinct
  // descriptions are looked for (a set is compared with the last 16 new ones; the columns a ReLU step appended --
  // no scales -- are a set's own list, and only the last description is looked at).
  std::vector<GatherSet> uniq;
  uniq.reserve((size_t)count);
  slot->assign((size_t)count, 0);
  for (int64_t i = 0; i < count; ++i) {
    int64_t found = -1;
    const int64_t back = sets[i].scale != nullptr ? 16 : 1;
    for (int64_t k = (int64_t)uniq.size() - 1; k >= 0 && k >= (int64_t)uniq.size() - back && found < 0; --k) {
      const GatherSet& u = uniq[(size_t)k];
      if (u.idx == sets[i].idx && u.scale == sets[i].scale && u.plb == sets[i].plb && u.pub == sets[i].pub && u.m == sets[i].m) found = k;
    }
    if (found < 0) {
      found = (int64_t)uniq.size();
      uniq.push_back(sets[i]);
    }
    (*slot)[(size_t)i] = found;
  }
  const int64_t nu = (int64_t)uniq.size();
  BufRef X, tab;
  NNV_TRY(ctx->alloc(sizeof(double) * Kp * 2 * nu, &X));
  NNV_TRY(ctx->upload(uniq.data(), sizeof(GatherSet) * nu, &tab));
  hipLaunchKernelGGL(sum_vectors_kernel, dim3((unsigned)nu), dim3(256), 0, ctx->stream, tab->as<GatherSet>(), X->as<double>(), (int)Kp);
  NNV_HIP_TRY(hipGetLastError());
  // a = scatter(sc * plb) is zero for every set: its products [xmin1; xmax2] are +0 (a fill), and only the columns
  // of b = scatter(sc * pub) go through the matrix cores
  if (plb_zero && nu < (int64_t(1) << 30)) return range_sums_upper_half(ctx, fc, nu, X, out);
  NNV_TRY(ctx->alloc(sizeof(double) * 2 * Mp * 2 * nu, out));
  return launch_gemm(ctx, fc->Wpn->as<double>(), 2 * Mp, X->as<double>(), Kp, (*out)->as<double>(), 2 * Mp, 2 * Mp, 2 * nu, Kp,
                     nullptr);
}

// Whether the range scan of a set reads its generator images inside their windows only: the windows must cover
// every column the scan reads (all stored ones), describe this set's image, and be small next to it.
static bool scan_in_windows(const nnvhip_star* t) {
  if (t->box == nullptr || t->rows_pending || t->box_H <= 0 || t->box_W <= 0) return false;
  const int64_t P = (int64_t)t->box_H * t->box_W;
  if (t->N % P != 0 || t->box_cols < t->stored_cols()) return false;
  return 2 * (int64_t)t->box_eh * t->box_ew <= P;
}

int compute_ranges(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* s, RangeCounts* counts) {
  // sets that already carry ranges are skipped
  std::vector<nnvhip_star*> todo;
  todo.reserve((size_t)count);
  const uint64_t visit = ++ctx->visit_seq;  // (a handle may be listed twice)
  for (int64_t i = 0; i < count; ++i)
    if (!s[i]->lb && s[i]->visit != visit) {
      s[i]->visit = visit;
      todo.push_back(s[i]);
    }
  if (todo.empty()) return NNVHIP_OK;
  // Sets whose generator images are in memory inside their windows only are scanned inside the windows (all
  // sets of the call, or none: one launch serves them all; the same sums to the bit either way).
  bool in_windows = tune_knobs().ranges_row_waves == 0;
  {
    bool any_win = false;
    for (auto* t : todo) {
      in_windows = in_windows && scan_in_windows(t) && t->box_H == todo[0]->box_H && t->box_W == todo[0]->box_W && t->N == todo[0]->N;
      any_win = any_win || t->cs.win_pending();
    }
    in_windows = in_windows && any_win;
  }
  // The scan reads the columns the producer left no sums for.  Columns that are described but not in
  // memory yet are written first only if they are among those (they normally come with their sums).
  {
    std::vector<nnvhip_star*> cols;
    for (auto* t : todo) {
      const int64_t scan_end = (t->has_producer_sums() && t->rng_first_col >= 1) ? t->rng_first_col : t->n + 1;
      // (columns that are in memory inside their windows only are fine for a scan that stays inside the windows)
      const bool win = t->cs.win_pending() && scan_end > t->cs.win_from && !in_windows;
      if ((t->cs.pending && scan_end > t->cs.from) || (t->cs.zero_to > 1 && scan_end > 1) || win ||
          (t->cs.delta_pending() && scan_end > 1))
        cols.push_back(t);
    }
    if (!cols.empty()) NNV_TRY(write_pending_columns(ctx, (int64_t)cols.size(), cols.data()));
  }
  NNV_TRY(ensure_dense_batch(ctx, (int64_t)todo.size(), todo.data(), true, false));
  const int64_t nset = (int64_t)todo.size();
  if (nset > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  int64_t ld = todo[0]->ld;
  int64_t nmax = 0;
  for (auto* t : todo) {
    if (t->ld != ld) NNV_FAIL(NNVHIP_ERR_SHAPE, "sets of one array must have the same dimension");
    nmax = std::max(nmax, t->n);
  }
  // Column chunking: enough blocks to cover the chip a few times over, at least 64 columns per
  // chunk so the partial-sum traffic stays below ~6 % of V.
  int row_waves = 1;  // measured best: all eight waves on the same 128 rows, interleaving columns
  if (const int v = tune_knobs().ranges_row_waves) row_waves = v == 8 ? 8 : v == 4 ? 4 : v == 2 ? 2 : 1;
  const int64_t row_blocks = ceil_div(ld, kRowsPerWave * row_waves);
  int64_t want_blocks = 2048;
  if (const int v = tune_knobs().ranges_blocks) want_blocks = std::max(1, v);
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(want_blocks, row_blocks * nset), ceil_div(nmax, 64)));
  chunks = std::min<int64_t>(chunks, 1024);
  // one buffer for all lb/ub, one for all partials
  BufRef rb, pb;
  NNV_TRY(ctx->alloc(sizeof(double) * 2 * ld * nset, &rb));
  bool pending = false;
  for (auto* t : todo) pending = pending || t->has_producer_sums();
  if (chunks > 1 || pending) NNV_TRY(ctx->alloc(sizeof(double) * 4 * ld * chunks * nset, &pb));
  std::vector<RangeDesc> descs(nset);
  bool any_pending = false;
  for (int64_t i = 0; i < nset; ++i) {
    nnvhip_star* t = todo[i];
    RangeDesc& d = descs[i];
    d.V = t->V;
    d.plb = t->plb;
    d.pub = t->pub;
    d.ld = ld;
    d.n = (int32_t)t->n;
    int64_t ch = std::max<int64_t>(1, std::min<int64_t>(chunks, ceil_div(t->n, 64)));
    d.chunks = (int32_t)ch;
    d.cols_per_chunk = (int32_t)std::max<int64_t>(1, ceil_div(t->n, ch));
    d.part = pb ? pb->as<double>() + 4 * ld * chunks * i : nullptr;
    d.lb = rb->as<double>() + 2 * ld * i;
    d.ub = d.lb + ld;
    d.row_waves = row_waves;
    d.part2 = nullptr;
    d.part3 = nullptr;
    d.chunks2 = 0;
    d.chunks2_at = 0;
    d.part2_at = nullptr;
    d.cchunks = 0;
    d.cpart = nullptr;
    d.cbias = nullptr;
    d.cout = nullptr;
    d.box = nullptr;
    d.bH = d.bW = 0;
    d.blk3 = nullptr;
    d.nrows = 0;
    if (in_windows) {
      d.box = t->box;
      d.bH = t->box_H;
      d.bW = t->box_W;
    }
    if (t->has_producer_sums() && t->rng_first_col >= 1) {
      // the producer of the trailing columns left their sums: scan only the columns before them
      d.part2 = t->rng_chunks > 0 ? t->rng_part : nullptr;
      d.chunks2 = d.part2 ? (int32_t)t->rng_chunks : 0;
      if (d.part2 && t->rng_part_at != nullptr) {
        d.part2_at = t->rng_part_at;
        d.chunks2_at = (int32_t)std::min(t->rng_chunks_at, t->rng_chunks);
      }
      d.part3 = t->rng_mm;
      d.n = (int32_t)(t->rng_first_col - 1);
      ch = std::max<int64_t>(1, std::min<int64_t>(chunks, ceil_div(std::max<int64_t>(d.n, 1), 64)));
      d.chunks = (int32_t)ch;
      d.cols_per_chunk = (int32_t)std::max<int64_t>(1, ceil_div(std::max<int64_t>(d.n, 1), ch));
      any_pending = true;
    }
  }
  // every column of every set already has its sums from the producing kernels: no scan at all
  bool scan = false;
  for (int64_t i = 0; i < nset; ++i) scan = scan || !(descs[i].n == 0 && (descs[i].chunks2 > 0 || descs[i].part3 != nullptr));
  if (!scan)
    for (int64_t i = 0; i < nset; ++i) descs[i].chunks = 0;
  // an array of sets has blocks to spare for the last step: two rows per lane, read 16 bytes at a time
  bool wide_final = ceil_div(ld, 64) * nset >= 4096;
  {
    auto aligned16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    for (int64_t i = 0; i < nset && wide_final; ++i)
      wide_final = aligned16(descs[i].part) && aligned16(descs[i].part2) && aligned16(descs[i].part3) && aligned16(descs[i].V) &&
                   aligned16(descs[i].lb);
  }
  if (counts != nullptr && counts->base != nullptr && (chunks > 1 || any_pending) && nset == count) {
    // (every set of the call is in the table, in the caller's order)
    for (int64_t i = 0; i < nset; ++i) {
      descs[i].blk3 = counts->base + counts->stride * i;
      descs[i].nrows = counts->nrows;
    }
    counts->gran = wide_final ? 128 : 64;
  }
  const RangeDesc* table = nullptr;
  BufRef tab;
  if (nset > 1) {
    NNV_TRY(ctx->upload_table(descs.data(), sizeof(RangeDesc) * nset, &tab));
    table = tab->as<RangeDesc>();
  }
  dim3 grid((unsigned)row_blocks, (unsigned)chunks, (unsigned)nset);
  double bytes = 0.0;  // algorithmic: V once, the predicate bounds, lb/ub out
  for (int64_t i = 0; i < nset; ++i)
    bytes += 8.0 * (double)todo[i]->N * (double)(descs[i].n + 1) + 16.0 * (double)descs[i].n + 16.0 * (double)todo[i]->N;
  if (scan && in_windows) {
    const int P = descs[0].bH * descs[0].bW;
    const int C = (int)(todo[0]->N / P);
    // two positions per lane (16-byte loads) where every image row then starts on a 16-byte boundary
    bool wide = P % 2 == 0;
    for (int64_t i = 0; i < nset && wide; ++i) wide = (reinterpret_cast<uintptr_t>(descs[i].V) & 15) == 0;
    NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
    if (wide) {
      const int nposb = (int)ceil_div(P, 128);
      NNV_LAUNCH(ctx, ctx->kernel_timing, ranges_window_kernel<2>, dim3((unsigned)(nposb * ceil_div(C, 2)), (unsigned)chunks, (unsigned)nset),
                 dim3(512), 0, table, descs[0], nposb, C);
    } else {
      const int nposb = (int)ceil_div(P, 64);
      NNV_LAUNCH(ctx, ctx->kernel_timing, ranges_window_kernel<1>, dim3((unsigned)(nposb * ceil_div(C, 4)), (unsigned)chunks, (unsigned)nset),
                 dim3(512), 0, table, descs[0], nposb, C);
    }
    NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 2, bytes));
  } else if (scan) {
    NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
    NNV_LAUNCH(ctx, ctx->kernel_timing, (ranges_partial_kernel<8, 4>), grid, dim3(64 * kRangeWaves), 0, table, descs[0]);
    NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 2, bytes));
  }
  if (chunks > 1 || any_pending) {
    double fbytes = 0.0;  // every chunk's four sums read, lb and ub written
    for (int64_t i = 0; i < nset; ++i) fbytes += 8.0 * (double)ld * (4.0 * (double)(descs[i].chunks + descs[i].chunks2) + 3.0);
    if (wide_final)
      NNV_LAUNCH(ctx, ctx->kernel_timing, ranges_final_kernel<2>, dim3((unsigned)ceil_div(ld, 128), 1, (unsigned)nset), dim3(256), 0,
                 table, descs[0]);
    else
      NNV_LAUNCH(ctx, ctx->kernel_timing, ranges_final_kernel<1>, dim3((unsigned)ceil_div(ld, 64), 1, (unsigned)nset), dim3(256), 0,
                 table, descs[0]);
    NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 7, fbytes));
  }
  NNV_HIP_TRY(hipGetLastError());
  for (int64_t i = 0; i < nset; ++i) {
    todo[i]->rbuf = rb;
    todo[i]->lb = descs[i].lb;
    todo[i]->ub = descs[i].ub;
    todo[i]->rng_buf.reset();  // the sums are folded in
    todo[i]->rng_part = nullptr;
    todo[i]->rng_chunks = 0;
    todo[i]->rng_at_buf.reset();
    todo[i]->rng_part_at = nullptr;
    todo[i]->rng_chunks_at = 0;
    todo[i]->rng_mm_buf.reset();
    todo[i]->rng_mm = nullptr;
  }
  return NNVHIP_OK;
}

int finalize_fused_ranges(nnvhip_ctx* ctx, nnvhip_star* s, const BufRef& part, int64_t chunks, const double* cpart,
                          int64_t cchunks, const double* cbias) {
  if (s->lb || chunks < 1) return NNVHIP_OK;
  BufRef rb;
  NNV_TRY(ctx->alloc(sizeof(double) * 2 * s->ld, &rb));
  RangeDesc d{};
  d.V = s->V;
  d.plb = s->plb;
  d.pub = s->pub;
  d.part = part->as<double>();
  d.lb = rb->as<double>();
  d.ub = d.lb + s->ld;
  d.ld = s->ld;
  d.n = (int32_t)s->n;
  d.chunks = (int32_t)chunks;
  d.cols_per_chunk = 0;
  d.row_waves = 1;
  d.part2 = nullptr;
  d.part3 = nullptr;
  d.chunks2 = 0;
  d.cchunks = (int32_t)cchunks;
  d.cpart = cpart;
  d.cbias = cbias;
  d.cout = s->V;
  NNV_LAUNCH(ctx, ctx->kernel_timing, ranges_final_kernel<1>, dim3((unsigned)ceil_div(s->ld, 64), 1, 1),
             dim3(cchunks > 0 ? 320 : 256), 0, nullptr, d);
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 7, 8.0 * (double)s->ld * (4.0 * (double)chunks + 3.0)));
  NNV_HIP_TRY(hipGetLastError());
  s->rbuf = rb;
  s->lb = d.lb;
  s->ub = d.ub;
  return NNVHIP_OK;
}

// ---- estimateRanges without any allocation ----------------------------------------------------------
// The column pass leaves one [4][ld] block of partial sums per column chunk, which the reduction kernel
// then combines; nnvhip_estimate_ranges takes that workspace (and the lb / ub vectors) from the context's
// pool.  The variant below takes both from a fixed array in device memory instead, so that it never
// allocates.  Every GPU holds its own copy of the array at its own address: the address is looked up
// once per context (with the context's device current) and the kernels get it as an argument.
constexpr int64_t kStaticScratchDoubles = int64_t(4) << 20;  // 32 MiB per GPU, held until the process ends
static __device__ __align__(256) double scratch[kStaticScratchDoubles];

// Every context has a stream of its own, and all contexts on one GPU share the array: the last use on each
// device is marked by an event, and a call from another context makes its stream wait for that event first, so
// that calls from several contexts of one host thread (or of threads that do not overlap in time) are ordered
// on the device as well.  The events are made when a device sees its first context and live until the process ends.
namespace {
constexpr int kMaxDevices = 64;
struct StaticUse {
  hipEvent_t done = nullptr;
  const nnvhip_ctx* last = nullptr;  // whose stream recorded `done` (compared, never dereferenced)
};
StaticUse g_static_use[kMaxDevices];
std::mutex g_static_use_mutex;
}  // namespace

int init_static_scratch(nnvhip_ctx* ctx) {
  void* p = nullptr;
  NNV_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  ctx->static_scratch = static_cast<double*>(p);
  ctx->static_scratch_doubles = kStaticScratchDoubles;
  if (ctx->device >= 0 && ctx->device < kMaxDevices) {
    std::lock_guard<std::mutex> lock(g_static_use_mutex);
    StaticUse& u = g_static_use[ctx->device];
    if (u.done == nullptr) NNV_HIP_TRY(hipEventCreateWithFlags(&u.done, hipEventDisableTiming));
  }
  return NNVHIP_OK;
}

__global__ __launch_bounds__(256) void copy_ranges_kernel(const double* __restrict__ lb, const double* __restrict__ ub,
                                                           double* __restrict__ lb_out, double* __restrict__ ub_out,
                                                           int64_t N) {
  const int64_t r = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (r < N) {
    if (lb_out != nullptr) lb_out[r] = lb[r];
    if (ub_out != nullptr) ub_out[r] = ub[r];
  }
}

int ranges_into_static(nnvhip_ctx* ctx, const nnvhip_star* s, double* lb_dev, double* ub_dev) {
  if (ctx->static_scratch == nullptr) NNV_FAIL(NNVHIP_ERR_HIP, "internal: the static workspace has no address on this device");
  if (s->lb != nullptr && s->ub != nullptr) {
    // the handle already caches its ranges (an earlier estimateRanges, a producing layer): no workspace is needed
    hipLaunchKernelGGL(copy_ranges_kernel, dim3((unsigned)ceil_div(s->N, 256)), dim3(256), 0, ctx->stream, s->lb, s->ub, lb_dev,
                       ub_dev, s->N);
    NNV_HIP_TRY(hipGetLastError());
    return NNVHIP_OK;
  }
  if (ctx->device < 0 || ctx->device >= kMaxDevices) NNV_FAIL(NNVHIP_ERR_ARG, "device number %d is out of range", ctx->device);
  // the set must be a plain stored matrix: writing pending columns or rows would need a buffer
  if (s->rows_pending || s->cs.any_pending() || s->stored_cols() != s->n + 1)
    NNV_FAIL(NNVHIP_ERR_ARG, "nnvhip_estimate_ranges_static: parts of this set are not in memory yet (read it once, or use "
                             "nnvhip_estimate_ranges)");
  const int64_t ld = s->ld, n = s->n;
  if (n >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "too many predicate variables");
  // workspace: lb (ld), ub (ld), then chunks x [4][ld] partial sums
  if (6 * ld > ctx->static_scratch_doubles)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "nnvhip_estimate_ranges_static: a set of dimension %lld does not fit the static workspace "
                               "(at most %lld rows)", (long long)s->N, (long long)(ctx->static_scratch_doubles / 6 / kLdAlign * kLdAlign));
  const int64_t row_blocks = ceil_div(ld, kRowsPerWave);
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(2048, row_blocks), ceil_div(n, 64)));
  chunks = std::min<int64_t>(chunks, 1024);
  chunks = std::min<int64_t>(chunks, (ctx->static_scratch_doubles - 2 * ld) / (4 * ld));  // >= 1, checked above
  RangeDesc d{};
  d.V = s->V;
  d.plb = s->plb;
  d.pub = s->pub;
  d.lb = ctx->static_scratch;
  d.ub = d.lb + ld;
  d.part = d.ub + ld;
  d.ld = ld;
  d.n = (int32_t)n;
  d.chunks = (int32_t)chunks;
  d.cols_per_chunk = (int32_t)std::max<int64_t>(1, ceil_div(std::max<int64_t>(n, 1), chunks));
  d.row_waves = 1;
  std::lock_guard<std::mutex> lock(g_static_use_mutex);
  StaticUse& use = g_static_use[ctx->device];
  if (use.last != nullptr && use.last != ctx) NNV_HIP_TRY(hipStreamWaitEvent(ctx->stream, use.done, 0));
  hipLaunchKernelGGL((ranges_partial_kernel<8, 4>), dim3((unsigned)row_blocks, (unsigned)chunks, 1), dim3(64 * kRangeWaves), 0,
                     ctx->stream, nullptr, d);
  if (chunks > 1)
    hipLaunchKernelGGL(ranges_final_kernel<1>, dim3((unsigned)ceil_div(ld, 64), 1, 1), dim3(256), 0, ctx->stream, nullptr, d);
  hipLaunchKernelGGL(copy_ranges_kernel, dim3((unsigned)ceil_div(s->N, 256)), dim3(256), 0, ctx->stream, d.lb, d.ub, lb_dev, ub_dev,
                     s->N);
  NNV_HIP_TRY(hipGetLastError());
  NNV_HIP_TRY(hipEventRecord(use.done, ctx->stream));
  use.last = ctx;
  return NNVHIP_OK;
}

// ---- columns an FC map described but did not write ------------------------------------------------
namespace {
struct PendingCols {
  double* V;
  int64_t ld;
  ColSource* cs;
};

// Writes the zeros outside the windows of the columns [j0, j1) of a matrix of N = H * W * C rows (the rows inside
// a window hold values and are left alone).  Lane = one row, the waves of a block interleave columns.
__global__ __launch_bounds__(512) void zero_outside_windows_kernel(double* __restrict__ V, int64_t ld, int64_t N,
                                                                   const ColBox* __restrict__ box, int64_t j0, int64_t j1, int H,
                                                                   int W, int cols_per_chunk) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r = (int64_t)blockIdx.x * 64 + lane;
  if (r >= N) return;
  const int p = (int)(r % ((int64_t)H * W));
  const int w = p / H, h = p - w * H;
  const int64_t ja = j0 + (int64_t)blockIdx.y * cols_per_chunk;
  const int64_t jb = min(j1, ja + cols_per_chunk);
  for (int64_t j = ja + wave; j < jb; j += 8) {
    const ColBox b = box[j];
    if (!(h >= b.h0 && h <= b.h1 && w >= b.w0 && w <= b.w1)) V[r + j * ld] = 0.0;
  }
}

static int write_window_zeros(nnvhip_ctx* ctx, double* V, int64_t ld, ColSource* cs) {
  const int64_t ncols = cs->win_to - cs->win_from;
  if (ncols > 0) {
    const int64_t rows = cs->win_rows;  // (the padding rows up to ld are zero already)
    const int64_t row_blocks = ceil_div(rows, 64);
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(8192, row_blocks), ceil_div(ncols, 32)));
    const int64_t cpc = ceil_div(ncols, chunks);
    chunks = ceil_div(ncols, cpc);
    hipLaunchKernelGGL(zero_outside_windows_kernel, dim3((unsigned)row_blocks, (unsigned)chunks), dim3(512), 0, ctx->stream, V, ld, rows,
                       cs->win_box, cs->win_from, cs->win_to, (int)cs->win_H, (int)cs->win_W, (int)cpc);
    NNV_HIP_TRY(hipGetLastError());
  }
  cs->win_from = cs->win_to = 0;
  return NNVHIP_OK;
}

// One gather launch per run of sets that share the weight matrix and the leading dimension.
int write_cols(nnvhip_ctx* ctx, std::vector<PendingCols>& todo) {
  // matrices a shared-product call described and did not store: all sets of such a call in one pass
  for (auto& t : todo)
    if (t.cs->delta_pending()) {
      DeltaCall& dc = *t.cs->delta;
      NNV_TRY(launch_delta_tiles(ctx, dc.A, dc.lda, dc.Mp, dc.bias_ptr, dc.ldo, (int64_t)dc.outs.size(), dc.outs.data(), dc.group.data(),
                                 dc.max_cols, dc.bytes, true));
      dc.written = true;
    }
  {  // columns written inside their windows only: the zeros around them
    std::vector<PendingCols> rest;
    for (auto& t : todo) {
      if (t.cs->win_pending()) NNV_TRY(write_window_zeros(ctx, t.V, t.ld, t.cs));
      if (t.cs->any_pending()) rest.push_back(t);
    }
    todo.swap(rest);
  }
  size_t a = 0;
  while (a < todo.size()) {
    size_t b = a + 1;
    while (b < todo.size() && b - a < 65535 && todo[b].cs->W == todo[a].cs->W && todo[b].ld == todo[a].ld &&
           todo[b].cs->ldw == todo[a].cs->ldw && todo[b].cs->rows == todo[a].cs->rows)
      ++b;
    std::vector<GatherSet> gs(b - a);
    for (size_t i = a; i < b; ++i) {
      const ColSource& cs = *todo[i].cs;
      GatherSet& g = gs[i - a];
      g = GatherSet{};
      g.idx = cs.idx;
      g.scale = cs.scale;
      g.out = todo[i].V + cs.from * todo[i].ld;
      g.m = cs.pending ? (int32_t)cs.cols : 0;
      if (cs.zero_to > 1) {  // column 0 (the centre) is in memory already
        g.nfill = (int32_t)(cs.zero_to - 1);
        g.fill = todo[i].V + todo[i].ld;
      }
    }
    const ColSource& c0 = *todo[a].cs;
    NNV_TRY(launch_gather_columns(ctx, c0.W, c0.ldw, c0.rows, todo[a].ld, (int64_t)(b - a), gs.data(), 0));
    for (size_t i = a; i < b; ++i) {
      todo[i].cs->pending = false;
      todo[i].cs->zero_to = 0;
    }
    a = b;
  }
  return NNVHIP_OK;
}
}  // namespace

int write_pending_columns(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* sets) {
  std::vector<PendingCols> todo;
  for (int64_t i = 0; i < count; ++i)
    if (sets[i]->cs.any_pending()) todo.push_back(PendingCols{sets[i]->V, sets[i]->ld, &sets[i]->cs});
  return todo.empty() ? NNVHIP_OK : write_cols(ctx, todo);
}

int write_pending_columns(nnvhip_ctx* ctx, double* V, int64_t ld, ColSource* cs) {
  if (!cs->any_pending()) return NNVHIP_OK;
  std::vector<PendingCols> todo{PendingCols{V, ld, cs}};
  return write_cols(ctx, todo);
}

}  // namespace nnvhip
