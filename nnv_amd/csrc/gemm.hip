// affineMap of a fully connected layer: C = W * [c V] on fp64 MFMA (v_mfma_f64_16x16x4_f64).
//
// Both operands are staged through LDS in K-tiles of 16.  The MFMA operand roles are chosen for
// column-major stores: the instruction's "b" operand carries 16 consecutive ROWS of W (the
// memory-contiguous direction of C), its "a" operand 16 columns of V, so lane l, register r of
// an accumulator holds C[row0 + l%16][col0 + l/16 + 4r] and lanes 0..15 store one 128-byte line.
#include <algorithm>
#include <cstdlib>
#include <string>

#include "internal.h"
#include "mfma_tile.h"

namespace nnvhip {

// TM x TN output tile per block of WR x WC waves, each wave owning
// (TM/WR) x (TN/WC) = (16*FM) x (16*FN).
// MAPPED = false: the plain product.  MAPPED = true additionally honours a row list (kmap), a per-tile
// segment table (segs) and a column map (colmap); kept apart so that the plain kernel pays nothing.
// WPE: waves per SIMD the register allocation is held to (1: whatever the code needs).
template <int TM, int TN, int WR, int WC, int KT, bool MAPPED, int WPE = 1>
__global__ __launch_bounds__(64 * WR * WC, WPE) void gemm_f64_kernel(const double* __restrict__ A, int64_t lda,
                                                        const double* __restrict__ B, int64_t ldb,
                                                        double* __restrict__ C, int64_t ldc, int Mp, int64_t ncols,
                                                        int Kp, const double* __restrict__ bias, int tiles_m,
                                                        int tiles_n, int xr, int local_m, int ksplit,
                                                        double* __restrict__ part,
                                                        const double* __restrict__ plb,
                                                        const double* __restrict__ pub,
                                                        double* __restrict__ rpart,
                                                        const int32_t* __restrict__ kmap,
                                                        const GemmSeg* __restrict__ segs,
                                                        const int32_t* __restrict__ colmap,
                                                        const double* __restrict__ Bk, int64_t ldbk) {
  constexpr int NT = 64 * WR * WC;  // threads per block
  constexpr int FM = TM / WR / 16;
  constexpr int FN = TN / WC / 16;
  constexpr int LDA_S = TM + kPadRow;  // Ws[k][row]
  constexpr int LDB_S = KT + kPadK;    // Vs[col][k]
  __shared__ double Ws[2][KT * LDA_S];
  __shared__ double Vs[2][TN * LDB_S];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wr = wave % WR;
  const int wc = wave / WR;
  // XCD-aware tile mapping.  Workgroups are dealt round-robin to the 8 XCDs (each with its own
  // 4 MiB L2) by linear id, so blockIdx.x % 8 names the XCD.  The XCDs form an xr x (8/xr) grid over
  // the tile matrix: XCD (i, j) owns the row tiles congruent to i mod xr and the column tiles
  // congruent to j mod 8/xr, i.e. it touches 1/xr of W and xr/8 of V instead of all of V.  Inside
  // an XCD consecutive blocks walk down the row tiles of one column tile, keeping its V tile hot.
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int xc = 8 / xr;
  const int mt = (slot % local_m) * xr + (xcd % xr);
  const int64_t nt = (int64_t)(slot / local_m) * xc + (xcd / xr);
  if (mt >= tiles_m || nt >= tiles_n) return;
  const int m0 = mt * TM;
  const int64_t n0 = nt * TN;
  // Row-compacted contraction: kmap lists the rows of B (= columns of A) that can be non-zero, padded
  // to whole K-tiles with -1; with a segment table every column tile has its own list (one per set).
  int64_t col_base = n0;       // column of B and C behind the tile's first column
  int64_t col_end = ncols;     // first column past the valid ones, in the same numbering as col_base
  int64_t bk_col0 = n0;        // column of Bk behind the tile's first column
  int64_t b_col_base = n0;     // column of B behind the tile's first column
  // fused range sums: the tile's first column and the end of the valid ones in the numbering of plb / pub
  // (the set's own columns), and the chunk of partial sums the tile fills
  int64_t rcol0 = n0, rcol_end = ncols, rchunk = nt;
  if (MAPPED && segs != nullptr) {
    const GemmSeg sg = segs[nt];
    rpart = sg.rpart;
    plb = sg.plb;
    pub = sg.pub;
    rcol0 = sg.col_local0;
    rcol_end = sg.col_local0 + sg.valid;
    rchunk = 0;
    kmap = sg.kmap;
    Kp = sg.kp;
    col_base = sg.col_base;
    col_end = sg.col_base + sg.valid;
    b_col_base = sg.b_col_base;
    Bk = sg.Bk;
    ldbk = sg.ldbk;
    bk_col0 = sg.col_local0;
  }
  // Bk: the listed rows of B already packed into a matrix of their own (row t of Bk = row kmap[t] of B);
  // only A is gathered then
  const bool b_packed = MAPPED && Bk != nullptr;
  // The row list of this tile is copied into LDS first: the staging loads then take their row numbers
  // from there instead of through a dependent global load ahead of every operand load.
  constexpr int kMapLds = 2048;
  __shared__ int kmap_s[MAPPED ? kMapLds : 1];
  const bool map_lds = MAPPED && kmap != nullptr && Kp <= kMapLds;  // uniform over the block
  if (map_lds) {
    for (int k = tid; k < Kp; k += NT) kmap_s[k] = kmap[k];
    __syncthreads();
  }

  // ---- global -> register staging ----------------------------------------------------------
  constexpr int A_VEC = TM * KT / 2;           // double2 elements in a W tile
  constexpr int A_PASS = (A_VEC + NT - 1) / NT;
  constexpr int B_VEC = TN * KT / 2;
  constexpr int B_PASS = (B_VEC + NT - 1) / NT;
  double2 ra[A_PASS], rb[B_PASS];
  // column of B behind each staged element (-1: none)
  int64_t bcol[B_PASS];
#pragma unroll
  for (int p = 0; p < B_PASS; ++p) {
    const int64_t jl = (tid + p * NT) / (KT / 2);
    const int64_t col = col_base + jl;
    bcol[p] = col < col_end ? ((MAPPED && colmap != nullptr) ? (int64_t)colmap[col] : b_col_base + jl) : -1;
  }

  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int p = 0; p < A_PASS; ++p) {
      int idx = tid + p * NT;
      int i2 = idx % (TM / 2);
      int k = idx / (TM / 2);
      int row = m0 + 2 * i2;
      double2 v = make_double2(0.0, 0.0);
      if (idx < A_VEC && row < Mp) {
        const int kk = (MAPPED && kmap != nullptr) ? (map_lds ? kmap_s[k0 + k] : kmap[k0 + k]) : k0 + k;
        if (kk >= 0) v = *reinterpret_cast<const double2*>(A + row + (int64_t)kk * lda);
      }
      ra[p] = v;
    }
#pragma unroll
    for (int p = 0; p < B_PASS; ++p) {
      int idx = tid + p * NT;
      int k2 = idx % (KT / 2);
      int j = idx / (KT / 2);
      double2 v = make_double2(0.0, 0.0);
      if (idx < B_VEC && bcol[p] >= 0) {
        if (b_packed) {
          v = *reinterpret_cast<const double2*>(Bk + (k0 + 2 * k2) + (bk_col0 + j) * ldbk);
        } else if (MAPPED && kmap != nullptr) {
          const int ka = map_lds ? kmap_s[k0 + 2 * k2] : kmap[k0 + 2 * k2];
          const int kb = map_lds ? kmap_s[k0 + 2 * k2 + 1] : kmap[k0 + 2 * k2 + 1];
          if (ka >= 0) v.x = B[ka + bcol[p] * ldb];
          if (kb >= 0) v.y = B[kb + bcol[p] * ldb];
        } else {
          v = *reinterpret_cast<const double2*>(B + (k0 + 2 * k2) + bcol[p] * ldb);
        }
      }
      rb[p] = v;
    }
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int p = 0; p < A_PASS; ++p) {
      int idx = tid + p * NT;
      int i2 = idx % (TM / 2);
      int k = idx / (TM / 2);
      if (idx < A_VEC) *reinterpret_cast<double2*>(&Ws[buf][k * LDA_S + 2 * i2]) = ra[p];
    }
#pragma unroll
    for (int p = 0; p < B_PASS; ++p) {
      int idx = tid + p * NT;
      int k2 = idx % (KT / 2);
      int j = idx / (KT / 2);
      if (idx < B_VEC) {  // odd column stride: two 64-bit stores
        Vs[buf][j * LDB_S + 2 * k2] = rb[p].x;
        Vs[buf][j * LDB_S + 2 * k2 + 1] = rb[p].y;
      }
    }
  };

  double4_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};

  // split-K: block row blockIdx.y owns the K-tiles [kt0, kt1) and writes a partial product
  const int nk_all = Kp / KT;
  const int kt0 = (int)((int64_t)nk_all * blockIdx.y / ksplit);
  const int kt1 = (int)((int64_t)nk_all * (blockIdx.y + 1) / ksplit);
  // two LDS stages: tile t+1 travels global -> registers while tile t is multiplied, then goes to the
  // other stage; one barrier per K-tile.  (A three-stage variant with the barrier hidden behind the
  // first MFMA step measured no faster: the limit is the per-wave MFMA issue cadence, not the barrier.)
  const int nk = kt1 - kt0;
  load_tiles(kt0 * KT);
  store_tiles(0);
  __syncthreads();
  for (int t = 0; t < nk; ++t) {
    const int cur = t & 1;
    if (t + 1 < nk) load_tiles((kt0 + t + 1) * KT);
    mfma_tile_k16<FM, FN, KT>(&Ws[cur][wr * (TM / WR)], LDA_S, &Vs[cur][(wc * (TN / WC)) * LDB_S], LDB_S, lane, acc);
    if (t + 1 < nk) store_tiles(cur ^ 1);
    __syncthreads();
  }
  if (ksplit > 1) {  // partial sums go to the workspace (ld = Mp); bias is added by the reduction
    C = part + (int64_t)blockIdx.y * Mp * ncols;
    ldc = Mp;
    bias = nullptr;
  }

  const int lrow = lane & 15;
  const int lcol = lane >> 4;
  // ---- fused estimateRanges: partial sums of this column tile ----------------------------------
  // xmin1 = sum max(v,0)*plb, xmin2 = sum min(v,0)*pub, xmax1 = sum max(v,0)*pub, xmax2 = sum min(v,0)*plb
  // over the tile's generator columns (column 0, the centre, is skipped), per output row.
  if (rpart != nullptr) {
    double* red = &Ws[0][0];  // the K loop is over (last barrier passed): reuse the W stage
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
#pragma unroll
      for (int j = 0; j < FN; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int64_t col = rcol0 + wc * (TN / WC) + j * 16 + lcol + 4 * r;
          if (col >= 1 && col < rcol_end) {
            const double v = acc[i][j][r];
            const double pl = plb[col - 1], pu = pub[col - 1];
            const double p = fmax(v, 0.0), q = fmin(v, 0.0);
            s0 = fma(p, pl, s0);
            s1 = fma(q, pu, s1);
            s2 = fma(p, pu, s2);
            s3 = fma(q, pl, s3);
          }
        }
      }
      // the four lane groups (lcol) hold different columns of the same rows
      s0 += __shfl_xor(s0, 16);
      s1 += __shfl_xor(s1, 16);
      s2 += __shfl_xor(s2, 16);
      s3 += __shfl_xor(s3, 16);
      s0 += __shfl_xor(s0, 32);
      s1 += __shfl_xor(s1, 32);
      s2 += __shfl_xor(s2, 32);
      s3 += __shfl_xor(s3, 32);
      if (lcol == 0) {
        double* dst = red + ((wc * TM) + wr * (TM / WR) + i * 16 + lrow) * 4;
        dst[0] = s0;
        dst[1] = s1;
        dst[2] = s2;
        dst[3] = s3;
      }
    }
    __syncthreads();
    for (int t = tid; t < TM * 4; t += NT) {  // waves along the columns are combined in order
      const int row = t >> 2, q = t & 3;
      double s = 0.0;
#pragma unroll
      for (int w = 0; w < WC; ++w) s += red[(w * TM + row) * 4 + q];
      if (m0 + row < Mp) rpart[(rchunk * 4 + q) * ldc + m0 + row] = s;
    }
  }

  // ---- epilogue: bias on column 0, 128-byte line stores --------------------------------------
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    int row = m0 + wr * (TM / WR) + i * 16 + lrow;
    if (row >= Mp) continue;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int64_t col = n0 + wc * (TN / WC) + j * 16 + lcol + 4 * r;
        const int64_t ccol = col_base + (col - n0);
        if (ccol < col_end) {
          double v = acc[i][j][r];
          if (bias != nullptr && ccol == 0) v = v + bias[row];
          // (partial products of a split go to the workspace column by column; the reduction maps them)
          C[row + ((MAPPED && colmap != nullptr && ksplit == 1) ? (int64_t)colmap[ccol] : ccol) * ldc] = v;
        }
      }
    }
  }
}

// colmap (or null): column t of the partial products belongs at column colmap[t] of C.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const double* __restrict__ part, int ksplit, int Mp,
                                                             int64_t ncols, double* __restrict__ C, int64_t ldc,
                                                             const double* __restrict__ bias,
                                                             const int32_t* __restrict__ colmap) {
  const int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)Mp * ncols;
  if (t >= total) return;
  double s = 0.0;
  for (int k0 = 0; k0 < ksplit; k0 += 16) {  // sixteen loads in flight, added in split order
    double v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = k0 + u < ksplit ? part[(int64_t)(k0 + u) * total + t] : 0.0;
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (k0 + u < ksplit) s += v[u];
  }
  const int64_t col = t / Mp;
  const int row = (int)(t - col * Mp);
  if (bias != nullptr && col == 0) s = s + bias[row];
  C[row + (colmap != nullptr ? (int64_t)colmap[col] : col) * ldc] = s;
}

template <int TM, int TN, int WR, int WC, int KT>
static int launch_cfg(nnvhip_ctx* ctx, const double* A, int64_t lda, const double* B, int64_t ldb, double* C,
                      int64_t ldc, int64_t Mp, int64_t ncols, int64_t Kp, const double* bias, RangeFuse* fuse,
                      const GemmRows* rows, SplitKDefer* defer) {
  int64_t tiles_m = ceil_div(Mp, TM);
  int64_t tiles_n = ceil_div(ncols, TN);
  int64_t blocks = tiles_m * tiles_n;
  if (blocks >= (int64_t(1) << 28)) NNV_FAIL(NNVHIP_ERR_SHAPE, "matrix too large for one launch");
  // XCD grid xr x (8/xr): least HBM/fabric traffic (8/xr)*|W| + xr*|V| among the shapes whose
  // busiest XCD has (almost) the fewest tiles
  int64_t best_xr = 8, best_slots = 0;
  double best_cost = 0.0;
  for (int64_t xr = 1; xr <= 8; xr *= 2) {
    const int64_t slots = ceil_div(tiles_m, xr) * ceil_div(tiles_n, 8 / xr);
    const double traffic = (8.0 / xr) * (double)Mp * Kp + (double)xr * Kp * (double)ncols;
    // an XCD has 32 CUs: up to 32 tiles per XCD still run in one round, so small imbalances are free
    const int64_t eff_slots = slots < 128 ? ceil_div(slots, 32) * 32 : slots;
    const double cost = (double)eff_slots * (1.0 + 0.03 * traffic / ((double)Mp * Kp + (double)Kp * ncols) / 8.0);
    if (best_slots == 0 || cost < best_cost) {
      best_cost = cost;
      best_xr = xr;
      best_slots = slots;
    }
  }
  if (const int v = tune_knobs().gemm_xr) {
    best_xr = std::max(1, std::min(8, v));
    best_slots = ceil_div(tiles_m, best_xr) * ceil_div(tiles_n, 8 / best_xr);
  }
  const int64_t local_m = ceil_div(tiles_m, best_xr);
  const int64_t grid_x = 8 * best_slots;
  // Split-K when the output has too few tiles to occupy the chip: partial products into a workspace,
  // summed in split order by a second kernel (deterministic, no floating-point atomics).
  const int64_t nk = Kp / KT;
  int64_t ksplit = 1;
  if (blocks < 128 && nk >= 8) ksplit = std::min<int64_t>(std::min<int64_t>(16, nk / 4), ceil_div(512, blocks));
  if (const int v = tune_knobs().gemm_ksplit) ksplit = std::max<int64_t>(1, std::min<int64_t>(v, nk));
  // the split-K workspace is laid out for one plain column range: no segment tables (a column map is
  // applied by the reduction)
  if (rows != nullptr && rows->segs != nullptr) ksplit = 1;
  if (rows != nullptr && rows->colmap != nullptr && defer != nullptr) ksplit = 1;
  if (rows != nullptr && rows->segs != nullptr && rows->seg_cols != TN)
    NNV_FAIL(NNVHIP_ERR_ARG, "internal: segment table built for another tile width");
  BufRef ws;
  if (ksplit > 1) NNV_TRY(ctx->alloc(sizeof(double) * ksplit * Mp * ncols, &ws));
  double* rpart = nullptr;
  if (fuse != nullptr && ksplit == 1) {  // the epilogue sees final values: fuse the range sums
    NNV_TRY(ctx->alloc(sizeof(double) * 4 * ldc * (tiles_n + fuse->extra_chunks), &fuse->part));
    fuse->chunks = tiles_n;
    rpart = fuse->part->as<double>();
  }
  const bool timed = ctx->kernel_timing && TM >= 64;
  NNV_TRY(ctx->kernel_timer_begin(timed));
  if (rows != nullptr) {
    // The mapped 128 x 128 tile needs a few registers more than let two blocks share a CU.  With a short
    // contraction (few kept rows) the start and the end of a tile weigh as much as its K loop, and a
    // second resident block hides them: for launches of many such tiles the allocation is held to 128
    // registers (at the price of a few reloads per K-tile; measured: 12% quicker at K = 240 over
    // 57344 tiles, 8% slower over 460 tiles, where two rounds of one block per CU do as well).
    auto kern = gemm_f64_kernel<TM, TN, WR, WC, KT, true>;
    if (TM == 128 && TN == 128 && Kp <= 512 && blocks >= 2048) kern = gemm_f64_kernel<TM, TN, WR, WC, KT, true, (TM == 128 && TN == 128 ? 4 : 1)>;
    NNV_LAUNCH(ctx, timed, kern, dim3((unsigned)grid_x, (unsigned)ksplit),
                       dim3(64 * WR * WC), 0, A, lda, B, ldb, C, ldc, (int)Mp, ncols, (int)Kp, bias, (int)tiles_m,
                       (int)tiles_n, (int)best_xr, (int)local_m, (int)ksplit, ws ? ws->as<double>() : nullptr,
                       fuse ? fuse->plb : nullptr, fuse ? fuse->pub : nullptr, rpart, rows->kmap, rows->segs, rows->colmap,
                       rows->Bk, rows->ldbk);
  } else
    NNV_LAUNCH(ctx, timed, (gemm_f64_kernel<TM, TN, WR, WC, KT, false>), dim3((unsigned)grid_x, (unsigned)ksplit),
                       dim3(64 * WR * WC), 0, A, lda, B, ldb, C, ldc, (int)Mp, ncols, (int)Kp, bias, (int)tiles_m,
                       (int)tiles_n, (int)best_xr, (int)local_m, (int)ksplit, ws ? ws->as<double>() : nullptr,
                       fuse ? fuse->plb : nullptr, fuse ? fuse->pub : nullptr, rpart, nullptr, nullptr, nullptr, nullptr, 0);
  NNV_TRY(ctx->kernel_timer_end(timed, 0, rows && rows->flop > 0.0 ? rows->flop : 2.0 * (double)Mp * (double)Kp * (double)ncols));
  if (defer != nullptr) {
    defer->ws = ws;
    defer->ksplit = ksplit;
  } else if (ksplit > 1) {
    const int64_t total = Mp * ncols;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, ctx->stream,
                       ws->as<double>(), (int)ksplit, (int)Mp, ncols, C, ldc, bias, rows ? rows->colmap : nullptr);
  }
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

// Tile width of a segmented launch: 128 x 128 tiles when there are enough of them to cover the chip,
// 64 x 64 for small arrays (and the 16-row tile for skinny outputs).
int gemm_seg_cols(int64_t Mp, int64_t count, const int64_t* cols) {
  if (Mp <= 16) return 64;   // the 16 x 64 tile
  if (Mp <= 32) return 128;  // the 32 x 128 tile
  int64_t tiles = 0;
  for (int64_t i = 0; i < count; ++i) tiles += ceil_div(cols[i], 128);
  return tiles * ceil_div(Mp, 128) < 256 ? 64 : 128;
}

int launch_gemm(nnvhip_ctx* ctx, const double* A, int64_t lda, const double* B, int64_t ldb, double* C, int64_t ldc,
                int64_t Mp, int64_t ncols, int64_t Kp, const double* bias, RangeFuse* fuse, const GemmRows* rows,
                SplitKDefer* defer) {
  if (Mp % 16 || Kp % 16 || lda % 2 || ldb % 2 || Mp > lda || Kp > ldb || Mp > ldc)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: GEMM operands violate the padding contract");
  if (Mp >= (int64_t(1) << 31) || Kp >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "matrix too large");
  if (ncols == 0) return NNVHIP_OK;
  // Tile choice: the largest tile that still yields a few blocks per CU; skinny outputs (the last
  // layer has 10 rows) get a 16-row tile.  K must be a multiple of the K-tile (16 or 32).
#define NNV_GEMM(TM, TN, WR, WC, KT) \
  launch_cfg<TM, TN, WR, WC, KT>(ctx, A, lda, B, ldb, C, ldc, Mp, ncols, Kp, bias, fuse, rows, defer)
  const int64_t kCUs = 256;
  if (Mp <= 16) return NNV_GEMM(16, 64, 1, 4, 16);
  if (Mp <= 32) return NNV_GEMM(32, 128, 1, 4, 16);
  // Eight-wave tiles (two waves per SIMD issue MFMAs even with one block per CU).  The shape is
  // fitted to the problem: all tiles of a launch are resident at once and share the MFMA pipes, so
  // the time goes with ceil(tiles / CUs) * tile area / (measured rate of the shape).  Small outputs
  // thus get the shape that covers the chip in one round (e.g. 128x80 for 1024 x 2376: 240 tiles).
  struct Shape {
    int tm, tn;
    double rate;  // TFLOP/s measured on a 1024 x 1024 x 16384 product
  };
  static const Shape shapes[] = {{64, 64, 47.0},  {64, 96, 47.8},   {64, 128, 49.6},  {128, 48, 46.8},
                                 {128, 64, 49.9}, {128, 80, 48.0},  {128, 96, 47.3},  {128, 112, 47.6},
                                 {128, 128, 54.0}};
  int best = 0;
  double best_cost = 0.0;
  for (int i = 0; i < (int)(sizeof(shapes) / sizeof(shapes[0])); ++i) {
    const int64_t tiles = ceil_div(Mp, shapes[i].tm) * ceil_div(ncols, shapes[i].tn);
    const double cost = (double)ceil_div(tiles, kCUs) * shapes[i].tm * shapes[i].tn / shapes[i].rate;
    if (i == 0 || cost < best_cost * 0.999) {
      best = i;
      best_cost = cost;
    }
  }
  if (rows != nullptr && rows->segs != nullptr)  // the table was cut for this width: see gemm_seg_cols
    return rows->seg_cols == 64 ? NNV_GEMM(64, 64, 2, 4, 16) : NNV_GEMM(128, 128, 2, 4, 16);
  if (rows != nullptr && rows->tile_hint == 64 && tune_knobs().gemm_tile.empty()) return NNV_GEMM(64, 64, 2, 4, 16);
  if (!tune_knobs().gemm_tile.empty()) {  // tuning knob: "TMxTN" of one of the shapes above
    for (int i = 0; i < (int)(sizeof(shapes) / sizeof(shapes[0])); ++i)
      if (std::to_string(shapes[i].tm) + "x" + std::to_string(shapes[i].tn) == tune_knobs().gemm_tile) best = i;
  }
  switch (shapes[best].tm * 1000 + shapes[best].tn) {
    case 64064: return NNV_GEMM(64, 64, 2, 4, 16);
    case 64096: return NNV_GEMM(64, 96, 4, 2, 16);
    case 64128: return NNV_GEMM(64, 128, 4, 2, 16);
    case 128048: return NNV_GEMM(128, 48, 8, 1, 16);
    case 128064: return NNV_GEMM(128, 64, 4, 2, 16);
    case 128080: return NNV_GEMM(128, 80, 8, 1, 16);
    case 128096: return NNV_GEMM(128, 96, 8, 1, 16);
    case 128112: return NNV_GEMM(128, 112, 8, 1, 16);
    default: return NNV_GEMM(128, 128, 2, 4, 16);
  }
#undef NNV_GEMM
}

// Packs the listed rows of every set's leading columns: Vk(t, j) = V(kept[t], j), zero where kept[t] < 0.
// Lane = two packed rows, the waves of a block interleave columns.  Grid: (row blocks of 128, column
// chunks, sets).
__global__ __launch_bounds__(512) void pack_rows_kernel(const PackSet* __restrict__ table, PackSet one, int cols_per_chunk) {
  const PackSet d = table ? table[blockIdx.z] : one;
  const int j0 = blockIdx.y * cols_per_chunk;
  if (j0 >= d.ncols) return;
  const int j1 = min(d.ncols, j0 + cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int t0 = blockIdx.x * 128 + 2 * lane;
  if (t0 >= d.kp) return;
  const int ra = d.kept[t0], rb = d.kept[t0 + 1];
  // image positions of the two rows, for columns that are only defined inside their windows
  int ha = 0, wa = 0, hb = 0, wb = 0;
  if (d.box != nullptr) {
    const int P = d.bH * d.bW;
    const int pa = max(ra, 0) % P, pb = max(rb, 0) % P;
    wa = pa / d.bH, ha = pa - wa * d.bH;
    wb = pb / d.bH, hb = pb - wb * d.bH;
  }
  for (int jb = j0 + 4 * wave; jb < j1; jb += 32) {
    double2 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      v[u] = make_double2(0.0, 0.0);
      const int j = jb + u;
      if (j < j1 && !(j >= 1 && j < d.zero_to)) {
        if (d.W != nullptr && j >= d.wfrom && j < d.wend) {  // the value the gather pass wrote, recomputed
          const int src = d.widx[j - d.wfrom];
          const double sc = d.wscale ? d.wscale[src] : 1.0;
          const double* col = d.W + (int64_t)src * d.ldw;
          if (ra >= 0) v[u].x = __dadd_rn(0.0, __dmul_rn(col[ra], sc));
          if (rb >= 0) v[u].y = __dadd_rn(0.0, __dmul_rn(col[rb], sc));
        } else {
          const double* col = d.V + (int64_t)j * d.ld;
          bool ina = ra >= 0, inb = rb >= 0;
          if (d.box != nullptr && j >= d.box_from && j < d.box_to) {
            const ColBox b = d.box[j];
            ina = ina && ha >= b.h0 && ha <= b.h1 && wa >= b.w0 && wa <= b.w1;
            inb = inb && hb >= b.h0 && hb <= b.h1 && wb >= b.w0 && wb <= b.w1;
          }
          if (ina) v[u].x = col[ra];
          if (inb) v[u].y = col[rb];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (jb + u < j1) *reinterpret_cast<double2*>(d.Vk + t0 + (int64_t)(jb + u) * d.kp) = v[u];
  }
}

PackSet pack_of(const nnvhip_star* s, const int32_t* kept, double* dst, int64_t kp, int64_t ncols) {
  PackSet p{s->V, kept, dst, s->ld, (int32_t)kp, (int32_t)ncols};
  const ColSource& cs = s->cs;
  if (cs.W != nullptr && cs.from < ncols) {
    p.W = cs.W;
    p.ldw = cs.ldw;
    p.Wt = cs.Wt;
    p.ldwt = cs.ldwt;
    p.wrows = cs.rows;
    p.widx = cs.idx;
    p.wscale = cs.scale;
    p.wfrom = (int32_t)cs.from;
    p.wend = (int32_t)std::min<int64_t>(ncols, cs.from + cs.cols);
  }
  p.zero_to = (int32_t)std::min<int64_t>(ncols, cs.zero_to);
  if (cs.win_pending() && cs.win_from < ncols) {
    p.box = cs.win_box;
    p.box_from = (int32_t)cs.win_from;
    p.box_to = (int32_t)std::min<int64_t>(ncols, cs.win_to);
    p.bH = cs.win_H;
    p.bW = cs.win_W;
  }
  return p;
}

int launch_pack_rows(nnvhip_ctx* ctx, int64_t count, const PackSet* sets) {
  if (count <= 0) return NNVHIP_OK;
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  int64_t max_kp = 0, max_cols = 0;
  for (int64_t i = 0; i < count; ++i) {
    max_kp = std::max<int64_t>(max_kp, sets[i].kp);
    max_cols = std::max<int64_t>(max_cols, sets[i].ncols);
  }
  if (max_kp == 0 || max_cols == 0) return NNVHIP_OK;
  const int64_t row_blocks = ceil_div(max_kp, 128);
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(8192, row_blocks * count), ceil_div(max_cols, 32)));
  const int64_t cpc = ceil_div(max_cols, chunks);
  chunks = ceil_div(max_cols, cpc);
  const PackSet* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(ctx->upload_table(sets, sizeof(PackSet) * count, &tab));
    table = tab->as<PackSet>();
  }
  hipLaunchKernelGGL(pack_rows_kernel, dim3((unsigned)row_blocks, (unsigned)chunks, (unsigned)count), dim3(512), 0, ctx->stream,
                     table, sets[0], (int)cpc);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

__global__ void bias_columns_kernel(double* const* __restrict__ cols, const double* __restrict__ bias, int Mp) {
  double* col = cols[blockIdx.y];
  int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < Mp) col[r] = col[r] + bias[r];
}

int launch_bias_columns(nnvhip_ctx* ctx, double* const* centre_cols_dev, int64_t count, const double* bias,
                        int64_t Mp) {
  if (count <= 0) return NNVHIP_OK;
  for (int64_t off = 0; off < count; off += 65535) {
    int64_t n = std::min<int64_t>(65535, count - off);
    hipLaunchKernelGGL(bias_columns_kernel, dim3((unsigned)ceil_div(Mp, 256), (unsigned)n), dim3(256), 0, ctx->stream,
                       centre_cols_dev + off, bias, (int)Mp);
  }
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

}  // namespace nnvhip
