// affineMap of a fully connected layer: C = W * [c V] on fp64 MFMA (v_mfma_f64_16x16x4_f64).
//
// Both operands are staged through LDS in K-tiles of 16.  The MFMA operand roles are chosen for
// column-major stores: the instruction's "b" operand carries 16 consecutive ROWS of W (the
// memory-contiguous direction of C), its "a" operand 16 columns of V, so lane l, register r of
// an accumulator holds C[row0 + l%16][col0 + l/16 + 4r] and lanes 0..15 store one 128-byte line.
#include "internal.h"
#include "mfma_tile.h"

namespace nnvhip {

// TM x TN output tile per 256-thread block, waves arranged WR x WC, each wave owning
// (TM/WR) x (TN/WC) = (16*FM) x (16*FN).
template <int TM, int TN, int WR, int WC>
__global__ __launch_bounds__(256) void gemm_f64_kernel(const double* __restrict__ A, int64_t lda,
                                                        const double* __restrict__ B, int64_t ldb,
                                                        double* __restrict__ C, int64_t ldc, int Mp, int64_t ncols,
                                                        int Kp, const double* __restrict__ bias, int tiles_m) {
  static_assert(WR * WC == 4, "four waves per block");
  constexpr int FM = TM / WR / 16;
  constexpr int FN = TN / WC / 16;
  constexpr int LDA_S = TM + kPadRow;  // Ws[k][row]
  constexpr int LDB_S = kKt + kPadK;   // Vs[col][k]
  __shared__ double Ws[2][kKt * LDA_S];
  __shared__ double Vs[2][TN * LDB_S];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wr = wave % WR;
  const int wc = wave / WR;
  // consecutive blocks walk down the rows of one column band, so the band's V tile stays hot
  const int64_t bid = blockIdx.x;
  const int m0 = (int)(bid % tiles_m) * TM;
  const int64_t n0 = (bid / tiles_m) * TN;

  // ---- global -> register staging ----------------------------------------------------------
  constexpr int A_VEC = TM * kKt / 2;          // double2 elements in a W tile
  constexpr int A_PASS = (A_VEC + 255) / 256;
  constexpr int B_VEC = TN * kKt / 2;
  constexpr int B_PASS = (B_VEC + 255) / 256;
  double2 ra[A_PASS], rb[B_PASS];

  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int p = 0; p < A_PASS; ++p) {
      int idx = tid + p * 256;
      int i2 = idx % (TM / 2);
      int k = idx / (TM / 2);
      int row = m0 + 2 * i2;
      double2 v = make_double2(0.0, 0.0);
      if (idx < A_VEC && row < Mp) v = *reinterpret_cast<const double2*>(A + row + (int64_t)(k0 + k) * lda);
      ra[p] = v;
    }
#pragma unroll
    for (int p = 0; p < B_PASS; ++p) {
      int idx = tid + p * 256;
      int k2 = idx % (kKt / 2);
      int j = idx / (kKt / 2);
      int64_t col = n0 + j;
      double2 v = make_double2(0.0, 0.0);
      if (idx < B_VEC && col < ncols) v = *reinterpret_cast<const double2*>(B + (k0 + 2 * k2) + col * ldb);
      rb[p] = v;
    }
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int p = 0; p < A_PASS; ++p) {
      int idx = tid + p * 256;
      int i2 = idx % (TM / 2);
      int k = idx / (TM / 2);
      if (idx < A_VEC) *reinterpret_cast<double2*>(&Ws[buf][k * LDA_S + 2 * i2]) = ra[p];
    }
#pragma unroll
    for (int p = 0; p < B_PASS; ++p) {
      int idx = tid + p * 256;
      int k2 = idx % (kKt / 2);
      int j = idx / (kKt / 2);
      if (idx < B_VEC) *reinterpret_cast<double2*>(&Vs[buf][j * LDB_S + 2 * k2]) = rb[p];
    }
  };

  double4_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};

  const int nk = Kp / kKt;
  load_tiles(0);
  store_tiles(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) load_tiles((kt + 1) * kKt);
    mfma_tile_k16<FM, FN>(&Ws[cur][wr * (TM / WR)], LDA_S, &Vs[cur][(wc * (TN / WC)) * LDB_S], LDB_S, lane, acc);
    if (kt + 1 < nk) store_tiles(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue: bias on column 0, 128-byte line stores --------------------------------------
  const int lrow = lane & 15;
  const int lcol = lane >> 4;
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    int row = m0 + wr * (TM / WR) + i * 16 + lrow;
    if (row >= Mp) continue;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int64_t col = n0 + wc * (TN / WC) + j * 16 + lcol + 4 * r;
        if (col < ncols) {
          double v = acc[i][j][r];
          if (bias != nullptr && col == 0) v = v + bias[row];
          C[row + col * ldc] = v;
        }
      }
    }
  }
}

template <int TM, int TN, int WR, int WC>
static int launch_cfg(nnvhip_ctx* ctx, const double* A, int64_t lda, const double* B, int64_t ldb, double* C,
                      int64_t ldc, int64_t Mp, int64_t ncols, int64_t Kp, const double* bias) {
  int64_t tiles_m = ceil_div(Mp, TM);
  int64_t tiles_n = ceil_div(ncols, TN);
  int64_t blocks = tiles_m * tiles_n;
  if (blocks >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "matrix too large for one launch");
  hipLaunchKernelGGL((gemm_f64_kernel<TM, TN, WR, WC>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, A, lda, B,
                     ldb, C, ldc, (int)Mp, ncols, (int)Kp, bias, (int)tiles_m);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

int launch_gemm(nnvhip_ctx* ctx, const double* A, int64_t lda, const double* B, int64_t ldb, double* C, int64_t ldc,
                int64_t Mp, int64_t ncols, int64_t Kp, const double* bias) {
  if (Mp % 16 || Kp % 16 || lda % 2 || ldb % 2 || Mp > lda || Kp > ldb || Mp > ldc)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: GEMM operands violate the padding contract");
  if (Mp >= (int64_t(1) << 31) || Kp >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "matrix too large");
  if (ncols == 0) return NNVHIP_OK;
  // Tile choice: the largest tile that still yields a few blocks per CU; skinny outputs (the last
  // layer has 10 rows) get a 16-row tile.
  const int64_t kCUs = 256;
  if (Mp <= 16) return launch_cfg<16, 256, 1, 4>(ctx, A, lda, B, ldb, C, ldc, Mp, ncols, Kp, bias);
  if (Mp <= 32) return launch_cfg<32, 128, 1, 4>(ctx, A, lda, B, ldb, C, ldc, Mp, ncols, Kp, bias);
  int64_t b128 = ceil_div(Mp, 128) * ceil_div(ncols, 128);
  if (b128 >= 3 * kCUs) return launch_cfg<128, 128, 2, 2>(ctx, A, lda, B, ldb, C, ldc, Mp, ncols, Kp, bias);
  int64_t b64 = ceil_div(Mp, 64) * ceil_div(ncols, 64);
  if (b64 >= 2 * kCUs || Mp % 64 == 0 || Mp > 256)
    return launch_cfg<64, 64, 2, 2>(ctx, A, lda, B, ldb, C, ldc, Mp, ncols, Kp, bias);
  return launch_cfg<32, 128, 1, 4>(ctx, A, lda, B, ldb, C, ldc, Mp, ncols, Kp, bias);
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
