// fp64 MFMA tile core shared by the fully connected GEMM and the implicit-GEMM convolution.
#pragma once
#include <hip/hip_runtime.h>

namespace nnvhip {

typedef double double4_t __attribute__((ext_vector_type(4)));

constexpr int kKt = 16;      // K-tile of the convolution kernel
// LDS has 32 four-byte banks; a 64-bit read is served 16 lanes per cycle, so a read is conflict free
// when each group of 16 consecutive lanes touches 16 distinct bank pairs.
constexpr int kPadRow = 0;  // [k][row] array: a lane group reads 16 consecutive doubles - always distinct
constexpr int kPadK = 1;    // [col][k] array: odd column stride -> 16 columns hit 16 distinct bank pairs

// One K-tile (KT deep = KT/4 16x16x4 MFMA steps) of a (16*FM) x (16*FN) wave tile.
//   rows_s: LDS, element (k, row) at rows_s[k * ld_rows + row]   -> MFMA operand "b"
//   cols_s: LDS, element (col, k) at cols_s[col * ld_cols + k]   -> MFMA operand "a"
// v_mfma_f64_16x16x4_f64 operand layout on gfx950 (measured): lane l supplies a[i = l%16][k = l/16]
// and b[k = l/16][j = l%16]; result register r of lane l is D[i = l/16 + 4r][j = l%16].
template <int FM, int FN, int KT = kKt>
__device__ __forceinline__ void mfma_tile_k16(const double* __restrict__ rows_s, int ld_rows,
                                              const double* __restrict__ cols_s, int ld_cols, int lane,
                                              double4_t (&acc)[FM][FN]) {
  const int l16 = lane & 15;
  const int kq = lane >> 4;
#pragma unroll
  for (int kk = 0; kk < KT / 4; ++kk) {
    const int k = kk * 4 + kq;
    double b[FM], a[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) b[i] = rows_s[k * ld_rows + i * 16 + l16];
#pragma unroll
    for (int j = 0; j < FN; ++j) a[j] = cols_s[(j * 16 + l16) * ld_cols + k];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[j], b[i], acc[i][j], 0, 0, 0);
  }
}

}  // namespace nnvhip
