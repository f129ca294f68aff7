// affineMap of a Conv2DLayer on an ImageStar (nn/layers/Conv2DLayer.m:559-601): the same
// cross-correlation applied to the centre image (plus bias) and to every generator image.
//
// Implicit GEMM on fp64 MFMA.  With P = Ho*Wo output positions per image and G = n+1 images the
// output, in MATLAB's H x W x C x (n+1) layout, is a (P*G) x Cout matrix whose rows are contiguous in
// memory per (channel, image); the reduction runs over the K = FH*FW*Cin filter taps, which is
// exactly the row order of MATLAB's FH x FW x Cin x Cout weight array.  The im2col operand is never
// materialised: each block gathers its 128-position x 16-tap tile straight from the input images
// (zero for padding taps) into LDS; the weight tile is loaded like the generator tile of the dense
// GEMM.  MFMA operand "b" carries positions (the memory-contiguous direction of the output), "a"
// carries output channels.
#include <algorithm>
#include <cstring>
#include <type_traits>

#include "internal.h"
#include "lds_dma.h"
#include "mfma_tile.h"
#include "relu_sort.h"

namespace nnvhip {

struct ConvGeom {
  int H, W, Cin, Ho, Wo, Cout;
  int FH, FW, sh, sw, dh, dw, pt, pl;
  int K, Kp;
  int P;   // Ho * Wo
  int HW;  // H * W
};

constexpr int kMaxTaps = 4096;  // tap table held in LDS: 8 bytes per (padded) tap
constexpr size_t kConvLdsLimit = 64 * 1024;  // LDS of one block: operand tiles + tap table + row mask

// Tap k = fh + FH*(fw + FW*ci) -> packed (input offset ci*H*W : 32 | fh*dh : 16 | fw*dw : 16).
__device__ __forceinline__ unsigned long long pack_tap(const ConvGeom& g, int k) {
  if (k >= g.K) return ~0ull;  // padded tap: never valid
  const int fh = k % g.FH;
  const int t = k / g.FH;
  const int fw = t % g.FW;
  const int ci = t / g.FW;
  return ((unsigned long long)(unsigned)(ci * g.HW) << 32) | ((unsigned long long)(fh * g.dh) << 16) |
         (unsigned long long)(fw * g.dw);
}

// How the rows of the implicit GEMM map to (image, output position).  box == null: row R is position R % P of
// image R / P.  Otherwise rows [0, P) are the centre image and every further image owns `area` = eh x ew rows,
// the positions of its window's corner onwards (row t of the slot: ho = h0 + t % eh, wo = w0 + t / eh; slots of
// positions outside the window are idle): a generator image is computed inside its window only.
struct ConvRows {
  const ColBox* box;
  int eh, area;
  const ColBox* in_box;  // windows of the input images, or null: a tap outside its image's window is not read
};

template <bool COMPACT>
__device__ __forceinline__ bool conv_row(const ConvGeom& g, const ConvRows& cr, int64_t R, int64_t total_rows, int64_t* gi,
                                         int* ho, int* wo) {
  if (R >= total_rows) return false;
  if (!COMPACT || R < g.P) {
    const int64_t im = COMPACT ? 0 : R / g.P;
    const int p = (int)(R - im * g.P);
    *gi = im;
    *wo = p / g.Ho;
    *ho = p - *wo * g.Ho;
    return true;
  }
  const int64_t q = R - g.P;
  const int64_t im = q / cr.area;
  const int t = (int)(q - im * cr.area);
  const ColBox bb = cr.box[1 + im];
  *gi = 1 + im;
  const int tw = t / cr.eh;
  *ho = bb.h0 + (t - tw * cr.eh);
  *wo = bb.w0 + tw;
  return *ho <= bb.h1 && *wo <= bb.w1;
}

template <bool COMPACT>
__device__ __forceinline__ int64_t conv_first_image(const ConvGeom& g, const ConvRows& cr, int64_t R0) {
  if (!COMPACT) return R0 / g.P;
  return R0 < g.P ? 0 : 1 + (R0 - g.P) / cr.area;
}

// Stores a block's accumulators: lane l, register r of acc[i][j] holds out[row R0 + ... + l%16][channel c0 +
// ... + l/16 + 4r]; the bias goes onto the centre image only.
template <int TP, int TC, int WR, int WC, int FM, int FN, bool COMPACT = false>
__device__ __forceinline__ void conv_store_tile(const double4_t (&acc)[FM][FN], double* __restrict__ out, int64_t ldout,
                                                const double* __restrict__ bias, const ConvGeom& g, int64_t total_rows,
                                                int64_t R0, int c0, int wr, int wc, int lane,
                                                const ConvRows cr = ConvRows{nullptr, 0, 0, nullptr}) {
  const int lrow = lane & 15;
  const int lcol = lane >> 4;
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int64_t Rr = R0 + wr * (TP / WR) + i * 16 + lrow;
    int64_t gi;
    int ho, wo;
    if (!conv_row<COMPACT>(g, cr, Rr, total_rows, &gi, &ho, &wo)) continue;
    const int p = ho + wo * g.Ho;
    double* o = out + gi * ldout + p;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int co = c0 + wc * (TC / WC) + j * 16 + lcol + 4 * r;
        if (co < g.Cout) {
          double v = acc[i][j][r];
          if (bias != nullptr && gi == 0) v = v + bias[co];  // centre image only
          o[(int64_t)co * g.P] = v;
        }
      }
    }
  }
}

// MASK: the input is the matrix in front of a ReLU step whose row reset has not been run; `keep` holds one
// bit per input row (1 = the row is kept, 0 = it reads as zero: PosLin.m:700-709, Star.m:1442-1461), copied
// into LDS behind the tap table.  A reset row is never loaded.
template <int TP, int TC, int WR, int WC, bool MASK>
__global__ __launch_bounds__(64 * WR * WC) void conv2d_f64_kernel(const double* __restrict__ in, int64_t ldin,
                                                          double* __restrict__ out, int64_t ldout,
                                                          const double* __restrict__ Wt,
                                                          const double* __restrict__ bias, ConvGeom g,
                                                          int64_t total_rows, int tiles_c,
                                                          const uint32_t* __restrict__ keep, int keep_words) {
  constexpr int NT = 64 * WR * WC;  // threads per block
  static_assert(NT % TP == 0 && (TP * kKt) % NT == 0, "gather mapping needs NT = TP * (taps per pass)");
  constexpr int FM = TP / WR / 16;
  constexpr int FN = TC / WC / 16;
  constexpr int LDP_S = TP + kPadRow;  // Ps[k][position]
  constexpr int LDW_S = kKt + kPadK;   // Wts[cout][k]
  __shared__ double Ps[2][kKt * LDP_S];
  __shared__ double Wts[2][TC * LDW_S];
  extern __shared__ unsigned long long taps[];  // Kp entries

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wr = wave % WR;
  const int wc = wave / WR;
  const int64_t bid = blockIdx.x;
  const int c0 = (int)(bid % tiles_c) * TC;
  const int64_t R0 = (bid / tiles_c) * TP;

  for (int k = tid; k < g.Kp; k += NT) taps[k] = pack_tap(g, k);
  uint32_t* keep_s = reinterpret_cast<uint32_t*>(taps + g.Kp);
  if (MASK)
    for (int k = tid; k < keep_words; k += NT) keep_s[k] = keep[k];

  // this thread's gather position (fixed for the whole K loop)
  constexpr int P_PASS = TP * kKt / NT;  // gathered elements per thread per K-tile
  constexpr int K_STEP = NT / TP;        // taps covered by one pass
  const int p_local = tid % TP;
  const int k_first = tid / TP;
  const int64_t R = R0 + p_local;
  const bool rvalid = R < total_rows;
  int h0 = 0, w0 = 0;
  const double* img = in;
  if (rvalid) {
    const int64_t gi = R / g.P;
    const int p = (int)(R - gi * g.P);
    const int wo = p / g.Ho;
    const int ho = p - wo * g.Ho;
    h0 = ho * g.sh - g.pt;
    w0 = wo * g.sw - g.pl;
    img = in + gi * ldin;
  }

  constexpr int W_VEC = TC * kKt / 2;
  constexpr int W_PASS = (W_VEC + NT - 1) / NT;
  double rp[P_PASS];
  double2 rw[W_PASS];

  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int q = 0; q < P_PASS; ++q) {
      const unsigned long long t = taps[k0 + k_first + q * K_STEP];
      const int h = h0 + (int)((t >> 16) & 0xffffu);
      const int w = w0 + (int)(t & 0xffffu);
      bool ok = rvalid && t != ~0ull && (unsigned)h < (unsigned)g.H && (unsigned)w < (unsigned)g.W;
      const int row = ok ? (int)(unsigned)(t >> 32) + h + w * g.H : 0;  // row of the input set (< 2^31)
      if (MASK) ok = ok && ((keep_s[row >> 5] >> (row & 31)) & 1u) != 0;
      rp[q] = ok ? img[row] : 0.0;
    }
#pragma unroll
    for (int q = 0; q < W_PASS; ++q) {
      const int idx = tid + q * NT;
      const int k2 = idx % (kKt / 2);
      const int j = idx / (kKt / 2);
      double2 v = make_double2(0.0, 0.0);
      if (idx < W_VEC && c0 + j < g.Cout) v = *reinterpret_cast<const double2*>(Wt + (k0 + 2 * k2) + (int64_t)(c0 + j) * g.Kp);
      rw[q] = v;
    }
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int q = 0; q < P_PASS; ++q) Ps[buf][(k_first + q * K_STEP) * LDP_S + p_local] = rp[q];
#pragma unroll
    for (int q = 0; q < W_PASS; ++q) {
      const int idx = tid + q * NT;
      const int k2 = idx % (kKt / 2);
      const int j = idx / (kKt / 2);
      if (idx < W_VEC) {  // odd column stride: two 64-bit stores
        Wts[buf][j * LDW_S + 2 * k2] = rw[q].x;
        Wts[buf][j * LDW_S + 2 * k2 + 1] = rw[q].y;
      }
    }
  };

  double4_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};

  __syncthreads();  // tap table ready
  const int nk = g.Kp / kKt;
  load_tiles(0);
  store_tiles(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) load_tiles((kt + 1) * kKt);
    mfma_tile_k16<FM, FN>(&Ps[cur][wr * (TP / WR)], LDP_S, &Wts[cur][(wc * (TC / WC)) * LDW_S], LDW_S, lane, acc);
    if (kt + 1 < nk) store_tiles(cur ^ 1);
    __syncthreads();
  }

  conv_store_tile<TP, TC, WR, WC, FM, FN>(acc, out, ldout, bias, g, total_rows, R0, c0, wr, wc, lane);
}

// ---- the same convolution with little vector-ALU work per MFMA ------------------------------------
// On this chip the vector ALU does not issue in the shadow of an fp64 MFMA (measured: every extra VALU
// instruction of a wave costs about as many matrix-pipe cycles as it takes to issue), so the gather of the
// kernel above - tap decode, bounds checks, a 32-bit multiply and 64-bit address arithmetic per element -
// costs a third of the MFMA time.  Here a tap is a wave-uniform (row offset, spatial bit) pair read through
// the scalar unit from a table in global memory, a thread's padding pattern is one 32-bit mask computed once
// (bit fh + FH*fw: that tap falls inside the image), the element's row is one addition, and its address a
// 32-bit offset from a block-uniform base.  The weight tile comes k-major from a second copy of the weights
// straight into LDS (global_load_lds_dwordx4), with no registers or address arithmetic in between.
// Needs FH*FW <= 32 and a tile's images within 2 GiB of its first one; the host checks both.
struct FastTap {
  int32_t off;   // ci*H*W + fh*dh + fw*dw*H: row of the tap relative to the row of tap (0, 0, 0)
  uint32_t bit;  // 1 << (fh + FH*fw); 0 for a padding entry
};

__global__ void conv_fast_taps_kernel(FastTap* __restrict__ tab, ConvGeom g) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  if (k >= g.Kp) return;
  FastTap t{0, 0u};
  if (k < g.K) {
    const int fh = k % g.FH;
    const int r = k / g.FH;
    const int fw = r % g.FW;
    const int ci = r / g.FW;
    t.off = ci * g.HW + fh * g.dh + fw * g.dw * g.H;
    t.bit = 1u << (fh + g.FH * fw);
  }
  tab[k] = t;
}

// Wk(k, co) = W(k, co) for co < Cout, zero up to coutp: the weights k-major (row k contiguous over channels)
__global__ void conv_weights_kmajor_kernel(const double* __restrict__ W, double* __restrict__ Wk, int Kp, int Cout, int coutp) {
  const int64_t idx = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (idx >= (int64_t)Kp * coutp) return;
  const int k = (int)(idx / coutp), co = (int)(idx % coutp);
  Wk[idx] = co < Cout ? W[k + (int64_t)co * Kp] : 0.0;
}

struct ConvFastArgs {
  const double* in;
  int64_t ldin;
  double* out;
  int64_t ldout;
  const double* Wk;
  int coutp;
  const double* bias;
  ConvGeom g;
  int64_t total_rows;
  int tiles_c;
  const FastTap* taps;
  const uint32_t* keep;
  int keep_words;
  ConvRows cr;
};

// LDS of a block of the kernel below: the weight tiles [2][k][channel] first (their transfers want 1 KiB alignment),
// then the position tiles [2][k][position]; the row mask (MASK only) sits in the dynamic part behind them.
constexpr size_t conv_fast_lds_bytes(int tc) { return sizeof(double) * 2 * kKt * (128 + (size_t)tc); }

template <int TC, int WR, int WC, bool MASK, bool COMPACT>
__device__ __forceinline__ void conv2d_fast_block(const ConvFastArgs& a, int64_t bid, double* __restrict__ lds, uint32_t* keep_s) {
  constexpr int TP = 128, NT = 512;
  static_assert(WR * WC == 8, "eight waves");
  constexpr int FM = TP / WR / 16;
  constexpr int FN = TC / WC / 16;
  constexpr int kWLoads = kKt * TC / 128;  // 1 KiB wave transfers per K-tile of weights
  constexpr int kRowsPerLoad = 128 / TC;   // rows of Wk per transfer
  double(*Wts)[kKt * TC] = reinterpret_cast<double(*)[kKt * TC]>(lds);                // [k][channel]
  double(*Ps)[kKt * TP] = reinterpret_cast<double(*)[kKt * TP]>(lds + 2 * kKt * TC);  // [k][position]
  const double* __restrict__ in = a.in;
  const int64_t ldin = a.ldin;
  double* __restrict__ out = a.out;
  const int64_t ldout = a.ldout;
  const double* __restrict__ Wk = a.Wk;
  const int coutp = a.coutp;
  const double* __restrict__ bias = a.bias;
  const ConvGeom& g = a.g;
  const int64_t total_rows = a.total_rows;
  const int tiles_c = a.tiles_c;
  const FastTap* __restrict__ taps = a.taps;
  const uint32_t* __restrict__ keep = a.keep;
  const int keep_words = a.keep_words;
  const ConvRows& cr = a.cr;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave % WR;
  const int wc = wave / WR;
  const int c0 = (int)(bid % tiles_c) * TC;
  const int64_t R0 = (bid / tiles_c) * TP;

  if (MASK)
    for (int k = tid; k < keep_words; k += NT) keep_s[k] = keep[k];

  // this thread's position (fixed for the whole K loop) and the four consecutive taps of a K-tile it gathers
  const int p_local = tid & (TP - 1);
  const int kq = __builtin_amdgcn_readfirstlane(tid >> 7);
  const int64_t R = R0 + p_local;
  const int64_t gi0 = conv_first_image<COMPACT>(g, cr, R0);
  const char* const base = reinterpret_cast<const char*>(in + gi0 * ldin);  // block-uniform
  uint32_t toff = 0;
  int base_row = 0;
  uint32_t vmask = 0;
  int64_t gi = 0;
  int ho = 0, wo = 0;
  if (conv_row<COMPACT>(g, cr, R, total_rows, &gi, &ho, &wo)) {
    const int h0 = ho * g.sh - g.pt;
    const int w0 = wo * g.sw - g.pl;
    toff = (uint32_t)((gi - gi0) * ldin * 8);
    base_row = h0 + w0 * g.H;
    // taps inside the image - and, where the input images come with windows, inside this image's window (the
    // rows outside it are zero and may not be in memory)
    int ha = 0, hb = g.H - 1, wa = 0, wb = g.W - 1;
    if (COMPACT && cr.in_box != nullptr) {
      const ColBox b = cr.in_box[gi];
      ha = max(ha, (int)b.h0), hb = min(hb, (int)b.h1), wa = max(wa, (int)b.w0), wb = min(wb, (int)b.w1);
    }
    for (int fw = 0; fw < g.FW; ++fw)
      for (int fh = 0; fh < g.FH; ++fh) {
        const int h = h0 + fh * g.dh, w = w0 + fw * g.dw;
        if (h >= ha && h <= hb && w >= wa && w <= wb) vmask |= 1u << (fh + g.FH * fw);
      }
  }

  double rp[4];
  struct alignas(32) Tap4 {
    FastTap t[4];
  };
  auto gather = [&](int k0) {
    const Tap4 t4 = *reinterpret_cast<const Tap4*>(taps + k0 + kq * 4);  // wave-uniform: one scalar load
    int row[4];
    bool ok[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      row[q] = base_row + t4.t[q].off;
      ok[q] = (vmask & t4.t[q].bit) != 0;
    }
    if (MASK) {
      // (the row of a tap outside the image may lie outside the mask, even outside the block's LDS, where a
      // read returns zero: the word read for it is not used)
      uint32_t b[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) b[q] = keep_s[row[q] >> 5];
#pragma unroll
      for (int q = 0; q < 4; ++q) ok[q] = ok[q] && __builtin_amdgcn_ubfe(b[q], (uint32_t)row[q] & 31u, 1u) != 0;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      double v = 0.0;
      if (ok[q]) v = *reinterpret_cast<const double*>(base + (toff + ((uint32_t)row[q] << 3)));
      rp[q] = v;
    }
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 4; ++q) Ps[buf][(kq * 4 + q) * TP + p_local] = rp[q];
  };
  // weights: transfer w of a K-tile brings rows w*kRowsPerLoad ... of the tile; lane l its 16 bytes
  const unsigned w_lds = lds_addr_of(&Wts[0][0]) + (unsigned)wave * 1024u;
  const unsigned w_voff = (unsigned)(((lane / (TC / 2)) * coutp + 2 * (lane % (TC / 2))) * 8);
  const double* const w_base = Wk + (int64_t)(wave * kRowsPerLoad) * coutp + c0;
  auto dma = [&](int k0, int buf) {
    if (wave < kWLoads) lds_dma16(w_base + (int64_t)k0 * coutp, w_voff, w_lds + (unsigned)(buf * kKt * TC * 8));
  };

  double4_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};

  __syncthreads();  // row mask in place
  const int nk = g.Kp / kKt;
  gather(0);
  dma(0, 0);
  store(0);
  wait_vm<0>();
  block_barrier();
  const int l16 = lane & 15, lq = lane >> 4;
  const double* const ps0 = &Ps[0][wr * (TP / WR) + l16 + lq * TP];
  const double* const ws0 = &Wts[0][wc * (TC / WC) + l16 + lq * TC];
  // one K-tile out of buffer `cur` (a constant, so that every LDS address is a base register plus an immediate)
  auto step = [&](int kt, auto cur_c) {
    constexpr int cur = decltype(cur_c)::value;
    if (kt + 1 < nk) {
      gather((kt + 1) * kKt);
      dma((kt + 1) * kKt, cur ^ 1);
    }
    const double* ps = ps0 + cur * (kKt * TP);
    const double* ws = ws0 + cur * (kKt * TC);
#pragma unroll
    for (int kk = 0; kk < kKt / 4; ++kk) {
      double b[FM], a[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) b[i] = ps[kk * 4 * TP + i * 16];
#pragma unroll
      for (int j = 0; j < FN; ++j) a[j] = ws[kk * 4 * TC + j * 16];
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[j], b[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) store(cur ^ 1);
    wait_vm<0>();     // this wave's weight transfer has landed ...
    block_barrier();  // ... and everybody's; everybody is done with the tiles of this step
  };
  for (int kt = 0; kt < nk; kt += 2) {
    step(kt, std::integral_constant<int, 0>());
    if (kt + 1 < nk) step(kt + 1, std::integral_constant<int, 1>());
  }
  conv_store_tile<TP, TC, WR, WC, FM, FN, COMPACT>(acc, out, ldout, bias, g, total_rows, R0, c0, wr, wc, lane, cr);
}

template <int TC, int WR, int WC, bool MASK, bool COMPACT>
__global__ __launch_bounds__(512) void conv2d_fast_kernel(ConvFastArgs a) {
  __shared__ __attribute__((aligned(1024))) double lds[2 * kKt * (128 + TC)];
  extern __shared__ uint32_t keep_s[];  // row mask (MASK only)
  conv2d_fast_block<TC, WR, WC, MASK, COMPACT>(a, blockIdx.x, lds, keep_s);
}

// Windows of the output columns of a convolution (see launch_conv_boxes in internal.h).
__global__ void conv_boxes_kernel(const ColBox* __restrict__ in_box, int64_t dense, const int32_t* __restrict__ onehot_idx,
                                  int64_t m, ColBox* __restrict__ out_box, ConvGeom g) {
  const int64_t j = blockIdx.x * (int64_t)256 + threadIdx.x;
  if (j >= dense + m) return;
  int h0 = 0, h1 = g.H - 1, w0 = 0, w1 = g.W - 1;  // window of the input column
  if (j >= dense) {
    const int src = onehot_idx[j - dense] % g.HW;
    w0 = w1 = src / g.H;
    h0 = h1 = src - w0 * g.H;
  } else if (j > 0 && in_box != nullptr) {
    const ColBox b = in_box[j];
    h0 = b.h0, h1 = b.h1, w0 = b.w0, w1 = b.w1;
  }
  ColBox o;
  if (j == 0) {
    // the centre image is not sparse: where every tap falls into the padding it still holds the bias
    o = ColBox{0, (int16_t)(g.Ho - 1), 0, (int16_t)(g.Wo - 1)};
  } else if (h0 > h1 || w0 > w1) {
    o = ColBox{1, 0, 1, 0};
  } else {
    // output rows whose taps ho*sh - pt + fh*dh (0 <= fh < FH) reach [h0, h1]
    auto floordiv = [](int a, int s) { return a >= 0 ? a / s : -((-a + s - 1) / s); };
    const int a0 = h0 + g.pt - (g.FH - 1) * g.dh, a1 = h1 + g.pt;
    const int b0 = w0 + g.pl - (g.FW - 1) * g.dw, b1 = w1 + g.pl;
    const int ho0 = max(0, -floordiv(-a0, g.sh)), ho1 = min(g.Ho - 1, floordiv(a1, g.sh));
    const int wo0 = max(0, -floordiv(-b0, g.sw)), wo1 = min(g.Wo - 1, floordiv(b1, g.sw));
    o = (ho0 > ho1 || wo0 > wo1) ? ColBox{1, 0, 1, 0} : ColBox{(int16_t)ho0, (int16_t)ho1, (int16_t)wo0, (int16_t)wo1};
  }
  out_box[j] = o;
}

__global__ void zero_pad_rows_kernel(double* __restrict__ V, int64_t ld, int64_t N, int64_t ncols) {
  const int64_t pad = ld - N;
  const int64_t total = pad * ncols;
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x)
    V[N + t % pad + (t / pad) * ld] = 0.0;
}


// ---- convolution of one-hot generator images -----------------------------------------------------
// A generator that is s * e_r (r = pixel (h, w, ci)) maps to the filter "stamped" around that pixel:
// out(ho, wo, co) = s * W(fh, fw, ci, co) for the one tap with ho*sh - pt + fh*dh = h and
// wo*sw - pl + fw*dw = w, and zero elsewhere.  The dense accumulation would add exact zeros to that
// one product, so 0 + w*s is the same value.  One pass that writes the output columns (HBM bound);
// lane = two adjacent output rows, the waves of a block interleave columns.
struct StampSet {
  const int32_t* idx;   // input row of every one-hot column
  const double* scale;  // by input row, or null (= 1)
  double* out;          // first of these columns in the output set
  const double* plb;    // predicate bounds of these columns
  const double* pub;
  double* part;         // [chunks][4][ldout] range sums of these columns (as the estimateRanges pass leaves them)
  int32_t m;
  int32_t win_only;     // 1: only the rows inside a column's window (the positions whose taps span its pixel) are written
  const int32_t* pixel_col;  // (by-row pass) input row -> its column here, -1: none
};

__global__ __launch_bounds__(512) void conv_stamp_kernel(const StampSet* __restrict__ table, StampSet one, ConvGeom g,
                                                         const double* __restrict__ Wt, int64_t ldout, int cols_per_chunk) {
  const StampSet d = table ? table[blockIdx.z] : one;
  const int j0 = min(d.m, (int)blockIdx.y * cols_per_chunk);  // an empty chunk still writes its (zero) sums
  const int j1 = min(d.m, j0 + cols_per_chunk);
  if (d.m == 0) return;
  double2 xmin1 = {0, 0}, xmin2 = {0, 0}, xmax1 = {0, 0}, xmax2 = {0, 0};
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r0 = (int64_t)blockIdx.x * 128 + 2 * lane;
  const int64_t Nout = (int64_t)g.P * g.Cout;
  // the two output rows of this lane: (ho, wo, co), fixed for all columns
  int hb[2], wb[2], co[2];
  bool real[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int64_t r = r0 + e;
    real[e] = r < Nout;
    const int p = real[e] ? (int)(r % g.P) : 0;
    co[e] = real[e] ? (int)(r / g.P) : 0;
    const int wo = p / g.Ho;
    const int ho = p - wo * g.Ho;
    hb[e] = ho * g.sh - g.pt;  // input row reached by tap fh = 0
    wb[e] = wo * g.sw - g.pl;
  }
  // the columns of the chunk are decoded once per block (pixel position, channel offset into the
  // weights, scale) in batches of kStampBatch and then read back from LDS by all lanes
  constexpr int kStampBatch = 256;
  __shared__ int s_h[kStampBatch], s_w[kStampBatch], s_k[kStampBatch];
  __shared__ double s_s[kStampBatch];
  const bool unit_dil = g.dh == 1 && g.dw == 1;
  for (int jb = j0; jb < j1; jb += kStampBatch) {
    const int nb = min(kStampBatch, j1 - jb);
    __syncthreads();
    for (int t = threadIdx.x; t < nb; t += 512) {
      const int src = d.idx[jb + t];
      const int ci = src / g.HW;
      const int q = src - ci * g.HW;
      const int w = q / g.H;
      s_h[t] = q - w * g.H;
      s_w[t] = w;
      s_k[t] = g.FH * g.FW * ci;
      s_s[t] = d.scale != nullptr ? d.scale[src] : 1.0;
    }
    __syncthreads();
    for (int t = wave; t < nb; t += 8) {
      const int h = s_h[t], w = s_w[t], kc = s_k[t];
      const double s = s_s[t];
      double v[2];
      bool inwin[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        v[e] = 0.0;
        const int th = h - hb[e], tw = w - wb[e];
        inwin[e] = real[e] && th >= 0 && tw >= 0 && th <= (g.FH - 1) * g.dh && tw <= (g.FW - 1) * g.dw;
        if (real[e] && th >= 0 && tw >= 0) {
          int fh = th, fw = tw;
          bool hit = true;
          if (!unit_dil) {
            fh = th / g.dh;
            fw = tw / g.dw;
            hit = fh * g.dh == th && fw * g.dw == tw;
          }
          if (hit && fh < g.FH && fw < g.FW) {
            const double wv = Wt[fh + g.FH * fw + kc + (int64_t)co[e] * g.Kp];
            v[e] = __dadd_rn(0.0, __dmul_rn(wv, s));
          }
        }
      }
      if (d.win_only) {
        double* o = d.out + r0 + (int64_t)(jb + t) * ldout;
        if (inwin[0]) o[0] = v[0];
        if (inwin[1]) o[1] = v[1];
      } else if (r0 < ldout) {
        *reinterpret_cast<double2*>(d.out + r0 + (int64_t)(jb + t) * ldout) = make_double2(v[0], v[1]);
      }
      const double pl = d.plb[jb + t], pu = d.pub[jb + t];
      const double px = fmax(v[0], 0.0), nx = fmin(v[0], 0.0);
      const double py = fmax(v[1], 0.0), ny = fmin(v[1], 0.0);
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
  // range sums of this chunk: the eight waves hold different columns of the same rows
  __shared__ double2 red[8][4][64];
  __syncthreads();
  if (wave > 0) {
    red[wave][0][lane] = xmin1;
    red[wave][1][lane] = xmin2;
    red[wave][2][lane] = xmax1;
    red[wave][3][lane] = xmax2;
  }
  __syncthreads();
  if (wave == 0 && r0 < ldout) {
    for (int w = 1; w < 8; ++w) {
      xmin1.x += red[w][0][lane].x;
      xmin1.y += red[w][0][lane].y;
      xmin2.x += red[w][1][lane].x;
      xmin2.y += red[w][1][lane].y;
      xmax1.x += red[w][2][lane].x;
      xmax1.y += red[w][2][lane].y;
      xmax2.x += red[w][3][lane].x;
      xmax2.y += red[w][3][lane].y;
    }
    double* p = d.part + ((int64_t)blockIdx.y * 4) * ldout + r0;
    *reinterpret_cast<double2*>(p) = xmin1;
    *reinterpret_cast<double2*>(p + ldout) = xmin2;
    *reinterpret_cast<double2*>(p + 2 * ldout) = xmax1;
    *reinterpret_cast<double2*>(p + 3 * ldout) = xmax2;
  }
}

// One bit per row of a set with a pending row reset: 1 where the row is kept.  Word w covers rows 32w..32w+31.
__global__ __launch_bounds__(256) void keep_bits_kernel(const int32_t* __restrict__ cls, int64_t N, uint32_t* __restrict__ bits,
                                                        int words) {
  const int64_t r = blockIdx.x * (int64_t)256 + threadIdx.x;
  const unsigned long long b = __ballot(r < N && cls[r] == kKeep);
  const int lane = threadIdx.x & 63;
  const int64_t w = r >> 5;
  if ((lane & 31) == 0 && w < words) bits[w] = (uint32_t)(b >> lane);
}

// ---- the stamps by output row (undilated filters) ---------------------------------------------------
// Row r = (ho, wo, co) of the output meets the stamps of the pixels under its filter window, one per tap: for
// tap k = (fh, fw, ci) the pixel (ho*sh - pt + fh, wo*sw - pl + fw, ci), whose unit-vector column t (pixel_col,
// -1: none) gets out(r, t) = 0 + W(k, co) * scale.  One thread per row writes those elements - exactly the
// non-zero candidates, i.e. the rows inside every column's window - and adds up the row's four range sums tap
// by tap.  Everything else in the columns is zero and is written by the caller (or left for later).
__global__ void stamp_pixel_columns_kernel(const int32_t* __restrict__ idx, int m, int32_t* __restrict__ pixel_col) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t < m) pixel_col[idx[t]] = t;
}

// S lanes share a row, lane s taking the taps k = s, s + S, ...; their sums are combined by a butterfly (a fixed
// order).  S = 1 for filters with few taps, 16 otherwise (a row's taps are then walked by 16 lanes at once).
// A block first decodes the taps once into LDS (filter position and the tap's offset from the pixel under the
// filter's corner), so that the walk has no division in it, and looks up four taps' pixels before it handles them.
constexpr int kStampTapTable = kMaxTaps;  // taps per output (FH * FW * Cin): no layer has more
// Block `blk` of NT threads; taps: LDS for g.K entries.
template <int S, int NT>
__device__ __forceinline__ void conv_stamp_rows_block(int64_t blk, int2* taps, const StampSet& d, const ConvGeom& g,
                                                      const double* __restrict__ Wt, const int32_t* __restrict__ pixel_col,
                                                      int64_t ldout) {
  for (int k = threadIdx.x; k < g.K; k += NT) {
    const int fh = k % g.FH;
    const int q = k / g.FH;
    const int fw = q % g.FW;
    const int ci = q / g.FW;
    taps[k] = make_int2(fh | (fw << 16), fh + g.H * (fw + g.W * ci));  // x: fh | fw << 16, y: fh + H * (fw + W * ci)
  }
  __syncthreads();
  const int64_t gt = blk * (int64_t)NT + threadIdx.x;
  const int64_t r = gt / S;
  const int s = (int)(gt % S);
  const bool row = r < ldout;
  const int64_t Nout = (int64_t)g.P * g.Cout;
  double x1 = 0.0, x2 = 0.0, y1 = 0.0, y2 = 0.0;
  if (row && r < Nout) {
    const int co = (int)(r / g.P);
    const int p = (int)(r - (int64_t)co * g.P);
    const int wo = p / g.Ho, ho = p - wo * g.Ho;
    const int hb = ho * g.sh - g.pt, wb = wo * g.sw - g.pl;
    const int pbase = hb + g.H * wb;  // the pixel under the filter's corner (may lie outside the image)
    const double* wcol = Wt + (int64_t)co * g.Kp;
    for (int k0 = s; k0 < g.K; k0 += 4 * S) {
      int t[4], pix[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + u * S;
        t[u] = -1;
        pix[u] = 0;
        if (k < g.K) {
          const int2 tp = taps[k];
          const int h = hb + (tp.x & 0xffff), w = wb + (tp.x >> 16);
          if ((unsigned)h < (unsigned)g.H && (unsigned)w < (unsigned)g.W) {
            pix[u] = pbase + tp.y;
            t[u] = pixel_col[pix[u]];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (t[u] < 0) continue;
        const int k = k0 + u * S;
        const double sc = d.scale != nullptr ? d.scale[pix[u]] : 1.0;
        const double v = __dadd_rn(0.0, __dmul_rn(wcol[k], sc));
        d.out[r + (int64_t)t[u] * ldout] = v;
        const double pl = d.plb[t[u]], pu = d.pub[t[u]];
        const double vp = fmax(v, 0.0), vn = fmin(v, 0.0);
        x1 = fma(vp, pl, x1);  // xmin1
        x2 = fma(vn, pu, x2);  // xmin2
        y1 = fma(vp, pu, y1);  // xmax1
        y2 = fma(vn, pl, y2);  // xmax2
      }
    }
  }
#pragma unroll
  for (int off = 1; off < S; off <<= 1) {
    x1 += __shfl_xor(x1, off);
    x2 += __shfl_xor(x2, off);
    y1 += __shfl_xor(y1, off);
    y2 += __shfl_xor(y2, off);
  }
  if (row && s == 0) {
    d.part[r] = x1;
    d.part[ldout + r] = x2;
    d.part[2 * ldout + r] = y1;
    d.part[3 * ldout + r] = y2;
  }
}

template <int S>
__global__ __launch_bounds__(256) void conv_stamp_rows_kernel(StampSet d, ConvGeom g, const double* __restrict__ Wt,
                                                              const int32_t* __restrict__ pixel_col, int64_t ldout) {
  __shared__ int2 taps[kStampTapTable];
  conv_stamp_rows_block<S, 256>(blockIdx.x, taps, d, g, Wt, pixel_col, ldout);
}

// The dense images' convolution and the stamps of the unit-vector columns of the same layer in one launch: the two
// write different columns of the output and read nothing of each other, the first is bound by the matrix pipe and the
// second by scattered stores, so their blocks are dealt to the chip in turn (every stride-th block of the grid is a
// stamp block, until there are no more) and run side by side on a compute unit.
struct ConvStampArgs {
  StampSet d;
  const double* Wt;
  const int32_t* pixel_col;
  int32_t blocks;  // stamp blocks in the grid
  int32_t stride;  // grid position p is stamp block (p + 1) / stride - 1 where (p + 1) % stride == 0 (and that is < blocks)
};

template <int TC, int WR, int WC, bool MASK, bool COMPACT, int S>
__global__ __launch_bounds__(512) void conv2d_fast_stamps_kernel(ConvFastArgs a, ConvStampArgs st) {
  static_assert(sizeof(int2) * kStampTapTable <= conv_fast_lds_bytes(TC), "the stamp blocks' tap table fits the tiles' LDS");
  __shared__ __attribute__((aligned(1024))) double lds[2 * kKt * (128 + TC)];
  extern __shared__ uint32_t keep_s[];  // row mask (MASK only)
  const int p = blockIdx.x;
  const int k = (p + 1) / st.stride;
  if ((p + 1) % st.stride == 0 && k <= st.blocks) {
    conv_stamp_rows_block<S, 512>(k - 1, reinterpret_cast<int2*>(lds), st.d, a.g, st.Wt, st.pixel_col, a.ldout);
    return;
  }
  conv2d_fast_block<TC, WR, WC, MASK, COMPACT>(a, p - min(st.blocks, p / st.stride), lds, keep_s);
}

// LDS of the convolution kernel beside its tap table and row mask: the two double-buffered operand tiles
template <int TP, int TC>
constexpr size_t conv_static_lds() {
  return sizeof(double) * 2 * (kKt * (TP + kPadRow) + TC * (kKt + kPadK));
}

template <int TP, int TC, int WR, int WC>
static int launch_conv_cfg(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, const ConvGeom& g, const double* in, int64_t ldin,
                           double* out, int64_t ldout, int64_t ncols, const uint32_t* keep, int keep_words) {
  const int64_t total_rows = (int64_t)g.P * ncols;
  const int64_t tiles_c = ceil_div(g.Cout, TC);
  const int64_t blocks = ceil_div(total_rows, TP) * tiles_c;
  if (blocks >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "convolution too large for one launch");
  const size_t dyn = sizeof(unsigned long long) * g.Kp + (keep ? sizeof(uint32_t) * (size_t)keep_words : 0);
  if (conv_static_lds<TP, TC>() + dyn > kConvLdsLimit)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "filters with %d taps (FH*FW*Cin) and %d output channels are not supported: at most %d taps", g.K, g.Cout,
             (int)((kConvLdsLimit - conv_static_lds<TP, TC>()) / sizeof(unsigned long long) / kKt * kKt));
  NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
  if (keep)
    NNV_LAUNCH(ctx, ctx->kernel_timing, (conv2d_f64_kernel<TP, TC, WR, WC, true>), dim3((unsigned)blocks), dim3(64 * WR * WC), dyn, in,
               ldin, out, ldout, cv->W->as<double>(), cv->bias ? cv->bias->as<double>() : nullptr, g, total_rows, (int)tiles_c, keep,
               keep_words);
  else
    NNV_LAUNCH(ctx, ctx->kernel_timing, (conv2d_f64_kernel<TP, TC, WR, WC, false>), dim3((unsigned)blocks), dim3(64 * WR * WC), dyn, in,
               ldin, out, ldout, cv->W->as<double>(), cv->bias ? cv->bias->as<double>() : nullptr, g, total_rows, (int)tiles_c, keep,
               keep_words);
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 1, 2.0 * (double)total_rows * g.Cout * g.K));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

static void fill_geom(ConvGeom& g, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo);

// ---- which kernel, and whether it can mask rows on load --------------------------------------------
constexpr size_t conv_fast_static_lds(int tc) { return sizeof(double) * 2 * kKt * (128 + (size_t)tc); }
static int conv_tile_channels(const nnvhip_conv2d* cv) { return cv->Cout <= 16 ? 16 : cv->Cout <= 32 ? 32 : 64; }

// The kernel with scalar tap decoding: at most 32 spatial taps (one mask bit each), every byte offset it forms
// (a row of the image plus the images a 128-position tile can span) below 2^31.
static bool conv_fast_ok(const nnvhip_conv2d* cv, const ConvGeom& g, int64_t ldin, int64_t rows_per_image = 0) {
  if (tune_knobs().conv_general != 0 || cv->Wk == nullptr) return false;
  if (cv->FH * cv->FW > 32) return false;
  const int64_t n_in = (int64_t)g.HW * g.Cin;
  const int64_t images_per_tile = 127 / (rows_per_image > 0 ? rows_per_image : g.P) + 2;
  return (n_in + images_per_tile * ldin) * 8 < (int64_t(1) << 31);
}

bool conv2d_can_mask(const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int64_t ldin) {
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
  const int64_t n_in = H * W * cv->Cin;
  if (n_in >= (int64_t(1) << 31) || cv->Kp > kMaxTaps) return false;
  const size_t mask = sizeof(uint32_t) * (size_t)ceil_div(n_in, 32);
  if (conv_fast_ok(cv, g, ldin)) return conv_fast_static_lds(conv_tile_channels(cv)) + mask <= kConvLdsLimit;
  // the general kernel, sized for its widest tile (128 x 64): the mask shares the dynamic LDS with the tap table
  return conv_static_lds<128, 64>() + sizeof(unsigned long long) * (size_t)cv->Kp + mask <= kConvLdsLimit;
}

int conv2d_prepare_weights(nnvhip_ctx* ctx, nnvhip_conv2d* cv) {
  cv->coutp = round_up(cv->Cout, 64);
  if (cv->Kp * cv->coutp >= (int64_t(1) << 28)) return NNVHIP_OK;  // stays on the general kernel
  NNV_TRY(ctx->alloc(sizeof(double) * cv->Kp * cv->coutp, &cv->Wk));
  hipLaunchKernelGGL(conv_weights_kmajor_kernel, dim3((unsigned)ceil_div(cv->Kp * cv->coutp, 256)), dim3(256), 0, ctx->stream,
                     cv->W->as<double>(), cv->Wk->as<double>(), (int)cv->Kp, (int)cv->Cout, (int)cv->coutp);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

static int conv_fast_taps(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, const ConvGeom& g, const FastTap** tab) {
  for (const auto& t : cv->tap_tables)
    if (t.H == g.H && t.W == g.W) {
      *tab = t.tab->as<FastTap>();
      return NNVHIP_OK;
    }
  nnvhip_conv2d::TapTable t;
  t.H = g.H;
  t.W = g.W;
  NNV_TRY(ctx->alloc(sizeof(FastTap) * (size_t)g.Kp, &t.tab));
  hipLaunchKernelGGL(conv_fast_taps_kernel, dim3((unsigned)ceil_div(g.Kp, 256)), dim3(256), 0, ctx->stream, t.tab->as<FastTap>(), g);
  NNV_HIP_TRY(hipGetLastError());
  if (cv->tap_tables.size() >= 8) cv->tap_tables.erase(cv->tap_tables.begin());
  cv->tap_tables.push_back(t);
  *tab = t.tab->as<FastTap>();
  return NNVHIP_OK;
}

// stamp != null (a set's unit-vector columns, pixel_col and part filled in, filters undilated): their stamps go into
// the same launch.
template <int TC, int WR, int WC>
static int launch_conv_fast(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, const ConvGeom& g, const double* in, int64_t ldin, double* out,
                            int64_t ldout, int64_t ncols, const uint32_t* keep, int keep_words, const ConvRows& cr,
                            const StampSet* stamp) {
  const bool compact = cr.box != nullptr;
  const int64_t total_rows = compact ? (int64_t)g.P + (ncols - 1) * cr.area : (int64_t)g.P * ncols;
  const int64_t tiles_c = ceil_div(g.Cout, TC);
  const int64_t blocks = ceil_div(total_rows, 128) * tiles_c;
  const size_t dyn = keep ? sizeof(uint32_t) * (size_t)keep_words : 0;
  if (conv_fast_static_lds(TC) + dyn > kConvLdsLimit) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: row mask too large for the convolution kernel");
  ConvFastArgs a{};
  NNV_TRY(conv_fast_taps(ctx, cv, g, &a.taps));
  a.in = in;
  a.ldin = ldin;
  a.out = out;
  a.ldout = ldout;
  a.Wk = cv->Wk->as<double>();
  a.coutp = (int)cv->coutp;
  a.bias = cv->bias ? cv->bias->as<double>() : nullptr;
  a.g = g;
  a.total_rows = total_rows;
  a.tiles_c = (int)tiles_c;
  a.keep = keep;
  a.keep_words = keep_words;
  a.cr = cr;
  // lanes per output row of the stamp blocks: 8 for filters with many taps (beside the tile blocks that measured best:
  // config 4 0.747 ms against 0.752 with 16 lanes, 0.756 with 4, 0.782 with 32), else 1
  const bool wide_stamps = g.K > 32;
  ConvStampArgs sa{};
  if (stamp != nullptr) {
    sa.d = *stamp;
    sa.Wt = cv->W->as<double>();
    sa.pixel_col = stamp->pixel_col;
    sa.blocks = (int32_t)ceil_div(ldout * (wide_stamps ? 8 : 1), 512);
    sa.stride = (int32_t)std::max<int64_t>(1, (blocks + sa.blocks) / sa.blocks);
  }
  const int64_t grid = blocks + sa.blocks;
  if (grid >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "convolution too large for one launch");
  NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
#define NNV_CONV_FAST(MASK, COMPACT)                                                                                                    \
  do {                                                                                                                                  \
    if (stamp == nullptr)                                                                                                               \
      NNV_LAUNCH(ctx, ctx->kernel_timing, (conv2d_fast_kernel<TC, WR, WC, MASK, COMPACT>), dim3((unsigned)grid), dim3(512), dyn, a);    \
    else if (wide_stamps)                                                                                                               \
      NNV_LAUNCH(ctx, ctx->kernel_timing, (conv2d_fast_stamps_kernel<TC, WR, WC, MASK, COMPACT, 8>), dim3((unsigned)grid), dim3(512), \
                 dyn, a, sa);                                                                                                           \
    else                                                                                                                                \
      NNV_LAUNCH(ctx, ctx->kernel_timing, (conv2d_fast_stamps_kernel<TC, WR, WC, MASK, COMPACT, 1>), dim3((unsigned)grid), dim3(512),  \
                 dyn, a, sa);                                                                                                           \
  } while (0)
  if (keep && compact)
    NNV_CONV_FAST(true, true);
  else if (keep)
    NNV_CONV_FAST(true, false);
  else if (compact)
    NNV_CONV_FAST(false, true);
  else
    NNV_CONV_FAST(false, false);
#undef NNV_CONV_FAST
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 1, 2.0 * (double)total_rows * g.Cout * g.K));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

int launch_zero_pad_rows(nnvhip_ctx* ctx, double* V, int64_t ld, int64_t N, int64_t ncols) {
  if (ld == N || ncols <= 0) return NNVHIP_OK;
  hipLaunchKernelGGL(zero_pad_rows_kernel, dim3(256), dim3(256), 0, ctx->stream, V, ld, N, ncols);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

int64_t conv_box_extent(const nnvhip_conv2d* cv, int dim, int64_t e, int64_t out_size) {
  // output positions whose taps reach a run of e input positions: floor((e - 1 + (F - 1) * dil) / stride) + 1
  const int64_t F = dim == 0 ? cv->FH : cv->FW;
  return std::min<int64_t>(out_size, (e - 1 + (F - 1) * cv->dil[dim]) / cv->stride[dim] + 1);
}

int launch_conv_boxes(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                      const ColBox* in_box, int64_t dense, const int32_t* onehot_idx, int64_t m, ColBox* out_box) {
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
  hipLaunchKernelGGL(conv_boxes_kernel, dim3((unsigned)ceil_div(dense + m, 256)), dim3(256), 0, ctx->stream, in_box, dense, onehot_idx, m,
                     out_box, g);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

bool conv2d_in_windows(const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int64_t ldin, int64_t ncols,
                       const ColBox* out_box, int eh, int ew) {
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
  return out_box != nullptr && ncols > 1 && eh > 0 && ew > 0 && 2 * (int64_t)eh * ew <= g.P &&
         conv_fast_ok(cv, g, ldin, (int64_t)eh * ew);
}

int launch_conv2d(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                  const double* in, int64_t ldin, double* out, int64_t ldout, int64_t ncols,
                  const int32_t* pending_cls, const ColBox* out_box, int eh, int ew, const ColBox* in_box, bool leave_outside,
                  const uint32_t* pending_bits, const ConvStampSet* stamp, bool* stamped) {
  if (stamped != nullptr) *stamped = false;
  if (cv->Kp > kMaxTaps) NNV_FAIL(NNVHIP_ERR_SHAPE, "filters with more than %d taps (FH*FW*Cin) are not supported", kMaxTaps);
  if ((cv->FH - 1) * cv->dil[0] > 0xffff || (cv->FW - 1) * cv->dil[1] > 0xffff)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "dilated filter extent too large");
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
  const int64_t Nout = Ho * Wo * cv->Cout;
  // a pending row reset of the input is applied on load, from one bit per input row
  const int64_t n_in = H * W * cv->Cin;
  const uint32_t* keep = nullptr;
  int keep_words = 0;
  BufRef bits;
  if (pending_cls != nullptr) {
    if (!conv2d_can_mask(cv, H, W, Ho, Wo, ldin)) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: row mask too large for the convolution kernel");
    keep_words = (int)ceil_div(n_in, 32);
    if (pending_bits != nullptr) {
      keep = pending_bits;
    } else {
      NNV_TRY(ctx->alloc(sizeof(uint32_t) * (size_t)keep_words, &bits));
      // whole waves only, so that every word is written by a lane that exists
      hipLaunchKernelGGL(keep_bits_kernel, dim3((unsigned)ceil_div(n_in, 256)), dim3(256), 0, ctx->stream, pending_cls, n_in,
                         bits->as<uint32_t>(), keep_words);
      NNV_HIP_TRY(hipGetLastError());
      keep = bits->as<uint32_t>();
    }
  }
  // 128 positions x Cout tile, eight waves per block (two per SIMD keep the MFMA pipe fed while
  // the other wave gathers)
  int st;
  // Generator images with known windows are computed inside them only (the caller has zeroed the rest) when that
  // at least halves the rows; it takes the kernel with scalar tap decoding.
  ConvRows cr{nullptr, 0, 0, nullptr};
  if (conv2d_in_windows(cv, H, W, Ho, Wo, ldin, ncols, out_box, eh, ew)) cr = ConvRows{out_box, eh, eh * ew, in_box};
  if (cr.box == nullptr && (in_box != nullptr || leave_outside))
    NNV_FAIL(NNVHIP_ERR_ARG, "internal: the convolution was to stay inside the images' windows");
  if (cr.box != nullptr && !leave_outside)  // everything outside the windows
    NNV_HIP_TRY(hipMemsetAsync(out + ldout, 0, sizeof(double) * (size_t)ldout * (size_t)(ncols - 1), ctx->stream));
  if (cr.box != nullptr || conv_fast_ok(cv, g, ldin)) {
    // the stamps of the set's unit-vector columns ride along where they are made row by row and come with their
    // pixel table and a place for their range sums
    static_assert(sizeof(ConvStampSet) == sizeof(StampSet), "same layout");
    StampSet one;
    const StampSet* merge = nullptr;
    if (stamp != nullptr && stamped != nullptr && stamp->m > 0 && stamp->pixel_col != nullptr && stamp->part != nullptr &&
        cv->dil[0] == 1 && cv->dil[1] == 1 && g.K <= kStampTapTable) {
      memcpy(&one, stamp, sizeof one);
      merge = &one;
      if (!one.win_only)  // whole columns: the zeros first
        NNV_HIP_TRY(hipMemsetAsync(one.out, 0, sizeof(double) * (size_t)ldout * (size_t)one.m, ctx->stream));
      *stamped = true;
    }
    if (cv->Cout <= 16)
      st = launch_conv_fast<16, 8, 1>(ctx, cv, g, in, ldin, out, ldout, ncols, keep, keep_words, cr, merge);
    else if (cv->Cout <= 32)
      st = launch_conv_fast<32, 4, 2>(ctx, cv, g, in, ldin, out, ldout, ncols, keep, keep_words, cr, merge);
    else
      st = launch_conv_fast<64, 4, 2>(ctx, cv, g, in, ldin, out, ldout, ncols, keep, keep_words, cr, merge);
  } else if (cv->Cout <= 16) {
    st = launch_conv_cfg<128, 16, 8, 1>(ctx, cv, g, in, ldin, out, ldout, ncols, keep, keep_words);
  } else if (cv->Cout <= 32) {
    st = launch_conv_cfg<128, 32, 4, 2>(ctx, cv, g, in, ldin, out, ldout, ncols, keep, keep_words);
  } else {
    st = launch_conv_cfg<128, 64, 4, 2>(ctx, cv, g, in, ldin, out, ldout, ncols, keep, keep_words);
  }
  NNV_TRY(st);
  if (ldout != Nout) {  // keep the padding rows of the output at zero
    hipLaunchKernelGGL(zero_pad_rows_kernel, dim3(256), dim3(256), 0, ctx->stream, out, ldout, Nout, ncols);
    NNV_HIP_TRY(hipGetLastError());
  }
  return NNVHIP_OK;
}

static void fill_geom(ConvGeom& g, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo) {
  g.H = (int)H;
  g.W = (int)W;
  g.Cin = (int)cv->Cin;
  g.Ho = (int)Ho;
  g.Wo = (int)Wo;
  g.Cout = (int)cv->Cout;
  g.FH = (int)cv->FH;
  g.FW = (int)cv->FW;
  g.sh = (int)cv->stride[0];
  g.sw = (int)cv->stride[1];
  g.dh = (int)cv->dil[0];
  g.dw = (int)cv->dil[1];
  g.pt = (int)cv->pad[0];
  g.pl = (int)cv->pad[2];
  g.K = (int)cv->K;
  g.Kp = (int)cv->Kp;
  g.P = (int)(Ho * Wo);
  g.HW = (int)(H * W);
}

static bool conv_stamps_by_row(const nnvhip_conv2d* cv) { return cv->dil[0] == 1 && cv->dil[1] == 1; }
bool conv_stamps_by_pixel(const nnvhip_conv2d* cv) { return conv_stamps_by_row(cv); }

int launch_pixel_columns(nnvhip_ctx* ctx, const int32_t* idx, int64_t m, int64_t n_in, BufRef* inv) {
  NNV_TRY(ctx->alloc(sizeof(int32_t) * (size_t)n_in, inv));
  NNV_HIP_TRY(hipMemsetAsync((*inv)->ptr, 0xff, sizeof(int32_t) * (size_t)n_in, ctx->stream));
  if (m > 0) {
    hipLaunchKernelGGL(stamp_pixel_columns_kernel, dim3((unsigned)ceil_div(m, 256)), dim3(256), 0, ctx->stream, idx, (int)m,
                       (*inv)->as<int32_t>());
    NNV_HIP_TRY(hipGetLastError());
  }
  return NNVHIP_OK;
}

int64_t conv_stamp_chunks(const nnvhip_conv2d* cv, int64_t ldout, int64_t count, int64_t max_m) {
  if (conv_stamps_by_row(cv)) return 1;
  const int64_t row_blocks = ceil_div(ldout, 128);
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(8192, row_blocks * count), ceil_div(std::max<int64_t>(max_m, 1), 32)));
  const int64_t cpc = ceil_div(std::max<int64_t>(max_m, 1), chunks);
  return ceil_div(std::max<int64_t>(max_m, 1), cpc);
}

int launch_conv_stamps(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                       int64_t ldout, int64_t count, const ConvStampSet* sets, int64_t chunks) {
  static_assert(sizeof(ConvStampSet) == sizeof(StampSet), "same layout");
  if (count <= 0) return NNVHIP_OK;
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  int64_t max_m = 0;
  double bytes = 0.0;
  for (int64_t i = 0; i < count; ++i) {
    max_m = std::max<int64_t>(max_m, sets[i].m);
    // algorithmic: the output columns -- whole ones, or, when only the rows inside each column's window are written,
    // the filter stamp itself (at most FH * FW positions of every output channel)
    const double rows_written = sets[i].win_only ? (double)std::min<int64_t>(Ho * Wo, cv->FH * cv->FW) * (double)cv->Cout
                                                 : (double)(Ho * Wo * cv->Cout);
    bytes += 8.0 * rows_written * (double)sets[i].m;
  }
  if (max_m == 0) return NNVHIP_OK;
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
  if (conv_stamps_by_row(cv)) {
    if (chunks != 1) NNV_FAIL(NNVHIP_ERR_ARG, "internal: one chunk of range sums per set");
    if (g.K > kStampTapTable) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: more taps than the stamp kernel's table holds");
    const int64_t n_in = H * W * cv->Cin;
    std::vector<BufRef> made;  // tables of the sets that came without one
    NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
    for (int64_t i = 0; i < count; ++i) {
      if (sets[i].m == 0) continue;
      StampSet one;
      memcpy(&one, &sets[i], sizeof one);
      const int32_t* pc = one.pixel_col;
      if (pc == nullptr) {
        BufRef inv;
        NNV_TRY(launch_pixel_columns(ctx, one.idx, one.m, n_in, &inv));
        pc = inv->as<int32_t>();
        made.push_back(inv);
      }
      if (!one.win_only)  // whole columns: the zeros first
        NNV_HIP_TRY(hipMemsetAsync(one.out, 0, sizeof(double) * (size_t)ldout * (size_t)one.m, ctx->stream));
      if (g.K <= 32)
        NNV_LAUNCH(ctx, ctx->kernel_timing && i == 0, conv_stamp_rows_kernel<1>, dim3((unsigned)ceil_div(ldout, 256)), dim3(256), 0, one, g,
                   cv->W->as<double>(), pc, ldout);
      else
        NNV_LAUNCH(ctx, ctx->kernel_timing && i == 0, conv_stamp_rows_kernel<16>, dim3((unsigned)ceil_div(ldout * 16, 256)), dim3(256), 0,
                   one, g, cv->W->as<double>(), pc, ldout);
    }
    NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 5, bytes));
    NNV_HIP_TRY(hipGetLastError());
    return NNVHIP_OK;
  }
  const int64_t row_blocks = ceil_div(ldout, 128);
  const int64_t cpc = ceil_div(max_m, chunks);
  const StampSet* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(ctx->upload_table(sets, sizeof(StampSet) * count, &tab));
    table = tab->as<StampSet>();
  }
  StampSet one;
  memcpy(&one, &sets[0], sizeof one);
  NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
  NNV_LAUNCH(ctx, ctx->kernel_timing, conv_stamp_kernel, dim3((unsigned)row_blocks, (unsigned)chunks, (unsigned)count), dim3(512), 0,
             table, one, g, cv->W->as<double>(), ldout, (int)cpc);
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 5, bytes));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

}  // namespace nnvhip
