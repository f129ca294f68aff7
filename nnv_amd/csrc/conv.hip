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

#include "internal.h"
#include "mfma_tile.h"

namespace nnvhip {

struct ConvGeom {
  int H, W, Cin, Ho, Wo, Cout;
  int FH, FW, sh, sw, dh, dw, pt, pl;
  int K, Kp;
  int P;   // Ho * Wo
  int HW;  // H * W
};

constexpr int kMaxTaps = 4096;  // tap table held in LDS: 8 bytes per (padded) tap

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

template <int TP, int TC, int WR, int WC>
__global__ __launch_bounds__(64 * WR * WC) void conv2d_f64_kernel(const double* __restrict__ in, int64_t ldin,
                                                          double* __restrict__ out, int64_t ldout,
                                                          const double* __restrict__ Wt,
                                                          const double* __restrict__ bias, ConvGeom g,
                                                          int64_t total_rows, int tiles_c) {
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
      const bool ok = rvalid && t != ~0ull && (unsigned)h < (unsigned)g.H && (unsigned)w < (unsigned)g.W;
      rp[q] = ok ? img[(int64_t)(unsigned)(t >> 32) + h + (int64_t)w * g.H] : 0.0;
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

  // epilogue: lane l, register r holds out[position R0 + ... + l%16][channel c0 + ... + l/16 + 4r]
  const int lrow = lane & 15;
  const int lcol = lane >> 4;
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int64_t Rr = R0 + wr * (TP / WR) + i * 16 + lrow;
    if (Rr >= total_rows) continue;
    const int64_t gi = Rr / g.P;
    const int p = (int)(Rr - gi * g.P);
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
  int32_t pad_;
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
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        v[e] = 0.0;
        const int th = h - hb[e], tw = w - wb[e];
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
      if (r0 < ldout) *reinterpret_cast<double2*>(d.out + r0 + (int64_t)(jb + t) * ldout) = make_double2(v[0], v[1]);
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

template <int TP, int TC, int WR, int WC>
static int launch_conv_cfg(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, const ConvGeom& g, const double* in, int64_t ldin,
                           double* out, int64_t ldout, int64_t ncols) {
  const int64_t total_rows = (int64_t)g.P * ncols;
  const int64_t tiles_c = ceil_div(g.Cout, TC);
  const int64_t blocks = ceil_div(total_rows, TP) * tiles_c;
  if (blocks >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "convolution too large for one launch");
  const size_t dyn = sizeof(unsigned long long) * g.Kp;
  NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
  NNV_LAUNCH(ctx, ctx->kernel_timing, (conv2d_f64_kernel<TP, TC, WR, WC>), dim3((unsigned)blocks), dim3(64 * WR * WC), dyn, in, ldin,
             out, ldout, cv->W->as<double>(), cv->bias ? cv->bias->as<double>() : nullptr, g, total_rows,
                     (int)tiles_c);
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 1, 2.0 * (double)total_rows * g.Cout * g.K));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

static void fill_geom(ConvGeom& g, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo);

int launch_conv2d(nnvhip_ctx* ctx, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                  const double* in, int64_t ldin, double* out, int64_t ldout, int64_t ncols,
                  const int32_t* /*centre_flags*/) {
  if (cv->Kp > kMaxTaps) NNV_FAIL(NNVHIP_ERR_SHAPE, "filters with more than %d taps (FH*FW*Cin) are not supported", kMaxTaps);
  if ((cv->FH - 1) * cv->dil[0] > 0xffff || (cv->FW - 1) * cv->dil[1] > 0xffff)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "dilated filter extent too large");
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
  const int64_t Nout = Ho * Wo * cv->Cout;
  // 128 positions x Cout tile, eight waves per block (two per SIMD keep the MFMA pipe fed while
  // the other wave gathers)
  int st;
  if (cv->Cout <= 16)
    st = launch_conv_cfg<128, 16, 8, 1>(ctx, cv, g, in, ldin, out, ldout, ncols);
  else if (cv->Cout <= 32)
    st = launch_conv_cfg<128, 32, 4, 2>(ctx, cv, g, in, ldin, out, ldout, ncols);
  else
    st = launch_conv_cfg<128, 64, 4, 2>(ctx, cv, g, in, ldin, out, ldout, ncols);
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

int64_t conv_stamp_chunks(int64_t ldout, int64_t count, int64_t max_m) {
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
    bytes += 8.0 * (double)(Ho * Wo * cv->Cout) * (double)sets[i].m;  // algorithmic: the output columns
  }
  if (max_m == 0) return NNVHIP_OK;
  ConvGeom g;
  fill_geom(g, cv, H, W, Ho, Wo);
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
