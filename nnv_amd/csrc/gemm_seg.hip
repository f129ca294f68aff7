// affineMap of a fully connected layer over an array of sets whose rows were mostly reset by the ReLU
// step before it: C_s = W(:, kept_s) * [c V]_s(kept_s, :) for every set s, in one launch.
//
// Every set contracts over its own short list of kept rows (config 5: 240 of 1024), so the product is
// cut into 128-row x TN-column tiles that each belong to one set (SegTile).  The B operand comes from the
// set's packed rows, stored transposed (row k of the packed matrix = the set's columns, contiguous), and
// the A operand is gathered column by column from the weight matrix; both reach LDS through the direct
// global-to-LDS path (global_load_lds_dwordx4: no staging registers, four stages in flight), one 1 KiB
// wave transfer per stage row.  The MFMA operand roles follow gemm.hip, but every lane owns FM consecutive
// rows and FN consecutive columns of its wave's sub-tile: operands are read from LDS with 128-bit loads
// and the result is stored in 128-bit pieces.  The epilogue leaves the tile's four Star.estimateRanges
// partial sums (set/Star.m:1098-1104) as gemm.hip's fused epilogue does, and adds the bias to a set's
// centre column.  Sets whose column count is not a multiple of 128 end in a narrower tile (32 or 64
// columns) from a second launch, so a 785-column set costs 6.3 tiles instead of 7.
#include <algorithm>
#include <cstdlib>

#include "internal.h"
#include "lds_dma.h"
#include "mfma_tile.h"

namespace nnvhip {

typedef double double2_t __attribute__((ext_vector_type(2)));

namespace {

constexpr int kSegTM = 128;  // rows of a tile
constexpr int kSegKS = 8;    // rows of W / of the packed matrix per pipeline stage
constexpr int kSegS = 4;     // stages in LDS
constexpr int kSegNT = 512;  // threads per block

// TN columns per tile; WR x WC waves, each owning (16*FM) rows x (16*FN) columns.
template <int TN, int WR, int WC, int FM, int FN, bool GATHER = false>
__global__ __launch_bounds__(kSegNT, 4) void gemm_seg_kernel(const double* __restrict__ A, int64_t lda,
                                                            double* __restrict__ C, int64_t ldc, int Mp,
                                                            const double* __restrict__ bias, int tiles_m, int64_t tiles_n,
                                                            int xr, int local_m, const SegTile* __restrict__ segs) {
  static_assert(WR * WC == 8 && 16 * FM * WR == kSegTM && 16 * FN * WC == TN, "eight waves cover the tile");
  constexpr int kStageA = kSegKS * kSegTM;        // doubles per stage of A
  constexpr int kStageB = kSegKS * TN;            // ... of B
  constexpr int kBLoads = kStageB / 128;          // 1 KiB wave transfers per stage of B
  constexpr int kRed = WC * 4 * 4 * kSegTM;       // epilogue: [WC * 4 partials][4 sums][128 rows]
  constexpr int kLds = kSegS * (kStageA + kStageB) > kRed ? kSegS * (kStageA + kStageB) : kRed;
  __shared__ __attribute__((aligned(1024))) double smem[kLds];
  __shared__ double pbs[2][TN];
  double* const As = smem;
  double* const Bs = smem + kSegS * kStageA;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave % WR, wc = wave / WR;
  const int l16 = lane & 15, q = lane >> 4;
  // XCD-aware tile mapping, as in gemm.hip
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int xc = 8 / xr;
  const int mt = (slot % local_m) * xr + (xcd % xr);
  const int64_t nt = (int64_t)(slot / local_m) * xc + (xcd / xr);
  if (mt >= tiles_m || nt >= tiles_n) return;
  const int m0 = mt * kSegTM;
  const SegTile sg = segs[nt];
  const int nst = sg.kp / kSegKS;

  // predicate bounds of the tile's columns (zero for the centre and for columns past the set's end, which
  // then add nothing to the sums): loaded now, parked in a register, stored to LDS after the K loop
  double pb_reg = 0.0;
  if (tid < 2 * TN) {
    const int t = tid % TN;
    const int64_t sc = sg.col_local0 + t;
    const bool ok = t < sg.valid && sc >= 1 && sg.rpart != nullptr;
    const double* src = tid < TN ? sg.plb : sg.pub;
    if (ok) pb_reg = src[sc - 1];
  }
  // row list: wave w stages row 8 * st + w of stage st; lane j keeps the entries of stages j, j + 64, ...
  static_assert(!GATHER || TN == 128, "rows of B are gathered one per wave");
  const bool centre_tile = GATHER && sg.col_local0 == 0 && sg.centre != nullptr;
  int kq[4];
  double cq[4];  // GATHER, a set's first tile: the centre's entries of the same rows
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int st = u * 64 + lane;
    const int c = st < nst ? sg.kmap[st * kSegKS + wave] : 0;
    // a padding entry: its packed row is zero, any column of W will do (GATHER: the entry stays negative and the
    // row of B is taken from the row of zeros)
    kq[u] = (c < 0 && !GATHER) ? 0 : c;
    cq[u] = 0.0;
    if (GATHER && centre_tile && st < nst && c >= 0) cq[u] = sg.centre[c];
  }
  const unsigned a_lds = lds_addr_of(As + wave * kSegTM);
  const unsigned a_voff = lane * 16;
  const double* a_base = A + m0;
  // B: the stage's kSegKS x TN block is kBLoads transfers; transfer w (waves 0 .. kBLoads-1) brings 128 / TN rows
  constexpr int kRowsPerLoad = 128 / TN;
  const unsigned b_lds = lds_addr_of(Bs + wave * 128);
  const unsigned b_voff = (unsigned)(((lane / (TN / 2)) * sg.ldbt + 2 * (lane % (TN / 2))) * 8);
  const double* b_base = sg.Bt + sg.b_col0 + (GATHER ? 0 : (int64_t)wave * kRowsPerLoad * sg.ldbt);
  auto issue = [&](int st) {
    const int u = st >> 6;
    const int c = __builtin_amdgcn_readlane(u == 0 ? kq[0] : u == 1 ? kq[1] : u == 2 ? kq[2] : kq[3], st & 63);
    const int b = st % kSegS;
    if constexpr (GATHER) {
      lds_dma16(a_base + (int64_t)(c < 0 ? 0 : c) * lda, a_voff, a_lds + (unsigned)(b * kStageA * 8));
      lds_dma16(b_base + (int64_t)(c < 0 ? sg.zero_row : c) * sg.ldbt, b_voff, b_lds + (unsigned)(b * kStageB * 8));
    } else {
      lds_dma16(a_base + (int64_t)c * lda, a_voff, a_lds + (unsigned)(b * kStageA * 8));
      if (wave < kBLoads) lds_dma16(b_base + (int64_t)st * kSegKS * sg.ldbt, b_voff, b_lds + (unsigned)(b * kStageB * 8));
    }
  };
  // transfers a wave has in flight per stage (vmcnt is per wave)
  const bool two = wave < kBLoads;

  double4_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};

#pragma unroll
  for (int st = 0; st < kSegS - 1; ++st)
    if (st < nst) issue(st);

  for (int t = 0; t < nst; ++t) {
    // this wave's transfers of stage t have landed (those of up to two later stages may be in flight) ...
    const int ahead = nst - 1 - t;
    if (two) {
      if (ahead >= kSegS - 2) wait_vm<2 * (kSegS - 2)>();
      else if (ahead == 1) wait_vm<2>();
      else wait_vm<0>();
    } else {
      if (ahead >= kSegS - 2) wait_vm<kSegS - 2>();
      else if (ahead == 1) wait_vm<1>();
      else wait_vm<0>();
    }
    if constexpr (GATHER) {
      // a set's first tile: column 0 of the row this wave brought is the centre's entry, not the shared matrix's
      if (centre_tile) {
        const int u = t >> 6;
        const double cu = u == 0 ? cq[0] : u == 1 ? cq[1] : u == 2 ? cq[2] : cq[3];
        const int lo = __builtin_amdgcn_readlane((int)(unsigned)(__double_as_longlong(cu) & 0xffffffffll), t & 63);
        const int hi = __builtin_amdgcn_readlane((int)(__double_as_longlong(cu) >> 32), t & 63);
        if (lane == 0) Bs[(t % kSegS) * kStageB + wave * TN] = __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
        __builtin_amdgcn_s_waitcnt(0xf | (0x3 << 14) | (0x7 << 4) | (0x0 << 8));  // lgkmcnt(0): the patch is in LDS
      }
    }
    block_barrier();  // ... and everybody's; everybody is done with stage t - 1, whose buffer the next transfer takes
    if (t + kSegS - 1 < nst) issue(t + kSegS - 1);
    const double* as = As + (t % kSegS) * kStageA + wr * (16 * FM) + l16 * FM;
    const double* bs = Bs + (t % kSegS) * kStageB + wc * (16 * FN) + l16 * FN;
#pragma unroll
    for (int s = 0; s < kSegKS / 4; ++s) {
      const int k = s * 4 + q;
      double wv[FM], vv[FN];
      if constexpr (FM == 4) {
        const double2_t w01 = *reinterpret_cast<const double2_t*>(as + k * kSegTM);
        const double2_t w23 = *reinterpret_cast<const double2_t*>(as + k * kSegTM + 2);
        wv[0] = w01[0], wv[1] = w01[1], wv[2] = w23[0], wv[3] = w23[1];
      } else if constexpr (FM == 2) {
        const double2_t w01 = *reinterpret_cast<const double2_t*>(as + k * kSegTM);
        wv[0] = w01[0], wv[1] = w01[1];
      } else {
        wv[0] = as[k * kSegTM];
      }
      if constexpr (FN == 2) {
        const double2_t v01 = *reinterpret_cast<const double2_t*>(bs + k * TN);
        vv[0] = v01[0], vv[1] = v01[1];
      } else {
        vv[0] = bs[k * TN];
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(vv[j], wv[i], acc[i][j], 0, 0, 0);
    }
  }
  // lane (l16, q), accumulator (i, j), register r: row = wr*16*FM + l16*FM + i, column = wc*16*FN + (q + 4r)*FN + j

  // ---- fused estimateRanges: partial sums of this column tile ------------------------------------
  // xmin1 = sum max(v,0)*plb, xmin2 = sum min(v,0)*pub, xmax1 = sum max(v,0)*pub, xmax2 = sum min(v,0)*plb
  if (sg.rpart != nullptr) {
    if (tid < 2 * TN) pbs[tid / TN][tid % TN] = pb_reg;
    __syncthreads();  // the stages are free, the bounds in place
    double* red = smem;
    double s[4][FM];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int i = 0; i < FM; ++i) s[a][i] = 0.0;
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int ct = wc * (16 * FN) + (q + 4 * r) * FN + j;
        const double pl = pbs[0][ct], pu = pbs[1][ct];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const double v = acc[i][j][r];
          const double p = fmax(v, 0.0), n = fmin(v, 0.0);
          s[0][i] = fma(p, pl, s[0][i]);
          s[1][i] = fma(n, pu, s[1][i]);
          s[2][i] = fma(p, pu, s[2][i]);
          s[3][i] = fma(n, pl, s[3][i]);
        }
      }
    const int part = wc * 4 + q;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      double* dst = red + (part * 4 + a) * kSegTM + wr * (16 * FM) + l16 * FM;
#pragma unroll
      for (int i = 0; i < FM; ++i) dst[i] = s[a][i];
    }
    __syncthreads();
    {  // the partial sums of a row are added in a fixed order
      const int row = tid & (kSegTM - 1), a = tid >> 7;
      double sum = 0.0;
#pragma unroll
      for (int pp = 0; pp < WC * 4; ++pp) sum += red[(pp * 4 + a) * kSegTM + row];
      if (m0 + row < Mp) sg.rpart[(int64_t)a * ldc + m0 + row] = sum;
    }
  }

  // ---- epilogue: bias on a set's centre column, FM consecutive rows per store -----------------------
  const int row = m0 + wr * (16 * FM) + l16 * FM;
  if (row < Mp) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int ct = wc * (16 * FN) + (q + 4 * r) * FN + j;
        if (ct < sg.valid) {
          double v[FM];
#pragma unroll
          for (int i = 0; i < FM; ++i) v[i] = acc[i][j][r];
          if (bias != nullptr && sg.col_local0 + ct == 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i) v[i] = v[i] + bias[row + i];
          }
          double* dst = C + (sg.col_base + ct) * ldc + row;
          if constexpr (FM == 1) {
            dst[0] = v[0];
          } else {
#pragma unroll
            for (int i = 0; i < FM; i += 2) *reinterpret_cast<double2_t*>(dst + i) = double2_t{v[i], v[i + 1]};
          }
        }
      }
  }
}

// Packs the listed rows of a set's leading columns transposed: Vt(t, j) = V(kept[t], j) for t < kp
// (zero where kept[t] < 0) and j < ncols, zero for ncols <= j < ldt; Vt is kp x ldt, row-major.  A block
// transposes a 64 x 64 piece through LDS: it reads like pack_rows_kernel (lanes along the kept rows of one
// column) and writes 512 contiguous bytes per row, 16 per lane.
__global__ __launch_bounds__(256) void pack_rows_t_kernel(const PackSet* __restrict__ table, PackSet one) {
  const PackSet d = table ? table[blockIdx.z] : one;
  const int t0 = blockIdx.x * 64, j0 = blockIdx.y * 64;
  if (t0 >= d.kp || j0 >= d.ldt) return;
  __shared__ double tile[64][65];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int t = t0 + lane;
  const int ra = t < d.kp ? d.kept[t] : -1;
  int ha = 0, wa = 0;  // image position of the row, for columns that are only defined inside their windows
  if (d.box != nullptr) {
    const int pa = max(ra, 0) % (d.bH * d.bW);
    wa = pa / d.bH, ha = pa - wa * d.bH;
  }
  for (int cc = wave; cc < 64; cc += 4) {
    const int j = j0 + cc;
    double v = 0.0;
    bool in = ra >= 0 && j < d.ncols && !(j >= 1 && j < d.zero_to);
    if (in && d.box != nullptr && j >= d.box_from && j < d.box_to) {
      const ColBox b = d.box[j];
      in = ha >= b.h0 && ha <= b.h1 && wa >= b.w0 && wa <= b.w1;
    }
    if (in) {
      if (d.W != nullptr && j >= d.wfrom && j < d.wend) {  // the value the gather pass wrote, recomputed
        const int src = d.widx[j - d.wfrom];
        const double sc = d.wscale ? d.wscale[src] : 1.0;
        v = __dadd_rn(0.0, __dmul_rn(d.W[(int64_t)src * d.ldw + ra], sc));
      } else {
        v = d.V[(int64_t)j * d.ld + ra];
      }
    }
    tile[cc][lane] = v;
  }
  __syncthreads();
  // two columns per lane (16-byte stores), two rows per wave and pass; ldt is even
  const int jl = 2 * (lane & 31), kh = lane >> 5;
  if (j0 + jl < d.ldt)
    for (int kk = 2 * wave + kh; kk < 64 && t0 + kk < d.kp; kk += 8)
      *reinterpret_cast<double2_t*>(d.Vk + (int64_t)(t0 + kk) * d.ldt + j0 + jl) = double2_t{tile[jl][kk], tile[jl + 1][kk]};
}

// The same packing when every column but the centre is a scaled weight column and the weights are at hand
// row-major: row t of Vt is a row of the weights, read and written contiguously.  The weights are larger than
// an XCD's L2, so the grid walks them in slices of kPackSlice rows with the sets innermost (blockIdx.x = set):
// while a slice is being read by every set it stays in the cache.  Block (set, slice) packs the kept rows of the
// set that fall into the slice (the list is ascending; its -1 padding belongs to the last slice).
constexpr int kPackSlice = 64;
__global__ __launch_bounds__(256) void pack_rows_t_direct_kernel(const PackSet* __restrict__ table, PackSet one, int slices) {
  const PackSet d = table ? table[blockIdx.x] : one;
  const int lo_row = blockIdx.y * kPackSlice, hi_row = lo_row + kPackSlice;
  // first entry >= lo_row and first entry >= hi_row among the real (non-negative, ascending) entries
  int nreal = 0;
  {
    int a = 0, b = d.kp;  // first padding entry
    while (a < b) {
      const int m = (a + b) >> 1;
      if (d.kept[m] >= 0) a = m + 1; else b = m;
    }
    nreal = a;
  }
  auto lower = [&](int row) {
    int a = 0, b = nreal;
    while (a < b) {
      const int m = (a + b) >> 1;
      if (d.kept[m] < row) a = m + 1; else b = m;
    }
    return a;
  };
  const int t0 = lower(lo_row);
  const int t1 = (int)blockIdx.y == slices - 1 ? d.kp : lower(hi_row);
  // a thread's four columns (and, if a row is longer than 1024 columns, the ones 1024 further on) and what they
  // read do not depend on the row: weight column and scale are looked up once, the rows then stream out in
  // 16-byte pieces.  Short rows (the narrow last tile of a set packed on its own) share the block's threads:
  // 256 / (ldt / 4) rows per pass.
  constexpr int kQ = 4;
  const int qpr = min(d.ldt / kQ, 256);  // column quads of a row that one pass covers
  const int rp = 256 / qpr;              // rows per pass
  const int q = (int)threadIdx.x % qpr, ro = (int)threadIdx.x / qpr;
  for (int jb = 0; jb < d.ldt; jb += qpr * kQ) {
    const int j0 = jb + kQ * q;
    int src[kQ];
    double sc[kQ];
    int kind[kQ];  // 0: zero, 1: the centre, 2: a weight column
#pragma unroll
    for (int e = 0; e < kQ; ++e) {
      const int j = j0 + e;
      src[e] = 0;
      sc[e] = 0.0;
      kind[e] = 0;
      if (j < d.ncols) {
        const int js = d.col0 + j;  // the set's column
        if (js == 0) {
          kind[e] = 1;
        } else if (js >= d.zero_to) {
          kind[e] = 2;
          src[e] = d.widx[js - d.wfrom];
          sc[e] = d.wscale ? d.wscale[src[e]] : 1.0;
        }
      }
    }
    if (j0 >= d.ldt || ro >= rp) continue;  // (ldt is a multiple of four)
#pragma unroll 2
    for (int t = t0 + ro; t < t1; t += rp) {
      const int ra = d.kept[t];
      const double* wrow = d.Wt + (int64_t)max(ra, 0) * d.ldwt;
      double* dst = d.Vk + (int64_t)t * d.ldt + j0;
      double v[kQ];
#pragma unroll
      for (int e = 0; e < kQ; ++e) {
        v[e] = 0.0;
        if (ra >= 0 && kind[e] == 2) v[e] = __dadd_rn(0.0, __dmul_rn(wrow[src[e]], sc[e]));
        if (ra >= 0 && kind[e] == 1) v[e] = d.V[ra];
      }
      *reinterpret_cast<double2_t*>(dst) = double2_t{v[0], v[1]};
      *reinterpret_cast<double2_t*>(dst + 2) = double2_t{v[2], v[3]};
    }
  }
}

template <int TN, int WR, int WC, int FM, int FN, bool GATHER = false>
int launch_seg_cfg(nnvhip_ctx* ctx, const double* A, int64_t lda, double* C, int64_t ldc, int64_t Mp, const double* bias,
                   const SegTile* segs, int64_t ntiles, double flop) {
  const int64_t tiles_m = ceil_div(Mp, kSegTM);
  if (tiles_m * ntiles >= (int64_t(1) << 28)) NNV_FAIL(NNVHIP_ERR_SHAPE, "matrix too large for one launch");
  // all row tiles of a column tile on one XCD, next to one another: the tile's packed rows are fetched once
  // and the gathered columns of W (short row lists) stay in that XCD's L2
  const int64_t xr = 1, local_m = tiles_m;
  const int64_t slots = local_m * ceil_div(ntiles, 8 / xr);
  const bool timed = ctx->kernel_timing;
  NNV_LAUNCH(ctx, timed, (gemm_seg_kernel<TN, WR, WC, FM, FN, GATHER>), dim3((unsigned)(8 * slots)), dim3(kSegNT), 0, A, lda, C, ldc, (int)Mp,
             bias, (int)tiles_m, ntiles, (int)xr, (int)local_m, segs);
  NNV_TRY(ctx->kernel_timer_end(timed, 9, flop));  // a timing group of its own
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

}  // namespace

int launch_pack_rows_t(nnvhip_ctx* ctx, int64_t count, const PackSet* sets) {
  if (count <= 0) return NNVHIP_OK;
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  int64_t max_kp = 0, max_ld = 0;
  for (int64_t i = 0; i < count; ++i) {
    if (sets[i].ldt % 2) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: packed rows must have an even length");
    max_kp = std::max<int64_t>(max_kp, sets[i].kp);
    max_ld = std::max<int64_t>(max_ld, sets[i].ldt);
  }
  if (max_kp == 0 || max_ld == 0) return NNVHIP_OK;
  const PackSet* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(ctx->upload_table(sets, sizeof(PackSet) * count, &tab));
    table = tab->as<PackSet>();
  }
  // every column but the centre a scaled weight column, the weights at hand row-major, no windows: rows of the weights
  bool direct = true;
  int64_t wrows = 0;
  for (int64_t i = 0; i < count; ++i) {
    direct = direct && sets[i].Wt != nullptr && sets[i].wfrom == 1 && sets[i].wend >= sets[i].col0 + sets[i].ncols &&
             sets[i].box == nullptr && sets[i].ldt % 4 == 0;
    wrows = std::max<int64_t>(wrows, sets[i].wrows);
  }
  direct = direct && wrows > 0 && ceil_div(wrows, kPackSlice) <= 65535;
  for (int64_t i = 0; i < count; ++i)
    if (sets[i].col0 != 0 && !direct) NNV_FAIL(NNVHIP_ERR_ARG, "internal: a column offset needs the rows of the weights");
  if (direct) {
    const int slices = (int)ceil_div(wrows, kPackSlice);
    hipLaunchKernelGGL(pack_rows_t_direct_kernel, dim3((unsigned)count, (unsigned)slices), dim3(256), 0, ctx->stream, table, sets[0],
                       slices);
    NNV_HIP_TRY(hipGetLastError());
    return NNVHIP_OK;
  }
  hipLaunchKernelGGL(pack_rows_t_kernel, dim3((unsigned)ceil_div(max_kp, 64), (unsigned)ceil_div(max_ld, 64), (unsigned)count), dim3(256),
                     0, ctx->stream, table, sets[0]);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

namespace {
__global__ __launch_bounds__(256) void scaled_rows_kernel(ScaledRows a) {
  const ScaledRows::One d = a.s[blockIdx.y];
  const int r = blockIdx.x;  // row `rows` is the row of zeros
  if (r > d.rows) return;
  double* o = d.out + (int64_t)r * d.ld;
  const double* w = d.Wt + (int64_t)min(r, d.rows - 1) * d.ldwt;
  for (int j = threadIdx.x; j < d.ld; j += 256) {
    double v = 0.0;
    if (r < d.rows && j >= 1 && j < d.ncols) {  // the value the gather pass would write, as the packing kernels form it
      const int src = d.idx[j - 1];
      v = __dadd_rn(0.0, __dmul_rn(w[src], d.scale ? d.scale[src] : 1.0));
    }
    o[j] = v;
  }
}
}  // namespace

int launch_scaled_rows(nnvhip_ctx* ctx, const ScaledRows& a) {
  if (a.count < 1 || a.count > 16) NNV_FAIL(NNVHIP_ERR_ARG, "internal: one to sixteen matrices per launch");
  int32_t max_rows = 0;
  for (int k = 0; k < a.count; ++k) {
    if (a.s[k].rows <= 0 || a.s[k].ncols > a.s[k].ld) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: scaled rows out of range");
    max_rows = std::max(max_rows, a.s[k].rows);
  }
  hipLaunchKernelGGL(scaled_rows_kernel, dim3((unsigned)(max_rows + 1), (unsigned)a.count), dim3(256), 0, ctx->stream, a);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

int launch_gemm_seg(nnvhip_ctx* ctx, const double* A, int64_t lda, double* C, int64_t ldc, int64_t Mp, const double* bias,
                    int tn, const SegTile* segs, int64_t ntiles, double flop, bool gather_b) {
  if (ntiles == 0) return NNVHIP_OK;
  if (Mp % 16 || lda % 2 || Mp > ldc) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: GEMM operands violate the padding contract");
  if (gather_b && tn != 128) NNV_FAIL(NNVHIP_ERR_ARG, "internal: rows of B are gathered by the 128-column tile only");
  if (gather_b) return launch_seg_cfg<128, 2, 4, 4, 2, true>(ctx, A, lda, C, ldc, Mp, bias, segs, ntiles, flop);
  switch (tn) {
    case 128: return launch_seg_cfg<128, 2, 4, 4, 2>(ctx, A, lda, C, ldc, Mp, bias, segs, ntiles, flop);
    case 64: return launch_seg_cfg<64, 4, 2, 2, 2>(ctx, A, lda, C, ldc, Mp, bias, segs, ntiles, flop);
    case 32: return launch_seg_cfg<32, 4, 2, 2, 1>(ctx, A, lda, C, ldc, Mp, bias, segs, ntiles, flop);
  }
  NNV_FAIL(NNVHIP_ERR_ARG, "internal: no tile of %d columns", tn);
}

}  // namespace nnvhip
