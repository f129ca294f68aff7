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

// ---- row lists of an array of sets against their group's majority list --------------------------------------
__global__ __launch_bounds__(256) void vote_rows_kernel(const DeltaSet* __restrict__ sets, int32_t* __restrict__ votes, int rows) {
  const DeltaSet d = sets[blockIdx.x];
  for (int t = threadIdx.x; t < d.kp; t += 256) {
    const int r = d.kept[t];
    if (r >= 0 && r < rows) atomicAdd(&votes[(int64_t)d.group * rows + r], 1);
  }
}

// one block per group: the rows more than half of the group's sets keep, ascending, -1 padded to a multiple of 16
__global__ __launch_bounds__(1024) void common_rows_kernel(const int32_t* __restrict__ votes, const int32_t* __restrict__ group_size,
                                                           int rows, int rows_pad, int32_t* __restrict__ common,
                                                           int32_t* __restrict__ ncommon) {
  const int g = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = group_size[g];
  __shared__ int wsum[16];
  __shared__ int base;
  if (tid == 0) base = 0;
  __syncthreads();
  int32_t* out = common + (int64_t)g * rows_pad;
  for (int r0 = 0; r0 < rows; r0 += 1024) {
    const int r = r0 + tid;
    const bool in = r < rows && 2 * votes[(int64_t)g * rows + r] > half;
    const unsigned long long bal = __ballot(in);
    if (lane == 0) wsum[wave] = __popcll(bal);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wsum[w];
    if (in) out[off + __popcll(bal & ((1ull << lane) - 1))] = r;
    __syncthreads();
    if (tid == 0) {
      int t = 0;
      for (int w = 0; w < 16; ++w) t += wsum[w];
      base += t;
    }
    __syncthreads();
  }
  const int n = base, npad = (n + 15) / 16 * 16;
  for (int t = n + tid; t < npad; t += 1024) out[t] = -1;
  if (tid == 0) ncommon[g] = npad;
}

// one block per set: the rows in which the set's list differs from its group's majority list
__global__ __launch_bounds__(1024) void delta_rows_kernel(const DeltaSet* __restrict__ sets, const int32_t* __restrict__ votes,
                                                          const int32_t* __restrict__ group_size, int rows, int cap,
                                                          int32_t* __restrict__ delta, int32_t* __restrict__ dlen,
                                                          int32_t* __restrict__ head) {
  extern __shared__ unsigned keptbits[];  // one bit per row
  const DeltaSet d = sets[blockIdx.x];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int words = (rows + 31) / 32;
  for (int w = tid; w < words; w += 1024) keptbits[w] = 0u;
  __shared__ int wsum[16];
  __shared__ int base;
  if (tid == 0) base = 0;
  __syncthreads();
  for (int t = tid; t < d.kp; t += 1024) {
    const int r = d.kept[t];
    if (r >= 0 && r < rows) atomicOr(&keptbits[r >> 5], 1u << (r & 31));
  }
  __syncthreads();
  const int half = group_size[d.group];
  int32_t* out = delta + (int64_t)blockIdx.x * cap;
  for (int r0 = 0; r0 < rows; r0 += 1024) {
    const int r = r0 + tid;
    bool kept = false, common = false;
    if (r < rows) {
      kept = (keptbits[r >> 5] >> (r & 31)) & 1u;
      common = 2 * votes[(int64_t)d.group * rows + r] > half;
    }
    const bool diff = kept != common;
    const unsigned long long bal = __ballot(diff);
    if (lane == 0) wsum[wave] = __popcll(bal);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wsum[w];
    if (diff) {
      const int pos = off + __popcll(bal & ((1ull << lane) - 1));
      if (pos < cap) out[pos] = kept ? r : (r | kSegSubtract);  // kept but not common: add; common but not kept: take away
    }
    __syncthreads();
    if (tid == 0) {
      int t = 0;
      for (int w = 0; w < 16; ++w) t += wsum[w];
      base += t;
    }
    __syncthreads();
  }
  const int n = base;
  if (n > cap) {
    if (tid == 0) dlen[blockIdx.x] = -1;
    return;
  }
  const int npad = (n + kSegKS - 1) / kSegKS * kSegKS;
  for (int t = n + tid; t < npad; t += 1024) out[t] = -1;
  if (tid == 0) dlen[blockIdx.x] = n;
  // the first four entries once more, next to the lengths: what the host reads back with them
  if (tid < 4) head[4 * blockIdx.x + tid] = tid < n ? out[tid] : -1;
}

// Sets that start from their group's shared product (DeltaOut).  A block takes 128 rows x 64 columns of that product
// into registers once (four waves of 16 columns each, a lane owns two adjacent rows) and then writes that piece of
// one set after the other of a batch of sets of the group: per set the few rank-one terms of its row differences,
// the four range sums of the piece, and 16-byte streaming stores.  The shared product is read once per batch, so
// the pass moves little more than the bytes it writes.
constexpr int kDeltaCols = 64;  // columns of a block's piece = columns per chunk of range sums
struct DeltaBatch {
  int32_t first, nsets;  // sets [first, first + nsets) of the table, all of one group
};
// Entry `src_lane` (wave-uniform) of a value that the lanes of a wave hold one each.
__device__ __forceinline__ double readlane_f64(double v, int src_lane) {
  const int lo = __builtin_amdgcn_readlane(__double2loint(v), src_lane);
  const int hi = __builtin_amdgcn_readlane(__double2hiint(v), src_lane);
  return __hiloint2double(hi, lo);
}

// A set's description with the first four entries of its difference list beside it: one trip to memory tells a block
// everything it needs to ask for the set's operands.
struct DeltaRec {
  DeltaOut d;
  int32_t e4[4];  // -1: no such entry
};
__global__ __launch_bounds__(256) void delta_recs_kernel(const DeltaOut* __restrict__ sets, DeltaRec* __restrict__ recs, int count) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  DeltaRec r;
  r.d = sets[i];
#pragma unroll
  for (int t = 0; t < 4; ++t) r.e4[t] = t < r.d.dlen ? r.d.delta[t] : -1;
  recs[i] = r;
}

__global__ __launch_bounds__(256) void delta_tiles_kernel(const DeltaRec* __restrict__ recs, const DeltaBatch* __restrict__ batches,
                                                          const double* __restrict__ A, int64_t lda, int Mp,
                                                          const double* __restrict__ bias, int64_t ldo) {
  const DeltaBatch bt = batches[blockIdx.z];
  const DeltaOut d0 = recs[bt.first].d;
  const int cc = blockIdx.x, rb = blockIdx.y;
  const int j0 = cc * kDeltaCols;
  if (j0 >= d0.ncols) return;  // (the sets of a group have the same columns)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r0 = rb * 128 + 2 * lane;
  const bool active = r0 < Mp;
  const int jw = j0 + 16 * wave;                // this wave's first column
  const int nj = max(0, min(16, d0.ncols - jw));  // ... and how many it has
  double2_t base[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    base[u] = double2_t{0.0, 0.0};
    if (active && u < nj) base[u] = *reinterpret_cast<const double2_t*>(d0.base + (int64_t)(jw + u) * Mp + r0);
  }
  __shared__ double2_t red[2][3][4][64];  // the sums of waves 1-3 of a set, two sets in flight
  // What a set brings besides the shared piece.  Its row differences (usually a handful): the first four come with
  // the set's record, and the weight column entries of the lane's rows and the rows of the shared operand they name
  // are looked up once per set; any more go through the loop per column.  What the wave's sixteen columns need of
  // those rows and the columns' predicate bounds is read by lane u (mod 16) for column u and handed round by lane
  // reads: one load each instead of a scalar load per column and value.  The look-ups run ahead of the arithmetic:
  // while set s is worked on, the operands of set s + 1 are in flight and the record of set s + 2 is on its way, so
  // that no set waits for its two dependent trips to memory (1.49 -> 1.22-1.39 ms for 6.7 GB of output; with the
  // stores left out the same loop is bound by its instruction count - 420 vector and 270 scalar instructions per
  // set and wave - which is why the pass that stores nothing is a kernel of its own, further down).
  struct SetOps {
    double2_t w4[4];
    double sv4[4];
    double pl16, pu16;
  };
  const int lcol = lane & 15;
  const bool lcol_in = lcol < nj;
  auto operands = [&](const DeltaRec& q, SetOps& o) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int r = max(q.e4[t], 0) & (kSegSubtract - 1);
      o.w4[t] = double2_t{0.0, 0.0};
      if (q.e4[t] >= 0 && active) o.w4[t] = *reinterpret_cast<const double2_t*>(A + (int64_t)r * lda + r0);
      if (q.e4[t] >= 0 && (q.e4[t] & kSegSubtract)) o.w4[t] = -o.w4[t];  // the row is taken away: -(w * s) = (-w) * s
      o.sv4[t] = (q.e4[t] >= 0 && lcol_in) ? q.d.S[(int64_t)r * q.d.lds + jw + lcol] : 0.0;
    }
    o.pl16 = o.pu16 = 0.0;
    if (q.d.rpart != nullptr && lcol_in && jw + lcol >= 1) {
      o.pl16 = q.d.plb[jw + lcol - 1];
      o.pu16 = q.d.pub[jw + lcol - 1];
    }
  };
  DeltaRec rec = recs[bt.first];                                     // set s
  DeltaRec rec1 = recs[bt.first + min(1, bt.nsets - 1)];             // set s + 1
  SetOps cur, nxt;
  operands(rec, cur);
  for (int s = 0; s < bt.nsets; ++s) {
    if (s + 1 < bt.nsets) operands(rec1, nxt);                       // (its record arrived an iteration ago)
    const DeltaRec rec2 = recs[bt.first + min(s + 2, bt.nsets - 1)];  // asked for now, read at the top of the next round
    const DeltaOut& d = rec.d;
    const int(&e4)[4] = rec.e4;
    const double2_t(&w4)[4] = cur.w4;
    const double(&sv4)[4] = cur.sv4;
    const double pl16 = cur.pl16, pu16 = cur.pu16;
    double2_t x1 = {0.0, 0.0}, x2 = {0.0, 0.0}, y1 = {0.0, 0.0}, y2 = {0.0, 0.0};
    // Columns whose predicate bounds mirror each other (plb = -pub: every generator of a box star) make xmin1 the
    // mirror image of xmax1 and xmax2 that of xmin2, rounding included (fl(a * (-p) + (-s)) = -fl(a * p + s)): half
    // of the products are then left out and the two sums negated at the end.
    const bool mirrored = d.rpart != nullptr && __all(pl16 == -pu16);
    if (active && nj > 0) {
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        if (u < nj) {
          const int j = jw + u;
          double2_t o = base[u];
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (e4[t] >= 0) {
              const double sv = readlane_f64(sv4[t], u);
              o[0] = fma(w4[t][0], sv, o[0]);
              o[1] = fma(w4[t][1], sv, o[1]);
            }
          for (int t = 4; t < d.dlen; ++t) {
            const int e = d.delta[t];
            const int r = e & (kSegSubtract - 1);
            const double2_t w = *reinterpret_cast<const double2_t*>(A + (int64_t)r * lda + r0);
            double sv = d.S[(int64_t)r * d.lds + j];
            if (e & kSegSubtract) sv = -sv;
            o[0] = fma(w[0], sv, o[0]);
            o[1] = fma(w[1], sv, o[1]);
          }
          if (j == 0) {  // the centre is the set's own product, bias last
            o = *reinterpret_cast<const double2_t*>(d.cprod + r0);
            if (bias != nullptr) {
              o[0] = o[0] + bias[r0];
              o[1] = o[1] + bias[r0 + 1];
            }
          } else if (d.rpart != nullptr) {
            const double pl = readlane_f64(pl16, u), pu = readlane_f64(pu16, u);
            const double px = fmax(o[0], 0.0), nx = fmin(o[0], 0.0), py = fmax(o[1], 0.0), ny = fmin(o[1], 0.0);
            x2[0] = fma(nx, pu, x2[0]);
            x2[1] = fma(ny, pu, x2[1]);
            y1[0] = fma(px, pu, y1[0]);
            y1[1] = fma(py, pu, y1[1]);
            if (!mirrored) {
              x1[0] = fma(px, pl, x1[0]);
              x1[1] = fma(py, pl, x1[1]);
              y2[0] = fma(nx, pl, y2[0]);
              y2[1] = fma(ny, pl, y2[1]);
            }
          }
          // (streaming store: the output is not read again here)
          __builtin_nontemporal_store(o, reinterpret_cast<double2_t*>(d.out + (int64_t)j * ldo + r0));
        }
      }
    }
    if (d.rpart == nullptr) {  // (all sets of a call agree on this)
      rec = rec1;
      rec1 = rec2;
      cur = nxt;
      continue;
    }
    if (mirrored) {  // (0 - s: a sum that is still +0 stays +0, as the left-out additions of -0 would have left it)
      x1 = double2_t{0.0 - y1[0], 0.0 - y1[1]};
      y2 = double2_t{0.0 - x2[0], 0.0 - x2[1]};
    }

    const int par = s & 1;
    if (wave > 0) {
      red[par][wave - 1][0][lane] = x1;
      red[par][wave - 1][1][lane] = x2;
      red[par][wave - 1][2][lane] = y1;
      red[par][wave - 1][3][lane] = y2;
    }
    // one barrier per set: wave 0 reads this buffer before it reaches the next barrier, and the buffer is written
    // again only after that one (two sets later).  The barrier waits for the LDS writes only: __syncthreads would
    // also sit out the round trip of every output store in flight.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (wave == 0 && active) {
      for (int w = 0; w < 3; ++w) {  // the waves in order
        x1 += red[par][w][0][lane];
        x2 += red[par][w][1][lane];
        y1 += red[par][w][2][lane];
        y2 += red[par][w][3][lane];
      }
      double* dst = d.rpart + (int64_t)cc * 4 * ldo + r0;
      *reinterpret_cast<double2_t*>(dst) = x1;            // xmin1 = sum max(v,0)*plb
      *reinterpret_cast<double2_t*>(dst + ldo) = x2;      // xmin2 = sum min(v,0)*pub
      *reinterpret_cast<double2_t*>(dst + 2 * ldo) = y1;  // xmax1 = sum max(v,0)*pub
      *reinterpret_cast<double2_t*>(dst + 3 * ldo) = y2;  // xmax2 = sum min(v,0)*plb
    }
    rec = rec1;
    rec1 = rec2;
    cur = nxt;
  }
}

// The pass that stores no matrix.  What a set adds to the shared piece is a product of rank four or less - (its
// rows' weight entries) x (those rows of the shared operand) - which is one 16x16x4 MFMA per 16 x 16 outputs with
// the shared piece as the accumulator going in (none for a set without differences, further ones for lists of more
// than four entries).  fp64 MFMA runs at the rate of the vector unit's fp64 FMAs and shares it: the instruction
// saves no time for the product itself but takes its operands per lane as they come from memory, where the
// vector form (the pass above) hands every operand round by lane reads: 421 vector + 266 scalar instructions per
// set and wave there, about 230 + 80 here.  A wave owns 32 rows x 64 columns (2 x 4 such tiles, held in registers
// for the batch of sets as above); the instruction's "a" operand carries columns and its "b" operand rows, so that
// result register r of lane l is O[row l % 16][column l / 16 + 4r]: a lane multiplies its four outputs by the
// bounds of its own four columns, the sums over all of the wave's columns are left in four lane groups, and two
// lane exchanges finish them - no LDS, no barrier.  Four waves of a block cover the 128 rows of the other pass's
// block, and a block's columns are one chunk of range sums there as here.
//
// What the pass reads of a set ahead of its turn (SumRec) and at its turn (SumTail).
struct SumRec {
  const double* pub;
  int32_t e4[4];  // the first four entries of the set's list; -1: no such entry
  int32_t dlen;
  int32_t flags;  // kSumMirrored, kSumSameAsLast
};
constexpr int32_t kSumMirrored = 1;    // every predicate of the set has plb = -pub (the sums then need one of the two)
constexpr int32_t kSumSameAsLast = 2;  // group, list and bounds are those of the set before it in the table: so are its sums
struct SumTail {
  const double* plb;
  double* rpart;
  const double* cprod;
  double* out;
  const int32_t* delta;
};
// One block per set.
__global__ __launch_bounds__(256) void delta_sum_recs_kernel(const DeltaOut* __restrict__ sets, SumRec* __restrict__ recs,
                                                             SumTail* __restrict__ tails, int shortcuts) {
  const int i = blockIdx.x;
  const int tid = threadIdx.x;
  const DeltaOut d = sets[i];
  const DeltaOut p = sets[max(i - 1, 0)];
  const bool alike = i > 0 && p.base == d.base && p.S == d.S && p.ncols == d.ncols && p.dlen == d.dlen;  // (the same for all threads)
  bool mine = true, eq = alike;
  for (int j = tid; j < d.ncols - 1; j += 256) {
    const double lo = d.plb[j], hi = d.pub[j];
    mine = mine && lo == -hi;
    if (alike)  // (to the bit: a zero's sign shows in the sums)
      eq = eq && __double_as_longlong(p.plb[j]) == __double_as_longlong(lo) && __double_as_longlong(p.pub[j]) == __double_as_longlong(hi);
  }
  if (alike)
    for (int t = tid; t < d.dlen; t += 256) eq = eq && p.delta[t] == d.delta[t];
  const bool mirrored = __syncthreads_and(mine) != 0;
  const bool same = __syncthreads_and(eq) != 0;
  if (tid == 0) {
    SumRec r;
    r.pub = d.pub;
#pragma unroll
    for (int t = 0; t < 4; ++t) r.e4[t] = t < d.dlen ? d.delta[t] : -1;
    r.dlen = d.dlen;
    r.flags = shortcuts ? (mirrored ? kSumMirrored : 0) | (same ? kSumSameAsLast : 0) : 0;
    recs[i] = r;
    tails[i] = SumTail{d.plb, d.rpart, d.cprod, d.out, d.delta};
  }
}

// Where the sums of set i of the table are: its own chunks, or - for a set the pass finds equal to the one before it
// in its batch - those of the set the run started with (the pass writes them once).
__global__ __launch_bounds__(256) void delta_sum_alias_kernel(const SumRec* __restrict__ recs, const DeltaOut* __restrict__ sets,
                                                              const int32_t* __restrict__ batch_first, const double** __restrict__ at,
                                                              int count) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  int k = i;
  while (k > batch_first[i] && (recs[k].flags & kSumSameAsLast) != 0) --k;
  at[i] = sets[k].rpart;
}

typedef const double __attribute__((address_space(1)))* gdouble_t;  // (a pointer known to be to device memory)
__device__ __forceinline__ gdouble_t in_global(const double* p) { return (gdouble_t)p; }
__device__ __forceinline__ double max0(double v) {  // (fmax / fmin without the pass that quiets signalling NaNs first)
  double r;
  asm("v_max_f64 %0, %1, 0" : "=v"(r) : "v"(v));
  return r;
}
__device__ __forceinline__ double min0(double v) {
  double r;
  asm("v_min_f64 %0, %1, 0" : "=v"(r) : "v"(v));
  return r;
}

// Two sums over the halves of a wave at once: lanes 0-31 get a(l) + a(l + 32), lanes 32-63 get b(l - 32) + b(l).
__device__ __forceinline__ double fold32(double a, double b) {
  const auto lo = __builtin_amdgcn_permlane32_swap((unsigned)__double2loint(a), (unsigned)__double2loint(b), false, false);
  const auto hi = __builtin_amdgcn_permlane32_swap((unsigned)__double2hiint(a), (unsigned)__double2hiint(b), false, false);
  return __hiloint2double((int)hi[0], (int)lo[0]) + __hiloint2double((int)hi[1], (int)lo[1]);
}
// ... and over neighbouring 16-lane rows: rows 0 and 2 get c.row0 + c.row1 and c.row2 + c.row3, rows 1 and 3 the same of d.
__device__ __forceinline__ double fold16(double c, double d) {
  const auto lo = __builtin_amdgcn_permlane16_swap((unsigned)__double2loint(c), (unsigned)__double2loint(d), false, false);
  const auto hi = __builtin_amdgcn_permlane16_swap((unsigned)__double2hiint(c), (unsigned)__double2hiint(d), false, false);
  return __hiloint2double((int)hi[0], (int)lo[0]) + __hiloint2double((int)hi[1], (int)lo[1]);
}

// EDGE: the block's columns include column 0 (the centre, which is the set's own and enters no sum) or columns past
// the last; their entries of the shared piece and of the shared operand are made zero, so that they add nothing.
template <bool EDGE, int RT>
__device__ __forceinline__ void delta_sums_body(const SumRec* __restrict__ recs, const SumTail* __restrict__ tails, const DeltaBatch bt,
                                                const double* __restrict__ basep, const double* __restrict__ S, int64_t lds, int ncols,
                                                const double* __restrict__ A, int64_t lda, int Mp, const double* __restrict__ bias,
                                                int64_t ldo, int cc, int row0, bool two) {
  const int lane = threadIdx.x & 63;
  const int l16 = lane & 15, g4 = lane >> 4;
  const int j0 = cc * kDeltaCols;
  int rows[RT];  // (a wave without a second row tile does the first twice)
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) rows[rt] = (rt == 0 || two ? row0 + 16 * rt : row0) + l16;
  const int nct = EDGE ? min(4, (ncols - j0 + 15) / 16) : 4;
  double4_t base[RT][4];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int col = j0 + 16 * ct + g4 + 4 * r;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        base[rt][ct][r] = 0.0;
        if (!EDGE || (col >= 1 && col < ncols)) base[rt][ct][r] = basep[(int64_t)col * Mp + rows[rt]];
      }
    }
  // A set's operands.  "a": entry l / 16 of its list, column l % 16 of column tile ct of the shared operand; "b":
  // the same entry, row l % 16 of row tile rt of the weights; the upper predicate bounds of the lane's sixteen
  // columns.  Each is asked for again - for the next set - right after its last use for this one, so that a whole
  // set's arithmetic lies between the request and the use and no second copy of the registers is needed.
  double sv[4], w[RT], pu[4][4];
  // (an entry that is not there reads row 0 of both operands and makes the weight entries zero)
  auto entry_of = [&](const SumRec& q) { return g4 == 0 ? q.e4[0] : g4 == 1 ? q.e4[1] : g4 == 2 ? q.e4[2] : q.e4[3]; };
  auto column_operand = [&](int e, int ct) {
    const int r = max(e, 0) & (kSegSubtract - 1);
    double v = (in_global(S) + ((int64_t)r * lds + j0 + l16))[16 * ct];  // (rows of S are padded past the last column)
    if (EDGE) {
      const int col = j0 + 16 * ct + l16;
      if (col < 1 || col >= ncols) v = 0.0;
    }
    return v;
  };
  auto row_operand = [&](int e, int row) {
    const int r = max(e, 0) & (kSegSubtract - 1);
    double v = (in_global(A) + (int64_t)r * lda)[row];
    if (e & kSegSubtract) v = -v;  // the row is taken away: -(w * s) = (-w) * s
    if (e < 0) v = 0.0;
    return v;
  };
  auto bounds_of = [&](const double* bounds, int ct, double (&out)[4]) {
    const gdouble_t b = in_global(bounds);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int col = j0 + 16 * ct + g4 + 4 * r;
      // (past the edges: some bound of the set; what it multiplies is zero)
      out[r] = EDGE ? b[min(max(col, 1), ncols - 1) - 1] : (b + (j0 + g4 - 1))[16 * ct + 4 * r];
    }
  };
  SumRec rec = recs[bt.first];                          // set s
  SumRec rec1 = recs[bt.first + min(1, bt.nsets - 1)];  // set s + 1
  {
    const int e = entry_of(rec);
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
      sv[ct] = column_operand(e, ct);
      bounds_of(rec.pub, ct, pu[ct]);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) w[rt] = row_operand(e, rows[rt]);
  }
  // A set that agrees with the one before it in list and bounds (a run of sub-boxes that differ from their
  // group's list in nothing, say) has the same pieces and the same sums: nothing is summed or written for it, and
  // whoever reads its sums is sent to those of the run's first set (delta_sum_alias_kernel).
  for (int s = 0; s < bt.nsets; ++s) {
    const SumRec rec2 = recs[bt.first + min(s + 2, bt.nsets - 1)];  // asked for now, read at the top of the next round
    const SumTail tl = tails[bt.first + s];                         // (needed at the end of the round)
    const bool again = s > 0 && (rec.flags & kSumSameAsLast) != 0;
    const bool ask = (rec1.flags & kSumSameAsLast) == 0;  // the next set needs its operands (the last set's "next" is itself)
    const int e1 = entry_of(rec1);
    if (!again) {
      double x1[RT] = {}, x2[RT] = {}, y1[RT] = {}, y2[RT] = {};
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        if (ct < nct) {
          double4_t o[RT];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) o[rt] = base[rt][ct];
          if (rec.dlen > 0) {  // (a set without differences: the shared piece as it is)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) o[rt] = __builtin_amdgcn_mfma_f64_16x16x4f64(sv[ct], w[rt], o[rt], 0, 0, 0);
          }
          for (int g = 1; 4 * g < rec.dlen; ++g) {  // (the list is padded with -1 to a multiple of 8)
            asm volatile("" ::: "memory");  // (keeps the branch a branch: the rare path is not to be run under an empty mask)
            const int e = tl.delta[4 * g + g4];
            const double sve = column_operand(e, ct);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) o[rt] = __builtin_amdgcn_mfma_f64_16x16x4f64(sve, row_operand(e, rows[rt]), o[rt], 0, 0, 0);
          }
          // Columns whose predicate bounds mirror each other (plb = -pub: every generator of a box star) make xmin1
          // the mirror image of xmax1 and xmax2 that of xmin2, rounding included (fl(a * (-p) + (-s)) =
          // -fl(a * p + s)): half of the products are then left out and the two sums negated at the end.
          if ((rec.flags & kSumMirrored) != 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const double v = o[rt][r];
                x2[rt] = fma(min0(v), pu[ct][r], x2[rt]);
                y1[rt] = fma(max0(v), pu[ct][r], y1[rt]);
              }
          } else {
            asm volatile("" ::: "memory");
            double pl[4];
            bounds_of(tl.plb, ct, pl);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const double v = o[rt][r];
                const double p = max0(v), q = min0(v);
                x1[rt] = fma(p, pl[r], x1[rt]);
                x2[rt] = fma(q, pu[ct][r], x2[rt]);
                y1[rt] = fma(p, pu[ct][r], y1[rt]);
                y2[rt] = fma(q, pl[r], y2[rt]);
              }
          }
          if (ask) {
            sv[ct] = column_operand(e1, ct);
            bounds_of(rec1.pub, ct, pu[ct]);
          }
        }
      }
      if (ask) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) w[rt] = row_operand(e1, rows[rt]);
      }
      // The four lane groups hold different columns of the same rows.  Two lane swaps add them up, two sums at a
      // time: fold32 leaves a(l) + a(l + 32) in the lower half of the wave and the same of b in the upper half,
      // fold16 then adds neighbouring 16-lane rows of two such values - lane row 0 and 1 end up with the finished
      // first sum of row tile 0 and 1, lane row 2 and 3 with the second sum (every sum as (g0 + g2) + (g1 + g3)).
      static_assert(RT == 2, "the lane rows of the finished sums are dealt to two row tiles");
      const int tile = g4 & 1, second = g4 >> 1;
      double* const dst = tl.rpart + (int64_t)cc * 4 * ldo + rows[tile];
      if ((rec.flags & kSumMirrored) != 0) {
        // lane rows 0, 1: xmin2; 2, 3: xmax1; the mirror images go out beside them (0 - s: a sum that is still +0
        // stays +0, as the left-out additions of -0 would have left it)
        const double v = fold16(fold32(x2[0], y1[0]), fold32(x2[1], y1[1]));
        if (tile == 0 || two) {
          dst[(second ? 2 : 1) * ldo] = v;
          dst[(second ? 0 : 3) * ldo] = 0.0 - v;
        }
      } else {
        asm volatile("" ::: "memory");
        const double va = fold16(fold32(x1[0], x2[0]), fold32(x1[1], x2[1]));  // lane rows 0, 1: xmin1; 2, 3: xmin2
        const double vb = fold16(fold32(y1[0], y2[0]), fold32(y1[1], y2[1]));  // xmax1; xmax2
        if (tile == 0 || two) {
          dst[(second ? 1 : 0) * ldo] = va;
          dst[(second ? 3 : 2) * ldo] = vb;
        }
      }
    } else if (ask) {
      asm volatile("" ::: "memory");
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        sv[ct] = column_operand(e1, ct);
        bounds_of(rec1.pub, ct, pu[ct]);
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) w[rt] = row_operand(e1, rows[rt]);
    }
    if (cc == 0 && lane < 16 * RT && (lane < 16 || two)) {  // the centre is the set's own product, bias last
      double c = tl.cprod[row0 + lane];
      if (bias != nullptr) c = c + bias[row0 + lane];
      __builtin_nontemporal_store(c, tl.out + row0 + lane);
    }
    rec = rec1;
    rec1 = rec2;
  }
}

template <int RT>
__global__ __launch_bounds__(256, 2) void delta_sums_kernel(const SumRec* __restrict__ recs, const SumTail* __restrict__ tails,
                                                            const DeltaBatch* __restrict__ batches, const DeltaOut* __restrict__ sets,
                                                            const double* __restrict__ A, int64_t lda, int Mp,
                                                            const double* __restrict__ bias, int64_t ldo) {
  const DeltaBatch bt = batches[blockIdx.z];
  const DeltaOut d0 = sets[bt.first];  // (the sets of a batch are of one group: same shared piece, operand and columns)
  const int cc = blockIdx.x, rb = blockIdx.y;
  const int j0 = cc * kDeltaCols;
  if (j0 >= d0.ncols) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row0 = rb * (64 * RT) + wave * (16 * RT);
  if (row0 >= Mp) return;           // (no barrier in this kernel)
  const bool two = RT == 2 && row0 + 16 < Mp;  // the wave's second row tile exists (Mp is a multiple of 16)
  if (cc == 0 || j0 + kDeltaCols > d0.ncols)
    delta_sums_body<true, RT>(recs, tails, bt, d0.base, d0.S, d0.lds, d0.ncols, A, lda, Mp, bias, ldo, cc, row0, two);
  else
    delta_sums_body<false, RT>(recs, tails, bt, d0.base, d0.S, d0.lds, d0.ncols, A, lda, Mp, bias, ldo, cc, row0, two);
}

__global__ __launch_bounds__(256) void masked_centres_kernel(const CentreSet* __restrict__ sets, double* __restrict__ Cm, int64_t Kp) {
  const CentreSet d = sets[blockIdx.x];
  double* col = Cm + (int64_t)blockIdx.x * Kp;
  for (int t = threadIdx.x; t < d.kp; t += 256) {
    const int r = d.kept[t];
    if (r >= 0) col[r] = d.centre[r];
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

int launch_delta_lists(nnvhip_ctx* ctx, int64_t count, const DeltaSet* sets_dev, int groups, const int32_t* group_size_dev,
                       int64_t rows, int64_t rows_pad, int cap, int32_t* votes, int32_t* common, int32_t* ncommon, int32_t* delta,
                       int32_t* dlen, int32_t* head) {
  if (count <= 0 || groups <= 0 || rows <= 0 || rows >= (int64_t(1) << 30) || cap % kSegKS != 0 || rows_pad % 16 != 0 ||
      rows_pad < rows)
    NNV_FAIL(NNVHIP_ERR_ARG, "internal: row-difference lists out of range");
  const size_t bits = sizeof(unsigned) * (size_t)ceil_div(rows, 32);
  if (bits > (size_t)48 << 10) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: too many rows for the row-difference lists");
  NNV_HIP_TRY(hipMemsetAsync(votes, 0, sizeof(int32_t) * (size_t)groups * (size_t)rows, ctx->stream));
  hipLaunchKernelGGL(vote_rows_kernel, dim3((unsigned)count), dim3(256), 0, ctx->stream, sets_dev, votes, (int)rows);
  hipLaunchKernelGGL(common_rows_kernel, dim3((unsigned)groups), dim3(1024), 0, ctx->stream, votes, group_size_dev, (int)rows,
                     (int)rows_pad, common, ncommon);
  hipLaunchKernelGGL(delta_rows_kernel, dim3((unsigned)count), dim3(1024), bits, ctx->stream, sets_dev, votes, group_size_dev, (int)rows,
                     cap, delta, dlen, head);
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

int delta_tile_chunks(int64_t ncols) { return (int)ceil_div(ncols, kDeltaCols); }

int launch_delta_tiles(nnvhip_ctx* ctx, const double* A, int64_t lda, int64_t Mp, const double* bias, int64_t ldo, int64_t count,
                       const DeltaOut* sets, const int32_t* group_of, int64_t max_cols, double bytes, bool store, BufRef* sums_at) {
  if (sums_at) sums_at->reset();
  if (count <= 0 || max_cols <= 0) return NNVHIP_OK;
  if (Mp % 16 || Mp > ldo || count >= (int64_t(1) << 24)) NNV_FAIL(NNVHIP_ERR_SHAPE, "internal: shared-product tiles out of range");
  // batches of neighbouring sets of one group: long enough to make the read of the shared piece small next to the
  // writes, short enough for a grid that covers the chip a few times over
  const int64_t row_blocks = ceil_div(Mp, 128), col_chunks = ceil_div(max_cols, kDeltaCols);
  int64_t per_batch = 16;
  while (per_batch > 2 && ceil_div(count, per_batch) * row_blocks * col_chunks < 4096) per_batch /= 2;
  std::vector<DeltaBatch> batches;
  for (int64_t a = 0; a < count;) {
    int64_t b = a + 1;
    while (b < count && b - a < per_batch && group_of[b] == group_of[a]) ++b;
    batches.push_back(DeltaBatch{(int32_t)a, (int32_t)(b - a)});
    a = b;
  }
  if (batches.size() > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "array too large for one launch");
  BufRef tab, btab, rtab, ttab;
  NNV_TRY(ctx->upload_table(sets, sizeof(DeltaOut) * count, &tab));
  NNV_TRY(ctx->upload_table(batches.data(), sizeof(DeltaBatch) * batches.size(), &btab));
  const bool timed = ctx->kernel_timing;
  const dim3 grid((unsigned)col_chunks, (unsigned)row_blocks, (unsigned)batches.size());
  if (store) {
    NNV_TRY(ctx->alloc(sizeof(DeltaRec) * (size_t)count, &rtab));
    hipLaunchKernelGGL(delta_recs_kernel, dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, ctx->stream, tab->as<DeltaOut>(),
                       rtab->as<DeltaRec>(), (int)count);
    NNV_LAUNCH(ctx, timed, delta_tiles_kernel, grid, dim3(256), 0, rtab->as<DeltaRec>(), btab->as<DeltaBatch>(), A, lda, (int)Mp, bias, ldo);
  } else {
    for (int64_t i = 0; i < count; ++i)
      if (sets[i].rpart == nullptr || sets[i].ncols < 2) NNV_FAIL(NNVHIP_ERR_ARG, "internal: the pass that stores no matrix is for range sums");
    NNV_TRY(ctx->alloc(sizeof(SumRec) * (size_t)count, &rtab));
    NNV_TRY(ctx->alloc(sizeof(SumTail) * (size_t)count, &ttab));
    if (sums_at == nullptr) NNV_FAIL(NNVHIP_ERR_ARG, "internal: the pass that stores no matrix says where its sums are");
    std::vector<int32_t> first((size_t)count);
    for (const DeltaBatch& b : batches)
      for (int32_t k = 0; k < b.nsets; ++k) first[(size_t)(b.first + k)] = b.first;
    BufRef ftab;
    NNV_TRY(ctx->upload_table(first.data(), sizeof(int32_t) * first.size(), &ftab));
    NNV_TRY(ctx->alloc(sizeof(const double*) * (size_t)count, sums_at));
    hipLaunchKernelGGL(delta_sum_recs_kernel, dim3((unsigned)count), dim3(256), 0, ctx->stream, tab->as<DeltaOut>(), rtab->as<SumRec>(),
                       ttab->as<SumTail>(), ctx->no_sum_shortcuts ? 0 : 1);
    hipLaunchKernelGGL(delta_sum_alias_kernel, dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, ctx->stream, rtab->as<SumRec>(),
                       tab->as<DeltaOut>(), ftab->as<int32_t>(), (*sums_at)->as<const double*>(), (int)count);
    NNV_LAUNCH(ctx, timed, delta_sums_kernel<2>, grid, dim3(256), 0, rtab->as<SumRec>(), ttab->as<SumTail>(), btab->as<DeltaBatch>(),
               tab->as<DeltaOut>(), A, lda, (int)Mp, bias, ldo);
  }
  NNV_TRY(ctx->kernel_timer_end(timed, 10, bytes));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

int launch_masked_centres(nnvhip_ctx* ctx, int64_t count, const CentreSet* sets_dev, double* Cm, int64_t Kp) {
  if (count <= 0) return NNVHIP_OK;
  NNV_HIP_TRY(hipMemsetAsync(Cm, 0, sizeof(double) * (size_t)Kp * (size_t)count, ctx->stream));
  hipLaunchKernelGGL(masked_centres_kernel, dim3((unsigned)count), dim3(256), 0, ctx->stream, sets_dev, Cm, Kp);
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
