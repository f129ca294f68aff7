// A whole reach of a small fully connected network in ONE launch: one 1024-thread block per input set
// walks the layer list of NN.reach_noConns (nn/NN.m:1529-1551) -- Star.affineMap (set/Star.m:313-343),
// Star.estimateRanges (set/Star.m:1078-1106) and the relax-star ReLU step at relaxFactor = 1
// (nn/funcs/PosLin.m:863-1650, 685-742; set/Star.m:1442-1461) -- and writes every layer's output set
// into buffers sized for the worst case (every neuron of every ReLU layer crossing).
//
// Networks of this size (tens of neurons per layer; an ACAS-Xu-shaped network is the type) are bound by
// the latency of a launch per layer step and of a host wait per ReLU on the layer-by-layer path; here the
// crossing counts never leave the block, the host reads them once at the end and only to fill in the
// handles.  Arrays of input sets (a branch-and-bound front over such a network) take one block each.
//
// The arithmetic is the layer kernels' (products accumulated in ascending row order from +0, the bias added
// last, lb = (c + xmin1) + xmin2), but sums are cut differently from the tiled kernels, so values agree with
// the layer-by-layer path to rounding, not bit for bit.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstring>

#include "internal.h"
#include "mfma_tile.h"
#include "relu_sort.h"

namespace nnvhip {

constexpr int kChainMaxLayers = 32;
constexpr int kChainThreads = 1024;
constexpr int kChainMaxN = 512;  // widest layer (the block's LDS holds a few vectors of that length)

struct ChainLayer {
  const double* W;     // fc: M rows (padded to ldw) x K, column-major
  const double* bias;  // fc: or null
  int32_t kind;        // NNVHIP_LAYER_FC / NNVHIP_LAYER_RELU
  int32_t M;           // dimension of the layer's output
  int32_t K;           // fc: columns of W
  int32_t ldw;
  int32_t ld;          // leading dimension of the output matrix
  int32_t npad;        // relu: padded worst-case number of predicates of the output
  // offsets (in doubles) into the set's slice of the arena
  int64_t v_off;       // the output matrix
  int64_t rng_off;     // lb[ld], ub[ld]: estimated ranges of the output (fc) / of the input when the layer before left none (relu)
  int64_t pred_off;    // relu: plb[npad], pub[npad]
  int64_t lbub_off;    // relu: lb[ld], ub[ld] of the crossing neurons in new-predicate order
  int64_t idx_off;     // relu, in ints, into the set's slice of the index arena: cross[ld], keep[ld + 16]
};

struct ChainSet {
  const double* V;    // the input set, fully in memory
  const double* plb;
  const double* pub;
  int64_t ld;
  int32_t N, n;
};

struct ChainArgs {
  ChainLayer layers[kChainMaxLayers];
  int32_t n_layers;
  int32_t order;
  double* arena;
  int64_t set_stride;
  int32_t* iarena;
  int64_t iset_stride;
  int32_t* counts;     // [set][layer][2]: crossing, inactive (zero for fc layers)
  int32_t* mailbox;    // host-pinned words, [relu ordinal * sets + set], or null
  int32_t mailbox_seq;
  int32_t n_sets;
};

// lb / ub of the N x (n+1) matrix V over the predicate box, 16 lanes per row (each lane takes every
// sixteenth generator in ascending order, then a fixed tree over the 16), into LDS and global memory.
// Only for a ReLU layer whose input did not come out of an FC layer of the same launch.
__device__ __forceinline__ void chain_ranges(const double* __restrict__ V, int ld, int N, int n, const double* __restrict__ plb,
                                             const double* __restrict__ pub, double* s_lb, double* s_ub, double* g_rng, int tid) {
  const int q = tid & 15;
  for (int r0 = 0; r0 < N; r0 += kChainThreads / 16) {
    const int i = r0 + (tid >> 4);
    double x1 = 0.0, x2 = 0.0, y1 = 0.0, y2 = 0.0;
    if (i < N) {
      for (int j = 1 + q; j <= n; j += 16) {
        const double v = V[i + (int64_t)j * ld];
        const double pl = plb[j - 1], pu = pub[j - 1];
        const double vp = fmax(v, 0.0), vn = fmin(v, 0.0);
        x1 = fma(vp, pl, x1);  // xmin1
        x2 = fma(vn, pu, x2);  // xmin2
        y1 = fma(vp, pu, y1);  // xmax1
        y2 = fma(vn, pl, y2);  // xmax2
      }
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      x1 += __shfl_xor(x1, off);
      x2 += __shfl_xor(x2, off);
      y1 += __shfl_xor(y1, off);
      y2 += __shfl_xor(y2, off);
    }
    if (q == 0 && i < N) {
      const double c = V[i];
      const double lb = (c + x1) + x2;  // set/Star.m:1098-1104, left to right
      const double ub = (c + y1) + y2;
      s_lb[i] = lb;
      s_ub[i] = ub;
      g_rng[i] = lb;
      g_rng[ld + i] = ub;
    }
  }
  __syncthreads();
}

// Barrier for data exchanged through LDS only: waits for the wave's LDS operations, not for its global stores
// (__syncthreads would also sit out the round trip of every store still in flight).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Scratch in LDS that the phases of a layer share: the sort stages its keys here, the FC phase its range sums.
struct ChainScratch {
  union {
    struct {
      double key[kChainMaxN];
      int idx[kChainMaxN];
      int rank[kChainMaxN];
    } sort;
    struct {
      double part[4][kChainMaxN];  // [sum][column group * ld + row]: range sums of the contracted columns per column group of waves
      double gat[2][kChainMaxN];   // S+ / S- of the gathered columns, by row
      double cen[kChainMaxN];      // the centre column
    } fc;
  };
};

__global__ __launch_bounds__(kChainThreads) void reach_chain_kernel(const ChainSet* __restrict__ sets, ChainSet one, ChainArgs a) {
  __shared__ double s_lb[kChainMaxN], s_ub[kChainMaxN];
  __shared__ ChainScratch sc;
  __shared__ int s_keep[kChainMaxN];
  __shared__ int s_cross[kChainMaxN];
  __shared__ int s_cls[kChainMaxN];
  __shared__ int4 wcnt[4];  // per wave: crossing | inactive << 10 | kept << 20 (each at most 64)
  __shared__ int s_counts[2 * kChainMaxLayers];
  const ChainSet S = sets ? sets[blockIdx.x] : one;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  double* A = a.arena + (int64_t)blockIdx.x * a.set_stride;
  int32_t* IA = a.iarena + (int64_t)blockIdx.x * a.iset_stride;
  int32_t* counts = a.counts + (int64_t)blockIdx.x * a.n_layers * 2;

  const double* V = S.V;        // the current set's matrix ...
  const double* Vsrc = S.V;     // ... and where an FC layer reads its kept rows from (a ReLU output: the ReLU's input,
  int ld = (int)S.ld, N = S.N, n = S.n;  // whose kept rows are the same values and were written a layer earlier)
  const double* plb = S.plb;
  const double* pub = S.pub;
  const double* plb_s = S.plb;  // likewise the bounds of the predicates in front of the ones a ReLU layer appended: the
  const double* pub_s = S.pub;  // ReLU's input holds the same values, written a layer earlier
  bool have_rng = false;        // s_lb / s_ub hold the ranges of V
  int n_keep = -1;              // >= 0: V is a ReLU output; its rows s_keep[0..n_keep) are the ones not reset,
  int oh_from = 0;              //       and its columns from oh_from on are the unit vectors of s_cross
  int relu_ord = 0;

  // every layer's weights are asked for once up front (one 128-byte line per thread and step), so that the
  // layers find them in the cache instead of each paying a trip to memory
  for (int l = 1; l < a.n_layers; ++l) {
    const ChainLayer& L = a.layers[l];
    if (L.kind != NNVHIP_LAYER_FC) continue;
    const int lines = (L.ldw * L.K) / 16;
    for (int t = tid; t < lines; t += kChainThreads) {
      const double w = L.W[(int64_t)t * 16];
      asm volatile("" ::"v"(w));
    }
  }

  for (int l = 0; l < a.n_layers; ++l) {
    const ChainLayer& L = a.layers[l];
    if (L.kind == NNVHIP_LAYER_FC) {
      // ---- Star.affineMap on the matrix cores, 16 x 16 output tiles, one wave each.  Operand layout of
      // v_mfma_f64_16x16x4_f64: lane l supplies a[i = l%16][k = l/16] (a column of V) and b[k = l/16][j = l%16]
      // (16 consecutive rows of W); result register r of lane l is out[row = l%16][column = l/16 + 4r].
      // The contraction runs over the kept rows only (reset rows hold +0) and over the columns in front of the
      // appended unit vectors; every wave keeps the four range sums of its rows over its columns.
      double* O = A + L.v_off;
      const int ldo = L.ld, ldw = L.ldw;
      const int R = ldo / 16;
      const int nd = n_keep >= 0 ? oh_from : n + 1;
      const int CT = (nd + 15) / 16;
      const int Kk = n_keep >= 0 ? n_keep : L.K;
      int RW = 1;
      while (RW * 2 <= min(R, 16)) RW *= 2;
      const int WC = 16 / RW;  // WC * ldo <= kChainMaxN (RW > R / 2, or WC = 1)
      const int wr = wave % RW, wc = wave / RW;
      const int l16 = lane & 15, kq = lane >> 4;
      for (int tr = wr; tr < R; tr += RW) {
        const int row = tr * 16 + l16;
        const double* wrow = L.W + row;
        double x1 = 0.0, x2 = 0.0, y1 = 0.0, y2 = 0.0;
        for (int tc = wc; tc < CT; tc += WC) {
          const int col_a = tc * 16 + l16;  // the column this lane feeds
          const bool col_ok = col_a < nd;
          const double* vcol = Vsrc + (int64_t)(col_ok ? col_a : 0) * ld;
          double pl[4], pu[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {  // predicate bounds of the lane's four result columns
            const int col = tc * 16 + kq + 4 * r;
            pl[r] = pu[r] = 0.0;
            if (col >= 1 && col < nd) {
              pl[r] = plb_s[col - 1];
              pu[r] = pub_s[col - 1];
            }
          }
          const double bias0 = (tc == 0 && kq == 0 && L.bias != nullptr) ? L.bias[row] : 0.0;
          double4_t acc = {0.0, 0.0, 0.0, 0.0};
          for (int k0 = 0; k0 < Kk; k0 += 32) {  // eight MFMA steps per round, their loads issued first
            double av[8], bv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              const int k = k0 + 4 * u + kq;
              av[u] = 0.0;
              bv[u] = 0.0;
              if (k < Kk) {
                const int kk = n_keep >= 0 ? s_keep[k] : k;
                bv[u] = wrow[(int64_t)kk * ldw];
                if (col_ok) av[u] = vcol[kk];
              }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f64_16x16x4f64(av[u], bv[u], acc, 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int col = tc * 16 + kq + 4 * r;
            if (col >= nd) continue;
            double v = acc[r];
            if (col == 0) {
              v = v + bias0;  // newV(:,1) = newV(:,1) + b
              sc.fc.cen[row] = v;
            } else {
              const double vp = fmax(v, 0.0), vn = fmin(v, 0.0);
              x1 = fma(vp, pl[r], x1);  // xmin1
              x2 = fma(vn, pu[r], x2);  // xmin2
              y1 = fma(vp, pu[r], y1);  // xmax1
              y2 = fma(vn, pl[r], y2);  // xmax2
            }
            O[row + (int64_t)col * ldo] = v;  // rows [M, ld): W's padding rows are zero
          }
        }
        // the four lane groups hold different columns of the same rows
        x1 += __shfl_xor(x1, 16);
        x2 += __shfl_xor(x2, 16);
        y1 += __shfl_xor(y1, 16);
        y2 += __shfl_xor(y2, 16);
        x1 += __shfl_xor(x1, 32);
        x2 += __shfl_xor(x2, 32);
        y1 += __shfl_xor(y1, 32);
        y2 += __shfl_xor(y2, 32);
        if (kq == 0) {
          sc.fc.part[0][wc * ldo + row] = x1;
          sc.fc.part[1][wc * ldo + row] = x2;
          sc.fc.part[2][wc * ldo + row] = y1;
          sc.fc.part[3][wc * ldo + row] = y2;
        }
      }
      // the appended unit vectors: W * e_r = W(:, r), and their range sums (bounds 0 / ub_r):
      // xmin2 += sum min(w, 0) * ub_r, xmax1 += sum max(w, 0) * ub_r
      const int mg = n_keep >= 0 ? n + 1 - oh_from : 0;
      if (mg > 0) {
        const int total = ldo * mg;
        for (int e = tid; e < total; e += kChainThreads) {
          const int i = e % ldo, t = e / ldo;
          O[i + (int64_t)(oh_from + t) * ldo] = 0.0 + L.W[i + (int64_t)s_cross[t] * ldw];
        }
        const int q = tid & 15;
        for (int r0 = 0; r0 < ldo; r0 += kChainThreads / 16) {
          const int i = r0 + (tid >> 4);
          double sp = 0.0, sn = 0.0;
          if (i < ldo) {
            for (int t0 = q; t0 < mg; t0 += 64) {
              double w[4], u[4];
#pragma unroll
              for (int s = 0; s < 4; ++s) {
                const int t = t0 + 16 * s;
                w[s] = u[s] = 0.0;
                if (t < mg) {
                  const int neuron = s_cross[t];
                  w[s] = L.W[i + (int64_t)neuron * ldw];
                  u[s] = s_ub[neuron];
                }
              }
#pragma unroll
              for (int s = 0; s < 4; ++s) {
                sp = fma(fmax(w[s], 0.0), u[s], sp);
                sn = fma(fmin(w[s], 0.0), u[s], sn);
              }
            }
          }
#pragma unroll
          for (int off = 1; off < 16; off <<= 1) {
            sp += __shfl_xor(sp, off);
            sn += __shfl_xor(sn, off);
          }
          if (q == 0 && i < ldo) {
            sc.fc.gat[0][i] = sp;
            sc.fc.gat[1][i] = sn;
          }
        }
      }
      lds_barrier();
      double* g = A + L.rng_off;
      if (tid < L.M) {  // the column groups in order, then the gathered columns; lb = (c + xmin1) + xmin2
        double x1 = 0.0, x2 = 0.0, y1 = 0.0, y2 = 0.0;
        for (int w2 = 0; w2 < WC; ++w2) {
          if (w2 >= CT) break;
          x1 += sc.fc.part[0][w2 * ldo + tid];
          x2 += sc.fc.part[1][w2 * ldo + tid];
          y1 += sc.fc.part[2][w2 * ldo + tid];
          y2 += sc.fc.part[3][w2 * ldo + tid];
        }
        if (mg > 0) {
          y1 += sc.fc.gat[0][tid];
          x2 += sc.fc.gat[1][tid];
        }
        const double c = sc.fc.cen[tid];
        const double lo = (c + x1) + x2, up = (c + y1) + y2;
        g[tid] = lo;
        g[ldo + tid] = up;
        s_lb[tid] = lo;
        s_ub[tid] = up;
      }
      if (tid == 0) {
        s_counts[2 * l] = 0;
        s_counts[2 * l + 1] = 0;
      }
      // A ReLU layer next reads the ranges from LDS and meets a full barrier before anybody loads the matrix; an FC
      // layer next loads the matrix other waves have just stored, so their stores must have completed.
      if (l + 1 < a.n_layers && a.layers[l + 1].kind == NNVHIP_LAYER_FC)
        __syncthreads();
      else
        lds_barrier();
      V = O;
      Vsrc = O;
      plb_s = plb;
      pub_s = pub;
      ld = ldo;
      N = L.M;
      n_keep = -1;
      oh_from = 0;
      have_rng = true;
    } else {
      if (!have_rng) {
        __syncthreads();  // the matrix may have been written a moment ago (a ReLU layer's output)
        chain_ranges(V, ld, N, n, plb, pub, s_lb, s_ub, A + L.rng_off, tid);
      }
      // ---- classification (N <= 1024: thread r owns neuron r), ascending lists by ballot + prefix sum
      int32_t* cross_g = IA + L.idx_off;
      int32_t* keep_g = cross_g + ld;
      const int r = tid;
      const bool valid = r < N;
      const double lo = valid ? s_lb[r] : 0.0;
      const double up = valid ? s_ub[r] : 1.0;
      const bool inactive = valid && (up <= 0.0);               // map1 = find(ub <= 0)
      const bool crossing = valid && (lo < 0.0) && (up > 0.0);  // map2 = find(lb < 0 & ub > 0)
      const bool kept = valid && !inactive && !crossing;
      const unsigned long long bc = __ballot(crossing);
      const unsigned long long bi = __ballot(inactive);
      const unsigned long long bk = __ballot(kept);
      if (lane == 0) reinterpret_cast<int*>(wcnt)[wave] = __popcll(bc) | (__popcll(bi) << 10) | (__popcll(bk) << 20);
      lds_barrier();
      int before = 0, all = 0;  // the three counts stay packed: none of the sums passes 2^10
#pragma unroll
      for (int w4 = 0; w4 < 4; ++w4) {
        const int4 c4 = wcnt[w4];
        const int cw[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          before += 4 * w4 + u < wave ? cw[u] : 0;
          all += cw[u];
        }
      }
      const int woff = before & 1023, koff = before >> 20;
      const int m = all & 1023, inact = (all >> 10) & 1023, nk = all >> 20;
      if (r < kChainMaxN) s_cls[r] = crossing ? 0 : inactive ? kZero : kKeep;  // rows past N: untouched (zero anyway)
      const int kpos = koff + __popcll(bk & ((1ull << lane) - 1ull));
      if (kept) s_keep[kpos] = r;
      const bool sorted = a.order != NNVHIP_ORDER_INDEX;
      if (crossing) {
        const int p = woff + __popcll(bc & ((1ull << lane) - 1ull));
        if (sorted) {
          // areas = 0.5*(abs(ub).*abs(lb))  |  ub - lb   (nn/funcs/PosLin.m:1049-1052, 934-936)
          sc.sort.key[p] = a.order == NNVHIP_ORDER_AREA ? 0.5 * (fabs(up) * fabs(lo)) : up - lo;
          sc.sort.idx[p] = r;
          sc.sort.rank[p] = 0;
        } else {
          s_cross[p] = r;
        }
      }
      if (tid == 0) {
        s_counts[2 * l] = m;
        s_counts[2 * l + 1] = inact;
      }
      lds_barrier();
      if (sorted && m > 0) {
        // stable descending key sort by counting: rank(i) = #{j : key_j > key_i, or key_j == key_i and j < i} over the
        // ascending list (j < i there is "smaller neuron index", what MATLAB's stable sort keeps).  The block's
        // threads share the m x m comparisons; the partial counts meet in integer adds, whose order does not matter.
        int mp = 64;
        while (mp < m) mp *= 2;
        const int tpi = kChainThreads / mp;  // threads per entry (m <= 512: at least two)
        const int i = tid % mp, c0 = tid / mp;
        if (i < m) {
          const double ki = sc.sort.key[i];
          int cnt = 0;
          for (int j = c0; j < m; j += tpi) {
            const double kj = sc.sort.key[j];
            cnt += (kj > ki || (kj == ki && j < i)) ? 1 : 0;
          }
          if (cnt) atomicAdd(&sc.sort.rank[i], cnt);
        }
        lds_barrier();
        if (tid < m) s_cross[sc.sort.rank[tid]] = sc.sort.idx[tid];
      }
      // (a full barrier: the layer's input matrix, written by other threads a few phases ago, is read below; every
      // store of this phase to global memory comes after it, so that no barrier has a fresh store to wait for)
      __syncthreads();
      if (kept) keep_g[kpos] = r;
      if (tid < 2 * (int)kLdAlign) {  // the kept-row list ends with -1 up to a whole group of 16 (at least one group)
        const int end = max((nk + (int)kLdAlign - 1) / (int)kLdAlign * (int)kLdAlign, (int)kLdAlign);
        if (nk + tid < end) keep_g[nk + tid] = -1;
      }
      if (tid < m) cross_g[tid] = s_cross[tid];
      if (tid == 0 && a.mailbox != nullptr)
        post_counts(a.mailbox + 2 * ((int64_t)relu_ord * a.n_sets + blockIdx.x), m, inact, a.mailbox_seq);
      // ---- the output set: V' = [V with the inactive and crossing rows reset, unit vectors of the crossing
      // neurons], new_pred_lb = [plb; 0], new_pred_ub = [pub; ub(index)]  (nn/funcs/PosLin.m:700-738).  Nothing
      // in this launch waits for these stores: the next FC layer reads the kept rows from V itself.
      double* O = A + L.v_off;
      const int ncols_in = n + 1;
      const int total = ld * (ncols_in + m);
      for (int e0 = tid; e0 < total; e0 += 4 * kChainThreads) {
        double val[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {  // the loads of four steps go out together
          const int e = e0 + u * kChainThreads;
          val[u] = 0.0;
          if (e < total) {
            const int i = e % ld, j = e / ld;
            if (j < ncols_in) val[u] = (i >= N || s_cls[i] == kKeep) ? V[e] : 0.0;
            else val[u] = i == s_cross[j - ncols_in] ? 1.0 : 0.0;
          }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int e = e0 + u * kChainThreads;
          if (e < total) O[e] = val[u];
        }
      }
      double* P = A + L.pred_off;
      double* LU = A + L.lbub_off;
      for (int j = tid; j < n + m; j += kChainThreads) {
        if (j < n) {
          P[j] = plb[j];
          P[L.npad + j] = pub[j];
        } else {
          const int neuron = s_cross[j - n];
          const double ubn = s_ub[neuron];
          P[j] = 0.0;
          P[L.npad + j] = ubn;
          LU[j - n] = s_lb[neuron];
          LU[ld + (j - n)] = ubn;
        }
      }
      if (n_keep >= 0) {  // ReLU after ReLU: its input has appended columns of its own
        __syncthreads();
        Vsrc = O;
        plb_s = P;
        pub_s = P + L.npad;
      } else {
        Vsrc = V;
        plb_s = plb;
        pub_s = pub;
      }
      V = O;
      oh_from = n + 1;
      n += m;
      n_keep = nk;
      plb = P;
      pub = P + L.npad;
      have_rng = false;
      ++relu_ord;
    }
  }
  lds_barrier();
  if (tid < 2 * a.n_layers) counts[tid] = s_counts[tid];
}

// Worst-case layout of one set's slice of the arenas for the given layer list.
struct ChainPlan {
  ChainArgs args{};
  std::vector<int64_t> ncap;  // worst-case predicate count of every layer's output
  int64_t doubles = 0, ints = 0;
  int n_relu = 0;
};

static bool plan_chain(nnvhip_ctx* c, int64_t n_layers, const int32_t* kind, const void* const* layer, int64_t N0, int64_t n0_max,
                       ChainPlan* plan) {
  if (n_layers < 1 || n_layers > kChainMaxLayers) return false;
  int64_t N = N0, ncap = n0_max;
  int64_t off = 0, ioff = 0;
  double work = 0.0;
  plan->ncap.resize((size_t)n_layers);
  for (int64_t l = 0; l < n_layers; ++l) {
    ChainLayer& L = plan->args.layers[l];
    L = ChainLayer{};
    L.kind = kind[l];
    if (kind[l] == NNVHIP_LAYER_FC) {
      const nnvhip_fc* fc = static_cast<const nnvhip_fc*>(layer[l]);
      if (!fc || fc->ctx != c || fc->K != N || fc->M > kChainMaxN) return false;
      L.W = fc->W->as<double>();
      L.bias = fc->bias ? fc->bias->as<double>() : nullptr;
      L.M = (int32_t)fc->M;
      L.K = (int32_t)fc->K;
      L.ldw = (int32_t)fc->Mp;
      N = fc->M;
      L.ld = (int32_t)round_up(N, kLdAlign);
      work += (double)L.ld * (double)fc->K * (double)(ncap + 1);
    } else if (kind[l] == NNVHIP_LAYER_RELU) {
      if (N > kChainMaxN) return false;
      L.M = (int32_t)N;
      L.ld = (int32_t)round_up(N, kLdAlign);
      ncap += N;
      L.npad = (int32_t)round_up(std::max<int64_t>(ncap, 1), kLdAlign);
      ++plan->n_relu;
    } else {
      return false;
    }
    plan->ncap[l] = ncap;
    L.v_off = off;
    off += (int64_t)L.ld * (ncap + 1);
    L.rng_off = off;
    off += 2 * (int64_t)L.ld;
    if (kind[l] == NNVHIP_LAYER_RELU) {
      L.pred_off = off;
      off += 2 * (int64_t)L.npad;
      L.lbub_off = off;
      off += 2 * (int64_t)L.ld;
      L.idx_off = ioff;
      ioff += 2 * (int64_t)L.ld + kLdAlign;
    }
  }
  // one block does all of it: only networks whose worst case is a few hundred thousand matrix entries
  if (off > (int64_t(1) << 18) || work > 6.4e7) return false;
  plan->doubles = off;
  plan->ints = std::max<int64_t>(ioff, kLdAlign);
  plan->args.n_layers = (int32_t)n_layers;
  return true;
}

int reach_small_chain(nnvhip_ctx* c, int64_t n_layers, const int32_t* kind, const void* const* layer, int order, int64_t count,
                      nnvhip_star* const* in, nnvhip_star** out, bool* taken) {
  *taken = false;
  if (!c->small_chain || c->dense_affine || count > 65535) return NNVHIP_OK;
  if (order != NNVHIP_ORDER_INDEX && order != NNVHIP_ORDER_AREA && order != NNVHIP_ORDER_RANGE) return NNVHIP_OK;
  int64_t n0_max = 0;
  for (int64_t i = 0; i < count; ++i) {
    if (!in[i] || in[i]->ctx != c || in[i]->N != in[0]->N) return NNVHIP_OK;  // the layer loop reports it
    n0_max = std::max(n0_max, in[i]->n);
  }
  ChainPlan plan;
  if (!plan_chain(c, n_layers, kind, layer, in[0]->N, n0_max, &plan)) return NNVHIP_OK;
  if ((double)plan.doubles * (double)count > 5.0e8) return NNVHIP_OK;  // 4 GB of worst-case buffers
  *taken = true;

  NNV_TRY(ensure_dense_batch(c, count, in, true, true));
  BufRef arena, iarena, cnt;
  NNV_TRY(c->alloc(sizeof(double) * plan.doubles * count, &arena));
  NNV_TRY(c->alloc(sizeof(int32_t) * plan.ints * count, &iarena));
  NNV_TRY(c->alloc(sizeof(int32_t) * 2 * n_layers * count, &cnt));
  ChainArgs& a = plan.args;
  a.order = order;
  a.arena = arena->as<double>();
  a.set_stride = plan.doubles;
  a.iarena = iarena->as<int32_t>();
  a.iset_stride = plan.ints;
  a.counts = cnt->as<int32_t>();
  a.n_sets = (int32_t)count;
  const int64_t words = (int64_t)plan.n_relu * count;
  const bool use_mailbox = words > 0 && words <= nnvhip_ctx::kMailboxSets && c->mailbox != nullptr;
  if (use_mailbox) {
    ++c->mailbox_seq;
    volatile unsigned long long* box = reinterpret_cast<volatile unsigned long long*>(c->mailbox);
    for (int64_t i = 0; i < words; ++i) box[i] = kMailboxEmpty;
    std::atomic_thread_fence(std::memory_order_seq_cst);
    a.mailbox = const_cast<int32_t*>(c->mailbox);
    a.mailbox_seq = (int32_t)(c->mailbox_seq & 0xffffu);
  }
  std::vector<ChainSet> sets((size_t)count);
  for (int64_t i = 0; i < count; ++i) sets[i] = ChainSet{in[i]->V, in[i]->plb, in[i]->pub, in[i]->ld, (int32_t)in[i]->N, (int32_t)in[i]->n};
  const ChainSet* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(c->upload(sets.data(), sizeof(ChainSet) * count, &tab));
    table = tab->as<ChainSet>();
  }
  NNV_LAUNCH(c, c->kernel_timing, reach_chain_kernel, dim3((unsigned)count), dim3(kChainThreads), 0, table, sets[0], a);
  NNV_HIP_TRY(hipGetLastError());

  // the crossing counts: all the host needs to know to fill in the handles
  std::vector<int32_t> counts((size_t)(2 * n_layers * count), 0);
  if (use_mailbox) {
    const auto t0 = std::chrono::steady_clock::now();
    long spins = 0;
    const volatile unsigned long long* box = reinterpret_cast<const volatile unsigned long long*>(c->mailbox);
    int ord = 0;
    for (int64_t l = 0; l < n_layers; ++l) {
      if (kind[l] != NNVHIP_LAYER_RELU) continue;
      for (int64_t i = 0; i < count; ++i) {
        const int64_t w_i = (int64_t)ord * count + i;
        unsigned long long w = box[w_i];
        while (w == kMailboxEmpty) {
          if ((++spins & 0xfff) == 0 && std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 10.0) {
            NNV_HIP_TRY(hipStreamSynchronize(c->stream));
            if (box[w_i] == kMailboxEmpty) NNV_FAIL(NNVHIP_ERR_HIP, "the reach kernel did not report its counts");
          }
          w = box[w_i];
        }
        int m_ = 0, inact_ = 0, seq_ = 0;
        mailbox_unpack(w, &m_, &inact_, &seq_);
        if (seq_ != (int)(c->mailbox_seq & 0xffffu)) NNV_FAIL(NNVHIP_ERR_HIP, "internal: mailbox word of another call");
        counts[(size_t)((i * n_layers + l) * 2)] = m_;
        counts[(size_t)((i * n_layers + l) * 2 + 1)] = inact_;
      }
      ++ord;
    }
  } else if (plan.n_relu > 0) {
    void* hc = nullptr;
    NNV_TRY(c->stage(sizeof(int32_t) * counts.size(), &hc));
    NNV_HIP_TRY(hipMemcpyAsync(hc, cnt->ptr, sizeof(int32_t) * counts.size(), hipMemcpyDeviceToHost, c->stream));
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
    memcpy(counts.data(), hc, sizeof(int32_t) * counts.size());
  }
  if (c->kernel_timing) {
    // algorithmic bytes: the weights read once per set, every layer's output matrix written once
    double bytes = 0.0;
    for (int64_t i = 0; i < count; ++i) {
      int64_t n = in[i]->n;
      for (int64_t l = 0; l < n_layers; ++l) {
        if (kind[l] == NNVHIP_LAYER_FC) bytes += 8.0 * (double)a.layers[l].M * (double)a.layers[l].K;
        n += counts[(size_t)((i * n_layers + l) * 2)];
        bytes += 8.0 * (double)a.layers[l].M * (double)(n + 1);
      }
    }
    NNV_TRY(c->kernel_timer_end(true, 8, bytes));
  }

  // ---- handles: every layer's output set, described exactly as the layer-by-layer path would leave it
  // once every pending piece had been written
  for (int64_t i = 0; i < count; ++i) {
    double* A = arena->as<double>() + i * plan.doubles;
    int32_t* IA = iarena->as<int32_t>() + i * plan.ints;
    const nnvhip_star* prev = in[i];
    const double* prev_ub = nullptr;  // upper bounds of prev's estimated ranges, when the kernel left them
    for (int64_t l = 0; l < n_layers; ++l) {
      const ChainLayer& L = a.layers[l];
      nnvhip_star* o = new_star(c);
      o->N = L.M;
      o->ld = L.ld;
      o->Vbuf = arena;
      o->V = A + L.v_off;
      if (L.kind == NNVHIP_LAYER_FC) {
        o->n = prev->n;
        o->pbuf = prev->pbuf;
        o->plb = prev->plb;
        o->pub = prev->pub;
        o->ptails = prev->ptails;
        o->pslot = prev->pslot;
        o->pcap = prev->pcap;
        o->cons = prev->cons;
        o->has_zono = prev->has_zono;
        o->rbuf = arena;
        o->lb = A + L.rng_off;
        o->ub = o->lb + L.ld;
        prev_ub = o->ub;
      } else {
        const int64_t m = counts[(size_t)((i * n_layers + l) * 2)];
        const int64_t inact = counts[(size_t)((i * n_layers + l) * 2 + 1)];
        o->n = prev->n + m;
        o->pbuf = arena;
        o->plb = A + L.pred_off;
        o->pub = o->plb + L.npad;
        o->n_inactive = inact;
        o->n_crossing = m;
        o->pre_ub_buf = arena;
        o->pre_ub = prev_ub ? prev_ub : A + L.rng_off + L.ld;
        o->n_kept = L.M - m - inact;
        o->kept_buf = iarena;
        o->kept_idx = IA + L.idx_off + L.ld;
        if (m > 0) {
          o->oh_from = prev->n + 1;
          o->oh_plb_zero = true;
          o->oh_idx_buf = iarena;
          o->oh_idx = IA + L.idx_off;
          auto node = make_ref<ConsNode>();
          node->prev = prev->cons;
          node->n_before = prev->n;
          node->src = prev->Vbuf;  // C2/C3 rows are rows of the pre-ReLU [c V]
          node->src_V = prev->V;
          node->src_ld = prev->ld;
          node->index = iarena;
          node->index_off = (IA + L.idx_off) - iarena->as<int32_t>();
          node->m = m;
          node->p_total = prev->cons->p_total + 3 * m;
          node->n_total = o->n;
          node->lbub = arena;
          node->lbub_off = (A + L.lbub_off) - arena->as<double>();
          node->ld_lbub = L.ld;
          o->cons = std::move(node);
        } else {
          o->cons = prev->cons;
        }
        prev_ub = nullptr;
      }
      out[l * count + i] = o;
      prev = o;
    }
  }
  return NNVHIP_OK;
}

}  // namespace nnvhip
