// The relax-star ReLU step at relaxFactor = 1 (nn/funcs/PosLin.m:863-1650, 685-742;
// set/Star.m:1442-1461), entirely on the device:
//   1. classify every neuron from its estimated range (inactive / crossing / active) and compact
//      the crossing indices in ascending order with wavefront ballots + prefix sums;
//   2. (area / range orders) rank the crossing neurons by a stable descending key sort;
//   3. one pass over V: zero the inactive and crossing rows, append the one-hot columns and the new
//      predicate bounds.  The crossing rows the constraints need are not copied: the constraint node
//      keeps the (immutable) pre-ReLU generator matrix alive and remembers the row indices.
// The dense constraint matrix is never built on this path; materialize_constraints() lays it out
// exactly as the reference does when the host asks for it.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>

#include "internal.h"
#include "relu_sort.h"

namespace nnvhip {

// One 1024-thread block per set.  SORT_CAP > 0: crossing lists of up to SORT_CAP neurons are sorted
// here by a bitonic network in LDS; longer lists are left to the tiled rank kernels.
template <int SORT_CAP>
__global__ __launch_bounds__(1024) void relu_classify_kernel(const ReluDesc* __restrict__ table, ReluDesc one) {
  const ReluDesc d = table ? table[blockIdx.x] : one;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  __shared__ int wcross[16];
  __shared__ int winact[16];
  __shared__ int wkeep[16];
  __shared__ double skey[SORT_CAP > 0 ? kSortInBlock : 1];
  __shared__ int sidx[SORT_CAP > 0 ? kSortInBlock : 1];
  static_assert(sizeof(double) == sizeof(long long), "keys are sorted through their bit patterns");
  int base = 0, inact_total = 0, keep_base = 0;
  int32_t* idx_out = d.order == NNVHIP_ORDER_INDEX ? d.cross_idx : d.asc_idx;
  // the first 1024 ranges are asked for before anything else ...
  const double l_first = tid < d.N ? d.lb[tid] : 0.0;
  const double u_first = tid < d.N ? d.ub[tid] : 1.0;
  // ... and while they travel, the bounds of the predicates the set already has are copied (new_pred_lb =
  // [plb; ...], new_pred_ub = [pub; ...]): nothing of that depends on the classification
  if (d.write_bounds && d.plb_out != d.plb_in) {  // (in place: the old bounds are where they belong)
    const int n_in = d.ncols_in - 1;
    for (int jb = tid; jb < n_in; jb += 4096) {
      double a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jb + u * 1024;
        a[u] = j < n_in ? d.plb_in[j] : 0.0;
        b[u] = j < n_in ? d.pub_in[j] : 0.0;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jb + u * 1024;
        if (j < n_in) {
          d.plb_out[j] = a[u];
          d.pub_out[j] = b[u];
        }
      }
    }
  }
  for (int r0 = 0; r0 < d.N; r0 += 1024) {
    const int r = r0 + tid;
    const bool valid = r < d.N;
    const double l = r0 == 0 ? l_first : valid ? d.lb[r] : 0.0;
    const double u = r0 == 0 ? u_first : valid ? d.ub[r] : 1.0;
    const bool inactive = valid && (u <= 0.0);              // map1 = find(ub <= 0)
    const bool crossing = valid && (l < 0.0) && (u > 0.0);  // map2 = find(lb < 0 & ub > 0)
    const bool kept = valid && !inactive && !crossing;
    const unsigned long long bc = __ballot(crossing);
    const unsigned long long bi = __ballot(inactive);
    const unsigned long long bk = __ballot(kept);
    if (lane == 0) {
      wcross[wave] = __popcll(bc);
      winact[wave] = __popcll(bi);
      wkeep[wave] = __popcll(bk);
      if (d.keep_bits != nullptr) *reinterpret_cast<uint2*>(d.keep_bits + ((r0 >> 5) + 2 * wave)) = make_uint2((uint32_t)bk, (uint32_t)(bk >> 32));
    }
    __syncthreads();
    int woff = 0, tot = 0, itot = 0, koff = 0, ktot = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int c = wcross[w];
      woff += w < wave ? c : 0;
      tot += c;
      itot += winact[w];
      const int k = wkeep[w];
      koff += w < wave ? k : 0;
      ktot += k;
    }
    if (kept) d.keep_idx[keep_base + koff + __popcll(bk & ((1ull << lane) - 1ull))] = r;
    keep_base += ktot;
    if (crossing) {
      const int pos = base + woff + __popcll(bc & ((1ull << lane) - 1ull));
      d.cls[r] = pos;
      if (d.order == NNVHIP_ORDER_INDEX) {
        idx_out[pos] = r;
        if (d.col_of != nullptr) d.col_of[r] = pos;
      } else {
        // areas = 0.5*(abs(ub).*abs(lb))  |  ub - lb.  Lists of up to kSortInBlock entries are sorted
        // below, straight from LDS; a set with more neurons than that may have a longer list, which the
        // multi-block rank kernels sort from the copies in global memory.
        const double key = d.order == NNVHIP_ORDER_AREA ? 0.5 * (fabs(u) * fabs(l))
                           : d.order == NNVHIP_ORDER_RANGE ? u - l : d.given_key[r];
        if (SORT_CAP > kSortInBlock) {
          idx_out[pos] = r;
          d.key[pos] = key;
        }
        if (SORT_CAP > 0 && pos < kSortInBlock) {
          skey[pos] = key;
          sidx[pos] = r;
        }
      }
    } else if (valid) {
      d.cls[r] = inactive ? kZero : kKeep;
      if (d.col_of != nullptr) d.col_of[r] = -1;
    }
    base += tot;
    inact_total += itot;
    __syncthreads();
  }
  for (int64_t r = d.N + tid; r < d.ld; r += 1024) d.cls[r] = kKeep;  // padding rows stay zero
  if (tid < 2 * (int)kLdAlign) {  // -1 up to the next multiple of 16 past the list (at least 16 entries in all)
    const int end = max((keep_base + (int)kLdAlign - 1) / (int)kLdAlign * (int)kLdAlign, (int)kLdAlign);
    if (keep_base + tid < end) d.keep_idx[keep_base + tid] = -1;
  }
  const int m = base;
  const bool sort_here = SORT_CAP > 0 && d.order != NNVHIP_ORDER_INDEX && m > 0 && m <= kSortInBlock;
  // order settled in this block (otherwise the rank kernels settle it and the bounds follow them)
  const bool order_known = d.order == NNVHIP_ORDER_INDEX || m <= kSortInBlock;
  if (sort_here) __syncthreads();  // the keys are staged; nothing of the stores below is in flight yet
  if (tid == 0) {
    d.counts[0] = m;
    d.counts[1] = inact_total;
    post_counts(d.mailbox, m, inact_total, d.mailbox_seq);  // the host can size the output while we sort
  }
  int mine = 0;  // entry tid of the sorted list
  if (sort_here)  // the staged doubles are read back as their bit patterns
    mine = sort_small_desc(reinterpret_cast<long long*>(skey), sidx, m, tid, d.cross_idx);
  if (sort_here && d.col_of != nullptr && tid < m) d.col_of[mine] = tid;
  if (d.write_bounds && sort_here) {
    // the output buffers were sized for the worst case: finish the set here.  New predicate tid belongs to the
    // neuron this thread holds: new_pred_lb = [plb; zeros(m,1)], new_pred_ub = [pub; ub(index)]
    if (tid < m) {
      const int n_in = d.ncols_in - 1;
      const double b = d.ub[mine], c = d.lb[mine];
      d.plb_out[n_in + tid] = 0.0;
      d.pub_out[n_in + tid] = b;
      d.lbub[tid] = c;
      d.lbub[d.ld_lbub + tid] = b;
    }
  } else if (d.write_bounds && order_known) {
    __syncthreads();     // cross_idx is complete
    const int n_in = d.ncols_in - 1;
    // the new predicates, four per thread and step, all loads issued before the first store (the dependent
    // index -> bound look-ups would otherwise queue up behind one another)
    for (int ib = tid; ib < m; ib += 4096) {
      double b[4], c[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = ib + u * 1024;
        b[u] = c[u] = 0.0;
        if (i < m) {
          const int neuron = d.cross_idx[i];
          b[u] = d.ub[neuron];
          c[u] = d.lb[neuron];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = ib + u * 1024;
        if (i >= m) break;
        d.plb_out[n_in + i] = 0.0;  // new_pred_lb = [plb; zeros(m,1)], new_pred_ub = [pub; ub(index)]
        d.pub_out[n_in + i] = b[u];
        d.lbub[i] = c[u];
        d.lbub[d.ld_lbub + i] = b[u];
      }
    }
  }
}

// What the kernels that settle the order of a crossing list write besides the list: kRankNewBounds: the bounds
// of the new predicates (new_pred_lb = [plb; zeros(m,1)], new_pred_ub = [pub; ub(index)]) and the crossing
// neurons' (lb, ub); kRankOldBounds: also the copy of the bounds of the predicates the set already has.
// kRankCountOnDevice: the length of the list is read from the set's counters (the kernel was queued before the host
// knew it, with a grid for the longest possible list).
constexpr int kRankNewBounds = 1, kRankOldBounds = 2, kRankCountOnDevice = 4;

// Sorts a crossing list of at most 1024 entries that the multi-block classification left in
// ascending order (keys in d.key, neurons in d.asc_idx).  One block per set; every thread ends up with entry
// tid of the sorted list and writes that predicate's bounds itself (see the flags above).
__global__ __launch_bounds__(1024) void relu_sort_small_kernel(const ReluDesc* __restrict__ table, ReluDesc one, int flags) {
  const ReluDesc d = table ? table[blockIdx.x] : one;
  const int m = d.m;
  const int tid = threadIdx.x;
  const int n_in = d.ncols_in - 1;
  if ((flags & kRankOldBounds) && d.plb_out != d.plb_in) {
    for (int j = tid; j < n_in; j += 1024) {
      d.plb_out[j] = d.plb_in[j];
      d.pub_out[j] = d.pub_in[j];
    }
  }
  if (m <= 0 || m > 1024) return;
  __shared__ double skey[1024];
  __shared__ int sidx[1024];
  if (tid < m) {
    skey[tid] = d.key[tid];
    sidx[tid] = d.asc_idx[tid];
  }
  __syncthreads();
  const int mine = sort_small_desc(reinterpret_cast<long long*>(skey), sidx, m, tid, d.cross_idx);
  if (d.col_of != nullptr && tid < m) d.col_of[mine] = tid;
  if ((flags & kRankNewBounds) && tid < m) {
    const double ub = d.ub[mine];
    d.plb_out[n_in + tid] = 0.0;
    d.pub_out[n_in + tid] = ub;
    d.lbub[tid] = d.lb[mine];
    d.lbub[d.ld_lbub + tid] = ub;
  }
}

// Multi-block classification for sets with more than 1024 neurons: pass 1 counts the crossing and
// inactive neurons of every 1024-row block, pass 2 turns the block counts into offsets (at most a
// few dozen values) and writes the ascending crossing list.  Grid: (row blocks, 1, sets).
__global__ __launch_bounds__(1024) void relu_count_kernel(const ReluDesc* __restrict__ table, ReluDesc one) {
  const ReluDesc d = table ? table[blockIdx.z] : one;
  const int r = blockIdx.x * 1024 + threadIdx.x;
  const bool valid = r < d.N;
  const double l = valid ? d.lb[r] : 0.0;
  const double u = valid ? d.ub[r] : 1.0;
  const bool inactive = valid && (u <= 0.0);
  const bool crossing = valid && (l < 0.0) && (u > 0.0);
  const unsigned long long bc = __ballot(crossing);
  const unsigned long long bi = __ballot(inactive);
  __shared__ int wc[16], wi[16];
  if ((threadIdx.x & 63) == 0) {
    wc[threadIdx.x >> 6] = __popcll(bc);
    wi[threadIdx.x >> 6] = __popcll(bi);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int c = 0, i = 0;
    for (int w = 0; w < 16; ++w) {
      c += wc[w];
      i += wi[w];
    }
    d.blk_counts[3 * blockIdx.x] = c;
    d.blk_counts[3 * blockIdx.x + 1] = i;
    d.blk_counts[3 * blockIdx.x + 2] = min(1024, d.N - (int)blockIdx.x * 1024) - c - i;  // kept rows of the block
  }
}

__global__ __launch_bounds__(1024) void relu_compact_kernel(const ReluDesc* __restrict__ table, ReluDesc one) {
  const ReluDesc d = table ? table[blockIdx.z] : one;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  __shared__ int wcross[16], wkeep[16];
  __shared__ int sbase, stot, sinact, skbase;
  if (wave == 0) {  // offset of this block = crossing (kept) counts of the blocks before it
    int before = 0, tot = 0, inact = 0, kbefore = 0;
    const int nent = d.blk_gran == 1024 ? (int)gridDim.x : (int)((d.ld + d.blk_gran - 1) / d.blk_gran);
    const int mine = (int)blockIdx.x * (1024 / d.blk_gran);  // first entry of this block's rows
    for (int b = lane; b < nent; b += 64) {
      const int c = d.blk_counts[3 * b];
      before += b < mine ? c : 0;
      tot += c;
      inact += d.blk_counts[3 * b + 1];
      kbefore += b < mine ? d.blk_counts[3 * b + 2] : 0;
    }
    for (int off = 32; off > 0; off >>= 1) {
      before += __shfl_xor(before, off);
      tot += __shfl_xor(tot, off);
      inact += __shfl_xor(inact, off);
      kbefore += __shfl_xor(kbefore, off);
    }
    if (lane == 0) {
      sbase = before;
      stot = tot;
      sinact = inact;
      skbase = kbefore;
    }
  }
  const int r = blockIdx.x * 1024 + tid;
  const bool valid = r < d.N;
  const double l = valid ? d.lb[r] : 0.0;
  const double u = valid ? d.ub[r] : 1.0;
  const bool inactive = valid && (u <= 0.0);
  const bool crossing = valid && (l < 0.0) && (u > 0.0);
  const bool kept = valid && !inactive && !crossing;
  const unsigned long long bc = __ballot(crossing);
  const unsigned long long bk = __ballot(kept);
  if (lane == 0) {
    wcross[wave] = __popcll(bc);
    wkeep[wave] = __popcll(bk);
    if (d.keep_bits != nullptr)
      *reinterpret_cast<uint2*>(d.keep_bits + (blockIdx.x * 32 + 2 * wave)) = make_uint2((uint32_t)bk, (uint32_t)(bk >> 32));
  }
  __syncthreads();
  int woff = 0, koff = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    woff += w < wave ? wcross[w] : 0;
    koff += w < wave ? wkeep[w] : 0;
  }
  if (kept) d.keep_idx[skbase + koff + __popcll(bk & ((1ull << lane) - 1ull))] = r;
  int32_t* idx_out = d.order == NNVHIP_ORDER_INDEX ? d.cross_idx : d.asc_idx;
  if (crossing) {
    const int pos = sbase + woff + __popcll(bc & ((1ull << lane) - 1ull));
    idx_out[pos] = r;
    d.cls[r] = pos;
    if (d.order == NNVHIP_ORDER_INDEX && d.col_of != nullptr) d.col_of[r] = pos;
    if (d.order != NNVHIP_ORDER_INDEX) {
      d.key[pos] = d.order == NNVHIP_ORDER_AREA ? 0.5 * (fabs(u) * fabs(l)) : d.order == NNVHIP_ORDER_RANGE ? u - l : d.given_key[r];
    }
  } else if (valid) {
    d.cls[r] = inactive ? kZero : kKeep;
    if (d.col_of != nullptr) d.col_of[r] = -1;
  }
  if (blockIdx.x == gridDim.x - 1) {
    for (int64_t p = d.N + tid; p < d.ld; p += 1024) d.cls[p] = kKeep;  // padding rows stay zero
    if (tid < 2 * (int)kLdAlign) {  // pad the kept-row list with -1 to a whole K-tile (at least one)
      const int nkeep = d.N - stot - sinact;
      const int end = max((nkeep + (int)kLdAlign - 1) / (int)kLdAlign * (int)kLdAlign, (int)kLdAlign);
      if (nkeep + tid < end) d.keep_idx[nkeep + tid] = -1;
    }
    if (tid == 0) {
      d.counts[0] = stot;
      d.counts[1] = sinact;
      post_counts(d.mailbox, stot, sinact, d.mailbox_seq);
    }
  }
}

// Stable descending sort by counting: rank(i) = #{j : key_j > key_i or (key_j == key_i and j < i)}.
// j < i in the ascending list is "smaller neuron index", which is what MATLAB's stable sort keeps.
// A block owns kRankI entries of the list and compares them with the whole list, staged through LDS in pieces of
// kRankStage keys: thread (entry, slice) counts over every 16th key, the 16 slices of an entry are then added.
// No block needs anything from another one (the XCDs of this chip share no cache, so counters and atomics
// between blocks are the expensive part of a tiled count), and a block knows the final places of its entries:
// it puts their neurons there and, with kRankNewBounds, writes what the new predicates need (new_pred_lb =
// [plb; zeros(m,1)], new_pred_ub = [pub; ub(index)], and the crossing neurons' (lb, ub)).  kRankOldBounds: the
// blocks also share out the copy of the bounds of the predicates the set already has.
constexpr int kRankI = 16;
constexpr int kRankStage = 2048;
__global__ __launch_bounds__(256) void relu_rank_kernel(const ReluDesc* __restrict__ table, ReluDesc one, int flags) {
  const ReluDesc d = table ? table[blockIdx.z] : one;
  const int m = (flags & kRankCountOnDevice) ? d.counts[0] : d.m;
  const int tid = threadIdx.x;
  const int n_in = d.ncols_in - 1;
  if ((flags & kRankOldBounds) && d.plb_out != d.plb_in) {
    for (int j = blockIdx.x * 256 + tid; j < n_in; j += gridDim.x * 256) {
      d.plb_out[j] = d.plb_in[j];
      d.pub_out[j] = d.pub_in[j];
    }
  }
  const int i0 = blockIdx.x * kRankI;
  if (i0 >= m) return;
  const int il = tid & (kRankI - 1), slice = tid / kRankI;  // 256 / kRankI = 16 slices
  const int i = i0 + il;
  const double ki = i < m ? d.key[i] : 0.0;
  __shared__ double keys[kRankStage];
  __shared__ int part[16][kRankI];
  int cnt = 0;
  for (int base = 0; base < m; base += kRankStage) {
    const int n = min(kRankStage, m - base);
    if (base > 0) __syncthreads();  // everybody is done with the previous piece
    for (int t = tid; t < n; t += 256) keys[t] = d.key[base + t];
    __syncthreads();
#pragma unroll 8
    for (int t = slice; t < n; t += 16) {
      const double kj = keys[t];
      cnt += (kj > ki || (kj == ki && (base + t) < i)) ? 1 : 0;
    }
  }
  part[slice][il] = cnt;
  __syncthreads();
  if (slice != 0 || i >= m) return;
  int r = 0;
#pragma unroll
  for (int q = 0; q < 16; ++q) r += part[q][il];
  const int neuron = d.asc_idx[i];
  d.cross_idx[r] = neuron;
  if (d.col_of != nullptr) d.col_of[neuron] = r;
  if (flags & kRankNewBounds) {
    const double ub = d.ub[neuron];
    d.plb_out[n_in + r] = 0.0;
    d.pub_out[n_in + r] = ub;
    d.lbub[r] = d.lb[neuron];
    d.lbub[d.ld_lbub + r] = ub;
  }
}

constexpr int kApplyRows = 128;  // 64 lanes x 2 rows, the four waves interleave columns

constexpr int kApplyWaves = 8;  // waves per block of the apply pass

__global__ __launch_bounds__(64 * kApplyWaves) void relu_apply_kernel(const ReluDesc* __restrict__ table, ReluDesc one) {
  const ReluDesc d = table ? table[blockIdx.z] : one;
  const int ncols_out = d.ncols_in + (d.write_tail ? d.m : 0);  // columns of V' that are stored
  const int j0 = blockIdx.y * d.cols_per_chunk;
  if (j0 >= ncols_out) return;
  const int j1 = min(ncols_out, j0 + d.cols_per_chunk);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // row_waves waves of the block sit next to each other along the rows (contiguous memory of one
  // column), the others take different columns
  const int wrow = wave % d.row_waves;
  const int wcol = wave / d.row_waves;
  const int col_waves = kApplyWaves / d.row_waves;
  const int64_t r0 = ((int64_t)blockIdx.x * d.row_waves + wrow) * kApplyRows + 2 * lane;
  const bool active = r0 < d.ld;
  int cx = kKeep, cy = kKeep;
  if (active) {
    const int2 c = *reinterpret_cast<const int2*>(d.cls + r0);
    cx = c.x;
    cy = c.y;
  }
  // rows that are zeroed anyway are not read: lines whose 16 rows are all inactive or crossing never
  // leave HBM
  const bool need = active && (cx == kKeep || cy == kKeep);
  const int n_in = d.ncols_in - 1;
  // predicate bounds and the (lb, ub) of the crossing neurons: one thread per column of this block's
  // chunk, done by the first row block only
  if (blockIdx.x == 0 && d.write_bounds) {
    for (int j = j0 + (int)threadIdx.x; j < j1; j += 64 * kApplyWaves) {
      if (j < d.ncols_in) {
        if (j >= 1 && d.plb_out != d.plb_in) {
          d.plb_out[j - 1] = d.plb_in[j - 1];
          d.pub_out[j - 1] = d.pub_in[j - 1];
        }
      } else {
        const int i = j - d.ncols_in;
        const int neuron = d.cross_idx[i];
        const double ub = d.ub[neuron];
        d.plb_out[n_in + i] = 0.0;  // new_pred_lb = [plb; zeros(m,1)]
        d.pub_out[n_in + i] = ub;   // new_pred_ub = [pub; ub]
        d.lbub[i] = d.lb[neuron];
        d.lbub[d.ld_lbub + i] = ub;
      }
    }
    if (!d.write_tail && blockIdx.y == 0) {  // implicit columns: their predicate bounds all the same
      for (int i = (int)threadIdx.x; i < d.m; i += 64 * kApplyWaves) {
        const int neuron = d.cross_idx[i];
        const double ub = d.ub[neuron];
        d.plb_out[n_in + i] = 0.0;
        d.pub_out[n_in + i] = ub;
        d.lbub[i] = d.lb[neuron];
        d.lbub[d.ld_lbub + i] = ub;
      }
    }
  }
  // each wave takes 4 consecutive columns per step; the 4 loads are issued before any is used
  for (int jb = j0 + 4 * wcol; jb < j1; jb += 4 * col_waves) {
    double2 v[4];
    int hot[4];  // the neuron of an appended column (asked for together, ahead of the stores)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = jb + u;
      v[u] = make_double2(0.0, 0.0);
      if (need && j < j1 && j < d.ncols_in) v[u] = *reinterpret_cast<const double2*>(d.Vin + r0 + (int64_t)j * d.ld);
      hot[u] = (j >= d.ncols_in && j < j1) ? d.cross_idx[j - d.ncols_in] : -1;
    }
    if (!active) continue;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = jb + u;
      if (j >= j1) break;
      double2 o;
      if (j < d.ncols_in) {
        o.x = cx == kKeep ? v[u].x : 0.0;  // V1(map,:) = 0
        o.y = cy == kKeep ? v[u].y : 0.0;
      } else {
        const int neuron = hot[u];
        o.x = r0 == neuron ? 1.0 : 0.0;  // V2(index(i), i) = 1
        o.y = r0 + 1 == neuron ? 1.0 : 0.0;
      }
      typedef double dd2 __attribute__((ext_vector_type(2)));  // (streaming store: the pass does not read its output)
      __builtin_nontemporal_store(dd2{o.x, o.y}, reinterpret_cast<dd2*>(d.Vout + r0 + (int64_t)j * d.ld));
    }
  }
}

// unit-vector columns of a set: column j (of ncols) = e_idx[j]
__global__ void onehot_columns_kernel(double* __restrict__ V, int64_t ld, const int32_t* __restrict__ idx, int ncols) {
  for (int j = blockIdx.y; j < ncols; j += gridDim.y) {
    const int hot = idx[j];
    for (int64_t r = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; r < ld; r += (int64_t)gridDim.x * blockDim.x)
      V[r + (int64_t)j * ld] = r == hot ? 1.0 : 0.0;
  }
}

// Predicate bounds of the output and (lb, ub) of the crossing neurons, for the ReLU step that leaves
// the row reset pending: new_pred_lb = [plb; zeros(m,1)], new_pred_ub = [pub; ub(index)].
__global__ __launch_bounds__(256) void relu_bounds_kernel(const ReluDesc* __restrict__ table, ReluDesc one) {
  const ReluDesc d = table ? table[blockIdx.y] : one;
  const int n_in = d.ncols_in - 1;
  for (int j = blockIdx.x * 256 + threadIdx.x; j < n_in + d.m; j += gridDim.x * 256) write_pred_bound(d, n_in, j);
}

// The apply pass over an array of sets with a common leading dimension.  The descriptors carry Vin,
// Vout, cls, cross_idx, ncols_in, m, ld, write_tail and write_bounds (plus what the bounds need);
// the column chunking is chosen here.
static int launch_apply(nnvhip_ctx* ctx, int64_t count, std::vector<ReluDesc>& descs, double bytes) {
  const int64_t ld = descs[0].ld;
  int64_t max_cols = 0;
  for (int64_t i = 0; i < count; ++i)
    max_cols = std::max<int64_t>(max_cols, descs[i].ncols_in + (descs[i].write_tail ? descs[i].m : 0));
  // a couple of thousand blocks, at least two steps per wave
  int row_waves = ld >= 8 * kApplyRows ? 8 : ld >= 4 * kApplyRows ? 4 : ld >= 2 * kApplyRows ? 2 : 1;
  if (const int v = tune_knobs().apply_row_waves) row_waves = v == 8 ? 8 : v == 4 ? 4 : v == 2 ? 2 : 1;
  const int64_t row_blocks = ceil_div(ld, kApplyRows * row_waves);
  const int64_t min_cpc = (const int64_t)8 * (kApplyWaves / row_waves);  // two 4-column steps per wave
  int64_t want_blocks = 8192;
  if (const int v = tune_knobs().apply_blocks) want_blocks = std::max(1, v);
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(want_blocks, row_blocks * count), ceil_div(max_cols, min_cpc)));
  const int64_t cpc = ceil_div(max_cols, chunks);
  chunks = ceil_div(max_cols, cpc);
  for (int64_t i = 0; i < count; ++i) {
    descs[i].cols_per_chunk = (int32_t)cpc;
    descs[i].row_waves = row_waves;
  }
  const ReluDesc* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(ctx->upload_table(descs.data(), sizeof(ReluDesc) * count, &tab));
    table = tab->as<ReluDesc>();
  }
  NNV_TRY(ctx->kernel_timer_begin(ctx->kernel_timing));
  NNV_LAUNCH(ctx, ctx->kernel_timing, relu_apply_kernel, dim3((unsigned)row_blocks, (unsigned)chunks, (unsigned)count),
             dim3(64 * kApplyWaves), 0, table, descs[0]);
  NNV_TRY(ctx->kernel_timer_end(ctx->kernel_timing, 3, bytes));
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

// implicit unit-vector columns of a set whose rows are in place: copy and append
static int write_tail_columns(nnvhip_ctx* ctx, nnvhip_star* s) {
  const int64_t have = s->stored_cols();
  if (s->oh_idx == nullptr || s->oh_from != have || s->oh_scale != nullptr)
    NNV_FAIL(NNVHIP_ERR_ARG, "internal: implicit columns without their description");
  BufRef full;
  NNV_TRY(ctx->alloc(sizeof(double) * s->ld * (s->n + 1), &full));
  NNV_HIP_TRY(hipMemcpyAsync(full->ptr, s->V, sizeof(double) * s->ld * have, hipMemcpyDeviceToDevice, ctx->stream));
  const int m = (int)(s->n + 1 - have);
  hipLaunchKernelGGL(onehot_columns_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(s->ld, 256), 64), (unsigned)std::min(m, 4096)),
                     dim3(256), 0, ctx->stream, full->as<double>() + have * s->ld, s->ld, s->oh_idx, m);
  NNV_HIP_TRY(hipGetLastError());
  s->Vbuf = full;
  s->V = full->as<double>();
  s->vcols = -1;
  return NNVHIP_OK;
}

int ensure_dense_batch(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* sets, bool need_tail, bool need_cols) {
  // columns that were described but not written: wanted by the caller, or read by the steps below
  {
    std::vector<nnvhip_star*> cols;
    for (int64_t i = 0; i < count; ++i) {
      nnvhip_star* s = sets[i];
      if (s->cs.any_pending() && (need_cols || s->rows_pending || (need_tail && s->stored_cols() != s->n + 1))) cols.push_back(s);
    }
    if (!cols.empty()) NNV_TRY(write_pending_columns(ctx, (int64_t)cols.size(), cols.data()));
  }
  // sets with a pending row reset: one arena and one apply launch per leading dimension
  std::vector<nnvhip_star*> pend;
  const uint64_t visit = ++ctx->visit_seq;  // (a handle may be listed twice)
  for (int64_t i = 0; i < count; ++i) {
    nnvhip_star* s = sets[i];
    if (s->rows_pending) {
      if (s->visit != visit) {
        s->visit = visit;
        pend.push_back(s);
      }
    } else if (need_tail && s->stored_cols() != s->n + 1) {
      NNV_TRY(write_tail_columns(ctx, s));
    }
  }
  while (!pend.empty()) {
    std::vector<nnvhip_star*> grp, rest;
    for (auto* s : pend) (s->ld == pend[0]->ld ? grp : rest).push_back(s);
    const int64_t ld = grp[0]->ld;
    int64_t total_cols = 0;
    std::vector<ReluDesc> descs(grp.size());
    double bytes = 0.0;
    for (size_t i = 0; i < grp.size(); ++i) {
      nnvhip_star* s = grp[i];
      const int64_t have = s->stored_cols();
      const int64_t m = s->n + 1 - have;
      if (s->cls == nullptr || (m > 0 && (s->oh_idx == nullptr || s->oh_from != have)) || s->n_kept < 0)
        NNV_FAIL(NNVHIP_ERR_ARG, "internal: pending row reset without its description");
      ReluDesc& d = descs[i];
      d = ReluDesc{};
      d.Vin = s->V;
      d.cls = const_cast<int32_t*>(s->cls);
      d.cross_idx = const_cast<int32_t*>(s->oh_idx);
      d.ld = ld;
      d.N = (int32_t)s->N;
      d.ncols_in = (int32_t)have;
      d.m = (int32_t)m;
      d.write_tail = need_tail ? 1 : 0;
      d.write_bounds = 0;
      total_cols += have + (need_tail ? m : 0);
      bytes += 8.0 * (double)s->n_kept * (double)have + 8.0 * (double)s->N * (double)(have + (need_tail ? m : 0));
    }
    BufRef arena;
    NNV_TRY(ctx->alloc(sizeof(double) * ld * total_cols, &arena));
    int64_t off = 0;
    for (size_t i = 0; i < grp.size(); ++i) {
      descs[i].Vout = arena->as<double>() + off * ld;
      off += descs[i].ncols_in + (need_tail ? descs[i].m : 0);
    }
    NNV_TRY(launch_apply(ctx, (int64_t)grp.size(), descs, bytes));
    for (size_t i = 0; i < grp.size(); ++i) {
      nnvhip_star* s = grp[i];
      s->Vbuf = arena;
      s->V = descs[i].Vout;
      s->rows_pending = false;
      s->cls_buf.reset();
      s->cls = nullptr;
      s->keep_bits = nullptr;
      // The rows that were kept still hold the gathered weight columns, which is all a later packing of kept rows
      // asks of this description; nothing of it is pending any more (the apply pass read whole columns).
      s->cs.pending = false;
      s->cs.zero_to = 0;
      s->cs.win_from = s->cs.win_to = 0;
      s->cs.rows_reset = true;
      if (need_tail) s->vcols = -1;
    }
    pend.swap(rest);
  }
  return NNVHIP_OK;
}

int ensure_dense(nnvhip_ctx* ctx, nnvhip_star* s, bool need_tail) {
  if (!s->rows_pending && !s->cs.any_pending() && (!need_tail || s->stored_cols() == s->n + 1)) return NNVHIP_OK;
  return ensure_dense_batch(ctx, 1, &s, need_tail);
}

// Sets of up to this many neurons are classified by one block each (one launch for the whole step when the
// crossing list fits the in-block sort); larger ones by the multi-block kernels.  The one-block kernel walks a set
// 1024 neurons at a time, two barriers a round: 19 us at 7200 neurons, where count + compact take 4 us each.
static int64_t one_block_limit() {
  const int n = tune_knobs().one_block_n;
  return n >= 1024 && n <= 8192 ? n : 2048;
}

int relu_relax(nnvhip_ctx* ctx, int order, int64_t count, nnvhip_star* const* in, nnvhip_star** out, const ReluGiven* given) {
  // (a hint about the layer that follows is for this step, whatever becomes of it)
  const nnvhip_fc* const next_fc = ctx->next_fc;
  ctx->next_fc = nullptr;
  if (count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "at most 65535 sets per call");
  if ((order == kOrderGiven) != (given != nullptr)) NNV_FAIL(NNVHIP_ERR_ARG, "internal: explicit lists and their order go together");
  // the appended unit-vector columns are stored only on request or when the FC / conv maps are told to
  // contract over every column anyway; the row reset itself is left to whoever needs the whole matrix
  const bool eager_tail = ctx->eager_tail || ctx->dense_affine;
  const bool lazy_rows = !eager_tail && !ctx->eager_rows;
  // (with the reset left pending nothing here reads the inputs' columns: those not written yet stay so)
  NNV_TRY(ensure_dense_batch(ctx, count, in, true, !lazy_rows));
  const int64_t N = in[0]->N;
  const int64_t ld = in[0]->ld;
  const int64_t kOneBlockN = one_block_limit();
  // Larger sets are classified by several blocks, which need the class counts of the blocks before them: the kernel
  // that finishes the range estimate counts as it writes lb / ub where it is the one that runs; a counting launch
  // otherwise.
  BufRef blk_buf;
  const int64_t nblk = ceil_div(N, 1024);
  const int64_t blk_stride = 3 * std::max<int64_t>(nblk, ceil_div(ld, 64));
  RangeCounts rc;
  if (N > kOneBlockN) {
    NNV_TRY(ctx->alloc(sizeof(int32_t) * blk_stride * count, &blk_buf));
    rc.base = blk_buf->as<int32_t>();
    rc.stride = blk_stride;
    rc.nrows = (int32_t)std::min<int64_t>(N, INT32_MAX);
  }
  if (given == nullptr) NNV_TRY(compute_ranges(ctx, count, in, &rc));
  if (N >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "set dimension too large");
  const bool sorted = order != NNVHIP_ORDER_INDEX;

  // scratch shared by all sets: cls | counts ; cross_idx is kept (it becomes the node's index list)
  BufRef cls_buf, cnt_buf, asc_buf, key_buf;
  // (behind the classes: one bit per row, 1 = kept, in whole 1024-row blocks per set -- what a convolution that
  // applies the pending reset as it loads wants)
  const int64_t bit_words = ceil_div(N, 1024) * 32;
  NNV_TRY(ctx->alloc(sizeof(int32_t) * (ld + bit_words) * count, &cls_buf));
  NNV_TRY(ctx->alloc(sizeof(int32_t) * 2 * count, &cnt_buf));
  // kept-row lists of all sets in one buffer; the classification pads each list with -1 up to a whole
  // K-tile (at least one), which is what the GEMM's row map expects
  const int64_t keep_ld = round_up(N, kLdAlign) + kLdAlign;
  BufRef keep_buf;
  NNV_TRY(ctx->alloc(sizeof(int32_t) * keep_ld * count, &keep_buf));
  if (sorted) {
    NNV_TRY(ctx->alloc(sizeof(int32_t) * ld * count, &asc_buf));
    NNV_TRY(ctx->alloc(sizeof(double) * ld * count, &key_buf));
  }
  // With the reset pending, all that is left to write are the predicate bounds and the crossing
  // neurons' (lb, ub).  The one-block classification does that itself, into buffers sized for the worst
  // case (every neuron crossing), and the step is a single launch.
  // Larger sets with the reset pending: the multi-block classification leaves the counts on the device, and the
  // kernel that ranks the crossing list is queued right behind it, sized for the longest possible list; the host
  // reads the counts while it runs.
  const bool early_rank = lazy_rows && sorted && N > kOneBlockN;
  const bool fold_bounds = lazy_rows && (N <= kOneBlockN || early_rank);
  BufRef pred_buf, lbub_buf;
  std::vector<int64_t> pred_off(count), lbub_off(count), pred_cap(count, 0);
  // (sets whose predicate-bound arrays end where the set ends and have room for this step's worst case: the new
  // bounds go behind the old ones, in place; the others get arrays of their own, with room for the steps to come)
  std::vector<char> in_place(count, 0);
  Ref<PredTails> tails;
  const int64_t ldr_max = round_up(N, kLdAlign);
  if (fold_bounds) {
    int64_t total_pred = 0;
    for (int64_t i = 0; i < count; ++i) {
      const nnvhip_star* s = in[i];
      lbub_off[i] = 2 * ldr_max * i;
      in_place[i] = s->ptails && s->ptails->used[(size_t)s->pslot] == s->n && s->n + N <= s->pcap;
      if (in_place[i]) continue;
      pred_off[i] = total_pred;
      pred_cap[i] = round_up(s->n + 4 * N, kLdAlign);
      total_pred += 2 * pred_cap[i];
    }
    if (total_pred > 0) {
      NNV_TRY(ctx->alloc(sizeof(double) * total_pred, &pred_buf));
      tails = make_ref<PredTails>();
      tails->used.assign((size_t)count, -1);
    }
    NNV_TRY(ctx->alloc(sizeof(double) * 2 * ldr_max * count, &lbub_buf));
  }
  // crossing lists of all sets in one buffer (they become the constraint nodes' index lists)
  BufRef idx_buf;
  NNV_TRY(ctx->alloc(sizeof(int32_t) * ld * count, &idx_buf));
  // image sets (they carry windows): a convolution is likely to follow, whose stamp pass looks up the column of a
  // pixel; the kernels that settle the crossing list's order leave that inverse behind
  const bool want_inv = in[0]->box != nullptr && given == nullptr;
  BufRef inv_buf;
  if (want_inv) NNV_TRY(ctx->alloc(sizeof(int32_t) * ld * count, &inv_buf));
  std::vector<ReluDesc> descs(count);
  for (int64_t i = 0; i < count; ++i) {
    ReluDesc& d = descs[i];
    d = ReluDesc{};
    if (fold_bounds) {
      d.plb_out = in_place[i] ? in[i]->plb : pred_buf->as<double>() + pred_off[i];
      d.pub_out = in_place[i] ? in[i]->pub : d.plb_out + pred_cap[i];
      d.lbub = lbub_buf->as<double>() + lbub_off[i];
      d.ld_lbub = ldr_max;
      d.write_bounds = 1;
    }
    d.Vin = in[i]->V;
    d.lb = given ? given[i].lb : in[i]->lb;
    d.ub = given ? given[i].ub : in[i]->ub;
    d.given_key = given ? given[i].key : nullptr;
    d.plb_in = in[i]->plb;
    d.pub_in = in[i]->pub;
    d.cls = cls_buf->as<int32_t>() + ld * i;
    d.col_of = inv_buf ? inv_buf->as<int32_t>() + ld * i : nullptr;
    d.keep_bits = lazy_rows ? cls_buf->as<uint32_t>() + ld * count + bit_words * i : nullptr;
    d.cross_idx = idx_buf->as<int32_t>() + ld * i;
    d.asc_idx = sorted ? asc_buf->as<int32_t>() + ld * i : nullptr;
    d.key = sorted ? key_buf->as<double>() + ld * i : nullptr;
    d.counts = cnt_buf->as<int32_t>() + 2 * i;
    d.blk_counts = blk_buf ? blk_buf->as<int32_t>() + blk_stride * i : nullptr;
    d.blk_gran = rc.gran > 0 ? rc.gran : 1024;
    d.keep_idx = keep_buf->as<int32_t>() + keep_ld * i;
    d.mailbox = nullptr;
    d.ld = ld;
    d.N = (int32_t)N;
    d.ncols_in = (int32_t)(in[i]->n + 1);
    d.order = order;
  }
  const bool use_mailbox = count <= nnvhip_ctx::kMailboxSets && ctx->mailbox != nullptr && N < (int64_t(1) << kMailboxCountBits);
  if (use_mailbox) {  // every set's block posts into a word of its own
    ++ctx->mailbox_seq;
    volatile unsigned long long* box = reinterpret_cast<volatile unsigned long long*>(ctx->mailbox);
    for (int64_t i = 0; i < count; ++i) {
      box[i] = kMailboxEmpty;  // whatever an earlier call posted here is gone before the kernel is queued
      descs[i].mailbox = const_cast<int32_t*>(ctx->mailbox) + 2 * i;
      descs[i].mailbox_seq = (int32_t)(ctx->mailbox_seq & 0xffffu);
    }
    std::atomic_thread_fence(std::memory_order_seq_cst);
  }
  const ReluDesc* table = nullptr;
  BufRef tab;
  if (count > 1) {
    NNV_TRY(ctx->upload_table(descs.data(), sizeof(ReluDesc) * count, &tab));
    table = tab->as<ReluDesc>();
  }
  // Up to 8192 neurons: one block per set classifies, compacts and sorts crossing lists of up to 1024
  // entries (sorting network).  Larger sets: two multi-block passes.  Whatever is still unsorted after
  // the read-back of the counts goes to the multi-block rank kernels.
  const int sort_cap = !sorted ? 0 : N <= kOneBlockN ? kSortInBlock : 0;
  // algorithmic bytes of the classification: lb and ub read, the per-row class and the two index lists
  // written (plus, when it also writes the predicate bounds, the copy of the input's)
  double cls_bytes = 0.0;
  for (int64_t i = 0; i < count; ++i) cls_bytes += 24.0 * (double)N + (fold_bounds && !early_rank && !in_place[i] ? 32.0 * (double)in[i]->n : 0.0);
  const bool tk = ctx->kernel_timing;
  if (N <= kOneBlockN) {
    if (!sorted)
      NNV_LAUNCH(ctx, tk, relu_classify_kernel<0>, dim3((unsigned)count), dim3(1024), 0, table, descs[0]);
    else if (N <= 1024)
      NNV_LAUNCH(ctx, tk, relu_classify_kernel<1024>, dim3((unsigned)count), dim3(1024), 0, table, descs[0]);
    else
      NNV_LAUNCH(ctx, tk, relu_classify_kernel<8192>, dim3((unsigned)count), dim3(1024), 0, table, descs[0]);
    NNV_TRY(ctx->kernel_timer_end(tk, 6, cls_bytes));
  } else {
    const dim3 grid((unsigned)ceil_div(N, 1024), 1, (unsigned)count);
    if (rc.gran == 0) {
      NNV_LAUNCH(ctx, tk, relu_count_kernel, grid, dim3(1024), 0, table, descs[0]);
      NNV_TRY(ctx->kernel_timer_end(tk, 6, 0.5 * cls_bytes));
    }
    NNV_LAUNCH(ctx, tk, relu_compact_kernel, grid, dim3(1024), 0, table, descs[0]);
    NNV_TRY(ctx->kernel_timer_end(tk, 6, 0.5 * cls_bytes));
    if (early_rank)
      hipLaunchKernelGGL(relu_rank_kernel, dim3((unsigned)ceil_div(N, kRankI), 1, (unsigned)count), dim3(256), 0, ctx->stream, table,
                         descs[0], kRankNewBounds | kRankOldBounds | kRankCountOnDevice);
  }
  NNV_HIP_TRY(hipGetLastError());

  // An array whose caller has said which FC layer comes next: that layer's range sums of the columns this step
  // appends need only the per-row classes and the input's upper bounds, both on the device by now, and no count.
  // Queued here, the product runs while the host reads the counts, makes the handles and sets the layer call up.
  BufRef ahead_mm;
  if (next_fc != nullptr && given == nullptr && lazy_rows && count >= 64 && !ctx->eager_cols && !ctx->dense_affine &&
      next_fc->K == N && next_fc->ctx == ctx) {
    std::vector<AheadSet> as((size_t)count);
    for (int64_t i = 0; i < count; ++i) as[(size_t)i] = AheadSet{descs[i].cls, descs[i].ub};
    NNV_TRY(launch_range_sums_mm_ahead(ctx, next_fc, count, as.data(), N, &ahead_mm));
  }

  // Output handles: whatever does not depend on the counts is set up while the kernel runs (with the
  // row reset pending and the bounds written by the kernel, that is nearly everything).
  auto init_static = [&](nnvhip_star* o, ConsNode* node, int64_t i) {
    o->N = N;
    o->ld = ld;
    if (lazy_rows) {  // shares the input's matrix until somebody needs the rows reset in memory
      o->Vbuf = in[i]->Vbuf;
      o->V = in[i]->V;
      o->vcols = in[i]->n + 1;
      o->rows_pending = true;
      o->cls_buf = cls_buf;
      o->cls = cls_buf->as<int32_t>() + ld * i;
      o->keep_bits = cls_buf->as<uint32_t>() + ld * count + bit_words * i;
      // ... and what is known about where its columns came from (and whether they are in memory yet)
      // holds for the rows that are kept -- unless rows of the input's matrix were reset in memory after the gather
      // (this step may keep such a row)
      o->cs = in[i]->cs.rows_reset ? ColSource() : in[i]->cs;
    }
    {
      // resetting rows leaves every generator image inside its window (the columns the step appends come
      // after the ones the windows describe)
      o->box_buf = in[i]->box_buf;
      o->box = in[i]->box;
      o->box_cols = in[i]->box_cols;
      o->box_H = in[i]->box_H;
      o->box_W = in[i]->box_W;
      o->box_eh = in[i]->box_eh;
      o->box_ew = in[i]->box_ew;
    }
    o->kept_buf = keep_buf;
    o->kept_idx = keep_buf->as<int32_t>() + keep_ld * i;
    node->prev = in[i]->cons;
    node->n_before = in[i]->n;
    node->src = in[i]->Vbuf;  // zero-copy: C2/C3 rows are rows of the input's immutable [c V]
    node->src_V = in[i]->V;
    node->src_ld = in[i]->ld;
    node->src_cs = in[i]->cs;
    node->index = idx_buf;
    node->index_off = ld * i;
  };
  struct PreCreated {
    std::vector<nnvhip_star*> v;
    ~PreCreated() { release_all(v); }  // only what was not handed over
  } pre;
  std::vector<ConsRef> nodes;
  const bool precreate = lazy_rows && fold_bounds && count > 1;
  if (precreate) {
    pre.v.reserve(count);
    nodes.resize(count);
    for (int64_t i = 0; i < count; ++i) {
      pre.v.push_back(new_star(ctx));
      nodes[i] = make_ref<ConsNode>();
      init_static(pre.v[i], nodes[i].get(), i);
    }
  }

  // the column count of the output depends on m: fetch the counts
  std::vector<int32_t> counts(2 * count);
  if (use_mailbox) {
    // the kernels post the counts to pinned host memory; spin until every word has been overwritten
    const auto t0 = std::chrono::steady_clock::now();
    long spins = 0;
    const volatile unsigned long long* box = reinterpret_cast<const volatile unsigned long long*>(ctx->mailbox);
    for (int64_t i = 0; i < count; ++i) {
      unsigned long long w = box[i];
      while (w == kMailboxEmpty) {
        if (!ctx->deferred.empty()) ctx->drain_deferred(16);  // something useful to do while the device works
        if ((++spins & 0xfff) == 0 &&
            std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 10.0) {
          NNV_HIP_TRY(hipStreamSynchronize(ctx->stream));  // surfaces a launch failure, if any
          if (box[i] == kMailboxEmpty) NNV_FAIL(NNVHIP_ERR_HIP, "classification kernel did not report its counts");
        }
        w = box[i];
      }
      int m_ = 0, inact_ = 0, seq_ = 0;
      mailbox_unpack(w, &m_, &inact_, &seq_);
      if (seq_ != (int)(ctx->mailbox_seq & 0xffffu)) NNV_FAIL(NNVHIP_ERR_HIP, "internal: mailbox word of another call");
      counts[2 * i] = m_;
      counts[2 * i + 1] = inact_;
    }
  } else {
    void* hc = nullptr;
    NNV_TRY(ctx->stage(sizeof(int32_t) * 2 * count, &hc));
    NNV_HIP_TRY(hipMemcpyAsync(hc, cnt_buf->ptr, sizeof(int32_t) * 2 * count, hipMemcpyDeviceToHost, ctx->stream));
    NNV_HIP_TRY(hipStreamSynchronize(ctx->stream));
    memcpy(counts.data(), hc, sizeof(int32_t) * 2 * count);
  }

  // outputs: one V arena, one predicate-bound buffer, one buffer for the crossing bounds
  int64_t total_cols = 0, total_pred = 0, total_lbub = 0, max_m = 0, max_pred = 0;
  std::vector<int64_t> col_off(count);
  for (int64_t i = 0; i < count; ++i) {
    const int64_t m = counts[2 * i];
    const int64_t ncols_out = in[i]->n + 1 + (eager_tail ? m : 0);  // stored columns
    const int64_t ldr = round_up(std::max<int64_t>(m, 1), kLdAlign);
    col_off[i] = total_cols;
    total_cols += ncols_out;
    if (!fold_bounds) {
      pred_off[i] = total_pred;
      lbub_off[i] = total_lbub;
      total_pred += 2 * round_up(std::max<int64_t>(in[i]->n + m, 1), kLdAlign);
      total_lbub += m > 0 ? 2 * ldr : 0;
    }
    max_m = std::max(max_m, m);
    max_pred = std::max(max_pred, in[i]->n + m);
  }
  BufRef arena;
  if (!lazy_rows) NNV_TRY(ctx->alloc(sizeof(double) * ld * total_cols, &arena));
  if (!fold_bounds) {
    NNV_TRY(ctx->alloc(sizeof(double) * total_pred, &pred_buf));
    if (total_lbub > 0) NNV_TRY(ctx->alloc(sizeof(double) * total_lbub, &lbub_buf));
  }
  for (int64_t i = 0; i < count; ++i) {
    ReluDesc& d = descs[i];
    const int64_t m = counts[2 * i];
    d.m = (int32_t)m;
    d.Vout = lazy_rows ? nullptr : arena->as<double>() + col_off[i] * ld;
    d.write_tail = eager_tail ? 1 : 0;
    if (fold_bounds) continue;  // bounds are in place already
    const int64_t ldr = round_up(std::max<int64_t>(m, 1), kLdAlign);
    const int64_t npad = round_up(std::max<int64_t>(in[i]->n + m, 1), kLdAlign);
    d.plb_out = pred_buf->as<double>() + pred_off[i];
    d.pub_out = d.plb_out + npad;
    d.lbub = m > 0 ? lbub_buf->as<double>() + lbub_off[i] : nullptr;
    d.ld_lbub = ldr;
    d.write_bounds = 1;
  }
  // lists the classification block left unsorted (and, with them, bounds it left unwritten)
  const bool need_rank = sorted && sort_cap > 0 && max_m > sort_cap;
  // lists too long for any in-LDS sort go to the rank kernel
  const bool rank_lists = sorted && max_m > sort_cap && !(sort_cap == 0 && max_m <= 1024);
  bool ranked_with_bounds = false;
  if (count > 1 && (!fold_bounds || need_rank)) {
    NNV_TRY(ctx->upload_table(descs.data(), sizeof(ReluDesc) * count, &tab));
    table = tab->as<ReluDesc>();
  }
  if (early_rank) {
    // ranked already
  } else if (sorted && sort_cap == 0 && max_m > 0 && max_m <= 1024) {
    // (with the reset pending the kernel also writes the predicate bounds, as the rank kernel below does)
    ranked_with_bounds = lazy_rows;
    const int flags = lazy_rows ? (kRankNewBounds | (fold_bounds ? 0 : kRankOldBounds)) : 0;
    hipLaunchKernelGGL(relu_sort_small_kernel, dim3((unsigned)count), dim3(1024), 0, ctx->stream, table, descs[0], flags);
  } else if (rank_lists) {

    // with the reset pending the kernel also writes the predicate bounds (the old ones were copied by the
    // one-block classification where that ran with the output buffers in place)
    ranked_with_bounds = lazy_rows;
    const int flags = lazy_rows ? (kRankNewBounds | (fold_bounds ? 0 : kRankOldBounds)) : 0;
    hipLaunchKernelGGL(relu_rank_kernel, dim3((unsigned)ceil_div(max_m, kRankI), 1, (unsigned)count), dim3(256), 0, ctx->stream, table,
                       descs[0], flags);
  }
  if ((fold_bounds && !need_rank) || ranked_with_bounds) {
    // nothing left to launch
  } else if (lazy_rows) {
    if (max_pred > 0) {
      hipLaunchKernelGGL(relu_bounds_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(max_pred, 256), 64), (unsigned)count),
                         dim3(256), 0, ctx->stream, table, descs[0]);
      NNV_HIP_TRY(hipGetLastError());
    }
  } else {
    double bytes = 0.0;  // algorithmic: read the rows that are kept, write N x (n+1+m)
    for (int64_t i = 0; i < count; ++i) {
      const double kept = (double)(N - counts[2 * i] - counts[2 * i + 1]);
      bytes += 8.0 * kept * (double)(in[i]->n + 1) +
               8.0 * (double)N * (double)(in[i]->n + 1 + (eager_tail ? descs[i].m : 0));
    }
    NNV_TRY(launch_apply(ctx, count, descs, bytes));
  }

  for (int64_t i = 0; i < count; ++i) {
    const ReluDesc& d = descs[i];
    nnvhip_star* o = precreate ? pre.v[i] : new_star(ctx);
    ConsRef node = precreate ? std::move(nodes[i]) : make_ref<ConsNode>();
    if (!precreate) init_static(o, node.get(), i);
    o->n = in[i]->n + d.m;
    if (!lazy_rows) {
      o->Vbuf = arena;
      o->V = d.Vout;
      // where the input's columns were gathered from: still true of the rows this step keeps (a later packing of
      // kept rows reads the cache-resident weights instead of this matrix); everything is in memory
      o->cs = in[i]->cs.rows_reset ? ColSource() : in[i]->cs;
      o->cs.pending = false;
      o->cs.zero_to = 0;
      o->cs.win_from = o->cs.win_to = 0;
      o->cs.rows_reset = true;
    }
    (fold_bounds && in_place[i] ? ctx->n_bounds_in_place : ctx->n_bounds_copied)++;
    if (fold_bounds && in_place[i]) {
      o->pbuf = in[i]->pbuf;
      o->ptails = in[i]->ptails;
      o->pslot = in[i]->pslot;
      o->pcap = in[i]->pcap;
      o->ptails->used[(size_t)o->pslot] = o->n;
    } else {
      o->pbuf = pred_buf;
      if (fold_bounds) {
        o->ptails = tails;
        o->pslot = i;
        o->pcap = pred_cap[i];
        tails->used[(size_t)i] = o->n;
      }
    }
    o->plb = d.plb_out;
    o->pub = d.pub_out;
    o->n_inactive = counts[2 * i + 1];
    o->n_crossing = d.m;
    if (given == nullptr) {  // the input's estimated upper bounds, by neuron
      o->pre_ub_buf = in[i]->rbuf;
      o->pre_ub = in[i]->ub;
    }
    if (ahead_mm) {
      o->ahead_mm_buf = ahead_mm;
      o->ahead_mm_uid = next_fc->uid;
      o->ahead_mm_slot = i;
    }
    if (d.m > 0) {  // the appended columns are the unit vectors of the crossing neurons
      o->oh_from = in[i]->n + 1;
      o->oh_plb_zero = true;
      o->oh_idx_buf = idx_buf;
      o->oh_idx = idx_buf->as<int32_t>() + ld * i;
      if (inv_buf) {
        o->oh_inv_buf = inv_buf;
        o->oh_inv = inv_buf->as<int32_t>() + ld * i;
      }
      if (!eager_tail) o->vcols = in[i]->n + 1;  // ... and exist only as that list
    }
    // rows of the leading columns that were not reset
    o->n_kept = N - counts[2 * i] - counts[2 * i + 1];
    if (d.m > 0) {
      node->m = d.m;
      node->p_total = in[i]->cons->p_total + 3 * (int64_t)d.m;
      node->n_total = o->n;
      node->ld_lbub = d.ld_lbub;
      node->lbub = lbub_buf;
      node->lbub_off = lbub_off[i];  // a view into a shared buffer: the element offset
      o->cons = std::move(node);
    } else {
      o->cons = in[i]->cons;  // no crossing neuron: C, d unchanged
    }
    out[i] = o;
  }
  pre.v.clear();  // handed over
  return NNVHIP_OK;
}

// ---- dense constraint materialisation -----------------------------------------------------------

__global__ void cons_copy_kernel(double* __restrict__ C, int64_t ldC, const double* __restrict__ C0, int64_t ldc0,
                                 int64_t p0, int64_t n0) {
  const int64_t total = p0 * n0;
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = t % p0, c = t / p0;
    C[r + c * ldC] = C0[r + c * ldc0];
  }
}

// Rows of one ReLU node (nn/funcs/PosLin.m:711-735), r0 = rows before it, nb = n_before:
//   C1 = [0 -I], d1 = 0;  C2 = [V(index,2:n+1) -I], d2 = -V(index,1);
//   a = ub./(ub-lb); b = a.*lb;  C3 = [-a.*V(index,2:n+1) I], d3 = a.*V(index,1) - b.
__global__ void cons_relu_kernel(double* __restrict__ C, int64_t ldC, double* __restrict__ dvec, int64_t r0, int m,
                                 int nb, const double* __restrict__ rows, int64_t ld_rows,
                                 const int32_t* __restrict__ index, const double* __restrict__ lb,
                                 const double* __restrict__ ub) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= m) return;
  const int src = index[i];  // I.V(index(i), :)
  const double a = ub[i] / (ub[i] - lb[i]);
  const int64_t row1 = r0 + i, row2 = r0 + m + i, row3 = r0 + 2 * (int64_t)m + i;
  for (int j = blockIdx.y; j <= nb; j += gridDim.y) {
    const double v = rows[src + (int64_t)j * ld_rows];
    if (j == 0) {
      dvec[row1] = 0.0;
      dvec[row2] = -v;
      dvec[row3] = __dsub_rn(__dmul_rn(a, v), __dmul_rn(a, lb[i]));
      C[row1 + (int64_t)(nb + i) * ldC] = -1.0;
      C[row2 + (int64_t)(nb + i) * ldC] = -1.0;
      C[row3 + (int64_t)(nb + i) * ldC] = 1.0;
    } else {
      C[row2 + (int64_t)(j - 1) * ldC] = v;
      C[row3 + (int64_t)(j - 1) * ldC] = __dmul_rn(-a, v);
    }
  }
}

int materialize_constraints(const nnvhip_star* s, double* C_host, double* d_host) {
  nnvhip_ctx* ctx = s->ctx;
  const int64_t p = s->cons->p_total, n = s->n;
  if (p == 0) return NNVHIP_OK;
  std::vector<const ConsNode*> chain;
  for (const ConsNode* nd = s->cons.get(); nd; nd = nd->prev.get()) chain.push_back(nd);
  std::reverse(chain.begin(), chain.end());
  BufRef Cd, dd;
  if (n > 0) {
    NNV_TRY(ctx->alloc(sizeof(double) * p * n, &Cd));
    NNV_HIP_TRY(hipMemsetAsync(Cd->ptr, 0, sizeof(double) * p * n, ctx->stream));
  }
  NNV_TRY(ctx->alloc(sizeof(double) * p, &dd));
  NNV_HIP_TRY(hipMemsetAsync(dd->ptr, 0, sizeof(double) * p, ctx->stream));
  double* Cp = Cd ? Cd->as<double>() : nullptr;
  int64_t r0 = 0;
  for (const ConsNode* nd : chain) {
    if (!nd->prev) {  // base node
      if (nd->C0 && Cp && nd->n_total > 0)
        hipLaunchKernelGGL(cons_copy_kernel, dim3(1024), dim3(256), 0, ctx->stream, Cp, p, nd->C0->as<double>(), nd->ldc,
                           nd->p_total, nd->n_total);
      if (nd->d0)
        NNV_HIP_TRY(hipMemcpyAsync(dd->ptr, nd->d0->ptr, sizeof(double) * nd->p_total, hipMemcpyDeviceToDevice, ctx->stream));
      r0 = nd->p_total;
    } else {
      double* Cuse = Cp;
      const int64_t ldC = p;
      // the crossing rows are read from the pre-ReLU matrix: columns of it that were never needed until
      // now are written first (into the matrix itself; the node's copy of the description is updated)
      NNV_TRY(write_pending_columns(ctx, const_cast<double*>(nd->src_V), nd->src_ld, const_cast<ColSource*>(&nd->src_cs)));
      const double* rows = nd->src_V;
      const double* lbp = nd->lbub->as<double>() + nd->lbub_off;
      dim3 grid((unsigned)ceil_div(nd->m, 128), (unsigned)std::min<int64_t>(nd->n_before + 1, 1024));
      hipLaunchKernelGGL(cons_relu_kernel, grid, dim3(128), 0, ctx->stream, Cuse, ldC, dd->as<double>(), r0, (int)nd->m,
                         (int)nd->n_before, rows, nd->src_ld, nd->index->as<int32_t>() + nd->index_off, lbp, lbp + nd->ld_lbub);
      r0 += 3 * nd->m;
    }
  }
  NNV_HIP_TRY(hipGetLastError());
  if (Cp && C_host) NNV_HIP_TRY(hipMemcpyAsync(C_host, Cp, sizeof(double) * p * n, hipMemcpyDeviceToHost, ctx->stream));
  if (d_host) NNV_HIP_TRY(hipMemcpyAsync(d_host, dd->ptr, sizeof(double) * p, hipMemcpyDeviceToHost, ctx->stream));
  NNV_HIP_TRY(hipStreamSynchronize(ctx->stream));
  return NNVHIP_OK;
}

}  // namespace nnvhip
