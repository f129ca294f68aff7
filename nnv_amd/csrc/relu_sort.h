// The descriptor of one set's ReLU step and the in-block sorting network of the classification kernel.
#pragma once
#include "internal.h"

namespace nnvhip {

constexpr int kKeep = -1;  // active neuron (lb >= 0, ub > 0): row untouched
constexpr int kZero = -2;  // inactive neuron (ub <= 0): row reset to 0

struct ReluDesc {
  const double* Vin;
  double* Vout;
  const double* lb;  // estimated ranges of the input set
  const double* ub;
  const double* plb_in;
  const double* pub_in;
  double* plb_out;
  double* pub_out;
  int32_t* cls;        // per row: kKeep, kZero or the crossing neuron's position in ascending order
  int32_t* cross_idx;  // crossing neuron indices in new-predicate order
  int32_t* asc_idx;    // crossing neuron indices in ascending order (sort orders only)
  double* key;         // sort keys, ascending-index order
  const double* given_key;  // order kOrderGiven: the key of every row is handed in (callers with an explicit list)
  int32_t* counts;     // [0] = m (crossing), [1] = inactive
  int32_t* keep_idx;   // rows left untouched (active neurons), ascending, then -1 up to a multiple of 16
  int32_t* blk_counts; // multi-block classification: {crossing, inactive, kept} per block of blk_gran rows (1024, or the
                       // 64 / 128 rows of a block of the kernel that finished the range estimate and counted as it went)
  int32_t* col_of;     // per row: the crossing neuron's place in new-predicate order, -1 for the other rows; or null
  uint32_t* keep_bits; // one bit per row, 1 = kept (word w: rows 32w .. 32w+31), for whole 1024-row blocks; or null
  int32_t* mailbox;    // host-pinned {m, inactive, seq}; null = counts are fetched by a copy instead
  int32_t mailbox_seq;
  int32_t blk_gran;
  double* lbub;        // lb then ub (offset ld_lbub) of the crossing neurons, new-predicate order
  int64_t ld;
  int64_t ld_lbub;
  int32_t N;
  int32_t ncols_in;  // n + 1
  int32_t m;
  int32_t order;
  int32_t cols_per_chunk;
  int32_t row_waves;  // apply pass: waves of a block laid along rows (1, 2, 4 or 8); the rest along columns
  int32_t write_tail; // apply pass: 1 = store the appended unit-vector columns, 0 = leave them implicit
  int32_t write_bounds; // apply pass: 1 = also write the predicate bounds and the crossing neurons' (lb, ub)
};

// Posts the counts to the host mailbox.  Payload and call number travel in one naturally aligned
// 64-bit store (call number in the top 16 bits, the two counts in 24 bits each), so there is nothing
// to order and nothing for the posting wave to wait for.  The host does not recognise a fresh word by
// its call number: before the launch it overwrites every word the call will use with kMailboxEmpty
// and waits until the word differs from that.  A posted word can never equal kMailboxEmpty (both
// counts would have to be 2^24 - 1, and their sum is at most the set's dimension, which is below
// 2^24), so a word some earlier call left behind cannot be taken for this call's, whatever the call
// numbers are.  The 16-bit call number is only cross-checked after the word has arrived.
__device__ __forceinline__ void post_counts(int32_t* mailbox, int m, int inactive, int seq) {
  if (mailbox == nullptr) return;
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(mailbox), mailbox_word(m, inactive, seq), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_SYSTEM);
}

// "a sorts before b" under the stable descending key order: larger key first, ties by smaller
// neuron index (MATLAB's sort(...,'descend') keeps equal keys in their original, ascending order).
__device__ __forceinline__ bool sorts_before(double ka, int ia, double kb, int ib) {
  return ka > kb || (ka == kb && ia < ib);
}

constexpr int kSortInBlock = 1024;  // longest crossing list the classification block sorts itself

// ---- sorting network for lists of at most 1024 entries, one entry per thread -------------------
// Keys are non-negative doubles, so their bit patterns order like signed 64-bit integers; the
// sentinel (minimum integer) sorts after every real entry.  The network is the "flip" form of the
// bitonic sort: for k = 2, 4, ..., P every block of k entries first exchanges i <-> i ^ (k-1), then
// i <-> i ^ j for j = k/4, ..., 1, always leaving the entry that sorts first in the lower slot.
// All exchange distances are compile-time constants, so distances inside a row of 16 lanes use DPP
// moves, distances inside 32 lanes ds_swizzle, 32..63 ds_bpermute, and only the 10 widest of the 55
// stages go through LDS with block barriers.
template <int MASK>
__device__ __forceinline__ int lane_xor(int v) {
  static_assert(MASK >= 1 && MASK < 64, "exchange inside one wave");
  if constexpr (MASK == 1) {
    return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
  } else if constexpr (MASK == 2) {
    return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
  } else if constexpr (MASK == 3) {
    return __builtin_amdgcn_update_dpp(v, v, 0x1B, 0xF, 0xF, false);  // quad_perm [3,2,1,0]
  } else if constexpr (MASK == 7) {
    return __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false);  // row_half_mirror
  } else if constexpr (MASK == 15) {
    return __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false);  // row_mirror
  } else if constexpr (MASK == 8) {
    return __builtin_amdgcn_update_dpp(v, v, 0x128, 0xF, 0xF, false);  // row_ror:8
  } else if constexpr (MASK == 4) {
    // banks 0 and 2 (lanes 0-3, 8-11 of a row) read lane+4, banks 1 and 3 read lane-4
    const int r = __builtin_amdgcn_update_dpp(v, v, 0x104, 0xF, 0x5, false);  // row_shl:4
    return __builtin_amdgcn_update_dpp(r, v, 0x114, 0xF, 0xA, false);         // row_shr:4
  } else if constexpr (MASK < 32) {
    return __builtin_amdgcn_ds_swizzle(v, 0x1F | (MASK << 10));  // bit-mask mode: lane ^ MASK within 32
  } else {
    return __shfl_xor(v, MASK);
  }
}

// One compare-exchange stage: partner = tid ^ MASK; the slot whose LOWBIT bit of tid is clear keeps
// the entry that sorts first (larger key; equal keys: smaller neuron index).
template <int MASK, int LOWBIT>
__device__ __forceinline__ void sort_stage(long long& key, int& idx, long long* skey, int* sidx, int tid) {
  long long pk;
  int pi;
  if constexpr (MASK >= 64) {
    __syncthreads();
    skey[tid] = key;
    sidx[tid] = idx;
    __syncthreads();
    pk = skey[tid ^ MASK];
    pi = sidx[tid ^ MASK];
  } else {
    const int lo = lane_xor<MASK>((int)(unsigned)(key & 0xffffffffll));
    const int hi = lane_xor<MASK>((int)(key >> 32));
    pk = ((long long)hi << 32) | (unsigned)lo;
    pi = lane_xor<MASK>(idx);
  }
  const bool mine_first = key > pk || (key == pk && idx < pi);
  const bool lower = (tid & LOWBIT) == 0;
  if (mine_first != lower) {
    key = pk;
    idx = pi;
  }
}

template <int K, int J>
__device__ __forceinline__ void sort_steps(long long& key, int& idx, long long* skey, int* sidx, int tid) {
  if constexpr (J >= 1) {
    sort_stage<J, J>(key, idx, skey, sidx, tid);
    sort_steps<K, J / 2>(key, idx, skey, sidx, tid);
  }
}

template <int P, int K>
__device__ __forceinline__ void sort_merges(long long& key, int& idx, long long* skey, int* sidx, int tid) {
  if constexpr (K <= P) {
    sort_stage<K - 1, K / 2>(key, idx, skey, sidx, tid);  // flip: i <-> i ^ (k-1)
    sort_steps<K, K / 4>(key, idx, skey, sidx, tid);
    sort_merges<P, 2 * K>(key, idx, skey, sidx, tid);
  }
}

// Sorts m <= 1024 (key bits, neuron) pairs staged in skey/sidx[0..m) and writes the neuron indices
// in sorted order to out[0..m).  All 1024 threads of the block must call it; thread t < m gets back entry t of
// the sorted list.
__device__ __forceinline__ int sort_small_desc(long long* skey, int* sidx, int m, int tid, int32_t* __restrict__ out) {
  long long key = tid < m ? skey[tid] : (long long)0x8000000000000000ull;
  int idx = tid < m ? sidx[tid] : 0x7fffffff;
  if (m <= 64) sort_merges<64, 2>(key, idx, skey, sidx, tid);
  else if (m <= 128) sort_merges<128, 2>(key, idx, skey, sidx, tid);
  else if (m <= 256) sort_merges<256, 2>(key, idx, skey, sidx, tid);
  else if (m <= 512) sort_merges<512, 2>(key, idx, skey, sidx, tid);
  else sort_merges<1024, 2>(key, idx, skey, sidx, tid);
  if (tid < m) out[tid] = idx;
  return idx;
}

// Entry j of the output's predicate bounds, new_pred_lb = [plb; zeros(m,1)], new_pred_ub = [pub; ub(index)]
// (nn/funcs/PosLin.m:737-738), plus the (lb, ub) of crossing neuron j - n_in that the constraint rows need.
__device__ __forceinline__ void write_pred_bound(const ReluDesc& d, int n_in, int j) {
  if (j < n_in) {
    d.plb_out[j] = d.plb_in[j];
    d.pub_out[j] = d.pub_in[j];
  } else {
    const int i = j - n_in;
    const int neuron = d.cross_idx[i];
    const double ub = d.ub[neuron];
    d.plb_out[j] = 0.0;
    d.pub_out[j] = ub;
    d.lbub[i] = d.lb[neuron];
    d.lbub[d.ld_lbub + i] = ub;
  }
}


}  // namespace nnvhip
