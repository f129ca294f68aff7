// Internal definitions shared by the translation units of libnnvhip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "nnvhip.h"

namespace nnvhip {

// Leading dimensions of every device matrix are multiples of 16 doubles (one 128-byte line), and
// the padding rows [N, ld) of every generator matrix are kept at exactly zero, so kernels may
// read whole 16-row groups and the GEMM K loop needs no tail handling.
constexpr int64_t kLdAlign = 16;

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline int64_t ceil_div(int64_t x, int64_t m) { return (x + m - 1) / m; }

void set_error(const char* fmt, ...);

#define NNV_HIP_TRY(expr)                                                                       \
  do {                                                                                          \
    hipError_t e_ = (expr);                                                                     \
    if (e_ != hipSuccess) {                                                                     \
      ::nnvhip::set_error("HIP error '%s' at %s:%d in %s", hipGetErrorString(e_), __FILE__,     \
                          __LINE__, #expr);                                                     \
      return e_ == hipErrorOutOfMemory ? NNVHIP_ERR_OOM : NNVHIP_ERR_HIP;                       \
    }                                                                                           \
  } while (0)

#define NNV_TRY(expr)                 \
  do {                                \
    int s_ = (expr);                  \
    if (s_ != NNVHIP_OK) return s_;   \
  } while (0)

// start of every entry point that takes a context: rejects null and selects the context's device
#define CHECK_CTX(c)                                                  \
  do {                                                                \
    if (!(c)) NNV_FAIL(NNVHIP_ERR_ARG, "null context");               \
    NNV_TRY(nnvhip::enter_ctx(c));                                    \
  } while (0)

#define NNV_FAIL(code, ...)             \
  do {                                  \
    ::nnvhip::set_error(__VA_ARGS__);   \
    return (code);                      \
  } while (0)

// Reference-counted pointer with a plain count inside the object it points to.  A context and everything made from
// it are used from one host thread at a time (the reference's layer loop is single-threaded, and the pool below
// has no lock either), so the count needs no atomic operations: an array of a thousand sets copies tens of
// thousands of these per layer, and the locked increments of std::shared_ptr were most of the host time of a
// ReLU step over such an array.
template <class T>
class Ref {
 public:
  Ref() = default;
  Ref(std::nullptr_t) {}
  explicit Ref(T* p) : p_(p) {
    if (p_) ++p_->ref_count;
  }
  Ref(const Ref& o) : p_(o.p_) {
    if (p_) ++p_->ref_count;
  }
  Ref(Ref&& o) noexcept : p_(o.p_) { o.p_ = nullptr; }
  Ref& operator=(const Ref& o) {
    if (o.p_) ++o.p_->ref_count;
    release();
    p_ = o.p_;
    return *this;
  }
  Ref& operator=(Ref&& o) noexcept {
    if (this != &o) {
      release();
      p_ = o.p_;
      o.p_ = nullptr;
    }
    return *this;
  }
  ~Ref() { release(); }
  void reset() {
    release();
    p_ = nullptr;
  }
  T* get() const { return p_; }
  T* operator->() const { return p_; }
  T& operator*() const { return *p_; }
  explicit operator bool() const { return p_ != nullptr; }
  bool operator==(const Ref& o) const { return p_ == o.p_; }
  bool operator!=(const Ref& o) const { return p_ != o.p_; }
  bool operator==(std::nullptr_t) const { return p_ == nullptr; }
  bool operator!=(std::nullptr_t) const { return p_ != nullptr; }

 private:
  void release() {
    if (p_ && --p_->ref_count == 0) delete p_;
  }
  T* p_ = nullptr;
};
template <class T>
Ref<T> make_ref() {
  return Ref<T>(new T());
}

struct Buffer {
  int64_t ref_count = 0;
  nnvhip_ctx* ctx = nullptr;
  void* ptr = nullptr;
  size_t bytes = 0;  // size class the block belongs to
  ~Buffer();
  template <class T>
  T* as() const { return static_cast<T*>(ptr); }
};
using BufRef = Ref<Buffer>;

// Word a ReLU classification kernel posts to the host mailbox: call number in the top 16 bits, the
// crossing and the inactive count in 24 bits each.  kMailboxEmpty is what the host stores into a word
// before the launch that will post to it; no posted word equals it (see post_counts in relu.hip).
constexpr int kMailboxCountBits = 24;
constexpr unsigned long long kMailboxEmpty = ~0ull;
__host__ __device__ inline unsigned long long mailbox_word(int m, int inactive, int seq) {
  return ((unsigned long long)((unsigned)seq & 0xffffu) << (2 * kMailboxCountBits)) |
         ((unsigned long long)((unsigned)m & ((1u << kMailboxCountBits) - 1)) << kMailboxCountBits) |
         (unsigned long long)((unsigned)inactive & ((1u << kMailboxCountBits) - 1));
}
inline void mailbox_unpack(unsigned long long w, int* m, int* inactive, int* seq) {
  *m = (int)((w >> kMailboxCountBits) & ((1u << kMailboxCountBits) - 1));
  *inactive = (int)(w & ((1u << kMailboxCountBits) - 1));
  *seq = (int)(w >> (2 * kMailboxCountBits));
}

// Tuning knobs for experiments, read from the environment once per process (0 / empty: not set):
// NNVHIP_GEMM_XR, NNVHIP_GEMM_KSPLIT, NNVHIP_GEMM_TILE ("TMxTN"), NNVHIP_RANGES_ROW_WAVES,
// NNVHIP_RANGES_BLOCKS, NNVHIP_APPLY_ROW_WAVES, NNVHIP_APPLY_BLOCKS, NNVHIP_CONV_GENERAL (1: every convolution
// on the general kernel), NNVHIP_ONE_BLOCK_N (1024 .. 8192: largest set the one-block classification takes).
struct TuneKnobs {
  int gemm_xr = 0, gemm_ksplit = 0;
  std::string gemm_tile;
  int ranges_row_waves = 0, ranges_blocks = 0, apply_row_waves = 0, apply_blocks = 0;
  int conv_general = 0;
  int one_block_n = 0;
};
const TuneKnobs& tune_knobs();

// Window of an image (rows h0..h1, columns w0..w1, inclusive) outside which a generator image is zero.
struct ColBox {
  int16_t h0, h1, w0, w1;
};

// One set of launch_delta_tiles (declared further down): its output is its group's shared product (base) plus the
// row differences of (+/-) A(:, r) * S(r, j), the centre column replaced by cprod (+ bias).
struct DeltaOut {
  const int32_t* delta;  // dlen entries: r or r | kSegSubtract
  const double* base;    // Mp x ncols, leading dimension Mp
  const double* S;       // the group's scaled rows, row-major: S(r, j) at S[r * lds + j]
  int64_t lds;
  const double* cprod;   // Mp entries
  double* out;           // the set's column 0 (leading dimension ldo)
  const double* plb;     // the set's predicate bounds, by generator column
  const double* pub;
  double* rpart;
  int32_t dlen;
  int32_t ncols;
};
// Predicate-bound arrays with room behind their last entry (one record per ReLU call that allocated such arrays,
// shared by the handles that point into them).  used[slot] = entries of the slot's arrays that are taken: a ReLU step
// whose input ends exactly there, and whose worst case fits the room, appends its new predicates' bounds in place
// instead of copying the old ones into arrays of its own (the input keeps reading its first n entries).
struct PredTails {
  int64_t ref_count = 0;
  std::vector<int64_t> used;
};
// A call of the shared-product route of an FC layer over an array whose output matrices have not been written: the
// range sums and the centre columns are in place, the dense columns are what `outs` says and are written - for all
// sets of the call at once - when somebody first reads any of them (write_pending_columns).  The buffers the
// description points into are kept alive here.
struct DeltaCall {
  int64_t ref_count = 0;
  BufRef W, bias, base, S, cprod, lists, arena;
  const double* A = nullptr;
  const double* bias_ptr = nullptr;
  int64_t lda = 0, Mp = 0, ldo = 0, max_cols = 0;
  double bytes = 0.0;
  std::vector<DeltaOut> outs;  // rpart == null: the sums were delivered with the call
  std::vector<int32_t> group;
  bool written = false;
};

// Where an FC map gathered stored columns of a set from, and whether they are in memory yet.  Column
// from + t holds 0 + W(:, r) * scale[r] with r = idx[t] (scale == null: 1).  A later packing of kept rows
// reads the cache-resident weight matrix instead of the set's own matrix in HBM; and the FC map may leave
// the columns unwritten (`pending`) when it has left their range sums behind: nothing on the way to the
// next layers reads them then, and whoever does (a host read, a layer that needs the whole matrix) has
// them written first.  Writing them is idempotent, so every handle that shares the matrix keeps a copy
// of this description with its own flags.  W == null: no such knowledge.
struct ColSource {
  BufRef W_buf, idx_buf, scale_buf, Wt_buf;
  const double* Wt = nullptr;  // the same matrix row-major (row r at Wt + r * ldwt), or null
  int64_t ldwt = 0;
  const double* W = nullptr;  // the layer's weight matrix: `rows` rows (a multiple of 16), leading dimension ldw
  int64_t ldw = 0;
  int64_t rows = 0;
  const int32_t* idx = nullptr;
  const double* scale = nullptr;
  int64_t from = 0;
  int64_t cols = 0;
  bool pending = false;  // the columns [from, from + cols) are not in memory yet
  // Rows of the matrix have been reset (zeroed in memory) since the columns were gathered: the description then holds
  // for the rows on the handle's own kept-row list only, and does not pass on to a set that lists its rows anew
  // (a ReLU step on top may keep a row the earlier reset zeroed: one that crossed and now carries a unit vector).
  bool rows_reset = false;
  int64_t zero_to = 0;   // > 1: the columns [1, zero_to) are +0 and not in memory yet
  // Generator images of a convolution's output that are in memory inside their windows only (win_box[j], an
  // image of win_H x win_W positions per channel): columns [win_from, win_to); the rows outside the windows,
  // which are zero, have not been written.  The next convolution and the range scan read inside the windows
  // only; whoever reads whole columns has the zeros written first (write_pending_columns).
  BufRef win_box_buf;
  const ColBox* win_box = nullptr;
  int64_t win_from = 0, win_to = 0;
  int64_t win_rows = 0;  // rows of the image (H * W * channels)
  int32_t win_H = 0, win_W = 0;
  bool win_pending() const { return win_to > win_from; }
  // The leading (contracted) columns 1 .. of the matrix are the output of a shared-product call that has not written
  // them yet (column 0, the centre, is in memory).
  Ref<DeltaCall> delta;
  bool delta_pending() const { return delta && !delta->written; }
  bool any_pending() const { return pending || zero_to > 1 || win_pending() || delta_pending(); }
};

// One node per ReLU layer of the structured constraint store.  The dense NNV matrix
// [C0; C1; C2; C3] (nn/funcs/PosLin.m:711-735) is only materialised when the host reads it.
struct ConsNode {
  int64_t ref_count = 0;
  Ref<ConsNode> prev;  // null for the base node
  int64_t p_total = 0;             // constraint rows up to and including this node
  int64_t n_total = 0;             // predicate variables up to and including this node
  // base node: dense C0 (p_total x n_total, ld = ldc) and d0
  BufRef C0;
  int64_t ldc = 0;
  BufRef d0;
  // ReLU node: the C2/C3 rows are the crossing rows of the pre-ReLU [c V].  They are not copied:
  // the node keeps the input set's (immutable) generator buffer alive and gathers rows by index
  // when the dense matrix is materialised.
  int64_t m = 0;
  int64_t n_before = 0;
  BufRef src;                    // owner of the pre-ReLU generator matrix
  const double* src_V = nullptr; // its N x (n_before+1) matrix
  int64_t src_ld = 0;
  ColSource src_cs;              // columns of it that may not be in memory yet
  BufRef lbub;                   // lb[0..m), then ub[0..m) at offset ld_lbub; data starts at lbub_off
  int64_t lbub_off = 0;
  int64_t ld_lbub = 0;
  BufRef index;                  // crossing neuron indices in new-predicate order: int32[m] at index_off
  int64_t index_off = 0;
};
using ConsRef = Ref<ConsNode>;

// start of every entry point that touches device data: selects the context's device
int enter_ctx(nnvhip_ctx* ctx);

// Key of the per-context weight cache: a 128-bit hash of the layer's host arrays plus its geometry.  Layers are
// created from host arrays by value (FullyConnectedLayer(W, b), Star.affineMap(W, b) have no handle to pass
// around), so "the same layer again" can only be recognised by content.
struct WeightKey {
  uint64_t h0 = 0, h1 = 0;
  int64_t geo[12] = {};
  int kind = 0;  // 0 fc, 1 conv2d
  int salt = 0;  // > 0: another layer whose hash and geometry equal those of the entries with lower salts
  bool operator<(const WeightKey& o) const {
    if (kind != o.kind) return kind < o.kind;
    if (salt != o.salt) return salt < o.salt;
    if (h0 != o.h0) return h0 < o.h0;
    if (h1 != o.h1) return h1 < o.h1;
    for (int i = 0; i < 12; ++i)
      if (geo[i] != o.geo[i]) return geo[i] < o.geo[i];
    return false;
  }
};
struct WeightEntry {
  void* handle = nullptr;  // nnvhip_fc* / nnvhip_conv2d*; the cache owns one reference
  // The host arrays the layer was made from, by value.  A hit on the hash is only taken after they compare equal
  // to the caller's arrays: equal hashes prove nothing, and a wrong hit would run another network's weights.
  std::vector<double> host_w, host_b;
  int64_t bytes = 0;
  uint64_t last_use = 0;
};
// 128-bit content hash (multiply-fold streams that carry their previous state along) of a host array; only a
// filter in front of the byte-wise comparison
void hash_bytes(const void* data, size_t bytes, uint64_t* h0, uint64_t* h1);

}  // namespace nnvhip

struct nnvhip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  // size-class caching pool
  std::multimap<size_t, void*> free_blocks;
  int64_t bytes_in_use = 0;
  int64_t bytes_cached = 0;
  int64_t live_handles = 0;
  // Handles of large arrays that the caller has released but that have not been let go yet: destroying
  // thousands of handles costs hundreds of microseconds of host time, which is spent where the host waits
  // for the device anyway (the ReLU step's wait for its counts, a synchronisation) or when the pool runs
  // short of a block; pool_stats, trim and destroy let them go first.
  std::vector<nnvhip_star*> deferred;
  void drain_deferred(size_t at_most = ~size_t(0));
  // counters for diagnosing a slow step: hipMalloc calls of the pool, waits for the stream because the pinned
  // staging ring wrapped or grew, mailbox waits that went through the slow path
  int64_t n_device_mallocs = 0, n_staging_waits = 0;
  uint64_t visit_seq = 0;
  uint64_t next_layer_uid = 0;
  // nnvhip_hint_next_fc: the FC layer the caller will apply to the output of its next ReLU step (consumed by that step)
  const nnvhip_fc* next_fc = nullptr;
  // memory of released handles, reused by new_star (at most kMaxFreeStars of them are kept)
  static constexpr size_t kMaxFreeStars = 32768;
  std::vector<void*> free_stars;
  int64_t device_bytes = 0;  // memory of the device (the pool grows past a released array only below a share of it)
  // pinned staging ring for descriptor tables and small read-backs
  char* pinned = nullptr;
  std::vector<char*> retired_rings;
  size_t pinned_bytes = 0;
  size_t pinned_off = 0;
  // mailbox in pinned host memory: a kernel posts {m, inactive, call number} there and the host spins
  // on it (after having stored kMailboxEmpty there), which is quicker than a device-to-host copy plus
  // stream synchronisation
  volatile int32_t* mailbox = nullptr;  // kMailboxSets words of 64 bits, one per set of an array
  static constexpr int64_t kMailboxSets = 8192;
  // fixed workspace in device memory of the entry point that must not allocate (ranges.hip): this
  // device's address of the array and its length
  double* static_scratch = nullptr;
  int64_t static_scratch_doubles = 0;
  // Layer weights by content: creating a layer whose arrays are already on the device returns the resident
  // handle (one more reference) instead of uploading them again.  Entries nobody else holds are dropped,
  // least recently used first, once the cache passes its budget (environment NNVHIP_WEIGHT_CACHE_MB, default 8192).
  std::map<nnvhip::WeightKey, nnvhip::WeightEntry> weight_cache;
  int64_t weight_cache_bytes = 0;
  int64_t weight_cache_budget = int64_t(8192) << 20;
  uint64_t weight_clock = 0;
  // uploads since the context was created: layers whose weights went to the device, their bytes, and all
  // bytes the library copied from host to device (sets, bounds, descriptor tables, weights)
  int64_t weight_uploads = 0, weight_upload_bytes = 0, h2d_bytes = 0;
  void drop_weight_cache(bool all);
  // frees the device memory of every cached layer that nobody but the cache holds; returns how many went
  int64_t drop_unreferenced_weights();
  uint32_t mailbox_seq = 0;  // number of the ReLU call (wraps; only its low 16 bits travel, as a cross-check)
  // FC layers as the full dense contraction (no skipping of structural zeros); default from the
  // environment variable NNVHIP_DENSE_AFFINE
  bool dense_affine = false;
  // ReLU outputs always store their appended unit-vector columns (environment NNVHIP_EAGER_TAIL)
  bool eager_tail = false;
  // ReLU outputs reset their rows at once instead of leaving that to the first reader that needs the
  // whole matrix (environment NNVHIP_EAGER_ROWS; implied by the two switches above)
  bool eager_rows = false;
  // FC maps always write the columns they gather (environment NNVHIP_EAGER_COLS)
  bool eager_cols = false;
  // small fully connected networks are reached in one launch (chain.hip); environment NNVHIP_NO_SMALL_CHAIN
  // or nnvhip_set_small_chain(ctx, 0) keeps them on the layer-by-layer path
  bool small_chain = true;
  // a convolution whose input has a pending row reset runs that reset first instead of masking the rows as
  // it loads them (environment NNVHIP_NO_CONV_MASK)
  bool no_conv_mask = false;
  // convolutions compute every generator image in full instead of inside its window (nnvhip_star::box;
  // environment NNVHIP_NO_CONV_BOXES)
  bool no_conv_boxes = false;
  // arrays of sets of one shape always contract over their whole kept-row lists instead of starting from their
  // group's shared product and contracting over the rows in which they differ (environment NNVHIP_NO_ROW_DELTAS)
  bool no_row_deltas = false;
  int64_t n_bounds_in_place = 0, n_bounds_copied = 0;  // sets through ReLU steps, by where their predicate bounds went
  bool no_sum_shortcuts = false;  // the pass that sums unwritten pieces: every set in full, with both bounds of every predicate
  // debugging aid (environment NNVHIP_POISON_PENDING): columns left unwritten are filled with NaNs
  bool poison_pending = false;
  // per-layer timing
  bool timing = false;         // per-layer events (nnvhip_last_op_time_ms)
  bool kernel_timing = false;  // additionally one event pair per launch of the timed kernel groups
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  double last_ms = 0.0;
  // timing of the dominant kernel alone (events directly around its launch), per instantiation group
  hipEvent_t kev0 = nullptr, kev1 = nullptr;
  hipEvent_t read_ev = nullptr;  // marks a read-back in the stream whose arrival the host waits for while later work runs
  // [0] dense MFMA GEMM (tiles of at least 64 rows), [1] implicit-GEMM convolution (work = flop),
  // [2] estimateRanges column pass, [3] ReLU apply pass, [4] row-wise affine layers (batch
  // normalisation, input normalisation, average pooling, flatten), [5] gather of W's columns for the
  // one-hot generator columns of an FC layer (work = algorithmic bytes)
  // [6] ReLU classification, [7] range reduction, [8] whole-reach kernel of small networks (chain.hip)
  // [9] tile kernel of gemm_seg.hip (work = flop), [10] outputs that start from a product shared by many sets and
  // add only the rows in which a set differs from it (delta_tiles_kernel; work = bytes written)
  static constexpr int kKernelGroups = 11;
  double kern_ms[kKernelGroups] = {};
  int64_t kern_launches[kKernelGroups] = {};
  double kern_flop[kKernelGroups] = {};
  int kernel_timer_begin(bool on);
  int kernel_timer_end(bool on, int which, double flop);

  int alloc(size_t bytes, nnvhip::BufRef* out);
  void release_block(void* p, size_t bytes);
  int trim();
  // Returns host-pinned scratch of `bytes`; waits for the stream when the ring wraps.
  int stage(size_t bytes, void** host);
  // Copies a host table to a fresh device buffer through the pinned ring (async on the stream).
  int upload(const void* host, size_t bytes, nnvhip::BufRef* out);
  // A descriptor table that only the launches of the current call read.  Small ones stay in the pinned
  // staging ring and the kernels read them from there (no copy on the stream); the slot is not reused
  // before the stream has been synchronised.
  int upload_table(const void* host, size_t bytes, nnvhip::BufRef* out);
  int begin_op();
  int end_op();
};

// Launch on the context's stream.  With `on` the start and stop events ride on the kernel's own
// dispatch, so kernel_timer_end() reads the duration of the kernel alone (what a profiler reports),
// not that of an event-launch-event sequence.
#define NNV_LAUNCH(ctx, on, kernel, grid, block, shmem, ...)                                                       \
  do {                                                                                                              \
    if (on)                                                                                                         \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, (ctx)->stream, (ctx)->kev0, (ctx)->kev1, 0, __VA_ARGS__); \
    else                                                                                                            \
      hipLaunchKernelGGL(kernel, grid, block, shmem, (ctx)->stream, __VA_ARGS__);                                  \
  } while (0)

struct nnvhip_star {
  std::atomic<int> refs{1};
  nnvhip_ctx* ctx = nullptr;
  int64_t N = 0;   // dim
  int64_t n = 0;   // nVar
  int64_t ld = 0;  // leading dimension of V (multiple of 16, >= N)
  nnvhip::BufRef Vbuf;
  double* V = nullptr;  // N x (n+1), may point inside a shared arena
  // Number of columns of V that exist in memory.  A ReLU output keeps its appended unit-vector columns
  // [oh_from, n] implicit (vcols = oh_from): the FC and conv maps never read them, and whoever needs the
  // full matrix calls ensure_dense() first.  -1 = all n+1 columns.
  int64_t vcols = -1;
  int64_t stored_cols() const { return vcols >= 0 ? vcols : n + 1; }
  // A ReLU output may also leave the reset of its rows pending: V then still points at the input set's
  // matrix (shared, never written) and every row that kept_idx does not list counts as zero.  The FC map
  // contracts over the listed rows only and never notices; everybody else calls ensure_dense(), which
  // runs the pending pass (it needs the per-row classification cls) into a buffer of the set's own.
  bool rows_pending = false;
  nnvhip::BufRef cls_buf;
  const uint32_t* keep_bits = nullptr;  // with cls (in cls_buf): bit r & 31 of word r >> 5 is set where row r is kept
  const int32_t* cls = nullptr;
  nnvhip::BufRef pbuf;
  double* plb = nullptr;
  double* pub = nullptr;
  nnvhip::Ref<nnvhip::PredTails> ptails;  // not null: plb / pub have room for pcap entries each (see PredTails)
  int64_t pslot = 0, pcap = 0;
  nnvhip::ConsRef cons;
  // cached estimateRanges result
  nnvhip::BufRef rbuf;
  double* lb = nullptr;
  double* ub = nullptr;
  // set by the ReLU step: the estimated upper bounds of its input, by neuron (the range buffer is kept alive)
  nnvhip::BufRef pre_ub_buf;
  const double* pre_ub = nullptr;
  // filled for sets produced by the ReLU step
  int64_t n_inactive = -1;
  int64_t n_crossing = -1;
  // Structure hint for the FC affine map: columns [oh_from, n] of V are scaled unit vectors,
  // column j = oh_scale[r] * e_r with r = oh_idx[j - oh_from] (oh_scale == null: scale 1).  Box stars
  // (all generators) and ReLU outputs (the appended columns) carry it; 0 = no such block.  V itself is
  // always fully materialised, the hint only lets W*V skip products with structural zeros.
  int64_t oh_from = 0;
  const int32_t* oh_idx = nullptr;
  const double* oh_scale = nullptr;
  nnvhip::BufRef oh_idx_buf, oh_scale_buf;
  // The inverse of oh_idx where somebody has made it: oh_inv[r] = t with oh_idx[t] = r, -1 for rows no column names
  // (N entries).  The ReLU step leaves it for image sets; the convolution's stamp pass makes it otherwise and keeps it.
  nnvhip::BufRef oh_inv_buf;
  const int32_t* oh_inv = nullptr;
  // Second hint, set by the ReLU step: only the rows kept_idx[0..n_kept) (ascending; the list is padded
  // with -1 up to a multiple of 16 and at least 16 entries) of the columns before the one-hot block can
  // be non-zero -- every other row was reset.  n_kept < 0 = no such knowledge.
  int64_t n_kept = -1;
  const int32_t* kept_idx = nullptr;
  nnvhip::BufRef kept_buf;
  // Range sums left behind by the kernel that produced the trailing columns (filter stamps, gathered
  // columns): rng_chunks chunks of [4][ld] partial sums at rng_part that cover the generator columns
  // [rng_first_col, n].  estimateRanges then scans only the columns before rng_first_col.
  nnvhip::BufRef rng_buf;
  const double* rng_part = nullptr;
  int64_t rng_chunks = 0;
  int64_t rng_first_col = 0;
  // The first rng_chunks_at of those chunks were not written here: they equal another set's, whose address the
  // device holds at *rng_part_at (the producer found that out on the device; it may be this set's own).
  nnvhip::BufRef rng_at_buf;
  const double* const* rng_part_at = nullptr;
  int64_t rng_chunks_at = 0;
  // The same four sums for the gathered columns of a set in an array, as one matrix product left them
  // (launch_range_sums_mm): two vectors of 2 * ld entries, [xmin1; xmax2] and then [xmax1; xmin2].  They
  // cover columns from rng_first_col on, like the chunks above, and are added after them.
  nnvhip::BufRef rng_mm_buf;
  const double* rng_mm = nullptr;
  // A ReLU output of an array whose caller had said which FC layer comes next (nnvhip_hint_next_fc): the range sums
  // of the columns that layer will gather for the columns this step appended, as launch_range_sums_mm leaves them
  // (slot ahead_mm_slot of the product), queued behind the classification so that the device forms them while the
  // host reads the counts and sets the layer call up.  For the layer with uid ahead_mm_uid only.
  nnvhip::BufRef ahead_mm_buf;
  uint64_t ahead_mm_uid = 0;
  int64_t ahead_mm_slot = 0;
  bool has_producer_sums() const { return (rng_part != nullptr && rng_chunks > 0) || rng_mm != nullptr; }
  // some scale of the unit-vector block is negative (a box with ub < lb): sign-split products do not apply
  bool oh_scale_neg = false;
  // the predicates of the unit-vector block all have lower bound 0 (the block was appended by a ReLU step:
  // new_pred_lb = [plb; zeros(m,1)], nn/funcs/PosLin.m:737): products with those bounds are zero
  bool oh_plb_zero = false;
  uint64_t visit = 0;  // nnvhip_ctx::visit_seq of the last pass that listed this handle (passes over an array skip repeats)
  // The reference's Star carries an outer zonotope Z from Star(lb, ub) on (set/Star.m:220-237) and maps it along in
  // affineMap (:332-340, set/Zono.m:47-74) until the ReLU step returns a Star without one (nn/funcs/PosLin.m:740).
  // Z = Zono(V(:,1), V(:,2:end)) of the same set all the way -- Star(lb, ub) builds both from the same centre and
  // generators, and both are mapped by the same W, b -- so it is not stored: the handle only remembers whether
  // the reference's set would have one.
  bool has_zono = false;
  // where gathered columns came from, and whether they (and leading zero columns) are in memory yet
  nnvhip::ColSource cs;
  // Spatial support of the generator images of an ImageStar that a convolution produced: stored column j
  // (j < box_cols) is zero in every row (h, w, channel) of the box_H x box_W x C image outside the window
  // box[j] (h0..h1, w0..w1, inclusive; h0 > h1: the whole column is zero).  Generators of a box ImageStar
  // start as single pixels and grow by a filter's reach per convolution; a ReLU step only resets rows, so
  // its output keeps the windows.  box_eh x box_ew bounds the window of every column but the centre's.  The
  // next convolution computes a generator's image inside its (grown) window only.  null: no such knowledge.
  nnvhip::BufRef box_buf;
  const nnvhip::ColBox* box = nullptr;
  int64_t box_cols = 0;
  int32_t box_H = 0, box_W = 0, box_eh = 0, box_ew = 0;
};

struct nnvhip_fc {
  std::atomic<int> refs{1};
  nnvhip_ctx* ctx = nullptr;
  int64_t M = 0, K = 0, Mp = 0, Kp = 0;
  uint64_t uid = 0;     // of this context's layers, never reused (a set remembers which layer a product made ahead is for)
  nnvhip::BufRef W;     // Mp x Kp, zero padded, ld = Mp
  nnvhip::BufRef bias;  // Mp entries (zero padded) or null
  // [max(W, 0); min(W, 0)], 2*Mp x Kp with ld = 2*Mp: made on first use by launch_range_sums_mm
  mutable nnvhip::BufRef Wpn;
  // the weights row-major (Mp rows of Kp entries), made on first use for arrays of sets: the next layer packs
  // kept rows of columns that are scaled weight columns, i.e. reads rows of W
  mutable nnvhip::BufRef Wt;
};

struct nnvhip_conv2d {
  std::atomic<int> refs{1};
  nnvhip_ctx* ctx = nullptr;
  int64_t FH = 0, FW = 0, Cin = 0, Cout = 0;
  int64_t pad[4] = {0, 0, 0, 0}, stride[2] = {1, 1}, dil[2] = {1, 1};
  int64_t K = 0, Kp = 0;  // K = FH*FW*Cin taps, Kp = padded
  nnvhip::BufRef W;       // Kp x Cout, zero padded rows, ld = Kp (MATLAB layout is already K x Cout)
  nnvhip::BufRef bias;    // Cout entries or null
  // the same weights k-major for the kernel that brings its weight tiles straight into LDS: Kp rows of
  // coutp channels (Cout padded with zeros to a multiple of 64); null if the layer is too large for it
  nnvhip::BufRef Wk;
  int64_t coutp = 0;
  // tap tables of that kernel, one per input size the layer has seen (they depend on H and W)
  struct TapTable {
    int64_t H = 0, W = 0;
    nnvhip::BufRef tab;
  };
  mutable std::vector<TapTable> tap_tables;
};

namespace nnvhip {

nnvhip_star* new_star(nnvhip_ctx* ctx);
void delete_star(nnvhip_star* s);  // the last reference is gone

// Shared set-up of the affine layers (ctx.hip): validates the handle array; allocates one output arena
// with the sets back to back and creates output handles that share constraints and predicate bounds
// with their inputs; releases a vector of handles after a failure.
int check_set_array(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, nnvhip_star** out);
int make_affine_outputs(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, int64_t Nout,
                        std::vector<nnvhip_star*>* outs, bool* contiguous, int64_t* total_cols);
void release_all(std::vector<nnvhip_star*>& v);

// Optional fusion of Star.estimateRanges into the GEMM epilogue (one set per launch): every column
// tile leaves the four partial range sums of its rows in `part` ([chunks][4][ldc]); the caller then
// runs the range reduction over the chunks instead of a separate pass over the output.
struct RangeFuse {
  const double* plb = nullptr;  // predicate bounds of the set's n = ncols - 1 generator columns
  const double* pub = nullptr;
  int64_t extra_chunks = 0;     // in: room to leave behind the GEMM's chunks (for launch_gather_columns)
  BufRef part;                  // out: partial sums (allocated by the launcher)
  int64_t chunks = 0;           // out: number of column tiles; 0 = not fused (split-K was used)
};

// gemm.hip: C(Mp x ncols, ldc) = A(Mp x Kp, lda) * B(Kp x ncols, ldb); bias (Mp) is added to
// column 0 when non-null.  Mp, Kp multiples of 16; padding rows of A and B are zero.
// rows (optional): contraction over a subset of the K rows.  kmap lists the rows of B (= columns of A)
// that can be non-zero, padded with -1 to a multiple of 16; Kp passed to launch_gemm is then the padded
// length of that list.  With segs (arrays of sets), column tile t of seg_cols columns has its own
// description: its row list (null = all rows), the arena column of its first column and how many of
// its columns exist; ncols is then seg_cols * (number of tiles), seg_cols = gemm_seg_cols(...) (64 for
// small arrays and skinny outputs).
struct GemmSeg {
  const int32_t* kmap;
  const double* Bk;    // the set's packed rows (see GemmRows::Bk), or null
  int64_t ldbk;
  int64_t col_local0;  // column of Bk behind the tile's first column
  int64_t b_col_base;  // column of B behind the tile's first column (input arena)
  int64_t col_base;    // column of C behind the tile's first column (output arena)
  int32_t kp;
  int32_t valid;
  // fused range sums of this tile's columns (null: none): the set's predicate bounds (indexed by the
  // set's own generator column) and the [4][ldc] chunk the tile fills
  const double* plb;
  const double* pub;
  double* rpart;
};
struct GemmRows {
  const int32_t* kmap = nullptr;
  // the listed rows of B packed into their own matrix (row t = row kmap[t] of B, zero where kmap[t] < 0,
  // leading dimension ldbk): B is then read from here and only A is gathered
  const double* Bk = nullptr;
  int64_t ldbk = 0;
  const GemmSeg* segs = nullptr;
  // without segs: product column t reads column colmap[t] of B and writes column colmap[t] of C
  // (columns picked from an arena of sets that share the row list)
  const int32_t* colmap = nullptr;
  int32_t seg_cols = 128;
  double flop = 0.0;  // flop actually executed (for the kernel timers)
  // 64: take the 64 x 64 tile whatever the shape model says (short products of a few hundred tiles, whose blocks
  // then sit two or more to a CU and cover each other's start and end: 2048 x 1024 x 1024 runs in 105 us on it,
  // 141 us on the 128 x 64 tile the model picks)
  int32_t tile_hint = 0;
};
int gemm_seg_cols(int64_t Mp, int64_t count, const int64_t* cols);
// Vk(t, j) = V(kept[t], j) for t < kp (a multiple of 16; zero where kept[t] < 0), j < ncols; Vk has
// leading dimension kp.
struct PackSet {
  const double* V;
  const int32_t* kept;
  double* Vk;
  int64_t ld;
  int32_t kp;
  int32_t ncols;
  // columns [wfrom, wend) are read as 0 + W(:, widx[j - wfrom]) * wscale[...] instead (W == null: none)
  const double* W = nullptr;
  int64_t ldw = 0;
  const double* Wt = nullptr;  // W row-major (row r at Wt + r * ldwt), or null
  int64_t ldwt = 0;
  int64_t wrows = 0;           // rows of W
  const int32_t* widx = nullptr;
  const double* wscale = nullptr;
  int32_t wfrom = 0;
  int32_t wend = 0;
  int32_t zero_to = 0;  // > 1: columns [1, zero_to) are +0 whatever the memory holds
  int64_t ldt = 0;      // launch_pack_rows_t: Vk is kp x ldt, row-major (columns [ncols, ldt) are written as zeros)
  int32_t col0 = 0;     // launch_pack_rows_t, rows of the weights only: packed column j is the set's column col0 + j
                        // (ncols counts from there)
  // columns [box_from, box_to) are +0 outside their windows box[j] (images of bH x bW positions per channel),
  // whatever the memory holds there (box == null: none)
  const ColBox* box = nullptr;
  int32_t box_from = 0, box_to = 0;
  int32_t bH = 0, bW = 0;
};
// the packing of the first `ncols` columns of a set, with what is known about where they came from
PackSet pack_of(const nnvhip_star* s, const int32_t* kept, double* dst, int64_t kp, int64_t ncols);
int launch_pack_rows(nnvhip_ctx* ctx, int64_t count, const PackSet* sets);

// gemm_seg.hip: tiles of 128 rows x tn columns (tn = 128, 64 or 32), each belonging to one set:
// C(:, col_base + [0, valid)) = A(:, kmap) * Bt(:, col_local0 + [0, valid)), with the bias on the column whose
// number in the set (col_local0 + offset) is 0 and, with rpart, the tile's four range sums ([4][ldc]).
struct SegTile {
  const int32_t* kmap;  // kp entries (a multiple of 16), -1 where the list is padded
  const double* Bt;     // the set's packed rows, transposed: kp x ldbt, row-major (launch_pack_rows_t); or, with
                        // gather_b, a matrix shared by all sets whose row kmap[t] is the set's packed row t
  int64_t ldbt;
  int64_t b_col0;       // the tile's first column in Bt
  int64_t col_local0;   // the tile's first column in the set's own numbering
  int64_t col_base;     // ... and in C
  // gather_b (128-column tiles only): Bt holds one row per input row plus a row of zeros at index zero_row (for
  // the padded entries of kmap); a tile with col_local0 == 0 takes its column 0 from centre[kmap[t]] instead
  const double* centre;
  int32_t gather_b;
  int32_t zero_row;
  int32_t kp;
  int32_t valid;        // columns of the tile that exist
  const double* plb;    // the set's predicate bounds (indexed by generator column), for the range sums
  const double* pub;
  double* rpart;        // or null
};
// flag of an entry of a row-difference list (launch_delta_lists): the row is taken away, not added
constexpr int32_t kSegSubtract = 1 << 30;
int launch_pack_rows_t(nnvhip_ctx* ctx, int64_t count, const PackSet* sets);
int launch_gemm_seg(nnvhip_ctx* ctx, const double* A, int64_t lda, double* C, int64_t ldc, int64_t Mp, const double* bias,
                    int tn, const SegTile* segs, int64_t ntiles, double flop, bool gather_b = false);
// Row lists of the sets of an array, by group (sets whose packed rows agree wherever they keep the same row): the
// rows a majority of a group keeps (`common`, ascending, padded with -1 to a multiple of 16; its padded length in
// ncommon[group]) and, per set, the rows in which it differs from its group's list (`delta`: at most cap entries
// per set, ascending, r or r | kSegSubtract, padded with -1 to a multiple of 8; dlen[set] = their number, or -1
// if the set differs in more than cap rows).
struct DeltaSet {
  const int32_t* kept;  // ascending, kp entries, -1 padded
  int32_t kp;
  int32_t group;
};
int launch_delta_lists(nnvhip_ctx* ctx, int64_t count, const DeltaSet* sets_dev, int groups, const int32_t* group_size_dev,
                       int64_t rows, int64_t rows_pad, int cap, int32_t* votes /* groups x rows, scratch */, int32_t* common /* groups x rows_pad */,
                       int32_t* ncommon, int32_t* delta /* count x cap */, int32_t* dlen,
                       int32_t* head /* count x 4: the first entries of every list, -1 where there is none */);
// The output of one set that starts from its group's shared product: out(:, j) = base(:, j) + sum over the set's
// row differences of (+/-) A(:, r) * S(r, j) for j < ncols, the centre column (j = 0) replaced by cprod (+ bias), and
// the four Star.estimateRanges partial sums of every piece of delta_tile_chunks' columns in rpart ([piece][4][ldo]).  A streaming
// pass (gemm_seg.hip, delta_tiles_kernel): bound by the bytes it writes.
// (sets: host table, neighbours of one group next to one another; group_of[i]: group of set i of the table; the
// pass leaves delta_tile_chunks(ncols) chunks of range sums per set)
// store == false: only the centre columns and the range sums are written (the matrices are left to a later call with
// store == true and no rpart), and not for every set: sums_at receives a device array with, per set of the table,
// the address of the chunks that hold its sums - its own rpart, or that of an earlier set with the same sums.
int launch_delta_tiles(nnvhip_ctx* ctx, const double* A, int64_t lda, int64_t Mp, const double* bias, int64_t ldo, int64_t count,
                       const DeltaOut* sets, const int32_t* group_of, int64_t max_cols, double bytes, bool store = true,
                       BufRef* sums_at = nullptr);
int delta_tile_chunks(int64_t ncols);
// Cm(r, s) = centre of set s at row r if the set keeps row r, else +0: Cm is Kp x count (ld = Kp), zeroed here.
struct CentreSet {
  const int32_t* kept;
  const double* centre;
  int32_t kp;
};
int launch_masked_centres(nnvhip_ctx* ctx, int64_t count, const CentreSet* sets_dev, double* Cm, int64_t Kp);
// The matrices the gathering tiles read, up to 16 per launch: row r < rows of one is [0, Wt(r, idx[j - 1]) *
// scale[idx[j - 1]] for 1 <= j < ncols, zeros up to ld], row `rows` is all zeros.  out: (rows + 1) x ld, row-major.
struct ScaledRows {
  struct One {
    const double* Wt;
    int64_t ldwt;
    const int32_t* idx;
    const double* scale;
    double* out;
    int64_t ld;
    int32_t rows, ncols;
  } s[16];
  int32_t count;
};
int launch_scaled_rows(nnvhip_ctx* ctx, const ScaledRows& a);
// A split-K product leaves `ksplit` partial matrices (Mp x ncols each, ld = Mp) in a workspace; a caller
// that has a pass over the output coming anyway can take the workspace instead of having the reduction
// kernel launched (sum in split order, then the bias on column 0).  ksplit = 1: C is final.
struct SplitKDefer {
  BufRef ws;
  int64_t ksplit = 1;
};
int launch_gemm(nnvhip_ctx* ctx, const double* A, int64_t lda, const double* B, int64_t ldb, double* C,
                int64_t ldc, int64_t Mp, int64_t ncols, int64_t Kp, const double* bias, RangeFuse* fuse = nullptr,
                const GemmRows* rows = nullptr, SplitKDefer* defer = nullptr);
// Adds bias to the centre columns of sets 1..count-1 of an arena (set 0 is fused in the GEMM).
int launch_bias_columns(nnvhip_ctx* ctx, double* const* centre_cols_dev, int64_t count, const double* bias,
                        int64_t Mp);

// conv.hip
// Convolution of the one-hot generator columns of every set ("stamps" of the filter), conv.hip.
struct ConvStampSet {
  const int32_t* idx;   // input row of every one-hot column
  const double* scale;  // by input row, or null
  double* out;          // first of these columns in the output set
  const double* plb;    // predicate bounds of these columns
  const double* pub;
  double* part;         // this set's [chunks][4][ldout] range sums
  int32_t m;
  int32_t win_only;     // 1: write the rows inside each column's window only
  const int32_t* pixel_col;  // input row -> its one-hot column (index into idx), -1: none; or null (made by the launch)
};
int launch_conv2d(nnvhip_ctx* ctx, const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                  const double* in, int64_t ldin, double* out, int64_t ldout, int64_t ncols,
                  const int32_t* pending_cls /* per input row, or null: rows whose class is not kKeep read as zero */,
                  const ColBox* out_box = nullptr /* per output column, or null: with it (and conv2d_in_windows), columns
                                                    1.. are computed inside their windows only, at most eh x ew positions */,
                  int eh = 0, int ew = 0,
                  const ColBox* in_box = nullptr /* windows of the input columns: taps outside them are not read (the input
                                                    may be in memory inside its windows only); needs conv2d_in_windows */,
                  bool leave_outside = false /* do not write the zeros outside the output windows */,
                  const uint32_t* pending_bits = nullptr /* with pending_cls: the same as one bit per row (1 = kept), where
                                                            the step that classified the rows left them */,
                  const ConvStampSet* stamp = nullptr /* the set's unit-vector columns: their stamps go into the same
                                                                 launch where that is possible ... */,
                  bool* stamped = nullptr /* ... which this reports (launch_conv_stamps is then not needed for the set) */);
int launch_zero_pad_rows(nnvhip_ctx* ctx, double* V, int64_t ld, int64_t N, int64_t ncols);  // rows [N, ld) of ncols columns := 0
// whether launch_conv2d computes the generator images of such a call inside their windows only
bool conv2d_in_windows(const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int64_t ldin, int64_t ncols,
                       const ColBox* out_box, int eh, int ew);
// Windows of a convolution's output columns: column 0 the whole image; columns below `dense` from the input's
// windows (in_box null: whole image); the `m` columns from `dense` on from the pixels onehot_idx names.
int launch_conv_boxes(nnvhip_ctx* ctx, const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                      const ColBox* in_box, int64_t dense, const int32_t* onehot_idx, int64_t m, ColBox* out_box);
// Bound on the extent of an output window whose input window spans at most `e` rows (dim 0) or columns (dim 1).
int64_t conv_box_extent(const nnvhip_conv2d* conv, int dim, int64_t e, int64_t out_size);
// whether launch_conv2d takes pending_cls for such an input (H x W x Cin images, leading dimension ldin)
bool conv2d_can_mask(const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int64_t ldin);
int conv2d_prepare_weights(nnvhip_ctx* ctx, nnvhip_conv2d* conv);  // builds conv->Wk from conv->W (at creation)

// Whether the stamp launch of this layer looks columns up by pixel (ConvStampSet::pixel_col), and that table for one
// set: inv[idx[t]] = t, -1 elsewhere (n_in entries, allocated here).
bool conv_stamps_by_pixel(const nnvhip_conv2d* conv);
int launch_pixel_columns(nnvhip_ctx* ctx, const int32_t* idx, int64_t m, int64_t n_in, BufRef* inv);
// Number of column chunks (= range-sum chunks per set) the stamp launch will use.
int64_t conv_stamp_chunks(const nnvhip_conv2d* conv, int64_t ldout, int64_t count, int64_t max_m);
int launch_conv_stamps(nnvhip_ctx* ctx, const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                       int64_t ldout, int64_t count, const ConvStampSet* sets, int64_t chunks);

// ranges.hip
// counts != null: where the estimate of every set of the call ends in the kernel that combines partial sums, that
// kernel also counts the crossing / inactive / kept neurons (among the first nrows rows) of every `gran` rows of a
// set: three numbers per block at base + stride * (set's place in the call); gran == 0 afterwards: it did not.
struct RangeCounts {
  int32_t* base = nullptr;
  int64_t stride = 0;  // at least 3 * ceil(ld / 64)
  int32_t nrows = 0;
  int32_t gran = 0;    // out: rows per triple (64 or 128), 0: nothing was counted
};
int compute_ranges(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* s, RangeCounts* counts = nullptr);
// the fixed device workspace: address look-up (once per context) and Star.estimateRanges into it
int init_static_scratch(nnvhip_ctx* ctx);
int ranges_into_static(nnvhip_ctx* ctx, const nnvhip_star* s, double* lb_dev, double* ub_dev);
// W * (scaled unit vectors): out(:, j) = W(:, idx[j]) * scale[idx[j]] for the one-hot column block of
// every set (ranges.hip).  With part != null (one set) the four range sums of these columns are left
// as `chunks` further chunks at part + part_chunk0, in the layout finalize_fused_ranges reads.
struct GatherSet {
  const int32_t* idx;
  const double* scale;  // by row index, or null
  double* out;          // first one-hot column of the output set
  const double* plb;    // predicate bounds of these columns (range sums only)
  const double* pub;
  double* part;         // where this set's [chunks][4][ldout] range sums go, or null
  int32_t m;
  int32_t nfill;        // leading output columns that are known to be bias (column 0) and zeros: written here too
  double* fill;         // column 0 of the output set (nfill > 0)
  const double* bias;   // or null
  const double* red;    // split-K partials of the centre column (red_k vectors of Mp entries) to be summed into
  int32_t red_k;        // `centre`, plus the bias; null / 0 = the centre is final
  int32_t lazy;         // 1: only the range sums (and column 0 of the fill) are produced, the columns stay unwritten
  double* centre;
  // The gathered columns are all the columns of W (a box star without degenerate dimensions): the pass
  // also forms the centre's product W * cin, as one partial vector per chunk (cpart[chunk][ldout]) that
  // the range reduction sums in chunk order.  cin == null: not asked for.
  const double* cin;    // the input's centre, indexed by row
  double* cpart;
};
// Writes the columns of the sets that are described but not in memory yet (see ColSource).
int write_pending_columns(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* sets);
int write_pending_columns(nnvhip_ctx* ctx, double* V, int64_t ld, ColSource* cs);
int64_t gather_chunks(int64_t Mp, int64_t m);
int64_t gather_chunks_batch(int64_t ldout, int64_t count, int64_t max_m);
// chunks > 0: every set's `part` receives that many chunks (sets with part == null none); chunks = 0:
// no range sums, the launcher picks the chunking.
int launch_gather_columns(nnvhip_ctx* ctx, const double* W, int64_t ldw, int64_t Mp, int64_t ldout, int64_t count,
                          const GatherSet* sets, int64_t chunks);
// Range sums of the gathered columns of every set of an array as one matrix product.  For a column
// sc * e_r with sc >= 0 the product column is W(:, r) * sc, so
//   sum_j max(v_ij, 0) * pl_j = sum_r max(W_ir, 0) * (sc_r * pl_r)   (and likewise for min and for pu):
// with a = scatter(sc * plb), b = scatter(sc * pub) per set, [max(W,0); min(W,0)] * [a b] holds
// [xmin1; xmax2] and [xmax1; xmin2].  One fp64 MFMA product over all sets instead of a pass over the
// cache-resident weights per set.  out: 2*Mp x 2*count, ld = 2*Mp, columns 2i and 2i+1 belong to set i.
// The same product (every column's lower predicate bound zero, no scales) for the columns a ReLU step is about to
// append, from the step's per-row classes and the input's upper bounds instead of the lists the host does not have
// yet: x_s(r) = ub_s(r) where neuron r crosses (cls_s(r) >= 0), 0 elsewhere.  Set i's sums are slot i of *out.
struct AheadSet {
  const int32_t* cls;
  const double* ub;
};
int launch_range_sums_mm_ahead(nnvhip_ctx* ctx, const nnvhip_fc* fc, int64_t count, const AheadSet* sets, int64_t N, BufRef* out);
int launch_range_sums_mm(nnvhip_ctx* ctx, const nnvhip_fc* fc, int64_t count, const GatherSet* sets, BufRef* out,
                         std::vector<int64_t>* slot,  // slot[i]: which pair of columns of `out` holds set i's sums
                         bool plb_zero = false);      // every lower bound involved is 0: the first column of every pair is
                                                      // zero and only the second is multiplied out
// lb / ub (and, by centre_mode, the centre column) of a fully connected layer's output for one set whose
// gathered columns need no pass of their own, finished in one kernel (ranges.hip).
int launch_fc_rowsum(nnvhip_ctx* ctx, const nnvhip_fc* fc, nnvhip_star* out, int mode, const double* scale, const int32_t* cls,
                     const double* pre_ub, int centre_mode, const double* cin, const double* part, int64_t chunks);
// Turns the per-column-tile partial sums a fused GEMM left behind into the set's cached lb/ub.
// cpart / cchunks / cbias: the centre column of s is still to be formed as the sum of cchunks partial
// vectors (ld entries each) plus the bias (or null); the kernel writes it into column 0 of s first.
int finalize_fused_ranges(nnvhip_ctx* ctx, nnvhip_star* s, const BufRef& part, int64_t chunks,
                          const double* cpart = nullptr, int64_t cchunks = 0, const double* cbias = nullptr);

// relu.hip
// Makes V a plain stored matrix: writes columns that are still pending (need_cols; always when one of
// the other two steps reads them), runs a pending row reset and, with need_tail, writes the implicit
// unit-vector columns, into a fresh buffer.  The batch form keeps the sets of an array back to back.
int ensure_dense(nnvhip_ctx* ctx, nnvhip_star* s, bool need_tail = true);
int ensure_dense_batch(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* sets, bool need_tail = true,
                       bool need_cols = true);
// order: NNVHIP_ORDER_* (classification from the sets' estimated ranges), or kOrderGiven with one
// ReluGiven per set: per-row bounds to classify by (ub <= 0: reset, lb < 0 < ub: crossing, else left
// alone) and per-row keys whose descending order is the order of the new predicates.
constexpr int kOrderGiven = 3;
struct ReluGiven {
  const double* lb;
  const double* ub;
  const double* key;
};
int relu_relax(nnvhip_ctx* ctx, int order, int64_t count, nnvhip_star* const* in, nnvhip_star** out,
               const ReluGiven* given = nullptr);
int materialize_constraints(const nnvhip_star* s, double* C_host, double* d_host);

// chain.hip: the layer loop of a small FC / ReLU network as one launch (one block per set).  *taken = false:
// not applicable (nothing was done; the caller runs the layer loop).  out: n_layers x count handles.
int reach_small_chain(nnvhip_ctx* c, int64_t n_layers, const int32_t* kind, const void* const* layer, int order, int64_t count,
                      nnvhip_star* const* in, nnvhip_star** out, bool* taken);

}  // namespace nnvhip
