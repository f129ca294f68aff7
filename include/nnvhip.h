/*
 * nnvhip.h - C ABI of libnnvhip.so: NNV's relax-star reachability path on one MI355X.
 *
 * The library keeps star sets resident in HBM behind opaque handles and runs, entirely on the
 * device, the three layer operations NNV's NN.reach loop calls (relaxFactor = 1, fp64):
 *
 *   FullyConnectedLayer.reach  -> nnvhip_affine_fc        (Star.affineMap, W*[c V] + b)
 *   Conv2DLayer.reach          -> nnvhip_affine_conv2d    (dlconv over the generator axis)
 *   ReluLayer.reach            -> nnvhip_relu_relax       (PosLin.reach_relaxed_star_*)
 *   Star.estimateRanges        -> nnvhip_estimate_ranges
 *
 * "file:line" citations are relative to code/nnv/engine/ of the NNV reference tree.
 *
 * Conventions: all matrices are fp64, column-major, exactly MATLAB's memory layout, so a MEX
 * gateway passes mxGetDoubles() pointers straight through.  V is N x (n+1) with column 0 the
 * centre.  An ImageStar's H x W x C x (n+1) tensor is the same memory as an (H*W*C) x (n+1)
 * matrix (set/ImageStar.m:569-592, set/Star.m:1398-1418), so one handle type serves both.
 * Index vectors are 0-based int32 here (NNV's are 1-based doubles; the gateway adds 1).
 * Every function returns an nnvhip_status; on failure nnvhip_last_error() holds the message,
 * which for NNV's own argument checks is NNV's error text.
 *
 * Threading: one host thread per context (NNV's relax-star reach is single-core,
 * nn/NN.m:1227-1231).  Handles are reference counted; an operation never modifies its input.
 */
#ifndef NNVHIP_H
#define NNVHIP_H

#include <stdint.h>

#if defined(__GNUC__)
#define NNVHIP_API __attribute__((visibility("default")))
#else
#define NNVHIP_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nnvhip_ctx nnvhip_ctx;       /* device context: stream, memory pool, timers   */
typedef struct nnvhip_star nnvhip_star;     /* a Star / ImageStar resident in HBM            */
typedef struct nnvhip_fc nnvhip_fc;         /* FullyConnectedLayer weights resident in HBM   */
typedef struct nnvhip_conv2d nnvhip_conv2d; /* Conv2DLayer weights resident in HBM           */

typedef enum {
  NNVHIP_OK = 0,
  NNVHIP_ERR_SHAPE = 1,        /* a size check of the reference failed                      */
  NNVHIP_ERR_METHOD = 2,       /* unknown reachability method / crossing order              */
  NNVHIP_ERR_RELAX_FACTOR = 3, /* relaxFactor outside [0,1], or != 1 (LP path not built)    */
  NNVHIP_ERR_OOM = 4,          /* device allocation failed                                  */
  NNVHIP_ERR_HIP = 5,          /* a HIP runtime call failed                                 */
  NNVHIP_ERR_ARG = 6           /* null pointer / invalid handle / invalid argument          */
} nnvhip_status;

/* Order of the crossing neurons = order of the new predicate columns (nn/funcs/PosLin.m):
 * INDEX  ascending neuron index: relax-star-bound/-ub/-random/-static (:1167-1232, :1326-1397,
 *        :1488-1492, :1604-1605);
 * AREA   sort(0.5*|ub|.*|lb|, 'descend'), stable: relax-star-area (:1049-1052);
 * RANGE  sort(ub-lb, 'descend'), stable: relax-star-range (:934-936). */
typedef enum { NNVHIP_ORDER_INDEX = 0, NNVHIP_ORDER_AREA = 1, NNVHIP_ORDER_RANGE = 2 } nnvhip_order;

/* ---- context -------------------------------------------------------------------------- */
/* Replaces NN.reach's reachOptions.device hook (nn/NN.m:216-222): selects the GPU, creates the
 * stream and the device memory pool. */
NNVHIP_API int nnvhip_create(int device, nnvhip_ctx** ctx);
NNVHIP_API int nnvhip_destroy(nnvhip_ctx* ctx);
/* Message of the last failing call on this thread. */
NNVHIP_API const char* nnvhip_last_error(void);
/* Waits for all queued device work of the context (wait(gpuDevice) in the reference's GPU path). */
NNVHIP_API int nnvhip_synchronize(nnvhip_ctx* ctx);
/* Device time in ms of the most recent layer call (NN.reachTime(i) = toc, nn/NN.m:1542-1545).
 * Timing is off by default (enabled = 0); 1 brackets every layer call with HIP events and makes the
 * call wait for the layer to finish; 2 additionally brackets single kernels (nnvhip_kernel_time). */
NNVHIP_API int nnvhip_set_timing(nnvhip_ctx* ctx, int enabled);
NNVHIP_API int nnvhip_last_op_time_ms(nnvhip_ctx* ctx, double* ms);
/* Measurement switch (no counterpart in the reference).  By default nnvhip_affine_fc leaves out the
 * products with structural zeros that the producing step recorded on the set handle (one-hot
 * generator columns of box stars and of ReLU outputs, rows the ReLU step reset); the result is the
 * same.  enabled = 1 runs every FC layer as the full dense contraction W*[c V], which is how the
 * reference's Star.affineMap (set/Star.m:313-343) executes it.  Initial value: 1 if the environment
 * variable NNVHIP_DENSE_AFFINE is set, else 0. */
NNVHIP_API int nnvhip_set_dense_affine(nnvhip_ctx* ctx, int enabled);
/* Output switch of nnvhip_affine_fc (no counterpart in the reference, where every affineMap writes its
 * whole result, set/Star.m:313-343).  By default the columns an FC map gathers from its weight matrix
 * are described on the output handle and written only when somebody reads them (a property read, a
 * layer that needs the whole matrix): the ReLU step that follows works from the range sums the map
 * leaves behind, and the FC map after that packs its rows from the weights.  enabled = 1 writes them
 * in the call itself; a caller does that for the layer whose output it hands on (NN.reach's return
 * value, nn/NN.m:1529-1551).  Initial value: 1 if the environment variable NNVHIP_EAGER_COLS is set. */
NNVHIP_API int nnvhip_set_eager_columns(nnvhip_ctx* ctx, int enabled);
/* Output switch of nnvhip_relu_relax (no counterpart in the reference, where
 * multipleStepReachStarApprox_at_one builds the whole new_V = [V1 V2], nn/funcs/PosLin.m:700-709).  By
 * default the step's output shares the input's matrix: the row reset and the appended unit-vector
 * columns are recorded on the handle and written when somebody needs them in memory.  enabled = 1
 * writes the whole output matrix in the call.  Initial value: 1 if the environment variables
 * NNVHIP_EAGER_ROWS and NNVHIP_EAGER_TAIL are both set (each of them alone switches its half). */
NNVHIP_API int nnvhip_set_eager_relu(nnvhip_ctx* ctx, int enabled);
/* Measurement hook (no counterpart in the reference): while timing level 2 is set, every launch of a
 * kernel group is bracketed by its own pair of HIP events on the context's stream.  which = 0:
 * dense GEMM kernel of the FC layers (tiles of at least 64 rows); 1: implicit-GEMM convolution
 * kernel; 2: estimateRanges column pass; 3: ReLU apply pass; 4: row-wise affine layers (row map,
 * average pooling, row permutation); 5: column gather of an FC layer (its one-hot generator columns);
 * 6: classification of the ReLU step (incl. the sort of the crossing list and, for small sets,
 * the new predicate bounds); 7: the reduction of range partial sums into lb / ub; 8: the
 * whole-reach kernel of small fully connected networks (nnvhip_reach_layers); 9: the tile kernel that
 * contracts kept rows only, for arrays of sets and wide single sets (work: 2*Mp*kept*columns per set).
 * Returns accumulated kernel time,
 * launch count and work since the last reset.  Work is the flop executed for 0 and 1 (GEMM:
 * 2*Mp*Kp*ncols over the columns and rows the launch contracts, M and K padded to 16; conv:
 * 2*Ho*Wo*Cout*FH*FW*Cin*(n+1)) and algorithmic bytes for
 * 2 (8*N*(n+1) + 16*n + 16*N per set), 3 (8*kept*(n+1) read + 8*N*(n+1+m) written per set, kept =
 * rows that are neither inactive nor crossing), 4 (8*(Nin + Nout)*(n+1) per set), 5 (8*M per
 * gathered column written + W read once), 6 (24*N per set, + 32*n when the bounds are written too)
 * 7 (8*N*(4*chunks + 3) per set) and 8 (per set: 8*M*K per FC layer + 8*N_out*(n_out+1) per layer). */
NNVHIP_API int nnvhip_kernel_time(nnvhip_ctx* ctx, int which, double* total_ms, int64_t* launches, double* total_work,
                       int reset);
/* Measurement hook (no counterpart in the reference): runs a plain device-to-device copy kernel over
 * `bytes` (reps + 1 times) and returns the achieved read+write bandwidth of the timed reps in GB/s -
 * the practical HBM ceiling on this box, and the known-size kernel hardware counters are
 * calibrated against. */
NNVHIP_API int nnvhip_probe_copy_bandwidth(nnvhip_ctx* ctx, int64_t bytes, int reps, double* gbytes_per_s);
/* Measurement hook (no counterpart in the reference): a register-resident loop of fp64 16x16x4 MFMAs on
 * every CU (no memory traffic); returns the rate of the timed reps in TFLOP/s - the practical ceiling
 * of the matrix pipes on this box. */
NNVHIP_API int nnvhip_probe_mfma_peak(nnvhip_ctx* ctx, int reps, double* tflops);
/* Test hooks (no counterpart in the reference).  A ReLU step on up to 8192 sets learns its crossing /
 * inactive counts through one 64-bit word per set that the classification kernel posts to pinned host
 * memory: call number (16 bits) | n_crossing (24 bits) | n_inactive (24 bits).  Before the launch the host
 * overwrites the words with the all-ones pattern, which no posted word can equal; `posted` is 0 for it.
 * nnvhip_debug_set_relu_call_number sets the context's count of ReLU calls so that a test can place
 * itself next to the wrap of the 16-bit field. */
NNVHIP_API int nnvhip_debug_mailbox_pack(int32_t n_crossing, int32_t n_inactive, int32_t call_number, uint64_t* word);
NNVHIP_API int nnvhip_debug_mailbox_unpack(uint64_t word, int32_t* posted, int32_t* n_crossing, int32_t* n_inactive,
                                int32_t* call_number);
NNVHIP_API int nnvhip_debug_set_relu_call_number(nnvhip_ctx* ctx, int64_t call_number);
/* Returns every cached device block of the pool to the driver (hipFree). */
NNVHIP_API int nnvhip_trim_pool(nnvhip_ctx* ctx);
/* Bytes currently handed out by / cached in the pool. */
NNVHIP_API int nnvhip_pool_stats(nnvhip_ctx* ctx, int64_t* bytes_in_use, int64_t* bytes_cached);
/* Diagnostic counters of a context since it was created (no counterpart in the reference), none of which this call
 * changes: hipMalloc calls of the pool (a steady loop of reaches makes none after its first pass), waits for the
 * stream because the pinned staging ring wrapped or grew, handles of released arrays that are still queued for
 * destruction (this call does not drain the queue, unlike nnvhip_pool_stats), and live handles.  Any pointer may
 * be NULL.  A benchmark reads them around a step that took unusually long. */
NNVHIP_API int nnvhip_debug_counters(nnvhip_ctx* ctx, int64_t* device_mallocs, int64_t* staging_waits, int64_t* deferred_handles,
                          int64_t* live_handles);
/* Test hook (no counterpart in the reference): how many sets, since the context was created, went through a ReLU
 * step that wrote the bounds of its new predicates behind the input's in the arrays the input already had, and how
 * many through one that copied the input's bounds into arrays of its own (new_pred_lb = [predicate_lb; zeros(m,1)],
 * nn/funcs/PosLin.m:737-738, either way).  Either pointer may be NULL. */
NNVHIP_API int nnvhip_debug_relu_bounds(nnvhip_ctx* ctx, int64_t* appended_in_place, int64_t* copied);
/* Host-to-device traffic of the context since it was created (no counterpart in the reference, whose arrays
 * never leave the host): the number of layers whose weights were uploaded (nnvhip_fc_create /
 * nnvhip_conv2d_create calls that did not find their arrays resident), the bytes of those uploads, and all
 * bytes the library copied from host to device (sets, bounds, weights, descriptor tables that do not fit the
 * pinned ring the kernels read directly).  A repeated NN.reach or Star.affineMap(W, b) adds nothing to the
 * first two. */
NNVHIP_API int nnvhip_upload_stats(nnvhip_ctx* ctx, int64_t* weight_uploads, int64_t* weight_bytes, int64_t* h2d_bytes);

/* The weight cache (see nnvhip_fc_create), no counterpart in the reference: the number of cached layers, the
 * device bytes they hold, and how many of those bytes belong to layers that only the cache still references
 * (every layer object made from them has been destroyed). */
NNVHIP_API int nnvhip_weight_cache_stats(nnvhip_ctx* ctx, int64_t* entries, int64_t* device_bytes, int64_t* unreferenced_bytes);
/* Frees every cached layer that only the cache still references (the library does so itself before it reports
 * NNVHIP_ERR_OOM); *dropped (may be NULL) receives their number. */
NNVHIP_API int nnvhip_weight_cache_release(nnvhip_ctx* ctx, int64_t* dropped);
/* Test hook (no counterpart in the reference): with on != 0 every array hashes to the same value, so that a test
 * can show that the cache tells layers apart by comparing their arrays, not by their hash.  Process-wide. */
NNVHIP_API int nnvhip_debug_weak_weight_hash(int on);

/* ---- sets ----------------------------------------------------------------------------- */
/* Star(V, C, d, pred_lb, pred_ub), set/Star.m:153-189: uploads host arrays.  V is N x (n+1),
 * C is p x n, d has p entries; pred_lb/pred_ub may be NULL (both) for the -1/+1 default of
 * Star.estimateRanges (set/Star.m:1091-1096).  C/d may be NULL with p = 0. */
NNVHIP_API int nnvhip_star_create(nnvhip_ctx* ctx, int64_t N, int64_t n, const double* V, const double* pred_lb,
                       const double* pred_ub, const double* C, const double* d, int64_t p,
                       nnvhip_star** out);
/* Star(lb, ub), set/Star.m:220-237 with Box (set/Box.m:16-58): centre 0.5*(lb+ub), one
 * generator 0.5*(ub-lb)(i)*e_i per dimension with non-zero half-width, C = zeros(1,n), d = 0,
 * predicate bounds -1/+1.  Built on the device from the two N-vectors.  `count` boxes are given
 * as the columns of N x count matrices; out[] receives `count` handles laid out back to back in
 * one device arena (the array of Stars NN.reach accepts, nn/NN.m:204-207). */
NNVHIP_API int nnvhip_star_from_box(nnvhip_ctx* ctx, int64_t N, int64_t count, const double* lb, const double* ub,
                         nnvhip_star** out);
NNVHIP_API int nnvhip_star_retain(nnvhip_star* s);
NNVHIP_API int nnvhip_star_release(nnvhip_star* s);
/* Releases one reference of each of `count` handles (null entries are skipped): what clearing an
 * object array of sets does in the reference, e.g. when NN.reach overwrites the per-layer outputs
 * it keeps in reachSet (nn/NN.m:1531, 1547).  The handles are invalid once the call returns; for arrays of
 * 256 handles and more the library may give their device memory back to its pool later (during its next
 * wait for the device, or as soon as the pool needs a block). */
NNVHIP_API int nnvhip_star_release_array(int64_t count, nnvhip_star* const* sets);
/* dim, nVar and the number of constraint rows size(C,1). */
NNVHIP_API int nnvhip_star_dims(const nnvhip_star* s, int64_t* N, int64_t* n, int64_t* p);
/* flag = 1 when the set, or the set it was derived from by the layers of this library, was created with
 * constraint rows of the caller's (the five-argument Star(V, C, d, lb, ub), set/Star.m:153-189, with a non-empty
 * C).  Such a set may be empty; Star(lb, ub) and everything the affine and ReLU layers make of a non-empty set
 * is not.  verify_specification uses it to decide whether Star.isEmptySet (set/Star.m:1216-1232) may be
 * skipped for a set that lies inside a half-space. */
NNVHIP_API int nnvhip_star_has_user_constraints(const nnvhip_star* s, int32_t* flag);
/* flag = 1 when the reference's Star would carry an outer zonotope Z here: Star(lb, ub) sets
 * Z = Zono(center, gens) (set/Star.m:230-236), Star.affineMap maps it along (set/Star.m:332-340,
 * set/Zono.m:47-74), the five-argument constructor and the ReLU step leave it empty
 * (nn/funcs/PosLin.m:740).  Z is not stored: wherever it exists it is Zono(V(:,1), V(:,2:end)) of the same set
 * (both start from the same centre and generators and are mapped by the same W, b), so a caller that wants it
 * reads V. */
NNVHIP_API int nnvhip_star_has_zono(const nnvhip_star* s, int32_t* flag);
/* Property reads: dense MATLAB arrays.  V: N x (n+1).  Bounds: n each.  C: p x n, d: p, laid out
 * exactly as PosLin.multipleStepReachStarApprox_at_one builds them, [C0;C1;C2;C3]
 * (nn/funcs/PosLin.m:711-735), materialised from the device's structured store. */
NNVHIP_API int nnvhip_star_fetch_V(const nnvhip_star* s, double* V);
/* V(rows, :): R x (n+1), column-major, rows 0-based -- the objective rows f = V(index, 2:n+1) and
 * offsets V(index, 1) that Star.getMin / getMax / getMins / getMaxs hand to the LP solver
 * (set/Star.m:742-970), gathered on the device so that only those rows cross the bus. */
NNVHIP_API int nnvhip_star_fetch_rows(const nnvhip_star* s, int64_t R, const int32_t* rows, double* out);
NNVHIP_API int nnvhip_star_fetch_pred_bounds(const nnvhip_star* s, double* pred_lb, double* pred_ub);
NNVHIP_API int nnvhip_star_fetch_constraints(const nnvhip_star* s, double* C, double* d);
/* For a set returned by nnvhip_relu_relax: counts of inactive (ub <= 0) and crossing
 * (lb < 0 & ub > 0) neurons, and the crossing list in new-predicate order with its bounds
 * (map1/map2 and lb(map), ub(map) of nn/funcs/PosLin.m:921-925, 1094-1096).  Any output pointer
 * may be NULL. */
NNVHIP_API int nnvhip_star_relu_counts(const nnvhip_star* s, int64_t* n_inactive, int64_t* n_crossing);
NNVHIP_API int nnvhip_star_fetch_crossing(const nnvhip_star* s, int32_t* index, double* lb, double* ub);

/* ---- Star.estimateRanges, set/Star.m:1078-1106 ------------------------------------------ */
/* lb = c + max(V,0)*[0;pred_lb] + min(V,0)*[0;pred_ub]; ub likewise.  One pass over V; the
 * result is cached on the handle (nnvhip_relu_relax reuses it).  lb/ub: host, N entries each,
 * may be NULL to only compute and cache on the device. */
NNVHIP_API int nnvhip_estimate_ranges(nnvhip_ctx* ctx, nnvhip_star* s, double* lb, double* ub);
/* Array form: lb/ub are N x count (all sets must have the same dim). */
NNVHIP_API int nnvhip_estimate_ranges_batch(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* s, double* lb,
                                 double* ub);

/* Star.estimateRanges for callers that cannot allocate (no counterpart in the reference): tight serving
 * loops and harnesses that forbid hipMalloc (it allocates nothing, which is also what a caller under HIP
 * graph capture needs, but the library has not been exercised under capture).  Same kernels and the
 * same results as nnvhip_estimate_ranges, but the partial sums of the column pass go to a fixed
 * workspace in device memory (32 MiB per GPU, held until the process ends) instead of the context's
 * pool, nothing is cached on the handle, and the call issues no hipMalloc / hipFree / pool request.
 * A set whose handle already caches its ranges is served from that cache and uses no workspace.
 * lb_dev / ub_dev: DEVICE pointers to N doubles each (either may be NULL); they are written on the
 * context's stream (nnvhip_synchronize, or work queued on the same stream, orders later readers).
 * Limits: the set must be a plain stored matrix (sets made by nnvhip_star_create / _from_box always
 * are; a set whose rows or columns a layer left unwritten until first read is refused with
 * NNVHIP_ERR_ARG) and 6 * roundup(N, 16) doubles must fit the workspace (N <= 699040), else
 * NNVHIP_ERR_SHAPE.  All calls on one GPU share the workspace.  Calls on one context are ordered by its
 * stream; a call from another context of the same process first makes its stream wait for the previous
 * user's kernels (an event per device), so contexts driven one after the other are safe; calls issued
 * from several processes, or kernels of a caller's own that read lb_dev / ub_dev on another stream without
 * synchronising, still race. */
NNVHIP_API int nnvhip_estimate_ranges_static(nnvhip_ctx* ctx, const nnvhip_star* s, double* lb_dev, double* ub_dev);

/* ---- layers ---------------------------------------------------------------------------- */
/* FullyConnectedLayer(W, b), nn/layers/FullyConnectedLayer.m:39-99: W is M x K, b has M entries
 * (NULL = no bias, the affineMap(W, []) form).
 * Weight cache: the reference passes weights by value (FullyConnectedLayer(W, b), Star.affineMap(W, b),
 * set/Star.m:313-343), so a caller that builds the layer again -- every call of affineMap, every NN object a
 * sweep over properties or a branch-and-bound loop constructs -- would upload the same arrays again.  Each
 * context therefore keeps the layers it has created, found by a 128-bit hash of W and b plus the geometry and
 * confirmed by comparing the caller's arrays byte for byte with the host copy the cache keeps (equal hashes
 * alone never make a hit); creating a layer whose arrays are resident returns that handle with one more
 * reference and copies nothing (nnvhip_upload_stats).  Every create is paired with a destroy as before; entries nobody else holds are
 * dropped least recently used first beyond NNVHIP_WEIGHT_CACHE_MB (environment, default 8192; 0 = no cache).
 * The same holds for nnvhip_conv2d_create. */
NNVHIP_API int nnvhip_fc_create(nnvhip_ctx* ctx, const double* W, const double* b, int64_t M, int64_t K,
                     nnvhip_fc** out);
NNVHIP_API int nnvhip_fc_destroy(nnvhip_fc* fc);
/* Conv2DLayer(W, b, padding, stride, dilation), nn/layers/Conv2DLayer.m:15-33: W is
 * FH x FW x Cin x Cout, bias has Cout entries (NULL = 0), padding [t b l r], stride [sh sw],
 * dilation [dh dw]. */
NNVHIP_API int nnvhip_conv2d_create(nnvhip_ctx* ctx, const double* W, const double* bias, int64_t FH, int64_t FW,
                         int64_t Cin, int64_t Cout, const int64_t padding[4], const int64_t stride[2],
                         const int64_t dilation[2], nnvhip_conv2d** out);
NNVHIP_API int nnvhip_conv2d_destroy(nnvhip_conv2d* conv);
/* Output feature-map size for an H x W input, nn/layers/Conv2DLayer.m:1134-1135. */
NNVHIP_API int nnvhip_conv2d_output_size(const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t* Ho, int64_t* Wo);

/* FullyConnectedLayer.reach_star_single_input / Star.affineMap,
 * nn/layers/FullyConnectedLayer.m:295-316, 476-481; set/Star.m:313-343:
 * V' = W*V; V'(:,1) += b; constraints and predicate bounds are shared with the input.
 * `count` sets are mapped in one pass (reach_star_multipleInputs, :486-512). */
NNVHIP_API int nnvhip_affine_fc(nnvhip_ctx* ctx, const nnvhip_fc* fc, int64_t count, nnvhip_star* const* in,
                     nnvhip_star** out);
/* Conv2DLayer.reach_star_single_input, nn/layers/Conv2DLayer.m:559-601, 780: the input set is
 * read as an H x W x Cin x (n+1) ImageStar; centre gets conv + bias, generators conv only;
 * cross-correlation (no kernel flip), zero padding.  Output dim is Ho*Wo*Cout. */
NNVHIP_API int nnvhip_affine_conv2d(nnvhip_ctx* ctx, const nnvhip_conv2d* conv, int64_t H, int64_t W, int64_t count,
                         nnvhip_star* const* in, nnvhip_star** out);
/* ReluLayer.reach -> PosLin.reach(I, 'relax-star-*', [], relaxFactor, ...),
 * nn/layers/ReluLayer.m:72-150, nn/funcs/PosLin.m:863-1650, 685-742, set/Star.m:1442-1461.
 * estimateRanges; inactive rows -> 0; every crossing neuron gets a new predicate column, the
 * three triangle constraints and predicate bounds [0, ub].  relax_factor must be 1 (no LP). */
NNVHIP_API int nnvhip_relu_relax(nnvhip_ctx* ctx, int order, double relax_factor, int64_t count,
                      nnvhip_star* const* in, nnvhip_star** out);
/* The 'reduceMem' suffix of a relax-star method on a ReLU layer, nn/layers/ReluLayer.m:107-112, 119-146: the
 * ImageStar the ReLU step returned (in, of height H, width W, C channels) is replaced by the box-like ImageStar
 * the reference builds from its estimated ranges [l, u]: centre 0.5*(u+l), numel(find(l-u)) predicates with
 * bounds -1 / +1, C = zeros(1, n), d = 0, and one generator per pixel (rows outer, columns inner) whose
 * first-channel half-width 0.5*(u-l) is non-zero, holding that value on every channel of the pixel; generators
 * the loop never reaches stay zero -- the reference's statements as they stand, also for C > 1.  im_lb / im_ub
 * (host, H*W*C doubles each, or NULL) receive l and u, which the reference stores as the set's im_lb / im_ub.
 * The ranges come from the device; the N x (n+1) matrix is filled by one kernel and never crosses the bus. */
NNVHIP_API int nnvhip_relu_reduce_mem(nnvhip_ctx* ctx, nnvhip_star* in, int64_t H, int64_t W, int64_t C, nnvhip_star** out,
                           double* im_lb, double* im_ub);
/* The layer loop of NN.reach for a network made of the three layer kinds above, in one call
 * (NN.reach_noConns, nn/NN.m:1529-1551: rs = Layers{i}.reach(rs, method, ...); reachSet{i} = rs).  Layer i is
 * kind[i] = NNVHIP_LAYER_FC / _CONV2D / _RELU with handle layer[i] (nnvhip_fc*, nnvhip_conv2d*, NULL) and,
 * for a convolution, the input image size hw[2*i], hw[2*i+1].  The result is what calling nnvhip_affine_fc /
 * nnvhip_affine_conv2d / nnvhip_relu_relax one after the other gives -- the same kernels in the same order;
 * only the host's work between the layers shrinks, which is what a reach of a small network consists of.
 * out receives the n_layers * count handles of reachSet, layer-major (out[i*count + k] = set k after layer
 * i); the sets of the last layer are written in full (nnvhip_set_eager_columns), as for a caller that hands
 * them on.  On failure nothing is returned and every handle made on the way is released.
 * Small networks of FC and ReLU layers only (at most 32 layers, at most 512 neurons per layer, and a worst
 * case -- every neuron of every ReLU layer crossing -- of at most 2^18 matrix entries per set over all
 * layers) take ONE launch for the whole loop, one thread block per input set: such a reach is otherwise a
 * chain of launches and host waits, each longer than its work.  Every set of reachSet is then written in
 * full, in buffers sized for that worst case; values agree with the layer-by-layer calls to rounding (sums
 * are cut differently), structure and index lists exactly unless a bound or a sort key ties to the last bit.
 * nnvhip_set_small_chain(ctx, 0) (or the environment variable NNVHIP_NO_SMALL_CHAIN) keeps such networks
 * on the layer-by-layer path. */
NNVHIP_API int nnvhip_set_small_chain(nnvhip_ctx* ctx, int enabled);
/* The switches a context reads from the environment when it is created, by name, for the rest of its life or
 * until set again (no counterpart in the reference; they select between routes of this library that give the
 * same sets, and exist so that a test suite can drive every route in one process): "dense_affine"
 * (NNVHIP_DENSE_AFFINE), "eager_rows", "eager_tail", "eager_cols" (NNVHIP_EAGER_*), "poison_pending"
 * (NNVHIP_POISON_PENDING: whatever a layer leaves unwritten until first read is filled with NaNs),
 * "no_small_chain", "no_conv_mask", "no_conv_boxes" (NNVHIP_NO_*), "no_row_deltas" (NNVHIP_NO_ROW_DELTAS: an FC
 * layer over an array of sets of one shape contracts every set over its whole kept-row list instead of forming
 * the product over the rows most sets keep once and contracting each set over its differences from that list),
 * "no_sum_shortcuts" (NNVHIP_NO_SUM_SHORTCUTS: where that layer sums its sets' pieces without storing them, every
 * set is summed in full and with both bounds of every predicate - not once per run of sets that agree in list and
 * bounds, and not with one bound where the bounds mirror each other; the sums are the same to the bit).
 * A switch applies to the layer calls made
 * after it; sets produced before keep what they recorded.  Unknown name: NNVHIP_ERR_ARG. */
NNVHIP_API int nnvhip_set_switch(nnvhip_ctx* ctx, const char* name, int enabled);
/* A hint, with no counterpart in the reference (whose layer loop, nn/NN.m:1542-1547, calls one layer after the
 * other): the FC layer that the caller will apply to the output of its NEXT nnvhip_relu_relax call on this context.
 * For an array of at least 64 sets that ReLU step then queues, right behind its classification, the part of the FC
 * layer's range estimate that needs nothing but the classes (the sums over the columns the step appends), so that
 * the device works on it while the host reads the step's counts and sets the FC call up; nnvhip_affine_fc finds it
 * on the sets and does not form it again.  Results are the same to the bit with and without the hint; a hint that
 * does not come true (another layer follows, other sets are passed) costs the product and nothing else.  The hint
 * is consumed by the next nnvhip_relu_relax call; fc == NULL withdraws it. */
NNVHIP_API int nnvhip_hint_next_fc(nnvhip_ctx* ctx, const nnvhip_fc* fc);
enum { NNVHIP_LAYER_FC = 0, NNVHIP_LAYER_CONV2D = 1, NNVHIP_LAYER_RELU = 2 };
NNVHIP_API int nnvhip_reach_layers(nnvhip_ctx* ctx, int64_t n_layers, const int32_t* kind, const void* const* layer,
                        const int64_t* hw, int order, double relax_factor, int64_t count, nnvhip_star* const* in,
                        nnvhip_star** out);
/* PosLin.multipleStepReachStarApprox_at_one(I.resetRow(reset_rows), index, lb, ub),
 * nn/funcs/PosLin.m:685-742 and set/Star.m:1442-1461: the step with the lists handed in instead of
 * derived from estimateRanges -- what the relaxFactor < 1 branches call once the host LPs
 * (Star.getMaxs / getMins) have tightened some bounds (nn/funcs/PosLin.m:1066-1096 and the sibling
 * heuristics).  reset_rows (n_reset entries) are zeroed; index (m entries, 0-based, with
 * lb[i] < 0 < ub[i]) get the triangle relaxation, new predicates in the order of the list. */
NNVHIP_API int nnvhip_relu_apply_lists(nnvhip_ctx* ctx, nnvhip_star* in, int64_t n_reset, const int32_t* reset_rows,
                            int64_t m, const int32_t* index, const double* lb, const double* ub, nnvhip_star** out);

/* ---- specification check, utils/verify_specification.m:36-80 ----------------------------- */
/* verify_specification intersects every output set with every half-space {x | G x <= g} of the
 * unsafe region (Star.intersectHalfSpace, set/Star.m:555-589) and asks whether the result is empty
 * (Star.isEmptySet, set/Star.m:1216-1232, one LP over the dense C, d).  This call answers most of
 * those questions without C: for each set and each half-space it maps the set through G
 * (Y = G*[c V], the C1/d1 rows of set/Star.m:577-578) and bounds every row of Y over the predicate
 * box exactly as Star.estimateRanges does (set/Star.m:1078-1106).
 *   some row has lo > g          -> NNVHIP_HS_DISJOINT: the LP is infeasible, the intersection is empty
 *   every row has hi <= g        -> NNVHIP_HS_INSIDE: the whole set satisfies the half-space, so the
 *                                   intersection is the set itself
 *   otherwise                    -> NNVHIP_HS_UNDECIDED: only the LP over (C, d) can tell; the host
 *                                   builds it from nnvhip_star_fetch_constraints + nnvhip_halfspace_rows
 * The half-spaces are stacked: half-space h owns rows [row_ptr[h], row_ptr[h+1]) of G (R x N,
 * column-major, R = row_ptr[n_hs]) and of g.  Outputs (host, any may be NULL): verdict is
 * count x n_hs (set index fastest), lo and hi are R x count. */
enum { NNVHIP_HS_DISJOINT = 1, NNVHIP_HS_UNDECIDED = 2, NNVHIP_HS_INSIDE = 3 };
NNVHIP_API int nnvhip_halfspace_check(nnvhip_ctx* ctx, int64_t count, nnvhip_star* const* sets, int64_t n_hs,
                           const int64_t* row_ptr, const double* G, const double* g, int64_t N,
                           int32_t* verdict, double* lo, double* hi);
/* The rows Star.intersectHalfSpace appends for one set (set/Star.m:577-581):
 * C1 = G*V(:,2:n+1) (R x n, column-major) and d1 = g - G*V(:,1). */
NNVHIP_API int nnvhip_halfspace_rows(nnvhip_ctx* ctx, nnvhip_star* s, int64_t R, const double* G, const double* g,
                          int64_t N, double* C1, double* d1);

/* ---- row-wise affine layers -------------------------------------------------------------- */
/* A per-row affine program: up to 8 steps, step s applies `v = v <op> params[:, s]` to the centre
 * column only (NNVHIP_SCOPE_CENTRE) or to the centre and every generator (NNVHIP_SCOPE_ALL), in
 * order.  It carries, with the reference's own order of operations,
 *   BatchNormalizationLayer.reach_star_single_input, nn/layers/BatchNormalizationLayer.m:247-351
 *     (ImageStar: c - mean; all / sqrt(var + eps); all * scale; c + offset.  Star: all * l; c + b),
 *   ImageInputLayer.reach_star_single_input, nn/layers/ImageInputLayer.m:121-166
 *     (zerocenter, zscore, rescale-zero-one, rescale-symmetric),
 *   ImageStar.affineMap(scale, offset), set/ImageStar.m:431-460.
 * params is N x n_steps, column-major (per-channel values are expanded to rows by the caller). */
typedef struct nnvhip_rowmap nnvhip_rowmap;
enum { NNVHIP_OP_ADD = 0, NNVHIP_OP_SUB = 1, NNVHIP_OP_MUL = 2, NNVHIP_OP_DIV = 3 };
enum { NNVHIP_SCOPE_CENTRE = 0, NNVHIP_SCOPE_ALL = 1 };
NNVHIP_API int nnvhip_rowmap_create(nnvhip_ctx* ctx, int64_t N, int32_t n_steps, const int32_t* op,
                         const int32_t* scope, const double* params, nnvhip_rowmap** out);
NNVHIP_API int nnvhip_rowmap_destroy(nnvhip_rowmap* map);
NNVHIP_API int nnvhip_affine_rowmap(nnvhip_ctx* ctx, const nnvhip_rowmap* map, int64_t count,
                         nnvhip_star* const* in, nnvhip_star** out);

/* AveragePooling2DLayer(poolSize [h w], stride [sh sw], padding [t b l r]),
 * nn/layers/AveragePooling2DLayer.m:35-147; reach_star_single_input :424-436 applies evaluate
 * (:229-247, MatConvNet's vl_nnpool 'avg') to every H x W x C image of V: the mean over the part
 * of each window that lies inside the image.  Output dim is Ho*Wo*C. */
typedef struct nnvhip_avgpool2d nnvhip_avgpool2d;
NNVHIP_API int nnvhip_avgpool2d_create(nnvhip_ctx* ctx, const int64_t pool[2], const int64_t stride[2],
                            const int64_t padding[4], nnvhip_avgpool2d** out);
NNVHIP_API int nnvhip_avgpool2d_destroy(nnvhip_avgpool2d* layer);
NNVHIP_API int nnvhip_avgpool2d_output_size(const nnvhip_avgpool2d* layer, int64_t H, int64_t W, int64_t* Ho,
                                 int64_t* Wo);
NNVHIP_API int nnvhip_affine_avgpool2d(nnvhip_ctx* ctx, const nnvhip_avgpool2d* layer, int64_t H, int64_t W,
                            int64_t count, nnvhip_star* const* in, nnvhip_star** out);

/* Row permutation out(r, :) = in(src_row[r], :): the C-style variants of FlattenLayer.evaluate
 * applied to every image of V (nn/layers/FlattenLayer.m:118-170, 178-199).  The MATLAB-style
 * flatten is a plain reshape and needs no call.  src_row: N entries, 0-based, a permutation. */
NNVHIP_API int nnvhip_permute_rows(nnvhip_ctx* ctx, int64_t N, const int32_t* src_row, int64_t count,
                        nnvhip_star* const* in, nnvhip_star** out);

#ifdef __cplusplus
}
#endif
#endif /* NNVHIP_H */
