// Context: device memory pool, pinned staging ring, switches, timers and the measurement probes.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "internal.h"
#include "mfma_tile.h"

namespace nnvhip {

static thread_local char g_err[1024] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
}

Buffer::~Buffer() {
  if (ctx && ptr) ctx->release_block(ptr, bytes);
}

// Size classes: multiples of 256 B up to 64 KiB, then 1/8-octave steps (<= 12.5 % slack), so a
// repeated reach over the same network re-uses every block without calling hipMalloc again.
static size_t size_class(size_t bytes) {
  if (bytes < 256) return 256;
  if (bytes <= (64u << 10)) return (bytes + 255) & ~size_t(255);
  size_t p = size_t(1) << (63 - __builtin_clzll((unsigned long long)bytes));
  size_t step = p >> 3;
  return (bytes + step - 1) / step * step;
}

const TuneKnobs& tune_knobs() {
  static const TuneKnobs knobs = [] {
    TuneKnobs k;
    auto num = [](const char* name) {
      const char* e = getenv(name);
      return e ? atoi(e) : 0;
    };
    k.gemm_xr = num("NNVHIP_GEMM_XR");
    k.gemm_ksplit = num("NNVHIP_GEMM_KSPLIT");
    if (const char* e = getenv("NNVHIP_GEMM_TILE")) k.gemm_tile = e;
    k.ranges_row_waves = num("NNVHIP_RANGES_ROW_WAVES");
    k.ranges_blocks = num("NNVHIP_RANGES_BLOCKS");
    k.apply_row_waves = num("NNVHIP_APPLY_ROW_WAVES");
    k.apply_blocks = num("NNVHIP_APPLY_BLOCKS");
    k.conv_general = num("NNVHIP_CONV_GENERAL");
    k.one_block_n = num("NNVHIP_ONE_BLOCK_N");
    return k;
  }();
  return knobs;
}

int enter_ctx(nnvhip_ctx* ctx) {
  NNV_HIP_TRY(hipSetDevice(ctx->device));
  return NNVHIP_OK;
}

// Handles come from (and go back to) a list of released ones kept by the context: an array of a thousand sets makes
// and lets go of a thousand handles per layer, on the host's critical path.
nnvhip_star* new_star(nnvhip_ctx* ctx) {
  nnvhip_star* s;
  if (!ctx->free_stars.empty()) {
    void* mem = ctx->free_stars.back();
    ctx->free_stars.pop_back();
    s = new (mem) nnvhip_star();
  } else {
    s = new (::operator new(sizeof(nnvhip_star))) nnvhip_star();
  }
  s->ctx = ctx;
  ctx->live_handles++;
  return s;
}

void delete_star(nnvhip_star* s) {
  nnvhip_ctx* c = s->ctx;
  s->~nnvhip_star();
  if (c->free_stars.size() < nnvhip_ctx::kMaxFreeStars)
    c->free_stars.push_back(s);
  else
    ::operator delete(static_cast<void*>(s));
  c->live_handles--;
}

}  // namespace nnvhip

using namespace nnvhip;

void nnvhip_ctx::drain_deferred(size_t at_most) {
  while (!deferred.empty() && at_most-- > 0) {
    nnvhip_star* s = deferred.back();
    deferred.pop_back();
    nnvhip_star_release(s);
  }
}

int nnvhip_ctx::alloc(size_t bytes, BufRef* out) {
  size_t cls = size_class(bytes ? bytes : 1);
  void* p = nullptr;
  auto it = free_blocks.find(cls);
  // A released array that has not been let go yet may hold such a block.  While the pool is small next to the
  // device's memory it grows instead (a loop of reaches then alternates between two generations of blocks and
  // never waits for the handles of the previous one); past that share the array is let go now.
  if (it == free_blocks.end() && !deferred.empty() &&
      (double)(bytes_in_use + bytes_cached) + (double)cls > 0.4 * (double)device_bytes) {
    drain_deferred();
    it = free_blocks.find(cls);
  }
  if (it != free_blocks.end()) {
    p = it->second;
    free_blocks.erase(it);
    bytes_cached -= (int64_t)cls;
  } else {
    hipError_t e = hipMalloc(&p, cls);
    n_device_mallocs++;
    if (e != hipSuccess) {
      (void)hipGetLastError();
      drop_unreferenced_weights();  // layers that only the weight cache still holds
      trim();                       // let released arrays go, give cached blocks back and retry once
      e = hipMalloc(&p, cls);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        NNV_FAIL(NNVHIP_ERR_OOM, "out of device memory allocating %zu bytes", cls);
      }
    }
  }
  bytes_in_use += (int64_t)cls;
  auto b = make_ref<Buffer>();
  b->ctx = this;
  b->ptr = p;
  b->bytes = cls;
  *out = std::move(b);
  return NNVHIP_OK;
}

void nnvhip_ctx::release_block(void* p, size_t bytes) {
  // Blocks are recycled without waiting: every consumer runs on the context's single stream, so
  // a later user of the block is ordered after the earlier one.
  free_blocks.emplace(bytes, p);
  bytes_in_use -= (int64_t)bytes;
  bytes_cached += (int64_t)bytes;
}

int nnvhip_ctx::trim() {
  if (stream) (void)hipStreamSynchronize(stream);
  drain_deferred();
  for (auto& kv : free_blocks) (void)hipFree(kv.second);
  free_blocks.clear();
  bytes_cached = 0;
  return NNVHIP_OK;
}

int nnvhip_ctx::stage(size_t bytes, void** host) {
  bytes = (bytes + 255) & ~size_t(255);
  if (bytes > pinned_bytes) {
    n_staging_waits++;
    NNV_HIP_TRY(hipStreamSynchronize(stream));
    // a table handed out from the old ring may still be named by a launch that is about to be issued:
    // the old ring stays allocated until the context goes (rings only ever grow, by doubling)
    if (pinned) retired_rings.push_back(pinned);
    pinned = nullptr;
    pinned_bytes = std::max(bytes * 2, size_t(4) << 20);
    NNV_HIP_TRY(hipHostMalloc((void**)&pinned, pinned_bytes, hipHostMallocDefault));
    pinned_off = 0;
  }
  if (pinned_off + bytes > pinned_bytes) {
    n_staging_waits++;
    NNV_HIP_TRY(hipStreamSynchronize(stream));  // earlier async copies out of the ring are done
    pinned_off = 0;
  }
  *host = pinned + pinned_off;
  pinned_off += bytes;
  return NNVHIP_OK;
}

int nnvhip_ctx::upload_table(const void* host, size_t bytes, BufRef* out) {
  if (bytes > (size_t(64) << 10)) return upload(host, bytes, out);
  void* st = nullptr;
  NNV_TRY(stage(bytes, &st));
  memcpy(st, host, bytes);
  auto b = make_ref<Buffer>();  // no owner: the slot belongs to the ring
  b->ptr = st;
  b->bytes = bytes;
  *out = std::move(b);
  return NNVHIP_OK;
}

int nnvhip_ctx::upload(const void* host, size_t bytes, BufRef* out) {
  void* st = nullptr;
  NNV_TRY(stage(bytes, &st));
  memcpy(st, host, bytes);
  NNV_TRY(alloc(bytes, out));
  NNV_HIP_TRY(hipMemcpyAsync((*out)->ptr, st, bytes, hipMemcpyHostToDevice, stream));
  h2d_bytes += (int64_t)bytes;
  return NNVHIP_OK;
}

int nnvhip_ctx::kernel_timer_begin(bool) { return NNVHIP_OK; }  // the events travel with the launch (NNV_LAUNCH)

int nnvhip_ctx::kernel_timer_end(bool on, int which, double flop) {
  if (on) {  // start / stop events of the one kernel just launched
    NNV_HIP_TRY(hipEventSynchronize(kev1));
    float ms = 0.f;
    NNV_HIP_TRY(hipEventElapsedTime(&ms, kev0, kev1));
    kern_ms[which] += ms;
    kern_launches[which] += 1;
    kern_flop[which] += flop;
  }
  return NNVHIP_OK;
}

int nnvhip_ctx::begin_op() {
  if (timing) NNV_HIP_TRY(hipEventRecord(ev0, stream));
  return NNVHIP_OK;
}

int nnvhip_ctx::end_op() {
  if (timing) {
    NNV_HIP_TRY(hipEventRecord(ev1, stream));
    NNV_HIP_TRY(hipEventSynchronize(ev1));
    float ms = 0.f;
    NNV_HIP_TRY(hipEventElapsedTime(&ms, ev0, ev1));
    last_ms = ms;
  }
  return NNVHIP_OK;
}

extern "C" {

const char* nnvhip_last_error(void) { return g_err; }

int nnvhip_create(int device, nnvhip_ctx** out) {
  if (!out) NNV_FAIL(NNVHIP_ERR_ARG, "null output pointer");
  int ndev = 0;
  NNV_HIP_TRY(hipGetDeviceCount(&ndev));
  if (device < 0 || device >= ndev) NNV_FAIL(NNVHIP_ERR_ARG, "device %d not present (%d visible)", device, ndev);
  NNV_HIP_TRY(hipSetDevice(device));
  hipDeviceProp_t prop;
  NNV_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    NNV_FAIL(NNVHIP_ERR_ARG, "libnnvhip is built for gfx950 (MI355X); device %d is %s", device, prop.gcnArchName);
  nnvhip_ctx* c = new nnvhip_ctx();
  c->device = device;
  c->device_bytes = (int64_t)prop.totalGlobalMem;
  c->dense_affine = getenv("NNVHIP_DENSE_AFFINE") != nullptr;
  c->eager_tail = getenv("NNVHIP_EAGER_TAIL") != nullptr;
  c->eager_rows = getenv("NNVHIP_EAGER_ROWS") != nullptr;
  c->eager_cols = getenv("NNVHIP_EAGER_COLS") != nullptr;
  c->poison_pending = getenv("NNVHIP_POISON_PENDING") != nullptr;
  c->small_chain = getenv("NNVHIP_NO_SMALL_CHAIN") == nullptr;
  c->no_conv_mask = getenv("NNVHIP_NO_CONV_MASK") != nullptr;
  c->no_conv_boxes = getenv("NNVHIP_NO_CONV_BOXES") != nullptr;
  c->no_row_deltas = getenv("NNVHIP_NO_ROW_DELTAS") != nullptr;
  c->no_sum_shortcuts = getenv("NNVHIP_NO_SUM_SHORTCUTS") != nullptr;
  if (const char* e = getenv("NNVHIP_WEIGHT_CACHE_MB")) c->weight_cache_budget = (int64_t)atoll(e) << 20;
  NNV_HIP_TRY(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
  NNV_HIP_TRY(hipEventCreate(&c->ev0));
  NNV_HIP_TRY(hipEventCreate(&c->ev1));
  NNV_HIP_TRY(hipHostMalloc((void**)&c->mailbox, sizeof(int64_t) * nnvhip_ctx::kMailboxSets, hipHostMallocDefault));
  memset((void*)c->mailbox, 0xff, sizeof(int64_t) * nnvhip_ctx::kMailboxSets);  // kMailboxEmpty everywhere
  NNV_HIP_TRY(hipEventCreate(&c->kev0));
  NNV_HIP_TRY(hipEventCreate(&c->kev1));
  NNV_HIP_TRY(hipEventCreateWithFlags(&c->read_ev, hipEventDisableTiming));
  NNV_TRY(init_static_scratch(c));
  *out = c;
  return NNVHIP_OK;
}

int nnvhip_destroy(nnvhip_ctx* c) {
  if (!c) return NNVHIP_OK;
  c->drop_weight_cache(true);
  c->drain_deferred();
  if (c->live_handles != 0)
    NNV_FAIL(NNVHIP_ERR_ARG, "context still has %lld live handles", (long long)c->live_handles);
  NNV_TRY(nnvhip::enter_ctx(c));
  c->trim();
  for (void* mem : c->free_stars) ::operator delete(mem);
  c->free_stars.clear();
  if (c->pinned) (void)hipHostFree(c->pinned);
  if (c->mailbox) (void)hipHostFree((void*)c->mailbox);
  for (char* r : c->retired_rings) (void)hipHostFree(r);
  (void)hipEventDestroy(c->ev0);
  (void)hipEventDestroy(c->ev1);
  (void)hipEventDestroy(c->kev0);
  (void)hipEventDestroy(c->kev1);
  if (c->read_ev) (void)hipEventDestroy(c->read_ev);
  (void)hipStreamDestroy(c->stream);
  delete c;
  return NNVHIP_OK;
}

int nnvhip_synchronize(nnvhip_ctx* c) {
  CHECK_CTX(c);
  // released arrays are let go while the device works; whatever is left, once it is done
  while (!c->deferred.empty() && hipStreamQuery(c->stream) == hipErrorNotReady) c->drain_deferred(64);
  (void)hipGetLastError();
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  c->drain_deferred();
  return NNVHIP_OK;
}

int nnvhip_set_timing(nnvhip_ctx* c, int enabled) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->timing = enabled != 0;
  c->kernel_timing = enabled >= 2;
  return NNVHIP_OK;
}

int nnvhip_set_dense_affine(nnvhip_ctx* c, int enabled) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->dense_affine = enabled != 0;
  return NNVHIP_OK;
}

int nnvhip_set_eager_columns(nnvhip_ctx* c, int enabled) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->eager_cols = enabled != 0;
  return NNVHIP_OK;
}

int nnvhip_set_eager_relu(nnvhip_ctx* c, int enabled) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->eager_rows = enabled != 0;
  c->eager_tail = enabled != 0;
  return NNVHIP_OK;
}

int nnvhip_set_small_chain(nnvhip_ctx* c, int enabled) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->small_chain = enabled != 0;
  return NNVHIP_OK;
}

int nnvhip_set_switch(nnvhip_ctx* c, const char* name, int enabled) {
  if (!c || !name) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  const bool on = enabled != 0;
  const struct {
    const char* name;
    bool* flag;
    bool inverted;
  } table[] = {
      {"dense_affine", &c->dense_affine, false},   {"eager_rows", &c->eager_rows, false},
      {"eager_tail", &c->eager_tail, false},       {"eager_cols", &c->eager_cols, false},
      {"poison_pending", &c->poison_pending, false}, {"no_small_chain", &c->small_chain, true},
      {"no_conv_mask", &c->no_conv_mask, false},   {"no_conv_boxes", &c->no_conv_boxes, false},
      {"no_row_deltas", &c->no_row_deltas, false}, {"no_sum_shortcuts", &c->no_sum_shortcuts, false},
  };
  for (const auto& t : table)
    if (strcmp(t.name, name) == 0) {
      *t.flag = t.inverted ? !on : on;
      return NNVHIP_OK;
    }
  NNV_FAIL(NNVHIP_ERR_ARG, "unknown switch '%s'", name);
}

int nnvhip_last_op_time_ms(nnvhip_ctx* c, double* ms) {
  if (!c || !ms) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  *ms = c->last_ms;
  return NNVHIP_OK;
}

int nnvhip_kernel_time(nnvhip_ctx* c, int which, double* total_ms, int64_t* launches, double* total_flop, int reset) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (which < 0 || which >= nnvhip_ctx::kKernelGroups) NNV_FAIL(NNVHIP_ERR_ARG, "unknown kernel group %d", which);
  if (total_ms) *total_ms = c->kern_ms[which];
  if (launches) *launches = c->kern_launches[which];
  if (total_flop) *total_flop = c->kern_flop[which];
  if (reset) {
    c->kern_ms[which] = 0.0;
    c->kern_launches[which] = 0;
    c->kern_flop[which] = 0.0;
  }
  return NNVHIP_OK;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const double2* __restrict__ in, double2* __restrict__ out,
                                                          int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) out[i] = in[i];
}

int nnvhip_probe_copy_bandwidth(nnvhip_ctx* c, int64_t bytes, int reps, double* gbytes_per_s) {
  CHECK_CTX(c);
  if (bytes < 16 || reps < 1 || !gbytes_per_s) NNV_FAIL(NNVHIP_ERR_ARG, "invalid argument");
  bytes &= ~int64_t(15);
  BufRef a, b;
  NNV_TRY(c->alloc((size_t)bytes, &a));
  NNV_TRY(c->alloc((size_t)bytes, &b));
  NNV_HIP_TRY(hipMemsetAsync(a->ptr, 0, (size_t)bytes, c->stream));
  const int64_t n = bytes / 16;
  const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(n, 256), 256 * 32);
  hipLaunchKernelGGL(probe_copy_kernel, dim3(blocks), dim3(256), 0, c->stream, a->as<double2>(), b->as<double2>(), n);
  NNV_HIP_TRY(hipEventRecord(c->kev0, c->stream));
  for (int i = 0; i < reps; ++i)
    hipLaunchKernelGGL(probe_copy_kernel, dim3(blocks), dim3(256), 0, c->stream, a->as<double2>(), b->as<double2>(), n);
  NNV_HIP_TRY(hipEventRecord(c->kev1, c->stream));
  NNV_HIP_TRY(hipEventSynchronize(c->kev1));
  NNV_HIP_TRY(hipGetLastError());
  float ms = 0.f;
  NNV_HIP_TRY(hipEventElapsedTime(&ms, c->kev0, c->kev1));
  *gbytes_per_s = 2.0 * (double)bytes * reps / (ms * 1e-3) / 1e9;  // bytes read + bytes written
  return NNVHIP_OK;
}

// Register-resident fp64 MFMA loop: 8 independent accumulators per wave, 8 waves per block, no memory
// traffic.  What the matrix pipes deliver on this box when nothing else stands in their way.
__global__ __launch_bounds__(512) void probe_mfma_kernel(double* __restrict__ out, int iters) {
  double4_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = double4_t{0.0, 0.0, 0.0, 0.0};
  const double a = threadIdx.x * 1e-3, b = threadIdx.x * 2e-3;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
  }
  double s = 0.0;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}

int nnvhip_probe_mfma_peak(nnvhip_ctx* c, int reps, double* tflops) {
  CHECK_CTX(c);
  if (reps < 1 || !tflops) NNV_FAIL(NNVHIP_ERR_ARG, "invalid argument");
  const int blocks = 2048, iters = 2000;
  BufRef out;
  NNV_TRY(c->alloc(sizeof(double) * 512 * blocks, &out));
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(512), 0, c->stream, out->as<double>(), iters);
  NNV_HIP_TRY(hipEventRecord(c->kev0, c->stream));
  for (int i = 0; i < reps; ++i)
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(512), 0, c->stream, out->as<double>(), iters);
  NNV_HIP_TRY(hipEventRecord(c->kev1, c->stream));
  NNV_HIP_TRY(hipEventSynchronize(c->kev1));
  NNV_HIP_TRY(hipGetLastError());
  float ms = 0.f;
  NNV_HIP_TRY(hipEventElapsedTime(&ms, c->kev0, c->kev1));
  // one 16x16x4 MFMA = 2*16*16*4 flop; 8 per iteration and wave, 8 waves per block
  *tflops = 2048.0 * 8.0 * iters * 8.0 * blocks * reps / (ms * 1e-3) / 1e12;
  return NNVHIP_OK;
}

int nnvhip_debug_mailbox_pack(int32_t n_crossing, int32_t n_inactive, int32_t call_number, uint64_t* word) {
  if (!word) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  *word = mailbox_word(n_crossing, n_inactive, call_number);
  return NNVHIP_OK;
}

int nnvhip_debug_mailbox_unpack(uint64_t word, int32_t* posted, int32_t* n_crossing, int32_t* n_inactive,
                                int32_t* call_number) {
  int m = 0, inact = 0, seq = 0;
  mailbox_unpack(word, &m, &inact, &seq);
  if (posted) *posted = word != kMailboxEmpty;
  if (n_crossing) *n_crossing = m;
  if (n_inactive) *n_inactive = inact;
  if (call_number) *call_number = seq;
  return NNVHIP_OK;
}

int nnvhip_debug_set_relu_call_number(nnvhip_ctx* c, int64_t call_number) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->mailbox_seq = (uint32_t)call_number;
  return NNVHIP_OK;
}

int nnvhip_trim_pool(nnvhip_ctx* c) {
  CHECK_CTX(c);
  return c->trim();
}

int nnvhip_upload_stats(nnvhip_ctx* c, int64_t* weight_uploads, int64_t* weight_bytes, int64_t* h2d_bytes) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (weight_uploads) *weight_uploads = c->weight_uploads;
  if (weight_bytes) *weight_bytes = c->weight_upload_bytes;
  if (h2d_bytes) *h2d_bytes = c->h2d_bytes;
  return NNVHIP_OK;
}

int nnvhip_debug_counters(nnvhip_ctx* c, int64_t* device_mallocs, int64_t* staging_waits, int64_t* deferred_handles,
                          int64_t* live_handles) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (device_mallocs) *device_mallocs = c->n_device_mallocs;
  if (staging_waits) *staging_waits = c->n_staging_waits;
  if (deferred_handles) *deferred_handles = (int64_t)c->deferred.size();
  if (live_handles) *live_handles = c->live_handles;
  return NNVHIP_OK;
}

int nnvhip_debug_relu_bounds(nnvhip_ctx* c, int64_t* appended_in_place, int64_t* copied) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (appended_in_place) *appended_in_place = c->n_bounds_in_place;
  if (copied) *copied = c->n_bounds_copied;
  return NNVHIP_OK;
}

int nnvhip_pool_stats(nnvhip_ctx* c, int64_t* in_use, int64_t* cached) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->drain_deferred();
  if (in_use) *in_use = c->bytes_in_use;
  if (cached) *cached = c->bytes_cached;
  return NNVHIP_OK;
}

}  // extern "C"
