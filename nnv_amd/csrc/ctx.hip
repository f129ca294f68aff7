// Context, device memory pool, set handles and the host-side orchestration of the affine layers.
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

// Wt(r, k) = W(r, k): the Mp x Kp column-major weights row-major (ld = Kp), 32 x 32 tiles through LDS
__global__ __launch_bounds__(256) void transpose_weights_kernel(const double* __restrict__ W, double* __restrict__ Wt, int Mp, int Kp) {
  __shared__ double tile[32][33];
  const int k0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  for (int i = threadIdx.y; i < 32; i += 8) {
    const int k = k0 + i, r = r0 + threadIdx.x;
    tile[i][threadIdx.x] = (k < Kp && r < Mp) ? W[r + (int64_t)k * Mp] : 0.0;
  }
  __syncthreads();
  for (int i = threadIdx.y; i < 32; i += 8) {
    const int r = r0 + i, k = k0 + threadIdx.x;
    if (r < Mp && k < Kp) Wt[(int64_t)r * Kp + k] = tile[threadIdx.x][i];
  }
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

static bool g_weak_weight_hash = false;  // test hook: every array hashes alike, so only the byte comparison tells layers apart

void hash_bytes(const void* data, size_t bytes, uint64_t* h0, uint64_t* h1) {
  auto fold = [](uint64_t a, uint64_t b) {
    const __uint128_t r = (__uint128_t)a * b;
    return (uint64_t)r ^ (uint64_t)(r >> 64);
  };
  auto rotl = [](uint64_t x, int r) { return (x << r) | (x >> (64 - r)); };
  const uint64_t k0 = 0xa0761d6478bd642full, k1 = 0xe7037ed1a0b428dbull, k2 = 0x8ebc6af09c88c6e3ull, k3 = 0x589965cc75374cc3ull;
  if (g_weak_weight_hash) {
    *h0 = k0;
    *h1 = k1;
    return;
  }
  uint64_t a = k0 ^ bytes, b = k1 ^ bytes, c = k2 ^ bytes, d = k3 ^ bytes;
  const unsigned char* p = static_cast<const unsigned char*>(data);
  size_t i = 0;
  // Four words a round, four streams.  A product alone would forget its stream's past whenever one factor is zero
  // (a block that equals the constants it is mixed with), so every stream also carries its previous state and
  // the words along additively.
  for (; i + 32 <= bytes; i += 32) {
    uint64_t w[4];
    memcpy(w, p + i, 32);
    a = fold(a ^ w[0], k1 ^ w[1]) + rotl(a, 29) + w[1];
    b = fold(b ^ w[2], k2 ^ w[3]) + rotl(b, 31) + w[3];
    c = fold(c ^ w[1], k3 ^ w[2]) + rotl(c, 37) + w[2];
    d = fold(d ^ w[3], k0 ^ w[0]) + rotl(d, 41) + w[0];
  }
  uint64_t tail[4] = {0, 0, 0, 0};
  if (i < bytes) memcpy(tail, p + i, bytes - i);
  a = fold(a ^ tail[0], k1 ^ tail[1]) + rotl(a, 29) + tail[1];
  b = fold(b ^ tail[2], k2 ^ tail[3]) + rotl(b, 31) + tail[3];
  c = fold(c ^ tail[1], k3 ^ tail[2]) + rotl(c, 37) + tail[2];
  d = fold(d ^ tail[3], k0 ^ tail[0]) + rotl(d, 41) + tail[0];
  *h0 = fold(a ^ k2, b ^ k3) ^ a ^ rotl(b, 17);
  *h1 = fold(c ^ k0, d ^ k1) ^ d ^ rotl(c, 19);
}

int enter_ctx(nnvhip_ctx* ctx) {
  NNV_HIP_TRY(hipSetDevice(ctx->device));
  return NNVHIP_OK;
}

nnvhip_star* new_star(nnvhip_ctx* ctx) {
  nnvhip_star* s = new nnvhip_star();
  s->ctx = ctx;
  ctx->live_handles++;
  return s;
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
  auto b = std::make_shared<Buffer>();
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
  auto b = std::make_shared<Buffer>();  // no owner: the slot belongs to the ring
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

// Frees the cache's references: every entry (all), or least recently used entries that nobody else holds
// until the cache is back under its budget.
void nnvhip_ctx::drop_weight_cache(bool all) {
  while (!weight_cache.empty() && (all || weight_cache_bytes > weight_cache_budget)) {
    auto victim = weight_cache.end();
    for (auto it = weight_cache.begin(); it != weight_cache.end(); ++it) {
      const int refs = it->first.kind == 0 ? static_cast<nnvhip_fc*>(it->second.handle)->refs.load()
                                           : static_cast<nnvhip_conv2d*>(it->second.handle)->refs.load();
      if (!all && refs > 1) continue;  // in use by a layer object
      if (victim == weight_cache.end() || it->second.last_use < victim->second.last_use) victim = it;
    }
    if (victim == weight_cache.end()) break;
    weight_cache_bytes -= victim->second.bytes;
    if (victim->first.kind == 0) {
      nnvhip_fc* f = static_cast<nnvhip_fc*>(victim->second.handle);
      if (f->refs.fetch_sub(1) == 1) delete f;
    } else {
      nnvhip_conv2d* v = static_cast<nnvhip_conv2d*>(victim->second.handle);
      if (v->refs.fetch_sub(1) == 1) delete v;
    }
    weight_cache.erase(victim);
  }
}

int64_t nnvhip_ctx::drop_unreferenced_weights() {
  int64_t dropped = 0;
  for (auto it = weight_cache.begin(); it != weight_cache.end();) {
    const bool fc = it->first.kind == 0;
    const int refs = fc ? static_cast<nnvhip_fc*>(it->second.handle)->refs.load()
                        : static_cast<nnvhip_conv2d*>(it->second.handle)->refs.load();
    if (refs > 1) {
      ++it;
      continue;
    }
    weight_cache_bytes -= it->second.bytes;
    if (fc)
      delete static_cast<nnvhip_fc*>(it->second.handle);
    else
      delete static_cast<nnvhip_conv2d*>(it->second.handle);
    it = weight_cache.erase(it);
    ++dropped;
  }
  return dropped;
}

// The cached layer that was made from exactly these host arrays, or null.  Entries whose hash and geometry agree
// but whose arrays differ are stepped over by raising key.salt, which is then also the key a new entry goes under.
static void* weight_cache_find(nnvhip_ctx* c, WeightKey* key, const double* W, size_t nw, const double* b, size_t nb) {
  for (key->salt = 0;; ++key->salt) {
    auto hit = c->weight_cache.find(*key);
    if (hit == c->weight_cache.end()) return nullptr;
    const WeightEntry& e = hit->second;
    if (e.host_w.size() == nw && e.host_b.size() == nb && memcmp(e.host_w.data(), W, sizeof(double) * nw) == 0 &&
        (nb == 0 || memcmp(e.host_b.data(), b, sizeof(double) * nb) == 0)) {
      hit->second.last_use = ++c->weight_clock;
      return e.handle;
    }
  }
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

#define CHECK_CTX(c)                                                  \
  do {                                                                \
    if (!(c)) NNV_FAIL(NNVHIP_ERR_ARG, "null context");               \
    NNV_TRY(nnvhip::enter_ctx(c));                                    \
  } while (0)

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
  if (const char* e = getenv("NNVHIP_WEIGHT_CACHE_MB")) c->weight_cache_budget = (int64_t)atoll(e) << 20;
  NNV_HIP_TRY(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
  NNV_HIP_TRY(hipEventCreate(&c->ev0));
  NNV_HIP_TRY(hipEventCreate(&c->ev1));
  NNV_HIP_TRY(hipHostMalloc((void**)&c->mailbox, sizeof(int64_t) * nnvhip_ctx::kMailboxSets, hipHostMallocDefault));
  memset((void*)c->mailbox, 0xff, sizeof(int64_t) * nnvhip_ctx::kMailboxSets);  // kMailboxEmpty everywhere
  NNV_HIP_TRY(hipEventCreate(&c->kev0));
  NNV_HIP_TRY(hipEventCreate(&c->kev1));
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
  if (c->pinned) (void)hipHostFree(c->pinned);
  if (c->mailbox) (void)hipHostFree((void*)c->mailbox);
  for (char* r : c->retired_rings) (void)hipHostFree(r);
  (void)hipEventDestroy(c->ev0);
  (void)hipEventDestroy(c->ev1);
  (void)hipEventDestroy(c->kev0);
  (void)hipEventDestroy(c->kev1);
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
      {"no_row_deltas", &c->no_row_deltas, false},
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

int nnvhip_weight_cache_stats(nnvhip_ctx* c, int64_t* entries, int64_t* device_bytes, int64_t* unreferenced_bytes) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  int64_t unref = 0;
  for (const auto& kv : c->weight_cache) {
    const int refs = kv.first.kind == 0 ? static_cast<nnvhip_fc*>(kv.second.handle)->refs.load()
                                        : static_cast<nnvhip_conv2d*>(kv.second.handle)->refs.load();
    if (refs <= 1) unref += kv.second.bytes;
  }
  if (entries) *entries = (int64_t)c->weight_cache.size();
  if (device_bytes) *device_bytes = c->weight_cache_bytes;
  if (unreferenced_bytes) *unreferenced_bytes = unref;
  return NNVHIP_OK;
}

int nnvhip_weight_cache_release(nnvhip_ctx* c, int64_t* dropped) {
  CHECK_CTX(c);
  const int64_t n = c->drop_unreferenced_weights();
  if (dropped) *dropped = n;
  return NNVHIP_OK;
}

int nnvhip_debug_weak_weight_hash(int on) {
  g_weak_weight_hash = on != 0;
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

int nnvhip_pool_stats(nnvhip_ctx* c, int64_t* in_use, int64_t* cached) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  c->drain_deferred();
  if (in_use) *in_use = c->bytes_in_use;
  if (cached) *cached = c->bytes_cached;
  return NNVHIP_OK;
}

/* ------------------------------------------------------------------------------------------ */
/* sets                                                                                        */
/* ------------------------------------------------------------------------------------------ */

// Uploads a host column-major rows x cols matrix into a zero-padded device matrix with leading
// dimension ld.
static int upload_matrix(nnvhip_ctx* c, const double* host, int64_t rows, int64_t cols, int64_t ld,
                         double* dev) {
  if (rows == 0 || cols == 0) return NNVHIP_OK;
  if (ld != rows) NNV_HIP_TRY(hipMemsetAsync(dev, 0, sizeof(double) * ld * cols, c->stream));
  NNV_HIP_TRY(hipMemcpy2DAsync(dev, sizeof(double) * ld, host, sizeof(double) * rows, sizeof(double) * rows,
                               cols, hipMemcpyHostToDevice, c->stream));
  c->h2d_bytes += (int64_t)sizeof(double) * rows * cols;
  // the source is pageable caller memory: finish before returning
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_star_create(nnvhip_ctx* c, int64_t N, int64_t n, const double* V, const double* pred_lb,
                       const double* pred_ub, const double* C, const double* d, int64_t p,
                       nnvhip_star** out) {
  CHECK_CTX(c);
  if (!out || !V) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (N <= 0 || n < 0 || p < 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "invalid set size N=%lld n=%lld p=%lld", (long long)N, (long long)n, (long long)p);
  if ((pred_lb == nullptr) != (pred_ub == nullptr))
    NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistency between number of predicate variables and predicate lower- or upper-bounds vector");
  if (p > 0 && (!C || !d)) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistency between constraint matrix and constraint vector");
  nnvhip_star* s = new_star(c);
  std::unique_ptr<nnvhip_star, int (*)(nnvhip_star*)> guard(s, nnvhip_star_release);
  s->N = N;
  s->n = n;
  s->ld = round_up(N, kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * s->ld * (n + 1), &s->Vbuf));
  s->V = s->Vbuf->as<double>();
  NNV_TRY(upload_matrix(c, V, N, n + 1, s->ld, s->V));
  int64_t npad = round_up(std::max<int64_t>(n, 1), kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * 2 * npad, &s->pbuf));
  s->plb = s->pbuf->as<double>();
  s->pub = s->plb + npad;
  if (n > 0) {
    std::vector<double> tmp(2 * npad, 0.0);
    for (int64_t i = 0; i < n; ++i) {
      tmp[i] = pred_lb ? pred_lb[i] : -1.0;  // default of Star.estimateRanges, set/Star.m:1091-1096
      tmp[npad + i] = pred_ub ? pred_ub[i] : 1.0;
    }
    NNV_HIP_TRY(hipMemcpyAsync(s->plb, tmp.data(), sizeof(double) * 2 * npad, hipMemcpyHostToDevice, c->stream));
    c->h2d_bytes += (int64_t)sizeof(double) * 2 * npad;
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  auto base = std::make_shared<ConsNode>();
  base->p_total = p;
  base->n_total = n;
  if (p > 0 && n > 0) {
    base->ldc = round_up(p, kLdAlign);
    NNV_TRY(c->alloc(sizeof(double) * base->ldc * n, &base->C0));
    NNV_TRY(upload_matrix(c, C, p, n, base->ldc, base->C0->as<double>()));
  }
  if (p > 0) {
    NNV_TRY(c->alloc(sizeof(double) * p, &base->d0));
    NNV_HIP_TRY(hipMemcpyAsync(base->d0->ptr, d, sizeof(double) * p, hipMemcpyHostToDevice, c->stream));
    c->h2d_bytes += (int64_t)sizeof(double) * p;
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  s->cons = base;
  *out = guard.release();
  return NNVHIP_OK;
}

__global__ void box_fill_kernel(double* __restrict__ V, int64_t ld, int N, const double* __restrict__ center,
                                const double* __restrict__ vec, const int32_t* __restrict__ gen_dim,
                                const int64_t* __restrict__ col_off, const int64_t* __restrict__ gen_off) {
  // one block column per (set, column); rows across threads.  Column 0 is the centre; column
  // 1+g holds vec(dim_g) at row dim_g and zeros elsewhere (diag(vec) with empty columns removed).
  int set = blockIdx.z;
  int64_t ncols = col_off[set + 1] - col_off[set];
  for (int64_t j = blockIdx.y; j < ncols; j += gridDim.y) {
    double* col = V + (col_off[set] + j) * ld;
    int dim = j == 0 ? -1 : gen_dim[gen_off[set] + j - 1];
    // two rows per thread, one 16-byte store (ld is even and every column starts on a 16-byte boundary)
    for (int r = 2 * (blockIdx.x * blockDim.x + threadIdx.x); r < ld; r += 2 * gridDim.x * blockDim.x) {
      double v[2] = {0.0, 0.0};
#pragma unroll
      for (int e = 0; e < 2; ++e)
        if (r + e < N) {
          if (j == 0) v[e] = center[(int64_t)set * N + r + e];
          else if (r + e == dim) v[e] = vec[(int64_t)set * N + r + e];
        }
      *reinterpret_cast<double2*>(col + r) = make_double2(v[0], v[1]);
    }
  }
}

// info[2s] = offset of set s in the bounds buffer, info[2s+1] = its padded predicate count
__global__ void fill_pm_one_kernel(double* __restrict__ bounds, const int64_t* __restrict__ info) {
  const int64_t off = info[2 * blockIdx.y], n = info[2 * blockIdx.y + 1];
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i < n) {
    bounds[off + i] = -1.0;
    bounds[off + n + i] = 1.0;
  }
}

int nnvhip_star_from_box(nnvhip_ctx* c, int64_t N, int64_t count, const double* lb, const double* ub,
                         nnvhip_star** out) {
  CHECK_CTX(c);
  if (!lb || !ub || !out) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (N <= 0 || count <= 0 || count > 65535) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimensions between lb and ub");
  // Box constructor arithmetic on the host (set/Box.m:35-45): it decides the column count.
  std::vector<double> center(N * count), vec(N * count);
  std::vector<int32_t> gen_dim;
  std::vector<int64_t> col_off(count + 1, 0), gen_off(count + 1, 0);
  std::vector<char> neg_scale((size_t)count, 0);
  // Sets with the same half-widths, bit for bit (the boxes of a regular partition), share one scale vector and one
  // index list on the device: layers downstream recognise by the pointers that such sets gather the same scaled
  // weight columns.  shape_of[s] = the first set with set s's half-widths (among the first few distinct shapes).
  std::vector<int64_t> shape_of((size_t)count);
  std::vector<int64_t> shapes;
  std::vector<uint64_t> shape_hash;
  for (int64_t s = 0; s < count; ++s) {
    int64_t n = 0;
    uint64_t hash = 0x9E3779B97F4A7C15ull;  // of the half-widths' bit patterns: vectors are compared only when it matches
    for (int64_t i = 0; i < N; ++i) {
      double l = lb[s * N + i], u = ub[s * N + i];
      center[s * N + i] = 0.5 * (l + u);
      double v = 0.5 * (u - l);
      vec[s * N + i] = v;
      uint64_t bits;
      memcpy(&bits, &v, sizeof bits);
      hash = (hash ^ bits) * 0x100000001B3ull;
      hash ^= hash >> 29;
      if (v < 0.0) neg_scale[s] = 1;
      // zero columns are deleted only when the generator matrix has more than one element
      if (v != 0.0 || N == 1) {
        gen_dim.push_back((int32_t)i);
        ++n;
      }
    }
    gen_off[s + 1] = gen_off[s] + n;
    col_off[s + 1] = col_off[s] + n + 1;
    shape_of[s] = s;
    for (size_t k = 0; k < shapes.size(); ++k)
      if (shape_hash[k] == hash && memcmp(&vec[shapes[k] * N], &vec[s * N], sizeof(double) * N) == 0) {
        shape_of[s] = shapes[k];
        break;
      }
    if (shape_of[s] == s && shapes.size() < 16) {
      shapes.push_back(s);
      shape_hash.push_back(hash);
    }
  }
  int64_t ld = round_up(N, kLdAlign);
  int64_t total_cols = col_off[count];
  BufRef arena, dcenter, dvec, dgen, dcol, dgoff;
  NNV_TRY(c->alloc(sizeof(double) * ld * total_cols, &arena));
  NNV_TRY(c->upload(center.data(), sizeof(double) * center.size(), &dcenter));
  NNV_TRY(c->upload(vec.data(), sizeof(double) * vec.size(), &dvec));
  if (gen_dim.empty()) gen_dim.push_back(0);
  NNV_TRY(c->upload(gen_dim.data(), sizeof(int32_t) * gen_dim.size(), &dgen));
  NNV_TRY(c->upload(col_off.data(), sizeof(int64_t) * col_off.size(), &dcol));
  NNV_TRY(c->upload(gen_off.data(), sizeof(int64_t) * gen_off.size(), &dgoff));
  int64_t max_cols = 0;
  for (int64_t s = 0; s < count; ++s) max_cols = std::max(max_cols, col_off[s + 1] - col_off[s]);
  dim3 grid((unsigned)std::min<int64_t>(ceil_div(ld, 512), 64), (unsigned)std::min<int64_t>(max_cols, 4096),
            (unsigned)count);
  hipLaunchKernelGGL(box_fill_kernel, grid, dim3(256), 0, c->stream, arena->as<double>(), ld, (int)N,
                     dcenter->as<double>(), dvec->as<double>(), dgen->as<int32_t>(), dcol->as<int64_t>(),
                     dgoff->as<int64_t>());
  NNV_HIP_TRY(hipGetLastError());
  // predicate bounds -1/+1 for all sets in one buffer
  int64_t npad_total = 0;
  std::vector<int64_t> poff(count);
  for (int64_t s = 0; s < count; ++s) {
    poff[s] = npad_total;
    npad_total += 2 * round_up(std::max<int64_t>(gen_off[s + 1] - gen_off[s], 1), kLdAlign);
  }
  BufRef pb;
  NNV_TRY(c->alloc(sizeof(double) * npad_total, &pb));
  for (int64_t s = 0; s < count; ++s) {
    nnvhip_star* st = new_star(c);
    st->N = N;
    st->n = gen_off[s + 1] - gen_off[s];
    st->ld = ld;
    st->Vbuf = arena;
    st->V = arena->as<double>() + col_off[s] * ld;
    st->pbuf = pb;
    int64_t npad = round_up(std::max<int64_t>(st->n, 1), kLdAlign);
    st->plb = pb->as<double>() + poff[shape_of[s]];  // (the same -1 / +1 for every set of the shape)
    st->pub = st->plb + npad;
    // C = zeros(1, n), d = 0 (set/Star.m:226-227): a base node with one all-zero row
    auto base = std::make_shared<ConsNode>();
    base->p_total = 1;
    base->n_total = st->n;
    st->cons = base;  // C0/d0 left null = all zeros
    st->has_zono = true;  // Z = Zono(center, gens), set/Star.m:230-236
    if (st->n > 0) {  // every generator column is vec(dim) * e_dim
      st->oh_from = 1;
      st->oh_idx_buf = dgen;
      st->oh_idx = dgen->as<int32_t>() + gen_off[shape_of[s]];
      st->oh_scale_buf = dvec;
      st->oh_scale = dvec->as<double>() + shape_of[s] * N;
      st->oh_scale_neg = neg_scale[s] != 0;
    }
    out[s] = st;
  }
  // one launch fills every set's bounds: lb half gets -1, ub half +1
  {
    std::vector<int64_t> pinfo((size_t)(2 * count));
    int64_t max_npad = 0;
    for (int64_t s = 0; s < count; ++s) {
      pinfo[2 * s] = poff[s];
      pinfo[2 * s + 1] = round_up(std::max<int64_t>(out[s]->n, 1), kLdAlign);
      max_npad = std::max(max_npad, pinfo[2 * s + 1]);
    }
    BufRef dinfo;
    NNV_TRY(c->upload(pinfo.data(), sizeof(int64_t) * pinfo.size(), &dinfo));
    hipLaunchKernelGGL(fill_pm_one_kernel, dim3((unsigned)ceil_div(max_npad, 256), (unsigned)count), dim3(256), 0, c->stream,
                       pb->as<double>(), dinfo->as<int64_t>());
  }
  NNV_HIP_TRY(hipGetLastError());
  return NNVHIP_OK;
}

// Columns of the set the reduceMem suffix of the ReLU layer builds: column 0 the centre, column 1 + g the value
// val[g] on every channel of pixel pix[g] (rows pix[g] + k * HW), every other entry zero.
__global__ void rebox_fill_kernel(double* __restrict__ V, int64_t ld, int N, int HW, int64_t ncols, int ngen,
                                  const double* __restrict__ center, const int32_t* __restrict__ pix,
                                  const double* __restrict__ val) {
  for (int64_t j = blockIdx.y; j < ncols; j += gridDim.y) {
    double* col = V + j * ld;
    const int p = (j >= 1 && j - 1 < ngen) ? pix[j - 1] : -1;
    const double pv = p >= 0 ? val[j - 1] : 0.0;
    for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < ld; r += gridDim.x * blockDim.x) {
      double v = 0.0;
      if (r < N) {
        if (j == 0) v = center[r];
        else if (p >= 0 && r % HW == p) v = pv;
      }
      col[r] = v;
    }
  }
}

int nnvhip_relu_reduce_mem(nnvhip_ctx* c, nnvhip_star* in, int64_t H, int64_t W, int64_t C, nnvhip_star** out, double* im_lb,
                           double* im_ub) {
  CHECK_CTX(c);
  if (!in || in->ctx != c || !out) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle");
  if (H <= 0 || W <= 0 || C <= 0 || H * W * C != in->N)
    NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension in the ImageStar and the original Star set");
  const int64_t N = in->N, HW = H * W;
  // [l, u] = images(i).estimateRanges
  NNV_TRY(compute_ranges(c, 1, &in));
  std::vector<double> l((size_t)N), u((size_t)N);
  NNV_HIP_TRY(hipMemcpyAsync(l.data(), in->lb, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipMemcpyAsync(u.data(), in->ub, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  // center = 0.5*(u+l); v = 0.5*(u-l); n = numel(find(l-u)); one generator per pixel (i1 outer, i2 inner) whose
  // first-channel half-width is non-zero
  std::vector<double> center((size_t)N), val;
  std::vector<int32_t> pix;
  int64_t n = 0;
  for (int64_t i = 0; i < N; ++i) {
    center[i] = 0.5 * (u[i] + l[i]);
    if (l[i] - u[i] != 0.0) ++n;
  }
  for (int64_t i1 = 0; i1 < H; ++i1)
    for (int64_t i2 = 0; i2 < W; ++i2) {
      const double bv = 0.5 * (u[i1 + i2 * H] - l[i1 + i2 * H]);
      if (bv != 0.0) {
        pix.push_back((int32_t)(i1 + i2 * H));
        val.push_back(bv);
      }
    }
  if ((int64_t)pix.size() > n) NNV_FAIL(NNVHIP_ERR_SHAPE, "Index exceeds the number of array elements");  // (cannot happen: C >= 1)
  nnvhip_star* s = new_star(c);
  std::unique_ptr<nnvhip_star, int (*)(nnvhip_star*)> guard(s, nnvhip_star_release);
  s->N = N;
  s->n = n;
  s->ld = round_up(N, kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * s->ld * (n + 1), &s->Vbuf));
  s->V = s->Vbuf->as<double>();
  BufRef dcen, dpix, dval;
  NNV_TRY(c->upload(center.data(), sizeof(double) * N, &dcen));
  const int ngen = (int)pix.size();
  if (pix.empty()) {  // (something to upload)
    pix.push_back(0);
    val.push_back(0.0);
  }
  NNV_TRY(c->upload(pix.data(), sizeof(int32_t) * pix.size(), &dpix));
  NNV_TRY(c->upload(val.data(), sizeof(double) * val.size(), &dval));
  dim3 grid((unsigned)std::min<int64_t>(ceil_div(s->ld, 256), 64), (unsigned)std::min<int64_t>(n + 1, 4096));
  hipLaunchKernelGGL(rebox_fill_kernel, grid, dim3(256), 0, c->stream, s->V, s->ld, (int)N, (int)HW, n + 1, ngen,
                     dcen->as<double>(), dpix->as<int32_t>(), dval->as<double>());
  NNV_HIP_TRY(hipGetLastError());
  // predicate bounds -1 / +1; C = zeros(1, n), d = 0
  const int64_t npad = round_up(std::max<int64_t>(n, 1), kLdAlign);
  NNV_TRY(c->alloc(sizeof(double) * 2 * npad, &s->pbuf));
  s->plb = s->pbuf->as<double>();
  s->pub = s->plb + npad;
  {
    const int64_t pinfo[2] = {0, npad};
    BufRef dinfo;
    NNV_TRY(c->upload(pinfo, sizeof(pinfo), &dinfo));
    hipLaunchKernelGGL(fill_pm_one_kernel, dim3((unsigned)ceil_div(npad, 256), 1), dim3(256), 0, c->stream, s->plb, dinfo->as<int64_t>());
    NNV_HIP_TRY(hipGetLastError());
  }
  auto base = std::make_shared<ConsNode>();
  base->p_total = 1;
  base->n_total = n;
  s->cons = base;
  if (C == 1 && ngen == n && n > 0) {  // a plain box star: every generator is val * e_pix
    std::vector<double> scale((size_t)N, 0.0);
    bool neg = false;
    for (size_t g = 0; g < (size_t)ngen; ++g) {
      scale[pix[g]] = val[g];
      neg = neg || val[g] < 0.0;
    }
    BufRef dscale;
    NNV_TRY(c->upload(scale.data(), sizeof(double) * N, &dscale));
    s->oh_from = 1;
    s->oh_idx_buf = dpix;
    s->oh_idx = dpix->as<int32_t>();
    s->oh_scale_buf = dscale;
    s->oh_scale = dscale->as<double>();
    s->oh_scale_neg = neg;
  }
  if (im_lb) memcpy(im_lb, l.data(), sizeof(double) * N);
  if (im_ub) memcpy(im_ub, u.data(), sizeof(double) * N);
  *out = guard.release();
  return NNVHIP_OK;
}

int nnvhip_star_retain(nnvhip_star* s) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  s->refs.fetch_add(1);
  return NNVHIP_OK;
}

int nnvhip_star_release(nnvhip_star* s) {
  if (!s) return NNVHIP_OK;
  if (s->refs.fetch_sub(1) == 1) {
    nnvhip_ctx* c = s->ctx;
    delete s;
    c->live_handles--;
  }
  return NNVHIP_OK;
}

int nnvhip_star_release_array(int64_t count, nnvhip_star* const* sets) {
  if (count < 0 || (count > 0 && !sets)) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  // a large array is let go later, where the host waits for the device anyway (nnvhip_ctx::deferred)
  const bool later = count >= 256;
  for (int64_t i = 0; i < count; ++i) {
    if (later && sets[i] != nullptr)
      sets[i]->ctx->deferred.push_back(sets[i]);
    else
      nnvhip_star_release(sets[i]);
  }
  return NNVHIP_OK;
}

int nnvhip_star_dims(const nnvhip_star* s, int64_t* N, int64_t* n, int64_t* p) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  if (N) *N = s->N;
  if (n) *n = s->n;
  if (p) *p = s->cons ? s->cons->p_total : 0;
  return NNVHIP_OK;
}

int nnvhip_star_has_zono(const nnvhip_star* s, int32_t* flag) {
  if (!s || !flag) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  *flag = s->has_zono ? 1 : 0;
  return NNVHIP_OK;
}

int nnvhip_star_has_user_constraints(const nnvhip_star* s, int32_t* flag) {
  if (!s || !flag) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  const ConsNode* nd = s->cons.get();
  while (nd && nd->prev) nd = nd->prev.get();
  *flag = (nd && nd->C0) ? 1 : 0;  // the base node holds dense rows only when a caller handed some in
  return NNVHIP_OK;
}

int nnvhip_star_fetch_V(const nnvhip_star* s, double* V) {
  if (!s || !V) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  nnvhip_ctx* c = s->ctx;
  NNV_TRY(nnvhip::enter_ctx(c));
  NNV_TRY(ensure_dense(c, const_cast<nnvhip_star*>(s)));  // implicit columns are written out on first read
  NNV_HIP_TRY(hipMemcpy2DAsync(V, sizeof(double) * s->N, s->V, sizeof(double) * s->ld, sizeof(double) * s->N,
                               s->n + 1, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_star_fetch_rows(const nnvhip_star* s, int64_t R, const int32_t* rows, double* out) {
  if (!s || (R > 0 && (!rows || !out)) || R < 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (R == 0) return NNVHIP_OK;
  nnvhip_ctx* c = s->ctx;
  for (int64_t t = 0; t < R; ++t)
    if (rows[t] < 0 || rows[t] >= s->N) NNV_FAIL(NNVHIP_ERR_ARG, "Invalid index");
  NNV_TRY(nnvhip::enter_ctx(c));
  NNV_TRY(ensure_dense(c, const_cast<nnvhip_star*>(s)));
  // gather on the device into an Rp x (n+1) matrix (Rp = R rounded up to whole K-tiles, the packing
  // kernel's granularity), one contiguous copy, then drop the padding rows on the host
  const int64_t Rp = round_up(R, kLdAlign), nc = s->n + 1;
  std::vector<int32_t> list((size_t)Rp, -1);
  std::copy(rows, rows + R, list.begin());
  BufRef dlist, packed;
  NNV_TRY(c->upload(list.data(), sizeof(int32_t) * Rp, &dlist));
  NNV_TRY(c->alloc(sizeof(double) * Rp * nc, &packed));
  PackSet ps{s->V, dlist->as<int32_t>(), packed->as<double>(), s->ld, (int32_t)Rp, (int32_t)nc};
  NNV_TRY(launch_pack_rows(c, 1, &ps));
  std::vector<double> tmp((size_t)(Rp * nc));
  NNV_HIP_TRY(hipMemcpyAsync(tmp.data(), packed->ptr, sizeof(double) * Rp * nc, hipMemcpyDeviceToHost, c->stream));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  for (int64_t j = 0; j < nc; ++j) memcpy(out + j * R, tmp.data() + j * Rp, sizeof(double) * R);
  return NNVHIP_OK;
}

int nnvhip_star_fetch_pred_bounds(const nnvhip_star* s, double* lb, double* ub) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  nnvhip_ctx* c = s->ctx;
  NNV_TRY(nnvhip::enter_ctx(c));
  if (s->n > 0) {
    if (lb) NNV_HIP_TRY(hipMemcpyAsync(lb, s->plb, sizeof(double) * s->n, hipMemcpyDeviceToHost, c->stream));
    if (ub) NNV_HIP_TRY(hipMemcpyAsync(ub, s->pub, sizeof(double) * s->n, hipMemcpyDeviceToHost, c->stream));
  }
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_star_fetch_constraints(const nnvhip_star* s, double* C, double* d) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  NNV_TRY(nnvhip::enter_ctx(s->ctx));
  return materialize_constraints(s, C, d);
}

int nnvhip_star_relu_counts(const nnvhip_star* s, int64_t* n_inactive, int64_t* n_crossing) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  if (s->n_crossing < 0) NNV_FAIL(NNVHIP_ERR_ARG, "set was not produced by the ReLU step");
  if (n_inactive) *n_inactive = s->n_inactive;
  if (n_crossing) *n_crossing = s->n_crossing;
  return NNVHIP_OK;
}

int nnvhip_star_fetch_crossing(const nnvhip_star* s, int32_t* index, double* lb, double* ub) {
  if (!s) NNV_FAIL(NNVHIP_ERR_ARG, "null set handle");
  if (s->n_crossing < 0) NNV_FAIL(NNVHIP_ERR_ARG, "set was not produced by the ReLU step");
  nnvhip_ctx* c = s->ctx;
  NNV_TRY(nnvhip::enter_ctx(c));
  const ConsNode* node = s->cons.get();
  int64_t m = s->n_crossing;
  if (m > 0) {
    if (index) NNV_HIP_TRY(hipMemcpyAsync(index, node->index->as<int32_t>() + node->index_off, sizeof(int32_t) * m, hipMemcpyDeviceToHost, c->stream));
    const double* lbub = node->lbub->as<double>() + node->lbub_off;
    if (lb) NNV_HIP_TRY(hipMemcpyAsync(lb, lbub, sizeof(double) * m, hipMemcpyDeviceToHost, c->stream));
    if (ub) NNV_HIP_TRY(hipMemcpyAsync(ub, lbub + node->ld_lbub, sizeof(double) * m, hipMemcpyDeviceToHost, c->stream));
  }
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  return NNVHIP_OK;
}

int nnvhip_estimate_ranges(nnvhip_ctx* c, nnvhip_star* s, double* lb, double* ub) {
  return nnvhip_estimate_ranges_batch(c, 1, &s, lb, ub);
}

int nnvhip_estimate_ranges_static(nnvhip_ctx* c, const nnvhip_star* s, double* lb_dev, double* ub_dev) {
  CHECK_CTX(c);
  if (!s || s->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle");
  if (!lb_dev && !ub_dev) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  return ranges_into_static(c, s, lb_dev, ub_dev);
}

int nnvhip_estimate_ranges_batch(nnvhip_ctx* c, int64_t count, nnvhip_star* const* s, double* lb, double* ub) {
  CHECK_CTX(c);
  if (!s || count <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  for (int64_t i = 0; i < count; ++i) {
    if (!s[i] || s[i]->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle %lld", (long long)i);
    if (s[i]->N != s[0]->N) NNV_FAIL(NNVHIP_ERR_SHAPE, "sets of one array must have the same dimension");
  }
  NNV_TRY(c->begin_op());
  NNV_TRY(compute_ranges(c, count, s));
  NNV_TRY(c->end_op());
  if (lb || ub) {
    int64_t N = s[0]->N;
    // ranges computed by one call sit at a fixed stride in one buffer
    const int64_t stride = count > 1 ? s[1]->lb - s[0]->lb : 0;
    bool regular = count > 1 && stride >= N;
    for (int64_t i = 1; i < count && regular; ++i)
      regular = s[i]->rbuf == s[0]->rbuf && s[i]->lb == s[0]->lb + i * stride && s[i]->ub == s[0]->ub + i * stride;
    if (regular && stride <= 4 * N + 64) {
      // one contiguous copy of the whole range buffer, unpacked on the host (strided 2-D copies of
      // short rows are issued row by row by the runtime)
      const int64_t off_ub = s[0]->ub - s[0]->lb;
      std::vector<double> tmp((size_t)(stride * (count - 1) + std::max<int64_t>(N, off_ub + N)));
      NNV_HIP_TRY(hipMemcpyAsync(tmp.data(), s[0]->lb, sizeof(double) * tmp.size(), hipMemcpyDeviceToHost, c->stream));
      NNV_HIP_TRY(hipStreamSynchronize(c->stream));
      for (int64_t i = 0; i < count; ++i) {
        if (lb) std::copy(tmp.begin() + i * stride, tmp.begin() + i * stride + N, lb + i * N);
        if (ub) std::copy(tmp.begin() + i * stride + off_ub, tmp.begin() + i * stride + off_ub + N, ub + i * N);
      }
      return NNVHIP_OK;
    } else {
      for (int64_t i = 0; i < count; ++i) {
        if (lb) NNV_HIP_TRY(hipMemcpyAsync(lb + i * N, s[i]->lb, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
        if (ub) NNV_HIP_TRY(hipMemcpyAsync(ub + i * N, s[i]->ub, sizeof(double) * N, hipMemcpyDeviceToHost, c->stream));
      }
    }
    NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  return NNVHIP_OK;
}

/* ------------------------------------------------------------------------------------------ */
/* layers                                                                                      */
/* ------------------------------------------------------------------------------------------ */

int nnvhip_fc_create(nnvhip_ctx* c, const double* W, const double* b, int64_t M, int64_t K, nnvhip_fc** out) {
  CHECK_CTX(c);
  if (!W || !out) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (M <= 0 || K <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension between the weight matrix and bias vector");
  // the same arrays again (a layer object rebuilt around them, Star.affineMap called once more): the resident copy
  WeightKey key;
  key.kind = 0;
  key.geo[0] = M;
  key.geo[1] = K;
  key.geo[2] = b ? 1 : 0;
  hash_bytes(W, sizeof(double) * M * K, &key.h0, &key.h1);
  if (b) {
    uint64_t b0 = 0, b1 = 0;
    hash_bytes(b, sizeof(double) * M, &b0, &b1);
    key.geo[3] = (int64_t)b0;
    key.geo[4] = (int64_t)b1;
  }
  if (c->weight_cache_budget > 0) {
    if (void* hit = weight_cache_find(c, &key, W, (size_t)(M * K), b, b ? (size_t)M : 0)) {
      nnvhip_fc* f = static_cast<nnvhip_fc*>(hit);
      f->refs.fetch_add(1);
      c->live_handles++;
      *out = f;
      return NNVHIP_OK;
    }
  }
  std::unique_ptr<nnvhip_fc> fc(new nnvhip_fc());
  fc->ctx = c;
  fc->M = M;
  fc->K = K;
  fc->Mp = round_up(M, kLdAlign);
  fc->Kp = round_up(K, kLdAlign);
  // (128 doubles of slack: the tile kernel of gemm_seg.hip reads whole 128-row pieces of a column)
  NNV_TRY(c->alloc(sizeof(double) * (fc->Mp * fc->Kp + 128), &fc->W));
  NNV_HIP_TRY(hipMemsetAsync(fc->W->ptr, 0, sizeof(double) * fc->Mp * fc->Kp, c->stream));
  NNV_HIP_TRY(hipMemcpy2DAsync(fc->W->ptr, sizeof(double) * fc->Mp, W, sizeof(double) * M, sizeof(double) * M, K,
                               hipMemcpyHostToDevice, c->stream));
  if (b) {
    NNV_TRY(c->alloc(sizeof(double) * fc->Mp, &fc->bias));
    NNV_HIP_TRY(hipMemsetAsync(fc->bias->ptr, 0, sizeof(double) * fc->Mp, c->stream));
    NNV_HIP_TRY(hipMemcpyAsync(fc->bias->ptr, b, sizeof(double) * M, hipMemcpyHostToDevice, c->stream));
  }
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  const int64_t wbytes = (int64_t)sizeof(double) * (M * K + (b ? M : 0));
  c->weight_uploads++;
  c->weight_upload_bytes += wbytes;
  c->h2d_bytes += wbytes;
  c->live_handles++;
  *out = fc.release();
  if (c->weight_cache_budget > 0) {
    (*out)->refs.fetch_add(1);  // the cache's reference
    WeightEntry e;
    e.handle = *out;
    e.bytes = (int64_t)sizeof(double) * (*out)->Mp * ((*out)->Kp + 1);
    e.last_use = ++c->weight_clock;
    e.host_w.assign(W, W + M * K);
    if (b) e.host_b.assign(b, b + M);
    c->weight_cache[key] = std::move(e);
    c->weight_cache_bytes += e.bytes;
    c->drop_weight_cache(false);
  }
  return NNVHIP_OK;
}

int nnvhip_fc_destroy(nnvhip_fc* fc) {
  if (!fc) return NNVHIP_OK;
  nnvhip_ctx* c = fc->ctx;
  if (fc->refs.fetch_sub(1) == 1) delete fc;
  c->live_handles--;
  return NNVHIP_OK;
}

int nnvhip_conv2d_create(nnvhip_ctx* c, const double* W, const double* bias, int64_t FH, int64_t FW, int64_t Cin,
                         int64_t Cout, const int64_t padding[4], const int64_t stride[2], const int64_t dilation[2],
                         nnvhip_conv2d** out) {
  CHECK_CTX(c);
  if (!W || !out || !padding || !stride || !dilation) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  if (FH <= 0 || FW <= 0 || Cin <= 0 || Cout <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid weights array");
  for (int i = 0; i < 4; ++i)
    if (padding[i] < 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid padding matrix");
  if (stride[0] <= 0 || stride[1] <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid stride matrix");
  if (dilation[0] <= 0 || dilation[1] <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Invalid dilation matrix");
  WeightKey key;
  key.kind = 1;
  key.geo[0] = FH;
  key.geo[1] = FW;
  key.geo[2] = Cin;
  key.geo[3] = Cout;
  for (int i = 0; i < 4; ++i) key.geo[4 + i] = padding[i];
  key.geo[8] = stride[0] | (stride[1] << 20) | (dilation[0] << 40) | ((int64_t)(bias ? 1 : 0) << 62);
  key.geo[9] = dilation[1];
  hash_bytes(W, sizeof(double) * FH * FW * Cin * Cout, &key.h0, &key.h1);
  if (bias) {
    uint64_t b0 = 0, b1 = 0;
    hash_bytes(bias, sizeof(double) * Cout, &b0, &b1);
    key.geo[10] = (int64_t)b0;
    key.geo[11] = (int64_t)b1;
  }
  if (c->weight_cache_budget > 0) {
    if (void* hit = weight_cache_find(c, &key, W, (size_t)(FH * FW * Cin * Cout), bias, bias ? (size_t)Cout : 0)) {
      nnvhip_conv2d* v = static_cast<nnvhip_conv2d*>(hit);
      v->refs.fetch_add(1);
      c->live_handles++;
      *out = v;
      return NNVHIP_OK;
    }
  }
  std::unique_ptr<nnvhip_conv2d> cv(new nnvhip_conv2d());
  cv->ctx = c;
  cv->FH = FH;
  cv->FW = FW;
  cv->Cin = Cin;
  cv->Cout = Cout;
  for (int i = 0; i < 4; ++i) cv->pad[i] = padding[i];
  for (int i = 0; i < 2; ++i) {
    cv->stride[i] = stride[i];
    cv->dil[i] = dilation[i];
  }
  cv->K = FH * FW * Cin;
  cv->Kp = round_up(cv->K, kLdAlign);
  // MATLAB's FH x FW x Cin x Cout array is a (FH*FW*Cin) x Cout column-major matrix already
  NNV_TRY(c->alloc(sizeof(double) * cv->Kp * Cout, &cv->W));
  NNV_HIP_TRY(hipMemsetAsync(cv->W->ptr, 0, sizeof(double) * cv->Kp * Cout, c->stream));
  NNV_HIP_TRY(hipMemcpy2DAsync(cv->W->ptr, sizeof(double) * cv->Kp, W, sizeof(double) * cv->K, sizeof(double) * cv->K,
                               Cout, hipMemcpyHostToDevice, c->stream));
  if (bias) {
    NNV_TRY(c->alloc(sizeof(double) * Cout, &cv->bias));
    NNV_HIP_TRY(hipMemcpyAsync(cv->bias->ptr, bias, sizeof(double) * Cout, hipMemcpyHostToDevice, c->stream));
  }
  NNV_TRY(conv2d_prepare_weights(c, cv.get()));
  NNV_HIP_TRY(hipStreamSynchronize(c->stream));
  const int64_t wbytes = (int64_t)sizeof(double) * (cv->K * Cout + (bias ? Cout : 0));
  c->weight_uploads++;
  c->weight_upload_bytes += wbytes;
  c->h2d_bytes += wbytes;
  c->live_handles++;
  *out = cv.release();
  if (c->weight_cache_budget > 0) {
    (*out)->refs.fetch_add(1);  // the cache's reference
    WeightEntry e;
    e.handle = *out;
    e.bytes = (int64_t)sizeof(double) * (((*out)->Kp + 1) * Cout + ((*out)->Wk ? (*out)->Kp * (*out)->coutp : 0));
    e.last_use = ++c->weight_clock;
    e.host_w.assign(W, W + FH * FW * Cin * Cout);
    if (bias) e.host_b.assign(bias, bias + Cout);
    c->weight_cache[key] = std::move(e);
    c->weight_cache_bytes += e.bytes;
    c->drop_weight_cache(false);
  }
  return NNVHIP_OK;
}

int nnvhip_conv2d_destroy(nnvhip_conv2d* cv) {
  if (!cv) return NNVHIP_OK;
  nnvhip_ctx* c = cv->ctx;
  if (cv->refs.fetch_sub(1) == 1) delete cv;
  c->live_handles--;
  return NNVHIP_OK;
}

int nnvhip_conv2d_output_size(const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t* Ho, int64_t* Wo) {
  if (!cv) NNV_FAIL(NNVHIP_ERR_ARG, "null layer handle");
  // floor((H + t + b - (FH-1)*dh - 1)/sh + 1), nn/layers/Conv2DLayer.m:1134-1135
  int64_t eh = H + cv->pad[0] + cv->pad[1] - (cv->FH - 1) * cv->dil[0] - 1;
  int64_t ew = W + cv->pad[2] + cv->pad[3] - (cv->FW - 1) * cv->dil[1] - 1;
  if (eh < 0 || ew < 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "filter does not fit the padded input");
  if (Ho) *Ho = eh / cv->stride[0] + 1;
  if (Wo) *Wo = ew / cv->stride[1] + 1;
  return NNVHIP_OK;
}

}  // extern "C"

// Shared set-up of the affine layers: validates the input array, allocates one output arena with
// the sets back to back, and creates output handles that share constraints and predicate bounds
// with their inputs.
int nnvhip::make_affine_outputs(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, int64_t Nout,
                                std::vector<nnvhip_star*>* outs, bool* contiguous, int64_t* total_cols) {
  int64_t ldout = round_up(Nout, kLdAlign);
  int64_t cols = 0;
  bool contig = true;
  for (int64_t i = 0; i < count; ++i) {
    if (i > 0 && (in[i]->ld != in[0]->ld || in[i]->V != in[i - 1]->V + in[i - 1]->stored_cols() * in[i - 1]->ld)) contig = false;
    cols += in[i]->n + 1;
  }
  BufRef arena;
  NNV_TRY(c->alloc(sizeof(double) * ldout * cols, &arena));
  int64_t off = 0;
  for (int64_t i = 0; i < count; ++i) {
    nnvhip_star* o = new_star(c);
    o->N = Nout;
    o->n = in[i]->n;
    o->ld = ldout;
    o->Vbuf = arena;
    o->V = arena->as<double>() + off * ldout;
    o->pbuf = in[i]->pbuf;
    o->plb = in[i]->plb;
    o->pub = in[i]->pub;
    o->cons = in[i]->cons;
    off += in[i]->n + 1;
    outs->push_back(o);
  }
  *contiguous = contig;
  *total_cols = cols;
  return NNVHIP_OK;
}

void nnvhip::release_all(std::vector<nnvhip_star*>& v) {
  for (auto* s : v) nnvhip_star_release(s);
  v.clear();
}

int nnvhip::check_set_array(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, nnvhip_star** out) {
  if (!in || !out || count <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  for (int64_t i = 0; i < count; ++i)
    if (!in[i] || in[i]->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle %lld", (long long)i);
  return NNVHIP_OK;
}

extern "C" {

int nnvhip_affine_fc(nnvhip_ctx* c, const nnvhip_fc* fc, int64_t count, nnvhip_star* const* in, nnvhip_star** out) {
  CHECK_CTX(c);
  if (!fc || fc->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid layer handle");
  NNV_TRY(check_set_array(c, count, in, out));
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N != fc->K)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistency between the affine mapping matrix and dimension of the star set");
  std::vector<nnvhip_star*> outs;
  bool contig = false;
  int64_t cols = 0;
  NNV_TRY(c->begin_op());
  // A large array whose gathered columns will stay unwritten gets their range sums from one matrix product
  // (see below).  Nothing of it depends on the outputs, so it is queued before anything else: the device
  // works on it while the host sets up the outputs and the tiles of the contraction.
  BufRef mm_early;
  std::vector<int64_t> mm_slot;  // which pair of the product's columns holds a set's sums
  int st = NNVHIP_OK;
  if (count >= 64 && !c->eager_cols && !c->dense_affine) {
    std::vector<GatherSet> es((size_t)count);
    bool ok = true, any = false;
    for (int64_t i = 0; i < count; ++i) {
      const int64_t nc = in[i]->n + 1;
      int64_t d = (in[i]->oh_from > 0 && in[i]->oh_from < nc) ? in[i]->oh_from : nc;
      if ((double)fc->Mp * (double)fc->Kp * (double)(nc - d) * (double)count < 4.0e6) d = nc;
      GatherSet& g = es[i];
      g = GatherSet{};
      g.idx = in[i]->oh_idx;
      g.scale = in[i]->oh_scale;
      g.plb = in[i]->plb + (d - 1);  // the output shares the input's predicate bounds
      g.pub = in[i]->pub + (d - 1);
      g.m = (int32_t)(nc - d);
      ok = ok && !(g.m > 0 && in[i]->oh_scale_neg);
      any = any || g.m > 0;
    }
    if (ok && any) st = launch_range_sums_mm(c, fc, count, es.data(), &mm_early, &mm_slot);
  }
  if (st == NNVHIP_OK) st = make_affine_outputs(c, count, in, fc->M, &outs, &contig, &cols);
  if (st == NNVHIP_OK) {
    for (int64_t i = 0; i < count; ++i) outs[i]->has_zono = in[i]->has_zono;  // Z.affineMap(W, b), set/Star.m:332-340
    const double* bias = fc->bias ? fc->bias->as<double>() : nullptr;
    const double* Wd = fc->W->as<double>();
    // Columns of V that are scaled unit vectors (all generators of a box star, the columns a ReLU
    // appended) need no contraction: W * (s * e_r) = s * W(:, r).  dense[i] = leading columns that do.
    const bool dense_only = c->dense_affine;
    std::vector<int64_t> dense((size_t)count);
    std::vector<GatherSet> gs((size_t)count);
    int64_t total_dense = 0;
    bool any_onehot = false;
    for (int64_t i = 0; i < count; ++i) {
      const int64_t nc = in[i]->n + 1;
      dense[i] = (!dense_only && in[i]->oh_from > 0 && in[i]->oh_from < nc) ? in[i]->oh_from : nc;
      // tiny products are launch bound: one dense launch beats GEMM + gather
      if ((double)fc->Mp * (double)fc->Kp * (double)(nc - dense[i]) * (double)count < 4.0e6) dense[i] = nc;
      total_dense += dense[i];
      any_onehot = any_onehot || dense[i] < nc;
      GatherSet& g = gs[i];
      g.idx = in[i]->oh_idx;
      g.scale = in[i]->oh_scale;
      g.out = outs[i]->V + dense[i] * outs[i]->ld;
      g.plb = outs[i]->plb + (dense[i] - 1);
      g.pub = outs[i]->pub + (dense[i] - 1);
      g.part = nullptr;
      g.m = (int32_t)(nc - dense[i]);
      g.nfill = 0;
      g.fill = nullptr;
      g.bias = nullptr;
      g.red = nullptr;
      g.red_k = 0;
      g.lazy = 0;
      g.cin = nullptr;
      g.cpart = nullptr;
      g.centre = nullptr;
    }
    // One set whose gathered columns can stay unwritten and are either all the generators of a box star or the
    // columns a ReLU step appended (with that step's per-row classes still on the handle): the output's lb / ub
    // come from launch_fc_rowsum: one kernel over the weights instead of a gather pass plus a reduction.
    const bool lazy_ok = !c->eager_cols && !dense_only;
    const bool box_in = count == 1 && in[0]->oh_from == 1 && in[0]->oh_scale != nullptr && !in[0]->oh_scale_neg && dense[0] == 1 &&
                        gs[0].m > 0;
    const bool relu_in = count == 1 && in[0]->oh_from > 1 && in[0]->oh_scale == nullptr && gs[0].m > 0 && dense[0] == in[0]->oh_from &&
                         in[0]->rows_pending && in[0]->cls != nullptr && in[0]->pre_ub != nullptr;
    // (skinny layers keep the gather pass: a handful of 16-row blocks would not cover the chip)
    bool rowsum = (box_in || relu_in) && fc->Mp >= 128 && fc->K < (int64_t(1) << 31);
    // sets whose implicit unit-vector columns take part in the contraction after all get them written out
    // (which also runs a pending row reset)
    std::vector<nnvhip_star*> full;
    for (int64_t i = 0; i < count; ++i)
      if (dense[i] > in[i]->stored_cols() || (dense_only && (in[i]->rows_pending || in[i]->cs.any_pending()))) full.push_back(in[i]);
    if (!full.empty()) {
      st = ensure_dense_batch(c, (int64_t)full.size(), full.data());
      contig = true;  // the sets moved: look again
      for (int64_t i = 1; i < count; ++i)
        if (in[i]->ld != in[0]->ld || in[i]->V != in[i - 1]->V + in[i - 1]->stored_cols() * in[i - 1]->ld) contig = false;
    }
    // Rows of the dense columns that the ReLU step reset to zero need no contraction either: the
    // GEMM then runs over the kept rows only (used when that at least halves K).
    // *pack: gather the listed rows into a matrix of their own first (several row tiles of W would each
    // gather them otherwise; and a long list read through the map is slow, so a set that only takes this
    // route because its reset is pending always packs)
    auto rows_of = [&](int64_t i, GemmRows* r, int64_t* kp, bool* pack) {
      *kp = fc->Kp;
      *pack = fc->Mp > 128;
      // a set whose row reset is still pending shares its matrix with the ReLU's input: only the listed
      // rows may be read
      const bool must = in[i]->rows_pending;
      if (!must && (dense_only || in[i]->n_kept < 0 || in[i]->kept_idx == nullptr)) return false;
      // the kept-row list describes the columns before the one-hot block only (a one-hot column has its
      // 1 in a reset row): usable only if that block is not part of the contraction
      if (in[i]->oh_from > 0 && dense[i] > in[i]->oh_from) return false;
      const bool tiny = (double)fc->Mp * (double)fc->Kp * (double)dense[i] * (double)count < 4.0e6;
      if (!must && tiny) return false;
      const int64_t k = std::max<int64_t>(round_up(in[i]->n_kept, kLdAlign), kLdAlign);
      if (!must && 2 * k > fc->Kp) return false;
      if (tiny)
        *pack = false;  // launch bound: read through the map
      else if (must && 2 * k > fc->Kp)
        *pack = true;
      r->kmap = in[i]->kept_idx;
      r->flop = 2.0 * (double)fc->Mp * (double)k * (double)dense[i];
      *kp = k;
      return true;
    };
    // A set whose kept-row list is empty contracts over nothing: its dense columns are the bias and
    // zeros, which the gather pass writes along with its own columns (no GEMM, no packing).
    auto nothing_kept = [&](int64_t i, const GemmRows& r) { return r.kmap != nullptr && in[i]->n_kept == 0; };
    auto fill_by_gather = [&](int64_t i) {
      gs[i].nfill = (int32_t)dense[i];
      gs[i].fill = outs[i]->V;
      gs[i].bias = bias;
    };
    // Inputs with columns that are described but not in memory yet: the contraction reads them from
    // memory unless it goes over no row at all or through the packing pass (which takes such columns
    // from the weights they were gathered from).  Everybody else has them written now.
    if (st == NNVHIP_OK) {
      std::vector<nnvhip_star*> cols;
      for (int64_t i = 0; i < count; ++i) {
        if (!in[i]->cs.any_pending()) continue;
        GemmRows r;
        int64_t kp = 0;
        bool pack = false;
        const bool compact = rows_of(i, &r, &kp, &pack);
        if (!(compact && (nothing_kept(i, r) || (pack && r.kmap != nullptr)))) cols.push_back(in[i]);
      }
      if (!cols.empty()) st = write_pending_columns(c, (int64_t)cols.size(), cols.data());
    }
    // Gathered columns whose range sums this call leaves behind are not written: the ReLU step that
    // follows works from the sums, and the next FC map either contracts over no row or packs its rows
    // from the weights.  lazy[i] is set where the sums are produced.
    std::vector<char> lazy((size_t)count, 0);
    if (count == 1 && rowsum && st == NNVHIP_OK) {
      GemmRows rows;
      int64_t kp = fc->Kp;
      bool pack = false;
      const bool compact = rows_of(0, &rows, &kp, &pack);
      const int mode = box_in ? 0 : 1;
      if (box_in) {
        // the centre's product W * c + b is formed along the way: no GEMM launch at all
        st = launch_fc_rowsum(c, fc, outs[0], mode, in[0]->oh_scale, nullptr, nullptr, 1, in[0]->V, nullptr, 0);
        lazy[0] = lazy_ok;
      } else if (compact && nothing_kept(0, rows)) {
        // no row kept: the contracted columns are the bias and zeros, of which only the centre is stored
        fill_by_gather(0);
        st = launch_fc_rowsum(c, fc, outs[0], mode, nullptr, in[0]->cls, in[0]->pre_ub, 2, nullptr, nullptr, 0);
        lazy[0] = lazy_ok;
      } else {
        RangeFuse fuse;
        fuse.plb = outs[0]->plb;
        fuse.pub = outs[0]->pub;
        BufRef packed;
        // enough 128 x 128 tiles to go round: the tile kernel of gemm_seg.hip (rows packed transposed, operands
        // staged straight into LDS), as for an array of sets
        const int64_t tiles128 = ceil_div(dense[0], 128) * ceil_div(fc->Mp, 128);
        const bool tile_kernel = compact && pack && rows.kmap != nullptr && !dense_only && tiles128 >= 128 && kp <= 2048 &&
                                 dense[0] < (int64_t(1) << 24);
        if (tile_kernel) {
          const int64_t ldo = outs[0]->ld, ldt = round_up(dense[0], 128), ntiles = ceil_div(dense[0], 128);
          st = c->alloc(sizeof(double) * kp * ldt, &packed);
          if (st == NNVHIP_OK) {
            PackSet ps = pack_of(in[0], in[0]->kept_idx, packed->as<double>(), kp, dense[0]);
            ps.ldt = ldt;
            st = launch_pack_rows_t(c, 1, &ps);
          }
          if (st == NNVHIP_OK) st = c->alloc(sizeof(double) * 4 * ldo * ntiles, &fuse.part);
          fuse.chunks = ntiles;
          // tiles by width: [0] 128 columns, [1] 64, [2] 32 (the last tile, if the remainder fits)
          std::vector<SegTile> tiles[3];
          double flop[3] = {0.0, 0.0, 0.0};
          for (int64_t j = 0; j < dense[0] && st == NNVHIP_OK; j += 128) {
            const int64_t valid = std::min<int64_t>(128, dense[0] - j);
            const int w = valid > 64 ? 0 : valid > 32 ? 1 : 2;
            SegTile sg{};
            sg.kmap = rows.kmap;
            sg.Bt = packed->as<double>();
            sg.ldbt = ldt;
            sg.b_col0 = j;
            sg.col_local0 = j;
            sg.col_base = j;
            sg.kp = (int32_t)kp;
            sg.valid = (int32_t)valid;
            sg.plb = outs[0]->plb;
            sg.pub = outs[0]->pub;
            sg.rpart = fuse.part->as<double>() + 4 * ldo * (j / 128);
            tiles[w].push_back(sg);
            flop[w] += 2.0 * (double)fc->Mp * (double)kp * (double)valid;
          }
          static const int widths[3] = {128, 64, 32};
          for (int w = 0; w < 3 && st == NNVHIP_OK; ++w) {
            if (tiles[w].empty()) continue;
            BufRef dt;
            st = c->upload_table(tiles[w].data(), sizeof(SegTile) * tiles[w].size(), &dt);
            if (st == NNVHIP_OK)
              st = launch_gemm_seg(c, Wd, fc->Mp, outs[0]->V, ldo, fc->Mp, bias, widths[w], dt->as<SegTile>(), (int64_t)tiles[w].size(),
                                   flop[w]);
          }
        } else if (compact && pack) {
          st = c->alloc(sizeof(double) * kp * dense[0], &packed);
          if (st == NNVHIP_OK) {
            PackSet ps = pack_of(in[0], in[0]->kept_idx, packed->as<double>(), kp, dense[0]);
            st = launch_pack_rows(c, 1, &ps);
            rows.Bk = packed->as<double>();
            rows.ldbk = kp;
          }
        }
        if (st == NNVHIP_OK && !tile_kernel)
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, dense[0], kp, bias, &fuse,
                           compact ? &rows : nullptr);
        if (st == NNVHIP_OK && fuse.chunks > 0) {
          st = launch_fc_rowsum(c, fc, outs[0], mode, nullptr, in[0]->cls, in[0]->pre_ub, 0, nullptr, fuse.part->as<double>(), fuse.chunks);
          lazy[0] = lazy_ok;
        } else if (st == NNVHIP_OK) {
          // the product was split along K and left no sums: the columns are written
          if (st == NNVHIP_OK) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), 0);
        }
      }
      // a caller that wants the gathered columns in memory gets them written now (same values as a later
      // first read would write)
      if (st == NNVHIP_OK && outs[0]->lb != nullptr && !lazy_ok) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), 0);
    } else if (count == 1) {
      // one set: the GEMM epilogue also leaves the partial sums of Star.estimateRanges, so the
      // output set carries its ranges without another pass over V
      RangeFuse fuse;
      fuse.plb = outs[0]->plb;
      fuse.pub = outs[0]->pub;
      const int64_t gch = gather_chunks(fc->Mp, gs[0].m);
      fuse.extra_chunks = gch;
      GemmRows rows;
      int64_t kp = fc->Kp;
      bool pack = false;
      const bool compact = rows_of(0, &rows, &kp, &pack);
      if (compact && nothing_kept(0, rows)) {
        fill_by_gather(0);
        const int64_t ch = std::max<int64_t>(1, gather_chunks(fc->Mp, std::max<int64_t>(gs[0].m, gs[0].nfill)));
        BufRef part;
        if (gs[0].m > 0) {
          st = c->alloc(sizeof(double) * 4 * outs[0]->ld * ch, &part);
          if (st == NNVHIP_OK) gs[0].part = part->as<double>();
          lazy[0] = lazy_ok;
          gs[0].lazy = lazy[0];
        }
        if (st == NNVHIP_OK) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), gs[0].m > 0 ? ch : 0);
        if (st == NNVHIP_OK && gs[0].m > 0) st = finalize_fused_ranges(c, outs[0], part, ch);
      } else {
        BufRef packed;
        if (compact && pack) {
          st = c->alloc(sizeof(double) * kp * dense[0], &packed);
          if (st == NNVHIP_OK) {
            PackSet ps = pack_of(in[0], in[0]->kept_idx, packed->as<double>(), kp, dense[0]);
            st = launch_pack_rows(c, 1, &ps);
            rows.Bk = packed->as<double>();
            rows.ldbk = kp;
          }
        }
        // only the centre is contracted (a box star): the range sums are the gather's alone
        const bool centre_only = dense[0] == 1 && gs[0].m > 0;
        // ... and when the gathered columns are all the columns of W (no degenerate dimension), the gather
        // pass forms the centre's product as well, one partial vector per chunk: no GEMM launch at all
        const bool centre_in_gather = centre_only && !compact && gs[0].m == fc->K && in[0]->oh_from == 1 && gch > 0;
        SplitKDefer defer;  // (otherwise the gather pass sums the centre's split-K partials)
        BufRef cpart;
        if (st == NNVHIP_OK && centre_in_gather) {
          st = c->alloc(sizeof(double) * outs[0]->ld * gch, &cpart);
          if (st == NNVHIP_OK) {
            gs[0].cin = in[0]->V;
            gs[0].cpart = cpart->as<double>();
          }
        } else if (st == NNVHIP_OK) {
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, dense[0], kp, bias,
                           centre_only ? nullptr : &fuse, compact ? &rows : nullptr, centre_only ? &defer : nullptr);
        }
        if (st == NNVHIP_OK && centre_only) {
          st = c->alloc(sizeof(double) * 4 * outs[0]->ld * gch, &fuse.part);
          fuse.chunks = 0;
          if (defer.ksplit > 1) {
            gs[0].red = defer.ws->as<double>();
            gs[0].red_k = (int32_t)defer.ksplit;
            gs[0].centre = outs[0]->V;
            gs[0].bias = bias;
          }
        }
        const bool fused = st == NNVHIP_OK && (fuse.chunks > 0 || centre_only);
        if (st == NNVHIP_OK && gs[0].m > 0) {
          gs[0].part = fused ? fuse.part->as<double>() + fuse.chunks * 4 * outs[0]->ld : nullptr;
          lazy[0] = lazy_ok && fused;
          gs[0].lazy = lazy[0];
          st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), fused ? gch : 0);
        }
        if (st == NNVHIP_OK && fused)
          st = finalize_fused_ranges(c, outs[0], fuse.part, fuse.chunks + (gs[0].m > 0 ? gch : 0),
                                     centre_in_gather ? cpart->as<double>() : nullptr, centre_in_gather ? gch : 0, bias);
      }
    } else if (contig) {
      // one launch for the whole array.  With structure to exploit, every set's dense columns are cut
      // into tiles of 128 that carry their own description (row list, position in the arena).
      bool any_rows = false, bias_in_kernel = false;
      std::vector<GemmRows> rws((size_t)count);
      std::vector<int64_t> kps((size_t)count);
      std::vector<char> pk((size_t)count, 0);
      std::vector<char> filled((size_t)count, 0);
      bool any_fill = false;
      // Range sums: chunk_off[i] .. chunk_off[i+1] are set i's chunks of [4][ld] partial sums in `sums`,
      // first one per column tile of the segmented GEMM (tiles_of[i], filled by its epilogue), then the
      // gather pass's gch chunks if the set has gathered columns.
      BufRef sums;
      std::vector<int64_t> tiles_of((size_t)count, 0), chunk_off((size_t)count + 1, 0);
      int64_t gch = 0;
      {
        int64_t max_m = 0;
        for (int64_t i = 0; i < count; ++i) max_m = std::max<int64_t>(max_m, gs[i].m);
        gch = gather_chunks_batch(outs[0]->ld, count, max_m);  // 0: nothing to gather
      }
      // large arrays: the sums of the gathered columns come from one matrix product instead (gch_part = 0:
      // the gather pass leaves no chunks)
      bool use_mm = lazy_ok && gch > 0 && count >= 64;
      for (int64_t i = 0; i < count; ++i) use_mm = use_mm && !(gs[i].m > 0 && in[i]->oh_scale_neg);
      const int64_t gch_part = use_mm ? 0 : gch;
      BufRef mm_sums;
      for (int64_t i = 0; i < count; ++i) {
        bool pack = false;
        any_rows = rows_of(i, &rws[i], &kps[i], &pack) || any_rows;
        pk[i] = pack && rws[i].kmap != nullptr;
        if (nothing_kept(i, rws[i])) {
          fill_by_gather(i);
          filled[i] = 1;
          pk[i] = 0;
          any_fill = true;
        }
      }
      bool all_stored = true;
      for (int64_t i = 0; i < count; ++i) all_stored = all_stored && in[i]->stored_cols() == in[i]->n + 1;
      if (any_onehot && !any_rows && all_stored) {
        // all sets contract over every row: their dense columns are simply listed (tiles may span sets)
        if (cols >= (int64_t(1) << 31)) st = NNVHIP_ERR_SHAPE;
        std::vector<int32_t> map;
        map.reserve((size_t)total_dense);
        int64_t off = 0;
        for (int64_t i = 0; i < count; ++i) {
          for (int64_t j = 0; j < dense[i]; ++j) map.push_back((int32_t)(off + j));
          off += in[i]->n + 1;  // box stars: all columns stored, input and output arenas laid out alike
        }
        BufRef cmap;
        if (st == NNVHIP_OK) st = c->upload_table(map.data(), sizeof(int32_t) * map.size(), &cmap);
        if (st == NNVHIP_OK) {
          GemmRows rows;
          rows.colmap = cmap->as<int32_t>();
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, total_dense, fc->Kp, bias,
                           nullptr, &rows);
        }
      } else if (any_rows || any_onehot) {
        std::vector<GemmSeg> segs;
        GemmRows rows;
        const int64_t tn = gemm_seg_cols(fc->Mp, count, dense.data());
        rows.seg_cols = (int32_t)tn;
        // Large arrays whose sets all come with packed rows take the tile kernel of gemm_seg.hip: rows packed
        // transposed, operands staged straight into LDS, a narrow last tile per set, bias added in the kernel.
        bool seg_tiles = tn == 128 && !dense_only;
        for (int64_t i = 0; i < count; ++i)
          if (!filled[i] && (!pk[i] || kps[i] > 2048 || dense[i] >= (int64_t(1) << 24))) seg_tiles = false;
        if (seg_tiles) {
          const int64_t ldo = outs[0]->ld;
          BufRef packed, shared_rows;
          std::vector<PackSet> packs;
          std::vector<const double*> bt((size_t)count, nullptr);
          std::vector<int64_t> ldt((size_t)count, 0);
          // Sets whose generator columns are all the same scaled weight columns (boxes of one shape through an FC
          // layer and a ReLU: same index list, same scales) have the same packed rows wherever they keep the same
          // row.  One matrix then serves them all - row r = what any of them would pack for input row r - and the
          // 128-column tiles gather its rows through their own kept-row lists; only a set's centre column (patched
          // in by its first tile) and the columns past the last whole tile (packed as before) are its own.
          struct RowShape {  // what decides a set's packed rows besides its kept-row list
            const double* Wt;
            int64_t ldwt, rows;
            const int32_t* idx;
            const double* scale;
            int64_t dense, ldws, nfull, off;
          };
          std::vector<RowShape> shapes;
          std::vector<int> shape_of((size_t)count, -1);
          bool shared = true;
          for (int64_t i = 0; i < count && shared; ++i) {
            if (filled[i]) continue;
            const ColSource& cs = in[i]->cs;
            shared = cs.W != nullptr && cs.Wt != nullptr && cs.from == 1 && cs.from + cs.cols >= dense[i] && cs.zero_to <= 1 &&
                     !cs.win_pending() && dense[i] >= 128 && cs.rows < (int64_t(1) << 30);
            if (!shared) break;
            for (size_t k = 0; k < shapes.size() && shape_of[i] < 0; ++k) {
              const RowShape& r = shapes[k];
              if (r.Wt == cs.Wt && r.ldwt == cs.ldwt && r.rows == cs.rows && r.idx == cs.idx && r.scale == cs.scale && r.dense == dense[i])
                shape_of[i] = (int)k;
            }
            if (shape_of[i] < 0) {
              if (shapes.size() == 16) {  // too many different shapes for the matrices to pay
                shared = false;
                break;
              }
              shape_of[i] = (int)shapes.size();
              shapes.push_back(RowShape{cs.Wt, cs.ldwt, cs.rows, cs.idx, cs.scale, dense[i], round_up(dense[i], 128), dense[i] / 128, 0});
            }
          }
          shared = shared && !shapes.empty();
          // Sets of one shape differ in their products only through their kept-row lists (and their centres).  Where
          // the lists of a group are nearly the same - the sub-boxes of one box, whose first-layer bounds differ by
          // little - the group's product over the rows most of its sets keep is formed once (by the tile kernel), and a
          // set's output is that product plus the few rows in which the set differs, written by one streaming pass
          // (delta_try / delta_done below).
          bool delta_try = shared && count >= 32 && !c->no_row_deltas;
          for (size_t k = 1; k < shapes.size() && delta_try; ++k) delta_try = shapes[k].rows == shapes[0].rows;
          delta_try = delta_try && !shapes.empty() && shapes[0].rows == fc->Kp && shapes[0].rows < (int64_t(1) << 20);
          if (shared) {
            int64_t doubles = 0;
            for (RowShape& r : shapes) {
              r.off = doubles;
              doubles += (r.rows + 1) * r.ldws;
            }
            st = c->alloc(sizeof(double) * doubles, &shared_rows);
            ScaledRows sr{};
            for (size_t k = 0; k < shapes.size(); ++k) {
              const RowShape& r = shapes[k];
              sr.s[k] = ScaledRows::One{r.Wt, r.ldwt, r.idx, r.scale, shared_rows ? shared_rows->as<double>() + r.off : nullptr, r.ldws,
                                        (int32_t)r.rows, (int32_t)r.dense};
            }
            sr.count = (int32_t)shapes.size();
            if (st == NNVHIP_OK) st = launch_scaled_rows(c, sr);
          }
          bool delta_done = false;
          if (delta_try && st == NNVHIP_OK) {
            constexpr int kDeltaCap = 64;
            const int groups = (int)shapes.size();
            const int64_t rowsK = shapes[0].rows, rows_pad = round_up(rowsK, 16);
            std::vector<int64_t> act;  // the sets that take part (not filled)
            std::vector<DeltaSet> dsets;
            std::vector<CentreSet> csets;
            std::vector<int32_t> gsize((size_t)groups, 0);
            for (int64_t i = 0; i < count; ++i)
              if (!filled[i]) {
                act.push_back(i);
                dsets.push_back(DeltaSet{rws[i].kmap, (int32_t)kps[i], (int32_t)shape_of[i]});
                csets.push_back(CentreSet{rws[i].kmap, in[i]->V, (int32_t)kps[i]});
                gsize[(size_t)shape_of[i]]++;
              }
            const int64_t nact = (int64_t)act.size();
            BufRef dtab, ctab, gtab, votes, common, lens, delta;
            if (nact == 0) st = NNVHIP_OK;
            if (nact > 0) {
              st = c->upload_table(dsets.data(), sizeof(DeltaSet) * dsets.size(), &dtab);
              if (st == NNVHIP_OK) st = c->upload_table(gsize.data(), sizeof(int32_t) * gsize.size(), &gtab);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * groups * rowsK, &votes);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * groups * rows_pad, &common);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * (groups + nact), &lens);  // ncommon, then dlen
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * nact * kDeltaCap, &delta);
              if (st == NNVHIP_OK)
                st = launch_delta_lists(c, nact, dtab->as<DeltaSet>(), groups, gtab->as<int32_t>(), rowsK, rows_pad, kDeltaCap,
                                        votes->as<int32_t>(), common->as<int32_t>(), lens->as<int32_t>(), delta->as<int32_t>(),
                                        lens->as<int32_t>() + groups);
              std::vector<int32_t> hl((size_t)(groups + nact));
              if (st == NNVHIP_OK) {
                void* hp = nullptr;
                st = c->stage(sizeof(int32_t) * hl.size(), &hp);
                if (st == NNVHIP_OK) {
                  if (hipMemcpyAsync(hp, lens->ptr, sizeof(int32_t) * hl.size(), hipMemcpyDeviceToHost, c->stream) != hipSuccess ||
                      hipStreamSynchronize(c->stream) != hipSuccess) {
                    set_error("HIP error reading the row-difference lists back");
                    st = NNVHIP_ERR_HIP;
                  } else {
                    memcpy(hl.data(), hp, sizeof(int32_t) * hl.size());
                  }
                }
              }
              bool fits = st == NNVHIP_OK;
              int64_t delta_rows = 0;
              for (int64_t a = 0; a < nact && fits; ++a) {
                fits = hl[(size_t)(groups + a)] >= 0;
                delta_rows += std::max<int32_t>(hl[(size_t)(groups + a)], 0);
              }
              // worth it when a set's differences are a small part of its list
              int64_t kept_rows = 0;
              for (int64_t a = 0; a < nact; ++a) kept_rows += kps[act[(size_t)a]];
              fits = fits && 4 * delta_rows <= kept_rows;
              if (fits) {
                const int64_t ldo = outs[0]->ld, Mp = fc->Mp;
                // the groups' shared products: the same tiles, over the majority lists, into a buffer of their own
                int64_t base_cols = 0;
                std::vector<int64_t> base_off((size_t)groups);
                for (int g = 0; g < groups; ++g) {
                  base_off[(size_t)g] = base_cols;
                  base_cols += shapes[(size_t)g].ldws;
                }
                BufRef basebuf, cm, cprod;
                st = c->alloc(sizeof(double) * Mp * base_cols, &basebuf);
                std::vector<SegTile> bt_tiles;
                double base_flop = 0.0;
                for (int g = 0; g < groups && st == NNVHIP_OK; ++g) {
                  const RowShape& r = shapes[(size_t)g];
                  if (gsize[(size_t)g] == 0) continue;
                  for (int64_t j = 0; j < r.dense; j += 128) {
                    SegTile sg{};
                    sg.kmap = common->as<int32_t>() + (int64_t)g * rows_pad;
                    sg.Bt = shared_rows->as<double>() + r.off;
                    sg.ldbt = r.ldws;
                    sg.b_col0 = j;
                    sg.col_local0 = j;
                    sg.col_base = base_off[(size_t)g] + j;
                    sg.gather_b = 1;
                    sg.zero_row = (int32_t)r.rows;
                    sg.kp = hl[(size_t)g];
                    sg.valid = (int32_t)std::min<int64_t>(128, r.dense - j);
                    bt_tiles.push_back(sg);
                    base_flop += 2.0 * (double)Mp * (double)sg.kp * (double)sg.valid;
                  }
                }
                if (st == NNVHIP_OK && !bt_tiles.empty()) {
                  BufRef dt;
                  st = c->upload_table(bt_tiles.data(), sizeof(SegTile) * bt_tiles.size(), &dt);
                  if (st == NNVHIP_OK)
                    st = launch_gemm_seg(c, Wd, Mp, basebuf->as<double>(), Mp, Mp, nullptr, 128, dt->as<SegTile>(), (int64_t)bt_tiles.size(),
                                         base_flop, true);
                }
                // the centres, which are the sets' own: W * (centre masked to the kept rows), all sets in one product
                if (st == NNVHIP_OK) st = c->upload_table(csets.data(), sizeof(CentreSet) * csets.size(), &ctab);
                if (st == NNVHIP_OK) st = c->alloc(sizeof(double) * fc->Kp * nact, &cm);
                if (st == NNVHIP_OK) st = c->alloc(sizeof(double) * Mp * nact, &cprod);
                if (st == NNVHIP_OK) st = launch_masked_centres(c, nact, ctab->as<CentreSet>(), cm->as<double>(), fc->Kp);
                if (st == NNVHIP_OK)
                  st = launch_gemm(c, Wd, Mp, cm->as<double>(), fc->Kp, cprod->as<double>(), Mp, Mp, nact, fc->Kp, nullptr);
                // the sets' tiles, by column tile and group so that tiles that read the same piece of a shared product
                // run next to one another
                for (int64_t i = 0; i < count; ++i) {
                  tiles_of[i] = filled[i] ? 0 : delta_tile_chunks(dense[i]);
                  chunk_off[i + 1] = chunk_off[i] + tiles_of[i] + (gs[i].m > 0 ? gch_part : 0);
                }
                if (st == NNVHIP_OK && chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
                std::vector<int64_t> col_off((size_t)count, 0);
                {
                  int64_t off = 0;
                  for (int64_t i = 0; i < count; ++i) {
                    col_off[(size_t)i] = off;
                    off += in[i]->n + 1;
                  }
                }
                // the sets by group, so that neighbours in the table read the same shared product
                std::vector<DeltaOut> douts;
                std::vector<int32_t> dgroup;
                double dbytes = 0.0;
                int64_t max_cols = 0;
                for (int g = 0; g < groups && st == NNVHIP_OK; ++g)
                  for (int64_t a = 0; a < nact; ++a) {
                    const int64_t i = act[(size_t)a];
                    if (shape_of[i] != g) continue;
                    const RowShape& r = shapes[(size_t)g];
                    DeltaOut d{};
                    d.delta = delta->as<int32_t>() + a * kDeltaCap;
                    d.base = basebuf->as<double>() + base_off[(size_t)g] * Mp;
                    d.S = shared_rows->as<double>() + r.off;
                    d.lds = r.ldws;
                    d.cprod = cprod->as<double>() + a * Mp;
                    d.out = outs[0]->V + col_off[(size_t)i] * ldo;
                    d.plb = outs[i]->plb;
                    d.pub = outs[i]->pub;
                    d.rpart = sums->as<double>() + 4 * ldo * chunk_off[i];
                    d.dlen = hl[(size_t)(groups + a)];
                    d.ncols = (int32_t)dense[i];
                    douts.push_back(d);
                    dgroup.push_back((int32_t)g);
                    dbytes += 8.0 * (double)Mp * (double)dense[i];
                    max_cols = std::max<int64_t>(max_cols, dense[i]);
                  }
                if (st == NNVHIP_OK && !douts.empty())
                  st = launch_delta_tiles(c, Wd, Mp, Mp, bias, ldo, (int64_t)douts.size(), douts.data(), dgroup.data(), max_cols, dbytes);
                delta_done = true;
                bias_in_kernel = true;
              }
            }
          }
          auto nfull_of = [&](int64_t i) { return shared ? shapes[(size_t)shape_of[i]].nfull : 0; };
          int64_t total = 0;
          if (!delta_done) {
          for (int64_t i = 0; i < count; ++i)
            if (!filled[i]) {
              if (shared) {  // the columns past the last whole tile only, in a tile of their own width
                const int64_t rem = dense[i] - 128 * nfull_of(i);
                ldt[i] = rem > 64 ? 128 : rem > 32 ? 64 : rem > 0 ? 32 : 0;
              } else {
                ldt[i] = round_up(dense[i], 128);
              }
              total += kps[i] * ldt[i];
            }
          if (total > 0 && st == NNVHIP_OK) st = c->alloc(sizeof(double) * total, &packed);
          int64_t pos = 0;
          for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
            if (!filled[i] && ldt[i] > 0) {
              bt[i] = packed->as<double>() + pos;
              PackSet ps = pack_of(in[i], rws[i].kmap, packed->as<double>() + pos, kps[i], dense[i]);
              ps.ldt = ldt[i];
              if (shared) {
                ps.col0 = (int32_t)(128 * nfull_of(i));
                ps.ncols = (int32_t)(dense[i] - 128 * nfull_of(i));
              }
              packs.push_back(ps);
              pos += kps[i] * ldt[i];
            }
          if (st == NNVHIP_OK && !packs.empty()) st = launch_pack_rows_t(c, (int64_t)packs.size(), packs.data());
          for (int64_t i = 0; i < count; ++i) {
            tiles_of[i] = filled[i] ? 0 : ceil_div(dense[i], 128);
            chunk_off[i + 1] = chunk_off[i] + tiles_of[i] + (gs[i].m > 0 ? gch_part : 0);
          }
          if (st == NNVHIP_OK && chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
          // tiles by width: [0] 128 columns, [1] 64, [2] 32 (the last tile of a set whose remainder fits); [3]: the
          // 128-column tiles that gather their rows of B from the shared matrix
          std::vector<SegTile> tiles[4];
          double flop[4] = {0.0, 0.0, 0.0, 0.0};
          int64_t off = 0;
          for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
            for (int64_t j = 0; j < dense[i] && !filled[i]; j += 128) {
              const int64_t valid = std::min<int64_t>(128, dense[i] - j);
              const bool gather = shared && j < 128 * nfull_of(i);
              const int w = gather ? 3 : valid > 64 ? 0 : valid > 32 ? 1 : 2;
              SegTile sg{};
              sg.kmap = rws[i].kmap;
              if (gather) {
                const RowShape& r = shapes[(size_t)shape_of[i]];
                sg.Bt = shared_rows->as<double>() + r.off;
                sg.ldbt = r.ldws;
                sg.b_col0 = j;
                sg.centre = in[i]->V;
                sg.gather_b = 1;
                sg.zero_row = (int32_t)r.rows;
              } else {
                sg.Bt = bt[i];
                sg.ldbt = ldt[i];
                sg.b_col0 = shared ? 0 : j;
              }
              sg.col_local0 = j;
              sg.col_base = off + j;
              sg.kp = (int32_t)kps[i];
              sg.valid = (int32_t)valid;
              sg.plb = outs[i]->plb;
              sg.pub = outs[i]->pub;
              sg.rpart = sums->as<double>() + 4 * ldo * (chunk_off[i] + j / 128);
              tiles[w].push_back(sg);
              flop[w] += 2.0 * (double)fc->Mp * (double)kps[i] * (double)valid;
            }
            off += in[i]->n + 1;
          }
          static const int widths[4] = {128, 64, 32, 128};
          for (int w = 3; w >= 0 && st == NNVHIP_OK; --w) {
            if (tiles[w].empty()) continue;
            BufRef dt;
            st = c->upload_table(tiles[w].data(), sizeof(SegTile) * tiles[w].size(), &dt);
            if (st == NNVHIP_OK)
              st = launch_gemm_seg(c, Wd, fc->Mp, outs[0]->V, ldo, fc->Mp, bias, widths[w], dt->as<SegTile>(), (int64_t)tiles[w].size(),
                                   flop[w], w == 3);
          }
          bias_in_kernel = true;
          }  // !delta_done
        } else {
        // several row tiles would each gather the kept rows of B: pack them once per set instead
        BufRef packed;
        std::vector<PackSet> packs;
        std::vector<const double*> bk((size_t)count, nullptr);
        {
          int64_t total = 0;
          for (int64_t i = 0; i < count; ++i)
            if (pk[i]) total += kps[i] * dense[i];
          if (total > 0) st = c->alloc(sizeof(double) * total, &packed);
          int64_t pos = 0;
          for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
            if (pk[i]) {
              bk[i] = packed->as<double>() + pos;
              packs.push_back(pack_of(in[i], rws[i].kmap, packed->as<double>() + pos, kps[i], dense[i]));
              pos += kps[i] * dense[i];
            }
          if (st == NNVHIP_OK && !packs.empty()) st = launch_pack_rows(c, (int64_t)packs.size(), packs.data());
        }
        const int64_t ldo = outs[0]->ld;
        for (int64_t i = 0; i < count; ++i) {
          tiles_of[i] = filled[i] ? 0 : ceil_div(dense[i], tn);
          chunk_off[i + 1] = chunk_off[i] + tiles_of[i] + (gs[i].m > 0 ? gch_part : 0);
        }
        if (st == NNVHIP_OK && chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
        int64_t off = 0, off_in = 0, kp_max = kLdAlign;
        for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
          for (int64_t j = 0; j < dense[i] && !filled[i]; j += tn) {
            GemmSeg sg;
            sg.plb = outs[i]->plb;
            sg.pub = outs[i]->pub;
            sg.rpart = sums->as<double>() + 4 * ldo * (chunk_off[i] + j / tn);
            sg.kmap = rws[i].kmap;
            sg.Bk = bk[i];
            sg.ldbk = kps[i];
            sg.col_local0 = j;
            sg.b_col_base = off_in + j;
            sg.col_base = off + j;
            sg.kp = (int32_t)kps[i];
            sg.valid = (int32_t)std::min<int64_t>(tn, dense[i] - j);
            segs.push_back(sg);
          }
          if (!filled[i]) {
            rows.flop += 2.0 * (double)fc->Mp * (double)kps[i] * (double)dense[i];
            kp_max = std::max(kp_max, kps[i]);
          }
          off += in[i]->n + 1;
          off_in += in[i]->stored_cols();
        }
        BufRef dsegs;
        if (st == NNVHIP_OK && !segs.empty()) st = c->upload_table(segs.data(), sizeof(GemmSeg) * segs.size(), &dsegs);
        if (st == NNVHIP_OK && !segs.empty()) {
          rows.segs = dsegs->as<GemmSeg>();
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, tn * (int64_t)segs.size(),
                           kp_max, bias, nullptr, &rows);
        }
        }
      } else {
        st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, cols, fc->Kp, bias);
      }
      if (st == NNVHIP_OK && bias && count > 1 && !bias_in_kernel) {
        // the GEMM adds the bias to column 0 of the arena (the first set's centre); the other sets'
        // centres get it here (a set whose dense columns the gather pass fills has it from there)
        std::vector<double*> centres;
        for (int64_t i = 1; i < count; ++i)
          if (!filled[i]) centres.push_back(outs[i]->V);
        BufRef tab;
        if (!centres.empty()) st = c->upload_table(centres.data(), sizeof(double*) * centres.size(), &tab);
        if (st == NNVHIP_OK && !centres.empty()) st = launch_bias_columns(c, tab->as<double*>(), (int64_t)centres.size(), bias, fc->Mp);
      }
      if (st == NNVHIP_OK && (any_onehot || any_fill)) {
        // the gather also leaves the range sums of its columns on the output handles, so the ReLU
        // that follows scans only the contracted columns
        const int64_t ldo = outs[0]->ld;
        if (!sums) {  // no segmented GEMM ran: the gather's chunks are all there is
          for (int64_t i = 0; i < count; ++i) chunk_off[i + 1] = chunk_off[i] + (gs[i].m > 0 ? gch_part : 0);
          if (chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
        }
        if (st == NNVHIP_OK && use_mm) {
          if (mm_early) mm_sums = mm_early;  // queued at the start of the call, from the same lists
          else st = launch_range_sums_mm(c, fc, count, gs.data(), &mm_sums, &mm_slot);
        }
        if (st == NNVHIP_OK) {
          for (int64_t i = 0; i < count; ++i) {
            gs[i].part = (gch_part > 0 && gs[i].m > 0) ? sums->as<double>() + 4 * ldo * (chunk_off[i] + tiles_of[i]) : nullptr;
            lazy[i] = lazy_ok && (gs[i].part != nullptr || (use_mm && gs[i].m > 0));
            gs[i].lazy = lazy[i];
          }
          st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, ldo, count, gs.data(), gch_part);
        }
      }
      // what the two passes left: the GEMM tiles' chunks cover the contracted columns, the gather's its own;
      // columns covered by neither (a GEMM without the fused sums) still need a scan, filled zeros add nothing
      for (int64_t i = 0; i < count && st == NNVHIP_OK && (sums || mm_sums); ++i) {
        const int64_t nchunks = chunk_off[i + 1] - chunk_off[i];
        const bool mm = mm_sums && gs[i].m > 0;
        if (nchunks == 0 && !mm) continue;
        if (nchunks > 0) {
          outs[i]->rng_buf = sums;
          outs[i]->rng_part = sums->as<double>() + 4 * outs[0]->ld * chunk_off[i];
          outs[i]->rng_chunks = nchunks;
        }
        if (mm) {
          outs[i]->rng_mm_buf = mm_sums;
          outs[i]->rng_mm = mm_sums->as<double>() + 4 * outs[0]->ld * mm_slot[(size_t)i];  // two columns of 2 * ld entries
        }
        outs[i]->rng_first_col = (filled[i] || tiles_of[i] > 0) ? 1 : dense[i];
      }
    } else {
      for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
        GemmRows rows;
        int64_t kp = fc->Kp;
        bool pack = false;
        const bool compact = rows_of(i, &rows, &kp, &pack);
        if (compact && nothing_kept(i, rows)) {
          fill_by_gather(i);
          st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[i]->ld, 1, &gs[i], 0);
          continue;
        }
        BufRef packed;
        if (compact && pack) {
          st = c->alloc(sizeof(double) * kp * dense[i], &packed);
          if (st != NNVHIP_OK) break;
          PackSet ps = pack_of(in[i], in[i]->kept_idx, packed->as<double>(), kp, dense[i]);
          st = launch_pack_rows(c, 1, &ps);
          if (st != NNVHIP_OK) break;
          rows.Bk = packed->as<double>();
          rows.ldbk = kp;
        }
        st = launch_gemm(c, Wd, fc->Mp, in[i]->V, in[i]->ld, outs[i]->V, outs[i]->ld, fc->Mp, dense[i], kp, bias, nullptr,
                         compact ? &rows : nullptr);
        if (st == NNVHIP_OK && gs[i].m > 0) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[i]->ld, 1, &gs[i], 0);
      }
    }
    // the gathered columns remember where they came from
    // (arrays: the next layer packs kept rows of these columns, i.e. reads rows of W - from a row-major copy)
    if (st == NNVHIP_OK && count >= 64 && !fc->Wt && fc->Mp * fc->Kp < (int64_t(1) << 31)) {
      bool any = false;
      for (int64_t i = 0; i < count; ++i) any = any || gs[i].m > 0;
      if (any) {
        BufRef wt;
        st = c->alloc(sizeof(double) * fc->Mp * fc->Kp, &wt);
        if (st == NNVHIP_OK) {
          hipLaunchKernelGGL(transpose_weights_kernel, dim3((unsigned)ceil_div(fc->Kp, 32), (unsigned)ceil_div(fc->Mp, 32)), dim3(32, 8), 0,
                             c->stream, Wd, wt->as<double>(), (int)fc->Mp, (int)fc->Kp);
          if (hipGetLastError() != hipSuccess) st = NNVHIP_ERR_HIP;
          fc->Wt = wt;
        }
      }
    }
    for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
      if (gs[i].m > 0) {
        nnvhip_star* o = outs[i];
        ColSource& cs = o->cs;
        cs.W_buf = fc->W;
        cs.W = Wd;
        cs.ldw = fc->Mp;
        cs.rows = fc->Mp;
        if (fc->Wt) {
          cs.Wt_buf = fc->Wt;
          cs.Wt = fc->Wt->as<double>();
          cs.ldwt = fc->Kp;
        }
        cs.idx_buf = in[i]->oh_idx_buf;
        cs.idx = gs[i].idx;
        cs.scale_buf = in[i]->oh_scale_buf;
        cs.scale = gs[i].scale;
        cs.from = dense[i];
        cs.cols = gs[i].m;
        cs.pending = lazy[i] != 0;
        cs.zero_to = (lazy[i] && gs[i].nfill > 0) ? gs[i].nfill : 0;  // a filled set's leading columns
        // debugging aid: NaNs where nothing was written, so that a reader that forgets to ask for the
        // columns cannot pass a test on what an earlier call happened to leave in the memory
        auto poison = [&](double* p, int64_t ncols) -> int {
          NNV_HIP_TRY(hipMemsetAsync(p, 0xff, sizeof(double) * o->ld * ncols, c->stream));
          return NNVHIP_OK;
        };
        if (c->poison_pending && cs.pending) st = poison(o->V + cs.from * o->ld, cs.cols);
        if (c->poison_pending && cs.zero_to > 1 && st == NNVHIP_OK) st = poison(o->V + o->ld, cs.zero_to - 1);
      }
  }
  if (st == NNVHIP_OK) st = c->end_op();
  if (st != NNVHIP_OK) {
    release_all(outs);
    return st;
  }
  for (int64_t i = 0; i < count; ++i) out[i] = outs[i];
  return NNVHIP_OK;
}

int nnvhip_affine_conv2d(nnvhip_ctx* c, const nnvhip_conv2d* cv, int64_t H, int64_t W, int64_t count,
                         nnvhip_star* const* in, nnvhip_star** out) {
  CHECK_CTX(c);
  if (!cv || cv->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid layer handle");
  NNV_TRY(check_set_array(c, count, in, out));
  if (H <= 0 || W <= 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "The input is not an ImageStar object");
  for (int64_t i = 0; i < count; ++i) {
    if (in[i]->N % (H * W) != 0) NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistent dimension in the ImageStar and the original Star set");
    int64_t ch = in[i]->N / (H * W);
    if (ch != cv->Cin)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Input set contains %lld channels while the convolutional layers has %lld channels",
               (long long)ch, (long long)cv->Cin);
  }
  int64_t Ho = 0, Wo = 0;
  NNV_TRY(nnvhip_conv2d_output_size(cv, H, W, &Ho, &Wo));
  int64_t Nout = Ho * Wo * cv->Cout;
  if (Nout >= (int64_t(1) << 31) || in[0]->N >= (int64_t(1) << 31)) NNV_FAIL(NNVHIP_ERR_SHAPE, "image too large");
  std::vector<nnvhip_star*> outs;
  bool contig = false;
  int64_t cols = 0;
  NNV_TRY(c->begin_op());
  int st = make_affine_outputs(c, count, in, Nout, &outs, &contig, &cols);
  // generator images that are scaled unit vectors (box ImageStars, columns appended by a ReLU) turn
  // into stamps of the filter; the implicit GEMM runs over the leading dense images only
  std::vector<ConvStampSet> stamps((size_t)count);
  auto mask_on_load = [&](const nnvhip_star* s) {
    return !c->no_conv_mask && s->cls != nullptr && conv2d_can_mask(cv, H, W, Ho, Wo, s->ld);
  };
  bool any_stamps = false;
  int64_t max_m = 0;
  // Windows of the generator images (internal.h, nnvhip_star::box).  The output's come from the input's windows and
  // from the pixels of its unit-vector columns (without either an image counts as full); where the input's dense
  // images have small windows the implicit GEMM computes inside the output windows only.
  const bool track_boxes = !c->no_conv_boxes && H < 32768 && W < 32768 && Ho < 32768 && Wo < 32768;
  struct Plan {
    int64_t nc = 0, dense = 0, m = 0;
    bool in_ok = false;      // the input's windows describe its dense images
    bool out_boxes = false;  // the output gets windows
    bool compact = false;    // the dense images are computed inside their windows only
    int dense_eh = 0, dense_ew = 0;
  };
  std::vector<Plan> plan((size_t)count);
  for (int64_t i = 0; i < count; ++i) {
    Plan& pl = plan[i];
    pl.nc = in[i]->n + 1;
    pl.dense = (!c->dense_affine && in[i]->oh_from > 0 && in[i]->oh_from < pl.nc) ? in[i]->oh_from : pl.nc;
    pl.m = pl.nc - pl.dense;
    if (!track_boxes) continue;
    pl.in_ok = in[i]->box != nullptr && in[i]->box_H == H && in[i]->box_W == W && in[i]->box_cols >= pl.dense;
    pl.out_boxes = pl.in_ok || (pl.m > 0 && pl.dense == 1);
    if (pl.in_ok && pl.dense > 1) {
      pl.dense_eh = (int)conv_box_extent(cv, 0, in[i]->box_eh, Ho);
      pl.dense_ew = (int)conv_box_extent(cv, 1, in[i]->box_ew, Wo);
      // (any table will do for the question; the real one is made below)
      pl.compact = conv2d_in_windows(cv, H, W, Ho, Wo, in[i]->ld, pl.dense, in[i]->box, pl.dense_eh, pl.dense_ew);
    }
  }
  {
    // The implicit GEMM reads whole images: pending row resets are run first, and sets whose unit-vector
    // columns take part in the contraction get those written out.  (A pending reset alone is applied by the
    // kernel as it loads, from one bit per row, where that fits; images that are in memory inside their windows
    // only are fine for the kernel that stays inside the windows.)
    std::vector<nnvhip_star*> full, prefix;
    for (int64_t i = 0; i < count; ++i) {
      const ColSource& cs = in[i]->cs;
      if (plan[i].dense > in[i]->stored_cols())
        full.push_back(in[i]);
      else if (cs.pending || cs.zero_to > 1 || (cs.win_pending() && !plan[i].compact) ||
               (in[i]->rows_pending && !mask_on_load(in[i])))
        prefix.push_back(in[i]);
    }
    if (st == NNVHIP_OK && !full.empty()) st = ensure_dense_batch(c, (int64_t)full.size(), full.data());
    if (st == NNVHIP_OK && !prefix.empty()) st = ensure_dense_batch(c, (int64_t)prefix.size(), prefix.data(), false);
  }
  for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
    const Plan& pl = plan[i];
    nnvhip_star* o = outs[i];
    const ColBox* ob = nullptr;
    if (pl.out_boxes) {
      st = c->alloc(sizeof(ColBox) * (size_t)pl.nc, &o->box_buf);
      if (st != NNVHIP_OK) break;
      ColBox* tab = o->box_buf->as<ColBox>();
      st = launch_conv_boxes(c, cv, H, W, Ho, Wo, pl.in_ok ? in[i]->box : nullptr, pl.dense, in[i]->oh_idx, pl.m, tab);
      if (st != NNVHIP_OK) break;
      int64_t eh = pl.dense > 1 ? pl.dense_eh : 0, ew = pl.dense > 1 ? pl.dense_ew : 0;
      if (pl.m > 0) {
        eh = std::max(eh, conv_box_extent(cv, 0, 1, Ho));
        ew = std::max(ew, conv_box_extent(cv, 1, 1, Wo));
      }
      ob = tab;
      o->box = tab;
      o->box_cols = pl.nc;
      o->box_H = (int32_t)Ho;
      o->box_W = (int32_t)Wo;
      o->box_eh = (int32_t)eh;
      o->box_ew = (int32_t)ew;
    }
    // Images with windows are written inside them only; the zeros around them wait for a reader of whole
    // columns (ColSource::win_*).  Not when the caller wants every column in memory.
    const bool lazy = ob != nullptr && !c->eager_cols;
    const int64_t win_from = lazy ? (pl.compact ? 1 : pl.dense) : 0;
    const int64_t win_to = lazy ? (pl.m > 0 ? pl.nc : (pl.compact ? pl.dense : 0)) : 0;
    if (win_to > win_from) {
      o->cs.win_box_buf = o->box_buf;
      o->cs.win_box = ob;
      o->cs.win_from = win_from;
      o->cs.win_to = win_to;
      o->cs.win_rows = Nout;
      o->cs.win_H = (int32_t)Ho;
      o->cs.win_W = (int32_t)Wo;
      if (c->poison_pending)  // debugging aid: NaNs where nothing will be written
        NNV_HIP_TRY(hipMemsetAsync(o->V + win_from * o->ld, 0xff, sizeof(double) * o->ld * (win_to - win_from), c->stream));
    }
    stamps[i].idx = in[i]->oh_idx;
    stamps[i].scale = in[i]->oh_scale;
    stamps[i].out = o->V + pl.dense * o->ld;
    stamps[i].plb = o->plb + (pl.dense - 1);
    stamps[i].pub = o->pub + (pl.dense - 1);
    stamps[i].part = nullptr;
    stamps[i].m = (int32_t)pl.m;
    stamps[i].win_only = (lazy && pl.m > 0) ? 1 : 0;
    any_stamps = any_stamps || pl.m > 0;
    max_m = std::max<int64_t>(max_m, pl.m);
    st = launch_conv2d(c, cv, H, W, Ho, Wo, in[i]->V, in[i]->ld, o->V, o->ld, pl.dense,
                       in[i]->rows_pending ? in[i]->cls : nullptr, pl.compact ? ob : nullptr, pl.dense_eh, pl.dense_ew,
                       pl.compact ? in[i]->box : nullptr, pl.compact && lazy);
    // (launch_conv2d zeroes the padding rows of the columns it writes; the stamp kernel only writes them when
    // it writes whole columns)
    if (st == NNVHIP_OK && stamps[i].win_only && o->ld != Nout) st = launch_zero_pad_rows(c, stamps[i].out, o->ld, Nout, pl.m);
  }
  if (st == NNVHIP_OK && any_stamps) {
    // the stamp pass also leaves the range sums of its columns on the output handles
    const int64_t sch = conv_stamp_chunks(cv, outs[0]->ld, count, max_m);
    BufRef sums;
    st = c->alloc(sizeof(double) * 4 * outs[0]->ld * sch * count, &sums);
    if (st == NNVHIP_OK) {
      for (int64_t i = 0; i < count; ++i) stamps[i].part = sums->as<double>() + 4 * outs[0]->ld * sch * i;
      st = launch_conv_stamps(c, cv, H, W, Ho, Wo, outs[0]->ld, count, stamps.data(), sch);
    }
    for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
      if (stamps[i].m > 0) {
        outs[i]->rng_buf = sums;
        outs[i]->rng_part = stamps[i].part;
        outs[i]->rng_chunks = sch;
        outs[i]->rng_first_col = (in[i]->n + 1) - stamps[i].m;
      }
  }
  if (st == NNVHIP_OK) st = c->end_op();
  if (st != NNVHIP_OK) {
    release_all(outs);
    return st;
  }
  for (int64_t i = 0; i < count; ++i) out[i] = outs[i];
  return NNVHIP_OK;
}

int nnvhip_relu_relax(nnvhip_ctx* c, int order, double relax_factor, int64_t count, nnvhip_star* const* in,
                      nnvhip_star** out) {
  CHECK_CTX(c);
  NNV_TRY(check_set_array(c, count, in, out));
  if (order != NNVHIP_ORDER_INDEX && order != NNVHIP_ORDER_AREA && order != NNVHIP_ORDER_RANGE)
    NNV_FAIL(NNVHIP_ERR_METHOD, "This reachability method does not exist");
  if (!(relax_factor >= 0.0 && relax_factor <= 1.0)) NNV_FAIL(NNVHIP_ERR_RELAX_FACTOR, "Invalid relax factor");
  if (relax_factor != 1.0)
    NNV_FAIL(NNVHIP_ERR_RELAX_FACTOR, "relaxFactor < 1 needs the LP-based range optimisation, which this library does not provide");
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N != in[0]->N) NNV_FAIL(NNVHIP_ERR_SHAPE, "sets of one array must have the same dimension");
  NNV_TRY(c->begin_op());
  NNV_TRY(relu_relax(c, order, count, in, out));
  return c->end_op();
}

int nnvhip_reach_layers(nnvhip_ctx* c, int64_t n_layers, const int32_t* kind, const void* const* layer, const int64_t* hw,
                        int order, double relax_factor, int64_t count, nnvhip_star* const* in, nnvhip_star** out) {
  if (!c) NNV_FAIL(NNVHIP_ERR_ARG, "null context");
  if (n_layers < 0 || count <= 0 || !in || (n_layers > 0 && (!kind || !layer || !out))) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  nnvhip_star* const* cur = in;
  int st = NNVHIP_OK;
  int64_t done = 0;
  if (n_layers > 0 && relax_factor == 1.0) {
    // small fully connected networks: the whole loop below as one launch
    NNV_TRY(nnvhip::enter_ctx(c));
    bool taken = false;
    for (int64_t t = 0; t < n_layers * count; ++t) out[t] = nullptr;
    st = reach_small_chain(c, n_layers, kind, layer, order, count, in, out, &taken);
    if (taken) {
      if (st != NNVHIP_OK)
        for (int64_t t = 0; t < n_layers * count; ++t) {
          nnvhip_star_release(out[t]);
          out[t] = nullptr;
        }
      return st;
    }
  }
  for (int64_t l = 0; l < n_layers && st == NNVHIP_OK; ++l) {
    nnvhip_star** dst = out + l * count;
    // the set that is handed back is written in full by the layer that produces it
    const bool eager = l == n_layers - 1 && !c->eager_cols;
    if (eager) c->eager_cols = true;
    switch (kind[l]) {
      case NNVHIP_LAYER_FC:
        st = nnvhip_affine_fc(c, static_cast<const nnvhip_fc*>(layer[l]), count, cur, dst);
        break;
      case NNVHIP_LAYER_CONV2D:
        if (!hw) {
          set_error("null argument");
          st = NNVHIP_ERR_ARG;
        } else {
          st = nnvhip_affine_conv2d(c, static_cast<const nnvhip_conv2d*>(layer[l]), hw[2 * l], hw[2 * l + 1], count, cur, dst);
        }
        break;
      case NNVHIP_LAYER_RELU:
        st = nnvhip_relu_relax(c, order, relax_factor, count, cur, dst);
        break;
      default:
        set_error("unknown layer kind %d", (int)kind[l]);
        st = NNVHIP_ERR_ARG;
    }
    if (eager) c->eager_cols = false;
    if (st == NNVHIP_OK) {
      cur = dst;
      done = l + 1;
    }
  }
  if (st != NNVHIP_OK) {
    for (int64_t t = 0; t < done * count; ++t) {
      nnvhip_star_release(out[t]);
      out[t] = nullptr;
    }
  }
  return st;
}

int nnvhip_relu_apply_lists(nnvhip_ctx* c, nnvhip_star* in, int64_t n_reset, const int32_t* reset_rows, int64_t m,
                            const int32_t* index, const double* lb, const double* ub, nnvhip_star** out) {
  CHECK_CTX(c);
  if (!in || in->ctx != c || !out) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle");
  if (n_reset < 0 || m < 0 || (n_reset > 0 && !reset_rows) || (m > 0 && (!index || !lb || !ub)))
    NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  const int64_t N = in->N;
  // per-row bounds that make the classification reproduce the two lists: a reset row looks inactive
  // (ub = 0), a listed neuron carries its own (lb, ub), every other row looks active; the keys put the
  // new predicates in the order of the list
  std::vector<double> rows((size_t)(3 * N));
  double* L = rows.data();
  double* U = L + N;
  double* K = U + N;
  std::vector<char> seen((size_t)N, 0);
  for (int64_t r = 0; r < N; ++r) {
    L[r] = 0.0;
    U[r] = 1.0;
    K[r] = 0.0;
  }
  for (int64_t t = 0; t < n_reset; ++t) {
    const int64_t r = reset_rows[t];
    if (r < 0 || r >= N) NNV_FAIL(NNVHIP_ERR_ARG, "Invalid index");
    if (seen[r]) NNV_FAIL(NNVHIP_ERR_ARG, "row %lld is listed twice", (long long)r);
    seen[r] = 1;
    L[r] = -1.0;
    U[r] = 0.0;
  }
  for (int64_t t = 0; t < m; ++t) {
    const int64_t r = index[t];
    if (r < 0 || r >= N) NNV_FAIL(NNVHIP_ERR_ARG, "Invalid index");
    if (seen[r]) NNV_FAIL(NNVHIP_ERR_ARG, "row %lld is listed twice", (long long)r);
    if (!(lb[t] < 0.0 && ub[t] > 0.0)) NNV_FAIL(NNVHIP_ERR_ARG, "neuron %lld: the triangle relaxation needs lb < 0 < ub", (long long)r);
    seen[r] = 1;
    L[r] = lb[t];
    U[r] = ub[t];
    K[r] = (double)(m - t);
  }
  NNV_TRY(c->begin_op());
  BufRef dev;
  NNV_TRY(c->upload(rows.data(), sizeof(double) * 3 * N, &dev));
  ReluGiven g{dev->as<double>(), dev->as<double>() + N, dev->as<double>() + 2 * N};
  NNV_TRY(relu_relax(c, kOrderGiven, 1, &in, out, &g));
  return c->end_op();
}

}  // extern "C"
