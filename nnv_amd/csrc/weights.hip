// Layer handles (fully connected, convolution) and the per-context weight cache that recognises arrays it has
// uploaded before.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>

#include "internal.h"

namespace nnvhip {

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

}  // namespace nnvhip

using namespace nnvhip;

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

extern "C" {

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
  fc->uid = ++c->next_layer_uid;
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
  if (fc->refs.fetch_sub(1) == 1) {
    if (c->next_fc == fc) c->next_fc = nullptr;
    delete fc;
  }
  c->live_handles--;
  return NNVHIP_OK;
}

int nnvhip_hint_next_fc(nnvhip_ctx* c, const nnvhip_fc* fc) {
  CHECK_CTX(c);
  if (fc != nullptr && fc->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "layer of another context");
  c->next_fc = fc;
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
