// Slot-mapped KV-cache write (reference: tinyvllm/layers/attention.py:9-48).
//
// A K (or V) row is Hkv*Dh elements = 2 KiB in bf16: the first half of a workgroup moves K rows, the
// second half V rows, 16 bytes per lane, so every global access is a fully coalesced 128-bit one.
// A workgroup moves TOK consecutive tokens and a lane has all its TOK loads in flight before its first
// store: with one token per workgroup the kernel is bound by load latency and by the rate at which
// 4 KiB workgroups can be started, not by HBM.
// HBM bound: 2 * row_bytes read + 2 * row_bytes written per token.
#include "common.h"

namespace tlf {

constexpr int kStoreThreads = 256;

template <int TOK>
__global__ __launch_bounds__(kStoreThreads) void store_kvcache_kernel(
    const unsigned char *__restrict__ key, int64_t key_stride,
    const unsigned char *__restrict__ value, int64_t value_stride,
    unsigned char *__restrict__ k_cache, unsigned char *__restrict__ v_cache,
    const int32_t *__restrict__ slot_mapping, int32_t num_tokens, int32_t row_bytes, int64_t num_slots) {
  const int half = kStoreThreads / 2;
  const bool is_v = threadIdx.x >= half;
  const int lane = is_v ? threadIdx.x - half : threadIdx.x;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * TOK;
  const unsigned char *src = is_v ? value : key;
  const int64_t stride = is_v ? value_stride : key_stride;
  unsigned char *cache = is_v ? v_cache : k_cache;
  int64_t slot[TOK];
#pragma unroll
  for (int i = 0; i < TOK; ++i) {
    slot[i] = tok0 + i < num_tokens ? slot_mapping[tok0 + i] : -1;
    if (slot[i] >= num_slots) slot[i] = -1;   // padding row: leave the cache alone
  }
  for (int off = lane * 16; off < row_bytes; off += half * 16) {
    uint4 v[TOK];
#pragma unroll
    for (int i = 0; i < TOK; ++i)
      if (slot[i] >= 0) v[i] = load_nt_u4(src + (tok0 + i) * stride + off);
#pragma unroll
    for (int i = 0; i < TOK; ++i)
      if (slot[i] >= 0) *reinterpret_cast<uint4 *>(cache + slot[i] * static_cast<int64_t>(row_bytes) + off) = v[i];
  }
}

// bf16 rows -> e4m3 rows: each lane converts 8 elements (16 B in, 8 B out).
__global__ __launch_bounds__(kStoreThreads) void store_kvcache_fp8_kernel(
    const unsigned char *__restrict__ key, int64_t key_stride,
    const unsigned char *__restrict__ value, int64_t value_stride,
    unsigned char *__restrict__ k_cache, unsigned char *__restrict__ v_cache,
    const int32_t *__restrict__ slot_mapping, int32_t num_kv_heads, int32_t head_dim,
    const float *__restrict__ k_scale, const float *__restrict__ v_scale, int64_t num_slots) {
  const int token = blockIdx.x;
  const int64_t slot = slot_mapping[token];
  if (slot < 0 || slot >= num_slots) return;
  const int half = kStoreThreads / 2;
  const bool is_v = threadIdx.x >= half;
  const int lane = is_v ? threadIdx.x - half : threadIdx.x;
  const int row_elems = num_kv_heads * head_dim;
  const unsigned char *src = is_v ? value + token * value_stride : key + token * key_stride;
  unsigned char *dst = (is_v ? v_cache : k_cache) + slot * static_cast<int64_t>(row_elems);
  const float *scale = is_v ? v_scale : k_scale;
  for (int e = lane * 8; e < row_elems; e += half * 8) {
    const uint4 p = *reinterpret_cast<const uint4 *>(src + static_cast<int64_t>(e) * 2);
    float f[8];
    unpack8(p, f);
    const float s = scale[e / head_dim];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = fminf(fmaxf(f[i] / s, -448.0f), 448.0f);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
    *reinterpret_cast<int2 *>(dst + e) = make_int2(lo, hi);
  }
}

}  // namespace tlf

extern "C" int tlf_store_kvcache(const void *key, int64_t key_stride_bytes, const void *value,
                                 int64_t value_stride_bytes, void *k_cache, void *v_cache,
                                 const int32_t *slot_mapping, int32_t num_tokens,
                                 int32_t row_bytes, int64_t num_slots, void *stream) {
  using namespace tlf;
  if (num_tokens == 0) return TLF_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping) return TLF_E_NULL;
  if (num_tokens < 0 || row_bytes <= 0 || num_slots <= 0) return TLF_E_SHAPE;
  if (row_bytes % 16 || key_stride_bytes % 16 || value_stride_bytes % 16 || !aligned16(key) ||
      !aligned16(value) || !aligned16(k_cache) || !aligned16(v_cache))
    return TLF_E_ALIGN;
  if (key_stride_bytes < row_bytes || value_stride_bytes < row_bytes) return TLF_E_SHAPE;
  if (num_tokens >= 2048)
    TLF_LAUNCH(store_kvcache_kernel<8>, dim3((num_tokens + 7) / 8), dim3(kStoreThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const unsigned char *>(key),
                       key_stride_bytes, static_cast<const unsigned char *>(value),
                       value_stride_bytes, static_cast<unsigned char *>(k_cache),
                       static_cast<unsigned char *>(v_cache), slot_mapping, num_tokens, row_bytes, num_slots);
  else
    TLF_LAUNCH(store_kvcache_kernel<1>, dim3(num_tokens), dim3(kStoreThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<const unsigned char *>(key),
                       key_stride_bytes, static_cast<const unsigned char *>(value),
                       value_stride_bytes, static_cast<unsigned char *>(k_cache),
                       static_cast<unsigned char *>(v_cache), slot_mapping, num_tokens, row_bytes, num_slots);
  return launch_status();
}

extern "C" int tlf_store_kvcache_fp8(const void *key, int64_t key_stride_bytes, const void *value,
                                     int64_t value_stride_bytes, void *k_cache, void *v_cache,
                                     const int32_t *slot_mapping, int32_t num_tokens,
                                     int32_t num_kv_heads, int32_t head_dim, const float *k_scale,
                                     const float *v_scale, int64_t num_slots, void *stream) {
  using namespace tlf;
  if (num_tokens == 0) return TLF_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping || !k_scale || !v_scale)
    return TLF_E_NULL;
  if (num_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || num_slots <= 0) return TLF_E_SHAPE;
  if (head_dim % 8) return TLF_E_SHAPE;
  const int64_t row_bytes_in = static_cast<int64_t>(num_kv_heads) * head_dim * 2;
  if (key_stride_bytes % 16 || value_stride_bytes % 16 || !aligned16(key) || !aligned16(value) ||
      (reinterpret_cast<uintptr_t>(k_cache) & 7u) || (reinterpret_cast<uintptr_t>(v_cache) & 7u))
    return TLF_E_ALIGN;
  if (key_stride_bytes < row_bytes_in || value_stride_bytes < row_bytes_in) return TLF_E_SHAPE;
  TLF_LAUNCH(store_kvcache_fp8_kernel, dim3(num_tokens), dim3(kStoreThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const unsigned char *>(key),
                     key_stride_bytes, static_cast<const unsigned char *>(value),
                     value_stride_bytes, static_cast<unsigned char *>(k_cache),
                     static_cast<unsigned char *>(v_cache), slot_mapping, num_kv_heads, head_dim,
                     k_scale, v_scale, num_slots);
  return launch_status();
}
