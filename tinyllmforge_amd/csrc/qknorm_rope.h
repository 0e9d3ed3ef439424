// q/k RMSNorm + RoPE + KV-cache store of one 8-value piece of the qkv projection, shared by the kernel that
// reads the projection as bf16 rows and by the one that first sums the fp32 partials of a projection whose K
// was split across workgroups.
#pragma once

#include "common.h"

namespace tlf {

struct QkRopeStoreArgs {
  const unsigned short *qw;   // q_norm weight [128]
  const unsigned short *kw;   // k_norm weight [128]
  float eps;
  const int64_t *positions;
  const float *cos_sin;       // fp32 [max_pos, 128] = cos || sin
  int32_t max_pos;
  unsigned short *q_out;      // [n, Hq * 128]
  unsigned short *k_out;      // [n, Hkv * 128] or null
  unsigned short *v_out;
  unsigned char *k_cache;
  unsigned char *v_cache;
  const int32_t *slot_mapping;  // null: no cache store
  int64_t num_slots;
  int32_t kv_dtype;
  const float *k_scale;
  const float *v_scale;
  int32_t num_q_heads;
  int32_t num_kv_heads;
};

// (reference op sequence: tinyvllm/models/qwen3.py:79-94, layers/attention.py:94-95)
// 16 lanes own one head (8 dims each); lanes j < 8 hold the first half of the head, lanes j >= 8 the second,
// so the RoPE partner of lane j is lane j ^ 8.  The work on one 8-value piece comes in three steps, so that a
// kernel that handles several tokens per lane can issue every step's loads for all of them before it waits:
//   1. qk_piece_meta: the token's position and cache slot (one load each);
//   2. qk_piece_table: this lane's 8 cosines and 8 sines of that position (q and k heads only);
//   3. qk_piece_finish: norm, rotation and the stores.
struct QkPieceMeta {
  int64_t pos;    // the token's position (q and k heads)
  int64_t slot;   // cache slot of the token, or -1: no cache store (k and v heads)
};
struct QkPieceTable {
  float4 c0, c1, s0, s1;   // cos[8], sin[8] of this lane's dims
};

__device__ __forceinline__ QkPieceMeta qk_piece_meta(int64_t tok, int head, const QkRopeStoreArgs &a) {
  QkPieceMeta m;
  m.pos = 0;
  m.slot = -1;
  const bool is_q = head < a.num_q_heads;
  const bool is_v = head >= a.num_q_heads + a.num_kv_heads;
  if (!is_v) m.pos = a.positions[tok];
  if (!is_q && a.slot_mapping != nullptr) {
    m.slot = a.slot_mapping[tok];
    if (m.slot >= a.num_slots) m.slot = -1;
  }
  return m;
}

__device__ __forceinline__ QkPieceTable qk_piece_table(const QkPieceMeta &m, int head, int j, const QkRopeStoreArgs &a) {
  QkPieceTable t;
  t.c0 = t.c1 = t.s0 = t.s1 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (head < a.num_q_heads + a.num_kv_heads) {
    const bool pos_ok = m.pos >= 0 && m.pos < a.max_pos;
    const float *cs = a.cos_sin + (pos_ok ? m.pos : 0) * 128 + (j % 8) * 8;
    t.c0 = *reinterpret_cast<const float4 *>(cs);
    t.c1 = *reinterpret_cast<const float4 *>(cs + 4);
    t.s0 = *reinterpret_cast<const float4 *>(cs + 64);
    t.s1 = *reinterpret_cast<const float4 *>(cs + 68);
  }
  return t;
}

// raw = this lane's 8 bf16 values of token tok, head `head` (q heads first, then k, then v); all 16 lanes of
// a head call together.
__device__ __forceinline__ void qk_piece_finish(const uint4 raw, int64_t tok, int head, int j, const QkPieceMeta &m,
                                                const QkPieceTable &t, const QkRopeStoreArgs &a) {
  constexpr int kDh = 128;
  const int num_q_heads = a.num_q_heads, num_kv_heads = a.num_kv_heads;
  const bool is_q = head < num_q_heads;
  const bool is_k = !is_q && head < num_q_heads + num_kv_heads;
  const int kvh = is_q ? 0 : (is_k ? head - num_q_heads : head - num_q_heads - num_kv_heads);
  const int64_t slot = m.slot;
  uint4 outp = raw;
  if (is_q || is_k) {
    float v[8];
    unpack8(raw, v);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(v[i], v[i], ss);
    // sum over the head's 16 lanes: rotations by 8, 4, 2, 1 inside the row add the same pairs, in the same
    // order, as a butterfly over lane ^ 8, 4, 2, 1 would (after each step the partial sums repeat with that
    // period), so every lane of the head ends with the same bits
    ss += row_ror<8>(ss);
    ss += row_ror<4>(ss);
    ss += row_ror<2>(ss);
    ss += row_ror<1>(ss);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(kDh) + a.eps);
    float w[8];
    unpack8(*reinterpret_cast<const uint4 *>((is_q ? a.qw : a.kw) + j * 8), w);
    float nrm[8], other[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float nn = bf16_bits_to_float(float_to_bf16_bits(__fmul_rn(v[i], inv)));
      nrm[i] = bf16_bits_to_float(float_to_bf16_bits(__fmul_rn(nn, w[i])));
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) other[i] = row_ror<8>(nrm[i]);   // lane j ^ 8
    const bool pos_ok = m.pos >= 0 && m.pos < a.max_pos;
    const float cosv[8] = {t.c0.x, t.c0.y, t.c0.z, t.c0.w, t.c1.x, t.c1.y, t.c1.z, t.c1.w};
    const float sinv[8] = {t.s0.x, t.s0.y, t.s0.z, t.s0.w, t.s1.x, t.s1.y, t.s1.z, t.s1.w};
    float o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // lanes j < 8: cos*x1 - sin*x2 ; lanes j >= 8: cos*x2 + sin*x1
      const float x = __fmul_rn(cosv[i], nrm[i]);
      const float y = __fmul_rn(sinv[i], other[i]);
      o[i] = (j < 8) ? __fsub_rn(x, y) : __fadd_rn(x, y);
      if (!pos_ok) o[i] = nrm[i];
    }
    outp = pack8(o);
  }
  if (is_q) {
    *reinterpret_cast<uint4 *>(a.q_out + tok * static_cast<int64_t>(num_q_heads) * kDh + head * kDh + j * 8) = outp;
    return;
  }
  const int64_t row_elems = static_cast<int64_t>(num_kv_heads) * kDh;
  unsigned short *lin = is_k ? a.k_out : a.v_out;
  if (lin != nullptr) *reinterpret_cast<uint4 *>(lin + tok * row_elems + kvh * kDh + j * 8) = outp;
  if (slot < 0) return;
  unsigned char *cache = is_k ? a.k_cache : a.v_cache;
  if (a.kv_dtype == TLF_KV_BF16) {
    *reinterpret_cast<uint4 *>(cache + (slot * row_elems + kvh * kDh + j * 8) * 2) = outp;
  } else {
    float f[8];
    unpack8(outp, f);
    const float s = (is_k ? a.k_scale : a.v_scale)[kvh];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = fminf(fmaxf(f[i] / s, -448.0f), 448.0f);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
    *reinterpret_cast<int2 *>(cache + slot * row_elems + kvh * kDh + j * 8) = make_int2(lo, hi);
  }
}

// The three steps on one piece.
__device__ __forceinline__ void qknorm_rope_store_piece(const uint4 raw, int64_t tok, int head, int j,
                                                        const QkRopeStoreArgs &a) {
  const QkPieceMeta m = qk_piece_meta(tok, head, a);
  const QkPieceTable t = qk_piece_table(m, head, j, a);
  qk_piece_finish(raw, tok, head, j, m, t, a);
}

// Argument checks shared by the entry points that end in this step; fills `a` (q_out .. v_scale as given).
int check_qk_rope_store_args(const void *q_norm_weight, const void *k_norm_weight, const int64_t *positions,
                             const float *cos_sin, int32_t max_pos, const void *q_out, const void *k_out,
                             const void *v_out, const void *k_cache, const void *v_cache,
                             const int32_t *slot_mapping, int64_t num_slots, int32_t kv_dtype,
                             const float *k_scale, const float *v_scale, int32_t n, int32_t num_q_heads,
                             int32_t num_kv_heads, int32_t head_dim);

}  // namespace tlf
