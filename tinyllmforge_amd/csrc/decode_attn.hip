// Paged decode attention for gfx950 (reference: the decode branch of
// tinyvllm/layers/attention.py:106-109, flash_attn_with_kvcache with one query
// token per sequence).
//
// HBM-bound streaming kernel.  A K (or V) cache row of one token holds all KV
// heads contiguously (Hkv * 128 bf16 = 2 KiB), so one workgroup owns a run of
// tokens of one sequence and ALL its KV heads: wave w <-> KV head w.  Together
// the waves read whole contiguous rows with 128-bit loads, and the Hq/Hkv query
// heads that share a KV head are served from a single pass over its rows
// (GQA sharing), so every cache byte is fetched exactly once.
//
// Per wave and 16-token tile:
//   global (4 x 128-bit loads per lane for K, 4 for V, issued one tile ahead)
//     -> LDS (row-major [token][dim], padded rows)
//   S^T[token, head] = K_tile . Q^T        4 x v_mfma_f32_16x16x32_bf16
//   online softmax in fp32 (row max / sum by two cross-lane exchanges)
//   O^T[dim, head]  += V_tile^T . P^T      8 x v_mfma_f32_16x16x16_bf16
// The MFMA output layout of S^T (lane = head, 4 tokens per lane) is exactly the
// B-operand layout of the second product, so P never leaves registers, and the
// softmax statistics of a head live in the lanes that hold its O^T columns.
// P is fed as a bf16 hi + lo pair (two MFMAs): matrix-core time is free in a
// bandwidth-bound kernel and it removes the bf16 rounding of the probabilities.
//
// Long sequences are cut into fixed-size partitions (grid = partitions x
// batch, independent of device data, so the launch can be graph-captured);
// partitions beyond a sequence's length exit at once.  Each partition writes
// (max, sum, unnormalised O) and a small second kernel merges them.
#include <stdlib.h>

#include "common.h"

namespace tlf {

constexpr int kDh = 128;
constexpr int kTile = 16;             // tokens per tile
constexpr int kLdsRow = kDh + 8;      // padded LDS row (elements): 272 B, shifts rows by 4 banks
constexpr float kLog2e = 1.4426950408889634f;

struct DecodeParams {
  const unsigned short *q;
  int64_t q_stride;
  const unsigned char *k_cache;
  const unsigned char *v_cache;
  const float *k_scale;
  const float *v_scale;
  const int32_t *block_tables;
  int64_t bt_stride;
  const int32_t *context_lens;
  unsigned short *out;
  float *part_o;   // [batch, nparts, Hq, 128]
  float *part_ml;  // [batch, nparts, Hq, 2]  (max in log2 domain, sum)
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t block_size;
  int32_t max_blocks;
  int64_t num_cache_blocks;
  int32_t part_tokens;
  int32_t nparts;
  float scale_log2;  // softmax scale * log2(e)
};

// One tile's worth of global data of one wave: 16 tokens x 128 dims of K and V.
struct TileRegs {
  uint4 k[4];
  uint4 v[4];
  bool ok;  // the tile's block-table entry names a real cache block
};

template <int NW>
__global__ __launch_bounds__(NW * 64) void paged_decode_kernel(const DecodeParams p) {
  __shared__ __attribute__((aligned(16))) unsigned short lds[NW][2][kTile][kLdsRow];
  const int b = blockIdx.y;
  const int part = blockIdx.x;
  // a length beyond the table's capacity would overrun block_tables: clamp it
  const int ctx = min(p.context_lens[b], p.max_blocks * p.block_size);
  const int t_begin = part * p.part_tokens;
  const int w = threadIdx.x >> 6;  // KV head
  const int lane = threadIdx.x & 63;
  const int n = lane & 15;  // query head inside the group (MFMA column)
  const int g = lane >> 4;
  const int group = p.num_q_heads / p.num_kv_heads;
  const int head = w * group + n;
  const bool head_ok = n < group;

  if (t_begin >= ctx) {
    if (p.nparts == 1 && head_ok) {  // empty sequence: zeros, nobody else writes this row
      unsigned short *o = p.out + (static_cast<int64_t>(b) * p.num_q_heads + head) * kDh;
#pragma unroll
      for (int d = 0; d < 8; ++d)
        *reinterpret_cast<uint2 *>(o + d * 16 + g * 4) = make_uint2(0, 0);
    }
    return;
  }
  const int t_end = min(ctx, t_begin + p.part_tokens);

  // Q as the B operand of S^T = K . Q^T: lane (n, g) holds q[head n][c*32 + g*8 .. +8].
  bf16x8 qf[4];
  {
    const unsigned short *qp = p.q + b * p.q_stride + static_cast<int64_t>(head) * kDh;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      Pack16 t;
      t.u = make_uint4(0, 0, 0, 0);
      if (head_ok) t.u = *reinterpret_cast<const uint4 *>(qp + c * 32 + g * 8);
      qf[c] = t.v;
    }
  }

  const int64_t row_elems = static_cast<int64_t>(p.num_kv_heads) * kDh;
  const int32_t *bt = p.block_tables + b * p.bt_stride;
  unsigned short(*Ks)[kLdsRow] = lds[w][0];
  unsigned short(*Vs)[kLdsRow] = lds[w][1];

  // Issue the loads of the tile starting at token t0 (a tile never straddles a block).
  auto load_tile = [&](int t0, TileRegs &r) {
    const int bi = t0 / p.block_size;
    const int64_t blk = bt[bi];
    const bool ok = blk >= 0 && blk < p.num_cache_blocks;
    const int64_t tok0 = (ok ? blk : 0) * p.block_size + (t0 - bi * p.block_size);
    r.ok = ok;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tt = i * 4 + g;  // token of this lane inside the tile
      const int64_t off = ((tok0 + tt) * row_elems + w * kDh + n * 8) * 2;
      const bool valid = ok && (t0 + tt) < t_end;
      r.k[i] = make_uint4(0, 0, 0, 0);
      r.v[i] = make_uint4(0, 0, 0, 0);
      if (valid) {
        r.k[i] = *reinterpret_cast<const uint4 *>(p.k_cache + off);
        r.v[i] = *reinterpret_cast<const uint4 *>(p.v_cache + off);
      }
    }
  };

  floatx4 acc[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) acc[d] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;  // running max (log2 domain), identical in the 4 lanes of a head
  float l_run = 0.f;        // this lane's share of the running sum

  TileRegs regs;
  load_tile(t_begin, regs);
  for (int t0 = t_begin; t0 < t_end; t0 += kTile) {
    wave_lds_fence();  // previous tile's LDS reads are done
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<uint4 *>(&Ks[i * 4 + g][n * 8]) = regs.k[i];
      *reinterpret_cast<uint4 *>(&Vs[i * 4 + g][n * 8]) = regs.v[i];
    }
    wave_lds_fence();
    const bool tile_ok = regs.ok;
    if (t0 + kTile < t_end) load_tile(t0 + kTile, regs);

    // S^T = K . Q^T : lane (n, g) gets tokens g*4 + i of head n
    floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      Pack16 a;
      a.u = *reinterpret_cast<const uint4 *>(&Ks[n][c * 32 + g * 8]);
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[c], s, 0, 0, 0);
    }
    float sv[4];
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool valid = tile_ok && (t0 + g * 4 + i) < t_end;
      sv[i] = valid ? s[i] * p.scale_log2 : -INFINITY;
      mt = fmaxf(mt, sv[i]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m_run, mt);
    // -inf only while every token so far sat in a skipped block: keep the exponents finite
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = exp2f(m_run - m_use);
    float psum = 0.f;
    bf16x4 pb, pl;  // p = hi + lo in bf16: the matrix cores are idle here, so P.V keeps ~16 bits of p
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float pv = exp2f(sv[i] - m_use);
      psum += pv;
      pb[i] = static_cast<__bf16>(pv);
      pl[i] = static_cast<__bf16>(pv - static_cast<float>(pb[i]));
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    const shortx4 pbs = __builtin_bit_cast(shortx4, pb);
    const shortx4 pls = __builtin_bit_cast(shortx4, pl);
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      // A = V^T fragment: lane (dim = d*16 + n, g) holds tokens g*4 + i
      shortx4 vf;
#pragma unroll
      for (int i = 0; i < 4; ++i) vf[i] = static_cast<short>(Vs[g * 4 + i][d * 16 + n]);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[d][i] *= alpha;
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pbs, acc[d], 0, 0, 0);
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pls, acc[d], 0, 0, 0);
    }
  }

  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (!head_ok) return;
  // lane (n, g) holds O^T[dims d*16 + g*4 + i][head n]
  if (p.nparts == 1) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    unsigned short *o = p.out + (static_cast<int64_t>(b) * p.num_q_heads + head) * kDh;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      uint2 st;
      st.x = pack_bf16x2(acc[d][0] * inv, acc[d][1] * inv);
      st.y = pack_bf16x2(acc[d][2] * inv, acc[d][3] * inv);
      *reinterpret_cast<uint2 *>(o + d * 16 + g * 4) = st;
    }
  } else {
    const int64_t slot = (static_cast<int64_t>(b) * p.nparts + part) * p.num_q_heads + head;
    float *po = p.part_o + slot * kDh;
#pragma unroll
    for (int d = 0; d < 8; ++d)
      *reinterpret_cast<float4 *>(po + d * 16 + g * 4) =
          make_float4(acc[d][0], acc[d][1], acc[d][2], acc[d][3]);
    if (g == 0) *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m_run, l_run);
  }
}

// Merge the partitions of one (sequence, head): one wave, two dims per lane.
__global__ __launch_bounds__(64) void paged_decode_combine_kernel(const DecodeParams p) {
  const int b = blockIdx.y;
  const int head = blockIdx.x;
  const int lane = threadIdx.x;
  const int ctx = min(p.context_lens[b], p.max_blocks * p.block_size);
  unsigned short *o = p.out + (static_cast<int64_t>(b) * p.num_q_heads + head) * kDh + lane * 2;
  if (ctx <= 0) {
    *reinterpret_cast<unsigned int *>(o) = 0u;
    return;
  }
  const int np = min(p.nparts, (ctx + p.part_tokens - 1) / p.part_tokens);
  const int64_t base = (static_cast<int64_t>(b) * p.nparts) * p.num_q_heads + head;
  float m = -INFINITY;
  for (int i = 0; i < np; ++i)
    m = fmaxf(m, p.part_ml[(base + static_cast<int64_t>(i) * p.num_q_heads) * 2]);
  float l = 0.f, a0 = 0.f, a1 = 0.f;
  for (int i = 0; i < np; ++i) {
    const int64_t slot = base + static_cast<int64_t>(i) * p.num_q_heads;
    const float2 ml = *reinterpret_cast<const float2 *>(p.part_ml + slot * 2);
    const float wgt = (ml.x == -INFINITY) ? 0.f : exp2f(ml.x - m);
    const float2 v = *reinterpret_cast<const float2 *>(p.part_o + slot * kDh + lane * 2);
    l += wgt * ml.y;
    a0 += wgt * v.x;
    a1 += wgt * v.y;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  *reinterpret_cast<unsigned int *>(o) = pack_bf16x2(a0 * inv, a1 * inv);
}

inline int decode_part_tokens() {
  static int cached = 0;
  if (cached == 0) {
    int v = 256;
    if (const char *e = getenv("TLF_DECODE_PART_TOKENS")) {
      const int x = atoi(e);
      if (x >= kTile && x % kTile == 0) v = x;
    }
    cached = v;
  }
  return cached;
}

inline int decode_nparts(int32_t max_blocks, int32_t block_size) {
  const int64_t max_tokens = static_cast<int64_t>(max_blocks) * block_size;
  const int pt = decode_part_tokens();
  return static_cast<int>((max_tokens + pt - 1) / pt);
}

}  // namespace tlf

using namespace tlf;

extern "C" size_t tlf_paged_decode_attn_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                        int32_t head_dim, int32_t max_blocks,
                                                        int32_t block_size) {
  if (batch <= 0 || num_q_heads <= 0 || head_dim <= 0 || max_blocks <= 0 || block_size <= 0)
    return 0;
  const size_t np = static_cast<size_t>(decode_nparts(max_blocks, block_size));
  const size_t slots = static_cast<size_t>(batch) * np * num_q_heads;
  return slots * (static_cast<size_t>(head_dim) + 2) * sizeof(float) + 256;
}

extern "C" int tlf_paged_decode_attn(const void *q, int64_t q_stride, const void *k_cache,
                                     const void *v_cache, int32_t kv_dtype, const float *k_scale,
                                     const float *v_scale, const int32_t *block_tables,
                                     int64_t block_table_stride, const int32_t *context_lens,
                                     void *out, int32_t batch, int32_t num_q_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                     int32_t max_blocks, int64_t num_cache_blocks, float scale,
                                     void *workspace, size_t workspace_bytes, void *stream) {
  if (batch == 0) return TLF_OK;
  if (!q || !k_cache || !v_cache || !block_tables || !context_lens || !out) return TLF_E_NULL;
  if (head_dim != kDh) return TLF_E_UNSUPPORTED;
  if (kv_dtype != TLF_KV_BF16) return TLF_E_UNSUPPORTED;
  if (batch < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || block_size <= 0 || max_blocks <= 0 ||
      num_cache_blocks <= 0)
    return TLF_E_SHAPE;
  if (num_q_heads % num_kv_heads || num_q_heads / num_kv_heads > 16 || block_size % kTile)
    return TLF_E_SHAPE;
  if (block_table_stride < max_blocks || q_stride < static_cast<int64_t>(num_q_heads) * head_dim)
    return TLF_E_SHAPE;
  if (!aligned16(q) || q_stride % 8 || !aligned16(k_cache) || !aligned16(v_cache) ||
      !aligned16(out))
    return TLF_E_ALIGN;
  (void)k_scale;
  (void)v_scale;

  DecodeParams p;
  p.q = static_cast<const unsigned short *>(q);
  p.q_stride = q_stride;
  p.k_cache = static_cast<const unsigned char *>(k_cache);
  p.v_cache = static_cast<const unsigned char *>(v_cache);
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.block_tables = block_tables;
  p.bt_stride = block_table_stride;
  p.context_lens = context_lens;
  p.out = static_cast<unsigned short *>(out);
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.block_size = block_size;
  p.max_blocks = max_blocks;
  p.num_cache_blocks = num_cache_blocks;
  p.part_tokens = decode_part_tokens();
  p.nparts = decode_nparts(max_blocks, block_size);
  p.scale_log2 = scale * kLog2e;
  p.part_o = nullptr;
  p.part_ml = nullptr;
  if (p.nparts > 1) {
    const size_t need =
        tlf_paged_decode_attn_workspace_bytes(batch, num_q_heads, head_dim, max_blocks, block_size);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
      return TLF_E_WORKSPACE;
    const size_t slots = static_cast<size_t>(batch) * p.nparts * num_q_heads;
    p.part_o = static_cast<float *>(workspace);
    p.part_ml = p.part_o + slots * kDh;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(p.nparts, batch);
  switch (num_kv_heads) {
    case 1: hipLaunchKernelGGL(paged_decode_kernel<1>, grid, dim3(64), 0, s, p); break;
    case 2: hipLaunchKernelGGL(paged_decode_kernel<2>, grid, dim3(128), 0, s, p); break;
    case 4: hipLaunchKernelGGL(paged_decode_kernel<4>, grid, dim3(256), 0, s, p); break;
    case 8: hipLaunchKernelGGL(paged_decode_kernel<8>, grid, dim3(512), 0, s, p); break;
    case 16: hipLaunchKernelGGL(paged_decode_kernel<16>, grid, dim3(1024), 0, s, p); break;
    default: return TLF_E_UNSUPPORTED;
  }
  int rc = launch_status();
  if (rc != TLF_OK) return rc;
  if (p.nparts > 1) {
    hipLaunchKernelGGL(paged_decode_combine_kernel, dim3(num_q_heads, batch), dim3(64), 0, s, p);
    rc = launch_status();
  }
  return rc;
}
