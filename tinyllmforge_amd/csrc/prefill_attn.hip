// Varlen causal prefill attention for gfx950 (reference: the prefill branch of
// tinyvllm/layers/attention.py:96-105, flash_attn_varlen_func with causal=True,
// optionally reading K/V from the paged cache through block tables).
//
// MFMA-bound flash-style kernel.  A workgroup owns one sequence, one KV head and
// a tile of query rows, and serves ALL Hq/Hkv query heads of that KV head, so a
// K/V tile staged in LDS is reused by every head of the group.  The (row, head)
// pairs of the tile are flattened into 64*CT "units"; a wave owns CT column
// tiles of 16 units.
//
// Per 64-token K/V tile (global -> registers one tile ahead -> LDS, row-major):
//   S^T[token, unit] = K . Q^T          v_mfma_f32_16x16x32_bf16, Q fragments in registers
//   online softmax in fp32; causal mask bottom-right aligned
//   O^T[dim, unit]  += V^T . P^T        v_mfma_f32_16x16x32_bf16; the V^T operand comes
//                                       straight from the row-major tile with
//                                       ds_read_b64_tr_b16 (LDS transpose read)
// The rows of the K operand are permuted so that the S^T accumulator layout of
// two 16-token sub-tiles is exactly the 32-token B operand of the second product:
// P never leaves registers.
//
// The second product runs in fp16 (v_mfma_f32_16x16x32_f16): fp16 keeps 11 significant bits of P (a single
// bf16 P, 8 bits, misses the 1e-3 relative-L2 bar against an exact softmax; a bf16 hi + lo pair meets it at
// twice the MFMAs and three more vector-ALU operations per score), and V is converted to fp16 once, when its
// tile is staged (exact for e4m3 rows).  Two guards keep the input domain that of bf16 operands:
//  - P is carried as 2^15 p (the factor sits in the exponent argument and in the running sum alike, so it
//    cancels in O / l): weights down to 2^-29 of the row maximum are normal fp16 numbers.  Unscaled, every
//    weight below 2^-14 would be an fp16 subnormal, and a row with one dominant key and thousands of faint ones
//    would lose their mass from the numerator but not from the denominator.
//  - a bf16 V tile that fp16 cannot hold (some |v| >= 65536, or no element as large as 2^-9, where the whole
//    tile would sit in or near the subnormal range) ends the workgroup: the staging threads vote on every
//    64-token tile, and on such a tile the workgroup writes a marker (a NaN pattern no arithmetic produces) into
//    the first output element of its row tile and leaves.  A second launch of the same grid (MODE 1) looks at
//    that element, returns at once where the marker is absent, and otherwise computes the row tile again with
//    both products in bf16 (P as a bf16 hi + lo pair, no 2^15 factor), which holds whatever bf16 holds.  Real
//    checkpoints never take it; keeping it in a launch of its own keeps its registers and branches out of the
//    fp16 kernel (inside one kernel the same choice cost 20-30 % on every call).
#include <stdlib.h>

#include "common.h"

namespace tlf {

constexpr int kPDh = 128;
constexpr int kBKV = 64;            // K/V tokens per LDS tile
// Padded LDS rows (elements; LDS has 32 banks of 4 bytes).  K fragments are read 16 bytes per lane from 8
// consecutive rows at a time: 272-byte rows.  V is read transposed, 8 bytes per lane, 4 lanes per row and
// 4 rows at a time: 288-byte rows.
constexpr int kPRowK = kPDh + 8;
constexpr int kPRowV = kPDh + 16;
typedef _Float16 f16x8 __attribute__((__vector_size__(8 * sizeof(_Float16))));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// LDS row of token t (0..63) of a K tile: within each half of 32 tokens, token 8 a + 4 s + b sits in row
// 16 s + 4 a + b, so that the 16 rows a fragment read addresses (tokens 8 a + b, or 8 a + 4 + b) are
// consecutive.
__device__ __forceinline__ int k_tile_row(int t) {
  return (t & 32) | ((t & 4) << 2) | ((t & 24) >> 1) | (t & 3);
}

// Head dimension held by LDS column c of a K or V tile.  bf16 rows are stored as they come.  e4m3 rows are
// stored with their 16-byte halves regrouped (columns 0..63: dims 16 j + 0..7, columns 64..127: dims
// 16 j + 8..15) so that the conversion's LDS writes are conflict free; the first product sums over columns
// (q is read with the same permutation) and the second product's output rows are columns (mapped back when
// written).  Runs of 8 columns stay runs of 8 dims.
template <bool KV8>
__device__ __forceinline__ int tile_col_dim(int c) {
  if (!KV8) return c;
  const int j = (c >> 3) & 7;
  return j * 16 + (c >= 64 ? 8 : 0) + (c & 7);
}

// Two bf16 (one dword) -> two fp16 (see the head of this file for the range).
__device__ __forceinline__ unsigned int bf16x2_to_f16x2(unsigned int w) {
  return __builtin_bit_cast(unsigned int,
                            __builtin_amdgcn_cvt_pkrtz(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u)));
}
__device__ __forceinline__ unsigned int pack_f16x2(float lo, float hi) {  // round to nearest even
  f16x2 r;
  r[0] = static_cast<_Float16>(lo);
  r[1] = static_cast<_Float16>(hi);
  return __builtin_bit_cast(unsigned int, r);
}
constexpr float kPLog2e = 1.4426950408889634f;
constexpr float kPShift = 15.0f;          // P is carried as 2^15 p
// bf16 bit patterns (sign cleared) that bound what a tile may hold for the fp16 product
constexpr unsigned int kVBigBits = 0x4780u;     // 65536: the first bf16 above the largest finite fp16
constexpr unsigned int kVDecentBits = 0x3b00u;  // 2^-9
constexpr unsigned short kRedoMarker = 0xffa5u;  // bf16 NaN with a payload: "compute this row tile again in bf16"
typedef unsigned short ushortx2 __attribute__((ext_vector_type(2)));

struct PrefillParams {
  const unsigned short *q;
  int64_t q_stride;
  const unsigned char *k;
  const unsigned char *v;
  int64_t k_stride, v_stride;  // elements, packed layout only
  const float *k_scale;
  const float *v_scale;
  const int32_t *cu_q;
  const int32_t *cu_k;
  const int32_t *block_tables;  // NULL: packed K/V
  int64_t bt_stride;
  unsigned short *out;
  int32_t num_q_heads, num_kv_heads;
  int32_t block_size;
  int64_t num_cache_blocks;
  float scale_log2;
  int32_t pair_group;  // (sequence, KV head) pairs an XCD walks together, row tiles outermost
};

// LDS transpose read: within each group of 16 lanes, lane i receives
// {row0[i], row1[i], row2[i], row3[i]} where row j is the 16 elements addressed
// (4 each) by lanes 4j .. 4j+3 of the group.
__device__ __forceinline__ shortx4 lds_read_tr16(const unsigned short *p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (shortx4 __attribute__((address_space(3))) *)(p));
}

__device__ __forceinline__ void fp8x16_to_bf16(const uint4 &in, uint4 &lo, uint4 &hi) {
  fp8x4_to_bf16x4(in.x, lo.x, lo.y);
  fp8x4_to_bf16x4(in.y, lo.z, lo.w);
  fp8x4_to_bf16x4(in.z, hi.x, hi.y);
  fp8x4_to_bf16x4(in.w, hi.z, hi.w);
}
__device__ __forceinline__ void fp8x4_to_f16x4(unsigned int w, unsigned int &lo, unsigned int &hi) {
  lo = __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
  hi = __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
}
__device__ __forceinline__ void fp8x16_to_f16(const uint4 &in, uint4 &lo, uint4 &hi) {
  fp8x4_to_f16x4(in.x, lo.x, lo.y);
  fp8x4_to_f16x4(in.y, lo.z, lo.w);
  fp8x4_to_f16x4(in.z, hi.x, hi.y);
  fp8x4_to_f16x4(in.w, hi.z, hi.w);
}

// acc[d0 .. d0 + 3] *= alpha unless alpha == 1 in every lane.
__device__ __forceinline__ void rescale16(floatx4 (&acc)[8], int d0, float alpha) {
  const unsigned long long moved = __builtin_amdgcn_ballot_w64(alpha != 1.0f);
  float t[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) t[e] = acc[d0 + e / 4][e % 4];
  asm volatile(
      "s_cmp_eq_u64 %[m], 0\n\t"
      "s_cbranch_scc1 .Ltlf_keep%=\n\t"
      "v_mul_f32_e32 %0, %[a], %0\n\tv_mul_f32_e32 %1, %[a], %1\n\tv_mul_f32_e32 %2, %[a], %2\n\t"
      "v_mul_f32_e32 %3, %[a], %3\n\tv_mul_f32_e32 %4, %[a], %4\n\tv_mul_f32_e32 %5, %[a], %5\n\t"
      "v_mul_f32_e32 %6, %[a], %6\n\tv_mul_f32_e32 %7, %[a], %7\n\tv_mul_f32_e32 %8, %[a], %8\n\t"
      "v_mul_f32_e32 %9, %[a], %9\n\tv_mul_f32_e32 %10, %[a], %10\n\tv_mul_f32_e32 %11, %[a], %11\n\t"
      "v_mul_f32_e32 %12, %[a], %12\n\tv_mul_f32_e32 %13, %[a], %13\n\tv_mul_f32_e32 %14, %[a], %14\n\t"
      "v_mul_f32_e32 %15, %[a], %15\n"
      ".Ltlf_keep%=:"
      : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]),
        "+v"(t[8]), "+v"(t[9]), "+v"(t[10]), "+v"(t[11]), "+v"(t[12]), "+v"(t[13]), "+v"(t[14]), "+v"(t[15])
      : [a] "v"(alpha), [m] "s"(moved)
      : "scc");
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[d0 + e / 4][e % 4] = t[e];
}

// MODE 0: second product in fp16 (bf16 rows: leaves a marker and returns on a tile fp16 cannot hold);
// MODE 1 (bf16 rows only): both products in bf16, for the row tiles that carry the marker.
template <int CT, bool KV8, int NWV, int MODE>
__global__ __launch_bounds__(64 * NWV) __attribute__((amdgpu_waves_per_eu(2, 2)))  // 256 registers: two waves per SIMD
void prefill_attn_kernel(const PrefillParams p) {
  static_assert(MODE == 0 || !KV8, "e4m3 rows always fit fp16");
  constexpr bool VB16 = MODE == 1;
  __shared__ __attribute__((aligned(16))) unsigned short Ks[kBKV][kPRowK];  // bf16, rows in k_tile_row order
  __shared__ __attribute__((aligned(16))) unsigned short Vs[kBKV][kPRowV];  // fp16 (bf16 for a tile fp16 cannot hold)
  __shared__ __attribute__((aligned(16))) unsigned int vvote[8];            // per wave: what its V slice holds
  // Workgroup -> (sequence, KV head, row tile).  Workgroups go to the 8 XCDs round robin by their linear id, and
  // each XCD has its own L2: when the (sequence, KV head) pairs divide evenly, pair j runs entirely on XCD j % 8,
  // so the K/V rows its row tiles share are fetched into one L2 instead of eight.  An XCD takes its pairs
  // pair_group at a time and walks their row tiles together, the last row tiles (the longest key ranges) first,
  // so that the launch ends on short workgroups.
  int seq = blockIdx.z, h = blockIdx.y, xt = blockIdx.x;
  const int pairs = gridDim.y * gridDim.z;
  if (pairs % 8 == 0) {
    const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const int slot = lin >> 3;
    const int gx = static_cast<int>(gridDim.x), G = p.pair_group;   // G divides pairs / 8 (host)
    const int grp = slot / (G * gx), within = slot % (G * gx);
    const int pair = (lin & 7) + 8 * (grp * G + within % G);
    xt = within / G;
    h = pair % static_cast<int>(gridDim.y);
    seq = pair / static_cast<int>(gridDim.y);
  }
  const int group = p.num_q_heads / p.num_kv_heads;
  const int bq = (16 * NWV * CT) / group;  // query rows per workgroup
  const int row0 = (gridDim.x - 1 - xt) * bq;
  const int q_begin = p.cu_q[seq];
  const int lq = p.cu_q[seq + 1] - q_begin;
  if (row0 >= lq) return;
  const int k_begin = p.cu_k[seq];
  const int lk = p.cu_k[seq + 1] - k_begin;
  const int shift = lk - lq;  // cached prefix length: query i sees keys 0 .. shift + i
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int n = lane & 15, g = lane >> 4;
  // first output element of this workgroup's row tile (row row0, first head of the KV head's group)
  unsigned short *const marker =
      p.out + (static_cast<int64_t>(q_begin + row0) * p.num_q_heads + static_cast<int64_t>(h) * group) * kPDh;
  if (MODE == 1 && *marker != kRedoMarker) return;   // workgroup uniform

  // units of this lane: u = wave*CT*16 + c*16 + n -> (row, head)
  int urow[CT];
  bool uok[CT];
  bf16x8 qf[CT][4];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int u = wave * CT * 16 + c * 16 + n;
    urow[c] = row0 + u / group;
    const int head = h * group + u % group;
    uok[c] = urow[c] < lq;
    const unsigned short *qp =
        p.q + static_cast<int64_t>(q_begin + urow[c]) * p.q_stride + static_cast<int64_t>(head) * kPDh;
#pragma unroll
    for (int kc = 0; kc < 4; ++kc) {
      Pack16 t;
      t.u = make_uint4(0, 0, 0, 0);
      if (uok[c]) t.u = *reinterpret_cast<const uint4 *>(qp + tile_col_dim<KV8>(kc * 32 + g * 8));
      qf[c][kc] = t.v;
    }
  }

  const int last_row = min(row0 + bq, lq) - 1;
  const int kv_end = min(lk, shift + last_row + 1);
  const int32_t *bt = p.block_tables ? p.block_tables + seq * p.bt_stride : nullptr;
  // e4m3 rows are dequantised as float(c) * scale[h]: the K scale is a constant factor of the scores
  const float scale_log2 = p.scale_log2 * (KV8 ? p.k_scale[h] : 1.0f);
  const int64_t cache_row = static_cast<int64_t>(p.num_kv_heads) * kPDh;

  // K/V tile loader: bf16 rows are 16 chunks of 16 B, e4m3 rows 8 chunks of 16 B.
  constexpr int kChunks = KV8 ? 8 : 16;
  constexpr int kThreads = 64 * NWV;
  constexpr int kPasses = kBKV * kChunks / kThreads;
  uint4 kreg[kPasses], vreg[kPasses];
  // Address arithmetic is kept off the vector ALU as far as possible (this kernel is VALU bound):
  // everything that depends on the thread only is computed once, the tile's share is scalar.
  constexpr int kRowsPerPass = kThreads / kChunks;
  const int trow = tid / kChunks, ch = tid % kChunks;
  const int64_t k_thread = (static_cast<int64_t>(k_begin + trow) * p.k_stride + h * kPDh + ch * 8) * 2;
  const int64_t v_thread = (static_cast<int64_t>(k_begin + trow) * p.v_stride + h * kPDh + ch * 8) * 2;
  const int64_t cache_row_bytes = cache_row * (KV8 ? 1 : 2);
  const int64_t paged_thread = static_cast<int64_t>(h) * kPDh * (KV8 ? 1 : 2) + ch * 16;
  const int bs_shift = (p.block_size & (p.block_size - 1)) == 0 ? __builtin_ctz(p.block_size) : -1;
  // Rows at or past kv_end are masked for every unit of this workgroup and get probability 0, so
  // they only have to be finite: their loads re-read row kv_end-1 instead of being predicated.
  auto load_tile = [&](int kv0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int tk = kv0 + i * kRowsPerPass + trow;
      if (bt == nullptr) {  // uniform
        // scalar part of the row index, clamped per thread through a row delta
        const int back = max(tk - (kv_end - 1), 0);  // rows to step back, 0 for a real row
        const int64_t tile_k = static_cast<int64_t>(kv0 + i * kRowsPerPass) * p.k_stride * 2;
        const int64_t tile_v = static_cast<int64_t>(kv0 + i * kRowsPerPass) * p.v_stride * 2;
        kreg[i] = *reinterpret_cast<const uint4 *>(p.k + (k_thread + tile_k - back * (p.k_stride * 2)));
        vreg[i] = *reinterpret_cast<const uint4 *>(p.v + (v_thread + tile_v - back * (p.v_stride * 2)));
      } else {
        const int tc = min(tk, kv_end - 1);
        int bi, within;
        if (bs_shift >= 0) {  // uniform: block sizes are powers of two in practice
          bi = tc >> bs_shift;
          within = tc & (p.block_size - 1);
        } else {
          bi = tc / p.block_size;
          within = tc - bi * p.block_size;
        }
        const int64_t blk = bt[bi];
        kreg[i] = make_uint4(0, 0, 0, 0);
        vreg[i] = make_uint4(0, 0, 0, 0);
        if (blk >= 0 && blk < p.num_cache_blocks) {  // an unmapped block reads as zeros
          const int64_t o = (blk * p.block_size + within) * cache_row_bytes + paged_thread;
          kreg[i] = *reinterpret_cast<const uint4 *>(p.k + o);
          vreg[i] = *reinterpret_cast<const uint4 *>(p.v + o);
        }
      }
    }
  };
  // What this wave's slice of the V tile in vreg holds: bit 0 some |v| >= 65536, bit 1 some |v| >= 2^-9,
  // bit 2 anything but zeros.
  auto vote_tile = [&]() __attribute__((always_inline)) {
    if constexpr (!KV8 && MODE == 0) {
      ushortx2 mx = ushortx2{0, 0};
#pragma unroll
      for (int i = 0; i < kPasses; ++i) {
        const unsigned int w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          mx = __builtin_elementwise_max(mx, __builtin_bit_cast(ushortx2, w[e] & 0x7fff7fffu));
      }
      const unsigned int m = mx[0] > mx[1] ? mx[0] : mx[1];
      const unsigned int bits = (__builtin_amdgcn_ballot_w64(m >= kVBigBits) ? 1u : 0u) |
                                (__builtin_amdgcn_ballot_w64(m >= kVDecentBits) ? 2u : 0u) |
                                (__builtin_amdgcn_ballot_w64(m != 0u) ? 4u : 0u);
      if (lane == 0) vvote[wave] = bits;
    }
  };
  // After the barrier that follows vote_tile(): true when fp16 cannot hold the tile (workgroup uniform)
  auto tile_needs_bf16 = [&]() __attribute__((always_inline)) -> bool {
    if constexpr (KV8 || MODE == 1) return false;
    unsigned int any = 0;
#pragma unroll
    for (int w = 0; w < NWV; w += 4) {
      const uint4 t = *reinterpret_cast<const uint4 *>(&vvote[w]);
      any |= t.x | t.y | t.z | t.w;
    }
    any = __builtin_amdgcn_readfirstlane(any);
    return (any & 1u) || ((any & 6u) == 4u);
  };
  auto store_tile = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int t = i * kRowsPerPass + trow;
      const int kr = k_tile_row(t);
      if (KV8) {
        // a thread holds dims 16 ch .. 16 ch + 15: columns 8 ch .. and 64 + 8 ch .. (tile_col_dim)
        uint4 lo, hi;
        fp8x16_to_bf16(kreg[i], lo, hi);
        *reinterpret_cast<uint4 *>(&Ks[kr][ch * 8]) = lo;
        *reinterpret_cast<uint4 *>(&Ks[kr][64 + ch * 8]) = hi;
        fp8x16_to_f16(vreg[i], lo, hi);
        *reinterpret_cast<uint4 *>(&Vs[t][ch * 8]) = lo;
        *reinterpret_cast<uint4 *>(&Vs[t][64 + ch * 8]) = hi;
      } else {
        *reinterpret_cast<uint4 *>(&Ks[kr][ch * 8]) = kreg[i];
        if constexpr (VB16)
          *reinterpret_cast<uint4 *>(&Vs[t][ch * 8]) = vreg[i];
        else
          *reinterpret_cast<uint4 *>(&Vs[t][ch * 8]) =
              make_uint4(bf16x2_to_f16x2(vreg[i].x), bf16x2_to_f16x2(vreg[i].y), bf16x2_to_f16x2(vreg[i].z),
                         bf16x2_to_f16x2(vreg[i].w));
      }
    }
  };

  floatx4 acc[CT][8];
  float m_run[CT], l_run[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    m_run[c] = -INFINITY;
    l_run[c] = 0.f;
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[c][d] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  load_tile(0);
  vote_tile();
  lds_barrier();
  if (tile_needs_bf16()) {   // workgroup uniform
    if (tid == 0) *marker = kRedoMarker;
    return;
  }
  constexpr float pshift = VB16 ? 0.f : kPShift;   // P is carried as 2^pshift p
  store_tile();
  lds_barrier();
  for (int kv0 = 0; kv0 < kv_end; kv0 += kBKV) {
    const bool more = kv0 + kBKV < kv_end;
    if (more) load_tile(kv0 + kBKV);
    // tiles that end at or before the first row's limit and inside lk need no mask
    const bool need_mask = (kv0 + kBKV - 1 > shift + row0) || (kv0 + kBKV > lk);
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      if (kv0 + hh * 32 >= kv_end) break;  // uniform
      // S^T for two 16-token sub-tiles; A row m of sub-tile s <-> token hh*32 + (m/4)*8 + s*4 + m%4
      floatx4 s0[CT], s1[CT];
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        s0[c] = floatx4{0.f, 0.f, 0.f, 0.f};
        s1[c] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
      const int tr0 = hh * 32 + n;  // k_tile_row of token hh*32 + (n/4)*8 + n%4; the token 4 further on is 16 rows on
#pragma unroll
      for (int kc = 0; kc < 4; ++kc) {
        Pack16 a0, a1;
        a0.u = *reinterpret_cast<const uint4 *>(&Ks[tr0][kc * 32 + g * 8]);
        a1.u = *reinterpret_cast<const uint4 *>(&Ks[tr0 + 16][kc * 32 + g * 8]);
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          s0[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, qf[c][kc], s0[c], 0, 0, 0);
          s1[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, qf[c][kc], s1[c], 0, 0, 0);
        }
      }
      // lane (n, g) of column tile c holds tokens kv0 + hh*32 + g*8 + j, j = 0..7
      uint4 ph[CT], pl[CT];  // fp16 P; or bf16 P as a hi + lo pair for a tile multiplied in bf16
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        // (the softmax is where this kernel's vector-ALU time goes: raw v_exp_f32, one fused
        // multiply-add per score, no mask arithmetic on tiles that lie wholly below the diagonal,
        // P converted two scores per instruction)
        float sv[8];
        if (need_mask) {  // workgroup-uniform
          const int tbase = kv0 + hh * 32 + g * 8;
          const int limit = min(shift + urow[c], lk - 1);  // last visible key of this unit
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float raw = j < 4 ? s0[c][j] : s1[c][j - 4];
            sv[j] = tbase + j <= limit ? raw : -INFINITY;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) sv[j] = j < 4 ? s0[c][j] : s1[c][j - 4];
        }
        float mt = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), sv[2]), fmaxf(fmaxf(sv[3], sv[4]), sv[5]));
        mt = fmaxf(fmaxf(mt, sv[6]), sv[7]);
        mt = max_lanes_16_32_48(mt);
        // running max in the scaled (log2) domain; scale_log2 > 0, so scaling commutes with max
        const float m_new = fmaxf(m_run[c], mt * scale_log2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[c] - m_use);
        float pv[8];
        const float shift_m = pshift - m_use;
#pragma unroll
        for (int j = 0; j < 8; ++j)  // 2^15 p = 2^(s * scale - m + 15): at most 2^15; a flushed denormal result is an exact 0 weight
          pv[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[j], scale_log2, shift_m));
        const float psum = ((pv[0] + pv[1]) + (pv[2] + pv[3])) + ((pv[4] + pv[5]) + (pv[6] + pv[7]));
        if constexpr (VB16) {
          unsigned int hi[4], lo[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            hi[j] = pack_bf16x2(pv[2 * j], pv[2 * j + 1]);
            lo[j] = pack_bf16x2(pv[2 * j] - __uint_as_float(hi[j] << 16), pv[2 * j + 1] - __uint_as_float(hi[j] & 0xffff0000u));
          }
          ph[c] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
          pl[c] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        } else {
          ph[c] = make_uint4(pack_f16x2(pv[0], pv[1]), pack_f16x2(pv[2], pv[3]), pack_f16x2(pv[4], pv[5]),
                             pack_f16x2(pv[6], pv[7]));
        }
        l_run[c] = l_run[c] * alpha + psum;
        m_run[c] = m_new;
        // Rescale of the accumulators, skipped (wave-uniform branch) while no lane's running max moved, which is
        // the rule after the first tiles.  Branch and multiplies are one asm block per 16 accumulators, so that
        // each accumulator stays in its register: written as a C++ branch, the scaled values land in new
        // registers and the path that skips the rescale copies all 32 accumulators there on every tile.
        rescale16(acc[c], 0, alpha);
        rescale16(acc[c], 4, alpha);
      }
      // O^T += V^T . P^T ; V^T fragment: lane (dim = d*16 + n, g) <- tokens hh*32 + g*8 + 0..7
      const int vt = hh * 32 + g * 8 + (n >> 2);
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        const shortx4 v0 = lds_read_tr16(&Vs[vt][d * 16 + (n & 3) * 4]);
        const shortx4 v1 = lds_read_tr16(&Vs[vt + 4][d * 16 + (n & 3) * 4]);
        const uint4 vraw = make_uint4(__builtin_bit_cast(uint2, v0).x, __builtin_bit_cast(uint2, v0).y,
                                      __builtin_bit_cast(uint2, v1).x, __builtin_bit_cast(uint2, v1).y);
        if constexpr (VB16) {
          const bf16x8 vb = __builtin_bit_cast(bf16x8, vraw);
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vb, __builtin_bit_cast(bf16x8, ph[c]), acc[c][d], 0, 0, 0);
            acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vb, __builtin_bit_cast(bf16x8, pl[c]), acc[c][d], 0, 0, 0);
          }
        } else {
          const f16x8 vf = __builtin_bit_cast(f16x8, vraw);
#pragma unroll
          for (int c = 0; c < CT; ++c)
            acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, __builtin_bit_cast(f16x8, ph[c]), acc[c][d], 0, 0, 0);
        }
      }
    }
    if (more) vote_tile();   // of the tile that was loaded while this one was multiplied
    lds_barrier();
    if (more) {
      if (tile_needs_bf16()) {   // workgroup uniform
        if (tid == 0) *marker = kRedoMarker;
        return;
      }
      store_tile();
      lds_barrier();
    }
  }

  const float vscale = KV8 ? p.v_scale[h] : 1.0f;
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    float l = l_run[c];
    l = sum_lanes_16_32_48(l);
    if (!uok[c]) continue;
    const int u = wave * CT * 16 + c * 16 + n;
    const int head = h * group + u % group;
    const float inv = l > 0.f ? vscale / l : 0.f;
    unsigned short *o = p.out + (static_cast<int64_t>(q_begin + urow[c]) * p.num_q_heads + head) * kPDh;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      uint2 st;
      st.x = pack_bf16x2(acc[c][d][0] * inv, acc[c][d][1] * inv);
      st.y = pack_bf16x2(acc[c][d][2] * inv, acc[c][d][3] * inv);
      *reinterpret_cast<uint2 *>(o + tile_col_dim<KV8>(d * 16 + g * 4)) = st;
    }
  }
}

}  // namespace tlf

using namespace tlf;

extern "C" int tlf_varlen_prefill_attn(const void *q, int64_t q_stride, const void *k,
                                       int64_t k_stride, const void *v, int64_t v_stride,
                                       int32_t kv_dtype, const float *k_scale, const float *v_scale,
                                       const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k,
                                       const int32_t *block_tables, int64_t block_table_stride,
                                       void *out, int32_t num_seqs, int32_t max_seqlen_q,
                                       int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                       int32_t block_size, int64_t num_cache_blocks, float scale,
                                       void *stream) {
  if (num_seqs == 0 || max_seqlen_q == 0) return TLF_OK;
  if (!q || !k || !v || !cu_seqlens_q || !cu_seqlens_k || !out) return TLF_E_NULL;
  if (head_dim != kPDh) return TLF_E_UNSUPPORTED;
  if (num_seqs < 0 || max_seqlen_q < 0 || num_q_heads <= 0 || num_kv_heads <= 0) return TLF_E_SHAPE;
  if (num_q_heads % num_kv_heads) return TLF_E_SHAPE;
  const int group = num_q_heads / num_kv_heads;
  if (group != 1 && group != 2 && group != 4 && group != 8 && group != 16) return TLF_E_UNSUPPORTED;
  if (q_stride < static_cast<int64_t>(num_q_heads) * head_dim || q_stride % 8) return TLF_E_SHAPE;
  const bool paged = block_tables != nullptr;
  if (paged) {
    if (block_size <= 0 || num_cache_blocks <= 0 || block_table_stride <= 0) return TLF_E_SHAPE;
    if (kv_dtype == TLF_KV_FP8_E4M3) {
      if (!k_scale || !v_scale) return TLF_E_NULL;
    } else if (kv_dtype != TLF_KV_BF16) {
      return TLF_E_UNSUPPORTED;
    }
  } else {
    if (kv_dtype != TLF_KV_BF16) return TLF_E_UNSUPPORTED;
    if (k_stride < static_cast<int64_t>(num_kv_heads) * head_dim || k_stride % 8 ||
        v_stride < static_cast<int64_t>(num_kv_heads) * head_dim || v_stride % 8)
      return TLF_E_SHAPE;
  }
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return TLF_E_ALIGN;

  PrefillParams p;
  p.q = static_cast<const unsigned short *>(q);
  p.q_stride = q_stride;
  p.k = static_cast<const unsigned char *>(k);
  p.v = static_cast<const unsigned char *>(v);
  p.k_stride = k_stride;
  p.v_stride = v_stride;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.cu_q = cu_seqlens_q;
  p.cu_k = cu_seqlens_k;
  p.block_tables = block_tables;
  p.bt_stride = block_table_stride;
  p.out = static_cast<unsigned short *>(out);
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.block_size = block_size;
  p.num_cache_blocks = num_cache_blocks;
  p.scale_log2 = scale * kPLog2e;
  // Eight waves of 48 (row, head) units each (CT = 3 column tiles of 16: 384 units, one workgroup per CU), or four
  // waves of 32 (CT = 2, two workgroups per CU).  Every wave reads the whole K and V tile out of LDS for its own
  // units, so LDS bytes per MFMA fall as 1 / CT, and with two column tiles the LDS reads alone take as long as
  // the MFMAs; three is what 256 registers hold.  Measured, 3 x 8 against 2 x 8 / 2 x 4: 16 x 1024 tokens
  // 284 us against 297 (2 x 4), 4 x 4096 740 against 793, 2 x 8192 on e4m3 rows 2362 against 2579.
  // TLF_PREFILL_WAVES=4 picks the four-wave form for tuning.
  static const int forced = [] {
    const char *e = getenv("TLF_PREFILL_WAVES");
    return e && atoi(e) == 4 ? 4 : 0;
  }();
  const int nwv = forced ? forced : 8;
  const int ct = nwv == 8 ? 3 : 2;
  // An XCD walks its (sequence, KV head) pairs four at a time with the row tiles outermost, longest first: with
  // one pair after the other the last pair's long row tiles start when most slots are already idle (16 x 1024
  // tokens 304 -> 287 us, 28 x 560 190 -> 182, 4 x 4096 779 -> 757); four pairs' K/V rows (2 MB at 1024 tokens)
  // still share the XCD's L2.  TLF_PREFILL_PAIR_GROUP overrides for tuning (a power of two).
  static const int forced_group = [] {
    const char *e = getenv("TLF_PREFILL_PAIR_GROUP");
    const int v = e ? atoi(e) : 0;
    return v >= 1 && v <= 64 && (v & (v - 1)) == 0 ? v : 0;
  }();
  {
    const int per_xcd = (num_kv_heads * num_seqs) / 8;  // only used when the pairs divide evenly over the XCDs
    int grp = forced_group ? forced_group : 4;
    while (grp > 1 && (per_xcd < 1 || per_xcd % grp)) grp >>= 1;
    p.pair_group = grp;
  }
  const int bq = (16 * nwv * ct) / group;
  const dim3 grid((max_seqlen_q + bq - 1) / bq, num_kv_heads, num_seqs);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (paged && kv_dtype == TLF_KV_FP8_E4M3) {
    // the K scale is a per-head constant of the scores: fold it in on the device side per head
    if (nwv == 8) TLF_LAUNCH((prefill_attn_kernel<3, true, 8, 0>), grid, dim3(512), 0, s, p);
    else TLF_LAUNCH((prefill_attn_kernel<2, true, 4, 0>), grid, dim3(256), 0, s, p);
  } else {
    if (nwv == 8) TLF_LAUNCH((prefill_attn_kernel<3, false, 8, 0>), grid, dim3(512), 0, s, p);
    else TLF_LAUNCH((prefill_attn_kernel<2, false, 4, 0>), grid, dim3(256), 0, s, p);
    int rc = launch_status();
    if (rc != TLF_OK) return rc;
    // the row tiles that met a V tile outside fp16's range, again in bf16 (every other workgroup returns at once)
    if (nwv == 8) TLF_LAUNCH((prefill_attn_kernel<3, false, 8, 1>), grid, dim3(512), 0, s, p);
    else TLF_LAUNCH((prefill_attn_kernel<2, false, 4, 1>), grid, dim3(256), 0, s, p);
  }
  return launch_status();
}
