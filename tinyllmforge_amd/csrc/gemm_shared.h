// Pieces shared by the GEMM kernels of libtlf_hip.so: parameters, the int8 -> bf16
// conversion, the epilogue over MFMA accumulator tiles and the global -> LDS copy instruction.
#pragma once

#include "common.h"

namespace tlf {

constexpr int kBK = 64;           // K elements per LDS tile
constexpr int kSkinnyMaxM = 16;   // at or below this many tokens the skinny kernel runs

// four int8 (one dword) -> four bf16, exact
__device__ __forceinline__ uint2 cvt4_i8_bf16(unsigned int w) {
  const float f0 = static_cast<float>(static_cast<signed char>(w & 0xff));
  const float f1 = static_cast<float>(static_cast<signed char>((w >> 8) & 0xff));
  const float f2 = static_cast<float>(static_cast<signed char>((w >> 16) & 0xff));
  const float f3 = static_cast<float>(static_cast<signed char>(w >> 24));
  return make_uint2(pack_bf16x2(f0, f1), pack_bf16x2(f2, f3));
}

struct GemmParams {
  const unsigned char *x;
  int64_t ldx_bytes;
  const unsigned char *w;
  const float *scale;
  unsigned short *y;
  float *partial;  // [splits, M, N] fp32 when splits > 1
  int32_t M, N, K;
  int32_t k_per_split;
  int32_t splits;
  int32_t m_tiles, n_tiles;
  int32_t group_n;  // N-tile columns (xcd_rows: M-tile rows) walked together by one XCD
  int32_t xcd_rows; // 1: an XCD owns M-tile rows 8 c + xcd and walks all N-tile columns; 0: it owns N-tile columns
  int32_t map_main; // workgroups of the owned part: 8 * (rows or columns per XCD) * tiles walked
  int32_t map_full; // rows (columns) covered by ownership: a multiple of 8
  int32_t map_rem;  // the rest of them (1 ... 7; 1 when there is none): their tiles follow, dealt out one by one
  int32_t act;      // 1: SiLU-and-mul epilogue over interleaved gate/up channels, y is [M, N/2]
                    // 2: greedy-sample epilogue, nothing but argmax keys [M, amax_parts] is stored
  unsigned long long *amax;
  int32_t amax_parts;  // key columns per token: one per (N-tile, wave along N)
};

// Epilogue of the tiled kernel (BN output channels x BM tokens per workgroup, waves laid out as
// WAVES_N x WAVES_M): scale (W8), round once to bf16, 8-byte stores; or fp32 partials when K is
// split across workgroups; or the fused SiLU-and-mul over interleaved gate/up channels.
// The channel scales of a lane's accumulator registers (plans without a split of K): fetched once, before the
// first store.  Read where they are used, each load sits behind the previous store (the compiler cannot rule out
// that y and scale overlap) and the epilogue becomes a chain of load -> multiply -> store round trips, 32 of
// them for a 256-token tile.
template <int TN, int WN>
__device__ __forceinline__ void gemm_load_scales(const GemmParams &p, float4 (&sc)[TN][4], int n0, int wn, int kg) {
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wn * WN + i * 32 + q * 8 + kg * 4;
      sc[i][q] = p.splits == 1 && n < p.N ? *reinterpret_cast<const float4 *>(p.scale + n) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

template <int TN, int TM, int WN, int WM, bool W8>
__device__ __forceinline__ void gemm_epilogue_sc(const GemmParams &p, floatx16 (&acc)[TN][TM], int m0, int n0, int wn,
                                                 int wm, int r, int kg, int split, const float4 (&sc)[TN][4]);

template <int TN, int TM, int WN, int WM, bool W8>
__device__ __forceinline__ void gemm_epilogue(const GemmParams &p, floatx16 (&acc)[TN][TM], int m0,
                                              int n0, int wn, int wm, int r, int kg, int split) {
  float4 sc[TN][4];
  if (W8) gemm_load_scales<TN, WN>(p, sc, n0, wn, kg);
  gemm_epilogue_sc<TN, TM, WN, WM, W8>(p, acc, m0, n0, wn, wm, r, kg, split, sc);
}

// acc[i][j][v]: token m = m0 + wm*WM + j*32 + r, channel n = n0 + wn*WN + i*32 + (v/4)*8 + kg*4 + (v%4).
template <int TN, int TM, int WN, int WM, bool W8>
__device__ __forceinline__ void gemm_epilogue_sc(const GemmParams &p, floatx16 (&acc)[TN][TM], int m0, int n0, int wn,
                                                 int wm, int r, int kg, int split, const float4 (&sc)[TN][4]) {
  if (p.act == 2) {
    // LM head + greedy sample (reference: tinyvllm/layers/embed_head.py:63, sampler.py:13-14,21): the
    // logits are never stored.  A token's channels of this wave sit in the registers of lanes r and
    // r + 32: each lane keeps the best key of its bf16-rounded values, the pair is merged with one
    // exchange, and the key goes to column (N-tile, wave) of the token's row.
    const int part = (n0 + wn * WN) / WN;
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int m = m0 + wm * WM + j * 32 + r;
      unsigned long long best = 0;
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * WN + i * 32 + q * 8 + kg * 4;
          if (n >= p.N) continue;
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = acc[i][j][q * 4 + e];
          if (W8) {
            const float4 s = sc[i][q];
            o[0] *= s.x; o[1] *= s.y; o[2] *= s.z; o[3] *= s.w;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const unsigned long long key = argmax_key(float_to_bf16_bits(o[e]), static_cast<unsigned int>(n + e));
            best = key > best ? key : best;
          }
        }
      const unsigned int lo = __shfl_xor(static_cast<unsigned int>(best), 32, 64);
      const unsigned int hi = __shfl_xor(static_cast<unsigned int>(best >> 32), 32, 64);
      const unsigned long long other = (static_cast<unsigned long long>(hi) << 32) | lo;
      best = other > best ? other : best;
      if (kg == 0 && m < p.M) p.amax[static_cast<int64_t>(m) * p.amax_parts + part] = best;
    }
    return;
  }
  // bf16 results leave as 16-byte stores: lanes r and r + 32 hold the same token and alternate groups of 4
  // channels, so one half-wave exchange (v_permlane32_swap) hands lane r the 8 consecutive channels 16 h ..
  // 16 h + 7 and lane r + 32 the next 8 -- half the store instructions, rows written 32 bytes at a time.
  auto swap_pairs = [](uint2 &a, uint2 &b) {
    // before: lane kg holds channel groups (2 h) and (2 h + 1) of its own; after: lane 0 holds group 2 h of
    // both lanes (channels 0..7 of the 16), lane 1 group 2 h + 1 of both (channels 8..15)
    auto rx = __builtin_amdgcn_permlane32_swap(a.x, b.x, false, false);
    auto ry = __builtin_amdgcn_permlane32_swap(a.y, b.y, false, false);
    a = make_uint2(rx[0], ry[0]);
    b = make_uint2(rx[1], ry[1]);
  };
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = m0 + wm * WM + j * 32 + r;
    const bool m_ok = m < p.M;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      if (p.act == 1) {
        // channels come in groups of 16 = 8 gate rows then the 8 matching up rows, so this lane's
        // registers q = 0, 2 hold gate values and q = 1, 3 the up values of the same 4 channels
        uint2 st[2];
#pragma unroll
        for (int q = 0; q < 4; q += 2) {
          float gt[4], up[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            gt[e] = acc[i][j][q * 4 + e];
            up[e] = acc[i][j][(q + 1) * 4 + e];
          }
          if (W8) {
            const float4 sg = sc[i][q], su = sc[i][q + 1];
            gt[0] *= sg.x; gt[1] *= sg.y; gt[2] *= sg.z; gt[3] *= sg.w;
            up[0] *= su.x; up[1] *= su.y; up[2] *= su.z; up[3] *= su.w;
          }
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)  // both factors rounded to bf16 first, as the unfused sequence does
            o[e] = silu_mul_bf16(bf16_bits_to_float(float_to_bf16_bits(gt[e])),
                                 bf16_bits_to_float(float_to_bf16_bits(up[e])));
          st[q / 2] = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
        }
        // this lane: output channels c0 + kg*4 .. (q = 0) and c0 + 8 + kg*4 .. (q = 2) of the 16 of this tile
        swap_pairs(st[0], st[1]);
        const int nfirst = n0 + wn * WN + i * 32;
        if (m_ok && nfirst + kg * 16 < p.N) {  // lane r + 32 stores what came from the tile's second 16 rows
          const int c = nfirst / 2 + kg * 8;
          *reinterpret_cast<uint4 *>(p.y + static_cast<int64_t>(m) * (p.N / 2) + c) =
              make_uint4(st[0].x, st[0].y, st[1].x, st[1].y);
        }
        continue;
      }
      if (p.splits > 1) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * WN + i * 32 + q * 8 + kg * 4;
          if (!m_ok || n >= p.N) continue;  // N % 4 == 0, so a group of 4 is all in or all out
          float *dst = p.partial + (static_cast<int64_t>(split) * p.M + m) * p.N + n;
          *reinterpret_cast<float4 *>(dst) =
              make_float4(acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
        }
        continue;
      }
      uint2 st[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = acc[i][j][q * 4 + e];
        if (W8) {
          const float4 s = sc[i][q];
          o[0] *= s.x; o[1] *= s.y; o[2] *= s.z; o[3] *= s.w;
        }
        st[q] = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        swap_pairs(st[2 * h], st[2 * h + 1]);
        const int n = n0 + wn * WN + i * 32 + h * 16 + kg * 8;  // N % 16 == 0: 16 channels are all in or all out
        if (m_ok && n < p.N)
          *reinterpret_cast<uint4 *>(p.y + static_cast<int64_t>(m) * p.N + n) =
              make_uint4(st[2 * h].x, st[2 * h].y, st[2 * h + 1].x, st[2 * h + 1].y);
      }
    }
  }
}

// Workgroup barrier for a global -> LDS copy pipeline, the copy instruction itself and the LDS address of a
// __shared__ object (see the tiled kernel in gemm.hip for why these are inline asm).
#define TLF_LPTR(p) ((__attribute__((address_space(3))) void *)(p))
// Workgroup barrier for the copy pipeline: wait until at most N of this wave's copies are still
// in flight and its LDS reads have returned, then s_barrier.  Written as one asm block: a
// workgroup-scope release fence would make the compiler wait for every outstanding copy
// (they count as LDS writes), which is exactly the wait the pipeline must not do.
#define TLF_DL_BARRIER(N) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory")

// The copies are issued from inline asm so that the compiler does not see them: it cannot tell
// which LDS object a copy writes, and would otherwise wait for every outstanding copy (and for
// every outstanding LDS read) before each ds_read.  Ordering is explicit instead: TLF_DL_BARRIER.
// m0 (the LDS base of a copy) is a reserved register that nothing else in this kernel uses:
// LDS reads and writes need no m0 on this ISA.
#define TLF_DL_COPY(VOFF, SBASE, LDS)                                                     \
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(VOFF), \
               "s"(SBASE), "s"(LDS)                                                       \
               : "memory")
#define TLF_DL_LDSADDR(P) static_cast<unsigned int>(reinterpret_cast<uintptr_t>(TLF_LPTR(P)))

}  // namespace tlf
