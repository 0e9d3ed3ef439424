// y[M, N] = x[M, K] . W[N, K]^T  for gfx950 matrix cores: W is int8 with a
// per-output-channel fp32 scale (weight-only quantised linear) or bf16
// (reference: tinyvllm/layers/linear.py:48-49, 82-83, 180-181, nn.Linear layout).
//
// MFMA-bound for M >= 256, weight-bandwidth-bound for small M.
//
// Orientation: W rows are the MFMA A operand, x rows the B operand, so an
// accumulator lane owns one token (x row) and 4 consecutive output channels:
// the per-channel scale is a per-register constant and the bf16 result is
// written as 8-byte pieces of a y row.
//
//   global --128-bit loads--> registers --(int8 -> bf16, exact)--> LDS (padded rows)
//   LDS --ds_read_b128--> v_mfma_f32_32x32x16_bf16, fp32 accumulators
//
// LDS is double buffered: while the matrix cores work on K-tile i, the loads of
// K-tile i+1 are in flight to registers, then converted and written to the
// other buffer; one barrier per K-tile.
//
// Tile order is XCD aware: hardware deals workgroups round-robin to the 8 XCDs
// (each with a private L2), so workgroup b belongs to XCD b % 8.  Each XCD is
// given whole columns of N-tiles and walks the M-tiles of a column first, so
// the workgroups that share an L2 share W panels and step through K together.
#include <stdio.h>
#include <stdlib.h>

#include "common.h"

namespace tlf {

constexpr int kBK = 64;           // K elements per LDS tile
constexpr int kLdsK = kBK + 8;    // padded LDS row: 144 B
constexpr int kSkinnyMaxM = 16;   // at or below this many tokens the skinny kernel runs

template <int ROWS, bool W8>
struct TileLoader;

// bf16 source rows: 128 B per row per K-tile = 8 lanes x 16 B.
template <int ROWS>
struct TileLoader<ROWS, false> {
  static constexpr int kPasses = ROWS / 32;  // 256 threads cover 32 rows per pass
  uint4 r[kPasses];
  __device__ __forceinline__ void load(const unsigned char *base, int64_t ld_bytes, int row0,
                                       int rows_total, int k0, int tid) {
    const int c = tid & 7;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int row = p * 32 + (tid >> 3);
      r[p] = make_uint4(0, 0, 0, 0);
      if (row0 + row < rows_total)
        r[p] = *reinterpret_cast<const uint4 *>(base + (row0 + row) * ld_bytes +
                                                (static_cast<int64_t>(k0) + c * 8) * 2);
    }
  }
  __device__ __forceinline__ void store(unsigned short (*lds)[kLdsK], int tid) const {
    const int c = tid & 7;
#pragma unroll
    for (int p = 0; p < kPasses; ++p)
      *reinterpret_cast<uint4 *>(&lds[p * 32 + (tid >> 3)][c * 8]) = r[p];
  }
};

// int8 source rows: 64 B per row per K-tile = 4 lanes x 16 B, converted to bf16 on the way.
template <int ROWS>
struct TileLoader<ROWS, true> {
  static constexpr int kPasses = ROWS / 64;
  uint4 r[kPasses];
  __device__ __forceinline__ void load(const unsigned char *base, int64_t ld_bytes, int row0,
                                       int rows_total, int k0, int tid) {
    const int c = tid & 3;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int row = p * 64 + (tid >> 2);
      r[p] = make_uint4(0, 0, 0, 0);
      if (row0 + row < rows_total)
        r[p] = *reinterpret_cast<const uint4 *>(base + (row0 + row) * ld_bytes + k0 + c * 16);
    }
  }
  static __device__ __forceinline__ uint2 cvt4(unsigned int w) {
    const float f0 = static_cast<float>(static_cast<signed char>(w & 0xff));
    const float f1 = static_cast<float>(static_cast<signed char>((w >> 8) & 0xff));
    const float f2 = static_cast<float>(static_cast<signed char>((w >> 16) & 0xff));
    const float f3 = static_cast<float>(static_cast<signed char>(w >> 24));
    return make_uint2(pack_bf16x2(f0, f1), pack_bf16x2(f2, f3));
  }
  __device__ __forceinline__ void store(unsigned short (*lds)[kLdsK], int tid) const {
    const int c = tid & 3;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const uint2 a = cvt4(r[p].x), b = cvt4(r[p].y), cc = cvt4(r[p].z), d = cvt4(r[p].w);
      unsigned short *dst = &lds[p * 64 + (tid >> 2)][c * 16];
      *reinterpret_cast<uint4 *>(dst) = make_uint4(a.x, a.y, b.x, b.y);
      *reinterpret_cast<uint4 *>(dst + 8) = make_uint4(cc.x, cc.y, d.x, d.y);
    }
  }
};

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
};

// BN x BM output tile per workgroup (BN output channels, BM tokens), 4 waves as WAVES_N x WAVES_M.
// Epilogue shared by the tiled kernels: scale (W8), round once to bf16, 8-byte stores;
// or fp32 partials when K is split.
template <int TN, int TM, int WN, int WM, bool W8>
__device__ __forceinline__ void gemm_epilogue(const GemmParams &p, floatx16 (&acc)[TN][TM], int m0,
                                              int n0, int wn, int wm, int r, int kg, int split) {
  // Epilogue.  acc[i][j][v]: token m = m0 + wm*WM + j*32 + r,
  // channel n = n0 + wn*WN + i*32 + (v/4)*8 + kg*4 + (v%4).
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = m0 + wm * WM + j * 32 + r;
    if (m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * WN + i * 32 + q * 8 + kg * 4;
        if (n >= p.N) continue;  // N % 4 == 0, so a group of 4 is all in or all out
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = acc[i][j][q * 4 + e];
        if (p.splits > 1) {
          float *dst = p.partial + (static_cast<int64_t>(split) * p.M + m) * p.N + n;
          *reinterpret_cast<float4 *>(dst) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
          if (W8) {
            const float4 s = *reinterpret_cast<const float4 *>(p.scale + n);
            o[0] *= s.x; o[1] *= s.y; o[2] *= s.z; o[3] *= s.w;
          }
          uint2 st;
          st.x = pack_bf16x2(o[0], o[1]);
          st.y = pack_bf16x2(o[2], o[3]);
          *reinterpret_cast<uint2 *>(p.y + static_cast<int64_t>(m) * p.N + n) = st;
        }
      }
    }
  }
}

// NBUF = LDS buffers: 2 overlaps the LDS write of tile i+1 with the math of tile i inside one
// workgroup; 1 halves the LDS footprint so that more workgroups share a CU and overlap each other.
template <int BN, int BM, int WAVES_N, int WAVES_M, bool W8, int NBUF>
__global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(BN * BM >= 256 * 256 ? 1 : 2, 8)))  // all but the largest tile: <= 256 registers
void gemm_kernel(const GemmParams p) {
  static_assert(WAVES_N * WAVES_M == 4, "4 waves");
  constexpr int WN = BN / WAVES_N, WM = BM / WAVES_M;  // per-wave tile
  constexpr int TN = WN / 32, TM = WM / 32;            // 32x32 MFMA tiles per wave
  __shared__ __attribute__((aligned(16))) unsigned short Ws[NBUF][BN][kLdsK];
  __shared__ __attribute__((aligned(16))) unsigned short Xs[NBUF][BM][kLdsK];

  // XCD-aware tile order
  const int xcd = blockIdx.x & 7;
  const int local = blockIdx.x >> 3;
  const int mt = local % p.m_tiles;
  const int nt = (local / p.m_tiles) * 8 + xcd;
  if (nt >= p.n_tiles) return;  // uniform per workgroup
  const int n0 = nt * BN, m0 = mt * BM;
  const int split = blockIdx.y;
  const int k_begin = split * p.k_per_split;
  const int k_end = min(p.K, k_begin + p.k_per_split);

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wn = wave % WAVES_N, wm = wave / WAVES_N;
  const int r = lane & 31, kg = lane >> 5;

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  TileLoader<BN, W8> wl;
  TileLoader<BM, false> xl;
  const int64_t ldw_bytes = W8 ? p.K : static_cast<int64_t>(p.K) * 2;
  wl.load(p.w, ldw_bytes, n0, p.N, k_begin, tid);
  xl.load(p.x, p.ldx_bytes, m0, p.M, k_begin, tid);
  wl.store(Ws[0], tid);
  xl.store(Xs[0], tid);
  __syncthreads();

  int buf = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += kBK) {
    const bool more = k0 + kBK < k_end;
    if (more) {
      wl.load(p.w, ldw_bytes, n0, p.N, k0 + kBK, tid);
      xl.load(p.x, p.ldx_bytes, m0, p.M, k0 + kBK, tid);
    }
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      bf16x8 af[TN], bfr[TM];
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        Pack16 t;
        t.u = *reinterpret_cast<const uint4 *>(&Ws[buf][wn * WN + i * 32 + r][ks * 16 + kg * 8]);
        af[i] = t.v;
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        Pack16 t;
        t.u = *reinterpret_cast<const uint4 *>(&Xs[buf][wm * WM + j * 32 + r][ks * 16 + kg * 8]);
        bfr[j] = t.v;
      }
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (NBUF == 2) {
      if (more) {
        wl.store(Ws[buf ^ 1], tid);
        xl.store(Xs[buf ^ 1], tid);
      }
      __syncthreads();
      buf ^= 1;
    } else {
      __syncthreads();  // every wave is done reading the tile
      if (more) {
        wl.store(Ws[0], tid);
        xl.store(Xs[0], tid);
      }
      __syncthreads();
    }
  }

  gemm_epilogue<TN, TM, WN, WM, W8>(p, acc, m0, n0, wn, wm, r, kg, split);
}

// ---------------------------------------------------------------------------
// Pipelined variant of the tiled kernel for tiles up to 128 x 128 (the mid-size GEMMs of a
// decode step).  Same tiling and numerics as gemm_kernel; what differs is the schedule:
//   * two register sets: the global loads of K-tiles t+1 and t+2 are both in flight while tile t
//     is computed, so a load has two steps to land (loads are unconditional - rows and tiles past
//     the end are clamped - so that the compiler can count them and never drains the queue);
//   * the workgroup barrier orders LDS only (lds_barrier), global loads stay in flight across it;
//   * the int8 -> bf16 conversion and LDS write of tile t+1 are issued in four slices between the
//     four MFMA groups of tile t, so VALU / LDS work overlaps matrix-core time.
// Written without lambdas or arrays of loader objects: those end up in scratch memory.
template <int ROWS, bool W8>
struct PipeLoader;

template <int ROWS>
struct PipeLoader<ROWS, false> {  // bf16 rows: 8 lanes x 16 B per row and K-tile
  static constexpr int kPasses = ROWS / 32;
  u32x4 r[kPasses];  // native vectors: arrays of HIP's struct uint4 are not promoted to registers here
  __device__ __forceinline__ void load(const unsigned char *base, int64_t ld_bytes, int row0,
                                       int rows_total, int k0, int tid) {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int row = min(row0 + p * 32 + (tid >> 3), rows_total - 1);
      r[p] = *reinterpret_cast<const u32x4 *>(base + row * ld_bytes +
                                              (static_cast<int64_t>(k0) + (tid & 7) * 8) * 2);
    }
  }
  template <int PART, int NPARTS>
  __device__ __forceinline__ void store_part(unsigned short (*lds)[kLdsK], int tid) const {
#pragma unroll
    for (int p = 0; p < kPasses; ++p)
      if (p % NPARTS == PART)
        *reinterpret_cast<u32x4 *>(&lds[p * 32 + (tid >> 3)][(tid & 7) * 8]) = r[p];
  }
};

template <int ROWS>
struct PipeLoader<ROWS, true> {  // int8 rows: 4 lanes x 16 B per row and K-tile
  static constexpr int kPasses = ROWS / 64;
  u32x4 r[kPasses];  // native vectors: arrays of HIP's struct uint4 are not promoted to registers here
  __device__ __forceinline__ void load(const unsigned char *base, int64_t ld_bytes, int row0,
                                       int rows_total, int k0, int tid) {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int row = min(row0 + p * 64 + (tid >> 2), rows_total - 1);
      r[p] = *reinterpret_cast<const u32x4 *>(base + row * ld_bytes + k0 + (tid & 3) * 16);
    }
  }
  template <int PART, int NPARTS>
  __device__ __forceinline__ void store_part(unsigned short (*lds)[kLdsK], int tid) const {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      // each pass is cut in two halves so that even a one-pass tile spreads over the slices
      unsigned short *dst = &lds[p * 64 + (tid >> 2)][(tid & 3) * 16];
      if ((2 * p) % NPARTS == PART) {
        const uint2 a = TileLoader<64, true>::cvt4(r[p].x), b = TileLoader<64, true>::cvt4(r[p].y);
        *reinterpret_cast<uint4 *>(dst) = make_uint4(a.x, a.y, b.x, b.y);
      }
      if ((2 * p + 1) % NPARTS == PART) {
        const uint2 c = TileLoader<64, true>::cvt4(r[p].z), d = TileLoader<64, true>::cvt4(r[p].w);
        *reinterpret_cast<uint4 *>(dst + 8) = make_uint4(c.x, c.y, d.x, d.y);
      }
    }
  }
};

#define TLF_PIPE_MFMA(BUF, KS)                                                                    \
  {                                                                                               \
    bf16x8 af[TN], bfr[TM];                                                                       \
    _Pragma("unroll") for (int i = 0; i < TN; ++i) {                                              \
      Pack16 t;                                                                                   \
      t.u = *reinterpret_cast<const uint4 *>(&Ws[BUF][wn * WN + i * 32 + r][(KS) * 16 + kg * 8]); \
      af[i] = t.v;                                                                                \
    }                                                                                             \
    _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                              \
      Pack16 t;                                                                                   \
      t.u = *reinterpret_cast<const uint4 *>(&Xs[BUF][wm * WM + j * 32 + r][(KS) * 16 + kg * 8]); \
      bfr[j] = t.v;                                                                               \
    }                                                                                             \
    _Pragma("unroll") for (int i = 0; i < TN; ++i)                                                \
      _Pragma("unroll") for (int j = 0; j < TM; ++j)                                              \
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);   \
  }
// one pipeline step: compute buffer BUF while tile (T)+2 is requested into set LD and the already
// requested tile (T)+1 in set ST is converted and written to the other buffer, slice by slice
#define TLF_PIPE_STEP(BUF, LDW, LDX, STW, STX, T)                                      \
  {                                                                                    \
    const int kl = k_begin + min((T) + 2, nkt - 1) * kBK;                              \
    LDW.load(p.w, ldw_bytes, n0, p.N, kl, tid);                                        \
    LDX.load(p.x, p.ldx_bytes, m0, p.M, kl, tid);                                      \
    TLF_PIPE_MFMA(BUF, 0)                                                              \
    STW.template store_part<0, 4>(Ws[(BUF) ^ 1], tid);                                 \
    STX.template store_part<0, 4>(Xs[(BUF) ^ 1], tid);                                 \
    TLF_PIPE_MFMA(BUF, 1)                                                              \
    STW.template store_part<1, 4>(Ws[(BUF) ^ 1], tid);                                 \
    STX.template store_part<1, 4>(Xs[(BUF) ^ 1], tid);                                 \
    TLF_PIPE_MFMA(BUF, 2)                                                              \
    STW.template store_part<2, 4>(Ws[(BUF) ^ 1], tid);                                 \
    STX.template store_part<2, 4>(Xs[(BUF) ^ 1], tid);                                 \
    TLF_PIPE_MFMA(BUF, 3)                                                              \
    STW.template store_part<3, 4>(Ws[(BUF) ^ 1], tid);                                 \
    STX.template store_part<3, 4>(Xs[(BUF) ^ 1], tid);                                 \
    lds_barrier();                                                                     \
  }

template <int BN, int BM, int WAVES_N, int WAVES_M, bool W8>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8)))
void gemm_pipe_kernel(const GemmParams p) {
  static_assert(WAVES_N * WAVES_M == 4, "4 waves");
  constexpr int WN = BN / WAVES_N, WM = BM / WAVES_M;
  constexpr int TN = WN / 32, TM = WM / 32;
  __shared__ __attribute__((aligned(16))) unsigned short Ws[2][BN][kLdsK];
  __shared__ __attribute__((aligned(16))) unsigned short Xs[2][BM][kLdsK];
  const int xcd = blockIdx.x & 7;
  const int local = blockIdx.x >> 3;
  const int mt = local % p.m_tiles;
  const int nt = (local / p.m_tiles) * 8 + xcd;
  if (nt >= p.n_tiles) return;
  const int n0 = nt * BN, m0 = mt * BM;
  const int split = blockIdx.y;
  const int k_begin = split * p.k_per_split;
  const int k_end = min(p.K, k_begin + p.k_per_split);
  const int nkt = (k_end - k_begin) / kBK;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wn = wave % WAVES_N, wm = wave / WAVES_N;
  const int r = lane & 31, kg = lane >> 5;
  const int64_t ldw_bytes = W8 ? p.K : static_cast<int64_t>(p.K) * 2;

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  PipeLoader<BN, W8> w0, w1;
  PipeLoader<BM, false> x0, x1;
  w0.load(p.w, ldw_bytes, n0, p.N, k_begin, tid);
  x0.load(p.x, p.ldx_bytes, m0, p.M, k_begin, tid);
  {
    const int k1 = k_begin + min(1, nkt - 1) * kBK;
    w1.load(p.w, ldw_bytes, n0, p.N, k1, tid);
    x1.load(p.x, p.ldx_bytes, m0, p.M, k1, tid);
  }
  w0.template store_part<0, 1>(Ws[0], tid);
  x0.template store_part<0, 1>(Xs[0], tid);
  lds_barrier();
  // tile t sits in buffer t & 1; set 1 holds tile t+1 at even t, set 0 at odd t
  const int pairs = nkt / 2;
  for (int t = 0; t < 2 * pairs; t += 2) {
    TLF_PIPE_STEP(0, w0, x0, w1, x1, t)
    TLF_PIPE_STEP(1, w1, x1, w0, x0, t + 1)
  }
  if (nkt & 1) {  // the last tile of an odd count sits in buffer 0 (written by the last odd step)
    TLF_PIPE_MFMA(0, 0)
    TLF_PIPE_MFMA(0, 1)
    TLF_PIPE_MFMA(0, 2)
    TLF_PIPE_MFMA(0, 3)
  }
  gemm_epilogue<TN, TM, WN, WM, W8>(p, acc, m0, n0, wn, wm, r, kg, split);
}
#undef TLF_PIPE_STEP
#undef TLF_PIPE_MFMA

// Sum the split-K partials, apply the channel scale, round once to bf16.
template <bool W8>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmParams p) {
  const int64_t i4 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t total4 = static_cast<int64_t>(p.M) * p.N / 4;
  if (i4 >= total4) return;
  const int64_t mn = static_cast<int64_t>(p.M) * p.N;
  float4 s = *reinterpret_cast<const float4 *>(p.partial + i4 * 4);
  for (int k = 1; k < p.splits; ++k) {
    const float4 t = *reinterpret_cast<const float4 *>(p.partial + k * mn + i4 * 4);
    s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
  }
  if (W8) {
    const int n = static_cast<int>((i4 * 4) % p.N);
    const float4 sc = *reinterpret_cast<const float4 *>(p.scale + n);
    s.x *= sc.x; s.y *= sc.y; s.z *= sc.z; s.w *= sc.w;
  }
  uint2 st;
  st.x = pack_bf16x2(s.x, s.y);
  st.y = pack_bf16x2(s.z, s.w);
  *reinterpret_cast<uint2 *>(p.y + i4 * 4) = st;
}

// ---------------------------------------------------------------------------
// Skinny GEMM for a handful of tokens (decode at small batch; up to 64 rows): weight-bandwidth bound.
//
// W is streamed exactly once, straight from HBM into MFMA A-operand registers
// (non-temporal 128-bit loads, no LDS staging): lane (r, g) of a wave loads 16
// consecutive K elements of channel r; the K index inside an MFMA is only a
// summation label, so the two halves of that load feed two
// v_mfma_f32_16x16x32_bf16 whose B operand (the activations, read from L2) uses
// the same labelling.  A workgroup owns 16*TN output channels; its 8 waves split
// K and the partial accumulators are summed through LDS, so nothing but the
// final bf16 rows goes back to memory.
template <int MT, int TN, bool W8>
__global__ __launch_bounds__(512) void skinny_gemm_kernel(const GemmParams p) {
  constexpr int kWaves = 8;
  constexpr int kU = 4;  // K-blocks of 64 whose weight loads are in flight together
  __shared__ __attribute__((aligned(16))) float red[kWaves][TN * MT][64][4];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16 * TN;
  const int nkb = p.K / kBK;
  const int kb_begin = static_cast<int>(static_cast<int64_t>(nkb) * wave / kWaves);
  const int kb_end = static_cast<int>(static_cast<int64_t>(nkb) * (wave + 1) / kWaves);
  const int64_t ldw = W8 ? p.K : static_cast<int64_t>(p.K) * 2;  // bytes per weight row

  floatx4 acc[TN][MT];
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[t][m] = floatx4{0.f, 0.f, 0.f, 0.f};

  const unsigned char *wrow[TN];
  bool wok[TN];
#pragma unroll
  for (int t = 0; t < TN; ++t) {
    const int n = n0 + t * 16 + r;
    wok[t] = n < p.N;
    wrow[t] = p.w + static_cast<int64_t>(wok[t] ? n : 0) * ldw;
  }
  const unsigned char *xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int row = m * 16 + r;
    xok[m] = row < p.M;
    xrow[m] = p.x + static_cast<int64_t>(xok[m] ? row : 0) * p.ldx_bytes;
  }

  for (int kb0 = kb_begin; kb0 < kb_end; kb0 += kU) {
    // issue the weight loads of up to kU K-blocks
    uint4 wraw[kU][TN][W8 ? 1 : 2];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int kb = kb0 + u;
#pragma unroll
      for (int t = 0; t < TN; ++t) {
        if (W8) {
          wraw[u][t][0] = make_uint4(0, 0, 0, 0);
          if (kb < kb_end && wok[t]) wraw[u][t][0] = load_nt_u4(wrow[t] + kb * kBK + g * 16);
        } else {
          wraw[u][t][0] = make_uint4(0, 0, 0, 0);
          wraw[u][t][W8 ? 0 : 1] = make_uint4(0, 0, 0, 0);
          if (kb < kb_end && wok[t]) {
            const unsigned char *src = wrow[t] + (static_cast<int64_t>(kb) * kBK + g * 16) * 2;
            wraw[u][t][0] = load_nt_u4(src);
            wraw[u][t][W8 ? 0 : 1] = load_nt_u4(src + 16);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int kb = kb0 + u;
      if (kb >= kb_end) break;  // uniform per wave
      bf16x8 a0[TN], a1[TN];
#pragma unroll
      for (int t = 0; t < TN; ++t) {
        Pack16 lo, hi;
        if (W8) {
          const uint4 q = wraw[u][t][0];
          const uint2 c0 = TileLoader<64, true>::cvt4(q.x), c1 = TileLoader<64, true>::cvt4(q.y);
          const uint2 c2 = TileLoader<64, true>::cvt4(q.z), c3 = TileLoader<64, true>::cvt4(q.w);
          lo.u = make_uint4(c0.x, c0.y, c1.x, c1.y);
          hi.u = make_uint4(c2.x, c2.y, c3.x, c3.y);
        } else {
          lo.u = wraw[u][t][0];
          hi.u = wraw[u][t][W8 ? 0 : 1];
        }
        a0[t] = lo.v;
        a1[t] = hi.v;
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        Pack16 b0, b1;
        b0.u = make_uint4(0, 0, 0, 0);
        b1.u = make_uint4(0, 0, 0, 0);
        if (xok[m]) {
          const unsigned char *src = xrow[m] + (static_cast<int64_t>(kb) * kBK + g * 16) * 2;
          b0.u = *reinterpret_cast<const uint4 *>(src);
          b1.u = *reinterpret_cast<const uint4 *>(src + 16);
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) {
          acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[t], b0.v, acc[t][m], 0, 0, 0);
          acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[t], b1.v, acc[t][m], 0, 0, 0);
        }
      }
    }
  }
  // acc[t][m]: token m*16 + r, channels n0 + t*16 + 4g + i
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m)
      *reinterpret_cast<float4 *>(&red[wave][t * MT + m][lane][0]) =
          make_float4(acc[t][m][0], acc[t][m][1], acc[t][m][2], acc[t][m][3]);
  __syncthreads();
  for (int item = tid; item < TN * MT * 64; item += 512) {
    const int tile = item >> 6, l = item & 63;
    const int t = tile / MT, m = tile % MT;
    float4 s = *reinterpret_cast<const float4 *>(&red[0][tile][l][0]);
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      const float4 v = *reinterpret_cast<const float4 *>(&red[w][tile][l][0]);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const int token = m * 16 + (l & 15);
    const int n = n0 + t * 16 + (l >> 4) * 4;
    if (token >= p.M || n >= p.N) continue;
    if (W8) {
      const float4 sc = *reinterpret_cast<const float4 *>(p.scale + n);
      s.x *= sc.x; s.y *= sc.y; s.z *= sc.z; s.w *= sc.w;
    }
    uint2 st;
    st.x = pack_bf16x2(s.x, s.y);
    st.y = pack_bf16x2(s.z, s.w);
    *reinterpret_cast<uint2 *>(p.y + static_cast<int64_t>(token) * p.N + n) = st;
  }
}

template <bool W8>
int launch_skinny(const GemmParams &p, hipStream_t stream) {
  const int mt = (p.M + 15) / 16;
  const int tiles16 = (p.N + 15) / 16;
  // more channels per workgroup reuse the activation fragments, as long as the grid stays large
  int tn = 1;
  if (tiles16 >= 4 * 512) tn = 4;
  else if (tiles16 >= 2 * 512) tn = 2;
  if (const char *e = getenv("TLF_GEMM_SKINNY_TN")) {  // tuning override
    const int v = atoi(e);
    if (v == 1 || v == 2 || v == 4) tn = v;
  }
  const dim3 grid((tiles16 + tn - 1) / tn);
#define TLF_SK(MT_, TN_) \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT_, TN_, W8>), grid, dim3(512), 0, stream, p)
#define TLF_SK_TN(MT_)          \
  if (tn == 4) TLF_SK(MT_, 4);  \
  else if (tn == 2) TLF_SK(MT_, 2); \
  else TLF_SK(MT_, 1)
  switch (mt) {
    case 1: TLF_SK_TN(1); break;
    case 2: TLF_SK_TN(2); break;
    case 3: TLF_SK_TN(3); break;
    default: TLF_SK_TN(4); break;
  }
#undef TLF_SK_TN
#undef TLF_SK
  return launch_status();
}

struct GemmPlan {
  bool pipe = false;  // use the pipelined kernel (tiles up to 128 x 128)
  int nbuf = 2; // LDS buffers
  int bn, bm;   // tile
  int splits;   // split-K factor
  int k_per_split;
};

// Tile and split-K choice, from a sweep over the Qwen3-8B projection shapes on MI355X.
// A K-tile step of this kernel costs roughly the same whatever the tile (it is latency bound),
// so mid-size problems want many small tiles plus a moderate split of K (each split keeps at
// least 16 K-tiles), and only problems with thousands of tiles use the large MFMA-friendly tiles.
inline GemmPlan plan_gemm(int M, int N, int K, bool w8) {
  GemmPlan g;
  auto tiles = [&](int bn, int bm) { return ((N + bn - 1) / bn) * ((M + bm - 1) / bm); };
  auto pow2_floor = [](int v) { int p = 1; while (p * 2 <= v) p *= 2; return p; };
  const int ktiles = K / kBK;
  const int max_split = ktiles / 16 > 1 ? pow2_floor(ktiles / 16) : 1;
  int splits = 1;
  if (tiles(64, 64) <= 512) {
    g.bn = 64; g.bm = 64;
    splits = pow2_floor(1024 / tiles(64, 64));
  } else if (tiles(128, 128) <= 1024) {
    g.bn = 128; g.bm = 128;
    splits = tiles(128, 128) <= 256 ? pow2_floor(512 / tiles(128, 128)) : 1;
    // plenty of tiles: one LDS buffer, so that three workgroups share a CU (measured +5-15 %)
    if (tiles(128, 128) > 256) g.nbuf = 1;
  } else {
    // thousands of tiles: 128 channels x 256 tokens, one LDS buffer, two workgroups per CU
    // (measured 427 us against 456 us for a 256 x 256 tile on 24576 x 4096 at M = 2048)
    g.bn = 128; g.bm = 256; g.nbuf = 1;
    // the bf16-weight variant of that tile does not fit 256 registers: keep the 256 x 256 tile
    if (!w8) { g.bn = 256; g.bm = 256; g.nbuf = 2; }
  }
  // small tiles with two LDS buffers run the pipelined schedule (measured 5-25 % faster)
  g.pipe = g.bn <= 128 && g.bm <= 128 && g.nbuf == 2;
  if (splits > max_split) splits = max_split;
  if (splits > 16) splits = 16;
  if (splits < 1) splits = 1;
  const int kt_per = (ktiles + splits - 1) / splits;
  g.k_per_split = kt_per * kBK;
  g.splits = (ktiles + kt_per - 1) / kt_per;
  return g;
}

// TLF_GEMM_PLAN="bn,bm,splits" forces one plan (tuning sweeps); TLF_GEMM_SKINNY_MAX_M moves the
// hand-over point between the skinny and the tiled kernel.
inline bool plan_override(GemmPlan &g, int K) {
  const char *e = getenv("TLF_GEMM_PLAN");
  if (!e) return false;
  int bn = 0, bm = 0, sp = 0, nb = 2;
  if (sscanf(e, "%d,%d,%d,%d", &bn, &bm, &sp, &nb) < 3) return false;
  g.nbuf = nb == 1 ? 1 : 2;
  g.pipe = nb == 3;
  const int ktiles = K / kBK;
  if (sp < 1) sp = 1;
  if (sp > ktiles) sp = ktiles;
  const int kt_per = (ktiles + sp - 1) / sp;
  g.bn = bn; g.bm = bm;
  g.k_per_split = kt_per * kBK;
  g.splits = (ktiles + kt_per - 1) / kt_per;
  return true;
}

inline int skinny_max_m() {
  static int v = -1;
  if (v < 0) {
    v = kSkinnyMaxM;
    if (const char *e = getenv("TLF_GEMM_SKINNY_MAX_M")) v = atoi(e);
  }
  return v;
}

template <bool W8>
int launch_gemm(const void *x, int64_t x_stride, const void *w, const float *scale, void *y,
                int32_t M, int32_t N, int32_t K, void *workspace, size_t workspace_bytes,
                hipStream_t stream) {
  GemmParams p;
  p.x = static_cast<const unsigned char *>(x);
  p.ldx_bytes = x_stride * 2;
  p.w = static_cast<const unsigned char *>(w);
  p.scale = scale;
  p.y = static_cast<unsigned short *>(y);
  p.partial = nullptr;
  p.M = M; p.N = N; p.K = K;
  if (M <= skinny_max_m()) {
    p.k_per_split = K; p.splits = 1; p.m_tiles = 1; p.n_tiles = 1;
    return launch_skinny<W8>(p, stream);
  }
  GemmPlan g = plan_gemm(M, N, K, W8);
  plan_override(g, K);
  p.k_per_split = g.k_per_split;
  p.splits = g.splits;
  p.m_tiles = (M + g.bm - 1) / g.bm;
  p.n_tiles = (N + g.bn - 1) / g.bn;
  if (g.splits > 1) {
    const size_t need = static_cast<size_t>(g.splits) * M * N * sizeof(float);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u))
      return TLF_E_WORKSPACE;
    p.partial = static_cast<float *>(workspace);
  }
  const dim3 grid(((p.n_tiles + 7) / 8) * 8 * p.m_tiles, g.splits);
#define TLF_TILE(BN_, BM_, WN_, WM_)                                                               \
  if (g.bn == BN_ && g.bm == BM_) {                                                                \
    if (g.nbuf == 1)                                                                               \
      hipLaunchKernelGGL((gemm_kernel<BN_, BM_, WN_, WM_, W8, 1>), grid, dim3(256), 0, stream, p); \
    else                                                                                           \
      hipLaunchKernelGGL((gemm_kernel<BN_, BM_, WN_, WM_, W8, 2>), grid, dim3(256), 0, stream, p); \
    launched = true;                                                                               \
  }
  bool launched = false;
  if (g.pipe && g.bm <= 128 && g.bn <= 128) {
#define TLF_PIPE(BN_, BM_, WN_, WM_)                                                                \
  if (g.bn == BN_ && g.bm == BM_) {                                                                 \
    hipLaunchKernelGGL((gemm_pipe_kernel<BN_, BM_, WN_, WM_, W8>), grid, dim3(256), 0, stream, p);  \
    launched = true;                                                                                \
  }
    TLF_PIPE(128, 128, 2, 2)
    TLF_PIPE(64, 128, 1, 4)
    TLF_PIPE(128, 64, 4, 1)
    TLF_PIPE(64, 64, 2, 2)
#undef TLF_PIPE
  }
  if (!launched) {
  TLF_TILE(256, 256, 2, 2)
  TLF_TILE(128, 256, 2, 2)
  TLF_TILE(64, 256, 1, 4)
  TLF_TILE(256, 128, 2, 2)
  TLF_TILE(128, 128, 2, 2)
  TLF_TILE(64, 128, 1, 4)
  TLF_TILE(128, 64, 4, 1)
  TLF_TILE(64, 64, 2, 2)
  }
#undef TLF_TILE
  if (!launched) return TLF_E_UNSUPPORTED;
  int rc = launch_status();
  if (rc != TLF_OK) return rc;
  if (g.splits > 1) {
    const int64_t total4 = static_cast<int64_t>(M) * N / 4;
    hipLaunchKernelGGL((splitk_reduce_kernel<W8>), dim3(static_cast<unsigned>((total4 + 255) / 256)),
                       dim3(256), 0, stream, p);
    rc = launch_status();
  }
  return rc;
}

inline int check_gemm_args(const void *x, int64_t x_stride, const void *w, const void *y, int32_t M,
                           int32_t N, int32_t K) {
  if (!x || !w || !y) return TLF_E_NULL;
  if (M < 0 || N <= 0 || K <= 0 || K % kBK || N % 16 || x_stride < K) return TLF_E_SHAPE;
  if (!aligned16(x) || !aligned16(w) || !aligned16(y) || x_stride % 8) return TLF_E_ALIGN;
  return TLF_OK;
}

}  // namespace tlf

using namespace tlf;

extern "C" size_t tlf_w8a16_gemm_workspace_bytes(int32_t M, int32_t N, int32_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % kBK) return 0;
  // room for the deepest split any plan may use (16), so that tuning overrides stay in bounds
  if (M <= skinny_max_m()) return 0;
  return static_cast<size_t>(16) * M * N * sizeof(float);
}

extern "C" int tlf_w8a16_gemm(const void *x, int64_t x_stride, const void *wq, const float *scale,
                              void *y, int32_t M, int32_t N, int32_t K, void *workspace,
                              size_t workspace_bytes, void *stream) {
  if (M == 0) return TLF_OK;
  const int rc = check_gemm_args(x, x_stride, wq, y, M, N, K);
  if (rc != TLF_OK) return rc;
  if (!scale) return TLF_E_NULL;
  if (reinterpret_cast<uintptr_t>(scale) & 15u) return TLF_E_ALIGN;
  return launch_gemm<true>(x, x_stride, wq, scale, y, M, N, K, workspace, workspace_bytes,
                           static_cast<hipStream_t>(stream));
}

extern "C" int tlf_bf16_gemm(const void *x, int64_t x_stride, const void *w, void *y, int32_t M,
                             int32_t N, int32_t K, void *workspace, size_t workspace_bytes,
                             void *stream) {
  if (M == 0) return TLF_OK;
  const int rc = check_gemm_args(x, x_stride, w, y, M, N, K);
  if (rc != TLF_OK) return rc;
  return launch_gemm<false>(x, x_stride, w, nullptr, y, M, N, K, workspace, workspace_bytes,
                            static_cast<hipStream_t>(stream));
}
