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
#include "common.h"

namespace tlf {

constexpr int kBK = 64;           // K elements per LDS tile
constexpr int kLdsK = kBK + 8;    // padded LDS row: 144 B

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
template <int BN, int BM, int WAVES_N, int WAVES_M, bool W8>
__global__ __launch_bounds__(256) void gemm_kernel(const GemmParams p) {
  static_assert(WAVES_N * WAVES_M == 4, "4 waves");
  constexpr int WN = BN / WAVES_N, WM = BM / WAVES_M;  // per-wave tile
  constexpr int TN = WN / 32, TM = WM / 32;            // 32x32 MFMA tiles per wave
  __shared__ __attribute__((aligned(16))) unsigned short Ws[2][BN][kLdsK];
  __shared__ __attribute__((aligned(16))) unsigned short Xs[2][BM][kLdsK];

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
    if (more) {
      wl.store(Ws[buf ^ 1], tid);
      xl.store(Xs[buf ^ 1], tid);
    }
    __syncthreads();
    buf ^= 1;
  }

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

struct GemmPlan {
  int bn, bm;   // tile
  int splits;   // split-K factor
  int k_per_split;
};

// Fill the 256 CUs: largest tile whose grid still has >= ~1 workgroup per CU,
// then split K when even the smallest tile leaves CUs idle.
inline GemmPlan plan_gemm(int M, int N, int K) {
  GemmPlan g;
  const int cus = 256;
  auto tiles = [&](int bn, int bm) { return ((N + bn - 1) / bn) * ((M + bm - 1) / bm); };
  if (M > 128 && tiles(256, 256) >= cus) {
    g.bn = 256; g.bm = 256;
  } else if (M > 64 && tiles(128, 128) >= cus) {
    g.bn = 128; g.bm = 128;
  } else if (M > 64) {
    g.bn = 128; g.bm = 128;
  } else {
    g.bn = 128; g.bm = 64;
  }
  const int t = tiles(g.bn, g.bm);
  int splits = 1;
  const int ktiles = K / kBK;
  while (t * splits * 2 <= cus * 2 && splits * 2 <= 16 && ktiles / (splits * 2) >= 4) splits *= 2;
  if (t >= cus) splits = 1;
  g.splits = splits;
  const int kt_per = (ktiles + splits - 1) / splits;
  g.k_per_split = kt_per * kBK;
  g.splits = (ktiles + kt_per - 1) / kt_per;
  return g;
}

template <bool W8>
int launch_gemm(const void *x, int64_t x_stride, const void *w, const float *scale, void *y,
                int32_t M, int32_t N, int32_t K, void *workspace, size_t workspace_bytes,
                hipStream_t stream) {
  const GemmPlan g = plan_gemm(M, N, K);
  GemmParams p;
  p.x = static_cast<const unsigned char *>(x);
  p.ldx_bytes = x_stride * 2;
  p.w = static_cast<const unsigned char *>(w);
  p.scale = scale;
  p.y = static_cast<unsigned short *>(y);
  p.partial = nullptr;
  p.M = M; p.N = N; p.K = K;
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
  if (g.bn == 256 && g.bm == 256)
    hipLaunchKernelGGL((gemm_kernel<256, 256, 2, 2, W8>), grid, dim3(256), 0, stream, p);
  else if (g.bn == 128 && g.bm == 128)
    hipLaunchKernelGGL((gemm_kernel<128, 128, 2, 2, W8>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_kernel<128, 64, 4, 1, W8>), grid, dim3(256), 0, stream, p);
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
  const GemmPlan g = plan_gemm(M, N, K);
  if (g.splits <= 1) return 0;
  return static_cast<size_t>(g.splits) * M * N * sizeof(float);
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
