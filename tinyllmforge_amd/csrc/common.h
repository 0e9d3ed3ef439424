// Shared device/host helpers for the gfx950 kernels of libtlf_hip.so.
#pragma once
#include <atomic>

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tlf_hip.h"

namespace tlf {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short shortx4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

constexpr int kWave = 64;

// 16 bytes = 8 bf16, moved as one 128-bit access.
union Pack16 {
  uint4 u;
  bf16x8 v;
  unsigned short s[8];
  unsigned int w[4];
};

__device__ __forceinline__ float bf16_bits_to_float(unsigned short b) {
  return __uint_as_float(static_cast<unsigned int>(b) << 16);
}

// Round-to-nearest-even fp32 -> bf16 (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ unsigned short float_to_bf16_bits(float f) {
  __bf16 h = static_cast<__bf16>(f);
  return __builtin_bit_cast(unsigned short, h);
}

// SiLU-and-mul with the eager rounding points of the reference (tinyvllm/layers/activation.py:11-14):
// bf16(silu(g)) * u, the product rounded to bf16 by the caller's pack.  g and u are bf16 values.
// exp and the division run on the quarter-rate hardware approximations, corrected to about 2 ulp of fp32 in
// all (the product g * log2(e) keeps its rounding error as a second term, the reciprocal gets one Newton step):
// with the library expf and an IEEE division the kernel is bound by the vector ALU, not by HBM.  Beyond
// |g| = 80 the reciprocal's operand nears the end of the fp32 range; those (rare) values take the library path.
__device__ __forceinline__ float silu_mul_bf16(float g, float u) {
  float s;
  if (fabsf(g) <= 80.0f) {
    const float kL2eHi = 1.44269502162933349609375f, kL2eLo = 1.925963033500011e-08f, kLn2 = 0.693147182464599609375f;
    const float x = -g;
    const float hi = __fmul_rn(x, kL2eHi);
    const float lo = fmaf(x, kL2eLo, fmaf(x, kL2eHi, -hi));    // x * log2(e) - hi
    const float e0 = __builtin_amdgcn_exp2f(hi);
    const float d = 1.0f + fmaf(e0, __fmul_rn(lo, kLn2), e0);   // 1 + 2^(hi + lo)
    float r = __builtin_amdgcn_rcpf(d);
    r = fmaf(fmaf(-d, r, 1.0f), r, r);
    s = __fmul_rn(g, r);
  } else {
    s = g / (1.0f + expf(-g));
  }
  return __fmul_rn(bf16_bits_to_float(float_to_bf16_bits(s)), u);
}

// Value of lane (l - N) mod 16 of the same row of 16 lanes (a DPP move on the vector ALU, no LDS round trip).
template <int N>
__device__ __forceinline__ float row_ror(float v) {
  static_assert(N >= 1 && N <= 15, "rotation inside a row of 16 lanes");
  const int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + N, 0xf, 0xf, false);
  return __int_as_float(r);
}

__device__ __forceinline__ unsigned int pack_bf16x2(float lo, float hi) {
  bf16x2 r;
  r[0] = static_cast<__bf16>(lo);
  r[1] = static_cast<__bf16>(hi);
  return __builtin_bit_cast(unsigned int, r);
}

__device__ __forceinline__ void unpack8(const uint4 &p, float (&f)[8]) {
  f[0] = __uint_as_float(p.x << 16);
  f[1] = __uint_as_float(p.x & 0xffff0000u);
  f[2] = __uint_as_float(p.y << 16);
  f[3] = __uint_as_float(p.y & 0xffff0000u);
  f[4] = __uint_as_float(p.z << 16);
  f[5] = __uint_as_float(p.z & 0xffff0000u);
  f[6] = __uint_as_float(p.w << 16);
  f[7] = __uint_as_float(p.w & 0xffff0000u);
}

__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  uint4 p;
  p.x = pack_bf16x2(f[0], f[1]);
  p.y = pack_bf16x2(f[2], f[3]);
  p.z = pack_bf16x2(f[4], f[5]);
  p.w = pack_bf16x2(f[6], f[7]);
  return p;
}

// Four e4m3 values (one dword) -> four bf16, exact: v_cvt_scalef32_pk_bf16_fp8 converts a pair per
// instruction (scale 1.0), half the vector-ALU work of going through fp32.
__device__ __forceinline__ void fp8x4_to_bf16x4(unsigned int w, unsigned int &lo, unsigned int &hi) {
  lo = __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
  hi = __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true));
}

// 128-bit load with the non-temporal hint: data that is read once (KV-cache rows,
// weights at small batch) should not displace L2 / Infinity Cache lines; on MI355X a
// read-only stream is ~10% faster with it (measured: 7.1 vs 6.3 TB/s).
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_nt_u4(const void *p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Exchanges among the four lanes l, l ^ 16, l ^ 32, l ^ 48 on the vector ALU (v_permlane16_swap /
// v_permlane32_swap), without the LDS round trip of a ds_bpermute: a = {row 0, row 0, row 2, row 2},
// b = {row 1, row 1, row 3, row 3} of 16-lane rows after the first swap, lower and upper half after the second.
__device__ __forceinline__ float max_lanes_16_32_48(float v) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_lanes_16_32_48(float v) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Orders this wave's LDS writes before its later LDS reads (other lanes' data).
// LDS operations of one wave execute in program order; this only stops the
// compiler from moving them across.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() fences every address space,
// i.e. it also waits for all outstanding global loads (s_waitcnt vmcnt(0)) and so defeats any
// register prefetch that is meant to stay in flight across the barrier.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Second half of every RMSNorm kernel: TPR threads share a row, thread `sub` holds chunks
// sub + c * TPR (8 values each) of s in v, of the norm weight in pw, and its own sum of squares in ss.
//   n = bf16(s * rsqrt(mean(s^2) + eps));  y = bf16(float(n) * float(w))
// (reference: tinyvllm/layers/layernorm.py:21-45).  The reduction tree is part of the result's bits,
// which is why every kernel that ends in an RMSNorm shares this function and TLF_RMS_SHAPES.
template <int TPR, int MAXC>
__device__ __forceinline__ void rmsnorm_finish(const float (&v)[MAXC][8], const uint4 (&pw)[MAXC], float ss,
                                               bool active, int sub, int nchunks, int cols, float eps,
                                               unsigned short *__restrict__ y_row) {
  if (TPR <= 64) {
#pragma unroll
    for (int o = TPR / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
  } else {
    __shared__ float part[256 / 64];
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int w = 0; w < TPR / 64; ++w) ss += part[w];
  }
  const float var = ss / static_cast<float>(cols);
  const float inv = 1.0f / sqrtf(var + eps);
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int chunk = sub + c * TPR;
    if (active && chunk < nchunks) {
      float w[8];
      unpack8(pw[c], w);
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float n = bf16_bits_to_float(float_to_bf16_bits(__fmul_rn(v[c][i], inv)));
        o[i] = __fmul_rn(n, w[i]);
      }
      *reinterpret_cast<uint4 *>(y_row + chunk * 8) = pack8(o);
    }
  }
}

// threads per row and chunks per thread for a row of `cols` values (256-thread workgroups,
// 256 / TPR rows each); CALL(TPR, MAXC) is expanded for the matching shape
#define TLF_RMS_SHAPES(cols, CALL) \
  do {                             \
    if ((cols) <= 128) {           \
      CALL(16, 1);                 \
    } else if ((cols) <= 512) {    \
      CALL(64, 1);                 \
    } else if ((cols) <= 2048) {   \
      CALL(64, 4);                 \
    } else if ((cols) <= 4096) {   \
      CALL(256, 2);                \
    } else if ((cols) <= 8192) {   \
      CALL(256, 4);                \
    } else {                       \
      CALL(256, 8);                \
    }                              \
  } while (0)

// Greedy argmax (reference: tinyvllm/layers/sampler.py:13-14,21) as a maximum over 64-bit keys:
// key = (order-preserving image of the bf16 value) << 32 | (~index), so the largest key is the
// largest value with the smallest index among ties.  Key 0 is below every real key.
__device__ __forceinline__ unsigned long long argmax_key(unsigned short bits, unsigned int idx) {
  if (bits == 0x8000u) bits = 0;  // -0 == +0
  const unsigned int ord = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
  return (static_cast<unsigned long long>(ord) << 32) | (0xffffffffu - idx);
}

__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    unsigned int lo = __shfl_xor(static_cast<unsigned int>(v), o, 64);
    unsigned int hi = __shfl_xor(static_cast<unsigned int>(v >> 32), o, 64);
    unsigned long long other = (static_cast<unsigned long long>(hi) << 32) | lo;
    v = other > v ? other : v;
  }
  return v;
}

int launch_argmax_final(const unsigned long long *keys, int32_t nparts, int64_t *out, int32_t rows,
                        hipStream_t stream);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Kernels this library has launched in this process: a statistic for benchmarks (kernels per engine step are
// counted around one eager step or one graph capture); every launch of the library goes through TLF_LAUNCH.
extern std::atomic<long long> g_kernel_launches;
#define TLF_LAUNCH(...)                                                      \
  do {                                                                       \
    tlf::g_kernel_launches.fetch_add(1, std::memory_order_relaxed);          \
    hipLaunchKernelGGL(__VA_ARGS__);                                         \
  } while (0)

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TLF_OK : static_cast<int>(e);
}

}  // namespace tlf
