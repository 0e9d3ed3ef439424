// Shared device/host helpers for the gfx950 kernels of libtlf_hip.so.
#pragma once

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
__device__ __forceinline__ float silu_mul_bf16(float g, float u) {
  const float s = g / (1.0f + expf(-g));
  return __fmul_rn(bf16_bits_to_float(float_to_bf16_bits(s)), u);
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

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TLF_OK : static_cast<int>(e);
}

}  // namespace tlf
