// Library-level entry points of libtlf_hip.so.
#include "common.h"

namespace tlf {
std::atomic<long long> g_kernel_launches{0};
}

extern "C" int tlf_version(void) { return TLF_ABI_VERSION; }

extern "C" int64_t tlf_kernel_launches(void) { return tlf::g_kernel_launches.load(std::memory_order_relaxed); }

extern "C" const char *tlf_error_string(int code) {
  switch (code) {
    case TLF_OK: return "ok";
    case TLF_E_NULL: return "a required pointer is NULL";
    case TLF_E_SHAPE: return "a size or stride is out of range";
    case TLF_E_ALIGN: return "a pointer or stride is not 16-byte aligned";
    case TLF_E_WORKSPACE: return "workspace missing, misaligned or too small";
    case TLF_E_UNSUPPORTED: return "no kernel for this combination";
    case TLF_E_TOO_LARGE: return "size beyond the fixed scratch array of this no-allocation entry point";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}

extern "C" int tlf_device_info(int32_t *num_cus, int32_t *lds_bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (num_cus) *num_cus = prop.multiProcessorCount;
  if (lds_bytes) *lds_bytes = static_cast<int32_t>(prop.sharedMemPerBlock);
  return TLF_OK;
}

// ---------------------------------------------------------------------------
// Bandwidth probes: the rate a plain streaming kernel reaches on this box.
namespace tlf {

// Each workgroup streams its own contiguous region with non-temporal 128-bit loads, sixteen in
// flight per lane (64 KB per workgroup, 16 MB over the chip): the best read pattern found on
// MI355X; with eight in flight the same kernel stops at 6.3 TB/s instead of 7.1.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4 *__restrict__ src, size_t n16,
                                                         unsigned int *__restrict__ sink) {
  const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
  const size_t begin = per * blockIdx.x;
  const size_t end = begin + per < n16 ? begin + per : n16;
  unsigned int acc = 0;
  size_t i = begin + threadIdx.x;
  for (; i + 15 * 256 < end; i += 16 * 256) {
    uint4 v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = load_nt_u4(src + i + u * 256);
#pragma unroll
    for (int u = 0; u < 16; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < end; i += 256) {
    const uint4 a = load_nt_u4(src + i);
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u && threadIdx.x == 1023) *sink = acc;  // keeps the loads alive, never taken
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4 *__restrict__ src,
                                                         uint4 *__restrict__ dst, size_t n16) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride)
    dst[i] = src[i];
}

// Register-only MFMA stream: what the matrix cores sustain with nothing to wait for.  Every wave issues
// 16 * iters v_mfma_f32_32x32x16_bf16 on four independent accumulators from operands that never change:
// small integers (mode 0, 2) or pseudo-random bf16 activations times int8-valued weights (mode 1, 3).  The two
// differ on this part: the clock drops under the switching activity of random data.  Modes 2 and 3 leave idle
// cycles after every MFMA.
__global__ __launch_bounds__(256) void probe_mfma_kernel(float *__restrict__ out, int iters, int mode) {
  bf16x8 a, b;
  unsigned int h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 17u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    h = h * 1664525u + 1013904223u;
    const bool random = mode & 1;
    const float fa = random ? (static_cast<int>(h >> 8) % 2001 - 1000) * 1e-3f : static_cast<float>((threadIdx.x + i) & 3);
    h = h * 1664525u + 1013904223u;
    const float fb = random ? static_cast<float>(static_cast<int>(h >> 8) % 255 - 127) : static_cast<float>(i & 1);
    a[i] = static_cast<__bf16>(fa);
    b[i] = static_cast<__bf16>(fb);
  }
  floatx16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
  if (mode & 2) {
    // the same stream with two s_nop 7 after every MFMA: the matrix pipe runs at a duty of about 0.9, so the clock
    // the part answers with separates the power that goes with the clock from the power that goes with the MFMAs
#define TLF_GAPPED(J) "v_mfma_f32_32x32x16_bf16 %" #J ", %4, %5, %" #J "\n\ts_nop 7\n\ts_nop 7\n\t"
#define TLF_GAPPED4 TLF_GAPPED(0) TLF_GAPPED(1) TLF_GAPPED(2) TLF_GAPPED(3)
    for (int it = 0; it < iters; ++it)
      asm volatile(TLF_GAPPED4 TLF_GAPPED4 TLF_GAPPED4 TLF_GAPPED4
                   : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])
                   : "v"(a), "v"(b));
#undef TLF_GAPPED4
#undef TLF_GAPPED
  } else {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[j][v];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Two streams through one CU's vector-memory path at once: waves 0 .. 3 of every workgroup read a region of
// their own once (from HBM), waves 4 .. 7 re-read a small region that stays in L2, l2_units KiB for every KiB
// of the first kind.  Measured on MI355X the launch takes the SUM of the times the two streams take alone
// (loads return in order through a CU's L1, so an L2 hit queues behind the HBM misses issued before it):
// a decode-size GEMM, whose workgroups all re-read the activations out of L2 while they stream their weights
// from HBM, pays for both in full.
__global__ __launch_bounds__(512) void probe_mix_kernel(const unsigned char *__restrict__ big, size_t kib_per_wave,
                                                        const unsigned char *__restrict__ small_, size_t small_kib,
                                                        int l2_eighths, unsigned int *__restrict__ sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned int acc = 0;
  uint4 v[16];
  if (wave < 4) {
    const unsigned char *p = big + (static_cast<size_t>(blockIdx.x) * 4 + wave) * kib_per_wave * 1024 + lane * 16;
    for (size_t i = 0; i + 16 <= kib_per_wave; i += 16) {
#pragma unroll
      for (int d = 0; d < 16; ++d) v[d] = load_nt_u4(p + (i + d) * 1024);
#pragma unroll
      for (int d = 0; d < 16; ++d) acc ^= v[d].x ^ v[d].w;
    }
  } else {
    const size_t n = kib_per_wave * l2_eighths / 8;
    size_t c = (static_cast<size_t>(wave) * 37 + blockIdx.x * 11) % small_kib;
    for (size_t i = 0; i + 16 <= n; i += 16) {
#pragma unroll
      for (int d = 0; d < 16; ++d) {
        v[d] = *reinterpret_cast<const uint4 *>(small_ + c * 1024 + lane * 16);
        c = c + 1 == small_kib ? 0 : c + 1;
      }
#pragma unroll
      for (int d = 0; d < 16; ++d) acc ^= v[d].x ^ v[d].w;
    }
  }
  if (acc == 0x9e3779b9u && threadIdx.x == 1023) *sink = acc;  // keeps the loads alive, never taken
}

}  // namespace tlf

extern "C" int tlf_probe_mfma(void *out, int32_t iters, int32_t mode, void *stream) {
  if (!out) return TLF_E_NULL;
  if (iters < 0 || mode < 0 || mode > 3) return TLF_E_SHAPE;
  // one workgroup of four waves per CU slot, twice the CUs: two waves per SIMD keep the pipe full
  TLF_LAUNCH(tlf::probe_mfma_kernel, dim3(512), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<float *>(out), iters, mode);
  return tlf::launch_status();
}

extern "C" int tlf_probe_mix(const void *big, size_t big_bytes, const void *small_region, size_t small_bytes,
                             int32_t l2_eighths, void *sink, void *stream) {
  if (!big || !small_region || !sink) return TLF_E_NULL;
  if (!tlf::aligned16(big) || !tlf::aligned16(small_region)) return TLF_E_ALIGN;
  const size_t kib_per_wave = big_bytes / 1024 / (256 * 4) / 16 * 16;
  if (kib_per_wave == 0 || small_bytes < 16 * 1024 || small_bytes % 1024 || l2_eighths < 0) return TLF_E_SHAPE;
  TLF_LAUNCH(tlf::probe_mix_kernel, dim3(256), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const unsigned char *>(big), kib_per_wave,
                     static_cast<const unsigned char *>(small_region), small_bytes / 1024, l2_eighths,
                     static_cast<unsigned int *>(sink));
  return tlf::launch_status();
}

extern "C" int tlf_probe_read(const void *src, size_t bytes, void *sink, void *stream) {
  if (!src || !sink) return TLF_E_NULL;
  if (bytes % 16 || !tlf::aligned16(src)) return TLF_E_ALIGN;
  if (bytes == 0) return TLF_OK;
  TLF_LAUNCH(tlf::probe_read_kernel, dim3(256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4 *>(src), bytes / 16,
                     static_cast<unsigned int *>(sink));
  return tlf::launch_status();
}

extern "C" int tlf_probe_copy(const void *src, void *dst, size_t bytes, void *stream) {
  if (!src || !dst) return TLF_E_NULL;
  if (bytes % 16 || !tlf::aligned16(src) || !tlf::aligned16(dst)) return TLF_E_ALIGN;
  if (bytes == 0) return TLF_OK;
  TLF_LAUNCH(tlf::probe_copy_kernel, dim3(256 * 8), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4 *>(src),
                     static_cast<uint4 *>(dst), bytes / 16);
  return tlf::launch_status();
}
