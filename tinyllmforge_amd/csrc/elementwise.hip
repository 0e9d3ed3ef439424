// Single-pass, 128-bit vectorised elementwise / row-reduction kernels:
// RMSNorm (+ residual), RoPE, SiLU-and-mul, embedding gather, greedy argmax.
// All are HBM bound; each element is read once and written once.
#include <mutex>

#include "common.h"
#include "qknorm_rope.h"

namespace tlf {

// --------------------------------------------------------------------------
// RMSNorm / add-RMSNorm (reference: tinyvllm/layers/layernorm.py:21-45).
// TPR threads share one row, each holding up to MAXC chunks of 8 elements in
// registers, so x is read once.  Rounding points follow the reference:
//   n = bf16(s * rsqrt(mean(s^2) + eps));  y = bf16(float(n) * float(w)).
template <int TPR, int MAXC, bool ADD>
__global__ __launch_bounds__(256) void rmsnorm_kernel(
    const unsigned short *__restrict__ x, int64_t x_outer_stride,
    const unsigned short *__restrict__ residual, const unsigned short *__restrict__ weight,
    unsigned short *__restrict__ y, unsigned short *__restrict__ residual_out, int64_t rows,
    int32_t inner, int32_t cols, float eps) {
  constexpr int kRowsPerBlock = 256 / TPR;
  const int tid = threadIdx.x;
  const int sub = tid % TPR;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + tid / TPR;
  const bool active = row < rows;
  const int nchunks = cols / 8;
  const int64_t safe_row = active ? row : 0;
  const unsigned short *xr = x + (safe_row / inner) * x_outer_stride + (safe_row % inner) * cols;
  const int64_t out_off = safe_row * cols;

  float v[MAXC][8];
  uint4 pw[MAXC];  // the weights do not depend on the row: fetched together with it, not after the reduction
  uint4 px[MAXC], pres[MAXC];
  // every load of the row is unconditional (a chunk past the row re-reads the row's last chunk, an idle thread row 0)
  // and stands before the first use, so that all of them are in flight at once; only the arithmetic and the stores
  // are predicated
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int at = min(sub + c * TPR, nchunks - 1) * 8;
    pw[c] = *reinterpret_cast<const uint4 *>(weight + at);
    px[c] = *reinterpret_cast<const uint4 *>(xr + at);
    if (ADD) pres[c] = *reinterpret_cast<const uint4 *>(residual + out_off + at);
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int chunk = sub + c * TPR;
    if (active && chunk < nchunks) {
      unpack8(px[c], v[c]);
      if (ADD) {
        float r[8];
        const uint4 pr = pres[c];
        unpack8(pr, r);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[c][i] = __fadd_rn(v[c][i], r[i]);
        *reinterpret_cast<uint4 *>(residual_out + out_off + chunk * 8) = pack8(v[c]);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) ss = fmaf(v[c][i], v[c][i], ss);
    }
  }
  rmsnorm_finish<TPR, MAXC>(v, pw, ss, active, sub, nchunks, cols, eps, y + out_off);
}

template <bool ADD>
int launch_rmsnorm(const void *x, int64_t x_outer_stride, const void *residual, const void *weight,
                   void *y, void *residual_out, int64_t rows, int32_t inner, int32_t cols,
                   float eps, hipStream_t stream) {
  auto xs = static_cast<const unsigned short *>(x);
  auto rs = static_cast<const unsigned short *>(residual);
  auto ws = static_cast<const unsigned short *>(weight);
  auto ys = static_cast<unsigned short *>(y);
  auto ro = static_cast<unsigned short *>(residual_out);
#define TLF_RMS(TPR, MAXC)                                                                       \
  TLF_LAUNCH((rmsnorm_kernel<TPR, MAXC, ADD>),                                            \
                     dim3(static_cast<unsigned>((rows + (256 / TPR) - 1) / (256 / TPR))),         \
                     dim3(256), 0, stream, xs, x_outer_stride, rs, ws, ys, ro, rows, inner, cols, \
                     eps)
  TLF_RMS_SHAPES(cols, TLF_RMS);
#undef TLF_RMS
  return launch_status();
}

// --------------------------------------------------------------------------
// RoPE (reference: tinyvllm/layers/rotary_embedding.py:5-15, 41-57).
// One thread rotates 8 pairs (i, i + head_dim/2) of one head of one token.
__global__ __launch_bounds__(256) void rope_kernel(
    const int64_t *__restrict__ positions, const unsigned short *__restrict__ q, int64_t q_stride,
    const unsigned short *__restrict__ k, int64_t k_stride, const float *__restrict__ cos_sin,
    unsigned short *__restrict__ q_out, unsigned short *__restrict__ k_out, int32_t n,
    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t max_pos) {
  const int half = head_dim / 2;
  const int cpt = half / 8;  // chunks per head
  const int heads = num_q_heads + num_kv_heads;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t total = static_cast<int64_t>(n) * heads * cpt;
  if (item >= total) return;
  const int c = static_cast<int>(item % cpt);
  const int h = static_cast<int>((item / cpt) % heads);
  const int64_t tok = item / (static_cast<int64_t>(cpt) * heads);
  const int64_t pos = positions[tok];
  const bool pos_ok = pos >= 0 && pos < max_pos;  // outside the table: the row is passed through unrotated
  const bool is_q = h < num_q_heads;
  const int hh = is_q ? h : h - num_q_heads;
  const unsigned short *src = (is_q ? q + tok * q_stride : k + tok * k_stride) + hh * head_dim;
  unsigned short *dst = (is_q ? q_out + tok * static_cast<int64_t>(num_q_heads) * head_dim
                              : k_out + tok * static_cast<int64_t>(num_kv_heads) * head_dim) +
                        hh * head_dim;
  float x1[8], x2[8];
  unpack8(*reinterpret_cast<const uint4 *>(src + c * 8), x1);
  unpack8(*reinterpret_cast<const uint4 *>(src + half + c * 8), x2);
  const float *cs = cos_sin + (pos_ok ? pos : 0) * head_dim;
  float y1[8], y2[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float co = cs[c * 8 + i];
    const float si = cs[half + c * 8 + i];
    y1[i] = pos_ok ? __fsub_rn(__fmul_rn(co, x1[i]), __fmul_rn(si, x2[i])) : x1[i];
    y2[i] = pos_ok ? __fadd_rn(__fmul_rn(co, x2[i]), __fmul_rn(si, x1[i])) : x2[i];
  }
  *reinterpret_cast<uint4 *>(dst + c * 8) = pack8(y1);
  *reinterpret_cast<uint4 *>(dst + half + c * 8) = pack8(y2);
}

// --------------------------------------------------------------------------
// Fused q/k RMSNorm + RoPE + KV-cache store over the qkv projection (qknorm_rope.h): one workgroup handles
// 16 heads of TOK consecutive tokens, 16 lanes per head.  A lane has the loads of all its TOK pieces in flight
// before it touches the first (then their table rows, then the arithmetic): with one piece per lane the kernel
// is bound by the latency of its two dependent loads and by the rate at which 4 KB workgroups can be started.
template <int TOK>
__global__ __launch_bounds__(256) void qknorm_rope_store_kernel(const unsigned short *__restrict__ qkv,
                                                                int64_t qkv_stride, int32_t n,
                                                                const QkRopeStoreArgs a) {
  constexpr int kDh = 128;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * TOK;
  const int head = blockIdx.y * 16 + threadIdx.x / 16;
  const int j = threadIdx.x % 16;
  if (head >= a.num_q_heads + 2 * a.num_kv_heads) return;  // whole 16-lane groups leave together
  uint4 raw[TOK];
  QkPieceMeta meta[TOK];
  QkPieceTable tab[TOK];
#pragma unroll
  for (int i = 0; i < TOK; ++i) {
    const int64_t tok = min(tok0 + i, static_cast<int64_t>(n) - 1);
    raw[i] = load_nt_u4(qkv + tok * qkv_stride + head * kDh + j * 8);
    meta[i] = qk_piece_meta(tok, head, a);
  }
#pragma unroll
  for (int i = 0; i < TOK; ++i) tab[i] = qk_piece_table(meta[i], head, j, a);
#pragma unroll
  for (int i = 0; i < TOK; ++i)
    if (tok0 + i < n) qk_piece_finish(raw[i], tok0 + i, head, j, meta[i], tab[i], a);
}

// --------------------------------------------------------------------------
// SiLU-and-mul (reference: tinyvllm/layers/activation.py:11-14, eager rounding).
// A lane handles kSiluUnroll 8-element pieces, 256 lanes apart, and has the loads of all of them in flight
// before the first exponential.
constexpr int kSiluUnroll = 4;
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const unsigned short *__restrict__ x,
                                                           unsigned short *__restrict__ y,
                                                           int64_t rows, int32_t inter) {
  const int cpr = inter / 8;
  const int64_t total = rows * cpr;
  const int64_t item0 = static_cast<int64_t>(blockIdx.x) * (256 * kSiluUnroll) + threadIdx.x;
  uint4 gp[kSiluUnroll], up[kSiluUnroll];
  int64_t dst[kSiluUnroll];
#pragma unroll
  for (int k = 0; k < kSiluUnroll; ++k) {
    const int64_t item = item0 + k * 256;
    dst[k] = -1;
    if (item < total) {
      const int64_t r = item / cpr;
      const int c = static_cast<int>(item - r * cpr);
      const unsigned short *xr = x + r * 2 * inter;
      gp[k] = load_nt_u4(xr + c * 8);
      up[k] = load_nt_u4(xr + inter + c * 8);
      dst[k] = r * inter + c * 8;
    }
  }
#pragma unroll
  for (int k = 0; k < kSiluUnroll; ++k) {
    if (dst[k] < 0) continue;
    float g[8], u[8], o[8];
    unpack8(gp[k], g);
    unpack8(up[k], u);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = silu_mul_bf16(g[i], u[i]);
    *reinterpret_cast<uint4 *>(y + dst[k]) = pack8(o);
  }
}

// --------------------------------------------------------------------------
// Embedding gather (reference: tinyvllm/layers/embed_head.py:38).
__global__ __launch_bounds__(256) void embedding_kernel(const int64_t *__restrict__ ids,
                                                        const unsigned short *__restrict__ weight,
                                                        unsigned short *__restrict__ y,
                                                        int32_t vocab, int32_t cols) {
  const int64_t tok = blockIdx.x;
  const int64_t id = ids[tok];
  const bool ok = id >= 0 && id < vocab;
  const unsigned short *src = weight + (ok ? id : 0) * cols;
  unsigned short *dst = y + tok * cols;
  for (int c = threadIdx.x * 8; c < cols; c += blockDim.x * 8) {
    uint4 p = make_uint4(0, 0, 0, 0);
    if (ok) p = *reinterpret_cast<const uint4 *>(src + c);
    *reinterpret_cast<uint4 *>(dst + c) = p;
  }
}

// --------------------------------------------------------------------------
// Greedy argmax (reference: tinyvllm/layers/sampler.py:13-14,21).
// key = (order-preserving image of the bf16 value) << 32 | (~index): the maximum
// key is the largest value with the smallest index among ties.
constexpr int kArgmaxMaxChunks = 128;

__global__ __launch_bounds__(256) void argmax_partial_kernel(
    const unsigned short *__restrict__ logits, int64_t row_stride, int32_t vocab,
    unsigned long long *__restrict__ partial, int32_t nchunks) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const unsigned short *lr = logits + row * row_stride;
  const int nvec = vocab / 8;
  const int vec_per_chunk = (nvec + nchunks - 1) / nchunks;
  const int v0 = chunk * vec_per_chunk;
  const int v1 = min(v0 + vec_per_chunk, nvec);
  unsigned long long best = 0;
  auto take = [&](const uint4 &u, int v) {
    Pack16 p;
    p.u = u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const unsigned long long key = argmax_key(p.s[i], static_cast<unsigned int>(v * 8 + i));
      best = key > best ? key : best;
    }
  };
  int v = v0 + threadIdx.x;
  for (; v + 3 * 256 < v1; v += 4 * 256) {   // four loads in flight per lane
    uint4 u[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) u[k] = load_nt_u4(lr + static_cast<int64_t>(v + k * 256) * 8);
#pragma unroll
    for (int k = 0; k < 4; ++k) take(u[k], v + k * 256);
  }
  for (; v < v1; v += 256) take(load_nt_u4(lr + static_cast<int64_t>(v) * 8), v);
  if (chunk == 0) {  // scalar tail when vocab is not a multiple of 8
    const int t = nvec * 8 + threadIdx.x;
    if (t < vocab) {
      const unsigned long long key = argmax_key(lr[t], static_cast<unsigned int>(t));
      best = key > best ? key : best;
    }
  }
  __shared__ unsigned long long part[4];
  best = wave_max_u64(best);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) best = part[w] > best ? part[w] : best;
    partial[static_cast<int64_t>(row) * nchunks + chunk] = best;
  }
}

// One workgroup of THREADS (64 or 256) per row.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void argmax_final_kernel(
    const unsigned long long *__restrict__ partial, int32_t nchunks, int64_t *__restrict__ out) {
  const int row = blockIdx.x;
  unsigned long long best = 0;
  for (int c = threadIdx.x; c < nchunks; c += THREADS) {
    const unsigned long long k = partial[static_cast<int64_t>(row) * nchunks + c];
    best = k > best ? k : best;
  }
  best = wave_max_u64(best);
  if (THREADS > 64) {
    __shared__ unsigned long long part[THREADS / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0)
      for (int w = 1; w < THREADS / 64; ++w) best = part[w] > best ? part[w] : best;
  }
  if (threadIdx.x == 0) out[row] = static_cast<int64_t>(0xffffffffu - static_cast<unsigned int>(best));
}

// --------------------------------------------------------------------------
// Sampler with temperatures (reference: tinyvllm/layers/sampler.py:13-20).
//   T == 0:  first index of the largest logit
//   T  > 0:  argmax_i softmax(l / T)_i / (e_i + 1e-10),  e_i ~ Exp(1)
// The softmax normaliser is common to a row and log is monotone, so the sampled index is
//   argmax_i  l_i / T - log(e_i + 1e-10),   e_i = -log(u_i)
// in one pass over the row, with no exp and no row sum.  The reference draws e from torch's
// device generator; here u comes from Philox4x32-10 (Salmon et al., SC'11) keyed by the caller's
// seed: counter = (i / 4, row, offset_lo, offset_hi) yields the uniforms of elements 4*(i/4)..+3,
// u = (x >> 8) * 2^-24 + 2^-25 in (0, 1).  Same law, a stream of its own.
__device__ __forceinline__ void philox4x32_10(unsigned int (&c)[4], unsigned int k0, unsigned int k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const unsigned long long p0 = 0xD2511F53ull * c[0];
    const unsigned long long p1 = 0xCD9E8D57ull * c[2];
    const unsigned int n0 = static_cast<unsigned int>(p1 >> 32) ^ c[1] ^ k0;
    const unsigned int n2 = static_cast<unsigned int>(p0 >> 32) ^ c[3] ^ k1;
    c[1] = static_cast<unsigned int>(p1);
    c[3] = static_cast<unsigned int>(p0);
    c[0] = n0;
    c[2] = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

// key of an fp32 score: order-preserving image of the value << 32 | ~index (cf. argmax_key)
__device__ __forceinline__ unsigned long long score_key(float v, unsigned int idx) {
  v += 0.0f;  // -0 -> +0
  const unsigned int b = __float_as_uint(v);
  const unsigned int ord = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  return (static_cast<unsigned long long>(ord) << 32) | (0xffffffffu - idx);
}

__device__ __forceinline__ float sample_score(float logit, float temp, unsigned int x) {
  if (temp == 0.f) return logit;
  const float u = static_cast<float>(x >> 8) * 0x1p-24f + 0x1p-25f;
  const float e = -logf(u);
  return __fsub_rn(__fdiv_rn(logit, temp), logf(__fadd_rn(e, 1e-10f)));
}

__global__ __launch_bounds__(256) void sample_partial_kernel(
    const unsigned short *__restrict__ logits, int64_t row_stride, int32_t vocab,
    const float *__restrict__ temperatures, unsigned int seed_lo, unsigned int seed_hi,
    unsigned int off_lo, unsigned int off_hi, unsigned long long *__restrict__ partial,
    int32_t nchunks) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const unsigned short *lr = logits + row * row_stride;
  const float temp = temperatures[row];
  const int nvec = vocab / 8;
  const int vec_per_chunk = (nvec + nchunks - 1) / nchunks;
  const int v0 = chunk * vec_per_chunk;
  const int v1 = min(v0 + vec_per_chunk, nvec);
  unsigned long long best = 0;
  for (int v = v0 + threadIdx.x; v < v1; v += blockDim.x) {
    const uint4 p = *reinterpret_cast<const uint4 *>(lr + static_cast<int64_t>(v) * 8);
    float l[8];
    unpack8(p, l);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      unsigned int c[4] = {static_cast<unsigned int>(v * 2 + h), static_cast<unsigned int>(row), off_lo, off_hi};
      if (temp != 0.f) philox4x32_10(c, seed_lo, seed_hi);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const unsigned long long key = score_key(sample_score(l[h * 4 + i], temp, c[i]),
                                                 static_cast<unsigned int>(v * 8 + h * 4 + i));
        best = key > best ? key : best;
      }
    }
  }
  if (chunk == 0) {  // scalar tail when vocab is not a multiple of 8
    const int t = nvec * 8 + threadIdx.x;
    if (t < vocab) {
      unsigned int c[4] = {static_cast<unsigned int>(t / 4), static_cast<unsigned int>(row), off_lo, off_hi};
      if (temp != 0.f) philox4x32_10(c, seed_lo, seed_hi);
      const unsigned int x = (t & 3) == 0 ? c[0] : (t & 3) == 1 ? c[1] : (t & 3) == 2 ? c[2] : c[3];
      const unsigned long long key =
          score_key(sample_score(bf16_bits_to_float(lr[t]), temp, x), static_cast<unsigned int>(t));
      best = key > best ? key : best;
    }
  }
  __shared__ unsigned long long part[4];
  best = wave_max_u64(best);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) best = part[w] > best ? part[w] : best;
    partial[static_cast<int64_t>(row) * nchunks + chunk] = best;
  }
}

// Last stage of the greedy sample on its own: rows x nparts keys (argmax_key) -> token ids.
int launch_argmax_final(const unsigned long long *keys, int32_t nparts, int64_t *out, int32_t rows,
                        hipStream_t stream) {
  if (nparts > 256)  // the keys of an LM-head epilogue: thousands per row
    TLF_LAUNCH(argmax_final_kernel<256>, dim3(rows), dim3(256), 0, stream, keys, nparts, out);
  else
    TLF_LAUNCH(argmax_final_kernel<64>, dim3(rows), dim3(64), 0, stream, keys, nparts, out);
  return launch_status();
}

inline int argmax_chunks(int32_t rows, int32_t vocab) {
  int by_rows = (2048 + rows - 1) / rows;   // enough workgroups for eight on every CU
  int by_vocab = (vocab + 2047) / 2048;
  int n = by_rows < by_vocab ? by_rows : by_vocab;
  if (n < 1) n = 1;
  if (n > kArgmaxMaxChunks) n = kArgmaxMaxChunks;
  return n;
}

}  // namespace tlf

// ============================================================================ C ABI
using namespace tlf;

extern "C" int tlf_rmsnorm(const void *x, int64_t x_outer_stride, const void *weight, void *y,
                           int32_t outer, int32_t inner, int32_t cols, float eps, void *stream) {
  if (outer == 0 || inner == 0) return TLF_OK;
  if (!x || !weight || !y) return TLF_E_NULL;
  if (outer < 0 || inner < 0 || cols <= 0 || cols % 8 || cols > 16384) return TLF_E_SHAPE;
  if (x_outer_stride < static_cast<int64_t>(inner) * cols) return TLF_E_SHAPE;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || x_outer_stride % 8) return TLF_E_ALIGN;
  return launch_rmsnorm<false>(x, x_outer_stride, nullptr, weight, y, nullptr,
                               static_cast<int64_t>(outer) * inner, inner, cols, eps,
                               static_cast<hipStream_t>(stream));
}

extern "C" int tlf_add_rmsnorm(const void *x, const void *residual, const void *weight, void *y,
                               void *residual_out, int32_t rows, int32_t cols, float eps,
                               void *stream) {
  if (rows == 0) return TLF_OK;
  if (!x || !residual || !weight || !y || !residual_out) return TLF_E_NULL;
  if (rows < 0 || cols <= 0 || cols % 8 || cols > 16384) return TLF_E_SHAPE;
  if (!aligned16(x) || !aligned16(residual) || !aligned16(weight) || !aligned16(y) ||
      !aligned16(residual_out))
    return TLF_E_ALIGN;
  return launch_rmsnorm<true>(x, cols, residual, weight, y, residual_out, rows, 1, cols, eps,
                              static_cast<hipStream_t>(stream));
}

extern "C" int tlf_rope(const int64_t *positions, const void *q, int64_t q_stride, const void *k,
                        int64_t k_stride, const float *cos_sin, void *q_out, void *k_out,
                        int32_t n, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                        int32_t max_pos, void *stream) {
  if (n == 0) return TLF_OK;
  if (!positions || !q || !k || !cos_sin || !q_out || !k_out) return TLF_E_NULL;
  if (n < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || head_dim % 16 ||
      max_pos <= 0)
    return TLF_E_SHAPE;
  if (q_stride < static_cast<int64_t>(num_q_heads) * head_dim ||
      k_stride < static_cast<int64_t>(num_kv_heads) * head_dim)
    return TLF_E_SHAPE;
  if (!aligned16(q) || !aligned16(k) || !aligned16(q_out) || !aligned16(k_out) || q_stride % 8 ||
      k_stride % 8)
    return TLF_E_ALIGN;
  const int64_t total = static_cast<int64_t>(n) * (num_q_heads + num_kv_heads) * (head_dim / 16);
  TLF_LAUNCH(rope_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), positions,
                     static_cast<const unsigned short *>(q), q_stride,
                     static_cast<const unsigned short *>(k), k_stride, cos_sin,
                     static_cast<unsigned short *>(q_out), static_cast<unsigned short *>(k_out), n,
                     num_q_heads, num_kv_heads, head_dim, max_pos);
  return launch_status();
}

int tlf::check_qk_rope_store_args(const void *q_norm_weight, const void *k_norm_weight,
                                  const int64_t *positions, const float *cos_sin, int32_t max_pos,
                                  const void *q_out, const void *k_out, const void *v_out,
                                  const void *k_cache, const void *v_cache, const int32_t *slot_mapping,
                                  int64_t num_slots, int32_t kv_dtype, const float *k_scale,
                                  const float *v_scale, int32_t n, int32_t num_q_heads,
                                  int32_t num_kv_heads, int32_t head_dim) {
  if (!q_norm_weight || !k_norm_weight || !positions || !cos_sin || !q_out) return TLF_E_NULL;
  if (head_dim != 128) return TLF_E_UNSUPPORTED;
  if (n < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_pos <= 0) return TLF_E_SHAPE;
  if (slot_mapping != nullptr) {
    if (!k_cache || !v_cache) return TLF_E_NULL;
    if (num_slots <= 0) return TLF_E_SHAPE;
    if (kv_dtype == TLF_KV_FP8_E4M3) {
      if (!k_scale || !v_scale) return TLF_E_NULL;
    } else if (kv_dtype != TLF_KV_BF16) {
      return TLF_E_UNSUPPORTED;
    }
    if (!aligned16(k_cache) || !aligned16(v_cache)) return TLF_E_ALIGN;
  }
  if (!aligned16(q_out) || !aligned16(q_norm_weight) || !aligned16(k_norm_weight) || !aligned16(cos_sin) ||
      (k_out && !aligned16(k_out)) || (v_out && !aligned16(v_out)))
    return TLF_E_ALIGN;
  return TLF_OK;
}

extern "C" int tlf_qknorm_rope_store(const void *qkv, int64_t qkv_stride, const void *q_norm_weight,
                                     const void *k_norm_weight, float eps, const int64_t *positions,
                                     const float *cos_sin, int32_t max_pos, void *q_out,
                                     void *k_out, void *v_out, void *k_cache, void *v_cache,
                                     const int32_t *slot_mapping, int64_t num_slots,
                                     int32_t kv_dtype, const float *k_scale, const float *v_scale,
                                     int32_t n, int32_t num_q_heads, int32_t num_kv_heads,
                                     int32_t head_dim, void *stream) {
  if (n == 0) return TLF_OK;
  if (!qkv) return TLF_E_NULL;
  const int rc = check_qk_rope_store_args(q_norm_weight, k_norm_weight, positions, cos_sin, max_pos, q_out, k_out,
                                          v_out, k_cache, v_cache, slot_mapping, num_slots, kv_dtype, k_scale,
                                          v_scale, n, num_q_heads, num_kv_heads, head_dim);
  if (rc != TLF_OK) return rc;
  const int heads = num_q_heads + 2 * num_kv_heads;
  if (qkv_stride < static_cast<int64_t>(heads) * head_dim) return TLF_E_SHAPE;
  if (!aligned16(qkv) || qkv_stride % 8) return TLF_E_ALIGN;
  const QkRopeStoreArgs a{static_cast<const unsigned short *>(q_norm_weight),
                          static_cast<const unsigned short *>(k_norm_weight), eps, positions, cos_sin, max_pos,
                          static_cast<unsigned short *>(q_out), static_cast<unsigned short *>(k_out),
                          static_cast<unsigned short *>(v_out), static_cast<unsigned char *>(k_cache),
                          static_cast<unsigned char *>(v_cache), slot_mapping, num_slots, kv_dtype, k_scale,
                          v_scale, num_q_heads, num_kv_heads};
  if (n >= 2048)   // a prefill step: 4 tokens per workgroup
    TLF_LAUNCH(qknorm_rope_store_kernel<4>, dim3((n + 3) / 4, (heads + 15) / 16), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const unsigned short *>(qkv), qkv_stride, n, a);
  else             // a decode step: as many workgroups as there are pieces of 16 heads
    TLF_LAUNCH(qknorm_rope_store_kernel<1>, dim3(n, (heads + 15) / 16), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const unsigned short *>(qkv), qkv_stride, n, a);
  return launch_status();
}

extern "C" int tlf_silu_and_mul(const void *x, void *y, int32_t rows, int32_t inter, void *stream) {
  if (rows == 0) return TLF_OK;
  if (!x || !y) return TLF_E_NULL;
  if (rows < 0 || inter <= 0 || inter % 8) return TLF_E_SHAPE;
  if (!aligned16(x) || !aligned16(y)) return TLF_E_ALIGN;
  const int64_t total = static_cast<int64_t>(rows) * (inter / 8);
  TLF_LAUNCH(silu_and_mul_kernel, dim3(static_cast<unsigned>((total + 256 * kSiluUnroll - 1) / (256 * kSiluUnroll))),
                     dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const unsigned short *>(x), static_cast<unsigned short *>(y),
                     static_cast<int64_t>(rows), inter);
  return launch_status();
}

extern "C" int tlf_embedding(const int64_t *ids, const void *weight, void *y, int32_t n,
                             int32_t vocab, int32_t cols, void *stream) {
  if (n == 0) return TLF_OK;
  if (!ids || !weight || !y) return TLF_E_NULL;
  if (n < 0 || vocab <= 0 || cols <= 0 || cols % 8) return TLF_E_SHAPE;
  if (!aligned16(weight) || !aligned16(y)) return TLF_E_ALIGN;
  TLF_LAUNCH(embedding_kernel, dim3(n), dim3(256), 0, static_cast<hipStream_t>(stream), ids,
                     static_cast<const unsigned short *>(weight), static_cast<unsigned short *>(y),
                     vocab, cols);
  return launch_status();
}

extern "C" size_t tlf_argmax_workspace_bytes(int32_t rows, int32_t vocab) {
  (void)vocab;
  if (rows <= 0) return 0;
  return static_cast<size_t>(rows) * kArgmaxMaxChunks * sizeof(unsigned long long);
}

extern "C" int tlf_argmax(const void *logits, int64_t row_stride, int64_t *out, int32_t rows,
                          int32_t vocab, void *workspace, size_t workspace_bytes, void *stream) {
  if (rows == 0) return TLF_OK;
  if (!logits || !out) return TLF_E_NULL;
  if (rows < 0 || vocab <= 0 || row_stride < vocab) return TLF_E_SHAPE;
  if (!aligned16(logits) || row_stride % 8) return TLF_E_ALIGN;
  if (!workspace || workspace_bytes < tlf_argmax_workspace_bytes(rows, vocab) ||
      (reinterpret_cast<uintptr_t>(workspace) & 7u))
    return TLF_E_WORKSPACE;
  const int nchunks = argmax_chunks(rows, vocab);
  auto part = static_cast<unsigned long long *>(workspace);
  TLF_LAUNCH(argmax_partial_kernel, dim3(nchunks, rows), dim3(256), 0,
                     static_cast<hipStream_t>(stream),
                     static_cast<const unsigned short *>(logits), row_stride, vocab, part, nchunks);
  TLF_LAUNCH(argmax_final_kernel<64>, dim3(rows), dim3(64), 0,
                     static_cast<hipStream_t>(stream), part, nchunks, out);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Greedy argmax for callers that cannot allocate (code under hipGraph capture, tight serving loops,
// harnesses that forbid hipMalloc): same two kernels as tlf_argmax, the partial keys go to a
// file-scope device array instead of a caller workspace.  Each GPU the library runs on holds its own
// copy of the array (1 MiB) until the process ends.
constexpr int kNoAllocMaxRows = 1024;
constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) unsigned long long scratch[kNoAllocMaxRows * kArgmaxMaxChunks];

// Device address of `scratch` on the current device, resolved once per device.  In host code the
// array's name is only a handle for this lookup, never an address a kernel may be given.
static int scratch_of_current_device(unsigned long long **out) {
  static std::mutex mu;
  static unsigned long long *ptrs[kNoAllocMaxDevices] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kNoAllocMaxDevices) return TLF_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (p == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    ptrs[dev] = static_cast<unsigned long long *>(p);
  }
  *out = ptrs[dev];
  return TLF_OK;
}

extern "C" int tlf_argmax_noalloc_max_rows(void) { return kNoAllocMaxRows; }

extern "C" int tlf_argmax_noalloc(const void *logits, int64_t row_stride, int64_t *out, int32_t rows,
                                  int32_t vocab, void *stream) {
  if (rows == 0) return TLF_OK;
  if (!logits || !out) return TLF_E_NULL;
  if (rows < 0 || vocab <= 0 || row_stride < vocab) return TLF_E_SHAPE;
  if (rows > kNoAllocMaxRows) return TLF_E_TOO_LARGE;
  if (!aligned16(logits) || row_stride % 8) return TLF_E_ALIGN;
  unsigned long long *part = nullptr;
  const int rc = scratch_of_current_device(&part);
  if (rc != TLF_OK) return rc;
  // every (row, chunk) key that the second kernel reads is written by the first one in this call:
  // nothing of an earlier call's contents is read, so the array needs no clearing
  const int nchunks = argmax_chunks(rows, vocab);
  TLF_LAUNCH(argmax_partial_kernel, dim3(nchunks, rows), dim3(256), 0,
                     static_cast<hipStream_t>(stream),
                     static_cast<const unsigned short *>(logits), row_stride, vocab, part, nchunks);
  TLF_LAUNCH(argmax_final_kernel<64>, dim3(rows), dim3(64), 0,
                     static_cast<hipStream_t>(stream), part, nchunks, out);
  return launch_status();
}

extern "C" int tlf_sample(const void *logits, int64_t row_stride, const float *temperatures,
                          int64_t *out, int32_t rows, int32_t vocab, uint64_t seed, uint64_t offset,
                          void *workspace, size_t workspace_bytes, void *stream) {
  if (rows == 0) return TLF_OK;
  if (!logits || !out || !temperatures) return TLF_E_NULL;
  if (rows < 0 || vocab <= 0 || row_stride < vocab) return TLF_E_SHAPE;
  if (!aligned16(logits) || row_stride % 8) return TLF_E_ALIGN;
  if (!workspace || workspace_bytes < tlf_argmax_workspace_bytes(rows, vocab) ||
      (reinterpret_cast<uintptr_t>(workspace) & 7u))
    return TLF_E_WORKSPACE;
  const int nchunks = argmax_chunks(rows, vocab);
  auto part = static_cast<unsigned long long *>(workspace);
  TLF_LAUNCH(sample_partial_kernel, dim3(nchunks, rows), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const unsigned short *>(logits),
                     row_stride, vocab, temperatures, static_cast<unsigned int>(seed),
                     static_cast<unsigned int>(seed >> 32), static_cast<unsigned int>(offset),
                     static_cast<unsigned int>(offset >> 32), part, nchunks);
  TLF_LAUNCH(argmax_final_kernel<64>, dim3(rows), dim3(64), 0,
                     static_cast<hipStream_t>(stream), part, nchunks, out);
  return launch_status();
}
