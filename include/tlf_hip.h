/*
 * tlf_hip.h - C ABI of libtlf_hip.so: the per-token hot path of a TinyLLMForge
 * (tinyvllm) engine as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions (all entry points):
 *   - extern "C", plain pointers and sizes; no C++ or torch types.
 *   - Every pointer is a DEVICE pointer owned by the caller (the reference lets
 *     PyTorch own every buffer, so the binding passes tensor.data_ptr()).
 *   - The last argument is a hipStream_t passed as void*; work is only enqueued
 *     on that stream.  No entry point allocates, frees, synchronises or reads
 *     device memory on the host, so every call can be stream-captured into a
 *     hipGraph.  Launch geometry depends only on the integer arguments, never
 *     on device data.
 *   - Return value: 0 = ok, < 0 = rejected argument (TLF_E_*), > 0 = hipError_t
 *     of the failed launch.  Nothing is launched when an argument is rejected.
 *   - "bf16" is bfloat16 stored as uint16; "rows" are tokens unless said otherwise.
 *   - Scratch memory is caller provided: ask tlf_*_workspace_bytes() and pass a
 *     buffer of at least that size (256-byte aligned).
 *
 * Each declaration cites the reference interface (file:line under the
 * reference's tinyvllm/ package) that it replaces.
 */
#ifndef TLF_HIP_H
#define TLF_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TLF_ABI_VERSION 1

#define TLF_OK 0
#define TLF_E_NULL (-1)        /* a required pointer is NULL                         */
#define TLF_E_SHAPE (-2)       /* a size is negative, zero where not allowed, or unsupported */
#define TLF_E_ALIGN (-3)       /* a pointer or stride breaks the stated alignment    */
#define TLF_E_WORKSPACE (-4)   /* workspace missing or too small                     */
#define TLF_E_UNSUPPORTED (-5) /* a combination this build has no kernel for          */
#define TLF_E_TOO_LARGE (-6)   /* a size beyond the fixed scratch of a no-allocation entry point */

/* KV-cache element types */
#define TLF_KV_BF16 0
#define TLF_KV_FP8_E4M3 1 /* OCP e4m3fn, per-KV-head fp32 scale */

/* ABI version of the loaded library (== TLF_ABI_VERSION it was built with). */
int tlf_version(void);
/* Static, human readable text for a return code of this library. */
const char *tlf_error_string(int code);
/* Multiprocessor count and LDS bytes per workgroup of the current device
 * (host query; either out pointer may be NULL). */
int tlf_device_info(int32_t *num_cus, int32_t *lds_bytes);
/* Number of kernels this library has launched in this process so far (host counter, every entry point).
 * A statistic for benchmarks: read it before and after one eager engine step, or around a graph capture,
 * to count the kernels of a step.  No counterpart in the reference. */
int64_t tlf_kernel_launches(void);

/* ---------------------------------------------------------------------------
 * a1  store_kvcache   replaces layers/attention.py:33-48 (Triton kernel 9-30)
 *
 *   cache_row(slot[i]) = key[i] / value[i]  for every token i with slot[i] >= 0
 *
 * key/value: [num_tokens, row_bytes] rows, 16-byte aligned, row strides in
 * BYTES (value is a strided view into the qkv projection in the reference,
 * models/qwen3.py:79).  k_cache/v_cache: [num_slots, row_bytes] contiguous
 * (= [nblk, block_size, Hkv, Dh]).  row_bytes % 16 == 0.  A negative slot is
 * skipped (graph padding rows); slot >= num_slots is also skipped, never
 * written.  Pure byte copy: exact for any element type.
 */
int tlf_store_kvcache(const void *key, int64_t key_stride_bytes,
                      const void *value, int64_t value_stride_bytes,
                      void *k_cache, void *v_cache,
                      const int32_t *slot_mapping, int32_t num_tokens,
                      int32_t row_bytes, int64_t num_slots, void *stream);

/* a13 (build-defined, no reference counterpart): bf16 rows -> e4m3 cache rows,
 * c = e4m3(sat(x / scale[h])).  key/value rows are [Hkv, Dh] bf16 (strides in
 * bytes), cache rows are Hkv*Dh bytes.  k_scale/v_scale: fp32 [Hkv].  Dh % 8 == 0. */
int tlf_store_kvcache_fp8(const void *key, int64_t key_stride_bytes,
                          const void *value, int64_t value_stride_bytes,
                          void *k_cache, void *v_cache,
                          const int32_t *slot_mapping, int32_t num_tokens,
                          int32_t num_kv_heads, int32_t head_dim,
                          const float *k_scale, const float *v_scale,
                          int64_t num_slots, void *stream);

/* ---------------------------------------------------------------------------
 * a5  RMSNorm.rms_forward   replaces layers/layernorm.py:21-31
 *
 *   y = bf16( bf16( x * rsqrt(mean(x^2) + eps) ) * w )      (fp32 math)
 *
 * x is viewed as [outer, inner, cols] bf16 with element strides
 * (x_outer_stride, cols, 1): the q/k-norm call normalises every head of a
 * strided slice of the qkv projection (models/qwen3.py:80-83), the layer norm
 * uses inner = 1.  y is [outer, inner, cols] contiguous.  cols % 8 == 0,
 * cols <= 16384, 16-byte aligned rows.
 */
int tlf_rmsnorm(const void *x, int64_t x_outer_stride, const void *weight, void *y,
                int32_t outer, int32_t inner, int32_t cols, float eps, void *stream);

/* a6  RMSNorm.add_rms_forward   replaces layers/layernorm.py:33-45
 *
 *   s = x + residual (fp32); residual_out = bf16(s);
 *   y = bf16( bf16( s * rsqrt(mean(s^2) + eps) ) * w )
 *
 * All [rows, cols] bf16 contiguous.  y may alias x and residual_out may alias
 * residual (each thread reads its elements before writing them).
 */
int tlf_add_rmsnorm(const void *x, const void *residual, const void *weight,
                    void *y, void *residual_out,
                    int32_t rows, int32_t cols, float eps, void *stream);

/* ---------------------------------------------------------------------------
 * a7  RotaryEmbedding.forward   replaces layers/rotary_embedding.py:41-57 (+5-15)
 *
 *   cs = cos_sin[positions[i]]  (fp32 [max_pos, head_dim] = cos || sin)
 *   per head: y[:d/2] = cos*x[:d/2] - sin*x[d/2:], y[d/2:] = cos*x[d/2:] + sin*x[:d/2]
 *   (neox half split, fp32 products rounded separately, one bf16 rounding)
 *
 * q: [n, num_q_heads*head_dim] bf16 with row stride q_stride (elements), k
 * likewise; outputs contiguous and may alias the inputs.  positions int64 [n],
 * each in [0, max_pos) (a row whose position lies outside the table is copied
 * to the output unrotated; tlf_qknorm_rope_store does the same).  head_dim % 16 == 0.
 */
int tlf_rope(const int64_t *positions, const void *q, int64_t q_stride,
             const void *k, int64_t k_stride, const float *cos_sin,
             void *q_out, void *k_out, int32_t n, int32_t num_q_heads,
             int32_t num_kv_heads, int32_t head_dim, int32_t max_pos, void *stream);

/* Fused form of the reference's op sequence models/qwen3.py:79-94 +
 * layers/attention.py:94-95: q/k RMSNorm over head_dim (a5), RoPE (a7) and the
 * KV-cache store (a1; bf16 or e4m3 by kv_dtype) in one pass over the qkv
 * projection [n, (Hq + 2 Hkv) * head_dim] (row stride qkv_stride elements).
 * Writes q_out [n, Hq*head_dim] contiguous; k/v go only to the caches when
 * slot_mapping is non-NULL, and k_out/v_out (contiguous, may be NULL) receive
 * the rotated K and the V rows for the prefill attention.  Every intermediate
 * rounding of the unfused sequence is kept, so results are bit-identical to
 * running tlf_rmsnorm, tlf_rope and tlf_store_kvcache one after the other.
 * head_dim == 128.
 */
int tlf_qknorm_rope_store(const void *qkv, int64_t qkv_stride,
                          const void *q_norm_weight, const void *k_norm_weight, float eps,
                          const int64_t *positions, const float *cos_sin, int32_t max_pos,
                          void *q_out, void *k_out, void *v_out,
                          void *k_cache, void *v_cache, const int32_t *slot_mapping,
                          int64_t num_slots, int32_t kv_dtype,
                          const float *k_scale, const float *v_scale,
                          int32_t n, int32_t num_q_heads, int32_t num_kv_heads,
                          int32_t head_dim, void *stream);

/* ---------------------------------------------------------------------------
 * a8  SiluAndMul.forward   replaces layers/activation.py:11-14
 *
 *   y = bf16( bf16(silu(x[:, :I])) * x[:, I:] )      x [rows, 2I] -> y [rows, I]
 *
 * bf16, contiguous, I % 8 == 0.
 */
int tlf_silu_and_mul(const void *x, void *y, int32_t rows, int32_t inter, void *stream);

/* ---------------------------------------------------------------------------
 * a9  Sampler.forward, greedy branch   replaces layers/sampler.py:13-14,21
 *
 *   out[b] = first index of max(logits[b, :])       logits bf16 [rows, vocab]
 *
 * (bf16 -> fp32 is monotone, so the argmax over bf16 equals the reference's
 * argmax over the fp32 cast; -0 == +0; NaN logits are not supported.)
 * out: int64 [rows].  logits row stride in elements.  Needs a workspace.
 */
size_t tlf_argmax_workspace_bytes(int32_t rows, int32_t vocab);
int tlf_argmax(const void *logits, int64_t row_stride, int64_t *out,
               int32_t rows, int32_t vocab, void *workspace, size_t workspace_bytes,
               void *stream);

/* tlf_argmax without a workspace argument and without any allocation.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory - code under hipGraph capture, tight
 * serving loops, harnesses that forbid hipMalloc - and so cannot provide (or grow) the workspace that
 * tlf_argmax asks for.  Same kernels and result as tlf_argmax; the partial keys live in a 1 MiB
 * file-scope device array of the library (one copy per GPU, held until the process ends), which
 * bounds rows <= tlf_argmax_noalloc_max_rows() (1024): more rows return TLF_E_TOO_LARGE.  The
 * array's device address is looked up on the first call on each device (a host-side query, no
 * allocation; make that first call outside a stream capture).  Calls on one GPU share the array:
 * calls that may overlap in time (different streams) race; calls on one stream are ordered.
 * Nothing needs clearing between calls (every key read was written by the same call). */
int tlf_argmax_noalloc_max_rows(void);
int tlf_argmax_noalloc(const void *logits, int64_t row_stride, int64_t *out,
                       int32_t rows, int32_t vocab, void *stream);

/* Sampler.forward with temperatures   replaces layers/sampler.py:13-21
 *
 *   T[b] == 0:  out[b] = first index of max(logits[b, :])
 *   T[b]  > 0:  out[b] = argmax_i softmax(logits[b, :] / T[b])_i / (e_i + 1e-10),  e_i ~ Exp(1)
 *               computed as argmax_i logits[b, i] / T[b] - log(e_i + 1e-10)  (same index: the row's
 *               normaliser is common and log is monotone), one pass over the row.
 *
 * The reference takes e from torch's device generator, whose stream no kernel can reproduce; here
 * e_i = -log(u_i) with u from Philox4x32-10: key = seed, counter = (i / 4, b, offset) gives the
 * uniforms of elements 4 (i / 4) .. + 3, u = (x >> 8) * 2^-24 + 2^-25.  Same distribution, its
 * own stream; the caller advances offset once per call.
 * logits bf16 [rows, vocab] (row stride in elements), temperatures fp32 [rows] >= 0, out int64
 * [rows].  workspace: tlf_argmax_workspace_bytes(rows, vocab). */
int tlf_sample(const void *logits, int64_t row_stride, const float *temperatures, int64_t *out,
               int32_t rows, int32_t vocab, uint64_t seed, uint64_t offset,
               void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * a10  weight-only int8 linear (build-defined; the reference has bf16 F.linear
 * only: layers/linear.py:48-49, 82-83, 180-181; same [N, K] weight layout)
 *
 *   y[m, n] = bf16( (sum_k x[m, k] * float(wq[n, k])) * scale[n] )   fp32 accumulate
 *
 * x: bf16 [M, K] row stride x_stride (elements); wq: the int8 weight IN TILE ORDER, i.e. the output
 * of tlf_w8a16_pack_weight for the row-major [N, K] weight (same bytes, re-ordered so that every wave
 * reads contiguous runs: the 16-byte piece W[n, 16 a .. 16 a + 15] sits at byte
 * ((n / 32) * (K / 32) + a / 2) * 1024 + (a % 2) * 512 + (n % 32) * 16; rows are padded to a multiple of
 * 32); scale: fp32 [N]; y: bf16 [M, N] contiguous.  K % 64 == 0, N % 16 == 0.  Every W8A16 entry point
 * below takes the weight in this order.
 * workspace: fp32 partial sums when the kernel plan for (M, N, K) splits K across workgroups
 * (few output tiles, long K); tlf_w8a16_gemm_workspace_bytes gives the size for this and for
 * tlf_bf16_gemm (0 when neither plan splits), 16-byte aligned.
 */
size_t tlf_w8a16_packed_bytes(int32_t N, int32_t K);   /* = round_up(N, 32) * K */
int tlf_w8a16_pack_weight(const void *wq_rowmajor, void *packed, int32_t N, int32_t K, void *stream);
size_t tlf_w8a16_gemm_workspace_bytes(int32_t M, int32_t N, int32_t K);
int tlf_w8a16_gemm(const void *x, int64_t x_stride, const void *wq, const float *scale,
                   void *y, int32_t M, int32_t N, int32_t K,
                   void *workspace, size_t workspace_bytes, void *stream);

/* a10 / f1  bf16 linear   replaces layers/linear.py:48-49, 82-83, 180-181 and the
 * logits product layers/embed_head.py:63
 *
 *   y[m, n] = bf16( sum_k x[m, k] * w[n, k] )      fp32 accumulate
 *
 * Same shapes and constraints as tlf_w8a16_gemm with w bf16 [N, K].
 */
int tlf_bf16_gemm(const void *x, int64_t x_stride, const void *w, void *y,
                  int32_t M, int32_t N, int32_t K,
                  void *workspace, size_t workspace_bytes, void *stream);

/* gate_up projection fused with the activation: replaces MergedColumnParallelLinear.forward
 * (layers/linear.py:82-83) followed by SiluAndMul.forward (layers/activation.py:11-14) in
 * Qwen3MLP.forward (models/qwen3.py:123-130).
 *
 *   g = bf16(scale[..] * sum_k x[m,k] wq[.., k]),  u likewise
 *   y[m, c] = bf16( bf16(silu(g[m, c])) * u[m, c] )          y: bf16 [M, N/2] contiguous
 *
 * wq / scale rows are INTERLEAVED (before tlf_w8a16_pack_weight): rows 16 j .. 16 j + 7 are gate channels 8 j .. 8 j + 7 and rows
 * 16 j + 8 .. 16 j + 15 the matching up channels (N = 2 x intermediate size, N % 16 == 0), so that
 * both halves of a product sit in one lane's accumulators.  Bit-identical to tlf_w8a16_gemm on
 * the same interleaved weight followed by tlf_silu_and_mul on the de-interleaved result.
 * Needs no workspace (K is never split across workgroups).  Other constraints as tlf_w8a16_gemm. */
int tlf_w8a16_gemm_silu_mul(const void *x, int64_t x_stride, const void *wq, const float *scale,
                            void *y, int32_t M, int32_t N, int32_t K, void *stream);
/* The same with bf16 weights: w bf16 [N, K] row-major with its rows interleaved the same way (no scale). */
int tlf_bf16_gemm_silu_mul(const void *x, int64_t x_stride, const void *w, void *y,
                           int32_t M, int32_t N, int32_t K, void *stream);

/* Row-parallel projection fused with what follows it in a decoder layer: replaces
 * RowParallelLinear.forward (layers/linear.py:181-183; o_proj, down_proj) followed by
 * RMSNorm.add_rms_forward (layers/layernorm.py:33-45) of post_attention_layernorm, of the next
 * layer's input_layernorm, or of the final norm (models/qwen3.py:163-166, 188-190).
 *
 *   h = bf16(scale[n] * sum_k x[m,k] wq[n,k])          (tlf_bf16_gemm_add_rmsnorm: no scale, w bf16)
 *   s = h + residual (fp32);  residual_out = bf16(s)
 *   y = bf16( bf16( s * rsqrt(mean(s^2) + eps) ) * norm_weight )
 *
 * residual, y, residual_out: bf16 [M, N] contiguous; norm_weight bf16 [N]; N <= 16384;
 * residual_out may alias residual.  Bit-identical to the GEMM entry point followed by
 * tlf_add_rmsnorm.  When the plan for (M, N, K) splits K across workgroups, the
 * sum of the partial products, the residual add and the norm are one kernel (h never goes to
 * memory); otherwise h is staged in the workspace and the two kernels run back to back.
 * workspace: tlf_gemm_add_rmsnorm_workspace_bytes(M, N, K) bytes, 256-byte aligned.
 * Other constraints as tlf_w8a16_gemm. */
size_t tlf_gemm_add_rmsnorm_workspace_bytes(int32_t M, int32_t N, int32_t K);
int tlf_w8a16_gemm_add_rmsnorm(const void *x, int64_t x_stride, const void *wq, const float *scale,
                               const void *residual, const void *norm_weight, void *y,
                               void *residual_out, int32_t M, int32_t N, int32_t K, float eps,
                               void *workspace, size_t workspace_bytes, void *stream);
int tlf_bf16_gemm_add_rmsnorm(const void *x, int64_t x_stride, const void *w, const void *residual,
                              const void *norm_weight, void *y, void *residual_out, int32_t M,
                              int32_t N, int32_t K, float eps, void *workspace,
                              size_t workspace_bytes, void *stream);

/* qkv projection fused with what follows it in the attention block: replaces
 * QKVParallelLinear.forward (layers/linear.py:82-83 through models/qwen3.py:78) followed by the
 * q/k RMSNorm, RoPE and KV-cache store that tlf_qknorm_rope_store performs (models/qwen3.py:79-94,
 * layers/attention.py:94-95).
 *
 *   qkv = bf16(scale[c] * sum_k x[t,k] wq[c,k])   [n, (Hq + 2 Hkv) * head_dim]   (bf16 entry: no scale, w bf16)
 *   then exactly tlf_qknorm_rope_store(qkv, ...): same arguments, same outputs, same bits.
 *
 * When the plan for (n, (Hq + 2 Hkv) * head_dim, K) splits K across workgroups, the sum of the partial
 * products, the norms, the rotation and the store are one kernel (qkv never goes to memory); otherwise qkv
 * is staged in the workspace and the two kernels run back to back.
 * workspace: tlf_gemm_qknorm_rope_store_workspace_bytes(n, (Hq + 2 Hkv) * head_dim, K) bytes, 256-byte
 * aligned.  Other constraints as tlf_w8a16_gemm / tlf_bf16_gemm and tlf_qknorm_rope_store. */
size_t tlf_gemm_qknorm_rope_store_workspace_bytes(int32_t M, int32_t N, int32_t K);
int tlf_w8a16_gemm_qknorm_rope_store(const void *x, int64_t x_stride, const void *wq, const float *scale,
                                     const void *q_norm_weight, const void *k_norm_weight, float eps,
                                     const int64_t *positions, const float *cos_sin, int32_t max_pos,
                                     void *q_out, void *k_out, void *v_out,
                                     void *k_cache, void *v_cache, const int32_t *slot_mapping,
                                     int64_t num_slots, int32_t kv_dtype,
                                     const float *k_scale, const float *v_scale,
                                     int32_t n, int32_t num_q_heads, int32_t num_kv_heads,
                                     int32_t head_dim, int32_t K,
                                     void *workspace, size_t workspace_bytes, void *stream);
int tlf_bf16_gemm_qknorm_rope_store(const void *x, int64_t x_stride, const void *w,
                                    const void *q_norm_weight, const void *k_norm_weight, float eps,
                                    const int64_t *positions, const float *cos_sin, int32_t max_pos,
                                    void *q_out, void *k_out, void *v_out,
                                    void *k_cache, void *v_cache, const int32_t *slot_mapping,
                                    int64_t num_slots, int32_t kv_dtype,
                                    const float *k_scale, const float *v_scale,
                                    int32_t n, int32_t num_q_heads, int32_t num_kv_heads,
                                    int32_t head_dim, int32_t K,
                                    void *workspace, size_t workspace_bytes, void *stream);

/* LM head fused with the greedy sample: replaces ParallelLMHead.forward's product
 * (layers/embed_head.py:63) followed by Sampler.forward's greedy branch (layers/sampler.py:13-14,21)
 * when every temperature of the batch is 0.
 *
 *   token_ids[m] = argmax_n bf16( sum_k x[m,k] * w[n,k] ),  first index among ties      int64 [M]
 *
 * The [M, N] logits are never stored (more than 16 tokens; a smaller batch stages them in the
 * workspace): the GEMM epilogue keeps one (value, index) key per token, N-tile and wave, and a
 * second small kernel takes their maximum.  Identical to tlf_bf16_gemm followed by tlf_argmax.
 * workspace: tlf_gemm_argmax_workspace_bytes(M, N, K) bytes, 256-byte aligned.
 * Other constraints as tlf_bf16_gemm. */
size_t tlf_gemm_argmax_workspace_bytes(int32_t M, int32_t N, int32_t K);
int tlf_bf16_gemm_argmax(const void *x, int64_t x_stride, const void *w, int64_t *token_ids,
                         int32_t M, int32_t N, int32_t K,
                         void *workspace, size_t workspace_bytes, void *stream);

/* Diagnostic, no counterpart in the reference, touches no GPU: the kernel plan the two GEMM entry
 * points would use for a shape.  plan8 = {tile channels, tile tokens, LDS stages, waves/SIMD budget,
 * K-groups per workgroup, split-K factor, K per split, N-tile columns per XCD patch}; tile 0 x 0
 * means the skinny kernel.  Returns TLF_OK when a kernel instance exists for the plan,
 * TLF_E_UNSUPPORTED otherwise (the GEMM call would return the same). */
int tlf_gemm_plan(int32_t M, int32_t N, int32_t K, int32_t w8, int32_t *plan8);

/* ---------------------------------------------------------------------------
 * a3  paged decode attention   replaces the decode branch layers/attention.py:106-109
 *     (flash_attn_with_kvcache, one query token per sequence)
 *
 *   out[b, h] = softmax(scale * q[b, h] . K_b^T) V_b    over rows 0..context_lens[b]-1,
 *   row t of sequence b = cache[block_tables[b, t / block_size], t % block_size, h / (Hq/Hkv), :]
 *
 * q: bf16 [batch, Hq, Dh] with row stride q_stride (elements); caches
 * [num_cache_blocks, block_size, Hkv, Dh] contiguous, bf16 or e4m3 (kv_dtype;
 * e4m3 rows are dequantised as float(c) * scale[kvh], k_scale/v_scale fp32 [Hkv],
 * NULL for bf16); block_tables int32 [batch, max_blocks] with row stride
 * block_table_stride; entries at or beyond ceil(context_len / block_size) are
 * never dereferenced (the reference pads them with -1 or 0); entries outside
 * [0, num_cache_blocks) inside that range make the kernel skip the block.
 * context_lens int32 [batch]; a sequence with context_len <= 0 gets zeros.
 * out: bf16 [batch, Hq*Dh] contiguous.  fp32 softmax and accumulation; the
 * probabilities enter the P.V product as a bf16 hi + lo pair (about 16 significant bits;
 * flash-attn rounds them to one bf16).
 * Dh == 128, Hq % Hkv == 0, Hq/Hkv <= 16, Hkv in {1,2,4,8,16}, block_size % 16 == 0,
 * batch <= 1024.
 * Calls that share a workspace must not overlap in time.
 */
size_t tlf_paged_decode_attn_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                             int32_t head_dim, int32_t max_blocks,
                                             int32_t block_size);
int tlf_paged_decode_attn(const void *q, int64_t q_stride,
                          const void *k_cache, const void *v_cache, int32_t kv_dtype,
                          const float *k_scale, const float *v_scale,
                          const int32_t *block_tables, int64_t block_table_stride,
                          const int32_t *context_lens, void *out,
                          int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                          int32_t head_dim, int32_t block_size, int32_t max_blocks,
                          int64_t num_cache_blocks, float scale,
                          void *workspace, size_t workspace_bytes, void *stream);

/* a3 with the split of the work made once per decode step instead of once per layer (build-defined; the reference
 * calls flash_attn_with_kvcache per layer, layers/attention.py:106-109, and every layer of a step passes the same
 * context_lens and block_tables).  tlf_paged_decode_plan scans the lengths, finds every workgroup's first sequence
 * and copies the block-table entries it needs first into plan (tlf_paged_decode_plan_bytes() bytes, 16-byte
 * aligned); tlf_paged_decode_attn_planned is tlf_paged_decode_attn reading that plan: same arguments (the lengths
 * and tables must be the ones the plan was made from, with the same batch, block_size and max_blocks), same
 * results bit for bit, and its first cache rows are requested one memory round trip after the kernel starts
 * instead of three.  The plan is read-only to the attention calls: one plan serves all layers of the step.  A plan
 * made for another batch size (or for a grid another max_blocks / block_size gives) is recognised by its header
 * and turns every output row into NaN; one made from other lengths of the same batch cannot be told apart and gives
 * what those lengths would give. */
size_t tlf_paged_decode_plan_bytes(void);
int tlf_paged_decode_plan(const int32_t *context_lens, const int32_t *block_tables,
                          int64_t block_table_stride, int32_t batch, int32_t block_size,
                          int32_t max_blocks, void *plan, size_t plan_bytes, void *stream);
int tlf_paged_decode_attn_planned(const void *q, int64_t q_stride,
                                  const void *k_cache, const void *v_cache, int32_t kv_dtype,
                                  const float *k_scale, const float *v_scale,
                                  const int32_t *block_tables, int64_t block_table_stride,
                                  const int32_t *context_lens, void *out,
                                  int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                  int32_t head_dim, int32_t block_size, int32_t max_blocks,
                                  int64_t num_cache_blocks, float scale,
                                  void *workspace, size_t workspace_bytes, const void *plan, void *stream);

/* ---------------------------------------------------------------------------
 * a4  varlen causal prefill attention   replaces the prefill branch
 *     layers/attention.py:96-105 (flash_attn_varlen_func, causal=True)
 *
 * q: bf16 [total_q, Hq, Dh] row stride q_stride (elements).  Sequence s owns
 * query rows cu_seqlens_q[s]..cu_seqlens_q[s+1]-1 and keys
 * 0..len_k-1 with len_k = cu_seqlens_k[s+1] - cu_seqlens_k[s].  The causal mask
 * is bottom-right aligned: query i sees keys 0..(len_k - len_q) + i.
 *   block_tables == NULL: k/v are packed rows [total_k, Hkv, Dh] with row
 *     strides k_stride/v_stride (elements; v is a strided view in the reference).
 *   block_tables != NULL: k/v are the paged caches (layout and kv_dtype as in
 *     tlf_paged_decode_attn) and EVERY sequence reads its keys from them
 *     (layers/attention.py:99-100).
 * out: bf16 [total_q, Hq*Dh] contiguous.  max_seqlen_q bounds the grid.
 * fp32 softmax and accumulation.  The P.V product runs in fp16: P with 11 significant bits (flash-attn rounds
 * it to one bf16, 8 bits), carried as 2^15 p so that weights down to 2^-29 of the row maximum are normal fp16
 * numbers (the factor cancels in O / l), and V converted to fp16 when its tile is staged (exact for e4m3 rows).
 * The input domain stays that of bf16 operands: a 64-token tile of bf16 V rows that fp16 cannot hold (some
 * |v| >= 65536, or no element as large as 2^-9) makes the workgroup leave a marker in its first output element,
 * and a second launch inside this call recomputes exactly those row tiles with both products in bf16 (P as a
 * bf16 hi + lo pair).  So the call is two launches for bf16 rows and one for e4m3 rows; out is complete when
 * the call's work on the stream is.
 * Dh == 128, Hq % Hkv == 0.
 */
int tlf_varlen_prefill_attn(const void *q, int64_t q_stride,
                            const void *k, int64_t k_stride,
                            const void *v, int64_t v_stride, int32_t kv_dtype,
                            const float *k_scale, const float *v_scale,
                            const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k,
                            const int32_t *block_tables, int64_t block_table_stride,
                            void *out, int32_t num_seqs, int32_t max_seqlen_q,
                            int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t block_size, int64_t num_cache_blocks, float scale,
                            void *stream);

/* ---------------------------------------------------------------------------
 * K9  embedding row gather   replaces layers/embed_head.py:38 (F.embedding)
 *   y[i] = weight[ids[i]]   ids int64 [n], weight bf16 [vocab, cols], cols % 8 == 0.
 *   Rows with an id outside [0, vocab) are zero filled.
 */
int tlf_embedding(const int64_t *ids, const void *weight, void *y,
                  int32_t n, int32_t vocab, int32_t cols, void *stream);

/* ---------------------------------------------------------------------------
 * Bandwidth probes (no reference counterpart): plain streaming kernels that
 * bench.py uses to measure the HBM rate a read-only / copy kernel reaches on
 * the box and to scale the profiler's traffic counters.  bytes % 16 == 0,
 * 16-byte aligned pointers; sink is a 4-byte device word that is never
 * actually written for ordinary data.
 */
int tlf_probe_read(const void *src, size_t bytes, void *sink, void *stream);
int tlf_probe_copy(const void *src, void *dst, size_t bytes, void *stream);

/* Two more probes for the GEMM's rooflines (no reference counterpart).
 * tlf_probe_mfma: 512 workgroups x 4 waves each issue 16 * iters v_mfma_f32_32x32x16_bf16 from registers:
 *   2 * 32*32*16 * 16 * iters * 2048 flop per launch.  mode 0: small-integer operands, mode 1: pseudo-random
 *   bf16 values times int8-valued weights (the clock a kernel sees on real data); mode 2 / 3: the same two with
 *   idle cycles after every MFMA (a duty of about 0.9: how the clock answers to the load).  out: 512 * 256 floats.
 * tlf_probe_mix: 256 workgroups of 8 waves; waves 0..3 stream big (read once: floor(big_bytes / 16 MiB) * 16 KiB
 *   per wave, from HBM), waves 4..7 re-read small_region (L2 resident: at least 16 KiB, a multiple of 1 KiB)
 *   l2_eighths / 8 times as many bytes.  Shows what a CU's vector-memory path does with both at once. */
int tlf_probe_mfma(void *out, int32_t iters, int32_t mode, void *stream);
int tlf_probe_mix(const void *big, size_t big_bytes, const void *small_region, size_t small_bytes,
                  int32_t l2_eighths, void *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TLF_HIP_H */
