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
// int8 weights are held in TILE ORDER (tlf_w8a16_pack_weight), not row-major: the 16-byte atom
// W[n, 16 a .. 16 a + 15] of row n sits at byte
//     ((n / 32) * (K / 32) + a / 2) * 1024 + (a % 2) * 512 + (n % 32) * 16,
// i.e. 32 rows x 32 K values form one contiguous 1 KiB chunk whose 64 atoms are, in order, the
// A operands of v_mfma_f32_32x32x16_bf16 for lanes 0..63 (lane = (a % 2) * 32 + n % 32), and the
// chunks of one 32-row group follow each other along K.  A wave that owns a 32-row group streams
// one contiguous run with 1 KiB per load instruction (measured on MI355X: 5.4 TB/s, against
// 3.3 TB/s for the 32 rows x 32 bytes per instruction that row-major weights give this MFMA).
// bf16 weights stay row-major (the reference's nn.Linear layout).
//
// Three kernels: a tiled one whose K-tiles travel global -> LDS without passing through
// registers (gemm_dlds_kernel), a W-streaming one for decode-size batches in which every wave
// streams its own weight rows global -> registers and only the activations go through LDS
// (gemm_wstream_kernel), and a skinny one for a handful of tokens (skinny_gemm_kernel).
//
// Tile order is XCD aware: hardware deals workgroups round-robin to the 8 XCDs
// (each with a private L2), so workgroup b belongs to XCD b % 8.  Each XCD is
// given whole columns of N-tiles, so the workgroups that share an L2 share W
// and x panels and step through K together.
#include <stdio.h>
#include <type_traits>
#include <stdlib.h>

#include "common.h"
#include "gemm_shared.h"
#include "qknorm_rope.h"

namespace tlf {

// Tiled kernel: global_load_lds_dwordx4 copies each lane's 16 bytes from global memory
// straight into LDS (the wave's 64 pieces land contiguously at a wave-uniform LDS base), so a K-tile
// costs no staging registers, no ds_write and - for int8 weights - half the LDS bytes: W stays
// int8 in LDS and is converted to bf16 after the fragment read.  NS LDS stages carved out of
// one pool: with three, the copies of tiles t+1 and t+2 are in flight while tile t is computed;
// two suffice where the copies are L2 hits, four and more help where few workgroups stream
// weights from HBM.
//
// LDS rows are unpadded (a wave's copy is contiguous), conflicts are avoided by an XOR swizzle of
// the 16-byte pieces instead: piece c of a 128-byte bf16 row R sits at position c ^ ((R>>1)&7),
// piece c of a 64-byte int8 row at c ^ ((R>>2)&3); the lane that fills a position picks the
// matching global piece.  Any 16 consecutive rows then cover all 64 banks once per ds_read_b128.
//
// int8 weights: lane (r, kg) reads 16 consecutive K values of channel r with one ds_read_b128 and
// feeds them to two MFMAs; the K index inside an MFMA is only a summation label, so the x operand
// of those two MFMAs is read with the same labelling (pieces 2c and 2c+1 of the x row).
// Copy setup for one step: global bases and LDS bases of tile T's destination stage.
#define TLF_DL_ISSUE_SETUP(XS, WS, T)                                                             \
  const int kt_ = min((T), nkt - 1);                                                              \
  const unsigned char *xg_ = xbase + static_cast<int64_t>(kt_) * (kBK * 2);                       \
  const unsigned char *wg_ = wbase + static_cast<int64_t>(kt_) * kWStep;                          \
  const unsigned int xl_ = TLF_DL_LDSADDR(XS) + set_u * kXBytes + wave_u * 1024,                  \
                     wl_ = TLF_DL_LDSADDR(WS) + set_u * kWBytes + wave_u * 1024;
// Slice PART of 4 of the copies.  The copies are spread over the step, between the MFMA groups:
// issued back to back, the workgroup's copies queue up in the texture-address unit and every
// wave sits in that queue with nothing on the matrix cores.
#define TLF_DL_ISSUE_PART(PART)                                                                   \
  {                                                                                               \
    _Pragma("unroll") for (int q = 0; q < XP; ++q)                                                \
      if (q % 4 == (PART)) TLF_DL_COPY(xoff[q], xg_, xl_ + q * kPass);                            \
    _Pragma("unroll") for (int q = 0; q < WP; ++q)                                                \
      if ((q + XP) % 4 == (PART)) TLF_DL_COPY(woff[q], wg_, wl_ + q * kPass);                     \
  }
#define TLF_DL_ISSUE(XS, WS, T)        \
  {                                    \
    TLF_DL_ISSUE_SETUP(XS, WS, T)      \
    TLF_DL_ISSUE_PART(0)               \
    TLF_DL_ISSUE_PART(1)               \
    TLF_DL_ISSUE_PART(2)               \
    TLF_DL_ISSUE_PART(3)               \
  }

// Copy slices issued after MFMA group G (0..3) of a step.  Three stages: one slice per group.
// Two stages: the copy has to land within the step, so everything goes out in its first half.
#define TLF_DL_AFTER_GROUP(G)                          \
  if (do_issue_) {                                     \
    if constexpr (NS >= 3) {                           \
      if ((G) == 0) TLF_DL_ISSUE_PART(0)               \
      if ((G) == 1) TLF_DL_ISSUE_PART(1)               \
      if ((G) == 2) TLF_DL_ISSUE_PART(2)               \
      if ((G) == 3) TLF_DL_ISSUE_PART(3)               \
    } else {                                           \
      if ((G) == 0) { TLF_DL_ISSUE_PART(0) TLF_DL_ISSUE_PART(1) } \
      if ((G) == 1) { TLF_DL_ISSUE_PART(2) TLF_DL_ISSUE_PART(3) } \
    }                                                  \
  }
// Compute on stage (XS, WS); the four copy slices of the step go between its MFMA groups.
#define TLF_DL_COMPUTE(XS, WS)                                                                    \
  if constexpr (W8) {                                                                             \
    _Pragma("unroll") for (int ksp = 0; ksp < 2; ++ksp) {                                         \
      bf16x8 af[TN][2], bfr[TM][2];                                                               \
      _Pragma("unroll") for (int i = 0; i < TN; ++i) {                                            \
        const u32x4 raw = *reinterpret_cast<const u32x4 *>(WS + wrow + i * (32 * 64) + wq[ksp]);  \
        const uint2 a = cvt4_i8_bf16(raw.x), b = cvt4_i8_bf16(raw.y); \
        const uint2 c = cvt4_i8_bf16(raw.z), d = cvt4_i8_bf16(raw.w); \
        Pack16 t;                                                                                 \
        t.u = make_uint4(a.x, a.y, b.x, b.y);                                                     \
        af[i][0] = t.v;                                                                           \
        t.u = make_uint4(c.x, c.y, d.x, d.y);                                                     \
        af[i][1] = t.v;                                                                           \
      }                                                                                           \
      _Pragma("unroll") for (int h = 0; h < 2; ++h)                                               \
        _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                          \
          Pack16 t;                                                                               \
          t.u = *reinterpret_cast<const uint4 *>(XS + xrow + j * (32 * 128) + xq[ksp * 2 + h]);   \
          bfr[j][h] = t.v;                                                                        \
        }                                                                                         \
      _Pragma("unroll") for (int h = 0; h < 2; ++h) {                                             \
        _Pragma("unroll") for (int i = 0; i < TN; ++i)                                            \
          _Pragma("unroll") for (int j = 0; j < TM; ++j)                                          \
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i][h], bfr[j][h], acc[i][j], 0, 0, 0); \
        TLF_DL_AFTER_GROUP(ksp * 2 + h)                                                           \
      }                                                                                           \
    }                                                                                             \
  } else {                                                                                        \
    _Pragma("unroll") for (int ks = 0; ks < 4; ++ks) {                                            \
      bf16x8 af[TN], bfr[TM];                                                                     \
      _Pragma("unroll") for (int i = 0; i < TN; ++i) {                                            \
        Pack16 t;                                                                                 \
        t.u = *reinterpret_cast<const uint4 *>(WS + wrow + i * (32 * 128) + xq[ks]);              \
        af[i] = t.v;                                                                              \
      }                                                                                           \
      _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                            \
        Pack16 t;                                                                                 \
        t.u = *reinterpret_cast<const uint4 *>(XS + xrow + j * (32 * 128) + xq[ks]);              \
        bfr[j] = t.v;                                                                             \
      }                                                                                           \
      _Pragma("unroll") for (int i = 0; i < TN; ++i)                                              \
        _Pragma("unroll") for (int j = 0; j < TM; ++j)                                            \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0); \
      TLF_DL_AFTER_GROUP(ks)                                                                      \
    }                                                                                             \
  }

// One step: tile T sits in stage (XS, WS).  Own copies of tile T have landed once at most one
// later tile (kLoads copies) is outstanding; the barrier then makes every wave's copies visible
// and says that every wave is done with the stage tile T+2 goes to (it held tile T-1).
#define TLF_DL_STEP(XS, WS, XS_NEXT2, WS_NEXT2, T) \
  {                                                \
    TLF_DL_BARRIER(kLoads);                        \
    TLF_DL_ISSUE_SETUP(XS_NEXT2, WS_NEXT2, (T) + 2) \
    constexpr bool do_issue_ = true;               \
    TLF_DL_COMPUTE(XS, WS)                         \
  }
// Two-stage form: the copy of tile T+1 is issued right after the barrier of step T into the stage
// tile T-1 was read from, and has the whole step to land (an L2 hit takes a few hundred cycles,
// a step a thousand or more).  Half the LDS of the three-stage form, so more workgroups per CU.
#define TLF_DL_STEP2(XS, WS, XS_NEXT, WS_NEXT, T) \
  {                                               \
    TLF_DL_BARRIER(0);                            \
    TLF_DL_ISSUE_SETUP(XS_NEXT, WS_NEXT, (T) + 1) \
    constexpr bool do_issue_ = true;              \
    TLF_DL_COMPUTE(XS, WS)                        \
  }

// NS = LDS stages (2 ... 8), OCC = waves per SIMD the register budget is cut for.
// KG = K-groups: the workgroup holds KG independent sets of WAVES_N x WAVES_M waves; set g runs the
// pipeline over its own 1/KG of the K range in its own LDS stages and the sets' accumulators are
// summed through LDS at the end.  A latency-bound problem (few tiles, long K) then takes 1/KG of
// the steps without partial sums in global memory.
template <int BN, int BM, int WAVES_N, int WAVES_M, bool W8, int NS, int OCC, int KG>
__global__ __launch_bounds__(WAVES_N * WAVES_M * KG * 64) __attribute__((amdgpu_waves_per_eu(OCC, 8)))
void gemm_dlds_kernel(const GemmParams p) {
  static_assert(NS >= 2 && NS <= 8, "2 to 8 stages");
  constexpr int NW = WAVES_N * WAVES_M;       // waves of one set
  static_assert(NW == 2 || NW == 4 || NW == 8, "2, 4 or 8 waves");  // 8: two waves share each SIMD (not faster in the sweeps)
  static_assert(NW * KG <= 16, "at most 1024 threads");
  constexpr int WN = BN / WAVES_N, WM = BM / WAVES_M;
  constexpr int TN = WN / 32, TM = WM / 32;
  constexpr int kWRow = W8 ? kBK : kBK * 2;   // bytes of one W row in a K-tile
  constexpr int kWStep = W8 ? 2 * 1024 : kBK * 2;  // global bytes from one K-tile to the next (int8: two 1 KiB chunks)
  constexpr int kPass = NW * 1024;            // bytes one copy instruction moves per wave set
  constexpr int XP = BM * 128 / kPass;        // copies per lane and stage: x
  constexpr int WP = BN * kWRow / kPass;      // ... and W
  constexpr int kLoads = XP + WP;
  constexpr int kXBytes = BM * 128, kWBytes = BN * kWRow;      // one set's x / W tile
  constexpr int kStage = KG * (kXBytes + kWBytes);             // one stage: x tiles of all sets, then W tiles
  constexpr int kReduce = (KG - 1) * BN * BM * 4;              // fp32 accumulators of sets 1..KG-1
  constexpr int kPool = NS * kStage > kReduce ? NS * kStage : kReduce;
  static_assert(XP >= 1 && WP >= 1 && TN >= 1 && TM >= 1, "tile too small");
  static_assert(kPool <= 160 * 1024, "the stages must fit LDS");
  static_assert((NS - 2) * kLoads <= 63, "vmcnt range");
  __shared__ __attribute__((aligned(1024))) unsigned char pool[kPool];
  unsigned char *const Xs0 = pool, *const Xs1 = pool + kStage, *const Xs2 = pool + 2 * (NS > 2) * kStage;
  unsigned char *const Ws0 = Xs0 + KG * kXBytes, *const Ws1 = Xs1 + KG * kXBytes,
                      *const Ws2 = Xs2 + KG * kXBytes;

  // XCD b % 8 owns the N-tile columns nt = 8 c + xcd.  Its workgroups walk those columns in
  // groups of group_n: inside a group the M-tiles are walked with the group's columns innermost,
  // so the ~32 workgroups resident on an XCD form a patch of (32 / group_n) x panels times
  // group_n W panels and the XCD's L2 fetches each panel once per K-tile.
  // With many more tokens than channels the roles are swapped (xcd_rows): XCD b % 8 owns the M-tile rows
  // mt = 8 r + xcd and walks all columns, group_n rows at a time with the rows innermost, so each XCD's L2 holds an
  // eighth of x and streams W, instead of holding an eighth of W and streaming all of x (at 16384 tokens x is 6 x the
  // bytes of a 5120 x 8192 weight), and 20 tile columns, which do not divide by 8, no longer leave four XCDs with
  // half as much to do again as the other four.
  // Ownership covers the first 8 * floor(T / 8) rows (columns) of the T there are; the tiles of the remaining T % 8
  // are dealt to the XCDs one by one after them (map_main workgroups in, consecutive workgroups sit on consecutive
  // XCDs): an XCD with a whole extra row of tiles would finish a round of tiles after the others (50 tile rows of
  // 256 tokens over 8 XCDs: 7 rows on two of them, 6.25 on average).
  const int walked = p.xcd_rows ? p.n_tiles : p.m_tiles;     // tiles along the dimension the XCD walks in full
  int owned, across;
  if (static_cast<int>(blockIdx.x) < p.map_main) {
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int per_group = p.group_n * walked;
    const int within = local % per_group;
    across = within / p.group_n;
    owned = ((local / per_group) * p.group_n + within % p.group_n) * 8 + xcd;
  } else {
    const int t = static_cast<int>(blockIdx.x) - p.map_main;
    owned = p.map_full + t % p.map_rem;
    across = t / p.map_rem;
  }
  const int mt = p.xcd_rows ? owned : across;
  const int nt = p.xcd_rows ? across : owned;
  if (nt >= p.n_tiles || mt >= p.m_tiles) return;
  const int n0 = nt * BN, m0 = mt * BM;
  const int split = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const unsigned int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned int set_u = wave_all / NW, wave_u = wave_all % NW;  // wave-uniform
  const int wave = static_cast<int>(wave_u);
  // K range of this workgroup, then of this wave set (the host makes the tile count divide by KG)
  const int k_wg = split * p.k_per_split;
  const int nkt = (min(p.K, k_wg + p.k_per_split) - k_wg) / kBK / KG;
  const int k_begin = k_wg + static_cast<int>(set_u) * nkt * kBK;
  const int wn = wave % WAVES_N, wm = wave / WAVES_N;
  const int r = lane & 31, kg = lane >> 5;
  const int64_t ldw_bytes = W8 ? p.K : static_cast<int64_t>(p.K) * 2;

  // copy side: byte offset of this lane's piece for each pass, relative to the tile's first row
  // (rows past the end are clamped to the last row; their results are never stored)
  const unsigned char *xbase = p.x + m0 * p.ldx_bytes + static_cast<int64_t>(k_begin) * 2;
  // int8 weights are in tile order: the tile's first 32-row group and the K term (1 KiB chunks of 32) make the
  // 64-bit base, woff counts row groups from there (a weight may exceed 2 GiB; a tile never does)
  const unsigned char *wbase = W8 ? p.w + (static_cast<int64_t>(n0 >> 5) * (p.K / 32) + k_begin / 32) * 1024
                                  : p.w + n0 * ldw_bytes + static_cast<int64_t>(k_begin) * 2;
  unsigned int xoff[XP], woff[WP];
  {
    const int rl = wave * 8 + (lane >> 3);  // row inside a pass of NW * 8 rows
    const int piece = (lane & 7) ^ ((rl >> 1) & 7);
#pragma unroll
    for (int q = 0; q < XP; ++q) {
      const int row = min(m0 + q * (NW * 8) + rl, p.M - 1) - m0;
      xoff[q] = static_cast<unsigned int>(row * p.ldx_bytes + piece * 16);
    }
    if constexpr (W8) {
      const int rw = wave * 16 + (lane >> 2);  // row inside a pass of NW * 16 rows
      const int pw = (lane & 3) ^ ((rw >> 2) & 3);
#pragma unroll
      for (int q = 0; q < WP; ++q) {
        // atom (row n, piece pw of the K-tile) of the tile-ordered weight, relative to the K-tile's first chunk
        const int n = min(n0 + q * (NW * 16) + rw, p.N - 1);
        woff[q] = static_cast<unsigned int>(((n - n0) >> 5) * (p.K * 32) + (pw >> 1) * 1024 + (pw & 1) * 512 + (n & 31) * 16);
      }
    } else {
#pragma unroll
      for (int q = 0; q < WP; ++q) {
        const int row = min(n0 + q * (NW * 8) + rl, p.N - 1) - n0;
        woff[q] = static_cast<unsigned int>(row * ldw_bytes + piece * 16);
      }
    }
  }
  // fragment side: LDS byte offsets of this lane's pieces
  const int xrow = static_cast<int>(set_u) * kXBytes + (wm * WM + r) * 128;
  const int wrow = static_cast<int>(set_u) * kWBytes + (wn * WN + r) * kWRow;
  int xq[4], wq[2];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    // int8 weights: step (ksp, h) = (s>>1, s&1) uses x piece (2*ksp + kg)*2 + h; bf16: piece 2*ks + kg
    const int c = W8 ? ((s >> 1) * 2 + kg) * 2 + (s & 1) : s * 2 + kg;
    xq[s] = (c ^ ((r >> 1) & 7)) * 16;
  }
#pragma unroll
  for (int s = 0; s < 2; ++s) wq[s] = ((s * 2 + kg) ^ ((r >> 2) & 3)) * 16;

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  TLF_DL_ISSUE(Xs0, Ws0, 0)
  if constexpr (NS == 3) {
    TLF_DL_ISSUE(Xs1, Ws1, 1)
    const int triples = nkt / 3;
    for (int t = 0; t < 3 * triples; t += 3) {
      TLF_DL_STEP(Xs0, Ws0, Xs2, Ws2, t)
      TLF_DL_STEP(Xs1, Ws1, Xs0, Ws0, t + 1)
      TLF_DL_STEP(Xs2, Ws2, Xs1, Ws1, t + 2)
    }
    const int rem = nkt - 3 * triples;
    if (rem >= 1) TLF_DL_STEP(Xs0, Ws0, Xs2, Ws2, 3 * triples)
    if (rem >= 2) TLF_DL_STEP(Xs1, Ws1, Xs0, Ws0, 3 * triples + 1)
  } else if constexpr (NS == 2) {
    const int pairs = nkt / 2;
    for (int t = 0; t < 2 * pairs; t += 2) {
      TLF_DL_STEP2(Xs0, Ws0, Xs1, Ws1, t)
      TLF_DL_STEP2(Xs1, Ws1, Xs0, Ws0, t + 1)
    }
    if (nkt & 1) TLF_DL_STEP2(Xs0, Ws0, Xs1, Ws1, nkt - 1)
  } else {
    // NS >= 4: a ring of stages addressed at run time, NS-1 tiles in flight.  For shapes whose
    // workgroups are few and stream from HBM: a CU's copy rate is (bytes in flight) / latency.
    // Tiles past the end are not requested; the last NS-1 steps then wait for everything.
    for (int t = 1; t < NS - 1; ++t)
      if (t < nkt) TLF_DL_ISSUE(pool + t * kStage, pool + t * kStage + KG * kXBytes, t)
    int cur = 0;
    for (int t = 0; t < nkt; ++t) {
      const int nxt = cur == 0 ? NS - 1 : cur - 1;  // the stage tile t-1 was read from
      unsigned char *const xs = pool + cur * kStage, *const xn = pool + nxt * kStage;
      const bool do_issue_ = t + NS - 1 < nkt;
      if (do_issue_) TLF_DL_BARRIER((NS - 2) * kLoads); else TLF_DL_BARRIER(0);
      TLF_DL_ISSUE_SETUP(xn, xn + KG * kXBytes, t + NS - 1)
      TLF_DL_COMPUTE(xs, xs + KG * kXBytes)
      cur = cur + 1 == NS ? 0 : cur + 1;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped copies of the last two steps must land before LDS is released
  if constexpr (KG > 1) {
    // sum the sets' accumulators: sets 1.. park theirs in LDS (lane-major, conflict free), set 0 adds
    __syncthreads();  // every set is done with the stages
    float *red = reinterpret_cast<float *>(pool);
    const int slot = wave * 64 + lane;
    if (set_u > 0) {
      float *dst = red + (set_u - 1) * (BN * BM) + slot;
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) dst[((i * TM + j) * 16 + v) * (NW * 64)] = acc[i][j][v];
    }
    __syncthreads();
    if (set_u > 0) return;
#pragma unroll
    for (int g = 0; g < KG - 1; ++g) {
      const float *src = red + g * (BN * BM) + slot;
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] += src[((i * TM + j) * 16 + v) * (NW * 64)];
    }
  }
  gemm_epilogue<TN, TM, WN, WM, W8>(p, acc, m0, n0, wn, wm, r, kg, split);
}

// ---------------------------------------------------------------------------
// W-streaming kernel for decode-size batches, int8 weights in tile order.
//
// At these sizes every weight byte is used once per token tile and the kernel lives or dies by how
// the 256 CUs pull the weight matrix out of HBM.  A workgroup owns 32 COLS channels and all tokens.
// Its COLS x KG compute waves are COLS side by side along N times KG along K: wave (n, kh) owns one
// 32-row group of W for the kh-th part of the workgroup's K range and streams it global -> registers:
// one contiguous run, 1 KiB per load instruction, PF K-tiles (2 KiB each) in flight per wave, no LDS
// and no workgroup barrier on the weight side; each lane's 16 bytes are its MFMA A operand after the
// int8 -> bf16 conversion.  Only the activations are shared: one more wave does nothing but copy
// x K-tiles (all tokens x 64 K values, one per K part) global -> LDS into a ring of NS stages, with a
// load counter of its own, so the compute waves' counted waits see nothing but their weight loads;
// one barrier per step hands a stage over.  KG = 2 puts two compute waves on every SIMD, which take
// turns in the matrix pipe while the other one waits for LDS or converts; their accumulators are
// added through LDS at the end.  Accumulator layout and epilogue are those of the tiled kernel.
// COLS = compute waves side by side along N (3 or 4: 96 or 128 channels per workgroup; the host picks
// the width whose workgroup count fills the 256 CUs best - a kernel that is bound by HBM needs every
// CU pulling: 24576 channels are 192 workgroups of 128 but 256 of 96).
template <int TM, int NS, int PF, int KG, int COLS>
__global__ __launch_bounds__((COLS * KG + 1) * 64) __attribute__((amdgpu_waves_per_eu(1, (COLS * KG + 4) / 4)))
void gemm_wstream_kernel(const GemmParams p) {
  constexpr int kWsCols = COLS;
  constexpr int BM = TM * 32;
  constexpr int kCompute = kWsCols * KG;
  constexpr int kXBytes = BM * 128;        // one x tile: BM rows of 64 bf16
  constexpr int kStage = KG * kXBytes;     // one stage: the x tile of every K part
  constexpr int XP = BM / 8;               // copy instructions per x tile (8 rows of 128 bytes each)
  constexpr int kReduce = (KG - 1) * kWsCols * TM * 16 * 64 * 4;
  constexpr int kPool = NS * kStage > kReduce ? NS * kStage : kReduce;
  static_assert(NS >= 2 && kPool <= 160 * 1024, "the stages must fit LDS");
  static_assert((NS - 2) * KG * XP <= 63, "vmcnt range");
  static_assert(PF == 2 || PF == 4 || PF == 8, "2, 4 or 8 tiles in flight");
  __shared__ __attribute__((aligned(1024))) unsigned char pool[kPool];
  const int lane = threadIdx.x & 63;
  const unsigned int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int split = blockIdx.y;
  const int k_begin = split * p.k_per_split;
  const int nh = (min(p.K, k_begin + p.k_per_split) - k_begin) / kBK / KG;  // steps = K-tiles per K part, >= 1 (host)
  const int n0 = blockIdx.x * (kWsCols * 32);

  if (wave == kCompute) {
    // ---- the copy wave: step s brings tile s of every K part to stage s % NS; piece c of LDS row R
    // sits at c ^ ((R >> 1) & 7)
    const unsigned char *xbase = p.x + static_cast<int64_t>(k_begin) * 2;
    unsigned int xoff[XP];
#pragma unroll
    for (int q = 0; q < XP; ++q) {
      const int R = q * 8 + (lane >> 3);
      const int piece = (lane & 7) ^ ((R >> 1) & 7);
      xoff[q] = static_cast<unsigned int>(min(R, p.M - 1) * p.ldx_bytes + piece * 16);  // rows past M: a copy of the last row
    }
    const unsigned int lds0 = TLF_DL_LDSADDR(pool);
#define TLF_WS_ISSUE(S, STAGE)                                                             \
  {                                                                                        \
    const int s_ = min((S), nh - 1);                                                       \
    _Pragma("unroll") for (int h = 0; h < KG; ++h) {                                       \
      const unsigned char *xg_ = xbase + static_cast<int64_t>(h * nh + s_) * (kBK * 2);    \
      const unsigned int xl_ = lds0 + static_cast<unsigned int>(STAGE) * kStage + h * kXBytes; \
      _Pragma("unroll") for (int q = 0; q < XP; ++q) TLF_DL_COPY(xoff[q], xg_, xl_ + q * 1024); \
    }                                                                                      \
  }
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) TLF_WS_ISSUE(s, s)
    int stage = NS - 1;
    for (int s = 0; s < nh; ++s) {
      // step s has landed once at most the NS - 2 steps after it are in flight; the barrier publishes it
      // and says that every compute wave is done with step s - 1, whose stage the next copy overwrites
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NS - 2) * KG * XP) : "memory");
      TLF_WS_ISSUE(s + NS - 1, stage)
      stage = stage + 1 == NS ? 0 : stage + 1;
    }
#undef TLF_WS_ISSUE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no copy may land after the stages are re-used or released
    if constexpr (KG > 1) {  // the two barriers of the accumulator exchange
      asm volatile("s_barrier" ::: "memory");
      asm volatile("s_barrier" ::: "memory");
    }
    return;
  }

  // ---- compute waves
  const int r = lane & 31, kg = lane >> 5;
  const int col = static_cast<int>(wave) % kWsCols, kh = static_cast<int>(wave) / kWsCols;
  const int nt = n0 / 32 + col;
  const bool has_rows = nt * 32 < p.N;
  const int ntc = has_rows ? nt : (p.N - 1) / 32;  // a wave without rows streams the last group and stores nothing
  // chunk c (32 K values of the 32-row group) of this wave's K part is the 1 KiB at wp + c * 1024
  const unsigned char *wp = p.w + (static_cast<int64_t>(ntc) * (p.K / 32) + k_begin / 32 + kh * nh * 2) * 1024 + lane * 16;
  const int xrow = kh * kXBytes + r * 128;
  int xq[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)  // chunk c = i / 2, half h = i % 2 of the tile: x piece 4 c + 2 kg + h
    xq[i] = (((i >> 1) * 4 + kg * 2 + (i & 1)) ^ ((r >> 1) & 7)) * 16;

  floatx16 acc[1][TM];
#pragma unroll
  for (int j = 0; j < TM; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[0][j][v] = 0.f;

  // Tile t of this wave's stream = chunks 2 t and 2 t + 1.  Every load below is unconditional (an index
  // past the end re-reads the last tile, an L2 hit): with branches around them the compiler gives up
  // counting and waits for ALL outstanding loads before every use, which is the end of the prefetch.
  auto load_tile = [&](int t, u32x4 (&dst)[2]) {
    const unsigned char *src = wp + static_cast<int64_t>(min(t, nh - 1)) * 2048;
    dst[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
    dst[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + 1024));
  };
  // quarter q of a tile's 32 weights per lane -> the A operand of MFMA group q
  auto convert_quarter = [&](const u32x4 (&raw)[2], int q, bf16x8 &a) {
    const unsigned int d0 = (q & 1) ? raw[q >> 1].z : raw[q >> 1].x;
    const unsigned int d1 = (q & 1) ? raw[q >> 1].w : raw[q >> 1].y;
    const uint2 c0 = cvt4_i8_bf16(d0), c1 = cvt4_i8_bf16(d1);
    Pack16 t;
    t.u = make_uint4(c0.x, c0.y, c1.x, c1.y);
    a = t.v;
  };
  int cur = 0;
  uint4 bfrag[2][TM];
  auto read_group = [&](int g, uint4 (&dst)[TM]) {
    const unsigned char *xs = pool + cur * kStage + xrow + xq[g];
#pragma unroll
    for (int j = 0; j < TM; ++j) dst[j] = *reinterpret_cast<const uint4 *>(xs + j * (32 * 128));
  };
  auto mfma_group = [&](const bf16x8 &a, const uint4 (&b)[TM]) {
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      Pack16 t;
      t.u = b[j];
      acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, t.v, acc[0][j], 0, 0, 0);
    }
  };

  u32x4 wreg[PF][2];
#pragma unroll
  for (int u = 0; u < PF; ++u) load_tile(u, wreg[u]);
  // One step: tile t = t0 + u of this wave's K part.  GUARDED = the last trip, where tiles may lie past
  // the end of the stream; the trips before it run without a branch.  Within a step the x fragments of
  // MFMA group g + 1 are requested before the MFMAs of group g are issued (two fragment buffers).
  auto tile_step = [&](auto guarded, int t0, auto uc) {
    constexpr bool G = decltype(guarded)::value;
    constexpr int u = decltype(uc)::value;
    const int t = t0 + u;
    const bool live = !G || t < nh;  // uniform
    bf16x8 a[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) convert_quarter(wreg[u], q, a[q]);
    load_tile(t + PF, wreg[u]);  // the registers just read take tile t + PF
    if (live) {
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // step t is in stage cur
      read_group(0, bfrag[0]);
      read_group(1, bfrag[1]);
      mfma_group(a[0], bfrag[0]);
      read_group(2, bfrag[0]);
      mfma_group(a[1], bfrag[1]);
      read_group(3, bfrag[1]);
      mfma_group(a[2], bfrag[0]);
      mfma_group(a[3], bfrag[1]);
      cur = cur + 1 == NS ? 0 : cur + 1;
    }
  };
  auto trip = [&](auto guarded, int t0) {
    tile_step(guarded, t0, std::integral_constant<int, 0>{});
    tile_step(guarded, t0, std::integral_constant<int, 1>{});
    if constexpr (PF > 2) {
      tile_step(guarded, t0, std::integral_constant<int, 2>{});
      tile_step(guarded, t0, std::integral_constant<int, 3>{});
    }
    if constexpr (PF > 4) {
      tile_step(guarded, t0, std::integral_constant<int, 4>{});
      tile_step(guarded, t0, std::integral_constant<int, 5>{});
      tile_step(guarded, t0, std::integral_constant<int, 6>{});
      tile_step(guarded, t0, std::integral_constant<int, 7>{});
    }
  };
  // full trips run unguarded; one guarded trip takes the rest (0 .. PF - 1 tiles)
  const int full = nh / PF;
  int t0 = 0;
  for (int i = 0; i < full; ++i, t0 += PF) trip(std::false_type{}, t0);
  if (t0 < nh) trip(std::true_type{}, t0);

  if constexpr (KG > 1) {
    // add the K parts' accumulators: parts 1.. park theirs in LDS (lane-major, conflict free), part 0 adds.
    // The copy wave has drained its copies before it joins the first barrier.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float *red = reinterpret_cast<float *>(pool);
    const int slot = col * 64 + lane;
    if (kh > 0) {
      float *dst = red + (kh - 1) * (kWsCols * TM * 16 * 64) + slot;
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(j * 16 + v) * (kWsCols * 64)] = acc[0][j][v];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    if (kh > 0) return;
#pragma unroll
    for (int g = 0; g < KG - 1; ++g) {
      const float *src = red + g * (kWsCols * TM * 16 * 64) + slot;
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[0][j][v] += src[(j * 16 + v) * (kWsCols * 64)];
    }
  }
  if (has_rows)
    gemm_epilogue<1, TM, 32, BM, true>(p, acc, 0, n0, col, 0, r, kg, split);
}
#undef TLF_DL_STEP
#undef TLF_DL_STEP2
#undef TLF_DL_COMPUTE
#undef TLF_DL_ISSUE
#undef TLF_DL_ISSUE_PART
#undef TLF_DL_AFTER_GROUP
#undef TLF_DL_ISSUE_SETUP

// s += partial_k for k = 1 .. splits - 1, in that order.  All loads go out before the first add (1, 3 or 7 at a time,
// by a branch the whole grid takes alike): in a rolled loop each load would wait for the add before it, one memory
// round trip per partial in kernels that last a few microseconds.  An index past the end re-reads the last partial
// and is not added.
template <int C, int H>
__device__ __forceinline__ void add_partials_n(const float *src, int64_t mn, int splits, float4 (&s)[H]) {
  float4 t[C][H];
#pragma unroll
  for (int u = 0; u < C; ++u)
#pragma unroll
    for (int h = 0; h < H; ++h) t[u][h] = *reinterpret_cast<const float4 *>(src + min(u + 1, splits - 1) * mn + 4 * h);
#pragma unroll
  for (int u = 0; u < C; ++u)
    if (u + 1 < splits) {
#pragma unroll
      for (int h = 0; h < H; ++h) { s[h].x += t[u][h].x; s[h].y += t[u][h].y; s[h].z += t[u][h].z; s[h].w += t[u][h].w; }
    }
}
// H = consecutive float4 per thread (1 or 2)
template <int H>
__device__ __forceinline__ void add_partials(const float *src, int64_t mn, int splits, float4 (&s)[H]) {
  if (splits <= 2) {
    add_partials_n<1, H>(src, mn, splits, s);
  } else if (splits <= 4) {
    add_partials_n<3, H>(src, mn, splits, s);
  } else {
    add_partials_n<7, H>(src, mn, splits, s);
    for (int k = 8; k < splits; ++k)
#pragma unroll
      for (int h = 0; h < H; ++h) {
        const float4 t = *reinterpret_cast<const float4 *>(src + k * mn + 4 * h);
        s[h].x += t.x; s[h].y += t.y; s[h].z += t.z; s[h].w += t.w;
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
  float4 s1[1] = {*reinterpret_cast<const float4 *>(p.partial + i4 * 4)};
  add_partials<1>(p.partial + i4 * 4, mn, p.splits, s1);
  float4 s = s1[0];
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

// What follows the qkv projection in the decoder is the q/k RMSNorm, RoPE and the KV-cache store
// (reference: tinyvllm/models/qwen3.py:79-94, layers/attention.py:94-95).  When K was split across
// workgroups this kernel is the sum of the partials and that step in one pass: the 16 lanes of a head first
// form h = bf16(sum_k partial_k * scale), exactly what splitk_reduce_kernel would store, and go on from
// there as the kernel that reads the projection from memory does (same bits).
template <bool W8>
__global__ __launch_bounds__(256) void splitk_reduce_qknorm_rope_store_kernel(const GemmParams p,
                                                                              const QkRopeStoreArgs a) {
  const int64_t tok = blockIdx.x;
  const int head = blockIdx.y * 16 + threadIdx.x / 16;
  const int j = threadIdx.x % 16;
  if (head >= a.num_q_heads + 2 * a.num_kv_heads) return;  // whole 16-lane groups leave together
  const int n = head * 128 + j * 8;
  const int64_t mn = static_cast<int64_t>(p.M) * p.N;
  const float *src = p.partial + tok * p.N + n;
  // the token's position and slot, then its cosines and sines, are on their way while the partials are summed
  const QkPieceMeta meta = qk_piece_meta(tok, head, a);
  float4 sum[2] = {*reinterpret_cast<const float4 *>(src), *reinterpret_cast<const float4 *>(src + 4)};
  const QkPieceTable table = qk_piece_table(meta, head, j, a);
  add_partials<2>(src, mn, p.splits, sum);
  float4 s0 = sum[0], s1 = sum[1];
  if (W8) {
    const float4 c0 = *reinterpret_cast<const float4 *>(p.scale + n);
    const float4 c1 = *reinterpret_cast<const float4 *>(p.scale + n + 4);
    s0.x *= c0.x; s0.y *= c0.y; s0.z *= c0.z; s0.w *= c0.w;
    s1.x *= c1.x; s1.y *= c1.y; s1.z *= c1.z; s1.w *= c1.w;
  }
  const uint4 raw = make_uint4(pack_bf16x2(s0.x, s0.y), pack_bf16x2(s0.z, s0.w), pack_bf16x2(s1.x, s1.y),
                               pack_bf16x2(s1.z, s1.w));
  qk_piece_finish(raw, tok, head, j, meta, table, a);
}

// What follows a row-parallel projection in the decoder (o_proj, down_proj) is the residual add and
// an RMSNorm (reference: tinyvllm/models/qwen3.py:163-166 after linear.py:181-183).  When K was
// split across workgroups the projection's value only exists after the partial sums are added, so
// this kernel is that sum and the add-RMSNorm in one pass:
//   h = bf16(sum_k partial_k * scale)            -- exactly what splitk_reduce_kernel would store
//   s = h + residual;  residual_out = bf16(s)
//   y = bf16( bf16(s * rsqrt(mean(s^2) + eps)) * w )
// Thread layout, summation order and rounding points are those of the stand-alone add-RMSNorm
// kernel, so the two routes give the same bits.
struct NormTail {
  const unsigned short *residual;
  const unsigned short *weight;
  unsigned short *y;
  unsigned short *residual_out;
  float eps;
};

// C = partials loaded ahead per chunk (1, 3 or 7: splits <= 2, <= 4, more; fewer where a thread has many chunks).  Every load of the row is unconditional
// (a chunk past the row re-reads the row's last chunk, an idle thread row 0) and stands before the first use, so all of
// them are in flight at once; only the arithmetic and the stores are predicated.
template <int TPR, int MAXC, bool W8, int C>
__device__ __forceinline__ void splitk_reduce_add_rmsnorm_body(const GemmParams &p, const NormTail &t) {
  constexpr int kRowsPerBlock = 256 / TPR;
  const int tid = threadIdx.x;
  const int sub = tid % TPR;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + tid / TPR;
  const bool active = row < p.M;
  const int nchunks = p.N / 8;
  const int64_t mn = static_cast<int64_t>(p.M) * p.N;
  const int64_t off = (active ? row : 0) * p.N;
  float v[MAXC][8];
  uint4 pw[MAXC], pr[MAXC];
  float4 ab[MAXC][2], part[MAXC][C][2], sc[MAXC][2];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int at = min(sub + c * TPR, nchunks - 1) * 8;
    pw[c] = *reinterpret_cast<const uint4 *>(t.weight + at);
    pr[c] = *reinterpret_cast<const uint4 *>(t.residual + off + at);
    const float *src = p.partial + off + at;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      ab[c][h] = *reinterpret_cast<const float4 *>(src + 4 * h);
#pragma unroll
      for (int u = 0; u < C; ++u)
        part[c][u][h] = *reinterpret_cast<const float4 *>(src + min(u + 1, p.splits - 1) * mn + 4 * h);
      if (W8) sc[c][h] = *reinterpret_cast<const float4 *>(p.scale + at + 4 * h);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int chunk = sub + c * TPR;
    if (active && chunk < nchunks) {
      float4 a = ab[c][0], b = ab[c][1];
#pragma unroll
      for (int u = 0; u < C; ++u)
        if (u + 1 < p.splits) {
          const float4 a2 = part[c][u][0], b2 = part[c][u][1];
          a.x += a2.x; a.y += a2.y; a.z += a2.z; a.w += a2.w;
          b.x += b2.x; b.y += b2.y; b.z += b2.z; b.w += b2.w;
        }
      {  // partials beyond those loaded ahead, one at a time
        const float *src = p.partial + off + chunk * 8;
        for (int k = C + 1; k < p.splits; ++k) {
          const float4 a2 = *reinterpret_cast<const float4 *>(src + k * mn);
          const float4 b2 = *reinterpret_cast<const float4 *>(src + k * mn + 4);
          a.x += a2.x; a.y += a2.y; a.z += a2.z; a.w += a2.w;
          b.x += b2.x; b.y += b2.y; b.z += b2.z; b.w += b2.w;
        }
      }
      if (W8) {
        const float4 s0 = sc[c][0], s1 = sc[c][1];
        a.x *= s0.x; a.y *= s0.y; a.z *= s0.z; a.w *= s0.w;
        b.x *= s1.x; b.y *= s1.y; b.z *= s1.z; b.w *= s1.w;
      }
      uint4 hb;  // the projection's bf16 output
      hb.x = pack_bf16x2(a.x, a.y);
      hb.y = pack_bf16x2(a.z, a.w);
      hb.z = pack_bf16x2(b.x, b.y);
      hb.w = pack_bf16x2(b.z, b.w);
      float r[8];
      unpack8(hb, v[c]);
      unpack8(pr[c], r);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[c][i] = __fadd_rn(v[c][i], r[i]);
      *reinterpret_cast<uint4 *>(t.residual_out + off + chunk * 8) = pack8(v[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss = fmaf(v[c][i], v[c][i], ss);
    }
  }
  rmsnorm_finish<TPR, MAXC>(v, pw, ss, active, sub, nchunks, p.N, t.eps, t.y + off);
}

template <int TPR, int MAXC, bool W8>
__global__ __launch_bounds__(256) void splitk_reduce_add_rmsnorm_kernel(const GemmParams p,
                                                                        const NormTail t) {
  constexpr int kAhead = MAXC <= 2 ? 7 : MAXC <= 4 ? 3 : 1;   // what the registers hold: 8 x MAXC x C values per thread
  if (p.splits <= 2 || kAhead == 1)
    splitk_reduce_add_rmsnorm_body<TPR, MAXC, W8, 1>(p, t);
  else if (p.splits <= 4 || kAhead == 3)
    splitk_reduce_add_rmsnorm_body<TPR, MAXC, W8, 3>(p, t);
  else
    splitk_reduce_add_rmsnorm_body<TPR, MAXC, W8, 7>(p, t);
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
//
// PIPE: two batches of weight and activation loads in flight (see below); measured faster up to 8 tokens, where
// a wave's stream is bound by the latency of its own loads (down projection, 1 token: 15.4 -> 11.4 us), slower
// from 9 tokens on, where the activation fragments are twice the weight bytes of a K-block.
template <int MT, int TN, bool W8, bool PIPE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(PIPE ? 4 : 2, PIPE ? 4 : 8)))
void skinny_gemm_kernel(const GemmParams p) {
  constexpr int kWaves = 8;
  // K-blocks of 64 per batch of loads: as many as two batches fit in about 64 registers per lane (the kernel
  // keeps to 128 registers, so that two workgroups share a CU)
  constexpr int kRegsPerBlock = TN * (W8 ? 4 : 8) + MT * 8;
  constexpr int kU = 2 * 4 * kRegsPerBlock <= 64 ? 4 : 2 * 2 * kRegsPerBlock <= 64 ? 2 : 1;
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
    const int nn = wok[t] ? n : 0;
    // int8: tile-ordered weight, this lane's atoms are (row nn, 16 K values 64 kb + 16 g ..)
    wrow[t] = W8 ? p.w + static_cast<int64_t>(nn >> 5) * p.K * 32 + (nn & 31) * 16 + (g >> 1) * 1024 + (g & 1) * 512
                 : p.w + static_cast<int64_t>(nn) * ldw;
  }
  const unsigned char *xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int row = m * 16 + r;
    xok[m] = row < p.M;
    xrow[m] = p.x + static_cast<int64_t>(xok[m] ? row : 0) * p.ldx_bytes;
  }

  if constexpr (PIPE) {
    // Two batches of kU K-blocks are in flight: the loads of batch i + 1 (weights and activations) are issued
    // before batch i is consumed.  Every load is unconditional (a K-block past the wave's range re-reads its
    // last block, a row past N or M reads row 0; what they produce is never stored), so that the waits are
    // counted and a batch is consumed while the next one is still on its way.
    constexpr int kWL = W8 ? 1 : 2;  // 128-bit weight loads per lane, tile and K-block
    struct Batch {
      uint4 w[kU][TN][kWL];
      uint4 x[kU][MT][2];
    };
    auto issue = [&](int kb0, Batch &bt) {
  #pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int kb = min(kb0 + u, kb_end - 1);
  #pragma unroll
        for (int t = 0; t < TN; ++t) {
          if (W8) {
            bt.w[u][t][0] = load_nt_u4(wrow[t] + static_cast<int64_t>(kb) * 2048);
          } else {
            const unsigned char *src = wrow[t] + (static_cast<int64_t>(kb) * kBK + g * 16) * 2;
            bt.w[u][t][0] = load_nt_u4(src);
            bt.w[u][t][kWL - 1] = load_nt_u4(src + 16);
          }
        }
  #pragma unroll
        for (int m = 0; m < MT; ++m) {
          const unsigned char *src = xrow[m] + (static_cast<int64_t>(kb) * kBK + g * 16) * 2;
          bt.x[u][m][0] = *reinterpret_cast<const uint4 *>(src);
          bt.x[u][m][1] = *reinterpret_cast<const uint4 *>(src + 16);
        }
      }
    };
    auto consume = [&](int kb0, const Batch &bt) {
  #pragma unroll
      for (int u = 0; u < kU; ++u) {
        if (kb0 + u >= kb_end) break;  // uniform per wave
        bf16x8 a0[TN], a1[TN];
  #pragma unroll
        for (int t = 0; t < TN; ++t) {
          Pack16 lo, hi;
          if (W8) {
            const uint4 q = bt.w[u][t][0];
            const uint2 c0 = cvt4_i8_bf16(q.x), c1 = cvt4_i8_bf16(q.y);
            const uint2 c2 = cvt4_i8_bf16(q.z), c3 = cvt4_i8_bf16(q.w);
            lo.u = make_uint4(c0.x, c0.y, c1.x, c1.y);
            hi.u = make_uint4(c2.x, c2.y, c3.x, c3.y);
          } else {
            lo.u = bt.w[u][t][0];
            hi.u = bt.w[u][t][kWL - 1];
          }
          a0[t] = lo.v;
          a1[t] = hi.v;
        }
  #pragma unroll
        for (int m = 0; m < MT; ++m) {
          Pack16 b0, b1;
          b0.u = bt.x[u][m][0];
          b1.u = bt.x[u][m][1];
  #pragma unroll
          for (int t = 0; t < TN; ++t) {
            acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[t], b0.v, acc[t][m], 0, 0, 0);
            acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[t], b1.v, acc[t][m], 0, 0, 0);
          }
        }
      }
    };
    if (kb_begin < kb_end) {
      Batch ba, bb;
      issue(kb_begin, ba);
      for (int kb0 = kb_begin; kb0 < kb_end; kb0 += 2 * kU) {
        issue(kb0 + kU, bb);
        consume(kb0, ba);
        issue(kb0 + 2 * kU, ba);
        consume(kb0 + kU, bb);
      }
    }
  } else {
    // weights four K-blocks ahead, activations read from L2 where they are used (predicated: rows past M load nothing)
    constexpr int kUOld = 4;
    for (int kb0 = kb_begin; kb0 < kb_end; kb0 += kUOld) {
      // issue the weight loads of up to kUOld K-blocks
      uint4 wraw[kUOld][TN][W8 ? 1 : 2];
  #pragma unroll
      for (int u = 0; u < kUOld; ++u) {
        const int kb = kb0 + u;
  #pragma unroll
        for (int t = 0; t < TN; ++t) {
          if (W8) {
            wraw[u][t][0] = make_uint4(0, 0, 0, 0);
            if (kb < kb_end && wok[t]) wraw[u][t][0] = load_nt_u4(wrow[t] + static_cast<int64_t>(kb) * 2048);
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
      for (int u = 0; u < kUOld; ++u) {
        const int kb = kb0 + u;
        if (kb >= kb_end) break;  // uniform per wave
        bf16x8 a0[TN], a1[TN];
  #pragma unroll
        for (int t = 0; t < TN; ++t) {
          Pack16 lo, hi;
          if (W8) {
            const uint4 q = wraw[u][t][0];
            const uint2 c0 = cvt4_i8_bf16(q.x), c1 = cvt4_i8_bf16(q.y);
            const uint2 c2 = cvt4_i8_bf16(q.z), c3 = cvt4_i8_bf16(q.w);
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
    if (p.act) {
      // a 16-channel tile is 8 gate rows then the 8 matching up rows: lanes 0..31 hold gate values,
      // lane l + 32 the up values of the same 4 channels; the gate lanes finish the pair
      if (l >= 32) continue;
      float4 u = *reinterpret_cast<const float4 *>(&red[0][tile][l + 32][0]);
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        const float4 v = *reinterpret_cast<const float4 *>(&red[w][tile][l + 32][0]);
        u.x += v.x; u.y += v.y; u.z += v.z; u.w += v.w;
      }
      if (W8) {
        const float4 sc = *reinterpret_cast<const float4 *>(p.scale + n + 8);
        u.x *= sc.x; u.y *= sc.y; u.z *= sc.z; u.w *= sc.w;
      }
      auto rb = [](float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); };
      uint2 st;
      st.x = pack_bf16x2(silu_mul_bf16(rb(s.x), rb(u.x)), silu_mul_bf16(rb(s.y), rb(u.y)));
      st.y = pack_bf16x2(silu_mul_bf16(rb(s.z), rb(u.z)), silu_mul_bf16(rb(s.w), rb(u.w)));
      const int c = (n0 + t * 16) / 2 + (l >> 4) * 4;
      *reinterpret_cast<uint2 *>(p.y + static_cast<int64_t>(token) * (p.N / 2) + c) = st;
      continue;
    }
    uint2 st;
    st.x = pack_bf16x2(s.x, s.y);
    st.y = pack_bf16x2(s.z, s.w);
    *reinterpret_cast<uint2 *>(p.y + static_cast<int64_t>(token) * p.N + n) = st;
  }
}

// Tuning knobs for sweeps, read from the environment ONCE per process (the first GEMM call or
// workspace query): what a query returned stays valid for every later call.
//   TLF_GEMM_PLAN="bn,bm,splits,stages,occ[,kgroups,wn]"  forces one tiled plan
//   TLF_GEMM_SKINNY_MAX_M   hand-over point between the skinny and the tiled kernel (0 ... 64)
//   TLF_GEMM_SKINNY_TN      16-channel tiles per skinny workgroup (1, 2 or 4)
//   TLF_GEMM_GROUP_N        N-tile columns per XCD patch
//   TLF_GEMM_XCD_ROWS=0|1   an XCD owns tile columns | tile rows (the planner picks by tile counts)
//   TLF_GEMM_WSTREAM_M="lo,hi"  token range served by the W-streaming kernel ("0,0": never)
//   TLF_GEMM_WSTREAM_SPLITS     its split of K across workgroups
//   TLF_GEMM_WSTREAM_KG         its K parts inside a workgroup (1 or 2)
//   TLF_GEMM_WSTREAM_COLS       its workgroup width in 32-channel groups (3 or 4)
//   TLF_GEMM_WSTREAM_FORCE=1    take it for every shape in its token range, not only where it measured faster
struct GemmTuning {
  bool has_plan = false;
  int plan[7] = {0, 0, 0, 0, 0, 1, 0};
  int skinny_max_m = kSkinnyMaxM;
  int skinny_tn = 0;
  int skinny_pipe_m = -1;  // forced token limit of the skinny kernel's two-batch pipeline
  int group_n = 0;
  int xcd_rows = -1;   // TLF_GEMM_XCD_ROWS: -1 planner's choice
  int ws_min_m = 13, ws_max_m = 224;  // token range of the W-streaming kernel (int8 weights)
  bool ws_range_set = false;          // the range came from TLF_GEMM_WSTREAM_M: taken literally
  int ws_splits = 0;                               // forced split of K for it
  int ws_kg = 0;                                   // forced K parts per workgroup (1 or 2)
  bool ws_force = false;                           // take it for every shape in its token range
  int ws_cols = 0;                                 // forced workgroup width in 32-channel groups (3 or 4)
};

inline const GemmTuning &gemm_tuning() {
  static const GemmTuning t = [] {
    GemmTuning g;
    if (const char *e = getenv("TLF_GEMM_PLAN")) {
      int v[7] = {0, 0, 0, 0, 0, 1, 0};
      if (sscanf(e, "%d,%d,%d,%d,%d,%d,%d", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5], &v[6]) >= 5) {
        g.has_plan = true;
        for (int i = 0; i < 7; ++i) g.plan[i] = v[i];
      }
    }
    if (const char *e = getenv("TLF_GEMM_SKINNY_MAX_M")) {
      const int v = atoi(e);  // the skinny kernel covers at most 4 x 16 tokens
      g.skinny_max_m = v < 0 ? 0 : v > 64 ? 64 : v;
    }
    if (const char *e = getenv("TLF_GEMM_SKINNY_TN")) {
      const int v = atoi(e);
      if (v == 1 || v == 2 || v == 4) g.skinny_tn = v;
    }
    if (const char *e = getenv("TLF_GEMM_SKINNY_PIPE_M")) g.skinny_pipe_m = atoi(e);
    if (const char *e = getenv("TLF_GEMM_GROUP_N")) g.group_n = atoi(e) > 0 ? atoi(e) : 1;
    if (const char *e = getenv("TLF_GEMM_XCD_ROWS")) g.xcd_rows = atoi(e) != 0;
    if (const char *e = getenv("TLF_GEMM_WSTREAM_M")) {
      int lo = 0, hi = 0;
      if (sscanf(e, "%d,%d", &lo, &hi) == 2) {
        g.ws_min_m = lo < 1 ? 1 : lo;
        g.ws_max_m = hi > 224 ? 224 : hi;  // seven token tiles of 32 is the tallest instance
        g.ws_range_set = true;
      }
    }
    if (const char *e = getenv("TLF_GEMM_WSTREAM_SPLITS")) g.ws_splits = atoi(e) > 0 ? atoi(e) : 0;
    if (const char *e = getenv("TLF_GEMM_WSTREAM_FORCE")) g.ws_force = atoi(e) != 0;
    if (const char *e = getenv("TLF_GEMM_WSTREAM_COLS")) g.ws_cols = atoi(e);
    if (const char *e = getenv("TLF_GEMM_WSTREAM_KG")) g.ws_kg = atoi(e) == 1 || atoi(e) == 2 ? atoi(e) : 0;
    return g;
  }();
  return t;
}

template <bool W8>
int launch_skinny(const GemmParams &p, hipStream_t stream) {
  if (p.M > 64) return TLF_E_UNSUPPORTED;  // four 16-token MFMA tiles at most
  const int mt = (p.M + 15) / 16;
  const int tiles16 = (p.N + 15) / 16;
  // more channels per workgroup reuse the activation fragments, as long as the grid stays large
  int tn = 1;
  if (tiles16 >= 4 * 512) tn = 4;
  else if (tiles16 >= 2 * 512) tn = 2;
  if (gemm_tuning().skinny_tn) tn = gemm_tuning().skinny_tn;
  const dim3 grid((tiles16 + tn - 1) / tn);
  // two batches in flight pay where a CU holds one workgroup or less (N <= 4096: o_proj 5.8 / 6.0 us at 6 / 8 tokens
  // against 6.4 / 6.7, down 12.3 / 12.7 against 14.5 / 15.5) and up to 4 tokens everywhere; a wide N at 5 ... 8 tokens
  // is 3-5 % faster on the plain loop
  const int pipe_m = gemm_tuning().skinny_pipe_m >= 0 ? gemm_tuning().skinny_pipe_m : tiles16 <= 256 ? 8 : 4;
#define TLF_SK(MT_, TN_)                                                                                 \
  if (MT_ == 1 && p.M <= pipe_m)                                                                         \
    TLF_LAUNCH((skinny_gemm_kernel<MT_, TN_, W8, MT_ == 1>), grid, dim3(512), 0, stream, p);     \
  else                                                                                                   \
    TLF_LAUNCH((skinny_gemm_kernel<MT_, TN_, W8, false>), grid, dim3(512), 0, stream, p)
#define TLF_SK_TN(MT_)      \
  if (tn == 4) {            \
    TLF_SK(MT_, 4);         \
  } else if (tn == 2) {     \
    TLF_SK(MT_, 2);         \
  } else {                  \
    TLF_SK(MT_, 1);         \
  }
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
  int bn, bm;         // tile: output channels x tokens
  int stages;         // LDS stages (2 or 3)
  int occ;            // waves per SIMD the kernel's registers are budgeted for
  int splits;         // split-K factor
  int k_per_split;
  int group_n = 1;    // N-tile columns per XCD patch
  int kgroups = 1;    // wave sets splitting K inside a workgroup
  int wn = 0;         // waves along the channel side of the tile (0: the tile's default layout)
  bool wstream = false;  // the W-streaming kernel: bn = 128 channels, bm = all tokens rounded to 32
};

// Plan of the W-streaming kernel (int8 weights, at most 256 tokens).  A workgroup takes 128 channels
// and all tokens; K is split across workgroups until about 256 of them exist (small N), each split
// keeping at least 8 K-tiles.  The fused activation needs whole sums, so it takes the kernel only
// when N alone fills the machine.
inline bool plan_wstream(int M, int N, int K, int act, GemmPlan &g) {
  const GemmTuning &t = gemm_tuning();
  if (t.has_plan || M > t.ws_max_m || M < 1 || act == 2) return false;
  if (M < t.ws_min_m) {
    // Below 13 tokens the skinny kernel runs, except on big matrices, where one workgroup per 96 or 128 channels
    // streaming its rows beats the skinny kernel's many small workgroups.  Cold weights, us, W-streaming / skinny
    // at 1 / 4 / 8 / 12 tokens: 51200 x 5120 44.8 / 45.1 / 45.8 / 46.7 against 53.6 / 55.0 / 49.8 / 51.5;
    // 5120 x 25600 27.5 / 26.6 / 26.7 / 26.8 against 34.5 / 35.5 / 42.7 / 49.0; 10240 x 5120 15.5 / 14.4 / 15.0 / 14.5
    // against 14.5 / 14.8 / 15.8 / 18.3; 5120 x 8192 13.6 / 13.5 / 13.5 / 13.9 against 12.5 / 13.0 / 15.4 / 17.6;
    // 24576 x 4096 18.8 / 18.8 / 18.9 / 18.8 against 18.6 / 18.4 / 19.4 / 20.5; but 4096 x 12288 16.4 / 15.3 / 15.6 / 15.7
    // against 11.4 / 11.2 / 12.8 / 16.6 and 6144 x 4096 10.0 against 8.2 ... 10.3.
    const int64_t nk = static_cast<int64_t>(N) * K;
    const bool big = nk >= 120000000;
    const bool mid = M >= 8 && nk >= 40000000 && N >= 5120;
    if (t.ws_range_set || !(big || mid)) return false;
  }
  if (M > 128 && !(N >= 256 * 96)) return false;  // 129 ... 224 tokens: 96-channel workgroups on a wide N only (below)
  // 13 ... 16 tokens, cold weights, W-streaming / skinny kernel at 16 tokens: qkv 10.5 / 11.8 us, gate_up 20.1 / 22.2,
  // down 16.5 / 18.1, but o_proj (N = 4096, K = 4096: 43 workgroups x 4 splits) 9.3 / 7.8
  if (M <= kSkinnyMaxM && !t.ws_force && N <= 4096 && K <= 4096) return false;
  // 128 or 96 channels per workgroup: whichever count of workgroups fills whole rounds of 256 CUs better
  auto fill = [](int wgs) { return static_cast<double>(wgs) / ((wgs + 255) / 256 * 256); };
  const int ktiles = K / kBK;
  const bool narrow = (N + 127) / 128 < 96;  // fewer than 96 workgroups of 128 channels: K has to be split
  int cols = 4;
  if (N >= 256 * 96 && fill((N + 95) / 96) > fill((N + 127) / 128) + 0.1) cols = 3;
  if (narrow) cols = 3;
  // 160 ... 224 tokens: seven waves of up to 256 registers (96-channel workgroups, two K parts); measured on
  // gate_up with cold weights 46.7 / 49.8 / 58.9 us at 160 / 192 / 224 tokens against 53.3 / 56.2 / 65.5 for the
  // tiled plans, and no faster than the 256 x 128 tile at 256
  if (M > 128) cols = 3;
  if (t.ws_cols == 3 || t.ws_cols == 4) cols = t.ws_cols;
  const int n_wg = (N + cols * 32 - 1) / (cols * 32);
  // ... and only when those workgroups fill whole rounds of the CUs: 51200 channels are 534 workgroups (2.1 rounds), and
  // the tiled plans win there (160 / 192 / 224 tokens 114.3 / 130.4 / 146.4 us against 122.6 / 143.1 / 164.3)
  if (M > 128 && !t.ws_force && fill(n_wg) < 0.9) return false;
  int splits = 1;
  // Measured against the tiled plans on the Qwen3-8B projections with cold weights: a wide N (gate_up)
  // wins at every size up to 128 tokens (24 / 28 / 37 us at 32 / 64 / 128 tokens against 36 / 38 / 43);
  // a narrow N needs a split of K, whose activation traffic and partial sums grow with the token count:
  // with 96-channel workgroups, K split 4 ways and one K part per workgroup (two for a long K) it wins up to
  // 80 tokens (qkv 10.5 / 11.2 / 14.4 / 16.2 us at 17 / 32 / 64 / 80 tokens against 14.3 / 14.7 / 16.3 / 17.3 for
  // the tiled plans, o_proj 9.5 / 9.7 / 12.1 / 14.2 against 13.1 / 13.5 / 14.9 / 14.7) and, with a long K (down
  // projection), up to 32 (16.0 / 16.9 at 17 / 32 against 25.8 / 25.9); above that the tiled plans are faster.
  // The bigger narrow matrices of the Qwen3-32B shape keep winning up to 128 tokens (cold weights, us, W-streaming /
  // tiled at 64 / 96 / 128 tokens: 10240 x 5120 20.0 / 24.3 / 28.2 against 20.0 / 31.3 / 35.8; 5120 x 8192 18.0 / 21.6 /
  // 25.1 against 23.2 / 26.2 / 31.0; 5120 x 25600 36.7 / 44.3 / 49.8 against 48.6 / 56.6 / 65.8).
  const bool big_narrow = static_cast<int64_t>(N) * K >= 40000000 && N >= 5120 && M <= 128;
  if (!t.ws_force && narrow && M > (ktiles >= 128 ? 32 : 80) && !big_narrow) return false;
  if (act) {
    if (narrow) return false;
  } else {
    splits = (256 + n_wg / 2) / n_wg;
    if (narrow && splits > 4) splits = 4;
    if (splits > ktiles / 8) splits = ktiles / 8;
    if (splits > 16) splits = 16;
    if (t.ws_splits) splits = t.ws_splits < ktiles ? t.ws_splits : ktiles;
    if (splits < 1) splits = 1;
  }
  const int kt_per = (ktiles + splits - 1) / splits;
  const int tm = (M + 31) / 32;
  g.wstream = true;
  g.bn = cols * 32;
  g.bm = tm * 32;
  // two K parts (two compute waves per SIMD) for a wide N from 33 tokens on and for a narrow N with a long K;
  // elsewhere one part is 5-15 % faster (gate_up at 32 tokens 19.5 against 20.8 us, qkv 11.2 against 12.0)
  int kg = ktiles % 2 == 0 && kt_per >= 4 && (narrow ? ktiles >= 128 : M > 32) ? 2 : 1;
  if (t.ws_kg && (t.ws_kg == 1 || ktiles % 2 == 0)) kg = t.ws_kg;
  if (tm > 7 || (tm > 4 && !(kg == 2 && cols == 3))) return false;  // the tall instances exist in that form only
  g.stages = tm >= 7 ? 2 : kg == 2 && tm >= 3 ? 3 : 4;
  g.occ = kg;
  g.kgroups = kg;
  g.group_n = 1;
  g.k_per_split = kt_per * kBK;
  g.splits = (ktiles + kt_per - 1) / kt_per;
  return true;
}

// Tile, stage and split-K choice, from sweeps over the Qwen3-8B projection shapes on MI355X
// (M from 24 to 8192, int8 and bf16 weights).  Few tiles: small tiles and a split of K so that
// about a thousand workgroups exist (each split keeps at least 16 K-tiles); from 256 tiles of
// 128 x 128 on: no split; from 1024 on: 256 channels x 128 tokens.
inline GemmPlan plan_gemm(int M, int N, int K, bool w8) {
  GemmPlan g;
  auto tiles = [&](int bn, int bm) { return ((N + bn - 1) / bn) * ((M + bm - 1) / bm); };
  auto pow2_floor = [](int v) { int p = 1; while (p * 2 <= v) p *= 2; return p; };
  const int ktiles = K / kBK;
  const int max_split = ktiles / 16 > 1 ? pow2_floor(ktiles / 16) : 1;
  int splits = 1;
  const int n128 = (N + 127) / 128;
  // Decode-size batches of int8 weights, from a sweep of every tile instance and split over the four Qwen3-8B
  // projections on cold weights (us, this plan / the plan it replaced):
  //  - moderate N, long K (down projection, 4096 x 12288): one M-tile as tall as the batch, 128 channels wide, K
  //    split 8 ways (256 workgroups): 48 / 64 / 96 / 160 / 192 tokens 20.8 / 20.3 / 24.3 / 29.3 / 32.7 against
  //    23.8 / 23.1 / 28.9 / 31.0 / 36.5;
  //  - moderate N, K of 64 tiles, 48 tile columns and more (qkv, 6144 x 4096) above 160 tokens: the same tall
  //    tile with K split 4 ways up to 224 tokens (176 / 192 / 208: 23.9 / 24.5 / 26.1 against 32.8 / 32.3 / 33.4),
  //    two 128 x 128 tiles with K split in two above (256 tokens: 27.0 against 33.4);
  //  - wide N (gate_up) from 193 to 256 tokens: 256 x 128 tile with eight waves (256 tokens: 60.8 against 71.2).
  const bool tall_long_k = w8 && n128 < 128 && ktiles > 64 && M > 32 && M <= 208;
  const bool mid_k64 = w8 && n128 < 128 && n128 >= 48 && ktiles <= 64 && ktiles % 4 == 0 && M > 160 && M <= 256;
  // The narrow projections of the Qwen3-32B shape (10240 x 5120, 5120 x 8192, 5120 x 25600) above the W-streaming
  // kernel's 128 tokens, from a sweep of 16 plans on cold weights (us, this plan / the rules below): 192 tokens
  // 128 x 64 tiles with K split 2 (4 from K = 8192 on) 40.4 / 33.3 / 81.3 against 48.4 / 42.3 / 88.9; 256 tokens 256 x 128
  // tiles, same splits, 45.2 / 37.4 / 88.8 against 52.8 / 43.9 / 97.8.  (The Qwen3-8B shapes keep the rules below: the
  // same sweep found nothing faster for them.)
  const bool big_narrow = w8 && n128 < 128 && N >= 5120 && static_cast<int64_t>(N) * K >= 40000000;
  bool measured_splits = false;   // the split came out of a sweep: the long-K adjustment below leaves it alone
  if (big_narrow && M > 128 && M <= 256) {
    if (M <= 192) {
      g.bn = 128; g.bm = 64; g.stages = 4; g.occ = 3; g.wn = 4;
    } else {
      g.bn = 256; g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 8;
    }
    splits = K >= 8192 ? 4 : 2;
    measured_splits = true;
  } else if (tall_long_k || (mid_k64 && M <= 224)) {
    g.bn = 128; g.bm = M <= 64 ? 64 : (M + 31) / 32 * 32; g.wn = 4;
    g.stages = g.bm == 64 ? 4 : 3; g.occ = g.bm == 64 ? 3 : 2;
    splits = tall_long_k ? 8 : 4;
  } else if (mid_k64) {
    g.bn = 128; g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 4;
    splits = 2;
  } else if (w8 && n128 >= 128 && M > 192 && M <= 256 && tiles(256, 128) >= 160) {
    g.bn = 256; g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 8;
  } else if (M > 64 && M <= 224 && (N + 127) / 128 >= 128) {
    // a decode-size batch against a very wide N (gate_up, LM head): one M-tile as tall as the
    // batch (rounded to 32 tokens), so nothing is padded to a power of two and W passes through
    // each CU once; four waves side by side along N.  Measured on 24576 x 4096 at M = 130:
    // 62 -> 49 us (int8), 56 -> 40 us (bf16); LM head 342 -> 300 us.
    g.bn = 128; g.bm = (M + 31) / 32 * 32; g.stages = 3; g.occ = 2; g.wn = 4;
  } else if (w8 && M > 64 && M <= 160 && (N + 63) / 64 <= 128 && ktiles % 2 == 0 &&
             (ktiles > 64 || (M > 128 && tiles(64, 64) > 256))) {
    // decode-size batch, moderate N: again one M-tile as tall as the batch, here 64 channels wide
    // with two waves per set and two sets splitting K inside the workgroup, three stages, plus a
    // split of K across workgroups.  Measured at M = 130 (M = 96): 6144 x 4096 25 -> 20 us,
    // 4096 x 12288 40 -> 30 us (29 -> 24 us); 4096 x 4096 is better off below.
    g.bn = 64; g.bm = (M + 31) / 32 * 32; g.stages = 3; g.occ = 2; g.wn = 2; g.kgroups = 2;
    splits = ktiles >= 128 ? 4 : 2;
  } else if (tiles(64, 64) <= 512) {
    g.bn = 64; g.bm = 64; g.stages = 2; g.occ = 4;
    splits = pow2_floor(1024 / tiles(64, 64));
    if (ktiles <= 64 && ktiles % 4 == 0) {
      // moderate K: split it between wave sets inside the workgroup instead (no partial sums in
      // global memory, no reduce kernel); measured 5-20 % faster on 4096 x 4096 and 6144 x 4096
      g.kgroups = tiles(64, 64) <= 256 ? 4 : 2;
      splits = tiles(64, 64) <= 128 ? 2 : 1;
      // weights stream from HBM: a third stage keeps two tiles per wave set in flight
      // (int8 only: 144 KB of LDS; measured 17.1 -> 14.1 us on 4096 x 4096 at M = 130)
      if (w8 && g.kgroups == 4) g.stages = 3;
    } else if (M > 64 && ktiles > 64) {
      // long K (down projection): 128 channels x 64 tokens, split of K, four-stage ring
      // (measured 42.6 -> 38.2 us at M = 130, 55.7 -> 44.5 us at M = 256 on 4096 x 12288)
      g.bn = 128; g.bm = 64; g.stages = 4; g.occ = 3;
      splits = 4;
      if (M > 160) {
        // two M-tiles of 128 with cold weights: 43.3 -> 41.2 us at M = 192, 46.4 -> 40.7 us at M = 256
        g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 2;
      }
    }
  } else if (tiles(128, 128) < 256) {
    g.bn = 128; g.bm = 64; g.stages = 2; g.occ = 3;
    splits = pow2_floor(1024 / tiles(128, 64));
  } else if (M <= 64) {
    // one M-tile and a very wide N (the LM head at small batch): pure weight streaming
    g.bn = 128; g.bm = 64; g.stages = 2; g.occ = 3;
  } else if (w8) {
    // int8 weights: every wave of a tile spans all of its tokens (waves side by side along N), so
    // each weight is converted to bf16 by one wave only; a 2 x 2 wave layout converts it twice and
    // is 5-10 % slower although it reads fewer LDS bytes per MFMA.
    const int t256 = tiles(256, 256);
    const int m256 = (M + 255) / 256 * 256;  // rows the 256-token tiles would compute
    if (t256 >= 160 && !(t256 > 256 && t256 < 512) && m256 * 20 <= M * 23) {
      // 256 x 256 tile, eight waves of 32 channels x 256 tokens, one workgroup per CU: fewest
      // copied bytes per flop (1.19-1.31 PFLOP/s at M = 8192 against 1.09-1.16 for 256 x 128).
      // Between one and two tiles per CU the second round would be half empty; more than 15 % of
      // padding rows costs more than the tile saves.
      g.bn = 256; g.bm = 256; g.stages = 3; g.occ = 2; g.wn = 8;
    } else if (const int t = tiles(256, 128); t >= 224 && t * 100 >= (t + 255) / 256 * 256 * 85) {
      // 256 x 128 tile, eight waves of 32 channels x 128 tokens, one workgroup per CU, when such tiles fill
      // whole rounds of the CUs (4096 x 4096 and 4096 x 12288 at 2048 tokens: one tile per CU, +8 % and +11 %
      // over two 128 x 128 tiles per CU; 6144 x 4096 at 4096 tokens: three rounds, +13 % over the four-wave form)
      g.bn = 256; g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 8;
    } else if (tiles(128, 128) < 1024) {
      g.bn = 128; g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 4;
    } else {
      g.bn = 256; g.bm = 128; g.stages = 2; g.occ = 2; g.wn = 4;  // 64 KB of LDS: two workgroups per CU
    }
  } else if (tiles(128, 128) < 1024 && tiles(256, 128) < 256) {
    g.bn = 128; g.bm = 128; g.stages = 3; g.occ = 2; g.wn = 2;
  } else if (!w8 && M >= 2048 && ktiles <= 64 && tiles(256, 256) >= 512 && (M + 255) / 256 * 256 * 20 <= M * 23) {
    // bf16 weights at prefill sizes, two rounds of 256 x 256 tiles or more, K up to 4096: the eight-wave 256 x 256 tile with two LDS
    // stages (a bf16 K-tile of it is 64 KB; three stages do not fit).  TFLOP/s against the 256 x 128 tile at 8192 /
    // 16384 tokens: 6144 x 4096 1125 / 1207 against 944 / 1102, 4096 x 4096 1272 / 1252 against 1117 / 1157,
    // 24576 x 4096 1196 / 1189 against 1109 / 1122; 4096 x 12288 (192 K-tiles) ties or loses 1-3 %, hence the bound on K.
    g.bn = 256; g.bm = 256; g.stages = 2; g.occ = 2; g.wn = 8;
  } else {  // bf16, one 256 x 128 tile per CU or more (measured 7-10 % faster than 128 x 128 from there on)
    g.bn = 256; g.bm = 128; g.stages = 3; g.occ = 1;
  }
  // a long K wants a split of its own: no workgroup walks more than ~48 K-tiles when splitting
  if (!measured_splits && splits > 1 && splits < pow2_floor(ktiles / 48)) splits = pow2_floor(ktiles / 48);
  if (splits > max_split) splits = max_split;
  if (splits > 16) splits = 16;
  if (splits < 1) splits = 1;
  const int kt_per = (ktiles + splits - 1) / splits;
  g.k_per_split = kt_per * kBK;
  g.splits = (ktiles + kt_per - 1) / kt_per;
  return g;
}

// A forced plan (GemmTuning) replaces the planner's choice.
inline bool plan_override(GemmPlan &g, int K) {
  const GemmTuning &t = gemm_tuning();
  if (!t.has_plan) return false;
  int sp = t.plan[2];
  g.kgroups = t.plan[5];
  g.wn = t.plan[6];
  const int ktiles = K / kBK;
  if (sp < 1) sp = 1;
  if (sp > ktiles) sp = ktiles;
  const int kt_per = (ktiles + sp - 1) / sp;
  g.bn = t.plan[0]; g.bm = t.plan[1]; g.stages = t.plan[3]; g.occ = t.plan[4];
  g.k_per_split = kt_per * kBK;
  g.splits = (ktiles + kt_per - 1) / kt_per;
  return true;
}

inline int skinny_max_m() { return gemm_tuning().skinny_max_m; }

// plan_out != nullptr: nothing is launched; the eight plan fields are written there instead and the
// return code says whether a kernel instance exists for the plan.
template <bool W8>
int launch_gemm(const void *x, int64_t x_stride, const void *w, const float *scale, void *y,
                int32_t M, int32_t N, int32_t K, void *workspace, size_t workspace_bytes,
                hipStream_t stream, int32_t *plan_out = nullptr, int32_t act = 0,
                const NormTail *tail = nullptr, const QkRopeStoreArgs *qk = nullptr) {
  const bool dry = plan_out != nullptr;
  GemmParams p;
  p.x = static_cast<const unsigned char *>(x);
  p.ldx_bytes = x_stride * 2;
  p.w = static_cast<const unsigned char *>(w);
  p.scale = scale;
  p.y = static_cast<unsigned short *>(y);
  p.partial = nullptr;
  p.M = M; p.N = N; p.K = K;
  p.act = act;
  p.amax = nullptr;
  p.amax_parts = 0;
  p.xcd_rows = 0;
  p.map_main = 0; p.map_full = 0; p.map_rem = 1;
  GemmPlan g;
  const bool wstream = W8 && plan_wstream(M, N, K, act, g);
  if (M <= skinny_max_m() && !wstream) {
    p.k_per_split = K; p.splits = 1; p.m_tiles = 1; p.n_tiles = 1; p.group_n = 1; p.xcd_rows = 0;
    p.map_main = 0; p.map_full = 0; p.map_rem = 1;
    if (dry) {
      const int32_t skinny[8] = {0, 0, 0, 0, 1, 1, K, 1};  // tile 0 x 0 = the skinny kernel
      for (int i = 0; i < 8; ++i) plan_out[i] = skinny[i];
      return TLF_OK;
    }
    if (act == 2) return TLF_E_UNSUPPORTED;  // the caller stages the logits and runs tlf_argmax
    return launch_skinny<W8>(p, stream);
  }
  if (!wstream) {
    g = plan_gemm(M, N, K, W8);
    plan_override(g, K);
  }
  if (act) {  // the activation needs whole sums: no split of K across workgroups
    g.splits = 1;
    g.k_per_split = K;
  }
  if (g.kgroups > 1) {
    // every split must hand each wave set the same whole number of K-tiles
    const int ktiles = K / kBK;
    if (ktiles % g.kgroups) return TLF_E_UNSUPPORTED;
    int kt_per = g.k_per_split / kBK;
    kt_per = (kt_per + g.kgroups - 1) / g.kgroups * g.kgroups;
    g.k_per_split = kt_per * kBK;
    g.splits = (ktiles + kt_per - 1) / kt_per;
  }
  p.k_per_split = g.k_per_split;
  p.splits = g.splits;
  p.m_tiles = (M + g.bm - 1) / g.bm;
  p.n_tiles = (N + g.bn - 1) / g.bn;
  if (act == 2 && !dry) {  // argmax keys: at most N / 32 + 8 columns per token for any tile shape
    const size_t need = static_cast<size_t>(M) * (N / 32 + 8) * sizeof(unsigned long long);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u))
      return TLF_E_WORKSPACE;
    p.amax = static_cast<unsigned long long *>(workspace);
  }
  if (g.splits > 1 && !dry) {
    const size_t need = static_cast<size_t>(g.splits) * M * N * sizeof(float);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u))
      return TLF_E_WORKSPACE;
    p.partial = static_cast<float *>(workspace);
  }
  // XCD patch: group as many N-tile columns as divide this XCD's share evenly (up to 4), once
  // there are enough M-tiles for the patch to matter
  // An XCD owns tile rows instead of tile columns (see the kernel) from 16 tile rows on.  Either way the rows
  // (columns) that do not divide by 8 are dealt out tile by tile, so both forms keep the XCDs level; rows then win by
  // the traffic: TFLOP/s rows / columns at 8192, 12800 and 16384 tokens: 10240 x 5120 1128 / 1057, 1219 / 1159,
  // 1282 / 1251; 51200 x 5120 1293 / 1232, 1275 / 1233, 1302 / 1241; 5120 x 8192 and 5120 x 25600 within 2 %; the
  // Qwen3-8B shapes 0 ... +4 %; at 4096 tokens (16 tile rows) -4 ... +6 %.  (With whole rows or columns per XCD 50 tile
  // rows cost 7 rounds on two XCDs against 6.25 on average: 5120 x 8192 at 12800 tokens 1104 -> 1281 TFLOP/s.)
  // TLF_GEMM_XCD_ROWS = 0 / 1 forces the choice for tuning.
  p.xcd_rows = p.m_tiles >= 16;
  if (gemm_tuning().xcd_rows >= 0) p.xcd_rows = gemm_tuning().xcd_rows && p.m_tiles >= 8;
  const int owned_total = p.xcd_rows ? p.m_tiles : p.n_tiles, walked = p.xcd_rows ? p.n_tiles : p.m_tiles;
  const int owned_each = owned_total / 8;     // rows (columns) every XCD owns; the other owned_total % 8 are dealt out tile by tile
  {
    g.group_n = 1;
    if (walked >= 8 && owned_each > 0) g.group_n = owned_each % 4 == 0 ? 4 : owned_each % 3 == 0 ? 3 : owned_each % 2 == 0 ? 2 : 1;
    if (gemm_tuning().group_n && owned_each > 0 && owned_each % gemm_tuning().group_n == 0) g.group_n = gemm_tuning().group_n;
  }
  p.group_n = g.group_n;
  p.map_full = owned_each * 8;
  p.map_rem = owned_total - p.map_full;
  p.map_main = owned_each * 8 * walked;
  if (p.map_rem == 0) p.map_rem = 1;          // never used then (no workgroup past map_main); keeps the kernel's % defined
  const dim3 grid(static_cast<unsigned>(p.map_main + (owned_total - p.map_full) * walked), g.splits);
  bool launched = false;
  if constexpr (W8) {
    if (g.wstream) {
      const dim3 wgrid(p.n_tiles, g.splits);
#define TLF_WS(TM_, NS_, PF_, KG_, COLS_)                                                           \
  if (!launched && g.bm == TM_ * 32 && g.kgroups == KG_ && g.bn == COLS_ * 32) {                    \
    if (!dry)                                                                                       \
      TLF_LAUNCH((gemm_wstream_kernel<TM_, NS_, PF_, KG_, COLS_>), wgrid,                   \
                         dim3((COLS_ * KG_ + 1) * 64), 0, stream, p);                               \
    launched = true;                                                                                \
  }
      // registers per wave: 9 waves (4 x 2 + 1) leave 168, so the tall tiles keep 4 weight tiles in flight there
      TLF_WS(1, 4, 8, 1, 4) TLF_WS(2, 4, 8, 1, 4) TLF_WS(3, 4, 8, 1, 4) TLF_WS(4, 4, 8, 1, 4)
      TLF_WS(1, 4, 8, 2, 4) TLF_WS(2, 4, 8, 2, 4) TLF_WS(3, 3, 4, 2, 4) TLF_WS(4, 3, 4, 2, 4)
      TLF_WS(1, 4, 8, 1, 3) TLF_WS(2, 4, 8, 1, 3) TLF_WS(3, 4, 8, 1, 3) TLF_WS(4, 4, 8, 1, 3)
      TLF_WS(1, 4, 8, 2, 3) TLF_WS(2, 4, 8, 2, 3) TLF_WS(3, 3, 8, 2, 3) TLF_WS(4, 3, 8, 2, 3)
      TLF_WS(5, 3, 4, 2, 3) TLF_WS(6, 3, 4, 2, 3)  // seven waves: 256 registers each
      TLF_WS(7, 2, 4, 2, 3)
#undef TLF_WS
    }
  }
#define TLF_TILE_KG(BN_, BM_, WN_, WM_, NS_, OCC_, KG_)                                     \
  if (!launched && g.bn == BN_ && g.bm == BM_ && g.stages == NS_ && g.occ == OCC_ &&        \
      g.kgroups == KG_ && (g.wn == 0 || g.wn == WN_)) {                                                                   \
    p.amax_parts = p.n_tiles * WN_;                                                         \
    if (!dry)                                                                               \
      TLF_LAUNCH((gemm_dlds_kernel<BN_, BM_, WN_, WM_, W8, NS_, OCC_, KG_>), grid,  \
                         dim3(WN_ * WM_ * KG_ * 64), 0, stream, p);                         \
    launched = true;                                                                        \
  }
#define TLF_TILE(BN_, BM_, WN_, WM_, NS_, OCC_) TLF_TILE_KG(BN_, BM_, WN_, WM_, NS_, OCC_, 1)
  // the instances plan_gemm() uses (TLF_GEMM_PLAN can only pick among these)
  TLF_TILE(64, 64, 2, 2, 2, 4)
  TLF_TILE_KG(64, 64, 2, 2, 2, 4, 2)
  TLF_TILE_KG(64, 64, 2, 2, 2, 4, 4)
  TLF_TILE(128, 64, 4, 1, 2, 3)
  TLF_TILE(128, 64, 4, 1, 4, 3)
  TLF_TILE(128, 128, 2, 2, 3, 2)
  TLF_TILE(256, 128, 2, 2, 3, 1)
  TLF_TILE(256, 128, 4, 1, 2, 2)
  TLF_TILE(128, 96, 4, 1, 3, 2)   // one M-tile of 96 ... 224 tokens, waves side by side along N
  TLF_TILE(128, 128, 4, 1, 3, 2)
  TLF_TILE(128, 160, 4, 1, 3, 2)
  TLF_TILE(128, 192, 4, 1, 3, 2)
  TLF_TILE(128, 224, 4, 1, 3, 2)
  TLF_TILE(256, 256, 8, 1, 2, 2)   // two stages: the bf16 form of the eight-wave 256 x 256 tile (128 KB of LDS)
  if constexpr (W8) {  // these fit LDS with int8 weights only
    TLF_TILE_KG(64, 96, 2, 1, 3, 2, 2)   // one M-tile, 64 channels, two sets of two waves
    TLF_TILE_KG(64, 128, 2, 1, 3, 2, 2)
    TLF_TILE_KG(64, 160, 2, 1, 3, 2, 2)
    TLF_TILE_KG(64, 64, 2, 2, 3, 4, 4)
    TLF_TILE(256, 256, 8, 1, 3, 2)   // eight waves of 32 channels x 256 tokens
    TLF_TILE(256, 128, 8, 1, 3, 2)   // eight waves of 32 channels x 128 tokens
  }
#undef TLF_TILE
#undef TLF_TILE_KG
  if (dry) {
    const int32_t fields[8] = {g.bn, g.bm, g.stages, g.occ, g.kgroups, g.splits, g.k_per_split, g.group_n};
    for (int i = 0; i < 8; ++i) plan_out[i] = fields[i];
    return launched ? TLF_OK : TLF_E_UNSUPPORTED;
  }
  if (!launched) return TLF_E_UNSUPPORTED;
  int rc = launch_status();
  if (rc != TLF_OK) return rc;
  if (act == 2)  // y is the int64 token-id vector here
    return launch_argmax_final(p.amax, p.amax_parts, static_cast<int64_t *>(y), M, stream);
  if (g.splits > 1) {
    if (tail) {  // the caller checked that this plan splits K and that the row fits the kernel
#define TLF_TAIL(TPR_, MAXC_)                                                                 \
  TLF_LAUNCH((splitk_reduce_add_rmsnorm_kernel<TPR_, MAXC_, W8>),                     \
                     dim3(static_cast<unsigned>((M + (256 / TPR_) - 1) / (256 / TPR_))), dim3(256), 0, \
                     stream, p, *tail)
      TLF_RMS_SHAPES(N, TLF_TAIL);
#undef TLF_TAIL
      return launch_status();
    }
    if (qk) {  // likewise: N = (Hq + 2 Hkv) * 128
      TLF_LAUNCH((splitk_reduce_qknorm_rope_store_kernel<W8>),
                         dim3(static_cast<unsigned>(M), static_cast<unsigned>((N / 128 + 15) / 16)), dim3(256), 0,
                         stream, p, *qk);
      return launch_status();
    }
    const int64_t total4 = static_cast<int64_t>(M) * N / 4;
    TLF_LAUNCH((splitk_reduce_kernel<W8>), dim3(static_cast<unsigned>((total4 + 255) / 256)),
                       dim3(256), 0, stream, p);
    rc = launch_status();
  }
  return rc;
}

inline size_t align256(size_t n) { return (n + 255) & ~static_cast<size_t>(255); }

// Row-major int8 [N, K] -> tile order (see the head of this file).  One thread moves one 16-byte
// atom; rows N .. round_up(N, 32) - 1 of the last group are zero filled.
__global__ __launch_bounds__(256) void pack_w8_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                      int32_t N, int32_t K, int64_t atoms) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= atoms) return;
  const int64_t chunk = i >> 6;
  const int within = static_cast<int>(i & 63);
  const int kg = within >> 5, r = within & 31;
  const int chunks_per_group = K / 32;
  const int64_t group = chunk / chunks_per_group;
  const int j = static_cast<int>(chunk % chunks_per_group);
  const int64_t n = group * 32 + r;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (n < N) v = src[(n * K + (j * 2 + kg) * 16) >> 4];
  dst[i] = v;
}

// Projection followed by add-RMSNorm.  A plan that splits K across workgroups ends in the fused
// reduce + norm kernel; every other plan writes the projection to the head of the workspace and
// runs the stand-alone add-RMSNorm on it.
template <bool W8>
int launch_gemm_add_rmsnorm(const void *x, int64_t x_stride, const void *w, const float *scale,
                            const NormTail &tail, int32_t M, int32_t N, int32_t K, void *workspace,
                            size_t workspace_bytes, hipStream_t stream) {
  int32_t plan[8];
  int rc = launch_gemm<W8>(nullptr, K, nullptr, nullptr, nullptr, M, N, K, nullptr, 0, nullptr, plan);
  if (rc != TLF_OK) return rc;
  const bool fused = plan[5] > 1;
  if (fused)
    return launch_gemm<W8>(x, x_stride, w, scale, nullptr, M, N, K, workspace, workspace_bytes, stream,
                           nullptr, 0, &tail);
  const size_t tmp_bytes = align256(static_cast<size_t>(M) * N * 2);
  if (!workspace || workspace_bytes < tmp_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return TLF_E_WORKSPACE;
  unsigned char *ws = static_cast<unsigned char *>(workspace);
  rc = launch_gemm<W8>(x, x_stride, w, scale, ws, M, N, K, ws + tmp_bytes, workspace_bytes - tmp_bytes,
                       stream);
  if (rc != TLF_OK) return rc;
  return tlf_add_rmsnorm(ws, tail.residual, tail.weight, tail.y, tail.residual_out, M, N, tail.eps,
                         stream);
}

// qkv projection followed by q/k RMSNorm + RoPE + KV-cache store, the same way: a plan that splits K ends in
// the fused reduce kernel, every other plan stages the projection at the head of the workspace.
template <bool W8>
int launch_gemm_qknorm_rope_store(const void *x, int64_t x_stride, const void *w, const float *scale,
                                  const QkRopeStoreArgs &a, int32_t M, int32_t N, int32_t K, void *workspace,
                                  size_t workspace_bytes, hipStream_t stream) {
  int32_t plan[8];
  int rc = launch_gemm<W8>(nullptr, K, nullptr, nullptr, nullptr, M, N, K, nullptr, 0, nullptr, plan);
  if (rc != TLF_OK) return rc;
  if (plan[5] > 1)
    return launch_gemm<W8>(x, x_stride, w, scale, nullptr, M, N, K, workspace, workspace_bytes, stream, nullptr, 0,
                           nullptr, &a);
  const size_t tmp_bytes = align256(static_cast<size_t>(M) * N * 2);
  if (!workspace || workspace_bytes < tmp_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return TLF_E_WORKSPACE;
  unsigned char *ws = static_cast<unsigned char *>(workspace);
  rc = launch_gemm<W8>(x, x_stride, w, scale, ws, M, N, K, ws + tmp_bytes, workspace_bytes - tmp_bytes, stream);
  if (rc != TLF_OK) return rc;
  return tlf_qknorm_rope_store(ws, N, a.qw, a.kw, a.eps, a.positions, a.cos_sin, a.max_pos, a.q_out, a.k_out,
                               a.v_out, a.k_cache, a.v_cache, a.slot_mapping, a.num_slots, a.kv_dtype, a.k_scale,
                               a.v_scale, M, a.num_q_heads, a.num_kv_heads, 128, stream);
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

extern "C" size_t tlf_w8a16_packed_bytes(int32_t N, int32_t K) {
  if (N <= 0 || K <= 0 || K % kBK) return 0;
  return static_cast<size_t>((N + 31) / 32) * 32 * static_cast<size_t>(K);
}

extern "C" int tlf_w8a16_pack_weight(const void *wq_rowmajor, void *packed, int32_t N, int32_t K,
                                     void *stream) {
  if (!wq_rowmajor || !packed) return TLF_E_NULL;
  if (N <= 0 || K <= 0 || K % kBK) return TLF_E_SHAPE;
  if (!aligned16(wq_rowmajor) || !aligned16(packed)) return TLF_E_ALIGN;
  if (wq_rowmajor == packed) return TLF_E_UNSUPPORTED;  // not in place
  const int64_t atoms = static_cast<int64_t>(tlf_w8a16_packed_bytes(N, K) / 16);
  TLF_LAUNCH(pack_w8_kernel, dim3(static_cast<unsigned>((atoms + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4 *>(wq_rowmajor),
                     static_cast<uint4 *>(packed), N, K, atoms);
  return launch_status();
}

extern "C" size_t tlf_w8a16_gemm_workspace_bytes(int32_t M, int32_t N, int32_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % kBK) return 0;
  // fp32 partial sums of the plan's split of K (the larger of the int8 and the bf16 plan: both
  // entry points share this query); a tuning override may pick any split up to 16
  int splits = 16;
  if (!gemm_tuning().has_plan) {
    int32_t p8[8], p16[8];
    if (launch_gemm<true>(nullptr, K, nullptr, nullptr, nullptr, M, N, K, nullptr, 0, nullptr, p8) == TLF_OK &&
        launch_gemm<false>(nullptr, K, nullptr, nullptr, nullptr, M, N, K, nullptr, 0, nullptr, p16) == TLF_OK)
      splits = p8[5] > p16[5] ? p8[5] : p16[5];
  }
  if (splits <= 1) return 0;
  return static_cast<size_t>(splits) * M * N * sizeof(float);
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

extern "C" int tlf_gemm_plan(int32_t M, int32_t N, int32_t K, int32_t w8, int32_t *plan8) {
  if (!plan8) return TLF_E_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || K % kBK || N % 16) return TLF_E_SHAPE;
  return w8 ? launch_gemm<true>(nullptr, K, nullptr, nullptr, nullptr, M, N, K, nullptr, 0, nullptr, plan8)
            : launch_gemm<false>(nullptr, K, nullptr, nullptr, nullptr, M, N, K, nullptr, 0, nullptr, plan8);
}

extern "C" int tlf_w8a16_gemm_silu_mul(const void *x, int64_t x_stride, const void *wq,
                                       const float *scale, void *y, int32_t M, int32_t N, int32_t K,
                                       void *stream) {
  if (M == 0) return TLF_OK;
  const int rc = check_gemm_args(x, x_stride, wq, y, M, N, K);
  if (rc != TLF_OK) return rc;
  if (!scale) return TLF_E_NULL;
  if (reinterpret_cast<uintptr_t>(scale) & 15u) return TLF_E_ALIGN;
  return launch_gemm<true>(x, x_stride, wq, scale, y, M, N, K, nullptr, 0,
                           static_cast<hipStream_t>(stream), nullptr, 1);
}

extern "C" int tlf_bf16_gemm_silu_mul(const void *x, int64_t x_stride, const void *w, void *y, int32_t M,
                                      int32_t N, int32_t K, void *stream) {
  if (M == 0) return TLF_OK;
  const int rc = check_gemm_args(x, x_stride, w, y, M, N, K);
  if (rc != TLF_OK) return rc;
  return launch_gemm<false>(x, x_stride, w, nullptr, y, M, N, K, nullptr, 0, static_cast<hipStream_t>(stream),
                            nullptr, 1);
}

extern "C" size_t tlf_gemm_add_rmsnorm_workspace_bytes(int32_t M, int32_t N, int32_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % kBK) return 0;
  return align256(static_cast<size_t>(M) * N * 2) + align256(tlf_w8a16_gemm_workspace_bytes(M, N, K));
}

static int check_norm_tail(const void *residual, const void *norm_weight, const void *y,
                           const void *residual_out, int32_t N) {
  if (!residual || !norm_weight || !y || !residual_out) return TLF_E_NULL;
  if (N > 16384) return TLF_E_SHAPE;
  if (!aligned16(residual) || !aligned16(norm_weight) || !aligned16(y) || !aligned16(residual_out))
    return TLF_E_ALIGN;
  return TLF_OK;
}

extern "C" int tlf_w8a16_gemm_add_rmsnorm(const void *x, int64_t x_stride, const void *wq,
                                          const float *scale, const void *residual,
                                          const void *norm_weight, void *y, void *residual_out,
                                          int32_t M, int32_t N, int32_t K, float eps,
                                          void *workspace, size_t workspace_bytes, void *stream) {
  if (M == 0) return TLF_OK;
  int rc = check_gemm_args(x, x_stride, wq, y, M, N, K);
  if (rc != TLF_OK) return rc;
  if (!scale) return TLF_E_NULL;
  if (reinterpret_cast<uintptr_t>(scale) & 15u) return TLF_E_ALIGN;
  rc = check_norm_tail(residual, norm_weight, y, residual_out, N);
  if (rc != TLF_OK) return rc;
  const NormTail tail{static_cast<const unsigned short *>(residual),
                      static_cast<const unsigned short *>(norm_weight),
                      static_cast<unsigned short *>(y), static_cast<unsigned short *>(residual_out), eps};
  return launch_gemm_add_rmsnorm<true>(x, x_stride, wq, scale, tail, M, N, K, workspace, workspace_bytes,
                                       static_cast<hipStream_t>(stream));
}

extern "C" int tlf_bf16_gemm_add_rmsnorm(const void *x, int64_t x_stride, const void *w,
                                         const void *residual, const void *norm_weight, void *y,
                                         void *residual_out, int32_t M, int32_t N, int32_t K, float eps,
                                         void *workspace, size_t workspace_bytes, void *stream) {
  if (M == 0) return TLF_OK;
  int rc = check_gemm_args(x, x_stride, w, y, M, N, K);
  if (rc != TLF_OK) return rc;
  rc = check_norm_tail(residual, norm_weight, y, residual_out, N);
  if (rc != TLF_OK) return rc;
  const NormTail tail{static_cast<const unsigned short *>(residual),
                      static_cast<const unsigned short *>(norm_weight),
                      static_cast<unsigned short *>(y), static_cast<unsigned short *>(residual_out), eps};
  return launch_gemm_add_rmsnorm<false>(x, x_stride, w, nullptr, tail, M, N, K, workspace, workspace_bytes,
                                        static_cast<hipStream_t>(stream));
}

// LM head + greedy sample.  Tiled plans never store the logits; for a handful of tokens (skinny
// kernel) they are staged in the workspace and tlf_argmax runs on them.
extern "C" size_t tlf_gemm_argmax_workspace_bytes(int32_t M, int32_t N, int32_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % kBK) return 0;
  const size_t keys = align256(static_cast<size_t>(M) * (N / 32 + 8) * sizeof(unsigned long long));
  const size_t staged = align256(static_cast<size_t>(M) * N * 2) + align256(tlf_argmax_workspace_bytes(M, N));
  return keys > staged ? keys : staged;
}

extern "C" int tlf_bf16_gemm_argmax(const void *x, int64_t x_stride, const void *w, int64_t *token_ids,
                                    int32_t M, int32_t N, int32_t K, void *workspace,
                                    size_t workspace_bytes, void *stream) {
  if (M == 0) return TLF_OK;
  int rc = check_gemm_args(x, x_stride, w, token_ids, M, N, K);
  if (rc != TLF_OK) return rc;
  if (!workspace || workspace_bytes < tlf_gemm_argmax_workspace_bytes(M, N, K) ||
      (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return TLF_E_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (M <= skinny_max_m()) {
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    const size_t tmp = align256(static_cast<size_t>(M) * N * 2);
    rc = launch_gemm<false>(x, x_stride, w, nullptr, ws, M, N, K, nullptr, 0, st);
    if (rc != TLF_OK) return rc;
    return tlf_argmax(ws, N, token_ids, M, N, ws + tmp, workspace_bytes - tmp, stream);
  }
  return launch_gemm<false>(x, x_stride, w, nullptr, token_ids, M, N, K, workspace, workspace_bytes, st,
                            nullptr, 2);
}

extern "C" size_t tlf_gemm_qknorm_rope_store_workspace_bytes(int32_t M, int32_t N, int32_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % kBK) return 0;
  return align256(static_cast<size_t>(M) * N * 2) + align256(tlf_w8a16_gemm_workspace_bytes(M, N, K));
}

namespace {
template <bool W8>
int gemm_qknorm_rope_store_entry(const void *x, int64_t x_stride, const void *w, const float *scale,
                                 const void *q_norm_weight, const void *k_norm_weight, float eps,
                                 const int64_t *positions, const float *cos_sin, int32_t max_pos, void *q_out,
                                 void *k_out, void *v_out, void *k_cache, void *v_cache,
                                 const int32_t *slot_mapping, int64_t num_slots, int32_t kv_dtype,
                                 const float *k_scale, const float *v_scale, int32_t n, int32_t num_q_heads,
                                 int32_t num_kv_heads, int32_t head_dim, int32_t K, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  if (n == 0) return TLF_OK;
  int rc = check_qk_rope_store_args(q_norm_weight, k_norm_weight, positions, cos_sin, max_pos, q_out, k_out, v_out,
                                    k_cache, v_cache, slot_mapping, num_slots, kv_dtype, k_scale, v_scale, n,
                                    num_q_heads, num_kv_heads, head_dim);
  if (rc != TLF_OK) return rc;
  const int64_t N64 = (static_cast<int64_t>(num_q_heads) + 2 * num_kv_heads) * head_dim;
  if (N64 > (1 << 30)) return TLF_E_SHAPE;
  const int32_t N = static_cast<int32_t>(N64);
  rc = check_gemm_args(x, x_stride, w, q_out, n, N, K);
  if (rc != TLF_OK) return rc;
  if (W8) {
    if (!scale) return TLF_E_NULL;
    if (reinterpret_cast<uintptr_t>(scale) & 15u) return TLF_E_ALIGN;
  }
  const QkRopeStoreArgs a{static_cast<const unsigned short *>(q_norm_weight),
                          static_cast<const unsigned short *>(k_norm_weight), eps, positions, cos_sin, max_pos,
                          static_cast<unsigned short *>(q_out), static_cast<unsigned short *>(k_out),
                          static_cast<unsigned short *>(v_out), static_cast<unsigned char *>(k_cache),
                          static_cast<unsigned char *>(v_cache), slot_mapping, num_slots, kv_dtype, k_scale,
                          v_scale, num_q_heads, num_kv_heads};
  return launch_gemm_qknorm_rope_store<W8>(x, x_stride, w, scale, a, n, N, K, workspace, workspace_bytes,
                                           static_cast<hipStream_t>(stream));
}
}  // namespace

extern "C" int tlf_w8a16_gemm_qknorm_rope_store(
    const void *x, int64_t x_stride, const void *wq, const float *scale, const void *q_norm_weight,
    const void *k_norm_weight, float eps, const int64_t *positions, const float *cos_sin, int32_t max_pos,
    void *q_out, void *k_out, void *v_out, void *k_cache, void *v_cache, const int32_t *slot_mapping,
    int64_t num_slots, int32_t kv_dtype, const float *k_scale, const float *v_scale, int32_t n,
    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t K, void *workspace,
    size_t workspace_bytes, void *stream) {
  return gemm_qknorm_rope_store_entry<true>(x, x_stride, wq, scale, q_norm_weight, k_norm_weight, eps, positions,
                                            cos_sin, max_pos, q_out, k_out, v_out, k_cache, v_cache, slot_mapping,
                                            num_slots, kv_dtype, k_scale, v_scale, n, num_q_heads, num_kv_heads,
                                            head_dim, K, workspace, workspace_bytes, stream);
}

extern "C" int tlf_bf16_gemm_qknorm_rope_store(
    const void *x, int64_t x_stride, const void *w, const void *q_norm_weight, const void *k_norm_weight,
    float eps, const int64_t *positions, const float *cos_sin, int32_t max_pos, void *q_out, void *k_out,
    void *v_out, void *k_cache, void *v_cache, const int32_t *slot_mapping, int64_t num_slots,
    int32_t kv_dtype, const float *k_scale, const float *v_scale, int32_t n, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t head_dim, int32_t K, void *workspace, size_t workspace_bytes,
    void *stream) {
  return gemm_qknorm_rope_store_entry<false>(x, x_stride, w, nullptr, q_norm_weight, k_norm_weight, eps, positions,
                                             cos_sin, max_pos, q_out, k_out, v_out, k_cache, v_cache, slot_mapping,
                                             num_slots, kv_dtype, k_scale, v_scale, n, num_q_heads, num_kv_heads,
                                             head_dim, K, workspace, workspace_bytes, stream);
}
