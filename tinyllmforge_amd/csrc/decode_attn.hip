// Paged decode attention for gfx950 (reference: the decode branch of
// tinyvllm/layers/attention.py:106-109, flash_attn_with_kvcache with one query
// token per sequence).
//
// HBM-bound streaming kernel.  A K (or V) cache row of one token holds all KV
// heads contiguously (Hkv * 128 bf16 = 2 KiB), so a workgroup owns a run of
// tokens and ALL KV heads: wave w <-> KV head w.  Together the waves read whole
// contiguous rows with 128-bit loads, and the Hq/Hkv query heads that share a KV
// head are served from one pass over its rows (GQA sharing): every cache byte is
// fetched exactly once.
//
// Work split (data-independent grid, so the launch can be graph-captured):
// the 16-token tiles of all sequences form one flat list; the G persistent
// workgroups take equal contiguous shares of it (computed on the device from
// context_lens by a block scan), so every workgroup streams the same number of
// bytes whatever the mix of lengths.  A share may cover the end of one sequence
// and the start of the next.  A sequence that lies inside one share is finished
// there; a sequence cut by share boundaries gets one partial (max, sum,
// unnormalised O) per share, and a small second kernel merges the partials of
// the cut sequences.  (Merging inside the first kernel needs device-scope
// fences, i.e. an L2 write-back and invalidate per workgroup on this multi-XCD
// part: measured at +80 us on a 120 us kernel, against ~5 us for the second
// launch.)
//
// Per wave and 16-token tile:
//   global (128-bit loads, issued one tile ahead) -> LDS (row-major, padded rows)
//   S^T[token, head] = K_tile . Q^T        4 x v_mfma_f32_16x16x32_bf16
//   online softmax in fp32 (row max / sum by two cross-lane exchanges)
//   O^T[dim, head]  += V_tile^T . P^T      v_mfma_f32_16x16x16_bf16; the V^T operand is
//                                          read from the row-major tile by ds_read_b64_tr_b16
// The MFMA output layout of S^T (lane = head, 4 tokens per lane) is exactly the
// B-operand layout of the second product, so P never leaves registers, and the
// softmax statistics of a head live in the lanes that hold its O^T columns.
// P is fed as a bf16 hi + lo pair (two MFMAs): matrix-core time is free in a
// bandwidth-bound kernel and it removes the bf16 rounding of the probabilities.
#include <stdlib.h>

#include "common.h"

namespace tlf {

constexpr int kDh = 128;
constexpr int kTile = 16;             // tokens per tile
// Padded LDS rows (elements).  LDS has 32 banks of 4 bytes.  K rows are read 16 bytes per lane by 8 lanes of 8
// consecutive rows at a time: a 272-byte row shifts each row by 4 banks.  V rows are read transposed, 8 bytes
// per lane, 4 lanes per row and 4 rows at a time: a 288-byte row shifts each row by 8 banks.
constexpr int kLdsRowK = kDh + 8;
constexpr int kLdsRowV = kDh + 16;
constexpr int kMaxBatch = 1024;       // sequences per call (prefix table lives in LDS)
constexpr int kMinTiles = 4;          // smallest share of a workgroup, in tiles
constexpr int kMaxGrid = 1024;        // workspace is sized for this many workgroups
constexpr float kLog2e = 1.4426950408889634f;

struct DecodeParams {
  const unsigned short *q;
  int64_t q_stride;
  const unsigned char *k_cache;
  const unsigned char *v_cache;
  const float *k_scale;
  const float *v_scale;
  const int32_t *block_tables;
  int64_t bt_stride;
  const int32_t *context_lens;
  unsigned short *out;
  int32_t *meta;      // [batch, 2]: first workgroup and number of shares of each sequence
  float *part_ml;     // [slots, Hq, 2]  (max in log2 domain, sum)
  float *part_o;      // [slots, Hq, 128]
  int32_t batch;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t block_size;
  int32_t max_blocks;
  int64_t num_cache_blocks;
  float scale_log2;  // softmax scale * log2(e)
  const int32_t *plan;  // null, or the output of plan_decode_kernel for these lengths, tables and this grid
};

// Layout of a plan (int32): header {total tiles, tiles per workgroup, grid, batch}, the prefix table, the clamped
// lengths, then one record per workgroup: {first sequence, its first tile, its end tile, its length, 0 ...} and the
// 64 block-table entries a wave holds for that sequence from the share's first block on.
constexpr int kPlanPrefix = 16;
constexpr int kPlanCtx = kPlanPrefix + kMaxBatch + 16;
constexpr int kPlanRec = kPlanCtx + kMaxBatch;
constexpr int kPlanRecInts = 8 + 64;
constexpr int kPlanInts = kPlanRec + kMaxGrid * kPlanRecInts;

__device__ __forceinline__ shortx4 lds_read_tr16_b64(const unsigned short *p) {
  // within each group of 16 lanes, lane i receives {row0[i], row1[i], row2[i], row3[i]},
  // row j being the 16 elements addressed (4 each) by lanes 4j .. 4j+3 of the group
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (shortx4 __attribute__((address_space(3))) *)(p));
}

__device__ __forceinline__ void fp8x16_to_bf16x16(const uint4 &in, uint4 &lo, uint4 &hi) {
  fp8x4_to_bf16x4(in.x, lo.x, lo.y);
  fp8x4_to_bf16x4(in.y, lo.z, lo.w);
  fp8x4_to_bf16x4(in.z, hi.x, hi.y);
  fp8x4_to_bf16x4(in.w, hi.z, hi.w);
}

// Head dimension held by LDS column c of a K or V tile.  bf16 rows are stored as they come.  e4m3 rows are
// stored with their 16-byte halves regrouped (columns 0..63: dims 16 j + 0..7, columns 64..127: dims 16 j + 8..15)
// so that the conversion's LDS writes are conflict free; the first product sums over columns (q is read with the
// same permutation) and the second product's output rows are columns (mapped back when written).  Runs of 8
// columns stay runs of 8 dims.
template <bool KV8>
__device__ __forceinline__ int lds_col_dim(int c) {
  if (!KV8) return c;
  const int j = (c >> 3) & 7;
  return j * 16 + (c >= 64 ? 8 : 0) + (c & 7);
}

// One tile's worth of global data of one wave: 16 tokens x 128 dims of K and V
// (4 + 4 128-bit loads per lane for bf16, 2 + 2 for e4m3).
template <bool KV8>
struct TileRegs {
  static constexpr int kLoads = KV8 ? 2 : 4;
  uint4 k[kLoads];
  uint4 v[kLoads];
  bool ok;  // the tile's block-table entry names a real cache block
};

// TS = 16-token tiles per loop trip.  bf16 rows: 1.  e4m3 rows: 2, so that a trip moves the same bytes per wave
// as a bf16 trip does (a wave with 4 KB in flight per trip does not cover the latency of its own loads), and
// the 32 tokens share one softmax step (one pair of cross-lane exchanges, one rescale) and feed the second
// product through v_mfma_f32_16x16x32_bf16: the K index inside an MFMA is only a summation label, so label
// g*8 + j stands for token g*4 + j%4 of tile j/4, which is where the first product left the scores.
template <int NW, bool KV8, int TS>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 4)))  // one workgroup of 8 waves per CU
void paged_decode_kernel(const DecodeParams p) {
  constexpr int kThreads = NW * 64;
  constexpr int kTrip = TS * kTile;  // tokens per loop trip
  static_assert(TS == 1 || TS == 2, "one or two tiles per trip");
  __shared__ __attribute__((aligned(16))) unsigned short lds_k[NW][kTrip][kLdsRowK];
  __shared__ __attribute__((aligned(16))) unsigned short lds_v[NW][kTrip][kLdsRowV];
  __shared__ int s_prefix[kMaxBatch + 1];  // tiles before sequence b
  __shared__ int s_ctx[kMaxBatch];         // context length of sequence b (clamped to the table)
  __shared__ int s_wave_tot[16];
  __shared__ int s_start_b;

  const int tid = threadIdx.x;
  const int w = tid >> 6;  // KV head
  const int lane = tid & 63;
  const int n = lane & 15;  // query head inside the group (MFMA column)
  const int g = lane >> 4;
  const int group = p.num_q_heads / p.num_kv_heads;
  const int head = w * group + n;
  const bool head_ok = n < group;
  const int max_ctx = p.max_blocks * p.block_size;  // a longer length would overrun the table
  // fetched first: behind the scan their latency would sit in front of the first tile's loads
  const float kscale = KV8 ? p.k_scale[w] : 1.0f;
  const float vscale = KV8 ? p.v_scale[w] : 1.0f;

  const int64_t row_elems = static_cast<int64_t>(p.num_kv_heads) * kDh;
  unsigned short(*Ks)[kLdsRowK] = lds_k[w];
  unsigned short(*Vs)[kLdsRowV] = lds_v[w];
  const float scale_log2 = p.scale_log2 * kscale;

  // A segment = the part of one sequence that lies in this workgroup's share: sequence b, whose tiles are
  // [seq_first, seq_end) of the flat list, tokens [t_begin, t_end); last = nothing of the share lies behind it.
  // (plain scalars, all wave-uniform)
#define TLF_SEG_DECL(P) int P##b, P##seq_first, P##seq_end, P##t_begin, P##t_end, P##last
#define TLF_SEG_MAKE(P, CUR, B0)                                          \
  {                                                                        \
    int b_ = (B0);                                                         \
    while (s_prefix[b_ + 1] <= (CUR)) ++b_; /* skip empty sequences */     \
    P##b = b_;                                                             \
    P##seq_first = s_prefix[b_];                                           \
    P##seq_end = s_prefix[b_ + 1];                                         \
    const int seg_end_ = min(te, P##seq_end);                              \
    P##t_begin = ((CUR) - P##seq_first) * kTile;                           \
    P##t_end = min(s_ctx[b_], (seg_end_ - P##seq_first) * kTile);          \
    P##last = seg_end_ >= te;                                              \
  }
  // What a segment needs before its first tile: q as the B operand of S^T = K . Q^T (lane (n, g) holds
  // q[head n][c*32 + g*8 .. +8]) and its block-table entries.  Lane i holds entry bt_base + i (64 blocks at a
  // time), and a tile's entry is read out of that register by lane index: a per-tile fetch would sit in the
  // in-order load queue between the tile loads, and waiting for it would drain the tile loads issued before it.
  struct SegRegs {
    bf16x8 qf[4];
    int bt_vec, bt_base;
  };
  auto fetch_q = [&](int sb, SegRegs &r) {
    const unsigned short *qp = p.q + sb * p.q_stride + static_cast<int64_t>(head) * kDh;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      Pack16 t;
      t.u = make_uint4(0, 0, 0, 0);
      if (head_ok) t.u = *reinterpret_cast<const uint4 *>(qp + lds_col_dim<KV8>(c * 32 + g * 8));
      r.qf[c] = t.v;
    }
  };
  auto fetch_seg = [&](int sb, int t_begin, SegRegs &r) {
    fetch_q(sb, r);
    r.bt_base = t_begin / p.block_size;
    r.bt_vec = (p.block_tables + sb * p.bt_stride)[min(r.bt_base + lane, p.max_blocks - 1)];
  };
  // empty sequences get zeros: workgroup i looks after sequences i, i + G, ... (one workgroup walking the whole
  // batch would finish its own share that much later, and the launch with it)
  auto zero_empty = [&]() {
    for (int b = blockIdx.x; b < p.batch; b += gridDim.x) {
      if (s_prefix[b + 1] == s_prefix[b]) {
        if (tid == 0) *reinterpret_cast<int2 *>(p.meta + 2 * b) = make_int2(0, 0);
        unsigned short *o = p.out + static_cast<int64_t>(b) * p.num_q_heads * kDh;
        for (int i = tid * 8; i < p.num_q_heads * kDh; i += kThreads * 8)
          *reinterpret_cast<uint4 *>(o + i) = make_uint4(0, 0, 0, 0);
      }
    }
  };

  // Issue the loads of the tile starting at token t0 (a tile never straddles a block); blk is its
  // block-table entry.  The address is a wave-uniform base (the tile's first row) plus a per-lane byte
  // offset that never changes: no vector-ALU address arithmetic per tile.  A tile that lies wholly inside
  // the segment (all but a segment's last) loads without predicates.
  // bf16: 4 tokens x 16 chunks of 8 elements per instruction; e4m3: 8 tokens x 8 chunks of 16
  const unsigned int lane_off = KV8 ? static_cast<unsigned int>((lane >> 3) * row_elems + w * kDh + (lane & 7) * 16)
                                    : static_cast<unsigned int>((g * row_elems + w * kDh + n * 8) * 2);
  const unsigned int load_stride = static_cast<unsigned int>(KV8 ? 8 * row_elems : 4 * row_elems * 2);
  auto load_tile = [&](int t0, int t_end, int blk, TileRegs<KV8> &r) {
    const int bi = t0 / p.block_size;
    const bool ok = blk >= 0 && blk < p.num_cache_blocks;
    const int64_t tok0 = static_cast<int64_t>(ok ? blk : 0) * p.block_size + (t0 - bi * p.block_size);
    const int64_t base = tok0 * row_elems * (KV8 ? 1 : 2);
    const unsigned char *kb = p.k_cache + base, *vb = p.v_cache + base;
    r.ok = ok;
    if (ok && t0 + kTile <= t_end) {  // uniform
#pragma unroll
      for (int i = 0; i < TileRegs<KV8>::kLoads; ++i) {
        r.k[i] = load_nt_u4(kb + (lane_off + i * load_stride));
        r.v[i] = load_nt_u4(vb + (lane_off + i * load_stride));
      }
    } else {
#pragma unroll
      for (int i = 0; i < TileRegs<KV8>::kLoads; ++i) {
        const int tt = KV8 ? i * 8 + (lane >> 3) : i * 4 + g;
        r.k[i] = make_uint4(0, 0, 0, 0);
        r.v[i] = make_uint4(0, 0, 0, 0);
        if (ok && (t0 + tt) < t_end) {
          r.k[i] = load_nt_u4(kb + (lane_off + i * load_stride));
          r.v[i] = load_nt_u4(vb + (lane_off + i * load_stride));
        }
      }
    }
  };
  // the tiles of the trip that starts at token t0 of a segment that ends at t_end, block-table entries from
  // (bt_vec, bt_base); a tile at or past t_end is not loaded
  TileRegs<KV8> regs[TS];
  auto load_trip = [&](int t0, int t_end, int bt_vec, int bt_base) {
#pragma unroll
    for (int h = 0; h < TS; ++h) {
      const int tj = t0 + h * kTile;
      if (tj < t_end) {
        const int bi = __builtin_amdgcn_readfirstlane(tj / p.block_size);
        load_tile(tj, t_end, __builtin_amdgcn_readlane(bt_vec, bi - bt_base), regs[h]);
      }
    }
  };
  auto store_tile = [&](const TileRegs<KV8> &r, int row0) {
    unsigned short(*Ks)[kLdsRowK] = lds_k[w] + row0;
    unsigned short(*Vs)[kLdsRowV] = lds_v[w] + row0;
#pragma unroll
    for (int i = 0; i < TileRegs<KV8>::kLoads; ++i) {
      if (KV8) {
        // a lane holds dims 16 c .. 16 c + 15 (c = lane % 8): the first eight go to LDS columns 8 c ..,
        // the other eight to columns 64 + 8 c .., so that 8 lanes write 128 contiguous bytes (lds_col_dim)
        const int tt = i * 8 + (lane >> 3);
        const int ch = (lane & 7) * 8;
        uint4 lo, hi;
        fp8x16_to_bf16x16(r.k[i], lo, hi);
        *reinterpret_cast<uint4 *>(&Ks[tt][ch]) = lo;
        *reinterpret_cast<uint4 *>(&Ks[tt][64 + ch]) = hi;
        fp8x16_to_bf16x16(r.v[i], lo, hi);
        *reinterpret_cast<uint4 *>(&Vs[tt][ch]) = lo;
        *reinterpret_cast<uint4 *>(&Vs[tt][64 + ch]) = hi;
      } else {
        *reinterpret_cast<uint4 *>(&Ks[i * 4 + g][n * 8]) = r.k[i];
        *reinterpret_cast<uint4 *>(&Vs[i * 4 + g][n * 8]) = r.v[i];
      }
    }
  };


  int total_tiles, tpw, ts, te;
  TLF_SEG_DECL(sg_);
  TLF_SEG_DECL(sn_);
  SegRegs cur_regs, next_regs;
  if (p.plan == nullptr) {
  // ---- 1. tiles per sequence -> exclusive prefix in LDS (block scan, chunks of kThreads)
  if (tid == 0) s_prefix[0] = 0;
  int carry = 0;
  for (int base = 0; base < p.batch; base += kThreads) {
    const int b = base + tid;
    int tiles = 0;
    if (b < p.batch) {
      const int c = min(p.context_lens[b], max_ctx);
      s_ctx[b] = c;
      tiles = c > 0 ? (c + kTile - 1) / kTile : 0;
    }
    int incl = tiles;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) s_wave_tot[w] = incl;
    __syncthreads();
    int before = carry;
    for (int ww = 0; ww < w; ++ww) before += s_wave_tot[ww];
    if (b < p.batch) s_prefix[b + 1] = before + incl;
    int total = 0;
    for (int ww = 0; ww < NW; ++ww) total += s_wave_tot[ww];
    carry += total;
    __syncthreads();
  }
  total_tiles = carry;

  // ---- 2. empty sequences get zeros
  zero_empty();

  // ---- 3. this workgroup's share [ts, te) of the flat tile list
  const int G = gridDim.x;
  tpw = (total_tiles + G - 1) / G;
  if (tpw < kMinTiles) tpw = kMinTiles;
  ts = blockIdx.x * tpw;
  te = min(total_tiles, ts + tpw);
  if (ts >= total_tiles) return;  // uniform
  for (int b = tid; b < p.batch; b += kThreads)
    if (s_prefix[b] <= ts && ts < s_prefix[b + 1]) s_start_b = b;
  __syncthreads();

  // One trip is in flight per wave (deeper register prefetch was measured and is no faster: the stream is not
  // bound by this wave's latency once every CU has 64 KB in flight).  What is pipelined is the change of
  // segment: q and the block-table entries of the next segment are fetched while the current one runs, and the
  // first trip of the next segment is loaded during the last trip of the current one, so a workgroup whose
  // share covers several sequences does not stop streaming between them.
  TLF_SEG_MAKE(sg_, ts, s_start_b)
  fetch_seg(sg_b, sg_t_begin, next_regs);
  load_trip(sg_t_begin, sg_t_end, next_regs.bt_vec, next_regs.bt_base);
  } else {
    // ---- the same three steps from a plan made once per decode step (plan_decode_kernel) instead of once per
    // layer: the prefix table and the lengths are copied, and the record of this workgroup names its first sequence
    // and holds that sequence's block-table entries, so the first rows are requested one memory round trip after
    // the kernel starts instead of three (lengths -> scan and search -> block table -> rows).
    const int32_t *pl = p.plan;
    const int4 hdr = *reinterpret_cast<const int4 *>(pl);   // total tiles, tiles per workgroup, grid, batch
    const int32_t *recp = pl + kPlanRec + static_cast<int64_t>(blockIdx.x) * kPlanRecInts;
    const int4 rec = *reinterpret_cast<const int4 *>(recp);  // first sequence of the share, its tiles [first, end), its length
    const int bt_first = recp[8 + lane];
    constexpr int kCopies = kMaxBatch / kThreads + 1;
    int cp[kCopies], cc[kCopies];
#pragma unroll
    for (int i = 0; i < kCopies; ++i) {
      const int b = min(tid + i * kThreads, p.batch);
      cp[i] = pl[kPlanPrefix + b];
      cc[i] = pl[kPlanCtx + min(b, p.batch - 1)];
    }
    if (hdr.z != static_cast<int>(gridDim.x) || hdr.w != p.batch || hdr.y < kMinTiles) {
      // a plan made for another grid or batch: nothing of it can be trusted; every output row becomes NaN
      for (int b = blockIdx.x; b < p.batch; b += gridDim.x) {
        unsigned short *o = p.out + static_cast<int64_t>(b) * p.num_q_heads * kDh;
        for (int i = tid * 8; i < p.num_q_heads * kDh; i += kThreads * 8)
          *reinterpret_cast<uint4 *>(o + i) = make_uint4(0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u);
        if (tid == 0) *reinterpret_cast<int2 *>(p.meta + 2 * b) = make_int2(0, 0);
      }
      return;
    }
    total_tiles = __builtin_amdgcn_readfirstlane(hdr.x);
    tpw = __builtin_amdgcn_readfirstlane(hdr.y);
    ts = blockIdx.x * tpw;
    te = min(total_tiles, ts + tpw);
    const bool has_work = ts < total_tiles;
    if (has_work) {
      sg_b = __builtin_amdgcn_readfirstlane(rec.x);
      sg_seq_first = __builtin_amdgcn_readfirstlane(rec.y);
      sg_seq_end = __builtin_amdgcn_readfirstlane(rec.z);
      const int seg_end_ = min(te, sg_seq_end);
      sg_t_begin = (ts - sg_seq_first) * kTile;
      sg_t_end = min(__builtin_amdgcn_readfirstlane(rec.w), (seg_end_ - sg_seq_first) * kTile);
      sg_last = seg_end_ >= te;
      fetch_q(sg_b, next_regs);
      next_regs.bt_base = sg_t_begin / p.block_size;
      next_regs.bt_vec = bt_first;
      load_trip(sg_t_begin, sg_t_end, next_regs.bt_vec, next_regs.bt_base);
    }
#pragma unroll
    for (int i = 0; i < kCopies; ++i) {
      const int b = tid + i * kThreads;
      if (b <= p.batch) s_prefix[b] = cp[i];
      if (b < p.batch) s_ctx[b] = cc[i];
    }
    __syncthreads();
    zero_empty();
    if (!has_work) return;  // uniform
  }
  while (true) {
    cur_regs = next_regs;
    sn_b = sg_b; sn_seq_first = sg_seq_first; sn_seq_end = sg_seq_end; sn_t_begin = 0; sn_t_end = 0; sn_last = 1;
    if (!sg_last) {
      TLF_SEG_MAKE(sn_, sg_seq_end, sg_b + 1)
      fetch_seg(sn_b, sn_t_begin, next_regs);
    }
    const bf16x8(&qf)[4] = cur_regs.qf;

    floatx4 acc[8];
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[d] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;  // running max (log2 domain), identical in the 4 lanes of a head
    float l_run = 0.f;        // this lane's share of the running sum

    for (int t0 = sg_t_begin; t0 < sg_t_end; t0 += kTrip) {
      wave_lds_fence();  // previous trip's LDS reads are done
      bool tile_ok[TS];
#pragma unroll
      for (int h = 0; h < TS; ++h) {
        // a tile past the end of the segment (second tile of the last trip) was never loaded: zeros, masked below
        if (t0 + h * kTile >= sg_t_end) {
#pragma unroll
          for (int i = 0; i < TileRegs<KV8>::kLoads; ++i) {
            regs[h].k[i] = make_uint4(0, 0, 0, 0);
            regs[h].v[i] = make_uint4(0, 0, 0, 0);
          }
          regs[h].ok = false;
        }
        store_tile(regs[h], h * kTile);
        tile_ok[h] = regs[h].ok;
      }
      wave_lds_fence();
      {
        // next trip: of this segment, or the first of the next one (t_end 0 when there is none: nothing loads)
        const bool more = t0 + kTrip < sg_t_end;
        if (more) {  // 64 block-table entries per register: move the window on (uniform, rare)
          const int bi = __builtin_amdgcn_readfirstlane((t0 + kTrip + (TS - 1) * kTile) / p.block_size);
          if (bi - cur_regs.bt_base >= 64) {
            cur_regs.bt_base = (t0 + kTrip) / p.block_size;
            cur_regs.bt_vec =
                (p.block_tables + sg_b * p.bt_stride)[min(cur_regs.bt_base + lane, p.max_blocks - 1)];
          }
        }
        load_trip(more ? t0 + kTrip : sn_t_begin, more ? sg_t_end : sn_t_end,
                  more ? cur_regs.bt_vec : next_regs.bt_vec, more ? cur_regs.bt_base : next_regs.bt_base);
      }

      // S^T = K . Q^T : lane (n, g) gets tokens g*4 + i of head n, for each tile of the trip
      floatx4 s[TS];
#pragma unroll
      for (int h = 0; h < TS; ++h) s[h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int h = 0; h < TS; ++h) {
          Pack16 a;
          a.u = *reinterpret_cast<const uint4 *>(&Ks[h * kTile + n][c * 32 + g * 8]);
          s[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[c], s[h], 0, 0, 0);
        }
      float sv[TS][4];
      float mt = -INFINITY;
#pragma unroll
      for (int h = 0; h < TS; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const bool valid = tile_ok[h] && (t0 + h * kTile + g * 4 + i) < sg_t_end;
          sv[h][i] = valid ? s[h][i] * scale_log2 : -INFINITY;
          mt = fmaxf(mt, sv[h][i]);
        }
      mt = max_lanes_16_32_48(mt);
      const float m_new = fmaxf(m_run, mt);
      // -inf only while every token so far sat in a skipped block: keep the exponents finite
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      // raw v_exp_f32: results below 2^-126 (which the library routine would denormalise) weigh nothing here
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
      float pv[TS][4];
      float psum = 0.f;
#pragma unroll
      for (int h = 0; h < TS; ++h) {
#pragma unroll
        for (int i = 0; i < 4; ++i) pv[h][i] = __builtin_amdgcn_exp2f(sv[h][i] - m_use);
        psum += (pv[h][0] + pv[h][1]) + (pv[h][2] + pv[h][3]);
      }
      l_run = l_run * alpha + psum;
      m_run = m_new;
      // P as a bf16 hi + lo pair, converted two at a time
      unsigned int hi[TS][2], lo[TS][2];
#pragma unroll
      for (int h = 0; h < TS; ++h)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          hi[h][e] = pack_bf16x2(pv[h][2 * e], pv[h][2 * e + 1]);
          lo[h][e] = pack_bf16x2(pv[h][2 * e] - __uint_as_float(hi[h][e] << 16),
                                 pv[h][2 * e + 1] - __uint_as_float(hi[h][e] & 0xffff0000u));
        }
      // the running max rarely moves after the first tiles: skip the 32 multiplies then.  The branch is
      // wave-uniform and must stay a branch (the empty asm keeps the compiler from turning it into 32
      // multiplies and 32 selects on every trip).
      if (__any(alpha != 1.0f)) {
        asm volatile("" ::);
#pragma unroll
        for (int d = 0; d < 8; ++d)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[d][i] *= alpha;
      }
      if constexpr (TS == 1) {
        const shortx4 pbs = __builtin_bit_cast(shortx4, make_uint2(hi[0][0], hi[0][1]));
        const shortx4 pls = __builtin_bit_cast(shortx4, make_uint2(lo[0][0], lo[0][1]));
#pragma unroll
        for (int d = 0; d < 8; ++d) {
          // A = V^T fragment: lane (dim = d*16 + n, g) <- tokens g*4 + 0..3 (transpose read)
          const shortx4 vf = lds_read_tr16_b64(&Vs[g * 4 + (n >> 2)][d * 16 + (n & 3) * 4]);
          acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pbs, acc[d], 0, 0, 0);
          acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pls, acc[d], 0, 0, 0);
        }
      } else {
        Pack16 ph, pl;
        ph.u = make_uint4(hi[0][0], hi[0][1], hi[1][0], hi[1][1]);
        pl.u = make_uint4(lo[0][0], lo[0][1], lo[1][0], lo[1][1]);
#pragma unroll
        for (int d = 0; d < 8; ++d) {
          // A = V^T fragment of both tiles: summation labels g*8 + 0..3 <- tokens g*4 + 0..3 of tile 0,
          // labels g*8 + 4..7 <- the same tokens of tile 1
          const shortx4 v0 = lds_read_tr16_b64(&Vs[g * 4 + (n >> 2)][d * 16 + (n & 3) * 4]);
          const shortx4 v1 = lds_read_tr16_b64(&Vs[kTile + g * 4 + (n >> 2)][d * 16 + (n & 3) * 4]);
          Pack16 vf;
          vf.u = make_uint4(__builtin_bit_cast(uint2, v0).x, __builtin_bit_cast(uint2, v0).y,
                            __builtin_bit_cast(uint2, v1).x, __builtin_bit_cast(uint2, v1).y);
          acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, ph.v, acc[d], 0, 0, 0);
          acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pl.v, acc[d], 0, 0, 0);
        }
      }
    }
    l_run = sum_lanes_16_32_48(l_run);

    // ---- finish the segment.  lane (n, g) holds O^T[dims d*16 + g*4 + i][head n]
    const int w_first = sg_seq_first / tpw;
    const int w_last = (sg_seq_end - 1) / tpw;
    const int nseg = w_last - w_first + 1;
    if (nseg == 1) {
      if (head_ok) {
        const float inv = l_run > 0.f ? vscale / l_run : 0.f;
        unsigned short *o = p.out + (static_cast<int64_t>(sg_b) * p.num_q_heads + head) * kDh;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
          uint2 st;
          st.x = pack_bf16x2(acc[d][0] * inv, acc[d][1] * inv);
          st.y = pack_bf16x2(acc[d][2] * inv, acc[d][3] * inv);
          *reinterpret_cast<uint2 *>(o + lds_col_dim<KV8>(d * 16 + g * 4)) = st;
        }
      }
    } else {
      // (workgroup, sequence) pairs form a staircase, so blockIdx + b is a unique slot
      const int64_t slot = (static_cast<int64_t>(blockIdx.x) + sg_b) * p.num_q_heads;
      if (head_ok) {
        float *po = p.part_o + (slot + head) * kDh;
#pragma unroll
        for (int d = 0; d < 8; ++d)
          *reinterpret_cast<float4 *>(po + lds_col_dim<KV8>(d * 16 + g * 4)) =
              make_float4(acc[d][0] * vscale, acc[d][1] * vscale, acc[d][2] * vscale,
                          acc[d][3] * vscale);
        if (g == 0) *reinterpret_cast<float2 *>(p.part_ml + (slot + head) * 2) = make_float2(m_run, l_run);
      }
    }
    if (tid == 0 && sg_t_begin == 0)  // the share holding the sequence's first tile records its split
      *reinterpret_cast<int2 *>(p.meta + 2 * sg_b) = make_int2(w_first, nseg);
    if (sg_last) break;
    sg_b = sn_b; sg_seq_first = sn_seq_first; sg_seq_end = sn_seq_end; sg_t_begin = sn_t_begin; sg_t_end = sn_t_end;
    sg_last = sn_last;
  }
#undef TLF_SEG_DECL
#undef TLF_SEG_MAKE
}

// Merge the partials of the sequences that were cut by share boundaries.
// grid = (Hq / 8, batch); a thread owns 4 dims of one head and walks the shares
// four at a time, so that 8 independent loads are in flight per step (the loop is
// latency bound: partials were just written by other CUs).
__global__ __launch_bounds__(256) void paged_decode_merge_kernel(const DecodeParams p) {
  const int b = blockIdx.y;
  const int2 meta = *reinterpret_cast<const int2 *>(p.meta + 2 * b);
  const int w_first = meta.x, nseg = meta.y;
  if (nseg <= 1) return;  // finished by the first kernel (or empty)
  const int hh = blockIdx.x * 8 + (threadIdx.x >> 5);
  if (hh >= p.num_q_heads) return;
  const int c4 = (threadIdx.x & 31) * 4;
  const int64_t base = (static_cast<int64_t>(w_first) + b) * p.num_q_heads + hh;
  float M = -INFINITY, L = 0.f;
  float4 A = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = 0; s0 < nseg; s0 += 4) {
    float2 ml[4];
    float4 o4[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = min(s0 + u, nseg - 1);  // clamped duplicate gets weight 0 below
      const int64_t sl = base + static_cast<int64_t>(s) * p.num_q_heads;
      ml[u] = *reinterpret_cast<const float2 *>(p.part_ml + sl * 2);
      o4[u] = *reinterpret_cast<const float4 *>(p.part_o + sl * kDh + c4);
    }
    float Mn = M;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (s0 + u < nseg) Mn = fmaxf(Mn, ml[u].x);
    if (Mn == -INFINITY) continue;
    const float a = exp2f(M - Mn);
    L *= a;
    A.x *= a; A.y *= a; A.z *= a; A.w *= a;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float wgt = (s0 + u < nseg && ml[u].x != -INFINITY) ? exp2f(ml[u].x - Mn) : 0.f;
      L += wgt * ml[u].y;
      A.x += wgt * o4[u].x;
      A.y += wgt * o4[u].y;
      A.z += wgt * o4[u].z;
      A.w += wgt * o4[u].w;
    }
    M = Mn;
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  uint2 st;
  st.x = pack_bf16x2(A.x * inv, A.y * inv);
  st.y = pack_bf16x2(A.z * inv, A.w * inv);
  *reinterpret_cast<uint2 *>(p.out + (static_cast<int64_t>(b) * p.num_q_heads + hh) * kDh + c4) = st;
}

// The work split of paged_decode_kernel, made once per decode step for all layers (their lengths and block tables
// are the same).  Every workgroup scans the lengths as step 1 of that kernel does (1024 threads, one chunk), then
// writes the records of 16 of the G attention workgroups: 16 threads find their first sequences, all 1024 copy the
// 64 block-table entries of each; workgroup 0 also writes the header, the prefix table and the lengths.
constexpr int kPlanRecsPerWg = 16;
__global__ __launch_bounds__(1024) void plan_decode_kernel(const int32_t *__restrict__ context_lens,
                                                           const int32_t *__restrict__ block_tables, int64_t bt_stride,
                                                           int32_t batch, int32_t block_size, int32_t max_blocks, int32_t G,
                                                           int32_t *__restrict__ plan) {
  __shared__ int s_prefix[kMaxBatch + 1];
  __shared__ int s_ctx[kMaxBatch];
  __shared__ int s_wave_tot[16];
  __shared__ int s_rec_b[kPlanRecsPerWg];
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
  const int max_ctx = max_blocks * block_size;
  int tiles = 0;
  if (tid < batch) {
    const int c = min(context_lens[tid], max_ctx);
    s_ctx[tid] = c;
    tiles = c > 0 ? (c + kTile - 1) / kTile : 0;
  }
  int incl = tiles;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) s_wave_tot[w] = incl;
  if (tid == 0) s_prefix[0] = 0;
  __syncthreads();
  int before = 0, total = 0;
  for (int ww = 0; ww < 16; ++ww) {
    if (ww < w) before += s_wave_tot[ww];
    total += s_wave_tot[ww];
  }
  if (tid < batch) s_prefix[tid + 1] = before + incl;
  __syncthreads();
  int tpw = (total + G - 1) / G;
  if (tpw < kMinTiles) tpw = kMinTiles;
  if (blockIdx.x == 0) {
    if (tid == 0) *reinterpret_cast<int4 *>(plan) = make_int4(total, tpw, G, batch);
    for (int b = tid; b <= batch; b += 1024) plan[kPlanPrefix + b] = s_prefix[b];
    if (tid < batch) plan[kPlanCtx + tid] = s_ctx[tid];
  }
  const int i0 = blockIdx.x * kPlanRecsPerWg;
  if (tid < kPlanRecsPerWg && i0 + tid < G) {
    const int i = i0 + tid;
    const int ts = i * tpw;
    int b = -1;
    if (ts < total) {  // the sequence whose tiles [prefix[b], prefix[b + 1]) hold tile ts (never an empty one)
      int lo = 0, hi = batch - 1;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (s_prefix[mid + 1] > ts) hi = mid; else lo = mid + 1;
      }
      b = lo;
    }
    s_rec_b[tid] = b;
    int32_t *rec = plan + kPlanRec + static_cast<int64_t>(i) * kPlanRecInts;
    *reinterpret_cast<int4 *>(rec) = b >= 0 ? make_int4(b, s_prefix[b], s_prefix[b + 1], s_ctx[b]) : make_int4(-1, 0, 0, 0);
    *reinterpret_cast<int4 *>(rec + 4) = make_int4(0, 0, 0, 0);
  }
  __syncthreads();
  const int i = i0 + w;   // wave w copies the entries of record i0 + w
  if (i < G) {
    const int b = s_rec_b[w];
    int v = -1;
    if (b >= 0) {
      const int bt_base = (i * tpw - s_prefix[b]) * kTile / block_size;
      v = block_tables[b * bt_stride + min(bt_base + lane, max_blocks - 1)];
    }
    plan[kPlanRec + static_cast<int64_t>(i) * kPlanRecInts + 8 + lane] = v;
  }
}

inline int device_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

// Workgroups per CU of the persistent grid.  Measured on MI355X (config: B=64, ctx 512..4096):
// 1 -> 109 us, 2 -> 116 us, 3 -> 119 us, 4 -> 125 us per call: fewer, longer shares mean fewer
// partials and less contention.  TLF_DECODE_WGS_PER_CU overrides the grid size for tuning (one workgroup
// is resident per CU: LDS, and a register budget of 256 per lane).
inline int decode_wgs_per_cu() {
  static int v = 0;
  if (v == 0) {
    v = 1;
    if (const char *e = getenv("TLF_DECODE_WGS_PER_CU")) {
      const int x = atoi(e);
      if (x >= 1 && x <= 4) v = x;
    }
  }
  return v;
}

inline size_t decode_meta_bytes() { return 2 * kMaxBatch * sizeof(int32_t); }

}  // namespace tlf

using namespace tlf;

extern "C" size_t tlf_paged_decode_attn_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                        int32_t head_dim, int32_t max_blocks,
                                                        int32_t block_size) {
  (void)max_blocks;
  (void)block_size;
  if (batch <= 0 || num_q_heads <= 0 || head_dim <= 0) return 0;
  const size_t slots = static_cast<size_t>(kMaxGrid) + batch;
  return decode_meta_bytes() +
         slots * num_q_heads * (static_cast<size_t>(head_dim) + 2) * sizeof(float);
}

namespace tlf {
// persistent grid: one workgroup per CU (decode_wgs_per_cu), fewer when the largest possible job is small
inline int decode_grid(int32_t batch, int32_t max_blocks, int32_t block_size) {
  const int64_t max_tiles = static_cast<int64_t>(batch) * ((static_cast<int64_t>(max_blocks) * block_size + kTile - 1) / kTile);
  int64_t grid = static_cast<int64_t>(decode_wgs_per_cu()) * device_cu_count();
  if (grid > kMaxGrid) grid = kMaxGrid;
  const int64_t by_work = (max_tiles + kMinTiles - 1) / kMinTiles;
  if (grid > by_work) grid = by_work;
  if (grid < 1) grid = 1;
  return static_cast<int>(grid);
}
}  // namespace tlf

extern "C" size_t tlf_paged_decode_plan_bytes(void) { return static_cast<size_t>(kPlanInts) * sizeof(int32_t); }

extern "C" int tlf_paged_decode_plan(const int32_t *context_lens, const int32_t *block_tables,
                                     int64_t block_table_stride, int32_t batch, int32_t block_size,
                                     int32_t max_blocks, void *plan, size_t plan_bytes, void *stream) {
  if (batch == 0) return TLF_OK;
  if (!context_lens || !block_tables || !plan) return TLF_E_NULL;
  if (batch < 0 || batch > kMaxBatch || block_size <= 0 || max_blocks <= 0 || block_size % kTile) return TLF_E_SHAPE;
  if (static_cast<int64_t>(max_blocks) * block_size > (1ll << 30) || block_table_stride < max_blocks) return TLF_E_SHAPE;
  if (plan_bytes < tlf_paged_decode_plan_bytes() || !aligned16(plan)) return TLF_E_WORKSPACE;
  const int grid = decode_grid(batch, max_blocks, block_size);
  TLF_LAUNCH(plan_decode_kernel, dim3((grid + kPlanRecsPerWg - 1) / kPlanRecsPerWg), dim3(1024), 0,
             static_cast<hipStream_t>(stream), context_lens, block_tables, block_table_stride, batch, block_size,
             max_blocks, grid, static_cast<int32_t *>(plan));
  return launch_status();
}

static int decode_attn_impl(const void *q, int64_t q_stride, const void *k_cache,
                                     const void *v_cache, int32_t kv_dtype, const float *k_scale,
                                     const float *v_scale, const int32_t *block_tables,
                                     int64_t block_table_stride, const int32_t *context_lens,
                                     void *out, int32_t batch, int32_t num_q_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                     int32_t max_blocks, int64_t num_cache_blocks, float scale,
                                     void *workspace, size_t workspace_bytes, const int32_t *plan, void *stream) {
  if (batch == 0) return TLF_OK;
  if (!q || !k_cache || !v_cache || !block_tables || !context_lens || !out) return TLF_E_NULL;
  if (head_dim != kDh) return TLF_E_UNSUPPORTED;
  if (kv_dtype != TLF_KV_BF16 && kv_dtype != TLF_KV_FP8_E4M3) return TLF_E_UNSUPPORTED;
  if (kv_dtype == TLF_KV_FP8_E4M3 && (!k_scale || !v_scale)) return TLF_E_NULL;
  if (batch < 0 || batch > kMaxBatch || num_q_heads <= 0 || num_kv_heads <= 0 || block_size <= 0 ||
      max_blocks <= 0 || num_cache_blocks <= 0)
    return TLF_E_SHAPE;
  if (num_q_heads % num_kv_heads || num_q_heads / num_kv_heads > 16 || block_size % kTile)
    return TLF_E_SHAPE;
  if (static_cast<int64_t>(max_blocks) * block_size > (1ll << 30)) return TLF_E_SHAPE;
  if (block_table_stride < max_blocks || q_stride < static_cast<int64_t>(num_q_heads) * head_dim)
    return TLF_E_SHAPE;
  if (!aligned16(q) || q_stride % 8 || !aligned16(k_cache) || !aligned16(v_cache) ||
      !aligned16(out))
    return TLF_E_ALIGN;
  const size_t need =
      tlf_paged_decode_attn_workspace_bytes(batch, num_q_heads, head_dim, max_blocks, block_size);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return TLF_E_WORKSPACE;

  DecodeParams p;
  p.q = static_cast<const unsigned short *>(q);
  p.q_stride = q_stride;
  p.k_cache = static_cast<const unsigned char *>(k_cache);
  p.v_cache = static_cast<const unsigned char *>(v_cache);
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.block_tables = block_tables;
  p.bt_stride = block_table_stride;
  p.context_lens = context_lens;
  p.out = static_cast<unsigned short *>(out);
  p.batch = batch;
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.block_size = block_size;
  p.max_blocks = max_blocks;
  p.num_cache_blocks = num_cache_blocks;
  p.scale_log2 = scale * kLog2e;
  unsigned char *ws = static_cast<unsigned char *>(workspace);
  const size_t slots = static_cast<size_t>(kMaxGrid) + batch;
  p.meta = reinterpret_cast<int32_t *>(ws);
  p.part_ml = reinterpret_cast<float *>(ws + decode_meta_bytes());
  p.part_o = p.part_ml + slots * num_q_heads * 2;

  p.plan = plan;
  const int grid = decode_grid(batch, max_blocks, block_size);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 g(static_cast<unsigned>(grid));
  const bool f8 = kv_dtype == TLF_KV_FP8_E4M3;
  // e4m3 rows: two tiles per trip where the bf16 image of both fits LDS (up to 8 KV heads)
#define TLF_DECODE(NW)                                                                              \
  if (f8)                                                                                           \
    TLF_LAUNCH((paged_decode_kernel<NW, true, (NW <= 8 ? 2 : 1)>), g, dim3(NW * 64), 0, s, p); \
  else                                                                                              \
    TLF_LAUNCH((paged_decode_kernel<NW, false, 1>), g, dim3(NW * 64), 0, s, p)
  switch (num_kv_heads) {
    case 1: TLF_DECODE(1); break;
    case 2: TLF_DECODE(2); break;
    case 4: TLF_DECODE(4); break;
    case 8: TLF_DECODE(8); break;
    case 16: TLF_DECODE(16); break;
    default: return TLF_E_UNSUPPORTED;
  }
#undef TLF_DECODE
  int rc = launch_status();
  if (rc != TLF_OK) return rc;
  TLF_LAUNCH(paged_decode_merge_kernel, dim3((num_q_heads + 7) / 8, batch), dim3(256), 0, s, p);
  return launch_status();
}

extern "C" int tlf_paged_decode_attn(const void *q, int64_t q_stride, const void *k_cache,
                                     const void *v_cache, int32_t kv_dtype, const float *k_scale,
                                     const float *v_scale, const int32_t *block_tables,
                                     int64_t block_table_stride, const int32_t *context_lens,
                                     void *out, int32_t batch, int32_t num_q_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                     int32_t max_blocks, int64_t num_cache_blocks, float scale,
                                     void *workspace, size_t workspace_bytes, void *stream) {
  return decode_attn_impl(q, q_stride, k_cache, v_cache, kv_dtype, k_scale, v_scale, block_tables, block_table_stride,
                          context_lens, out, batch, num_q_heads, num_kv_heads, head_dim, block_size, max_blocks,
                          num_cache_blocks, scale, workspace, workspace_bytes, nullptr, stream);
}

extern "C" int tlf_paged_decode_attn_planned(const void *q, int64_t q_stride, const void *k_cache,
                                             const void *v_cache, int32_t kv_dtype, const float *k_scale,
                                             const float *v_scale, const int32_t *block_tables,
                                             int64_t block_table_stride, const int32_t *context_lens,
                                             void *out, int32_t batch, int32_t num_q_heads,
                                             int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                             int32_t max_blocks, int64_t num_cache_blocks, float scale,
                                             void *workspace, size_t workspace_bytes, const void *plan, void *stream) {
  if (batch != 0 && (!plan || !aligned16(plan))) return plan ? TLF_E_ALIGN : TLF_E_NULL;
  return decode_attn_impl(q, q_stride, k_cache, v_cache, kv_dtype, k_scale, v_scale, block_tables, block_table_stride,
                          context_lens, out, batch, num_q_heads, num_kv_heads, head_dim, block_size, max_blocks,
                          num_cache_blocks, scale, workspace, workspace_bytes, static_cast<const int32_t *>(plan), stream);
}
