// Paged decode attention for gfx950: one query token per sequence against the block-table-addressed
// KV cache (layout [num_blocks, block_size, hkv, 128] bf16).  HBM-bandwidth bound: every K/V byte of
// the live context is read exactly once, 16 bytes per lane, 256 contiguous bytes per token and head.
//
// Work is split "flat": the 32-token stages of all sequences are laid end to end and cut into ncols
// equal runs, one per column of workgroups, so every column streams the same number of bytes no
// matter how ragged the context lengths are.  A run may start in the middle of a sequence and may
// cover several short ones; each (column, sequence) intersection is a piece.
//
// Three launches per call, all on the caller's stream (the host never sees the lengths):
//   1. paged_decode_plan_kernel (one workgroup): prefix sum of stage counts, run length, and for each
//      column the sequence and stage it starts at.
//   2. paged_decode_kernel: ncols x (hkv/HPW) workgroups of HPW waves; a workgroup takes HPW kv heads
//      of its column's run (one head per wave), so it streams HPW*256 contiguous bytes per token.
//      The first stage of the next piece (and its query rows) is already in flight while the last
//      stage of the current piece is consumed: a wave never drains its load queue inside its run.
//      A piece that covers a whole sequence is normalised and written to `out`; a piece that shares
//      its sequence with other columns leaves (max, sum, unnormalised O) in one of the column's two
//      partial slots (slot 0: the sequence began in an earlier column, slot 1: it began here).
//   3. paged_decode_combine_kernel: merges the partials of sequences spread over several columns and
//      writes zero rows for empty sequences.
//
// Inside a wave (one kv head, all hq/hkv query heads of its group served from one read of K and V)
//   stage = 32 consecutive tokens (inside one cache block): 8 KiB of K + 8 KiB of V.  Stage i+1 is in
//           flight from HBM into registers while stage i is consumed out of the wave's private LDS tile.
//   S^T[token, qhead] = K[token, :] . Q^T            8 x v_mfma_f32_16x16x32_bf16 (K tile as A operand,
//                                                     read back from LDS with a 16-byte XOR swizzle)
//   online softmax over tokens (base-2 exponent, fp32 running max / sum per query head)
//   O^T[d, qhead]    += V^T[d, token] . P^T           8 x v_mfma_f32_16x16x32_bf16; V^T comes out of
//                                                     LDS through ds_read_b64_tr_b16 (transposing read)
//   The accumulator layout of S^T is exactly the B-operand layout the second product needs, so P never
//   moves between lanes.
#include "mops_common.h"
#include <stdlib.h>
#include <mutex>

namespace mops {

constexpr int kHeadDim = 128;
constexpr int kStageTokens = 32;
constexpr int kRowBytes = kHeadDim * 2;                  // one token, one kv head
constexpr int kTileBytes = kStageTokens * kRowBytes;     // 8 KiB
constexpr int kPlanThreads = 256;
constexpr int kPlanLdsSeqs = 4096;                       // prefix array kept in LDS up to this batch
constexpr int kHdrInts = 64;                             // workspace header, see PlanHeader
// Header words.  [2..8] are the signature of the launch the plan was made for: a kernel that is handed
// a workspace whose plan does not fit its own parameters (never planned, or planned for another batch or
// head geometry) must not follow it, because the sequence indices in it would be out of range.
enum PlanHeader { kHdrTotal = 0, kHdrPerCol = 1, kHdrMagic = 2, kHdrBatch = 3, kHdrCols = 4, kHdrHq = 5, kHdrHkv = 6,
                  kHdrBlockSize = 7, kHdrMaxBlocks = 8 };
constexpr int kPlanMagic = 0x6d6f7073;

// Byte offset of 16-byte piece `slice` of token row `t` inside a swizzled LDS tile.
__device__ __forceinline__ int tile_offset(int t, int slice) {
  return t * kRowBytes + ((slice ^ (t & 15)) << 4);
}

struct DecodeParams {
  const uint16_t* q;
  int64_t q_batch_stride;
  const uint16_t* k_cache;
  const uint16_t* v_cache;
  const int32_t* cache_seqlens;
  const int32_t* block_table;
  int64_t block_table_row_stride;
  uint16_t* out;
  int32_t* hdr;        // [kHdrInts]
  int32_t* prefix;     // [batch + 1] exclusive prefix sum of per-sequence stage counts
  int32_t* col_start;  // [ncols][2]  first sequence of the column's run, stage offset inside it
  float* ws_acc;       // [ncols][2][hq][128]
  float* ws_ml;        // [ncols][2][hq][2]   (running max in the base-2 scaled domain, sum)
  int batch, hq, hkv, group;       // group = hq / hkv  (<= 16)
  int block_size, num_blocks, max_blocks_per_seq;
  int ncols;
  int min_per_col;      // shortest run of stages a column is given
  float scale_log2;                // softmax_scale * log2(e)
};

__device__ __forceinline__ int clamp_seqlen(int s, const DecodeParams& p) {
  const int cap = p.max_blocks_per_seq * p.block_size;
  return s < 0 ? 0 : (s > cap ? cap : s);
}
__device__ __forceinline__ int stages_of(int seqlen) { return (seqlen + kStageTokens - 1) / kStageTokens; }

// True when the plan in the workspace was made for a launch with these parameters.
__device__ __forceinline__ bool plan_fits(const DecodeParams& p) {
  const int32_t* h = p.hdr;
  return h[kHdrMagic] == kPlanMagic && h[kHdrBatch] == p.batch && h[kHdrCols] == p.ncols && h[kHdrHq] == p.hq &&
         h[kHdrHkv] == p.hkv && h[kHdrBlockSize] == p.block_size && h[kHdrMaxBlocks] == p.max_blocks_per_seq &&
         h[kHdrPerCol] > 0 && h[kHdrTotal] >= 0;
}

// Scalar (constant-cache) load of a wave-uniform int that no kernel in flight writes.  Used inside
// the main loop, where a vector load would have to wait behind the whole queue of KV loads.
__device__ __forceinline__ int sload_i32(const int32_t* ptr) {
  const uint64_t a = reinterpret_cast<uint64_t>(ptr);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  const uint64_t u = ((uint64_t)hi << 32) | lo;
  int v;
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(u) : "memory");
  return v;
}

// ---------------------------------------------------------------------------------------------------
// 1. plan
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kPlanThreads) void paged_decode_plan_kernel(const DecodeParams p) {
  __shared__ int scan[kPlanThreads];
  __shared__ int prefix_lds[kPlanLdsSeqs + 1];
  const int tid = threadIdx.x;
  const bool use_lds = p.batch <= kPlanLdsSeqs;
  const int per_thread = (p.batch + kPlanThreads - 1) / kPlanThreads;
  const int b0 = min(tid * per_thread, p.batch), b1 = min(b0 + per_thread, p.batch);
  int mine = 0;
  for (int b = b0; b < b1; ++b) mine += stages_of(clamp_seqlen(p.cache_seqlens[b], p));
  scan[tid] = mine;
  __syncthreads();
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    const int v = tid >= off ? scan[tid - off] : 0;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  const int total = scan[kPlanThreads - 1];
  int pos = scan[tid] - mine;
  for (int b = b0; b < b1; ++b) {
    p.prefix[b] = pos;
    if (use_lds) prefix_lds[b] = pos;
    pos += stages_of(clamp_seqlen(p.cache_seqlens[b], p));
  }
  if (tid == 0) {
    p.prefix[p.batch] = total;
    if (use_lds) prefix_lds[p.batch] = total;
  }
  const int per_col = max(p.min_per_col, (total + p.ncols - 1) / p.ncols);
  if (tid == 0) {
    p.hdr[kHdrTotal] = total;
    p.hdr[kHdrPerCol] = per_col;
    p.hdr[kHdrMagic] = kPlanMagic;
    p.hdr[kHdrBatch] = p.batch;
    p.hdr[kHdrCols] = p.ncols;
    p.hdr[kHdrHq] = p.hq;
    p.hdr[kHdrHkv] = p.hkv;
    p.hdr[kHdrBlockSize] = p.block_size;
    p.hdr[kHdrMaxBlocks] = p.max_blocks_per_seq;
  }
  __syncthreads();
  const int* pre = use_lds ? prefix_lds : p.prefix;
  for (int j = tid; j < p.ncols; j += kPlanThreads) {
    const int64_t flat64 = (int64_t)j * per_col;
    int b = 0, s = 0;
    if (flat64 < total) {
      const int flat = (int)flat64;
      // largest b with prefix[b] <= flat; ties (empty sequences) resolve to the last of them,
      // which is the non-empty one that owns the stage
      int lo = 0, hi = p.batch;  // invariant: prefix[lo] <= flat < prefix[hi]
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (pre[mid] <= flat) lo = mid; else hi = mid;
      }
      b = lo;
      s = flat - pre[lo];
    }
    p.col_start[2 * j] = b;
    p.col_start[2 * j + 1] = s;
  }
}

// ---------------------------------------------------------------------------------------------------
// 2. main kernel
// ---------------------------------------------------------------------------------------------------
struct Piece {       // wave-uniform: the part of one sequence that lies inside this column's run
  int valid;
  int b;
  int tok_begin, tok_end, nstages;
  int complete;      // covers the whole sequence: normalise and write `out` directly
  int slot;          // partial slot of the column when not complete
  int blk0;          // cache block of the first stage
};

template <int HPW>
__global__ __launch_bounds__(kWave * HPW, 2) void paged_decode_kernel(const DecodeParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds_all[HPW * 2 * kTileBytes];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  unsigned char* const lds_k = lds_all + wave * 2 * kTileBytes;
  unsigned char* const lds_v = lds_k + kTileBytes;

  const int n_hg = p.hkv / HPW;                      // head groups (workgroups) per column
  const int col = blockIdx.x / n_hg;
  const int g = (blockIdx.x % n_hg) * HPW + wave;    // this wave's kv head
  if (!plan_fits(p)) return;   // the combine kernel writes zero rows in that case
  const int total = p.hdr[kHdrTotal];
  const int per_col = p.hdr[kHdrPerCol];
  const int64_t flat0 = (int64_t)col * per_col;
  if (flat0 >= total) return;
  int remaining = min(per_col, total - (int)flat0);  // stages left in this column's run

  const int n = lane & 15;                           // query head inside the group (MFMA column)
  const int jj = lane >> 4;                          // MFMA row quad / k slice
  const int ld_tok = lane >> 4;                      // token (mod 4) this lane loads
  const int ld_slice = lane & 15;                    // 16-byte piece of the 256-byte row
  const int64_t tok_stride = (int64_t)p.hkv * kHeadDim;
  const bool head_ok = n < p.group;

  auto block_ok = [&](int blk) -> bool { return blk >= 0 && blk < p.num_blocks; };
  auto table_at = [&](int b, int tok) -> int {
    return sload_i32(p.block_table + (int64_t)b * p.block_table_row_stride + tok / p.block_size);
  };
  // piece of sequence b starting at its stage s, limited to `budget` stages
  auto make_piece = [&](int b, int s, int budget) -> Piece {
    Piece d;
    const int seqlen = clamp_seqlen(sload_i32(p.cache_seqlens + b), p);
    const int nst = stages_of(seqlen);
    const int e = min(nst, s + budget);
    d.valid = e > s;
    d.b = b;
    d.tok_begin = s * kStageTokens;
    d.tok_end = min(seqlen, e * kStageTokens);
    d.nstages = e - s;
    d.complete = (s == 0 && e == nst);
    d.slot = s > 0 ? 0 : 1;
    d.blk0 = d.valid ? table_at(b, d.tok_begin) : -1;
    return d;
  };
  // first non-empty sequence after b (the run still has stages left, so one exists)
  auto next_piece = [&](int b, int budget) -> Piece {
    Piece d;
    d.valid = 0;
    d.b = b;
    d.tok_begin = d.tok_end = d.nstages = d.complete = d.slot = 0;
    d.blk0 = -1;
    if (budget <= 0) return d;
    for (int nb = b + 1; nb < p.batch; ++nb) {
      d = make_piece(nb, 0, budget);
      if (d.valid) break;
    }
    return d;
  };

  // Per-lane byte offsets of the eight rows a lane loads per stage: fixed for the whole kernel, so an
  // issue only has to form two wave-uniform base addresses.
  uint32_t voff[8];
#pragma unroll
  for (int qi = 0; qi < 8; ++qi)
    voff[qi] = (uint32_t)(((int64_t)(4 * qi + ld_tok) * tok_stride + (ld_slice << 3)) * 2);
  u32x4 kreg[8], vreg[8];
  auto issue_loads = [&](int tok0, int blk) {   // tok0: first token of the stage inside its sequence
    const int64_t base = (((int64_t)blk * p.block_size + (tok0 % p.block_size)) * tok_stride + (int64_t)g * kHeadDim) * 2;
    const char* kb = reinterpret_cast<const char*>(p.k_cache) + base;
    const char* vb = reinterpret_cast<const char*>(p.v_cache) + base;
#pragma unroll
    for (int qi = 0; qi < 8; ++qi) {
      kreg[qi] = load16_stream(kb + voff[qi]);
      vreg[qi] = load16_stream(vb + voff[qi]);
    }
  };
  // Q as the B operand of S^T = K . Q^T: lane (n, jj) holds Q[g*group + n][(4*kb + jj)*8 .. +8).
  auto load_q = [&](int b, bf16x8 (&dst)[4]) {
    const uint16_t* qrow = p.q + (int64_t)b * p.q_batch_stride + (int64_t)(g * p.group + (head_ok ? n : 0)) * kHeadDim;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      u32x4 w = {0u, 0u, 0u, 0u};
      if (head_ok) w = load16(qrow + ((4 * kb + jj) << 3));
      dst[kb] = __builtin_bit_cast(bf16x8, w);
    }
  };

  const int b_first = p.col_start[2 * col], s_first = p.col_start[2 * col + 1];
  if (b_first < 0 || b_first >= p.batch || s_first < 0) return;   // cannot happen for a planned run
  Piece cur = make_piece(b_first, s_first, remaining);
  if (!cur.valid) return;  // a plan made for other lengths: nothing of this sequence lies in the run

  bf16x8 qb[4];
  f32x4 acc[8];
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;  // running max of scaled (base-2) scores for query head n
  float l_run = 0.f;        // this lane's share of the running sum

  // Block of the stage whose data is in (or on its way to) the registers.  A table entry outside the
  // cache is read as block 0 with every token masked, so control flow never depends on it.
  int blk_ld = cur.blk0;
  load_q(cur.b, qb);
  issue_loads(cur.tok_begin, block_ok(blk_ld) ? blk_ld : 0);
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) asm volatile("" : "+v"(qb[kb]));

  while (true) {
    remaining -= cur.nstages;
    // the piece after this one: looked up now, while this piece's first stage is still in flight
    const Piece nxt = next_piece(cur.b, remaining);
    int st = 0;
    do {
      const int tok0 = cur.tok_begin + st * kStageTokens;
      const int valid = block_ok(blk_ld) ? min(kStageTokens, cur.tok_end - tok0) : 0;
      // registers -> LDS (swizzled); V rows past the end of the context become zeros so that a
      // zero probability times stale cache contents can never produce a NaN.
#pragma unroll
      for (int qi = 0; qi < 8; ++qi) {
        const int t = 4 * qi + ld_tok;
        const int off = tile_offset(t, ld_slice);
        *reinterpret_cast<u32x4*>(lds_k + off) = kreg[qi];
        *reinterpret_cast<u32x4*>(lds_v + off) = vreg[qi];
      }
      if (valid < kStageTokens) {
#pragma unroll
        for (int qi = 0; qi < 8; ++qi) {
          const int t = 4 * qi + ld_tok;
          if (t >= valid) *reinterpret_cast<u32x4*>(lds_v + tile_offset(t, ld_slice)) = u32x4{0u, 0u, 0u, 0u};
        }
      }
      // Everything older than the rows just consumed has landed; the only loads that can still be
      // outstanding are a new piece's query rows.  Waiting for them here, with the queue empty, keeps
      // the compute section free of a wait that would also cover the stage issued below.
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) asm volatile("" : "+v"(qb[kb]));
      // ---- put the next stage in flight before this one is consumed: the next stage of this piece,
      //      or the first stage (and the query rows) of the next piece
      const bool last_stage = st + 1 >= cur.nstages;
      {
        int tok1 = tok0 + kStageTokens;
        bool more = true;
        if (!last_stage) {
          if (tok1 % p.block_size == 0) blk_ld = table_at(cur.b, tok1);
        } else {
          tok1 = nxt.tok_begin;
          blk_ld = nxt.blk0;
          more = nxt.valid;
        }
        if (more) issue_loads(tok1, block_ok(blk_ld) ? blk_ld : 0);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      // ---- S^T = K . Q^T for the two 16-token tiles
      f32x4 s[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
          const u32x4 w = *reinterpret_cast<const u32x4*>(lds_k + tile_offset(16 * tt + n, 4 * kb + jj));
          s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), qb[kb], s[tt], 0, 0, 0);
        }
      }
      // ---- online softmax; lane (n, jj) holds tokens 16*tt + 4*jj + r of query head n
      float sv[8];
      float m_loc = -INFINITY;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = 16 * tt + 4 * jj + r;
          float x = s[tt][r] * p.scale_log2;
          x = (t < valid) ? x : -INFINITY;
          sv[4 * tt + r] = x;
          m_loc = fmaxf(m_loc, x);
        }
      m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 16, kWave));
      m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32, kWave));
      const float m_new = fmaxf(m_run, m_loc);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
      float psum = 0.f;
      float pv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pv[e] = __builtin_amdgcn_exp2f(sv[e] - m_safe);
        psum += pv[e];
      }
      l_run = l_run * alpha + psum;
      m_run = m_new;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) acc[dt] *= alpha;
      }
      u32x4 pw;
#pragma unroll
      for (int e = 0; e < 4; ++e) pw[e] = pack_bf16x2(pv[2 * e], pv[2 * e + 1]);
      const bf16x8 pb = __builtin_bit_cast(bf16x8, pw);
      // ---- O^T += V^T . P^T ; transposing LDS reads assemble V^T[d, 8 tokens] per lane
      const int src_row = (lane & 15) >> 2;   // which of the 4 token rows this lane addresses
      const int src_chunk = lane & 3;         // which 4-wide d chunk of the 16-wide window
#pragma unroll
      for (int dt = 0; dt < 8; ++dt) {
        const int slice = 2 * dt + (src_chunk >> 1);
        const int t_lo = 4 * jj + src_row;
        const int t_hi = 16 + t_lo;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)(lds_v + tile_offset(t_lo, slice) + ((src_chunk & 1) << 3)));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)(lds_v + tile_offset(t_hi, slice) + ((src_chunk & 1) << 3)));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        const s16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), pb, acc[dt], 0, 0, 0);
      }
      // the query rows are free now: on the last stage, fetch the next piece's into the same registers
      if (last_stage && nxt.valid) load_q(nxt.b, qb);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      ++st;
    } while (st < cur.nstages);

    // ---- piece finished: total sum for query head n over the four row-quads, then write out
    float l_tot = l_run + __shfl_xor(l_run, 16, kWave);
    l_tot += __shfl_xor(l_tot, 32, kWave);
    if (head_ok) {
      const int h = g * p.group + n;
      if (cur.complete) {
        const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        uint16_t* orow = p.out + ((int64_t)cur.b * p.hq + h) * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
          u32x2 w;
          w[0] = pack_bf16x2(acc[dt][0] * inv, acc[dt][1] * inv);
          w[1] = pack_bf16x2(acc[dt][2] * inv, acc[dt][3] * inv);
          *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * jj) = w;
        }
      } else {
        const int64_t slot = ((int64_t)col * 2 + cur.slot) * p.hq + h;
        float* arow = p.ws_acc + slot * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) *reinterpret_cast<f32x4*>(arow + 16 * dt + 4 * jj) = acc[dt];
        if (jj == 0) {
          p.ws_ml[2 * slot] = m_run;
          p.ws_ml[2 * slot + 1] = l_tot;
        }
      }
    }
    if (!nxt.valid) break;
    cur = nxt;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run = -INFINITY;
    l_run = 0.f;
  }
}

// ---------------------------------------------------------------------------------------------------
// 3. combine: one wave per (sequence, query head); lane owns two output elements.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kWave) void paged_decode_combine_kernel(const DecodeParams p) {
  const int bh = blockIdx.x;
  const int b = bh / p.hq;
  const int h = bh % p.hq;
  const int lane = threadIdx.x;
  if (!plan_fits(p)) {  // no usable plan: the main kernel did nothing; leave a defined (zero) row
    reinterpret_cast<uint32_t*>(p.out + (int64_t)bh * kHeadDim)[lane] = 0u;
    return;
  }
  const int f0 = p.prefix[b], f1 = p.prefix[b + 1];
  if (f1 <= f0) {  // an empty context attends to nothing: zeros
    reinterpret_cast<uint32_t*>(p.out + (int64_t)bh * kHeadDim)[lane] = 0u;
    return;
  }
  const int per_col = p.hdr[kHdrPerCol];
  const int j0 = f0 / per_col, j1 = (f1 - 1) / per_col;
  if (j0 == j1) return;  // one piece: written directly by the main kernel
  // partial of column j: slot 1 in the column where the sequence begins, slot 0 in the following ones
  auto slot_of = [&](int j) -> int64_t { return ((int64_t)j * 2 + (j == j0 ? 1 : 0)) * p.hq + h; };
  // A short batch of long sequences spreads one sequence over many columns, so neither pass may be a
  // chain of dependent loads: the maxima are read one per lane and reduced across the wave, and the
  // weighted sum keeps eight independent partial rows in flight.
  const int n_parts = j1 - j0 + 1;
  float m = -INFINITY;
  for (int i = lane; i < n_parts; i += kWave) m = fmaxf(m, p.ws_ml[2 * slot_of(j0 + i)]);
  m = group_max<kWave>(m);
  const float m_safe = (m == -INFINITY) ? 0.f : m;
  float l = 0.f, o0 = 0.f, o1 = 0.f;
  for (int i0 = 0; i0 < n_parts; i0 += 8) {
    float ml[8][2];
    float2 a[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const bool ok = i0 + u < n_parts;
      const int64_t sl = slot_of(j0 + (ok ? i0 + u : 0));
      ml[u][0] = ok ? p.ws_ml[2 * sl] : -INFINITY;
      ml[u][1] = ok ? p.ws_ml[2 * sl + 1] : 0.f;
      a[u] = *reinterpret_cast<const float2*>(p.ws_acc + sl * kHeadDim + 2 * lane);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {   // same order of additions as a plain loop over the columns
      const float w = (i0 + u < n_parts) ? __builtin_amdgcn_exp2f(ml[u][0] - m_safe) : 0.f;
      l += w * ml[u][1];
      o0 += w * a[u].x;
      o1 += w * a[u].y;
    }
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  reinterpret_cast<uint32_t*>(p.out + (int64_t)bh * kHeadDim)[lane] = pack_bf16x2(o0 * inv, o1 * inv);
}

// ---------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------
static int env_int(const char* name) {
  const char* e = getenv(name);
  return e ? atoi(e) : 0;
}

// Waves (= kv heads) per workgroup: 2 streams 512 contiguous bytes per token per workgroup and still
// leaves four independent workgroups per CU.
static int choose_hpw(int hkv) {
  static const int forced = env_int("MOPS_HIP_DECODE_HPW");  // tuning override: 1, 2, 4 or 8
  int want = (forced == 1 || forced == 2 || forced == 4 || forced == 8) ? forced : 2;
  while (want > 1 && hkv % want != 0) want >>= 1;
  return want;
}

static int device_cu_count() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    return n;
  }();
  return cus;
}

// Columns of the flat split: every CU holds 8 waves (16 KiB of LDS tiles each, two per SIMD), a
// column needs hkv waves.
static int choose_ncols(int64_t hkv) {
  static const int forced = env_int("MOPS_HIP_DECODE_NCOLS");  // tuning override
  if (forced > 0) return forced;
  const int64_t n = (int64_t)device_cu_count() * 8 / hkv;
  return (int)(n < 1 ? 1 : n);
}

static int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

struct WorkspaceLayout {
  int64_t hdr, prefix, col_start, acc, ml, total;
};

static WorkspaceLayout workspace_layout(int64_t batch, int64_t hq, int64_t ncols) {
  WorkspaceLayout w;
  w.hdr = 0;
  w.prefix = align_up(kHdrInts * 4, 256);
  w.col_start = w.prefix + align_up((batch + 1) * 4, 256);
  w.acc = w.col_start + align_up(ncols * 2 * 4, 256);
  w.ml = w.acc + align_up(ncols * 2 * hq * kHeadDim * 4, 256);
  w.total = w.ml + align_up(ncols * 2 * hq * 2 * 4, 256);
  return w;
}

}  // namespace mops

extern "C" int64_t mops_hip_paged_decode_workspace_bytes(int64_t batch, int64_t hq, int64_t hkv,
                                                         int64_t max_blocks_per_seq, int64_t block_size) {
  using namespace mops;
  if (batch <= 0 || hq <= 0 || hkv <= 0 || max_blocks_per_seq <= 0 || block_size <= 0) return 0;
  return workspace_layout(batch, hq, choose_ncols(hkv)).total;
}

namespace mops {

// Validates the arguments and launches plan (unless reused), main and combine kernels with `workspace` as scratch.
static int launch_paged_decode(const void* q, int64_t q_batch_stride,
                               const void* k_cache, const void* v_cache,
                               const int32_t* cache_seqlens,
                               const int32_t* block_table, int64_t block_table_row_stride,
                               void* out,
                               int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                               int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                               float softmax_scale,
                               void* workspace, int64_t workspace_bytes,
                               int plan_mode, void* stream) {
  if (batch < 0 || hq <= 0 || hkv <= 0 || block_size <= 0 || num_blocks < 0 || max_blocks_per_seq < 0)
    return MOPS_HIP_EINVAL;
  if (plan_mode != MOPS_HIP_DECODE_PLAN_AND_ATTEND && plan_mode != MOPS_HIP_DECODE_REUSE_PLAN) return MOPS_HIP_EINVAL;
  if (batch == 0) return MOPS_HIP_OK;
  if (!q || !k_cache || !v_cache || !cache_seqlens || !block_table || !out) return MOPS_HIP_EINVAL;
  if (hq % hkv != 0 || block_table_row_stride < max_blocks_per_seq || num_blocks == 0) return MOPS_HIP_EINVAL;
  if (q_batch_stride < hq * head_dim) return MOPS_HIP_EINVAL;
  if (head_dim != kHeadDim || hq / hkv > 16 || block_size % kStageTokens != 0) return MOPS_HIP_EUNSUPPORTED;
  if (batch >= (1 << 20) || hq > 4096 || hkv > 1024 || max_blocks_per_seq * block_size > (1 << 24) ||
      num_blocks * block_size > (int64_t)0x7fffffff)
    return MOPS_HIP_EUNSUPPORTED;
  // the flat split counts 32-token stages in int32
  if (batch * ((max_blocks_per_seq * block_size + kStageTokens - 1) / kStageTokens) > (int64_t)0x7fffffff) return MOPS_HIP_EUNSUPPORTED;
  if ((q_batch_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out)) return MOPS_HIP_EALIGN;
  hipStream_t s = (hipStream_t)stream;

  DecodeParams p;
  p.q = (const uint16_t*)q;
  p.q_batch_stride = q_batch_stride;
  p.k_cache = (const uint16_t*)k_cache;
  p.v_cache = (const uint16_t*)v_cache;
  p.cache_seqlens = cache_seqlens;
  p.block_table = block_table;
  p.block_table_row_stride = block_table_row_stride;
  p.out = (uint16_t*)out;
  p.batch = (int)batch;
  p.hq = (int)hq;
  p.hkv = (int)hkv;
  p.group = (int)(hq / hkv);
  p.block_size = (int)block_size;
  p.num_blocks = (int)num_blocks;
  p.max_blocks_per_seq = (int)max_blocks_per_seq;
  p.ncols = choose_ncols(hkv);
  {
    // With few stages in all (a short batch) runs of one stage would spread a sequence over as many partial
    // results as it has stages; two stages per column halve the combine's work at no cost to the streaming.
    static const int forced = env_int("MOPS_HIP_DECODE_MIN_PER_COL");  // tuning override
    p.min_per_col = forced > 0 ? forced : 2;
  }
  p.scale_log2 = softmax_scale * 1.44269504088896340736f;
  const WorkspaceLayout w = workspace_layout(batch, hq, p.ncols);
  if (!workspace || workspace_bytes < w.total) return MOPS_HIP_EWORKSPACE;
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return MOPS_HIP_EALIGN;
  char* base = (char*)workspace;
  p.hdr = (int32_t*)(base + w.hdr);
  p.prefix = (int32_t*)(base + w.prefix);
  p.col_start = (int32_t*)(base + w.col_start);
  p.ws_acc = (float*)(base + w.acc);
  p.ws_ml = (float*)(base + w.ml);

  int st = MOPS_HIP_OK;
  if (plan_mode != MOPS_HIP_DECODE_REUSE_PLAN) {
    hipLaunchKernelGGL(paged_decode_plan_kernel, dim3(1), dim3(kPlanThreads), 0, s, p);
    st = finish_launch();
    if (st != MOPS_HIP_OK) return st;
  }

  const int hpw = choose_hpw(p.hkv);
  const dim3 grid((unsigned)((int64_t)p.ncols * (p.hkv / hpw))), block((unsigned)(kWave * hpw));
  switch (hpw) {
    case 8: hipLaunchKernelGGL(paged_decode_kernel<8>, grid, block, 0, s, p); break;
    case 4: hipLaunchKernelGGL(paged_decode_kernel<4>, grid, block, 0, s, p); break;
    case 2: hipLaunchKernelGGL(paged_decode_kernel<2>, grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL(paged_decode_kernel<1>, grid, block, 0, s, p); break;
  }
  st = finish_launch();
  if (st != MOPS_HIP_OK) return st;
  hipLaunchKernelGGL(paged_decode_combine_kernel, dim3((unsigned)(batch * hq)), dim3(kWave), 0, s, p);
  return finish_launch();
}

// Scratch of the allocation-free entry point: one copy per GPU, held until the process ends.  In host code
// this name is only a handle for hipGetSymbolAddress; the device address it yields is what the kernels get.
constexpr int64_t kStaticScratchBytes = MOPS_HIP_DECODE_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each GPU, looked up once
static std::mutex g_scratch_mutex;

// Device address of this GPU's copy of `scratch` (nullptr and a status on failure).
static int static_scratch(void** ptr) {
  *ptr = nullptr;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return record_hip_error(e != hipSuccess ? e : hipErrorInvalidDevice);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !addr) return record_hip_error(e != hipSuccess ? e : hipErrorInvalidSymbol);
    g_scratch_ptr[dev] = addr;
  }
  *ptr = g_scratch_ptr[dev];
  return MOPS_HIP_OK;
}

}  // namespace mops

extern "C" int mops_hip_attn_paged_decode_planned_bf16(const void* q, int64_t q_batch_stride,
                                                       const void* k_cache, const void* v_cache,
                                                       const int32_t* cache_seqlens,
                                                       const int32_t* block_table, int64_t block_table_row_stride,
                                                       void* out,
                                                       int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                                                       int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                                       float softmax_scale,
                                                       void* workspace, int64_t workspace_bytes,
                                                       int plan_mode, void* stream) {
  return mops::launch_paged_decode(q, q_batch_stride, k_cache, v_cache, cache_seqlens, block_table, block_table_row_stride,
                                   out, batch, hq, hkv, head_dim, block_size, num_blocks, max_blocks_per_seq, softmax_scale,
                                   workspace, workspace_bytes, plan_mode, stream);
}

extern "C" int mops_hip_attn_paged_decode_noalloc_bf16(const void* q, int64_t q_batch_stride,
                                                       const void* k_cache, const void* v_cache,
                                                       const int32_t* cache_seqlens,
                                                       const int32_t* block_table, int64_t block_table_row_stride,
                                                       void* out,
                                                       int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                                                       int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                                       float softmax_scale, void* stream) {
  using namespace mops;
  if (batch <= 0 || hq <= 0 || hkv <= 0) {
    // let the shared validation name the problem (or accept the empty batch); no scratch is needed for either
    return launch_paged_decode(q, q_batch_stride, k_cache, v_cache, cache_seqlens, block_table, block_table_row_stride, out,
                               batch, hq, hkv, head_dim, block_size, num_blocks, max_blocks_per_seq, softmax_scale,
                               nullptr, 0, MOPS_HIP_DECODE_PLAN_AND_ATTEND, stream);
  }
  if (workspace_layout(batch, hq, choose_ncols(hkv)).total > kStaticScratchBytes) return MOPS_HIP_ETOOLARGE;
  void* ws = nullptr;
  const int st = static_scratch(&ws);
  if (st != MOPS_HIP_OK) return st;
  return launch_paged_decode(q, q_batch_stride, k_cache, v_cache, cache_seqlens, block_table, block_table_row_stride, out,
                             batch, hq, hkv, head_dim, block_size, num_blocks, max_blocks_per_seq, softmax_scale,
                             ws, kStaticScratchBytes, MOPS_HIP_DECODE_PLAN_AND_ATTEND, stream);
}

extern "C" int mops_hip_attn_paged_decode_bf16(const void* q, int64_t q_batch_stride,
                                               const void* k_cache, const void* v_cache,
                                               const int32_t* cache_seqlens,
                                               const int32_t* block_table, int64_t block_table_row_stride,
                                               void* out,
                                               int64_t batch, int64_t hq, int64_t hkv, int64_t head_dim,
                                               int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                               float softmax_scale,
                                               void* workspace, int64_t workspace_bytes,
                                               void* stream) {
  return mops_hip_attn_paged_decode_planned_bf16(q, q_batch_stride, k_cache, v_cache, cache_seqlens, block_table,
                                                 block_table_row_stride, out, batch, hq, hkv, head_dim, block_size,
                                                 num_blocks, max_blocks_per_seq, softmax_scale, workspace, workspace_bytes,
                                                 MOPS_HIP_DECODE_PLAN_AND_ATTEND, stream);
}
