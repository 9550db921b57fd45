// Paged decode attention for gfx950: one query token per sequence against the block-table-addressed
// KV cache (layout [num_blocks, block_size, hkv, 128] bf16).  HBM-bandwidth bound: every K/V byte of
// the live context is read exactly once, 16 bytes per lane, 256 contiguous bytes per token row.
//
// Work decomposition
//   unit  = (chunk c, sequence b, kv head g): the tokens [c*chunk, (c+1)*chunk) of sequence b for one
//           kv head, served for ALL hq/hkv query heads of that group from one read of K and V.
//   one unit = one 64-lane workgroup (a single wave64): no workgroup barriers, the wave owns a private
//           16 KiB LDS tile.  Units are numbered chunk-major so the units that fall beyond a
//           sequence's length (they exit at once) collect at the end of the launch.
//   stage = 32 consecutive tokens of the unit (inside one cache block): 8 KiB of K + 8 KiB of V.
//           Stage i+1 is in flight from HBM into registers while stage i is consumed out of LDS.
//
// Per stage, per wave
//   S^T[token, qhead] = K[token, :] . Q^T            8 x v_mfma_f32_16x16x32_bf16 (K tile as A operand,
//                                                     read back from LDS with a 16-byte XOR swizzle)
//   online softmax over tokens (base-2 exponent, fp32 running max / sum per query head)
//   O^T[d, qhead]    += V^T[d, token] . P^T           8 x v_mfma_f32_16x16x32_bf16; V^T comes out of
//                                                     LDS through ds_read_b64_tr_b16 (transposing read)
//   The accumulator layout of S^T is exactly the B-operand layout the second product needs, so P never
//   moves between lanes.
//
// A sequence whose context fits one chunk is written straight to `out`; longer ones leave
// (max, sum, unnormalised O) partials in the workspace for paged_decode_combine_kernel.
#include "mops_common.h"

namespace mops {

constexpr int kHeadDim = 128;
constexpr int kStageTokens = 32;
constexpr int kRowBytes = kHeadDim * 2;                  // one token, one kv head
constexpr int kTileBytes = kStageTokens * kRowBytes;     // 8 KiB

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
  float* ws_acc;   // [batch*hq, max_chunks, 128]
  float* ws_ml;    // [batch*hq, max_chunks, 2]   (running max in the base-2 scaled domain, sum)
  int batch, hq, hkv, group;       // group = hq / hkv  (<= 16)
  int block_size, num_blocks, max_blocks_per_seq;
  int chunk_tokens, max_chunks;
  float scale_log2;                // softmax_scale * log2(e)
};

__device__ __forceinline__ int clamp_seqlen(int s, const DecodeParams& p) {
  const int cap = p.max_blocks_per_seq * p.block_size;
  return s < 0 ? 0 : (s > cap ? cap : s);
}

__global__ __launch_bounds__(kWave) void paged_decode_kernel(const DecodeParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kTileBytes];
  unsigned char* const lds_k = lds;
  unsigned char* const lds_v = lds + kTileBytes;

  const int lane = threadIdx.x;
  const int unit = blockIdx.x;
  const int g = unit % p.hkv;
  const int b = (unit / p.hkv) % p.batch;
  const int c = unit / (p.hkv * p.batch);

  const int seqlen = clamp_seqlen(p.cache_seqlens[b], p);
  const int nchunks = (seqlen + p.chunk_tokens - 1) / p.chunk_tokens;
  if (c >= (nchunks > 0 ? nchunks : 1)) return;

  const int n = lane & 15;   // query head inside the group (MFMA column)
  const int jj = lane >> 4;  // MFMA row quad / k slice
  const int tok_begin = c * p.chunk_tokens;
  const int tok_end = min(seqlen, tok_begin + p.chunk_tokens);
  const int nstages = (tok_end - tok_begin + kStageTokens - 1) / kStageTokens;  // 0 when seqlen == 0

  // Q as the B operand of S^T = K . Q^T: lane (n, jj) holds Q[g*group + n][(4*kb + jj)*8 .. +8).
  bf16x8 qb[4];
  {
    const bool head_ok = n < p.group;
    const uint16_t* qrow = p.q + (int64_t)b * p.q_batch_stride + (int64_t)(g * p.group + (head_ok ? n : 0)) * kHeadDim;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      u32x4 w = {0u, 0u, 0u, 0u};
      if (head_ok) w = load16(qrow + ((4 * kb + jj) << 3));
      qb[kb] = __builtin_bit_cast(bf16x8, w);
    }
  }

  const int32_t* table = p.block_table + (int64_t)b * p.block_table_row_stride;
  const int64_t tok_stride = (int64_t)p.hkv * kHeadDim;  // elements between consecutive tokens of a block
  const int ld_tok = lane >> 4;                           // token (mod 4) this lane loads
  const int ld_slice = lane & 15;                         // 16-byte piece of the 256-byte row

  u32x4 kreg[8], vreg[8];
  auto issue_loads = [&](int stage, int blk) {
    const int t0 = tok_begin + stage * kStageTokens;
    const int64_t base = ((int64_t)blk * p.block_size + (t0 % p.block_size) + ld_tok) * tok_stride +
                         (int64_t)g * kHeadDim + (ld_slice << 3);
#pragma unroll
    for (int qi = 0; qi < 8; ++qi) {
      kreg[qi] = load16_stream(p.k_cache + base + (int64_t)(4 * qi) * tok_stride);
      vreg[qi] = load16_stream(p.v_cache + base + (int64_t)(4 * qi) * tok_stride);
    }
  };
  auto block_of = [&](int stage) -> int {
    const int t0 = tok_begin + stage * kStageTokens;
    return table[t0 / p.block_size];
  };
  auto block_ok = [&](int blk) -> bool { return blk >= 0 && blk < p.num_blocks; };

  f32x4 acc[8];
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;  // running max of scaled (base-2) scores for query head n
  float l_run = 0.f;        // this lane's share of the running sum

  int blk_cur = nstages > 0 ? block_of(0) : -1;
  int blk_next = nstages > 1 ? block_of(1) : -1;
  if (nstages > 0 && block_ok(blk_cur)) issue_loads(0, blk_cur);
  // Pin the wait for Q here, behind the first stage's loads, so the loop body never has to wait for
  // "everything outstanding" on Q's account.
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) asm volatile("" : "+v"(qb[kb]));

  for (int st = 0; st < nstages; ++st) {
    const bool cur_ok = block_ok(blk_cur);
    const int valid = min(kStageTokens, tok_end - (tok_begin + st * kStageTokens));
    if (cur_ok) {
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
    }
    // next stage goes in flight before this one is consumed
    const int blk_after = (st + 2 < nstages) ? block_of(st + 2) : -1;
    if (st + 1 < nstages && block_ok(blk_next)) issue_loads(st + 1, blk_next);
    __syncthreads();

    if (cur_ok) {
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
    }
    __syncthreads();
    blk_cur = blk_next;
    blk_next = blk_after;
  }

  // total sum for query head n over the four row-quads
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);

  if (n >= p.group) return;
  const int h = g * p.group + n;
  if (nchunks <= 1) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    uint16_t* orow = p.out + ((int64_t)b * p.hq + h) * kHeadDim;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      u32x2 w;
      w[0] = pack_bf16x2(acc[dt][0] * inv, acc[dt][1] * inv);
      w[1] = pack_bf16x2(acc[dt][2] * inv, acc[dt][3] * inv);
      *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * jj) = w;
    }
  } else {
    const int64_t slot = ((int64_t)b * p.hq + h) * p.max_chunks + c;
    float* arow = p.ws_acc + slot * kHeadDim;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) *reinterpret_cast<f32x4*>(arow + 16 * dt + 4 * jj) = acc[dt];
    if (jj == 0) {
      p.ws_ml[2 * slot] = m_run;
      p.ws_ml[2 * slot + 1] = l_run;
    }
  }
}

// Merges the per-chunk partials of every (sequence, query head) that needed more than one chunk.
// One wave per (b, h); lane owns two output elements.
__global__ __launch_bounds__(kWave) void paged_decode_combine_kernel(const DecodeParams p) {
  const int bh = blockIdx.x;
  const int b = bh / p.hq;
  const int seqlen = clamp_seqlen(p.cache_seqlens[b], p);
  const int nchunks = (seqlen + p.chunk_tokens - 1) / p.chunk_tokens;
  if (nchunks <= 1) return;
  const int lane = threadIdx.x;
  const float* ml = p.ws_ml + (int64_t)bh * p.max_chunks * 2;
  const float* accp = p.ws_acc + (int64_t)bh * p.max_chunks * kHeadDim + 2 * lane;
  float m = -INFINITY;
  for (int c = 0; c < nchunks; ++c) m = fmaxf(m, ml[2 * c]);
  const float m_safe = (m == -INFINITY) ? 0.f : m;
  float l = 0.f, o0 = 0.f, o1 = 0.f;
  for (int c = 0; c < nchunks; ++c) {
    const float w = __builtin_amdgcn_exp2f(ml[2 * c] - m_safe);
    l += w * ml[2 * c + 1];
    const float2 a = *reinterpret_cast<const float2*>(accp + (int64_t)c * kHeadDim);
    o0 += w * a.x;
    o1 += w * a.y;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  reinterpret_cast<uint32_t*>(p.out + (int64_t)bh * kHeadDim)[lane] = pack_bf16x2(o0 * inv, o1 * inv);
}

// Chunk length (tokens, multiple of the stage) chosen from launch-time upper bounds only: enough
// units to keep every SIMD of the 256 CUs busy for several rounds, but not so many that the
// partials traffic shows up next to the KV stream.
static int choose_chunk_tokens(int64_t batch, int64_t hkv, int64_t max_tokens) {
  const int64_t target_units = 16384;
  int64_t chunk = (batch * hkv * max_tokens + target_units - 1) / target_units;
  chunk = (chunk + kStageTokens - 1) / kStageTokens * kStageTokens;
  if (chunk < 2 * kStageTokens) chunk = 2 * kStageTokens;
  if (chunk > 512) chunk = 512;
  return (int)chunk;
}

static int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

}  // namespace mops

extern "C" int64_t mops_hip_paged_decode_workspace_bytes(int64_t batch, int64_t hq, int64_t hkv,
                                                         int64_t max_blocks_per_seq, int64_t block_size) {
  using namespace mops;
  if (batch <= 0 || hq <= 0 || hkv <= 0 || max_blocks_per_seq <= 0 || block_size <= 0) return 0;
  const int64_t max_tokens = max_blocks_per_seq * block_size;
  const int chunk = choose_chunk_tokens(batch, hkv, max_tokens);
  const int64_t max_chunks = (max_tokens + chunk - 1) / chunk;
  if (max_chunks <= 1) return 256;
  return align_up(batch * hq * max_chunks * kHeadDim * 4, 256) + align_up(batch * hq * max_chunks * 2 * 4, 256);
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
  using namespace mops;
  if (batch < 0 || hq <= 0 || hkv <= 0 || block_size <= 0 || num_blocks < 0 || max_blocks_per_seq < 0)
    return MOPS_HIP_EINVAL;
  if (batch == 0) return MOPS_HIP_OK;
  if (!q || !k_cache || !v_cache || !cache_seqlens || !block_table || !out) return MOPS_HIP_EINVAL;
  if (hq % hkv != 0 || block_table_row_stride < max_blocks_per_seq) return MOPS_HIP_EINVAL;
  if (q_batch_stride < hq * head_dim) return MOPS_HIP_EINVAL;
  if (head_dim != kHeadDim || hq / hkv > 16 || block_size % kStageTokens != 0) return MOPS_HIP_EUNSUPPORTED;
  if (batch > (1 << 20) || hq > 4096 || max_blocks_per_seq * block_size > (1 << 24) ||
      num_blocks * block_size > (int64_t)0x7fffffff)
    return MOPS_HIP_EUNSUPPORTED;
  if ((q_batch_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out)) return MOPS_HIP_EALIGN;
  if (max_blocks_per_seq == 0) {
    hipError_t e = hipMemsetAsync(out, 0, (size_t)(batch * hq * kHeadDim * 2), (hipStream_t)stream);
    return e == hipSuccess ? MOPS_HIP_OK : MOPS_HIP_ELAUNCH;
  }

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
  const int64_t max_tokens = max_blocks_per_seq * block_size;
  p.chunk_tokens = choose_chunk_tokens(batch, hkv, max_tokens);
  p.max_chunks = (int)((max_tokens + p.chunk_tokens - 1) / p.chunk_tokens);
  p.scale_log2 = softmax_scale * 1.44269504088896340736f;
  p.ws_acc = nullptr;
  p.ws_ml = nullptr;
  if (p.max_chunks > 1) {
    const int64_t need = mops_hip_paged_decode_workspace_bytes(batch, hq, hkv, max_blocks_per_seq, block_size);
    if (!workspace || workspace_bytes < need) return MOPS_HIP_EWORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return MOPS_HIP_EALIGN;
    p.ws_acc = (float*)workspace;
    p.ws_ml = (float*)((char*)workspace + align_up(batch * hq * p.max_chunks * kHeadDim * 4, 256));
  }
  const int64_t units = batch * hkv * p.max_chunks;
  if (units > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL(paged_decode_kernel, dim3((unsigned)units), dim3(kWave), 0, (hipStream_t)stream, p);
  int st = finish_launch();
  if (st != MOPS_HIP_OK) return st;
  if (p.max_chunks > 1) {
    hipLaunchKernelGGL(paged_decode_combine_kernel, dim3((unsigned)(batch * hq)), dim3(kWave), 0,
                       (hipStream_t)stream, p);
    st = finish_launch();
  }
  return st;
}
