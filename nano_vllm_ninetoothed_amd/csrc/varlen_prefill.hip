// Varlen (packed THD) causal prefill attention for gfx950, grouped-query heads, head_dim 128.
// bf16 MFMA for both products, fp32 online softmax, K/V tiles staged through LDS.
//
// Work decomposition
//   workgroup (256 lanes, 4 waves) = one 128-row Q tile of one sequence for one query head; wave w owns
//   rows 32w..32w+31.  Workgroups are numbered so that the query heads of one kv group are neighbours
//   (their K/V tiles hit in L2) and the tiles with the longest causal prefix are dispatched first.
//   The launch is sized from max_seqlen; tiles past a sequence's end exit at once.
//
// Per 64-token K/V tile (double-buffered in LDS, next tile in flight from HBM into registers)
//   S^T[token, qrow] = K . Q^T        16 x v_mfma_f32_32x32x16_bf16 per wave; Q^T lives in registers as
//                                      the B operand for the whole kernel, K rows are read from LDS
//                                      with a 16-byte XOR swizzle
//   online softmax down the token axis: each lane owns one q row, so max/sum are register-local
//                                      plus one cross-half exchange
//   O^T[d, qrow]   += V^T . P^T        16 x v_mfma_f32_32x32x16_bf16; the accumulator layout of S^T is
//                                      already the B-operand layout, V^T comes out of LDS through
//                                      ds_read_b64_tr_b16
#include "mops_common.h"

namespace mops {

constexpr int kPD = 128;            // head dim
constexpr int kPBM = 128;           // q rows per workgroup
constexpr int kPBN = 64;            // kv tokens per tile
constexpr int kPThreads = 256;
constexpr int kPRowBytes = kPD * 2;
constexpr int kPTileBytes = kPBN * kPRowBytes;  // 16 KiB

// Byte offset of 16-byte piece `slice` of token row `t` inside an LDS tile.  The piece index is XORed
// with the row's low four bits with the bit pairs swapped: 16 consecutive rows at one slice (the K
// operand read) and 4 consecutive rows x 4 consecutive slices (the transposing V read) both spread
// over all 64 banks.
__device__ __forceinline__ int ptile_offset(int t, int slice) {
  const int g = ((t & 3) << 2) | ((t >> 2) & 3);
  return t * kPRowBytes + ((slice ^ g) << 4);
}

struct PrefillParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  int64_t q_ts, k_ts, v_ts, o_ts;  // token strides (elements)
  const int32_t* cu_seqlens;
  int batch, total_tokens, m_tiles, hq, hkv, group;
  float scale_log2;
};

__global__ __launch_bounds__(kPThreads, 2) void varlen_prefill_kernel(const PrefillParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[4 * kPTileBytes];  // [buf][K|V]

  const int idx = blockIdx.x;
  const int h = idx % p.hq;
  const int b = (idx / p.hq) % p.batch;
  const int m = p.m_tiles - 1 - idx / (p.hq * p.batch);
  const int seq_begin = p.cu_seqlens[b];
  const int seq_len = min(p.cu_seqlens[b + 1], p.total_tokens) - seq_begin;
  const int q0 = m * kPBM;
  if (seq_begin < 0 || q0 >= seq_len) return;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int n = lane & 31;   // q row inside the wave's 32-row slab (MFMA column)
  const int jj = lane >> 5;  // half: k slice / row-quad selector
  const int g = h / p.group;

  const int kv_end = min(seq_len, q0 + kPBM);
  const int ntiles = (kv_end + kPBN - 1) / kPBN;
  const int wave_row0 = q0 + 32 * wave;          // first q row (sequence-relative) of this wave
  const int my_row = wave_row0 + n;

  // ---- Q^T as B operand: lane (n, jj) holds Q[my_row][16*kb + 8*jj .. +8) for kb = 0..7
  bf16x8 qb[8];
  {
    const bool row_ok = my_row < seq_len;
    const uint16_t* qrow = p.q + (int64_t)(seq_begin + (row_ok ? my_row : 0)) * p.q_ts + (int64_t)h * kPD;
#pragma unroll
    for (int kb = 0; kb < 8; ++kb) {
      u32x4 w = {0u, 0u, 0u, 0u};
      if (row_ok) w = load16(qrow + 16 * kb + 8 * jj);
      qb[kb] = __builtin_bit_cast(bf16x8, w);
    }
  }

  // ---- cooperative tile loads: thread moves 16-byte piece (tid & 15) of rows (tid >> 4) + 16*i
  const int ld_row = tid >> 4;
  const int ld_slice = tid & 15;
  const uint16_t* kbase = p.k + (int64_t)seq_begin * p.k_ts + (int64_t)g * kPD + (ld_slice << 3);
  const uint16_t* vbase = p.v + (int64_t)seq_begin * p.v_ts + (int64_t)g * kPD + (ld_slice << 3);
  u32x4 kreg[4], vreg[4];
  auto issue_loads = [&](int tile) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = tile * kPBN + ld_row + 16 * i;
      u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
      if (t < seq_len) {
        kk = load16(kbase + (int64_t)t * p.k_ts);
        vv = load16(vbase + (int64_t)t * p.v_ts);
      }
      kreg[i] = kk;
      vreg[i] = vv;
    }
  };
  auto store_tile = [&](int buf) {
    unsigned char* kt = lds + buf * 2 * kPTileBytes;
    unsigned char* vt = kt + kPTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int off = ptile_offset(ld_row + 16 * i, ld_slice);
      *reinterpret_cast<u32x4*>(kt + off) = kreg[i];
      *reinterpret_cast<u32x4*>(vt + off) = vreg[i];
    }
  };

  f32x16 acc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  issue_loads(0);
#pragma unroll
  for (int kb = 0; kb < 8; ++kb) asm volatile("" : "+v"(qb[kb]));

  for (int tile = 0; tile < ntiles; ++tile) {
    const int buf = tile & 1;
    store_tile(buf);
    __syncthreads();
    if (tile + 1 < ntiles) issue_loads(tile + 1);

    const int j0 = tile * kPBN;
    if (j0 <= wave_row0 + 31) {  // some key of the tile is visible to some row of this wave
      const unsigned char* kt = lds + buf * 2 * kPTileBytes;
      const unsigned char* vt = kt + kPTileBytes;
      // ---- S^T = K . Q^T : two 32-token row tiles
      f32x16 s[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[tt][r] = 0.f;
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) {
          const u32x4 w = *reinterpret_cast<const u32x4*>(kt + ptile_offset(32 * tt + n, 2 * kb + jj));
          s[tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), qb[kb], s[tt], 0, 0, 0);
        }
      }
      // ---- causal mask (only where the tile crosses the diagonal), running max of the raw scores;
      //      the softmax scale is folded into the exponent: p = 2^(s*c - m*c)
      const bool need_mask = j0 + kPBN - 1 > wave_row0;
      float m_loc = -INFINITY;
      if (need_mask) {
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = j0 + 32 * tt + 8 * (r >> 2) + 4 * jj + (r & 3);
            s[tt][r] = key <= my_row ? s[tt][r] : -INFINITY;
          }
      }
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 16; ++r) m_loc = fmaxf(m_loc, s[tt][r]);
      m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32, kWave));
      const float m_new = fmaxf(m_run, m_loc);                  // raw-score domain
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float mc = m_safe * p.scale_log2;
      const float alpha = __builtin_amdgcn_exp2f(m_run * p.scale_log2 - mc);
      float psum = 0.f;
      u32x4 pw[4];  // P^T as B operand for the four 16-token k blocks
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tt][r], p.scale_log2, -mc));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tt][r + 1], p.scale_log2, -mc));
          psum += p0 + p1;
          pw[2 * tt + (r >> 3)][(r & 7) >> 1] = pack_bf16x2(p0, p1);
        }
      l_run = l_run * alpha + psum;
      m_run = m_new;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) acc[dt] *= alpha;
      }
      // ---- O^T += V^T . P^T
      const int grp = lane >> 4;              // 16-lane group: (d half, jj)
      const int src_row = (lane & 15) >> 2;   // token row this lane addresses inside a 4-row set
      const int src_chunk = lane & 3;         // 4-wide d chunk inside the 16-wide window
      const int d_half = grp & 1;
#pragma unroll
      for (int kb2 = 0; kb2 < 4; ++kb2) {
        const bf16x8 pb = __builtin_bit_cast(bf16x8, pw[kb2]);
        const int t_lo = 16 * kb2 + 4 * jj + src_row;
        const int t_hi = t_lo + 8;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          const int d0 = 32 * dt + 16 * d_half + 4 * src_chunk;  // first of 4 consecutive d
          const int slice = d0 >> 3;
          const int sub = (d0 & 7) << 1;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(vt + ptile_offset(t_lo, slice) + sub));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(vt + ptile_offset(t_hi, slice) + sub));
          typedef short s16x8 __attribute__((ext_vector_type(8)));
          const s16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), pb, acc[dt], 0, 0, 0);
        }
      }
    }
  }

  l_run += __shfl_xor(l_run, 32, kWave);
  if (my_row < seq_len) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    uint16_t* orow = p.out + (int64_t)(seq_begin + my_row) * p.o_ts + (int64_t)h * kPD;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        u32x2 w;
        w[0] = pack_bf16x2(acc[dt][4 * rq] * inv, acc[dt][4 * rq + 1] * inv);
        w[1] = pack_bf16x2(acc[dt][4 * rq + 2] * inv, acc[dt][4 * rq + 3] * inv);
        *reinterpret_cast<u32x2*>(orow + 32 * dt + 8 * rq + 4 * jj) = w;
      }
  }
}

}  // namespace mops

extern "C" int mops_hip_attn_varlen_causal_bf16(const void* q, int64_t q_token_stride,
                                                const void* k, int64_t k_token_stride,
                                                const void* v, int64_t v_token_stride,
                                                void* out, int64_t out_token_stride,
                                                const int32_t* cu_seqlens,
                                                int64_t batch, int64_t total_tokens, int64_t max_seqlen,
                                                int64_t hq, int64_t hkv, int64_t head_dim,
                                                float softmax_scale,
                                                void* stream) {
  using namespace mops;
  if (batch < 0 || total_tokens < 0 || max_seqlen < 0 || hq <= 0 || hkv <= 0) return MOPS_HIP_EINVAL;
  if (batch == 0 || total_tokens == 0 || max_seqlen == 0) return MOPS_HIP_OK;
  if (!q || !k || !v || !out || !cu_seqlens) return MOPS_HIP_EINVAL;
  if (hq % hkv != 0) return MOPS_HIP_EINVAL;
  if (head_dim != kPD) return MOPS_HIP_EUNSUPPORTED;
  if (q_token_stride < hq * kPD || out_token_stride < hq * kPD || k_token_stride < hkv * kPD ||
      v_token_stride < hkv * kPD)
    return MOPS_HIP_EINVAL;
  if (total_tokens > 0x3fffffffLL || batch > (1 << 20) || hq > 4096) return MOPS_HIP_EUNSUPPORTED;
  if ((q_token_stride & 7) || (k_token_stride & 7) || (v_token_stride & 7) || (out_token_stride & 3))
    return MOPS_HIP_EALIGN;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return MOPS_HIP_EALIGN;
  if (max_seqlen > total_tokens) max_seqlen = total_tokens;

  PrefillParams p;
  p.q = (const uint16_t*)q;
  p.k = (const uint16_t*)k;
  p.v = (const uint16_t*)v;
  p.out = (uint16_t*)out;
  p.q_ts = q_token_stride;
  p.k_ts = k_token_stride;
  p.v_ts = v_token_stride;
  p.o_ts = out_token_stride;
  p.cu_seqlens = cu_seqlens;
  p.batch = (int)batch;
  p.total_tokens = (int)total_tokens;
  p.m_tiles = (int)((max_seqlen + kPBM - 1) / kPBM);
  p.hq = (int)hq;
  p.hkv = (int)hkv;
  p.group = (int)(hq / hkv);
  p.scale_log2 = softmax_scale * 1.44269504088896340736f;
  const int64_t grid = (int64_t)p.m_tiles * batch * hq;
  if (grid > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL(varlen_prefill_kernel, dim3((unsigned)grid), dim3(kPThreads), 0, (hipStream_t)stream, p);
  return finish_launch();
}
