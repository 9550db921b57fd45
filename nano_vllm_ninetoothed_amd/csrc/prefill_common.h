// Pieces shared by the two varlen prefill kernels: tile geometry, launch parameters, half-wave reductions,
// the tile barrier.
#pragma once
#include "mops_common.h"

namespace mops {

constexpr int kPD = 128;            // head dim
constexpr int kPBM = 128;           // q rows per workgroup
constexpr int kPBN = 64;            // kv tokens per tile
constexpr int kPThreads = 256;
constexpr int kPRow = 256;          // bytes of one K or V row in LDS (128 bf16, no padding)
constexpr int kPTile = kPBN * kPRow;        // 16384: a K or V tile
constexpr int kPKChunk = 4 * kPRow;         // a tile is 16 chunks of 4 rows
constexpr int kPKTile = kPTile;
constexpr int kPAhead = 4;          // LDS operand reads run this many MFMAs ahead of use
constexpr float kLazyLog2 = 8.0f;    // the softmax reference moves when a row maximum outgrows it by this much (base-2 exponent)
constexpr int kPCompactChunks = 4;  // the compact launch handles up to 64 * 4 sequences

struct PrefillParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  int64_t q_ts, k_ts, v_ts, o_ts;  // token strides (elements)
  const int32_t* cu_seqlens;     // query side [batch+1]
  const int32_t* cu_seqlens_k;   // key side [batch+1]; equal to cu_seqlens when there is no cached prefix
  const int32_t* block_table;    // null: k/v are packed [total_k_tokens, hkv, 128]; else they are the paged caches
  int64_t block_table_row_stride;
  int block_size, num_blocks, max_blocks_per_seq;
  int batch, total_tokens, total_k_tokens, m_tiles, hq, hkv, group;
  int compact;   // workgroup ids enumerate only existing (q tile, sequence) pairs
  float scale_log2;
};

// max / sum across the two 32-lane halves of the wave; every lane gets the result
__device__ __forceinline__ float half_swap_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// inclusive prefix sum over the 64 lanes of the wave (row shifts, then the two row broadcasts)
__device__ __forceinline__ int wave_prefix_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
  return v;
}

// max of three; the compiler fuses the nested form into one v_max3_f32.  It has to stay a compiler-visible
// operation: the wait states between an MFMA and the first VALU read of its result are inserted by the
// compiler's hazard recognizer, which does not look inside inline assembly.
__device__ __forceinline__ float max3(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }
// workgroup barrier once this wave's LDS traffic is done and its loads into LDS have landed: what it publishes is the next tile
__device__ __forceinline__ void tile_barrier() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// the form of the kernel that packs the two query heads of a kv head into one wave (varlen_prefill_pair.hip);
// returns a status, or MOPS_HIP_EUNSUPPORTED without launching when the problem is outside what it handles
int launch_prefill_pair(const PrefillParams& p, hipStream_t stream);

}  // namespace mops
