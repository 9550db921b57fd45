// store_kvcache: slot_mapping scatter of K and V rows into the paged cache (HBM-bound copy).
// Semantics follow mops/triton/attention.py:18-38 of the reference: one row of num_kv_heads*head_dim
// elements per token, skipped when the slot is -1, source row stride honoured.
//
// One 256-thread workgroup moves TOKENS_PER_WG tokens; each thread moves 16-byte pieces, K pieces
// first and V pieces after them, so a 2 KiB K row + 2 KiB V row is exactly one piece per thread.
#include "mops_common.h"

namespace mops {

constexpr int kStoreThreads = 256;
constexpr int kStoreTokensPerWg = 2;

__global__ __launch_bounds__(kStoreThreads) void store_kvcache_kernel(
    const uint16_t* __restrict__ key, int64_t key_row_stride,
    const uint16_t* __restrict__ value, int64_t value_row_stride,
    uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
    const int32_t* __restrict__ slot_mapping,
    int64_t n_tokens, int row_elems, int64_t num_slots) {
  const int pieces_per_row = row_elems >> 3;  // 16-byte pieces
  const int pieces = 2 * pieces_per_row;
#pragma unroll
  for (int t = 0; t < kStoreTokensPerWg; ++t) {
    const int64_t tok = (int64_t)blockIdx.x * kStoreTokensPerWg + t;
    if (tok >= n_tokens) return;
    const int64_t slot = slot_mapping[tok];
    if (slot < 0 || slot >= num_slots) continue;
    for (int p = threadIdx.x; p < pieces; p += kStoreThreads) {
      const bool is_v = p >= pieces_per_row;
      const int col = (is_v ? p - pieces_per_row : p) << 3;
      const uint16_t* src = is_v ? value + tok * value_row_stride : key + tok * key_row_stride;
      uint16_t* dst = (is_v ? v_cache : k_cache) + slot * (int64_t)row_elems;
      store16(dst + col, load16_stream(src + col));
    }
  }
}

}  // namespace mops

extern "C" int mops_hip_store_kvcache(const void* key, int64_t key_row_stride,
                                      const void* value, int64_t value_row_stride,
                                      void* k_cache, void* v_cache,
                                      const int32_t* slot_mapping,
                                      int64_t n_tokens, int64_t row_elems, int64_t num_slots,
                                      void* stream) {
  using namespace mops;
  if (n_tokens < 0 || row_elems <= 0 || num_slots < 0) return MOPS_HIP_EINVAL;
  if (n_tokens == 0) return MOPS_HIP_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping) return MOPS_HIP_EINVAL;
  if (key_row_stride < row_elems || value_row_stride < row_elems) return MOPS_HIP_EINVAL;
  if (row_elems > (1 << 20)) return MOPS_HIP_EUNSUPPORTED;
  if ((row_elems & 7) || (key_row_stride & 7) || (value_row_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(key) || !aligned16(value) || !aligned16(k_cache) || !aligned16(v_cache))
    return MOPS_HIP_EALIGN;
  const int64_t grid = (n_tokens + kStoreTokensPerWg - 1) / kStoreTokensPerWg;
  if (grid > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL(store_kvcache_kernel, dim3((unsigned)grid), dim3(kStoreThreads), 0,
                     (hipStream_t)stream,
                     (const uint16_t*)key, key_row_stride, (const uint16_t*)value, value_row_stride,
                     (uint16_t*)k_cache, (uint16_t*)v_cache, slot_mapping, n_tokens, (int)row_elems,
                     num_slots);
  return finish_launch();
}
