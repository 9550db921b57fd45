// embedding: out[i, :] = weight[ids[i], :] — a row gather (HBM-bound copy), 16 bytes per lane.
// Semantics follow mops/torch/ops.py:57-59 (F.embedding); ids may be int32 or int64
// (nanovllm/engine/model_runner.py:156 hands int64).
#include "mops_common.h"

namespace mops {

constexpr int kEmbThreads = 256;

template <typename IdT>
__global__ __launch_bounds__(kEmbThreads) void embedding_kernel(
    const IdT* __restrict__ ids, const uint16_t* __restrict__ weight, int64_t weight_row_stride,
    uint16_t* __restrict__ out, int64_t n_ids, int64_t vocab, int hidden, int lanes_per_row) {
  // lanes_per_row is a power of two <= 256: narrow rows share a workgroup, wide rows loop.
  const int rows_per_wg = kEmbThreads / lanes_per_row;
  const int lane = threadIdx.x % lanes_per_row;
  const int64_t row = (int64_t)blockIdx.x * rows_per_wg + threadIdx.x / lanes_per_row;
  if (row >= n_ids) return;
  const int pieces = hidden >> 3;
  const int64_t id = (int64_t)ids[row];
  const bool ok = id >= 0 && id < vocab;
  const uint16_t* src = weight + (ok ? id : 0) * weight_row_stride;
  uint16_t* dst = out + row * (int64_t)hidden;
  for (int p = lane; p < pieces; p += lanes_per_row) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (ok) v = load16(src + (p << 3));
    store16_stream(dst + (p << 3), v);
  }
}

}  // namespace mops

extern "C" int mops_hip_embedding(const void* ids, int ids_are_int64,
                                  const void* weight, int64_t weight_row_stride,
                                  void* out,
                                  int64_t n_ids, int64_t vocab, int64_t hidden,
                                  void* stream) {
  using namespace mops;
  if (n_ids < 0 || vocab <= 0 || hidden <= 0) return MOPS_HIP_EINVAL;
  if (n_ids == 0) return MOPS_HIP_OK;
  if (!ids || !weight || !out) return MOPS_HIP_EINVAL;
  if (weight_row_stride < hidden) return MOPS_HIP_EINVAL;
  if (hidden > (1 << 20)) return MOPS_HIP_EUNSUPPORTED;
  if ((hidden & 7) || (weight_row_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(weight) || !aligned16(out)) return MOPS_HIP_EALIGN;
  const int64_t pieces = hidden >> 3;
  int lanes_per_row = 16;
  while (lanes_per_row < kEmbThreads && lanes_per_row < pieces) lanes_per_row <<= 1;
  const int rows_per_wg = kEmbThreads / lanes_per_row;
  const int64_t grid = (n_ids + rows_per_wg - 1) / rows_per_wg;
  if (grid > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  if (ids_are_int64) {
    hipLaunchKernelGGL(embedding_kernel<int64_t>, dim3((unsigned)grid), dim3(kEmbThreads), 0,
                       (hipStream_t)stream, (const int64_t*)ids, (const uint16_t*)weight,
                       weight_row_stride, (uint16_t*)out, n_ids, vocab, (int)hidden, lanes_per_row);
  } else {
    hipLaunchKernelGGL(embedding_kernel<int32_t>, dim3((unsigned)grid), dim3(kEmbThreads), 0,
                       (hipStream_t)stream, (const int32_t*)ids, (const uint16_t*)weight,
                       weight_row_stride, (uint16_t*)out, n_ids, vocab, (int)hidden, lanes_per_row);
  }
  return finish_launch();
}
