// rms_forward / add_rms_forward: one-pass row normalisation, the row held in registers between the
// statistics pass and the scaling pass so every element is read from HBM exactly once.
//
// Rounding order follows mops/torch/ops.py:9-30 of the reference:
//   rms_forward:      y = bf16( bf16(x * rstd) * w )                       rstd = 1/sqrt(mean(x^2)+eps)
//   add_rms_forward:  s = f32(x) + f32(r);  r_out = bf16(s);  y = bf16( bf16(s * rstd) * w )
//                     with the statistics taken on the unrounded fp32 s.
//
// A row of n elements is owned by GROUP consecutive lanes (16, 64 or 256), each lane keeping up to
// ITERS 16-byte pieces.  GROUP <= 64 reduces with wave shuffles only; GROUP == 256 is one workgroup
// per row and finishes the reduction through LDS.
#include "mops_common.h"

namespace mops {

constexpr int kNormThreads = 256;

template <int GROUP, int ITERS, bool FUSE_ADD>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual,
    const uint16_t* __restrict__ weight, uint16_t* __restrict__ y, uint16_t* __restrict__ residual_out,
    int64_t rows, int64_t rows_inner, int n, int64_t x_stride_outer, int64_t x_stride_inner,
    int64_t r_row_stride, float eps) {
  constexpr int kRowsPerWg = kNormThreads / GROUP;
  const int lane = threadIdx.x % GROUP;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + threadIdx.x / GROUP;
  const bool row_ok = row < rows;
  const int pieces = n >> 3;

  const int64_t ro = row_ok ? row / rows_inner : 0;
  const int64_t ri = row_ok ? row % rows_inner : 0;
  const uint16_t* xr = x + ro * x_stride_outer + ri * x_stride_inner;
  const uint16_t* rr = FUSE_ADD ? residual + (row_ok ? row : 0) * r_row_stride : nullptr;

  float v[ITERS][8];
  u32x4 wv[ITERS];   // the weight pieces are requested together with the row, not behind the reduction: at decode
                     // sizes the kernel's whole life is a few microseconds and a second trip to memory is a third of it
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int p = lane + it * GROUP;
    const bool ok = row_ok && p < pieces;
    u32x4 a = {0u, 0u, 0u, 0u}, b = {0u, 0u, 0u, 0u};
    wv[it] = u32x4{0u, 0u, 0u, 0u};
    if (ok) {
      a = load16_stream(xr + (p << 3));
      if (FUSE_ADD) b = load16_stream(rr + (p << 3));
      wv[it] = load16(weight + (p << 3));
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float lo = bf16lo_to_f32(a[e]), hi = bf16hi_to_f32(a[e]);
      if (FUSE_ADD) {
        lo += bf16lo_to_f32(b[e]);
        hi += bf16hi_to_f32(b[e]);
      }
      v[it][2 * e] = lo;
      v[it][2 * e + 1] = hi;
      ss += lo * lo;
      ss += hi * hi;
    }
    if (FUSE_ADD && ok) {
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(v[it][2 * e], v[it][2 * e + 1]);
      store16_stream(residual_out + row * (int64_t)n + (p << 3), o);
    }
  }

  if (GROUP <= kWave) {
    ss = group_sum<(GROUP <= kWave ? GROUP : kWave)>(ss);
  } else {
    __shared__ float partial[kNormThreads / kWave];
    ss = group_sum<kWave>(ss);
    if ((threadIdx.x & (kWave - 1)) == 0) partial[threadIdx.x / kWave] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int w = 0; w < kNormThreads / kWave; ++w) ss += partial[w];
  }
  const float rstd = 1.0f / sqrtf(ss / (float)n + eps);

#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int p = lane + it * GROUP;
    if (row_ok && p < pieces) {
      const u32x4 w = wv[it];
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = round_to_bf16(v[it][2 * e] * rstd) * bf16lo_to_f32(w[e]);
        const float hi = round_to_bf16(v[it][2 * e + 1] * rstd) * bf16hi_to_f32(w[e]);
        o[e] = pack_bf16x2(lo, hi);
      }
      store16_stream(y + row * (int64_t)n + (p << 3), o);
    }
  }
}

template <bool FUSE_ADD>
static int launch_rmsnorm(const void* x, const void* residual, const void* weight, void* y,
                          void* residual_out, int64_t rows, int64_t rows_inner, int64_t n,
                          int64_t x_stride_outer, int64_t x_stride_inner, int64_t r_row_stride,
                          float eps, void* stream) {
  const int64_t pieces = n >> 3;
#define MOPS_NORM_LAUNCH(G, I)                                                                     \
  do {                                                                                             \
    const int64_t per_wg = kNormThreads / (G);                                                     \
    const int64_t grid = (rows + per_wg - 1) / per_wg;                                             \
    if (grid > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;                                         \
    hipLaunchKernelGGL((rmsnorm_kernel<G, I, FUSE_ADD>), dim3((unsigned)grid), dim3(kNormThreads), \
                       0, (hipStream_t)stream, (const uint16_t*)x, (const uint16_t*)residual,      \
                       (const uint16_t*)weight, (uint16_t*)y, (uint16_t*)residual_out, rows,       \
                       rows_inner, (int)n, x_stride_outer, x_stride_inner, r_row_stride, eps);     \
  } while (0)
  if (pieces <= 16) MOPS_NORM_LAUNCH(16, 1);
  else if (pieces <= 64) MOPS_NORM_LAUNCH(64, 1);
  else if (pieces <= 128) MOPS_NORM_LAUNCH(64, 2);
  else if (pieces <= 256) MOPS_NORM_LAUNCH(256, 1);
  else if (pieces <= 512) MOPS_NORM_LAUNCH(256, 2);
  else if (pieces <= 1024) MOPS_NORM_LAUNCH(256, 4);
  else MOPS_NORM_LAUNCH(256, 8);
#undef MOPS_NORM_LAUNCH
  return finish_launch();
}

}  // namespace mops

extern "C" int mops_hip_rms_forward(const void* x, const void* weight, void* y,
                                    int64_t rows_outer, int64_t rows_inner, int64_t n,
                                    int64_t stride_outer, int64_t stride_inner,
                                    float eps, void* stream) {
  using namespace mops;
  if (rows_outer < 0 || rows_inner < 0 || n <= 0) return MOPS_HIP_EINVAL;
  const int64_t rows = rows_outer * rows_inner;
  if (rows == 0) return MOPS_HIP_OK;
  if (!x || !weight || !y) return MOPS_HIP_EINVAL;
  if (stride_outer < 0 || stride_inner < 0) return MOPS_HIP_EINVAL;
  if (n > 16384) return MOPS_HIP_EUNSUPPORTED;
  if ((n & 7) || (stride_outer & 7) || (stride_inner & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(y)) return MOPS_HIP_EALIGN;
  return launch_rmsnorm<false>(x, nullptr, weight, y, nullptr, rows, rows_inner, n, stride_outer,
                               stride_inner, 0, eps, stream);
}

extern "C" int mops_hip_add_rms_forward(const void* x, int64_t x_row_stride,
                                        const void* residual, int64_t residual_row_stride,
                                        const void* weight,
                                        void* y, void* residual_out,
                                        int64_t rows, int64_t n,
                                        float eps, void* stream) {
  using namespace mops;
  if (rows < 0 || n <= 0) return MOPS_HIP_EINVAL;
  if (rows == 0) return MOPS_HIP_OK;
  if (!x || !residual || !weight || !y || !residual_out) return MOPS_HIP_EINVAL;
  if (x_row_stride < n || residual_row_stride < n) return MOPS_HIP_EINVAL;
  if (y == x || y == residual || y == residual_out) return MOPS_HIP_EINVAL;
  if (residual_out == residual && residual_row_stride != n) return MOPS_HIP_EINVAL;
  if (n > 16384) return MOPS_HIP_EUNSUPPORTED;
  if ((n & 7) || (x_row_stride & 7) || (residual_row_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(x) || !aligned16(residual) || !aligned16(weight) || !aligned16(y) ||
      !aligned16(residual_out))
    return MOPS_HIP_EALIGN;
  return launch_rmsnorm<true>(x, residual, weight, y, residual_out, rows, 1, n, x_row_stride, 0,
                              residual_row_stride, eps, stream);
}
