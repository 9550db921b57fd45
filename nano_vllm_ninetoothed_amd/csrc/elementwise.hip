// siluAndMul and apply_rotary_emb: the two per-layer elementwise operators between the GEMMs and the
// attention kernels.  Both are HBM-bound streams; what matters at decode batch sizes is that each is ONE
// launch instead of a chain of library elementwise kernels.
//
// Rounding follows the reference's torch backend exactly:
//   siluAndMul (mops/torch/ops.py:32-34):  out = bf16( bf16(silu(f32(x))) * y )   — F.silu rounds to bf16
//                                          before the bf16 multiply
//   apply_rotary_emb (ops.py:45-54):       y1 = x1*cos - x2*sin, y2 = x2*cos + x1*sin in fp32 with each
//                                          product rounded on its own (no fused multiply-add), then bf16
#include "mops_common.h"

namespace mops {

constexpr int kEwThreads = 256;

__device__ __forceinline__ float silu_bf16(float x) {
  // x / (1 + exp(-x)) with IEEE divide, rounded to bf16 like the library kernel's output
  return round_to_bf16(x / (1.0f + expf(-x)));
}

__global__ __launch_bounds__(kEwThreads) void silu_and_mul_kernel(
    const uint16_t* __restrict__ x, int64_t x_row_stride, const uint16_t* __restrict__ y, int64_t y_row_stride,
    uint16_t* __restrict__ out, int64_t rows, int n) {
  const int pieces = n >> 3;
  const int64_t total = rows * pieces;
  for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kEwThreads) {
    const int64_t r = i / pieces;
    const int c = (int)(i - r * pieces) << 3;
    const u32x4 a = load16_stream(x + r * x_row_stride + c);
    const u32x4 b = load16_stream(y + r * y_row_stride + c);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = silu_bf16(bf16lo_to_f32(a[e])) * bf16lo_to_f32(b[e]);
      const float hi = silu_bf16(bf16hi_to_f32(a[e])) * bf16hi_to_f32(b[e]);
      o[e] = pack_bf16x2(lo, hi);
    }
    store16_stream(out + r * (int64_t)n + c, o);
  }
}

// One lane rotates 8 pairs (x1[8], x2[8]) of one (token, head): 16 lanes per head at head_dim 128... for
// a general even head_dim, half = head_dim/2 must be a multiple of 8.
__global__ __launch_bounds__(kEwThreads) void rotary_kernel(
    const uint16_t* __restrict__ x, int64_t x_token_stride, int64_t x_head_stride,
    const float* __restrict__ cos, int64_t cos_token_stride, const float* __restrict__ sin, int64_t sin_token_stride,
    uint16_t* __restrict__ out, int64_t tokens, int heads, int half) {
#pragma clang fp contract(off)  // products and sums stay separate roundings, as in the library expression
  const int pieces = half >> 3;                       // 16-byte pieces per half
  const int64_t total = tokens * heads * pieces;
  for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kEwThreads) {
    const int pc = (int)(i % pieces);
    const int64_t th = i / pieces;
    const int hd = (int)(th % heads);
    const int64_t t = th / heads;
    const uint16_t* xp = x + t * x_token_stride + hd * x_head_stride + (pc << 3);
    const u32x4 a = load16(xp);
    const u32x4 b = load16(xp + half);
    const float* cp = cos + t * cos_token_stride + (pc << 3);
    const float* sp = sin + t * sin_token_stride + (pc << 3);
    float c[8], s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      c[e] = cp[e];
      s[e] = sp[e];
    }
    u32x4 o1, o2;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float x1l = bf16lo_to_f32(a[e]), x1h = bf16hi_to_f32(a[e]);
      const float x2l = bf16lo_to_f32(b[e]), x2h = bf16hi_to_f32(b[e]);
      const float y1l = x1l * c[2 * e] - x2l * s[2 * e];
      const float y1h = x1h * c[2 * e + 1] - x2h * s[2 * e + 1];
      const float y2l = x2l * c[2 * e] + x1l * s[2 * e];
      const float y2h = x2h * c[2 * e + 1] + x1h * s[2 * e + 1];
      o1[e] = pack_bf16x2(y1l, y1h);
      o2[e] = pack_bf16x2(y2l, y2h);
    }
    uint16_t* op = out + (t * heads + hd) * (int64_t)(2 * half) + (pc << 3);
    store16(op, o1);
    store16(op + half, o2);
  }
}

static unsigned ew_grid(int64_t total_items) {
  int64_t g = (total_items + kEwThreads - 1) / kEwThreads;
  const int64_t cap = 256 * 16;  // 16 workgroups per CU are plenty for a stream
  if (g > cap) g = cap;
  return (unsigned)(g < 1 ? 1 : g);
}

}  // namespace mops

extern "C" int mops_hip_silu_and_mul(const void* x, int64_t x_row_stride, const void* y, int64_t y_row_stride,
                                     void* out, int64_t rows, int64_t n, void* stream) {
  using namespace mops;
  if (rows < 0 || n <= 0) return MOPS_HIP_EINVAL;
  if (rows == 0) return MOPS_HIP_OK;
  if (!x || !y || !out) return MOPS_HIP_EINVAL;
  if (x_row_stride < n || y_row_stride < n) return MOPS_HIP_EINVAL;
  if (n > (1 << 24)) return MOPS_HIP_EUNSUPPORTED;
  if ((n & 7) || (x_row_stride & 7) || (y_row_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(x) || !aligned16(y) || !aligned16(out)) return MOPS_HIP_EALIGN;
  hipLaunchKernelGGL(silu_and_mul_kernel, dim3(ew_grid(rows * (n >> 3))), dim3(kEwThreads), 0, (hipStream_t)stream,
                     (const uint16_t*)x, x_row_stride, (const uint16_t*)y, y_row_stride, (uint16_t*)out, rows, (int)n);
  return finish_launch();
}

extern "C" int mops_hip_apply_rotary_emb(const void* x, int64_t x_token_stride, int64_t x_head_stride,
                                         const float* cos, int64_t cos_token_stride,
                                         const float* sin, int64_t sin_token_stride,
                                         void* out, int64_t tokens, int64_t heads, int64_t head_dim, void* stream) {
  using namespace mops;
  if (tokens < 0 || heads <= 0 || head_dim <= 0) return MOPS_HIP_EINVAL;
  if (tokens == 0) return MOPS_HIP_OK;
  if (!x || !cos || !sin || !out) return MOPS_HIP_EINVAL;
  if (head_dim % 16 != 0 || head_dim > 1024 || heads > 65536) return MOPS_HIP_EUNSUPPORTED;
  const int64_t half = head_dim / 2;
  if (x_head_stride < head_dim || x_token_stride < heads * head_dim || cos_token_stride < half || sin_token_stride < half)
    return MOPS_HIP_EINVAL;
  if ((x_token_stride & 7) || (x_head_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(x) || !aligned16(out) || (reinterpret_cast<uintptr_t>(cos) & 3u) || (reinterpret_cast<uintptr_t>(sin) & 3u))
    return MOPS_HIP_EALIGN;
  hipLaunchKernelGGL(rotary_kernel, dim3(ew_grid(tokens * heads * (half >> 3))), dim3(kEwThreads), 0, (hipStream_t)stream,
                     (const uint16_t*)x, x_token_stride, x_head_stride, cos, cos_token_stride, sin, sin_token_stride,
                     (uint16_t*)out, tokens, (int)heads, (int)half);
  return finish_launch();
}

// ---------------------------------------------------------------------------------------------------
// sampler_forward: token = argmax(softmax(logits / T)) per row (the reference's sampler is greedy: its
// Gumbel line is commented out, mops/torch/ops.py:37-43).  Dividing by a positive temperature and
// applying softmax are monotonic, so this is the index of the row's largest logit; the first such index
// on ties, as torch.argmax returns.  One workgroup per row streams the row once.
// ---------------------------------------------------------------------------------------------------
namespace mops {

constexpr int kArgmaxThreads = 1024;

__global__ __launch_bounds__(kArgmaxThreads) void row_argmax_kernel(const uint16_t* __restrict__ logits, int64_t row_stride,
                                                                   int64_t* __restrict__ out, int n) {
  __shared__ float best_v[kArgmaxThreads / kWave];
  __shared__ int best_i[kArgmaxThreads / kWave];
  __shared__ int spoiled_w[kArgmaxThreads / kWave];
  const uint16_t* row = logits + (int64_t)blockIdx.x * row_stride;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  // A NaN or +inf logit turns the whole softmax row into NaN, and the library's argmax of an all-NaN row is 0.
  bool spoiled = false;
  const int pieces = n >> 3;
  auto take = [&](const u32x4 w, int pc) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = bf16lo_to_f32(w[e]), hi = bf16hi_to_f32(w[e]);
      const int i0 = (pc << 3) + 2 * e;
      spoiled |= !(lo < INFINITY) || !(hi < INFINITY);
      if (lo > bv) { bv = lo; bi = i0; }        // strictly greater: within a lane indices only grow
      if (hi > bv) { bv = hi; bi = i0 + 1; }
    }
  };
  // four loads in flight per lane (eight are slower again): one workgroup per row leaves the memory system too little to do otherwise
  constexpr int kDeep = 4;
  int pc = threadIdx.x;
  for (; pc + (kDeep - 1) * kArgmaxThreads < pieces; pc += kDeep * kArgmaxThreads) {
    u32x4 w[kDeep];
#pragma unroll
    for (int u = 0; u < kDeep; ++u) w[u] = load16_stream(row + ((int64_t)(pc + u * kArgmaxThreads) << 3));
#pragma unroll
    for (int u = 0; u < kDeep; ++u) take(w[u], pc + u * kArgmaxThreads);
  }
  for (; pc < pieces; pc += kArgmaxThreads) take(load16_stream(row + ((int64_t)pc << 3)), pc);
  for (int i = (pieces << 3) + threadIdx.x; i < n; i += kArgmaxThreads) {  // tail when n % 8 != 0
    const float x = bf16lo_to_f32(row[i]);
    spoiled |= !(x < INFINITY);
    if (x > bv) { bv = x; bi = i; }
  }
  // an all -inf row is all NaN after the softmax as well: bi stays unset and becomes 0 below
#pragma unroll
  for (int off = kWave / 2; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    best_v[threadIdx.x / kWave] = bv;
    best_i[threadIdx.x / kWave] = bi;
  }
  const bool wave_spoiled = __any(spoiled);
  if ((threadIdx.x & (kWave - 1)) == 0) spoiled_w[threadIdx.x / kWave] = wave_spoiled;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxThreads / kWave; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
    bool any_spoiled = false;
    for (int w = 0; w < kArgmaxThreads / kWave; ++w) any_spoiled |= spoiled_w[w] != 0;
    out[blockIdx.x] = (bi == 0x7fffffff || any_spoiled) ? 0 : bi;
  }
}

}  // namespace mops

extern "C" int mops_hip_sampler_argmax(const void* logits, int64_t row_stride, int64_t* out, int64_t rows, int64_t n,
                                       void* stream) {
  using namespace mops;
  if (rows < 0 || n <= 0) return MOPS_HIP_EINVAL;
  if (rows == 0) return MOPS_HIP_OK;
  if (!logits || !out) return MOPS_HIP_EINVAL;
  if (row_stride < n) return MOPS_HIP_EINVAL;
  if (n > 0x7ffffff0LL || rows > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  if ((row_stride & 7) || !aligned16(logits)) return MOPS_HIP_EALIGN;
  hipLaunchKernelGGL(row_argmax_kernel, dim3((unsigned)rows), dim3(kArgmaxThreads), 0, (hipStream_t)stream,
                     (const uint16_t*)logits, row_stride, out, (int)n);
  return finish_launch();
}

// An empty kernel: what a launch costs on this device with nothing to do, as a floor to read the small operators'
// durations against (bench.py --op launch_floor).
namespace mops {
__global__ void launch_floor_kernel() {}
}  // namespace mops

extern "C" int mops_hip_launch_floor(void* stream) {
  hipLaunchKernelGGL(mops::launch_floor_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream);
  return mops::finish_launch();
}
