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

// The same value from the hardware's exp2 and reciprocal (a quarter of the instructions), together with whether it can be
// trusted: the fp32 result of this route is within a few units of its last place of the exact route's, so the two round
// to the same bf16 unless the result lies within kSiluMargin units of a rounding midpoint (its low 16 bits near 0x8000).
// Arguments beyond +-8 (where the error of the scaled exponent grows), NaNs and infinities are never trusted.  The kernel
// recomputes untrusted elements with silu_bf16; the test that walks all 65536 bf16 patterns shows the outputs bit-equal.
constexpr unsigned kSiluMargin = 8;
__device__ __forceinline__ float silu_bf16_quick(float x, bool& unsure) {
  const float s = x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
  unsure = ((__float_as_uint(s) + kSiluMargin - 0x8000u) & 0xffffu) < 2u * kSiluMargin || !(fabsf(x) <= 8.0f);
  return round_to_bf16(s);
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
    // silu by the quick route; elements it cannot vouch for (about one in a thousand) are redone by the exact one, one
    // element position at a time and only where some lane of the wave asks for it
    float sv[8];
    unsigned redo = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      bool unsure;
      sv[e] = silu_bf16_quick((e & 1) ? bf16hi_to_f32(a[e >> 1]) : bf16lo_to_f32(a[e >> 1]), unsure);
      redo |= unsure ? 1u << e : 0u;
    }
    if (__any(redo != 0)) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (__any((redo >> e) & 1u)) {
          if ((redo >> e) & 1u) sv[e] = silu_bf16((e & 1) ? bf16hi_to_f32(a[e >> 1]) : bf16lo_to_f32(a[e >> 1]));
        }
    }
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(sv[2 * e] * bf16lo_to_f32(b[e]), sv[2 * e + 1] * bf16hi_to_f32(b[e]));
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

typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

// One workgroup per row, in two passes.  Pass 1 streams the row once and keeps three running values per lane and 16-bit
// half, over the raw bf16 bit patterns: their maximum and minimum as signed integers and their maximum as unsigned ones,
// three packed instructions per two logits (comparing widened values with an index kept beside the maximum took twelve,
// and at this size the kernel was as much instruction- as memory-bound).  Non-negative numbers order like their patterns
// read as signed integers and lie above all negative ones, so a signed maximum >= 0 is the row's maximum; when it is
// negative every logit is, negative numbers order against their patterns, and the signed minimum is the row's maximum.
// The unsigned maximum is the negative pattern of largest magnitude when there is one: above 0xff80 it is a NaN.
// Pass 2 finds the first index of the row maximum: only lanes whose own maximum equals it look again, at the one batch of
// pieces in which their maximum first appeared (noted in pass 1 at the price of a few instructions per batch), which is
// still in the L2.
__device__ __forceinline__ float bits_to_f32(int b) { return __uint_as_float((unsigned)b << 16); }

__global__ __launch_bounds__(kArgmaxThreads) void row_argmax_kernel(const uint16_t* __restrict__ logits, int64_t row_stride,
                                                                   int64_t* __restrict__ out, int n) {
  __shared__ int smax_w[kArgmaxThreads / kWave], smin_w[kArgmaxThreads / kWave], umax_w[kArgmaxThreads / kWave];
  __shared__ int first_i;
  const uint16_t* row = logits + (int64_t)blockIdx.x * row_stride;
  s16x2 smax2 = {(short)-32768, (short)-32768}, smin2 = {(short)32767, (short)32767};
  u16x2 umax2 = {0, 0};
  const int pieces = n >> 3;
  auto take = [&](const u32x4 w) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // (a copy of the element first: a bit cast applied to the vector's element directly reads element 0 whatever e is)
      const uint32_t d = w[e];
      smax2 = __builtin_elementwise_max(smax2, __builtin_bit_cast(s16x2, d));
      smin2 = __builtin_elementwise_min(smin2, __builtin_bit_cast(s16x2, d));
      umax2 = __builtin_elementwise_max(umax2, __builtin_bit_cast(u16x2, d));
    }
  };
  // The lane's maximum so far as a score that grows with the number: the pattern itself when there is a non-negative
  // logit, else below zero and falling with the signed minimum.  `at_pc`, `at_cnt`: the batch in which the score last
  // grew, i.e. in which the lane's maximum first appeared (its first piece, its number of pieces; 0 pieces: the tail).
  int smax = -32768, smin = 32767, score = -0x7fffffff, at_pc = 0, at_cnt = 0;
  auto score_of = [](int mx, int mn) { return mx >= 0 ? mx : -1 - (mn + 32768); };
  auto note = [&](int pc0, int cnt) {
    smax = max((int)smax2[0], (int)smax2[1]);
    smin = min((int)smin2[0], (int)smin2[1]);
    const int sc = score_of(smax, smin);
    if (sc > score) {
      score = sc;
      at_pc = pc0;
      at_cnt = cnt;
    }
  };
  // two loads in flight per lane (four and eight are slower): one workgroup per row leaves the memory system too little to do otherwise
  constexpr int kDeep = 2;
  int pc = threadIdx.x;
  for (; pc + (kDeep - 1) * kArgmaxThreads < pieces; pc += kDeep * kArgmaxThreads) {
    u32x4 w[kDeep];
#pragma unroll
    for (int u = 0; u < kDeep; ++u) w[u] = load16_stream(row + ((int64_t)(pc + u * kArgmaxThreads) << 3));
#pragma unroll
    for (int u = 0; u < kDeep; ++u) take(w[u]);
    note(pc, kDeep);
  }
  for (; pc < pieces; pc += kArgmaxThreads) {
    take(load16_stream(row + ((int64_t)pc << 3)));
    note(pc, 1);
  }
  int umax = max((int)umax2[0], (int)umax2[1]);
  for (int i = (pieces << 3) + threadIdx.x; i < n; i += kArgmaxThreads) {  // tail when n % 8 != 0
    const int x = (int)(short)row[i];
    smax = max(smax, x);
    smin = min(smin, x);
    umax = max(umax, x & 0xffff);
    const int sc = score_of(smax, smin);
    if (sc > score) {
      score = sc;
      at_cnt = 0;
    }
  }
  const int lane_smax = smax, lane_smin = smin;
#pragma unroll
  for (int off = kWave / 2; off >= 1; off >>= 1) {
    smax = max(smax, __shfl_xor(smax, off, kWave));
    smin = min(smin, __shfl_xor(smin, off, kWave));
    umax = max(umax, __shfl_xor(umax, off, kWave));
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    smax_w[threadIdx.x / kWave] = smax;
    smin_w[threadIdx.x / kWave] = smin;
    umax_w[threadIdx.x / kWave] = umax;
  }
  if (threadIdx.x == 0) first_i = 0x7fffffff;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kArgmaxThreads / kWave; ++w) {
    smax = max(smax, smax_w[w]);
    smin = min(smin, smin_w[w]);
    umax = max(umax, umax_w[w]);
  }
  // A NaN or +inf logit turns the whole softmax row into NaN, and so does a row of -inf; the library's argmax of an
  // all-NaN row is 0.  Patterns: +inf 0x7f80, NaNs above it; -inf 0xff80 (-128 as a signed value), NaNs above it.
  const bool spoiled = smax >= 0x7f80 || umax > 0xff80 || (smax < 0 && smin >= -128) || smin > smax;
  if (spoiled) {
    if (threadIdx.x == 0) out[blockIdx.x] = 0;
    return;
  }
  const float gv = bits_to_f32(smax >= 0 ? smax : smin);
  // the lane's own maximum as a number (lanes that read nothing say -inf, which a row that got here does not have as its maximum)
  const float lane_v = lane_smin > lane_smax ? -INFINITY : bits_to_f32(lane_smax >= 0 ? lane_smax : lane_smin);
  // pass 2 (numbers compared as numbers: -0 and +0 tie, the first of them wins, as in the library)
  if (__any(lane_v == gv)) {
    int bi = 0x7fffffff;
    if (lane_v == gv) {
      // -0 and +0 are one number with two patterns: a lane that met -0 first and +0 later noted the later batch, so zeros
      // are looked for from the lane's first piece on
      const bool zero = gv == 0.f;
      const int q0 = zero ? (int)threadIdx.x : at_pc;
      const int q1 = zero ? pieces : (at_cnt == 0 ? 0 : min(pieces, at_pc + at_cnt * kArgmaxThreads));
      for (int q = q0; q < q1 && bi == 0x7fffffff; q += kDeep * kArgmaxThreads) {
        u32x4 w[kDeep];
#pragma unroll
        for (int u = 0; u < kDeep; ++u) {
          const int qq = q + u * kArgmaxThreads;
          w[u] = qq < q1 ? load16(row + ((int64_t)qq << 3)) : u32x4{0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};   // NaNs match nothing
        }
#pragma unroll
        for (int u = kDeep - 1; u >= 0; --u)
#pragma unroll
          for (int e = 3; e >= 0; --e) {
            const int i0 = ((q + u * kArgmaxThreads) << 3) + 2 * e;
            if (bf16hi_to_f32(w[u][e]) == gv) bi = i0 + 1;
            if (bf16lo_to_f32(w[u][e]) == gv) bi = i0;
          }
      }
      if (bi == 0x7fffffff)
        for (int i = (pieces << 3) + threadIdx.x; i < n && bi == 0x7fffffff; i += kArgmaxThreads)
          if (bf16lo_to_f32(row[i]) == gv) bi = i;
    }
#pragma unroll
    for (int off = kWave / 2; off >= 1; off >>= 1) bi = min(bi, __shfl_xor(bi, off, kWave));
    if ((threadIdx.x & (kWave - 1)) == 0) atomicMin(&first_i, bi);
  }
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = first_i == 0x7fffffff ? 0 : first_i;
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
