// Fused per-head RMSNorm(q), RMSNorm(k), rotary embedding of both, and the scatter of k and v into the
// paged KV cache: the four small kernels that sit between the qkv projection and the attention call of a
// Qwen3 layer (nanovllm/models/qwen3.py:74-80, layers/rotary_embedding.py:27-37, layers/attention.py:29-31
// of the reference) as one launch.  In a decode step those launches cost more than the work they do.
//
// The arithmetic repeats the separate kernels step by step, including their roundings, so the result is
// bit-identical to rms_forward -> apply_rotary_emb -> store_kvcache run one after the other:
//   n   = bf16( bf16(x * rstd) * w )            rstd = 1/sqrt(mean(x^2) + eps), per head, fp32 statistics
//   y1  = bf16( n1 * cos - n2 * sin )           n1, n2 the two halves of the head, products and sums rounded separately
//   y2  = bf16( n2 * cos + n1 * sin )
// Sixteen lanes own one (token, head) row of 128 elements, one 16-byte piece each; lane p and lane p ^ 8
// hold the two halves of the same rotary pairs and swap their normalised pieces.
#include "mops_common.h"

namespace mops {

constexpr int kFusedThreads = 256;
constexpr int kFusedDim = 128;

__global__ __launch_bounds__(kFusedThreads) void qk_norm_rope_store_kernel(
    const uint16_t* __restrict__ qkv, int64_t qkv_token_stride, const uint16_t* __restrict__ q_weight,
    const uint16_t* __restrict__ k_weight, const float* __restrict__ cos, int64_t cos_token_stride,
    const float* __restrict__ sin, int64_t sin_token_stride, const int32_t* __restrict__ slot_mapping,
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out, uint16_t* __restrict__ k_cache,
    uint16_t* __restrict__ v_cache, int64_t tokens, int hq, int hkv, int64_t num_slots, float eps) {
  const int heads = hq + 2 * hkv;
  const int lane = threadIdx.x & 15;
  const int64_t row = (int64_t)blockIdx.x * (kFusedThreads / 16) + (threadIdx.x >> 4);
  const bool row_ok = row < tokens * heads;
  const int64_t t = row_ok ? row / heads : 0;
  const int hd = row_ok ? (int)(row % heads) : 0;
  const uint16_t* xp = qkv + t * qkv_token_stride + (int64_t)hd * kFusedDim + (lane << 3);
  u32x4 a = {0u, 0u, 0u, 0u};
  if (row_ok) a = load16_stream(xp);
  // Everything else the row needs is requested here as well, in front of the reduction and not behind it: the norm
  // weight, the token's cos / sin, its cache slot.  At decode sizes the kernel lives a few microseconds, and each
  // further trip to memory behind the statistics was a third of that.
  const bool is_q = hd < hq;
  const bool is_v = hd >= hq + hkv;
  int slot = -1;
  if (row_ok && !is_q) slot = slot_mapping[t];
  u32x4 w = {0u, 0u, 0u, 0u};
  f32x4 cv[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, sv[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  if (!is_v) {
    w = load16((is_q ? q_weight : k_weight) + (lane << 3));
    const float* cp = cos + t * cos_token_stride + ((lane & 7) << 3);
    const float* sp = sin + t * sin_token_stride + ((lane & 7) << 3);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      cv[h] = *reinterpret_cast<const f32x4*>(cp + 4 * h);
      sv[h] = *reinterpret_cast<const f32x4*>(sp + 4 * h);
    }
  }

  if (is_v) {   // a v head: straight into the cache
    if (row_ok) {
      if (slot >= 0 && slot < num_slots)
        store16(v_cache + ((int64_t)slot * hkv + (hd - hq - hkv)) * kFusedDim + (lane << 3), a);
    }
    return;   // rows of one head type fill whole 16-lane groups, so the shuffles below never miss a lane
  }

  // ---- RMSNorm, as rmsnorm_kernel<16, 1, false>
  float v[8];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = bf16lo_to_f32(a[e]), hi = bf16hi_to_f32(a[e]);
    v[2 * e] = lo;
    v[2 * e + 1] = hi;
    ss += lo * lo;
    ss += hi * hi;
  }
  ss = group_sum<16>(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)kFusedDim + eps);
  u32x4 nrm;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = round_to_bf16(v[2 * e] * rstd) * bf16lo_to_f32(w[e]);
    const float hi = round_to_bf16(v[2 * e + 1] * rstd) * bf16hi_to_f32(w[e]);
    nrm[e] = pack_bf16x2(lo, hi);
  }

  // ---- rotary, as rotary_kernel: lanes 0..7 hold x1 pieces, lanes 8..15 the matching x2 pieces
  u32x4 other;
#pragma unroll
  for (int e = 0; e < 4; ++e) other[e] = __float_as_uint(row_rotate<8>(__uint_as_float(nrm[e])));   // lane ^ 8 is 8 places around the row of 16
  const bool upper = lane >= 8;
  u32x4 o;
  {
#pragma clang fp contract(off)  // products and sums stay separate roundings, as in the library expression
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float c0 = cv[e >> 1][2 * (e & 1)], c1 = cv[e >> 1][2 * (e & 1) + 1], s0 = sv[e >> 1][2 * (e & 1)], s1 = sv[e >> 1][2 * (e & 1) + 1];
      const float ml = bf16lo_to_f32(nrm[e]), mh = bf16hi_to_f32(nrm[e]);       // this lane's half
      const float ol = bf16lo_to_f32(other[e]), oh = bf16hi_to_f32(other[e]);   // the partner's half
      float yl, yh;
      if (!upper) {   // y1 = x1 * cos - x2 * sin
        yl = ml * c0 - ol * s0;
        yh = mh * c1 - oh * s1;
      } else {        // y2 = x2 * cos + x1 * sin
        yl = ml * c0 + ol * s0;
        yh = mh * c1 + oh * s1;
      }
      o[e] = pack_bf16x2(yl, yh);
    }
  }
  if (!row_ok) return;
  if (is_q) {
    store16(q_out + (t * hq + hd) * (int64_t)kFusedDim + (lane << 3), o);
  } else {
    const int kh = hd - hq;
    if (k_out) store16(k_out + (t * hkv + kh) * (int64_t)kFusedDim + (lane << 3), o);
    if (slot >= 0 && slot < num_slots) store16(k_cache + ((int64_t)slot * hkv + kh) * kFusedDim + (lane << 3), o);
  }
}

}  // namespace mops

extern "C" int mops_hip_qk_norm_rope_store(const void* qkv, int64_t qkv_token_stride, const void* q_weight,
                                           const void* k_weight, const float* cos, int64_t cos_token_stride,
                                           const float* sin, int64_t sin_token_stride,
                                           const int32_t* slot_mapping, void* q_out, void* k_out, void* k_cache,
                                           void* v_cache, int64_t tokens, int64_t hq, int64_t hkv, int64_t head_dim,
                                           int64_t num_slots, float eps, void* stream) {
  using namespace mops;
  if (tokens < 0 || hq <= 0 || hkv <= 0 || num_slots < 0) return MOPS_HIP_EINVAL;
  if (head_dim != kFusedDim) return MOPS_HIP_EUNSUPPORTED;
  if (tokens == 0) return MOPS_HIP_OK;
  if (!qkv || !q_weight || !k_weight || !cos || !sin || !slot_mapping || !q_out || !k_cache || !v_cache) return MOPS_HIP_EINVAL;
  const int64_t heads = hq + 2 * hkv;
  if (qkv_token_stride < heads * kFusedDim || cos_token_stride < kFusedDim / 2 || sin_token_stride < kFusedDim / 2)
    return MOPS_HIP_EINVAL;
  if (qkv_token_stride & 7) return MOPS_HIP_EALIGN;
  if (!aligned16(qkv) || !aligned16(q_weight) || !aligned16(k_weight) || !aligned16(q_out) || (k_out && !aligned16(k_out)) ||
      !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(cos) || !aligned16(sin) || (cos_token_stride & 3) || (sin_token_stride & 3))
    return MOPS_HIP_EALIGN;   // cos / sin are read as 16-byte pieces
  if (heads > 4096 || tokens > (int64_t)1 << 40 || num_slots * hkv > ((int64_t)1 << 40)) return MOPS_HIP_EUNSUPPORTED;
  const int64_t rows = tokens * heads;
  const int64_t grid = (rows + kFusedThreads / 16 - 1) / (kFusedThreads / 16);
  if (grid > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  hipLaunchKernelGGL(qk_norm_rope_store_kernel, dim3((unsigned)grid), dim3(kFusedThreads), 0, (hipStream_t)stream,
                     (const uint16_t*)qkv, qkv_token_stride, (const uint16_t*)q_weight, (const uint16_t*)k_weight, cos,
                     cos_token_stride, sin, sin_token_stride, slot_mapping, (uint16_t*)q_out, (uint16_t*)k_out,
                     (uint16_t*)k_cache, (uint16_t*)v_cache, tokens, (int)hq, (int)hkv, num_slots, eps);
  return finish_launch();
}
