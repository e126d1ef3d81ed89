// Differential attention, the step behind the attention kernels.  Every head runs two softmax
// maps over the same values (two heads of queries to the attention kernels: map m of head h is
// their head `m * heads + h`, or `2 * h + m`); here the second map is taken off the
// first, the head's difference is divided by its root mean square (no weight), scaled by a
// constant and, where the layer has one, multiplied element by element with the sigmoid of a
// gate that was projected from the layer's input:
//
//   o = a0 - lambda a1,   out = o / sqrt(mean(o^2) + eps) * factor * sigmoid(g)
//
// over the head's `value_dim` values.  The difference, the norm and the sigmoid are 32-bit.
// A wave per (token, head); a lane owns the values lane, lane + 64, ... (value_dim <= 256).
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

template <typename T>
__global__ __launch_bounds__(256) void differential_combine_kernel(
    const T* __restrict__ ctx, int64_t ctx_ld, const float* __restrict__ lambda, float factor,
    float eps, const float* __restrict__ gate, int64_t gate_ld, T* __restrict__ out, int64_t out_ld,
    int tokens, int heads, int value_dim, int cache_dim, int map_major) {
  const int lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= (int64_t)tokens * heads) return;
  const int64_t t = pair / heads;
  const int head = (int)(pair - t * heads);
  const T* first = ctx + t * ctx_ld + (int64_t)(map_major ? head : 2 * head) * cache_dim;
  const T* second = ctx + t * ctx_ld + (int64_t)(map_major ? heads + head : 2 * head + 1) * cache_dim;
  const float l = lambda[0];
  float o[4];
  float squares = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    o[i] = d < value_dim ? to_float<T>(first[d]) - l * to_float<T>(second[d]) : 0.f;
    squares = fmaf(o[i], o[i], squares);
  }
  const float scale = factor / sqrtf(wave_sum(squares) / (float)value_dim + eps);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d >= value_dim) continue;
    float v = o[i] * scale;
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[t * gate_ld + (int64_t)head * value_dim + d]));
    out[t * out_ld + (int64_t)head * value_dim + d] = from_float<T>(v);
  }
}

// The same step for decoded tokens, straight from the records that the split-KV kernels leave
// per (token, head, key range): [head_dim accumulators | running maximum in units of log 2 | sum].
// A wave per (token, head) merges the ranges of both maps in float (out_m = sum_s acc_s 2^(m_s - M)
// / sum_s l_s 2^(m_s - M)), takes the difference, norms, scales and gates: the maps never pass
// through the storage type, and the launch that merges ranges is this one.
template <typename T>
__global__ __launch_bounds__(64) void differential_merge_kernel(
    const float* __restrict__ partial, const int* __restrict__ tok_list,
    const float* __restrict__ lambda, float factor, float eps, const float* __restrict__ gate,
    int64_t gate_ld, T* __restrict__ out, int64_t out_ld, int heads, int head_dim, int value_dim,
    int splits, int map_major) {
  const int n = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int64_t t = tok_list ? tok_list[n] : n;
  const int stride = head_dim + 2;
  float merged[2][4];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    const int seen = map_major ? m * heads + head : 2 * head + m;
    const float* src = partial + ((int64_t)n * 2 * heads + seen) * splits * stride;
    const float m_s = lane < splits ? src[lane * stride + head_dim] : -INFINITY;
    const float l_s = lane < splits ? src[lane * stride + head_dim + 1] : 0.f;
    const float total_m = wave_max(m_s);
    const float weight = (m_s == -INFINITY) ? 0.f : exp2f(m_s - total_m);
    const float total_l = wave_sum(l_s * weight);
    // (eight ranges' values of all of a lane's dimensions are asked for at once: a merge of many
    // ranges is a few trips to memory, not one per range)
    float value[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 8) {
      float part[4][8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int d = k * 64 + lane;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          part[k][j] = (d < value_dim && s0 + j < splits) ? src[(s0 + j) * stride + d] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float w = __shfl(weight, (s0 + j) & 63, 64);
#pragma unroll
        for (int k = 0; k < 4; ++k) value[k] = fmaf(part[k][j], w, value[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) merged[m][k] = value[k] / total_l;
  }
  const float l = lambda[0];
  float o[4];
  float squares = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    o[k] = k * 64 + lane < value_dim ? merged[0][k] - l * merged[1][k] : 0.f;
    squares = fmaf(o[k], o[k], squares);
  }
  const float scale = factor / sqrtf(wave_sum(squares) / (float)value_dim + eps);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int d = k * 64 + lane;
    if (d >= value_dim) continue;
    float v = o[k] * scale;
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[t * gate_ld + (int64_t)head * value_dim + d]));
    out[t * out_ld + (int64_t)head * value_dim + d] = from_float<T>(v);
  }
}

extern "C" int ps_differential_merge(const float* partial, int64_t partial_floats, const int* tok_list,
                                     int count, const float* lambda, float factor, float eps,
                                     const float* gate, int64_t gate_ld, void* out, int64_t out_ld,
                                     int heads, int head_dim, int value_dim, int splits, int map_major,
                                     int dtype, void* stream) {
  PS_REQUIRE(count >= 0 && heads > 0 && heads <= 65535 && splits >= 1 && splits <= 64,
             "ps_differential_merge: bad sizes");
  PS_REQUIRE(value_dim > 0 && value_dim <= 256 && head_dim >= value_dim,
             "ps_differential_merge: heads of %d values cached %d wide (1..256)", value_dim, head_dim);
  PS_REQUIRE(partial != nullptr &&
                 partial_floats >= (int64_t)count * 2 * heads * splits * (head_dim + 2),
             "ps_differential_merge: too few records");
  PS_REQUIRE(out_ld >= (int64_t)heads * value_dim && (gate == nullptr || gate_ld >= (int64_t)heads * value_dim),
             "ps_differential_merge: rows too short");
  PS_REQUIRE(lambda != nullptr && eps > 0.f, "ps_differential_merge: lambda and a positive eps needed");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_differential_merge: unknown dtype %d", dtype);
  if (count == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(differential_merge_kernel<float>, dim3(count, heads), dim3(64), 0, s, partial, tok_list,
                       lambda, factor, eps, gate, gate_ld, (float*)out, out_ld, heads, head_dim, value_dim,
                       splits, map_major);
  else
    hipLaunchKernelGGL(differential_merge_kernel<bf16_t>, dim3(count, heads), dim3(64), 0, s, partial, tok_list,
                       lambda, factor, eps, gate, gate_ld, (bf16_t*)out, out_ld, heads, head_dim, value_dim,
                       splits, map_major);
  PS_CHECK_LAUNCH("ps_differential_merge");
  return 0;
}

extern "C" int ps_differential_combine(const void* ctx, int64_t ctx_ld, const float* lambda,
                                       float factor, float eps, const float* gate, int64_t gate_ld,
                                       void* out, int64_t out_ld, int tokens, int heads,
                                       int value_dim, int cache_dim, int map_major, int dtype,
                                       void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && value_dim > 0 && value_dim <= 256 && cache_dim >= value_dim,
             "ps_differential_combine: heads of %d values cached %d wide (1..256)", value_dim, cache_dim);
  PS_REQUIRE(ctx_ld >= 2 * (int64_t)heads * cache_dim && out_ld >= (int64_t)heads * value_dim,
             "ps_differential_combine: rows too short");
  PS_REQUIRE(gate == nullptr || gate_ld >= (int64_t)heads * value_dim,
             "ps_differential_combine: gate rows too short");
  PS_REQUIRE(lambda != nullptr && eps > 0.f, "ps_differential_combine: lambda and a positive eps needed");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_differential_combine: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)(((int64_t)tokens * heads + 3) / 4));
  if (dtype == PS_F32)
    hipLaunchKernelGGL(differential_combine_kernel<float>, grid, dim3(256), 0, s, (const float*)ctx,
                       ctx_ld, lambda, factor, eps, gate, gate_ld, (float*)out, out_ld, tokens, heads,
                       value_dim, cache_dim, map_major);
  else
    hipLaunchKernelGGL(differential_combine_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)ctx,
                       ctx_ld, lambda, factor, eps, gate, gate_ld, (bf16_t*)out, out_ld, tokens, heads,
                       value_dim, cache_dim, map_major);
  PS_CHECK_LAUNCH("ps_differential_combine");
  return 0;
}
