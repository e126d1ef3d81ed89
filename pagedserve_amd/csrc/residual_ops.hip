// Steps on the float residual stream of layers whose sublayers add into a scratch row y that is
// folded into the stream with a factor, and what mixers that run side by side need.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

// One pass over the stream's rows, every piece optional:
//   h <- h + factor * column_scale * y + bias;   zero <- 0 (may be y);
//   normed <- h / sqrt(mean(h^2) + eps) * gamma
// (column_scale: a float per column, null for ones).  A block per token.
template <typename T>
__global__ __launch_bounds__(256) void stream_step_kernel(
    float* __restrict__ h, const float* y, float factor, const float* __restrict__ column_scale,
    const float* __restrict__ bias, const float* __restrict__ gamma, float eps, T* __restrict__ normed, float* zero, int width) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  float* row = h + t * width;
  float sum = 0.f;
  for (int d = threadIdx.x; d < width; d += blockDim.x) {
    float v = row[d];
    if (y != nullptr) v = fmaf(column_scale ? factor * column_scale[d] : factor, y[t * width + d], v);
    if (bias != nullptr) v += bias[d];
    if (y != nullptr || bias != nullptr) row[d] = v;
    if (zero != nullptr) zero[t * width + d] = 0.f;
    sum = fmaf(v, v, sum);
  }
  if (gamma == nullptr) return;
  const float inv = 1.0f / sqrtf(block_sum(sum, scratch) / (float)width + eps);
  // (each thread reads back what it wrote itself)
  for (int d = threadIdx.x; d < width; d += blockDim.x)
    normed[t * width + d] = from_float<T>(row[d] * inv * gamma[d]);
}

// out[t, c] = act(gu[t, c]) * gu[t, inner + c]; act: silu, or (GELU) the tanh form of gelu
template <typename T, bool GELU>
__global__ __launch_bounds__(256) void silu_gate_kernel(const float* __restrict__ gu, int64_t ld,
                                                        T* __restrict__ out, int64_t out_ld,
                                                        int inner) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= inner) return;
  const float g = gu[t * ld + c];
  const float u = gu[t * ld + inner + c];
  out[t * out_ld + c] = from_float<T>((GELU ? gelu_tanh_f(g) : g / (1.0f + expf(-g))) * u);
}

// p[t, c] <- silu(p[t, c]) for columns first .. first + count - 1 of rows ld floats apart
__global__ __launch_bounds__(256) void silu_columns_kernel(float* __restrict__ p, int64_t ld, int first,
                                                           int count) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= count) return;
  float* at = p + (int64_t)blockIdx.x * ld + first + c;
  const float v = *at;
  *at = v / (1.0f + expf(-v));
}

// y <- y + share * (a / rms(a) * wa + b / rms(b) * wb);  a <- 0;  b <- 0.   A block per token.
__global__ __launch_bounds__(256) void pair_norm_mix_kernel(
    float* __restrict__ a, float* __restrict__ b, const float* __restrict__ wa,
    const float* __restrict__ wb, float eps, float share, float* __restrict__ y, int width) {
  __shared__ float scratch_a[16], scratch_b[16];
  const int64_t t = blockIdx.x;
  float* ra = a + t * width;
  float* rb = b + t * width;
  float sa = 0.f, sb = 0.f;
  for (int d = threadIdx.x; d < width; d += blockDim.x) {
    sa = fmaf(ra[d], ra[d], sa);
    sb = fmaf(rb[d], rb[d], sb);
  }
  const float ia = 1.0f / sqrtf(block_sum(sa, scratch_a) / (float)width + eps);
  const float ib = 1.0f / sqrtf(block_sum(sb, scratch_b) / (float)width + eps);
  for (int d = threadIdx.x; d < width; d += blockDim.x) {
    const float va = ra[d] * ia * wa[d];
    const float vb = rb[d] * ib * wb[d];
    y[t * width + d] += share * (va + vb);
    ra[d] = 0.f;
    rb[d] = 0.f;
  }
}

extern "C" int ps_stream_step(float* h, const float* y, float factor, const float* column_scale,
                              const float* bias, const float* gamma, float eps, void* normed,
                              float* zero, int tokens, int width, int out_dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0, "ps_stream_step: bad sizes");
  PS_REQUIRE(gamma == nullptr || (normed != nullptr && eps > 0.f),
             "ps_stream_step: a norm needs an output and a positive eps");
  PS_REQUIRE(out_dtype == PS_F32 || out_dtype == PS_BF16, "ps_stream_step: unknown dtype %d", out_dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == PS_F32)
    hipLaunchKernelGGL(stream_step_kernel<float>, dim3(tokens), dim3(256), 0, s, h, y, factor,
                       column_scale, bias, gamma, eps, (float*)normed, zero, width);
  else
    hipLaunchKernelGGL(stream_step_kernel<bf16_t>, dim3(tokens), dim3(256), 0, s, h, y, factor,
                       column_scale, bias, gamma, eps, (bf16_t*)normed, zero, width);
  PS_CHECK_LAUNCH("ps_stream_step");
  return 0;
}

extern "C" int ps_silu_gate(const float* gu, int64_t ld, void* out, int64_t out_ld, int tokens,
                            int inner, int activation, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && inner > 0 && ld >= 2 * (int64_t)inner && out_ld >= inner,
             "ps_silu_gate: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_silu_gate: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(tokens, (inner + 255) / 256);
  PS_REQUIRE(activation == 0 || activation == 1, "ps_silu_gate: activation %d (0: silu, 1: gelu_tanh)", activation);
  if (dtype == PS_F32 && activation)
    hipLaunchKernelGGL((silu_gate_kernel<float, true>), grid, dim3(256), 0, s, gu, ld, (float*)out, out_ld, inner);
  else if (dtype == PS_F32)
    hipLaunchKernelGGL((silu_gate_kernel<float, false>), grid, dim3(256), 0, s, gu, ld, (float*)out, out_ld, inner);
  else if (activation)
    hipLaunchKernelGGL((silu_gate_kernel<bf16_t, true>), grid, dim3(256), 0, s, gu, ld, (bf16_t*)out, out_ld, inner);
  else
    hipLaunchKernelGGL((silu_gate_kernel<bf16_t, false>), grid, dim3(256), 0, s, gu, ld, (bf16_t*)out, out_ld, inner);
  PS_CHECK_LAUNCH("ps_silu_gate");
  return 0;
}

extern "C" int ps_silu_columns(float* p, int64_t ld, int first, int count, int tokens, void* stream) {
  PS_REQUIRE(tokens >= 0 && first >= 0 && count > 0 && ld >= first + count, "ps_silu_columns: bad sizes");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(silu_columns_kernel, dim3(tokens, (count + 255) / 256), dim3(256), 0,
                     (hipStream_t)stream, p, ld, first, count);
  PS_CHECK_LAUNCH("ps_silu_columns");
  return 0;
}

extern "C" int ps_pair_norm_mix(float* a, float* b, const float* wa, const float* wb, float eps,
                                float share, float* y, int tokens, int width, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && eps > 0.f, "ps_pair_norm_mix: bad sizes");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(pair_norm_mix_kernel, dim3(tokens), dim3(256), 0, (hipStream_t)stream, a, b, wa,
                     wb, eps, share, y, width);
  PS_CHECK_LAUNCH("ps_pair_norm_mix");
  return 0;
}
