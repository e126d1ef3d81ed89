// A product with a block-diagonal matrix: `blocks` small matrices w[b] ([n, k], stored [out, in])
// that each read their own columns of a row and write their own columns of the result,
//
//   out[t, b * out_step + j] = (sum_i x[t, b * x_step + i] * w[b, j, i] + bias[b * n + j])
//                              * (gate ? sigmoid(gate[t * gate_ld + b * n + j]) : 1)
//
// (gates of a recurrence that are computed block by block; the per-head matrices of latent
// attention, which take a head's columns of the queries or of the attention's result).  The
// rows may be float or of the storage type on either side; sums are 32-bit.
//
// A block of 256 threads takes 16 tokens x 64 output columns of one matrix: the tokens' inputs
// and the matrix's rows pass through LDS in pieces of 32 along k, a thread owns one column for
// four tokens.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define BL_TOKENS 16
#define BL_COLS 64
#define BL_K 32

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void block_linear_kernel(
    const TX* __restrict__ x, int64_t x_ld, int x_step, const TW* __restrict__ w,
    const float* __restrict__ bias, TO* __restrict__ out, int64_t out_ld, int out_step,
    const float* __restrict__ gate, int64_t gate_ld, int n, int k, int tokens) {
  __shared__ float s_x[BL_TOKENS][BL_K];
  __shared__ float s_w[BL_COLS][BL_K + 1];
  const int b = blockIdx.z;
  const int t0 = blockIdx.x * BL_TOKENS;
  const int j0 = blockIdx.y * BL_COLS;
  const int col = threadIdx.x & 63;          // the thread's output column of the tile
  const int group = threadIdx.x >> 6;        // its four tokens: group * 4 ..
  const TW* wb = w + (int64_t)b * n * k;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k; k0 += BL_K) {
    for (int i = threadIdx.x; i < BL_TOKENS * BL_K; i += 256) {
      const int tt = i / BL_K, kk = i - tt * BL_K;
      const int t = t0 + tt;
      s_x[tt][kk] = (t < tokens && k0 + kk < k)
                        ? to_float<TX>(x[(int64_t)t * x_ld + (int64_t)b * x_step + k0 + kk]) : 0.f;
    }
    for (int i = threadIdx.x; i < BL_COLS * BL_K; i += 256) {
      const int jj = i / BL_K, kk = i - jj * BL_K;
      s_w[jj][kk] = (j0 + jj < n && k0 + kk < k) ? to_float<TW>(wb[(int64_t)(j0 + jj) * k + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BL_K; ++kk) {
      const float weight = s_w[col][kk];
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = fmaf(s_x[group * 4 + r][kk], weight, acc[r]);
    }
    __syncthreads();
  }
  const int j = j0 + col;
  if (j >= n) return;
  const float shift = bias ? bias[b * n + j] : 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = t0 + group * 4 + r;
    if (t >= tokens) continue;
    float v = acc[r] + shift;
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(int64_t)t * gate_ld + b * n + j]));
    out[(int64_t)t * out_ld + (int64_t)b * out_step + j] = from_float<TO>(v);
  }
}

extern "C" int ps_block_linear(const void* x, int x_dtype, int64_t x_ld, int x_step, const void* w,
                               int w_dtype, const float* bias, void* out, int out_dtype,
                               int64_t out_ld, int out_step, const float* gate, int64_t gate_ld,
                               int blocks, int n, int k, int tokens, void* stream) {
  PS_REQUIRE(blocks > 0 && n > 0 && k > 0 && tokens >= 0, "ps_block_linear: bad sizes");
  PS_REQUIRE(x_step >= 0 && out_step >= n && x_ld >= (int64_t)(blocks - 1) * x_step + k &&
                 out_ld >= (int64_t)(blocks - 1) * out_step + n,
             "ps_block_linear: the rows are too short for %d blocks of %d inputs and %d outputs",
             blocks, k, n);
  PS_REQUIRE(gate == nullptr || gate_ld >= (int64_t)blocks * n, "ps_block_linear: gate rows too short");
  PS_REQUIRE(blocks <= 65535 && (n + BL_COLS - 1) / BL_COLS <= 65535, "ps_block_linear: too many blocks");
  const bool known = (x_dtype == PS_F32 || x_dtype == PS_BF16) && (w_dtype == PS_F32 || w_dtype == PS_BF16) &&
                     (out_dtype == PS_F32 || out_dtype == PS_BF16);
  PS_REQUIRE(known, "ps_block_linear: unknown dtype");
  PS_REQUIRE(w_dtype == PS_BF16 || (x_dtype == PS_F32 && out_dtype == PS_F32),
             "ps_block_linear: float matrices take and give float rows");
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((tokens + BL_TOKENS - 1) / BL_TOKENS, (n + BL_COLS - 1) / BL_COLS, blocks);
#define PS_LAUNCH_BL(TX, TW, TO)                                                                  \
  hipLaunchKernelGGL((block_linear_kernel<TX, TW, TO>), grid, dim3(256), 0, s, (const TX*)x, x_ld,  \
                     x_step, (const TW*)w, bias, (TO*)out, out_ld, out_step, gate, gate_ld, n, k, \
                     tokens)
  if (w_dtype == PS_F32) {
    PS_LAUNCH_BL(float, float, float);
  } else if (x_dtype == PS_F32) {
    if (out_dtype == PS_F32) PS_LAUNCH_BL(float, bf16_t, float);
    else PS_LAUNCH_BL(float, bf16_t, bf16_t);
  } else {
    if (out_dtype == PS_F32) PS_LAUNCH_BL(bf16_t, bf16_t, float);
    else PS_LAUNCH_BL(bf16_t, bf16_t, bf16_t);
  }
#undef PS_LAUNCH_BL
  PS_CHECK_LAUNCH("ps_block_linear");
  return 0;
}
