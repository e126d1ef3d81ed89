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
// Two kernels.  bfloat16 matrices whose rows are whole runs of 8 (and rows of x and out that
// keep a lane's pieces aligned) go to the matrix cores: a wave owns 16 tokens x 16 CT columns,
// reads its operands of v_mfma_f32_16x16x32_bf16 straight from memory (a lane: 8 consecutive k
// of one token and of one matrix row; the matrices are small and stay in the caches) and writes
// 4 consecutive columns of a token per lane.  Float rows of x are not rounded to bfloat16: they
// are split into a rounded part and the rest, x = hi + lo, and both parts are multiplied, so
// the sum has the float input's digits.  A block's four waves lie along the tokens (prompts) or
// along the columns (decode steps of up to 16 tokens).
// Everything else (float matrices, odd sizes): a block of 256 threads takes 16 tokens x 64
// output columns of one matrix, the tokens' inputs and the matrix's rows pass through LDS in
// pieces of 32 along k, a thread owns one column for four tokens.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

// 8 consecutive values of a row as the matrix cores' operand: `hi` the values rounded to
// bfloat16, `lo` what the rounding left (zero for rows that are bfloat16 already).
template <typename TX>
__device__ inline void bl_operand(const TX* p, bool live, uint4& hi, uint4& lo);

template <>
__device__ inline void bl_operand<bf16_t>(const bf16_t* p, bool live, uint4& hi, uint4& lo) {
  hi = live ? *reinterpret_cast<const uint4*>(p) : make_uint4(0, 0, 0, 0);
  lo = make_uint4(0, 0, 0, 0);
}

template <>
__device__ inline void bl_operand<float>(const float* p, bool live, uint4& hi, uint4& lo) {
  float v[8];
  if (live) {
    *reinterpret_cast<float4*>(&v[0]) = *reinterpret_cast<const float4*>(p);
    *reinterpret_cast<float4*>(&v[4]) = *reinterpret_cast<const float4*>(p + 4);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.f;
  }
  uint32_t h[4], l[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16_t a = float_to_bf16(v[2 * i]), c = float_to_bf16(v[2 * i + 1]);
    h[i] = (uint32_t)a.bits | ((uint32_t)c.bits << 16);
    l[i] = pack2_bf16(v[2 * i] - bf16_to_float(a), v[2 * i + 1] - bf16_to_float(c));
  }
  hi = make_uint4(h[0], h[1], h[2], h[3]);
  lo = make_uint4(l[0], l[1], l[2], l[3]);
}

// WT waves along the tokens x WC along the columns (WT * WC = 4), CT tiles of 16 columns a wave.
template <typename TX, typename TO, int WT, int WC, int CT>
__global__ __launch_bounds__(256) void block_linear_mfma_kernel(
    const TX* __restrict__ x, int64_t x_ld, int x_step, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, TO* __restrict__ out, int64_t out_ld, int out_step,
    const float* __restrict__ gate, int64_t gate_ld, int n, int k, int tokens) {
  const int b = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t0 = (blockIdx.x * WT + wave % WT) * 16;
  const int j0 = (blockIdx.y * WC + wave / WT) * 16 * CT;
  if (t0 >= tokens || j0 >= n) return;       // (the whole wave; nothing below waits for another)
  const int r = lane & 15, g = lane >> 4;
  const int t = min(t0 + r, tokens - 1);
  const TX* xr = x + (int64_t)t * x_ld + (int64_t)b * x_step + 8 * g;
  const bf16_t* wr[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c)
    wr[c] = w + ((int64_t)b * n + min(j0 + c * 16 + r, n - 1)) * k + 8 * g;
  f32x4 acc[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k; k0 += 32) {
    const bool live = k0 + 8 * g < k;
    uint4 hi, lo, wv[CT];
    bl_operand<TX>(xr + k0, live, hi, lo);
#pragma unroll
    for (int c = 0; c < CT; ++c)
      wv[c] = live ? *reinterpret_cast<const uint4*>(wr[c] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&wv[c]),
                                                       *reinterpret_cast<const bf16x8*>(&hi), acc[c], 0, 0, 0);
      if (sizeof(TX) == 4)
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&wv[c]),
                                                         *reinterpret_cast<const bf16x8*>(&lo), acc[c], 0, 0, 0);
    }
  }
  // element i of an accumulator: matrix row (lane / 16) * 4 + i of the tile, token lane % 16
  if (t0 + r >= tokens) return;
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int j = j0 + c * 16 + 4 * g;
    if (j >= n) continue;                    // (n is a multiple of 4: a lane's four are in or out)
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = acc[c][i] + (bias ? bias[b * n + j + i] : 0.f);
    if (gate != nullptr) {
      const float4 gv = *reinterpret_cast<const float4*>(gate + (int64_t)t * gate_ld + b * n + j);
      v[0] *= 1.0f / (1.0f + expf(-gv.x));
      v[1] *= 1.0f / (1.0f + expf(-gv.y));
      v[2] *= 1.0f / (1.0f + expf(-gv.z));
      v[3] *= 1.0f / (1.0f + expf(-gv.w));
    }
    TO* o = out + (int64_t)t * out_ld + (int64_t)b * out_step + j;
    if (sizeof(TO) == 4) {
      *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      *reinterpret_cast<uint2*>(o) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
    }
  }
}

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
  // the matrix cores: every piece of 8 inputs, 4 outputs and 4 gates that a lane moves at once is whole and aligned
  const int x_unit = x_dtype == PS_F32 ? 4 : 8, out_unit = 4;
  const bool cores =
      w_dtype == PS_BF16 && k % 8 == 0 && n % 4 == 0 && ((uintptr_t)w % 16) == 0 &&
      x_ld % x_unit == 0 && x_step % x_unit == 0 && ((uintptr_t)x % 16) == 0 &&
      out_ld % out_unit == 0 && out_step % out_unit == 0 && ((uintptr_t)out % 16) == 0 &&
      (gate == nullptr || (gate_ld % 4 == 0 && ((uintptr_t)gate % 16) == 0));
  if (cores) {
    const bool few = tokens <= 16;
    // few tokens: the four waves of a block take 16 columns each; many: 16 tokens x 64 columns each
    const dim3 tiles = few ? dim3(1, (n + 63) / 64, blocks) : dim3((tokens + 63) / 64, (n + 63) / 64, blocks);
    PS_REQUIRE(tiles.y <= 65535, "ps_block_linear: too many columns");
#define PS_LAUNCH_BLM(TX, TO)                                                                           \
  do {                                                                                                  \
    if (few)                                                                                            \
      hipLaunchKernelGGL((block_linear_mfma_kernel<TX, TO, 1, 4, 1>), tiles, dim3(256), 0, s,           \
                         (const TX*)x, x_ld, x_step, (const bf16_t*)w, bias, (TO*)out, out_ld,          \
                         out_step, gate, gate_ld, n, k, tokens);                                        \
    else                                                                                                \
      hipLaunchKernelGGL((block_linear_mfma_kernel<TX, TO, 4, 1, 4>), tiles, dim3(256), 0, s,           \
                         (const TX*)x, x_ld, x_step, (const bf16_t*)w, bias, (TO*)out, out_ld,          \
                         out_step, gate, gate_ld, n, k, tokens);                                        \
  } while (0)
    if (x_dtype == PS_F32) {
      if (out_dtype == PS_F32) PS_LAUNCH_BLM(float, float);
      else PS_LAUNCH_BLM(float, bf16_t);
    } else {
      if (out_dtype == PS_F32) PS_LAUNCH_BLM(bf16_t, float);
      else PS_LAUNCH_BLM(bf16_t, bf16_t);
    }
#undef PS_LAUNCH_BLM
    PS_CHECK_LAUNCH("ps_block_linear");
    return 0;
  }
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
