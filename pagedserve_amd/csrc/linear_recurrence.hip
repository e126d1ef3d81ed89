// A gated linear recurrence with one number of state per channel (the real-gated linear
// recurrent unit of Griffin: De et al., "Griffin: Mixing Gated Linear Recurrences with Local
// Attention for Efficient Language Models").  Per token t and channel c, all in 32-bit:
//
//   r = sigmoid(gr[t, c]),   i = sigmoid(gi[t, c])            (gr, gi: the gates' pre-activations;
//       a row of `gates` holds, for every run of `block` channels, their gr and then their gi)
//   log a = -decay_scale * r * softplus(lam[c]),   a = exp(log a)
//   S_t = a S_(t-1) + sqrt(1 - a^2) * i * u[t, c]              (the first token too, from S = 0)
//   out[t, c] = S_t * gelu_tanh(proj[t, y_col + c])
//
// state: [slots, channels, 1 + taps - 1] float per request: S and behind it the channel's last
// taps - 1 raw inputs of the short convolution (proj[:, x_col + c], oldest first), which the
// convolution kernel of selective_scan.hip reads at the next step.
//
// The recurrence is linear in S, so a run of tokens acts on S as S -> A S + B.  A block owns CH
// channels of one item; its SEG x CH threads cut the item's tokens into runs of L: every thread
// works out a and b of its run's tokens and the run's (A, B), the runs' starts follow from the
// carried state through LDS, and every thread walks its run again from its true start, out of
// registers.  The dependent chain of an item of n tokens is n / SEG steps long, not n.  Long
// portions of few items take 16 channels and 64 runs a block, so that two prompts of a model
// 768 wide are 96 blocks and not 24 (a wave then reads four tokens' 64 bytes, not one token's
// 256); many items or many channels fill the chip with 64 channels a block.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

struct LruArgs {
  const float* proj;
  int64_t ld;
  int y_col, x_col;
  const float* u;
  const float* gates;   // [tokens, 2 * channels]: per run of `block` channels, r then i
  int block;
  const float* lam;
  float decay_scale;
  float* state;
  const int* cu_tokens;
  const int* slots;
  int channels, taps;
};

__device__ inline float lru_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ inline float lru_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T, int CH, int SEG, int L>
__global__ __launch_bounds__(CH * SEG) void lru_scan_kernel(LruArgs p, T* __restrict__ out) {
  __shared__ float s_a[SEG][CH], s_b[SEG][CH];
  __shared__ float s_carry[CH];
  const int item = blockIdx.x;
  const int lane = threadIdx.x % CH;
  const int seg = threadIdx.x / CH;
  const int c = blockIdx.y * CH + lane;
  const bool live = c < p.channels;
  const int cc = live ? c : p.channels - 1;
  const int t0 = p.cu_tokens[item], t1 = p.cu_tokens[item + 1];
  if (t1 <= t0) return;     // (the whole block)
  const int row = p.taps;   // 1 + taps - 1 floats per channel
  float* slot = p.state + ((int64_t)p.slots[item] * p.channels + cc) * row;
  const float rate = -p.decay_scale * lru_softplus(p.lam[cc]);
  const int gate_at = (cc / p.block) * 2 * p.block + cc % p.block;
  if (seg == 0) s_carry[lane] = slot[0];
  __syncthreads();
  const int width = p.channels;
  for (int base = t0; base < t1; base += SEG * L) {
    const int first = base + seg * L;
    float a[L], b[L];
    float run_a = 1.f, run_b = 0.f;
#pragma unroll
    for (int j = 0; j < L; ++j) {
      const int t = first + j;
      a[j] = 1.f;
      b[j] = 0.f;
      if (t < t1) {
        const float* g = p.gates + (int64_t)t * 2 * width;
        const float log_a = rate * lru_sigmoid(g[gate_at]);
        a[j] = expf(log_a);
        // 1 - a^2 without the cancellation next to a = 1
        b[j] = sqrtf(-expm1f(2.f * log_a)) * lru_sigmoid(g[gate_at + p.block]) * p.u[(int64_t)t * width + cc];
      }
      run_b = fmaf(a[j], run_b, b[j]);
      run_a *= a[j];
    }
    if (SEG > 1) {
      s_a[seg][lane] = run_a;
      s_b[seg][lane] = run_b;
      __syncthreads();
    }
    // the state before this run: the carried one through the runs ahead of it
    float s = s_carry[lane];
    for (int k = 0; k < seg; ++k) s = fmaf(s_a[k][lane], s, s_b[k][lane]);
#pragma unroll
    for (int j = 0; j < L; ++j) {
      const int t = first + j;
      s = fmaf(a[j], s, b[j]);
      if (t < t1 && live)
        out[(int64_t)t * width + c] = from_float<T>(s * gelu_tanh_f(p.proj[(int64_t)t * p.ld + p.y_col + c]));
    }
    __syncthreads();      // everyone has read the carried state and the runs
    if (seg == SEG - 1) s_carry[lane] = s;   // (runs beyond the item's end leave s as it is)
    __syncthreads();
  }
  if (seg == 0 && live) {
    slot[0] = s_carry[lane];
    // the slot's last taps - 1 raw inputs of (what it kept, then this step's tokens), oldest first
    float* kept = slot + 1;
    const int count = t1 - t0;
    for (int j = 0; j < p.taps - 1; ++j) {
      const int local = count - (p.taps - 1) + j;
      // (ascending j reads kept[j + count] with count >= 1: never a place already written)
      kept[j] = local >= 0 ? p.proj[(int64_t)(t0 + local) * p.ld + p.x_col + c] : kept[j + count];
    }
  }
}

extern "C" int ps_lru_scan(const float* proj, int64_t ld, int y_col, int x_col, const float* u,
                           const float* gates, int block, const float* lam, float decay_scale, float* state,
                           void* out, const int* cu_tokens, const int* slots, int items, int tokens,
                           int channels, int taps, int dtype, void* stream) {
  PS_REQUIRE(items >= 0 && tokens >= 0 && channels > 0 && taps >= 1, "ps_lru_scan: bad sizes");
  PS_REQUIRE(y_col >= 0 && x_col >= 0 && ld >= (int64_t)y_col + channels && ld >= (int64_t)x_col + channels,
             "ps_lru_scan: the projection's rows are too short for its channels");
  PS_REQUIRE(decay_scale > 0.f, "ps_lru_scan: the decay's factor must be positive");
  PS_REQUIRE(block > 0 && channels % block == 0, "ps_lru_scan: %d channels in runs of %d", channels, block);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_lru_scan: unknown dtype %d", dtype);
  if (items == 0 || tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const LruArgs p = {proj, ld, y_col, x_col, u, gates, block, lam, decay_scale, state, cu_tokens, slots, channels, taps};
  const dim3 grid(items, (channels + 63) / 64);
  const dim3 narrow_grid(items, (channels + 15) / 16);
  // decoded tokens and short portions: one wave walks an item; long portions: 16 runs side by
  // side, or 64 runs of 16 channels where blocks of 64 channels would leave most of the chip idle
  const bool wide = tokens - items >= 64;
  const bool narrow = wide && (int64_t)grid.x * grid.y < 192;
#define PS_LAUNCH_LRU(T)                                                                              \
  do {                                                                                                \
    if (narrow)                                                                                       \
      hipLaunchKernelGGL((lru_scan_kernel<T, 16, 64, 4>), narrow_grid, dim3(1024), 0, s, p, (T*)out); \
    else if (wide)                                                                                    \
      hipLaunchKernelGGL((lru_scan_kernel<T, 64, 16, 8>), grid, dim3(1024), 0, s, p, (T*)out);        \
    else                                                                                              \
      hipLaunchKernelGGL((lru_scan_kernel<T, 64, 1, 4>), grid, dim3(64), 0, s, p, (T*)out);           \
  } while (0)
  if (dtype == PS_F32)
    PS_LAUNCH_LRU(float);
  else
    PS_LAUNCH_LRU(bf16_t);
#undef PS_LAUNCH_LRU
  PS_CHECK_LAUNCH("ps_lru_scan");
  return 0;
}
