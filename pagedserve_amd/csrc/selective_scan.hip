// A selective state-space mixer (Mamba): a short causal convolution per channel, then a
// recurrence whose state is a vector of `states` numbers per channel with a step size that
// depends on the token:
//
//   x_t   = silu(sum_j conv[c, j] u_(t - taps + 1 + j) + conv_bias[c])      (u: the raw inputs)
//   dt_t  = softplus(dt_bias[c] + sum_r low_t[r] w_dt[c, r])
//   S_t[c, n] = exp(dt_t A[c, n]) S_(t-1)[c, n] + dt_t x_t B_t[n],   A = -exp(A_log)
//   y_t[c] = (sum_n S_t[c, n] C_t[n] + D[c] x_t) * silu(z_t[c])
//
// Per request the slot keeps, for every channel, the `states` numbers of S and behind them the
// last taps - 1 raw inputs (oldest first): [slots, channels, states + taps - 1] float.  The
// step sizes, the decays, the state and the sums are 32-bit in both engine dtypes.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

__device__ inline float silu_f(float v) { return v / (1.0f + expf(-v)); }

// softplus(v) = max(v, 0) + log1p(exp(-|v|))
__device__ inline float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// exp(rate * step) of the recurrence's decays, rate = A (or A * log2(e), see decay_rate).  The
// float engine takes the library's exponential; the bfloat16 engine, whose inputs carry three
// decimal digits, takes the hardware's base-2 exponential (one instruction after the product
// instead of a dozen: the walk over the tokens is bound by the instructions it issues).
template <typename T>
__device__ inline float decay_rate(float a);
template <>
__device__ inline float decay_rate<float>(float a) { return a; }
template <>
__device__ inline float decay_rate<bf16_t>(float a) { return a * 1.4426950408889634f; }
template <typename T>
__device__ inline float decay_of(float rate, float step);
template <>
__device__ inline float decay_of<float>(float rate, float step) { return expf(rate * step); }
template <>
__device__ inline float decay_of<bf16_t>(float rate, float step) { return __builtin_amdgcn_exp2f(rate * step); }

// x[t, c] = silu(conv(u)[t, c]): a thread per (token, channel).  Inputs before the step's first
// token of the item come from the slot (zeros for a new request: the slot was cleared).
template <typename T>
__global__ __launch_bounds__(256) void conv_silu_kernel(
    const float* __restrict__ proj, int64_t ld, int u_col, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ state, int row, int tail,
    T* __restrict__ x, const int* __restrict__ tok_item, const int* __restrict__ cu_tokens,
    const int* __restrict__ slots, int channels, int taps, int activation) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int item = tok_item[t];
  const int first = cu_tokens[item];
  const float* kept = state + ((int64_t)slots[item] * channels + c) * row + tail;
  float sum = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;           // the input `back` tokens before this one
    const int local = (t - first) - back;    // its place among the item's tokens of this step
    const float u = local >= 0 ? proj[(int64_t)(t - back) * ld + u_col + c]
                               : kept[taps - 1 + local];
    sum = fmaf(w[(int64_t)c * taps + j], u, sum);
  }
  x[(int64_t)t * channels + c] = from_float<T>(activation ? silu_f(sum) : sum);
}

// dt[t, c] = softplus(bias[c] + sum_r low[t, r] w[c, r]).  A thread per channel and SS_STEP_TOKENS
// tokens: a weight is read once for all of them.
#define SS_STEP_TOKENS 4
template <typename T>
__global__ __launch_bounds__(256) void step_size_kernel(
    const float* __restrict__ low, int64_t ld, int rank, const T* __restrict__ w,
    const float* __restrict__ bias, float* __restrict__ dt, int tokens, int channels) {
  extern __shared__ float s_low[];           // [SS_STEP_TOKENS][rank]
  const int t0 = blockIdx.x * SS_STEP_TOKENS;
  const int count = tokens - t0 < SS_STEP_TOKENS ? tokens - t0 : SS_STEP_TOKENS;
  for (int i = threadIdx.x; i < SS_STEP_TOKENS * rank; i += blockDim.x) {
    const int tt = i / rank;
    s_low[i] = tt < count ? low[(int64_t)(t0 + tt) * ld + (i - tt * rank)] : 0.f;
  }
  __syncthreads();
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  float z[SS_STEP_TOKENS];
  const float start = bias ? bias[c] : 0.f;
#pragma unroll
  for (int tt = 0; tt < SS_STEP_TOKENS; ++tt) z[tt] = start;
  const T* w_row = w + (int64_t)c * rank;
  for (int r = 0; r < rank; ++r) {
    const float weight = to_float<T>(w_row[r]);
#pragma unroll
    for (int tt = 0; tt < SS_STEP_TOKENS; ++tt) z[tt] = fmaf(s_low[tt * rank + r], weight, z[tt]);
  }
#pragma unroll
  for (int tt = 0; tt < SS_STEP_TOKENS; ++tt)
    if (tt < count) dt[(int64_t)(t0 + tt) * channels + c] = softplus_f(z[tt]);
}

// The recurrence.  A block of one wave owns 64 / LPC channels of one item and walks tokens in
// order; a channel's states are dealt to LPC neighbouring lanes (state n to lane n % LPC), SPL to a
// lane, in registers.  B and C of SS_CHUNK tokens wait in LDS.
#define SS_CHUNK 16
struct ScanArgs {
  const float* dt;
  const float* bc;
  int64_t bc_ld;
  int b_col, c_col;
  const float* proj;
  int64_t ld;
  int u_col, z_col;
  const float* a_log;
  const float* skip;
  float* state;
  const int* cu_tokens;
  const int* slots;
  int channels, states, taps;
  // where dt is null, the step sizes are worked out on the way: softplus(step_bias[c] + sum_r
  // bc[t, low_col + r] step_w[c, r]) with weights of the storage type
  const void* step_w;
  const float* step_bias;
  int low_col, rank;
};

// Tokens first .. last - 1 of one item for the block's channels, from the states in S.  EMIT:
// the outputs are written; else only the states move, and the lanes get the sum of the step sizes.
// Everything that a token's step reads waits in LDS, SS_CHUNK tokens at a time (B and C, the
// block's channels of the step sizes, inputs and gates, loaded by all lanes side by side), so
// that the walk from token to token never waits for memory; the outputs of a chunk leave
// together, gated, after its walk.
// LDS: [SS_CHUNK][2 * states] | [SS_CHUNK][rank] (own step sizes only) | 4 x [SS_CHUNK][CPB].
template <typename T, int LPC, int SPL, bool EMIT>
__device__ inline float scan_range(const ScanArgs& p, const T* __restrict__ x, T* __restrict__ y,
                                   int first, int last, int c, int cc, bool live, float (&S)[SPL],
                                   const float (&A)[SPL], float* s_bc) {
  constexpr int CPB = 64 / LPC;
  const int lane = threadIdx.x;
  const int part = lane % LPC;
  const int mine = lane / LPC;                       // the lane's channel within the block
  const int states = p.states, channels = p.channels;
  const float d_skip = EMIT ? p.skip[cc] : 0.f;
  const bool own_steps = p.dt == nullptr;
  const T* step_row = (const T*)p.step_w + (int64_t)cc * p.rank;
  const float step_bias = own_steps && p.step_bias != nullptr ? p.step_bias[cc] : 0.f;
  float* s_low = s_bc + SS_CHUNK * 2 * states;       // [SS_CHUNK][rank], only with own step sizes
  float* s_dt = s_low + (own_steps ? SS_CHUNK * p.rank : 0);
  float* s_x = s_dt + SS_CHUNK * CPB;
  float* s_z = s_x + SS_CHUNK * CPB;
  float* s_y = s_z + SS_CHUNK * CPB;
  const int c0 = c - mine;                           // the block's first channel
  float steps = 0.f;
  for (int base = first; base < last; base += SS_CHUNK) {
    const int count = (last - base) < SS_CHUNK ? (last - base) : SS_CHUNK;
    __syncthreads();
    for (int idx = lane; idx < count * 2 * states; idx += 64) {
      const int tt = idx / (2 * states);
      const int n = idx - tt * 2 * states;
      s_bc[idx] = p.bc[(int64_t)(base + tt) * p.bc_ld + (n < states ? p.b_col + n : p.c_col + n - states)];
    }
    if (own_steps) {
      for (int idx = lane; idx < count * p.rank; idx += 64) {
        const int tt = idx / p.rank;
        s_low[idx] = p.bc[(int64_t)(base + tt) * p.bc_ld + p.low_col + (idx - tt * p.rank)];
      }
    }
    for (int idx = lane; idx < count * CPB; idx += 64) {
      const int tt = idx / CPB;
      const int64_t t = base + tt;
      const int channel = c0 + (idx - tt * CPB) < channels ? c0 + (idx - tt * CPB) : channels - 1;
      if (!own_steps) s_dt[idx] = p.dt[t * channels + channel];
      s_x[idx] = to_float<T>(x[t * channels + channel]);
      if (EMIT) s_z[idx] = p.proj[t * p.ld + p.z_col + channel];
    }
    __syncthreads();
    for (int tt = 0; tt < count; ++tt) {
      float step;
      if (own_steps) {
        // the channel's lanes share the low-rank sum
        float z = 0.f;
        for (int r = part; r < p.rank; r += LPC) z = fmaf(s_low[tt * p.rank + r], to_float<T>(step_row[r]), z);
        step = softplus_f(lanes_sum<LPC>(z) + step_bias);
      } else {
        step = s_dt[tt * CPB + mine];
      }
      const float xv = s_x[tt * CPB + mine];
      const float* b_row = s_bc + tt * 2 * states;
      const float* c_row = b_row + states;
      const float sx = step * xv;
      float sum = 0.f;
      steps += step;
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        const int n = part + i * LPC;
        if (n < states) {
          S[i] = fmaf(decay_of<T>(A[i], step), S[i], sx * b_row[n]);
          if (EMIT) sum = fmaf(S[i], c_row[n], sum);
        }
      }
      if (EMIT) {
        sum = lanes_sum<LPC>(sum);
        if (part == 0) s_y[tt * CPB + mine] = fmaf(d_skip, xv, sum);
      }
    }
    if (EMIT) {
      __syncthreads();
      for (int idx = lane; idx < count * CPB; idx += 64) {
        const int tt = idx / CPB;
        const int channel = c0 + (idx - tt * CPB);
        if (channel < channels)
          y[(int64_t)(base + tt) * channels + channel] = from_float<T>(s_y[idx] * silu_f(s_z[idx]));
      }
    }
  }
  (void)live;
  return steps;
}

// The slot's last taps - 1 raw inputs of (what it kept, then tokens t0 .. t1 - 1), oldest first.
__device__ inline void keep_inputs(const ScanArgs& p, float* kept, int t0, int t1, int c) {
  const int count = t1 - t0;
  for (int j = 0; j < p.taps - 1; ++j) {
    const int local = count - (p.taps - 1) + j;      // place among this step's tokens
    // (ascending j reads kept[j + count] with count >= 1: never a place already written)
    kept[j] = local >= 0 ? p.proj[(int64_t)(t0 + local) * p.ld + p.u_col + c] : kept[j + count];
  }
}

// One block walks all tokens of its item: the shape for decoded tokens and short portions.
template <typename T, int LPC, int SPL>
__global__ __launch_bounds__(64) void selective_scan_kernel(ScanArgs p, const T* __restrict__ x,
                                                            T* __restrict__ y) {
  constexpr int CPB = 64 / LPC;
  extern __shared__ float s_bc[];            // [SS_CHUNK][2 * states]
  const int item = blockIdx.x;
  const int lane = threadIdx.x;
  const int part = lane % LPC;
  const int c = blockIdx.y * CPB + lane / LPC;
  const bool live = c < p.channels;
  const int cc = live ? c : p.channels - 1;
  const int t0 = p.cu_tokens[item], t1 = p.cu_tokens[item + 1];
  const int row = p.states + p.taps - 1;
  float* mine = p.state + ((int64_t)p.slots[item] * p.channels + cc) * row;
  float S[SPL], A[SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = part + i * LPC;
    S[i] = n < p.states ? mine[n] : 0.f;
    A[i] = n < p.states ? decay_rate<T>(-expf(p.a_log[(int64_t)cc * p.states + n])) : 0.f;
  }
  scan_range<T, LPC, SPL, true>(p, x, y, t0, t1, c, cc, live, S, A, s_bc);
  if (!live) return;
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = part + i * LPC;
    if (n < p.states) mine[n] = S[i];
  }
  if (part == 0 && t1 > t0) keep_inputs(p, mine + p.states, t0, t1, c);
}

// Long portions are cut into pieces of SS_PIECE tokens that run side by side.  The recurrence
// is linear in the state, S_end = P S_start + E with P = exp(A * sum of the piece's step sizes)
// and E what the piece leaves from a zero state, so three launches do it:
//   1. every piece from zero: E and the sum of its step sizes (the first piece of an item also
//      copies the slot's state aside);
//   2. per item, piece after piece: the state at each piece's start, and the item's last state
//      into the slot;
//   3. every piece again from its true start, now writing the outputs.
// Records: [entry][channels][states] floats and [entry][channels] sums, an item's entries one
// behind the other: its start, then its pieces.
#define SS_PIECE 32
struct PieceOf {
  int item, piece, pieces, entry;     // entry: the record of the item's start
};

// The (item, piece) of the block's place among all pieces of the step; item < 0: none.
__device__ inline PieceOf find_piece(const int* cu_tokens, int items, int place) {
  PieceOf found = {-1, 0, 0, 0};
  int entry = 0;
  for (int i = 0; i < items; ++i) {
    const int pieces = (cu_tokens[i + 1] - cu_tokens[i] + SS_PIECE - 1) / SS_PIECE;
    if (place < pieces) {
      found.item = i;
      found.piece = place;
      found.pieces = pieces;
      found.entry = entry;
      return found;
    }
    place -= pieces;
    entry += pieces + 1;
  }
  return found;
}

template <typename T, int LPC, int SPL, bool EMIT>
__global__ __launch_bounds__(64) void selective_pieces_kernel(ScanArgs p, const T* __restrict__ x,
                                                              T* __restrict__ y, int items,
                                                              float* __restrict__ records,
                                                              float* __restrict__ sums) {
  constexpr int CPB = 64 / LPC;
  extern __shared__ float s_bc[];
  const PieceOf at = find_piece(p.cu_tokens, items, blockIdx.x);
  if (at.item < 0) return;
  const int lane = threadIdx.x;
  const int part = lane % LPC;
  const int c = blockIdx.y * CPB + lane / LPC;
  const bool live = c < p.channels;
  const int cc = live ? c : p.channels - 1;
  const int t0 = p.cu_tokens[at.item], t1 = p.cu_tokens[at.item + 1];
  const int first = t0 + at.piece * SS_PIECE;
  const int last = first + SS_PIECE < t1 ? first + SS_PIECE : t1;
  const int64_t per_entry = (int64_t)p.channels * p.states;
  float* record = records + (at.entry + 1 + at.piece) * per_entry + (int64_t)cc * p.states;
  const int row = p.states + p.taps - 1;
  float* mine = p.state + ((int64_t)p.slots[at.item] * p.channels + cc) * row;
  float S[SPL], A[SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = part + i * LPC;
    A[i] = n < p.states ? decay_rate<T>(-expf(p.a_log[(int64_t)cc * p.states + n])) : 0.f;
    S[i] = (EMIT && n < p.states) ? record[n] : 0.f;
  }
  if (!EMIT && at.piece == 0 && live) {
    float* start = records + at.entry * per_entry + (int64_t)cc * p.states;
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const int n = part + i * LPC;
      if (n < p.states) start[n] = mine[n];
    }
  }
  const float steps = scan_range<T, LPC, SPL, EMIT>(p, x, y, first, last, c, cc, live, S, A, s_bc);
  if (!live) return;
  if (!EMIT) {
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const int n = part + i * LPC;
      if (n < p.states) record[n] = S[i];
    }
    if (part == 0) sums[(int64_t)(at.entry + 1 + at.piece) * p.channels + c] = steps;
  } else if (at.piece == at.pieces - 1 && part == 0) {
    keep_inputs(p, mine + p.states, t0, t1, c);
  }
}

// Launch 2: a thread per (channel, state) of an item.
__global__ __launch_bounds__(256) void selective_join_kernel(ScanArgs p, float* __restrict__ records,
                                                             const float* __restrict__ sums) {
  const int item = blockIdx.x;
  const int64_t per_entry = (int64_t)p.channels * p.states;
  const int64_t index = (int64_t)blockIdx.y * 256 + threadIdx.x;
  if (index >= per_entry) return;
  int entry = 0;
  for (int i = 0; i < item; ++i)
    entry += (p.cu_tokens[i + 1] - p.cu_tokens[i] + SS_PIECE - 1) / SS_PIECE + 1;
  const int pieces = (p.cu_tokens[item + 1] - p.cu_tokens[item] + SS_PIECE - 1) / SS_PIECE;
  if (pieces == 0) return;
  const int c = (int)(index / p.states), n = (int)(index - (int64_t)c * p.states);
  const float a = -expf(p.a_log[index]);
  float s = records[entry * per_entry + index];
  for (int j = 0; j < pieces; ++j) {
    float* record = records + (entry + 1 + j) * per_entry + index;
    const float left = *record;
    const float decay = expf(a * sums[(int64_t)(entry + 1 + j) * p.channels + c]);
    *record = s;
    s = fmaf(decay, s, left);
  }
  const int row = p.states + p.taps - 1;
  p.state[((int64_t)p.slots[item] * p.channels + c) * row + n] = s;
}

extern "C" int ps_conv_silu(const float* proj, int64_t ld, int u_col, const float* w,
                            const float* bias, const float* state, int states, void* x,
                            const int* tok_item, const int* cu_tokens, const int* slots, int tokens,
                            int channels, int taps, int activation, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && channels > 0 && taps >= 1 && taps <= 64 && states >= 0,
             "ps_conv_silu: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_conv_silu: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(tokens, (channels + 255) / 256);
  const int row = states + taps - 1;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(conv_silu_kernel<float>, grid, dim3(256), 0, s, proj, ld, u_col, w, bias, state,
                       row, states, (float*)x, tok_item, cu_tokens, slots, channels, taps, activation);
  else
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, grid, dim3(256), 0, s, proj, ld, u_col, w, bias, state,
                       row, states, (bf16_t*)x, tok_item, cu_tokens, slots, channels, taps, activation);
  PS_CHECK_LAUNCH("ps_conv_silu");
  return 0;
}

extern "C" int ps_step_size(const float* low, int64_t ld, int rank, const void* w, const float* bias,
                            float* dt, int tokens, int channels, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && rank > 0 && rank <= 2048 && channels > 0, "ps_step_size: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_step_size: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)SS_STEP_TOKENS * rank * sizeof(float);
  const dim3 grid((tokens + SS_STEP_TOKENS - 1) / SS_STEP_TOKENS, (channels + 255) / 256);
  if (dtype == PS_F32)
    hipLaunchKernelGGL(step_size_kernel<float>, grid, dim3(256), lds, s, low, ld, rank,
                       (const float*)w, bias, dt, tokens, channels);
  else
    hipLaunchKernelGGL(step_size_kernel<bf16_t>, grid, dim3(256), lds, s, low, ld, rank,
                       (const bf16_t*)w, bias, dt, tokens, channels);
  PS_CHECK_LAUNCH("ps_step_size");
  return 0;
}

extern "C" int ps_selective_pieces(int tokens, int items) {
  return tokens / SS_PIECE + items;      // no step of that many tokens and items has more pieces
}

// records / sums: scratch for the launch in pieces, [(pieces + items) * channels * states] and
// [(pieces + items) * channels] floats with pieces = ps_selective_pieces(tokens, items); null:
// every item is walked by one block.
extern "C" int ps_selective_scan(const void* x, const float* dt, const float* bc, int64_t bc_ld,
                                 int b_col, int c_col, const float* proj, int64_t ld, int u_col,
                                 int z_col, const float* a_log, const float* skip, float* state,
                                 void* y, const int* cu_tokens, const int* slots, int items,
                                 int channels, int states, int taps, int tokens, float* records,
                                 float* sums, const void* step_w, const float* step_bias,
                                 int low_col, int rank, int dtype, void* stream) {
  PS_REQUIRE(items >= 0 && channels > 0 && states > 0 && taps >= 1, "ps_selective_scan: bad sizes");
  PS_REQUIRE(states <= 256, "ps_selective_scan: %d states per channel, at most 256", states);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_selective_scan: unknown dtype %d", dtype);
  PS_REQUIRE((records == nullptr) == (sums == nullptr), "ps_selective_scan: records and sums go together");
  PS_REQUIRE(dt != nullptr || (step_w != nullptr && rank > 0 && rank <= 256 && low_col >= 0),
             "ps_selective_scan: neither step sizes nor weights (of rank 1..256) to work them out");
  if (items == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int staged = 2 * states + (dt == nullptr ? rank : 0);     // floats per token beside the channels' own
  const ScanArgs p = {dt, bc, bc_ld, b_col, c_col, proj, ld, u_col, z_col, a_log, skip, state,
                      cu_tokens, slots, channels, states, taps, step_w, step_bias, low_col, rank};
  const int pieces = ps_selective_pieces(tokens, items);
#define PS_LAUNCH_SS_T(T, LPC, SPL)                                                               \
  do {                                                                                            \
    const int blocks = (channels + 64 / LPC - 1) / (64 / LPC);                                    \
    const size_t lds = (size_t)SS_CHUNK * (staged + 4 * (64 / LPC)) * sizeof(float);               \
    if (records == nullptr) {                                                                     \
      hipLaunchKernelGGL((selective_scan_kernel<T, LPC, SPL>), dim3(items, blocks), dim3(64), lds, s, \
                         p, (const T*)x, (T*)y);                                                  \
    } else {                                                                                      \
      hipLaunchKernelGGL((selective_pieces_kernel<T, LPC, SPL, false>), dim3(pieces, blocks),     \
                         dim3(64), lds, s, p, (const T*)x, (T*)y, items, records, sums);          \
      hipLaunchKernelGGL(selective_join_kernel, dim3(items, (channels * states + 255) / 256),     \
                         dim3(256), 0, s, p, records, sums);                                      \
      hipLaunchKernelGGL((selective_pieces_kernel<T, LPC, SPL, true>), dim3(pieces, blocks),      \
                         dim3(64), lds, s, p, (const T*)x, (T*)y, items, records, sums);          \
    }                                                                                             \
  } while (0)
#define PS_LAUNCH_SS(LPC, SPL)                  \
  do {                                          \
    if (dtype == PS_F32) {                      \
      PS_LAUNCH_SS_T(float, LPC, SPL);          \
    } else {                                    \
      PS_LAUNCH_SS_T(bf16_t, LPC, SPL);         \
    }                                           \
  } while (0)
  // a lane keeps at most 16 states; few states are dealt to few lanes
  if (states <= 4) PS_LAUNCH_SS(1, 4);
  else if (states <= 8) PS_LAUNCH_SS(2, 4);
  else if (states <= 16) PS_LAUNCH_SS(4, 4);
  else if (states <= 32) PS_LAUNCH_SS(4, 8);
  else if (states <= 64) PS_LAUNCH_SS(8, 8);
  else if (states <= 128) PS_LAUNCH_SS(16, 8);
  else PS_LAUNCH_SS(16, 16);
#undef PS_LAUNCH_SS
#undef PS_LAUNCH_SS_T
  PS_CHECK_LAUNCH("ps_selective_scan");
  return 0;
}
