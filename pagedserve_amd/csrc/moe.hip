// Mixture of experts: the router, and the experts' products for rows that are dealt to them
// token by token.
//
//   z = W_r x (32-bit),  s = softmax(z) over all experts
//   the experts form `groups` equal groups of neighbours; a group's score is its largest s; only
//   experts of the `keep` best groups may be chosen; the `top` largest s among them are, with
//   the weights s * scale (not renormalised)
//   out = sum over the chosen e of weight_e * W_down,e (silu(W_gate,e x) * (W_up,e x))
//
// Options of the router: sigmoid scores instead of the softmax; a correction per expert that is
// added to the scores for the choice only (the weights use the scores without it; closed
// experts count as minus infinity, since corrected scores may be negative); a group's score as
// the sum of its `group_top` largest choice scores; weights divided by their sum (+ 1e-20).
// Option of the experts: the plain form W_down,e relu(W_up,e x)^2 with one first matrix.
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

#define MOE_MAX_EXPERTS 1024

// What a router does beyond the softmax choice.
struct RouteOptions {
  int sigmoid;                 // scores are sigmoid(z) instead of softmax(z)
  const float* correction;     // added to the scores for the choice (null: none)
  int group_top;               // a group's score: the sum of this many largest choice scores
  int normalise;               // the chosen weights are divided by their sum
  int fixed;                   // experts behind the routed ones that every token uses with weight 1:
                               // a row of ids and weights is [top chosen | fixed], the fixed ones
                               // numbered from `experts` on
};

// The sum of the `count` largest of choice[first .. first + size - 1].  The numbers are walked in
// the order (larger first, lower index first); each round takes the first one behind the last
// taken, so nothing has to be remembered but that one.
__device__ inline float largest_sum(const float* choice, int first, int size, int count) {
  float total = 0.f;
  float last = INFINITY;
  int last_at = -1;
  if (count > size) count = size;
  for (int r = 0; r < count; ++r) {
    int best = -1;
    float best_score = -INFINITY;
    for (int e = first; e < first + size; ++e) {
      const float v = choice[e];
      const bool behind = v < last || (v == last && e > last_at);
      if (behind && (best < 0 || v > best_score)) {
        best_score = v;
        best = e;
      }
    }
    if (best < 0) break;      // (numbers that are no numbers)
    total += best_score;
    last = best_score;
    last_at = best;
  }
  return total;
}

// A lane's share of the dot product of a token's row with an expert's router row: four strides
// of the wave at a time, so that eight loads are on their way together instead of two.
template <typename T>
__device__ inline float router_dot(const T* __restrict__ row, const float* __restrict__ w_row, int width,
                                   int lane) {
  float sum = 0.f;
  int d = lane;
  for (; d + 192 < width; d += 256) {
    const float x0 = to_float<T>(row[d]), x1 = to_float<T>(row[d + 64]);
    const float x2 = to_float<T>(row[d + 128]), x3 = to_float<T>(row[d + 192]);
    const float w0 = w_row[d], w1 = w_row[d + 64], w2 = w_row[d + 128], w3 = w_row[d + 192];
    sum = fmaf(x0, w0, sum);
    sum = fmaf(x1, w1, sum);
    sum = fmaf(x2, w2, sum);
    sum = fmaf(x3, w3, sum);
  }
  for (; d < width; d += 64) sum = fmaf(to_float<T>(row[d]), w_row[d], sum);
  return sum;
}

// A block of one wave per token.  The logits are sums over the width dealt to the lanes; the
// choice itself is a few dozen comparisons and is left to lane 0.
template <typename T>
__global__ __launch_bounds__(64) void moe_route_kernel(
    const T* __restrict__ x, int64_t x_ld, const float* __restrict__ w, int width, int experts,
    int groups, int keep, int top, float scale, RouteOptions options, int* __restrict__ ids,
    float* __restrict__ weights) {
  __shared__ float s_score[MOE_MAX_EXPERTS];
  __shared__ float s_choice[MOE_MAX_EXPERTS];
  __shared__ unsigned char s_open[MOE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const T* row = x + t * x_ld;
  for (int e = 0; e < experts; ++e) {
    const float sum = wave_sum(router_dot<T>(row, w + (int64_t)e * width, width, lane));
    if (lane == 0) s_score[e] = sum;
  }
  __syncthreads();
  if (lane != 0) return;
  const int cols = top + options.fixed;
  if (options.sigmoid) {
    for (int e = 0; e < experts; ++e) s_score[e] = 1.0f / (1.0f + expf(-s_score[e]));
  } else {
    float top_z = -INFINITY;
    for (int e = 0; e < experts; ++e) top_z = fmaxf(top_z, s_score[e]);
    float total = 0.f;
    for (int e = 0; e < experts; ++e) {
      s_score[e] = expf(s_score[e] - top_z);
      total += s_score[e];
    }
    const float inv = 1.0f / total;
    for (int e = 0; e < experts; ++e) s_score[e] *= inv;
  }
  for (int e = 0; e < experts; ++e) {
    s_choice[e] = s_score[e] + (options.correction ? options.correction[e] : 0.f);
    s_open[e] = groups <= 1 || keep >= groups;
  }
  if (groups > 1 && keep < groups) {
    // the best groups one after the other; a group that was taken has its experts open
    const int size = experts / groups;
    for (int round = 0; round < keep; ++round) {
      int best = -1;
      float best_score = -INFINITY;
      for (int g = 0; g < groups; ++g) {
        if (s_open[g * size]) continue;
        const float score = largest_sum(s_choice, g * size, size, options.group_top);
        if (best < 0 || score > best_score) {
          best_score = score;
          best = g;
        }
      }
      if (best < 0) best = 0;      // (scores that are no numbers: any choice, but a valid one)
      for (int e = best * size; e < (best + 1) * size; ++e) s_open[e] = 1;
    }
  }
  float chosen_sum = 0.f;
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float best_score = -INFINITY;
    for (int e = 0; e < experts; ++e) {
      if (s_open[e] == 1 && (best < 0 || s_choice[e] > best_score)) {
        best_score = s_choice[e];
        best = e;
      }
    }
    if (best < 0) best = 0;       // (scores that are no numbers: any choice, but a valid one)
    s_open[best] = 2;     // chosen: not again
    ids[t * cols + j] = best;
    const float own = s_score[best] == s_score[best] ? s_score[best] : 0.f;
    weights[t * cols + j] = own;
    chosen_sum += own;
  }
  const float factor = options.normalise ? scale / (chosen_sum + 1e-20f) : scale;
  for (int j = 0; j < top; ++j) weights[t * cols + j] *= factor;
  for (int j = 0; j < options.fixed; ++j) {
    ids[t * cols + top + j] = experts + j;
    weights[t * cols + top + j] = 1.0f;
  }
}

// The same for up to 64 experts: a block of four waves per token, the waves share the experts'
// logits between them, and the choice is made with an expert per lane.  Ties go to the
// expert (and the group) with the lower number, as above.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_wave_kernel(
    const T* __restrict__ x, int64_t x_ld, const float* __restrict__ w, int width, int experts,
    int groups, int keep, int top, float scale, RouteOptions options, int* __restrict__ ids,
    float* __restrict__ weights) {
  __shared__ float s_score[64];
  __shared__ float s_group[64];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const T* row = x + t * x_ld;
  for (int e = wave; e < experts; e += 4) {
    const float sum = wave_sum(router_dot<T>(row, w + (int64_t)e * width, width, lane));
    if (lane == 0) s_score[e] = sum;
  }
  __syncthreads();
  // (all four waves choose, from the same numbers; the first one writes)
  const bool mine = lane < experts;
  const float z = mine ? s_score[lane] : -INFINITY;
  __syncthreads();
  float score;
  if (options.sigmoid) {
    score = mine ? 1.0f / (1.0f + expf(-z)) : 0.f;
  } else {
    const float p = mine ? expf(z - wave_max(z)) : 0.f;
    score = p / wave_sum(p);
  }
  const float choice = score + ((mine && options.correction) ? options.correction[lane] : 0.f);
  bool open = mine;
  if (groups > 1 && keep < groups) {
    const int size = experts / groups;
    s_score[lane] = choice;
    __syncthreads();
    if (lane < groups) s_group[lane] = largest_sum(s_score, lane * size, size, options.group_top);
    __syncthreads();
    if (mine) {
      const int g = lane / size;
      const float own = s_group[g];
      int ahead = 0;
      for (int other = 0; other < groups; ++other) {
        const float theirs = s_group[other];
        ahead += (theirs > own || (theirs == own && other < g)) ? 1 : 0;
      }
      open = ahead < keep;
    }
  }
  const int cols = top + options.fixed;
  int slot = -1;       // which of the token's choices this lane's expert is
  for (int j = 0; j < top; ++j) {
    const float offer = open ? choice : -INFINITY;
    const float best = wave_max(offer);
    const unsigned long long holders = __ballot(open && offer == best);
    const int chosen = holders ? __builtin_ctzll(holders) : 0;
    if (lane == chosen) {
      open = false;
      slot = j;
      if (wave == 0) ids[t * cols + j] = chosen;
    }
  }
  const float own = (slot >= 0 && score == score) ? score : 0.f;
  const float chosen_sum = wave_sum(own);
  if (slot >= 0 && wave == 0) {
    weights[t * cols + slot] = options.normalise ? own / (chosen_sum + 1e-20f) * scale : own * scale;
  }
  if (wave == 1 && lane < options.fixed) {
    ids[t * cols + top + lane] = experts + lane;
    weights[t * cols + top + lane] = 1.0f;
  }
}

// What a hidden column becomes: silu(g) * u of the gated form, relu(g)^2 of the plain one.
template <bool GATED>
__device__ inline float moe_activation(float g, float u) {
  if (GATED) return g / (1.0f + expf(-g)) * u;
  const float r = fmaxf(g, 0.f);
  return r * r;
}

// hidden[(t, j), c] = silu(W_gate,e[c] . x_t) * (W_up,e[c] . x_t) for e = ids[t, j].  The
// experts' first matrices lie one behind the other, [experts][gate rows | up rows][width].
// A block of four waves per (token, choice) and 4 * ROWS hidden columns; the lanes share a dot
// product's width.  GATED false: the plain form, hidden = relu(W_up,e[c] . x_t)^2, the experts' first
// matrices [experts][up rows][width].
template <typename T, int ROWS, bool GATED>
__global__ __launch_bounds__(256) void moe_hidden_kernel(
    const T* __restrict__ x, int64_t x_ld, const T* __restrict__ w1, const int* __restrict__ ids,
    T* __restrict__ hidden, int width, int inner, int experts, const T* __restrict__ w1x) {
  extern __shared__ float s_x[];
  // (blockIdx.x: the token, blockIdx.z: which of its choices)
  const int64_t row_index = (int64_t)blockIdx.x * gridDim.z + blockIdx.z;
  int e = ids[row_index];
  // (experts numbered from `experts` on lie in a tensor of their own)
  if (e >= experts) {
    e = w1x != nullptr ? e - experts : 0;
    if (w1x != nullptr) w1 = w1x;
  }
  const T* x_row = x + (int64_t)blockIdx.x * x_ld;
  for (int d = threadIdx.x; d < width; d += 256) s_x[d] = to_float<T>(x_row[d]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const T* base = w1 + (int64_t)e * (GATED ? 2 : 1) * inner * width;
  const int first = (blockIdx.y * 4 + wave) * ROWS;
  for (int r = 0; r < ROWS; ++r) {
    const int c = first + r;
    if (c >= inner) break;
    const T* g_row = base + (int64_t)c * width;
    const T* u_row = base + (int64_t)(inner + c) * width;
    float g = 0.f, u = 0.f;
    for (int d = lane; d < width; d += 64) {
      g = fmaf(to_float<T>(g_row[d]), s_x[d], g);
      if (GATED) u = fmaf(to_float<T>(u_row[d]), s_x[d], u);
    }
    g = wave_sum(g);
    if (GATED) u = wave_sum(u);
    if (lane == 0) hidden[row_index * inner + c] = from_float<T>(moe_activation<GATED>(g, u));
  }
}

// y[t, d] += sum_j weights[t, j] * (W_down,e_j[d] . hidden[(t, j)]).  A block of four waves per
// token and 4 * ROWS output columns.
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void moe_down_kernel(
    const T* __restrict__ hidden, const T* __restrict__ w2, const int* __restrict__ ids,
    const float* __restrict__ weights, float* __restrict__ y, int width, int inner, int top,
    int experts, const T* __restrict__ w2x) {
  extern __shared__ float s_h[];        // [top][inner]
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < top * inner; i += 256)
    s_h[i] = to_float<T>(hidden[t * top * inner + i]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int first = (blockIdx.y * 4 + wave) * ROWS;
  for (int r = 0; r < ROWS; ++r) {
    const int d = first + r;
    if (d >= width) break;
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = ids[t * top + j];
      const T* w_row = (e < experts || w2x == nullptr)
                           ? w2 + ((int64_t)(e < experts ? e : 0) * width + d) * inner
                           : w2x + ((int64_t)(e - experts) * width + d) * inner;
      float sum = 0.f;
      for (int c = lane; c < inner; c += 64) sum = fmaf(to_float<T>(w_row[c]), s_h[j * inner + c], sum);
      total = fmaf(weights[t * top + j], wave_sum(sum), total);
    }
    if (lane == 0) y[t * width + d] += total;
  }
}

extern "C" int ps_moe_route(const void* x, int64_t x_ld, const float* w, int tokens, int width,
                            int experts, int groups, int keep, int top, float scale, int sigmoid,
                            const float* correction, int group_top, int normalise, int fixed, int* ids,
                            float* weights, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && experts > 0 && experts <= MOE_MAX_EXPERTS,
             "ps_moe_route: %d experts, at most %d", experts, MOE_MAX_EXPERTS);
  PS_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups,
             "ps_moe_route: %d groups (keep %d) do not divide %d experts", groups, keep, experts);
  PS_REQUIRE(top >= 1 && top <= (experts / groups) * keep,
             "ps_moe_route: %d experts per token, %d may be chosen", top, (experts / groups) * keep);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_moe_route: unknown dtype %d", dtype);
  PS_REQUIRE(group_top >= 1 && group_top <= 8,
             "ps_moe_route: a group's score sums its %d largest scores, 1 to 8 are taken", group_top);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  PS_REQUIRE(fixed >= 0 && fixed <= 64, "ps_moe_route: %d fixed experts, up to 64 are taken", fixed);
  const RouteOptions options = {sigmoid, correction, group_top, normalise, fixed};
  if (experts <= 64) {
    if (dtype == PS_F32)
      hipLaunchKernelGGL(moe_route_wave_kernel<float>, dim3(tokens), dim3(256), 0, s, (const float*)x,
                         x_ld, w, width, experts, groups, keep, top, scale, options, ids, weights);
    else
      hipLaunchKernelGGL(moe_route_wave_kernel<bf16_t>, dim3(tokens), dim3(256), 0, s, (const bf16_t*)x,
                         x_ld, w, width, experts, groups, keep, top, scale, options, ids, weights);
  } else if (dtype == PS_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(tokens), dim3(64), 0, s, (const float*)x, x_ld, w,
                       width, experts, groups, keep, top, scale, options, ids, weights);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(tokens), dim3(64), 0, s, (const bf16_t*)x, x_ld,
                       w, width, experts, groups, keep, top, scale, options, ids, weights);
  PS_CHECK_LAUNCH("ps_moe_route");
  return 0;
}


// ---- few rows: every (token, choice) reads its expert's rows once, 16 bytes of k per lane ------
// Eight consecutive k of a row as floats.
template <typename T>
__device__ inline void load8(const T* p, float (&v)[8]);
template <>
__device__ inline void load8<bf16_t>(const bf16_t* p, float (&v)[8]) {
  const uint4 raw = *reinterpret_cast<const uint4*>(p);
  const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(words[i] << 16);
    v[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
  }
}
template <>
__device__ inline void load8<float>(const float* p, float (&v)[8]) {
  const float4 lo = *reinterpret_cast<const float4*>(p);
  const float4 hi = *reinterpret_cast<const float4*>(p + 4);
  v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
  v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
}

// As moe_hidden_kernel for a width that is a multiple of 8: a wave owns ROWS hidden columns and
// keeps the sums of their gate and up rows apart, so that 2 * ROWS loads are in flight per lane.
template <typename T, int ROWS, bool GATED>
__global__ __launch_bounds__(256) void moe_hidden_wide_kernel(
    const T* __restrict__ x, int64_t x_ld, const T* __restrict__ w1, const int* __restrict__ ids,
    T* __restrict__ hidden, int width, int inner, int experts, const T* __restrict__ w1x) {
  extern __shared__ float s_x[];
  const int64_t row_index = (int64_t)blockIdx.x * gridDim.z + blockIdx.z;
  int e = ids[row_index];
  if (e >= experts) {
    e = w1x != nullptr ? e - experts : 0;
    if (w1x != nullptr) w1 = w1x;
  }
  const T* x_row = x + (int64_t)blockIdx.x * x_ld;
  for (int d = threadIdx.x; d < width; d += 256) s_x[d] = to_float<T>(x_row[d]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const T* base = w1 + (int64_t)e * (GATED ? 2 : 1) * inner * width;
  const int first = (blockIdx.y * 4 + wave) * ROWS;
  if (first >= inner) return;
  float g[ROWS], u[ROWS];
  const T* rows_g[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    g[r] = u[r] = 0.f;
    const int c = first + r < inner ? first + r : inner - 1;
    rows_g[r] = base + (int64_t)c * width;
  }
  const int64_t up = (int64_t)inner * width;
  for (int d = lane * 8; d < width; d += 512) {
    float xv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xv[i] = s_x[d + i];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      float a[8], b[8];
      load8<T>(rows_g[r] + d, a);
      if (GATED) load8<T>(rows_g[r] + up + d, b);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        g[r] = fmaf(a[i], xv[i], g[r]);
        if (GATED) u[r] = fmaf(b[i], xv[i], u[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const float gs = wave_sum(g[r]), us = GATED ? wave_sum(u[r]) : 0.f;
    if (lane == 0 && first + r < inner)
      hidden[row_index * inner + first + r] = from_float<T>(moe_activation<GATED>(gs, us));
  }
}

// As moe_down_kernel for an inner width that is a multiple of 8.
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void moe_down_wide_kernel(
    const T* __restrict__ hidden, const T* __restrict__ w2, const int* __restrict__ ids,
    const float* __restrict__ weights, float* __restrict__ y, int width, int inner, int top,
    int experts, const T* __restrict__ w2x) {
  extern __shared__ float s_h[];        // [top][inner]
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < top * inner; i += 256)
    s_h[i] = to_float<T>(hidden[t * top * inner + i]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int first = (blockIdx.y * 4 + wave) * ROWS;
  if (first >= width) return;
  float total[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) total[r] = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[t * top + j];
    const float weight = weights[t * top + j];
    float sum[ROWS];
    const T* rows[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      sum[r] = 0.f;
      const int d = first + r < width ? first + r : width - 1;
      rows[r] = (e < experts || w2x == nullptr) ? w2 + ((int64_t)(e < experts ? e : 0) * width + d) * inner
                                                : w2x + ((int64_t)(e - experts) * width + d) * inner;
    }
    for (int c = lane * 8; c < inner; c += 512) {
      float hv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) hv[i] = s_h[j * inner + c + i];
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        float a[8];
        load8<T>(rows[r] + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) sum[r] = fmaf(a[i], hv[i], sum[r]);
      }
    }
    // (a lane's share of all experts is summed first and the lanes meet once at the end: no
    // expert's loads wait for the one before)
#pragma unroll
    for (int r = 0; r < ROWS; ++r) total[r] = fmaf(weight, sum[r], total[r]);
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const float whole = wave_sum(total[r]);
    if (lane == 0 && first + r < width) y[t * width + first + r] += whole;
  }
}

// ---- many rows: the (token, choice) pairs sorted by expert, products on the matrix cores -------
#define MOE_TILE 128     // pairs per tile; an expert's pairs are padded up to whole tiles

// One block.  order[pos] = the pair at sorted place pos (-1: padding), tile_expert[tile] = the
// expert of the MOE_TILE places of a tile (-1: the tile is not used).  The place of a pair within its
// expert's run depends on the order in which the threads arrive; nothing that is computed does.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int pairs,
                                                        int experts, int* __restrict__ order,
                                                        int* __restrict__ tile_expert, int max_tiles) {
  __shared__ int s_count[MOE_MAX_EXPERTS];
  __shared__ int s_start[MOE_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < experts; e += blockDim.x) s_count[e] = 0;
  for (int i = threadIdx.x; i < max_tiles * MOE_TILE; i += blockDim.x) order[i] = -1;
  for (int i = threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&s_count[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      s_start[e] = at;
      at += (s_count[e] + MOE_TILE - 1) / MOE_TILE * MOE_TILE;
    }
    s_start[experts] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += blockDim.x) {
    for (int tile = s_start[e] / MOE_TILE; tile < s_start[e + 1] / MOE_TILE; ++tile) tile_expert[tile] = e;
    s_count[e] = s_start[e];     // from here on: the next free place of the expert's run
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) order[atomicAdd(&s_count[ids[p]], 1)] = p;
}

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float moe_f32x16;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8;
#define MOE_LDS_STRIDE 80   // bytes between rows of a stage (64 bytes of k, padded)
#define MOE_DEPTH 4         // k tiles whose global loads are in flight

// A tile of 128 sorted pairs times 128 weight rows of the tile's expert, k in stages of 32.
// HIDDEN: the weight rows are 64 gate rows and the 64 up rows of the same hidden columns, and
// hidden[pair, column] = silu(gate) * up; the rows of A are the pairs' tokens (pair / top).
// MODE 2, the plain form's hidden rows: 128 up rows, hidden[pair, column] = relu(up)^2 (a tile of
// pairs is staged once for twice the columns).
// MODE 0: 64 output columns (so that the narrower product still gives every compute unit a
// block), out[pair, column] = weights[pair] * sum; the rows of A are the pairs' hidden rows.
// Four waves, 2 x 2: a wave has 64 pairs and 32 weight rows, twice in the first case.
template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int64_t expert_stride,
    int w_rows, int k, const int* __restrict__ order, const int* __restrict__ tile_expert, int top,
    const float* __restrict__ weights, bf16_t* __restrict__ hidden, float* __restrict__ out,
    int64_t out_ld) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  __shared__ __attribute__((aligned(16))) unsigned char lds[2][(MOE_TILE + 128) * MOE_LDS_STRIDE];
  __shared__ int s_pair[MOE_TILE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 1, wave_n = wave & 1;
  constexpr bool HIDDEN = MODE == 1;                     // gate and up rows side by side
  constexpr bool FROM_TOKENS = MODE != 0;                // the rows of A are the pairs' tokens
  const int columns = HIDDEN ? w_rows / 2 : w_rows;      // output columns
  constexpr int NJ = MODE == 0 ? 1 : 2;                  // runs of 64 weight rows in a stage
  const int n0 = blockIdx.y * (MODE == 2 ? 128 : 64);
  if (tid < MOE_TILE) s_pair[tid] = order[blockIdx.x * MOE_TILE + tid];
  __syncthreads();
  // staging: 16-byte chunks, 4 per row; A and W: 128 rows each, two chunks a thread
  const int chunk = (tid & 3) * 8;
  const int a_row = tid >> 2;
  const bf16_t* a_src[2];
  bool a_ok[2];
  const bf16_t* w_src[2];
  bool w_ok[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int a_pair = s_pair[a_row + i * 64];
    a_ok[i] = a_pair >= 0;
    a_src[i] = a + (int64_t)(a_pair < 0 ? 0 : (FROM_TOKENS ? a_pair / top : a_pair)) * lda;
    const int local = a_row + i * 64;      // 0..127
    int row;
    if (HIDDEN) row = (local < 64 ? 0 : columns) + n0 + (local & 63);
    else row = n0 + local;
    w_ok[i] = HIDDEN ? n0 + (local & 63) < columns : ((MODE == 2 || local < 64) && row < w_rows);
    w_src[i] = w + (int64_t)e * expert_stride + (int64_t)(w_ok[i] ? row : 0) * k;
  }
  // a ring of MOE_DEPTH stages in registers keeps that many k tiles' loads in flight
  uint4 ring_a[MOE_DEPTH][2], ring_w[MOE_DEPTH][2];
  const uint4 zero = {0u, 0u, 0u, 0u};
  auto load_global = [&](uint4* stage_a, uint4* stage_w, int k0) {
    // (a chunk behind the row's end is not read at all: the row's own first chunk stands in for
    // it and is thrown away; with k under 32 the old stand-in, this chunk of the first k tile, lay
    // behind the end of the row, and for the last row of the last expert behind the tensor)
    const bool k_ok = k0 + chunk < k;
    const int kk = k_ok ? k0 + chunk : 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      stage_a[i] = *reinterpret_cast<const uint4*>(a_src[i] + kk);
      if (!(k_ok && a_ok[i])) stage_a[i] = zero;
      if (i < NJ) {
        stage_w[i] = *reinterpret_cast<const uint4*>(w_src[i] + kk);
        if (!(k_ok && w_ok[i])) stage_w[i] = zero;
      }
    }
  };
  auto store_lds = [&](int buffer, const uint4* stage_a, const uint4* stage_w) {
    const int offset = a_row * MOE_LDS_STRIDE + (tid & 3) * 16;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<uint4*>(&lds[buffer][i * 64 * MOE_LDS_STRIDE + offset]) = stage_a[i];
      if (i < NJ)
        *reinterpret_cast<uint4*>(&lds[buffer][(MOE_TILE + i * 64) * MOE_LDS_STRIDE + offset]) = stage_w[i];
    }
  };
  moe_f32x16 acc[2][2];      // [rows of 32 pairs][weight rows]
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[r][j][i] = 0.f;
  const int k_tiles = (k + 31) / 32;
  auto compute = [&](int buffer) {
    const unsigned char* stage = lds[buffer];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int kbyte = half * 32 + (lane >> 5) * 16;
      uint4 fa[2], fw[2];
#pragma unroll
      for (int r = 0; r < 2; ++r)
        fa[r] = *reinterpret_cast<const uint4*>(
            &stage[(wave_m * 64 + r * 32 + (lane & 31)) * MOE_LDS_STRIDE + kbyte]);
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        fw[j] = *reinterpret_cast<const uint4*>(
            &stage[(MOE_TILE + j * 64 + wave_n * 32 + (lane & 31)) * MOE_LDS_STRIDE + kbyte]);
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          acc[r][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              *reinterpret_cast<const moe_bf16x8*>(&fa[r]), *reinterpret_cast<const moe_bf16x8*>(&fw[j]),
              acc[r][j], 0, 0, 0);
    }
  };
#pragma unroll
  for (int d = 0; d < MOE_DEPTH; ++d) load_global(ring_a[d], ring_w[d], d * 32);
  store_lds(0, ring_a[0], ring_w[0]);
  __syncthreads();
  for (int kt0 = 0; kt0 < k_tiles; kt0 += MOE_DEPTH) {
#pragma unroll
    for (int d = 0; d < MOE_DEPTH; ++d) {
      const int kt = kt0 + d;
      if (kt < k_tiles) {
        // stage d held tile kt, which is in LDS already: refill it with tile kt + MOE_DEPTH
        load_global(ring_a[d], ring_w[d], (kt + MOE_DEPTH) * 32);
        compute(kt & 1);
        // tile kt + 1 left MOE_DEPTH - 1 iterations ago
        store_lds((kt + 1) & 1, ring_a[(d + 1) % MOE_DEPTH], ring_w[(d + 1) % MOE_DEPTH]);
        __syncthreads();
      }
    }
  }
  // element i of an accumulator: row (i / 4) * 8 + (lane / 32) * 4 + i % 4, column lane % 32
#pragma unroll
  for (int ri = 0; ri < 32; ++ri) {
    const int r = ri >> 4, i = ri & 15;
    const int pair = s_pair[wave_m * 64 + r * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3)];
    if (pair < 0) continue;
    if (HIDDEN) {
      const int col = n0 + wave_n * 32 + (lane & 31);
      const float g = acc[r][0][i], u = acc[r][1][i];
      if (col < columns) hidden[(int64_t)pair * columns + col] = from_float<bf16_t>(g / (1.0f + expf(-g)) * u);
    } else if (MODE == 2) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + j * 64 + wave_n * 32 + (lane & 31);
        if (col < columns)
          hidden[(int64_t)pair * columns + col] = from_float<bf16_t>(moe_activation<false>(acc[r][j][i], 0.f));
      }
    } else {
      const int col = n0 + wave_n * 32 + (lane & 31);
      if (col < columns) out[(int64_t)pair * out_ld + col] = weights[pair] * acc[r][0][i];
    }
  }
}

// y[t, :] += sum_j out[t * top + j, :]
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ out,
                                                          float* __restrict__ y, int width, int top) {
  const int64_t t = blockIdx.x;
  for (int d = threadIdx.x; d < width; d += 256) {
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += out[(t * top + j) * width + d];
    y[t * width + d] += sum;
  }
}

extern "C" int ps_moe_experts(const void* x, int64_t x_ld, const void* w1, const void* w2,
                              const int* ids, const float* weights, void* hidden, float* y,
                              int tokens, int width, int inner, int top, int gated, int experts,
                              const void* w1x, const void* w2x, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && inner > 0 && top > 0 && top <= 65535,
             "ps_moe_experts: bad sizes");
  PS_REQUIRE((size_t)width * 4 <= 64 * 1024 && (size_t)top * inner * 4 <= 64 * 1024,
             "ps_moe_experts: width %d or %d x %d hidden columns do not fit LDS", width, top, inner);
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_moe_experts: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool wide1 = width % 8 == 0 && x_ld % 8 == 0, wide2 = inner % 8 == 0;
  // hidden columns / output columns per wave: four, or two while that still leaves the chip
  // short of blocks (a handful of decoded tokens)
  const bool few = (int64_t)tokens * ((width + 15) / 16) < 4 * ps_compute_units();
#define PS_MOE_HIDDEN(T, ROWS, GATED)                                                              \
  do {                                                                                             \
    const dim3 grid1(tokens, (inner + 4 * ROWS - 1) / (4 * ROWS), top);                            \
    if (wide1)                                                                                     \
      hipLaunchKernelGGL((moe_hidden_wide_kernel<T, ROWS, GATED>), grid1, dim3(256),               \
                         (size_t)width * 4, s, (const T*)x, x_ld, (const T*)w1, ids, (T*)hidden,   \
                         width, inner, experts, (const T*)w1x);                                    \
    else                                                                                           \
      hipLaunchKernelGGL((moe_hidden_kernel<T, ROWS, GATED>), grid1, dim3(256), (size_t)width * 4, \
                         s, (const T*)x, x_ld, (const T*)w1, ids, (T*)hidden, width, inner,        \
                         experts, (const T*)w1x);                                                  \
  } while (0)
#define PS_MOE_ROWS(T, ROWS)                                                                       \
  do {                                                                                             \
    const dim3 grid2(tokens, (width + 4 * ROWS - 1) / (4 * ROWS));                                 \
    if (gated) PS_MOE_HIDDEN(T, ROWS, true);                                                       \
    else PS_MOE_HIDDEN(T, ROWS, false);                                                            \
    if (wide2)                                                                                     \
      hipLaunchKernelGGL((moe_down_wide_kernel<T, ROWS>), grid2, dim3(256), (size_t)top * inner * 4, \
                         s, (const T*)hidden, (const T*)w2, ids, weights, y, width, inner, top,    \
                         experts, (const T*)w2x);                                                  \
    else                                                                                           \
      hipLaunchKernelGGL((moe_down_kernel<T, ROWS>), grid2, dim3(256), (size_t)top * inner * 4, s, \
                         (const T*)hidden, (const T*)w2, ids, weights, y, width, inner, top,       \
                         experts, (const T*)w2x);                                                  \
  } while (0)
  if (dtype == PS_F32) {
    if (few) PS_MOE_ROWS(float, 2);
    else PS_MOE_ROWS(float, 4);
  } else {
    if (few) PS_MOE_ROWS(bf16_t, 2);
    else PS_MOE_ROWS(bf16_t, 4);
  }
#undef PS_MOE_ROWS
#undef PS_MOE_HIDDEN
  PS_CHECK_LAUNCH("ps_moe_experts");
  return 0;
}

extern "C" int ps_moe_grouped_tiles(int pairs, int experts) {
  return (pairs + MOE_TILE - 1) / MOE_TILE + experts;
}

extern "C" int ps_moe_experts_grouped(const void* x, int64_t x_ld, const void* w1, const void* w2,
                                      const int* ids, const float* weights, void* hidden,
                                      float* out, int* order, int* tile_expert, float* y,
                                      int tokens, int width, int inner, int experts, int top,
                                      int gated, void* stream) {
  PS_REQUIRE(tokens >= 0 && width > 0 && inner > 0 && top > 0 && experts > 0 &&
                 experts <= MOE_MAX_EXPERTS, "ps_moe_experts_grouped: bad sizes");
  PS_REQUIRE(width % 8 == 0 && inner % 8 == 0 && x_ld % 8 == 0,
             "ps_moe_experts_grouped: width %d and inner width %d must be multiples of 8", width, inner);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int pairs = tokens * top;
  const int tiles = ps_moe_grouped_tiles(pairs, experts);
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, s, ids, pairs, experts, order, tile_expert,
                     tiles);
  if (gated)
    hipLaunchKernelGGL(moe_grouped_kernel<1>, dim3(tiles, (inner + 63) / 64), dim3(256), 0, s,
                       (const bf16_t*)x, x_ld, (const bf16_t*)w1, (int64_t)2 * inner * width, 2 * inner,
                       width, order, tile_expert, top, weights, (bf16_t*)hidden, (float*)nullptr,
                       (int64_t)0);
  else
    hipLaunchKernelGGL(moe_grouped_kernel<2>, dim3(tiles, (inner + 127) / 128), dim3(256), 0, s,
                       (const bf16_t*)x, x_ld, (const bf16_t*)w1, (int64_t)inner * width, inner,
                       width, order, tile_expert, top, weights, (bf16_t*)hidden, (float*)nullptr,
                       (int64_t)0);
  hipLaunchKernelGGL(moe_grouped_kernel<0>, dim3(tiles, (width + 63) / 64), dim3(256), 0, s,
                     (const bf16_t*)hidden, (int64_t)inner, (const bf16_t*)w2, (int64_t)width * inner,
                     width, inner, order, tile_expert, top, weights, (bf16_t*)nullptr, out,
                     (int64_t)width);
  hipLaunchKernelGGL(moe_combine_kernel, dim3(tokens), dim3(256), 0, s, out, y, width, top);
  PS_CHECK_LAUNCH("ps_moe_experts_grouped");
  return 0;
}
