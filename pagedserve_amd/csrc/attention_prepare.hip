// Between the projection of an attention layer and the attention itself, one launch, a block
// per token: the float columns [q | k | v] of the projection become
//
//   * queries and keys normed over the WHOLE projection (all heads at once) with a weight per
//     column:  x / sqrt(mean(x^2) + eps) * w          (optional),
//   * rotated by the token's position on the first `rot_dims` dimensions of every head,
//     dimension 2i paired with 2i+1:  (a, b) -> (a cos t - b sin t, b cos t + a sin t) with
//     t = position * freqs[i]                          (optional),
//   * values mixed with the values that an earlier layer left for the same token:
//     v <- (1 - lambda) v + lambda v_first             (v_mode 2; v_mode 1 leaves them there),
//
// and the keys and values go straight into their cache pages while the queries are written in
// the storage type.  Heads are stored `cache_dim` wide (>= the key and the value head size,
// zeros behind), the one head size that the attention kernels then see for all three.
// Norm statistics, angles and the mixing are 32-bit.
//
// `v_heads` < kv_heads: the projection holds that many value heads and key/value head j caches
// value head j % v_heads (several maps of keys over the same values).  `store` 0: the layer reads
// another layer's keys and values; only its queries are prepared.  `q_maps` > 1: a query head has
// `q_dim` dimensions of its own and query head j stands at places (j % q_maps) * q_dim onward of
// its row, zeros elsewhere, so that it meets only its own run of a key head that holds q_maps
// runs side by side (key_dim = q_maps * q_dim; no rotation then).
#include <math.h>

#include "common.h"
#include "pagedserve_hip.h"

template <typename T>
__global__ __launch_bounds__(1024) void attention_prepare_kernel(
    const float* __restrict__ proj, int64_t ld, int q_col, int k_col, int v_col,
    T* __restrict__ q_out, int64_t q_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
    const float* __restrict__ q_gamma, const float* __restrict__ k_gamma, float eps,
    const float* __restrict__ freqs, int rot_dims, T* __restrict__ v_first,
    const float* __restrict__ v_lambda, int v_mode, const int* __restrict__ tok_item,
    const int* __restrict__ tok_pos, const int* __restrict__ tables, int table_width, int heads,
    int kv_heads, int key_dim, int value_dim, int cache_dim, int page_size, int num_pages,
    int v_heads, int store, int q_dim, int q_maps) {
  __shared__ float red[2][16];
  __shared__ float s_cos[128], s_sin[128];   // the token's angles, one per rotated pair of a head
  const int t = blockIdx.x;
  const float* row = proj + (int64_t)t * ld;
  const int pos = tok_pos[t];
  const int q_cols = heads * q_dim, k_cols = kv_heads * key_dim;
  const int logical = pos / page_size;
  int page = -1;
  if (logical < table_width) page = tables[(int64_t)tok_item[t] * table_width + logical];
  const bool stored = page >= 0 && page < num_pages;
  const int offset = pos - logical * page_size;
  const int half = cache_dim / 2;   // cache_dim is even
  // Queries and keys, a pair of neighbouring dimensions per thread and turn.  A pair's values
  // and weights do not wait for the norms: a thread loads its first pair
  // before the block meets for the sums of squares (which the same values feed), so that a
  // step of few tokens makes one trip to memory; further pairs of a thread are read again.
  const int q_pairs = heads * half, k_pairs = store ? kv_heads * half : 0;
  struct Pair {
    float a, b, wa, wb;
    int head, d0;
    bool is_q;
  };
  auto load_pair = [&](const int i) -> Pair {
    Pair p;
    p.is_q = i < q_pairs;
    const int j = p.is_q ? i : i - q_pairs;
    p.head = j / half;
    p.d0 = (j - p.head * half) * 2;
    // the head's own dimensions: `own` of them, from place `begin` of its row on
    const int own = p.is_q ? q_dim : key_dim;
    const int begin = p.is_q ? (p.head % q_maps) * q_dim : 0;
    const int at = p.d0 - begin;
    const int src = (p.is_q ? q_col : k_col) + p.head * own + at;
    const float* gamma = p.is_q ? q_gamma : k_gamma;
    const bool has_a = at >= 0 && at < own, has_b = at + 1 >= 0 && at + 1 < own;
    p.a = has_a ? row[src] : 0.f;
    p.b = has_b ? row[src + 1] : 0.f;
    p.wa = (gamma && has_a) ? gamma[p.head * own + at] : 1.f;
    p.wb = (gamma && has_b) ? gamma[p.head * own + at + 1] : 1.f;
    return p;
  };
  const int pairs = q_pairs + k_pairs;
  // every head turns by the same angles: they are worked out once per token, not once per head
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) sincosf((float)pos * freqs[i], &s_sin[i], &s_cos[i]);
  const bool has_first = (int)threadIdx.x < pairs;
  Pair first = {};
  if (has_first) first = load_pair(threadIdx.x);
  float q_inv = 1.f, k_inv = 1.f;
  if (q_gamma != nullptr || k_gamma != nullptr) {
    float q_sum = 0.f, k_sum = 0.f;
    if (has_first) {
      const float sq = first.a * first.a + first.b * first.b;
      if (first.is_q) q_sum = sq; else k_sum = sq;
    }
    for (int i = threadIdx.x + blockDim.x; i < pairs; i += blockDim.x) {
      const Pair p = load_pair(i);
      const float sq = p.a * p.a + p.b * p.b;
      if (p.is_q) q_sum += sq; else k_sum += sq;
    }
    q_sum = wave_sum(q_sum);
    k_sum = wave_sum(k_sum);
    const int wave = threadIdx.x >> 6;
    const int waves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) {
      red[0][wave] = q_sum;
      red[1][wave] = k_sum;
    }
    __syncthreads();
    q_sum = 0.f;
    k_sum = 0.f;
    for (int w = 0; w < waves; ++w) {
      q_sum += red[0][w];
      k_sum += red[1][w];
    }
    if (q_gamma != nullptr) q_inv = 1.0f / sqrtf(q_sum / (float)q_cols + eps);
    if (k_gamma != nullptr) k_inv = 1.0f / sqrtf(k_sum / (float)k_cols + eps);
  } else {
    __syncthreads();      // the angles
  }
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const Pair p = i == (int)threadIdx.x ? first : load_pair(i);
    const float inv = p.is_q ? q_inv : k_inv;
    const float a = p.a * inv * p.wa, b = p.b * inv * p.wb;
    const bool turned = p.d0 + 1 < rot_dims;
    const float cs = turned ? s_cos[p.d0 >> 1] : 1.f, sn = turned ? s_sin[p.d0 >> 1] : 0.f;
    const float ra = a * cs - b * sn;
    const float rb = b * cs + a * sn;
    if (p.is_q) {
      T* dst = q_out + (int64_t)t * q_stride + (int64_t)p.head * cache_dim + p.d0;
      dst[0] = from_float<T>(ra);
      dst[1] = from_float<T>(rb);
    } else if (stored) {
      T* dst = k_pool + (((int64_t)page * kv_heads + p.head) * page_size + offset) * cache_dim + p.d0;
      dst[0] = from_float<T>(ra);
      dst[1] = from_float<T>(rb);
    }
  }
  const float lambda = v_mode == 2 ? v_lambda[0] : 0.f;
  for (int i = threadIdx.x; i < (store ? kv_heads * cache_dim : 0); i += blockDim.x) {
    const int head = i / cache_dim;
    const int d = i - head * cache_dim;
    float v = 0.f;
    if (d < value_dim) {
      v = row[v_col + (head % v_heads) * value_dim + d];
      const int64_t at = ((int64_t)t * kv_heads + head) * value_dim + d;
      if (v_mode == 1) v_first[at] = from_float<T>(v);
      if (v_mode == 2) v = (1.f - lambda) * v + lambda * to_float<T>(v_first[at]);
    }
    if (stored)
      v_pool[(((int64_t)page * kv_heads + head) * page_size + offset) * cache_dim + d] = from_float<T>(v);
  }
}

extern "C" int ps_attention_prepare(const float* proj, int64_t ld, int q_col, int k_col, int v_col,
                                    void* q_out, int64_t q_stride, void* k_pool, void* v_pool,
                                    const float* q_gamma, const float* k_gamma, float eps,
                                    const float* freqs, int rot_dims, void* v_first,
                                    const float* v_lambda, int v_mode, const int* tok_item,
                                    const int* tok_pos, const int* tables, int table_width,
                                    int tokens, int heads, int kv_heads, int key_dim,
                                    int value_dim, int cache_dim, int page_size, int num_pages,
                                    int v_heads, int store, int q_dim, int q_maps, int dtype,
                                    void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0 &&
                 page_size > 0 && num_pages > 0 && table_width > 0,
             "ps_attention_prepare: bad sizes");
  PS_REQUIRE(cache_dim >= key_dim && cache_dim >= value_dim && cache_dim % 2 == 0,
             "ps_attention_prepare: cached head size %d must be even and hold keys of %d and values of %d",
             cache_dim, key_dim, value_dim);
  PS_REQUIRE(rot_dims <= 256, "ps_attention_prepare: %d rotated dimensions, the kernel keeps angles for 256", rot_dims);
  PS_REQUIRE(rot_dims >= 0 && rot_dims <= key_dim && rot_dims % 2 == 0,
             "ps_attention_prepare: %d rotated dimensions do not fit heads of %d", rot_dims, key_dim);
  PS_REQUIRE(rot_dims == 0 || freqs != nullptr, "ps_attention_prepare: rotation without frequencies");
  PS_REQUIRE(v_mode >= 0 && v_mode <= 2 && (v_mode == 0 || v_first != nullptr) &&
                 (v_mode != 2 || v_lambda != nullptr),
             "ps_attention_prepare: value mixing needs its buffer and its weight");
  PS_REQUIRE(q_stride >= (int64_t)heads * cache_dim, "ps_attention_prepare: query rows too short");
  PS_REQUIRE(v_heads >= 1 && v_heads <= kv_heads && kv_heads % v_heads == 0 &&
                 (v_mode == 0 || v_heads == kv_heads),
             "ps_attention_prepare: %d value heads under %d key heads", v_heads, kv_heads);
  PS_REQUIRE(q_maps >= 1 && q_dim >= 1 && q_maps * q_dim <= cache_dim &&
                 (q_maps == 1 ? q_dim == key_dim : (rot_dims == 0 && q_maps * q_dim == key_dim)),
             "ps_attention_prepare: %d runs of %d query dimensions do not fit keys of %d", q_maps, q_dim,
             key_dim);
  PS_REQUIRE((q_gamma == nullptr && k_gamma == nullptr) || eps > 0.f, "ps_attention_prepare: eps must be positive");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_attention_prepare: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  // as many threads as the widest of the three passes has elements (the queries' columns, the
  // pairs of queries and keys), so that a pass is one round of loads where the row allows
  int widest = heads * key_dim;
  if ((heads + kv_heads) * (cache_dim / 2) > widest) widest = (heads + kv_heads) * (cache_dim / 2);
  int threads = widest >= 1024 ? 1024 : (widest + 63) / 64 * 64;
  if (tokens > 256 && threads > 256) threads = 256;   // (many rows fill the chip anyway)
  if (dtype == PS_F32)
    hipLaunchKernelGGL(attention_prepare_kernel<float>, dim3(tokens), dim3(threads), 0, s, proj, ld, q_col,
                       k_col, v_col, (float*)q_out, q_stride, (float*)k_pool, (float*)v_pool, q_gamma,
                       k_gamma, eps, freqs, rot_dims, (float*)v_first, v_lambda, v_mode, tok_item,
                       tok_pos, tables, table_width, heads, kv_heads, key_dim, value_dim, cache_dim,
                       page_size, num_pages, v_heads, store, q_dim, q_maps);
  else
    hipLaunchKernelGGL(attention_prepare_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, s, proj, ld, q_col,
                       k_col, v_col, (bf16_t*)q_out, q_stride, (bf16_t*)k_pool, (bf16_t*)v_pool,
                       q_gamma, k_gamma, eps, freqs, rot_dims, (bf16_t*)v_first, v_lambda, v_mode,
                       tok_item, tok_pos, tables, table_width, heads, kv_heads, key_dim, value_dim,
                       cache_dim, page_size, num_pages, v_heads, store, q_dim, q_maps);
  PS_CHECK_LAUNCH("ps_attention_prepare");
  return 0;
}

// ctx[t, h, :] *= sigmoid(gate[t, h]): a gate per token and head on the attention's output.
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ ctx, int64_t stride, const float* __restrict__ gate,
                                 int64_t gate_ld, int heads, int head_dim) {
  const int t = blockIdx.x;
  const int row = heads * head_dim;
  for (int i = threadIdx.x; i < row; i += blockDim.x) {
    const int head = i / head_dim;
    const float g = gate[(int64_t)t * gate_ld + head];
    const float s = 1.0f / (1.0f + expf(-g));
    T* p = ctx + (int64_t)t * stride + i;
    *p = from_float<T>(to_float<T>(*p) * s);
  }
}

extern "C" int ps_head_gate(void* ctx, int64_t stride, const float* gate, int64_t gate_ld,
                            int tokens, int heads, int head_dim, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && head_dim > 0 && stride >= (int64_t)heads * head_dim &&
                 gate_ld >= heads,
             "ps_head_gate: bad sizes");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_head_gate: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = heads * head_dim >= 256 ? 256 : 64;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(head_gate_kernel<float>, dim3(tokens), dim3(threads), 0, s, (float*)ctx, stride,
                       gate, gate_ld, heads, head_dim);
  else
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, s, (bf16_t*)ctx,
                       stride, gate, gate_ld, heads, head_dim);
  PS_CHECK_LAUNCH("ps_head_gate");
  return 0;
}

// The angle's cosine and sine of rotated dimension d of a head, by the layout of the pairs:
// halves (dimension i with i + rot_dims / 2) or neighbours (2i with 2i + 1).
struct RotationPlace {
  int partner;     // the other dimension of the pair
  int angle;       // index of the pair's frequency
  float sign;      // -1 for the pair's first dimension, +1 for its second
};
__device__ inline RotationPlace rotation_place(int d, int rot_dims, bool halves) {
  RotationPlace p;
  if (halves) {
    const int half = rot_dims >> 1;
    const bool first = d < half;
    p.partner = first ? d + half : d - half;
    p.angle = first ? d : d - half;
    p.sign = first ? -1.f : 1.f;
  } else {
    const bool first = (d & 1) == 0;
    p.partner = first ? d + 1 : d - 1;
    p.angle = d >> 1;
    p.sign = first ? -1.f : 1.f;
  }
  return p;
}

// The same step for layers that treat every head on its own: the first `rot_dims` dimensions
// of each query and key head are rotated by the token's position (pairs laid out as halves
// or as neighbours; cosine and sine times `magnitude`), then, with head_norm, each head is
// divided by its root mean square over its key_dim dimensions (no weight).  Values are the
// columns at v_col as projected (they may be the key columns themselves: values that are the
// unrotated, unnormed keys).  A block per token, a wave per head in turn; a lane holds up to
// four dimensions of the head.
template <typename T>
__global__ __launch_bounds__(256) void attention_prepare_heads_kernel(
    const float* __restrict__ proj, int64_t ld, int q_col, int k_col, int v_col,
    T* __restrict__ q_out, int64_t q_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
    const float* __restrict__ freqs, int rot_dims, int halves, float magnitude, int head_norm,
    float eps, const int* __restrict__ tok_item, const int* __restrict__ tok_pos,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int key_dim,
    int value_dim, int cache_dim, int page_size, int num_pages) {
  __shared__ float s_cos[128], s_sin[128];
  const int t = blockIdx.x;
  const float* row = proj + (int64_t)t * ld;
  const int pos = tok_pos[t];
  const int logical = pos / page_size;
  int page = -1;
  if (logical < table_width) page = tables[(int64_t)tok_item[t] * table_width + logical];
  const bool stored = page >= 0 && page < num_pages;
  const int offset = pos - logical * page_size;
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
    float sn, cs;
    sincosf((float)pos * freqs[i], &sn, &cs);
    s_cos[i] = cs * magnitude;
    s_sin[i] = sn * magnitude;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int hh = wave; hh < heads + kv_heads; hh += waves) {
    const bool is_q = hh < heads;
    const int head = is_q ? hh : hh - heads;
    const float* src = row + (is_q ? q_col : k_col) + head * key_dim;
    float value[4];
    float squares = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = lane + 64 * r;
      float v = 0.f;
      if (d < key_dim) {
        v = src[d];
        if (d < rot_dims) {
          const RotationPlace place = rotation_place(d, rot_dims, halves != 0);
          v = v * s_cos[place.angle] + place.sign * src[place.partner] * s_sin[place.angle];
        }
      }
      value[r] = v;
      squares = fmaf(v, v, squares);
    }
    float inv = 1.f;
    if (head_norm) inv = 1.0f / sqrtf(wave_sum(squares) / (float)key_dim + eps);
    T* dst = nullptr;
    if (is_q) dst = q_out + (int64_t)t * q_stride + (int64_t)head * cache_dim;
    else if (stored) dst = k_pool + (((int64_t)page * kv_heads + head) * page_size + offset) * cache_dim;
    if (dst != nullptr) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d = lane + 64 * r;
        if (d < cache_dim) dst[d] = from_float<T>(value[r] * inv);   // (zeros behind key_dim)
      }
    }
  }
  if (!stored) return;
  for (int i = threadIdx.x; i < kv_heads * cache_dim; i += blockDim.x) {
    const int head = i / cache_dim;
    const int d = i - head * cache_dim;
    const float v = d < value_dim ? row[v_col + head * value_dim + d] : 0.f;
    v_pool[(((int64_t)page * kv_heads + head) * page_size + offset) * cache_dim + d] = from_float<T>(v);
  }
}

extern "C" int ps_attention_prepare_heads(const float* proj, int64_t ld, int q_col, int k_col,
                                          int v_col, void* q_out, int64_t q_stride, void* k_pool,
                                          void* v_pool, const float* freqs, int rot_dims,
                                          int halves, float magnitude, int head_norm, float eps,
                                          const int* tok_item, const int* tok_pos,
                                          const int* tables, int table_width, int tokens, int heads,
                                          int kv_heads, int key_dim, int value_dim, int cache_dim,
                                          int page_size, int num_pages, int dtype, void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0 &&
                 page_size > 0 && num_pages > 0 && table_width > 0,
             "ps_attention_prepare_heads: bad sizes");
  PS_REQUIRE(cache_dim >= key_dim && cache_dim >= value_dim && cache_dim <= 256,
             "ps_attention_prepare_heads: cached head size %d must hold keys of %d and values of %d, up to 256",
             cache_dim, key_dim, value_dim);
  PS_REQUIRE(rot_dims >= 0 && rot_dims <= key_dim && rot_dims % 2 == 0,
             "ps_attention_prepare_heads: %d rotated dimensions do not fit heads of %d", rot_dims, key_dim);
  PS_REQUIRE(rot_dims == 0 || freqs != nullptr, "ps_attention_prepare_heads: rotation without frequencies");
  PS_REQUIRE(q_stride >= (int64_t)heads * cache_dim, "ps_attention_prepare_heads: query rows too short");
  PS_REQUIRE(!head_norm || eps > 0.f, "ps_attention_prepare_heads: eps must be positive");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_attention_prepare_heads: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(attention_prepare_heads_kernel<float>, dim3(tokens), dim3(256), 0, s, proj, ld,
                       q_col, k_col, v_col, (float*)q_out, q_stride, (float*)k_pool, (float*)v_pool,
                       freqs, rot_dims, halves, magnitude, head_norm, eps, tok_item, tok_pos, tables,
                       table_width, heads, kv_heads, key_dim, value_dim, cache_dim, page_size, num_pages);
  else
    hipLaunchKernelGGL(attention_prepare_heads_kernel<bf16_t>, dim3(tokens), dim3(256), 0, s, proj, ld,
                       q_col, k_col, v_col, (bf16_t*)q_out, q_stride, (bf16_t*)k_pool, (bf16_t*)v_pool,
                       freqs, rot_dims, halves, magnitude, head_norm, eps, tok_item, tok_pos, tables,
                       table_width, heads, kv_heads, key_dim, value_dim, cache_dim, page_size, num_pages);
  PS_CHECK_LAUNCH("ps_attention_prepare_heads");
  return 0;
}

// Latent attention, between its projection and the attention kernels.  The float row of a
// token holds, per head, [dim unrotated | rot_dims rotated] query dimensions from q_col on, and
// from kv_col on the latent (rank numbers) and one rotated key part (rot_dims) that all heads
// share.  One cached "head" per token, cache_dim wide:
//
//   key row   = [ latent / rms(latent) * gamma | rotated key part | zeros ]
//   query row = [ (left to the caller: the head's unrotated part taken through the transposed
//                 key matrix, rank numbers) | rotated query part | zeros ]      per head
//
// so that a query's product with a key row is the score, and the weighted sum of the key rows
// holds the weighted latent in its first `rank` places.  A block per token.
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const float* __restrict__ proj, int64_t ld, const float* __restrict__ queries, int64_t queries_ld,
    int q_col, int kv_col, T* __restrict__ q_out,
    int64_t q_stride, T* __restrict__ k_pool, const float* __restrict__ gamma, float eps,
    const float* __restrict__ freqs, int rot_dims, int halves, float magnitude,
    const int* __restrict__ tok_item, const int* __restrict__ tok_pos,
    const int* __restrict__ tables, int table_width, int heads, int dim, int rank, int cache_dim,
    int page_size, int num_pages) {
  __shared__ float s_cos[128], s_sin[128];
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* row = proj + (int64_t)t * ld;
  const float* q_row = queries + (int64_t)t * queries_ld;
  const int pos = tok_pos[t];
  const int logical = pos / page_size;
  int page = -1;
  if (logical < table_width) page = tables[(int64_t)tok_item[t] * table_width + logical];
  const bool stored = page >= 0 && page < num_pages;
  const int offset = pos - logical * page_size;
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
    float sn, cs;
    sincosf((float)pos * freqs[i], &sn, &cs);
    s_cos[i] = cs * magnitude;
    s_sin[i] = sn * magnitude;
  }
  float squares = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) squares = fmaf(row[kv_col + i], row[kv_col + i], squares);
  const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)rank + eps);   // (also the barrier for the angles)
  T* key = stored ? k_pool + ((int64_t)page * page_size + offset) * cache_dim : nullptr;
  if (key != nullptr) {
    for (int i = threadIdx.x; i < rank; i += blockDim.x)
      key[i] = from_float<T>(row[kv_col + i] * inv * gamma[i]);
    for (int i = rank + rot_dims + threadIdx.x; i < cache_dim; i += blockDim.x) key[i] = from_float<T>(0.f);
  }
  // the rotated parts: vector 0 is the key's, vector 1 + h the query's of head h
  const int behind = cache_dim - rank - rot_dims;
  for (int i = threadIdx.x; i < (heads + 1) * rot_dims; i += blockDim.x) {
    const int vec = i / rot_dims;
    const int d = i - vec * rot_dims;
    const float* src = vec == 0 ? row + kv_col + rank : q_row + q_col + (vec - 1) * (dim + rot_dims) + dim;
    const RotationPlace place = rotation_place(d, rot_dims, halves != 0);
    const float v = src[d] * s_cos[place.angle] + place.sign * src[place.partner] * s_sin[place.angle];
    if (vec == 0) {
      if (key != nullptr) key[rank + d] = from_float<T>(v);
    } else {
      q_out[(int64_t)t * q_stride + (int64_t)(vec - 1) * cache_dim + rank + d] = from_float<T>(v);
    }
  }
  for (int i = threadIdx.x; i < heads * behind; i += blockDim.x) {
    const int head = i / behind;
    q_out[(int64_t)t * q_stride + (int64_t)head * cache_dim + rank + rot_dims + (i - head * behind)] =
        from_float<T>(0.f);
  }
}

extern "C" int ps_latent_prepare(const float* proj, int64_t ld, const float* queries,
                                 int64_t queries_ld, int q_col, int kv_col, void* q_out,
                                 int64_t q_stride, void* k_pool, const float* gamma, float eps,
                                 const float* freqs, int rot_dims, int halves, float magnitude,
                                 const int* tok_item, const int* tok_pos, const int* tables,
                                 int table_width, int tokens, int heads, int dim, int rank,
                                 int cache_dim, int page_size, int num_pages, int dtype,
                                 void* stream) {
  PS_REQUIRE(tokens >= 0 && heads > 0 && dim >= 0 && rank > 0 && page_size > 0 && num_pages > 0 &&
                 table_width > 0,
             "ps_latent_prepare: bad sizes");
  PS_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= 256,
             "ps_latent_prepare: %d rotated dimensions: an even number up to 256", rot_dims);
  PS_REQUIRE(rot_dims == 0 || freqs != nullptr, "ps_latent_prepare: rotation without frequencies");
  PS_REQUIRE(cache_dim >= rank + rot_dims, "ps_latent_prepare: cached rows of %d do not hold %d + %d",
             cache_dim, rank, rot_dims);
  PS_REQUIRE(q_stride >= (int64_t)heads * cache_dim, "ps_latent_prepare: query rows too short");
  PS_REQUIRE(gamma != nullptr && eps > 0.f, "ps_latent_prepare: the latent's norm needs its weight and a positive eps");
  PS_REQUIRE(queries != nullptr && queries_ld >= q_col + (int64_t)heads * (dim + rot_dims),
             "ps_latent_prepare: the queries' rows are too short");
  PS_REQUIRE(dtype == PS_F32 || dtype == PS_BF16, "ps_latent_prepare: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PS_F32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(tokens), dim3(256), 0, s, proj, ld, queries, queries_ld, q_col,
                       kv_col, (float*)q_out, q_stride, (float*)k_pool, gamma, eps, freqs, rot_dims,
                       halves, magnitude, tok_item, tok_pos, tables, table_width, heads, dim, rank,
                       cache_dim, page_size, num_pages);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, dim3(tokens), dim3(256), 0, s, proj, ld, queries, queries_ld, q_col,
                       kv_col, (bf16_t*)q_out, q_stride, (bf16_t*)k_pool, gamma, eps, freqs, rot_dims,
                       halves, magnitude, tok_item, tok_pos, tables, table_width, heads, dim, rank,
                       cache_dim, page_size, num_pages);
  PS_CHECK_LAUNCH("ps_latent_prepare");
  return 0;
}
