// Paged attention for single queries whose heads share their keys: the decode kernel for
// layers with many query heads per key/value head (one cached latent row that every head reads,
// or grouped heads with large groups).
//
// ps_attention_decode runs one block per (token, head, range of keys): the heads of a group
// each fetch the same keys again.  Here one block of 256 threads takes (token, up to 16 heads
// of one group, range): a tile of 64 keys (and of their values, unless values and keys are the
// same pool) goes to LDS once, in pieces of 16 bytes, and serves every head, on the matrix
// cores (v_mfma_f32_16x16x32_bf16, the heads in the place of a product's 16 tokens).
//
//   scores   wave w takes keys 16 w .. 16 w + 15 of the tile: S[key][head] = K Q^T, both
//            operands read from LDS as they lie (a lane: 8 consecutive dimensions of one key
//            and of one head's query); scaled in float and laid down as s[head][key].
//   softmax  online per head across the tiles: wave w owns heads w, w + 4, ..; its lanes hold
//            one head's 64 scores, so maximum and sum are wave reductions; p goes to LDS as
//            bfloat16 (the operand of the next product), the head's rescaling factor beside it.
//   values   O^T[dimension][head] = V^T P^T: wave w takes the tiles of 16 dimensions w, w + 4,
//            ..; a lane gathers one dimension of 8 keys from LDS.
//
// Scores, softmax and sums in float.  The block writes one record per head, (unnormalised sum
// [head_dim], maximum in units of log 2, sum), in the layout of ps_attention_decode's records,
// and the launch that merges ranges (attention_decode.hip) follows, also behind a single one.
#include <math.h>

#include <mutex>

#include "common.h"
#include "pagedserve_hip.h"

#define ADS_KEYS 64
#define ADS_HEADS 16
#define ADS_PROW (ADS_KEYS + 8)
#define ADS_LOADS 8           // 16-byte pieces of a tile per thread: 64 keys x 32 pieces / 256

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

int ps_attention_reduce(const float* partial, void* out, int64_t out_stride, const int* tok_list, int count,
                        int heads, int head_dim, int splits, const float* gate, int64_t gate_ld, int dtype,
                        void* stream);

struct AdsArgs {
  const bf16_t* q;
  int64_t q_stride;
  const bf16_t* k_pool;
  const bf16_t* v_pool;
  float* partial;
  const int* tok_list;
  const int* tok_item;
  const int* tok_pos;
  const int* tables;
  int table_width, heads, kv_heads, head_dim, page_size, num_pages;
  float scale_log2;
  int window, splits;
  float softcap_log2;
  int page_shift, pieces_shift;     // log2 of the page size and of head_dim / 8, or -1
};

// dynamic LDS: keys [64][D + 8] bf16 | values the same (absent when they are the keys) |
// queries [16][D + 8] bf16 | p [16][64 + 8] bf16 | scores [16][64] float | m, l, factor [16] float
__global__ __launch_bounds__(256) void attention_decode_shared_kernel(const AdsArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ads_lds[];
  const int D = a.head_dim;
  const int row = D + 8;                         // bf16 per cached row in LDS
  const bool same = a.v_pool == a.k_pool;
  bf16_t* s_k = reinterpret_cast<bf16_t*>(ads_lds);
  bf16_t* s_v = same ? s_k : s_k + ADS_KEYS * row;
  bf16_t* s_q = s_k + (same ? 1 : 2) * ADS_KEYS * row;
  bf16_t* s_p = s_q + ADS_HEADS * row;
  float* s_s = reinterpret_cast<float*>(s_p + ADS_HEADS * ADS_PROW);
  float* s_m = s_s + ADS_HEADS * ADS_KEYS;
  float* s_l = s_m + ADS_HEADS;
  float* s_f = s_l + ADS_HEADS;

  const int n = blockIdx.x;
  const int group = a.heads / a.kv_heads;        // query heads per key/value head
  const int parts = (group + ADS_HEADS - 1) / ADS_HEADS;
  const int kv_head = blockIdx.y / parts;
  const int head0 = kv_head * group + (blockIdx.y % parts) * ADS_HEADS;
  const int nh = min(ADS_HEADS, kv_head * group + group - head0);
  const int split = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int t = a.tok_list ? a.tok_list[n] : n;
  const int pos = a.tok_pos[t];
  const int* table = a.tables + (int64_t)(a.tok_item ? a.tok_item[t] : t) * a.table_width;
  const int first_key = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const int end_key = pos + 1;
  int chunk = (end_key - first_key + a.splits - 1) / a.splits;
  chunk = (chunk + ADS_KEYS - 1) / ADS_KEYS * ADS_KEYS;
  const int range_begin = first_key + split * chunk;
  const int range_end = min(range_begin + chunk, end_key);
  const int pieces = D / 8;                      // 16-byte pieces of a cached row

  // the heads' queries as they are; rows of heads that the block does not have are zero
  for (int i = tid; i < ADS_HEADS * pieces; i += 256) {
    const int h = i / pieces, piece = i - h * pieces;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (h < nh) {
      const bf16_t* src = a.q + (int64_t)t * a.q_stride + (int64_t)(head0 + h) * D + piece * 8;
      v = *reinterpret_cast<const uint4*>(src);
    }
    *reinterpret_cast<uint4*>(s_q + h * row + piece * 8) = v;
  }
  for (int i = tid; i < ADS_HEADS * ADS_PROW / 2; i += 256) reinterpret_cast<uint32_t*>(s_p)[i] = 0u;
  if (tid < ADS_HEADS) {
    s_m[tid] = -INFINITY;
    s_l[tid] = 0.f;
    s_f[tid] = 1.f;
  }
  // O^T: tile j of the wave covers dimensions 16 (wave + 4 j) ..; element i of a lane: dimension
  // 4 g + i of the tile, head r
  f32x4 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int d_tiles = (D + 15) / 16;

  for (int base = range_begin; base < range_end; base += ADS_KEYS) {
    __syncthreads();                             // the tile before is done with (and s_q is there)
    {
      // a thread's pieces of the tile: first every page number, then every row, then LDS, so
      // that the trips to memory overlap
      int key[ADS_LOADS], piece[ADS_LOADS], page[ADS_LOADS];
      bool live[ADS_LOADS];
      uint4 kv[ADS_LOADS], vv[ADS_LOADS];
#pragma unroll
      for (int u = 0; u < ADS_LOADS; ++u) {
        const int i = tid + 256 * u;
        key[u] = a.pieces_shift >= 0 ? i >> a.pieces_shift : i / pieces;
        piece[u] = i - key[u] * pieces;
        const int p = base + key[u];
        live[u] = key[u] < ADS_KEYS && p < range_end;
        const int logical = a.page_shift >= 0 ? p >> a.page_shift : p / a.page_size;
        page[u] = table[live[u] ? logical : 0];
      }
#pragma unroll
      for (int u = 0; u < ADS_LOADS; ++u) {
        const int p = base + key[u];
        const int within = a.page_shift >= 0 ? p & (a.page_size - 1) : p % a.page_size;
        const int safe = min(max(page[u], 0), a.num_pages - 1);
        const int64_t at = (((int64_t)safe * a.kv_heads + kv_head) * a.page_size + within) * D + piece[u] * 8;
        kv[u] = live[u] ? *reinterpret_cast<const uint4*>(a.k_pool + at) : make_uint4(0, 0, 0, 0);
        if (!same) vv[u] = live[u] ? *reinterpret_cast<const uint4*>(a.v_pool + at) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < ADS_LOADS; ++u) {
        if (key[u] < ADS_KEYS) {
          *reinterpret_cast<uint4*>(s_k + key[u] * row + piece[u] * 8) = kv[u];
          if (!same) *reinterpret_cast<uint4*>(s_v + key[u] * row + piece[u] * 8) = vv[u];
        }
      }
    }
    __syncthreads();
    {
      // S[key 16 wave + 4 g + i][head r]
      f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* kr = s_k + (16 * wave + r) * row + 8 * g;
      const bf16_t* qr = s_q + r * row + 8 * g;
      for (int d0 = 0; d0 < D; d0 += 32) {
        uint4 kf = make_uint4(0, 0, 0, 0), qf = make_uint4(0, 0, 0, 0);
        if (d0 + 8 * g < D) {
          kf = *reinterpret_cast<const uint4*>(kr + d0);
          qf = *reinterpret_cast<const uint4*>(qr + d0);
        }
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&kf),
                                                     *reinterpret_cast<const bf16x8*>(&qf), sc, 0, 0, 0);
      }
      *reinterpret_cast<float4*>(s_s + r * ADS_KEYS + 16 * wave + 4 * g) =
          make_float4(sc[0] * a.scale_log2, sc[1] * a.scale_log2, sc[2] * a.scale_log2, sc[3] * a.scale_log2);
    }
    __syncthreads();
    const bool visible = base + lane < range_end;
    for (int h = wave; h < nh; h += 4) {
      float s = s_s[h * ADS_KEYS + lane];
      if (a.softcap_log2 > 0.f) s = capped_score_fast(s, a.softcap_log2);
      if (!visible) s = -INFINITY;
      const float before = s_m[h];
      const float m_new = fmaxf(before, wave_max(s));          // (a tile has at least one visible key)
      const float p = visible ? __builtin_amdgcn_exp2f(s - m_new) : 0.f;
      // the sum is of the rounded weights, which are what multiplies the values
      const bf16_t rounded = float_to_bf16(p);
      const float sum = wave_sum(bf16_to_float(rounded));
      s_p[h * ADS_PROW + lane] = rounded;
      if (lane == 0) {
        const float factor = before == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(before - m_new);
        s_f[h] = factor;
        s_l[h] = s_l[h] * factor + sum;
        s_m[h] = m_new;
      }
    }
    __syncthreads();
    {
      const float factor = s_f[r];
      uint4 pf[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        pf[ks] = *reinterpret_cast<const uint4*>(s_p + r * ADS_PROW + 32 * ks + 8 * g);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int tile = wave + 4 * j;
        if (tile >= d_tiles) break;              // (the same in every lane of the wave)
        const int d = min(16 * tile + r, D - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] *= factor;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          // V^T[dimension d][keys 32 ks + 8 g ..]
          const bf16_t* vr = s_v + (32 * ks + 8 * g) * row + d;
          uint32_t w[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            w[e] = (uint32_t)vr[(2 * e) * row].bits | ((uint32_t)vr[(2 * e + 1) * row].bits << 16);
          const uint4 vf = make_uint4(w[0], w[1], w[2], w[3]);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(&vf),
                                                           *reinterpret_cast<const bf16x8*>(&pf[ks]), acc[j], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();
  // one record per head; a range without keys leaves (0, -inf, 0)
  if (r < nh) {
    float* dst = a.partial + (((int64_t)n * a.heads + head0 + r) * a.splits + split) * (D + 2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tile = wave + 4 * j;
      if (tile >= d_tiles) break;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 16 * tile + 4 * g + i;
        if (d < D) dst[d] = acc[j][i];
      }
    }
    if (wave == 0 && g == 0) {
      dst[D] = s_m[r];
      dst[D + 1] = s_l[r];
    }
  }
}

static int ads_shift(int value) {
  if (value <= 0 || (value & (value - 1)) != 0) return -1;
  int shift = 0;
  while ((1 << shift) < value) ++shift;
  return shift;
}

static size_t ads_lds_bytes(int head_dim, bool same) {
  return ((size_t)((same ? 1 : 2) * ADS_KEYS + ADS_HEADS) * (head_dim + 8) + ADS_HEADS * ADS_PROW) * sizeof(bf16_t) +
         ((size_t)ADS_HEADS * ADS_KEYS + 3 * ADS_HEADS) * sizeof(float);
}

// ps_attention_decode's result for bfloat16 layers, by blocks that share a tile of keys among
// the heads of a group.  `partial`: count * heads * splits * (head_dim + 2) floats, needed with
// one range too.  No sink.  v_pool may be k_pool (the values are the cached keys).
extern "C" int ps_attention_decode_shared(const void* q, int64_t q_stride, const void* k_pool,
                                          const void* v_pool, void* out, int64_t out_stride,
                                          float* partial, int64_t partial_floats, const int* tok_list,
                                          const int* tok_item, const int* tok_pos, const int* tables,
                                          int table_width, int count, int heads, int kv_heads,
                                          int head_dim, int page_size, int num_pages, float scale,
                                          int window, int splits, const float* gate, int64_t gate_ld,
                                          float softcap, void* stream) {
  PS_REQUIRE(count >= 0 && heads > 0 && kv_heads > 0 && page_size > 0 && num_pages > 0 && table_width > 0,
             "ps_attention_decode_shared: bad sizes");
  PS_REQUIRE(heads % kv_heads == 0, "ps_attention_decode_shared: heads (%d) must be a multiple of kv_heads (%d)",
             heads, kv_heads);
  PS_REQUIRE(head_dim > 0 && head_dim % 8 == 0 && head_dim <= 256,
             "ps_attention_decode_shared: head_dim %d must be a multiple of 8 up to 256", head_dim);
  PS_REQUIRE(window >= 0 && splits >= 1 && splits <= 64, "ps_attention_decode_shared: window %d / splits %d",
             window, splits);
  PS_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 &&
                 ((uintptr_t)v_pool % 16) == 0,
             "ps_attention_decode_shared: queries and pools must be aligned to 16 bytes");
  const int group = heads / kv_heads;
  const int parts = (group + ADS_HEADS - 1) / ADS_HEADS;
  PS_REQUIRE((int64_t)kv_heads * parts <= 65535, "ps_attention_decode_shared: too many heads");
  const int64_t need = (int64_t)count * heads * splits * (head_dim + 2);
  PS_REQUIRE(partial != nullptr && partial_floats >= need,
             "ps_attention_decode_shared: the records need %lld floats", (long long)need);
  if (count == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool same = v_pool == k_pool;
  const size_t lds = ads_lds_bytes(head_dim, same);
  static std::once_flag raised;
  // (up to 82 KB: beyond the 64 KB that a kernel may ask for without saying so)
  std::call_once(raised, [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(attention_decode_shared_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)ads_lds_bytes(256, false));
  });
  const AdsArgs a = {(const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, partial,
                     tok_list, tok_item, tok_pos, tables, table_width, heads, kv_heads, head_dim,
                     page_size, num_pages, scale * 1.4426950408889634f, window, splits,
                     softcap * 1.4426950408889634f, ads_shift(page_size), ads_shift(head_dim / 8)};
  hipLaunchKernelGGL(attention_decode_shared_kernel, dim3(count, kv_heads * parts, splits), dim3(256), lds, s, a);
  PS_CHECK_LAUNCH("ps_attention_decode_shared");
  if (out == nullptr) return 0;      // the records are all that is asked for: the caller merges them
  return ps_attention_reduce(partial, out, out_stride, tok_list, count, heads, head_dim, splits, gate, gate_ld,
                             PS_BF16, stream);
}
