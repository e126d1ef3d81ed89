// C interface of libpagedserve_hip.so: the gfx950 kernels of the engine.
//
// Conventions
//   * every function returns 0 on success; otherwise ps_last_error() names the fault
//     (a rejected size, an alignment that a kernel needs, a failed launch);
//   * pointers are device pointers; `stream` is a hipStream_t;
//   * `dtype` is PS_F32 (0) or PS_BF16 (1) and names the storage type of activations,
//     matrices and the cache; norm scales, biases, the residual stream and logits are
//     always float;
//   * matrices are stored [out, in] (row n holds the weights of output n), so a product
//     is C[m, n] = sum_k A[m, k] * W[n, k].
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* ps_last_error(void);
int ps_device_info(int* compute_units, int* lds_bytes, char* arch, int arch_len);

// out[t, :] = scale * table[id(t), :] + (pos_table ? pos_table[positions[t], :] : 0), in float,
// where id(t) = ids[t], or carried[src[t]] if src is given and src[t] >= 0.  norm_gamma (null:
// none): the row is then RMS-normed, out / sqrt(mean(out^2) + norm_eps) * norm_gamma.
int ps_embed(const void* table, const void* pos_table, const int* ids, const int* src,
             const int* carried, const int* positions, float* out, int tokens, int width,
             int vocab, int max_positions, float scale, const float* norm_gamma, float norm_eps,
             int dtype, void* stream);

// out[r, :] = norm(x[rows ? rows[r] : r, :]) * gamma (+ beta).  rms != 0: no mean, no beta.
int ps_norm(const float* x, const int* rows, const float* gamma, const float* beta, void* out,
            int n_rows, int width, float eps, int rms, int out_dtype, void* stream);

// C[m, n] = epilogue(sum_k A[m, k] W[n, k] + bias[n]).
//   c_dtype is the storage type of C; PS_EPI_RESIDUAL needs float C and adds into it.
int ps_gemm_nt(const void* a, const void* w, const float* bias, void* c, int m, int n, int k,
               int lda, int ldc, int dtype, int c_dtype, int epilogue, void* stream);

// A linear layer with what may be fused around it.
//   * norm_h != null: the input rows are norm(norm_h[norm_rows ? norm_rows[r] : r]) * gamma
//     (+ beta) instead of `a`; `norm_out` ([m, k] of `dtype`) is scratch for when the norm
//     cannot be fused into the product (it is fused for bfloat16, m <= 16, k <= 1024);
//   * k_pool != null: the output is [q | k | v] columns (q_cols, then kv_cols twice); besides
//     being written to c, the k and v columns of row t are stored in the cache at the page
//     slot of position tok_pos[t] of item tok_item[t] (what ps_kv_write does).
//   * w_packed != null (bfloat16, k a multiple of 64): a second copy of w for the products of
//     few rows, which stream the weights once and are bound by how they read them.  Rows are
//     padded to a multiple of 16; the 16 x 64 tile of rows 16 t .. 16 t + 15 and columns
//     64 s .. 64 s + 63 lies at element ((t * (k / 64) + s) * 1024 as two runs of 512: run h
//     holds, for lane = g * 16 + r (g = 0..3, r = 0..15), the 8 values w[16 t + r][64 s + 16 g +
//     8 h ..]: the order in which a wave's lanes hold the operand of v_mfma_f32_16x16x32_bf16,
//     so that one load of a wave is 1 KB of consecutive memory.
//   * packed activations: between two products of 17 to 64 rows (a decode step of a larger
//     batch) the rows may be kept in the order in which the second product's lanes hold their
//     operand, rows in blocks of 16 and tiles of 16 x 64 as for w_packed; it is bound by the
//     loads of its activations as much as of its weights.  The norm in front of a product is
//     written that way by ps_linear itself; for c the caller asks (c_packed_request, bfloat16
//     output, n a multiple of 64, no residual epilogue, no scatter), is told through c_layout,
//     and passes a_packed to the call that reads the buffer.
typedef struct PsLinearArgs {
  const void* a;
  const void* w;
  const float* bias;
  void* c;
  int m, n, k, lda, ldc;
  int dtype, c_dtype, epilogue;
  const float* norm_h;
  const int* norm_rows;
  const float* gamma;
  const float* beta;
  void* norm_out;
  float eps;
  int rms;
  int ldh;
  void* k_pool;
  void* v_pool;
  const int* tok_item;
  const int* tok_pos;
  const int* tables;
  int table_width, q_cols, kv_cols, head_dim, kv_heads, page_size, num_pages;
  const void* w_packed;   // null, or the copy of w described above
  int a_packed;           // the rows of a lie in the packed activation order (see below)
  int c_packed_request;   // c may be written in that order if the kernel chosen can
  int c_rows;             // rows that c has room for (the packed order rounds m up to 16)
  int norm_out_rows;      // rows that norm_out has room for
  int* c_layout;          // null, or where ps_linear says how it wrote c: 0 rows, 1 packed
  // Null, or: the caller also wants tokens[r] = the column of the largest value of row r of c
  // (the lowest such column on ties), as ps_sample gives it without a temperature.  Float
  // output and the plain epilogue only.  The kernels for few bfloat16 rows do it in their
  // epilogue and *top_done becomes 1; otherwise it becomes 0, nothing is written to tokens,
  // and the caller runs ps_sample.  top_keys: m * 16 * 32 64-bit words, top_ticket: 17 * 64 ints; both
  // zero before the first call and left at zero by every call, and not shared by launches
  // that may overlap.
  int* top_tokens;
  void* top_keys;
  int* top_ticket;
  int* top_done;
  // With a scatter: nobody reads the key and value columns of c (attention takes them from
  // the pages), so a kernel may leave them unwritten; they are unspecified afterwards.  The
  // tiled kernel for many rows does, which takes 40 % off what a prompt's QKV product writes.
  int scatter_only;
} PsLinearArgs;

int ps_linear(const PsLinearArgs* args, void* stream);
int ps_linear_args_size(void);   // sizeof(PsLinearArgs) as this library was built

// Store keys and values of the step's tokens into their pages.
//   k, v: [tokens, kv_heads * head_dim] with row stride `stride`;
//   pools: [pages, kv_heads, page_size, head_dim].
int ps_kv_write(const void* k, const void* v, int64_t stride, void* k_pool, void* v_pool,
                const int* tok_item, const int* tok_pos, const int* tables, int table_width,
                int tokens, int kv_heads, int head_dim, int page_size, int num_pages, int dtype,
                void* stream);

// Attention of `tokens` tokens of the step (those listed in tok_list, or all when it is
// null) over their requests' cached keys 0..position (or the last `window` of them), one
// wave per (token, head).  Any head_dim from 1 to 256; heads must be a multiple of kv_heads.
// sink: null, or one float per head that enters the softmax's denominator as exp(sink[head])
// (a score without key or value, not scaled); gate: null, or a float per token and head, rows
// gate_ld apart: the output of token t and head h is multiplied by sigmoid(gate[t * gate_ld + h]);
// the same in the attention kernels below (ps_attention_decode_partial leaves the gate to
// whoever merges its records).  softcap: 0, or c > 0: a scaled score s enters the softmax as
// c * tanh(s / c).
int ps_attention_rowwise(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                         void* out, int64_t out_stride, const int* tok_list, const int* tok_item,
                         const int* tok_pos, const int* tables, int table_width, int tokens,
                         int heads, int kv_heads, int head_dim, int page_size, int num_pages,
                         float scale, int window, const float* sink, const float* gate,
                         int64_t gate_ld, float softcap, int dtype, void* stream);

// The same result in true 32-bit for the items of several tokens (prompt portions), a block
// of four waves per (tile of ps_attention_tiled_f32_tile() queries, head): float pools, float
// q and out, keys and values through LDS, scores by plain fused multiply-adds.  The tiles are
// listed as for ps_attention_prefill (item and first query of each, cut at the tile size).
// head_dim a multiple of 4 up to 128 (ps_attention_tiled_f32_supported); 16-byte aligned rows.
int ps_attention_tiled_f32_supported(int head_dim);
int ps_attention_tiled_f32_tile();
int ps_attention_tiled_f32(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                           void* out, int64_t out_stride, const int* tile_item, const int* tile_q0,
                           int tiles, const int* cu_tokens, const int* kv_lens, const int* tables,
                           int table_width, int heads, int kv_heads, int head_dim, int page_size,
                           int num_pages, float scale, int window, const float* sink, const float* gate,
                           int64_t gate_ld, float softcap, void* stream);

// The same result for single queries, with each token's keys cut into `splits` ranges that
// run as separate blocks of `waves` (4 or 16) waves; `partial` is scratch of
// count * heads * splits * (head_dim + 2) floats (unused when splits == 1).  head_dim is a
// multiple of 8 up to 256.  tok_item may be null (here and in the two variants below): token t
// is then item t, row t of `tables`, as in a step of single tokens, and the kernel asks for its
// block table beside the position instead of behind the item index.
int ps_attention_decode(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                        void* out, int64_t out_stride, float* partial, int64_t partial_floats,
                        const int* tok_list, const int* tok_item, const int* tok_pos,
                        const int* tables, int table_width, int count, int heads, int kv_heads,
                        int head_dim, int page_size, int num_pages, float scale, int window,
                        int splits, int waves, const float* sink, const float* gate, int64_t gate_ld,
                        float softcap, int dtype, void* stream);

// The same result for bfloat16 layers whose query heads share key/value heads in large groups
// (one cached row that all heads read): a block takes a token's heads of one group (up to 16)
// and a range of keys, loads the keys once and serves every head on the matrix cores.  `partial`
// (count * heads * splits * (head_dim + 2) floats) is needed with one range too; no sink.
// v_pool may be k_pool.
int ps_attention_decode_shared(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                               void* out, int64_t out_stride, float* partial, int64_t partial_floats,
                               const int* tok_list, const int* tok_item, const int* tok_pos,
                               const int* tables, int table_width, int count, int heads, int kv_heads,
                               int head_dim, int page_size, int num_pages, float scale, int window,
                               int splits, const float* gate, int64_t gate_ld, float softcap,
                               void* stream);

// Only the records of ps_attention_decode: (unnormalised sum of values [head_dim], maximum in
// units of log 2, sum) per (token, head, range) at partial[((n * heads + head) * splits + s) *
// (head_dim + 2)], also with one range; nothing is merged and no output rows are written.
int ps_attention_decode_partial(const void* q, int64_t q_stride, const void* k_pool,
                                const void* v_pool, float* partial, int64_t partial_floats,
                                const int* tok_list, const int* tok_item, const int* tok_pos,
                                const int* tables, int table_width, int count, int heads,
                                int kv_heads, int head_dim, int page_size, int num_pages,
                                float scale, int window, int splits, int waves, const float* sink,
                                float softcap, int dtype, void* stream);

// The merge of those records inside the output projection, for up to 16 tokens and head sizes
// that are multiples of 64 (bfloat16 weights in their packed copy, n output columns,
// k = heads * head_dim):  residual[t(r), :] += merged context of row r  W^T + bias, where
// t(r) = tok_list ? tok_list[r] : r.  One wave per (tile of 16 columns, head), up to four heads
// to a block, whose sum is added with float atomics.  tiles_per_block: 0 (the library chooses),
// or the heads per block: 1, 2 or 4.
int ps_attention_merge_linear(const float* partial, int64_t partial_floats, const int* tok_list,
                              int count, int heads, int head_dim, int splits,
                              const void* w_packed, const float* bias, float* residual,
                              int64_t ld_res, int n, int tiles_per_block, void* stream);

// ps_attention_decode for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
// reference.  The partial results of the key ranges go into a device array that is part of the
// library (PS_DECODE_STATIC_SCRATCH_FLOATS floats = 8 MiB, held by every GPU the library runs
// on until the process ends) instead of a buffer of the caller; the call allocates and frees
// nothing.  count * heads * splits * (head_dim + 2) beyond that size is refused with an error.
// All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
// streams, or threads) race on it and give wrong results; calls on one stream are ordered and
// safe.  Nothing in the array has to be cleared between calls.
#define PS_DECODE_STATIC_SCRATCH_FLOATS (2 * 1024 * 1024)
int ps_attention_decode_static(const void* q, int64_t q_stride, const void* k_pool,
                               const void* v_pool, void* out, int64_t out_stride,
                               const int* tok_list, const int* tok_item, const int* tok_pos,
                               const int* tables, int table_width, int count, int heads,
                               int kv_heads, int head_dim, int page_size, int num_pages,
                               float scale, int window, int splits, int waves, int dtype,
                               void* stream);

// Tiled attention on the matrix cores for items that bring several tokens (bfloat16, head_dim a
// multiple of 16 up to 256).  Tile i covers queries tile_q0[i] .. tile_q0[i] + 63 of item
// tile_item[i]; cu_tokens and kv_lens describe the step's items.  Blocks start in the order of
// the list (all heads of tile 0, then of tile 1, ...): list the tiles that see the most keys first.
// max_kv_len: no query sees more keys than that (0: unknown); it only steers the launch shape.
// query_tile: the queries per tile that the list was cut for: ps_attention_prefill_query_tile(),
// or, for head sizes up to 128, ps_attention_prefill_small_tile() (steps with so few tiles that
// the larger ones would leave compute units without a block), or, for head sizes up to
// ps_attention_prefill_large_tile_head_dim(), ps_attention_prefill_large_tile() (long prompts:
// a block then takes in half as many keys and values per score).
int ps_attention_prefill(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                         void* out, int64_t out_stride, const int* tile_item, const int* tile_q0,
                         int tiles, const int* cu_tokens, const int* kv_lens, const int* tables,
                         int table_width, int heads, int kv_heads, int head_dim, int page_size,
                         int num_pages, float scale, int window, int max_kv_len, int query_tile,
                         const float* sink, const float* gate, int64_t gate_ld, float softcap,
                         int dtype, void* stream);

// Both of the above in one launch, for a step that has items of one token (tok_list lists the
// `singles` tokens; tok_item and tok_pos are indexed by token as in ps_attention_decode, which
// this computes with one range of keys) and items of several (tiles of
// ps_attention_prefill_query_tile() queries as in ps_attention_prefill): blocks of both kinds
// share the compute units, where two launches would leave most of them waiting twice.
// bfloat16 and head sizes of 16 to 64 in steps of 16 (ps_attention_mixed_supported).
int ps_attention_mixed_supported(int dtype, int head_dim, int table_width);
int ps_attention_mixed(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                       void* out, int64_t out_stride, const int* tok_list, int singles,
                       const int* tok_item, const int* tok_pos, const int* tile_item,
                       const int* tile_q0, int tiles, const int* cu_tokens, const int* kv_lens,
                       const int* tables, int table_width, int heads, int kv_heads, int head_dim,
                       int page_size, int num_pages, float scale, int window, const float* sink,
                       const float* gate, int64_t gate_ld, float softcap, int dtype, void* stream);

// The constants of that kernel that a caller builds its index arrays by: queries per tile (of
// the two sizes), and the widest block table (entries per item) that it takes.
int ps_attention_prefill_query_tile(void);
int ps_attention_prefill_small_tile(void);
int ps_attention_prefill_large_tile(void);
int ps_attention_prefill_large_tile_head_dim(void);
int ps_attention_prefill_table_max(void);

// tokens[r] = argmax (inv_temperature[r] == 0) or a draw from softmax(logits * inv_temperature[r])
// by inverse CDF at uniform[r] in [0, 1).
int ps_sample(const float* logits, int64_t ld, const float* inv_temperature, const float* uniform,
              int* tokens, int rows, int vocab, void* stream);

// Record the launches issued on `stream` between begin and end into an executable graph.
int ps_graph_begin(void* stream);
int ps_graph_end(void* stream, void** exec_out, int* node_count);
int ps_graph_abort(void* stream);
int ps_graph_launch(void* exec, void* stream);
int ps_graph_destroy(void* exec);

// ---- several copies of the residual stream -----------------------------------------------
// x: [tokens, streams, width] float.  One launch does, per token:
//   * if y != null:       x'_t = sum_s mix[s * streams + t] x_s + out_w[t] * y   (all t at once)
//   * if normed != null:  u = sum_s in_w[s] x'_s;  normed = u / sqrt(mean(u^2) + eps) * gamma
//   * if zero != null:    zero[token, :] = 0        (may be the buffer that y was read from)
int ps_hyper_step(float* x, const float* y, const float* mix, const float* out_w,
                  const float* in_w, const float* gamma, float eps, void* normed, float* zero,
                  int tokens, int width, int streams, int out_dtype, void* stream);
// x[t, s, :] = e[t, :];   out[r, :] = sum_s x[rows ? rows[r] : r, s, :].
int ps_streams_expand(const float* e, float* x, int tokens, int width, int streams, void* stream);
int ps_streams_collapse(const float* x, const int* rows, float* out, int n_rows, int width,
                        int streams, void* stream);

// ---- attention: what lies between the projection and the attention kernels ---------------
// proj: [tokens, ld] float with the query, key and value columns at q_col, k_col, v_col
// (heads * key_dim, kv_heads * key_dim, kv_heads * value_dim of them).  Queries and keys are
// normed over their whole row (q_gamma / k_gamma: a weight per column, null: no norm), rotated
// on the first rot_dims dimensions of every head (dimension 2i with 2i+1, angle position *
// freqs[i]), values are kept (v_mode 1: v_first[t] = v) or mixed (v_mode 2: v = (1 - *v_lambda)
// v + *v_lambda v_first[t]); keys and values go into their pages, queries to q_out, every head
// cache_dim wide with zeros behind its own size.
int ps_attention_prepare(const float* proj, int64_t ld, int q_col, int k_col, int v_col,
                         void* q_out, int64_t q_stride, void* k_pool, void* v_pool,
                         const float* q_gamma, const float* k_gamma, float eps, const float* freqs,
                         int rot_dims, void* v_first, const float* v_lambda, int v_mode,
                         const int* tok_item, const int* tok_pos, const int* tables,
                         int table_width, int tokens, int heads, int kv_heads, int key_dim,
                         int value_dim, int cache_dim, int page_size, int num_pages, int v_heads,
                         int store, int q_dim, int q_maps, int dtype, void* stream);
// The same step for layers that treat every head on its own: the first rot_dims dimensions of
// each query and key head rotated (halves != 0: dimension i with i + rot_dims / 2, else 2i with
// 2i + 1; cosine and sine times magnitude), then, with head_norm, every head divided by its root
// mean square over key_dim (no weight); values: the columns at v_col as projected (v_col may be
// k_col: values that are the keys before rotation and norm).  cache_dim up to 256.
int ps_attention_prepare_heads(const float* proj, int64_t ld, int q_col, int k_col, int v_col,
                               void* q_out, int64_t q_stride, void* k_pool, void* v_pool,
                               const float* freqs, int rot_dims, int halves, float magnitude,
                               int head_norm, float eps, const int* tok_item, const int* tok_pos,
                               const int* tables, int table_width, int tokens, int heads,
                               int kv_heads, int key_dim, int value_dim, int cache_dim,
                               int page_size, int num_pages, int dtype, void* stream);
// Latent attention: proj holds per head [dim | rot_dims] query dimensions from q_col on and, from
// kv_col on, a latent of `rank` numbers and one rotated key part of rot_dims.  The token's one
// cached row (k_pool: [pages, 1, page, cache_dim]) becomes [rms_norm(latent) * gamma | rotated key
// part | zeros]; of every head's query row (cache_dim wide) the places rank .. rank + rot_dims - 1
// get the rotated query part and the places behind zeros (the first `rank` are the caller's).
int ps_latent_prepare(const float* proj, int64_t ld, const float* queries, int64_t queries_ld,
                      int q_col, int kv_col, void* q_out,
                      int64_t q_stride, void* k_pool, const float* gamma, float eps,
                      const float* freqs, int rot_dims, int halves, float magnitude,
                      const int* tok_item, const int* tok_pos, const int* tables, int table_width,
                      int tokens, int heads, int dim, int rank, int cache_dim, int page_size,
                      int num_pages, int dtype, void* stream);
// ctx[t, h, :] *= sigmoid(gate[t * gate_ld + h]).
int ps_head_gate(void* ctx, int64_t stride, const float* gate, int64_t gate_ld, int tokens,
                 int heads, int head_dim, int dtype, void* stream);

// ---- gated linear attention ----------------------------------------------------------------
// alpha[t, c] = sigmoid(z)^(1 / tau) with z = bias[c] + sum_r proj[t, low_col + r] w[c, r].
int ps_gla_decay(const float* proj, int64_t ld, int low_col, int rank, const void* w,
                 const float* bias, float tau, float* alpha, int tokens, int channels, int dtype,
                 void* stream);
// For every item i of the step (tokens cu_tokens[i] .. cu_tokens[i + 1] - 1, state slot
// slots[i]) and head: S = diag(alpha_t) S + k_t v_t^T, out[t] = S^T (q_t * q_scale), token after
// token; state: [max_slots, heads, key_dim, value_dim] float, read at the start and written
// back at the end; out: [tokens, heads * value_dim] float.  longest: no item brings more
// tokens than that (0: unknown); it only steers the launch shape.  head_decay (or null): one
// decay per head that stands for all its key channels and all tokens (alpha is then not read).
// silu_inputs: q, k and v pass silu on their way in.
int ps_gla_scan(const float* proj, int64_t ld, int q_col, int k_col, int v_col,
                const float* alpha, float* state, float* out, const int* cu_tokens,
                const int* slots, int items, int max_slots, int heads, int key_dim, int value_dim,
                float q_scale, int longest, const float* head_decay, int silu_inputs, void* stream);
// Long portions in pieces (recurrences with a decay per head).  ps_scan_pieces cuts the items
// into pieces of `piece` tokens: piece_cu [max_pieces + 1] (empty pieces behind the last),
// item_first [items + 1]; max_pieces >= tokens / piece + items.  ps_decay_join: piece_states
// [max_pieces, heads, per_head] hold what every piece leaves from a zero state and get the
// state at every piece's start; the slots get the items' last states.
int ps_scan_pieces(const int* cu_tokens, int items, int piece, int max_pieces, int* piece_cu,
                   int* item_first, void* stream);
int ps_decay_join(float* piece_states, float* state, const int* piece_cu, const int* item_first,
                  const int* slots, const float* head_decay, int items, int heads, int per_head,
                  void* stream);
// out[t, :] = rms_norm(o[t, :]) * w * sigmoid(gate[t * gate_ld ...]) over the whole row.
int ps_row_norm_gate(const float* o, const float* w, float eps, const float* gate, int64_t gate_ld,
                     void* out, int64_t out_stride, int tokens, int columns, int dtype, void* stream);
// out[t, h, :] = rms_norm(o[t, h, :]) * w * silu(gate[t * gate_ld + h * value_dim ...]).
int ps_gla_output(const float* o, const float* w, float eps, const float* gate, int64_t gate_ld,
                  void* out, int64_t out_stride, int tokens, int heads, int value_dim, int dtype,
                  void* stream);

// logits[r, :vocab] = cap * tanh(logits[r, :vocab] / cap), rows ld floats apart.
int ps_softcap(float* logits, int64_t ld, int rows, int vocab, float cap, void* stream);

// ---- selective state-space mixer -------------------------------------------------------------
// state: [slots, channels, states + taps - 1] float per request: the recurrence's numbers of a
// channel and behind them its last taps - 1 raw inputs, oldest first.
// x[t, c] = act(bias[c] + sum_j w[c, j] u[t - taps + 1 + j, c]) with u = proj[:, u_col + c]; inputs
// from before the step come from the slot.  activation: 1 silu, 0 none.  dtype: that of x.
int ps_conv_silu(const float* proj, int64_t ld, int u_col, const float* w, const float* bias,
                 const float* state, int states, void* x, const int* tok_item,
                 const int* cu_tokens, const int* slots, int tokens, int channels, int taps,
                 int activation, int dtype, void* stream);
// dt[t, c] = softplus(bias[c] + sum_r low[t * ld + r] w[c, r]) in float.
int ps_step_size(const float* low, int64_t ld, int rank, const void* w, const float* bias, float* dt,
                 int tokens, int channels, int dtype, void* stream);
// Per item and channel, token after token: S[n] = exp(dt A[n]) S[n] + dt x B_t[n] with
// A = -exp(a_log[c, n]); y = (sum_n S[n] C_t[n] + skip[c] x) * silu(z) with z = proj[:, z_col + c].
// B and C: bc[t * bc_ld + b_col / c_col + n].  Writes the states and the last raw inputs back.
// records / sums (or null for both): scratch of (pieces + items) * channels * states and
// (pieces + items) * channels floats with pieces = ps_selective_pieces(tokens, items); with them
// the items are cut into pieces that run side by side (for steps with long portions).
// dt null: the step sizes are worked out on the way, softplus(step_bias[c] + sum_r bc[t * bc_ld +
// low_col + r] step_w[c, r]) with step_w [channels, rank] of the storage type, rank <= 256.
int ps_selective_pieces(int tokens, int items);
int ps_selective_scan(const void* x, const float* dt, const float* bc, int64_t bc_ld, int b_col,
                      int c_col, const float* proj, int64_t ld, int u_col, int z_col,
                      const float* a_log, const float* skip, float* state, void* y,
                      const int* cu_tokens, const int* slots, int items, int channels, int states,
                      int taps, int tokens, float* records, float* sums, const void* step_w,
                      const float* step_bias, int low_col, int rank, int dtype, void* stream);

// ---- a stream whose sublayers add into a scratch row ------------------------------------------
// h += factor * column_scale * y + bias (y, bias: null for none; column_scale: a float per
// column, null for ones); zero[...] = 0 (may be y); if gamma:
// normed = h / sqrt(mean(h^2) + eps) * gamma.
int ps_stream_step(float* h, const float* y, float factor, const float* column_scale,
                   const float* bias, const float* gamma, float eps, void* normed, float* zero,
                   int tokens, int width, int out_dtype, void* stream);
// out[t, c] = silu(gu[t * ld + c]) * gu[t * ld + inner + c].
int ps_silu_gate(const float* gu, int64_t ld, void* out, int64_t out_ld, int tokens, int inner,
                 int activation, int dtype, void* stream);
// p[t * ld + first + c] = silu(...) in place for c < count.
int ps_silu_columns(float* p, int64_t ld, int first, int count, int tokens, void* stream);
// y += share * (rms_norm(a) * wa + rms_norm(b) * wb) over rows of width floats; a and b are cleared.
int ps_pair_norm_mix(float* a, float* b, const float* wa, const float* wb, float eps, float share,
                     float* y, int tokens, int width, void* stream);

// ---- block-diagonal products -------------------------------------------------------------------
// out[t, b * out_step + j] = (sum_i x[t, b * x_step + i] w[b, j, i] + bias[b * n + j])
//                            * (gate ? sigmoid(gate[t * gate_ld + b * n + j]) : 1)
// for `blocks` matrices w[b] of [n, k]; x and out float or bfloat16 rows (x_ld, out_ld apart),
// w bfloat16, or everything float.
int ps_block_linear(const void* x, int x_dtype, int64_t x_ld, int x_step, const void* w, int w_dtype,
                    const float* bias, void* out, int out_dtype, int64_t out_ld, int out_step,
                    const float* gate, int64_t gate_ld, int blocks, int n, int k, int tokens,
                    void* stream);

// ---- gated linear recurrence with one state per channel ---------------------------------------
// state: [slots, channels, taps] float per request: S and behind it the last taps - 1 raw inputs
// of the short convolution (proj[:, x_col + c], oldest first).  Per item, token after token:
// a = exp(-decay_scale * sigmoid(gr[t, c]) * softplus(lam[c])),
// S = a S + sqrt(1 - a^2) sigmoid(gi[t, c]) u[t, c],
// out[t, c] = S * gelu_tanh(proj[t, y_col + c]); a row of gates (2 * channels floats) holds, for
// every run of `block` channels, their gr and then their gi.
int ps_lru_scan(const float* proj, int64_t ld, int y_col, int x_col, const float* u,
                const float* gates, int block, const float* lam, float decay_scale, float* state, void* out,
                const int* cu_tokens, const int* slots, int items, int tokens, int channels,
                int taps, int dtype, void* stream);

// ---- mixture of experts ------------------------------------------------------------------------
// ids / weights [tokens, top]: the experts that each row of x chooses and s * scale of each
// (softmax over all experts of the 32-bit logits w x; only experts of the keep best of groups
// equal groups of neighbours, a group's score being its largest s).
int ps_moe_route(const void* x, int64_t x_ld, const float* w, int tokens, int width, int experts,
                 int groups, int keep, int top, float scale, int sigmoid, const float* correction,
                 int group_top, int normalise, int fixed, int* ids, float* weights, int dtype,
                 void* stream);
// y[t] += sum_j weights[t, j] W2[e] (silu(W1[e][:inner] x_t) * (W1[e][inner:] x_t)), e = ids[t, j];
// w1: [experts, 2 * inner, width], w2: [experts, width, inner]; hidden: [tokens * top, inner] scratch.
int ps_moe_experts(const void* x, int64_t x_ld, const void* w1, const void* w2, const int* ids,
                   const float* weights, void* hidden, float* y, int tokens, int width, int inner,
                   int top, int gated, int experts, const void* w1x, const void* w2x, int dtype,
                   void* stream);
// The same for many rows in bfloat16 (width and inner multiples of 8): the (token, choice) pairs
// are sorted by expert into tiles of 128 and multiplied on the matrix cores.  order:
// [tiles * 128] int and tile_expert: [tiles] int scratch with tiles = ps_moe_grouped_tiles(tokens *
// top, experts); out: [tokens * top, width] float scratch.
int ps_moe_grouped_tiles(int pairs, int experts);
int ps_moe_experts_grouped(const void* x, int64_t x_ld, const void* w1, const void* w2, const int* ids,
                           const float* weights, void* hidden, float* out, int* order,
                           int* tile_expert, float* y, int tokens, int width, int inner, int experts,
                           int top, int gated, void* stream);

// Differential attention behind the attention kernels: ctx holds two softmax maps per head over
// the same values, cache_dim wide: map m of head h at head `m * heads + h` (map_major) or at head
// `2 * h + m`.
// out[t, h, d] = (o / sqrt(mean_d(o^2) + eps)) * factor * sigmoid(gate[t, h * value_dim + d]) with
// o = map0 - lambda[0] * map1 over the head's value_dim values (gate null: no gate).
int ps_differential_combine(const void* ctx, int64_t ctx_ld, const float* lambda, float factor,
                            float eps, const float* gate, int64_t gate_ld, void* out,
                            int64_t out_ld, int tokens, int heads, int value_dim, int cache_dim,
                            int map_major, int dtype, void* stream);
// The same for decoded tokens, from the records that ps_attention_decode_partial or
// ps_attention_decode_shared (without output rows) left for 2 * heads heads of head_dim: the
// ranges of both maps are merged in float, then as above.
int ps_differential_merge(const float* partial, int64_t partial_floats, const int* tok_list, int count,
                          const float* lambda, float factor, float eps, const float* gate,
                          int64_t gate_ld, void* out, int64_t out_ld, int heads, int head_dim,
                          int value_dim, int splits, int map_major, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
