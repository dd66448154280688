// The C interface of libholon_hip: one function per device operation, raw device pointers, a HIP stream.
// dtype: 0 = float32, 1 = bfloat16 (activations, weights and cache share it). Index arrays are int32.
// Every function returns 0 on success; otherwise holon_last_error() describes what was refused.
#pragma once
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* holon_last_error(void);
int holon_abi_version(void);

// out[t] = table[ids[t]]; with take_slot and last_token (both or neither), token t is last_token[take_slot[t]] where
// take_slot[t] >= 0: a token the previous step drew and left on the device.
// stats_out (nullable, tokens <= 16): [16] float32, the sum of squares of every row written.
int holon_embedding(const int32_t* ids, const int32_t* take_slot, const int32_t* last_token, const void* table, void* out,
                    int tokens, int hidden, int vocab, int dtype, float* stats_out, void* stream);
// stats[m] = sum of squares of row m of x [rows, dim], rows <= 16.
int holon_row_sumsq(const void* x, float* stats, int rows, int dim, int dtype, void* stream);
// y = rmsnorm(x) over rows of `dim`; with `residual`: residual += x (rounded), y = rmsnorm(residual).
int holon_rmsnorm(const void* x, void* residual, const void* weight, void* y, int64_t rows, int dim, float eps,
                  int dtype, void* stream);
// The same with what is added given as float32 sums over shares of K, parts [splits, rows, dim]: residual +=
// round(parts[0] + parts[1] + ...), y = rmsnorm(residual); residual, weight and y bfloat16.
int holon_rmsnorm_parts(const float* parts, int splits, void* residual, const void* weight, void* y, int64_t rows,
                        int dim, float eps, void* stream);
int holon_silu_mul(const void* gate_up, void* out, int64_t tokens, int inter, int dtype, void* stream);
// Per (token, head): optional rmsnorm over head_dim, optional half-split rotation with table[pos] = cos|sin, then
// q -> q_out [T, heads, D]; k, v -> the paged cache (pages == NULL: only q heads are processed).
int holon_qk_norm_rope_write(const void* qkv, int64_t qkv_stride, void* q_out, int tokens, int heads, int kv_heads,
                             int head_dim, const void* q_weight, const void* k_weight, float eps, const float* table,
                             int rotary_dim, int max_positions, const int32_t* positions, void* pages,
                             const int32_t* write_page, const int32_t* write_off, int page_size, int num_pages,
                             int dtype, void* stream);
int holon_kv_write(const void* k, const void* v, void* pages, const int32_t* write_page, const int32_t* write_off,
                   int tokens, int kv_heads, int head_dim, int page_size, int num_pages, int dtype, void* stream);
// Attention of every query token over its row's cached keys (any dtype, page size and head_dim % 8 == 0).
int holon_attention_generic(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                            const int32_t* slots, const int32_t* lens, const int32_t* query_start, int rows,
                            int tokens, int heads, int kv_heads, int head_dim, int page_size, int num_pages,
                            float scale, int window, int dtype, void* stream);
// Matrix-core attention (bfloat16, head_dim 64/128/256, page_size % 16 == 0). `row_ids` lists the rows served.
int holon_attention_mfma_supported(int head_dim, int page_size, int dtype);
int holon_attention_prefill_bf16(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                                 const int32_t* slots, const int32_t* lens, const int32_t* query_start,
                                 const int32_t* row_ids, int n_rows, int max_query, int max_len, int heads,
                                 int kv_heads, int head_dim, int page_size, float scale, int window, void* stream);
// Which kernel long prompt portions of groups of up to 32 heads take: 0 one tile of 32 rows a wave, 2 two tiles a wave,
// 1 (the default) two from 12,288 keys on. Returns the setting before; a negative argument changes nothing.
int holon_attention_prefill_form(int form);
// 1 (default): long portions at head_dim 128 copy their stages into LDS without passing registers; 0: through registers.
// Returns the setting before; a negative argument only asks.
int holon_attention_prefill_copies(int direct);
// One query token per row; the keys are split over `splits` waves of `keys_per_split` keys (a multiple of 32) whose
// partial results (part_o [n_rows, heads, splits, head_dim], part_ml [n_rows, heads, splits, 2], float32) are merged
// in split order.
int holon_attention_decode_bf16(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                                const int32_t* slots, const int32_t* lens, const int32_t* query_start,
                                const int32_t* row_ids, int n_rows, int max_len, int heads, int kv_heads, int head_dim,
                                int page_size, float scale, int window, float* part_o, float* part_ml, int splits,
                                int keys_per_split, void* stream);
// The same with `waves` waves a block (1 to 8, a divisor of `splits`), whose partials are combined through LDS: a
// (row, head) leaves splits / waves partials (the workspace's third dimension), and when that is one the block writes
// the result itself (the workspace may then be NULL, and no merge runs). rows_in_order: every row of the step is a
// decode row with row_ids[i] = i and query_start[i] = i (neither array is then read).
int holon_attention_decode_waves_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                      int table_stride, const int32_t* slots, const int32_t* lens,
                                      const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                      int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                      float* part_o, float* part_ml, int splits, int keys_per_split, int waves,
                                      int rows_in_order, void* stream);
// The prompt and the decode entry points with a sink per query head in the softmax's denominator (`sink` [heads]
// float32 in the scores' units, or NULL): exp(sink - max) is added to the sum of the weights; it has no key or value.
int holon_attention_prefill_sink_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                      int table_stride, const int32_t* slots, const int32_t* lens,
                                      const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_query,
                                      int max_len, int heads, int kv_heads, int head_dim, int page_size, float scale,
                                      int window, const float* sink, void* stream);
int holon_attention_decode_sink_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                     int table_stride, const int32_t* slots, const int32_t* lens,
                                     const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                     int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                     float* part_o, float* part_ml, int splits, int keys_per_split, int waves,
                                     int rows_in_order, const float* sink, void* stream);
// Both over pages whose key heads share value heads: kv_heads planes of keys, then kv_heads / v_share planes of values
// a page; key head hk reads value head hk / v_share (1: as ever). Sink nullable; softcap 0, r1 = r2 = null,
// keep_first 0: plain scores. hgate (nullable, bfloat16, rows hgate_stride apart): head h's result of token t times
// sigmoid(hgate[t, h]).
int holon_attention_prefill_shared_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                        int table_stride, const int32_t* slots, const int32_t* lens,
                                        const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_query,
                                        int max_len, int heads, int kv_heads, int head_dim, int page_size, float scale,
                                        int window, const float* sink, float softcap, const float* r1, const float* r2,
                                        int keep_first, int v_share, const void* hgate, int64_t hgate_stride,
                                        void* stream);
int holon_attention_decode_shared_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, const int32_t* slots, const int32_t* lens,
                                       const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                       int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                       float* part_o, float* part_ml, int splits, int keys_per_split, int waves,
                                       int rows_in_order, const float* sink, float softcap, const float* r1,
                                       const float* r2, int keep_first, int v_share, const void* hgate,
                                       int64_t hgate_stride, void* stream);
// The same from the step's raw q/k/v projection `qkv` [T, (heads + 2 kv_heads) head_dim]: per-head RMSNorm (q_weight
// and k_weight, both or neither), rotation (rope_table [max_positions, head_dim] = cos | sin, or NULL) and the cache
// write of every row's new token (write_page, write_off by token; its position is the row's len - 1) happen inside
// the attention kernel.
int holon_attention_decode_fused_bf16(const void* qkv, void* out, void* pages, const int32_t* table, int table_stride,
                                      const int32_t* slots, const int32_t* lens, const int32_t* query_start,
                                      const int32_t* row_ids, int n_rows, int max_len, int heads, int kv_heads,
                                      int head_dim, int page_size, float scale, int window, const void* q_weight,
                                      const void* k_weight, float eps, const float* rope_table,
                                      int max_positions, const int32_t* write_page, const int32_t* write_off,
                                      float* part_o, float* part_ml, int splits, int keys_per_split, int waves,
                                      int rows_in_order, void* stream);
// The same decode attention for callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. The split partials that
// holon_attention_decode_bf16 takes as a workspace live in a device array inside the library instead, of
// HOLON_DECODE_SCRATCH_BYTES on every GPU the library runs on, held until the process ends; no call allocates or frees.
// n_rows * heads * splits * (head_dim + 2) floats (the first part rounded up to 256 bytes) must fit, or the call is
// refused. All calls on one GPU share that GPU's array: calls that overlap on one GPU (other streams, other threads)
// race; calls in one stream's order do not. holon_decode_scratch_init() looks the array's address up for the current
// device ahead of time (the entry point does it at its first call on a device otherwise).
#define HOLON_DECODE_SCRATCH_BYTES (16 << 20)
int holon_decode_scratch_init(void);
int64_t holon_decode_scratch_bytes(void);
int holon_attention_decode_bf16_static(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, const int32_t* slots, const int32_t* lens,
                                       const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                       int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                       int splits, int keys_per_split, void* stream);
// y[M, N] = x[M, K] w[N, K]^T for M <= 16 rows, bfloat16 in, float32 accumulation; out_f32: 0 bfloat16 out, 1 float32
// out, 2 float32 out of values rounded to bfloat16 first, 4 bfloat16 out of max(rounded product, 0)^2;
// tiled says that `w` is holon_tile_weight_bf16's copy ([N/16, K/32, 64, 8]: lane-major 16-byte pieces).
int holon_gemm_skinny_supported(int M, int N, int K);
int holon_gemm_skinny_bf16(const void* x, const void* w, void* y, int M, int N, int K, int out_f32, int tiled,
                           void* stream);
// residual[M, N] = round(residual + round(x w^T)) in place, tiled weights: the product and the residual add that
// follows it in one kernel.
// With stats_out ([N / 16, 16] float32): per block of 16 columns, the sums of squares of the residual values written.
int holon_gemm_skinny_add_bf16(const void* x, const void* w_tiled, void* residual, int M, int N, int K, float* stats_out,
                               void* stream);
// A norm folded into the product: w_tiled holds W * diag(g) (holon_tile_weight_bf16 with `scale`), x the un-normed rows,
// stats [parts, 16] partial sums of squares of x's rows (row m in column m); row m of the result is scaled by
// rsqrt(sum(stats[:, m]) / K + eps) before rounding.
int holon_gemm_skinny_scaled_bf16(const void* x, const void* w_tiled, void* y, int M, int N, int K, int out_f32,
                                  const float* stats, int parts, float eps, void* stream);
// y[M, I] = round(silu(round(x gate^T))) * round(x up^T) with w = [gate; up] ([2I, K]), M <= 16.
// stats (nullable): as in holon_gemm_skinny_scaled_bf16 (tiled weights with the norm's weight folded in).
int holon_gemm_skinny_glu_bf16(const void* x, const void* w, void* y, int M, int I, int K, int tiled, const float* stats,
                               int parts, float eps, void* stream);
// The same products for 17 <= M <= 64 rows over tiled weights with many tiles (N / 16 a multiple of 8 and at least
// 1,024; K a multiple of 256): the rows of activations go through LDS, shared by a block's waves, and every wave sums
// its tile over all of K in order. `gated`: N is I and the weight has 2 I rows.
int holon_gemm_rows_supported(int M, int N, int K, int gated);
int holon_gemm_rows_bf16(const void* x, const void* w_tiled, void* y, int M, int N, int K, int out_f32, void* stream);
int holon_gemm_rows_glu_bf16(const void* x, const void* w_tiled, void* y, int M, int I, int K, void* stream);
// The same for narrow weights (a few hundred tiles) and up to 128 rows, with K cut into `splits` shares over the grid as well: blocks of
// four waves, N / 16 a multiple of 4, K a multiple of 128 * splits, splits <= 16. parts [splits, M, N]
// float32 holds each share's sums; the product is their sum in order (holon_sum_parts rounds it to bfloat16;
// holon_rmsnorm_parts, the residual add + norm, reads them itself). holon_gemm_rows_splits: the number of shares that
// serves this shape best (0: none does).
int holon_gemm_rows_splits(int M, int N, int K);
int holon_gemm_rows_parts_supported(int M, int N, int K, int splits);
int holon_gemm_rows_parts_bf16(const void* x, const void* w_tiled, void* parts, int M, int N, int K, int splits,
                               void* stream);
// The same for 129 to 1,024 rows over a weight whose K is at least twice its N (a feed-forward's second product;
// up to 768 rows: one and a half times):
// blocks of 128 rows against 256 columns. holon_gemm_tiles_splits: the shares to take, 0 where the shape is not served
// or not this kernel's to take.
int holon_gemm_tiles_splits(int M, int N, int K);
int holon_gemm_tiles_parts_supported(int M, int N, int K, int splits);
int holon_gemm_tiles_parts_bf16(const void* x, const void* w_tiled, void* parts, int M, int N, int K, int splits,
                                void* stream);
int holon_sum_parts(const void* parts, void* y, int splits, int64_t count, void* stream);
// y[M, N] = x[M, K] w[N, K]^T, all float32, true 32-bit products and sums in an order that depends on K alone: a row's
// result is bit for bit the same whatever other rows are in the call.
int holon_gemm_f32(const void* x, const void* w, void* y, int M, int N, int K, void* stream);
// scale (nullable, [K] bfloat16): tiled holds round(w[n][k] * scale[k]).
int holon_tile_weight_bf16(const void* w, void* tiled, int N, int K, const void* scale, void* stream);
// `pieces`: room for rows x holon_argmax_pieces(vocab) pairs (float32, int32) when that is not 0 (a wide row is then
// searched by many blocks and a second kernel picks among them), or NULL (one block a row).
int holon_argmax_pieces(int vocab);
int holon_argmax(const float* logits, int32_t* out, int rows, int vocab, void* pieces, void* stream);
// last_token[slots[r]] = tokens[r] for r < rows (slots are distinct; last_token has n_slots entries).
int holon_store_tokens(int32_t* last_token, const int32_t* slots, const int32_t* tokens, int rows, int n_slots,
                       void* stream);
// One token per row. Without `slots`, row r's parameters are temperature[r], top_k[r], ...; with `slots` ([rows]) they
// are tables by slot and row r reads entry slots[r]. `positions` ([rows]: the position of the token being drawn) is
// int32 when positions_i32 is set, int64 otherwise.
int holon_sample(const float* logits, int32_t* out, int rows, int vocab, const float* temperature,
                 const int32_t* top_k, const float* top_p, const float* min_p, const int64_t* seeds,
                 const void* positions, const int32_t* slots, int positions_i32, void* stream);
// dst[idx[r], :] = src[r, :], rows of `width` int32 values; idx outside [0, dst_rows) is skipped.
int holon_scatter_rows(int32_t* dst, const int32_t* idx, const int32_t* src, int rows, int width, int dst_rows,
                       void* stream);

// log_softmax of the raw logits: token_lp[r] for tokens[r], and the k (<= 32) largest with their ids, [rows, k].
int holon_logprobs(const float* logits, const int32_t* tokens, int rows, int vocab, int k, float* token_lp,
                   int32_t* top_ids, float* top_lp, void* stream);

// -- a float32 residual stream (stream32.hip) ---------------------------------------------------------------------------
// y[i] = x[i] as float32 (x float32 or bfloat16): a new copy.
int holon_widen_rows(const void* x, float* y, int64_t n, int dtype, void* stream);
// x32 [rows, dim] += s1 d1 + s2 d2 in place (d1, d2 nullable, each float32 or bfloat16 by dt1, dt2); then, with
// weight and y (both or neither): y = (x - mean) / sqrt(var + eps) * weight, weight and y of dtype dt_out.
int holon_stream_norm(float* x32, const void* d1, float s1, int dt1, const void* d2, float s2, int dt2,
                      const void* weight, void* y, int64_t rows, int dim, float eps, int dt_out, void* stream);
// y [rows, w1 + w2] = [x32 | origin] in dt_out.
int holon_pair_rows(const float* x32, const void* origin, void* y, int64_t rows, int w1, int w2, int dt_origin,
                    int dt_out, void* stream);
// logits <- cap * tanh(logits / cap) in place.
int holon_softcap(float* logits, int64_t n, float cap, void* stream);

// -- recurrent mixers (recurrent.hip); rows are ranges query_start[b] .. query_start[b + 1] of the flat tokens ----------
// y_t[c] = act(sum_j w[c, j] x_(t - taps + 1 + j)[c] (+ x_t[c])); state [state_slots, taps - 1, channels] holds each
// request's last inputs (ignored by a row that starts at 0) and takes the row's last ones afterwards.
// rows_in_order: every row has one token and token t is row t (a decode step): one kernel then does both.
int holon_causal_conv(const void* x, const void* w, void* state, void* y, const int32_t* slots, const int32_t* starts,
                      const int32_t* query_start, const int32_t* token_row, int tokens, int rows, int channels, int taps,
                      int state_slots, int add_input, int act, int dtype, int rows_in_order, void* stream);
// From filtered q, k, v [T, 2 G D + H V] and the projections ab [T, 2 H]: unit q (times D^-0.5) and k [T, G, D],
// beta = sigmoid(b), g = exp(-exp(a_log) softplus(a + dt_bias)) [T, H]; all outputs float32.
int holon_delta_prepare(const void* qkv, const void* ab, const float* a_log, const float* dt_bias, float* qn, float* kn,
                        float* beta, float* g, int tokens, int heads, int kv_heads, int dim, int vdim, int dtype,
                        void* stream);
// The gated delta rule over each row's tokens; v = qkv[t, v_offset + h V + j]; state [state_slots, H, D, V] float32.
// piece_tokens > 0: rows in pieces that run side by side, as for holon_memory_scan; workspaces ab [pieces, H, D, V + D]
// and sin [pieces, H, D, V], float32.
int holon_delta_scan(const float* qn, const float* kn, const void* qkv, int qkv_stride, int v_offset, const float* beta,
                     const float* g, float* state, float* out, const int32_t* slots, const int32_t* starts,
                     const int32_t* query_start, int rows, int heads, int kv_heads, int dim, int vdim, int state_slots,
                     int dtype, int piece_tokens, int max_pieces, const int32_t* piece_base, float* ab, float* sin,
                     void* stream);
// The decayed key-value memory over each row's tokens; r, k, v [T, H D]; w [T, H D] float32; u [H, D];
// state [state_slots, H, D, D] float32. piece_tokens > 0: rows are cut into pieces of that many tokens that run side by
// side in two passes (at most max_pieces a row; piece_base [rows]: the number of each row's first piece among all;
// workspaces sloc [pieces, H, D, D] and pw [pieces, H, D], float32).
int holon_memory_scan(const void* r, const void* k, const void* v, const float* w, const float* u, float* state,
                      float* out, const int32_t* slots, const int32_t* starts, const int32_t* query_start, int rows,
                      int heads, int dim, int state_slots, int dtype, int piece_tokens, int max_pieces,
                      const int32_t* piece_base, float* sloc, float* pw, void* stream);
// y [T, H V] = o / sqrt(mean_V(o^2) + eps) * weight * act(gate); weight [V], or [H V] with per_head; act is silu, or
// with plain_sigmoid the sigmoid alone; a token's H V gates start gate_stride values after the token before's. den
// [T, H] float32 or NULL: every head's o is divided by it first.
int holon_gated_out(const float* o, const void* gate, const void* weight, void* y, int tokens, int heads, int vdim,
                    int per_head, float eps, int dtype, int64_t gate_stride, int plain_sigmoid, const float* den,
                    void* stream);
// y [mixes, T, W] = x + (x' - x) mu_s, x' the row of the token before (state [state_slots, W] for a row's first
// token, zeros for a row that starts at 0); the state then takes each row's last x.
int holon_shift_mix(const void* x, const void* mu, void* state, void* y, const int32_t* slots, const int32_t* starts,
                    const int32_t* query_start, const int32_t* token_row, int tokens, int rows, int width, int mixes,
                    int state_slots, int dtype, int rows_in_order, void* stream);
// y [T, C] = exp(-exp(tanh(a [T, R]) w2^T + w0 [C])), float32; w2 comes transposed, w2t [R, C].
int holon_decay_lora(const float* a, const void* w2t, const float* w0, float* y, int tokens, int channels, int rank,
                     int dtype, void* stream);

// -- windowed sigmoid attention (sigmoid_attention.hip); a page is keys [Hkv, P, D] then values [Hkv, V, P] ---------------
int holon_head_prepare(const void* qkv, void* q_out, int tokens, int heads, int kv_heads, int dim, int vdim,
                       const void* q_weight, const void* k_weight, float eps, const float* table, int rot, int table_rows,
                       const int32_t* positions, void* pages, const int32_t* write_page, const int32_t* write_off,
                       int page_size, int num_pages, int dtype, const float* bias, int stride, int v_from_keys,
                       int v_share, void* stream);
int holon_sigmoid_attention(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                            const int32_t* slots, const int32_t* token_row, const int32_t* positions,
                            const int32_t* query_start, const int32_t* row_ids, int tokens, int heads, int kv_heads,
                            int dim, int vdim, int page_size, int num_pages, const float* bias, float scale, int window,
                            const void* gate, int dtype, void* stream);
// The prompt portions (rows listed in row_ids) on the matrix cores: bfloat16, keys and values of one width 64 or 128.
int holon_sigmoid_attention_prefill_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                         int table_stride, const int32_t* slots, const int32_t* lens,
                                         const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_query,
                                         int max_len, int heads, int kv_heads, int head_dim, int page_size, float scale,
                                         int window, const float* head_bias, const void* gate, void* stream);
// The decode rows (one token each) on the matrix cores, the same sizes.
int holon_sigmoid_attention_decode_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                        int table_stride, const int32_t* slots, const int32_t* lens,
                                        const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                        int heads, int kv_heads, int head_dim, int page_size, float scale, int window,
                                        const float* head_bias, const void* gate, int rows_in_order, void* stream);

// -- Dynamic Tanh and the adds around it (dyt.hip) ------------------------------------------------------------------------
// x [rows, dim] (float32 when anything is added): x += scale * (tanh(a1 term) w1 + b1) (with a term), x += extra (with
// extra, float32), y = tanh(a2 x) w2 + b2 (with y); the alphas are single values on the device, w and b [dim] float32.
int holon_dyt_stream(void* x, int x_dtype, const void* term, int term_dtype, const float* post_alpha,
                     const float* post_w, const float* post_b, float scale, const float* extra, const float* pre_alpha,
                     const float* pre_w, const float* pre_b, void* y, int y_dtype, int64_t rows, int dim, void* stream);

// -- softmax attention with a window and a sink over pages of keys [Hkv, P, D] then values [Hkv, V, P] ------------------
// (softmax_attention.hip) q [T, H, D] -> out [T, H V]; token t reads block table row slots[token_row[t]] and stands at
// positions[t]; sink [H] float32 or null; window 0: everything before. softcap > 0: scores become softcap tanh(s /
// softcap); r1, r2 [H] float32 (both or neither): r1 ln(1 + r2 (i - j)) is taken off the score of key j for query i;
// keep_first: under a window, keys 0 .. keep_first - 1 stay visible. v_share > 1: a page holds kv_heads / v_share value
// heads behind its kv_heads key heads, and key head h reads value head h / v_share.
int holon_softmax_attention(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                            int table_rows, const int32_t* slots, const int32_t* token_row, const int32_t* positions,
                            int tokens, int heads, int kv_heads, int dim, int vdim, int page_size, int num_pages,
                            const float* sink, float scale, int window, int dtype, float softcap, const float* r1,
                            const float* r2, int keep_first, int v_share, void* stream);
// x [T, H V] *= sigmoid(gates[t, h]) per head (gates: columns of rows gate_stride apart); x [rows, dim] += bias;
// y [T, 2 H V] (kv head, map, head in group) -> out [T, H V]: u = y1 - lam y2, u / sqrt(mean(u^2) + eps) * gain.
int holon_head_gate(void* x, const void* gates, int64_t gate_stride, int64_t tokens, int heads, int vdim, int dtype,
                    void* stream);
int holon_add_bias(void* x, const float* bias, int64_t rows, int dim, int dtype, void* stream);
int holon_diff_combine(const void* y, void* out, int64_t tokens, int heads, int kv_heads, int vdim, float lam, float eps,
                       float gain, int dtype, void* stream);
// qkv [T, H D + G D + G V]: the query values of a token RMS-normed as one vector with q_weight [H D], its key values
// with k_weight [G D]; queries to q [T, H, D], keys and values into the token's page.
int holon_whole_norm_prepare(const void* qkv, int tokens, int heads, int kv_heads, int dim, int vdim,
                             const void* q_weight, const void* k_weight, float eps, void* q, void* pages,
                             const int32_t* write_page, const int32_t* write_off, int page_size, int num_pages, int dtype,
                             void* stream);
// both [T, H (dim + rot) + kv_rank + rot]: the latent RMS-normed, the first rd of every rotated part's rot dimensions
// turned by the position (table [table_rows, rd] float32: cosines, then sines); unrotated query parts to qn [T, H, dim],
// rotated ones into the last rot columns of full [T, H, kv_rank + rot]; [latent, rotated key part] into the token's
// page as a key row and as a value column.
int holon_latent_rope_prepare(const void* both, int tokens, int heads, int dim, int rot, int kv_rank,
                              const void* c_weight, float eps, const float* table, int rd, int table_rows,
                              const int32_t* positions, void* qn, void* full, void* pages, const int32_t* write_page,
                              const int32_t* write_off, int page_size, int num_pages, int dtype, void* stream);

// The latent attention's two latents, side by side in `both` [T, q_rank + kv_rank]: each divided by its root mean square
// and multiplied by its weight; the first to cq [T, q_rank], the second into the token's page as a key row and as a
// value column (pages of [2, P * kv_rank]).
int holon_latent_prepare(const void* both, int tokens, int q_rank, int kv_rank, const void* q_weight,
                         const void* c_weight, float eps, void* cq, void* pages, const int32_t* write_page,
                         const int32_t* write_off, int page_size, int num_pages, int dtype, void* stream);
// y [rows, H, B] = x [rows, H, A] times every head's own w [H, B, A], for steps of up to 16 rows; a head's results lie
// y_head values apart (B, or more where y is part of wider rows).
int holon_head_linear_rows(const void* x, const void* w, void* y, int rows, int heads, int A, int B, int y_head,
                           int dtype, void* stream);

// -- a block of two sublayers over one float32 stream (parallel_block.hip) ----------------------------------------------
// x32 [rows, dim] += (d1 + d2) + row in place (each nullable; d1, d2 float32 or bfloat16 by dt1, dt2; row [dim] float32);
// then, with w1 and y1: y1 = x rsqrt(mean(x^2) + eps) w1, and with w2 and y2 the same rows with w2 (weights of dtype dtw,
// results of dt_out).
int holon_stream_rms(float* x32, const void* d1, int dt1, const void* d2, int dt2, const float* row, const void* w1,
                     const void* w2, int dtw, void* y1, void* y2, int64_t rows, int dim, float eps, int dt_out,
                     void* stream);
// The same for a step of single tokens (row b is token b) whose results each go through a causal filter, y <- y +
// conv(y), with the requests' last taps - 1 inputs in their slots (see parallel_block.hip).
int holon_stream_rms_filter_supported(int dim, int taps);
int holon_stream_rms_filter(float* x32, const void* d1, int dt1, const void* d2, int dt2, const float* row,
                            const void* w1, const void* w2, int dtw, void* y1, void* y2, int64_t rows, int dim,
                            float eps, int dt_out, const void* cw1, const void* cw2, void* held1, void* held2,
                            const int32_t* slots, const int32_t* starts, int taps, void* stream);
// y[i] = scale * x[i] as float32 (x float32 or bfloat16): a new copy.
int holon_scale_rows(const void* x, float* y, int64_t n, int dtype, float scale, void* stream);

// -- feed-forward kinds (ffn_kinds.hip) ---------------------------------------------------------------------------------
// y = coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] over rows of `dim`, N(v) = v / sqrt(mean(v^2) + eps).
int holon_polynorm(const void* z, const float* coef, void* y, int64_t rows, int dim, float eps, int dtype, void* stream);
// logits [rows, experts] float32 -> weights [rows, experts]: sigmoid scores; chosen by score + correction (nullable)
// among the `keep` best of `groups` groups of neighbours (a group's score: its two largest choices), `top` a row;
// a chosen expert's weight is score * scale, every other 0.
int holon_moe_route(const float* logits, const float* correction, float* weights, int64_t rows, int experts, int top,
                    int groups, int keep, float scale, void* stream);
// The same from the tokens' rows x [rows, width] (float32 or bfloat16): the float32 logits x . router[e] (router
// [experts, width] float32) and the choice, in one kernel.
int holon_moe_router(const void* x, const float* router, const float* correction, float* weights, int64_t rows,
                     int width, int experts, int top, int groups, int keep, float scale, int dtype, void* stream);
// gate_up [rows, 2 C], C = experts ff + shared: y [rows, C] = silu(gate) up times the weight of the column's expert
// (the last `shared` columns: 1, or column `shared_col` >= 0 of the weights' rows), exactly 0 where the weight is 0.
// A row of `weights` is `wstride` long.
int holon_moe_gate(const void* gate_up, const float* weights, void* y, int64_t rows, int experts, int ff, int shared,
                   int dtype, int wstride, int shared_col, void* stream);
// The other router: logits x . router[e] + bias[e] (nullable), the `top` largest chosen, weights the softmax over the
// chosen logits alone; router rows beyond the experts (none or one) are gates: their columns hold a sigmoid.
// weights [rows, router_rows].
int holon_moe_router_top(const void* x, const float* router, const float* bias, float* weights, int64_t rows, int width,
                         int experts, int router_rows, int top, int dtype, void* stream);
// y = max(z, 0)^2 over n values.
int holon_relu2(const void* z, void* y, int64_t n, int dtype, void* stream);

// -- the matrix memory of xLSTM (mlstm.hip) -------------------------------------------------------------------------------
// proj [T, width]: q, k [H D] and v [H V] and the gates' pre-activations [2 H] (input, then forget) from the given
// columns; gate_bias [2 H]; state S [slots, H, D, V + 1] (the last column is n) and m [slots, H, ceil((V + 1) / 8)] (a
// copy for every 8 columns), float32; out [T, H, V] the numerators S^T q and den [T, H] the denominators
// max(|n . q|, exp(-m)) + 1e-6, float32. piece_tokens > 0: rows are cut into pieces of that many tokens that run side
// by side in two passes (at most max_pieces a row; piece_base [rows]: the number of each row's first piece among all;
// workspaces gates [T, H, 3], sloc [pieces, H, D, V + 1], pk [pieces, H]).
int holon_mlstm_scan(const void* proj, int width, int q_off, int k_off, int v_off, int gate_off, const float* gate_bias,
                     float cap, float* S, float* m, float* out, float* den, const int32_t* slots, const int32_t* starts,
                     const int32_t* query_start, int rows, int heads, int dim, int vdim, int state_slots, int dtype,
                     int tokens, int piece_tokens, int max_pieces, const int32_t* piece_base, float* gates, float* sloc,
                     float* pk, void* stream);

#ifdef __cplusplus
}
#endif
