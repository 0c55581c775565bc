// C entry points of the kernel library.  Every function launches on the given stream and
// returns 0, a HIP error code (> 0), or a negative code for arguments it refuses:
//   -2 sizes or strides out of range, -3 misaligned pointer or stride,
//   -4 head size not compiled in, -5 page size not supported, -6 scratch smaller than asked for,
//   -7 sizes beyond what the library's own static scratch holds (inside the library also: not this kernel's shape),
//   -8 a decode attention whose partials do not fit a workgroup's LDS (a context too long for the kernel).
// All pointers are device pointers.  Nothing here allocates.
#pragma once
#include <stdint.h>

extern "C" {
int bw_embed(const int32_t* tokens, const int32_t* feedback, const void* table, int table_is_bf16, float* out,
             int rows, int width, int vocab, void* stream);
// out[r] = table[token] * scale + pair_table[hash(token before, token)] + pos_table[position], each of the two tables
// optional.  hash = (before * mul_prev + token * mul_cur) mod buckets; a request's first position takes row ``buckets``.
// The token before a request's first row of this step is state[slot] (a word per slot), which then takes the request's
// last token of this step.  seq_rows: [requests, 2] = (first row, rows).  Rows with a negative token or position are zero.
int bw_embed_sum(const int32_t* tokens, const int32_t* feedback, const int32_t* positions, const int32_t* row_seq,
                 const int32_t* seq_rows, const int32_t* slots, int32_t* state, const void* table, const void* pair_table,
                 const void* pos_table, int tables_are_bf16, float scale, int buckets, int mul_prev, int mul_cur,
                 int max_positions, float* out, int rows, int width, int vocab, void* stream);
int bw_rmsnorm(const float* x, const void* weight, int weight_is_bf16, void* y, int out_is_bf16, int rows,
               int dim, int ldy, float eps, void* stream);
int bw_add(float* x, const float* y, long long n, void* stream);
int bw_add_bias(float* x, const float* bias, int rows, int cols, int ldx, void* stream);
int bw_convert(const void* src, int src_is_bf16, void* dst, int dst_is_bf16, int rows, int cols, int lds, int ldd,
               void* stream);
int bw_swiglu_f32(const float* gate_up, float* h, int rows, int inter, void* stream);
int bw_gather_rows_f32(const float* x, const int32_t* idx, float* out, int count, int width, int ldx, void* stream);
int bw_rope_kvwrite(float* qkv, void* q_out, const int32_t* positions, const int32_t* row_seq,
                    const int32_t* block_table, int table_stride, const float* cos_table, const float* sin_table,
                    void* k_cache, void* v_cache, int is_bf16, int rows, int heads, int kv_heads, int head_dim,
                    int page_size, int write_cache, void* stream);
int bw_gemm_f32(const float* x, const void* w, int w_is_bf16, float* y, int M, int N, int K, int ldx, int ldy,
                int accumulate, void* stream);
int bw_gemm_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo, int epilogue,
                 void* stream);
int bw_gemm_clamped_glu_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo, float limit,
                             float alpha, void* stream);
int bw_gemm_add_scratch(int M, int N, int K, long long* scratch_floats, int* counters);
int bw_gemm_add_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo, float* scratch,
                     long long scratch_floats, int32_t* counters, int num_counters, void* stream);
// No counterpart in the reference.  For callers that cannot allocate device memory and cannot bring a
// workspace either (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
// bw_gemm_add_bf16 with its scratch (the segments' sums, the tiles' counters) in a static array of the
// library's device image, 8 MB + 4 KB on every GPU the library runs on, held until the process ends.
// Shapes whose scratch would exceed that (bw_gemm_add_bf16_static_max gives the limits, bw_gemm_add_scratch
// what a shape needs) are refused with -7.  It calls no hipMalloc, no hipFree and no allocating library
// routine.  All calls on one GPU share that GPU's array: calls that overlap on one GPU race; calls on one
// stream, one after the other, do not.  The bits are those of bw_gemm_add_bf16.
int bw_gemm_add_bf16_static(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo,
                            void* stream);
int bw_gemm_add_bf16_static_max(long long* scratch_floats, int* counters);
int bw_gemm_qkv_rope_bf16(const void* x, int ldx, const void* w_qkv, void* q_out, const int32_t* positions,
                          const int32_t* row_seq, const int32_t* block_table, int table_stride, const float* cos_table,
                          const float* sin_table, void* k_cache, void* v_cache, int M, int heads, int kv_heads,
                          int head_dim, int K, int page_size, int write_cache, void* stream);
int bw_attention_f32(const float* q, int q_stride, const int32_t* positions, const int32_t* row_seq,
                     const int32_t* block_table, int table_stride, const float* k_cache, const float* v_cache,
                     float* out, int out_stride, int rows, int heads, int kv_heads, int head_dim, int page_size,
                     int window, float scale, const float* sink, int chunk, float softcap, void* stream);
int bw_attention_f32_tiles(const float* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                           int table_stride, const int32_t* tiles, int num_tiles, int tiled, const float* k_cache,
                           const float* v_cache, float* out, int out_stride, int heads, int kv_heads, int head_dim,
                           int page_size, int window, float scale, const float* sink, int chunk, float softcap,
                           void* stream);
int bw_attention_bf16(const void* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                      int table_stride, const int32_t* tiles, int num_tiles, const void* k_cache,
                      const void* v_cache, int num_pages, void* out, int out_stride, int heads, int kv_heads,
                      int head_dim, int page_size, int window, float scale, int decode, float* scratch,
                      long long scratch_floats, int32_t* counters, int num_counters, const float* sink, int chunk,
                      float softcap, void* stream);
// (the three attention entry points above) chunk > 0: a query sees only the keys of its own run of ``chunk`` positions,
// runs counted from position 0 (not together with a window); softcap > 0: a score s becomes softcap * tanh(s / softcap).
int bw_attention_decode_scratch(int num_tiles, int heads, int kv_heads, int head_dim, int table_stride,
                                int page_size, long long* scratch_floats, int* counters);
int bw_attention_fold_group_tiles(int head_dim);
int bw_norm_gemm_supported(int M, int K);
// rows wider than one 2048-segment of K: whether the fused norm + product kernel with ``cols`` columns a workgroup takes them
int bw_norm_gemm_wide_supported(int M, int N, int K, int cols);
int bw_norm_gemm_bf16(const float* x, int ldx, const void* norm_w, int norm_w_is_bf16, float eps, const void* w,
                      void* out, int ldo, int M, int N, int K, int epilogue, void* stream);
int bw_norm_qkv_rope_bf16(const float* x, int ldx, const void* norm_w, int norm_w_is_bf16, float eps,
                          const void* w_qkv, void* q_out, const int32_t* positions, const int32_t* row_seq,
                          const int32_t* block_table, int table_stride, const float* cos_table,
                          const float* sin_table, void* k_cache, void* v_cache, int M, int heads, int kv_heads,
                          int head_dim, int K, int page_size, int write_cache, void* stream);
// Between bw_chain_begin and bw_chain_end (in the calling thread) the decode products of up to 16 rows that can run as
// phases of one launch (bw_norm_gemm_bf16 with SwiGLU or a 32-bit store, bw_norm_qkv_rope_bf16, the residual adds of
// bw_gemm_bf16 / bw_gemm_add_bf16 of few columns) are not launched when they are asked for: they wait, and leave as one
// launch whose phases wait for each other inside the kernel when anything else of gemm_bf16.hip or fused_decode.hip is
// launched, at bw_chain_flush, or at the end.  A caller that launches anything else on the stream meanwhile (this
// library's other entry points included) calls bw_chain_flush first.  sync: bw_chain_sync_words() 32-bit words, zero
// before the first chain (every launch leaves them zero); err: a word that gets a bit for every phase one of whose
// bounded waits gave up after spin_limit looks (then the results are void and the caller clears sync).  The same bits.
int bw_chain_sync_words();
int bw_chain_begin(void* sync, int sync_words, void* err, int spin_limit);
int bw_chain_flush(void* stream);
int bw_chain_end(void* stream);
int bw_sample(const float* logits, int vocab, int ld, int rows, const float* temperature, const double* uniform,
              int32_t* out, void* stream);
int bw_fingerprint(const float* logits, int vocab, int ld, int rows, const void* h_in, void* h_out, void* stream);
// Mixers with a fixed-size state per request (sequence_mix.hip).  seq_rows: [requests, 2] = (first row, rows) of every
// request of the step; slots: its state slot.  A request without rows, with a negative slot or a negative first
// position is padding: its state stays as it is.
// mix: [nmix, dim]; out: [rows, >= nmix*dim], block m of a row is the row shifted with mix[m]
int bw_norm_shift(const float* x, int ldx, const float* w, const float* mix, float* state, long long state_ld,
                  const int32_t* positions, const int32_t* row_seq, const int32_t* seq_rows, const int32_t* slots,
                  void* out, int out_is_bf16, int ldo, int rows, int dim, float eps, int nmix, void* stream);
// mode 0: a decay per key channel (gate: logits [rows, ldg] at gate_off, bias [heads*dim], param = 1/tau);
// mode 1: scalar input and forget gates per head (columns gate_off and gate2_off of proj, biases bias and bias2, param = cap)
// with normaliser and running maximum.  state: [slots, state_ld] of S [heads][dim][vdim] (mode 1: then n [heads][dim], m [heads]).
// mode 2: a decay per key channel exp(-exp(logit + bias)), the read-out taken before the update with the token's own
// k v^T weighted by bias2 [heads*dim]; mode 3: one constant decay a head, bias [heads] (gate is not read).
// q is multiplied by qscale, k by kscale.
int bw_linear_recurrence(int mode, const float* proj, int ldp, int q_off, int k_off, int v_off, const float* gate, int ldg,
                         int gate_off, int gate2_off, const float* bias, const float* bias2, float param, float qscale,
                         float kscale, float* state, long long state_ld, float* out, int ldo, const int32_t* seq_rows,
                         const int32_t* slots, const int32_t* positions, int nseq, int heads, int dim, int vdim,
                         const int32_t* chunks, int nchunks, const int32_t* spans, int nspans, float* scan_local,
                         float* scan_start, long long scan_floats, void* stream);
// gate 0: sigmoid, 1: SiLU.  weight: [heads, wstride] (wstride 0: one weight vector for all heads).
// Up to two sections of [heads][dim] 32-bit elements a row (at columns off0, off1) turned in place: of a head's first rot
// elements, element i is paired with element i + rot/2; tables [positions, rot/2].
int bw_rotate_halves_rows(float* x, int ldx, int rows, int heads, int dim, int rot, int sections, int off0, int off1,
                          const float* cos_table, const float* sin_table, const int32_t* positions, void* stream);
int bw_tanh_rows(float* x, int ld, int rows, int cols, void* stream);      // x <- tanh(x)
int bw_head_norm_gate(const float* o, int ldi, const float* weight, int wstride, const float* g, int ldg, int gate, void* out,
                      int out_is_bf16, int ldo, const int32_t* positions, int rows, int heads, int vdim, float eps,
                      void* stream);
// h = act(gate) * up of the stacked 32-bit product [rows, ldg] (gate at column 0, up at column inter); act 0: SiLU,
// 1: GELU in its tanh form, 2: g = min(gate, limit), u = clamp(up, -limit, limit), h = g sigmoid(alpha g) (u + 1).
// row_gate (optional): h of row r is multiplied by sigmoid(row_gate[r * ld_row_gate]).
int bw_glu(const float* gate_up, int ldg, void* h, int out_is_bf16, int rows, int inter, int act, float limit, float alpha,
           const float* row_gate, int ld_row_gate, void* stream);
// Attention over a compressed cache shared by all heads (latent_attention.hip).
int bw_latent_prep(const float* proj, int ldp, int q_off, int dkv_off, const float* norm_w, float eps,
                   const float* cos_table, const float* sin_table, const int32_t* positions, const int32_t* row_seq,
                   const int32_t* block_table, int table_stride, void* cache, void* latent_t, int cache_is_bf16, void* qa, int qa_is_bf16, int ldqa,
                   int rows, int heads, int dim, int rot, int rotary, int rank, int page_size, int write_cache,
                   void* stream);
int bw_headwise_linear(const float* x, int ldx, int xhs, const void* wt, int w_is_bf16, int in, int outn, void* out,
                       int out_is_bf16, int ldo, int ohs, int rows, int heads, void* stream);
int bw_shared_key_attention(const float* q, int ldq, const int32_t* positions, const int32_t* block_table,
                            int table_stride, const int32_t* tiles, int num_tiles, const void* cache, int cache_is_bf16,
                            int num_pages, const float* sink, float* out, int ldo, int heads, int dk, int dv,
                            int page_size, int window, float scale, int heads_per_group, void* stream);
int bw_shared_key_attention_mfma(const void* q, int ldq, const int32_t* positions, const int32_t* block_table,
                                 int table_stride, const int32_t* tiles, int num_tiles, const void* cache,
                                 const void* latent_t, int num_pages, const float* sink, float* out, int ldo, int heads,
                                 int dk, int dv, int page_size, int window, float scale, int heads_per_group, int nsplit,
                                 int kchunk, float* partial, long long partial_floats, void* stream);
// Mixers that convolve their projections over a few tokens, gate their outputs or carry a gated recurrence per channel,
// and row operations of layers whose norm sits behind the sublayer (gated_mix.hip).  sink (the attention entry points
// above): a score per head that joins the softmax's denominator and has no value, or null.
int bw_causal_conv(const float* x, int ldx, const float* in_bias, const void* w, const void* bias, int w_is_bf16, int taps, int channels,
                   float* state, long long state_ld, const int32_t* seq_rows, const int32_t* slots,
                   const int32_t* positions, int nseq, int max_seq_rows, float* out, int ldo, void* stream);
int bw_pair_rope_unit(const float* src, int lds, const int32_t* positions, const int32_t* row_seq,
                      const int32_t* block_table, int table_stride, const float* cos_table, const float* sin_table,
                      void* q_out, void* k_cache, void* v_cache, int is_bf16, int rows, int heads, int kv_heads,
                      int dim, int vdim, int hd, int rot, int page_size, int unit_norm, float eps, int has_kv,
                      int write_cache, int halves, int v_from_k, void* stream);
// (halves 1: pair i of the rotation is elements (i, i + rot/2) instead of (2i, 2i+1); v_from_k 1: src holds no values, a
// value head is its key head as projected, before rotation)
// Queries and keys normed over their whole projection (all heads at once): x / sqrt(mean(x^2) + eps) * w; values as they
// are or mixed with another layer's values of the same row, v <- (1 - lambda) v + lambda v_first (lambda: one number on
// the device); the cache write and the queries' copy as bw_pair_rope_unit.  src: [q | k | v] at columns 0, heads*dim,
// (heads + kv_heads)*dim.  v_keep (optional): receives the row's values as projected (32-bit, [rows, ldk]).
int bw_whole_norm_kv(const float* src, int lds, const int32_t* positions, const int32_t* row_seq,
                     const int32_t* block_table, int table_stride, const float* q_w, const float* k_w, float eps,
                     const float* v_first, int ldf, const float* lambda, float* v_keep, int ldk, void* q_out,
                     void* k_cache, void* v_cache, int is_bf16, int rows, int heads, int kv_heads, int dim, int vdim,
                     int hd, int page_size, int write_cache, void* stream);
// per_head 1: g holds one logit a head ([rows, heads]) instead of one an element
int bw_gate_mul(const void* av, int a_is_bf16, int lda, int hd, const float* g, int ldg, void* out, int out_is_bf16,
                int ldo, int rows, int heads, int vdim, int per_head, void* stream);
// (y and gates are overwritten: y by its activation, the gates' logits by the recurrence's factor and addend)
int bw_rglru_scan(float* y, int ldy, const float* y_bias, const float* u, int ldu, float* gates, int ldg, const float* ra_bias,
                  const float* ri_bias, const float* decay, float* state, long long state_ld, void* out,
                  int out_is_bf16, int ldo, const int32_t* seq_rows, const int32_t* slots, const int32_t* positions,
                  int nseq, int rows, int channels, int bs, void* stream);
// place, wts, top (optional): row r of the normed operand is sum_j wts[r][j] * y[place[r][j]] instead of y[r]
// scale: the normed row is multiplied by it on its way into x (1: added as it is)
int bw_norm_add(const float* y, int ldy, const void* w, int w_is_bf16, float* x, int ldx, void* rounded, int ldr,
                int rows, int dim, float eps, const int32_t* place, const float* wts, int top, float scale, void* stream);
// out[r] = (1/n) sum_b norm(y[b][r]) * w[b], n <= 4 (host arrays of device pointers)
int bw_norm_mean(const float* const* y, const int* ldy, const float* const* w, int n, float* out, int ldo, int rows, int dim,
                 float eps, void* stream);
// x[r] += scale * norm(that mean; w2, eps2), one launch, for rows of up to 2,048 elements: the bits of bw_norm_mean then bw_norm_add
int bw_norm_mean_add(const float* const* y, const int* ldy, const float* const* w, int n, float eps, const float* w2, float eps2,
                     float scale, float* x, int ldx, int rows, int dim, void* stream);
int bw_softcap(float* x, int ld, int rows, int cols, float cap, void* stream);
int bw_scale_rows(float* x, int ld, int rows, int cols, float factor, void* stream);      // x *= factor
// A feed-forward of routed experts (moe.hip).
// (weight_scale: the chosen scores are multiplied by it on their way into wts)
// score_kind 0: softmax over the experts, 1: sigmoid of each logit; correction (optional, [experts]): added to the scores
// for the choice only; group_best: a group's score is the sum of that many of its best choice scores (1 to 4)
int bw_moe_route(const float* logits, int ld, int rows, int experts, int top, int groups, int keep, float weight_scale,
                 int score_kind, const float* correction, int group_best, int32_t* ids, float* wts, void* stream);
// route, then plan; one launch for steps of up to 16 rows
int bw_moe_route_plan(const float* logits, int ld, int rows, int experts, int top, int groups, int keep, float weight_scale,
                      int score_kind, const float* correction, int group_best, int32_t* ids, float* wts, int32_t* sorted,
                      int32_t* place, int32_t* tiles, int32_t* meta, void* stream);
int bw_moe_max_tiles(int slots, int experts);
int bw_moe_plan(const int32_t* ids, int slots, int experts, int32_t* sorted, int32_t* place, int32_t* tiles,
                int32_t* meta, void* stream);
int bw_moe_experts(const void* x, int x_is_bf16, int ldx, int x_rows, const void* w, int w_is_bf16, void* out, int ldo,
                   const int32_t* sorted, const int32_t* tiles, const int32_t* meta, int slots, int max_tiles, int top,
                   int K, int N, int gate_up, float limit, float alpha, int round_out, void* stream);
// (gate_up's activation: limit > 0: g = min(G, limit), u = clamp(U, -limit, limit), h = g sigmoid(alpha g) (u + 1);
// limit = 0: h = G sigmoid(alpha G) U)
int bw_moe_tile_rows(int slots);
int bw_moe_combine(const float* y, int ldy, const int32_t* place, const float* wts, int top, float* out, int ldo,
                   int rows, int width, int accumulate, void* stream);
}
