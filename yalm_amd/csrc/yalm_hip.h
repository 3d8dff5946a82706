// C entry points of the gfx950 kernel library.  Every function launches on the
// given stream and returns 0, a YALM_ERR_* code for refused arguments, or the
// hipError_t of a failed launch.  Pointers are device pointers unless noted.
// dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* yalm_error_string(int code);
int yalm_abi_version(void);

// x[t, :] = float(table[tokens[t], :]); a negative token gives a row of zeros.
// reference: copy_embedding_* (src/infer.cu:636-658)
int yalm_embed(const void* table, int table_dtype, const int* tokens, float* out, int T, int D, int V,
               hipStream_t stream);

// out[r, :] = x[row(r), :] * rsqrt(mean(x^2) + eps) * w, row(r) = row_index ? row_index[r] : r.
// x is the float32 residual stream; w may be float32 or bfloat16; out float32 or bfloat16.
// reference: rmsnorm (src/infer.cu:525-539)
int yalm_rmsnorm(const float* x, const void* w, int w_dtype, void* out, int out_dtype, const int* row_index, int R,
                 int D, float eps, hipStream_t stream);

// C = A[M,K] * W[N,K]^T with float32 accumulation.  A and W have dtype `dtype`.
// epilogue 0: C float32 [M,N] = acc
//          1: C `dtype`  [M,N] = acc
//          2: C float32 [M,N] += acc                      (residual add)
//          3: gated: W holds gate and up rows interleaved in blocks of 16
//             (16 gate rows, 16 up rows, ...), N = 32 * ceil(H/16);
//             C `dtype` [M,H] = silu(gate) * up, silu(z) = z / (1 + exp(-z))
//          5: as 3 with gelu(z) = z/2 (1 + tanh(0.797885 (z + 0.044715 z^3))) in silu's place
//             (the reference's two activations, src/infer.cpp:189-195)
// reference: matmul_wide, fused_matmul_add_residuals, fused_qkv_matmul_clip,
// fused_ffn_w1_w3_glu_act (src/infer.cu:250-337, 610-634)
// workspace: float32 scratch (may be null) for kernels that split K across workgroups; they
// use as many slices as it holds (slices * M * N floats).
int yalm_gemm(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N, int K,
              int dtype, int epilogue, int H, int force_simple, hipStream_t stream);

// Floats of workspace with which the tiled bfloat16 kernel for more than 64 rows splits K (0: it does
// not; the output's tiles fill the chip).
long yalm_gemm_bf16_dma_workspace(int M, int N, int K);

// Decode GEMMs from the float32 residual stream, M <= 8 rows (M * (K + 8) * 2 bytes <= 72 KB), bfloat16 weights:
// C = epilogue(rmsnorm(x, norm_w, eps) * W^T); epilogue 0 (float32 store) or 3 or 5 (gated, as yalm_gemm).
// norm_w is float32 [K].  Refuses (YALM_ERR_ARG) other shapes: use yalm_rmsnorm + yalm_gemm then.
int yalm_gemm_norm(const float* x, const float* norm_w, float eps, const void* W, void* C, int M, int N, int K,
                   int epilogue, int H, hipStream_t stream);
// The same for the fused q/k/v projection of a decode step (row m = sequence m), followed by what
// yalm_rope_kv_write does: q rotated into q_out (bfloat16 [M, n_heads * head_dim]), k rotated and v
// into the pages of the cache at each row's position.  head_dim must be a multiple of 16.
int yalm_gemm_norm_qkv_rope(const float* x, const float* norm_w, float eps, const void* Wqkv, void* q_out,
                            void* k_pages, void* v_pages, const int* block_table, int table_stride, int ring_pages,
                            const int* tok_pos, const int* seq_slot, const float* cos_sin, int n_positions, int M,
                            int K, int n_heads, int n_kv_heads, int head_dim, int rotary_dim, int n_pages,
                            int page_layout, hipStream_t stream);

// The K slices of A[M,K] * W[N,K]^T for 17..64 rows, or more with K a multiple of 64 (bfloat16), left unadded:
// workspace [*slices][M][N] float32, for a consumer that adds them itself (yalm_rope_kv_write).  Needs at least
// M * N floats; refuses (YALM_ERR_ARG) other shapes.
int yalm_gemm_partial(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N, int K,
                      int* slices, hipStream_t stream);

// Residual add and the next RMSNorm in one for 17..64 rows, or more with K a multiple of 64 (bfloat16):
// C float32 [M,N] += A[M,K] * W[N,K]^T, then h_out bfloat16 [M,N] = C_new * rsqrt(mean(C_new^2) + eps) * norm_w.
// workspace: at least M * N floats (more lets it split K).  Refuses (YALM_ERR_ARG) other shapes.
int yalm_gemm_add_norm(const void* A, const void* W, float* C, float* workspace, long workspace_floats, int M, int N,
                       int K, const float* norm_w, float eps, void* h_out, hipStream_t stream);

// The norm chain for 17..128 rows (more than 64: K a multiple of 64).  yalm_gemm_add_emit is yalm_gemm_add_norm that
// only prepares the next norm: xn_out bfloat16 [M,N] = C_new * norm_w and ss_out float32
// [M, yalm_gemm_add_emit_parts(N)] = sums of squares of C_new over the columns of each part.  A consumer given those
// (ss, n_parts, eps; its K is the row's width) scales its float32 sums by rsqrt(sum(ss[m, :]) / K + eps) per row:
// yalm_gemm_scaled (epilogues of yalm_gemm) and yalm_gemm_partial_scaled (slices of yalm_gemm_partial, each scaled).
int yalm_gemm_add_emit(const void* A, const void* W, float* C, float* workspace, long workspace_floats, int M, int N,
                       int K, const float* norm_w, void* xn_out, float* ss_out, hipStream_t stream);
int yalm_gemm_add_emit_parts(int N);
int yalm_gemm_scaled(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N, int K,
                     int epilogue, int H, const float* ss, int n_parts, float eps, hipStream_t stream);
int yalm_gemm_partial_scaled(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N, int K,
                             int* slices, const float* ss, int n_parts, float eps, hipStream_t stream);

// Decode GEMMs (M <= 64, bfloat16) that chain norms without a norm kernel in between.
// Producer: epilogue 2 (C float32 += product) with emit_nw given also writes
// emit_xn[M,N] = bfloat16(C_new * emit_nw[n]) and emit_ss[M, parts] = sums of squares of
// C_new over the columns of each workgroup (parts = yalm_gemm_chain_parts(N), N < 16384).
// Consumer: X is such an emit_xn; with ss_in [M, n_parts_in] the float32 sums are scaled by
// rsqrt(sum(ss_in[m, :]) / K + eps) per row before the epilogue (0: float32 store, 2, 3 and 5: gated).
int yalm_gemm_chain(const void* X, const void* W, void* C, int M, int N, int K, int epilogue, int H,
                    const float* ss_in, int n_parts_in, float eps, const float* emit_nw, void* emit_xn,
                    float* emit_ss, hipStream_t stream);
int yalm_gemm_chain_parts(int N);
// The consumer form of the fused q/k/v projection with rotation and cache write (see yalm_gemm_norm_qkv_rope).
int yalm_gemm_chain_qkv_rope(const void* X, const float* ss_in, int n_parts_in, float eps, const void* Wqkv,
                             void* q_out, void* k_pages, void* v_pages, const int* block_table, int table_stride,
                             int ring_pages, const int* tok_pos, const int* seq_slot, const float* cos_sin,
                             int n_positions, int M, int K, int n_heads, int n_kv_heads, int head_dim,
                             int rotary_dim, int n_pages, int page_layout, hipStream_t stream);

// Rotates q and k of every token (adjacent pairs, angles from the table), writes q,
// optionally k and v into a staging area in page format (for attention over the step's
// own tokens: tile seq_tile0[sequence] + position / PAGE), and k and v into the pages
// of the cache.
//   k_stage [n_tiles, n_kv_heads, PAGE, head_dim], v_stage [n_tiles, n_kv_heads, head_dim, PAGE] or null
//   qkv      float32 [T, (n_heads + 2 n_kv_heads) * head_dim]
//   cos_sin  float32 [n_positions, rotary_dim/2, 2] or null (no rotation)
//   k_pages  [n_pages, n_kv_heads, PAGE, head_dim], v_pages [n_pages, n_kv_heads, head_dim, PAGE]; inside a
//            page of a head the elements lie as page_layout says (common.h: YALM_PAGE_ROWS as these shapes
//            read, YALM_PAGE_BLOCKS in blocks of 32 elements or rows for head sizes that are multiples of
//            32); the staging area is always YALM_PAGE_ROWS
//   block_table int32 [n_slots, table_stride]; page of position p: table[slot][(p / PAGE) % ring_pages]
//   a token is written iff its page is among the last ring_pages pages of its sequence
// reference: fused_rope_and_cache_update (src/infer.cu:660-705)
// slices > 1: qkv holds that many partial products [slices][T][...] of a GEMM that split K (yalm_gemm_partial);
// they are added in order while they are read.
int yalm_rope_kv_write(const float* qkv, void* q_out, void* k_stage, void* v_stage, const int* seq_tile0,
                       void* k_pages, void* v_pages, const int* block_table, int table_stride, int ring_pages, const int* tok_seq,
                       const int* tok_pos, const int* seq_slot, const int* seq_len, const float* cos_sin,
                       int n_positions, int T, int n_heads, int n_kv_heads, int head_dim, int rotary_dim,
                       int n_pages, int page_layout, int slices, int dtype, hipStream_t stream);

// The same for a step of whole prompts (every sequence from position 0; cu_seqlens [B + 1] token offsets,
// n_tiles = seq_tile0[B]): whole page-shaped tiles at a time.  Needs a staging area; refuses
// (YALM_ERR_ARG) head sizes whose transposed tile does not fit 64 KB of LDS.  slices as above.
int yalm_rope_kv_write_tiles(const float* qkv, void* q_out, void* k_stage, void* v_stage, const int* cu_seqlens,
                             const int* seq_tile0, void* k_pages, void* v_pages, const int* block_table,
                             int table_stride, int ring_pages, const int* seq_slot, const int* seq_len,
                             const float* cos_sin, int n_positions, int T, int B, int n_tiles, int n_heads,
                             int n_kv_heads, int head_dim, int rotary_dim, int n_pages, int page_layout, int slices,
                             int dtype, hipStream_t stream);

// Causal attention of a step's tokens over the same step's keys (sequences that
// start at position 0), packed without padding.  window 0 = all keys.
//   q, out [T, n_heads, hd]; k_stage, v_stage: the staging area rope_kv_write filled
//   (key j of sequence b: tile seq_tile0[b] + j / PAGE, row j % PAGE), all `dtype`
//   tile_order (may be null): n_order tiles of the staging area, every second tile of each
//   sequence from its first, those that see the most keys first; it changes the order of the
//   work and no result
// reference: attn_dot + attn_softmax + att_mix (src/infer.cu:339-523) for every position
int yalm_attn_prefill(const void* q, const void* k_stage, const void* v_stage, void* out, const int* cu_seqlens,
                      const int* seq_tile0, const int* tok_seq, const int* tok_pos, const int* tile_order, int n_order,
                      int T, int B, int n_tiles, int n_heads, int n_kv_heads, int head_dim, int window, int dtype,
                      int force_simple, hipStream_t stream);

// One query per sequence over the pages of the cache (the new key is already written).
//   q, out [B, n_heads, hd]; seq_len[b] = keys of sequence b including the new one;
//   seq_slot[b] < 0 marks a padding row (out = 0).
//   partial: float32 workspace of yalm_attn_decode_workspace(...) bytes
//   the pages are YALM_PAGE_ROWS (the variants below take a page_layout)
int yalm_attn_decode(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                     int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                     float* partial, int B, int n_heads, int n_kv_heads, int head_dim, int window, int n_splits,
                     int n_pages, int dtype, int force_simple, hipStream_t stream);
long yalm_attn_decode_workspace(int B, int n_heads, int head_dim, int n_splits);

// The two above, which also leave lse[token, head] (float32; may be null) = the natural logarithm of the
// sum of exp(score) over the keys the query saw (-FLT_MAX for a padding row), so that further keys can be
// mixed in afterwards (yalm_attn_sink_mix).  out_f32 (prefill only; float32 [T, n_heads, hd], may be null) receives
// the result before its rounding to `dtype`, for the same purpose.  step_max_len (device, one int, may be null): the length of the step's
// longest sequence; the matrix-core decode kernel then cuts every sequence into splits of that sequence's split size,
// so that sequences of unequal lengths give workgroups of equal work (no result depends on it).  seq_order (device,
// B ints, a permutation of the rows; may be null): the order in which that kernel's workgroups take the rows.
// score_bias (device, float32 [n_heads, n_bias]; may be null): a term added to every score (after the 1/sqrt(head_dim)
// scaling) by the distance between query and key, score_bias[head, min(distance, n_bias - 1)]: what a position
// encoding that is no rotation needs (not together with attention sinks).
// softcap (0: none): score <- softcap tanh(score / softcap), after the scaling and before score_bias's term.
// sink_logit (device, float32 [n_heads]; may be null): one more term exp(sink_logit[head]) of the softmax's denominator,
// to which no key and no row of values belongs (scale, cap and distance term shape the keys' scores only; lse holds it).
// slopes (device, float32 [n_heads]; may be null): -slopes[head] * distance is added to every score, as score_bias's
// term is, without a table.
// block (0: none): part of the mask; a query sees only the keys of its own block of `block` positions, blocks counted
// from position 0 of the sequence (not together with attention sinks).
int yalm_attn_prefill_lse(const void* q, const void* k_stage, const void* v_stage, void* out, float* out_f32, float* lse,
                          const int* cu_seqlens, const int* seq_tile0, const int* tok_seq, const int* tok_pos,
                          const int* tile_order, int n_order, int T, int B, int n_tiles, int n_heads, int n_kv_heads,
                          int head_dim, int window, int dtype, int force_simple, const float* score_bias, int n_bias,
                          float softcap, const float* sink_logit, const float* slopes, int block, const float* log_a,
                          const float* log_b, hipStream_t stream);
int yalm_attn_decode_lse(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                         int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                         float* lse, float* partial, int B, int n_heads, int n_kv_heads, int head_dim, int window,
                         int n_splits, int n_pages, int page_layout, int dtype, int force_simple,
                         const int* step_max_len, const int* seq_order, const float* score_bias, int n_bias,
                         float softcap, const float* sink_logit, const float* slopes, int block, const float* log_a,
                          const float* log_b, hipStream_t stream);

// Attention sinks beside a window (src/infer.cpp:305-319, 486-488): the first n_sinks positions of a
// sequence stay visible when the window has moved past them, and each then counts as lying
// window + n_sinks - 1 - j positions behind the query, however long the sequence is.  The reference
// turns the stored sink keys one position further every step; here they are kept as they were
// written and turned by the whole distance when they are read, which rounds once instead of once a step.
//
// The store: sink_k, sink_v [slots, n_kv_heads, n_sinks, hd].  1 <= n_sinks <= 16, window >= n_sinks.
// A step of whole prompts:
//   yalm_sink_store copies the keys and values of positions < min(n_sinks, seq_len[b]) from the staging
//   area (tile seq_tile0[b]) into the store of seq_slot[b].
//   yalm_attn_sink_mix adds the sinks that the window no longer covers to a finished attention result:
//   for token t at position p the sinks j < min(n_sinks, p - window + 1), keys turned by
//   max(0, p - window - n_sinks + 1) positions with cos_sin (null or rotary_dim 0: not turned);
//   out[t, h] = (e^lse out + sum_j e^s_j v_j) / (e^lse + sum_j e^s_j), s_j = q . k_j / sqrt(hd); with src_f32 (the
//   out_f32 of yalm_attn_prefill_lse; may be null) the unrounded result is read from there, so that the mixed row
//   is rounded once.
// A decode step: yalm_attn_decode_sinks is yalm_attn_decode whose merge of the splits takes those sinks in
//   as further splits of one key each (no rounding in between, no launch more; the merge runs with one
//   split too); with store != 0 a token at a position < n_sinks first stores its own key and value from its
//   page.
int yalm_sink_store(const void* k_stage, const void* v_stage, const int* seq_tile0, const int* seq_slot,
                    const int* seq_len, void* sink_k, void* sink_v, int B, int n_tiles, int n_slots, int n_kv_heads,
                    int head_dim, int n_sinks, int dtype, hipStream_t stream);
int yalm_attn_sink_mix(const void* q, void* out, const float* src_f32, const float* lse, const void* sink_k,
                       const void* sink_v,
                       const int* tok_seq, const int* tok_pos, const int* seq_slot, const float* cos_sin,
                       int n_positions, int T, int n_slots, int n_heads, int n_kv_heads, int head_dim, int rotary_dim,
                       int window, int n_sinks, int dtype, hipStream_t stream);
int yalm_attn_decode_sinks(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                           int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                           float* partial, void* sink_k, void* sink_v, int store, const float* cos_sin,
                           int n_positions, int n_slots, int rotary_dim, int n_sinks, int B, int n_heads,
                           int n_kv_heads, int head_dim, int window, int n_splits, int n_pages, int page_layout,
                           int dtype, int force_simple, const int* step_max_len, const int* seq_order,
                           hipStream_t stream);

// yalm_attn_decode without a workspace argument, for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
// counterpart in the reference.  The partial results of the splits go to a fixed array of
// YALM_ATTN_DECODE_STATIC_BYTES in device memory that belongs to the library; every GPU it runs on
// holds its own copy until the process ends.  The call allocates and frees nothing.  Sizes with
// yalm_attn_decode_workspace(B, n_heads, head_dim, n_splits) > YALM_ATTN_DECODE_STATIC_BYTES are
// refused with YALM_ERR_SCRATCH (1003).  All calls on one GPU share that GPU's array, which keeps
// the last call's contents (nothing in it has to be cleared between calls): calls that overlap on
// one GPU, on different streams or from different threads, race.  The first call on a device looks
// the array's address up and should not run under stream capture.
#define YALM_ATTN_DECODE_STATIC_BYTES (8l << 20)
int yalm_attn_decode_static(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                            int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                            int B, int n_heads, int n_kv_heads, int head_dim, int window, int n_splits, int n_pages,
                            int dtype, int force_simple, hipStream_t stream);

// out[r] = index of the maximum of logits[r, :], lowest index on ties (src/sampler.cpp:27-38)
int yalm_argmax(const float* logits, int* out, int R, int V, hipStream_t stream);
// out[r] = first index whose running sum of exp((l - max)/T) reaches u[r] * total, else V-1
// (src/sampler.cpp:40-65 with the uniform numbers given by the caller)
int yalm_sample(const float* logits, const float* u, float temperature, int* out, int R, int V, hipStream_t stream);
// prob[r] = softmax(logits[r, :])[index[r]] (src/sampler.cpp:11-25)
int yalm_token_prob(const float* logits, const int* index, float* prob, int R, int V, hipStream_t stream);

// Layers that norm a sublayer's OUTPUT before it joins the residual stream (postnorm.hip).
// yalm_cast: out[i] = dtype(x[i]).  yalm_norm_add: x[r, :] += y[r, :] * rsqrt(mean(y[r]^2) + eps) * w, and if h_out is
// given h_out[r, :] = dtype(x_new[r, :]) (the next sublayer's input), or, with next_w (float32 [D]: the weights of the
// norm that reads the stream next), dtype(x_new[r, :] * rsqrt(mean(x_new[r]^2) + next_eps) * next_w).  yalm_polynorm: out[r, :] = a N(z) + b N(z^2) +
// c N(z^3) + e with powers element by element, N(v) = v / sqrt(mean(v^2) + eps) over the row and coef = {a, b, c, e}
// (float32, on the device).
int yalm_cast(const float* x, void* out, long n, int out_dtype, hipStream_t stream);
int yalm_norm_add(const float* y, const void* w, int w_dtype, float eps, float* x, void* h_out, int h_dtype,
                  const float* next_w, float next_eps, int R, int D, hipStream_t stream);
int yalm_polynorm(const float* z, const float* coef, float eps, void* out, int out_dtype, int R, int F,
                  hipStream_t stream);

// Latent attention (latent.hip).  yalm_head_matmul: for every token t and head h,
//   out[t * out_row + h * out_head + out_off + n] = scale * sum_k in[t * in_row + h * in_head + in_off + k] * wt[h, k, n]
// (n < N, k < K <= 512), times sigmoid(gate[t * gate_row + h * N + n]) if gate (float32) is given.  Types (in, wt,
// out): all float32; float32, bfloat16, float32; all bfloat16.
// yalm_latent_pack fills out float32 [T, (H + 2) * Dk], the head-shaped rows that yalm_rope_kv_write reads with
// H query heads and one KV head of size Dk = [rot | rank | zeros]: query head h gets q_scale * proj[t, h * q_head +
// q_rot_off + i] in its first rot places and zeros behind rot + rank (the places between are the caller's, see
// yalm_head_matmul); with has_kv the key row is [proj[t, kv_off + rank + i] | c | 0] and the value row [0 | c | 0], c =
// proj[t, kv_off + i] * rsqrt(mean over the rank columns of their squares + eps) * norm_w[i].
int yalm_head_matmul(const void* in, int in_dtype, long in_row, int in_head, int in_off, const void* wt, int w_dtype,
                     void* out, int out_dtype, long out_row, int out_head, int out_off, float scale, const float* gate,
                     long gate_row, int T, int H, int K, int N, hipStream_t stream);
// yalm_head_matmul for many tokens on the matrix cores: wn is wt with its last two axes exchanged, bfloat16 [H, N, K]; the
// input (float32 or bfloat16) is rounded to bfloat16, the sums are float32, out float32 or bfloat16.  K must be a multiple
// of 8 and in_row, in_head, in_off multiples of 8; other shapes are refused (YALM_ERR_ARG: use yalm_head_matmul).
int yalm_head_matmul_mfma(const void* in, int in_dtype, long in_row, int in_head, int in_off, const void* wn, void* out,
                          int out_dtype, long out_row, int out_head, int out_off, float scale, const float* gate,
                          long gate_row, int T, int H, int K, int N, hipStream_t stream);
int yalm_latent_pack(const float* proj, long proj_row, int q_head, int q_rot_off, int kv_off, const void* norm_w,
                     int norm_dtype, float eps, float q_scale, float* out, int T, int H, int rot, int rank, int Dk,
                     int has_kv, hipStream_t stream);

// Mixture of experts (moe.hip).  yalm_moe_route: ids, wts [T, top] = the `top` experts with the largest
// softmax(w_router h) over all E experts (float32 arithmetic; the lowest index on ties) and those scores (renorm: divided
// by their sum).  The pair kernels serve every (token, choice) pair from its expert's weights: w_gate, w_up [E, F, D],
// w_down [E, D, F]; mid [T * top, F] = g sigmoid(alpha g) (u + 1) with g = min(w_gate h, limit), u = clamp(w_up h,
// -limit, limit) (limit <= 0: unclamped); out float32 [T, D] = (accumulate: out +) sum_k wts[t, k] * w_down[ids[t, k]] mid[t, k], k in order.
int yalm_moe_route(const void* h, const void* w_router, int dtype, int* ids, float* wts, int T, int D, int E, int top,
                   int renorm, hipStream_t stream);
// The same choice from logits that a product has made already (float32 [T, E]).
// bias (float32 [E], may be null) is added to the logits first.  renorm 2: the experts with the largest logits,
// weighted by the softmax over the chosen logits alone.
int yalm_moe_select(const float* logits, const float* bias, int* ids, float* wts, int T, int E, int top, int renorm,
                    hipStream_t stream);
// up_shift: the number added to the clamped up value (mid = g sigmoid(alpha g) (u + up_shift); the text above has 1;
// alpha 1, limit 0 and up_shift 0 give silu(gate) * up).
int yalm_moe_pair_gate_up(const void* h, const void* w_gate, const void* w_up, const int* ids, float limit, float alpha,
                          float up_shift, void* mid, int T, int top, int D, int F, int E, int dtype, hipStream_t stream);
int yalm_moe_pair_down(const void* mid, const void* w_down, const int* ids, const float* wts, float* out, int T, int top,
                       int D, int F, int E, int dtype, int accumulate, hipStream_t stream);

// The same result for many tokens (bfloat16, D and F multiples of 8): the pairs grouped by expert, each expert's rows
// padded to tiles of 128, one launch a product over all tiles on the matrix cores.  Scratch of the caller, with
// max_tiles = yalm_moe_grouped_tiles(T * top, E): pair_of_row int32 [max_tiles * 128], row_of_pair int32 [T * top],
// tile_expert int32 [max_tiles], mid bfloat16 [max_tiles * 128, F], y float32 [max_tiles * 128, D].
int yalm_moe_grouped_tiles(int n_pairs, int E);
int yalm_moe_grouped(const void* h, const void* w_gate, const void* w_up, const void* w_down, const int* ids,
                     const float* wts, float limit, float alpha, float up_shift, int* pair_of_row, int* row_of_pair,
                     int* tile_expert, void* mid, float* y, float* out, int T, int top, int D, int F, int E, int accumulate,
                     hipStream_t stream);

// x[t, :] = table[tokens[t], :] * scale + (freq not null) a sinusoidal position vector: entry 2i is sin(p f_i), entry
// 2i + 1 cos(p f_i), p = positions[t], f = freq (float64 [ceil(D / 2)] on the device).  A negative token gives zeros.
int yalm_embed_sinusoid(const void* table, int table_dtype, const int* tokens, const int* positions, const double* freq,
                        float scale, float* out, int T, int D, int V, hipStream_t stream);

// Between the q/k/v product and an attention without rotation (qkv_pack.hip): qkv float32 [T, H d + G d + G dv]
// (+ bias, float32 of that width or null); RMS norms over the whole query and key projections with the weights w_q
// [H d], w_k [G d] (float32; null: no norm); the queries times q_scale and, with temp_every > 0, times 1 + temp_coef
// ln(floor((p + 1) / temp_every) + 1); blend 1 stores the values in v_first (float32 [T, G dv]), blend 2 replaces them
// by (1 - lam) v + lam v_first (lam: one float32 on the device).  Heads are written `pad` wide with zeros behind
// (pad >= d, dv): q_out [T, H, pad]; keys and values into the cache pages (page_layout of head size pad) and, with
// k_stage, into the staging tiles of a step of whole prompts, as yalm_rope_kv_write does.  head_norm != 0: the norms run
// over each head's d elements instead, with w_q and w_k of d elements shared by the heads.  v_from_k != 0: qkv has no value
// part, [T, H d + G d], and a head's values are its keys as projected, before their norm (dv = d, no blend).  rot_dims > 0:
// behind the norms, the neighbours (2p, 2p + 1), p < rot_dims / 2, of every query and key head are turned by the angle
// cos_sin[position][p] ((cos, sin) float32 [n_positions, rot_dims / 2, 2]).
int yalm_qkv_pack(const float* qkv, const float* bias, const float* w_q, const float* w_k, float eps, float temp_coef,
                  int temp_every, float q_scale, float* v_first, int blend, const float* lam, void* q_out, void* k_stage,
                  void* v_stage, const int* seq_tile0, void* k_pages, void* v_pages, const int* block_table,
                  int table_stride, int ring_pages, const int* tok_seq, const int* tok_pos, const int* seq_slot,
                  const int* seq_len, int T, int n_heads, int n_kv_heads, int d, int dv, int pad, int n_pages,
                  int page_layout, int dtype, void* v_rows, int head_norm, int v_from_k, const float* cos_sin, int rot_dims,
                  int n_positions, hipStream_t stream);
// v_rows (`dtype` [T, G, pad]; may be null): yalm_qkv_pack then leaves the values there row by row instead of in their
// transposed places, and yalm_v_tiles brings them into v_stage [n_tiles, G, pad, 64] and the cache pages (v_pages null:
// none) a tile of 64 tokens at a time through LDS (pad a multiple of 16; 64 (pad + 8) elements must fit 64 KB).
int yalm_v_tiles(const void* v_rows, void* v_stage, void* v_pages, const int* cu_seqlens, const int* seq_tile0,
                 const int* block_table, int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, int B,
                 int n_tiles, int n_kv_heads, int pad, int n_pages, int page_layout, int dtype, hipStream_t stream);

// The matrix-memory recurrence (mlstm.hip): proj float32 [T, 2 H d + 2 H dv + 2 H] = q | k | v | g | z_i | z_f of
// every token; state float32 [n_slots, H, d dv + d + 1] (S, n, m of every head), read and left advanced; out `dtype`
// [T, H dv] = the heads' results divided by their root mean square, times w_norm, times sigmoid(g).  The tokens of
// sequence b are rows cu_seqlens[b] .. cu_seqlens[b + 1] - 1; seq_slot[b] < 0: a padding row, left alone.
int yalm_mlstm_scan(const float* proj, const float* b_i, const float* b_f, const float* w_norm, float* state,
                    const int* cu_seqlens, const int* seq_slot, void* out, int B, int H, int d, int dv, float q_scale,
                    float cap, float floor_, float eps, int n_slots, int dtype, hipStream_t stream);

// The same recurrence a chunk of tokens at a time on the matrix cores, in float32 (chunk 64: steps of whole prompts,
// 16: single tokens); a workgroup owns 64 columns of a (sequence, head).  raw float32 [T, H dv] and nm float32
// [B, H (d + 1)]: scratch of the caller.  T: rows of proj and out.  YALM_ERR_ARG where yalm_mlstm_chunks_lds(d, chunk)
// exceeds 150 KB.
int yalm_mlstm_chunks(const float* proj, const float* b_i, const float* b_f, const float* w_norm, float* state, float* raw,
                      float* nm, const int* cu_seqlens, const int* seq_slot, void* out, int T, int B, int H, int d, int dv,
                      float q_scale, float cap, float floor_, float eps, int n_slots, int chunk, int dtype,
                      hipStream_t stream);
long yalm_mlstm_chunks_lds(int d, int chunk);

// The gated delta rule with a decay per key channel, over the tokens of a step, float32 throughout.  H heads with values
// of dv, Hq query/key heads of d (head h uses query/key head h / (H / Hq)).
// proj float32 [T, 2 Hq d + H dv + H] = q | k | v | b: the projections before their short causal convolutions, and the step
// size's logit.  low float32 [T, H d + H dv]: the decay's and the output gate's pre-activations.  conv_w float32
// [2 Hq d + H dv, taps] (the last column is the current token's); decay_log [H], decay_bias [H d], w_norm [dv].
// Per token: q, k, v <- silu(convolution); q, k <- unit vectors a head (x / sqrt(sum x^2 + unit_floor)), q times q_scale;
// beta = sigmoid(b); g = exp(-exp(decay_log[h]) softplus(low + decay_bias)) per head and key channel; per head
//   S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
// out `dtype` [T, H dv] = o / rms(o over the head; eps) * w_norm * sigmoid(gate pre-activation).
// state float32 [n_slots, H d dv + (2 Hq d + H dv) (taps - 1)]: S [H, d, dv], then the convolutions' last taps - 1 inputs
// [channel, taps - 1] (the latest last); read and left advanced.  prep float32 [T, 2 Hq d + H dv + H + H d] and raw float32
// [T, H dv]: scratch of the caller.  The tokens of sequence b are rows cu_seqlens[b] .. cu_seqlens[b + 1] - 1, in order;
// tok_seq[t] is row t's sequence; seq_slot[b] < 0: a padding row, left alone (its output is zero).  d <= 256, taps <= 16.
int yalm_gated_delta(const float* proj, const float* low, const float* conv_w, const float* decay_log,
                     const float* decay_bias, const float* w_norm, float* state, float* prep, float* raw,
                     const int* tok_seq, const int* cu_seqlens, const int* seq_slot, void* out, int T, int B, int H, int Hq,
                     int d, int dv, int taps, float q_scale, float unit_floor, float eps, int n_slots, int dtype,
                     hipStream_t stream);

// x[t, :] = table[tokens[t], :] * scale + pos_table[positions[t], :] (both tables of `dtype`, [V, D] and [P, D]); a token
// outside the vocabulary gives a row of zeros.
int yalm_embed_learned(const void* table, const void* pos_table, int dtype, const int* tokens, const int* positions,
                       float scale, float* out, int T, int D, int V, int P, hipStream_t stream);
// out[i] = act(z[i]), out of `out_dtype`; kind 0: z/2 (1 + erf(z / sqrt 2)), 1: the tanh form of the same, 2: silu.
int yalm_activate(const float* z, void* out, long n, int kind, int out_dtype, hipStream_t stream);
// x[t, :] (+)= sigmoid(h[t, :] . w) * y[t, :]; h [T, D] and w [D] of `dtype`, x and y float32; accumulate 0: x is written.
int yalm_gated_add(const float* y, const void* h, const void* w, int dtype, float* x, int T, int D, int accumulate,
                   hipStream_t stream);
// out[t, c] = (residual ? h[t, c] : 0) + sum_j w[j, c] in(t - (taps - 1) + j, c): a causal convolution over the tokens of
// each sequence (h, out [T, D] of `dtype`, not the same memory; w float32 [taps, D], tap by tap, the last tap on the token itself).
// carried, float32 [n_slots, taps - 1, D], holds each sequence's last taps - 1 inputs (the newest last): read for the
// places in front of the step's first token, then left advanced.  Rows of padding (slot -1) read zeros and keep nothing.
// one_each != 0: every sequence brings one token (T = B, row t is sequence t), which lets one launch do both.
int yalm_time_conv(const void* h, const float* w, float* carried, void* out, const int* tok_seq, const int* cu_seqlens,
                   const int* seq_slot, int T, int B, int D, int taps, int residual, int one_each, int dtype, hipStream_t stream);
// out[t, i] = act(z[t, i] + bias[i]) * (z[t, F + i] + bias[F + i]), i < F: z float32 [T, 2 F] (gate | up), bias float32
// [2 F] or null, out of `out_dtype`, kind as yalm_activate; with x_bias (float32 [D]) also x[t, :] += x_bias (x float32 [T, D]).
int yalm_gated_bias_act(const float* z, const float* bias, void* out, int T, int F, int kind, int out_dtype, float* x,
                        const float* x_bias, int D, hipStream_t stream);
// o[t, h, e] *= sigmoid(g[t * g_stride + h * dv + e]), e < dv: o of `dtype` [T, n_heads, pad], g float32.
int yalm_sigmoid_gate(void* o, const float* g, long g_stride, int T, int n_heads, int dv, int pad, int dtype,
                      hipStream_t stream);
// both[t] = [x[t] | x0[t]] (`dtype` [T, 2 D]), then x[t] = start (x, x0 float32 [T, D], start float32 [D]).
int yalm_loop_pack(float* x, const float* x0, const float* start, void* both, int T, int D, int dtype, hipStream_t stream);
// The HGRN2 recurrence (hgrn2.hip): proj float32 [T, 2 H d + H dv] = z_q | z_f | v of every token; q = silu(z_q), f =
// lower + (1 - lower) sigmoid(z_f + f_bias) (f_bias, lower float32 [H d]); per head S <- diag(f) S + (1 - f) v^T, o = S^T q;
// out (`out_dtype` [T, H dv]) = o over its root mean square a head, times w_norm (float32 [dv]).  state float32 [n_slots, H,
// dv, d] (a head's S column by column), read and left advanced; raw float32 [T, H dv] scratch; the tokens of sequence b are
// cu_seqlens[b] .. cu_seqlens[b + 1] - 1, in order; a sequence with slot -1 touches no state and gives zeros.  d <= 256.
int yalm_hgrn2(const float* proj, const float* f_bias, const float* lower, const float* w_norm, float* state, float* raw,
               const int* cu_seqlens, const int* seq_slot, void* out, int T, int B, int n_heads, int d, int dv, float eps,
               int out_dtype, hipStream_t stream);

// Yardsticks for the measurement (probes.hip): a kernel that only reads `bytes` bytes once with `workgroups`
// workgroups (out: 1,024 words of scratch), and a loop of matrix-core instructions on registers (shape 32:
// v_mfma_f32_32x32x16_bf16, 16: v_mfma_f32_16x16x32_bf16; *flops, host memory, receives the launch's operations).
int yalm_probe_read(const void* src, long bytes, unsigned int* out, int workgroups, hipStream_t stream);
int yalm_probe_mfma(int shape, int iters, int workgroups, float* out, double* flops, hipStream_t stream);

#ifdef __cplusplus
}
#endif
