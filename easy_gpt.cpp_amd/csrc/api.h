// C entry points of the gfx950 kernel library.  Every function launches on `stream`
// and returns 0, or one of the EGPT_* error codes without launching anything.
// dtype: 0 = float32, 1 = bfloat16 (activations, weights and caches of one call share it).
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* egpt_error_string(int code);
int egpt_abi_version(void);

// The residual stream (`out` here, `h` below) is float32 [rows][hidden], or with fixed != 0 64-bit fixed point in
// units of 2^-32 (see common.h), which the products of steps of few tokens add their partial results into.
int egpt_embed(const int32_t* ids, const void* table, void* out, int fixed, int n_tokens, int hidden, int vocab,
               int dtype, void* stream);
// h += delta (delta may be null); out = rmsnorm(h) * weight.  rows == null: every row, h written back.
// rows != null: only the listed rows, gathered into out[n_rows], h untouched.
// A product may arrive as float32 partial sums of a split-k product, [n_splits][rows][cols]: then the
// *_splits argument is > 0 and the consumer adds the splits up; 0 means one tensor of the activation type.
int egpt_add_rmsnorm(void* h, int fixed, const void* delta, int delta_splits, int delta_rows, const int32_t* rows,
                     const void* weight, float eps, void* out, int n_rows, int hidden, int dtype, void* stream);
// row_ss (may be null) float32 [ss_splits, n_tokens]: gate_up are float32 partial sums that still lack each row's factor
// 1/sqrt(sum_s row_ss[s][t] / hidden + eps)
int egpt_swiglu(const void* gate_up, int n_splits, const float* row_ss, int ss_splits, int hidden, float eps, void* out,
                int n_tokens, int inter, int dtype, void* stream);
// qkv_out [n_tokens, (nq + 2 nkv) hd] of the activation type; may be qkv_in itself when n_splits == 0.
// row_ss != null: the product still lacks each row's factor 1 / sqrt(sum_s row_ss[s][row] / hidden + eps).
// cos_sin != null: the angles' cosines and sines from egpt_rope_table ([n_tokens][rotary_dim / 2][2]) instead of
// computing them from positions and inv_freq.
int egpt_qkv_rope_store(const void* qkv_in, int n_splits, const float* row_ss, int ss_splits, int hidden, float eps,
                        void* qkv_out, const void* bias, const int32_t* positions, const float* inv_freq,
                        const float* cos_sin, int rotary_dim, const int32_t* slots, void* k_cache, void* v_cache,
                        int n_tokens, int nq, int nkv, int hd, int page_size, int dtype, void* stream);
// cos_sin [n_tokens][half][2] = (cos, sin)(float(positions[t]) * inv_freq[i]) in float32: once per step for all layers.
int egpt_rope_table(const int32_t* positions, const float* inv_freq, float* cos_sin, int n_tokens, int half, void* stream);
// bfloat16 product for m <= 64 rows on the matrix cores, optionally split over k (see gemm_skinny.hip).
// waves: wavefronts (of 16 columns of the result each) per workgroup, 4, 8 or 16; here and below.
// acc_fixed != null (here and in the products below): instead of writing partial sums, every workgroup adds its
// part of the product into acc_fixed [m][n], a residual stream in fixed point, with integer atomics.
int egpt_gemm_skinny(const void* x, const void* w, const void* bias, float* out_f32, void* out_bf16, void* acc_fixed,
                     int m, int n, int k, int n_splits, int waves, void* stream);
// float32 product on the matrix cores (float32 operands and accumulation): out [n_splits][m][n] are partial sums over
// n_splits ranges of k (bias only with one).  k % 4 == 0.  A row's values do not depend on m or on the other rows.
int egpt_gemm_f32(const float* x, const float* w, const float* bias, float* out, int m, int n, int k, int n_splits,
                  void* stream);
// out = x w^T + bias; x [m,k], w [n,k], out [m,n]; out_f32 != 0 writes float32 whatever dtype is.
int egpt_linear(const void* x, const void* w, const void* bias, void* out, int m, int n, int k, int dtype,
                int out_f32, void* stream);
int egpt_paged_attention(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                         const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                         const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int hd, int page_size,
                         float scale, int window, int dtype, void* stream);
// The same on the matrix cores: bfloat16, head size 64 or 128, page size a multiple of 16.  With n_splits > 1
// the key range of every request is split and part_o [n_splits][n_tokens][nq][hd], part_ml
// [n_splits][n_tokens][nq][2] (float32) hold the partial results that a second kernel combines.
int egpt_paged_attention_mfma(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                              const void* v_cache, const int32_t* block_table, int table_width,
                              const int32_t* q_start, const int32_t* q_len, const int32_t* kv_len, int n_seqs,
                              int n_tokens, int nq, int nkv, int hd, int page_size, float scale, int window,
                              int n_splits, int rows_per_wave, int combine, void* stream);
// Prompt portions: the wavefronts of a workgroup share key/value tiles through LDS (n_splits == 1 semantics);
// page sizes that are powers of two; shape = 10 * row tiles + key splits per workgroup (41, 42, 44, 22, 24), or
// 100 + 10 * blocks of 32 rows + key splits (121, 122, 124, 141, 142; page sizes up to 64).
// key_splits > 1 (shapes from 100 on): the tiles of keys that a block of rows walks are dealt over as many workgroups,
// whose results part_o [key_splits][n_tokens][nq][hd] and part_ml [key_splits][n_tokens][nq][2] (float32) hold until a
// second kernel has combined them.
// single_waves > 0 (needs nq / nkv <= 16): the requests of the step that bring one token are left out here and taken
// by the decode kernel in a launch behind, which spreads a request's keys over the single_waves (1..8) wavefronts of a
// workgroup and over single_splits key ranges; with single_splits > 1, part_o [single_splits][n_seqs][nq][hd] and
// part_ml [single_splits][n_seqs][nq][2] hold those ranges' results until they are combined (the same memory as
// above, used after it: it must hold the larger of the two).
int egpt_paged_attention_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                               const int32_t* block_table, int table_width, const int32_t* q_start,
                               const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv,
                               int hd, int page_size, float scale, int window, int shape, int key_splits,
                               float* part_o, float* part_ml, int single_splits, int single_waves, int single_lean,
                               void* stream);
// One decoded token per request: workgroups of n_waves wavefronts per (request, kv head, key split); lean != 0: the
// variant with half the loads in flight per round and fewer registers.
int egpt_paged_attention_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                                const void* v_cache, const int32_t* block_table, int table_width,
                                const int32_t* q_start, const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd,
                                int page_size, float scale, int window, int n_splits, int n_waves, int combine,
                                int lean, void* stream);
// The same with the QKV epilogue (partial sums, 1/rms, bias, rotation, store of the new key and value) folded in;
// token t belongs to request t; rotation over the whole head.
int egpt_attention_decode_fused(const float* qkv_prod, int in_splits, const float* row_ss, int ss_splits, int hidden,
                                float eps, const void* bias, const float* cos_sin, const int32_t* slots, void* out,
                                float* part_o, float* part_ml, void* k_cache,
                                void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                                const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd, int page_size, float scale,
                                int window, int n_splits, int n_waves, int combine, int lean, void* stream);
// Paged attention on the matrix cores for every head size that is a multiple of 16 up to 256 and page sizes that are
// multiples of 16, bfloat16 or float32 (true float32: v_mfma_f32_16x16x4_f32); see attention_any.hip.  The tiled entry
// takes prompt portions and mixed batches (operands as egpt_paged_attention).  The decode entry takes one token per
// request (token q_start[b] belongs to request b): part_o [n_segments][n_seqs][nq][hd] and part_ml
// [n_segments][n_seqs][nq][2] (float32) take the results of the segments of 64 keys, n_segments >= ceil(longest
// context / 64), which a second kernel folds into out.  In float32 a row's result is the same bits from either.
int egpt_attention_any_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                             const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                             const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int hd, int page_size,
                             float scale, int window, int dtype, void* stream);
int egpt_attention_any_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                              const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                              const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd, int page_size, float scale,
                              int window, int n_segments, int dtype, void* stream);
int egpt_attention_combine(const float* part_o, const float* part_ml, void* out, int n_rows, int hd, int n_splits,
                           void* stream);
// Products for m <= 16 rows whose x operand is computed while it is staged (see gemm_skinny.hip).
// h_fixed != 0: h_in is a fixed-point residual stream that is complete as it is (no delta, h_out unused).
int egpt_gemm_skinny_norm(const void* h_in, int h_fixed, float* h_out, const float* delta, int delta_splits,
                          const void* norm_w, const void* w, float* out, float* ss_out, int m, int n, int k,
                          int n_splits, int waves, void* stream);
int egpt_gemm_skinny_swiglu(const float* gate_up, int gu_splits, const float* ss_in, int ss_splits, int hidden,
                            float eps, const void* w, float* out, void* acc_fixed, int m, int n, int k, int n_splits,
                            int waves, void* stream);
int egpt_gemm_skinny_attn(const float* part_o, const float* part_ml, int a_splits, int nq, int hd, const void* w,
                          float* out, void* acc_fixed, int m, int n, int n_splits, int waves, void* stream);
// Gate/up product with SwiGLU for up to 64 rows (see gemm_gate_up.hip): out bfloat16 [m][inter] from x bfloat16 [m][k]
// and w bfloat16 [2 * inter][k] (gate rows, then up rows); k % 8 == 0.
int egpt_gemm_gate_up_swiglu(const void* x, const void* w, void* out, int m, int inter, int k, int groups, void* stream);
// scratch: n_rows * 32 floats followed by n_rows * 32 int32 (two-stage search for wide vocabularies), or null.
int egpt_argmax(const float* logits, int32_t* out, void* scratch, int n_rows, int vocab, void* stream);
// egpt_argmax for callers that cannot allocate device memory and have no workspace to pass (code under graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The pieces
// of the two-stage search live in a buffer inside the library's device image (256 KiB per GPU, held until the process
// ends) instead of a workspace argument; the call allocates nothing and launches the same kernels as egpt_argmax.
// At most EGPT_ARGMAX_STATIC_MAX_ROWS rows (more: EGPT_STATIC_SCRATCH_TOO_SMALL, nothing is launched).  The buffer needs
// no clearing: every entry that the second stage reads is written by the first stage of the same call.  All calls on
// one GPU share that GPU's buffer, so calls that overlap there (on different streams, or from different threads)
// race; calls on one stream are ordered by the stream.  The stream must belong to the current device.
// egpt_argmax_static_init resolves the buffer's address on the current device (once per device; the entry point
// does it at its first call on a device otherwise): call it before a capture begins.
#define EGPT_ARGMAX_STATIC_MAX_ROWS 1024
int egpt_argmax_static_init(void);
int egpt_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, void* stream);
// weights: scratch for n_rows * vocab floats.
int egpt_sample(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                const float* uniform, int32_t* out, float* weights, int n_rows, int vocab, void* stream);
// The same in stages for wide vocabularies (several workgroups per row, then the selection on the tokens that can still
// be kept); workspace: egpt_sample_workspace(n_rows, vocab) bytes of device memory.
size_t egpt_sample_workspace(int n_rows, int vocab);
int egpt_sample_wide(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                     const float* uniform, int32_t* out, void* workspace, int n_rows, int vocab, void* stream);

#ifdef __cplusplus
}
#endif
