// C entry points of librbitnet_hip.so.  All pointers are device pointers unless a
// name starts with h_.  Every function returns 0 on success; otherwise
// rb_last_error() holds the reason.  `stream` is a hipStream_t.
//
// dtype codes: 0 = float32, 1 = bfloat16 (storage; arithmetic is float32 inside).
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* rb_last_error(void);
int rb_version(void);
int rb_page_size(void);

// x[t, :] = table[ids[t], :] widened to float32.  ids are checked by the caller.
int rb_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x, int n_tokens, int width,
                    void* stream);

// Residual add and RMS norm in one pass.
//   src = rows ? rows[r] : r
//   v = x[src] + (delta ? delta[src] : 0);  if (delta && !rows) x[src] = v
//   out[r] = v * gain * rsqrt(mean(v^2) + eps)
// delta may be n_terms terms, each laid out like x and term_stride floats after the one before:
// they are added up first, in their order (rb_gemm_bf16_terms leaves such terms).
int rb_add_rmsnorm(float* x, const float* delta, int n_terms, long long term_stride, const float* gain, float eps,
                   const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void* stream);

// Rotate q and k by the angle table, write q to q_out and k, v into the cache pages.
//   qkv      float32 [T, (Hq + 2 Hk) D]: q heads, then k heads, then v heads; as qkv_terms terms
//            to be added up in their order, qkv_term_stride floats apart (1 term: qkv itself)
//   cos, sin float32 [max_pos, D/2], or null for no rotation
//   style    0: pairs (2i, 2i+1); 1: pairs (i, i + D/2)
//   k_pages, v_pages [n_pages, Hk, 64, D] of cache_dtype; null when the layer keeps no cache
//   tok_pos, tok_seq int32 [T]; block_table int32 [B, bt_stride]
int rb_rope_kv_write(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos, const float* sin,
                     int style, void* q_out, void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                     const int32_t* block_table, int bt_stride, int n_tokens, int n_heads, int n_kv_heads,
                     int head_dim, void* stream);

// t[r, j] = silu(gu[r, j]) * gu[r, F + j]
int rb_swiglu(const float* gu, void* out, int out_dtype, int n_rows, int ff, void* stream);

// C[M, N] = A[M, K] * W[N, K]^T with float32 accumulation; any sizes.
// w_layout 0: W is N rows of K values.  1 (float32 with N % 16 == 0 and K % 128 == 0 only): fragment-major, blocks
// of 16 rows x 16 depth values, 1 KB each, in the order [N / 16][K / 16]; inside a block the value of row r and
// depth d lies at 4 * (16 * (d / 4) + r) + d % 4.  rb_place_rows writes either layout.
int rb_gemm_generic(const void* a, const void* w, int w_layout, void* c, int dtype_in, int dtype_out, int m, int n,
                    int k, void* stream);

// C[M, N] = A[M, K] * W[N, K]^T, bfloat16 inputs on the matrix cores.
//   epilogue 0: store C (float32 or bfloat16)
//   epilogue 1: W holds gate and up rows interleaved in blocks of 16
//               (16 gate rows, then the 16 up rows of the same columns); the result is
//               silu(gate) * up, [M, N/2]
// K must be a multiple of 8 (rows 16-byte aligned).
// w_layout says how W is stored.  0: N rows of K values.  1: fragment-major (K % 64 == 0 and
// N % 16 == 0 only): blocks of 16 rows x 32 depth values, 1 KB each, in the order [N / 16][K / 32];
// inside a block, the value of row r and depth d lies at 8 * (16 * (d / 8) + r) + d % 8.  A wave
// then reads 1 KB in a row per load, and a product of few tokens streams W with non-temporal
// loads: 6.0-6.8 TB/s instead of 5.3-5.8.  rb_place_rows writes either layout.
// workspace: rb_gemm_workspace_floats(m, n, k, epilogue) floats (0: none, null allowed); contents do
// not matter before or after.
long long rb_gemm_workspace_floats(int m, int n, int k, int epilogue);
int rb_gemm_bf16(const void* a, const void* w, int w_layout, void* c, int dtype_out, int epilogue, int m, int n, int k,
                 float* workspace, void* stream);

// The plain product (float32, epilogue 0) as the terms that the K slices of its kernel computed:
// terms [rb_gemm_bf16_terms_count(m, n, k), M, N], to be added up in their order.  One term is
// the product itself.  For a caller that adds them to something else anyway.
int rb_gemm_bf16_terms_count(int m, int n, int k);
int rb_gemm_bf16_terms(const void* a, const void* w, int w_layout, float* terms, int m, int n, int k, void* stream);

// The same product for 1..16 tokens with what stands before and after it in a decode step folded
// in, so that no kernel runs between the products.  rb_gemm_bf16_few_ok: whether it takes these
// sizes (few tokens, and no tiled kernel would).
//   a: bfloat16 rows of K values; row i of the product is row rows[i] (row i without rows).
//   squares_in (may be null): float32 [*, ceil(K / 16)], rows as in a.  Then a holds float32 rows
//     times a norm's gain and squares_in their sums of squares over every 16 columns, and the
//     product is multiplied by 1 / sqrt(sum of them / K + eps): the RMS norm's factor.
//   epilogue 0, 1: as above.  2: C (float32) += product.  3: as 2, and for the norm that follows
//     gained [M, N] = bf16(C * gain), squares_out [M, ceil(N / 16)] = sums of C^2 over 16 columns.
int rb_gemm_bf16_few_ok(int m, int n, int k);
int rb_gemm_bf16_few(const void* a, const float* squares_in, float eps, const int32_t* rows, const void* w,
                     int w_layout, void* c, int dtype_out, int epilogue, const float* gain, void* gained,
                     float* squares_out, int m, int n, int k, void* stream);

// Causal attention of every token over its sequence's cache (keys 0..pos, or the last
// `window` of them), any head_dim that is even and at most 256.
//   q [T, Hq, D], out [T, Hq * D], both of dtype; pages as in rb_rope_kv_write.
int rb_attention_generic(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                         const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                         int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale,
                         int window, void* stream);

// The same for bfloat16 and head_dim 64 or 128 on the matrix cores.
//   prefill: sequences b = 0..B-1 hold tokens cu_seqlens[b]..cu_seqlens[b+1] at positions past_len[b]...
int rb_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                              const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                              int bt_stride, int n_seqs, int max_q_len, int n_heads, int n_kv_heads, int head_dim,
                              float scale, int window, void* stream);
//   decode: one token per sequence at position tok_pos[b]; the keys are split into
//   n_splits ranges whose partial results are combined in a second kernel.
//   workspace: float32 [B, Hq, n_splits, D + 2]
int rb_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                             const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                             int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                             float* workspace, void* stream);

//   decode, fused: rotation of q and the new k, cache write and attention in one kernel (plus the
//   combination of the splits when there are several).  qkv float32 [B, (Hq + 2 Hk) D] as for
//   rb_rope_kv_write.
int rb_attention_decode_fused_bf16(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos,
                                   const float* sin, int style, void* k_pages, void* v_pages, void* out,
                                   const int32_t* tok_pos, const int32_t* block_table,
                                   int bt_stride, int n_seqs, int n_heads, int n_kv_heads, int head_dim, float scale,
                                   int window, int n_splits, float* workspace, void* stream);

// tokens[r] = argmax of logits[r, :] (NaN counts as -inf, lowest index among equals), or, where
// temperature[r] > 0, the first index whose running sum of exp(z/T - max) reaches u[r] times the total.
// workspace: rb_sample_workspace_bytes(n_rows, vocab) bytes, 8-byte aligned, contents do not matter.
int rb_sample_workspace_bytes(int n_rows, int vocab);
int rb_sample(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
              int32_t* tokens, void* workspace, void* stream);

// rb_sample for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The
// same kernels and the same result as rb_sample, but the chunk statistics go into device memory
// that the library holds itself (256 KiB on every GPU it runs on, until the process ends), so no
// workspace is passed and neither this call nor anything under it allocates or frees.
// Limit: n_rows * ceil(vocab / 4096) <= rb_sample_static_max_stats() (16384: 512 rows of a
// 128k vocabulary); more is refused with an error and nothing is launched.  The stream must belong
// to the current device.  All calls on one GPU share that memory: two calls whose kernels may
// overlap there (different streams, no dependency between them) race; calls on one stream do not.
// The first use on a device asks the runtime for the address of that device's copy; before the
// first call under stream capture, call rb_sample_static_max_stats() (or rb_sample_static once) on
// that device outside of any capture.
int rb_sample_static_max_stats(void);
int rb_sample_static(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
                     int32_t* tokens, void* stream);

// Load-time helpers (weights_init.hip).
// rb_fill_normal: out[i] = mean + std * z_i for i < n, z_i the standard normal number that (key, i)
// fixes; the same bits as weights/random_init.py draws on the host.
int rb_fill_normal(void* out, int dtype, long long n, unsigned long long key, double mean, double std, void* stream);
// rb_place_rows: row r of src [n_rows, width] goes, cast to dst's dtype, to row
// row0 + (r / block) * period + r % block of dst [dst_rows, width].  block = n_rows places the rows
// one after another from row0 (q, k, v in one matrix); block 16, period 32, row0 0 and 16 interleave
// gate and up rows in blocks of 16.
// dst_layout 1: dst is fragment-major for its type (bfloat16: see rb_gemm_bf16, dst_rows % 16 == 0, width % 32 == 0;
// float32: see rb_gemm_generic, dst_rows % 16 == 0, width % 16 == 0).
int rb_place_rows(const void* src, int src_dtype, void* dst, int dst_dtype, int dst_layout, long long n_rows,
                  long long width, long long dst_rows, long long row0, long long block, long long period, void* stream);

// What the GPU reaches, measured the simplest way: rb_probe_read reads `bytes` bytes (a multiple of
// 16) once with 16-byte loads from `blocks` workgroups of 256 lanes (mode 0: all workgroups stride
// through the buffer together, plain loads; mode 1: every workgroup walks pieces of 64 KB of its own
// with non-temporal loads, which is a quarter faster on this GPU); rb_probe_mfma runs 4 * iters bfloat16 32x32x16 MFMAs in each of `waves`
// waves (a multiple of 4).  `sink` is one float of device memory that is practically never written.
int rb_probe_read(const void* p, long long bytes, int blocks, int mode, float* sink, void* stream);
int rb_probe_mfma(int waves, int iters, float* sink, void* stream);

#ifdef __cplusplus
}
#endif
