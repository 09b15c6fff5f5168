// Plain C++ twins of the kernels: for every entry point of api.h that a step of a model
// calls, a function of the same name with the prefix rbp_ and the same parameters, working on
// host arrays with plain loops (the reference's loops, crates/bitnet-core/src/llama/model.rs:67-136
// and :229-315, written for a batch and a paged cache).  They are the kernels' oracle: built by
// the host compiler into a library of their own that needs no GPU, run under the address and
// undefined-behaviour sanitizers by a self-test, compared with the tests' plain implementation
// on the CPU and with the kernels on the GPU.
//
// Every pointer is a host pointer; `stream` and `workspace` are accepted and ignored.  Sums
// run in double and are rounded once to the result's type, so a twin is at least as exact as
// its kernel and the tests' tolerances are the kernels' own rounding.  Where a kernel's float32
// operations are part of its contract (the rotation of a pair, the order in which the terms of
// a product cut into K slices are added), the twin does the same operations in the same order.
// Each returns 0, or 1 after storing a message for rbp_last_error().
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* rbp_last_error(void);
int rbp_page_size(void);

int rbp_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x, int n_tokens, int width,
                     void* stream);
int rbp_add_rmsnorm(float* x, const float* delta, int n_terms, long long term_stride, const float* gain, float eps,
                    const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void* stream);
int rbp_rope_kv_write(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos, const float* sin,
                      int style, void* q_out, void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos,
                      const int32_t* tok_seq, const int32_t* block_table, int bt_stride, int n_tokens, int n_heads,
                      int n_kv_heads, int head_dim, void* stream);
int rbp_swiglu(const float* gu, void* out, int out_dtype, int n_rows, int ff, void* stream);
int rbp_gemm_generic(const void* a, const void* w, int w_layout, void* c, int dtype_in, int dtype_out, int m, int n,
                     int k, void* stream);
int rbp_gemm_bf16(const void* a, const void* w, int w_layout, void* c, int dtype_out, int epilogue, int m, int n, int k,
                  float* workspace, void* stream);
int rbp_gemm_bf16_few(const void* a, const float* squares_in, float eps, const int32_t* rows, const void* w,
                      int w_layout, void* c, int dtype_out, int epilogue, const float* gain, void* gained,
                      float* squares_out, int m, int n, int k, void* stream);
int rbp_attention_generic(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                          const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table, int bt_stride,
                          int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale, int window,
                          void* stream);
int rbp_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                               const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                               int bt_stride, int n_seqs, int max_q_len, int n_heads, int n_kv_heads, int head_dim,
                               float scale, int window, void* stream);
int rbp_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                              const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                              int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                              float* workspace, void* stream);
int rbp_attention_decode_fused_bf16(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos,
                                    const float* sin, int style, void* k_pages, void* v_pages, void* out,
                                    const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                                    int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                                    float* workspace, void* stream);
int rbp_sample(const float* logits, int n_rows, int vocab, const float* temperature, const float* u, int32_t* tokens,
               void* workspace, void* stream);
int rbp_place_rows(const void* src, int src_dtype, void* dst, int dst_dtype, int dst_layout, long long n_rows,
                   long long width, long long dst_rows, long long row0, long long block, long long period,
                   void* stream);

#ifdef __cplusplus
}
#endif
