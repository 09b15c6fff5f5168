// The plain C++ twins of the kernels (see plain.h): host arrays, plain loops, sums in double.
// Formulas: crates/bitnet-core/src/llama/model.rs (matvec :67-91, rmsnorm :93-100, softmax
// :102-114, silu :116-120, rope :122-136, one token's forward :229-315) and runtime.rs:81-107
// (the choice of the next token), written for packed batches of tokens and a cache in pages.
#include "plain.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <vector>

namespace {

constexpr int PAGE = 64;
enum { F32 = 0, BF16 = 1 };

thread_local char g_error[512];

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

#define REQUIRE(cond, ...) \
  do {                     \
    if (!(cond)) return fail(__VA_ARGS__); \
  } while (0)

// ---------------------------------------------------------------- storage types
float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// round to nearest, ties to even; NaN stays NaN
uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

double load(const void* p, int dtype, size_t i) {
  return dtype == F32 ? (double)((const float*)p)[i] : (double)bf16_to_f32(((const uint16_t*)p)[i]);
}

void store(void* p, int dtype, size_t i, double v) {
  if (dtype == F32)
    ((float*)p)[i] = (float)v;
  else
    ((uint16_t*)p)[i] = f32_to_bf16((float)v);
}

bool dtype_ok(int d) { return d == F32 || d == BF16; }

// p[0] + p[stride] + ... in float32 and in that order: how a product's K slices are added up
float sum_terms(const float* p, int n_terms, size_t stride) {
  float v = p[0];
  for (int t = 1; t < n_terms; ++t) v += p[(size_t)t * stride];
  return v;
}

// Where element (row, col) of W [N, K] lies.  layout 0: rows.  layout 1: fragment-major, blocks of
// 16 rows x 4 E columns (E = values of the type in 16 bytes: 8 bfloat16, 4 float32) in the order
// [N / 16][K / (4 E)]; inside a block the value of row r, column q at E * (16 * (q / E) + r) + q % E.
size_t w_at(int layout, int dtype, long long n_cols, long long row, long long col) {
  if (layout == 0) return (size_t)(row * n_cols + col);
  const long long e = dtype == F32 ? 4 : 8;
  const long long block = (row / 16) * (n_cols / (4 * e)) + col / (4 * e);
  const long long r = row % 16, q = col % (4 * e);
  return (size_t)(block * 64 * e + e * (16 * (q / e) + r) + q % e);
}

double silu(double v) { return v / (1.0 + exp(-v)); }      // model.rs:116-120

// The page and the place inside it of position `pos` of the sequence whose row of the block table is bt.
size_t page_base(const int32_t* bt, int pos, int n_kv, int head_dim) {
  const int page = bt[pos / PAGE];
  return ((size_t)page * n_kv) * PAGE * head_dim + (size_t)(pos % PAGE) * head_dim;
}

// One query (head qh of n_heads, reading kv head qh / group) over the keys lo..pos of its sequence:
// scores times scale, softmax, weighted sum of the values (model.rs:262-289).  q: D values.
void attend(const double* q, const void* k_pages, const void* v_pages, int dtype, const int32_t* bt, int pos, int lo,
            int kvh, int n_kv, int d, float scale, double* out) {
  const int n = pos - lo + 1;
  std::vector<double> s(n);
  double mx = -INFINITY;
  for (int j = 0; j < n; ++j) {
    const size_t base = page_base(bt, lo + j, n_kv, d) + (size_t)kvh * PAGE * d;
    double dot = 0.0;
    for (int i = 0; i < d; ++i) dot += q[i] * load(k_pages, dtype, base + i);
    s[j] = dot * (double)scale;
    if (s[j] > mx) mx = s[j];
  }
  double total = 0.0;
  for (int j = 0; j < n; ++j) {
    s[j] = exp(s[j] - mx);
    total += s[j];
  }
  for (int i = 0; i < d; ++i) out[i] = 0.0;
  for (int j = 0; j < n; ++j) {
    const size_t base = page_base(bt, lo + j, n_kv, d) + (size_t)kvh * PAGE * d;
    const double p = total > 0.0 ? s[j] / total : s[j];
    for (int i = 0; i < d; ++i) out[i] += p * load(v_pages, dtype, base + i);
  }
}

int attention_tokens(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                     const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table, int bt_stride,
                     int n_tokens, int n_heads, int n_kv, int d, float scale, int window) {
  REQUIRE(dtype_ok(dtype), "attention: unknown dtype %d", dtype);
  REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: %d heads on %d kv heads", n_heads, n_kv);
  REQUIRE(d > 0 && d % 2 == 0, "attention: head_dim %d", d);
  const int group = n_heads / n_kv;
  std::vector<double> qv(d), o(d);
  for (int t = 0; t < n_tokens; ++t) {
    const int pos = tok_pos[t];
    const int32_t* bt = block_table + (size_t)(tok_seq ? tok_seq[t] : t) * bt_stride;
    const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    for (int h = 0; h < n_heads; ++h) {
      for (int i = 0; i < d; ++i) qv[i] = load(q, dtype, ((size_t)t * n_heads + h) * d + i);
      attend(qv.data(), k_pages, v_pages, dtype, bt, pos, lo, h / group, n_kv, d, scale, o.data());
      for (int i = 0; i < d; ++i) store(out, dtype, ((size_t)t * n_heads + h) * d + i, o[i]);
    }
  }
  return 0;
}

// C[i, j] = sum_k A[rows ? rows[i] : i, k] * W[j, k] in double
void product(const void* a, int a_dtype, const int32_t* rows, const void* w, int w_dtype, int w_layout, int m, int n,
             int k, std::vector<double>& c) {
  c.assign((size_t)m * n, 0.0);
  std::vector<double> ar(k);
  for (int i = 0; i < m; ++i) {
    const size_t src = rows ? (size_t)rows[i] : (size_t)i;
    for (int kk = 0; kk < k; ++kk) ar[kk] = load(a, a_dtype, src * k + kk);
    for (int j = 0; j < n; ++j) {
      double acc = 0.0;
      for (int kk = 0; kk < k; ++kk) acc += ar[kk] * load(w, w_dtype, w_at(w_layout, w_dtype, k, j, kk));
      c[(size_t)i * n + j] = acc;
    }
  }
}

// epilogue 1: W's rows are blocks of 16 gate rows followed by the 16 up rows of the same columns
void store_gated(const std::vector<double>& c, void* out, int dtype_out, int m, int n) {
  const int half = n / 2;
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < half; ++j) {
      const int blk = j / 16, r = j % 16;
      const double g = c[(size_t)i * n + 32 * blk + r], u = c[(size_t)i * n + 32 * blk + 16 + r];
      store(out, dtype_out, (size_t)i * half + j, silu(g) * u);
    }
}

}  // namespace

extern "C" {

const char* rbp_last_error(void) { return g_error; }
int rbp_page_size(void) { return PAGE; }

// x[t, :] = table[ids[t], :]  (model.rs:229-232; ids outside the table are an error, :225-227)
int rbp_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x, int n_tokens, int width,
                     void*) {
  REQUIRE(dtype_ok(table_dtype), "rbp_embed_gather: unknown dtype %d", table_dtype);
  for (int t = 0; t < n_tokens; ++t) {
    REQUIRE(ids[t] >= 0, "rbp_embed_gather: token id %d", ids[t]);
    for (int j = 0; j < width; ++j) x[(size_t)t * width + j] = (float)load(table, table_dtype, (size_t)ids[t] * width + j);
  }
  return 0;
}

// v = x[src] + sum of the terms of delta[src];  x[src] = v when all rows are taken;
// out[r] = v * gain / sqrt(mean(v^2) + eps)   (model.rs:93-100, the residual sums of :292-294, :304-306)
int rbp_add_rmsnorm(float* x, const float* delta, int n_terms, long long term_stride, const float* gain, float eps,
                    const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void*) {
  REQUIRE(dtype_ok(out_dtype), "rbp_add_rmsnorm: unknown dtype %d", out_dtype);
  REQUIRE(width > 0 && n_terms >= 1, "rbp_add_rmsnorm: width %d, %d terms", width, n_terms);
  std::vector<float> v(width);
  for (int r = 0; r < n_rows; ++r) {
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    double ss = 0.0;
    for (int j = 0; j < width; ++j) {
      float val = x[src * width + j];
      if (delta) val = val + sum_terms(delta + src * width + j, n_terms, (size_t)term_stride);      // float32, as stored
      v[j] = val;
      ss += (double)val * (double)val;
    }
    if (delta && !rows)
      for (int j = 0; j < width; ++j) x[src * width + j] = v[j];
    const double factor = 1.0 / sqrt(ss / width + (double)eps);
    for (int j = 0; j < width; ++j) store(out, out_dtype, (size_t)r * width + j, (double)v[j] * (double)gain[j] * factor);
  }
  return 0;
}

// Rotation of q and k by the table's angles, k and v into the pages (model.rs:122-136, :242-257).
// The rotation's float32 operations are the kernels': y0 = fma(x0, c, -(x1 * s)), y1 = fma(x0, s, x1 * c).
int rbp_rope_kv_write(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos, const float* sin,
                      int style, void* q_out, void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos,
                      const int32_t* tok_seq, const int32_t* block_table, int bt_stride, int n_tokens, int n_heads,
                      int n_kv_heads, int head_dim, void*) {
  REQUIRE(dtype_ok(cache_dtype), "rbp_rope_kv_write: unknown dtype %d", cache_dtype);
  REQUIRE(head_dim > 0 && head_dim % 2 == 0, "rbp_rope_kv_write: head_dim %d", head_dim);
  REQUIRE(style == 0 || style == 1, "rbp_rope_kv_write: style %d", style);
  const int half = head_dim / 2;
  const size_t row_width = (size_t)(n_heads + 2 * n_kv_heads) * head_dim;
  const size_t stride = (size_t)qkv_term_stride;
  for (int t = 0; t < n_tokens; ++t) {
    const int pos = tok_pos[t];
    const float* src = qkv + (size_t)t * row_width;
    size_t base = 0;
    if (k_pages) base = page_base(block_table + (size_t)tok_seq[t] * bt_stride, pos, n_kv_heads, head_dim);
    for (int h = 0; h < n_heads + n_kv_heads; ++h)
      for (int i = 0; i < half; ++i) {
        const int i0 = style == 0 ? 2 * i : i, i1 = style == 0 ? 2 * i + 1 : i + half;
        const float x0 = sum_terms(src + (size_t)h * head_dim + i0, qkv_terms, stride);
        const float x1 = sum_terms(src + (size_t)h * head_dim + i1, qkv_terms, stride);
        float y0 = x0, y1 = x1;
        if (cos) {
          const float c = cos[(size_t)pos * half + i], s = sin[(size_t)pos * half + i];
          y0 = fmaf(x0, c, -(x1 * s));
          y1 = fmaf(x0, s, x1 * c);
        }
        if (h < n_heads) {
          const size_t dst = ((size_t)t * n_heads + h) * head_dim;
          store(q_out, cache_dtype, dst + i0, y0);
          store(q_out, cache_dtype, dst + i1, y1);
        } else if (k_pages) {
          const size_t dst = base + (size_t)(h - n_heads) * PAGE * head_dim;
          store(k_pages, cache_dtype, dst + i0, y0);
          store(k_pages, cache_dtype, dst + i1, y1);
        }
      }
    if (v_pages) {
      const float* vsrc = src + (size_t)(n_heads + n_kv_heads) * head_dim;
      for (int h = 0; h < n_kv_heads; ++h)
        for (int d = 0; d < head_dim; ++d)
          store(v_pages, cache_dtype, base + (size_t)h * PAGE * head_dim + d,
                sum_terms(vsrc + (size_t)h * head_dim + d, qkv_terms, stride));
    }
  }
  return 0;
}

// t[r, j] = silu(gu[r, j]) * gu[r, F + j]  (model.rs:297-302)
int rbp_swiglu(const float* gu, void* out, int out_dtype, int n_rows, int ff, void*) {
  REQUIRE(dtype_ok(out_dtype), "rbp_swiglu: unknown dtype %d", out_dtype);
  for (int r = 0; r < n_rows; ++r)
    for (int j = 0; j < ff; ++j)
      store(out, out_dtype, (size_t)r * ff + j,
            silu((double)gu[(size_t)r * 2 * ff + j]) * (double)gu[(size_t)r * 2 * ff + ff + j]);
  return 0;
}

// C[M, N] = A[M, K] W[N, K]^T  (model.rs:67-91)
int rbp_gemm_generic(const void* a, const void* w, int w_layout, void* c, int dtype_in, int dtype_out, int m, int n,
                     int k, void*) {
  REQUIRE(dtype_ok(dtype_in) && dtype_ok(dtype_out), "rbp_gemm_generic: unknown dtype %d / %d", dtype_in, dtype_out);
  REQUIRE(m >= 0 && n > 0 && k > 0, "rbp_gemm_generic: bad sizes M=%d N=%d K=%d", m, n, k);
  REQUIRE(w_layout == 0 || (w_layout == 1 && dtype_in == F32 && n % 16 == 0 && k % 128 == 0),
          "rbp_gemm_generic: W layout %d with dtype %d, N=%d K=%d", w_layout, dtype_in, n, k);
  std::vector<double> acc;
  product(a, dtype_in, nullptr, w, dtype_in, w_layout, m, n, k, acc);
  for (size_t i = 0; i < acc.size(); ++i) store(c, dtype_out, i, acc[i]);
  return 0;
}

int rbp_gemm_bf16(const void* a, const void* w, int w_layout, void* c, int dtype_out, int epilogue, int m, int n, int k,
                  float*, void*) {
  REQUIRE(m >= 0 && n > 0 && k > 0, "rbp_gemm_bf16: bad sizes M=%d N=%d K=%d", m, n, k);
  REQUIRE(w_layout == 0 || (w_layout == 1 && k % 64 == 0 && n % 16 == 0), "rbp_gemm_bf16: W layout %d with N=%d K=%d",
          w_layout, n, k);
  REQUIRE(epilogue == 0 || (epilogue == 1 && n % 32 == 0), "rbp_gemm_bf16: epilogue %d with N=%d", epilogue, n);
  REQUIRE(dtype_ok(dtype_out), "rbp_gemm_bf16: unknown output dtype %d", dtype_out);
  std::vector<double> acc;
  product(a, BF16, nullptr, w, BF16, w_layout, m, n, k, acc);
  if (epilogue == 1) {
    store_gated(acc, c, dtype_out, m, n);
    return 0;
  }
  for (size_t i = 0; i < acc.size(); ++i) store(c, dtype_out, i, acc[i]);
  return 0;
}

// The product of 1..16 tokens with its neighbours folded in (see api.h):
//   squares_in: the tokens are bf16(x * gain) and squares_in the sums of x^2 over every 16 columns; the product
//   is multiplied by 1 / sqrt(sum / K + eps);
//   epilogue 2: C += product;  3: as 2, and gained = bf16(C * gain), squares_out = sums of C^2 over 16 columns.
int rbp_gemm_bf16_few(const void* a, const float* squares_in, float eps, const int32_t* rows, const void* w,
                      int w_layout, void* c, int dtype_out, int epilogue, const float* gain, void* gained,
                      float* squares_out, int m, int n, int k, void*) {
  REQUIRE(m >= 1 && m <= 16 && n > 0 && k > 0, "rbp_gemm_bf16_few: bad sizes M=%d N=%d K=%d", m, n, k);
  REQUIRE(w_layout == 0 || (w_layout == 1 && k % 64 == 0 && n % 16 == 0), "rbp_gemm_bf16_few: W layout %d", w_layout);
  REQUIRE(epilogue >= 0 && epilogue <= 3, "rbp_gemm_bf16_few: unknown epilogue %d", epilogue);
  REQUIRE(epilogue != 1 || n % 32 == 0, "rbp_gemm_bf16_few: gated epilogue with N=%d", n);
  REQUIRE(dtype_out == F32 || (dtype_out == BF16 && epilogue <= 1), "rbp_gemm_bf16_few: output dtype %d", dtype_out);
  REQUIRE(!squares_in || epilogue <= 1, "rbp_gemm_bf16_few: prepared rows with epilogue %d", epilogue);
  REQUIRE(epilogue != 3 || (gain && gained && squares_out), "rbp_gemm_bf16_few: epilogue 3 without its outputs");
  std::vector<double> acc;
  product(a, BF16, rows, w, BF16, w_layout, m, n, k, acc);
  if (squares_in) {
    const int n_sq = (k + 15) / 16;
    for (int i = 0; i < m; ++i) {
      const size_t src = rows ? (size_t)rows[i] : (size_t)i;
      double ss = 0.0;
      for (int j = 0; j < n_sq; ++j) ss += (double)squares_in[src * n_sq + j];
      const double factor = 1.0 / sqrt(ss / k + (double)eps);
      for (int j = 0; j < n; ++j) acc[(size_t)i * n + j] *= factor;
    }
  }
  if (epilogue == 1) {
    store_gated(acc, c, dtype_out, m, n);
    return 0;
  }
  if (epilogue == 0) {
    for (size_t i = 0; i < acc.size(); ++i) store(c, dtype_out, i, acc[i]);
    return 0;
  }
  float* cf = (float*)c;
  const int n_sq = (n + 15) / 16;
  for (int i = 0; i < m; ++i) {
    for (int j = 0; j < n; ++j) cf[(size_t)i * n + j] = (float)((double)cf[(size_t)i * n + j] + acc[(size_t)i * n + j]);
    if (epilogue == 3) {
      for (int j = 0; j < n; ++j)
        ((uint16_t*)gained)[(size_t)i * n + j] = f32_to_bf16(cf[(size_t)i * n + j] * gain[j]);
      for (int b = 0; b < n_sq; ++b) {
        double ss = 0.0;
        for (int j = 16 * b; j < n && j < 16 * b + 16; ++j) ss += (double)cf[(size_t)i * n + j] * (double)cf[(size_t)i * n + j];
        squares_out[(size_t)i * n_sq + b] = (float)ss;
      }
    }
  }
  return 0;
}

int rbp_attention_generic(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                          const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table, int bt_stride,
                          int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale, int window, void*) {
  return attention_tokens(q, k_pages, v_pages, out, dtype, tok_pos, tok_seq, block_table, bt_stride, n_tokens, n_heads,
                          n_kv_heads, head_dim, scale, window);
}

// sequences b hold tokens cu_seqlens[b] .. cu_seqlens[b + 1] at positions past_len[b] ...
int rbp_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                               const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                               int bt_stride, int n_seqs, int max_q_len, int n_heads, int n_kv_heads, int head_dim,
                               float scale, int window, void*) {
  const int n_tokens = cu_seqlens[n_seqs];
  std::vector<int32_t> pos(n_tokens > 0 ? n_tokens : 1), seq(n_tokens > 0 ? n_tokens : 1);
  for (int b = 0; b < n_seqs; ++b) {
    REQUIRE(cu_seqlens[b + 1] - cu_seqlens[b] <= max_q_len, "rbp_attention_prefill_bf16: sequence %d brings more than %d tokens",
            b, max_q_len);
    for (int t = cu_seqlens[b]; t < cu_seqlens[b + 1]; ++t) {
      pos[t] = past_len[b] + (t - cu_seqlens[b]);
      seq[t] = b;
    }
  }
  return attention_tokens(q, k_pages, v_pages, out, BF16, pos.data(), seq.data(), block_table, bt_stride, n_tokens,
                          n_heads, n_kv_heads, head_dim, scale, window);
}

// one token per sequence at position tok_pos[b]
int rbp_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                              const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                              int n_heads, int n_kv_heads, int head_dim, float scale, int window, int, float*, void*) {
  return attention_tokens(q, k_pages, v_pages, out, BF16, tok_pos, nullptr, block_table, bt_stride, n_seqs, n_heads,
                          n_kv_heads, head_dim, scale, window);
}

// rotation of q and the new k, cache write and attention of one token per sequence
int rbp_attention_decode_fused_bf16(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos,
                                    const float* sin, int style, void* k_pages, void* v_pages, void* out,
                                    const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                                    int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                                    float* workspace, void* stream) {
  std::vector<uint16_t> q((size_t)(n_seqs > 0 ? n_seqs : 1) * n_heads * head_dim);
  std::vector<int32_t> seq(n_seqs > 0 ? n_seqs : 1);
  for (int b = 0; b < n_seqs; ++b) seq[b] = b;
  int rc = rbp_rope_kv_write(qkv, qkv_terms, qkv_term_stride, cos, sin, style, q.data(), k_pages, v_pages, BF16, tok_pos,
                             seq.data(), block_table, bt_stride, n_seqs, n_heads, n_kv_heads, head_dim, stream);
  if (rc) return rc;
  return rbp_attention_decode_bf16(q.data(), k_pages, v_pages, out, tok_pos, block_table, bt_stride, n_seqs, n_heads,
                                   n_kv_heads, head_dim, scale, window, n_splits, workspace, stream);
}

// The greatest logit, NaN counted as -inf, the lowest index among equals; or, where temperature[r] > 0,
// the first index whose running sum of exp(z / T - max / T) reaches u[r] times the total, the last index
// if none does (runtime.rs:81-107).
int rbp_sample(const float* logits, int n_rows, int vocab, const float* temperature, const float* u, int32_t* tokens,
               void*, void*) {
  REQUIRE(vocab > 0, "rbp_sample: vocabulary %d", vocab);
  for (int r = 0; r < n_rows; ++r) {
    const float* row = logits + (size_t)r * vocab;
    float best = -INFINITY;
    int arg = 0;
    bool any = false;
    for (int i = 0; i < vocab; ++i) {
      const float v = row[i] != row[i] ? -INFINITY : row[i];
      if (!any || v > best) {
        best = v;
        arg = i;
        any = true;
      }
    }
    const float temp = temperature ? temperature[r] : 0.f;
    if (!(temp > 0.f) || best == -INFINITY) {
      tokens[r] = arg;
      continue;
    }
    const float zmax = best / temp;
    double total = 0.0;
    for (int i = 0; i < vocab; ++i) {
      const float v = row[i] != row[i] ? -INFINITY : row[i];
      total += (double)expf(v / temp - zmax);
    }
    const double target = (double)u[r] * total;
    double run = 0.0;
    int pick = vocab - 1;
    for (int i = 0; i < vocab; ++i) {
      const float v = row[i] != row[i] ? -INFINITY : row[i];
      run += (double)expf(v / temp - zmax);
      if (run >= target) {
        pick = i;
        break;
      }
    }
    tokens[r] = pick;
  }
  return 0;
}

// Row r of src goes to row row0 + (r / block) * period + r % block of dst, cast to dst's type;
// dst_layout 1: dst is fragment-major.
int rbp_place_rows(const void* src, int src_dtype, void* dst, int dst_dtype, int dst_layout, long long n_rows,
                   long long width, long long dst_rows, long long row0, long long block, long long period, void*) {
  REQUIRE(dtype_ok(src_dtype) && dtype_ok(dst_dtype), "rbp_place_rows: unknown dtype %d / %d", src_dtype, dst_dtype);
  REQUIRE(block > 0 && period >= block, "rbp_place_rows: block %lld, period %lld", block, period);
  REQUIRE(dst_layout == 0 || (dst_layout == 1 && dst_rows % 16 == 0 && width % (dst_dtype == F32 ? 16 : 32) == 0),
          "rbp_place_rows: layout %d for %lld rows of %lld", dst_layout, dst_rows, width);
  for (long long r = 0; r < n_rows; ++r) {
    const long long to = row0 + (r / block) * period + r % block;
    REQUIRE(to >= 0 && to < dst_rows, "rbp_place_rows: row %lld goes to %lld of %lld", r, to, dst_rows);
    for (long long j = 0; j < width; ++j)
      store(dst, dst_dtype, w_at(dst_layout, dst_dtype, width, to, j), load(src, src_dtype, (size_t)(r * width + j)));
  }
  return 0;
}

}  // extern "C"
