// Embedding gather, fused residual-add + RMS norm, rotary encoding with cache write,
// SiLU gate.  All arithmetic in float32; storage float32 or bfloat16.
#include <stdarg.h>
#include <stdio.h>

#include "api.h"
#include "common.h"

// ---------------------------------------------------------------- errors
static thread_local char g_error[512];
void rb_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
extern "C" const char* rb_last_error(void) { return g_error; }
extern "C" int rb_version(void) { return 1; }
extern "C" int rb_page_size(void) { return RB_PAGE; }

// ---------------------------------------------------------------- the machine
static int g_tune_cus = 0;
extern "C" void rb_tune_compute_units(int n) { g_tune_cus = n; }      // tests and experiments; 0 = the device's own
int rb_compute_units(void) {
  if (g_tune_cus > 0) return g_tune_cus;
  static int known[64];                 // per device, 0 = not asked yet (a race writes the same number twice)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (known[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    known[dev] = n;
  }
  return known[dev];
}

// ---------------------------------------------------------------- embedding
// Reference: x[j] = token_embd[j + tok * n_embd] (llama/model.rs:229-232).
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                                    float* __restrict__ x, int width) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * width;
  float* dst = x + (size_t)t * width;
  for (int j = threadIdx.x; j < width; j += blockDim.x) dst[j] = Num<T>::load(row + j);
}

extern "C" int rb_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x, int n_tokens,
                               int width, void* stream) {
  RB_RECORDED(rb_embed_gather(table, table_dtype, ids, x, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0, "rb_embed_gather: bad sizes %d x %d", n_tokens, width);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == RB_F32)
    embed_gather_kernel<float><<<n_tokens, 256, 0, s>>>((const float*)table, ids, x, width);
  else if (table_dtype == RB_BF16)
    embed_gather_kernel<bf16_t><<<n_tokens, 256, 0, s>>>((const bf16_t*)table, ids, x, width);
  else
    RB_REQUIRE(false, "rb_embed_gather: unknown dtype %d", table_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- add + rmsnorm
// Reference: s = sum(x^2)/n; scale = 1/sqrt(s + eps); y = x * w * scale
// (llama/model.rs:93-100); residual adds are plain sums (:292-294, :304-306).
// delta may be several terms, term_stride floats apart (the partial sums that the K slices of a
// product left): they are added up first, in their order, and the total is added to x.
template <typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ delta, int n_terms,
                                   size_t term_stride, const float* __restrict__ gain, float eps,
                                   const int32_t* __restrict__ rows, int width, TO* __restrict__ out) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = x + src * width;
  const float* dr = delta ? delta + src * width : nullptr;
  const bool write_back = (delta != nullptr) && (rows == nullptr);
  float ss = 0.f;
  auto terms = [&](int j) {
    float d = dr[j];
    for (int p = 1; p < n_terms; ++p) d += dr[(size_t)p * term_stride + j];
    return d;
  };
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    float v = xr[j];
    if (dr) v += terms(j);
    if (write_back) xr[j] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)width + eps);
  TO* orow = out + (size_t)r * width;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    float v = xr[j];
    if (dr && !write_back) v += terms(j);
    Num<TO>::store(orow + j, v * gain[j] * scale);
  }
}

// The same for widths that are a multiple of 4 and fit the block's registers: every thread
// loads its share of the row once with 16-byte loads (the gain too, before the sum is
// known), so the row makes one trip from memory and the loads are all in flight together.
// Several terms are read by four times the threads, each with four terms' loads in flight.
__device__ __forceinline__ void add4(float4& d, const float4& e) {
  d.x += e.x;
  d.y += e.y;
  d.z += e.z;
  d.w += e.w;
}

template <typename TO, int VPT, int THREADS>          // VPT float4 per thread
__global__ __launch_bounds__(THREADS) void add_rmsnorm_vec_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                              int n_terms, size_t term_stride,
                                                              const float* __restrict__ gain, float eps,
                                                              const int32_t* __restrict__ rows, int width,
                                                              TO* __restrict__ out) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float4* xr = reinterpret_cast<float4*>(x + src * width);
  const float4* dr = delta ? reinterpret_cast<const float4*>(delta + src * width) : nullptr;
  const float4* gr = reinterpret_cast<const float4*>(gain);
  const bool write_back = (delta != nullptr) && (rows == nullptr);
  const int n4 = width / 4;
  float4 v[VPT], g[VPT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c < n4) {
      v[i] = xr[c];
      g[i] = gr[c];
      if (dr) {
        float4 d = dr[c];
        const float* term = delta + src * width + 4 * c;
        auto at = [&](int p) { return *reinterpret_cast<const float4*>(term + (size_t)p * term_stride); };
        int p = 1;
        for (; p + 3 < n_terms; p += 4) {
          const float4 e0 = at(p), e1 = at(p + 1), e2 = at(p + 2), e3 = at(p + 3);
          add4(d, e0);
          add4(d, e1);
          add4(d, e2);
          add4(d, e3);
        }
        for (; p < n_terms; ++p) add4(d, at(p));
        add4(v[i], d);
      }
    } else {
      v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      g[i] = v[i];
    }
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (write_back && c < n4) xr[c] = v[i];
    ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)width + eps);
  TO* orow = out + (size_t)r * width;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c < n4) {
      Num<TO>::store(orow + 4 * c + 0, v[i].x * g[i].x * scale);
      Num<TO>::store(orow + 4 * c + 1, v[i].y * g[i].y * scale);
      Num<TO>::store(orow + 4 * c + 2, v[i].z * g[i].z * scale);
      Num<TO>::store(orow + 4 * c + 3, v[i].w * g[i].w * scale);
    }
  }
}

template <typename TO>
static bool launch_add_rmsnorm_vec(float* x, const float* delta, int n_terms, size_t term_stride, const float* gain,
                                   float eps, const int32_t* rows, int n_rows, int width, TO* out, hipStream_t s) {
  if (width % 4 != 0 || term_stride % 4 != 0) return false;
  const int n4 = width / 4;
  if (delta && n_terms > 1 && n4 > 256 && n4 <= 2048) {
    if (n4 <= 1024)
      add_rmsnorm_vec_kernel<TO, 1, 1024><<<n_rows, 1024, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, out);
    else
      add_rmsnorm_vec_kernel<TO, 2, 1024><<<n_rows, 1024, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, out);
    return true;
  }
  if (n4 <= 256)
    add_rmsnorm_vec_kernel<TO, 1, 256><<<n_rows, 256, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, out);
  else if (n4 <= 512)
    add_rmsnorm_vec_kernel<TO, 2, 256><<<n_rows, 256, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, out);
  else if (n4 <= 1024)
    add_rmsnorm_vec_kernel<TO, 4, 256><<<n_rows, 256, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, out);
  else if (n4 <= 2048)
    add_rmsnorm_vec_kernel<TO, 8, 256><<<n_rows, 256, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, out);
  else
    return false;
  return true;
}

extern "C" int rb_add_rmsnorm(float* x, const float* delta, int n_terms, long long term_stride_ll, const float* gain,
                              float eps, const int32_t* rows, int n_rows, int width, void* out, int out_dtype,
                              void* stream) {
  RB_RECORDED(rb_add_rmsnorm(x, delta, n_terms, term_stride_ll, gain, eps, rows, n_rows, width, out, out_dtype, stream));
  RB_REQUIRE(n_rows >= 0 && width > 0, "rb_add_rmsnorm: bad sizes %d x %d", n_rows, width);
  RB_REQUIRE(!delta || (n_terms >= 1 && term_stride_ll >= 0), "rb_add_rmsnorm: %d terms, %lld apart", n_terms,
             term_stride_ll);
  const size_t term_stride = (size_t)term_stride_ll;
  if (n_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = width >= 2048 ? 512 : 256;
  if (out_dtype == RB_F32 && launch_add_rmsnorm_vec<float>(x, delta, n_terms, term_stride, gain, eps, rows, n_rows, width, (float*)out, s)) {
  } else if (out_dtype == RB_BF16 &&
             launch_add_rmsnorm_vec<bf16_t>(x, delta, n_terms, term_stride, gain, eps, rows, n_rows, width, (bf16_t*)out, s)) {
  } else if (out_dtype == RB_F32)
    add_rmsnorm_kernel<float><<<n_rows, threads, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, (float*)out);
  else if (out_dtype == RB_BF16)
    add_rmsnorm_kernel<bf16_t><<<n_rows, threads, 0, s>>>(x, delta, n_terms, term_stride, gain, eps, rows, width, (bf16_t*)out);
  else
    RB_REQUIRE(false, "rb_add_rmsnorm: unknown dtype %d", out_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- rope + cache write
// Reference: for i < D/2 the pair is rotated by pos * inv_i,
//   x0' = x0 cos - x1 sin, x1' = x0 sin + x1 cos (llama/model.rs:122-136), for every q
// head and k head (:242-252); k is cached rotated, v as it is (:254-257).
template <typename TC>
__global__ void rope_kv_write_kernel(const float* __restrict__ qkv, int n_terms, size_t term_stride,
                                     const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t, int style, TC* __restrict__ q_out,
                                     TC* __restrict__ k_pages, TC* __restrict__ v_pages,
                                     const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                                     const int32_t* __restrict__ block_table, int bt_stride, int n_heads,
                                     int n_kv, int head_dim) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int half = head_dim / 2;
  const int row_width = (n_heads + 2 * n_kv) * head_dim;
  const float* src = qkv + (size_t)t * row_width;
  const float* cr = cos_t ? cos_t + (size_t)pos * half : nullptr;
  const float* sr = sin_t ? sin_t + (size_t)pos * half : nullptr;
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * head_dim + (size_t)(pos % RB_PAGE) * head_dim;
  }
  // rotated pairs: q heads and k heads
  const int n_rot = (n_heads + n_kv) * half;
  for (int idx = threadIdx.x; idx < n_rot; idx += blockDim.x) {
    const int h = idx / half;
    const int i = idx - h * half;
    const int i0 = style == 0 ? 2 * i : i;
    const int i1 = style == 0 ? 2 * i + 1 : i + half;
    const float x0 = sum_terms(src + h * head_dim + i0, n_terms, term_stride);
    const float x1 = sum_terms(src + h * head_dim + i1, n_terms, term_stride);
    float y0 = x0, y1 = x1;
    if (cr) {
      const float c = cr[i], s = sr[i];
      rotate_pair(x0, x1, c, s, y0, y1);
    }
    if (h < n_heads) {
      TC* dst = q_out + ((size_t)t * n_heads + h) * head_dim;
      Num<TC>::store(dst + i0, y0);
      Num<TC>::store(dst + i1, y1);
    } else if (k_pages) {
      TC* dst = k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * head_dim;
      Num<TC>::store(dst + i0, y0);
      Num<TC>::store(dst + i1, y1);
    }
  }
  if (v_pages) {
    const float* vsrc = src + (size_t)(n_heads + n_kv) * head_dim;
    for (int idx = threadIdx.x; idx < n_kv * head_dim; idx += blockDim.x) {
      const int h = idx / head_dim;
      const int d = idx - h * head_dim;
      Num<TC>::store(v_pages + page_base + (size_t)h * RB_PAGE * head_dim + d,
                     sum_terms(vsrc + idx, n_terms, term_stride));
    }
  }
}

// The same with four pairs a thread: 16-byte loads of the projections and the angle tables, 8- and
// 16-byte stores (bfloat16) instead of 4-byte loads and 2-byte stores.  Needs head sizes that are
// multiples of 8 and 16-byte aligned rows, which the launcher checks.
__device__ __forceinline__ float4 sum_terms4(const float* __restrict__ p, int n_terms, size_t stride) {
  float4 v = *reinterpret_cast<const float4*>(p);
  for (int t = 1; t < n_terms; ++t) {
    const float4 e = *reinterpret_cast<const float4*>(p + (size_t)t * stride);
    v.x += e.x;
    v.y += e.y;
    v.z += e.z;
    v.w += e.w;
  }
  return v;
}
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}

template <typename TC>
__global__ void rope_kv_write_vec_kernel(const float* __restrict__ qkv, int n_terms, size_t term_stride,
                                         const float* __restrict__ cos_t, const float* __restrict__ sin_t, int style,
                                         TC* __restrict__ q_out, TC* __restrict__ k_pages, TC* __restrict__ v_pages,
                                         const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                                         const int32_t* __restrict__ block_table, int bt_stride, int n_heads,
                                         int n_kv, int head_dim) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int half = head_dim / 2;
  const int quads = half / 4;
  const int row_width = (n_heads + 2 * n_kv) * head_dim;
  const float* src = qkv + (size_t)t * row_width;
  const float* cr = cos_t ? cos_t + (size_t)pos * half : nullptr;
  const float* sr = sin_t ? sin_t + (size_t)pos * half : nullptr;
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * head_dim + (size_t)(pos % RB_PAGE) * head_dim;
  }
  const int first = q_out ? 0 : n_heads * quads;      // without q_out only k is rotated
  for (int idx = first + threadIdx.x; idx < (n_heads + n_kv) * quads; idx += blockDim.x) {
    const int h = idx / quads;
    const int i = 4 * (idx - h * quads);
    if (h >= n_heads && !k_pages) break;
    TC* dst = h < n_heads ? q_out + ((size_t)t * n_heads + h) * head_dim
                          : k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * head_dim;
    float4 c = make_float4(1.f, 1.f, 1.f, 1.f), sn = make_float4(0.f, 0.f, 0.f, 0.f);
    if (cr) {
      c = *reinterpret_cast<const float4*>(cr + i);
      sn = *reinterpret_cast<const float4*>(sr + i);
    }
    const float* hp = src + h * head_dim;
    if (style == 0) {
      // pairs (2 i, 2 i + 1): eight consecutive values
      const float4 a = sum_terms4(hp + 2 * i, n_terms, term_stride), b = sum_terms4(hp + 2 * i + 4, n_terms, term_stride);
      float y[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      if (cr) {
        rotate_pair(a.x, a.y, c.x, sn.x, y[0], y[1]);
        rotate_pair(a.z, a.w, c.y, sn.y, y[2], y[3]);
        rotate_pair(b.x, b.y, c.z, sn.z, y[4], y[5]);
        rotate_pair(b.z, b.w, c.w, sn.w, y[6], y[7]);
      }
      store4(dst + 2 * i, y[0], y[1], y[2], y[3]);
      store4(dst + 2 * i + 4, y[4], y[5], y[6], y[7]);
    } else {
      // pairs (i, i + half): four values of each half
      const float4 a = sum_terms4(hp + i, n_terms, term_stride), b = sum_terms4(hp + half + i, n_terms, term_stride);
      float y0[4] = {a.x, a.y, a.z, a.w}, y1[4] = {b.x, b.y, b.z, b.w};
      if (cr) {
        rotate_pair(a.x, b.x, c.x, sn.x, y0[0], y1[0]);
        rotate_pair(a.y, b.y, c.y, sn.y, y0[1], y1[1]);
        rotate_pair(a.z, b.z, c.z, sn.z, y0[2], y1[2]);
        rotate_pair(a.w, b.w, c.w, sn.w, y0[3], y1[3]);
      }
      store4(dst + i, y0[0], y0[1], y0[2], y0[3]);
      store4(dst + half + i, y1[0], y1[1], y1[2], y1[3]);
    }
  }
  if (v_pages) {
    const float* vsrc = src + (size_t)(n_heads + n_kv) * head_dim;
    for (int idx = 4 * threadIdx.x; idx < n_kv * head_dim; idx += 4 * blockDim.x) {
      const int h = idx / head_dim;
      const int d = idx - h * head_dim;
      const float4 v = sum_terms4(vsrc + idx, n_terms, term_stride);
      store4(v_pages + page_base + (size_t)h * RB_PAGE * head_dim + d, v.x, v.y, v.z, v.w);
    }
  }
}

extern "C" int rb_rope_kv_write(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos,
                                const float* sin, int style, void* q_out,
                                void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos,
                                const int32_t* tok_seq, const int32_t* block_table, int bt_stride, int n_tokens,
                                int n_heads, int n_kv_heads, int head_dim, void* stream) {
  RB_RECORDED(rb_rope_kv_write(qkv, qkv_terms, qkv_term_stride, cos, sin, style, q_out, k_pages, v_pages, cache_dtype,
                               tok_pos, tok_seq, block_table, bt_stride, n_tokens, n_heads, n_kv_heads, head_dim, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && head_dim > 0 && head_dim % 2 == 0,
             "rb_rope_kv_write: bad sizes T=%d Hq=%d Hk=%d D=%d", n_tokens, n_heads, n_kv_heads, head_dim);
  RB_REQUIRE(qkv_terms >= 1 && qkv_term_stride >= 0, "rb_rope_kv_write: %d terms, %lld apart", qkv_terms,
             qkv_term_stride);
  RB_REQUIRE((cos == nullptr) == (sin == nullptr), "rb_rope_kv_write: cos and sin tables go together");
  RB_REQUIRE(style == 0 || style == 1, "rb_rope_kv_write: unknown pairing style %d", style);
  RB_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rb_rope_kv_write: k and v pages go together");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool vec = head_dim % 8 == 0 && qkv_term_stride % 4 == 0 && aligned(qkv) && aligned(cos) && aligned(sin) &&
                   aligned(q_out) && aligned(k_pages) && aligned(v_pages);
  if (vec && cache_dtype == RB_F32)
    rope_kv_write_vec_kernel<float><<<n_tokens, 256, 0, s>>>(qkv, qkv_terms, (size_t)qkv_term_stride, cos, sin, style,
                                                             (float*)q_out, (float*)k_pages, (float*)v_pages, tok_pos,
                                                             tok_seq, block_table, bt_stride, n_heads, n_kv_heads,
                                                             head_dim);
  else if (vec && cache_dtype == RB_BF16)
    rope_kv_write_vec_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(qkv, qkv_terms, (size_t)qkv_term_stride, cos, sin, style,
                                                              (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages,
                                                              tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                              n_kv_heads, head_dim);
  else if (cache_dtype == RB_F32)
    rope_kv_write_kernel<float><<<n_tokens, 256, 0, s>>>(qkv, qkv_terms, (size_t)qkv_term_stride, cos, sin, style, (float*)q_out, (float*)k_pages,
                                                         (float*)v_pages, tok_pos, tok_seq, block_table,
                                                         bt_stride, n_heads, n_kv_heads, head_dim);
  else if (cache_dtype == RB_BF16)
    rope_kv_write_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(qkv, qkv_terms, (size_t)qkv_term_stride, cos, sin, style, (bf16_t*)q_out,
                                                          (bf16_t*)k_pages, (bf16_t*)v_pages, tok_pos, tok_seq,
                                                          block_table, bt_stride, n_heads, n_kv_heads, head_dim);
  else
    RB_REQUIRE(false, "rb_rope_kv_write: unknown dtype %d", cache_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- SiLU gate
// Reference: silu(v) = v / (1 + exp(-v)); t = silu(gate) * up (llama/model.rs:116-120, 297-302).
template <typename TO>
__global__ void swiglu_kernel(const float* __restrict__ gu, TO* __restrict__ out, int ff) {
  const size_t r = blockIdx.y;
  const float* g = gu + r * 2 * (size_t)ff;
  const float* u = g + ff;
  TO* o = out + r * (size_t)ff;
  for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < ff; j += gridDim.x * blockDim.x) {
    const float gv = g[j];
    Num<TO>::store(o + j, gv / (1.0f + expf(-gv)) * u[j]);
  }
}

extern "C" int rb_swiglu(const float* gu, void* out, int out_dtype, int n_rows, int ff, void* stream) {
  RB_RECORDED(rb_swiglu(gu, out, out_dtype, n_rows, ff, stream));
  RB_REQUIRE(n_rows >= 0 && ff > 0, "rb_swiglu: bad sizes %d x %d", n_rows, ff);
  RB_REQUIRE(n_rows <= 65535 * 64, "rb_swiglu: too many rows %d", n_rows);
  if (n_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  // rows go to grid.y in chunks so that any row count fits the launch limits
  for (int r0 = 0; r0 < n_rows; r0 += 65535) {
    const int nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    dim3 grid((ff + 255) / 256 < 64 ? (ff + 255) / 256 : 64, nr);
    const float* src = gu + (size_t)r0 * 2 * ff;
    if (out_dtype == RB_F32)
      swiglu_kernel<float><<<grid, 256, 0, s>>>(src, (float*)out + (size_t)r0 * ff, ff);
    else if (out_dtype == RB_BF16)
      swiglu_kernel<bf16_t><<<grid, 256, 0, s>>>(src, (bf16_t*)out + (size_t)r0 * ff, ff);
    else
      RB_REQUIRE(false, "rb_swiglu: unknown dtype %d", out_dtype);
  }
  RB_LAUNCH_CHECK();
  return 0;
}
