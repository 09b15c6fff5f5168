// Causal attention of each token over its sequence's paged cache: any even head_dim up to
// 256, any number of heads and groups, float32 or bfloat16 storage, float32 arithmetic
// throughout (scores, softmax, weighted sum).  One workgroup per (token, query head): one wave
// when the step has many tokens, up to 8 waves that share the pages of the context and merge
// their running softmax states through LDS when it has few (a decode step of 8 sequences and
// 32 heads would otherwise leave three quarters of the GPU idle, each wave walking its whole
// context alone).
//
// Reference: kv head = q head / (Hq / Hk); s[p] = (q . K[p]) * scale for p <= pos;
// softmax with the maximum subtracted; out = sum_p s[p] V[p]  (llama/model.rs:260-289,
// softmax :102-114).  The softmax is computed page by page with a running maximum, which
// is the same value up to rounding.
#include <math.h>

#include "api.h"
#include "common.h"

#define AG_MAX_D 256

#define AG_MAX_WAVES 8

template <typename T>
__global__ __launch_bounds__(RB_WAVE * AG_MAX_WAVES) void attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages, T* __restrict__ out,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ block_table, int bt_stride, int n_heads, int n_kv, int head_dim, float scale,
    int window) {
  __shared__ float qs[AG_MAX_D];
  __shared__ float ps_all[AG_MAX_WAVES][RB_PAGE];
  __shared__ float red_m[AG_MAX_WAVES], red_l[AG_MAX_WAVES];
  __shared__ float red_acc[AG_MAX_WAVES][AG_MAX_D];
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x & (RB_WAVE - 1);
  const int wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  float* ps = ps_all[wave];
  const int pos = tok_pos[t];
  const int kvh = h / (n_heads / n_kv);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* pages = block_table + (size_t)tok_seq[t] * bt_stride;

  const T* qrow = q + ((size_t)t * n_heads + h) * head_dim;
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) qs[d] = Num<T>::load(qrow + d);
  __syncthreads();

  float m_run = -INFINITY, l_run = 0.f;
  float acc[AG_MAX_D / RB_WAVE];
#pragma unroll
  for (int i = 0; i < AG_MAX_D / RB_WAVE; ++i) acc[i] = 0.f;

  for (int pg = lo / RB_PAGE + wave; pg <= pos / RB_PAGE; pg += n_waves) {
    const size_t base = ((size_t)pages[pg] * n_kv + kvh) * RB_PAGE * head_dim;
    const int p = pg * RB_PAGE + lane;
    float s = -INFINITY;
    if (p >= lo && p <= pos) {
      const T* krow = k_pages + base + (size_t)lane * head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], Num<T>::load(krow + d), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m_run, wave_max(s));      // finite: the page holds at least one valid key
    const float pexp = (s == -INFINITY) ? 0.f : expf(s - m_new);
    const float corr = (m_run == -INFINITY) ? 0.f : expf(m_run - m_new);
    l_run = l_run * corr + wave_sum(pexp);
    m_run = m_new;
    // ps belongs to this wave alone; a wave's LDS accesses complete in order
    ps[lane] = pexp;
    __builtin_amdgcn_wave_barrier();
    const int j_lo = (pg * RB_PAGE < lo) ? lo - pg * RB_PAGE : 0;
    const int j_hi = (pg * RB_PAGE + RB_PAGE - 1 > pos) ? pos - pg * RB_PAGE : RB_PAGE - 1;
#pragma unroll
    for (int i = 0; i < AG_MAX_D / RB_WAVE; ++i) {
      const int d = lane + i * RB_WAVE;
      if (d < head_dim) {
        float a = acc[i] * corr;
        const T* vcol = v_pages + base + d;
        for (int j = j_lo; j <= j_hi; ++j) a = fmaf(ps[j], Num<T>::load(vcol + (size_t)j * head_dim), a);
        acc[i] = a;
      }
    }
  }
  // ---- the waves' states into one (a wave without pages holds m = -inf, l = 0, acc = 0)
  if (n_waves > 1) {
    if (lane == 0) {
      red_m[wave] = m_run;
      red_l[wave] = l_run;
    }
#pragma unroll
    for (int i = 0; i < AG_MAX_D / RB_WAVE; ++i) {
      const int d = lane + i * RB_WAVE;
      if (d < head_dim) red_acc[wave][d] = acc[i];
    }
    __syncthreads();
    if (wave != 0) return;
    float mx = red_m[0];
    for (int w = 1; w < n_waves; ++w) mx = fmaxf(mx, red_m[w]);
    l_run = 0.f;
#pragma unroll
    for (int i = 0; i < AG_MAX_D / RB_WAVE; ++i) acc[i] = 0.f;
    for (int w = 0; w < n_waves; ++w) {
      const float f = (red_m[w] == -INFINITY) ? 0.f : expf(red_m[w] - mx);
      l_run += red_l[w] * f;
#pragma unroll
      for (int i = 0; i < AG_MAX_D / RB_WAVE; ++i) {
        const int d = lane + i * RB_WAVE;
        if (d < head_dim) acc[i] += red_acc[w][d] * f;
      }
    }
  }
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  T* orow = out + ((size_t)t * n_heads + h) * head_dim;
#pragma unroll
  for (int i = 0; i < AG_MAX_D / RB_WAVE; ++i) {
    const int d = lane + i * RB_WAVE;
    if (d < head_dim) Num<T>::store(orow + d, acc[i] * inv);
  }
}

// The same for head sizes that are multiples of 4 (every size a real model has), with 16-byte loads
// (8-byte ones of bfloat16).  Scores: lane j takes key j of the page and walks its row four values at a
// time.  Weighted sum: the lanes are dealt in groups of G = the next power of two >= D / 4; group g takes
// the keys j = g, g + 64 / G, ... and lane c of a group the values 4 c .. 4 c + 3 of each, so that a
// group's load is one row of V in a piece; the groups' sums meet by shuffles once, after the last page.
// The scalar kernel above took 125 us for a decode step of 8 sequences at 530 keys of the 8B shape
// in float32 (every load instruction of its score loop touched 64 cache lines for 4 bytes each).
template <typename T>
struct Vec4;
template <>
struct Vec4<float> {
  static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
};
template <>
struct Vec4<bf16_t> {
  static __device__ __forceinline__ float4 load(const bf16_t* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return make_float4(bf16_bits_to_f32(v.x & 0xffffu), bf16_bits_to_f32(v.x >> 16), bf16_bits_to_f32(v.y & 0xffffu),
                       bf16_bits_to_f32(v.y >> 16));
  }
};

template <typename T>
__global__ __launch_bounds__(RB_WAVE * AG_MAX_WAVES) void attention_generic_vec_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages, T* __restrict__ out,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
    const int32_t* __restrict__ block_table, int bt_stride, int n_heads, int n_kv, int head_dim, float scale,
    int window, int group_lanes) {
  __shared__ __attribute__((aligned(16))) float qs[AG_MAX_D];
  __shared__ float ps_all[AG_MAX_WAVES][RB_PAGE];
  __shared__ float red_m[AG_MAX_WAVES], red_l[AG_MAX_WAVES];
  __shared__ __attribute__((aligned(16))) float red_acc[AG_MAX_WAVES][AG_MAX_D];
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x & (RB_WAVE - 1);
  const int wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  float* ps = ps_all[wave];
  const int pos = tok_pos[t];
  const int kvh = h / (n_heads / n_kv);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* pages = block_table + (size_t)tok_seq[t] * bt_stride;
  const int chunks = head_dim / 4;
  const int c = lane % group_lanes, g = lane / group_lanes, n_groups = RB_WAVE / group_lanes;
  const bool c_on = c < chunks;

  const T* qrow = q + ((size_t)t * n_heads + h) * head_dim;
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) qs[d] = Num<T>::load(qrow + d);
  __syncthreads();

  float m_run = -INFINITY, l_run = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int pg = lo / RB_PAGE + wave; pg <= pos / RB_PAGE; pg += n_waves) {
    const size_t base = ((size_t)pages[pg] * n_kv + kvh) * RB_PAGE * head_dim;
    const int p = pg * RB_PAGE + lane;
    float s = -INFINITY;
    if (p >= lo && p <= pos) {
      const T* krow = k_pages + base + (size_t)lane * head_dim;
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
      for (int cc = 0; cc < chunks; ++cc) {
        const float4 kv = Vec4<T>::load(krow + 4 * cc);
        const float4 qv = *reinterpret_cast<const float4*>(qs + 4 * cc);
        d0 = fmaf(qv.x, kv.x, d0);
        d1 = fmaf(qv.y, kv.y, d1);
        d2 = fmaf(qv.z, kv.z, d2);
        d3 = fmaf(qv.w, kv.w, d3);
      }
      s = ((d0 + d1) + (d2 + d3)) * scale;
    }
    const float m_new = fmaxf(m_run, wave_max(s));      // finite: the page holds at least one valid key
    const float pexp = (s == -INFINITY) ? 0.f : expf(s - m_new);
    const float corr = (m_run == -INFINITY) ? 0.f : expf(m_run - m_new);
    l_run = l_run * corr + wave_sum(pexp);
    m_run = m_new;
    ps[lane] = pexp;                                    // this wave's alone; a wave's LDS accesses complete in order
    __builtin_amdgcn_wave_barrier();
    const int j_lo = (pg * RB_PAGE < lo) ? lo - pg * RB_PAGE : 0;
    const int j_hi = (pg * RB_PAGE + RB_PAGE - 1 > pos) ? pos - pg * RB_PAGE : RB_PAGE - 1;
    acc.x *= corr;
    acc.y *= corr;
    acc.z *= corr;
    acc.w *= corr;
    if (c_on) {
      const T* vcol = v_pages + base + 4 * c;
      for (int j = j_lo + g; j <= j_hi; j += n_groups) {
        const float4 vv = Vec4<T>::load(vcol + (size_t)j * head_dim);
        const float w = ps[j];
        acc.x = fmaf(w, vv.x, acc.x);
        acc.y = fmaf(w, vv.y, acc.y);
        acc.z = fmaf(w, vv.z, acc.z);
        acc.w = fmaf(w, vv.w, acc.w);
      }
    }
  }
  // the groups' sums meet in group 0
  for (int o = group_lanes; o < RB_WAVE; o <<= 1) {
    acc.x += __shfl_xor(acc.x, o, RB_WAVE);
    acc.y += __shfl_xor(acc.y, o, RB_WAVE);
    acc.z += __shfl_xor(acc.z, o, RB_WAVE);
    acc.w += __shfl_xor(acc.w, o, RB_WAVE);
  }
  const bool owner = g == 0 && c_on;
  // ---- the waves' states into one (a wave without pages holds m = -inf, l = 0, acc = 0)
  if (n_waves > 1) {
    if (lane == 0) {
      red_m[wave] = m_run;
      red_l[wave] = l_run;
    }
    if (owner) *reinterpret_cast<float4*>(&red_acc[wave][4 * c]) = acc;
    __syncthreads();
    if (wave != 0) return;
    float mx = red_m[0];
    for (int w = 1; w < n_waves; ++w) mx = fmaxf(mx, red_m[w]);
    l_run = 0.f;
    acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int w = 0; w < n_waves; ++w) {
      const float f = (red_m[w] == -INFINITY) ? 0.f : expf(red_m[w] - mx);
      l_run += red_l[w] * f;
      if (owner) {
        const float4 a = *reinterpret_cast<const float4*>(&red_acc[w][4 * c]);
        acc.x += a.x * f;
        acc.y += a.y * f;
        acc.z += a.z * f;
        acc.w += a.w * f;
      }
    }
  }
  if (owner) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    T* orow = out + ((size_t)t * n_heads + h) * head_dim + 4 * c;
    Num<T>::store(orow + 0, acc.x * inv);
    Num<T>::store(orow + 1, acc.y * inv);
    Num<T>::store(orow + 2, acc.z * inv);
    Num<T>::store(orow + 3, acc.w * inv);
  }
}

static int g_attention_vec = 1;
extern "C" void rb_tune_attention_vec(int on) { g_attention_vec = on; }      // experiments and tests: 0 = the scalar kernel for every head size

extern "C" int rb_attention_generic(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                                    const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                                    int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                    float scale, int window, void* stream) {
  RB_RECORDED(rb_attention_generic(q, k_pages, v_pages, out, dtype, tok_pos, tok_seq, block_table, bt_stride, n_tokens, n_heads,
                                   n_kv_heads, head_dim, scale, window, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
             "rb_attention_generic: bad head counts Hq=%d Hk=%d", n_heads, n_kv_heads);
  RB_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= AG_MAX_D,
             "rb_attention_generic: head_dim %d not supported (even, at most %d)", head_dim, AG_MAX_D);
  RB_REQUIRE(n_heads <= 65535, "rb_attention_generic: too many heads %d", n_heads);
  RB_REQUIRE(window >= 0, "rb_attention_generic: negative window");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(n_tokens, n_heads);
  // waves per (token, head): enough to give every SIMD of the GPU two waves, at most 8
  int n_waves = 1;
  while (n_waves < AG_MAX_WAVES && (long long)n_tokens * n_heads * n_waves < 8LL * rb_compute_units()) n_waves *= 2;
  const int threads = RB_WAVE * n_waves;
  if (head_dim % 4 == 0 && g_attention_vec) {
    int group_lanes = 1;
    while (group_lanes < head_dim / 4) group_lanes *= 2;
    RB_REQUIRE(dtype == RB_F32 || dtype == RB_BF16, "rb_attention_generic: unknown dtype %d", dtype);
    if (dtype == RB_F32)
      attention_generic_vec_kernel<float><<<grid, threads, 0, s>>>((const float*)q, (const float*)k_pages,
                                                                  (const float*)v_pages, (float*)out, tok_pos, tok_seq,
                                                                  block_table, bt_stride, n_heads, n_kv_heads, head_dim,
                                                                  scale, window, group_lanes);
    else
      attention_generic_vec_kernel<bf16_t><<<grid, threads, 0, s>>>((const bf16_t*)q, (const bf16_t*)k_pages,
                                                                   (const bf16_t*)v_pages, (bf16_t*)out, tok_pos,
                                                                   tok_seq, block_table, bt_stride, n_heads, n_kv_heads,
                                                                   head_dim, scale, window, group_lanes);
    RB_LAUNCH_CHECK();
    return 0;
  }
  if (dtype == RB_F32)
    attention_generic_kernel<float><<<grid, threads, 0, s>>>((const float*)q, (const float*)k_pages,
                                                            (const float*)v_pages, (float*)out, tok_pos, tok_seq,
                                                            block_table, bt_stride, n_heads, n_kv_heads, head_dim,
                                                            scale, window);
  else if (dtype == RB_BF16)
    attention_generic_kernel<bf16_t><<<grid, threads, 0, s>>>((const bf16_t*)q, (const bf16_t*)k_pages,
                                                             (const bf16_t*)v_pages, (bf16_t*)out, tok_pos,
                                                             tok_seq, block_table, bt_stride, n_heads, n_kv_heads,
                                                             head_dim, scale, window);
  else
    RB_REQUIRE(false, "rb_attention_generic: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}
