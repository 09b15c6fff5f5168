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
  // waves per (token, head): enough to give every SIMD of the GPU a wave, at most 8
  int n_waves = 1;
  while (n_waves < AG_MAX_WAVES && (long long)n_tokens * n_heads * n_waves < 1024) n_waves *= 2;
  const int threads = RB_WAVE * n_waves;
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
