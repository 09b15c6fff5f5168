// Next-token choice on the device, one block per sequence.
//
// Reference (llama/runtime.rs:81-107): temperature <= 0 -> the index of the greatest logit
// with NaN counted as -inf; otherwise z = logit / T, e = exp(z - max z), r = u * sum(e) and
// the first index whose running sum (in index order) reaches r, the last index if none does.
// Among equal maxima this kernel takes the lowest index.
#include <math.h>

#include "api.h"
#include "common.h"

#define SAMPLE_THREADS 1024

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ u,
                                                                int32_t* __restrict__ tokens) {
  __shared__ float s_val[SAMPLE_THREADS / RB_WAVE];
  __shared__ int s_idx[SAMPLE_THREADS / RB_WAVE];
  __shared__ double s_part[SAMPLE_THREADS];
  __shared__ float s_max;
  __shared__ int s_arg;
  __shared__ int s_choice;
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & (RB_WAVE - 1);
  const int wave = tid / RB_WAVE;
  const float* row = logits + (size_t)r * vocab;

  // ---- maximum and its lowest index
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
    float v = row[i];
    if (v != v) v = -INFINITY;
    if (v > best || (v == best && i < best_i)) {
      best = v;
      best_i = i;
    }
  }
#pragma unroll
  for (int o = RB_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, RB_WAVE);
    const int oi = __shfl_xor(best_i, o, RB_WAVE);
    if (ov > best || (ov == best && oi < best_i)) {
      best = ov;
      best_i = oi;
    }
  }
  if (lane == 0) {
    s_val[wave] = best;
    s_idx[wave] = best_i;
  }
  __syncthreads();
  if (tid == 0) {
    float b = s_val[0];
    int bi = s_idx[0];
    for (int w = 1; w < SAMPLE_THREADS / RB_WAVE; ++w)
      if (s_val[w] > b || (s_val[w] == b && s_idx[w] < bi)) {
        b = s_val[w];
        bi = s_idx[w];
      }
    s_max = b;
    s_arg = bi == 0x7fffffff ? 0 : bi;      // every logit NaN or -inf: index 0
    s_choice = -1;
  }
  __syncthreads();
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) tokens[r] = s_arg;
    return;
  }

  // ---- inverse CDF in index order: each thread owns one contiguous segment
  const float zmax = s_max / temp;
  const int seg = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int i0 = tid * seg;
  const int i1 = i0 + seg < vocab ? i0 + seg : vocab;
  double part = 0.0;
  for (int i = i0; i < i1; ++i) {
    float v = row[i];
    if (v != v) v = -INFINITY;
    part += (double)expf(v / temp - zmax);
  }
  s_part[tid] = part;
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int w = 0; w < SAMPLE_THREADS; ++w) total += s_part[w];
    const double target = (double)u[r] * total;
    double c = 0.0;
    int owner = -1;
    for (int w = 0; w < SAMPLE_THREADS; ++w) {
      if (c + s_part[w] >= target && w * seg < vocab) {
        owner = w;
        break;
      }
      c += s_part[w];
    }
    if (owner < 0) {
      tokens[r] = vocab - 1;
    } else {
      // walk the owner's segment
      int pick = -1;
      const int j1 = owner * seg + seg < vocab ? owner * seg + seg : vocab;
      for (int i = owner * seg; i < j1; ++i) {
        float v = row[i];
        if (v != v) v = -INFINITY;
        c += (double)expf(v / temp - zmax);
        if (c >= target) {
          pick = i;
          break;
        }
      }
      tokens[r] = pick >= 0 ? pick : j1 - 1;
    }
  }
}

extern "C" int rb_sample(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
                         int32_t* tokens, void* stream) {
  RB_REQUIRE(n_rows >= 0 && vocab > 0, "rb_sample: bad sizes %d x %d", n_rows, vocab);
  RB_REQUIRE(temperature == nullptr || u != nullptr, "rb_sample: temperature given without uniform numbers");
  if (n_rows == 0) return 0;
  sample_kernel<<<n_rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, vocab, temperature, u, tokens);
  RB_LAUNCH_CHECK();
  return 0;
}
