// Next-token choice on the device, in two kernels so that a 128k vocabulary is read by
// many workgroups: (1) per chunk of the vocabulary, the maximum with its lowest index and
// the sum of exponentials relative to it; (2) per sequence, the chunks combined and, for
// temperature sampling, the chunk that holds the target walked element by element.
//
// Reference (llama/runtime.rs:81-107): temperature <= 0 -> the index of the greatest logit
// with NaN counted as -inf; otherwise z = logit / T, e = exp(z - max z), r = u * sum(e) and
// the first index whose running sum (in index order) reaches r, the last index if none does.
// Among equal maxima the lowest index is taken.  Sums are kept in double, so that the order
// of summation (chunks, segments) cannot move the chosen index.
#include <math.h>

#include <mutex>

#include "api.h"
#include "common.h"

#define SAMPLE_CHUNK 4096
#define SAMPLE_THREADS 256
#define SAMPLE_SEG (SAMPLE_CHUNK / SAMPLE_THREADS)
#define SAMPLE_MAX_CHUNKS 1024

struct ChunkStat {
  float max;
  int arg;
  double sum;       // sum over the chunk of exp(z / T - max / T); 0 for greedy rows
};

__device__ __forceinline__ float clean(float v) { return v != v ? -INFINITY : v; }

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_chunk_kernel(const float* __restrict__ logits, int vocab,
                                                                      const float* __restrict__ temperature,
                                                                      ChunkStat* __restrict__ stats, int n_chunks) {
  __shared__ float s_val[SAMPLE_THREADS / RB_WAVE];
  __shared__ int s_idx[SAMPLE_THREADS / RB_WAVE];
  __shared__ double s_sum[SAMPLE_THREADS / RB_WAVE];
  __shared__ float s_max;
  const int c = blockIdx.x, r = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & (RB_WAVE - 1), wave = tid / RB_WAVE;
  const float* row = logits + (size_t)r * vocab;
  const int i0 = c * SAMPLE_CHUNK;
  const int i1 = i0 + SAMPLE_CHUNK < vocab ? i0 + SAMPLE_CHUNK : vocab;
  float v[SAMPLE_SEG];
  float best = -INFINITY;
  int best_i = 0x7fffffff;
#pragma unroll
  for (int k = 0; k < SAMPLE_SEG; ++k) {          // strided: coalesced loads
    const int i = i0 + tid + k * SAMPLE_THREADS;
    v[k] = i < i1 ? clean(row[i]) : -INFINITY;
    if (i < i1 && (v[k] > best || (v[k] == best && i < best_i))) {
      best = v[k];
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
    stats[(size_t)r * n_chunks + c].max = b;
    stats[(size_t)r * n_chunks + c].arg = bi;
  }
  __syncthreads();
  const float temp = temperature ? temperature[r] : 0.f;
  double sum = 0.0;
  if (temp > 0.f && s_max > -INFINITY) {
    const float zmax = s_max / temp;
#pragma unroll
    for (int k = 0; k < SAMPLE_SEG; ++k) sum += (double)expf(v[k] / temp - zmax);      // exp(-inf) = 0 beyond the end
#pragma unroll
    for (int o = RB_WAVE / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o, RB_WAVE);
  }
  if (lane == 0) s_sum[wave] = sum;
  __syncthreads();
  if (tid == 0) {
    double t = 0.0;
    for (int w = 0; w < SAMPLE_THREADS / RB_WAVE; ++w) t += s_sum[w];
    stats[(size_t)r * n_chunks + c].sum = t;
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_pick_kernel(const float* __restrict__ logits, int vocab,
                                                                     const float* __restrict__ temperature,
                                                                     const float* __restrict__ u,
                                                                     const ChunkStat* __restrict__ stats, int n_chunks,
                                                                     int32_t* __restrict__ tokens) {
  __shared__ double s_part[SAMPLE_THREADS];
  __shared__ int s_chunk;
  __shared__ double s_before, s_target, s_factor;
  __shared__ float s_gmax;
  const int r = blockIdx.x, tid = threadIdx.x;
  const ChunkStat* st = stats + (size_t)r * n_chunks;
  const float temp = temperature ? temperature[r] : 0.f;
  if (tid == 0) {
    float gmax = -INFINITY;
    int garg = 0x7fffffff;
    for (int c = 0; c < n_chunks; ++c)
      if (st[c].max > gmax || (st[c].max == gmax && st[c].arg < garg)) {
        gmax = st[c].max;
        garg = st[c].arg;
      }
    s_gmax = gmax;
    s_chunk = -1;
    if (!(temp > 0.f) || gmax == -INFINITY) {
      tokens[r] = garg == 0x7fffffff ? 0 : garg;          // every logit NaN or -inf: index 0
    } else {
      double total = 0.0;
      for (int c = 0; c < n_chunks; ++c)
        if (st[c].max > -INFINITY) total += st[c].sum * exp((double)(st[c].max / temp) - (double)(gmax / temp));
      const double target = (double)u[r] * total;
      double run = 0.0;
      int pick = -1;
      for (int c = 0; c < n_chunks; ++c) {
        if (!(st[c].max > -INFINITY)) continue;
        const double f = exp((double)(st[c].max / temp) - (double)(gmax / temp));
        if (run + st[c].sum * f >= target) {
          pick = c;
          s_factor = f;
          break;
        }
        run += st[c].sum * f;
      }
      if (pick < 0) {
        tokens[r] = vocab - 1;
      } else {
        s_chunk = pick;
        s_before = run;
        s_target = target;
      }
    }
  }
  __syncthreads();
  const int c = s_chunk;
  if (c < 0) return;
  // ---- walk the chosen chunk in index order: each thread a contiguous segment
  const float* row = logits + (size_t)r * vocab;
  const float zmax = s_gmax / temp;
  const int i0 = c * SAMPLE_CHUNK + tid * SAMPLE_SEG;
  const int cend = (c + 1) * SAMPLE_CHUNK < vocab ? (c + 1) * SAMPLE_CHUNK : vocab;
  double part = 0.0;
  for (int i = i0; i < i0 + SAMPLE_SEG && i < cend; ++i) part += (double)expf(clean(row[i]) / temp - zmax);
  s_part[tid] = part;
  __syncthreads();
  if (tid == 0) {
    double run = s_before;
    const double target = s_target;
    int owner = -1;
    for (int w = 0; w < SAMPLE_THREADS; ++w) {
      if (c * SAMPLE_CHUNK + w * SAMPLE_SEG >= cend) break;
      if (run + s_part[w] >= target) {
        owner = w;
        break;
      }
      run += s_part[w];
    }
    int pick = cend - 1;            // rounding kept the running sum just below the target
    if (owner >= 0) {
      const int j0 = c * SAMPLE_CHUNK + owner * SAMPLE_SEG;
      const int j1 = j0 + SAMPLE_SEG < cend ? j0 + SAMPLE_SEG : cend;
      pick = j1 - 1;
      for (int i = j0; i < j1; ++i) {
        run += (double)expf(clean(row[i]) / temp - zmax);
        if (run >= target) {
          pick = i;
          break;
        }
      }
    }
    tokens[r] = pick;
  }
}

extern "C" int rb_sample_workspace_bytes(int n_rows, int vocab) {
  const int n_chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  return (int)((size_t)n_rows * n_chunks * sizeof(ChunkStat));
}

extern "C" int rb_sample(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
                         int32_t* tokens, void* workspace, void* stream) {
  RB_RECORDED(rb_sample(logits, n_rows, vocab, temperature, u, tokens, workspace, stream));
  RB_REQUIRE(n_rows >= 0 && vocab > 0, "rb_sample: bad sizes %d x %d", n_rows, vocab);
  RB_REQUIRE(temperature == nullptr || u != nullptr, "rb_sample: temperature given without uniform numbers");
  RB_REQUIRE(workspace != nullptr, "rb_sample: no workspace");
  if (n_rows == 0) return 0;
  const int n_chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  RB_REQUIRE(n_chunks <= SAMPLE_MAX_CHUNKS && n_rows <= 65535, "rb_sample: vocabulary %d or batch %d too large", vocab,
             n_rows);
  hipStream_t s = (hipStream_t)stream;
  ChunkStat* stats = (ChunkStat*)workspace;
  sample_chunk_kernel<<<dim3(n_chunks, n_rows), SAMPLE_THREADS, 0, s>>>(logits, vocab, temperature, stats, n_chunks);
  sample_pick_kernel<<<n_rows, SAMPLE_THREADS, 0, s>>>(logits, vocab, temperature, u, stats, n_chunks, tokens);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- the variant that allocates nothing
// rb_sample_static is rb_sample with the chunk statistics in device memory that the library
// itself holds: a file-scope array, one copy on every GPU the library runs on, kept until the
// process ends.  Nothing in it has to start at zero: the first kernel writes every entry
// [row, chunk] that the second reads.  The array's name is only a host-side handle; the
// address that kernels get is asked for once per device with hipGetSymbolAddress and kept.
#define SAMPLE_STATIC_MAX_STATS 16384      // entries of 16 bytes: 256 KiB per GPU
#define SAMPLE_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[SAMPLE_STATIC_MAX_STATS * sizeof(ChunkStat)];
static void* g_scratch_ptr[SAMPLE_STATIC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  RB_REQUIRE(e == hipSuccess, "rb_sample_static: hipGetDevice failed: %s", hipGetErrorString(e));
  RB_REQUIRE(dev >= 0 && dev < SAMPLE_STATIC_MAX_DEVICES, "rb_sample_static: device %d beyond the %d this library keeps scratch for",
             dev, SAMPLE_STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    RB_REQUIRE(e == hipSuccess && p != nullptr, "rb_sample_static: hipGetSymbolAddress failed on device %d: %s", dev,
               hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// Also the set-up call: it asks for the current device's copy of the scratch array, so that a first
// rb_sample_static under stream capture finds the address known (the runtime may refuse the query
// while a stream captures).
extern "C" int rb_sample_static_max_stats(void) {
  void* ptr = nullptr;
  (void)scratch_of_current_device(&ptr);
  return SAMPLE_STATIC_MAX_STATS;
}

extern "C" int rb_sample_static(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
                                int32_t* tokens, void* stream) {
  RB_REQUIRE(n_rows >= 0 && vocab > 0, "rb_sample_static: bad sizes %d x %d", n_rows, vocab);
  RB_REQUIRE(temperature == nullptr || u != nullptr, "rb_sample_static: temperature given without uniform numbers");
  if (n_rows == 0) return 0;
  const long long n_chunks = ((long long)vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  RB_REQUIRE(n_chunks <= SAMPLE_MAX_CHUNKS && n_rows <= 65535 && (long long)n_rows * n_chunks <= SAMPLE_STATIC_MAX_STATS,
             "rb_sample_static: %d rows of %d logits need %lld chunk entries, the built-in scratch holds %d "
             "(use rb_sample with a workspace)",
             n_rows, vocab, (long long)n_rows * n_chunks, SAMPLE_STATIC_MAX_STATS);
  void* ptr = nullptr;
  if (int rc = scratch_of_current_device(&ptr)) return rc;
  hipStream_t s = (hipStream_t)stream;
  ChunkStat* stats = (ChunkStat*)ptr;
  sample_chunk_kernel<<<dim3((int)n_chunks, n_rows), SAMPLE_THREADS, 0, s>>>(logits, vocab, temperature, stats,
                                                                             (int)n_chunks);
  sample_pick_kernel<<<n_rows, SAMPLE_THREADS, 0, s>>>(logits, vocab, temperature, u, stats, (int)n_chunks, tokens);
  RB_LAUNCH_CHECK();
  return 0;
}
