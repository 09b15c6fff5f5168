// Shared device helpers for the gfx950 kernels: storage types, wave and block
// reductions, error reporting of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <functional>

#define RB_WAVE 64
#define RB_PAGE 64            // tokens per cache page; attention tiles are one page of keys

// ---------------------------------------------------------------- error reporting
// Every entry point returns 0, or a non-zero code after rb_set_error(); the text is
// read back with rb_last_error().  No entry point throws or aborts.
void rb_set_error(const char* fmt, ...);
#define RB_REQUIRE(cond, ...)                       \
  do {                                              \
    if (!(cond)) {                                  \
      rb_set_error(__VA_ARGS__);                    \
      return 1;                                     \
    }                                               \
  } while (0)
#define RB_LAUNCH_CHECK()                                                   \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      rb_set_error("%s: launch failed: %s", __func__, hipGetErrorString(e_)); \
      return 2;                                                             \
    }                                                                       \
  } while (0)

enum RbDtype { RB_F32 = 0, RB_BF16 = 1 };

// ---------------------------------------------------------------- the machine
// Compute units of the current device (asked of the runtime once per device): what one round
// of workgroups is.  Every choice of a tile, a number of K slices or of splits that depends on
// how a grid fills the GPU is an expression of this number, not of the 256 of an MI355X.
int rb_compute_units(void);

// ---------------------------------------------------------------- recorded steps (plan.hip)
// While a plan records on the calling thread, every entry point that launches kernels notes its
// own call (a closure over its arguments that takes the stream to launch on) before it does its
// work, so that the same launches can be issued again from C++ without the caller's host code
// between them.  RB_RECORDED(call) stands first in such an entry point, `call` being the entry
// point's own call with its own parameter names, `stream` among them.  An entry point that
// calls another one is recorded once, as itself.
bool rb_plan_wants_call(void);
void rb_plan_note(std::function<int(void*)> call);
struct RbPlanScope {
  RbPlanScope();
  ~RbPlanScope();
};
#define RB_RECORDED(call)  \
  RbPlanScope rb_plan_scope_; \
  if (rb_plan_wants_call()) rb_plan_note([=](void* stream) -> int { return call; })

// ---------------------------------------------------------------- bfloat16 storage
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round to nearest even, NaN stays NaN: the hardware's conversion (v_cvt_pk_bf16_f32)
typedef __attribute__((ext_vector_type(2))) __bf16 rb_bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float rb_f32x2_t;
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  union {
    __bf16 b;
    uint16_t u;
  } r;
  r.b = (__bf16)f;
  return r.u;
}
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(f);
  return r;
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  union {
    rb_bf16x2_t v;
    uint32_t u;
  } r;
  const rb_f32x2_t f = {lo, hi};
  r.v = __builtin_convertvector(f, rb_bf16x2_t);
  return r.u;
}

template <typename T>
struct Num;
template <>
struct Num<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <>
struct Num<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};

// ---------------------------------------------------------------- rotation of a pair
// (x0, x1) turned by the angle whose cosine and sine are c and s (llama/model.rs:122-136). The
// operations are spelled out so that every kernel that rotates rounds the same way, whatever
// the compiler would have contracted: the same q, k and logits whichever kernel rotated them.
__device__ __forceinline__ void rotate_pair(float x0, float x1, float c, float s, float& y0, float& y1) {
  y0 = __fmaf_rn(x0, c, -__fmul_rn(x1, s));
  y1 = __fmaf_rn(x0, s, __fmul_rn(x1, c));
}

// ---------------------------------------------------------------- terms of a product
// A product whose K was cut into slices may be left as its slices' sums, `stride` floats
// apart: p[0] + p[stride] + ... in that order (the order in which the product's own kernel
// adds them), four loads in flight.
__device__ __forceinline__ float sum_terms(const float* __restrict__ p, int n_terms, size_t stride) {
  float v = p[0];
  int t = 1;
  for (; t + 3 < n_terms; t += 4) {
    const float e0 = p[(size_t)t * stride], e1 = p[(size_t)(t + 1) * stride], e2 = p[(size_t)(t + 2) * stride],
                e3 = p[(size_t)(t + 3) * stride];
    v += e0;
    v += e1;
    v += e2;
    v += e3;
  }
  for (; t < n_terms; ++t) v += p[(size_t)t * stride];
  return v;
}

// ---------------------------------------------------------------- reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = RB_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, RB_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = RB_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, RB_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds at least 16 floats.
// Every thread gets the total.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (RB_WAVE - 1);
  const int wave = threadIdx.x / RB_WAVE;
  const int n_waves = (blockDim.x + RB_WAVE - 1) / RB_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < n_waves; ++i) t += scratch[i];
  return t;
}
