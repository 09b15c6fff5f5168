// Matrix-core (MFMA) operand types and layouts for gfx950, wave of 64 lanes.
//
// v_mfma_f32_16x16x32_bf16: D[16 x 16] += A[16 x 32] * B[32 x 16]
//   A: lane l holds row l % 16, the 8 depth values of group l / 16
//   B: lane l holds column l % 16, the 8 depth values of group l / 16
//   D: lane l holds column l % 16, rows 4 * (l / 16) + i for i = 0..3
// v_mfma_f32_32x32x16_bf16: D[32 x 32] += A[32 x 16] * B[16 x 32]
//   A: lane l holds row l % 32, the 8 depth values of group l / 32
//   B: lane l holds column l % 32, the 8 depth values of group l / 32
//   D: lane l holds column l % 32, rows 8 * (i / 4) + 4 * (l / 32) + i % 4 for i = 0..15
// Which depth values a group holds is free as long as A and B agree, since the product
// sums over them.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

union Frag8 {
  uint4 u;
  bf16x8_t v;
};

__device__ __forceinline__ f32x4_t mfma16(const Frag8& a, const Frag8& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16_t mfma32(const Frag8& a, const Frag8& b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}

__device__ __forceinline__ uint4 load16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
// 16 bytes that are read once and by nobody else (a weight on its way through a decode step):
// a non-temporal load, which leaves the caches to what is used again.  A plain streaming read of
// 1 GB reaches 5.3-5.6 TB/s on this GPU, a non-temporal one 5.7-6.1, and 7.0-7.1 when every
// workgroup walks memory of its own instead of striding with the others.
typedef unsigned int rb_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load16_stream(const void* p) {
  const rb_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const rb_u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 zero16() { return make_uint4(0u, 0u, 0u, 0u); }

// silu(v) = v / (1 + exp(-v)) (llama/model.rs:297-302) for the epilogues of the bfloat16 products,
// with the hardware's exp2 and reciprocal (each within 1 ulp of float32, where the output keeps 8
// bits): expf and a division took 30 us of the vector units for every 320 x 256 tile of a gated
// product, a fifth of its time.  The 32-bit path does not come through here.
__device__ __forceinline__ float silu_f32(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * v));
}

// ---- memory -> LDS without registers (global_load_lds_dwordx4): the 64 lanes of a wave fetch
// 16 bytes each from base + their byte offset, and the 1 KB lands at the given LDS address in
// lane order.  The instruction is inline assembly, so the compiler neither counts nor waits
// for it: wait with wait_vm<N>() (at most N vector memory operations of this wave still
// outstanding; they complete in issue order) before the data is read from LDS.
template <int N>
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// the same for data that is read once and by nobody else: past the caches
__device__ __forceinline__ void load_to_lds16_stream(const bf16_t* base, uint32_t byte_offset,
                                                     uint32_t lds_byte_address) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2 nt"
      :
      : "s"(lds_byte_address), "v"(byte_offset), "s"(base)
      : "memory");
}

__device__ __forceinline__ void load_to_lds16(const bf16_t* base, uint32_t byte_offset, uint32_t lds_byte_address) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_byte_address), "v"(byte_offset), "s"(base)
      : "memory");
}
