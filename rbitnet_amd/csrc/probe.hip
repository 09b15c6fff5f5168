// What this GPU reaches on the two things the model's kernels are bound by, measured the
// simplest way, so that a kernel's time can be read against more than the nominal peaks:
//  * rb_probe_read: every byte of a buffer once, 16 bytes per lane and load.  Mode 0: all
//    workgroups stride through the buffer together, plain loads (5.3-5.6 TB/s for 1 GB).  Mode 1:
//    every workgroup walks pieces of 64 KB of its own with non-temporal loads (7.0-7.1 TB/s): how
//    the decode products read their weights.
//  * rb_probe_mfma: back-to-back 32x32x16 bfloat16 MFMAs on four independent accumulators
//    per wave, operands in registers, nothing else.
// Neither has a counterpart in the reference (which measures nothing on a GPU).
#include "api.h"
#include "mfma.h"

__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ p, size_t n16, float* sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  uint32_t acc = 0;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  // four loads in flight per lane
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = p[i], b = p[i + stride], c = p[i + 2 * stride], d = p[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n16; i += stride) {
    const uint4 a = p[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) *sink = 1.f;      // keeps the loads alive; practically never true
}

__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* sink) {
  Frag8 a, b;
  a.u = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);      // bfloat16 ones
  b.u = make_uint4(threadIdx.x, 0u, 0u, 0u);
  f32x16_t c0, c1, c2, c3;
#pragma unroll
  for (int e = 0; e < 16; ++e) c0[e] = c1[e] = c2[e] = c3[e] = 0.f;
  for (int i = 0; i < iters; ++i) {
    c0 = mfma32(a, b, c0);
    c1 = mfma32(a, b, c1);
    c2 = mfma32(a, b, c2);
    c3 = mfma32(a, b, c3);
  }
  const float v = c0[0] + c1[1] + c2[2] + c3[3];
  if (v == 12345.678f) *sink = v;
}

// pieces of 64 KB dealt round robin to the workgroups; a piece is walked by the workgroup's 256
// lanes, four non-temporal loads in flight per lane
__global__ __launch_bounds__(256) void probe_read_pieces_kernel(const uint4* __restrict__ p, size_t n16, float* sink) {
  constexpr size_t PIECE = 65536 / 16;
  uint32_t acc = 0;
  const size_t n_pieces = n16 / PIECE;
  for (size_t c = blockIdx.x; c < n_pieces; c += gridDim.x) {
    const uint4* q = p + c * PIECE;
    for (size_t i = threadIdx.x; i < PIECE; i += 4 * 256) {
      const uint4 a = load16_stream(q + i), b = load16_stream(q + i + 256), e = load16_stream(q + i + 512),
                  d = load16_stream(q + i + 768);
      acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ e.x ^ e.y ^ e.z ^ e.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
  }
  for (size_t i = n_pieces * PIECE + (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) {
    const uint4 a = p[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) *sink = 1.f;
}

// Reads `bytes` bytes (a multiple of 16) starting at p with `blocks` workgroups of 256 lanes.
extern "C" int rb_probe_read(const void* p, long long bytes, int blocks, int mode, float* sink, void* stream) {
  RB_REQUIRE(p != nullptr && sink != nullptr && bytes > 0 && bytes % 16 == 0 && blocks > 0 && blocks <= 65536 &&
                 (mode == 0 || mode == 1),
             "rb_probe_read: bad arguments");
  if (mode == 1)
    probe_read_pieces_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const uint4*)p, (size_t)(bytes / 16), sink);
  else
    probe_read_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const uint4*)p, (size_t)(bytes / 16), sink);
  RB_LAUNCH_CHECK();
  return 0;
}

// Runs 4 * iters MFMAs in each of `waves` waves (a multiple of 4); that is
// waves * iters * 4 * 2 * 32 * 32 * 16 floating-point operations.
extern "C" int rb_probe_mfma(int waves, int iters, float* sink, void* stream) {
  RB_REQUIRE(waves > 0 && waves % 4 == 0 && iters > 0 && sink != nullptr, "rb_probe_mfma: bad arguments");
  probe_mfma_kernel<<<waves / 4, 256, 0, (hipStream_t)stream>>>(iters, sink);
  RB_LAUNCH_CHECK();
  return 0;
}
