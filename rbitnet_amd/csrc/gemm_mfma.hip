// C[M, N] = A[M, K] * W[N, K]^T for bfloat16 operands on the gfx950 matrix cores, float32
// accumulation: picks the kernel for the sizes.
//  * at most 16 tokens: W streamed straight into MFMA operands (gemm_skinny.hip); with more
//    than 8192 rows of W the variant that keeps the tokens in registers.
//  * more: tiles of W and of the tokens through LDS, with K cut into slices over workgroups
//    where the tiles alone are too few to fill the GPU (gemm_tiled.hip); 17..64 tokens with a
//    K that is no multiple of 64: the skinny kernel.
#include "api.h"
#include "tune.h"
#include "gemm_internal.h"

static int g_use_resident = 1, g_use_tiled_small = 1;
void gemm_resident_forced(int on);
extern "C" void rb_tune_use_resident(int on) {      // experiments only
  g_use_resident = on;
  gemm_resident_forced(on == 2);
}
extern "C" void rb_tune_use_stream(int on) { g_use_tiled_small = on; }     // experiments only: 0 = skinny up to 64 tokens

static int tiled_parts(int m, int n, int k, int epilogue) {
  if (m <= 64 && !g_use_tiled_small) return 0;
  return gemm_tiled_parts(m, n, k, epilogue);
}

extern "C" long long rb_gemm_workspace_floats(int m, int n, int k, int epilogue) {
  const int p = tiled_parts(m, n, k, epilogue);
  return p > 1 ? (long long)p * m * n : 0;
}

// products that no tiled kernel takes: the two kernels of gemm_skinny.hip
static int launch_few_tokens(const GemmTokens& x, const bf16_t* w, void* c, int dtype_out, const GemmAfter& after,
                             int m, int n, int k, hipStream_t s) {
  int rc = 0;
  if (g_use_resident && m <= 16 && (n > 8192 || g_use_resident == 2) &&
      gemm_resident_try(x, w, c, dtype_out, after, m, n, k, s, &rc))
    return rc;
  return gemm_skinny_launch(x, w, c, dtype_out, after, m, n, k, s);
}

// fragment-major W (w_layout 1) is for K % 64 == 0 and N % 16 == 0
static bool layout_ok(int w_layout, int n, int k) {
  return w_layout == 0 || (w_layout == 1 && k % 64 == 0 && n % 16 == 0);
}

extern "C" int rb_gemm_bf16(const void* a, const void* w, int w_layout, void* c, int dtype_out, int epilogue, int m,
                            int n, int k, float* workspace, void* stream) {
  RB_RECORDED(rb_gemm_bf16(a, w, w_layout, c, dtype_out, epilogue, m, n, k, workspace, stream));
  RB_REQUIRE(m >= 0 && n > 0 && k > 0, "rb_gemm_bf16: bad sizes M=%d N=%d K=%d", m, n, k);
  RB_REQUIRE(layout_ok(w_layout, n, k), "rb_gemm_bf16: W layout %d with N=%d K=%d (fragment-major needs N %% 16 == 0, K %% 64 == 0)",
             w_layout, n, k);
  RB_REQUIRE(k % 8 == 0, "rb_gemm_bf16: K=%d must be a multiple of 8 (use rb_gemm_generic)", k);
  RB_REQUIRE(epilogue == 0 || epilogue == 1, "rb_gemm_bf16: unknown epilogue %d", epilogue);
  RB_REQUIRE(epilogue == 0 || n % 32 == 0, "rb_gemm_bf16: gated epilogue needs N=%d to be a multiple of 32", n);
  RB_REQUIRE(dtype_out == RB_F32 || dtype_out == RB_BF16, "rb_gemm_bf16: unknown output dtype %d", dtype_out);
  if (m == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* xa = (const bf16_t*)a;
  const bf16_t* wa = (const bf16_t*)w;
  int rc = 0;
  if (tiled_parts(m, n, k, epilogue) >= 1) {
    rc = gemm_tiled_launch(xa, wa, w_layout == 1, c, workspace, dtype_out, epilogue, m, n, k, s);
  } else {
    const GemmTokens x = {xa, nullptr, 0.f, nullptr};
    const GemmAfter after = {epilogue, nullptr, nullptr, nullptr, w_layout == 1};
    rc = launch_few_tokens(x, wa, c, dtype_out, after, m, n, k, s);
  }
  if (rc) return rc;
  RB_LAUNCH_CHECK();
  return 0;
}

// The product as the terms its K slices computed, [terms, M, N] float32, for a caller that adds
// them up with something else (rb_add_rmsnorm does).  One term: the product itself.
extern "C" int rb_gemm_bf16_terms_count(int m, int n, int k) {
  const int p = (m > 0 && n > 0 && k > 0 && k % 8 == 0) ? tiled_parts(m, n, k, 0) : 0;
  return p > 1 ? p : 1;
}

extern "C" int rb_gemm_bf16_terms(const void* a, const void* w, int w_layout, float* terms, int m, int n, int k,
                                  void* stream) {
  RB_RECORDED(rb_gemm_bf16_terms(a, w, w_layout, terms, m, n, k, stream));
  const int p = rb_gemm_bf16_terms_count(m, n, k);
  if (p == 1) return rb_gemm_bf16(a, w, w_layout, terms, RB_F32, 0, m, n, k, nullptr, stream);
  RB_REQUIRE(layout_ok(w_layout, n, k), "rb_gemm_bf16_terms: W layout %d with N=%d K=%d", w_layout, n, k);
  const int rc = gemm_tiled_launch((const bf16_t*)a, (const bf16_t*)w, w_layout == 1, nullptr, terms, RB_F32, 0, m, n, k,
                                   (hipStream_t)stream);
  if (rc) return rc;
  RB_LAUNCH_CHECK();
  return 0;
}

extern "C" int rb_gemm_bf16_few_ok(int m, int n, int k) {
  return m >= 1 && m <= 16 && n > 0 && k > 0 && k % 8 == 0 && tiled_parts(m, n, k, 0) == 0;
}

extern "C" int rb_gemm_bf16_few(const void* a, const float* squares_in, float eps, const int32_t* rows, const void* w,
                                int w_layout, void* c, int dtype_out, int epilogue, const float* gain, void* gained,
                                float* squares_out, int m, int n, int k, void* stream) {
  RB_RECORDED(rb_gemm_bf16_few(a, squares_in, eps, rows, w, w_layout, c, dtype_out, epilogue, gain, gained, squares_out, m, n, k,
                               stream));
  RB_REQUIRE(layout_ok(w_layout, n, k), "rb_gemm_bf16_few: W layout %d with N=%d K=%d", w_layout, n, k);
  RB_REQUIRE(rb_gemm_bf16_few_ok(m, n, k), "rb_gemm_bf16_few: M=%d N=%d K=%d is not for it (1..16 tokens, K %% 8 == 0)",
             m, n, k);
  RB_REQUIRE(epilogue >= 0 && epilogue <= 3, "rb_gemm_bf16_few: unknown epilogue %d", epilogue);
  RB_REQUIRE(epilogue != 1 || n % 32 == 0, "rb_gemm_bf16_few: gated epilogue needs N=%d to be a multiple of 32", n);
  RB_REQUIRE(dtype_out == RB_F32 || (dtype_out == RB_BF16 && epilogue <= 1),
             "rb_gemm_bf16_few: output dtype %d with epilogue %d", dtype_out, epilogue);
  RB_REQUIRE(!squares_in || epilogue <= 1, "rb_gemm_bf16_few: prepared rows go with epilogues 0 and 1, not %d", epilogue);
  RB_REQUIRE(epilogue != 3 || (gain && gained && squares_out),
             "rb_gemm_bf16_few: epilogue 3 needs the gain and room for the prepared rows");
  const GemmTokens x = {(const bf16_t*)a, squares_in, eps, rows};
  const GemmAfter after = {epilogue, gain, (bf16_t*)gained, squares_out, w_layout == 1};
  const int rc = launch_few_tokens(x, (const bf16_t*)w, c, dtype_out, after, m, n, k, (hipStream_t)stream);
  if (rc) return rc;
  RB_LAUNCH_CHECK();
  return 0;
}
