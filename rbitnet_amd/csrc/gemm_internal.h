// Launchers of the bfloat16 matrix-core products, one per source file; rb_gemm_bf16 picks
// among them.  Each returns 0, or an error code with the message stored.
#pragma once
#include <hip/hip_runtime.h>

#include "mfma.h"

// The token operand of a product: bfloat16 rows of K values; row i of the product is row
// rows[i] of x (row i without rows).  With squares ([*, ceil(K / 16)], rows as in x) the rows are
// a float32 row times a norm's gain and squares holds that float32 row's sums of squares, one
// for every 16 columns: the product is multiplied by 1 / sqrt(their sum / K + eps), which makes
// it the product of the RMS-normalised row.
struct GemmTokens {
  const bf16_t* x;
  const float* squares;
  float eps;
  const int32_t* rows;
};

// What becomes of the sums.  epilogue 0: C = sums; 1: the gated pair; 2: C (float32) += sums;
// 3: as 2, and for the norm that follows gained [M, N] = bf16(C * gain) and
// squares [M, ceil(N / 16)] = the sums of C^2 over every 16 columns.
//
// w_frag says how W [N, K] is stored.  false: rows of K values.  true: fragment-major, for K % 64
// == 0 and N % 16 == 0: blocks of 16 rows x 32 depth values, 1 KB each, in the order [N / 16][K / 32];
// inside a block the 16 bytes of lane l of an MFMA's row operand (row l % 16, depth values
// 8 (l / 16) .. + 7) lie at 16 l.  A wave's load instruction then reads 1 KB in a row, and a
// product of few tokens reads W once with non-temporal loads: 6.0-6.8 TB/s instead of 5.3-5.8.
struct GemmAfter {
  int epilogue;
  const float* gain;
  bf16_t* gained;
  float* squares;
  bool w_frag;
};

// at most 64 tokens, any K % 8 == 0: W streamed straight into MFMA operands (gemm_skinny.hip);
// prepared tokens and epilogues 2 and 3: at most 16 tokens
int gemm_skinny_launch(const GemmTokens& x, const bf16_t* w, void* c, int dtype_out, const GemmAfter& after, int m,
                       int n, int k, hipStream_t s);
// at most 16 tokens kept in registers while a workgroup walks several row tiles; false: these
// sizes are not for it and nothing was launched
bool gemm_resident_try(const GemmTokens& x, const bf16_t* w, void* c, int dtype_out, const GemmAfter& after, int m,
                       int n, int k, hipStream_t s, int* rc);
// more than 16 tokens (more than 64 when K is no multiple of 64): tiles through LDS
// (gemm_tiled.hip).  gemm_tiled_parts: 0 when these sizes are not for it, else the number of K
// slices it will use; more than 1 needs parts * m * n floats of workspace.
int gemm_tiled_parts(int m, int n, int k, int epilogue);
int gemm_tiled_launch(const bf16_t* x, const bf16_t* w, bool w_frag, void* c, float* workspace, int dtype_out,
                      int epilogue, int m, int n, int k, hipStream_t s);
