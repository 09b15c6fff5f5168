// Launchers of the bfloat16 matrix-core products, one per source file; rb_gemm_bf16 picks
// among them.  Each returns 0, or an error code with the message stored.
#pragma once
#include <hip/hip_runtime.h>

#include "mfma.h"

// at most 64 tokens, any K % 8 == 0: W streamed straight into MFMA operands (gemm_skinny.hip)
int gemm_skinny_launch(const bf16_t* x, const bf16_t* w, void* c, int dtype_out, int epilogue, int m, int n, int k,
                       hipStream_t s);
// at most 16 tokens kept in registers while a workgroup walks several row tiles; false: these
// sizes are not for it and nothing was launched
bool gemm_resident_try(const bf16_t* x, const bf16_t* w, void* c, int dtype_out, int epilogue, int m, int n, int k,
                       hipStream_t s, int* rc);
// more than 16 tokens (more than 64 when K is no multiple of 64): tiles through LDS
// (gemm_tiled.hip).  gemm_tiled_parts: 0 when these sizes are not for it, else the number of K
// slices it will use; more than 1 needs parts * m * n floats of workspace.
int gemm_tiled_parts(int m, int n, int k, int epilogue);
int gemm_tiled_launch(const bf16_t* x, const bf16_t* w, void* c, float* workspace, int dtype_out, int epilogue, int m,
                      int n, int k, hipStream_t s);
