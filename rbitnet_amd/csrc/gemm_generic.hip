// C[M, N] = A[M, K] * W[N, K]^T for any sizes, float32 or bfloat16 storage, float32
// multiply-add on the vector units or, for float32 operands with K % 16 == 0, the float32
// MFMA (never a reduced-precision matrix mode).  This is the
// whole float32 path's matrix product and the bfloat16 path's product for shapes the
// matrix-core kernels refuse.
//
// Reference: y[o] = sum_i W[i + o * n_in] * x[i] (llama/model.rs:67-91).
#include "api.h"
#include "common.h"

#define GT 64      // tile of C: GT x GT
#define GK 16      // depth of one stage

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TI* __restrict__ a, const TI* __restrict__ w,
                                                           TO* __restrict__ c, int m, int n, int k) {
  __shared__ float as[GK][GT + 4];
  __shared__ float ws[GK][GT + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT;
  const int n0 = blockIdx.x * GT;
  const int tx = tid % 16;      // 4 columns of C each
  const int ty = tid / 16;      // 4 rows of C each
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // each thread loads 4 elements of the A tile and 4 of the W tile per stage
  const int lr = tid / 4;            // row of the tile, 0..63
  const int lk = (tid % 4) * 4;      // depth offset 0, 4, 8, 12
  for (int k0 = 0; k0 < k; k0 += GK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int kk = k0 + lk + q;
      const int am = m0 + lr;
      const int wn = n0 + lr;
      as[lk + q][lr] = (am < m && kk < k) ? Num<TI>::load(a + (size_t)am * k + kk) : 0.f;
      ws[lk + q][lr] = (wn < n && kk < k) ? Num<TI>::load(w + (size_t)wn * k + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int mm = m0 + ty * 4 + i;
    if (mm >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int nn = n0 + tx * 4 + j;
      if (nn < n) Num<TO>::store(c + (size_t)mm * n + nn, acc[i][j]);
    }
  }
}

// Float32 operands and at most 16 tokens (the float32 path's decode step): bound by reading W
// once.  A wave owns 4 rows of W and walks all of K with 16-byte loads (a row is read as
// 1 KB contiguous per instruction); the tokens' 1024-deep chunk goes through LDS once for
// the 4 waves; every lane keeps a partial sum per (row, token) and the wave adds them up at
// the end.  K must be a multiple of 4.
#define GS_ROWS 4
#define GS_KC 1024

template <int MT>
__global__ __launch_bounds__(256) void gemm_f32_skinny_kernel(const float* __restrict__ a, const float* __restrict__ w,
                                                              float* __restrict__ c, int m, int n, int k) {
  __shared__ float4 xs[MT][GS_KC / 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row0 = (blockIdx.x * 4 + wave) * GS_ROWS;
  float acc[GS_ROWS][MT];
#pragma unroll
  for (int r = 0; r < GS_ROWS; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = 0.f;
  const float* wrow[GS_ROWS];
#pragma unroll
  for (int r = 0; r < GS_ROWS; ++r) wrow[r] = w + (size_t)(row0 + r < n ? row0 + r : n - 1) * k;

  for (int k0 = 0; k0 < k; k0 += GS_KC) {
    __syncthreads();                  // the previous chunk has been used by every wave
    for (int idx = tid; idx < MT * (GS_KC / 4); idx += 256) {
      const int t = idx / (GS_KC / 4), q = idx % (GS_KC / 4);
      const int kk = k0 + 4 * q;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (t < m && kk < k) v = *reinterpret_cast<const float4*>(a + (size_t)t * k + kk);
      xs[t][q] = v;
    }
    __syncthreads();
#pragma unroll
    for (int step = 0; step < GS_KC / 256; ++step) {
      const int q = step * 64 + lane;
      const int kk = k0 + 4 * q;
      const int kl = kk < k ? kk : k - 4;            // beyond K: a valid address; the tokens' chunk holds zeros there
      float4 wv[GS_ROWS];
#pragma unroll
      for (int r = 0; r < GS_ROWS; ++r) wv[r] = *reinterpret_cast<const float4*>(wrow[r] + kl);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const float4 xv = xs[t][q];
#pragma unroll
        for (int r = 0; r < GS_ROWS; ++r) {
          acc[r][t] = fmaf(wv[r].x, xv.x, acc[r][t]);
          acc[r][t] = fmaf(wv[r].y, xv.y, acc[r][t]);
          acc[r][t] = fmaf(wv[r].z, xv.z, acc[r][t]);
          acc[r][t] = fmaf(wv[r].w, xv.w, acc[r][t]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < GS_ROWS; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const float v = wave_sum(acc[r][t]);
      if (lane == 0 && row0 + r < n && t < m) c[(size_t)t * n + row0 + r] = v;
    }
}

// Float32 operands, at most 64 tokens, K a multiple of 128 (the float32 path's decode step at the
// widths of real models): bound by reading W once, and built like the bfloat16 product for few
// tokens.  The float32 MFMA 16x16x4 (float32 inputs, products and sums): rows of W are the
// matrix cores' row operand, the tokens their columns.  Lane l (row r = l % 16, group kq = l / 16)
// loads 16 bytes of row r at depth 16 j + 4 kq and feeds its four values to four MFMAs; the tokens
// are loaded the same way, so that an MFMA sums over the depths 16 j + 4 kq + i of its four groups
// (which depth a group holds is free as long as both operands agree).  A stage is 128 depth values:
// 8 loads of W per row tile, non-temporal (W is read once per step), all in flight while the stage
// before is multiplied.  K is dealt to the waves of a workgroup in stages and their partial sums
// meet in LDS in a fixed order.
typedef __attribute__((ext_vector_type(4))) float gf_f32x4_t;

template <int MB, int R, bool WF>
__global__ __launch_bounds__(256) void gemm_f32_few_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                          float* __restrict__ c, int m, int n, int k) {
  extern __shared__ float red[];      // [waves - 1][R * MB * 4][64]
  constexpr int ACC = R * MB * 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
  const int r = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.x * (16 * R);
  gf_f32x4_t acc[R][MB];
#pragma unroll
  for (int rt = 0; rt < R; ++rt)
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) acc[rt][cb] = (gf_f32x4_t){0.f, 0.f, 0.f, 0.f};
  // Where a lane finds its 4 values at depth ks + 16 j + 4 kq of row tile rt: wrow[rt] + (ks + 16 j) * WK.
  // Rows [N, K]: the row's start + 4 kq, WK = 1.  Fragment-major (blocks of 16 rows x 16 depth values, 1 KB,
  // the 16 bytes of lane l at 16 l): the tile's start + 4 lane, WK = 16; a wave's load is then 1 KB in a
  // row, and W, read once per step, goes past the caches.
  constexpr int WK = WF ? 16 : 1;
  const float* wrow[R];
#pragma unroll
  for (int rt = 0; rt < R; ++rt) {
    const int row = n0 + 16 * rt + r;
    if (WF) wrow[rt] = w + (size_t)(n0 + 16 * rt < n ? n0 + 16 * rt : 0) * k + 4 * lane;
    else wrow[rt] = w + (size_t)(row < n ? row : 0) * k + 4 * kq;        // rows beyond N: row 0, never stored
  }
  const float* xrow[MB];
#pragma unroll
  for (int cb = 0; cb < MB; ++cb) {
    const int row = 16 * cb + r;
    xrow[cb] = x + (size_t)(row < m ? row : 0) * k + 4 * kq;
  }
  // the K / 128 stages dealt to the waves as evenly as they go (the host launches no more waves than stages)
  const int total = k / 128, base = total / n_waves, extra = total % n_waves;
  const int stages = base + (wave < extra ? 1 : 0);
  const int k_begin = 128 * (wave * base + (wave < extra ? wave : extra));
  gf_f32x4_t a[R][8], b[MB][8];
  auto load_stage = [&](int st) {
    const int ks = k_begin + 128 * st;
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int rt = 0; rt < R; ++rt)
        a[rt][j] = WF ? __builtin_nontemporal_load(reinterpret_cast<const gf_f32x4_t*>(wrow[rt] + (size_t)(ks + 16 * j) * WK))
                      : *reinterpret_cast<const gf_f32x4_t*>(wrow[rt] + ks + 16 * j);
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) b[cb][j] = *reinterpret_cast<const gf_f32x4_t*>(xrow[cb] + ks + 16 * j);
  };
  auto multiply_stage = [&]() {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
          for (int cb = 0; cb < MB; ++cb)
            acc[rt][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[rt][j][i], b[cb][j][i], acc[rt][cb], 0, 0, 0);
  };
  load_stage(0);
  for (int st = 1; st < stages; ++st) {
    multiply_stage();
    load_stage(st);
  }
  multiply_stage();

  if (n_waves > 1) {
    if (wave > 0) {
      float* dst = red + (size_t)(wave - 1) * ACC * 64 + lane;
#pragma unroll
      for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int cb = 0; cb < MB; ++cb)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[((rt * MB + cb) * 4 + i) * 64] = acc[rt][cb][i];
    }
    __syncthreads();
    if (wave != 0) return;
    for (int ww = 0; ww < n_waves - 1; ++ww) {
      const float* src = red + (size_t)ww * ACC * 64 + lane;
#pragma unroll
      for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int cb = 0; cb < MB; ++cb)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[rt][cb][i] += src[((rt * MB + cb) * 4 + i) * 64];
    }
  }
  // lane l holds, for token 16 cb + l % 16, the rows n0 + 16 rt + 4 (l / 16) + i
#pragma unroll
  for (int rt = 0; rt < R; ++rt)
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) {
      const int mm = 16 * cb + r, nn = n0 + 16 * rt + 4 * kq;
      if (mm >= m) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nn + i < n) c[(size_t)mm * n + nn + i] = acc[rt][cb][i];
    }
}

static int g_f32_few = 1;
// experiments only: 0 = the float32 product of few tokens (W as rows) on the vector units; 3 = one row tile a wave whatever the sizes
extern "C" void rb_tune_f32_few(int on) { g_f32_few = on; }

// One row tile per wave and at most 4 waves: measured at 1 to 16 tokens on the products of the 8B shape with W
// fragment-major, two row tiles a wave lose everywhere but in the output matrix at 16 tokens (28,672 rows at
// K = 4096, 8 tokens: 78 us against 93; 4,096 rows at K = 14336: 38 against 54), and 4 waves are as fast as 8
// or faster (4,096 rows at K = 4096: 13.2 us against 14.4).  The kernel is never launched with more.
template <int MB>
static void launch_f32_few(const float* x, const float* w, bool w_frag, float* c, int m, int n, int k, hipStream_t s) {
  int n_waves = k / 256;
  if (n_waves < 1) n_waves = 1;
  if (n_waves > 4) n_waves = 4;
  // From 33 tokens on a wave reads three to four times as many bytes of tokens as of W for every stage: two row
  // tiles a wave halve that (28,672 rows at K = 4096 with 64 tokens: 220 us against 305; 128,256 rows: 868
  // against 1,335; with 33 tokens 227 against 262).
  if constexpr (MB >= 3) {
    // (such a wave holds 246 registers, so a compute unit runs one workgroup of them: only where that still
    // gives every compute unit two workgroups and more)
    if (g_f32_few != 3 && (n + 31) / 32 >= 2 * rb_compute_units()) {
      const size_t lds2 = (size_t)(n_waves - 1) * 2 * MB * 4 * 64 * sizeof(float);
      const int grid2 = (n + 31) / 32;
      if (w_frag) gemm_f32_few_kernel<MB, 2, true><<<grid2, 64 * n_waves, lds2, s>>>(x, w, c, m, n, k);
      else gemm_f32_few_kernel<MB, 2, false><<<grid2, 64 * n_waves, lds2, s>>>(x, w, c, m, n, k);
      return;
    }
  }
  const size_t lds = (size_t)(n_waves - 1) * MB * 4 * 64 * sizeof(float);
  const int grid = (n + 15) / 16;
  if (w_frag) gemm_f32_few_kernel<MB, 1, true><<<grid, 64 * n_waves, lds, s>>>(x, w, c, m, n, k);
  else gemm_f32_few_kernel<MB, 1, false><<<grid, 64 * n_waves, lds, s>>>(x, w, c, m, n, k);
}

// Float32 operands and more than 16 tokens with K a multiple of 16 (the float32 path's
// prefill): the float32 MFMA (v_mfma_f32_32x32x2_f32: float32 inputs, float32 products and
// sums; no reduced-precision mode).  128 x 128 tiles, 16 deep, one wave per 64 x 64 piece.  W
// and the tokens are read with 16-byte loads along K and stored in LDS depth-major
// ([k][row], rows padded by 4 floats), so that the 32 lanes that read one depth value of 32
// rows hit 32 different banks; the next tile's loads are in flight in registers while the
// current one is multiplied.  D layout of the MFMA: lane l holds column l % 32 (a token),
// rows 8 * (i / 4) + 4 * (l / 32) + i % 4 (rows of W).
typedef __attribute__((ext_vector_type(16))) float gf32x16_t;
#define GM_T 128
#define GM_K 16
#define GM_LD (GM_T + 4)

template <bool WF>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            float* __restrict__ c, int m, int n, int k) {
  __shared__ float ws[2][GM_K][GM_LD];
  __shared__ float xs[2][GM_K][GM_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * GM_T, m0 = blockIdx.y * GM_T;
  const int wn0 = (wave & 1) * 64, wm0 = (wave >> 1) * 64;
  const int l32 = lane & 31, g = lane >> 5;

  gf32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // staging: thread t loads, for q = t and t + 256, row q / 4 of the tile, depth values 4 (q % 4) .. + 3;
  // of a fragment-major W (blocks of 16 rows x 16 depth values, the 16 bytes of lane l at 16 l) the 16 bytes
  // q % 64 of the tile's block q / 64: row 16 (q / 64) + q % 16, depth values 4 ((q % 64) / 16) .. + 3
  const float* wp[2];
  const float* xp[2];
  int w_row[2], w_kk[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = tid + 256 * i;
    int xr = m0 + q / 4;
    if (xr > m - 1) xr = m - 1;            // rows beyond the matrix: a valid row, never stored
    xp[i] = x + (size_t)xr * k + 4 * (q % 4);
    if (WF) {
      int tile = n0 / 16 + q / 64;
      if (tile > n / 16 - 1) tile = n / 16 - 1;
      w_row[i] = 16 * (q / 64) + q % 16;
      w_kk[i] = 4 * ((q % 64) / 16);
      wp[i] = w + (size_t)tile * 16 * k + 4 * (q % 64);
    } else {
      int wr = n0 + q / 4;
      if (wr > n - 1) wr = n - 1;
      w_row[i] = q / 4;
      w_kk[i] = 4 * (q % 4);
      wp[i] = w + (size_t)wr * k + 4 * (q % 4);
    }
  }
  float4 wreg[2], xreg[2];
  auto load_tile = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      wreg[i] = *reinterpret_cast<const float4*>(wp[i] + (size_t)kt * (WF ? 256 : GM_K));
      xreg[i] = *reinterpret_cast<const float4*>(xp[i] + (size_t)kt * GM_K);
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = tid + 256 * i;
      const int row = q / 4, kk = 4 * (q % 4);
      ws[buf][w_kk[i] + 0][w_row[i]] = wreg[i].x;
      ws[buf][w_kk[i] + 1][w_row[i]] = wreg[i].y;
      ws[buf][w_kk[i] + 2][w_row[i]] = wreg[i].z;
      ws[buf][w_kk[i] + 3][w_row[i]] = wreg[i].w;
      xs[buf][kk + 0][row] = xreg[i].x;
      xs[buf][kk + 1][row] = xreg[i].y;
      xs[buf][kk + 2][row] = xreg[i].z;
      xs[buf][kk + 3][row] = xreg[i].w;
    }
  };
  const int k_tiles = k / GM_K;
  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < k_tiles; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < k_tiles) load_tile(kt + 1);
#pragma unroll
    for (int ks = 0; ks < GM_K / 2; ++ks) {
      float a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i] = ws[buf][2 * ks + g][wn0 + 32 * i + l32];
#pragma unroll
      for (int j = 0; j < 2; ++j) b[j] = xs[buf][2 * ks + g][wm0 + 32 * j + l32];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < k_tiles) store_tile(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int mm = m0 + wm0 + 32 * j + l32;
      if (mm >= m) continue;
      float* dst = c + (size_t)mm * n;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int nn = n0 + wn0 + 32 * i + 8 * (e / 4) + 4 * g + (e % 4);
        if (nn < n) dst[nn] = acc[i][j][e];
      }
    }
}

extern "C" int rb_gemm_generic(const void* a, const void* w, int w_layout, void* c, int dtype_in, int dtype_out, int m,
                               int n, int k, void* stream) {
  RB_RECORDED(rb_gemm_generic(a, w, w_layout, c, dtype_in, dtype_out, m, n, k, stream));
  RB_REQUIRE(m >= 0 && n > 0 && k > 0, "rb_gemm_generic: bad sizes M=%d N=%d K=%d", m, n, k);
  // a fragment-major W is float32 with N % 16 == 0 and K % 128 == 0: sizes that the two matrix-core kernels take
  RB_REQUIRE(w_layout == 0 || (w_layout == 1 && dtype_in == RB_F32 && dtype_out == RB_F32 && n % 16 == 0 && k % 128 == 0),
             "rb_gemm_generic: W layout %d with dtype %d, N=%d K=%d (fragment-major: float32, N %% 16 == 0, K %% 128 == 0)",
             w_layout, dtype_in, n, k);
  const bool w_frag = w_layout == 1;
  if (m == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype_in == RB_F32 && dtype_out == RB_F32 && m <= 64 && k % 128 == 0 && (g_f32_few || w_frag)) {
    const float* af = (const float*)a;
    const float* wf = (const float*)w;
    const int mb = (m + 15) / 16;
    if (mb == 1) launch_f32_few<1>(af, wf, w_frag, (float*)c, m, n, k, s);
    else if (mb == 2) launch_f32_few<2>(af, wf, w_frag, (float*)c, m, n, k, s);
    else launch_f32_few<4>(af, wf, w_frag, (float*)c, m, n, k, s);
    RB_LAUNCH_CHECK();
    return 0;
  }
  if (dtype_in == RB_F32 && dtype_out == RB_F32 && m <= 16 && k % 4 == 0) {
    const unsigned blocks = (unsigned)((n + 4 * GS_ROWS - 1) / (4 * GS_ROWS));
    const float* af = (const float*)a;
    const float* wf = (const float*)w;
    if (m <= 4) gemm_f32_skinny_kernel<4><<<blocks, 256, 0, s>>>(af, wf, (float*)c, m, n, k);
    else if (m <= 8) gemm_f32_skinny_kernel<8><<<blocks, 256, 0, s>>>(af, wf, (float*)c, m, n, k);
    else gemm_f32_skinny_kernel<16><<<blocks, 256, 0, s>>>(af, wf, (float*)c, m, n, k);
    RB_LAUNCH_CHECK();
    return 0;
  }
  if (dtype_in == RB_F32 && dtype_out == RB_F32 && m > 16 && k % GM_K == 0) {
    dim3 tiles((n + GM_T - 1) / GM_T, (m + GM_T - 1) / GM_T);
    RB_REQUIRE(tiles.y <= 65535, "rb_gemm_generic: M=%d too large for one launch", m);
    if (w_frag) gemm_f32_mfma_kernel<true><<<tiles, 256, 0, s>>>((const float*)a, (const float*)w, (float*)c, m, n, k);
    else gemm_f32_mfma_kernel<false><<<tiles, 256, 0, s>>>((const float*)a, (const float*)w, (float*)c, m, n, k);
    RB_LAUNCH_CHECK();
    return 0;
  }
  RB_REQUIRE(!w_frag, "rb_gemm_generic: internal: a fragment-major W reached the kernels for rows");
  dim3 grid((n + GT - 1) / GT, (m + GT - 1) / GT);
  RB_REQUIRE(grid.y <= 65535, "rb_gemm_generic: M=%d too large for one launch", m);
  if (dtype_in == RB_F32 && dtype_out == RB_F32)
    gemm_generic_kernel<float, float><<<grid, 256, 0, s>>>((const float*)a, (const float*)w, (float*)c, m, n, k);
  else if (dtype_in == RB_BF16 && dtype_out == RB_F32)
    gemm_generic_kernel<bf16_t, float><<<grid, 256, 0, s>>>((const bf16_t*)a, (const bf16_t*)w, (float*)c, m, n, k);
  else if (dtype_in == RB_BF16 && dtype_out == RB_BF16)
    gemm_generic_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)c, m, n, k);
  else
    RB_REQUIRE(false, "rb_gemm_generic: unsupported dtypes in=%d out=%d", dtype_in, dtype_out);
  RB_LAUNCH_CHECK();
  return 0;
}
