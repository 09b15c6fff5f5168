// Products with few tokens (decode): bound by reading W once.  A wave owns 16*R rows of W and
// a slice of K, streams them with 16-byte loads straight into MFMA operands (W rows are the
// row operand, the tokens the columns, so a lane ends up with 4 consecutive outputs of one
// token), and the waves of a workgroup add their partial sums through LDS (no atomics: the
// sum order is fixed).
//
// Epilogue 1 expects W with gate and up rows interleaved in blocks of 16 and writes
// silu(gate) * up (llama/model.rs:297-302 of the reference) instead of the two products.
//
// Reference loop: y[o] = sum_i W[i + o * n_in] * x[i]  (llama/model.rs:67-91).
#include "api.h"
#include "gemm_internal.h"

template <int MB, int R, int U, bool FAST, int EPI, typename TO>
__global__ __launch_bounds__(512) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                          const bf16_t* __restrict__ w, TO* __restrict__ c,
                                                          int m, int n, int k, int k_per_wave) {
  extern __shared__ float red[];      // [waves - 1][ACC][64]
  constexpr int ACC = R * MB * 4;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n_waves = blockDim.x >> 6;
  const int r = lane & 15;
  const int kq = lane >> 4;
  const int n0 = blockIdx.x * (16 * R);

  f32x4_t acc[R][MB];
#pragma unroll
  for (int rt = 0; rt < R; ++rt)
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) acc[rt][cb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const bf16_t* wrow[R];
  bool wok[R];
#pragma unroll
  for (int rt = 0; rt < R; ++rt) {
    const int row = n0 + 16 * rt + r;
    wok[rt] = row < n;
    wrow[rt] = w + (size_t)(wok[rt] ? row : 0) * k;
  }
  const bf16_t* xrow[MB];
  bool xok[MB];
#pragma unroll
  for (int cb = 0; cb < MB; ++cb) {
    const int row = 16 * cb + r;
    xok[cb] = row < m;
    xrow[cb] = x + (size_t)(xok[cb] ? row : 0) * k;
  }

  int k_begin = wave * k_per_wave;
  const int k_end = (k_begin + k_per_wave < k) ? k_begin + k_per_wave : k;
  if (FAST) {
    // K and every wave's range are multiples of 128: no bounds checks.  Rows beyond N or M
    // are read from row 0 instead and their results never stored.  U stages of 128 depth
    // values stay in flight: as soon as a stage has been multiplied, its registers are
    // loaded again with the stage U further on.
    // Every wave has at least one stage (the host launches no more waves than stages), and a
    // wave's stage count is a multiple of U: the loads below are unconditional, which lets the
    // compiler count outstanding loads exactly and start multiplying when the oldest stage
    // arrives.  The K / 128 stages are dealt to the waves as evenly as they go: the first
    // K / 128 % waves waves take one more (K = 11008 = 86 stages over 8 waves: six times 11,
    // twice 10).
    static_assert(U == 1, "uneven stage counts per wave need one stage in flight");
    const int total = k / 128, base = total / n_waves, extra = total % n_waves;
    const int stages = base + (wave < extra ? 1 : 0);
    k_begin = 128 * (wave * base + (wave < extra ? wave : extra));
    Frag8 a[U][R][4], b[U][MB][4];
    auto load_stage = [&](int u, int st) {
      const int kk = k_begin + 128 * st + 8 * kq;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int rt = 0; rt < R; ++rt) a[u][rt][j].u = load16(wrow[rt] + kk + 32 * j);
#pragma unroll
        for (int cb = 0; cb < MB; ++cb) b[u][cb][j].u = load16(xrow[cb] + kk + 32 * j);
      }
    };
    auto multiply_stage = [&](int u) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
          for (int cb = 0; cb < MB; ++cb) acc[rt][cb] = mfma16(a[u][rt][j], b[u][cb][j], acc[rt][cb]);
    };
#pragma unroll
    for (int u = 0; u < U; ++u) load_stage(u, u);
    for (int s0 = 0; s0 + U < stages; s0 += U) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        multiply_stage(u);
        load_stage(u, s0 + u + U);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) multiply_stage(u);
  } else {
    for (int k0 = k_begin; k0 < k_end; k0 += 128) {
      Frag8 a[R][4], b[MB][4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kk = k0 + 32 * j + 8 * kq;
        const bool in = kk < k_end;
#pragma unroll
        for (int rt = 0; rt < R; ++rt) a[rt][j].u = (in && wok[rt]) ? load16(wrow[rt] + kk) : zero16();
#pragma unroll
        for (int cb = 0; cb < MB; ++cb) b[cb][j].u = (in && xok[cb]) ? load16(xrow[cb] + kk) : zero16();
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
          for (int cb = 0; cb < MB; ++cb) acc[rt][cb] = mfma16(a[rt][j], b[cb][j], acc[rt][cb]);
    }
  }

  // ---- partial sums of waves 1.. go through LDS to wave 0
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
    if (wave == 0) {
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
  }
  if (wave != 0) return;

  // ---- lane holds, per (rt, cb): token 16*cb + r, W rows n0 + 16*rt + 4*kq + 0..3
  if (EPI == 0) {
#pragma unroll
    for (int rt = 0; rt < R; ++rt)
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) {
        const int mm = 16 * cb + r;
        const int nn = n0 + 16 * rt + 4 * kq;
        if (mm >= m) continue;
        TO* dst = c + (size_t)mm * n + nn;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nn + i < n) Num<TO>::store(dst + i, acc[rt][cb][i]);
      }
  } else {
    const int half_n = n / 2;
#pragma unroll
    for (int rt = 0; rt + 1 < R; rt += 2)
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) {
        const int mm = 16 * cb + r;
        const int nn = n0 / 2 + 16 * (rt / 2) + 4 * kq;
        if (mm >= m) continue;
        TO* dst = c + (size_t)mm * half_n + nn;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nn + i < half_n) Num<TO>::store(dst + i, silu_f32(acc[rt][cb][i]) * acc[rt + 1][cb][i]);
      }
  }
}

static int g_tune_u = 0, g_tune_r = 0, g_tune_waves = 0;
extern "C" void rb_tune(int u, int r, int waves) {       // experiments only; 0 = the built-in choice
  g_tune_u = u;
  g_tune_r = r;
  g_tune_waves = waves;
}

template <int MB, int R, int U, bool FAST, int EPI, typename TO>
static int launch_skinny(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, int n_waves,
                         int k_per_wave, hipStream_t s) {
  const size_t lds = (size_t)(n_waves - 1) * R * MB * 4 * 64 * sizeof(float);
  RB_REQUIRE(lds <= 64 * 1024, "rb_gemm_bf16: internal: reduction buffer of %zu bytes", lds);
  const int grid = (n + 16 * R - 1) / (16 * R);
  gemm_skinny_kernel<MB, R, U, FAST, EPI, TO><<<grid, n_waves * 64, lds, s>>>(x, w, (TO*)c, m, n, k, k_per_wave);
  return 0;
}

// How K is dealt to the waves of a workgroup.  Fast path: K = 128 * T, the T stages dealt to
// the waves as evenly as they go.  Otherwise the checked path with up to 8 waves.  Measured on the Llama-3-8B
// products at M = 1..8: one stage in flight per wave (U = 1) is as fast as 2 or 4, and 4
// waves beat 8 at K = 4096, 8 beat 4 at K = 14336.
template <int MB, int R, int EPI, typename TO>
static int launch_skinny_u(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, hipStream_t s) {
  constexpr int max_waves = (R * MB <= 4) ? 8 : (R * MB <= 8 ? 4 : 3);      // bounds the reduction buffer
  if (k % 128 == 0) {
    const int t = k / 128;
    int nw = g_tune_waves ? g_tune_waves : ((k >= 8192 || max_waves < 4) ? max_waves : 4);
    if (nw > max_waves) nw = max_waves;
    if (nw > t) nw = t;
    return launch_skinny<MB, R, 1, true, EPI, TO>(x, w, c, m, n, k, nw, 0, s);
  }
  int n_waves = k / 256;
  if (n_waves < 1) n_waves = 1;
  if (n_waves > max_waves) n_waves = max_waves;
  int k_per_wave = (k + n_waves - 1) / n_waves;
  k_per_wave = (k_per_wave + 127) / 128 * 128;
  return launch_skinny<MB, R, 1, false, EPI, TO>(x, w, c, m, n, k, n_waves, k_per_wave, s);
}

template <int EPI, typename TO>
static int dispatch_skinny(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, hipStream_t s) {
  const int mb = (m + 15) / 16;
  // rows of W per wave: more of them reuse the token operand better, fewer give more
  // workgroups; keep at least about two workgroups per compute unit
  int r = 1;
  if (n >= 16384) r = 4;
  else if (n >= 6144) r = 2;
  if (g_tune_r) r = g_tune_r;
  if (EPI == 1 && r < 2) r = 2;
#define RB_SK(MBV, RV) return launch_skinny_u<MBV, RV, EPI, TO>(x, w, c, m, n, k, s)
  if (mb == 1) {
    if (r == 4) RB_SK(1, 4);
    if (r == 2) RB_SK(1, 2);
    if (EPI == 0) RB_SK(1, 1);
  } else if (mb == 2) {
    if (r == 4) RB_SK(2, 4);
    if (r == 2) RB_SK(2, 2);
    if (EPI == 0) RB_SK(2, 1);
  } else if (mb == 3) {
    if (r == 4) RB_SK(3, 4);
    if (r == 2) RB_SK(3, 2);
    if (EPI == 0) RB_SK(3, 1);
  } else {
    if (r == 4) RB_SK(4, 4);
    if (r == 2) RB_SK(4, 2);
    if (EPI == 0) RB_SK(4, 1);
  }
#undef RB_SK
  RB_REQUIRE(false, "rb_gemm_bf16: internal: no skinny kernel for M=%d R=%d", m, r);
}

// =============================================================================== skinny, tokens resident
// The same product for M <= 64 with the token operand held in registers: a wave owns a
// fixed slice of K (32 * XQ values), loads the tokens' fragments for it once, and then
// streams the W rows of one 16-row tile after the other through the matrix cores, the
// next tile's loads in flight while the current one is multiplied.  Inside the loop W is
// the only thing read from memory.  A workgroup's waves cover adjacent K slices and add
// their sums through LDS.
template <int MB, int XQ, int EPI, typename TO>
__global__ __launch_bounds__(512) void gemm_resident_kernel(const bf16_t* __restrict__ x,
                                                             const bf16_t* __restrict__ w, TO* __restrict__ c,
                                                             int m, int n, int k, int tiles_per_wg) {
  extern __shared__ float red[];      // [2][waves - 1][MB * 4][64]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n_waves = blockDim.x >> 6;
  const int r = lane & 15;
  const int kq = lane >> 4;
  const int n_tiles = (n + 15) / 16;
  const int tile0 = blockIdx.x * tiles_per_wg;
  int t_count = n_tiles - tile0;
  if (t_count > tiles_per_wg) t_count = tiles_per_wg;
  const int k0 = (blockIdx.y * n_waves + wave) * (32 * XQ) + 8 * kq;
  TO* cpart = c + (size_t)blockIdx.y * m * (EPI == 1 ? n / 2 : n);

  // ---- the tokens' fragments for this wave's slice of K
  Frag8 b[XQ][MB];
#pragma unroll
  for (int cb = 0; cb < MB; ++cb) {
    const int row = 16 * cb + r;
    const bf16_t* xrow = x + (size_t)(row < m ? row : 0) * k + k0;
#pragma unroll
    for (int j = 0; j < XQ; ++j) b[j][cb].u = load16(xrow + 32 * j);
  }

  Frag8 a0[XQ], a1[XQ];
  auto load_tile = [&](Frag8* a, int t) {
    int row = (tile0 + t) * 16 + r;
    if (row >= n) row = 0;                       // results of such rows are never stored
    const bf16_t* wrow = w + (size_t)row * k + k0;
#pragma unroll
    for (int j = 0; j < XQ; ++j) a[j].u = load16(wrow + 32 * j);
  };
  f32x4_t gate[MB];                              // EPI 1: the gate tile's sums wait for the up tile
  auto finish_tile = [&](const Frag8* a, int t) {
    f32x4_t acc[MB];
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) acc[cb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < XQ; ++j)
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) acc[cb] = mfma16(a[j], b[j][cb], acc[cb]);
    // the wave that gathers this tile's sums: tiles of a gate/up pair go to the same one
    const int owner = (EPI == 1 ? (t >> 1) : t) % n_waves;
    if (n_waves > 1) {
      float* buf = red + (size_t)(t & 1) * (n_waves - 1) * MB * 4 * 64;
      if (wave != owner) {
        const int slot = wave < owner ? wave : wave - 1;
        float* dst = buf + (size_t)slot * MB * 4 * 64 + lane;
#pragma unroll
        for (int cb = 0; cb < MB; ++cb)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[(cb * 4 + i) * 64] = acc[cb][i];
      }
      __syncthreads();
      if (wave == owner) {
        for (int ww = 0; ww < n_waves - 1; ++ww) {
          const float* src = buf + (size_t)ww * MB * 4 * 64 + lane;
#pragma unroll
          for (int cb = 0; cb < MB; ++cb)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[cb][i] += src[(cb * 4 + i) * 64];
        }
      }
    }
    if (wave != owner) return;
    const int tile = tile0 + t;
    if (EPI == 0) {
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) {
        const int mm = 16 * cb + r;
        const int nn = tile * 16 + 4 * kq;
        if (mm >= m) continue;
        TO* dst = cpart + (size_t)mm * n + nn;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nn + i < n) Num<TO>::store(dst + i, acc[cb][i]);
      }
    } else if ((t & 1) == 0) {
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) gate[cb] = acc[cb];
    } else {
      const int half_n = n / 2;
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) {
        const int mm = 16 * cb + r;
        const int nn = (tile >> 1) * 16 + 4 * kq;
        if (mm >= m) continue;
        TO* dst = cpart + (size_t)mm * half_n + nn;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nn + i < half_n) Num<TO>::store(dst + i, silu_f32(gate[cb][i]) * acc[cb][i]);
      }
    }
  };

  if (t_count <= 0) return;
  load_tile(a0, 0);
  int t = 0;
  for (; t + 2 < t_count; t += 2) {              // tiles t + 1 and t + 2 exist: loads are unconditional
    load_tile(a1, t + 1);
    finish_tile(a0, t);
    load_tile(a0, t + 2);
    finish_tile(a1, t + 1);
  }
  if (t + 1 < t_count) {
    load_tile(a1, t + 1);
    finish_tile(a0, t);
    finish_tile(a1, t + 1);
  } else {
    finish_tile(a0, t);
  }
}

static int g_res_tiles = 0;
extern "C" void rb_tune_resident(int waves, int parts, int tiles) {      // experiments only; 0 = built-in
  (void)waves;
  (void)parts;
  g_res_tiles = tiles;
}

template <int MB, int XQ, int EPI, typename TO>
static int launch_resident(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, int parts,
                           hipStream_t s) {
  const int slices = k / (32 * XQ);
  const int n_waves = slices / parts;
  const int n_tiles = (n + 15) / 16;
  // tiles per workgroup: as many as give every compute unit one workgroup at most, but no more
  // than 16 (measured: 22016 rows in 230 workgroups of 6 tiles take 35 us, in 344 of 4, which
  // come in two rounds, 44 us; 12288 rows 20 us in 256 workgroups, 31 us in 384; the 128256
  // rows of an output layer are as fast in 501 workgroups of 16 tiles as in 251 of 32)
  int tiles = g_res_tiles ? g_res_tiles : (n_tiles + 255) / 256;
  if (!g_res_tiles && tiles > 16) tiles = 16;
  if (EPI == 1 && (tiles & 1)) tiles += 1;
  const size_t lds = (size_t)2 * (n_waves > 1 ? n_waves - 1 : 0) * MB * 4 * 64 * sizeof(float);
  dim3 grid((n_tiles + tiles - 1) / tiles, parts);
  gemm_resident_kernel<MB, XQ, EPI, TO><<<grid, n_waves * 64, lds, s>>>(x, w, (TO*)c, m, n, k, tiles);
  return 0;
}

// true if the resident kernel takes these sizes
template <int EPI, typename TO>
static bool try_resident(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, int parts, hipStream_t s,
                         int* rc) {
  const int mb = (m + 15) / 16;
  const int xq = mb == 1 ? 16 : (mb == 2 ? 8 : 4);
  if (k % (32 * xq) != 0) return false;
  const int slices = k / (32 * xq);
  if (parts < 1 || slices % parts != 0) return false;
  const int n_waves = slices / parts;
  if (n_waves > 8) return false;
  if (EPI == 1 && (n % 32 != 0)) return false;
  if (mb == 1) *rc = launch_resident<1, 16, EPI, TO>(x, w, c, m, n, k, parts, s);
  else if (mb == 2) *rc = launch_resident<2, 8, EPI, TO>(x, w, c, m, n, k, parts, s);
  else if (mb == 3) *rc = launch_resident<3, 4, EPI, TO>(x, w, c, m, n, k, parts, s);
  else *rc = launch_resident<4, 4, EPI, TO>(x, w, c, m, n, k, parts, s);
  return true;
}


#define RB_BY_OUTPUT(FN, ...)                                                              \
  (epilogue == 0 ? (dtype_out == RB_F32 ? FN<0, float>(__VA_ARGS__) : FN<0, bf16_t>(__VA_ARGS__)) \
                 : (dtype_out == RB_F32 ? FN<1, float>(__VA_ARGS__) : FN<1, bf16_t>(__VA_ARGS__)))

int gemm_skinny_launch(const bf16_t* x, const bf16_t* w, void* c, int dtype_out, int epilogue, int m, int n, int k,
                       hipStream_t s) {
  return RB_BY_OUTPUT(dispatch_skinny, x, w, c, m, n, k, s);
}

bool gemm_resident_try(const bf16_t* x, const bf16_t* w, void* c, int dtype_out, int epilogue, int m, int n, int k,
                       hipStream_t s, int* rc) {
  return RB_BY_OUTPUT(try_resident, x, w, c, m, n, k, 1, s, rc);
}
