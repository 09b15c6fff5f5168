// Products with few tokens (decode): bound by reading W once.  A wave owns 16*R rows of W and
// a slice of K, streams them with 16-byte loads straight into MFMA operands (W rows are the
// row operand, the tokens the columns, so a lane ends up with 4 consecutive outputs of one
// token), and the waves of a workgroup add their partial sums through LDS (no atomics: the
// sum order is fixed).
//
// Epilogue 1 expects W with gate and up rows interleaved in blocks of 16 and writes
// silu(gate) * up (llama/model.rs:297-302 of the reference) instead of the two products.
//
// What stands between two products of a decode step is folded into them (1..16 tokens):
//  * epilogue 2 adds the product to the float32 C it finds, the residual sum of
//    llama/model.rs:292-294 and :304-306; every element is read and written by one lane.
//  * epilogue 3 does the same and prepares the RMS norm that follows (llama/model.rs:93-100,
//    y_i = x_i * w_i / sqrt(mean(x^2) + eps)): it also writes bf16(x_i * w_i) and, for every 16
//    columns, the sum of x_i^2.  Both need the new x_i only, which the lane has at hand.
//  * SCALED: the tokens are such prepared rows.  The waves add up the sums of squares (in a
//    fixed order) while the product runs and the row's factor 1 / sqrt(..) is applied to the
//    float32 sums at the end.
// With both, no kernel runs between the products, and no row is read more often than before.
//
// Reference loop: y[o] = sum_i W[i + o * n_in] * x[i]  (llama/model.rs:67-91).
#include "api.h"
#include "tune.h"
#include "gemm_internal.h"

struct FoldArgs {
  const float* squares_in;      // SCALED: [*, ceil(K / 16)]
  const int32_t* rows;          // which rows of x (and of squares_in) the tokens are; null: 0..M-1
  float eps;
  const float* gain;            // epilogue 3: [N]
  bf16_t* gained;               // epilogue 3: [M, N]
  float* squares_out;           // epilogue 3: [M, ceil(N / 16)]
  int w_frag;                   // W is stored fragment-major (see gemm_internal.h)
};

// What a lane does with its 4 consecutive sums of token mm, columns nn.. (epilogues 0, 2, 3).
// All 64 lanes come here together: the sums of squares go round the four lanes that share
// a token's 16 columns.
template <int EPI, typename TO>
__device__ __forceinline__ void store_sums(TO* __restrict__ c, const f32x4_t& sums, const f32x4_t& before,
                                           const f32x4_t& gain, int mm, int nn, int m, int n, int tile, int kq,
                                           const FoldArgs& fa) {
  const bool row_ok = mm < m;
  float sq = 0.f;
  if (row_ok) {
    TO* dst = c + (size_t)mm * n + nn;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (nn + i >= n) continue;
      const float v = EPI >= 2 ? before[i] + sums[i] : sums[i];
      Num<TO>::store(dst + i, v);
      if (EPI == 3) {
        sq += v * v;
        fa.gained[(size_t)mm * n + nn + i] = f32_to_bf16(v * gain[i]);
      }
    }
  }
  if (EPI == 3) {
    sq += __shfl_xor(sq, 16, RB_WAVE);
    sq += __shfl_xor(sq, 32, RB_WAVE);
    if (row_ok && kq == 0 && tile * 16 < n) fa.squares_out[(size_t)mm * ((n + 15) / 16) + tile] = sq;
  }
}

// A lane's share of a row's n_sq sums of squares: `share` of `shares` (4 lanes of every wave work
// on one row).  With n_sq a multiple of 4 the first 16 * shares * SQ_WIDE of them are asked for
// with 16-byte loads that are all in flight together, and added up by squares_sum() when they
// are needed; the rest, if any, one by one.
constexpr int SQ_WIDE = 4;
struct SquaresShare {
  float4 wide[SQ_WIDE];
  float rest;
};
__device__ __forceinline__ SquaresShare squares_ask(const float* __restrict__ sq, int n_sq, int share, int shares) {
  SquaresShare out;
  out.rest = 0.f;
  int done = 0;
  if (n_sq % 4 == 0) {
#pragma unroll
    for (int j = 0; j < SQ_WIDE; ++j) {
      const int at = 4 * (share + j * shares);
      out.wide[j] = at < n_sq ? *reinterpret_cast<const float4*>(sq + at) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    done = 4 * shares * SQ_WIDE;
  } else {
#pragma unroll
    for (int j = 0; j < SQ_WIDE; ++j) out.wide[j] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  for (int i = done + share; i < n_sq; i += shares) out.rest += sq[i];
  return out;
}
__device__ __forceinline__ float squares_sum(const SquaresShare& s) {
  float t = s.rest;
#pragma unroll
  for (int j = 0; j < SQ_WIDE; ++j) t += (s.wide[j].x + s.wide[j].y) + (s.wide[j].z + s.wide[j].w);
  return t;
}

template <int MB, int R, int U, bool FAST, int EPI, typename TO, bool SCALED>
__global__ __launch_bounds__(512) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                          const bf16_t* __restrict__ w, TO* __restrict__ c,
                                                          int m, int n, int k, int k_per_wave, FoldArgs fa) {
  extern __shared__ float red[];      // [waves - 1][ACCX][64]
  constexpr int ACC = R * MB * 4;
  constexpr int ACCX = ACC + (SCALED ? MB : 0);      // the sums of squares travel with the partial sums
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

  // Where a lane finds its 8 values at depth kstart (a multiple of 32) + 8 kq of row tile rt:
  // wrow[rt] + kstart * wk.  Rows [N, K]: the row's start + 8 kq, wk = 1.  Fragment-major: the
  // tile's start + 8 lane, wk = 16 (a block of 16 rows x 32 depth values is 512 values).
  const bool wf = fa.w_frag != 0;
  const int wk = wf ? 16 : 1;
  const bf16_t* wrow[R];
  bool wok[R];
#pragma unroll
  for (int rt = 0; rt < R; ++rt) {
    const int row = n0 + 16 * rt + r;
    wok[rt] = row < n;
    if (wf) wrow[rt] = w + (size_t)(n0 + 16 * rt < n ? n0 + 16 * rt : 0) * k + 8 * lane;
    else wrow[rt] = w + (size_t)(wok[rt] ? row : 0) * k + 8 * kq;
  }
  const bf16_t* xrow[MB];
  bool xok[MB];
  float ss[MB];
  SquaresShare asked[MB];
#pragma unroll
  for (int cb = 0; cb < MB; ++cb) {
    const int row = 16 * cb + r;
    xok[cb] = row < m;
    size_t src = xok[cb] ? row : 0;
    if (fa.rows) src = (size_t)fa.rows[src];
    xrow[cb] = x + src * k;
    ss[cb] = 0.f;
    if (SCALED) {
      const int n_sq = (k + 15) / 16;
      asked[cb] = squares_ask(fa.squares_in + src * n_sq, n_sq, wave * 4 + kq, n_waves * 4);
    }
  }

  // epilogues 2 and 3: what C holds now, and the gain, are asked for before the products, not
  // after them
  f32x4_t before[R][MB], gain[R];
#pragma unroll
  for (int rt = 0; rt < R; ++rt) {
    const int nn = n0 + 16 * rt + 4 * kq;
    gain[rt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    if (EPI == 3 && wave == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (nn + i < n) gain[rt][i] = fa.gain[nn + i];
    }
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) {
      before[rt][cb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
      if (EPI >= 2 && wave == 0) {
        const int mm = 16 * cb + r;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (mm < m && nn + i < n) before[rt][cb][i] = Num<TO>::load(c + (size_t)mm * n + nn + i);
      }
    }
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
      const int ks = k_begin + 128 * st;
      const int kk = ks + 8 * kq;
      if (wf) {           // read once, whole lines at a time: past the caches
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int rt = 0; rt < R; ++rt) a[u][rt][j].u = load16_stream(wrow[rt] + (size_t)(ks + 32 * j) * 16);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int rt = 0; rt < R; ++rt) a[u][rt][j].u = load16(wrow[rt] + ks + 32 * j);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int cb = 0; cb < MB; ++cb) b[u][cb][j].u = load16(xrow[cb] + kk + 32 * j);
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
    // the sums of squares were asked for before the first stage and arrive before it: added up
    // here, they do not occupy registers during the loop
    if (SCALED) {
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) ss[cb] = squares_sum(asked[cb]);
    }
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
    if (SCALED) {
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) ss[cb] = squares_sum(asked[cb]);
    }
    for (int k0 = k_begin; k0 < k_end; k0 += 128) {
      Frag8 a[R][4], b[MB][4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kk = k0 + 32 * j + 8 * kq;
        const bool in = kk < k_end;
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
          a[rt][j].u = (in && wok[rt]) ? load16(wrow[rt] + (size_t)(k0 + 32 * j) * wk) : zero16();
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

  // ---- a token's squares: the four lanes that share its row add their shares
  if (SCALED) {
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) {
      ss[cb] += __shfl_xor(ss[cb], 16, RB_WAVE);
      ss[cb] += __shfl_xor(ss[cb], 32, RB_WAVE);
    }
  }

  // ---- partial sums of waves 1.. go through LDS to wave 0
  if (n_waves > 1) {
    if (wave > 0) {
      float* dst = red + (size_t)(wave - 1) * ACCX * 64 + lane;
#pragma unroll
      for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int cb = 0; cb < MB; ++cb)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[((rt * MB + cb) * 4 + i) * 64] = acc[rt][cb][i];
      if (SCALED) {
#pragma unroll
        for (int cb = 0; cb < MB; ++cb) dst[(ACC + cb) * 64] = ss[cb];
      }
    }
    __syncthreads();
    if (wave == 0) {
      for (int ww = 0; ww < n_waves - 1; ++ww) {
        const float* src = red + (size_t)ww * ACCX * 64 + lane;
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
          for (int cb = 0; cb < MB; ++cb)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[rt][cb][i] += src[((rt * MB + cb) * 4 + i) * 64];
        if (SCALED) {
#pragma unroll
          for (int cb = 0; cb < MB; ++cb) ss[cb] += src[(ACC + cb) * 64];
        }
      }
    }
  }
  if (wave != 0) return;

  if (SCALED) {
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) {
      const float scale = 1.0f / sqrtf(ss[cb] / (float)k + fa.eps);
#pragma unroll
      for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rt][cb][i] *= scale;
    }
  }

  // ---- lane holds, per (rt, cb): token 16*cb + r, W rows n0 + 16*rt + 4*kq + 0..3
  if (EPI != 1) {
#pragma unroll
    for (int rt = 0; rt < R; ++rt)
#pragma unroll
      for (int cb = 0; cb < MB; ++cb)
        store_sums<EPI, TO>(c, acc[rt][cb], before[rt][cb], gain[rt], 16 * cb + r, n0 + 16 * rt + 4 * kq, m, n,
                            n0 / 16 + rt, kq, fa);
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

static int g_tune_r = 0, g_tune_waves = 0;
extern "C" void rb_tune(int r, int waves) {       // experiments only; 0 = the built-in choice
  g_tune_r = r;
  g_tune_waves = waves;
}

static FoldArgs fold_args(const GemmTokens& x, const GemmAfter& after) {
  return FoldArgs{x.squares, x.rows, x.eps, after.gain, after.gained, after.squares, after.w_frag ? 1 : 0};
}

template <int MB, int R, int U, bool FAST, int EPI, typename TO, bool SCALED>
static int launch_skinny(const GemmTokens& x, const bf16_t* w, void* c, const GemmAfter& after, int m, int n, int k,
                         int n_waves, int k_per_wave, hipStream_t s) {
  const size_t lds = (size_t)(n_waves - 1) * (R * MB * 4 + (SCALED ? MB : 0)) * 64 * sizeof(float);
  RB_REQUIRE(lds <= 64 * 1024, "rb_gemm_bf16: internal: reduction buffer of %zu bytes", lds);
  const int grid = (n + 16 * R - 1) / (16 * R);
  gemm_skinny_kernel<MB, R, U, FAST, EPI, TO, SCALED>
      <<<grid, n_waves * 64, lds, s>>>(x.x, w, (TO*)c, m, n, k, k_per_wave, fold_args(x, after));
  return 0;
}

// How K is dealt to the waves of a workgroup.  Fast path: K = 128 * T, the T stages dealt to
// the waves as evenly as they go.  Otherwise the checked path with up to 8 waves.  Measured on the Llama-3-8B
// products at M = 1..8: one stage in flight per wave (U = 1) is as fast as 2 or 4, and 4
// waves beat 8 at K = 4096, 8 beat 4 at K = 14336.  (With W fragment-major again: launched alone, products
// with K = 8192 and more gain up to 10 % from two or four stages in flight; the decode steps they belong to
// lose 4-6 % at the 8B and 70B shapes and gain 1-2 % at hidden sizes of 2,048 and 3,072.  One stage it stays.)
template <int MB, int R, int EPI, typename TO, bool SCALED>
static int launch_skinny_u(const GemmTokens& x, const bf16_t* w, void* c, const GemmAfter& after, int m, int n, int k,
                           hipStream_t s) {
  constexpr int max_waves = (R * MB <= 4) ? 8 : (R * MB <= 8 ? 4 : 3);      // bounds the reduction buffer
  if (k % 128 == 0) {
    const int t = k / 128;
    // 8 waves where K is long, or where every compute unit gets one workgroup at most and so needs
    // more loads in flight of its own (4,096 rows at K = 4096: 8.1-8.3 us against 8.6-9.0 with 4);
    // 4 where several workgroups share a compute unit (6,144 rows: 10.7 against 11.6 with 8)
    const long long wgs = (n + 16 * R - 1) / (16 * R);
    int nw = g_tune_waves ? g_tune_waves : ((k >= 8192 || wgs <= rb_compute_units() || max_waves < 4) ? max_waves : 4);
    if (nw > max_waves) nw = max_waves;
    if (nw > t) nw = t;
    return launch_skinny<MB, R, 1, true, EPI, TO, SCALED>(x, w, c, after, m, n, k, nw, 0, s);
  }
  int n_waves = k / 256;
  if (n_waves < 1) n_waves = 1;
  if (n_waves > max_waves) n_waves = max_waves;
  int k_per_wave = (k + n_waves - 1) / n_waves;
  k_per_wave = (k_per_wave + 127) / 128 * 128;
  return launch_skinny<MB, R, 1, false, EPI, TO, SCALED>(x, w, c, after, m, n, k, n_waves, k_per_wave, s);
}

template <int EPI, typename TO, bool SCALED>
static int dispatch_skinny(const GemmTokens& x, const bf16_t* w, void* c, const GemmAfter& after, int m, int n, int k,
                           hipStream_t s) {
  constexpr bool FOLDS = SCALED || EPI >= 2;      // compiled for up to 16 tokens only
  const int mb = (m + 15) / 16;
  RB_REQUIRE(!FOLDS || mb == 1, "rb_gemm_bf16: a product that folds its neighbours in takes at most 16 tokens, not %d",
             m);
  // Row tiles of W per wave (16 R rows per workgroup).  Up to K = 4096 (workgroups of 4 waves, several
  // of which share a compute unit) one tile per wave is the fastest at every N from 1024 to 16384
  // (measured with 8 tokens, W fragment-major; N = 6144: 11.1 us against 13.5 with two).  From
  // K = 8192 on (8 waves) more tiles reuse the token operand better and fewer deal the rows to the 256
  // compute units more evenly: the time goes with the rows that the busiest compute unit gets, at
  // a price per row that falls with R (about 15 % / R).  57344 rows at K = 8192: R = 4 gives 896
  // workgroups, 4 on some compute units and 3 on others, 194 us; R = 2 gives every one 7: 175 us.
  // 10240 rows at K = 8192 with one token: R = 1 35 us, R = 2 42; R = 4 takes 31 us by itself (160
  // workgroups), but the decode step of that shape is no faster with it (+0.3 % at batch 1, +0.5 % at
  // 8, -1.1 % at 16, each the mean of four runs in alternating order), so it is not taken.
  // Between K = 4096 and 8192 the same estimate holds: 15,360 rows at K = 5120 with 16 tokens 26.6 us
  // with R = 4 against 33.6 with R = 1 (8 tokens: 26.4 against 27.5, one token 26.9 against 26.5),
  // 5,120 rows 13.6 with R = 2 against 16.8 (8 tokens: 12.1 against 13.4).
  int r = 1;
  if (k > 4096) {
    double best = 0.0;
    const long long cus = rb_compute_units();
    for (int cand = (EPI == 1 ? 2 : 1); cand <= 4; cand *= 2) {
      const long long wgs = (n + 16 * cand - 1) / (16 * cand);
      const double cost = (double)((wgs + cus - 1) / cus * 16 * cand) * (1.0 + 0.15 / cand);
      if (best == 0.0 || cost <= best) {
        best = cost;
        r = cand;
      }
    }
  }
  if (g_tune_r) r = g_tune_r;
  if (EPI == 1 && r < 2) r = 2;
#define RB_SK(MBV, RV) return launch_skinny_u<MBV, RV, EPI, TO, SCALED>(x, w, c, after, m, n, k, s)
  if (mb == 1) {
    if (r == 4) RB_SK(1, 4);
    if (r == 2) RB_SK(1, 2);
    if (EPI != 1) RB_SK(1, 1);
  }
  if constexpr (!FOLDS) {
    if (mb == 2) {
      if (r == 4) RB_SK(2, 4);
      if (r == 2) RB_SK(2, 2);
      if (EPI != 1) RB_SK(2, 1);
    } else if (mb == 3) {
      if (r == 4) RB_SK(3, 4);
      if (r == 2) RB_SK(3, 2);
      if (EPI != 1) RB_SK(3, 1);
    } else {
      if (r == 4) RB_SK(4, 4);
      if (r == 2) RB_SK(4, 2);
      if (EPI != 1) RB_SK(4, 1);
    }
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
// their sums through LDS.  SCALED and epilogues 2 and 3 as in the kernel above (one workgroup
// covers all of K).
template <int MB, int XQ, int EPI, typename TO, bool SCALED>
__global__ __launch_bounds__(512) void gemm_resident_kernel(const bf16_t* __restrict__ x,
                                                             const bf16_t* __restrict__ w, TO* __restrict__ c,
                                                             int m, int n, int k, int tiles_per_wg, FoldArgs fa) {
  extern __shared__ float red[];      // [2][waves - 1][MB * 4][64], then SCALED: [waves][MB * 16]
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

  if (t_count <= 0) return;
  Frag8 a0[XQ], a1[XQ];
  auto load_tile = [&](Frag8* a, int t) {
    if (fa.w_frag) {
      // fragment-major: the wave's XQ blocks of a tile are XQ KB in a row; read once, past the caches
      int tile = tile0 + t;
      if (tile * 16 >= n) tile = 0;              // results of such rows are never stored
      const bf16_t* p = w + ((size_t)tile * k + (size_t)(blockIdx.y * n_waves + wave) * (32 * XQ)) * 16 + 8 * lane;
#pragma unroll
      for (int j = 0; j < XQ; ++j) a[j].u = load16_stream(p + (size_t)j * 512);
      return;
    }
    int row = (tile0 + t) * 16 + r;
    if (row >= n) row = 0;                       // results of such rows are never stored
    const bf16_t* wrow = w + (size_t)row * k + k0;
#pragma unroll
    for (int j = 0; j < XQ; ++j) a[j].u = load16(wrow + 32 * j);
  };
  load_tile(a0, 0);            // the first rows of W are on their way while the tokens are fetched

  // ---- the tokens' fragments for this wave's slice of K
  Frag8 b[XQ][MB];
  float scale[MB];
#pragma unroll
  for (int cb = 0; cb < MB; ++cb) {
    const int row = 16 * cb + r;
    size_t src = row < m ? row : 0;
    if (fa.rows) src = (size_t)fa.rows[src];
    const bf16_t* xrow = x + src * k + k0;
#pragma unroll
    for (int j = 0; j < XQ; ++j) b[j][cb].u = load16(xrow + 32 * j);
    scale[cb] = 0.f;
    if (SCALED) {
      const int n_sq = (k + 15) / 16;
      scale[cb] = squares_sum(squares_ask(fa.squares_in + src * n_sq, n_sq, wave * 4 + kq, n_waves * 4));
    }
  }
  // SCALED: the waves' shares of the squares meet in LDS behind the first tile's barrier
  float* squares = red + (size_t)2 * (n_waves - 1) * MB * 4 * 64;      // [waves][MB * 16]
  bool scale_known = !SCALED;
  if (SCALED) {
#pragma unroll
    for (int cb = 0; cb < MB; ++cb) {
      scale[cb] += __shfl_xor(scale[cb], 16, RB_WAVE);
      scale[cb] += __shfl_xor(scale[cb], 32, RB_WAVE);
      if (n_waves > 1) {
        if (kq == 0) squares[wave * (MB * 16) + cb * 16 + r] = scale[cb];
      } else {
        scale[cb] = 1.0f / sqrtf(scale[cb] / (float)k + fa.eps);
      }
    }
    if (n_waves == 1) scale_known = true;
  }

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
      if (SCALED && !scale_known) {
#pragma unroll
        for (int cb = 0; cb < MB; ++cb) {
          float ss = 0.f;
          for (int ww = 0; ww < n_waves; ++ww) ss += squares[ww * (MB * 16) + cb * 16 + r];
          scale[cb] = 1.0f / sqrtf(ss / (float)k + fa.eps);
        }
        scale_known = true;
      }
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
    if (SCALED) {
#pragma unroll
      for (int cb = 0; cb < MB; ++cb)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[cb][i] *= scale[cb];
    }
    const int tile = tile0 + t;
    if (EPI != 1) {
#pragma unroll
      for (int cb = 0; cb < MB; ++cb) {
        const int mm = 16 * cb + r;
        const int nn = tile * 16 + 4 * kq;
        f32x4_t before = (f32x4_t){0.f, 0.f, 0.f, 0.f}, gain = before;
        if (EPI >= 2) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (mm < m && nn + i < n) before[i] = Num<TO>::load(cpart + (size_t)mm * n + nn + i);
            if (EPI == 3 && nn + i < n) gain[i] = fa.gain[nn + i];
          }
        }
        store_sums<EPI, TO>(cpart, acc[cb], before, gain, mm, nn, m, n, tile, kq, fa);
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

static int g_res_tiles = 0, g_res_forced = 0;
extern "C" void rb_tune_resident(int tiles) { g_res_tiles = tiles; }      // experiments only; 0 = built-in
void gemm_resident_forced(int on) { g_res_forced = on; }                  // set by rb_tune_use_resident(2)

template <int MB, int XQ, int EPI, typename TO, bool SCALED>
static int launch_resident(const GemmTokens& x, const bf16_t* w, void* c, const GemmAfter& after, int m, int n, int k,
                           int parts, hipStream_t s) {
  const int slices = k / (32 * XQ);
  const int n_waves = slices / parts;
  const int n_tiles = (n + 15) / 16;
  // tiles per workgroup: as many as give every compute unit one workgroup at most, but no more
  // than 16 (measured: 22016 rows in 230 workgroups of 6 tiles take 35 us, in 344 of 4, which
  // come in two rounds, 44 us; 12288 rows 20 us in 256 workgroups, 31 us in 384; the 128256
  // rows of an output layer are as fast in 501 workgroups of 16 tiles as in 251 of 32)
  const int cus = rb_compute_units();
  int tiles = g_res_tiles ? g_res_tiles : (n_tiles + cus - 1) / cus;
  if (!g_res_tiles && tiles > 16) tiles = 16;
  if (EPI == 1 && (tiles & 1)) tiles += 1;
  const size_t lds = ((size_t)2 * (n_waves - 1) * MB * 4 * 64 + (SCALED ? n_waves * MB * 16 : 0)) * sizeof(float);
  dim3 grid((n_tiles + tiles - 1) / tiles, parts);
  gemm_resident_kernel<MB, XQ, EPI, TO, SCALED>
      <<<grid, n_waves * 64, lds, s>>>(x.x, w, (TO*)c, m, n, k, tiles, fold_args(x, after));
  return 0;
}

// true if the resident kernel takes these sizes
template <int EPI, typename TO, bool SCALED>
static bool try_resident(const GemmTokens& x, const bf16_t* w, void* c, const GemmAfter& after, int m, int n, int k,
                         int parts, hipStream_t s, int* rc) {
  constexpr bool FOLDS = SCALED || EPI >= 2;      // compiled for up to 16 tokens and all of K in one workgroup
  const int mb = (m + 15) / 16;
  const int xq = mb == 1 ? 16 : (mb == 2 ? 8 : 4);
  if (k % (32 * xq) != 0) return false;
  const int slices = k / (32 * xq);
  if (parts < 1 || slices % parts != 0) return false;
  const int n_waves = slices / parts;
  if (n_waves > 8) return false;
  // With fewer than 7 waves a workgroup has too few loads in flight for the one compute unit it has to
  // itself, and the skinny kernel, several workgroups to a compute unit, is faster (32,768 gated rows at
  // K = 2048: 12.4 us against 13.8 with 4 waves; at K = 3072: 17.3 against 18.4 with 6); forced on
  // (rb_tune_use_resident(2)) it still takes them.
  if (n_waves < 7 && g_res_forced == 0) return false;
  if (EPI == 1 && (n % 32 != 0)) return false;
  if (FOLDS && (mb != 1 || parts != 1)) return false;
  if (mb == 1) {
    *rc = launch_resident<1, 16, EPI, TO, SCALED>(x, w, c, after, m, n, k, parts, s);
    return true;
  }
  if constexpr (!FOLDS) {
    if (mb == 2) *rc = launch_resident<2, 8, EPI, TO, false>(x, w, c, after, m, n, k, parts, s);
    else if (mb == 3) *rc = launch_resident<3, 4, EPI, TO, false>(x, w, c, after, m, n, k, parts, s);
    else *rc = launch_resident<4, 4, EPI, TO, false>(x, w, c, after, m, n, k, parts, s);
    return true;
  }
  return false;
}


// One instance per (epilogue, output type, kind of tokens).  Epilogues 2 and 3 are float32 and
// take plain tokens; prepared tokens go with epilogues 0 and 1.
#define RB_PLAIN(FN, ...)                                                                                  \
  (after.epilogue == 3 ? FN<3, float, false>(__VA_ARGS__)                                                  \
   : after.epilogue == 2 ? FN<2, float, false>(__VA_ARGS__)                                                \
   : after.epilogue == 0 ? (dtype_out == RB_F32 ? FN<0, float, false>(__VA_ARGS__) : FN<0, bf16_t, false>(__VA_ARGS__)) \
                         : (dtype_out == RB_F32 ? FN<1, float, false>(__VA_ARGS__) : FN<1, bf16_t, false>(__VA_ARGS__)))
#define RB_SCALED(FN, ...)                                                                                 \
  (after.epilogue == 0 ? (dtype_out == RB_F32 ? FN<0, float, true>(__VA_ARGS__) : FN<0, bf16_t, true>(__VA_ARGS__)) \
                       : (dtype_out == RB_F32 ? FN<1, float, true>(__VA_ARGS__) : FN<1, bf16_t, true>(__VA_ARGS__)))

int gemm_skinny_launch(const GemmTokens& x, const bf16_t* w, void* c, int dtype_out, const GemmAfter& after, int m,
                       int n, int k, hipStream_t s) {
  if (x.squares) {
    RB_REQUIRE(after.epilogue <= 1, "rb_gemm_bf16: prepared rows go with epilogues 0 and 1, not %d", after.epilogue);
    return RB_SCALED(dispatch_skinny, x, w, c, after, m, n, k, s);
  }
  return RB_PLAIN(dispatch_skinny, x, w, c, after, m, n, k, s);
}

bool gemm_resident_try(const GemmTokens& x, const bf16_t* w, void* c, int dtype_out, const GemmAfter& after, int m,
                       int n, int k, hipStream_t s, int* rc) {
  if (x.squares) {
    if (after.epilogue > 1) return false;
    return RB_SCALED(try_resident, x, w, c, after, m, n, k, 1, s, rc);
  }
  return RB_PLAIN(try_resident, x, w, c, after, m, n, k, 1, s, rc);
}
