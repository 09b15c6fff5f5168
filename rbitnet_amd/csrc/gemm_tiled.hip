// Products with many tokens (prefill) and with 17..64 tokens: tiles of W and of the tokens
// through LDS, MFMA 32x32x16 bf16, float32 accumulation.  The tokens are the row operand of the
// MFMA and W's rows its columns, so that the lanes of a wave hold consecutive outputs of a token.
//
// Epilogue 1 expects W with gate and up rows interleaved in blocks of 16 and writes
// silu(gate) * up (llama/model.rs:297-302 of the reference) instead of the two products.
//
// Reference loop: y[o] = sum_i W[i + o * n_in] * x[i]  (llama/model.rs:67-91).
#include <type_traits>

#include "api.h"
#include "tune.h"
#include "gemm_internal.h"

// Adds up the [M, N] slabs of partial sums that the K slices of a product wrote, in slice
// order (the same order whatever else runs), and converts to the output type.
template <typename TO>
__global__ void gemm_sum_slabs_kernel(const float* __restrict__ slabs, TO* __restrict__ c, int parts, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = 0.f;
  for (int p = 0; p < parts; ++p) v += slabs[(size_t)p * count + i];
  Num<TO>::store(c + i, v);
}

// Which tile a workgroup computes.  Workgroup ids go round robin over the 8 XCDs, each with
// an L2 of its own: every XCD gets a contiguous range of the tile order, and the order runs
// through groups of TG_GROUP_M token tiles, all row tiles of a group before the next group.  The
// 32 workgroups that an XCD runs at a time then cover about 8 x 4 tiles and walk K together,
// so 12 tile rows come from beyond L2 per step for 32 tiles' worth of products.
#define TG_GROUP_M 8
__device__ __forceinline__ bool tile_of_workgroup(int m_tiles, int n_tiles, int* mt, int* nt) {
  const int tiles = m_tiles * n_tiles;
  const int per_xcd = (tiles + 7) / 8;
  const int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (t >= tiles) return false;
  const int in_group = TG_GROUP_M * n_tiles;
  const int first_m = t / in_group * TG_GROUP_M;
  const int rows = min(m_tiles - first_m, TG_GROUP_M);
  const int r = t % in_group;
  *mt = first_m + r % rows;
  *nt = r / rows;
  return true;
}

// What a lane holds of a 32 x 32 piece when the tokens were the MFMA's rows and W's rows its
// columns: W row first_row + l32 for the 16 tokens mbase + 8 (e / 4) + e % 4 (mbase includes the
// lane's 4 g).  A wave's store then covers 32 consecutive outputs of each of two tokens.  With
// `slab`, the sums go to that slice's [M, N] slab instead, to be added up later in a fixed order.
template <int EPI, typename TO>
__device__ __forceinline__ void store_piece(const f32x16_t& acc, TO* __restrict__ c, float* __restrict__ slab,
                                            int first_row, int l32, int mbase, int m, int n) {
  if (EPI == 0) {
    const int nn = first_row + l32;
    if (nn >= n) return;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int mm = mbase + 8 * (e / 4) + (e % 4);
      if (mm >= m) continue;
      if (slab) slab[(size_t)mm * n + nn] = acc[e];
      else Num<TO>::store(c + (size_t)mm * n + nn, acc[e]);
    }
  } else {
    // gate rows in lanes 0..15 of a half wave, up rows in lanes 16..31: the two halves swap what
    // the other needs, the lower one finishing the even tokens and the upper one the odd ones
    const int half_n = n / 2;
    const bool upper = (l32 & 16) != 0;
    const int col = first_row / 2 + (l32 & 15);
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
      const float mine = upper ? acc[e + 1] : acc[e];
      const float give = upper ? acc[e] : acc[e + 1];
      const float got = __shfl_xor(give, 16);
      const int mm = mbase + 8 * (e / 4) + (e % 4) + (upper ? 1 : 0);
      const float gate = upper ? got : mine, up = upper ? mine : got;
      if (mm < m && col < half_n) Num<TO>::store(c + (size_t)mm * half_n + col, silu_f32(gate) * up);
    }
  }
}

#define TG_BK 64
#define TG_LD 72          // bf16 elements per LDS row: 64 + 8 of padding, so that the 16 lanes
                          // of a quarter wave read 16 different 16-byte bank groups

template <int BN, int BM, int WN, int WM, int P, int EPI, bool KTAIL, typename TO>
__global__ __launch_bounds__(64 * (BN / WN) * (BM / WM)) void gemm_tiled_kernel(const bf16_t* __restrict__ x,
                                                         const bf16_t* __restrict__ w, TO* __restrict__ c,
                                                         int m, int n, int k, int m_tiles, int n_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int TN = WN / 32, TM = WM / 32;
  constexpr int WAVES_N = BN / WN;
  constexpr int NT = 64 * (BN / WN) * (BM / WM);      // threads: one wave per WN x WM piece of the tile
  constexpr int W_CHUNKS = BN * 8 / NT, X_CHUNKS = BM * 8 / NT;
  static_assert(BN * 8 % NT == 0 && BM * 8 % NT == 0 && NT % 8 == 0, "tile does not divide among the threads");
  bf16_t* ws = reinterpret_cast<bf16_t*>(smem);                      // [2][BN][TG_LD]
  bf16_t* xs = ws + 2 * BN * TG_LD;                                  // [2][BM][TG_LD]

  int mt, nt;
  if (!tile_of_workgroup(m_tiles, n_tiles, &mt, &nt)) return;
  const int m0 = mt * BM;
  const int n0 = nt * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wn0 = (wave % WAVES_N) * WN;
  const int wm0 = (wave / WAVES_N) * WM;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // ---- pipeline: tile kt is multiplied out of LDS while tiles kt + 1 .. kt + P - 1 are on
  // their way from memory in registers (P - 1 tiles of latency hidden) and one of them is
  // moved into the other LDS buffer.  Loads carry no conditions: rows beyond N or M are read
  // from the last row and never stored, chunks beyond K are read from the last chunk and
  // zeroed on their way into LDS.  (With conditions the compiler cannot count outstanding
  // loads and waits for all of them.)
  uint4 wreg[P][W_CHUNKS], xreg[P][X_CHUNKS];
  // addresses: a 64-bit base per tile (the same for the whole workgroup) plus a 32-bit
  // element offset per chunk; a tile spans at most 256 rows, so the offsets fit
  const bf16_t* wtile = w + (size_t)n0 * k;
  const bf16_t* xtile = x + (size_t)m0 * k;
  uint32_t woff[W_CHUNKS], xoff[X_CHUNKS];
#pragma unroll
  for (int i = 0; i < W_CHUNKS; ++i) {
    int row = (tid + NT * i) / 8;
    if (n0 + row > n - 1) row = n - 1 - n0;
    woff[i] = (uint32_t)row * (uint32_t)k;
  }
#pragma unroll
  for (int i = 0; i < X_CHUNKS; ++i) {
    int row = (tid + NT * i) / 8;
    if (m0 + row > m - 1) row = m - 1 - m0;
    xoff[i] = (uint32_t)row * (uint32_t)k;
  }
  const int kc = (tid % 8) * 8;             // this thread's chunk offset inside a tile (the same for all i)
  auto load_global = [&](int slot, int kt) {
    int col = kt * TG_BK + kc;
    if (col > k - 8) col = k - 8;           // beyond K: any valid address; the data is zeroed in store_lds
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) wreg[slot][i] = load16(wtile + (woff[i] + (uint32_t)col));
#pragma unroll
    for (int i = 0; i < X_CHUNKS; ++i) xreg[slot][i] = load16(xtile + (xoff[i] + (uint32_t)col));
  };
  auto store_lds = [&](int slot, int kt) {
    const int buf = kt & 1;
    const bool in = !KTAIL || kt * TG_BK + kc < k;
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int q = tid + NT * i;
      *reinterpret_cast<uint4*>(ws + ((size_t)buf * BN + q / 8) * TG_LD + kc) = in ? wreg[slot][i] : zero16();
    }
#pragma unroll
    for (int i = 0; i < X_CHUNKS; ++i) {
      const int q = tid + NT * i;
      *reinterpret_cast<uint4*>(xs + ((size_t)buf * BM + q / 8) * TG_LD + kc) = in ? xreg[slot][i] : zero16();
    }
  };
  auto multiply = [&](int kt) {
    const bf16_t* wb = ws + (size_t)(kt & 1) * BN * TG_LD;
    const bf16_t* xb = xs + (size_t)(kt & 1) * BM * TG_LD;
    if (NT <= 256) {
      // fragments of k-step ks + 1 are requested from LDS before the MFMAs of k-step ks
      Frag8 a[2][TN], b[2][TM];
      auto load_frags = [&](int buf2, int ks) {
#pragma unroll
        for (int i = 0; i < TN; ++i)
          a[buf2][i].u = *reinterpret_cast<const uint4*>(wb + (size_t)(wn0 + 32 * i + l32) * TG_LD + ks * 16 + g * 8);
#pragma unroll
        for (int j = 0; j < TM; ++j)
          b[buf2][j].u = *reinterpret_cast<const uint4*>(xb + (size_t)(wm0 + 32 * j + l32) * TG_LD + ks * 16 + g * 8);
      };
      load_frags(0, 0);
#pragma unroll
      for (int ks = 0; ks < TG_BK / 16; ++ks) {
        if (ks + 1 < TG_BK / 16) load_frags((ks + 1) & 1, ks + 1);
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
          for (int j = 0; j < TM; ++j) acc[i][j] = mfma32(b[ks & 1][j], a[ks & 1][i], acc[i][j]);
      }
    } else {
      // 8 waves: two per SIMD cover each other's LDS latency, and registers are scarce
#pragma unroll
      for (int ks = 0; ks < TG_BK / 16; ++ks) {
        Frag8 a[TN], b[TM];
#pragma unroll
        for (int i = 0; i < TN; ++i)
          a[i].u = *reinterpret_cast<const uint4*>(wb + (size_t)(wn0 + 32 * i + l32) * TG_LD + ks * 16 + g * 8);
#pragma unroll
        for (int j = 0; j < TM; ++j)
          b[j].u = *reinterpret_cast<const uint4*>(xb + (size_t)(wm0 + 32 * j + l32) * TG_LD + ks * 16 + g * 8);
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
          for (int j = 0; j < TM; ++j) acc[i][j] = mfma32(b[j], a[i], acc[i][j]);
      }
    }
  };

  const int k_tiles = (k + TG_BK - 1) / TG_BK;
  // tiles beyond the last are loaded as well (clamped) and never stored: the loop body stays
  // free of conditions on loads
#pragma unroll
  for (int sl = 0; sl < P; ++sl) load_global(sl, sl);
  store_lds(0, 0);
  __syncthreads();
  int kt = 0;
  for (; kt + P <= k_tiles; kt += P) {        // P iterations per trip, so that the register slots are static
#pragma unroll
    for (int u = 0; u < P; ++u) {
      // slot u held tile kt + u (now in LDS): reuse it for tile kt + u + P
      load_global(u, kt + u + P);
      multiply(kt + u);
      if (kt + u + 1 < k_tiles) store_lds((u + 1) % P, kt + u + 1);
      __syncthreads();
    }
  }
#pragma unroll
  for (int u = 0; u < P; ++u) {               // the last k_tiles % P tiles
    if (kt + u < k_tiles) {
      multiply(kt + u);
      if (kt + u + 1 < k_tiles) store_lds((u + 1) % P, kt + u + 1);
      __syncthreads();
    }
  }

  // ---- lane holds, per (i, j): W row n0 + wn0 + 32 i + l32, tokens base + 8 (e / 4) + 4 g + e % 4
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
      store_piece<EPI, TO>(acc[i][j], c, nullptr, n0 + wn0 + 32 * i, l32, m0 + wm0 + 32 * j + 4 * g, m, n);
}

// ---------------------------------------------------------------------------------------
// The same product with the tiles brought from memory straight into LDS
// (global_load_lds_dwordx4: no registers, no LDS store instruction), S stages deep.
//
// A wave's load instruction fills 1 KB of LDS in lane order, so rows cannot be padded.  Rows
// of BK elements are kept dense and the 16-byte chunks of a row are permuted instead: chunk c
// of row r lies in slot c ^ swz(r), swz(r) = (r / rows per 256 bytes) % chunks per row.  The
// permutation is applied on the memory side (which chunk a lane fetches), and the 16 lanes of
// a quarter wave that read one chunk column of 16 rows then hit 16 different bank groups.
//
// The loads are inline assembly, so the compiler neither counts nor waits for them: the
// kernel waits itself (s_waitcnt vmcnt) for the stage it is about to read, leaving the
// younger stages in flight.  There is no other memory access in the main loop.
template <int BN, int BM, int WN, int WM, int BK, int S, int EPI, typename TO, bool WF>
__global__ __launch_bounds__(64 * (BN / WN) * (BM / WM)) void gemm_dma_kernel(const bf16_t* __restrict__ x,
                                                       const bf16_t* __restrict__ w, TO* __restrict__ c,
                                                       float* __restrict__ slabs, int m, int n, int k, int m_tiles,
                                                       int n_tiles, int k_tiles) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr int TN = WN / 32, TM = WM / 32;
  constexpr int WAVES_N = BN / WN;
  constexpr int NWAVES = (BN / WN) * (BM / WM);
  constexpr int CPR = BK / 8;                   // 16-byte chunks per row
  constexpr int RPW = 64 / CPR;                 // rows one wave-wide load covers
  constexpr int RPB = 128 / BK;                 // rows per 256 bytes of LDS
  constexpr int W_LOADS = BN / RPW / NWAVES, X_LOADS = BM / RPW / NWAVES;
  constexpr int LOADS = W_LOADS + X_LOADS;      // per thread and stage
  constexpr int STAGE = (BN + BM) * BK;         // elements
  static_assert(BN % (RPW * NWAVES) == 0 && BM % (RPW * NWAVES) == 0, "tile does not divide among the waves");
  static_assert(WN % 32 == 0 && WM % 32 == 0 && BN % WN == 0 && BM % WM == 0, "wave tiles are made of 32 x 32 pieces");
  static_assert(S >= 2 && LOADS * (S - 1) < 64, "too many loads in flight for the counter");
  bf16_t* lds = reinterpret_cast<bf16_t*>(smem);

  int mt, nt;
  if (!tile_of_workgroup(m_tiles, n_tiles, &mt, &nt)) return;
  const int m0 = mt * BM;
  const int n0 = nt * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn0 = (wave % WAVES_N) * WN;
  const int wm0 = (wave / WAVES_N) * WM;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // ---- what this lane fetches: wave-wide load q covers rows q * RPW .. + RPW - 1 of a tile
  const bf16_t* wtile = w + (size_t)n0 * k;
  const bf16_t* xtile = x + (size_t)m0 * k;
  uint32_t woff[W_LOADS], xoff[X_LOADS];        // byte offsets from the tile's first element, without the k-tile
#pragma unroll
  for (int i = 0; i < W_LOADS; ++i) {
    if (WF) {
      // W fragment-major: wave-wide load q fetches one block of 16 rows x 32 depth values, 1 KB in
      // a row, and the stage holds the tile's blocks in the order [BN / 16][BK / 32]
      const int q = wave + NWAVES * i;
      int rt = q / (BK / 32);
      const int kb = q % (BK / 32);
      if (n0 + 16 * rt >= n) rt = 0;            // rows beyond N: any valid tile, never stored
      woff[i] = ((uint32_t)(16 * rt) * (uint32_t)k + (uint32_t)kb * 512u + (uint32_t)lane * 8u) * 2u;
    } else {
      const int row = (wave + NWAVES * i) * RPW + lane / CPR;
      const int chunk = (lane % CPR) ^ ((row / RPB) % CPR);
      int grow = row;
      if (n0 + grow > n - 1) grow = n - 1 - n0;   // rows beyond N: any valid row, never stored
      woff[i] = ((uint32_t)grow * (uint32_t)k + chunk * 8) * 2u;
    }
  }
#pragma unroll
  for (int i = 0; i < X_LOADS; ++i) {
    const int row = (wave + NWAVES * i) * RPW + lane / CPR;
    const int chunk = (lane % CPR) ^ ((row / RPB) % CPR);
    int grow = row;
    if (m0 + grow > m - 1) grow = m - 1 - m0;
    xoff[i] = ((uint32_t)grow * (uint32_t)k + chunk * 8) * 2u;
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;      // LDS byte address of stage 0
  const int kt0 = blockIdx.y * k_tiles;                    // this workgroup's slice of K: k_tiles tiles from here
  // a K tile further on: BK values along a row, or BK / 32 blocks of 1 KB (fragment-major)
  constexpr uint32_t W_KSTEP = WF ? BK * 32 : BK * 2;
  // With one tile of tokens every workgroup reads rows of W that nobody else reads, once: whole
  // lines (fragment-major) past the caches, as the products of few tokens do.  Only where a
  // workgroup's walk along K is long: the short walks of a product cut into many K slices are
  // bound by their first loads, which come sooner through the caches (64 tokens: 28,672 gated rows
  // 51 -> 43 us with such loads, but 4,096 rows in 8 slices of 8 tiles 15 -> 16.6 us).
  // The main loop is compiled for either kind of load (as a run-time choice it stood as eight branches
  // between the MFMAs of a K tile and cost 1.6 % of a long prefill).
  const bool w_once = WF && m_tiles == 1 && k_tiles >= 24;
  auto issue = [&](auto once, int kt) {
    const uint32_t stage = lds_base + (uint32_t)(kt % S) * (STAGE * 2);
    const uint32_t kbytes = (uint32_t)(kt0 + kt) * (BK * 2);
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      if constexpr (decltype(once)::value)
        load_to_lds16_stream(wtile, woff[i] + (uint32_t)(kt0 + kt) * W_KSTEP,
                             stage + (uint32_t)(wave + NWAVES * i) * 1024u);
      else
        load_to_lds16(wtile, woff[i] + (uint32_t)(kt0 + kt) * W_KSTEP, stage + (uint32_t)(wave + NWAVES * i) * 1024u);
    }
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i)
      load_to_lds16(xtile, xoff[i] + kbytes, stage + (uint32_t)(BN * BK * 2) + (uint32_t)(wave + NWAVES * i) * 1024u);
  };

  // ---- fragments: row base + 32 i + l32, chunk 2 ks + g, found in slot chunk ^ swz(l32)
  constexpr int KSTEPS = BK / 16;
  static_assert(KSTEPS % 2 == 0, "the fragment buffers alternate by depth step");
  const int sw = (l32 / RPB) % CPR;
  // W's fragments.  Rows: row wn0 + 32 i + l32, chunk 2 ks + g in slot chunk ^ sw.  Fragment-major:
  // block [(wn0 + 32 i + l32) / 16][chunk / 4], inside it 16 bytes at 16 ((chunk % 4) * 16 + l32 % 16);
  // the 16 lanes that are served together read 256 bytes in a row.
  const bf16_t* wfrag = WF ? lds + ((size_t)((wn0 + l32) / 16) * (BK / 32) * 64 + (l32 % 16)) * 8
                           : lds + (size_t)(wn0 + l32) * BK;
  constexpr int W_ISTEP = WF ? 2 * (BK / 32) * 512 : 32 * BK;       // 32 rows further on
  auto w_slot = [&](int ks) { return WF ? (((2 * ks + g) / 4) * 64 + ((2 * ks + g) % 4) * 16) * 8 : ((2 * ks + g) ^ sw) * 8; };
  const bf16_t* xfrag = lds + (size_t)BN * BK + (size_t)(wm0 + l32) * BK;
  Frag8 a[2][TN], b[2][TM];
  auto load_frags = [&](int buf2, int kt, int ks) {
    const bf16_t* wb = wfrag + (size_t)(kt % S) * STAGE;
    const bf16_t* xb = xfrag + (size_t)(kt % S) * STAGE;
    const int slot = ((2 * ks + g) ^ sw) * 8;
    const int wslot = w_slot(ks);
#pragma unroll
    for (int i = 0; i < TN; ++i) a[buf2][i].u = *reinterpret_cast<const uint4*>(wb + i * W_ISTEP + wslot);
#pragma unroll
    for (int j = 0; j < TM; ++j) b[buf2][j].u = *reinterpret_cast<const uint4*>(xb + 32 * j * BK + slot);
  };
  // the tokens are the MFMA's rows and W's rows its columns: a lane then holds one column of W's
  // rows for 16 tokens, and a wave's store covers 32 consecutive outputs of a token
  auto mfmas = [&](int buf2) {
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j) acc[i][j] = mfma32(b[buf2][j], a[buf2][i], acc[i][j]);
  };

  // ---- main loop.  The barrier that hands over tile kt + 1 stands before the last depth step
  // of tile kt, whose fragments are in registers by then: its MFMAs run while the first
  // fragments of tile kt + 1 come from LDS and while the other waves arrive, and the stage of
  // tile kt is free for tile kt + S from there on.
  // One load of tile kt (number l of the LOADS a wave has), one fragment of a depth step.
  auto issue_one = [&](auto once, int kt, int l) {
    const uint32_t stage = lds_base + (uint32_t)(kt % S) * (STAGE * 2);
    const uint32_t kbytes = (uint32_t)(kt0 + kt) * (BK * 2);
    if (l < W_LOADS) {
      if constexpr (decltype(once)::value)
        load_to_lds16_stream(wtile, woff[l] + (uint32_t)(kt0 + kt) * W_KSTEP,
                             stage + (uint32_t)(wave + NWAVES * l) * 1024u);
      else
        load_to_lds16(wtile, woff[l] + (uint32_t)(kt0 + kt) * W_KSTEP, stage + (uint32_t)(wave + NWAVES * l) * 1024u);
    }
    else
      load_to_lds16(xtile, xoff[l - W_LOADS] + kbytes,
                    stage + (uint32_t)(BN * BK * 2) + (uint32_t)(wave + NWAVES * (l - W_LOADS)) * 1024u);
  };
  // Fragment number f of a depth step, in the order in which the MFMAs first need them:
  // W's first, all of the tokens', the rest of W's.
  auto frag_one = [&](int buf2, int kt, int ks, int f) {
    const int slot = ((2 * ks + g) ^ sw) * 8;
    if (f == 0 || f > TM) {
      const int i = f == 0 ? 0 : f - TM;
      a[buf2][i].u = *reinterpret_cast<const uint4*>(wfrag + (size_t)(kt % S) * STAGE + i * W_ISTEP + w_slot(ks));
    } else {
      b[buf2][f - 1].u = *reinterpret_cast<const uint4*>(xfrag + (size_t)(kt % S) * STAGE + 32 * (f - 1) * BK + slot);
    }
  };
  // A depth step but the last of tile kt: its MFMAs, with the next step's fragments asked for
  // between them, one after each MFMA, so that a wave keeps the matrix core fed by itself (with
  // all the reads in a run before the MFMAs, a wave took 27-30 ns per MFMA where the core takes 16-20,
  // and the two waves of a SIMD, which the barrier keeps in step, did not cover each other).
  constexpr int NM = TN * TM, LASTBUF = (KSTEPS - 1) & 1;
  auto steps_but_last = [&](int kt) {
#pragma unroll
    for (int ks = 0; ks + 1 < KSTEPS; ++ks) {
#pragma unroll
      for (int q = 0; q < NM; ++q) {
        acc[q / TM][q % TM] = mfma32(b[ks & 1][q % TM], a[ks & 1][q / TM], acc[q / TM][q % TM]);
#pragma unroll
        for (int f = q; f < TN + TM; f += NM) frag_one((ks + 1) & 1, kt, ks + 1, f);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // The last depth step of tile kt, behind the barrier: between its MFMAs, one at a time, go the
  // loads of tile kt + S and the first fragments of tile kt + 1, so that the matrix core never
  // waits for a run of other instructions (both waves of a SIMD leave the barrier together, and
  // neither covers the other's).
  auto last_step = [&](auto once, int kt, bool fetch) {
#pragma unroll
    for (int q = 0; q < NM; ++q) {
      acc[q / TM][q % TM] = mfma32(b[LASTBUF][q % TM], a[LASTBUF][q / TM], acc[q / TM][q % TM]);
      if (fetch) {
#pragma unroll
        for (int l = q; l < LOADS; l += NM) issue_one(once, kt + S, l);
      }
#pragma unroll
      for (int f = q; f < TN + TM; f += NM) frag_one(0, kt + 1, 0, f);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto hand_over = [&](int kt) {
    // tile kt + 1 must have landed; in the steady state the S - 2 tiles after it stay in flight
    if (S == 2 || kt + S - 1 >= k_tiles) wait_vm<0>();
    else wait_vm<LOADS * (S - 2)>();
    // the last fragments of tile kt are in registers before anyone may overwrite its stage
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();                  // everyone's part of tile kt + 1 is in LDS, and nobody reads tile kt's stage any more
    __builtin_amdgcn_sched_barrier(0);
  };
  auto run = [&](auto once) {
#pragma unroll
    for (int s = 0; s < S; ++s)
      if (s < k_tiles) issue(once, s);
    if (S - 1 < k_tiles) wait_vm<LOADS * (S - 1)>();
    else wait_vm<0>();
    __syncthreads();
    load_frags(0, 0, 0);
    int kt = 0;
    for (; kt + S < k_tiles; ++kt) {
      steps_but_last(kt);
      hand_over(kt);
      last_step(once, kt, true);
    }
    for (; kt + 1 < k_tiles; ++kt) {
      steps_but_last(kt);
      hand_over(kt);
      last_step(once, kt, false);
    }
    steps_but_last(k_tiles - 1);
    mfmas(LASTBUF);
  };
  if (w_once) run(std::true_type{});
  else run(std::false_type{});

  // ---- lane holds, per (i, j): W row n0 + wn0 + 32 i + l32, tokens base + 8 (e / 4) + 4 g + e % 4
  if constexpr (EPI == 1 && sizeof(TO) == 2) {
    // The gated outputs of a piece are 16 columns wide: stored from the registers, a wave's store
    // would write 32 bytes of each of four tokens, and the tile's 80 such stores a lane took 27-35 us
    // of a 320 x 256 tile's 150.  They go through LDS instead (the tiles are done with) and leave
    // as whole rows of the tile, 16 bytes a lane.
    constexpr int HC = BN / 2;              // output columns of the tile
    constexpr int LD = HC + 8;              // 16 bytes of padding: the four tokens of a store hit different banks
    constexpr int CH = HC / 8;              // 16-byte chunks of a row
    static_assert((size_t)BM * LD <= (size_t)S * STAGE, "the tile's outputs do not fit the stages");
    const int half_n = n / 2;
    __syncthreads();                        // everyone has read its last fragments
    const bool upper = (l32 & 16) != 0;
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        // gate rows in lanes 0..15 of a half wave, up rows in lanes 16..31: the two halves swap what
        // the other needs, the lower one finishing the even tokens and the upper one the odd ones
        bf16_t* dst = lds + (size_t)(wm0 + 32 * j + 4 * g + (upper ? 1 : 0)) * LD + (wn0 + 32 * i) / 2 + (l32 & 15);
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
          const float mine = upper ? acc[i][j][e + 1] : acc[i][j][e];
          const float give = upper ? acc[i][j][e] : acc[i][j][e + 1];
          const float got = __shfl_xor(give, 16);
          const float gate = upper ? got : mine, up = upper ? mine : got;
          dst[(size_t)(8 * (e / 4) + (e % 4)) * LD] = f32_to_bf16(silu_f32(gate) * up);
        }
      }
    __syncthreads();
    const bool wide = (reinterpret_cast<uintptr_t>(c) & 15) == 0 && half_n % 8 == 0;
    for (int q = tid; q < BM * CH; q += 64 * NWAVES) {
      const int row = q / CH, ch = q - row * CH;
      const int mm = m0 + row, col = n0 / 2 + ch * 8;
      if (mm >= m || col >= half_n) continue;
      const bf16_t* src = lds + (size_t)row * LD + ch * 8;
      bf16_t* out = reinterpret_cast<bf16_t*>(c) + (size_t)mm * half_n + col;
      if (wide && col + 8 <= half_n) {
        *reinterpret_cast<uint4*>(out) = *reinterpret_cast<const uint4*>(src);
      } else {
        for (int u = 0; u < 8 && col + u < half_n; ++u) out[u] = src[u];
      }
    }
    return;
  }
  float* slab = slabs ? slabs + (size_t)blockIdx.y * m * n : nullptr;      // this slice of K's partial sums
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
      store_piece<EPI, TO>(acc[i][j], c, slab, n0 + wn0 + 32 * i, l32, m0 + wm0 + 32 * j + 4 * g, m, n);
}

template <int BN, int BM, int WN, int WM, int BK, int S, int EPI, typename TO, bool WF>
static int launch_dma_cfg(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, hipStream_t s,
                          int parts = 1, float* slabs = nullptr) {
  const int m_tiles = (m + BM - 1) / BM, n_tiles = (n + BN - 1) / BN;
  RB_REQUIRE(parts >= 1 && (k / BK) % parts == 0 && (parts == 1 || (slabs && EPI == 0)),
             "rb_gemm_bf16: internal: bad K split %d", parts);
  const long long tiles = (long long)m_tiles * n_tiles;
  RB_REQUIRE(tiles < (1LL << 30), "rb_gemm_bf16: too many tiles");
  RB_REQUIRE(k % BK == 0, "rb_gemm_bf16: the direct-to-LDS kernel needs K=%d to be a multiple of %d", k, BK);
  // byte offsets inside a tile are 32-bit
  RB_REQUIRE((long long)(BN > BM ? BN : BM) * k * 2 < (1LL << 32), "rb_gemm_bf16: K=%d too long for this kernel", k);
  const size_t lds = (size_t)S * (BN + BM) * BK * sizeof(bf16_t);
  RB_REQUIRE(!WF || (BN % 32 == 0 && n % 16 == 0), "rb_gemm_bf16: fragment-major W needs N=%d to be a multiple of 16", n);
  auto kern = gemm_dma_kernel<BN, BM, WN, WM, BK, S, EPI, TO, WF>;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    RB_REQUIRE(e == hipSuccess, "rb_gemm_bf16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    configured = true;
  }
  const dim3 grid((unsigned)((tiles + 7) / 8 * 8), (unsigned)parts);
  kern<<<grid, 64 * (BN / WN) * (BM / WM), lds, s>>>(x, w, (TO*)c, parts > 1 ? slabs : nullptr, m, n, k, m_tiles,
                                                      n_tiles, k / BK / parts);
  if (parts > 1 && c != nullptr) {      // without c the caller adds the slabs up itself
    const size_t count = (size_t)m * n;
    gemm_sum_slabs_kernel<TO><<<(unsigned)((count + 255) / 256), 256, 0, s>>>(slabs, (TO*)c, parts, count);
  }
  return 0;
}


template <int BN, int BM, int WN, int WM, int P, int EPI, typename TO>
static int launch_tiled_cfg(const bf16_t* x, const bf16_t* w, void* c, int m, int n, int k, hipStream_t s) {
  const int m_tiles = (m + BM - 1) / BM, n_tiles = (n + BN - 1) / BN;
  const long long tiles = (long long)m_tiles * n_tiles;
  RB_REQUIRE(tiles < (1LL << 30), "rb_gemm_bf16: too many tiles");
  const size_t lds = (size_t)2 * (BN + BM) * TG_LD * sizeof(bf16_t);
  const bool tail = k % TG_BK != 0;
  auto kern = tail ? gemm_tiled_kernel<BN, BM, WN, WM, P, EPI, true, TO>
                   : gemm_tiled_kernel<BN, BM, WN, WM, P, EPI, false, TO>;
  static bool configured[2] = {false, false};
  if (!configured[tail]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    RB_REQUIRE(e == hipSuccess, "rb_gemm_bf16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    configured[tail] = true;
  }
  const int grid = (int)((tiles + 7) / 8 * 8);
  kern<<<grid, 64 * (BN / WN) * (BM / WM), lds, s>>>(x, w, (TO*)c, m, n, k, m_tiles, n_tiles);
  return 0;
}

// ------------------------------------------------------------------ which tiles, how many K slices
// The kernels are bound by what they pull from L2 and LDS (a 128 x 128 x 64 tile needs a byte per
// 64 flop, a 256 x 256 one half of that), so the largest tile that still gives every compute unit
// work wins, and where even the smallest tiles are too few, K is cut into slices over workgroups
// (grid.y): each slice writes its partial sums to its own [M, N] slab of a workspace, and
// gemm_sum_slabs_kernel (or the kernel that reads them) adds them up in a fixed order.
//   cfg 4: 256 rows of W x 256 tokens (8 waves)      cfg 6: 192 x 256      cfg 9: 320 x 256
//   cfg 8: 256 x 128, 3 stages deep                  cfg 5: 128 x 128 (4 waves, 2 workgroups per compute unit)
//   cfg 7: 128 x 64, 3 stages deep (2 per compute unit)      cfg 13: the same with K tiles of 128
//   cfg 10: 64 x 64, 4 stages deep (2 per compute unit)
//   cfg 1..3: tiles staged through registers, for K that is no multiple of 64 (more than 64 tokens)
// Without K slices a product of 128 tokens by 4096 rows ran on 32 of the 256 compute units and
// took as long as one of 768 tokens (K = 14336: 194 us; 41 us with 4 slices of 64-token tiles).
struct TilePlan {
  int cfg;        // 0: not for the kernels of this file
  int parts;      // K slices; more than 1 needs parts * M * N floats of workspace
};

static int g_tile_cfg = 0, g_tile_parts = 0;
extern "C" void rb_tune_tiles(int cfg, int parts) {       // experiments only; 0 = built-in choice
  g_tile_cfg = cfg;
  g_tile_parts = parts;
}

// The choice among the direct-to-LDS tiles and the number of K slices is the least of an estimate
// of every candidate's time, a sum whose terms were fitted to 8,300 measured products: the four
// products of a layer of six model shapes (hidden sizes 2,048 to 8,192) at 24 to 4,096 tokens, every
// tile with 1 to 8 slices forced in turn (`bench.py --planner-sweep` repeats the sweep).
//
//   time [us] = c0 + K tiles of a slice x (what the compute units' tiles cost per K tile)
//               + fixed x (tiles on the busiest compute unit)
//               + slab x (MB of partial sums, when K is cut) + gate x (millions of gated outputs)
//
// A launch of w workgroups fills `slots` places at a time (the compute units, or twice as many for
// the tiles of which two fit on one): w / slots full rounds at `full` each, and a last round of
// rem workgroups.  A last round is cheaper than a full one and the cheaper the emptier (the
// compute units that have work share the memory system with fewer): `last + per_fill x rem / units`,
// and for the tiles that fit twice, once every unit has one, `second + per_second x (rem - units) / units`.
// The machine enters through the number of compute units alone.  The estimate's own choice is
// within 5 % of the best candidate in 258 of the 276 products of more than 64 tokens (0.8 % above
// the best in the mean, 21 % at worst) and in 90 of the 96 of 17 to 64 tokens (0.8 %, 10 %); fitted
// to the token counts that are powers of two alone it does as well on the others.
struct TileCost {
  int cfg, rows, tokens, bk, per_unit;
  float full, last, per_fill, second, per_second, fixed;
};
struct CostTable {
  float c0, slab, gate;
  const TileCost* tiles;
  int n_tiles;
};
static const TileCost kCostMany[] = {
    {4, 256, 256, 64, 1, 1.5794f, 1.1882f, 0.3369f, 0.f, 0.f, 4.5309f},
    {5, 128, 128, 64, 2, 1.0266f, 0.6988f, 0.1646f, 0.8664f, 0.2135f, 1.1148f},
    {6, 192, 256, 64, 1, 1.3217f, 1.0321f, 0.3024f, 0.f, 0.f, 3.2531f},
    {7, 128, 64, 64, 2, 0.6848f, 0.3279f, 0.1067f, 0.5481f, 0.2758f, 0.5548f},
    {8, 256, 128, 64, 1, 0.9282f, 0.7138f, 0.2021f, 0.f, 0.f, 2.674f},
    {9, 320, 256, 64, 1, 1.8295f, 1.3649f, 0.3086f, 0.f, 0.f, 7.2878f},
    {10, 64, 64, 64, 2, 0.4365f, 0.1927f, 0.0777f, 0.3422f, 0.1646f, 0.384f},
    {13, 128, 64, 128, 1, 0.4118f, 0.3109f, 0.1058f, 0.f, 0.f, 1.9912f}};
static const TileCost kCostFew[] = {{7, 128, 64, 64, 2, 1.2099f, 0.3352f, 0.2479f, 0.8967f, 0.3f, -0.4082f},
                                    {10, 64, 64, 64, 2, 0.6268f, 0.191f, 0.1144f, 0.4995f, 0.1176f, -0.1f},
                                    {13, 128, 64, 128, 1, 0.6506f, 0.3182f, 0.2568f, 0.f, 0.f, 0.2565f}};
static const CostTable kMany = {4.469f, 0.3738f, 0.2871f, kCostMany, 8};      // more than 64 tokens
static const CostTable kFew = {5.522f, 0.6852f, 0.f, kCostFew, 3};            // 17 to 64 tokens

static TilePlan plan_by_cost(int m, int n, int k, int epilogue) {
  const CostTable& table = m > 64 ? kMany : kFew;
  const long long units = rb_compute_units();
  const int kt = k / 64;
  TilePlan best = {0, 1};
  double best_cost = 0.0;
  for (int i = 0; i < table.n_tiles; ++i) {
    const TileCost& t = table.tiles[i];
    if (k % t.bk != 0) continue;
    const long long tiles = (long long)((n + t.rows - 1) / t.rows) * ((m + t.tokens - 1) / t.tokens);
    for (int p = 1; p <= (epilogue ? 1 : 8); ++p) {
      if ((k / t.bk) % p != 0 || (p > 1 && kt / p < 4)) continue;
      const long long w = tiles * p, slots = units * t.per_unit;
      const long long rounds = w / slots, rem = w - rounds * slots;
      double per_k = rounds * t.full;
      if (rem > 0 && rem <= units) per_k += t.last + t.per_fill * ((double)rem / units);
      if (rem > units) per_k += t.second + t.per_second * ((double)(rem - units) / units);
      double cost = table.c0 + (double)kt / p * per_k + t.fixed * ((w + units - 1) / units);
      if (p > 1) cost += table.slab * (4e-6 * p * m * n);
      if (epilogue) cost += table.gate * (1e-6 * m * n);
      if (best.cfg == 0 || cost < best_cost) {
        best = {t.cfg, p};
        best_cost = cost;
      }
    }
  }
  return best;
}

static TilePlan plan_tiles(int m, int n, int k, int epilogue) {
  const long long R = rb_compute_units();
  const bool dma = k % 64 == 0 && (long long)k * 512 < (1LL << 32);
  if (!dma) {
    if (m <= 64) return {0, 1};
    const long long t256 = (long long)((m + 255) / 256) * ((n + 255) / 256);
    const long long t256x128 = (long long)((m + 127) / 128) * ((n + 255) / 256);
    if (g_tile_cfg >= 1 && g_tile_cfg <= 3) return {g_tile_cfg, 1};
    return {t256 >= R * 5 / 8 ? 3 : (k >= 8192 && t256x128 >= R * 25 / 32 ? 2 : 1), 1};
  }
  if (m <= 16) return {0, 1};
  if (g_tile_cfg >= 4) {
    const int p = (epilogue == 0 && g_tile_parts > 0 && (k / 64) % g_tile_parts == 0) ? g_tile_parts : 1;
    return {g_tile_cfg, p};
  }
  return plan_by_cost(m, n, k, epilogue);
}

template <int EPI, typename TO, bool WF>
static int launch_planned(const bf16_t* x, const bf16_t* w, void* c, float* workspace, int m, int n, int k,
                          hipStream_t s) {
  const TilePlan plan = plan_tiles(m, n, k, EPI);
  RB_REQUIRE(plan.cfg != 0, "rb_gemm_bf16: internal: M=%d N=%d K=%d is not a product for the tiled kernels", m, n, k);
  RB_REQUIRE(plan.parts == 1 || workspace != nullptr, "rb_gemm_bf16: M=%d N=%d K=%d needs a workspace of %lld floats",
             m, n, k, (long long)plan.parts * m * n);
  const int p = plan.parts;
  switch (plan.cfg) {
    case 8: return launch_dma_cfg<256, 128, 64, 64, 64, 3, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 9: return launch_dma_cfg<320, 256, 160, 64, 64, 2, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 7: return launch_dma_cfg<128, 64, 32, 64, 64, 3, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 10: return launch_dma_cfg<64, 64, 32, 32, 64, 4, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 13: return launch_dma_cfg<128, 64, 32, 64, 128, 3, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 6: return launch_dma_cfg<192, 256, 96, 64, 64, 2, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 5: return launch_dma_cfg<128, 128, 64, 64, 64, 2, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    case 4: return launch_dma_cfg<256, 256, 128, 64, 64, 2, EPI, TO, WF>(x, w, c, m, n, k, s, p, workspace);
    default: break;
  }
  if constexpr (!WF) {
    switch (plan.cfg) {
      case 3: return launch_tiled_cfg<256, 256, 128, 64, 2, EPI, TO>(x, w, c, m, n, k, s);
      case 2: return launch_tiled_cfg<256, 128, 128, 64, 2, EPI, TO>(x, w, c, m, n, k, s);
      default: return launch_tiled_cfg<128, 128, 64, 64, 2, EPI, TO>(x, w, c, m, n, k, s);
    }
  }
  RB_REQUIRE(false, "rb_gemm_bf16: internal: fragment-major W with K=%d, which the direct-to-LDS kernels do not take", k);
  return 1;
}

#define RB_BY_OUTPUT(FN, WF, ...)                                                              \
  (epilogue == 0 ? (dtype_out == RB_F32 ? FN<0, float, WF>(__VA_ARGS__) : FN<0, bf16_t, WF>(__VA_ARGS__)) \
                 : (dtype_out == RB_F32 ? FN<1, float, WF>(__VA_ARGS__) : FN<1, bf16_t, WF>(__VA_ARGS__)))

// what the planner picks for these sizes, as 100 * cfg + parts (0: not a product for this file)
extern "C" int rb_tune_plan(int m, int n, int k, int epilogue) {
  const TilePlan plan = plan_tiles(m, n, k, epilogue);
  return plan.cfg == 0 ? 0 : 100 * plan.cfg + plan.parts;
}

int gemm_tiled_parts(int m, int n, int k, int epilogue) {
  const TilePlan plan = plan_tiles(m, n, k, epilogue);
  return plan.cfg == 0 ? 0 : plan.parts;
}

int gemm_tiled_launch(const bf16_t* x, const bf16_t* w, bool w_frag, void* c, float* workspace, int dtype_out,
                      int epilogue, int m, int n, int k, hipStream_t s) {
  if (w_frag) return RB_BY_OUTPUT(launch_planned, true, x, w, c, workspace, m, n, k, s);
  return RB_BY_OUTPUT(launch_planned, false, x, w, c, workspace, m, n, k, s);
}
