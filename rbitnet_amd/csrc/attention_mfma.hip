// Attention over the paged cache for bfloat16 and head sizes 64 and 128.
//
//  * prefill: causal flash attention on the matrix cores.  A workgroup of 4 waves takes
//    one kv head and 32-query blocks of the query heads that share it; the 64-key page
//    tiles of K and V are staged through LDS once for all of them.  Scores are computed
//    transposed (keys x queries) so that the probabilities come out of the first MFMA in
//    the lane layout the second one wants; V is transposed on its way into LDS.
//  * decode: one query per sequence.  The pages of a sequence are dealt out to n_splits
//    workgroups per kv head, each keeps a running softmax for the query heads of its kv
//    head, and a second kernel combines the splits.
//
// Scores, maxima, exponentials, sums and the output accumulators are float32; the
// probabilities are rounded to bfloat16 for the second MFMA in prefill only.
//
// Reference: s[p] = (q . K[p]) / sqrt(D) for p <= pos, softmax with the maximum
// subtracted, out = sum_p s[p] V[p]; q head qh reads kv head qh / (Hq / Hk)
// (llama/model.rs:260-289, softmax :102-114).
#include <math.h>

#include "api.h"
#include "tune.h"
#include "mfma.h"

#define LOG2E 1.4426950408889634f

// =============================================================================== prefill
template <int D, int NW>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    bf16_t* __restrict__ out, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ past_len,
    const int32_t* __restrict__ block_table, int bt_stride, int n_heads, int n_kv, float scale_log2, int window,
    int gw, int paired) {
  constexpr int KLD = D + 8;          // K tile row: D + 8 elements, rows 16 bytes apart in bank space
  constexpr int VLD = RB_PAGE + 8;    // V^T tile row: 64 keys + 8
  constexpr int DC = D / 8;           // 16-byte chunks per row
  constexpr int NT = 64 * NW;
  constexpr int KCH = RB_PAGE * DC / NT;
  // two tiles of each: the next one is written while the current one is read
  __shared__ __attribute__((aligned(16))) bf16_t ks2[2][RB_PAGE * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t vt2[2][D * VLD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int b = blockIdx.z;
  const int group = n_heads / n_kv;
  const int groups_per_kv = group / gw;
  // Which block of queries and which heads.  The blocks of late queries have the most keys:
  // they are started first (block index 0 is the last block), and the short ones fill the
  // compute units that finish early.  `paired` (the number of compute units, or 0): the workgroups
  // of a sequence, two of which fit a compute unit, are all resident at once (at most two per
  // compute unit); then the first `paired` are the heaviest in falling order and the rest the
  // lightest in rising order, so that the two that share a compute unit have about the same work
  // together everywhere.
  int bx = blockIdx.x, by = blockIdx.y;
  if (paired) {
    const int n = gridDim.x * gridDim.y, at = blockIdx.x + gridDim.x * blockIdx.y;
    const int rank = at < paired ? at : n - 1 - (at - paired);
    by = rank % gridDim.y;
    bx = rank / gridDim.y;
  }
  const int kvh = by / groups_per_kv;
  const int head = kvh * group + (by % groups_per_kv) * gw + (wave % gw);
  const int q_per_wg = 32 * (NW / gw);
  const int seq_start = cu_seqlens[b];
  const int q_len = cu_seqlens[b + 1] - seq_start;
  const int past = past_len[b];
  const int wg_q0 = (gridDim.x - 1 - bx) * q_per_wg;
  if (wg_q0 >= q_len) return;
  const int q0 = wg_q0 + (wave / gw) * 32;
  const bool wave_on = q0 < q_len;
  const int kv_last = past + q_len - 1;                       // last key this sequence holds

  // ---- this lane's query
  int ql = q0 + l32;
  const bool q_ok = ql < q_len;
  if (ql >= q_len) ql = q_len - 1;
  const int qpos = past + ql;
  const int q_lo = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
  Frag8 qf[D / 16];
  {
    const bf16_t* qrow = q + ((size_t)(seq_start + ql) * n_heads + head) * D;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) qf[s].u = load16(qrow + s * 16 + g * 8);
  }

  // ---- key tiles of the workgroup and of this wave
  const int wg_q_end = (wg_q0 + q_per_wg < q_len ? wg_q0 + q_per_wg : q_len) - 1;
  const int wg_min_pos = past + wg_q0;
  const int wg_lo = (window > 0 && wg_min_pos - window + 1 > 0) ? wg_min_pos - window + 1 : 0;
  const int first_tile = wg_lo / RB_PAGE;
  const int last_tile = (past + wg_q_end) / RB_PAGE;
  int wave_first = first_tile, wave_last = -1;
  int wave_min_pos = 0, wave_max_lo = 0;      // a tile all of whose keys lie in [wave_max_lo, wave_min_pos] needs no mask
  if (wave_on) {
    const int w_end = (q0 + 32 < q_len ? q0 + 32 : q_len) - 1;
    wave_last = (past + w_end) / RB_PAGE;
    const int w_min = past + q0;
    wave_first = ((window > 0 && w_min - window + 1 > 0) ? w_min - window + 1 : 0) / RB_PAGE;
    wave_min_pos = w_min;
    wave_max_lo = (window > 0 && past + w_end - window + 1 > 0) ? past + w_end - window + 1 : 0;
  }

  float m_run = -INFINITY, l_run = 0.f;
  f32x16_t oacc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[i][e] = 0.f;

  // ---- staging roles
  // V: a thread takes 4 consecutive keys x 8 consecutive d (one 16-byte chunk of 4 rows)
  const int v_dchunk = (tid & 3) + 4 * (tid >> 6);
  const int v_quad = (tid >> 2) & 15;
  const bool v_on = tid < 256 && v_dchunk < DC;
  // place of the quad in the permuted key order of a V^T row (see the second MFMA below)
  const int qq = v_quad & 7;
  const int v_col = (v_quad >> 3) * 32 + (2 * (qq >> 2) + (qq & 1)) * 8 + ((qq >> 1) & 1) * 4;

  uint4 kreg[KCH], vreg[4];
  auto load_tile = [&](int kt) {
    const int page = block_table[(size_t)b * bt_stride + kt];
    const size_t base = ((size_t)page * n_kv + kvh) * RB_PAGE * D;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + NT * i;
      kreg[i] = load16(k_pages + base + (size_t)(c / DC) * D + (c % DC) * 8);
    }
    if (v_on) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = kt * RB_PAGE + 4 * v_quad + e;
        // keys outside what the sequence holds may be anything, even NaN: make them zero
        vreg[e] = (key <= kv_last && key >= wg_lo) ? load16(v_pages + base + (size_t)(4 * v_quad + e) * D + v_dchunk * 8)
                                                   : zero16();
      }
    }
  };
  auto store_tile = [&](int buf) {
    bf16_t* ks = ks2[buf];
    bf16_t* vt = vt2[buf];
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + NT * i;
      *reinterpret_cast<uint4*>(ks + (c / DC) * KLD + (c % DC) * 8) = kreg[i];
    }
    if (v_on) {
      const uint32_t w0[4] = {vreg[0].x, vreg[1].x, vreg[2].x, vreg[3].x};
      const uint32_t w1[4] = {vreg[0].y, vreg[1].y, vreg[2].y, vreg[3].y};
      const uint32_t w2[4] = {vreg[0].z, vreg[1].z, vreg[2].z, vreg[3].z};
      const uint32_t w3[4] = {vreg[0].w, vreg[1].w, vreg[2].w, vreg[3].w};
      auto put = [&](int i, const uint32_t* w, bool hi) {
        uint2 o;
        if (!hi) {
          o.x = (w[0] & 0xffffu) | (w[1] << 16);
          o.y = (w[2] & 0xffffu) | (w[3] << 16);
        } else {
          o.x = (w[0] >> 16) | (w[1] & 0xffff0000u);
          o.y = (w[2] >> 16) | (w[3] & 0xffff0000u);
        }
        *reinterpret_cast<uint2*>(vt + (v_dchunk * 8 + i) * VLD + v_col) = o;
      };
      put(0, w0, false);
      put(1, w0, true);
      put(2, w1, false);
      put(3, w1, true);
      put(4, w2, false);
      put(5, w2, true);
      put(6, w3, false);
      put(7, w3, true);
    }
  };

  // Tile kt is read from buffer (kt - first_tile) % 2 while tile kt + 1 comes from memory into
  // registers and, after the products, goes into the other buffer: one barrier a tile, behind
  // which everyone has finished reading what the tile after next will overwrite.
  load_tile(first_tile);
  store_tile(0);
  __syncthreads();
  for (int kt = first_tile; kt <= last_tile; ++kt) {
    const int buf = (kt - first_tile) & 1;
    const bf16_t* ks = ks2[buf];
    const bf16_t* vt = vt2[buf];
    const bool next = kt + 1 <= last_tile;
    if (next) load_tile(kt + 1);
    if (wave_on && kt >= wave_first && kt <= wave_last) {

    // ---- S^T = K Q^T: rows keys, columns queries.  The fragments of K come from LDS a few MFMAs
    // ahead of their use, one read behind every MFMA: left to itself the compiler asked for two
    // and waited for them before every second MFMA, and a wave alone on its SIMD took 2.1 us a
    // tile where its 32 MFMAs take 0.55.
    constexpr int AHEAD = 4;                     // fragments on their way
    constexpr int SD = D / 16;                   // depth steps of the scores
    f32x16_t sacc[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) sacc[rt][e] = 0.f;
    Frag8 ring[AHEAD];
    auto k_read = [&](int f) {                   // fragment f: row tile f / SD, depth step f % SD
      ring[f % AHEAD].u = *reinterpret_cast<const uint4*>(ks + ((f / SD) * 32 + l32) * KLD + (f % SD) * 16 + g * 8);
    };
#pragma unroll
    for (int f = 0; f < AHEAD; ++f) k_read(f);
#pragma unroll
    for (int f = 0; f < 2 * SD; ++f) {
      sacc[f / SD] = mfma32(ring[f % AHEAD], qf[f % SD], sacc[f / SD]);
      if (f + AHEAD < 2 * SD) k_read(f + AHEAD);
      __builtin_amdgcn_sched_barrier(0);
    }
    // the first fragments of V^T are asked for now and arrive during the softmax arithmetic:
    // fragment f belongs to step f / VD (row tile and half, see below) and d tile f % VD
    constexpr int VD = D / 32;
    auto v_read = [&](int f) {
      const int q = f / VD, i = f % VD;
      ring[f % AHEAD].u = *reinterpret_cast<const uint4*>(vt + (i * 32 + l32) * VLD + (q / 2) * 32 + (2 * (q % 2) + g) * 8);
    };
#pragma unroll
    for (int f = 0; f < AHEAD; ++f) v_read(f);
    // ---- mask (only tiles that touch the diagonal or the window's edge), running maximum.
    // Scores stay unscaled: the scale is positive, so the maximum can be taken first and the
    // scale folded into the exponent's argument.
    const bool edge = (kt * RB_PAGE + RB_PAGE - 1 > wave_min_pos) || (window > 0 && kt * RB_PAGE < wave_max_lo);
    float mx = -INFINITY;
    if (edge) {
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = kt * RB_PAGE + rt * 32 + 8 * (e / 4) + 4 * g + (e % 4);
          if (key > qpos || key < q_lo) sacc[rt][e] = -INFINITY;
        }
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[rt][e]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale_log2;
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    float lsum = 0.f;
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = __builtin_amdgcn_exp2f(fmaf(sacc[rt][e], scale_log2, -m_safe));
        sacc[rt][e] = p;
        lsum += p;
      }
    lsum += __shfl_xor(lsum, 32, 64);
    // the accumulators are rescaled only when some query's maximum moved (rare after the
    // first tiles)
    if (__any(m_new != m_run)) {
      const float corr = __builtin_amdgcn_exp2f(m_run - m_safe);          // m_run = -inf gives 0
      l_run *= corr;
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[i][e] *= corr;
    }
    l_run += lsum;
    m_run = m_new;

    // ---- O^T += V^T P^T.  Step (rt, mm) takes the 16 keys whose probabilities sit in
    // registers 8 mm .. 8 mm + 7 of row tile rt: for lane group g these are keys
    // 32 rt + 16 mm + 8 h + 4 g + e (h = 0, 1; e = 0..3), and V^T was stored in that order.
    Frag8 pb[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int rt = q / 2, mm = q % 2;
      pb[q].u.x = pack_bf16x2(sacc[rt][8 * mm + 0], sacc[rt][8 * mm + 1]);
      pb[q].u.y = pack_bf16x2(sacc[rt][8 * mm + 2], sacc[rt][8 * mm + 3]);
      pb[q].u.z = pack_bf16x2(sacc[rt][8 * mm + 4], sacc[rt][8 * mm + 5]);
      pb[q].u.w = pack_bf16x2(sacc[rt][8 * mm + 6], sacc[rt][8 * mm + 7]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int f = 0; f < 4 * VD; ++f) {
      oacc[f % VD] = mfma32(ring[f % AHEAD], pb[f / VD], oacc[f % VD]);
      if (f + AHEAD < 4 * VD) v_read(f + AHEAD);
      __builtin_amdgcn_sched_barrier(0);
    }
    }
    if (next) store_tile(buf ^ 1);
    __syncthreads();
  }

  if (!wave_on || !q_ok) return;
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  bf16_t* orow = out + ((size_t)(seq_start + ql) * n_heads + head) * D;
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      uint2 o;
      o.x = pack_bf16x2(oacc[i][4 * e4 + 0] * inv, oacc[i][4 * e4 + 1] * inv);
      o.y = pack_bf16x2(oacc[i][4 * e4 + 2] * inv, oacc[i][4 * e4 + 3] * inv);
      *reinterpret_cast<uint2*>(orow + i * 32 + 8 * e4 + 4 * g) = o;
    }
}

static int g_prefill_waves = 0, g_prefill_paired = 1;
extern "C" void rb_tune_prefill_waves(int nw) { g_prefill_waves = nw; }      // experiments only; 0 = built-in
extern "C" void rb_tune_prefill_paired(int on) { g_prefill_paired = on; }    // experiments only

extern "C" int rb_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                                         const int32_t* cu_seqlens, const int32_t* past_len,
                                         const int32_t* block_table, int bt_stride, int n_seqs, int max_q_len,
                                         int n_heads, int n_kv_heads, int head_dim, float scale, int window,
                                         void* stream) {
  RB_RECORDED(rb_attention_prefill_bf16(q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, bt_stride, n_seqs,
                                        max_q_len, n_heads, n_kv_heads, head_dim, scale, window, stream));
  RB_REQUIRE(n_seqs > 0 && max_q_len > 0, "rb_attention_prefill_bf16: empty batch");
  RB_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
             "rb_attention_prefill_bf16: bad head counts Hq=%d Hk=%d", n_heads, n_kv_heads);
  RB_REQUIRE(head_dim == 64 || head_dim == 128,
             "rb_attention_prefill_bf16: head_dim %d not supported (64 or 128; use rb_attention_generic)", head_dim);
  RB_REQUIRE(window >= 0, "rb_attention_prefill_bf16: negative window");
  const int group = n_heads / n_kv_heads;
  const int gw = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
  // Workgroups of 4 waves, two of which share a compute unit (their waves cover each other's
  // softmax arithmetic), or of 8 waves with twice the queries, which stage every tile of keys
  // and values for twice the work.  Measured with 32 heads on 8 kv heads, head size 128: the
  // small ones are faster up to about 12k tokens (2,048: 74 us against 86, where 256 large
  // workgroups run in one round and the last block of queries sets the time; 8,192: 820
  // against 900), the large ones beyond (32,768: 9.7 ms against 10.3).
  int nw = max_q_len <= 8192 ? 4 : 8;
  if (g_prefill_waves) nw = g_prefill_waves;
  const int q_per_wg = 32 * (nw / gw);
  dim3 grid((max_q_len + q_per_wg - 1) / q_per_wg, n_kv_heads * (group / gw), n_seqs);
  const int cus = rb_compute_units();
  const int paired = (nw == 4 && g_prefill_paired && (int)(grid.x * grid.y) > cus && (int)(grid.x * grid.y) <= 2 * cus) ? cus : 0;
  RB_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "rb_attention_prefill_bf16: batch or head count too large");
  hipStream_t s = (hipStream_t)stream;
  const float sl2 = scale * LOG2E;
#define RB_PF(DV, NWV)                                                                                          \
  attn_prefill_kernel<DV, NWV><<<grid, 64 * NWV, 0, s>>>((const bf16_t*)q, (const bf16_t*)k_pages,              \
                                                         (const bf16_t*)v_pages, (bf16_t*)out, cu_seqlens,      \
                                                         past_len, block_table, bt_stride, n_heads, n_kv_heads, \
                                                         sl2, window, gw, paired)
  if (head_dim == 128) {
    if (nw == 8) RB_PF(128, 8);
    else RB_PF(128, 4);
  } else {
    if (nw == 8) RB_PF(64, 8);
    else RB_PF(64, 4);
  }
#undef RB_PF
  RB_LAUNCH_CHECK();
  return 0;
}

// =============================================================================== decode
// One query per sequence.  A workgroup takes one kv head of one sequence (and one of n_splits
// shares of its pages); each of its 4 waves walks its own pages, 64 keys at a time, with a
// running softmax for the G query heads of the kv head, and the waves' states are merged
// through LDS at the end.  No barrier inside the page loop: a page's 32 loads per lane are
// all issued before the first is used, and four pages are in flight per workgroup.
//
// FUSED: q, k, v come straight from the projection (float32): q and the new k are rotated
// here (angles from the table) and rounded through bfloat16 exactly as rope_kv_write_kernel
// does, the new k and v are stored in the cache by the workgroup that owns the last page,
// and where the loop reaches the token's own position it takes them from LDS, so that no
// workgroup reads what another has just written.  Otherwise q is read as bfloat16 and the
// cache already holds the token's key and value.
//
// With one split the result is written directly; with more, partial states go to the
// workspace and attn_decode_combine_kernel adds them.  (Combining inside this kernel by a
// ticket counter was tried twice.  With device-scope fences: they write back and invalidate
// the L2 of every XCD and cost far more than the launch they save.  With fence-free
// device-coherent stores, loads and a relaxed counter: correct, but the chain store
// acknowledgement -> counter -> uncached loads takes as long as the second launch at 4
// splits and much longer at 16 or more.)
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  union {
    uint32_t u;
    bf16x2_t v;
  } x, y;
  x.u = a;
  y.u = b;
  return __builtin_amdgcn_fdot2_f32_bf16(x.v, y.v, c, false);
}
// Cross-lane moves without LDS traffic (data-parallel primitives of the vector unit).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// sum over the 4 lanes of a quad; every lane gets it
__device__ __forceinline__ float quad_sum(float v) {
  v += dpp_move<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  return v;
}
// Reductions over the 16 quads of a wave for values that are equal within each quad: rotate
// the rows of 16 lanes by 4 and 8, then combine the four rows through scalar registers.
__device__ __forceinline__ float quads_max(float v) {
  v = fmaxf(v, dpp_move<0x124>(v));      // row_ror:4
  v = fmaxf(v, dpp_move<0x128>(v));      // row_ror:8
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}
__device__ __forceinline__ float quads_sum(float v) {
  v += dpp_move<0x124>(v);
  v += dpp_move<0x128>(v);
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (r0 + r1) + (r2 + r3);
}
__device__ __forceinline__ float lane_value(float v, int lane) {      // lane is the same for the whole wave
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

template <int D, int G, bool FUSED>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const float* __restrict__ qkv, const bf16_t* __restrict__ q_in, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int style, bf16_t* k_pages, bf16_t* v_pages, bf16_t* __restrict__ out,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_table, int bt_stride, int n_heads,
    int n_kv, float scale_log2, int window, int n_splits, float* __restrict__ ws, int qkv_terms, size_t qkv_stride) {
  constexpr int DL = D / 64;          // output elements per lane
  constexpr int QC = D / 32;          // 16-byte chunks of a quarter row of K
  constexpr int QP = D / 8;           // bfloat16 pairs of a quarter row
  constexpr int HALF = D / 2;
  __shared__ __attribute__((aligned(16))) uint16_t q_h[G][D];
  __shared__ __attribute__((aligned(16))) uint16_t knew_h[D], vnew_h[D];
  __shared__ float red_m[4][G], red_l[4][G];
  __shared__ float red_acc[4][G][D];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int pos = tok_pos[b];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first_page = lo / RB_PAGE, last_page = pos / RB_PAGE;
  const int32_t* pages = block_table + (size_t)b * bt_stride;
  const int j = lane >> 2, part = lane & 3;

  const int pg_first = first_page + split + n_splits * wave;

  // ---- q of the G heads as packed bfloat16 pairs in registers: this lane's quarter of each row
  uint32_t q_pk[G][QP];
  if (FUSED) {
    const int row_width = (n_heads + 2 * n_kv) * D;
    const float* src = qkv + (size_t)b * row_width;
    const float* cr = cos_t ? cos_t + (size_t)pos * HALF : nullptr;
    const float* sr = cos_t ? sin_t + (size_t)pos * HALF : nullptr;
    for (int idx = tid; idx < (G + 1) * HALF; idx += 256) {
      const int gg = idx / HALF, i = idx - gg * HALF;
      const int i0 = style == 0 ? 2 * i : i, i1 = style == 0 ? 2 * i + 1 : i + HALF;
      const float* h = gg < G ? src + (size_t)(kvh * G + gg) * D : src + (size_t)(n_heads + kvh) * D;
      const float x0 = sum_terms(h + i0, qkv_terms, qkv_stride), x1 = sum_terms(h + i1, qkv_terms, qkv_stride);
      float y0 = x0, y1 = x1;
      if (cr) {
        const float c = cr[i], sn = sr[i];
        rotate_pair(x0, x1, c, sn, y0, y1);
      }
      uint16_t* dst = gg < G ? q_h[gg] : knew_h;
      dst[i0] = f32_to_bf16_bits(y0);
      dst[i1] = f32_to_bf16_bits(y1);
    }
    for (int d = tid; d < D; d += 256)
      vnew_h[d] = f32_to_bf16_bits(sum_terms(src + (size_t)(n_heads + n_kv + kvh) * D + d, qkv_terms, qkv_stride));
    __syncthreads();
#pragma unroll
    for (int gg = 0; gg < G; ++gg)
#pragma unroll
      for (int i = 0; i < QP; ++i) q_pk[gg][i] = *reinterpret_cast<const uint32_t*>(&q_h[gg][part * (D / 4) + 2 * i]);
    if (split == (last_page - first_page) % n_splits) {      // this workgroup owns the last page
      const int page = pages[last_page];
      const size_t at = ((size_t)page * n_kv + kvh) * RB_PAGE * D + (size_t)(pos % RB_PAGE) * D;
      for (int d = tid; d < D; d += 256) {
        k_pages[at + d].bits = knew_h[d];
        v_pages[at + d].bits = vnew_h[d];
      }
    }
  } else {
#pragma unroll
    for (int gg = 0; gg < G; ++gg) {
      const bf16_t* qrow = q_in + ((size_t)b * n_heads + kvh * G + gg) * D + part * (D / 4);
#pragma unroll
      for (int c = 0; c < QC; ++c) {
        const uint4 u = load16(qrow + c * 8);
        q_pk[gg][4 * c + 0] = u.x;
        q_pk[gg][4 * c + 1] = u.y;
        q_pk[gg][4 * c + 2] = u.z;
        q_pk[gg][4 * c + 3] = u.w;
      }
    }
  }

  float m_run[G], l_run[G], acc[G][DL];
#pragma unroll
  for (int gg = 0; gg < G; ++gg) {
    m_run[gg] = -INFINITY;
    l_run[gg] = 0.f;
#pragma unroll
    for (int e = 0; e < DL; ++e) acc[gg][e] = 0.f;
  }
  // this wave's pages: first_page + split + n_splits * (wave + 4 i).  All of a page's loads
  // are issued before the first is used.  (Requesting the next page's keys ahead was tried:
  // the wave is bound by its arithmetic, not by the loads, and the extra registers cost a
  // workgroup per compute unit.)
  const int pg_step = 4 * n_splits;
  auto work_page = [&](int pg) {
    const int page = pages[pg];
    const size_t base = ((size_t)page * n_kv + kvh) * RB_PAGE * D;
    uint4 kreg[4][QC];
    uint32_t vreg[4][16];
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
      const bf16_t* krow = k_pages + base + (size_t)(ps * 16 + j) * D + part * (D / 4);
#pragma unroll
      for (int cidx = 0; cidx < QC; ++cidx) kreg[ps][cidx] = load16(krow + cidx * 8);
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
      const bf16_t* vcol = v_pages + base + (size_t)(ps * 16) * D + lane * DL;
#pragma unroll
      for (int jj = 0; jj < 16; ++jj) {
        if (DL == 2)
          vreg[ps][jj] = *reinterpret_cast<const uint32_t*>(vcol + (size_t)jj * D);
        else
          vreg[ps][jj] = (uint32_t)vcol[(size_t)jj * D].bits;
      }
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
      const int key0 = pg * RB_PAGE + ps * 16;
      if (key0 > pos || key0 + 15 < lo) continue;          // nothing valid in this pass (same for the whole wave)
      const int key = key0 + j;
      const bool valid = key >= lo && key <= pos;
      if (FUSED && pos >= key0 && pos < key0 + 16 && key == pos) {
        // the token's own key is not in the cache yet (or only just): take it from LDS
#pragma unroll
        for (int cidx = 0; cidx < QC; ++cidx)
          kreg[ps][cidx] = *reinterpret_cast<const uint4*>(&knew_h[part * (D / 4) + cidx * 8]);
      }
      float s[G];
#pragma unroll
      for (int gg = 0; gg < G; ++gg) s[gg] = 0.f;
#pragma unroll
      for (int cidx = 0; cidx < QC; ++cidx) {
        const uint32_t wds[4] = {kreg[ps][cidx].x, kreg[ps][cidx].y, kreg[ps][cidx].z, kreg[ps][cidx].w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int gg = 0; gg < G; ++gg) s[gg] = dot2_bf16(wds[e], q_pk[gg][4 * cidx + e], s[gg]);
      }
      float p[G];
#pragma unroll
      for (int gg = 0; gg < G; ++gg) {
        float v = quad_sum(s[gg]);
        v = valid ? v * scale_log2 : -INFINITY;
        const float m_new = fmaxf(m_run[gg], quads_max(v));
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m_run[gg] - m_safe);
        p[gg] = __builtin_amdgcn_exp2f(v - m_safe);
        l_run[gg] = l_run[gg] * corr + quads_sum(p[gg]);
        m_run[gg] = m_new;
#pragma unroll
        for (int e = 0; e < DL; ++e) acc[gg][e] *= corr;
      }
      // ---- weighted sum of the values: key jj's probability sits in lanes 4 jj .. 4 jj + 3;
      // rows outside [lo, pos] may hold anything and are made zero
      uint32_t vnew_pk = 0;
      if (FUSED) {
        if (DL == 2)
          vnew_pk = *reinterpret_cast<const uint32_t*>(&vnew_h[lane * DL]);
        else
          vnew_pk = vnew_h[lane];
      }
#pragma unroll
      for (int jj = 0; jj < 16; ++jj) {
        const int kk = key0 + jj;
        uint32_t raw = vreg[ps][jj];
        if (FUSED && kk == pos) raw = vnew_pk;
        if (kk < lo || kk > pos) raw = 0;
        float v[DL];
        v[0] = bf16_bits_to_f32(raw & 0xffffu);
        if (DL == 2) v[DL - 1] = bf16_bits_to_f32(raw >> 16);
#pragma unroll
        for (int gg = 0; gg < G; ++gg) {
          const float pj = lane_value(p[gg], 4 * jj);
#pragma unroll
          for (int e = 0; e < DL; ++e) acc[gg][e] = fmaf(pj, v[e], acc[gg][e]);
        }
      }
    }
  };
  for (int pg = pg_first; pg <= last_page; pg += pg_step) work_page(pg);

  // ---- the four waves' states into one
#pragma unroll
  for (int gg = 0; gg < G; ++gg) {
    if (lane == 0) {
      red_m[wave][gg] = m_run[gg];
      red_l[wave][gg] = l_run[gg];
    }
#pragma unroll
    for (int e = 0; e < DL; ++e) red_acc[wave][gg][lane * DL + e] = acc[gg][e];
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int gg = idx / D, d = idx % D;
    float mx = red_m[0][gg];
#pragma unroll
    for (int w = 1; w < 4; ++w) mx = fmaxf(mx, red_m[w][gg]);
    const float m_safe = (mx == -INFINITY) ? 0.f : mx;
    float a = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(red_m[w][gg] - m_safe);
      a += red_acc[w][gg][d] * f;
      l += red_l[w][gg] * f;
    }
    if (n_splits == 1) {
      out[((size_t)b * n_heads + kvh * G + gg) * D + d] = f32_to_bf16(l > 0.f ? a / l : 0.f);
    } else {
      float* dst = ws + (((size_t)b * n_heads + kvh * G + gg) * n_splits + split) * (D + 2);
      dst[d] = a;
      if (d == 0) {
        dst[D] = mx;
        dst[D + 1] = l;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// The same decode step on the matrix cores, for any number of query heads per kv head up to
// 16: scores S^T[key, head] = K q^T and outputs O^T[d, head] = V^T P^T as 16x16x32 MFMAs with
// the heads as the 16 columns (columns beyond the group are zero queries).  The vector
// kernel above spends 8 dot products and 8 multiply-adds per key element at 8 heads per kv
// head and is bound by that arithmetic; here the work per key does not grow with the group.
//
// A wave takes a page at a time.  K rows go from memory straight into MFMA operands.  The
// second product needs V^T (8 keys of one d per lane): the page of V is brought into the
// wave's own LDS area by direct loads (dense 256- or 128-byte rows, 16-byte chunks permuted
// by (key / 4) % 4 so that the four lane groups of a transposed read hit different banks)
// and read back as 16-bit values.  The probabilities leave the first MFMA as 4 keys per lane
// and tile; the k index of the second product is ordered so that a lane's own 8 values
// (keys 4 grp + 0..3 of two tiles) are its operand, and V^T is read in the same order.
// Rows of the last page beyond the position may hold anything (0 x NaN would spoil the
// product): they are cleared in LDS, and the token's own row is put there (FUSED).
// ds_read_b64_tr_b16: every lane gives the address of 4 consecutive 16-bit values; within each
// group of 16 lanes, lane j receives value j % 4 of lanes j / 4, j / 4 + 4, j / 4 + 8, j / 4 + 12.
typedef __attribute__((ext_vector_type(4))) short i16x4_t;
__device__ __forceinline__ uint2 lds_read_transposed(const uint16_t* p) {
  union {
    i16x4_t v;
    uint2 u;
  } r;
  r.v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t*)(p));
  return r.u;
}
// Which 16-byte chunk of a row of V a chunk is stored in is chunk ^ v_swizzle(key): a
// transposing read touches 16 consecutive keys at the same 32 bytes of their rows, and the
// swizzle spreads them over the 8 bank windows of 32 bytes (twice each: the read takes two
// cycles anyway).  Rows of 256 bytes (D = 128) all start at bank 0; of rows of 128 bytes
// (D = 64) every second one does.
template <int D>
__device__ __forceinline__ int v_swizzle(int key) {
  return D == 128 ? ((key & 7) << 1) : (((key >> 1) & 3) << 1);
}

template <int D, int NW, bool FUSED, int ONCE>
__global__ __launch_bounds__(64 * NW) void attn_decode_mfma_kernel(
    const float* __restrict__ qkv, const bf16_t* __restrict__ q_in, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int style, bf16_t* k_pages, bf16_t* v_pages, bf16_t* __restrict__ out,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_table, int bt_stride, int n_heads,
    int n_kv, float scale_log2, int window, int n_splits, float* __restrict__ ws, int qkv_terms, size_t qkv_stride) {
  constexpr int KS = D / 32;          // depth steps of the score product
  constexpr int DT = D / 16;          // d tiles of the output product
  constexpr int HALF = D / 2;
  constexpr int CPR = D / 8;          // 16-byte chunks per row of V
  constexpr int RPI = 64 / CPR;       // rows one direct load instruction covers
  constexpr int VI = RB_PAGE / RPI;   // direct load instructions per page
  constexpr int DL = D / 64;          // elements of a row per lane
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr int NT = 64 * NW;
  uint16_t* vpages = reinterpret_cast<uint16_t*>(smem);                    // [NW waves][64 keys][D]
  uint16_t* q_h = vpages + NW * RB_PAGE * D;                               // [16][D]
  uint16_t* knew_h = q_h + 16 * D;
  uint16_t* vnew_h = knew_h + D;
  float* red_m = reinterpret_cast<float*>(vnew_h + D);                     // [NW][16]
  float* red_l = red_m + NW * 16;                                          // [NW][64]
  float* red_acc = reinterpret_cast<float*>(smem);                         // [NW][16][D], over the pages at the end

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // the same for the whole wave: LDS addresses go to a scalar register
  const int c16 = lane & 15, grp = lane >> 4;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int G = n_heads / n_kv;
  const int pos = tok_pos[b];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first_page = lo / RB_PAGE, last_page = pos / RB_PAGE;
  const int32_t* pages = block_table + (size_t)b * bt_stride;

  // ---- A page's way from memory (its number in the table, then its rows) is the longest wait
  // of a short step, so it starts early: the numbers of the wave's first two pages are asked
  // for here, the first page's values and keys as soon as q has been prepared (before the
  // barrier), every further page's keys while the page before is worked on, and its number a
  // page before that.
  Frag8 kf[4][KS], kf_next[4][KS];
  const int pg_step = NW * n_splits;
  const int pg_first = first_page + split + n_splits * wave;
  int id_next = pg_first <= last_page ? pages[pg_first] : 0;                       // the page worked on next
  int id_after = pg_first + pg_step <= last_page ? pages[pg_first + pg_step] : 0;  // the one after it
  uint16_t* vpage = vpages + wave * RB_PAGE * D;
  const uint32_t vpage_lds = (uint32_t)(uintptr_t)vpage;
  // ONCE >= 1: the pages of V, whole rows that are read once in a step, go past the caches; ONCE = 2: the
  // keys as well (the launcher says when).  Compiled in: as a run-time choice it stood as a branch at
  // every load of a page.
  constexpr bool v_once = ONCE >= 1, k_once = ONCE >= 2;
  auto ask_values = [&](int page) {        // into this wave's area of LDS
    const bf16_t* rows = v_pages + ((size_t)page * n_kv + kvh) * RB_PAGE * D;
#pragma unroll
    for (int i = 0; i < VI; ++i) {
      const int key = i * RPI + lane / CPR;
      const int chunk = (lane % CPR) ^ v_swizzle<D>(key);
      if constexpr (v_once) load_to_lds16_stream(rows, (uint32_t)(key * D + chunk * 8) * 2u, vpage_lds + i * 1024u);
      else load_to_lds16(rows, (uint32_t)(key * D + chunk * 8) * 2u, vpage_lds + i * 1024u);
    }
  };
  auto ask_keys = [&](int page) {          // into kf_next
    const bf16_t* rows = k_pages + ((size_t)page * n_kv + kvh) * RB_PAGE * D;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int st = 0; st < KS; ++st) {
        const bf16_t* src = rows + (size_t)(16 * t + c16) * D + 32 * st + 8 * grp;
        if constexpr (k_once) kf_next[t][st].u = load16_stream(src);
        else kf_next[t][st].u = load16(src);
      }
  };

  // ---- q of the group (rotated here when FUSED) as bfloat16 rows in LDS, zero rows beyond it
  if (FUSED) {
    const int row_width = (n_heads + 2 * n_kv) * D;
    const float* src = qkv + (size_t)b * row_width;
    const float* cr = cos_t ? cos_t + (size_t)pos * HALF : nullptr;
    const float* sr = cos_t ? sin_t + (size_t)pos * HALF : nullptr;
    for (int idx = tid; idx < 17 * HALF; idx += NT) {
      const int gg = idx / HALF, i = idx - gg * HALF;
      const int i0 = style == 0 ? 2 * i : i, i1 = style == 0 ? 2 * i + 1 : i + HALF;
      uint16_t* dst = gg < 16 ? q_h + gg * D : knew_h;
      if (gg < 16 && gg >= G) {
        dst[i0] = 0;
        dst[i1] = 0;
        continue;
      }
      const float* h = gg < 16 ? src + (size_t)(kvh * G + gg) * D : src + (size_t)(n_heads + kvh) * D;
      const float x0 = sum_terms(h + i0, qkv_terms, qkv_stride), x1 = sum_terms(h + i1, qkv_terms, qkv_stride);
      float y0 = x0, y1 = x1;
      if (cr) {
        const float c = cr[i], sn = sr[i];
        rotate_pair(x0, x1, c, sn, y0, y1);
      }
      dst[i0] = f32_to_bf16_bits(y0);
      dst[i1] = f32_to_bf16_bits(y1);
    }
    for (int d = tid; d < D; d += NT)
      vnew_h[d] = f32_to_bf16_bits(sum_terms(src + (size_t)(n_heads + n_kv + kvh) * D + d, qkv_terms, qkv_stride));
  } else {
    for (int idx = tid; idx < 16 * D; idx += NT) {
      const int gg = idx / D, d = idx - gg * D;
      q_h[idx] = gg < G ? q_in[((size_t)b * n_heads + kvh * G + gg) * D + d].bits : (uint16_t)0;
    }
  }
  int page_cur = 0;
  if (pg_first <= last_page) {
    page_cur = __builtin_amdgcn_readfirstlane(id_next);
    ask_values(page_cur);
    ask_keys(page_cur);
  }
  __syncthreads();
  if (FUSED && split == (last_page - first_page) % n_splits) {      // this workgroup owns the last page
    const int page = pages[last_page];
    const size_t at = ((size_t)page * n_kv + kvh) * RB_PAGE * D + (size_t)(pos % RB_PAGE) * D;
    for (int d = tid; d < D; d += NT) {
      k_pages[at + d].bits = knew_h[d];
      v_pages[at + d].bits = vnew_h[d];
    }
  }
  Frag8 qf[KS];
#pragma unroll
  for (int st = 0; st < KS; ++st) qf[st].u = *reinterpret_cast<const uint4*>(q_h + c16 * D + 32 * st + 8 * grp);

  float m_run = -INFINITY, l_part = 0.f;
  f32x4_t acc_o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc_o[dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  for (int pg = pg_first; pg <= last_page; pg += pg_step) {
    // This page's keys must all have arrived here, before the loads into LDS below are issued:
    // the compiler does not see those (they are assembly) and would count them out wrongly if
    // it waited for keys later.  Touching every register makes it wait now.
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int st = 0; st < KS; ++st) {
        kf[t][st] = kf_next[t][st];
        asm volatile("" ::"v"(kf[t][st].u.x), "v"(kf[t][st].u.y), "v"(kf[t][st].u.z), "v"(kf[t][st].u.w) : "memory");
      }
    if (pg != pg_first) {
      // the reads of the previous page have all returned before its area is overwritten (the
      // first page's values were asked for before the barrier)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      ask_values(page_cur);
    }
    // the next page's keys (its number was asked for a page ago), and the number of the one after
    const bool more = pg + pg_step <= last_page;
    const bool more2 = pg + 2 * pg_step <= last_page;
    int page_nx = 0;
    if (more) {
      page_nx = __builtin_amdgcn_readfirstlane(id_after);
      ask_keys(page_nx);
      if (more2) id_after = pages[pg + 2 * pg_step];
    }
    if (FUSED && pg == last_page) {
      // the token's own key is not in the cache yet (or only just): take it from LDS
      const int t_new = (pos % RB_PAGE) / 16, r_new = pos % 16;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int st = 0; st < KS; ++st)
          if (t == t_new && c16 == r_new) kf[t][st].u = *reinterpret_cast<const uint4*>(knew_h + 32 * st + 8 * grp);
    }
    // ---- scores: lane holds keys 16 t + 4 grp + i of head c16
    f32x4_t sc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      sc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < KS; ++st) sc[t] = mfma16(kf[t][st], qf[st], sc[t]);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = pg * RB_PAGE + 16 * t + 4 * grp + i;
        const float v = (key >= lo && key <= pos) ? sc[t][i] * scale_log2 : -INFINITY;
        sc[t][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_safe);
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = __builtin_amdgcn_exp2f(sc[t][i] - m_safe);
        sc[t][i] = pv;
        psum += pv;
      }
    l_part = l_part * corr + psum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc_o[dt][i] *= corr;
    Frag8 pf[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      pf[s2].u.x = pack_bf16x2(sc[2 * s2][0], sc[2 * s2][1]);
      pf[s2].u.y = pack_bf16x2(sc[2 * s2][2], sc[2 * s2][3]);
      pf[s2].u.z = pack_bf16x2(sc[2 * s2 + 1][0], sc[2 * s2 + 1][1]);
      pf[s2].u.w = pack_bf16x2(sc[2 * s2 + 1][2], sc[2 * s2 + 1][3]);
    }
    // ---- the page of V has arrived (loads complete in issue order; the next page's keys,
    // asked for after it, may still be on their way)
    if (more2) wait_vm<4 * KS + 1>();
    else if (more) wait_vm<4 * KS>();
    else wait_vm<0>();
    if (pg == last_page) {
      const int r_pos = pos % RB_PAGE;
      for (int row = FUSED ? r_pos : r_pos + 1; row < RB_PAGE; ++row) {
        const int d = lane * DL;
        uint16_t* dst = vpage + row * D + (((d >> 3) ^ v_swizzle<D>(row)) * 8 + (d & 7));
        const bool own = FUSED && row == r_pos;
        if (DL == 2)
          *reinterpret_cast<uint32_t*>(dst) = own ? *reinterpret_cast<const uint32_t*>(vnew_h + d) : 0u;
        else
          *dst = own ? vnew_h[d] : (uint16_t)0;
      }
    }
    // ---- O^T[d, head] += V^T P^T.  A transposing LDS read hands every lane of a 16-lane group 4
    // keys of its own d: lane i of the group points at 4 consecutive d (4 (i % 4) ..) of key
    // i / 4, and lane j receives element j % 4 of lanes j / 4, j / 4 + 4, ...: keys 0..3 at d = j.
    // Two of them make the 8 keys of the group's MFMA operand.
    const int key_in = c16 >> 2;                       // which of the 4 keys this lane points at
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int d4 = 16 * dt + 4 * (c16 & 3);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        Frag8 vf;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int key = 32 * s2 + 16 * h + 4 * grp + key_in;
          const uint16_t* src = vpage + key * D + (((d4 >> 3) ^ v_swizzle<D>(key)) * 8 + (d4 & 7));
          const uint2 got = lds_read_transposed(src);
          if (h == 0) {
            vf.u.x = got.x;
            vf.u.y = got.y;
          } else {
            vf.u.z = got.x;
            vf.u.w = got.y;
          }
        }
        acc_o[dt] = mfma16(vf, pf[s2], acc_o[dt]);
      }
    }
    page_cur = page_nx;
  }

  // ---- the waves' states into one (the pages' area is reused for the outputs)
  __syncthreads();
  if (c16 < G) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red_acc[((size_t)wave * 16 + c16) * D + 16 * dt + 4 * grp + i] = acc_o[dt][i];
  }
  red_l[wave * 64 + lane] = l_part;
  if (grp == 0) red_m[wave * 16 + c16] = m_run;
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += NT) {
    const int gg = idx / D, d = idx % D;
    float mx = red_m[gg];
#pragma unroll
    for (int w = 1; w < NW; ++w) mx = fmaxf(mx, red_m[w * 16 + gg]);
    const float m_safe = (mx == -INFINITY) ? 0.f : mx;
    float a = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = exp2f(red_m[w * 16 + gg] - m_safe);
      a += red_acc[((size_t)w * 16 + gg) * D + d] * f;
      const float* lw = red_l + w * 64 + gg;
      l += ((lw[0] + lw[16]) + (lw[32] + lw[48])) * f;
    }
    if (n_splits == 1) {
      out[((size_t)b * n_heads + kvh * G + gg) * D + d] = f32_to_bf16(l > 0.f ? a / l : 0.f);
    } else {
      float* dst = ws + (((size_t)b * n_heads + kvh * G + gg) * n_splits + split) * (D + 2);
      dst[d] = a;
      if (d == 0) {
        dst[D] = mx;
        dst[D + 1] = l;
      }
    }
  }
}

template <int D>
__global__ void attn_decode_combine_kernel(const float* __restrict__ ws, bf16_t* __restrict__ out, int n_splits) {
  const size_t row = blockIdx.x;            // sequence * heads + head
  const int d = threadIdx.x;
  const float* src = ws + row * n_splits * (D + 2);
  float mx = -INFINITY;
  for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, src[(size_t)s * (D + 2) + D]);
  const float m_safe = (mx == -INFINITY) ? 0.f : mx;
  float a = 0.f, l = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float f = exp2f(src[(size_t)s * (D + 2) + D] - m_safe);
    a += src[(size_t)s * (D + 2) + d] * f;
    l += src[(size_t)s * (D + 2) + D + 1] * f;
  }
  out[row * D + d] = f32_to_bf16(l > 0.f ? a / l : 0.f);
}

struct DecodeArgs {
  const float* qkv;
  const bf16_t* q;
  const float* cos_t;
  const float* sin_t;
  int style;
  bf16_t* k;
  bf16_t* v;
  bf16_t* out;
  const int32_t* tok_pos;
  const int32_t* bt;
  int bt_stride, n_seqs, n_heads, n_kv;
  float sl2;
  int window, n_splits;
  float* ws;
  int qkv_terms;          // fused: qkv as so many terms to be added up, qkv_stride floats apart
  size_t qkv_stride;
};

template <int D, int G, bool FUSED>
static void launch_decode(const DecodeArgs& a, hipStream_t s) {
  dim3 grid(a.n_splits, a.n_kv, a.n_seqs);
  attn_decode_kernel<D, G, FUSED><<<grid, 256, 0, s>>>(a.qkv, a.q, a.cos_t, a.sin_t, a.style, a.k, a.v, a.out,
                                                       a.tok_pos, a.bt, a.bt_stride, a.n_heads, a.n_kv, a.sl2,
                                                       a.window, a.n_splits, a.ws, a.qkv_terms, a.qkv_stride);
  if (a.n_splits > 1) attn_decode_combine_kernel<D><<<a.n_seqs * a.n_heads, D, 0, s>>>(a.ws, a.out, a.n_splits);
}

template <int D, int NW, bool FUSED, int ONCE>
static int launch_decode_mfma_nw(const DecodeArgs& a, hipStream_t s) {
  const size_t lds = (size_t)NW * RB_PAGE * D * 2 + 16 * D * 2 + 2 * D * 2 + (size_t)NW * (16 + 64) * sizeof(float);
  auto kern = attn_decode_mfma_kernel<D, NW, FUSED, ONCE>;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    RB_REQUIRE(e == hipSuccess, "decode attention: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    configured = true;
  }
  dim3 grid(a.n_splits, a.n_kv, a.n_seqs);
  kern<<<grid, 64 * NW, lds, s>>>(a.qkv, a.q, a.cos_t, a.sin_t, a.style, a.k, a.v, a.out, a.tok_pos, a.bt,
                                  a.bt_stride, a.n_heads, a.n_kv, a.sl2, a.window, a.n_splits, a.ws, a.qkv_terms,
                                  a.qkv_stride);
  if (a.n_splits > 1) attn_decode_combine_kernel<D><<<a.n_seqs * a.n_heads, D, 0, s>>>(a.ws, a.out, a.n_splits);
  return 0;
}

// 8 waves (8 pages at a time) for short contexts (one split) while that still gives every
// workgroup a compute unit of its own (a wave's page of V takes 16 KB of LDS at head size
// 128): the step is then bound by latency and fewer rounds of pages count.  Else 4 waves and
// two workgroups per compute unit, which stream long contexts a little faster.
static int g_decode_waves = 0;
extern "C" void rb_tune_decode_waves(int nw) { g_decode_waves = nw; }      // experiments only; 0 = built-in
template <int D, bool FUSED>
static int launch_decode_mfma(const DecodeArgs& a, hipStream_t s) {
  const long long wgs = (long long)a.n_splits * a.n_kv * a.n_seqs;
  const int cus = rb_compute_units();
  const int nw = g_decode_waves ? g_decode_waves : (wgs <= cus && a.n_splits == 1 ? 8 : 4);
  // Pages past the caches.  V when the batch is large enough for the caches to matter (32 sequences x
  // kv heads and more: batch 64 1.9 % of the step, batch 8 0.8 %; with a single sequence the plain loads
  // are 1.2 % faster).  The keys as well where the launch is large (512 workgroups and more: batch 64
  // at 8,192 keys 4.7 % of the step, at 530 keys 1.9 %); in small launches, which wait for their first
  // page rather than for bandwidth, they lose (batch 8 at 530 keys: 0.9 %).
  const int once = (long long)a.n_kv * a.n_seqs < cus / 8 ? 0 : (wgs >= 2 * cus ? 2 : 1);
  if (nw == 8) {
    if (once == 0) return launch_decode_mfma_nw<D, 8, FUSED, 0>(a, s);
    if (once == 1) return launch_decode_mfma_nw<D, 8, FUSED, 1>(a, s);
    return launch_decode_mfma_nw<D, 8, FUSED, 2>(a, s);
  }
  if (once == 0) return launch_decode_mfma_nw<D, 4, FUSED, 0>(a, s);
  if (once == 1) return launch_decode_mfma_nw<D, 4, FUSED, 1>(a, s);
  return launch_decode_mfma_nw<D, 4, FUSED, 2>(a, s);
}

// Which decode kernel: 0 = by group size (matrix cores from 2 query heads per kv head on: the
// vector kernel's arithmetic grows with the group, and it is built for groups of 1, 2, 4 and 8
// only; with one head per kv head the two are equally fast), 1 = always the matrix-core
// kernel, 2 = never.  Experiments and tests only.
static int g_decode_mfma = 0;
extern "C" void rb_tune_decode_mfma(int mode) { g_decode_mfma = mode; }

template <bool FUSED>
static int dispatch_decode(const DecodeArgs& a, int head_dim, hipStream_t s, const char* who) {
  RB_REQUIRE(a.n_seqs > 0, "%s: empty batch", who);
  RB_REQUIRE(a.n_heads > 0 && a.n_kv > 0 && a.n_heads % a.n_kv == 0, "%s: bad head counts Hq=%d Hk=%d", who,
             a.n_heads, a.n_kv);
  RB_REQUIRE(head_dim == 64 || head_dim == 128, "%s: head_dim %d not supported (64 or 128; use rb_attention_generic)",
             who, head_dim);
  RB_REQUIRE(a.n_splits >= 1 && a.n_splits <= 65535, "%s: bad split count %d", who, a.n_splits);
  RB_REQUIRE(a.n_kv <= 65535 && a.n_seqs <= 65535, "%s: batch or head count too large", who);
  RB_REQUIRE(a.window >= 0, "%s: negative window", who);
  RB_REQUIRE(a.n_splits == 1 || a.ws != nullptr, "%s: splits need a workspace", who);
  const int group = a.n_heads / a.n_kv;
  const bool vector_ok = group == 1 || group == 2 || group == 4 || group == 8;
  RB_REQUIRE(group <= 16, "%s: %d query heads per kv head not supported (at most 16; use rb_attention_generic)", who,
             group);
  RB_REQUIRE(g_decode_mfma != 2 || vector_ok, "%s: the vector kernel is built for 1, 2, 4 or 8 heads per kv head", who);
  if (g_decode_mfma == 1 || !vector_ok || (g_decode_mfma == 0 && group > 1)) {
    const int rc = head_dim == 128 ? launch_decode_mfma<128, FUSED>(a, s) : launch_decode_mfma<64, FUSED>(a, s);
    if (rc) return rc;
    RB_LAUNCH_CHECK();
    return 0;
  }
  if (head_dim == 128) {
    if (group == 1) launch_decode<128, 1, FUSED>(a, s);
    else if (group == 2) launch_decode<128, 2, FUSED>(a, s);
    else if (group == 4) launch_decode<128, 4, FUSED>(a, s);
    else launch_decode<128, 8, FUSED>(a, s);
  } else {
    if (group == 1) launch_decode<64, 1, FUSED>(a, s);
    else if (group == 2) launch_decode<64, 2, FUSED>(a, s);
    else if (group == 4) launch_decode<64, 4, FUSED>(a, s);
    else launch_decode<64, 8, FUSED>(a, s);
  }
  RB_LAUNCH_CHECK();
  return 0;
}

extern "C" int rb_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                                        const int32_t* tok_pos, const int32_t* block_table, int bt_stride,
                                        int n_seqs, int n_heads, int n_kv_heads, int head_dim, float scale,
                                        int window, int n_splits, float* workspace, void* stream) {
  RB_RECORDED(rb_attention_decode_bf16(q, k_pages, v_pages, out, tok_pos, block_table, bt_stride, n_seqs, n_heads, n_kv_heads,
                                       head_dim, scale, window, n_splits, workspace, stream));
  DecodeArgs a = {nullptr, (const bf16_t*)q, nullptr, nullptr, 0, (bf16_t*)k_pages, (bf16_t*)v_pages, (bf16_t*)out,
                  tok_pos, block_table, bt_stride, n_seqs, n_heads, n_kv_heads, scale * LOG2E, window, n_splits,
                  workspace, 1, 0};
  return dispatch_decode<false>(a, head_dim, (hipStream_t)stream, "rb_attention_decode_bf16");
}

extern "C" int rb_attention_decode_fused_bf16(const float* qkv, int qkv_terms, long long qkv_term_stride,
                                              const float* cos, const float* sin, int style,
                                              void* k_pages, void* v_pages, void* out, const int32_t* tok_pos,
                                              const int32_t* block_table, int bt_stride, int n_seqs, int n_heads,
                                              int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                                              float* workspace, void* stream) {
  RB_RECORDED(rb_attention_decode_fused_bf16(qkv, qkv_terms, qkv_term_stride, cos, sin, style, k_pages, v_pages, out, tok_pos,
                                             block_table, bt_stride, n_seqs, n_heads, n_kv_heads, head_dim, scale, window,
                                             n_splits, workspace, stream));
  RB_REQUIRE((cos == nullptr) == (sin == nullptr), "rb_attention_decode_fused_bf16: cos and sin tables go together");
  RB_REQUIRE(style == 0 || style == 1, "rb_attention_decode_fused_bf16: unknown pairing style %d", style);
  RB_REQUIRE(qkv_terms >= 1 && qkv_term_stride >= 0, "rb_attention_decode_fused_bf16: %d terms, %lld apart", qkv_terms,
             qkv_term_stride);
  DecodeArgs a = {qkv, nullptr, cos, sin, style, (bf16_t*)k_pages, (bf16_t*)v_pages, (bf16_t*)out,
                  tok_pos, block_table, bt_stride, n_seqs, n_heads, n_kv_heads, scale * LOG2E, window, n_splits,
                  workspace, qkv_terms, (size_t)qkv_term_stride};
  return dispatch_decode<true>(a, head_dim, (hipStream_t)stream, "rb_attention_decode_fused_bf16");
}
