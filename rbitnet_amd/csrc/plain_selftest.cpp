// Runs every plain twin (plain.h) on small inputs whose buffers are exactly as large as the
// interface says, under the address and undefined-behaviour sanitizers (the build adds
// -fsanitize=address,undefined): an index that leaves its array ends the program.  Beside that it
// checks a few facts that need no second implementation: a one-token sequence attends to itself
// only; a product against the identity returns its input; both layouts of W give the same
// product; the norm of a constant row; sampling with u = 0 and u just below 1.
// Prints "plain twins ok" and exits with 0, or says what failed and exits with 1.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "plain.h"

static int g_failed = 0;
#define CHECK(cond, what)                              \
  do {                                                 \
    if (!(cond)) {                                     \
      printf("FAILED: %s (line %d)\n", what, __LINE__); \
      g_failed = 1;                                    \
    }                                                  \
  } while (0)
#define OK(call) CHECK((call) == 0, rbp_last_error())

static uint16_t bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float unbf16(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static float noise(uint32_t& s) {
  s = s * 1664525u + 1013904223u;
  return ((float)(s >> 8) / (float)(1 << 24) - 0.5f);
}

int main() {
  uint32_t seed = 7;
  // ---- embedding, both table types, the last row of the table
  {
    const int vocab = 5, width = 7;
    std::vector<float> table(vocab * width), x(3 * width);
    std::vector<uint16_t> table16(vocab * width);
    for (size_t i = 0; i < table.size(); ++i) {
      table[i] = noise(seed);
      table16[i] = bf16(table[i]);
    }
    const int32_t ids[3] = {4, 0, 4};
    OK(rbp_embed_gather(table.data(), 0, ids, x.data(), 3, width, nullptr));
    CHECK(x[0] == table[4 * width] && x[2 * width + 6] == table[4 * width + 6], "embedding rows");
    OK(rbp_embed_gather(table16.data(), 1, ids, x.data(), 3, width, nullptr));
    CHECK(x[width] == unbf16(table16[0]), "embedding widens bfloat16");
    const int32_t bad[1] = {-1};
    CHECK(rbp_embed_gather(table.data(), 0, bad, x.data(), 1, width, nullptr) != 0, "a negative id is refused");
  }
  // ---- norm: constant row, terms, chosen rows
  {
    const int width = 9, rows = 3, terms = 2;
    std::vector<float> x(rows * width, 0.003f), delta(terms * rows * width, 0.0f), gain(width, 1.0f), out(rows * width);
    OK(rbp_add_rmsnorm(x.data(), nullptr, 1, 0, gain.data(), 1e-5f, nullptr, rows, width, out.data(), 0, nullptr));
    CHECK(fabs(out[0] - 0.003 / sqrt(0.003 * 0.003 + 1e-5)) < 1e-7, "norm of a constant row, eps inside the root");
    for (auto& d : delta) d = 0.5f;
    OK(rbp_add_rmsnorm(x.data(), delta.data(), terms, rows * width, gain.data(), 1e-5f, nullptr, rows, width, out.data(),
                       0, nullptr));
    CHECK(fabs(x[4] - 1.003f) < 1e-6, "both terms were added to the stream");
    const int32_t pick[2] = {2, 0};
    std::vector<uint16_t> out16(2 * width);
    OK(rbp_add_rmsnorm(x.data(), delta.data(), terms, rows * width, gain.data(), 1e-5f, pick, 2, width, out16.data(), 1,
                       nullptr));
    CHECK(fabs(x[4] - 1.003f) < 1e-6, "chosen rows leave the stream as it is");
  }
  // ---- products: identity, both layouts, gate, folded forms
  {
    const int m = 3, n = 32, k = 64;
    std::vector<uint16_t> a(m * k), w(n * k), wf(n * k);
    for (auto& v : a) v = bf16(noise(seed));
    for (auto& v : w) v = bf16(noise(seed));
    OK(rbp_place_rows(w.data(), 1, wf.data(), 1, 1, n, k, n, 0, n, n, nullptr));
    std::vector<float> c0(m * n), c1(m * n);
    OK(rbp_gemm_bf16(a.data(), w.data(), 0, c0.data(), 0, 0, m, n, k, nullptr, nullptr));
    OK(rbp_gemm_bf16(a.data(), wf.data(), 1, c1.data(), 0, 0, m, n, k, nullptr, nullptr));
    CHECK(memcmp(c0.data(), c1.data(), c0.size() * 4) == 0, "rows and fragment-major W give the same product");
    std::vector<float> cg(m * n);
    OK(rbp_gemm_generic(a.data(), w.data(), 0, cg.data(), 1, 0, m, n, k, nullptr));
    CHECK(memcmp(c0.data(), cg.data(), c0.size() * 4) == 0, "the generic product is the same product");
    std::vector<uint16_t> gated(m * n / 2);
    OK(rbp_gemm_bf16(a.data(), w.data(), 0, gated.data(), 1, 1, m, n, k, nullptr, nullptr));
    const double g = c0[0], u = c0[16];
    CHECK(fabs(unbf16(gated[0]) - g / (1 + exp(-g)) * u) < 1e-2 * (1 + fabs(g * u)), "gate rows and up rows in blocks of 16");
    // C += product, then the rows prepared for the norm that follows
    std::vector<float> c(m * n, 1.0f), gain(n, 2.0f), squares((size_t)m * ((n + 15) / 16));
    std::vector<uint16_t> gained(m * n);
    OK(rbp_gemm_bf16_few(a.data(), nullptr, 0.f, nullptr, w.data(), 0, c.data(), 0, 3, gain.data(), gained.data(),
                         squares.data(), m, n, k, nullptr));
    CHECK(fabs(c[5] - (1.0f + c0[5])) < 1e-6, "epilogue 3 adds to C");
    CHECK(unbf16(gained[5]) == unbf16(bf16(c[5] * 2.0f)), "epilogue 3 leaves bf16(C * gain)");
    double ss = 0;
    for (int j = 16; j < 32; ++j) ss += (double)c[j] * c[j];
    CHECK(fabs(squares[1] - ss) < 1e-5 * (1 + ss), "epilogue 3 leaves the sums of squares of 16 columns");
    // prepared rows in: the product is scaled by the norm's factor; tokens chosen by `rows`
    std::vector<float> sq_in((size_t)m * (k / 16), 0.25f), cs(2 * n);
    const int32_t pick[2] = {2, 0};
    OK(rbp_gemm_bf16_few(a.data(), sq_in.data(), 1e-5f, pick, w.data(), 0, cs.data(), 0, 0, nullptr, nullptr, nullptr, 2,
                         n, k, nullptr));
    const double factor = 1.0 / sqrt(0.25 * (k / 16) / k + 1e-5);
    CHECK(fabs(cs[0] - c0[2 * n] * factor) < 1e-5 * (1 + fabs(cs[0])), "prepared rows: row 2 first, scaled");
    CHECK(rbp_gemm_bf16_few(a.data(), nullptr, 0.f, nullptr, w.data(), 0, c.data(), 0, 0, nullptr, nullptr, nullptr, 17,
                            n, k, nullptr) != 0, "17 tokens are refused");
    // the identity
    const int e = 8;
    std::vector<float> eye(e * e, 0.f), xin(2 * e), xout(2 * e);
    for (int i = 0; i < e; ++i) eye[i * e + i] = 1.f;
    for (auto& v : xin) v = noise(seed);
    OK(rbp_gemm_generic(xin.data(), eye.data(), 0, xout.data(), 0, 0, 2, e, e, nullptr));
    CHECK(memcmp(xin.data(), xout.data(), xin.size() * 4) == 0, "a product against the identity");
    // float32 W fragment-major: the same product
    const int fn = 32, fk = 128;
    std::vector<float> fw(fn * fk), fwf(fn * fk), fx(3 * fk), f0(3 * fn), f1(3 * fn);
    for (auto& v : fw) v = noise(seed);
    for (auto& v : fx) v = noise(seed);
    OK(rbp_place_rows(fw.data(), 0, fwf.data(), 0, 1, fn, fk, fn, 0, fn, fn, nullptr));
    OK(rbp_gemm_generic(fx.data(), fw.data(), 0, f0.data(), 0, 0, 3, fn, fk, nullptr));
    OK(rbp_gemm_generic(fx.data(), fwf.data(), 1, f1.data(), 0, 0, 3, fn, fk, nullptr));
    CHECK(memcmp(f0.data(), f1.data(), f0.size() * 4) == 0, "float32 rows and fragment-major W give the same product");
    CHECK(rbp_gemm_generic(fx.data(), fwf.data(), 1, f1.data(), 0, 0, 3, fn, 64, nullptr) != 0, "fragment-major float32 needs K % 128 == 0");
  }
  // ---- rotation and cache write, attention over pages, every form of it
  {
    const int hq = 4, hk = 2, d = 6, n_pages = 4, bt_stride = 2, n_seqs = 2;
    // sequence 0 brings 3 tokens on a past of 63 (so they straddle a page edge), sequence 1 its first token
    const int32_t cu[3] = {0, 3, 4}, past[2] = {63, 0};
    const int32_t tok_pos[4] = {63, 64, 65, 0}, tok_seq[4] = {0, 0, 0, 1};
    const int32_t bt[4] = {3, 1, 2, 0};                       // pages anywhere; sequence 1 has one page
    const int row = (hq + 2 * hk) * d, max_pos = 66;
    std::vector<float> qkv(2 * 4 * row), cosv(max_pos * d / 2), sinv(max_pos * d / 2);
    for (auto& v : qkv) v = noise(seed);
    for (int p = 0; p < max_pos; ++p)
      for (int i = 0; i < d / 2; ++i) {
        cosv[p * (d / 2) + i] = cosf(p * powf(100.f, -2.f * i / d));
        sinv[p * (d / 2) + i] = sinf(p * powf(100.f, -2.f * i / d));
      }
    for (int dtype = 0; dtype < 2; ++dtype) {
      const size_t esize = dtype == 0 ? 4 : 2;
      std::vector<unsigned char> q(4 * hq * d * esize), kp((size_t)n_pages * hk * 64 * d * esize, 0),
          vp((size_t)n_pages * hk * 64 * d * esize, 0), out(4 * hq * d * esize), out2(4 * hq * d * esize);
      // the past of sequence 0: positions 0..62 of page 3 hold something finite already (zeros)
      for (int style = 0; style < 2; ++style)
        OK(rbp_rope_kv_write(qkv.data(), 2, 4 * row, cosv.data(), sinv.data(), style, q.data(), kp.data(), vp.data(), dtype,
                             tok_pos, tok_seq, bt, bt_stride, 4, hq, hk, d, nullptr));
      OK(rbp_rope_kv_write(qkv.data(), 1, 0, nullptr, nullptr, 0, q.data(), nullptr, nullptr, dtype, tok_pos, tok_seq, bt,
                           bt_stride, 4, hq, 0, d, nullptr));          // a layer that keeps no cache: q only
      for (int window = 0; window <= 2; window += 2)
        OK(rbp_attention_generic(q.data(), kp.data(), vp.data(), out.data(), dtype, tok_pos, tok_seq, bt, bt_stride, 4, hq,
                                 hk, d, 0.4f, window, nullptr));
      if (dtype == 1) {
        OK(rbp_attention_generic(q.data(), kp.data(), vp.data(), out.data(), 1, tok_pos, tok_seq, bt, bt_stride, 4, hq, hk,
                                 d, 0.4f, 0, nullptr));
        OK(rbp_attention_prefill_bf16(q.data(), kp.data(), vp.data(), out2.data(), cu, past, bt, bt_stride, n_seqs, 3, hq,
                                      hk, d, 0.4f, 0, nullptr));
        CHECK(out == out2, "prefill attention is attention at the positions past + i");
        // the one-token sequence attends to itself: its output is its own value row
        const uint16_t* o16 = (const uint16_t*)out.data();
        const uint16_t* v16 = (const uint16_t*)vp.data();
        CHECK(o16[(3 * hq + 0) * d + 1] == v16[((size_t)bt[2] * hk + 0) * 64 * d + 1], "a one-token sequence returns its value");
        // decode: sequences 0 and 1 at positions 65 and 0, fused and not
        const int32_t dpos[2] = {65, 0};
        std::vector<float> qkv2(2 * row);
        memcpy(qkv2.data(), qkv.data() + 2 * row, row * 4);
        memcpy(qkv2.data() + row, qkv.data() + 3 * row, row * 4);
        std::vector<unsigned char> od(2 * hq * d * 2), of(2 * hq * d * 2), q2(2 * hq * d * 2);
        const int32_t dseq[2] = {0, 1};
        OK(rbp_rope_kv_write(qkv2.data(), 1, 0, cosv.data(), sinv.data(), 1, q2.data(), kp.data(), vp.data(), 1, dpos, dseq,
                             bt, bt_stride, 2, hq, hk, d, nullptr));
        OK(rbp_attention_decode_bf16(q2.data(), kp.data(), vp.data(), od.data(), dpos, bt, bt_stride, 2, hq, hk, d, 0.4f, 0, 1,
                                     nullptr, nullptr));
        OK(rbp_attention_decode_fused_bf16(qkv2.data(), 1, 0, cosv.data(), sinv.data(), 1, kp.data(), vp.data(), of.data(),
                                           dpos, bt, bt_stride, 2, hq, hk, d, 0.4f, 0, 1, nullptr, nullptr));
        CHECK(od == of, "fused decode attention is rotation, cache write and decode attention");
      }
    }
  }
  // ---- gate and sampling
  {
    const int rows = 2, ff = 5;
    std::vector<float> gu(rows * 2 * ff, 0.f), t(rows * ff);
    gu[0] = 40.f;
    gu[ff] = 3.f;
    OK(rbp_swiglu(gu.data(), t.data(), 0, rows, ff, nullptr));
    CHECK(fabs(t[0] - 120.f) < 1e-4 && t[1] == 0.f, "silu(40) * 3, silu(0) * 0");
    const int vocab = 6;
    const float nan = NAN;
    float logits[2 * 6] = {1.f, 5.f, nan, 5.f, -1.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    int32_t tok[2];
    OK(rbp_sample(logits, 2, vocab, nullptr, nullptr, tok, nullptr, nullptr));
    CHECK(tok[0] == 1 && tok[1] == 0, "argmax: NaN is -inf, the lowest index among equals");
    const float temp[2] = {1.f, 1.f}, u0[2] = {0.f, 0.9999f};
    OK(rbp_sample(logits, 2, vocab, temp, u0, tok, nullptr, nullptr));
    CHECK(tok[0] == 0 && tok[1] == 5, "inverse CDF: u = 0 takes the first index, u near 1 the last");
  }
  if (g_failed) return 1;
  printf("plain twins ok\n");
  return 0;
}
