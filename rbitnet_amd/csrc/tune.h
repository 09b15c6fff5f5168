// Hooks for measurements and for tests that must reach a kernel the dispatcher would not pick.
// They are no part of the library's interface: nothing on the product path calls them, and
// only tests and measurement scripts bind them.  The settings are process-wide and are read at
// every launch; 0 restores the built-in choice.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

void rb_tune_compute_units(int n);                              // every planner: pretend the GPU has n compute units
void rb_tune(int rows_per_wave, int waves);                     // skinny product
void rb_tune_resident(int tiles);                               // skinny product with resident tokens: row tiles per workgroup
void rb_tune_use_resident(int on);                              // 0: never the resident variant, 2: also below 8192 rows
void rb_tune_f32_few(int on);                                   // float32 product of few tokens: 0 = on the vector units, not the float32 MFMA; 3 = one row tile a wave always
void rb_tune_use_stream(int on);                                // 0: the skinny product up to 64 tokens
void rb_tune_tiles(int cfg, int parts);                         // tiled product: tile configuration and K slices
int rb_tune_plan(int m, int n, int k, int epilogue);            // tiled product: the built-in choice, 100 * cfg + parts
void rb_tune_attention_vec(int on);                             // generic attention: 0 = the scalar kernel also for head sizes that are multiples of 4
void rb_tune_prefill_waves(int waves);                          // prefill attention: 4 or 8
void rb_tune_prefill_paired(int on);                           // prefill attention: 0 = late blocks first only, no pairing of heavy and light workgroups
void rb_tune_decode_mfma(int mode);                             // decode attention: 1 matrix cores, 2 vector units
void rb_tune_decode_waves(int waves);                           // matrix-core decode attention: 4 or 8

#ifdef __cplusplus
}
#endif
