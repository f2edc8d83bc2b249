/* Runs every entry point of the CPU oracle (wo_oracle.c) once on small inputs
 * that reach its edge cases -- a ragged last group, an all-zero column, NaN and
 * infinity, int4 packing, outlier columns, an empty batch.  Built by
 * `make -C oracle sanitize` with -fsanitize=address,undefined (host code only)
 * and executed there; it checks memory and arithmetic hygiene, not values
 * (tests/test_oracle.py checks those). */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "wo_oracle.c"

static uint32_t rng_state = 12345u;
static float frand(void) {
  rng_state = rng_state * 1664525u + 1013904223u;
  return ((float)(rng_state >> 8) / 16777216.0f - 0.5f) * 2.0f;
}

int main(void) {
  const int64_t K = 192, N = 64, M = 5;
  for (int dtype = 0; dtype < 2; ++dtype) {
    uint16_t* w = malloc(K * N * 2);
    for (int64_t i = 0; i < K * N; ++i) w[i] = wo_from_f32(frand() * 0.05f, dtype, 0);
    for (int64_t k = 0; k < K; ++k) w[k * N + 3] = 0;                 /* an all-zero column */
    w[5] = wo_from_f32(NAN, dtype, 0);
    w[70] = wo_from_f32(INFINITY, dtype, 1);
    uint16_t* x = malloc(M * K * 2);
    for (int64_t i = 0; i < M * K; ++i) x[i] = wo_from_f32(frand(), dtype, 0);
    uint16_t* bias = malloc(N * 2);
    for (int64_t i = 0; i < N; ++i) bias[i] = wo_from_f32(frand() * 0.01f, dtype, 0);
    const int64_t groups[3] = {-1, 64, 128};
    for (int bits = 4; bits <= 8; bits += 4)
      for (int gi = 0; gi < 3; ++gi) {
        const int64_t g = groups[gi];
        const int64_t ng = g > 0 ? (K + g - 1) / g : 1;
        int8_t* codes = malloc(K * N);
        uint16_t* scale = malloc(ng * N * 2);
        if (wo_weight_quantize(w, K, N, dtype, bits, g, 0, 0, codes, scale) != 0) return 1;
        float* d32 = malloc(K * N * 4);
        uint16_t* dT = malloc(K * N * 2);
        wo_dequantize(codes, scale, K, N, dtype, bits, g, 0, 0, d32, dT);
        float* o32 = malloc(M * N * 4);
        uint16_t* oT = malloc(M * N * 2);
        wo_linear(x, codes, bias, scale, M, K, N, dtype, bits, g, 0, gi == 1, o32, oT);
        wo_linear(x, codes, NULL, scale, 0, K, N, dtype, bits, g, 0, 0, o32, oT); /* empty batch */
        float* a32 = malloc(M * N * 4);
        uint16_t* aT = malloc(M * N * 2);
        for (int act = 0; act < 3; ++act) wo_activation(o32, M, N, act, dtype, a32, aT);
        uint16_t* og = malloc(M * N * 2);
        for (int64_t i = 0; i < M * N; ++i) og[i] = wo_from_f32(frand(), dtype, 0);
        float* g32 = malloc(M * K * 4);
        uint16_t* gT = malloc(M * K * 2);
        wo_linear_grad(og, codes, scale, M, K, N, dtype, bits, g, 0, gi == 2, g32, gT);
        free(codes); free(scale); free(d32); free(dT); free(o32); free(oT); free(a32); free(aT);
        free(og); free(g32); free(gT);
      }
    /* llm.int8: fp32 scales, transposed codes, one outlier column */
    int8_t* lc = malloc(K * N);
    float* ls = malloc(N * 4);
    if (wo_weight_quantize_llm_int8(w, K, N, dtype, -1, lc, ls) != 0) return 1;
    int8_t* lt = malloc(K * N);
    wo_transpose_bytes(lc, K, N, lt);
    x[7] = wo_from_f32(9.0f, dtype, 0);
    uint16_t* lo = malloc(M * N * 2);
    int8_t* qx = malloc(M * K);
    int32_t* acc = malloc(M * N * 4);
    float* rng = malloc(M * 4);
    uint8_t* outl = malloc(K);
    wo_llm_int8_linear(x, lt, bias, ls, 6.0f, M, K, N, dtype, lo, qx, acc, rng, outl);
    uint16_t* ps = malloc(K * 2);
    for (int64_t i = 0; i < K; ++i) ps[i] = wo_from_f32(1.0f + frand() * 0.1f, dtype, 0);
    uint16_t* xs = malloc(M * K * 2);
    wo_apply_per_channel_scale(x, ps, M, K, dtype, xs);
    free(lc); free(ls); free(lt); free(lo); free(qx); free(acc); free(rng); free(outl); free(ps); free(xs);
    free(w); free(x); free(bias);
  }
  if (wo_div127_fma_mismatches(0x3f800000u, 977u, 100000) != 0) return 2;
  printf("oracle sanitize selftest ok\n");
  return 0;
}
