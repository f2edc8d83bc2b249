// Driver for oracle/_ref: exposes the float<->T conversions of the reference's
// own headers (paddle/phi/common/float16.h, bfloat16.h), compiled from where
// they lie in the reference tree, so the oracle's restated casts can be
// checked against the real thing.  TEST INFRASTRUCTURE ONLY: built by
// oracle/Makefile when the reference tree is present, loaded only by tests
// and by tests/golden/make_cast_vectors.py.
//
// Built three times (see Makefile):
//   plain      g++                      fp16 = software routine, bf16 = RNE
//   f16c       g++ -mf16c               fp16 = _cvtss_sh (RNE),  bf16 = RNE
//   hipflavour g++ -DPADDLE_WITH_HIP -DREF_BF16_ONLY   bf16 = truncation
#include <cstdint>

#include "paddle/phi/common/bfloat16.h"
#ifndef REF_BF16_ONLY
#include "paddle/phi/common/float16.h"
#endif

extern "C" {

uint16_t ref_f32_to_bf16(float f) { return phi::dtype::bfloat16(f).x; }

float ref_bf16_to_f32(uint16_t h) {
  phi::dtype::bfloat16 b;
  b.x = h;
  return static_cast<float>(b);
}

void ref_f32_to_bf16_array(const float* in, int64_t n, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = phi::dtype::bfloat16(in[i]).x;
}

#ifndef REF_BF16_ONLY
uint16_t ref_f32_to_f16(float f) { return phi::dtype::float16(f).x; }

float ref_f16_to_f32(uint16_t h) {
  phi::dtype::float16 v;
  v.x = h;
  return static_cast<float>(v);
}

void ref_f32_to_f16_array(const float* in, int64_t n, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = phi::dtype::float16(in[i]).x;
}

void ref_f16_to_f32_array(const uint16_t* in, int64_t n, float* out) {
  for (int64_t i = 0; i < n; ++i) {
    phi::dtype::float16 v;
    v.x = in[i];
    out[i] = static_cast<float>(v);
  }
}
#endif

}  // extern "C"
