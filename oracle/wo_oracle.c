/*
 * wo_oracle.c -- CPU restatement of Paddle's weight-only quantisation path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, the host
 * layer, the Python mirror of paddle.nn.quant) may link, load or call this
 * file.  It exists so that the GPU kernels can be compared with an
 * independent, single-threaded statement of the reference arithmetic, and so
 * that the benchmark can time a CPU baseline beside the GPU numbers.
 *
 * Each function cites the reference source it follows (paths relative to the
 * Paddle tree).  How each function is pinned:
 *   casts         : checked against the reference's own float16.h / bfloat16.h
 *                   compiled as oracle/_ref (exhaustive over the fp16 range,
 *                   dense sample for bf16) and against committed vectors made
 *                   from that build.
 *   scales, codes : closed form max|w|/bound -> cast -> round-half-away ->
 *                   clip; pinned by an independent numpy brute force, by
 *                   invariants (|q| <= bound, non-degenerate groups reach
 *                   |q| == bound, |w - q*s| <= s/2 unless clipped) and by the
 *                   known answers recorded from a run of the reference header
 *                   (all-zero column: scale bits 0x0000, int8 code 127, int4
 *                   nibble 0x9).
 *   dequant/linear: products of <=8-bit codes with <=11-bit scales are exact
 *                   in fp32, so dequant has one correct answer; the linear is
 *                   checked against a float64 matmul of the same operands.
 *   llm.int8      : activation codes pinned by a numpy statement and invariants,
 *                   the int32 accumulators by numpy's integer matmul, the merge
 *                   by float64 evaluation.  PARITY UNPINNED for the outlier
 *                   branch: the reference reads the weight there through the
 *                   index permutation of another layout
 *                   (impl/llm_int8_matmul_kernel_impl.h:351-362) that
 *                   weight_quantize(algo="llm.int8") does not produce, and its
 *                   own tests never reach the branch; this restatement indexes
 *                   the weight plainly, as the op's description has it.
 *   pre-scale     : one correctly rounded multiply in T; pinned against the
 *                   half-precision multiply of numpy (fp16) and torch (bf16),
 *                   which are library routines with that definition, and by
 *                   exactness cases (scale 1, powers of two).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define WO_F16 0
#define WO_BF16 1

/* cast flavours (which build of the reference the scale cast imitates) */
#define WO_CAST_RNE 0   /* bf16: CPU/CUDA build; fp16: F16C or device build */
#define WO_CAST_TRUNC 1 /* bf16: HIP build (>>16); fp16: stock host build    */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- bfloat16 ---------------------------------------------------------- */

/* paddle/phi/common/bfloat16.h:61-88 (cpu_float_to_bfloat16): zero keeps only
 * the sign, inf passes through, NaN becomes 0x7FFF, everything else (normal
 * and subnormal) is round-to-nearest-even on the raw bits. */
uint16_t wo_f32_to_bf16_rne(float f) {
  uint32_t u = f2u(f);
  uint32_t mag = u & 0x7FFFFFFFu;
  if (mag == 0) return (uint16_t)((u >> 16) & 0x8000u);
  if (mag == 0x7F800000u) return (uint16_t)(u >> 16);
  if (mag > 0x7F800000u) return 0x7FFFu;
  uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7FFFu + lsb) >> 16);
}

/* paddle/phi/common/bfloat16.h:103-110 (PADDLE_WITH_HIP): drop the low half. */
uint16_t wo_f32_to_bf16_trunc(float f) { return (uint16_t)(f2u(f) >> 16); }

/* paddle/phi/common/bfloat16.h:190-213: the bf16 bits are the high half. */
float wo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* ---- float16 ----------------------------------------------------------- */

/* paddle/phi/common/float16.h:118-119 (_cvtss_sh(val, 0)) and the device
 * __float2half: IEEE round-to-nearest-even with gradual underflow. */
uint16_t wo_f32_to_f16_rne(float f) {
  uint32_t u = f2u(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) /* NaN: quiet it, keep the top payload bits */
    return (uint16_t)(sign | 0x7E00u | ((mag >> 13) & 0x03FFu));
  if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536, inf */
  int32_t e = (int32_t)(mag >> 23) - 127;
  if (e >= -14) { /* normal half, may round up into the next binade or to inf */
    uint32_t m = mag & 0x007FFFFFu;
    uint32_t h = ((uint32_t)(e + 15) << 10) | (m >> 13);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
  }
  if (e < -25) return sign; /* below half of the smallest subnormal */
  /* subnormal half: value = m24 * 2^(e-23), target unit 2^-24 */
  uint32_t m24 = (mag & 0x007FFFFFu) | 0x00800000u;
  int shift = -e - 1; /* 14..24 */
  uint32_t h = m24 >> shift;
  uint32_t rem = m24 & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

/* paddle/phi/common/float16.h:121-139, the software routine a host build
 * without F16C falls into.  What it computes, case by case on |val|:
 *   below 2^-14   : floor(|val| * 2^24) (subnormal, magnitude truncated)
 *   up to 65504   : exponent rebias, mantissa truncated to 10 bits
 *   above 65504   : infinity (even where nearest-even would give 65504)
 *   NaN           : payload >> 13, but payloads that would shift to zero
 *                   become the smallest half NaN (0x7C01)
 */
uint16_t wo_f32_to_f16_trunc(float f) {
  uint32_t u = f2u(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) {
    if (mag < 0x7F802000u) return (uint16_t)(sign | 0x7C01u);
    return (uint16_t)(sign | 0x7C00u | ((mag >> 13) & 0x03FFu));
  }
  if (mag > 0x477FE000u) return (uint16_t)(sign | 0x7C00u);
  if (mag < 0x38800000u) {
    /* |val| * 2^37 truncated to an integer, then the common >> 13 */
    float scaled = u2f(mag) * u2f(0x52000000u);
    uint32_t q = (uint32_t)(int32_t)scaled;
    return (uint16_t)(sign | (q >> 13));
  }
  return (uint16_t)(sign | ((mag >> 13) - 0x1C000u));
}

/* paddle/phi/common/float16.h:315-345 (operator float): exact widening. */
float wo_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu;
  uint32_t m = h & 0x03FFu;
  if (e == 0) {
    if (m == 0) return u2f(sign);
    float v = (float)m * u2f(0x33800000u); /* m * 2^-24, exact */
    return u2f(f2u(v) | sign);
  }
  if (e == 31) return u2f(sign | 0x7F800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

float wo_to_f32(uint16_t h, int dtype) {
  return dtype == WO_BF16 ? wo_bf16_to_f32(h) : wo_f16_to_f32(h);
}

uint16_t wo_from_f32(float f, int dtype, int cast_mode) {
  if (dtype == WO_BF16)
    return cast_mode == WO_CAST_TRUNC ? wo_f32_to_bf16_trunc(f)
                                      : wo_f32_to_bf16_rne(f);
  return cast_mode == WO_CAST_TRUNC ? wo_f32_to_f16_trunc(f)
                                    : wo_f32_to_f16_rne(f);
}

void wo_cast_array_from_f32(const float* in, int64_t n, int dtype,
                            int cast_mode, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = wo_from_f32(in[i], dtype, cast_mode);
}

void wo_cast_array_to_f32(const uint16_t* in, int64_t n, int dtype, float* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = wo_to_f32(in[i], dtype);
}

/* |x| as the reference's xabs<T> takes it (impl/weight_quantize_kernel_impl.h:
 * 40-43): negate when x < 0, so -0 and NaN pass through unchanged. */
static inline float abs_like_ref(float v) { return v < 0.0f ? -v : v; }

/* ---- scales ------------------------------------------------------------ */

/* paddle/phi/kernels/impl/weight_quantize_kernel_impl.h:45-57
 * (per_channel_scale).  w is [K,N] row-major in T; the running maximum starts
 * from the signed first element of the column. */
void wo_per_channel_scale(const uint16_t* w, int64_t K, int64_t N, int dtype,
                          float bound, int cast_mode, uint16_t* scale) {
  for (int64_t n = 0; n < N; ++n) {
    float mx = wo_to_f32(w[n], dtype);
    for (int64_t k = 0; k < K; ++k) {
      float a = abs_like_ref(wo_to_f32(w[k * N + n], dtype));
      mx = a > mx ? a : mx;
    }
    scale[n] = wo_from_f32(mx / bound, dtype, cast_mode);
  }
}

/* paddle/phi/kernels/impl/weight_quantize_kernel_impl.h:59-78
 * (group_wise_scale).  scale is [ceil(K/g), N]; the maximum starts at 0 and
 * the last group may be short. */
void wo_group_wise_scale(const uint16_t* w, int64_t K, int64_t N, int dtype,
                         float bound, int64_t g, int cast_mode,
                         uint16_t* scale) {
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t k0 = 0; k0 < K; k0 += g) {
      float mx = 0.0f;
      for (int64_t k = k0; k < k0 + g && k < K; ++k) {
        float a = abs_like_ref(wo_to_f32(w[k * N + n], dtype));
        mx = a > mx ? a : mx;
      }
      scale[(k0 / g) * N + n] = wo_from_f32(mx / bound, dtype, cast_mode);
    }
  }
}

/* ---- codes ------------------------------------------------------------- */

/* The int8 branch of per_channel_quant / group_wise_quant
 * (impl/weight_quantize_kernel_impl.h:91-96, :143-149): C round() (halves
 * away from zero), then std::min(127.f, r) and std::max(-127.f, .) spelled
 * out so that a NaN quotient (0/0 in an all-zero column) lands on 127. */
static inline int8_t quant_code_int8(float w, float s) {
  float r = roundf(w / s);
  float lo = (r < 127.0f) ? r : 127.0f;      /* std::min(127.f, r)  */
  float cl = (-127.0f < lo) ? lo : -127.0f;  /* std::max(-127.f, lo) */
  return (int8_t)cl;
}

/* The int4 branch (impl/weight_quantize_kernel_impl.h:104-114, :155-166):
 * the rounded quotient is converted to int BEFORE clipping.  The conversion
 * of NaN, infinities and out-of-range values is undefined in C++; the
 * reference runs on x86, where it yields INT_MIN, so they clip to -7. */
static inline int quant_code_int4(float w, float s) {
  float r = roundf(w / s);
  int v;
  if (r >= -2147483648.0f && r < 2147483648.0f) v = (int)r;
  else v = INT32_MIN;
  int lo = v < 7 ? v : 7;
  return lo > -7 ? lo : -7;
}

/* per_channel_quant<T,bits> and group_wise_quant<T,bits>
 * (impl/weight_quantize_kernel_impl.h:80-183), group_size -1 meaning one
 * scale per column.  Output is the canonical code tensor: [K,N] int8, or
 * [K,N/2] bytes with column 2j in the low nibble and 2j+1 in the high one.
 * nibble_bias is 0 for the CPU/CUDA flavour and 8 for the HIP flavour
 * (:109-111). */
void wo_quant_codes(const uint16_t* w, const uint16_t* scale, int64_t K,
                    int64_t N, int dtype, int bits, int64_t group_size,
                    int nibble_bias, int8_t* codes) {
  for (int64_t k = 0; k < K; ++k) {
    const uint16_t* wrow = w + k * N;
    const uint16_t* srow =
        group_size > 0 ? scale + (k / group_size) * N : scale;
    if (bits == 8) {
      int8_t* out = codes + k * N;
      for (int64_t n = 0; n < N; ++n)
        out[n] = quant_code_int8(wo_to_f32(wrow[n], dtype),
                                 wo_to_f32(srow[n], dtype));
    } else {
      int8_t* out = codes + k * (N / 2);
      for (int64_t j = 0; j < N / 2; ++j) {
        int q0 = quant_code_int4(wo_to_f32(wrow[2 * j], dtype),
                                 wo_to_f32(srow[2 * j], dtype)) + nibble_bias;
        int q1 = quant_code_int4(wo_to_f32(wrow[2 * j + 1], dtype),
                                 wo_to_f32(srow[2 * j + 1], dtype)) + nibble_bias;
        out[j] = (int8_t)((q0 & 0x0F) | ((q1 & 0x0F) << 4));
      }
    }
  }
}

/* Scale + codes in one call: the arithmetic half of quant_compute
 * (paddle/phi/kernels/cpu/weight_quantize_kernel.cc:95-107), bound 127 or 7.
 * Returns 0, or -1 on an argument the reference's InferMeta would reject
 * (paddle/phi/infermeta/unary.cc:5961-5983). */
int wo_weight_quantize(const uint16_t* w, int64_t K, int64_t N, int dtype,
                       int bits, int64_t group_size, int cast_mode,
                       int nibble_bias, int8_t* codes, uint16_t* scale) {
  if (K % 64 != 0 || N % 16 != 0) return -1;
  if (!(group_size == -1 || group_size == 64 || group_size == 128)) return -1;
  if (bits != 8 && bits != 4) return -1;
  float bound = bits == 8 ? 127.0f : 7.0f;
  if (group_size == -1)
    wo_per_channel_scale(w, K, N, dtype, bound, cast_mode, scale);
  else
    wo_group_wise_scale(w, K, N, dtype, bound, group_size, cast_mode, scale);
  wo_quant_codes(w, scale, K, N, dtype, bits, group_size, nibble_bias, codes);
  return 0;
}

/* algo == "llm.int8" (paddle/phi/kernels/cpu/weight_quantize_kernel.cc:163-166:
 * quant_compute<..., int8_t, 8, float>): the same loops with ScaleT = float,
 * so the scale max/127 is not rounded to T and the codes divide by that fp32
 * value (impl/weight_quantize_kernel_impl.h:45-57, :80-96 and the group-wise
 * forms :59-78, :131-149).  codes [K,N] int8, scale [N] or [ceil(K/g),N] float.
 * Pinned like the T-scale flavour (closed form, invariants, numpy
 * restatement); the reference holds no vectors for it. */
int wo_weight_quantize_llm_int8(const uint16_t* w, int64_t K, int64_t N,
                                int dtype, int64_t group_size, int8_t* codes,
                                float* scale) {
  if (K % 64 != 0 || N % 16 != 0) return -1;
  if (!(group_size == -1 || group_size == 64 || group_size == 128)) return -1;
  for (int64_t n = 0; n < N; ++n) {
    if (group_size == -1) {
      float mx = wo_to_f32(w[n], dtype);
      for (int64_t k = 0; k < K; ++k) {
        float a = abs_like_ref(wo_to_f32(w[k * N + n], dtype));
        mx = a > mx ? a : mx;
      }
      scale[n] = mx / 127.0f;
    } else {
      for (int64_t k0 = 0; k0 < K; k0 += group_size) {
        float mx = 0.0f;
        for (int64_t k = k0; k < k0 + group_size && k < K; ++k) {
          float a = abs_like_ref(wo_to_f32(w[k * N + n], dtype));
          mx = a > mx ? a : mx;
        }
        scale[(k0 / group_size) * N + n] = mx / 127.0f;
      }
    }
  }
  for (int64_t k = 0; k < K; ++k) {
    const float* srow = group_size > 0 ? scale + (k / group_size) * N : scale;
    for (int64_t n = 0; n < N; ++n)
      codes[k * N + n] = quant_code_int8(wo_to_f32(w[k * N + n], dtype), srow[n]);
  }
  return 0;
}

/* The HIP-flavour layout step of quant_compute
 * (cpu/weight_quantize_kernel.cc:113-125): a byte transpose of the canonical
 * tensor, [K,N] -> [N,K] for int8 and [K,N/2] -> [N/2,K] for int4. */
void wo_transpose_bytes(const int8_t* in, int64_t rows, int64_t cols,
                        int8_t* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) out[c * rows + r] = in[r * cols + c];
}

/* Signed code of element (k,n) of a canonical tensor. */
static inline int code_at(const int8_t* codes, int64_t k, int64_t n, int64_t N,
                          int bits, int nibble_bias) {
  if (bits == 8) return codes[k * N + n];
  uint8_t b = (uint8_t)codes[k * (N / 2) + n / 2];
  int nib = (n & 1) ? (b >> 4) : (b & 0x0F);
  if (nibble_bias) return nib - nibble_bias; /* HIP flavour: nibble - 8 */
  return nib >= 8 ? nib - 16 : nib;          /* two's complement nibble  */
}

/* ---- dequantise -------------------------------------------------------- */

/* out32[k,n] = float(code) * float(scale), the formula of
 * paddle/phi/kernels/gpu/weight_dequantize_kernel.cu:44-65 and :116-173, with
 * the scale indexed [k/g, n] as weight_quantize writes it.  The reference then
 * rounds to T; outT (optional) holds that, with the chosen cast flavour. */
void wo_dequantize(const int8_t* codes, const uint16_t* scale, int64_t K,
                   int64_t N, int dtype, int bits, int64_t group_size,
                   int nibble_bias, int cast_mode, float* out32,
                   uint16_t* outT) {
  for (int64_t k = 0; k < K; ++k) {
    const uint16_t* srow =
        group_size > 0 ? scale + (k / group_size) * N : scale;
    for (int64_t n = 0; n < N; ++n) {
      float v = (float)code_at(codes, k, n, N, bits, nibble_bias) *
                wo_to_f32(srow[n], dtype);
      if (out32) out32[k * N + n] = v;
      if (outT) outT[k * N + n] = wo_from_f32(v, dtype, cast_mode);
    }
  }
}

/* ---- linear ------------------------------------------------------------ */

/* out[m,n] = sum_k x[m,k] * dequant(W)[k,n] + bias[n], the contract of
 * WeightOnlyLinearKernel (paddle/phi/kernels/gpu/weight_only_linear_kernel.cu:
 * 48-58; m = x.numel()/k, bias optional, output dtype = x dtype).  The
 * dequantised weight stays in fp32 and is never rounded to T.  acc64 != 0
 * accumulates in double (error-study variant), else in fp32 in k order.
 * out32 receives the unrounded result, outT (optional) its RNE cast to T. */
void wo_linear(const uint16_t* x, const int8_t* codes, const uint16_t* bias,
               const uint16_t* scale, int64_t M, int64_t K, int64_t N,
               int dtype, int bits, int64_t group_size, int nibble_bias,
               int acc64, float* out32, uint16_t* outT) {
  float* wrow = (float*)malloc((size_t)N * sizeof(float));
  float* acc_f = (float*)malloc((size_t)N * sizeof(float));
  double* acc_d = (double*)malloc((size_t)N * sizeof(double));
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) { acc_f[n] = 0.0f; acc_d[n] = 0.0; }
    for (int64_t k = 0; k < K; ++k) {
      const uint16_t* srow =
          group_size > 0 ? scale + (k / group_size) * N : scale;
      for (int64_t n = 0; n < N; ++n)
        wrow[n] = (float)code_at(codes, k, n, N, bits, nibble_bias) *
                  wo_to_f32(srow[n], dtype);
      float xv = wo_to_f32(x[m * K + k], dtype);
      if (acc64) {
        for (int64_t n = 0; n < N; ++n) acc_d[n] += (double)xv * (double)wrow[n];
      } else {
        for (int64_t n = 0; n < N; ++n) acc_f[n] += xv * wrow[n];
      }
    }
    for (int64_t n = 0; n < N; ++n) {
      float b = bias ? wo_to_f32(bias[n], dtype) : 0.0f;
      float v = acc64 ? (float)(acc_d[n] + (double)b) : acc_f[n] + b;
      out32[m * N + n] = v;
      if (outT) outT[m * N + n] = wo_from_f32(v, dtype, WO_CAST_RNE);
    }
  }
  free(wrow); free(acc_f); free(acc_d);
}

/* Dequantise once into fp32 [K,N] (the middle stage of the CPU baseline:
 * quantize, dequantize, fp32 matmul). */
void wo_dequantize_f32(const int8_t* codes, const uint16_t* scale, int64_t K,
                       int64_t N, int dtype, int bits, int64_t group_size,
                       int nibble_bias, float* out32) {
  wo_dequantize(codes, scale, K, N, dtype, bits, group_size, nibble_bias,
                WO_CAST_RNE, out32, NULL);
}

/* ---- fused epilogues ------------------------------------------------------ */

/* The activations that follow weight_only_linear, applied to the fp32 sum
 * (accumulator + bias) before the one cast to T.
 *   act 1, gelu: the tanh form of the reference's GEMV epilogue,
 *     paddle/phi/kernels/funcs/weight_only_gemv.cu:147-157 (GeluActivation:
 *     v * 0.5 * (1 + tanh(0.7978845608028654 * (v + 0.044715 v^3)))), applied
 *     as at :1045-1046 to v + bias in float.  The reference's tanh is the
 *     hardware approximation (tanh.approx.f32, :137-138); here the exact tanh
 *     in double, the value every approximation approximates.
 *   act 2, swiglu: out[m, n] = silu(g) * u for n < N/2 with g, u the sums of
 *     columns n and n + N/2 (the halves paddle.incubate.nn.functional.swiglu
 *     splits a single input into, paddle/phi/kernels/gpu/swiglu_kernel.cu:32-52;
 *     silu(g) = g / (1 + exp(-g)), SwiGLUFunctor in
 *     paddle/phi/kernels/funcs/activation_functor.h).  The reference applies
 *     it to the rounded output of the linear (fusion/cutlass/moe_ffn.cu:133-139);
 *     here, as in the fused kernel, to the fp32 sums, rounded once.
 * in32: [M, N] fp32 sums (wo_linear's out32).  out32/outT: [M, N] (gelu) or
 * [M, N/2] (swiglu). */
void wo_activation(const float* in32, int64_t M, int64_t N, int act, int dtype,
                   float* out32, uint16_t* outT) {
  if (act == 2) {
    const int64_t H = N / 2;
    for (int64_t m = 0; m < M; ++m)
      for (int64_t n = 0; n < H; ++n) {
        const double g = (double)in32[m * N + n], u = (double)in32[m * N + H + n];
        const float v = (float)(g / (1.0 + exp(-g)) * u);
        out32[m * H + n] = v;
        if (outT) outT[m * H + n] = wo_from_f32(v, dtype, WO_CAST_RNE);
      }
    return;
  }
  for (int64_t i = 0; i < M * N; ++i) {
    const double x = (double)in32[i];
    float v = in32[i];
    if (act == 1)
      v = (float)(x * 0.5 * (1.0 + tanh(0.7978845608028654 * (x + 0.044715 * x * x * x))));
    out32[i] = v;
    if (outT) outT[i] = wo_from_f32(v, dtype, WO_CAST_RNE);
  }
}

/* ---- x_grad of weight_only_linear ----------------------------------------- */

/* WeightOnlyLinearGradKernel, paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu:27-72:
 *   x_grad[M, K] = out_grad[M, N] . dequant(W)[K, N]^T.
 * The reference dequantises to T first (:52-60) and hands the product to a
 * library GEMM (:61-69), so code * scale is rounded to T there.  This path's
 * contract keeps the dequantised weight in fp32, float(code) * float(scale)
 * (exact), and accumulates in fp32 (acc64 = 0) or double (acc64 = 1) over n in
 * ascending order; one cast to T at the end. */
void wo_linear_grad(const uint16_t* out_grad, const int8_t* codes,
                    const uint16_t* scale, int64_t M, int64_t K, int64_t N,
                    int dtype, int bits, int64_t group_size, int nibble_bias,
                    int acc64, float* out32, uint16_t* outT) {
  float* wdq = (float*)malloc((size_t)K * (size_t)N * sizeof(float));
  wo_dequantize(codes, scale, K, N, dtype, bits, group_size, nibble_bias,
                WO_CAST_RNE, wdq, NULL);
  float* g = (float*)malloc((size_t)N * sizeof(float));
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) g[n] = wo_to_f32(out_grad[m * N + n], dtype);
    for (int64_t k = 0; k < K; ++k) {
      const float* wr = wdq + k * N;
      float v;
      if (acc64) {
        double a = 0.0;
        for (int64_t n = 0; n < N; ++n) a += (double)g[n] * (double)wr[n];
        v = (float)a;
      } else {
        float a = 0.0f;
        for (int64_t n = 0; n < N; ++n) a += g[n] * wr[n];
        v = a;
      }
      out32[m * K + k] = v;
      if (outT) outT[m * K + k] = wo_from_f32(v, dtype, WO_CAST_RNE);
    }
  }
  free(g); free(wdq);
}

/* The reference's own composition of the same gradient
 * (paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu:52-69): the
 * dequantised weight is written out in T (weight_dequantize, :52-60), i.e.
 * every code * scale is rounded to T, and that tensor goes through a library
 * GEMM with fp32 accumulation.  Same arguments as wo_linear_grad; the only
 * difference is the rounding of the weight.  It is what the kernel's distance
 * to the reference is measured against (tests/test_linear_grad.py). */
void wo_linear_grad_rounded_weight(const uint16_t* out_grad, const int8_t* codes,
                                   const uint16_t* scale, int64_t M, int64_t K, int64_t N,
                                   int dtype, int bits, int64_t group_size, int nibble_bias,
                                   int acc64, float* out32, uint16_t* outT) {
  uint16_t* wT = (uint16_t*)malloc((size_t)K * (size_t)N * sizeof(uint16_t));
  wo_dequantize(codes, scale, K, N, dtype, bits, group_size, nibble_bias,
                WO_CAST_RNE, NULL, wT);
  float* g = (float*)malloc((size_t)N * sizeof(float));
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) g[n] = wo_to_f32(out_grad[m * N + n], dtype);
    for (int64_t k = 0; k < K; ++k) {
      const uint16_t* wr = wT + k * N;
      double a = 0.0;
      float af = 0.0f;
      for (int64_t n = 0; n < N; ++n) {
        const float w = wo_to_f32(wr[n], dtype);
        if (acc64) a += (double)g[n] * (double)w;
        else af += g[n] * w;
      }
      const float v = acc64 ? (float)a : af;
      out32[m * K + k] = v;
      if (outT) outT[m * K + k] = wo_from_f32(v, dtype, WO_CAST_RNE);
    }
  }
  free(g); free(wT);
}

/* ---- pre-quant activation smoothing ------------------------------------ */

/* out[r,c] = T(x[r,c] * scales[c]): ApplyPerChannelScaleKernel
 * (paddle/phi/kernels/gpu/apply_per_channel_scale_kernel.cu:93-126), whose
 * __hmul2 is the exact product rounded once to nearest even.  The product of
 * two T values (at most 11 significant bits each) is exact in fp32. */
void wo_apply_per_channel_scale(const uint16_t* x, const uint16_t* scales,
                                int64_t rows, int64_t cols, int dtype,
                                uint16_t* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c)
      out[r * cols + c] = wo_from_f32(
          wo_to_f32(x[r * cols + c], dtype) * wo_to_f32(scales[c], dtype), dtype,
          WO_CAST_RNE);
}

/* ---- llm.int8 linear --------------------------------------------------- */

/* LLMGemm (paddle/phi/kernels/impl/llm_int8_matmul_kernel_impl.h:560-690) and
 * llm_int8_compute (gpu/llm_int8_linear_kernel.cu:29-64), stage by stage:
 *   ReduceAbsMaxKernel (:221-268): column k is an outlier if any |x[m,k]| >
 *     T(threshold) (compared in T); range[m] = max over the row of |x| with
 *     the elements above the threshold counted as 0.
 *   QuantActKernel (:270-303), QuantFunc (:153-164): q = 0 in outlier columns,
 *     else clip(round(x * 127 * (1 / range[m])), -127, 127), products left to
 *     right in fp32, C round().
 *   int8 GEMM: acc[m,n] = sum_k q[m,k] * w[n,k] in int32.
 *   outlier columns (:593-640): sub[m,n] = T(sum_k x[m,k] * T(w[n,k] *
 *     wscale[n])) over the outlier columns (fp32 accumulation), 0 without any.
 *   DequantMergeKernel (:415-447), DequantFunc (:172-176): out = T(sub +
 *     T(acc * range[m] * wscale[n] / 127)), products left to right.
 *   bias: out = T(out + bias[n]).
 * w is [N,K] signed int8, wscale fp32 [N].  qx (optional) receives the codes,
 * acc (optional) the int32 sums, ranges (optional) the row maxima, outlier
 * (optional, K bytes) the column flags. */
void wo_llm_int8_linear(const uint16_t* x, const int8_t* w, const uint16_t* bias,
                        const float* wscale, float threshold, int64_t M,
                        int64_t K, int64_t N, int dtype, uint16_t* out,
                        int8_t* qx_out, int32_t* acc_out, float* ranges_out,
                        uint8_t* outlier_out) {
  const float thr = wo_to_f32(wo_from_f32(threshold, dtype, WO_CAST_RNE), dtype);
  uint8_t* outlier = (uint8_t*)calloc((size_t)K, 1);
  float* range = (float*)malloc((size_t)M * sizeof(float));
  int8_t* q = (int8_t*)malloc((size_t)M * K);
  for (int64_t m = 0; m < M; ++m) {
    float mx = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      float a = fabsf(wo_to_f32(x[m * K + k], dtype));
      if (a > thr) { outlier[k] = 1; a = 0.0f; }
      if (a > mx) mx = a;
    }
    range[m] = mx;
  }
  for (int64_t m = 0; m < M; ++m) {
    const float inv = 1.0f / range[m];
    for (int64_t k = 0; k < K; ++k) {
      float t = 0.0f;
      if (!outlier[k]) {
        t = wo_to_f32(x[m * K + k], dtype) * 127.0f * inv;
        t = roundf(t);
        if (t > 127.0f) t = 127.0f; else if (t < -127.0f) t = -127.0f;
        if (t != t) t = 0.0f; /* 0 * inf in an all-zero row: undefined in the reference */
      }
      q[m * K + k] = (int8_t)t;
    }
  }
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int32_t acc = 0;
      float sub = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        acc += (int32_t)q[m * K + k] * (int32_t)w[n * K + k];
        if (outlier[k]) {
          float wd = wo_to_f32(wo_from_f32((float)w[n * K + k] * wscale[n], dtype, WO_CAST_RNE), dtype);
          sub += wo_to_f32(x[m * K + k], dtype) * wd;
        }
      }
      if (acc_out) acc_out[m * N + n] = acc;
      float subT = wo_to_f32(wo_from_f32(sub, dtype, WO_CAST_RNE), dtype);
      float dq = wo_to_f32(wo_from_f32((float)acc * range[m] * wscale[n] / 127.0f, dtype, WO_CAST_RNE), dtype);
      uint16_t o = wo_from_f32(subT + dq, dtype, WO_CAST_RNE);
      if (bias) o = wo_from_f32(wo_to_f32(o, dtype) + wo_to_f32(bias[n], dtype), dtype, WO_CAST_RNE);
      out[m * N + n] = o;
    }
  if (qx_out) memcpy(qx_out, q, (size_t)M * K);
  if (ranges_out) memcpy(ranges_out, range, (size_t)M * sizeof(float));
  if (outlier_out) memcpy(outlier_out, outlier, (size_t)K);
  free(outlier); free(range); free(q);
}

/* The division by 127 of DequantFunc as the HIP epilogue performs it: a
 * reciprocal multiply corrected by two FMAs.  Counts the inputs first,
 * first + stride, ... (count of them, as float bit patterns) for which it
 * differs from the IEEE division the reference uses
 * (impl/llm_int8_matmul_kernel_impl.h:172-176).  The full sweep (first 0,
 * stride 1, count 2^32) returns 0; the tests run a strided sample. */
int64_t wo_div127_fma_mismatches(uint32_t first, uint32_t stride, int64_t count) {
  const float y = 1.0f / 127.0f;
  int64_t bad = 0;
  uint32_t u = first;
  for (int64_t i = 0; i < count; ++i, u += stride) {
    float v, ref, q, r, q2;
    uint32_t a, b;
    memcpy(&v, &u, 4);
    ref = v / 127.0f;
    q = v * y;
    r = fmaf(-q, 127.0f, v);
    q2 = fmaf(r, y, q);
    if (!(r != 0.0f && r == r)) q2 = q;
    memcpy(&a, &ref, 4);
    memcpy(&b, &q2, 4);
    if (a != b && !(ref != ref && q2 != q2)) ++bad;
  }
  return bad;
}
