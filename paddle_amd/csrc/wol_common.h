// Shared definitions of the gfx950 weight-only library: scalar type casts,
// the three code layouts and the index arithmetic of the GFX950 layout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "wol_c_api.h"

namespace wol {

// ---------------------------------------------------------------------------
// GFX950 layout, version 1
//
// The weight is cut into strips of 16 output columns; strip tn holds columns
// [16*tn, 16*tn+16) for every k and is contiguous: 16*K*bits/8 bytes, so a
// slice of the tensor along N at a multiple of 16 is still a valid tensor.
// Inside a strip the bytes are ordered exactly as one wavefront consumes them
// as the B operand of v_mfma_f32_16x16x32_{bf16,f16}: lane = 16*kb + j reads
// column j and the eight k values 8*kb .. 8*kb+7 of a 32-deep k step, and one
// 16-byte load per lane covers KT = 64 (int8) or 128 (int4) consecutive k:
//
//   int8: tile = 64 k  -> 1 KiB.  lane's 16 B = [k step 0: 8 B][k step 1: 8 B],
//         byte i of a k step = code(k0 + 32*step + 8*kb + i, n) + 128.
//   int4: tile = 128 k -> 1 KiB.  lane's 16 B = 4 dwords, one per k step;
//         nibble position p of a dword holds i = 2*p (p < 4) or 2*(p-4)+1, so
//         that (dword >> 4*p) & 0x000F000F is the pair (i, i+1) = (2p, 2p+1)
//         in the low/high halves; nibble = code + 8.
//         A K that is 64 mod 128 ends with a half tile of 512 B (8 B per lane,
//         two k steps).
// Biased (unsigned) storage lets a code turn into a bf16/fp16 bit pattern with
// one AND-OR; the bias is removed exactly by the consumer.
// ---------------------------------------------------------------------------
constexpr int kLayoutVersion = 1;
constexpr int kStripCols = 16;

__host__ __device__ inline int64_t strip_bytes(int64_t K, int bits) {
  return kStripCols * K * bits / 8;
}

// Byte offset and nibble shift (0 or 4; always 0 for int8) of element (k, n).
__host__ __device__ inline int64_t gfx950_offset(int64_t K, int bits, int64_t k,
                                                int64_t n, int* nib_shift) {
  const int64_t tn = n / kStripCols;
  const int j = static_cast<int>(n % kStripCols);
  const int kb = static_cast<int>((k % 32) / 8);
  const int i = static_cast<int>(k % 8);
  const int lane = kb * 16 + j;
  if (bits == 8) {
    const int64_t kt = k / 64;
    const int step = static_cast<int>((k % 64) / 32);
    *nib_shift = 0;
    return tn * strip_bytes(K, 8) + kt * 1024 + lane * 16 + step * 8 + i;
  }
  const int pos = (i >> 1) + 4 * (i & 1);
  const int64_t full = K / 128;  // number of full tiles
  const int64_t kt = k / 128;
  *nib_shift = (pos & 1) * 4;
  if (kt < full) {
    const int step = static_cast<int>((k % 128) / 32);
    return tn * strip_bytes(K, 4) + kt * 1024 + lane * 16 + step * 4 + pos / 2;
  }
  const int step = static_cast<int>((k % 64) / 32);  // half tile at the end
  return tn * strip_bytes(K, 4) + full * 1024 + lane * 8 + step * 4 + pos / 2;
}

// Byte offset / nibble shift of element (k, n) in any layout.
__host__ __device__ inline int64_t code_offset(int layout, int64_t K, int64_t N,
                                              int bits, int64_t k, int64_t n,
                                              int* nib_shift) {
  if (layout == WOL_LAYOUT_GFX950) return gfx950_offset(K, bits, k, n, nib_shift);
  if (bits == 8) {
    *nib_shift = 0;
    return layout == WOL_LAYOUT_CANONICAL ? k * N + n : n * K + k;
  }
  *nib_shift = static_cast<int>(n & 1) * 4;
  return layout == WOL_LAYOUT_CANONICAL ? k * (N / 2) + n / 2
                                        : (n / 2) * K + k;
}

// Stored byte / nibble of a signed code q in a layout, and back.
__host__ __device__ inline int encode_code(int layout, int bits, int q) {
  if (bits == 8) return layout == WOL_LAYOUT_GFX950 ? ((q + 128) & 0xFF) : (q & 0xFF);
  return layout == WOL_LAYOUT_CANONICAL ? (q & 0xF) : ((q + 8) & 0xF);
}

__host__ __device__ inline int decode_code(int layout, int bits, int v) {
  if (bits == 8) return layout == WOL_LAYOUT_GFX950 ? (v & 0xFF) - 128
                                                    : static_cast<int8_t>(v & 0xFF);
  v &= 0xF;
  if (layout == WOL_LAYOUT_CANONICAL) return v >= 8 ? v - 16 : v;
  return v - 8;
}

// ---------------------------------------------------------------------------
// T <-> float.  Inputs are bit patterns (uint16_t); widening is exact.
// ---------------------------------------------------------------------------
__device__ inline float bf16_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

__device__ inline float f16_to_f32(uint16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h));
}

template <int DT>
__device__ inline float to_f32(uint16_t h) {
  return DT == WOL_DTYPE_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}

// Round-to-nearest-even float -> bf16, with the special cases of
// paddle/phi/common/bfloat16.h:61-88: zero keeps only its sign, infinity
// passes, NaN becomes 0x7FFF.
__device__ inline uint16_t f32_to_bf16_rne(float f) {
  // branch-free: the rounding add leaves zero and infinity as they are (their
  // low half is zero), so only NaN needs a select
  const uint32_t u = __float_as_uint(f);
  const uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
  return static_cast<uint16_t>((u & 0x7FFFFFFFu) > 0x7F800000u ? 0x7FFFu : r);
}

// Round-to-nearest-even float -> fp16 (v_cvt_f16_f32 under the default
// rounding mode, denormals on).  NaN is canonicalised like _cvtss_sh does:
// quiet bit set, top payload bits kept.
__device__ inline uint16_t f32_to_f16_rne(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t mag = u & 0x7FFFFFFFu;
  const uint16_t nan = static_cast<uint16_t>(((u >> 16) & 0x8000u) | 0x7E00u | ((mag >> 13) & 0x3FFu));
  const uint16_t num = __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
  return mag > 0x7F800000u ? nan : num;  // a select, not a branch
}

// The truncating flavours (WOL_ROUND_TRUNC): bf16 drops the low half
// (paddle/phi/common/bfloat16.h:103-110); fp16 follows the software routine of
// a host build without F16C (paddle/phi/common/float16.h:121-139): magnitudes
// truncate, anything above 65504 is infinity, subnormals are floor(|f|*2^24).
__device__ inline uint16_t f32_to_bf16_trunc(float f) {
  return static_cast<uint16_t>(__float_as_uint(f) >> 16);
}

__device__ inline uint16_t f32_to_f16_trunc(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
  const uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) {
    if (mag < 0x7F802000u) return sign | 0x7C01u;
    return sign | 0x7C00u | static_cast<uint16_t>((mag >> 13) & 0x3FFu);
  }
  if (mag > 0x477FE000u) return sign | 0x7C00u;
  if (mag < 0x38800000u) {
    // |f| < 2^-14: the product is exact (power-of-two factor) and < 2^23.
    const float scaled = __uint_as_float(mag) * __uint_as_float(0x52000000u);
    return sign | static_cast<uint16_t>(static_cast<uint32_t>(scaled) >> 13);
  }
  return sign | static_cast<uint16_t>((mag >> 13) - 0x1C000u);
}

template <int DT>
__device__ inline uint16_t from_f32(float f, int round_mode) {
  if (DT == WOL_DTYPE_BF16)
    return round_mode == WOL_ROUND_TRUNC ? f32_to_bf16_trunc(f) : f32_to_bf16_rne(f);
  return round_mode == WOL_ROUND_TRUNC ? f32_to_f16_trunc(f) : f32_to_f16_rne(f);
}

template <int DT>
__device__ inline uint16_t from_f32_rne(float f) {
  return DT == WOL_DTYPE_BF16 ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
}

// Output cast of the linear kernels: the hardware's round-to-nearest-even
// conversions (v_cvt_pk_bf16_f32 / v_cvt_f16_f32), branch-free.  They agree
// with from_f32_rne on every finite and infinite value; NaN payloads may differ.
// The fp16 flavour hides its operand from the optimiser first: otherwise the
// multiply-add that produced it is merged with the conversion into one
// v_fma_mixlo_f16, which rounds once, and the result would no longer be the
// cast of the fp32 value that the fp32 output mode reports.
template <int DT>
__device__ inline uint16_t cast_out(float f) {
  if (DT == WOL_DTYPE_BF16) return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
  asm volatile("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------
// What wol_linear_fused adds around the linear: the activation smoothing
// (apply_per_channel_scale) in front and an activation behind.
// ---------------------------------------------------------------------------

// x * s for two T values packed in a dword, each product rounded once to T
// (RNE): the arithmetic of apply_per_channel_scale (the product of two T values
// is exact in fp32).
template <int DT>
__device__ inline uint32_t prescale_pair(uint32_t x2, uint32_t s2) {
  const float lo = to_f32<DT>(static_cast<uint16_t>(x2 & 0xFFFFu)) * to_f32<DT>(static_cast<uint16_t>(s2 & 0xFFFFu));
  const float hi = to_f32<DT>(static_cast<uint16_t>(x2 >> 16)) * to_f32<DT>(static_cast<uint16_t>(s2 >> 16));
  return static_cast<uint32_t>(cast_out<DT>(lo)) | (static_cast<uint32_t>(cast_out<DT>(hi)) << 16);
}

// The same for the eight values of an A fragment and the scales of their eight k.
template <int DT>
__device__ inline u32x4 prescale_frag(u32x4 a, u32x4 s) {
  u32x4 o;
  o.x = prescale_pair<DT>(a.x, s.x);
  o.y = prescale_pair<DT>(a.y, s.y);
  o.z = prescale_pair<DT>(a.z, s.z);
  o.w = prescale_pair<DT>(a.w, s.w);
  return o;
}

// gelu in its tanh form (paddle/phi/kernels/funcs/weight_only_gemv.cu:147-157),
// on the fp32 sum; tanh(u) = 1 - 2 / (exp(2u) + 1), which saturates correctly
// at both ends.
__device__ inline float act_gelu(float v) {
  const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
  const float t = 1.0f - 2.0f / (__expf(2.0f * u) + 1.0f);
  return v * 0.5f * (1.0f + t);
}

// silu(g) * u, the swiglu of a gate and an up value
// (paddle/phi/kernels/gpu/swiglu_kernel.cu:32-52).
__device__ inline float act_swiglu(float g, float u) { return g / (1.0f + __expf(-g)) * u; }

// act: WOL_ACT_NONE or WOL_ACT_GELU (swiglu combines two sums and is applied where both are at hand)
__device__ inline float act_apply(float v, int act) { return act == WOL_ACT_GELU ? act_gelu(v) : v; }

// Strips (16 columns) that share a workgroup of the streaming linear kernel.
// Two halve the activation traffic out of L2 (N/16 * rows * K * 2 bytes, rows
// = M rounded up to a power of two, at most 16 per operand) but also the
// number of workgroups: worth it once that traffic is at least the weight
// bytes (rows >= bits) and enough workgroups remain (measured thresholds).
inline int stream_strips_per_workgroup(int64_t M, int64_t N, int bits) {
  if (M > 16) return 1;  // several 16-row operands per strip already fill the registers
  int rows = 1;
  while (rows < 16 && rows < M) rows *= 2;
  const int64_t groups = N / kStripCols / 2;
  if (rows >= 2 * bits) return groups >= 256 ? 2 : 1;  // a workgroup for every CU must remain
  // activation traffic equal to the weight bytes (8 rows of int8; the kernels
  // pair strips from 8 rows up): 25.7 against 26.9 us at 448 pairs, 13.4
  // against 12.8 us at 384
  if (rows >= 8 && rows >= bits) return groups >= 448 ? 2 : 1;
  return 1;
}

// What wol_linear_fused adds to a linear call.  pre_scale: [K] T or null.
// act: a WOL_ACT_* value.  The launchers say which parts they apply themselves.
struct Fuse {
  const void* pre_scale = nullptr;
  int act = 0;
};

// Launchers implemented in the .hip files; each returns a wol_status.
int launch_quantize(const void* w, int dtype, int64_t K, int64_t N, int bits, int group_size,
                    int round_mode, int layout, void* codes, void* scale, bool scale_f32,
                    void* workspace, hipStream_t stream);
// wol_quantize without a caller's workspace: the per-channel abs-max buffer is
// a file-scope device array of kQuantizeStaticMaxN words (256 KiB per GPU).
constexpr int64_t kQuantizeStaticMaxN = 65536;
int launch_quantize_static(const void* w, int dtype, int64_t K, int64_t N, int bits, int group_size,
                           int round_mode, int layout, void* codes, void* scale,
                           hipStream_t stream);
int launch_dequantize(const void* codes, int layout, const void* scale, int dtype, int64_t K,
                      int64_t N, int bits, int group_size, void* out, hipStream_t stream);
int launch_repack(const void* in, int layout_in, void* out, int layout_out, int64_t K, int64_t N,
                  int bits, hipStream_t stream);
int launch_linear_stream(const void* x, const void* codes, const void* bias, const void* scale,
                         int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                         void* out, bool out_f32, hipStream_t stream, const Fuse& f = Fuse());
// The batched decode kernel (2 to 16 rows; one row works too; K = 2048, 4096, and
// 8192 for int4 without groups of 64).
bool linear_batch_supports(int64_t M, int64_t K, int bits, int group_size);
bool linear_batch_fuses_pre_scale(int64_t K, int bits, int group_size);
int linear_batch_cus();  // CUs of the current device (256 when it cannot be asked)
void plan_linear_batch(int64_t K, int64_t N, int bits, int* grid, int* tpw, bool swi = false);
bool linear_batch_fuses_swiglu(int64_t K, int64_t N, int bits);
int launch_linear_batch(const void* x, const void* codes, const void* bias, const void* scale,
                        int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                        void* out, bool out_f32, hipStream_t stream, const Fuse& f = Fuse());
// The batched decode kernel with K cut into runs across workgroups (up to 32
// rows, any K of at least 16 whole weight tiles): the runs' fp32 sums go
// through ws (linear_batch_split_workspace bytes) and launch_reduce_partials
// adds them.  It applies no Fuse::pre_scale.
bool linear_batch_split_supports(int64_t M, int64_t K, int bits, int group_size);
size_t linear_batch_split_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size);
int launch_linear_batch_split(const void* x, const void* codes, const void* bias, const void* scale,
                              int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                              void* out, bool out_f32, void* ws, size_t ws_bytes, hipStream_t stream,
                              const Fuse& f = Fuse());
void describe_linear_batch_split(int64_t M, int64_t K, int64_t N, int bits, int group_size, char* buf, size_t n);
// out[m, n] = T(act(sum over the runs of part[run][m][n] + bias[n])): the second
// kernel of every K-split launch (wol_linear_gemm.hip).  N % 4 == 0.  act may also be
// WOL_ACT_SWIGLU (N % 8 == 0): out is then [M, N/2], silu of the first half of a row's sums
// times the second half.
int launch_reduce_partials(const float* part, int nsplit, const void* bias, int dtype, void* out,
                           bool out_f32, int64_t M, int64_t N, int act, hipStream_t stream);
// One-line descriptions of what the launchers would run for a problem.
void describe_linear_stream(int64_t M, int64_t K, int64_t N, int bits, int group_size, char* buf, size_t n);
// Whether the streaming kernel runs the problem with every load of a wavefront issued at once (K divides into a
// power of two of units per strip that a workgroup's wavefronts take whole) rather than walking its units.
bool linear_stream_loads_at_once(int64_t M, int64_t K, int64_t N, int bits);
void describe_linear_gemm(int64_t M, int64_t K, int64_t N, int bits, int group_size, size_t ws_bytes,
                          char* buf, size_t n);
int launch_linear_gemm(const void* x, const void* codes, const void* bias, const void* scale,
                       int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                       void* out, bool out_f32, void* workspace, size_t workspace_bytes,
                       hipStream_t stream, const Fuse& f = Fuse());
// x_grad[M, K] = out_grad[M, N] . dequant(W)[K, N]^T from the packed codes.
size_t linear_grad_workspace(int64_t M, int64_t K, int64_t N, int group_size);
void describe_linear_grad(int64_t M, int64_t K, int64_t N, char* buf, size_t n);
int launch_linear_grad(const void* out_grad, const void* codes, const void* scale, int dtype, int64_t M,
                       int64_t K, int64_t N, int bits, int group_size, void* x_grad, bool out_f32,
                       void* workspace, hipStream_t stream);
int launch_read_floor(const void* codes, int64_t K, int64_t N, int bits, void* out,
                      hipStream_t stream);
int launch_mfma_probe(int variant, const void* ops, int workgroups, int iters, float* out, hipStream_t stream);
// The headline decode kernel (bf16, int4 with group-wise scales, one row, K = 4096) with clock stamps per wavefront
// (wol_decode_phases).
int launch_decode_phases(const void* x, const void* codes, const void* scale, int64_t K, int64_t N, int group_size,
                         void* out, unsigned long long* stamps, hipStream_t stream);
// The prefill GEMM's 256 x 256 launch (int8 per-channel, bf16) with cycle stamps per wavefront (wol_prefill_phases).
int launch_prefill_phases(const void* x, const void* codes, const void* scale, int64_t M, int64_t K, int64_t N,
                          void* out, unsigned long long* stamps, hipStream_t stream);
int launch_mfma_ceiling(const void* operands, int workgroups, int iters, float* out,
                        hipStream_t stream);
int launch_prescale(const void* x, const void* scales, int dtype, int64_t rows, int64_t cols,
                    void* out, hipStream_t stream);
int launch_swiglu_t(const void* in, int dtype, int64_t M, int64_t N, void* out, hipStream_t stream);
size_t moe_ffn_workspace(int64_t rows, int64_t hidden, int64_t inter, int num_experts);
int launch_moe_ffn(const void* x, const int64_t* rows_before_expert, const void* ffn1_codes,
                   const void* ffn1_bias, const void* ffn1_scale, const void* ffn2_codes,
                   const void* ffn2_scale, int dtype, int64_t rows, int64_t hidden, int64_t inter,
                   int num_experts, int bits, void* out, void* workspace, hipStream_t stream);
int launch_swiglu_f32(const float* in, int dtype, int64_t M, int64_t N, void* out, hipStream_t stream);
int launch_llm_int8_linear(const void* x, const void* weight, const void* bias, const float* wscale,
                           float threshold, int dtype, int64_t M, int64_t K, int64_t N, void* out,
                           void* workspace, hipStream_t stream);
// Scratch bytes launch_llm_int8_linear needs, and where its stages lie in them
// (ranges, outlier mask, outlier count, outlier list, activation codes, int32
// sums of the K runs or -1 when the GEMM writes the output itself, number of
// K runs: seven values).
size_t llm_int8_workspace(int64_t M, int64_t K, int64_t N);
void llm_int8_workspace_offsets(int64_t M, int64_t K, int64_t N, int64_t* offsets);
// Scratch bytes with which launch_linear_gemm splits K across workgroups (0: none needed).
size_t linear_gemm_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size);
bool linear_gemm_fuses_swiglu(int64_t M, int64_t K, int64_t N, int bits, int group_size);
bool linear_stream_fuses_swiglu(int64_t M, int64_t N);

inline int check_launch() {
  return hipGetLastError() == hipSuccess ? WOL_OK : WOL_ERR_HIP;
}

}  // namespace wol
