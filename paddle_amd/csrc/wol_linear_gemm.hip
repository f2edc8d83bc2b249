// weight_only_linear for large M (prefill): an MFMA GEMM.
//
// A workgroup of four wavefronts (2 x 2) computes a BM x BN tile of the
// output.  The activations of a k tile are staged in LDS (padded rows, read
// back as 16x16x32 A fragments); the packed weights need no staging because
// the GFX950 layout already stores them in B-fragment order: every lane loads
// its 16 bytes for a strip straight from global memory and dequantises them in
// registers to exact signed bf16/fp16 integers.  Scales are applied to fp32
// accumulators -- in the epilogue (per-channel) or once per 64-k sub-block
// (group-wise) -- so the product code*scale is never rounded to T.
#include "wol_common.h"

namespace wol {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int DT>
__device__ inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  if (DT == WOL_DTYPE_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

__device__ inline uint32_t pack_bf16_hi(float lo, float hi) {
  // both values are small integers, exact in bf16: keep the high halves
  return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

__device__ inline uint32_t f16x2_add(uint32_t v, uint32_t c) {
  const f16x2 r = __builtin_bit_cast(f16x2, v) + __builtin_bit_cast(f16x2, c);
  return __builtin_bit_cast(uint32_t, r);
}

// Codes of one k step (8 per lane) -> four dwords of T pairs holding the exact
// signed code.
template <int DT, int BITS>
struct DequantExact;

template <>
struct DequantExact<WOL_DTYPE_BF16, 8> {
  __device__ static inline u32x4 run(const uint32_t* w) {
    u32x4 o;
    o.x = pack_bf16_hi(static_cast<float>(w[0] & 0xFFu) - 128.0f,
                       static_cast<float>((w[0] >> 8) & 0xFFu) - 128.0f);
    o.y = pack_bf16_hi(static_cast<float>((w[0] >> 16) & 0xFFu) - 128.0f,
                       static_cast<float>(w[0] >> 24) - 128.0f);
    o.z = pack_bf16_hi(static_cast<float>(w[1] & 0xFFu) - 128.0f,
                       static_cast<float>((w[1] >> 8) & 0xFFu) - 128.0f);
    o.w = pack_bf16_hi(static_cast<float>((w[1] >> 16) & 0xFFu) - 128.0f,
                       static_cast<float>(w[1] >> 24) - 128.0f);
    return o;
  }
};

template <>
struct DequantExact<WOL_DTYPE_F16, 8> {
  __device__ static inline u32x4 run(const uint32_t* w) {
    u32x4 o;  // byte | 0x6400 = 1024 + byte, minus 1152 = code
    o.x = f16x2_add(__builtin_amdgcn_perm(w[0], 0x64646464u, 0x00050004u), 0xE480E480u);
    o.y = f16x2_add(__builtin_amdgcn_perm(w[0], 0x64646464u, 0x00070006u), 0xE480E480u);
    o.z = f16x2_add(__builtin_amdgcn_perm(w[1], 0x64646464u, 0x00050004u), 0xE480E480u);
    o.w = f16x2_add(__builtin_amdgcn_perm(w[1], 0x64646464u, 0x00070006u), 0xE480E480u);
    return o;
  }
};

template <>
struct DequantExact<WOL_DTYPE_F16, 4> {
  __device__ static inline u32x4 run(const uint32_t* w) {
    const uint32_t v = w[0];
    u32x4 o;  // nibble<<4 | 0x5400 = 64 + nibble, minus 72 = code
    o.x = f16x2_add(((v << 4) & 0x00F000F0u) | 0x54005400u, 0xD480D480u);
    o.y = f16x2_add((v & 0x00F000F0u) | 0x54005400u, 0xD480D480u);
    o.z = f16x2_add(((v >> 4) & 0x00F000F0u) | 0x54005400u, 0xD480D480u);
    o.w = f16x2_add(((v >> 8) & 0x00F000F0u) | 0x54005400u, 0xD480D480u);
    return o;
  }
};

template <>
struct DequantExact<WOL_DTYPE_BF16, 4> {
  __device__ static inline uint32_t fix(uint32_t pair) {
    // pair = two bf16 holding 136 + code; widen, subtract, narrow (all exact)
    const float lo = __uint_as_float(pair << 16) - 136.0f;
    const float hi = __uint_as_float(pair & 0xFFFF0000u) - 136.0f;
    return pack_bf16_hi(lo, hi);
  }
  __device__ static inline u32x4 run(const uint32_t* w) {
    const uint32_t v = w[0];
    u32x4 o;
    o.x = fix((v & 0x000F000Fu) | 0x43004300u);
    o.y = fix(((v >> 4) & 0x000F000Fu) | 0x43004300u);
    o.z = fix(((v >> 8) & 0x000F000Fu) | 0x43004300u);
    o.w = fix(((v >> 12) & 0x000F000Fu) | 0x43004300u);
    return o;
  }
};

constexpr int kThreads = 256;

template <int DT, int BITS, bool GROUPED, int WMT, int WNT>
__global__ __launch_bounds__(kThreads) void gemm_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ codes,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ scale, void* __restrict__ out,
    int64_t M, int64_t K, int64_t N, int group_size, int out_f32) {
  constexpr int BM = 32 * WMT, BN = 32 * WNT;
  constexpr int TK = BITS == 8 ? 64 : 128;    // k per 16-byte lane load
  constexpr int kDwPerStep = BITS == 8 ? 2 : 1;
  constexpr int kRow = TK + 8;                // padded LDS row, in elements
  __shared__ __attribute__((aligned(16))) uint16_t As[BM * kRow];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int j = lane & 15, kb = lane >> 4;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int64_t strip0 = static_cast<int64_t>(blockIdx.x) * (BN / 16) + wn * WNT;
  const int64_t nstrips = N / kStripCols;

  f32x4 tot[WMT][WNT];
#pragma unroll
  for (int a = 0; a < WMT; ++a)
#pragma unroll
    for (int b = 0; b < WNT; ++b) tot[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int64_t nfull = K / TK;
  const int64_t niter = nfull + ((K % TK) ? 1 : 0);
  for (int64_t it = 0; it < niter; ++it) {
    const int64_t k0 = it * TK;
    const int kw = static_cast<int>(K - k0 < TK ? K - k0 : TK);  // 128 or 64 (int4 tail)
    __syncthreads();
    // stage the activations of this k tile: BM rows of kw elements
    for (int c = threadIdx.x; c < BM * (TK / 8); c += kThreads) {
      const int r = c / (TK / 8), cc = c % (TK / 8);
      u32x4 v = {0u, 0u, 0u, 0u};
      if (m0 + r < M && cc * 8 < kw)
        v = *reinterpret_cast<const u32x4*>(x + (m0 + r) * K + k0 + cc * 8);
      *reinterpret_cast<u32x4*>(&As[r * kRow + cc * 8]) = v;
    }
    // this lane's weights: one 16-byte load per strip (8 bytes in the int4 half tile)
    uint32_t wv[WNT][4];
#pragma unroll
    for (int s = 0; s < WNT; ++s) {
      wv[s][0] = wv[s][1] = wv[s][2] = wv[s][3] = BITS == 8 ? 0x80808080u : 0x88888888u;
      if (strip0 + s < nstrips) {
        const uint8_t* sp = codes + (strip0 + s) * strip_bytes(K, BITS);
        if (kw == TK) {
          const u32x4 q = *reinterpret_cast<const u32x4*>(sp + it * 1024 + lane * 16);
          wv[s][0] = q.x; wv[s][1] = q.y; wv[s][2] = q.z; wv[s][3] = q.w;
        } else {
          const u32x2 q = *reinterpret_cast<const u32x2*>(sp + nfull * 1024 + lane * 8);
          wv[s][0] = q.x; wv[s][1] = q.y;
        }
      }
    }
    __syncthreads();
    const int nsub = kw / 64;
#pragma unroll
    for (int sb = 0; sb < TK / 64; ++sb) {
      if (sb >= nsub) break;
      f32x4 part[WMT][WNT];
      if (GROUPED) {
#pragma unroll
        for (int a = 0; a < WMT; ++a)
#pragma unroll
          for (int b = 0; b < WNT; ++b) part[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const int step = sb * 2 + st;
        u32x4 bfrag[WNT];
#pragma unroll
        for (int s = 0; s < WNT; ++s) bfrag[s] = DequantExact<DT, BITS>::run(&wv[s][step * kDwPerStep]);
#pragma unroll
        for (int a = 0; a < WMT; ++a) {
          const int row = (wm * WMT + a) * 16 + j;
          const u32x4 af = *reinterpret_cast<const u32x4*>(&As[row * kRow + step * 32 + kb * 8]);
#pragma unroll
          for (int s = 0; s < WNT; ++s) {
            if (GROUPED) part[a][s] = mfma16<DT>(af, bfrag[s], part[a][s]);
            else tot[a][s] = mfma16<DT>(af, bfrag[s], tot[a][s]);
          }
        }
      }
      if (GROUPED) {
        const int64_t g = (k0 + sb * 64) / group_size;
#pragma unroll
        for (int s = 0; s < WNT; ++s) {
          float sc = 0.0f;
          if (strip0 + s < nstrips) sc = to_f32<DT>(scale[g * N + (strip0 + s) * 16 + j]);
#pragma unroll
          for (int a = 0; a < WMT; ++a) tot[a][s] += part[a][s] * sc;
        }
      }
    }
  }

#pragma unroll
  for (int s = 0; s < WNT; ++s) {
    if (strip0 + s >= nstrips) continue;
    const int64_t n = (strip0 + s) * 16 + j;
    const float sc = GROUPED ? 1.0f : to_f32<DT>(scale[n]);
    const float bv = bias != nullptr ? to_f32<DT>(bias[n]) : 0.0f;
#pragma unroll
    for (int a = 0; a < WMT; ++a) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t m = m0 + (wm * WMT + a) * 16 + kb * 4 + r;
        if (m >= M) continue;
        const float v = tot[a][s][r] * sc + bv;
        if (out_f32) static_cast<float*>(out)[m * N + n] = v;
        else static_cast<uint16_t*>(out)[m * N + n] = from_f32_rne<DT>(v);
      }
    }
  }
}

struct Args {
  const void* x; const void* codes; const void* bias; const void* scale; void* out;
  int64_t M, K, N; int group_size; int out_f32; hipStream_t stream;
};

template <int DT, int BITS, bool GROUPED, int WMT, int WNT>
void launch_one(const Args& a) {
  constexpr int BM = 32 * WMT, BN = 32 * WNT;
  const dim3 grid(static_cast<unsigned>((a.N + BN - 1) / BN), static_cast<unsigned>((a.M + BM - 1) / BM));
  gemm_kernel<DT, BITS, GROUPED, WMT, WNT><<<grid, dim3(kThreads), 0, a.stream>>>(
      static_cast<const uint16_t*>(a.x), static_cast<const uint8_t*>(a.codes),
      static_cast<const uint16_t*>(a.bias), static_cast<const uint16_t*>(a.scale), a.out, a.M, a.K,
      a.N, a.group_size, a.out_f32);
}

template <int DT, int BITS>
void launch_cfg(const Args& a) {
  if (a.group_size > 0) launch_one<DT, BITS, true, 4, 4>(a);
  else launch_one<DT, BITS, false, 4, 4>(a);
}

}  // namespace

int launch_linear_gemm(const void* x, const void* codes, const void* bias, const void* scale,
                       int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                       void* out, bool out_f32, hipStream_t stream) {
  const Args a{x, codes, bias, scale, out, M, K, N, group_size, out_f32 ? 1 : 0, stream};
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) launch_cfg<WOL_DTYPE_BF16, 8>(a); else launch_cfg<WOL_DTYPE_BF16, 4>(a);
  } else {
    if (bits == 8) launch_cfg<WOL_DTYPE_F16, 8>(a); else launch_cfg<WOL_DTYPE_F16, 4>(a);
  }
  return check_launch();
}

}  // namespace wol
