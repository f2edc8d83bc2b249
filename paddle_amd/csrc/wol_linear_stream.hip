// weight_only_linear for small M (decode): a bandwidth-bound kernel that
// streams the GFX950-packed weight once with 128-bit loads and feeds it to
// the matrix cores.
//
// One workgroup owns one strip of 16 output columns; its WK wavefronts split
// K between them.  A wavefront loads 16 bytes per lane (1 KiB per load, fully
// coalesced, one tile of 64 or 128 k), turns the biased codes into bf16/fp16
// bit patterns with AND-OR / byte-permute tricks (the code plus a constant
// offset, exact), and issues v_mfma_f32_16x16x32 with the activations as the
// A operand (rows >= M are zero) -- the MFMA does the multiply and the
// reduction over k across lanes.  The constant offset is removed by a second
// MFMA of the same A against a constant B, which is exact in fp32 up to the
// accumulator's rounding; accumulators restart every 64 k so the cancelling
// terms stay small.  Scales multiply the fp32 partial sums (once per group),
// never the weights, so nothing is rounded to T before the final cast.
// Partial sums of the WK wavefronts meet in LDS in a fixed order.
#include "wol_common.h"

namespace wol {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
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

// Codes of one k step (8 per lane) -> four dwords of T pairs holding
// code + offset exactly, and the B operand that cancels the offset.
//   int4/bf16: nibble | 0x4300      = 128 + (code + 8)      offset 136
//   int4/fp16: nibble<<4 | 0x5400   = 64 + (code + 8)       offset 72
//   int8/bf16: float(byte) high half = code + 128           offset 128
//   int8/fp16: byte | 0x6400        = 1024 + (code + 128)   offset 1152
template <int DT, int BITS>
struct Dequant;

template <>
struct Dequant<WOL_DTYPE_BF16, 4> {
  static constexpr uint32_t kCancel = 0xC308C308u;  // -136, -136
  __device__ static inline u32x4 run(const uint32_t* w) {
    const uint32_t v = w[0];
    u32x4 o;
    o.x = (v & 0x000F000Fu) | 0x43004300u;
    o.y = ((v >> 4) & 0x000F000Fu) | 0x43004300u;
    o.z = ((v >> 8) & 0x000F000Fu) | 0x43004300u;
    o.w = ((v >> 12) & 0x000F000Fu) | 0x43004300u;
    return o;
  }
};

template <>
struct Dequant<WOL_DTYPE_F16, 4> {
  static constexpr uint32_t kCancel = 0xD480D480u;  // -72, -72
  __device__ static inline u32x4 run(const uint32_t* w) {
    const uint32_t v = w[0];
    u32x4 o;
    o.x = ((v << 4) & 0x00F000F0u) | 0x54005400u;
    o.y = (v & 0x00F000F0u) | 0x54005400u;
    o.z = ((v >> 4) & 0x00F000F0u) | 0x54005400u;
    o.w = ((v >> 8) & 0x00F000F0u) | 0x54005400u;
    return o;
  }
};

template <>
struct Dequant<WOL_DTYPE_BF16, 8> {
  static constexpr uint32_t kCancel = 0xC300C300u;  // -128, -128
  __device__ static inline uint32_t pair(uint32_t lo_byte_val, uint32_t hi_byte_val) {
    // high halves of two fp32 values side by side (both are exact in bf16)
    return __builtin_amdgcn_perm(__float_as_uint(static_cast<float>(hi_byte_val)),
                                 __float_as_uint(static_cast<float>(lo_byte_val)), 0x07060302u);
  }
  __device__ static inline u32x4 run(const uint32_t* w) {
    u32x4 o;
    o.x = pair(w[0] & 0xFFu, (w[0] >> 8) & 0xFFu);
    o.y = pair((w[0] >> 16) & 0xFFu, w[0] >> 24);
    o.z = pair(w[1] & 0xFFu, (w[1] >> 8) & 0xFFu);
    o.w = pair((w[1] >> 16) & 0xFFu, w[1] >> 24);
    return o;
  }
};

template <>
struct Dequant<WOL_DTYPE_F16, 8> {
  static constexpr uint32_t kCancel = 0xE480E480u;  // -1152, -1152
  __device__ static inline u32x4 run(const uint32_t* w) {
    u32x4 o;
    o.x = __builtin_amdgcn_perm(w[0], 0x64646464u, 0x00050004u);
    o.y = __builtin_amdgcn_perm(w[0], 0x64646464u, 0x00070006u);
    o.z = __builtin_amdgcn_perm(w[1], 0x64646464u, 0x00050004u);
    o.w = __builtin_amdgcn_perm(w[1], 0x64646464u, 0x00070006u);
    return o;
  }
};

template <int DT, int BITS, int MT, int WK>
struct StreamKernel {
  static constexpr int kTileK = BITS == 8 ? 64 : 128;
  static constexpr int kSubs = kTileK / 64;         // 64-k sub-blocks per tile
  static constexpr int kDwPerStep = BITS == 8 ? 2 : 1;
  static constexpr int kUnroll = MT == 1 ? 4 : (MT == 2 ? 2 : 1);

  const uint16_t* x;
  const uint16_t* scale;
  int M;
  int64_t K, N;
  int group_size;
  int out_f32;
  int lane, j, kb;
  int64_t n;
  f32x4 tot[MT];

  __device__ inline u32x4 load_a(int mt, int64_t k) const {
    const int m = mt * 16 + j;
    u32x4 a = {0u, 0u, 0u, 0u};
    if (m < M) a = *reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(m) * K + k + 8 * kb);
    return a;
  }

  __device__ inline float load_scale(int64_t k) const {
    return to_f32<DT>(scale[(k / group_size) * N + n]);
  }

  // One 64-k sub-block: two k steps whose codes are in w[0 .. 2*kDwPerStep).
  __device__ inline void sub_block(const uint32_t* w, const u32x4 (&a)[2][MT], float s) {
    const u32x4 cancel = {Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel,
                          Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel};
    const u32x4 b0 = Dequant<DT, BITS>::run(w);
    const u32x4 b1 = Dequant<DT, BITS>::run(w + kDwPerStep);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      acc = mfma16<DT>(a[0][mt], b0, acc);
      acc = mfma16<DT>(a[0][mt], cancel, acc);
      acc = mfma16<DT>(a[1][mt], b1, acc);
      acc = mfma16<DT>(a[1][mt], cancel, acc);
      tot[mt] += acc * s;
    }
  }

  __device__ inline void run(const uint8_t* codes, const uint16_t* bias, void* out, float* red) {
    lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    j = lane & 15;
    kb = lane >> 4;
    const int64_t tn = blockIdx.x;
    n = tn * kStripCols + j;
    const uint8_t* strip = codes + tn * strip_bytes(K, BITS);
    const int ntile = static_cast<int>(K / kTileK);
    const int t0 = static_cast<int>(static_cast<int64_t>(ntile) * wave / WK);
    const int t1 = static_cast<int>(static_cast<int64_t>(ntile) * (wave + 1) / WK);
    const bool grouped = group_size > 0;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) tot[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const u32x4* tp = reinterpret_cast<const u32x4*>(strip) + lane;
    int t = t0;
    for (; t + kUnroll <= t1; t += kUnroll) {
      u32x4 wv[kUnroll];
      u32x4 av[kUnroll][kSubs][2][MT];
      float sv[kUnroll][kSubs];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) wv[u] = tp[static_cast<int64_t>(t + u) * 64];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int sb = 0; sb < kSubs; ++sb) {
          const int64_t k = static_cast<int64_t>(t + u) * kTileK + sb * 64;
          sv[u][sb] = grouped ? load_scale(k) : 1.0f;
#pragma unroll
          for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) av[u][sb][st][mt] = load_a(mt, k + 32 * st);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const uint32_t w[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
#pragma unroll
        for (int sb = 0; sb < kSubs; ++sb) sub_block(w + 2 * kDwPerStep * sb, av[u][sb], sv[u][sb]);
      }
    }
    for (; t < t1; ++t) {
      const u32x4 wv = tp[static_cast<int64_t>(t) * 64];
      const uint32_t w[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int sb = 0; sb < kSubs; ++sb) {
        const int64_t k = static_cast<int64_t>(t) * kTileK + sb * 64;
        u32x4 a[2][MT];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) a[st][mt] = load_a(mt, k + 32 * st);
        sub_block(w + 2 * kDwPerStep * sb, a, grouped ? load_scale(k) : 1.0f);
      }
    }
    if (BITS == 4 && (K % 128) != 0 && wave == WK - 1) {
      // half tile at the end of the strip: 8 bytes per lane, 64 k
      const int64_t k = static_cast<int64_t>(ntile) * 128;
      const u32x2 wv = *reinterpret_cast<const u32x2*>(strip + static_cast<int64_t>(ntile) * 1024 + lane * 8);
      const uint32_t w[2] = {wv.x, wv.y};
      u32x4 a[2][MT];
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[st][mt] = load_a(mt, k + 32 * st);
      sub_block(w, a, grouped ? load_scale(k) : 1.0f);
    }

    // Meet in LDS: red[wave][mt][r][lane], summed in wave order.
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[((wave * MT + mt) * 4 + r) * 64 + lane] = tot[mt][r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < MT * 256; idx += WK * 64) {
      const int mt = idx / 256, r = (idx % 256) / 64, l = idx % 64;
      float s = 0.0f;
#pragma unroll
      for (int w = 0; w < WK; ++w) s += red[((w * MT + mt) * 4 + r) * 64 + l];
      const int m = mt * 16 + (l / 16) * 4 + r;
      const int64_t nn = tn * kStripCols + (l % 16);
      if (m < M) {
        if (!grouped) s *= to_f32<DT>(scale[nn]);
        if (bias != nullptr) s += to_f32<DT>(bias[nn]);
        if (out_f32)
          static_cast<float*>(out)[static_cast<int64_t>(m) * N + nn] = s;
        else
          static_cast<uint16_t*>(out)[static_cast<int64_t>(m) * N + nn] = from_f32_rne<DT>(s);
      }
    }
  }
};

template <int DT, int BITS, int MT, int WK>
__global__ __launch_bounds__(WK * 64) void stream_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ codes,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ scale, void* __restrict__ out,
    int M, int64_t K, int64_t N, int group_size, int out_f32) {
  extern __shared__ float red[];
  StreamKernel<DT, BITS, MT, WK> k;
  k.x = x;
  k.scale = scale;
  k.M = M;
  k.K = K;
  k.N = N;
  k.group_size = group_size;
  k.out_f32 = out_f32;
  k.run(codes, bias, out, red);
}

struct Args {
  const void* x; const void* codes; const void* bias; const void* scale; void* out;
  int M; int64_t K, N; int group_size; int out_f32; hipStream_t stream;
};

template <int DT, int BITS, int MT, int WK>
void launch_one(const Args& a) {
  const size_t lds = static_cast<size_t>(WK) * MT * 256 * sizeof(float);
  stream_kernel<DT, BITS, MT, WK>
      <<<dim3(static_cast<unsigned>(a.N / kStripCols)), dim3(WK * 64), lds, a.stream>>>(
          static_cast<const uint16_t*>(a.x), static_cast<const uint8_t*>(a.codes),
          static_cast<const uint16_t*>(a.bias), static_cast<const uint16_t*>(a.scale), a.out, a.M,
          a.K, a.N, a.group_size, a.out_f32);
}

template <int DT, int BITS, int MT>
void launch_wk(const Args& a, int wk) {
  if (wk >= 16 && MT <= 2) launch_one<DT, BITS, MT, (MT <= 2 ? 16 : 8)>(a);
  else if (wk >= 8) launch_one<DT, BITS, MT, 8>(a);
  else if (wk >= 4) launch_one<DT, BITS, MT, 4>(a);
  else if (wk >= 2) launch_one<DT, BITS, MT, 2>(a);
  else launch_one<DT, BITS, MT, 1>(a);
}

template <int DT, int BITS>
void launch_mt(const Args& a, int wk) {
  const int mt = (a.M + 15) / 16;
  if (mt <= 1) launch_wk<DT, BITS, 1>(a, wk);
  else if (mt == 2) launch_wk<DT, BITS, 2>(a, wk);
  else if (mt == 3) launch_wk<DT, BITS, 3>(a, wk);
  else launch_wk<DT, BITS, 4>(a, wk);
}

template <int DT>
void launch_bits(const Args& a, int bits, int wk) {
  if (bits == 8) launch_mt<DT, 8>(a, wk);
  else launch_mt<DT, 4>(a, wk);
}

}  // namespace

// Wavefronts per workgroup: enough to put ~5 wavefronts on each of the 1024
// SIMDs, but no more than there are tiles along K.
static int pick_wk(int64_t K, int64_t N, int bits) {
  const int64_t strips = N / kStripCols;
  const int64_t ntile = K / (bits == 8 ? 64 : 128);
  int wk = 1;
  while (wk < 16 && strips * wk * 2 <= 6144 && wk * 2 <= ntile) wk *= 2;
  return wk;
}

int launch_linear_stream(const void* x, const void* codes, const void* bias, const void* scale,
                         int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                         void* out, bool out_f32, hipStream_t stream) {
  const Args a{x, codes, bias, scale, out, static_cast<int>(M), K, N, group_size, out_f32 ? 1 : 0, stream};
  const int wk = pick_wk(K, N, bits);
  if (dtype == WOL_DTYPE_BF16) launch_bits<WOL_DTYPE_BF16>(a, bits, wk);
  else launch_bits<WOL_DTYPE_F16>(a, bits, wk);
  return check_launch();
}

}  // namespace wol
