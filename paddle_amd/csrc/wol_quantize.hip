// weight_quantize, weight_dequantize and the layout re-packer for gfx950.
//
// All three work on blocks of 128 k x 64 n of the weight and pass the signed
// codes of a block through LDS (stage[r][c]); the layout-specific part is how
// the bytes of a block are enumerated in global memory (block_byte()).
//
// Quantisation arithmetic follows the reference's CPU kernel bit for bit
// (paddle/phi/kernels/impl/weight_quantize_kernel_impl.h:45-183):
//   amax  = max |w| over the column (group), compared in fp32
//   scale = cast_T(amax / bound)              bound = 127 (int8) | 7 (int4)
//   code  = clip(round_half_away(float(w) / float(scale)))
// including its corner cases: the per-channel maximum starts from the signed
// first element of the column (:49), NaN inputs never win a comparison, an
// all-zero column gives 0/0 = NaN which becomes code 127 (int8, through
// std::min/std::max :94-95) or -7 (int4, through the x86 float->int
// conversion :107).
#include <atomic>

#include "wol_common.h"

namespace wol {
namespace {

constexpr int kBlockK = 128;
constexpr int kBlockN = 64;
constexpr int kThreads = 256;

struct ByteRef {
  int64_t off;     // byte offset in the code tensor
  int r_lo, c_lo;  // block-local element in the low nibble (or the whole byte)
  int r_hi, c_hi;  // block-local element in the high nibble (int4 only)
};

// Number of code bytes a block of KR x NC elements owns.
__device__ inline int block_bytes(int bits, int KR, int NC) { return KR * NC * bits / 8; }

// The e-th byte (0 <= e < block_bytes) of block (k0, n0) in `layout`.
// Consecutive e are consecutive in memory within a run, so that neighbouring
// threads touch neighbouring bytes.
__device__ inline ByteRef block_byte(int layout, int bits, int64_t K, int64_t N, int64_t k0,
                                     int64_t n0, int KR, int NC, int e) {
  ByteRef b;
  if (layout == WOL_LAYOUT_CANONICAL) {
    if (bits == 8) {
      b.r_lo = e / NC; b.c_lo = e % NC; b.r_hi = b.r_lo; b.c_hi = b.c_lo;
      b.off = (k0 + b.r_lo) * N + n0 + b.c_lo;
    } else {
      const int half = NC / 2;
      b.r_lo = e / half; b.c_lo = 2 * (e % half); b.r_hi = b.r_lo; b.c_hi = b.c_lo + 1;
      b.off = (k0 + b.r_lo) * (N / 2) + n0 / 2 + e % half;
    }
  } else if (layout == WOL_LAYOUT_PADDLE_HIP) {
    if (bits == 8) {
      b.c_lo = e / KR; b.r_lo = e % KR; b.r_hi = b.r_lo; b.c_hi = b.c_lo;
      b.off = (n0 + b.c_lo) * K + k0 + b.r_lo;
    } else {
      const int cb = e / KR;
      b.r_lo = e % KR; b.c_lo = 2 * cb; b.r_hi = b.r_lo; b.c_hi = b.c_lo + 1;
      b.off = (n0 / 2 + cb) * K + k0 + b.r_lo;
    }
  } else {  // WOL_LAYOUT_GFX950
    const int per_strip = KR * kStripCols * bits / 8;
    const int s = e / per_strip;
    const int within_strip = e % per_strip;
    const int64_t strip0 = (n0 / kStripCols + s) * strip_bytes(K, bits);
    if (bits == 8) {
      const int t = within_strip / 1024, w = within_strip % 1024;
      const int lane = w / 16, b16 = w % 16;
      b.r_lo = t * 64 + (b16 / 8) * 32 + (lane / 16) * 8 + (b16 % 8);
      b.c_lo = s * 16 + lane % 16;
      b.r_hi = b.r_lo; b.c_hi = b.c_lo;
      b.off = strip0 + (k0 / 64) * 1024 + within_strip;
    } else {
      // k0 is a multiple of 128; KR == 128 is a full tile, KR == 64 the half tile.
      const int lane_bytes = KR == 128 ? 16 : 8;
      const int lane = within_strip / lane_bytes, bl = within_strip % lane_bytes;
      const int step = bl / 4, byte = bl % 4;
      const int p_lo = 2 * byte, p_hi = 2 * byte + 1;
      const int i_lo = p_lo < 4 ? 2 * p_lo : 2 * (p_lo - 4) + 1;
      const int i_hi = p_hi < 4 ? 2 * p_hi : 2 * (p_hi - 4) + 1;
      const int rbase = step * 32 + (lane / 16) * 8;
      b.r_lo = rbase + i_lo; b.r_hi = rbase + i_hi;
      b.c_lo = s * 16 + lane % 16; b.c_hi = b.c_lo;
      b.off = strip0 + (k0 / 128) * 1024 + within_strip;
    }
  }
  return b;
}

// LDS staging tile of signed codes; the +4 pad keeps column walks off one bank.
struct Stage {
  int8_t v[kBlockK][kBlockN + 4];
};

__device__ inline void store_block(const Stage& st, int layout, int bits, int64_t K, int64_t N,
                                   int64_t k0, int64_t n0, int KR, int NC, uint8_t* codes) {
  const int total = block_bytes(bits, KR, NC);
  for (int e = threadIdx.x; e < total; e += kThreads) {
    const ByteRef b = block_byte(layout, bits, K, N, k0, n0, KR, NC, e);
    int byte;
    if (bits == 8) {
      byte = encode_code(layout, 8, st.v[b.r_lo][b.c_lo]);
    } else {
      byte = encode_code(layout, 4, st.v[b.r_lo][b.c_lo]) |
             (encode_code(layout, 4, st.v[b.r_hi][b.c_hi]) << 4);
    }
    codes[b.off] = static_cast<uint8_t>(byte);
  }
}

__device__ inline void load_block(Stage& st, int layout, int bits, int64_t K, int64_t N,
                                  int64_t k0, int64_t n0, int KR, int NC, const uint8_t* codes) {
  const int total = block_bytes(bits, KR, NC);
  for (int e = threadIdx.x; e < total; e += kThreads) {
    const ByteRef b = block_byte(layout, bits, K, N, k0, n0, KR, NC, e);
    const int byte = codes[b.off];
    if (bits == 8) {
      st.v[b.r_lo][b.c_lo] = static_cast<int8_t>(decode_code(layout, 8, byte));
    } else {
      st.v[b.r_lo][b.c_lo] = static_cast<int8_t>(decode_code(layout, 4, byte & 0xF));
      st.v[b.r_hi][b.c_hi] = static_cast<int8_t>(decode_code(layout, 4, byte >> 4));
    }
  }
}

// Full blocks (128 k x 64 n) in the GFX950 layout move as whole 16-byte lane
// pieces: a piece is the 16 (int8) or 32 (int4) codes one lane of the
// consuming wavefront loads at once -- one column, rows as gfx950_offset()
// lays them out.  512 (int8) or 256 (int4) pieces per block.
template <int BITS>
__device__ inline void store_block_gfx950(const Stage& st, int64_t K, int64_t k0, int64_t n0,
                                          uint8_t* codes) {
  constexpr int kPieces = BITS == 8 ? 512 : 256;
  for (int q = threadIdx.x; q < kPieces; q += kThreads) {
    const int lane = q % 64, c = (BITS == 8 ? q / 128 : q / 64) * 16 + lane % 16;
    const int rb = (lane / 16) * 8;
    uint32_t d[4];
    int64_t off;
    if (BITS == 8) {
      const int t = (q / 64) % 2;
#pragma unroll
      for (int h = 0; h < 4; ++h) {  // dword h: k step h / 2, bytes 4 * (h % 2) ..
        uint32_t v = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = t * 64 + (h / 2) * 32 + rb + 4 * (h % 2) + e;
          v |= static_cast<uint32_t>((st.v[r][c] + 128) & 0xFF) << (8 * e);
        }
        d[h] = v;
      }
      off = (n0 / kStripCols + q / 128) * strip_bytes(K, 8) + (k0 / 64 + t) * 1024 + lane * 16;
    } else {
#pragma unroll
      for (int step = 0; step < 4; ++step) {
        uint32_t v = 0;
#pragma unroll
        for (int pn = 0; pn < 8; ++pn) {
          const int i = pn < 4 ? 2 * pn : 2 * (pn - 4) + 1;
          v |= static_cast<uint32_t>((st.v[step * 32 + rb + i][c] + 8) & 0xF) << (4 * pn);
        }
        d[step] = v;
      }
      off = (n0 / kStripCols + q / 64) * strip_bytes(K, 4) + (k0 / 128) * 1024 + lane * 16;
    }
    *reinterpret_cast<uint4*>(codes + off) = make_uint4(d[0], d[1], d[2], d[3]);
  }
}

template <int BITS>
__device__ inline void load_block_gfx950(Stage& st, int64_t K, int64_t k0, int64_t n0,
                                         const uint8_t* codes) {
  constexpr int kPieces = BITS == 8 ? 512 : 256;
  for (int q = threadIdx.x; q < kPieces; q += kThreads) {
    const int lane = q % 64, c = (BITS == 8 ? q / 128 : q / 64) * 16 + lane % 16;
    const int rb = (lane / 16) * 8;
    if (BITS == 8) {
      const int t = (q / 64) % 2;
      const int64_t off = (n0 / kStripCols + q / 128) * strip_bytes(K, 8) + (k0 / 64 + t) * 1024 + lane * 16;
      const uint4 v = *reinterpret_cast<const uint4*>(codes + off);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int h = 0; h < 4; ++h)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          st.v[t * 64 + (h / 2) * 32 + rb + 4 * (h % 2) + e][c] =
              static_cast<int8_t>(static_cast<int>((d[h] >> (8 * e)) & 0xFF) - 128);
    } else {
      const int64_t off = (n0 / kStripCols + q / 64) * strip_bytes(K, 4) + (k0 / 128) * 1024 + lane * 16;
      const uint4 v = *reinterpret_cast<const uint4*>(codes + off);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int step = 0; step < 4; ++step)
#pragma unroll
        for (int pn = 0; pn < 8; ++pn) {
          const int i = pn < 4 ? 2 * pn : 2 * (pn - 4) + 1;
          st.v[step * 32 + rb + i][c] = static_cast<int8_t>(static_cast<int>((d[step] >> (4 * pn)) & 0xF) - 8);
        }
    }
  }
}

union Pack8 {
  uint4 q;
  uint16_t h[8];
};

// Column-wise |w| maximum for the per-channel case: one block reduces
// 256 k x 64 n and merges with an integer atomic max (non-negative floats
// order like their bit patterns).  amax must be zero before the launch.
template <int DT>
__global__ __launch_bounds__(kThreads) void amax_kernel(const uint16_t* __restrict__ w, int64_t K,
                                                        int64_t N, uint32_t* __restrict__ amax) {
  __shared__ float part[32][kBlockN];
  const int tx = threadIdx.x % 8, ty = threadIdx.x / 8;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kBlockN;
  const int64_t k0 = static_cast<int64_t>(blockIdx.y) * 256;
  const int64_t kend = k0 + 256 < K ? k0 + 256 : K;
  const int64_t n = n0 + tx * 8;
  float mx[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) mx[c] = 0.0f;
  if (n < N) {
    for (int64_t k = k0 + ty; k < kend; k += 32) {
      Pack8 p;
      p.q = *reinterpret_cast<const uint4*>(w + k * N + n);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const float f = to_f32<DT>(p.h[c]);
        const float a = f < 0.0f ? -f : f;  // the reference's xabs
        mx[c] = a > mx[c] ? a : mx[c];      // NaN never wins
      }
    }
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) part[ty][tx * 8 + c] = mx[c];
  __syncthreads();
  if (threadIdx.x < kBlockN && n0 + threadIdx.x < N) {
    float m = 0.0f;
    for (int r = 0; r < 32; ++r) m = part[r][threadIdx.x] > m ? part[r][threadIdx.x] : m;
    atomicMax(amax + n0 + threadIdx.x, __float_as_uint(m));
  }
}

__global__ void zero_u32_kernel(uint32_t* p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

template <int BITS>
__device__ inline int quant_code(float w, float s) {
  const float r = roundf(w / s);  // IEEE divide, halves away from zero
  if (BITS == 8) {
    const float lo = (r < 127.0f) ? r : 127.0f;       // std::min(127.f, r): NaN -> 127
    const float cl = (-127.0f < lo) ? lo : -127.0f;   // std::max(-127.f, lo)
    return static_cast<int>(cl);
  }
  // float -> int of NaN / inf / out of range gives INT_MIN on x86, hence -7.
  const int v = (r >= -2147483648.0f && r < 2147483648.0f) ? static_cast<int>(r) : INT32_MIN;
  const int lo = v < 7 ? v : 7;
  return lo > -7 ? lo : -7;
}

// One block quantises 128 k x 64 n.  GROUPS is the number of scale groups the
// block spans along k: 0 = per-channel (scale from the amax workspace),
// 1 = group 128, 2 = group 64.
template <int DT, int BITS>
__global__ __launch_bounds__(kThreads) void quantize_kernel(
    const uint16_t* __restrict__ w, int64_t K, int64_t N, int group_size, int round_mode,
    int layout, const uint32_t* __restrict__ amax, uint8_t* __restrict__ codes,
    void* __restrict__ scale_out, int scale_f32) {
  // scale_f32: the "llm.int8" flavour -- the scale stays the fp32 quotient
  // (paddle/phi/kernels/cpu/weight_quantize_kernel.cc:163-166, ScaleT = float)
  uint16_t* scale = static_cast<uint16_t*>(scale_out);
  float* scale32 = static_cast<float*>(scale_out);
  __shared__ Stage st;
  __shared__ float part[2][32][kBlockN];
  __shared__ float sc[2][kBlockN];

  const int tx = threadIdx.x % 8, ty = threadIdx.x / 8;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kBlockN;
  const int64_t k0 = static_cast<int64_t>(blockIdx.y) * kBlockK;
  const int KR = static_cast<int>(K - k0 < kBlockK ? K - k0 : kBlockK);
  const int NC = static_cast<int>(N - n0 < kBlockN ? N - n0 : kBlockN);
  const float bound = BITS == 8 ? 127.0f : 7.0f;
  const bool col_ok = tx * 8 < NC;

  float f[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty + 32 * i;
    if (col_ok && r < KR) {
      Pack8 p;
      p.q = *reinterpret_cast<const uint4*>(w + (k0 + r) * N + n0 + tx * 8);
#pragma unroll
      for (int c = 0; c < 8; ++c) f[i][c] = to_f32<DT>(p.h[c]);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) f[i][c] = 0.0f;
    }
  }

  // rows [0,64) are i = 0,1 and rows [64,128) are i = 2,3
  const int ngroups = group_size == 64 ? 2 : 1;
  if (group_size > 0) {
#pragma unroll
    for (int g = 0; g < 2; ++g) {
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float m = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const bool mine = group_size == 64 ? (i / 2 == g) : (g == 0);
          const float a = f[i][c] < 0.0f ? -f[i][c] : f[i][c];
          if (mine) m = a > m ? a : m;
        }
        part[g][ty][tx * 8 + c] = m;
      }
    }
    __syncthreads();
    if (threadIdx.x < 2 * kBlockN) {
      const int g = threadIdx.x / kBlockN, c = threadIdx.x % kBlockN;
      if (g < ngroups && c < NC && g * 64 < KR) {
        float m = 0.0f;
        for (int r = 0; r < 32; ++r) m = part[g][r][c] > m ? part[g][r][c] : m;
        const int64_t si = (k0 / group_size + g) * N + n0 + c;
        if (scale_f32) {
          scale32[si] = m / bound;
          sc[g][c] = m / bound;
        } else {
          const uint16_t sb = from_f32<DT>(m / bound, round_mode);
          scale[si] = sb;
          sc[g][c] = to_f32<DT>(sb);
        }
      }
    }
  } else {
    if (threadIdx.x < NC) {
      const int c = threadIdx.x;
      // The reference starts the maximum from the signed first element, so a
      // NaN there poisons the scale and an all-zero column keeps its sign.
      const float v0 = to_f32<DT>(w[n0 + c]);
      const float m = __uint_as_float(amax[n0 + c]);
      const float src = (v0 != v0) ? v0 : (m == 0.0f ? (v0 < 0.0f ? m : v0) : m);
      if (scale_f32) {
        if (k0 == 0) scale32[n0 + c] = src / bound;
        sc[0][c] = src / bound;
      } else {
        const uint16_t sb = from_f32<DT>(src / bound, round_mode);
        if (k0 == 0) scale[n0 + c] = sb;
        sc[0][c] = to_f32<DT>(sb);
      }
    }
  }
  __syncthreads();

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty + 32 * i;
    if (col_ok && r < KR) {
      const int g = group_size == 64 ? i / 2 : 0;
#pragma unroll
      for (int c = 0; c < 8; ++c)
        st.v[r][tx * 8 + c] = static_cast<int8_t>(quant_code<BITS>(f[i][c], sc[g][tx * 8 + c]));
    }
  }
  __syncthreads();
  if (layout == WOL_LAYOUT_GFX950 && KR == kBlockK && NC == kBlockN)
    store_block_gfx950<BITS>(st, K, k0, n0, codes);
  else
    store_block(st, layout, BITS, K, N, k0, n0, KR, NC, codes);
}

// out[k,n] = cast_T(float(code) * float(scale)), written as [K,N] rows.
template <int DT, int BITS>
__global__ __launch_bounds__(kThreads) void dequantize_kernel(
    const uint8_t* __restrict__ codes, int layout, const uint16_t* __restrict__ scale, int64_t K,
    int64_t N, int group_size, uint16_t* __restrict__ out) {
  __shared__ Stage st;
  const int tx = threadIdx.x % 8, ty = threadIdx.x / 8;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kBlockN;
  const int64_t k0 = static_cast<int64_t>(blockIdx.y) * kBlockK;
  const int KR = static_cast<int>(K - k0 < kBlockK ? K - k0 : kBlockK);
  const int NC = static_cast<int>(N - n0 < kBlockN ? N - n0 : kBlockN);
  if (layout == WOL_LAYOUT_GFX950 && KR == kBlockK && NC == kBlockN)
    load_block_gfx950<BITS>(st, K, k0, n0, codes);
  else
    load_block(st, layout, BITS, K, N, k0, n0, KR, NC, codes);
  __syncthreads();
  if (tx * 8 >= NC) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty + 32 * i;
    if (r >= KR) continue;
    const int64_t k = k0 + r;
    const uint16_t* srow = group_size > 0 ? scale + (k / group_size) * N : scale;
    Pack8 s, o;
    s.q = *reinterpret_cast<const uint4*>(srow + n0 + tx * 8);
#pragma unroll
    for (int c = 0; c < 8; ++c)
      o.h[c] = from_f32_rne<DT>(static_cast<float>(st.v[r][tx * 8 + c]) * to_f32<DT>(s.h[c]));
    *reinterpret_cast<uint4*>(out + k * N + n0 + tx * 8) = o.q;
  }
}

template <int BITS>
__global__ __launch_bounds__(kThreads) void repack_kernel(const uint8_t* __restrict__ in,
                                                          int layout_in, uint8_t* __restrict__ out,
                                                          int layout_out, int64_t K, int64_t N) {
  __shared__ Stage st;
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * kBlockN;
  const int64_t k0 = static_cast<int64_t>(blockIdx.y) * kBlockK;
  const int KR = static_cast<int>(K - k0 < kBlockK ? K - k0 : kBlockK);
  const int NC = static_cast<int>(N - n0 < kBlockN ? N - n0 : kBlockN);
  const bool full = KR == kBlockK && NC == kBlockN;
  if (layout_in == WOL_LAYOUT_GFX950 && full)
    load_block_gfx950<BITS>(st, K, k0, n0, in);
  else
    load_block(st, layout_in, BITS, K, N, k0, n0, KR, NC, in);
  __syncthreads();
  if (layout_out == WOL_LAYOUT_GFX950 && full)
    store_block_gfx950<BITS>(st, K, k0, n0, out);
  else
    store_block(st, layout_out, BITS, K, N, k0, n0, KR, NC, out);
}

inline dim3 block_grid(int64_t K, int64_t N) {
  return dim3(static_cast<unsigned>((N + kBlockN - 1) / kBlockN),
              static_cast<unsigned>((K + kBlockK - 1) / kBlockK));
}

}  // namespace

int launch_quantize(const void* w, int dtype, int64_t K, int64_t N, int bits, int group_size,
                    int round_mode, int layout, void* codes, void* scale, bool scale_f32,
                    void* workspace, hipStream_t stream) {
  const uint16_t* wp = static_cast<const uint16_t*>(w);
  uint32_t* amax = static_cast<uint32_t*>(workspace);
  if (group_size == -1) {
    zero_u32_kernel<<<dim3(static_cast<unsigned>((N + 255) / 256)), dim3(256), 0, stream>>>(amax, N);
    const dim3 g(static_cast<unsigned>((N + kBlockN - 1) / kBlockN),
                 static_cast<unsigned>((K + 255) / 256));
    if (dtype == WOL_DTYPE_BF16)
      amax_kernel<WOL_DTYPE_BF16><<<g, dim3(kThreads), 0, stream>>>(wp, K, N, amax);
    else
      amax_kernel<WOL_DTYPE_F16><<<g, dim3(kThreads), 0, stream>>>(wp, K, N, amax);
  }
  const dim3 grid = block_grid(K, N);
  uint8_t* cp = static_cast<uint8_t*>(codes);
  const int sf = scale_f32 ? 1 : 0;
#define WOL_Q(DT, B)                                                                   \
  quantize_kernel<DT, B><<<grid, dim3(kThreads), 0, stream>>>(wp, K, N, group_size,   \
                                                              round_mode, layout, amax, cp, scale, sf)
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) WOL_Q(WOL_DTYPE_BF16, 8); else WOL_Q(WOL_DTYPE_BF16, 4);
  } else {
    if (bits == 8) WOL_Q(WOL_DTYPE_F16, 8); else WOL_Q(WOL_DTYPE_F16, 4);
  }
#undef WOL_Q
  return check_launch();
}

// ---------------------------------------------------------------------------
// The entry point for callers that cannot allocate (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc): the per-channel
// abs-max buffer lives in a file-scope device array instead of a caller's
// workspace.  Every GPU holds its own copy of the array at its own address,
// resolved once per device with that device current; host code only ever uses
// the resolved pointer, never the array's name.
// ---------------------------------------------------------------------------
constexpr int kStaticDevices = 64;
static __device__ __align__(256) uint32_t scratch[kQuantizeStaticMaxN];
static std::atomic<uint32_t*> scratch_ptr[kStaticDevices];

int launch_quantize_static(const void* w, int dtype, int64_t K, int64_t N, int bits, int group_size,
                           int round_mode, int layout, void* codes, void* scale,
                           hipStream_t stream) {
  uint32_t* amax = nullptr;
  if (group_size == -1) {  // group-wise scales need no scratch at all
    if (N > kQuantizeStaticMaxN) return WOL_ERR_BAD_SHAPE;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticDevices) return WOL_ERR_NO_DEVICE;
    amax = scratch_ptr[dev].load(std::memory_order_acquire);
    if (amax == nullptr) {
      void* p = nullptr;
      if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        return WOL_ERR_HIP;
      }
      amax = static_cast<uint32_t*>(p);
      scratch_ptr[dev].store(amax, std::memory_order_release);  // every thread resolves the same address
    }
  }
  // launch_quantize clears the first N words with a fill kernel before the
  // abs-max pass, so what an earlier call left behind does not matter
  return launch_quantize(w, dtype, K, N, bits, group_size, round_mode, layout, codes, scale, false,
                         amax, stream);
}

int launch_dequantize(const void* codes, int layout, const void* scale, int dtype, int64_t K,
                      int64_t N, int bits, int group_size, void* out, hipStream_t stream) {
  const dim3 grid = block_grid(K, N);
  const uint8_t* cp = static_cast<const uint8_t*>(codes);
  const uint16_t* sp = static_cast<const uint16_t*>(scale);
  uint16_t* op = static_cast<uint16_t*>(out);
#define WOL_DQ(DT, B) \
  dequantize_kernel<DT, B><<<grid, dim3(kThreads), 0, stream>>>(cp, layout, sp, K, N, group_size, op)
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) WOL_DQ(WOL_DTYPE_BF16, 8); else WOL_DQ(WOL_DTYPE_BF16, 4);
  } else {
    if (bits == 8) WOL_DQ(WOL_DTYPE_F16, 8); else WOL_DQ(WOL_DTYPE_F16, 4);
  }
#undef WOL_DQ
  return check_launch();
}

int launch_repack(const void* in, int layout_in, void* out, int layout_out, int64_t K, int64_t N,
                  int bits, hipStream_t stream) {
  const dim3 grid = block_grid(K, N);
  const uint8_t* ip = static_cast<const uint8_t*>(in);
  uint8_t* op = static_cast<uint8_t*>(out);
  if (bits == 8)
    repack_kernel<8><<<grid, dim3(kThreads), 0, stream>>>(ip, layout_in, op, layout_out, K, N);
  else
    repack_kernel<4><<<grid, dim3(kThreads), 0, stream>>>(ip, layout_in, op, layout_out, K, N);
  return check_launch();
}

}  // namespace wol
