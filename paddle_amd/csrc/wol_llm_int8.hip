// llm_int8_linear for gfx950: dynamic per-row int8 quantisation of the
// activations, an int8 x int8 -> int32 MFMA GEMM against the plain [N,K] int8
// weight that weight_quantize(algo="llm.int8") returns, the outlier columns in
// T x dequantised-weight arithmetic, and the merge of the two.
//
// Stages (paddle/phi/kernels/impl/llm_int8_matmul_kernel_impl.h:560-690 runs
// the same ones as separate kernels plus two library GEMMs and a device-to-host
// copy of the outlier count; here nothing returns to the host):
//   rowmax  : range[m] = max |x[m,k]| over the elements not above the
//             threshold; bit k set where any |x[m,k]| > threshold
//             (ReduceAbsMaxKernel, :221-268), per workgroup in LDS
//   mask    : ORs the workgroups' bits into the mask
//   quant   : qx = 0 in outlier columns, else clip(round(x * 127 * (1/range)))
//             (QuantActKernel :270-303, QuantFunc :153-164); one extra
//             workgroup turns the mask into an ascending list of columns
//             (one or two rows: these three as one single-workgroup kernel)
//   outlier : sub = T(sum over the outlier columns of x * T(w * wscale)), fp32
//             sum in ascending column order; leaves at once without outliers
//   gemm    : acc = qx . w^T in int32 on v_mfma_i32_32x32x32_i8, both operands
//             through direct-to-LDS loads, two or three k tiles deep.  The
//             epilogue is DequantMergeKernel (:415-447): out = T( sub + T(acc *
//             range * wscale / 127) ), then T(out + bias).
//   merge   : only when K is cut into runs (few rows): every run leaves its
//             int32 sums in a slab of its own and this kernel adds them (exact,
//             so the result does not depend on the cut) and applies the same
//             epilogue.
#include <atomic>

#include "wol_common.h"

namespace wol {
namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;


template <int N_>
__device__ inline void wait_vmcnt() {
  // gfx9 encoding: vmcnt = [15:14][3:0], expcnt = [6:4], lgkmcnt = [11:8]
  __builtin_amdgcn_s_waitcnt((N_ & 0xF) | ((N_ >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// ---------------------------------------------------------------------------
// activation side
// ---------------------------------------------------------------------------
// Row ranges and outlier bits.  A workgroup takes a run of rows, four at a time,
// and a thread the same columns of each (16-byte loads); the outlier bits of
// the run are ORed in an LDS mask and leave as the workgroup's own row of
// `part` -- no global atomics: device-wide atomics on one word serialise at
// 100-150 ns each across the XCDs, and outlier columns are the same in most
// rows (with them this kernel took 15 us for 2048 rows x 4096).  The mask
// kernel below ORs the rows of `part`.
constexpr int kRowChunk = 4;
constexpr int kMaxRowGroups = 512;

template <int DT>
__global__ __launch_bounds__(256) void llm_rowmax_kernel(const uint16_t* __restrict__ x, float threshold, int M,
                                                         int K, int rows_per_group, float* __restrict__ ranges,
                                                         uint32_t* __restrict__ part) {
  extern __shared__ uint32_t smask[];  // K / 32 words
  __shared__ float red[4][kRowChunk];
  const float thr = to_f32<DT>(from_f32_rne<DT>(threshold));  // the comparison is made in T
  const int nwords = K / 32;
  for (int w = threadIdx.x; w < nwords; w += 256) smask[w] = 0u;
  __syncthreads();
  const int m_begin = blockIdx.x * rows_per_group;
  const int m_end = m_begin + rows_per_group < M ? m_begin + rows_per_group : M;
  for (int m0 = m_begin; m0 < m_end; m0 += kRowChunk) {
    float mx[kRowChunk];
#pragma unroll
    for (int r = 0; r < kRowChunk; ++r) mx[r] = 0.0f;
    for (int k0 = threadIdx.x * 8; k0 < K; k0 += 256 * 8) {
      u32x4 v[kRowChunk];
#pragma unroll
      for (int r = 0; r < kRowChunk; ++r) {
        const int m = m0 + r < m_end ? m0 + r : m_end - 1;  // past the end: the last row again
        v[r] = *reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(m) * K + k0);
      }
      uint32_t bits = 0;
#pragma unroll
      for (int r = 0; r < kRowChunk; ++r) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float a = fabsf(to_f32<DT>(static_cast<uint16_t>(v[r][i >> 1] >> (16 * (i & 1)))));
          if (a > thr) {
            bits |= 1u << i;
            a = 0.0f;
          }
          mx[r] = a > mx[r] ? a : mx[r];
        }
      }
      if (bits != 0) atomicOr(&smask[k0 >> 5], bits << (k0 & 31));
    }
#pragma unroll
    for (int r = 0; r < kRowChunk; ++r) {
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) {
        const float o = __shfl_xor(mx[r], d, 64);
        mx[r] = o > mx[r] ? o : mx[r];
      }
      if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][r] = mx[r];
    }
    __syncthreads();
    if (threadIdx.x < kRowChunk && m0 + threadIdx.x < m_end) {
      float r = red[0][threadIdx.x];
#pragma unroll
      for (int i = 1; i < 4; ++i) r = red[i][threadIdx.x] > r ? red[i][threadIdx.x] : r;
      ranges[m0 + threadIdx.x] = r;
    }
    __syncthreads();  // red is reused by the next four rows
  }
  for (int w = threadIdx.x; w < nwords; w += 256) part[static_cast<int64_t>(blockIdx.x) * nwords + w] = smask[w];
}

// QuantFunc (:153-164).  NaN (0 * inf in a row whose range is 0) becomes 0.
__device__ inline uint32_t quant_one(float xv, float inv) {
  float t = xv * 127.0f * inv;
  t = roundf(t);
  t = t > 127.0f ? 127.0f : (t < -127.0f ? -127.0f : t);
  if (t != t) t = 0.0f;
  return static_cast<uint32_t>(static_cast<int>(t)) & 0xFFu;
}

// The mask (nwords words, word w from word_at(w)) as an ascending list of
// outlier columns and their count.  Called by every thread of a workgroup (of
// at least 256 threads; the first 256 do the work); scan (256 ints) and base_s
// are LDS.
template <class F>
__device__ inline void build_list(int nwords, F word_at, int32_t* list, int32_t* count, int* scan, int* base_s) {
  const int tid = threadIdx.x;
  const bool worker = tid < 256;
  if (tid == 0) *base_s = 0;
  __syncthreads();
  for (int w0 = 0; w0 < nwords; w0 += 256) {
    uint32_t word = worker && w0 + tid < nwords ? word_at(w0 + tid) : 0u;
    const int c = __popc(word);
    if (worker) scan[tid] = c;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int add = worker && tid >= d ? scan[tid - d] : 0;
      __syncthreads();
      if (worker) scan[tid] += add;
      __syncthreads();
    }
    const int base = *base_s;
    int o = worker ? base + scan[tid] - c : 0;
    while (word != 0) {
      const int b = __ffs(word) - 1;
      list[o++] = (w0 + tid) * 32 + b;
      word &= word - 1;
    }
    __syncthreads();
    if (tid == 0) *base_s = base + scan[255];
    __syncthreads();
  }
  if (tid == 0) *count = *base_s;
}

// Row ranges, outlier mask and list, activation codes of up to kSmallRows rows
// in one workgroup: the decode-sized case, where three launches cost more
// than the work.  The mask lives in LDS (K / 32 words, dynamic).
constexpr int kSmallRows = 2;  // beyond two rows the single workgroup takes longer than the three launches
constexpr int kSmallThreads = 1024;
constexpr int kSmallMaxK = 65536;

template <int DT>
__global__ __launch_bounds__(kSmallThreads) void llm_act_small_kernel(const uint16_t* __restrict__ x, float threshold,
                                                                      int M, int K, float* __restrict__ ranges,
                                                                      int32_t* __restrict__ mask,
                                                                      int8_t* __restrict__ qx,
                                                                      int32_t* __restrict__ count,
                                                                      int32_t* __restrict__ list) {
  extern __shared__ uint32_t smask[];
  __shared__ float part[kSmallThreads / 64][kSmallRows];
  __shared__ float srange[kSmallRows];
  __shared__ int scan[256];
  __shared__ int base_s;
  const int tid = threadIdx.x;
  const int nwords = K / 32;
  const float thr = to_f32<DT>(from_f32_rne<DT>(threshold));
  for (int w = tid; w < nwords; w += kSmallThreads) smask[w] = 0u;
  __syncthreads();
  float mx[kSmallRows];
#pragma unroll
  for (int r = 0; r < kSmallRows; ++r) mx[r] = 0.0f;
  for (int k0 = tid * 8; k0 < K; k0 += kSmallThreads * 8) {
    uint32_t bits = 0;
#pragma unroll
    for (int r = 0; r < kSmallRows; ++r) {
      if (r < M) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(r) * K + k0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float a = fabsf(to_f32<DT>(static_cast<uint16_t>(v[i >> 1] >> (16 * (i & 1)))));
          if (a > thr) {
            bits |= 1u << i;
            a = 0.0f;
          }
          mx[r] = a > mx[r] ? a : mx[r];
        }
      }
    }
    if (bits != 0) atomicOr(&smask[k0 >> 5], bits << (k0 & 31));
  }
#pragma unroll
  for (int r = 0; r < kSmallRows; ++r) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
      const float o = __shfl_xor(mx[r], d, 64);
      mx[r] = o > mx[r] ? o : mx[r];
    }
    if ((tid & 63) == 0) part[tid >> 6][r] = mx[r];
  }
  __syncthreads();
  if (tid < M) {
    float r = part[0][tid];
#pragma unroll
    for (int i = 1; i < kSmallThreads / 64; ++i) r = part[i][tid] > r ? part[i][tid] : r;
    ranges[tid] = r;
    srange[tid] = r;
  }
  for (int w = tid; w < nwords; w += kSmallThreads) mask[w] = static_cast<int32_t>(smask[w]);  // for whoever inspects the stages
  build_list(nwords, [&](int w) { return smask[w]; }, list, count, scan, &base_s);  // its barriers also publish srange
  const int64_t nvec = static_cast<int64_t>(M) * K / 16;
  for (int64_t v = tid; v < nvec; v += kSmallThreads) {
    const int64_t e = v * 16;
    const int m = static_cast<int>(e / K);
    const int k = static_cast<int>(e - static_cast<int64_t>(m) * K);
    const u32x4 lo = *reinterpret_cast<const u32x4*>(x + e);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(x + e + 8);
    const uint32_t out_bits = smask[k >> 5] >> (k & 31);
    const float inv = 1.0f / srange[m];
    u32x4 q = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t word = i < 8 ? lo[(i & 7) >> 1] : hi[(i & 7) >> 1];
      const float xv = to_f32<DT>(static_cast<uint16_t>(word >> (16 * (i & 1))));
      const uint32_t c = (out_bits >> i) & 1u ? 0u : quant_one(xv, inv);
      q[i >> 2] |= c << (8 * (i & 3));
    }
    *reinterpret_cast<u32x4*>(qx + e) = q;
  }
}

// ORs the row kernel's partial masks (groups rows of K / 32 words) into the
// mask.  A workgroup takes four words; 64 threads per word each take every
// 64th group and meet in LDS.
__global__ __launch_bounds__(256) void llm_mask_kernel(const uint32_t* __restrict__ part, int groups, int K,
                                                       int32_t* __restrict__ mask) {
  __shared__ uint32_t red[64][4];
  const int tid = threadIdx.x;
  const int nwords = K / 32;
  const int wl = tid & 3, sub = tid >> 2;
  const int w = blockIdx.x * 4 + wl;
  uint32_t v = 0u;
  if (w < nwords)
    for (int g = sub; g < groups; g += 64) v |= part[static_cast<int64_t>(g) * nwords + w];
  red[sub][wl] = v;
  __syncthreads();
  if (tid < 4 && w < nwords) {
    uint32_t o = 0u;
#pragma unroll
    for (int i = 0; i < 64; ++i) o |= red[i][tid];
    mask[w] = static_cast<int32_t>(o);
  }
}

// Activation codes; the last workgroup instead turns the mask into the
// ascending list of outlier columns.
template <int DT>
__global__ __launch_bounds__(256) void llm_quant_kernel(const uint16_t* __restrict__ x,
                                                        const float* __restrict__ ranges,
                                                        int32_t* mask, const uint32_t* __restrict__ part,
                                                        int groups, int M, int K, int8_t* __restrict__ qx,
                                                        int32_t* __restrict__ count, int32_t* __restrict__ list) {
  // groups > 0: the row kernel's few partial masks are ORed here (no mask
  // kernel ran); the list workgroup also leaves the combined mask in `mask`
  const int tid = threadIdx.x;
  const int nwords = K / 32;
  auto mask_word = [&](int w) {
    if (groups == 0) return static_cast<uint32_t>(mask[w]);
    uint32_t v = 0u;
    for (int g = 0; g < groups; ++g) v |= part[static_cast<int64_t>(g) * nwords + w];
    return v;
  };
  if (blockIdx.x == gridDim.x - 1) {
    __shared__ int scan[256];
    __shared__ int base_s;
    build_list(nwords, [&](int w) {
      const uint32_t v = mask_word(w);
      if (groups != 0) mask[w] = static_cast<int32_t>(v);
      return v;
    }, list, count, scan, &base_s);
    return;
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x - 1) * 256;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * 256 + tid;
  const int64_t nvec = static_cast<int64_t>(M) * K / 16;
  for (int64_t v = first; v < nvec; v += stride) {
    const int64_t e = v * 16;
    const int m = static_cast<int>(e / K);
    const int k = static_cast<int>(e - static_cast<int64_t>(m) * K);
    const u32x4 lo = *reinterpret_cast<const u32x4*>(x + e);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(x + e + 8);
    const uint32_t out_bits = mask_word(k >> 5) >> (k & 31);
    const float inv = 1.0f / ranges[m];
    u32x4 q = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t word = i < 8 ? lo[(i & 7) >> 1] : hi[(i & 7) >> 1];
      const float xv = to_f32<DT>(static_cast<uint16_t>(word >> (16 * (i & 1))));
      const uint32_t c = (out_bits >> i) & 1u ? 0u : quant_one(xv, inv);
      q[i >> 2] |= c << (8 * (i & 3));
    }
    *reinterpret_cast<u32x4*>(qx + e) = q;
  }
}

// ---------------------------------------------------------------------------
// the epilogue arithmetic, shared by the GEMM and the merge kernel
// ---------------------------------------------------------------------------
struct Epi {
  const uint16_t* x;      // [M,K] T
  const int8_t* w;        // [N,K]
  const float* wscale;    // [N]
  const float* ranges;    // [M]
  const uint16_t* bias;   // [N] T or null
  const int32_t* count;
  const int32_t* list;
  uint16_t* out;          // [M,N] T
  int M, K, N;
};

// v / 127, correctly rounded, in four instructions instead of the dozen of the
// IEEE division sequence: q = v * RN(1/127), r = v - 127 q (exact in an FMA),
// q + r * RN(1/127).  Equal to the division for every one of the 2^32 float
// inputs (checked exhaustively on a CPU with hardware FMA); q itself is the
// answer where r is zero or NaN (v = -0, infinities).
__device__ inline float div127(float v) {
  const float y = 1.0f / 127.0f;
  const float q = v * y;
  const float r = __builtin_fmaf(-q, 127.0f, v);
  const float q2 = __builtin_fmaf(r, y, q);
  return (r != 0.0f && r == r) ? q2 : q;
}

// DequantFunc (:172-176) and the two T additions that follow it.  The casts
// are the hardware's round-to-nearest-even conversions (the payload of a NaN
// result is unspecified).
template <int DT>
__device__ inline uint16_t merge_one(int acc, float sub, float range, float ws, bool has_bias, float bias) {
  const float dq = to_f32<DT>(cast_out<DT>(div127(static_cast<float>(acc) * range * ws)));
  const float o = to_f32<DT>(cast_out<DT>(sub + dq));  // sub is a T value
  return has_bias ? cast_out<DT>(o + bias) : cast_out<DT>(o);
}

// The same without outlier columns (sub = +0): T(0 + dq) is dq, -0 becoming +0.
template <int DT>
__device__ inline uint16_t merge_plain(int acc, float range, float ws, bool has_bias, float bias) {
  const uint16_t dq = cast_out<DT>(div127(static_cast<float>(acc) * range * ws));
  if (!has_bias) return dq == 0x8000u ? static_cast<uint16_t>(0) : dq;
  return cast_out<DT>(to_f32<DT>(dq) + 0.0f + bias);
}

// Eight neighbouring columns nn .. nn+7 of row m: the merge with the outlier
// columns' product (when there are any: out of LDS if xs is given, computed on
// the spot if wd_stride is negative, else as the outlier kernel left it in the
// output's own place) and one 16-byte store.  ws and bias hold the eight columns' values.
template <int DT>
__device__ inline void finish8(const Epi& e, int cnt, int m, int nn, float range, i32x4 s0, i32x4 s1,
                               const float* ws, const float* bias, const float* xs, int xs_stride,
                               const float* wd, int wd_stride) {
  u32x4 o;
  if (cnt == 0) {  // uniform: the count is one value for the whole launch
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const uint32_t lo = merge_plain<DT>(i < 4 ? s0[i] : s1[i - 4], range, ws[i], e.bias != nullptr, bias[i]);
      const uint32_t hi =
          merge_plain<DT>(i < 4 ? s0[i + 1] : s1[i - 3], range, ws[i + 1], e.bias != nullptr, bias[i + 1]);
      o[i >> 1] = lo | (hi << 16);
    }
    *reinterpret_cast<u32x4*>(e.out + static_cast<int64_t>(m) * e.N + nn) = o;
    return;
  }
  float sub[8];
  if (xs != nullptr) {
    // the workgroup holds this row's activations and these columns' dequantised
    // weights of every outlier column in LDS (xs[j * xs_stride], wd[j * wd_stride + i])
#pragma unroll
    for (int i = 0; i < 8; ++i) sub[i] = 0.0f;
#pragma unroll 1
    for (int j = 0; j < cnt; ++j) {
      const float xv = xs[j * xs_stride];
      const f32x4 w0 = *reinterpret_cast<const f32x4*>(wd + j * wd_stride);
      const f32x4 w1 = *reinterpret_cast<const f32x4*>(wd + j * wd_stride + 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sub[i] += xv * w0[i];
        sub[4 + i] += xv * w1[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) sub[i] = to_f32<DT>(cast_out<DT>(sub[i]));
  } else if (wd_stride < 0) {
    // very few rows: straight from x and the weight, no outlier kernel ran
#pragma unroll
    for (int i = 0; i < 8; ++i) sub[i] = 0.0f;
#pragma unroll 1
    for (int j = 0; j < cnt; ++j) {
      const int kj = e.list[j];
      const float xv = to_f32<DT>(e.x[static_cast<int64_t>(m) * e.K + kj]);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float w = static_cast<float>(e.w[static_cast<int64_t>(nn + i) * e.K + kj]);
        sub[i] += xv * to_f32<DT>(cast_out<DT>(w * ws[i]));
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) sub[i] = to_f32<DT>(cast_out<DT>(sub[i]));
  } else {
    const u32x4 sv = *reinterpret_cast<const u32x4*>(e.out + static_cast<int64_t>(m) * e.N + nn);
#pragma unroll
    for (int i = 0; i < 8; ++i) sub[i] = to_f32<DT>(static_cast<uint16_t>(sv[i >> 1] >> (16 * (i & 1))));
  }
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    const uint32_t lo = merge_one<DT>(i < 4 ? s0[i] : s1[i - 4], sub[i], range, ws[i], e.bias != nullptr, bias[i]);
    const uint32_t hi =
        merge_one<DT>(i < 4 ? s0[i + 1] : s1[i - 3], sub[i + 1], range, ws[i + 1], e.bias != nullptr, bias[i + 1]);
    o[i >> 1] = lo | (hi << 16);
  }
  *reinterpret_cast<u32x4*>(e.out + static_cast<int64_t>(m) * e.N + nn) = o;
}

// The eight columns' scales and biases.
template <int DT>
__device__ inline void load_ws_bias8(const Epi& e, int nn, float* ws, float* bias) {
  const f32x4 w0 = *reinterpret_cast<const f32x4*>(e.wscale + nn);
  const f32x4 w1 = *reinterpret_cast<const f32x4*>(e.wscale + nn + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ws[i] = w0[i];
    ws[4 + i] = w1[i];
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) bias[i] = e.bias != nullptr ? to_f32<DT>(e.bias[nn + i]) : 0.0f;
}

// sub[m,n] = T( sum over the outlier columns k, ascending, of x[m,k] * T(w[n,k] *
// wscale[n]) ), fp32 sum: what the reference computes with SplitKernel and a
// library GEMM (:305-362, :593-640).  A workgroup takes 64 rows x 256 columns,
// a thread one column of them; the rows' activations of 32 outlier columns at
// a time wait in LDS.  Workgroups leave at once when there is no outlier or
// the GEMM's epilogue computes the product itself (up to fused_cap columns).
template <int DT>
__global__ __launch_bounds__(256) void llm_outlier_kernel(Epi e, int fused_cap) {
  uint16_t* sub = e.out;  // the product waits where the output will go: whoever merges element (m, n) reads it first
  const int cnt = *e.count;
  if (cnt <= fused_cap) return;  // none, or few enough for the GEMM's epilogue to take them
  __shared__ __attribute__((aligned(16))) float xs[32][64];
  const int tid = threadIdx.x;
  const int nbx = (e.N + 255) / 256;
  const int m0 = static_cast<int>(blockIdx.x / nbx) * 64;
  const int n = static_cast<int>(blockIdx.x % nbx) * 256 + tid;
  const int nn = n < e.N ? n : e.N - 1;
  const float ws = e.wscale[nn];
  const int8_t* wrow = e.w + static_cast<int64_t>(nn) * e.K;
  float acc[64];
#pragma unroll
  for (int r = 0; r < 64; ++r) acc[r] = 0.0f;
  for (int j0 = 0; j0 < cnt; j0 += 32) {
    __syncthreads();
    for (int i = tid; i < 64 * 32; i += 256) {
      const int r = i & 63, c = i >> 6;
      int m = m0 + r;
      m = m < e.M ? m : e.M - 1;
      xs[c][r] = j0 + c < cnt ? to_f32<DT>(e.x[static_cast<int64_t>(m) * e.K + e.list[j0 + c]]) : 0.0f;
    }
    __syncthreads();
    const int cn = cnt - j0 < 32 ? cnt - j0 : 32;
#pragma unroll 1
    for (int c = 0; c < cn; ++c) {
      const float wd = to_f32<DT>(cast_out<DT>(static_cast<float>(wrow[e.list[j0 + c]]) * ws));
#pragma unroll
      for (int r = 0; r < 64; r += 4) {
        const f32x4 xv = *reinterpret_cast<const f32x4*>(&xs[c][r]);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[r + i] += xv[i] * wd;
      }
    }
  }
  if (n < e.N) {
#pragma unroll
    for (int r = 0; r < 64; ++r)
      if (m0 + r < e.M) sub[static_cast<int64_t>(m0 + r) * e.N + n] = cast_out<DT>(acc[r]);
  }
}

// ---------------------------------------------------------------------------
// int8 GEMM
// ---------------------------------------------------------------------------
struct GemmParams {
  const int8_t* qx;  // [M,K]
  Epi e;
  int32_t* acc;      // [runs][M,N] int32, one slab per K run; only with K runs
  int nbx, nby;      // tiles along N and M
  int n_lo, n_hi;    // columns [n_lo, n_hi) of the output belong to this launch
  int tiles_per_run; // k tiles per K run
  int cap;  // outlier columns the epilogue takes through LDS itself; more come from the outlier kernel
};

// XOR applied to the 16-byte piece index of a row in LDS (C pieces per row) so
// that the 16 rows a quarter of a wavefront reads hit distinct LDS banks,
// whether the LDS serves 8 or 16 lanes of a 128-bit read per cycle.
template <int C>
__device__ inline int row_swizzle(int row) {
  if (C == 8) return (row & 7) ^ ((row >> 3) & 1);                             // 128-byte rows
  return ((((row >> 1) ^ (row >> 3)) & 1) << 1) | ((row >> 2) & 1);            // 64-byte rows
}

// WM x WN wavefronts, each TM x TN blocks of 32x32; k tiles of TK bytes per row
// (128: whole cache lines per row and load; 64 for a K that is not a multiple
// of 128), STAGES of them in LDS.  RUNS: K is cut into runs across workgroups,
// each leaving its sums in its slab of acc; otherwise the epilogue writes out.
template <int DT, int WM, int WN, int TM, int TN, int TK, int STAGES, bool RUNS>
__global__ __launch_bounds__(WM* WN * 64) __attribute__((amdgpu_waves_per_eu(2))) void llm_gemm_kernel(GemmParams p) {
  constexpr int NW = WM * WN;
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int kTK = TK, kStages = STAGES, C = TK / 16;  // C: 16-byte pieces per row
  constexpr int kABytes = BM * kTK, kBBytes = BN * kTK, kStage = kABytes + kBBytes;
  constexpr int kABlocks = kABytes / 1024, kBBlocks = kBBytes / 1024;  // 1 KiB = one wavefront load
  constexpr int kALoads = (kABlocks + NW - 1) / NW, kBLoads = (kBBlocks + NW - 1) / NW;
  constexpr int kPerStage = kALoads + kBLoads;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int M = p.e.M, K = p.e.K, N = p.e.N;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int r32 = lane & 31, b = lane >> 5;

  // tile of this workgroup.  Consecutive workgroup ids go round the eight
  // XCDs; each XCD gets a band of column tiles with every row tile, so that
  // its L2 holds that band's weights once.
  const int ntiles = p.nbx * p.nby;
  const int run = blockIdx.x / ntiles;
  const int t = blockIdx.x - run * ntiles;
  int bx, by;
  if (p.nbx % 8 == 0) {
    const int xcd = t & 7, idx = t >> 3;
    bx = xcd * (p.nbx / 8) + idx / p.nby;
    by = idx % p.nby;
  } else {
    bx = t / p.nby;
    by = t % p.nby;
  }
  const int m0 = by * BM, n0 = p.n_lo + bx * BN;
  const int ktiles = K / kTK;
  const int t0 = run * p.tiles_per_run;
  const int niter = (ktiles - t0) < p.tiles_per_run ? (ktiles - t0) : p.tiles_per_run;

  // global sources of this lane's direct-to-LDS loads.  LDS piece q (16 bytes)
  // of a tile region is row q / C, slot q % C, and holds the row's logical
  // piece slot ^ swizzle(row).  Rows past M or N repeat the last valid row:
  // computed on valid data, never stored.  Where a region has fewer 1 KiB
  // blocks than there are wavefronts, some blocks are loaded twice.
  // (the casts at the load builtin are needed: with the array element passed as
  // it is, host compilation silently leaves out the kernel's stub and the
  // library does not link)
  const uint8_t* asrc[kALoads];
  int ablk[kALoads];
#pragma unroll
  for (int c = 0; c < kALoads; ++c) {
    ablk[c] = (c * NW + wave) % kABlocks;
    const int q = ablk[c] * 64 + lane;
    const int row = q / C, cc = (q % C) ^ row_swizzle<C>(row);
    int m = m0 + row;
    m = m < M ? m : M - 1;
    asrc[c] = reinterpret_cast<const uint8_t*>(p.qx) + static_cast<int64_t>(m) * K + static_cast<int64_t>(t0) * kTK + cc * 16;
  }
  const uint8_t* bsrc[kBLoads];
  int bblk[kBLoads];
#pragma unroll
  for (int c = 0; c < kBLoads; ++c) {
    bblk[c] = (c * NW + wave) % kBBlocks;
    const int q = bblk[c] * 64 + lane;
    const int row = q / C, cc = (q % C) ^ row_swizzle<C>(row);
    int n = n0 + row;
    n = n < N ? n : N - 1;
    bsrc[c] = reinterpret_cast<const uint8_t*>(p.e.w) + static_cast<int64_t>(n) * K + static_cast<int64_t>(t0) * kTK + cc * 16;
  }
  // tile `it` of this run into its stage; past the end of the run the last
  // tile again, into a spare stage, so that every iteration issues the same
  // number of loads
#define WOL_LLM_ISSUE(it_)                                                                           \
  do {                                                                                               \
    const int koff_ = ((it_) < niter ? (it_) : niter - 1) * kTK;                                      \
    unsigned char* stage_ = smem + ((it_) % kStages) * kStage;                                        \
    _Pragma("unroll") for (int c = 0; c < kALoads; ++c) __builtin_amdgcn_global_load_lds(             \
        reinterpret_cast<const uint8_t*>(asrc[c]) + koff_, (lds_ptr_t)(stage_ + ablk[c] * 1024), 16, 0, 0); \
    _Pragma("unroll") for (int c = 0; c < kBLoads; ++c) __builtin_amdgcn_global_load_lds(             \
        reinterpret_cast<const uint8_t*>(bsrc[c]) + koff_, (lds_ptr_t)(stage_ + kABytes + bblk[c] * 1024), \
        16, 0, 0);                                                                                   \
  } while (0)

  i32x16 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int c = 0; c < TN; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][c][v] = 0;

  // byte offsets of this lane's fragments inside a stage, for k step 0; k step
  // 1 is the same with the piece index XOR 2
  const int swz = row_swizzle<C>(r32);  // rows are 32 * block + r32: the swizzle has period 16
  int aoff[TM], boff[TN];
#pragma unroll
  for (int a = 0; a < TM; ++a) aoff[a] = ((wm * TM + a) * 32 + r32) * kTK;
#pragma unroll
  for (int c = 0; c < TN; ++c) boff[c] = kABytes + ((wn * TN + c) * 32 + r32) * kTK;

  WOL_LLM_ISSUE(0);
  if (kStages == 3) WOL_LLM_ISSUE(1);
  for (int it = 0; it < niter; ++it) {
    // loads complete in order: all but the newest stage have landed.  A bare
    // s_barrier, not __syncthreads(): the fence of the latter makes the
    // compiler wait for every load in flight, the prefetched tile included.
    wait_vmcnt<(kStages - 2) * kPerStage>();
    __builtin_amdgcn_s_barrier();
    const unsigned char* stage = smem + (it % kStages) * kStage;
    // the fragments of k step ks + 1 are read while the MFMAs of step ks run;
    // those of step 0 while the next tile's loads are issued
    constexpr int KS = C / 2;
    i32x4 af[2][TM], bf[2][TN];
    {
      const int piece = (b ^ swz) * 16;
#pragma unroll
      for (int a = 0; a < TM; ++a) af[0][a] = *reinterpret_cast<const i32x4*>(stage + aoff[a] + piece);
#pragma unroll
      for (int c = 0; c < TN; ++c) bf[0][c] = *reinterpret_cast<const i32x4*>(stage + boff[c] + piece);
    }
    __builtin_amdgcn_sched_barrier(0);
    WOL_LLM_ISSUE(it + kStages - 1);  // into the stage every wavefront finished reading before the barrier
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) {
        const int piece = (((ks + 1) * 2 + b) ^ swz) * 16;
#pragma unroll
        for (int a = 0; a < TM; ++a)
          af[(ks + 1) & 1][a] = *reinterpret_cast<const i32x4*>(stage + aoff[a] + piece);
#pragma unroll
        for (int c = 0; c < TN; ++c)
          bf[(ks + 1) & 1][c] = *reinterpret_cast<const i32x4*>(stage + boff[c] + piece);
      }
#pragma unroll
      for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int c = 0; c < TN; ++c)
          acc[a][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks & 1][a], bf[ks & 1][c], acc[a][c], 0, 0, 0);
      // issue order: the LDS reads of the next step spread between this step's
      // MFMAs (left alone the scheduler reads one fragment, waits, and issues
      // the two MFMAs that use it)
      constexpr int kMfma = TM * TN, kRead = TM + TN;
#pragma unroll
      for (int i = 0; i < kMfma; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        const int reads = ks + 1 < KS ? kRead * (i + 1) / kMfma - kRead * i / kMfma : 0;
#pragma unroll
        for (int r = 0; r < reads; ++r) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);  // nothing moves between k steps
    }
  }
#undef WOL_LLM_ISSUE
  wait_vmcnt<0>();  // the spare-stage loads must have landed before the LDS is reused (or the workgroup ends)

  // accumulator v of a 32x32 block: row 8 * (v / 4) + 4 * (lane / 32) + v % 4, column lane % 32
  const Epi& e = p.e;
  // Each wavefront passes its blocks one at a time through a slab of LDS of its
  // own (32 rows of kSlabRow ints: with that stride the two halves of the
  // wavefront write to disjoint banks) and takes them back as rows: a lane
  // owns eight neighbouring columns of one row, so the output leaves as
  // 16-byte stores (with K runs: as two 16-byte stores into this run's slab of
  // int32 sums).  The loop over the rows is a real loop, which keeps the
  // epilogue's registers few.
  constexpr int kSlabRow = 40;
  __syncthreads();  // every wavefront is done with the stages
  int* slab = reinterpret_cast<int*>(smem) + wave * (32 * kSlabRow);
  const int cnt = RUNS ? 0 : *e.count;
  const int cgrp = (lane & 3) * 8;  // first of this lane's eight columns inside the block
  // few outlier columns: their activations (this tile's rows) and dequantised
  // weights (this tile's columns) go to LDS behind the slabs, as floats
  float* rng = reinterpret_cast<float*>(smem + NW * 32 * kSlabRow * 4);  // [BM]: the tile's row ranges
  float* xs = rng + BM;                                                  // [cnt][BM]
  float* wdl = xs + p.cap * BM;                                          // [cnt][BN]
  const bool fused = !RUNS && cnt > 0 && cnt <= p.cap;
  if (!RUNS) {
    // (read per row out of global memory inside the row loop they cost a
    // memory latency per row, sixteen in a row per wavefront)
    for (int i = tid; i < BM; i += NW * 64) rng[i] = e.ranges[m0 + i < M ? m0 + i : M - 1];
    if (!fused) __syncthreads();
  }
  if (fused) {
    for (int i = tid; i < cnt * BM; i += NW * 64) {
      const int j = i / BM;
      int m = m0 + i % BM;
      m = m < M ? m : M - 1;
      xs[i] = to_f32<DT>(e.x[static_cast<int64_t>(m) * K + e.list[j]]);
    }
    for (int i = tid; i < cnt * BN; i += NW * 64) {
      const int j = i / BN;
      int n = n0 + i % BN;
      n = n < N ? n : N - 1;
      wdl[i] = to_f32<DT>(cast_out<DT>(static_cast<float>(e.w[static_cast<int64_t>(n) * K + e.list[j]]) * e.wscale[n]));
    }
    __syncthreads();
  }
#pragma unroll
  for (int c = 0; c < TN; ++c) {
    const int n = n0 + (wn * TN + c) * 32 + cgrp;
    const bool n_ok = n < p.n_hi;  // a multiple of 16: eight columns are all inside or all outside
    const int nn = n_ok ? n : 0;
    float ws[8], bias[8];
    if (!RUNS) load_ws_bias8<DT>(e, nn, ws, bias);
#pragma unroll
    for (int a = 0; a < TM; ++a) {
      __builtin_amdgcn_wave_barrier();  // the rows of the previous block have been read
#pragma unroll
      for (int v = 0; v < 16; ++v) slab[(8 * (v >> 2) + 4 * b + (v & 3)) * kSlabRow + r32] = acc[a][c][v];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll 1
      for (int h = 0; h < 2; ++h) {
        const int row = h * 16 + (lane >> 2);
        const int m = m0 + (wm * TM + a) * 32 + row;
        if (m >= M || !n_ok) continue;
        const i32x4 s0 = *reinterpret_cast<const i32x4*>(slab + row * kSlabRow + cgrp);
        const i32x4 s1 = *reinterpret_cast<const i32x4*>(slab + row * kSlabRow + cgrp + 4);
        if (RUNS) {  // this run's sums, to be added by the merge kernel
          int32_t* dst = p.acc + (static_cast<int64_t>(run) * M + m) * N + nn;
          *reinterpret_cast<i32x4*>(dst) = s0;
          *reinterpret_cast<i32x4*>(dst + 4) = s1;
          continue;
        }
        finish8<DT>(e, cnt, m, nn, rng[(wm * TM + a) * 32 + row], s0, s1, ws, bias, fused ? xs + (wm * TM + a) * 32 + row : nullptr, BM,
                    wdl + (wn * TN + c) * 32 + cgrp, BN);
      }
    }
  }
}

// Adds the K runs' int32 sums and finishes; one thread per eight columns.
template <int DT>
__global__ __launch_bounds__(256) void llm_merge_kernel(const int32_t* __restrict__ acc, int runs, Epi e,
                                                        int direct_outliers) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int groups = e.N / 8;
  if (i >= static_cast<int64_t>(e.M) * groups) return;
  const int m = static_cast<int>(i / groups);
  const int nn = static_cast<int>(i - static_cast<int64_t>(m) * groups) * 8;
  const int64_t slab = static_cast<int64_t>(e.M) * e.N;
  const int32_t* src = acc + static_cast<int64_t>(m) * e.N + nn;
  i32x4 s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0};
  for (int r = 0; r < runs; ++r) {
    s0 += *reinterpret_cast<const i32x4*>(src + r * slab);
    s1 += *reinterpret_cast<const i32x4*>(src + r * slab + 4);
  }
  float ws[8], bias[8];
  load_ws_bias8<DT>(e, nn, ws, bias);
  finish8<DT>(e, *e.count, m, nn, e.ranges[m], s0, s1, ws, bias, nullptr, 0, nullptr, direct_outliers ? -1 : 0);
}

inline void allow_lds(const void* kern, size_t lds, std::atomic<uint32_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const uint32_t bit = 1u << (dev & 31);
  if (done.load(std::memory_order_acquire) & bit) return;
  (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  done.fetch_or(bit, std::memory_order_release);
}

inline int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

struct Plan {
  int bm, bn;     // tile
  int tk;         // k bytes per tile row
  int whole_cols; // many rows: the first whole_cols columns get 256x256 tiles, the rest 128x256
  int runs;       // K runs (1: the GEMM writes the output itself)
  int tiles_per_run;
};

inline int num_cus() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}

// Up to 128 rows: one row tile of 32, 64 or 128 rows, 128 columns wide so that
// the column tiles spread over the CUs, and K cut into runs while CUs are
// still idle, every run keeps 256 k and the runs' int32 sums (written and read
// once each) stay below the weight bytes.
Plan make_plan(int64_t M, int64_t K, int64_t N) {
  Plan pl;
  pl.whole_cols = 0;
  const int tk = K % 128 == 0 ? 128 : 64;
  const int64_t ktiles = K / tk;
  int64_t runs = 1;
  if (M > 128) {
    // 128-deep tiles, eight wavefronts, one workgroup per CU: 256x256 with two
    // stages, or 128x256 with three where their rounds over the CUs come out
    // shorter (a half tile takes 0.55 of a whole one; 384 whole tiles on 256
    // CUs are two rounds, 768 half tiles three).  64-deep tiles (K not a
    // multiple of 128): 256x128, three stages, two workgroups of four per CU.
    pl.bm = 256;
    pl.bn = tk == 128 ? 256 : 128;
    if (tk == 128) {
      // a launch takes ceil(tiles / CUs) tile times: the columns are shared
      // out so that whole tiles fill whole rounds of the CUs
      const int64_t cus = num_cus();
      const int64_t cols = (N + 255) / 256, rows256 = (M + 255) / 256, rows128 = (M + 127) / 128;
      int64_t best_c = cols, best_t = INT64_MAX;
      for (int64_t c = cols; c >= 0; --c) {
        const int64_t t = 20 * ((c * rows256 + cus - 1) / cus) + 11 * (((cols - c) * rows128 + cus - 1) / cus);
        if (t < best_t) {
          best_t = t;
          best_c = c;
        }
      }
      pl.whole_cols = static_cast<int>(best_c * 256 < N ? best_c * 256 : N);
      if (best_c == 0) pl.bm = 128;
    }
  } else {
    pl.bm = M > 64 ? 128 : (M > 32 ? 64 : 32);
    pl.bn = 128;
    const int64_t tiles = (N + pl.bn - 1) / pl.bn;
    runs = 2 * num_cus() / tiles;  // two workgroups fit a CU: no second, nearly empty round
    if (runs > ktiles * tk / 256) runs = ktiles * tk / 256;  // at least 256 k per run
    if (runs > K / (8 * M)) runs = K / (8 * M);
    if (runs < 1) runs = 1;
  }
  int64_t per = (ktiles + runs - 1) / runs;
  runs = (ktiles + per - 1) / per;
  pl.tk = tk;
  pl.runs = static_cast<int>(runs);
  pl.tiles_per_run = static_cast<int>(per);
  return pl;
}

struct Workspace {
  float* ranges;
  int32_t* mask;
  uint32_t* part;
  int32_t* count;
  int32_t* list;
  int8_t* qx;
  int32_t* acc;
  int64_t bytes;
};

Workspace carve(void* base, int64_t M, int64_t K, int64_t N, int runs) {
  if (runs <= 1) runs = 0;
  unsigned char* p = static_cast<unsigned char*>(base);
  int64_t off = 0;
  Workspace w;
  w.ranges = reinterpret_cast<float*>(p + off);
  off += align256(M * 4);
  w.mask = reinterpret_cast<int32_t*>(p + off);
  off += align256(K / 32 * 4);
  w.part = reinterpret_cast<uint32_t*>(p + off);
  off += align256(static_cast<int64_t>(kMaxRowGroups) * (K / 32) * 4);
  w.count = reinterpret_cast<int32_t*>(p + off);
  off += 256;
  w.list = reinterpret_cast<int32_t*>(p + off);
  off += align256(K * 4);
  w.qx = reinterpret_cast<int8_t*>(p + off);
  off += align256(M * K);
  w.acc = reinterpret_cast<int32_t*>(p + off);
  off += align256(M * N * 4 * runs);
  w.bytes = off;
  return w;
}

template <int DT, int WM, int WN, int TM, int TN, int TK, int STAGES, bool RUNS>
int launch_gemm(const GemmParams& p, int runs, hipStream_t stream) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr size_t lds = static_cast<size_t>(STAGES) * (BM + BN) * TK;
  static_assert(lds >= static_cast<size_t>(WM * WN) * 32 * 40 * 4 + BM * 4,
                "the epilogue's slabs and row ranges must fit the stages");
  static std::atomic<uint32_t> done{0};
  auto kern = llm_gemm_kernel<DT, WM, WN, TM, TN, TK, STAGES, RUNS>;
  allow_lds(reinterpret_cast<const void*>(kern), lds, done);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(p.nbx * p.nby * runs)), dim3(WM * WN * 64), lds, stream,
                     p);
  return check_launch();
}

template <int DT, int TK, bool RUNS>
int launch_gemm_for(const GemmParams& p, const Plan& pl, hipStream_t stream) {
  switch (pl.bm) {
    case 256:
      if (RUNS) return WOL_ERR_BAD_SHAPE;  // make_plan cuts K only for tiles of at most 128 rows
      if (pl.bn == 256) return launch_gemm<DT, 2, 4, 4, 2, 128, 2, false>(p, pl.runs, stream);
      return launch_gemm<DT, 2, 2, 4, 2, 64, 3, false>(p, pl.runs, stream);
    case 128:
      if (pl.bn == 256) {
        if (RUNS || TK != 128) return WOL_ERR_BAD_SHAPE;  // make_plan: many rows, 128-deep tiles
        return launch_gemm<DT, 2, 4, 2, 2, 128, 3, false>(p, pl.runs, stream);
      }
      return launch_gemm<DT, 1, 4, 4, 1, TK, 3, RUNS>(p, pl.runs, stream);
    case 64: return launch_gemm<DT, 1, 4, 2, 1, TK, 3, RUNS>(p, pl.runs, stream);
    default: return launch_gemm<DT, 1, 4, 1, 1, TK, 3, RUNS>(p, pl.runs, stream);
  }
}

template <int DT, bool RUNS>
int launch_gemm_tk(const GemmParams& p, const Plan& pl, hipStream_t stream) {
  return pl.tk == 128 ? launch_gemm_for<DT, 128, RUNS>(p, pl, stream) : launch_gemm_for<DT, 64, RUNS>(p, pl, stream);
}

// Outlier columns the GEMM's epilogue can hold in LDS behind its slabs (at most
// 32): (rows + columns of the tile) floats each.
int fused_cap(const Plan& pl) {
  if (pl.runs > 1) return 0;  // the merge kernel reads the outlier kernel's product
  const bool eight = pl.bn == 256;  // the configurations of eight wavefronts
  const int64_t lds = static_cast<int64_t>(pl.bm == 256 && eight ? 2 : 3) * (pl.bm + pl.bn) * pl.tk;
  const int64_t room = lds - (eight ? 8 : 4) * 32 * 40 * 4 - pl.bm * 4;  // slabs, row ranges
  const int64_t cap = room / ((pl.bm + pl.bn) * 4);
  return static_cast<int>(cap > 32 ? 32 : (cap < 0 ? 0 : cap));
}

template <int DT>
int run_llm_int8(const void* x, const void* weight, const void* bias, const float* wscale, float threshold,
                 int64_t M, int64_t K, int64_t N, void* out, void* workspace, hipStream_t stream) {
  const Plan pl = make_plan(M, K, N);
  const Workspace ws = carve(workspace, M, K, N, pl.runs);
  const uint16_t* xs = static_cast<const uint16_t*>(x);
  const bool small = M <= kSmallRows && K <= kSmallMaxK;
  if (small) {
    hipLaunchKernelGGL(llm_act_small_kernel<DT>, dim3(1), dim3(kSmallThreads), static_cast<size_t>(K / 32 * 4), stream,
                       xs, threshold, static_cast<int>(M), static_cast<int>(K), ws.ranges, ws.mask, ws.qx, ws.count,
                       ws.list);
  }
  if (!small) {
    // at most kMaxRowGroups workgroups, each a whole number of four-row chunks
    int64_t rows_per_group = (M + kMaxRowGroups - 1) / kMaxRowGroups;
    rows_per_group = (rows_per_group + kRowChunk - 1) / kRowChunk * kRowChunk;
    const int groups = static_cast<int>((M + rows_per_group - 1) / rows_per_group);
    const size_t mask_lds = static_cast<size_t>(K / 32) * 4;
    hipLaunchKernelGGL(llm_rowmax_kernel<DT>, dim3(static_cast<unsigned>(groups)), dim3(256), mask_lds, stream, xs,
                       threshold, static_cast<int>(M), static_cast<int>(K), static_cast<int>(rows_per_group),
                       ws.ranges, ws.part);
    // up to four partial masks (16 rows) the quant kernel ORs itself: cheaper
    // than a launch (26.1 against 27.8 us at 8 rows; with 16 masks it loses 2 us)
    const bool or_in_quant = groups <= 4;
    if (!or_in_quant)
      hipLaunchKernelGGL(llm_mask_kernel, dim3(static_cast<unsigned>((K / 32 + 3) / 4)), dim3(256), 0, stream,
                         ws.part, groups, static_cast<int>(K), ws.mask);
    const int64_t nvec = M * K / 16;
    int64_t qblocks = (nvec + 255) / 256;
    if (qblocks > 8192) qblocks = 8192;
    hipLaunchKernelGGL(llm_quant_kernel<DT>, dim3(static_cast<unsigned>(qblocks + 1)), dim3(256), 0, stream, xs,
                       ws.ranges, ws.mask, ws.part, or_in_quant ? groups : 0, static_cast<int>(M),
                       static_cast<int>(K), ws.qx, ws.count, ws.list);
  }
  GemmParams p;
  p.qx = ws.qx;
  p.e = Epi{xs, static_cast<const int8_t*>(weight), wscale, ws.ranges, static_cast<const uint16_t*>(bias),
            ws.count, ws.list, static_cast<uint16_t*>(out), static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N)};
  p.acc = ws.acc;
  p.n_lo = 0;
  p.n_hi = static_cast<int>(N);
  p.nbx = static_cast<int>((N + pl.bn - 1) / pl.bn);
  p.nby = static_cast<int>((M + pl.bm - 1) / pl.bm);
  p.tiles_per_run = pl.tiles_per_run;
  p.cap = fused_cap(pl);
  if (pl.runs == 1 && pl.bm == 256 && pl.bn == 256 && pl.whole_cols < N) {
    Plan half = pl;
    half.bm = 128;
    const int c = fused_cap(half);  // both launches and the outlier kernel go by one limit
    p.cap = c < p.cap ? c : p.cap;
  }
  // up to four rows with K runs the merge kernel multiplies the outlier columns
  // itself (a launch costs more than that work)
  const bool direct = pl.runs > 1 && M <= 4;
  if (!direct)
    hipLaunchKernelGGL(llm_outlier_kernel<DT>, dim3(static_cast<unsigned>(((N + 255) / 256) * ((M + 63) / 64))),
                       dim3(256), 0, stream, p.e, p.cap);
  if (check_launch() != WOL_OK) return WOL_ERR_HIP;
  if (pl.runs == 1 && pl.bm == 256 && pl.bn == 256 && pl.whole_cols < N) {
    // 256x256 tiles on the first columns, 128x256 tiles on the rest
    p.n_hi = pl.whole_cols;
    p.nbx = pl.whole_cols / 256;
    const int rc = launch_gemm_tk<DT, false>(p, pl, stream);
    if (rc != WOL_OK) return rc;
    Plan half = pl;
    half.bm = 128;
    p.n_lo = pl.whole_cols;
    p.n_hi = static_cast<int>(N);
    p.nbx = static_cast<int>((N - pl.whole_cols + 255) / 256);
    p.nby = static_cast<int>((M + 127) / 128);
    return launch_gemm_tk<DT, false>(p, half, stream);
  }
  if (pl.runs == 1) return launch_gemm_tk<DT, false>(p, pl, stream);
  const int rc = launch_gemm_tk<DT, true>(p, pl, stream);
  if (rc != WOL_OK) return rc;
  const int64_t total = M * (N / 8);
  hipLaunchKernelGGL(llm_merge_kernel<DT>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream,
                     ws.acc, pl.runs, p.e, direct ? 1 : 0);
  return check_launch();
}

}  // namespace

size_t llm_int8_workspace(int64_t M, int64_t K, int64_t N) {
  const Plan pl = make_plan(M, K, N);
  return static_cast<size_t>(carve(nullptr, M, K, N, pl.runs).bytes);
}

void llm_int8_workspace_offsets(int64_t M, int64_t K, int64_t N, int64_t* offsets) {
  const Plan pl = make_plan(M, K, N);
  const Workspace w = carve(nullptr, M, K, N, pl.runs);
  offsets[0] = reinterpret_cast<intptr_t>(w.ranges);
  offsets[1] = reinterpret_cast<intptr_t>(w.mask);
  offsets[2] = reinterpret_cast<intptr_t>(w.count);
  offsets[3] = reinterpret_cast<intptr_t>(w.list);
  offsets[4] = reinterpret_cast<intptr_t>(w.qx);
  offsets[5] = pl.runs > 1 ? reinterpret_cast<intptr_t>(w.acc) : -1;
  offsets[6] = pl.runs;
}

int launch_llm_int8_linear(const void* x, const void* weight, const void* bias, const float* wscale,
                           float threshold, int dtype, int64_t M, int64_t K, int64_t N, void* out,
                           void* workspace, hipStream_t stream) {
  if (dtype == WOL_DTYPE_BF16)
    return run_llm_int8<WOL_DTYPE_BF16>(x, weight, bias, wscale, threshold, M, K, N, out, workspace, stream);
  return run_llm_int8<WOL_DTYPE_F16>(x, weight, bias, wscale, threshold, M, K, N, out, workspace, stream);
}

}  // namespace wol
