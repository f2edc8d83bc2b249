// apply_per_channel_scale: out[r, c] = T(x[r, c] * scales[c]), the pre-quant
// smoothing of activations that runs in front of weight_only_linear
// (paddle/phi/kernels/gpu/apply_per_channel_scale_kernel.cu:93-126: one
// multiply in T, i.e. the exact product rounded once to nearest even; the
// product of two T values is exact in fp32, so fp32 multiply + one cast gives
// the same bits).  HBM-bound: 2 bytes read and 2 written per element.
#include "wol_common.h"

namespace wol {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = 8;  // rows a thread walks with its scales in registers

template <int DT>
__device__ inline uint32_t mul_pair(uint32_t x2, float s_lo, float s_hi) {
  // the same arithmetic as prescale_pair (wol_common.h), with the scales already widened
  const float lo = to_f32<DT>(static_cast<uint16_t>(x2 & 0xFFFFu)) * s_lo;
  const float hi = to_f32<DT>(static_cast<uint16_t>(x2 >> 16)) * s_hi;
  return static_cast<uint32_t>(cast_out<DT>(lo)) | (static_cast<uint32_t>(cast_out<DT>(hi)) << 16);
}

// cols % 8 == 0 and 16-byte aligned pointers: thread = 8 columns, 16-byte
// accesses, all row loads of a thread issued before the first use.
template <int DT>
__global__ __launch_bounds__(kThreads) void prescale_vec_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ scales, int64_t rows,
    int64_t cols, uint16_t* __restrict__ out) {
  const int64_t c8 = static_cast<int64_t>(blockIdx.y) * kThreads + threadIdx.x;  // 8-column piece
  if (c8 * 8 >= cols) return;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock;
  const u32x4 sv = *reinterpret_cast<const u32x4*>(scales + c8 * 8);
  const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w};
  float s[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    s[2 * i] = to_f32<DT>(static_cast<uint16_t>(sw[i] & 0xFFFFu));
    s[2 * i + 1] = to_f32<DT>(static_cast<uint16_t>(sw[i] >> 16));
  }
  u32x4 v[kRowsPerBlock];
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; ++i) {
    const int64_t r = r0 + i < rows ? r0 + i : rows - 1;  // clamp: no branch around the load
    v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + r * cols + c8 * 8));
  }
#pragma unroll
  for (int i = 0; i < kRowsPerBlock; ++i) {
    u32x4 o;
    o.x = mul_pair<DT>(v[i].x, s[0], s[1]);
    o.y = mul_pair<DT>(v[i].y, s[2], s[3]);
    o.z = mul_pair<DT>(v[i].z, s[4], s[5]);
    o.w = mul_pair<DT>(v[i].w, s[6], s[7]);
    if (r0 + i < rows)
      __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(out + (r0 + i) * cols + c8 * 8));
  }
}

// any cols / alignment: one element per thread
template <int DT>
__global__ __launch_bounds__(kThreads) void prescale_scalar_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ scales, int64_t rows,
    int64_t cols, uint16_t* __restrict__ out) {
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock;
  for (int64_t c = static_cast<int64_t>(blockIdx.y) * kThreads + threadIdx.x; c < cols;
       c += static_cast<int64_t>(gridDim.y) * kThreads) {
    const float s = to_f32<DT>(scales[c]);
    for (int i = 0; i < kRowsPerBlock && r0 + i < rows; ++i)
      out[(r0 + i) * cols + c] = cast_out<DT>(to_f32<DT>(x[(r0 + i) * cols + c]) * s);
  }
}

template <int DT>
int launch(const void* x, const void* scales, int64_t rows, int64_t cols, void* out,
           hipStream_t stream) {
  const auto* xp = static_cast<const uint16_t*>(x);
  const auto* sp = static_cast<const uint16_t*>(scales);
  auto* op = static_cast<uint16_t*>(out);
  const bool vec = cols % 8 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(scales) |
                                      reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int64_t per_block = vec ? kThreads * 8 : kThreads;
  // rows along x (up to 2^31 - 1 blocks), column blocks along y (at most 65535:
  // the scalar kernel strides over the rest)
  const int64_t col_blocks = (cols + per_block - 1) / per_block;
  const dim3 grid(static_cast<unsigned>((rows + kRowsPerBlock - 1) / kRowsPerBlock),
                  static_cast<unsigned>(col_blocks < 65535 ? col_blocks : 65535));
  if (vec) prescale_vec_kernel<DT><<<grid, kThreads, 0, stream>>>(xp, sp, rows, cols, op);
  else prescale_scalar_kernel<DT><<<grid, kThreads, 0, stream>>>(xp, sp, rows, cols, op);
  return hipGetLastError() == hipSuccess ? WOL_OK : WOL_ERR_HIP;
}

// swiglu of fp32 sums: out[m, n] = T(silu(in[m, n]) * in[m, n + H]), H = N / 2,
// four columns per thread (H is a multiple of 16).
template <int DT>
__global__ __launch_bounds__(kThreads) void swiglu_f32_kernel(const float* __restrict__ in, int64_t M, int64_t N,
                                                              uint16_t* __restrict__ out) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  const int64_t H = N / 2;
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * 4;
  if (i >= M * H) return;
  const int64_t m = i / H, n = i % H;
  const f32x4 g = *reinterpret_cast<const f32x4*>(in + m * N + n);
  const f32x4 u = *reinterpret_cast<const f32x4*>(in + m * N + H + n);
  u32x2 o;
  o.x = cast_out<DT>(act_swiglu(g[0], u[0])) | (static_cast<uint32_t>(cast_out<DT>(act_swiglu(g[1], u[1]))) << 16);
  o.y = cast_out<DT>(act_swiglu(g[2], u[2])) | (static_cast<uint32_t>(cast_out<DT>(act_swiglu(g[3], u[3]))) << 16);
  *reinterpret_cast<u32x2*>(out + m * H + n) = o;
}

// swiglu of a T tensor: out[m, n] = T(silu(in[m, n]) * in[m, n + H]) computed in
// float (paddle/phi/kernels/gpu/swiglu_kernel.cu:32-52), eight columns per thread.
template <int DT>
__global__ __launch_bounds__(kThreads) void swiglu_t_kernel(const uint16_t* __restrict__ in, int64_t M, int64_t N,
                                                            uint16_t* __restrict__ out) {
  const int64_t H = N / 2;
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * 8;
  if (i >= M * H) return;
  const int64_t m = i / H, n = i % H;
  const u32x4 g = *reinterpret_cast<const u32x4*>(in + m * N + n);
  const u32x4 u = *reinterpret_cast<const u32x4*>(in + m * N + H + n);
  const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
  uint32_t ow[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float lo = act_swiglu(to_f32<DT>(static_cast<uint16_t>(gw[q] & 0xFFFFu)), to_f32<DT>(static_cast<uint16_t>(uw[q] & 0xFFFFu)));
    const float hi = act_swiglu(to_f32<DT>(static_cast<uint16_t>(gw[q] >> 16)), to_f32<DT>(static_cast<uint16_t>(uw[q] >> 16)));
    ow[q] = static_cast<uint32_t>(cast_out<DT>(lo)) | (static_cast<uint32_t>(cast_out<DT>(hi)) << 16);
  }
  *reinterpret_cast<u32x4*>(out + m * H + n) = u32x4{ow[0], ow[1], ow[2], ow[3]};
}

}  // namespace

// N / 2 must be a multiple of 8 and both tensors 16-byte aligned.
int launch_swiglu_t(const void* in, int dtype, int64_t M, int64_t N, void* out, hipStream_t stream) {
  const int64_t pieces = M * (N / 2) / 8;
  const dim3 grid(static_cast<unsigned>((pieces + kThreads - 1) / kThreads));
  if (dtype == WOL_DTYPE_BF16)
    swiglu_t_kernel<WOL_DTYPE_BF16><<<grid, kThreads, 0, stream>>>(static_cast<const uint16_t*>(in), M, N,
                                                                 static_cast<uint16_t*>(out));
  else
    swiglu_t_kernel<WOL_DTYPE_F16><<<grid, kThreads, 0, stream>>>(static_cast<const uint16_t*>(in), M, N,
                                                                static_cast<uint16_t*>(out));
  return hipGetLastError() == hipSuccess ? WOL_OK : WOL_ERR_HIP;
}

int launch_swiglu_f32(const float* in, int dtype, int64_t M, int64_t N, void* out, hipStream_t stream) {
  const int64_t quads = M * (N / 2) / 4;
  const dim3 grid(static_cast<unsigned>((quads + kThreads - 1) / kThreads));
  if (dtype == WOL_DTYPE_BF16)
    swiglu_f32_kernel<WOL_DTYPE_BF16><<<grid, kThreads, 0, stream>>>(in, M, N, static_cast<uint16_t*>(out));
  else
    swiglu_f32_kernel<WOL_DTYPE_F16><<<grid, kThreads, 0, stream>>>(in, M, N, static_cast<uint16_t*>(out));
  return hipGetLastError() == hipSuccess ? WOL_OK : WOL_ERR_HIP;
}

int launch_prescale(const void* x, const void* scales, int dtype, int64_t rows, int64_t cols,
                    void* out, hipStream_t stream) {
  return dtype == WOL_DTYPE_BF16 ? launch<WOL_DTYPE_BF16>(x, scales, rows, cols, out, stream)
                                 : launch<WOL_DTYPE_F16>(x, scales, rows, cols, out, stream);
}

}  // namespace wol
