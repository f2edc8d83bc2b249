// Diagnostic kernels (include/wol_diag.h).
//
// read_floor_kernel reads a packed weight with the launch shape of the
// one-row streaming kernel (one workgroup of 8 wavefronts per 16-column strip,
// every wavefront loading its 1/8 of the strip's k range with 16-byte
// non-temporal loads, all requested before the first use) and does nothing
// else.  Its time is the floor any decode kernel of that shape has on a given
// machine: launch, first-byte latency and the HBM stream, without a single
// MFMA, scale or activation.
#include "wol_common.h"
#include "wol_diag.h"

namespace wol {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(512) void read_floor_kernel(const uint8_t* __restrict__ codes,
                                                         int64_t strip_bytes_, int pieces_per_wave,
                                                         uint32_t* __restrict__ out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const u32x4* p = reinterpret_cast<const u32x4*>(codes + blockIdx.x * strip_bytes_) +
                   static_cast<int64_t>(wave) * pieces_per_wave * 64 + lane;
  uint32_t acc = 0;
  for (int i = 0; i < pieces_per_wave; i += 4) {
    u32x4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = i + j < pieces_per_wave ? i + j : pieces_per_wave - 1;
      v[j] = __builtin_nontemporal_load(p + static_cast<int64_t>(t) * 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  // one dword per wavefront keeps the loads alive
  if (lane == 0) out[blockIdx.x * 8 + wave] = acc;
}

// Nothing but matrix instructions: 4 x 2 blocks of 32 x 32 per wavefront (the
// register tile of the prefill GEMM), operands loaded once.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(512) void mfma_ceiling_kernel(const u32x4* __restrict__ operands, int iters,
                                                           float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  bf16x8 a[4], b[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = __builtin_bit_cast(bf16x8, operands[i * 64 + lane]);
#pragma unroll
  for (int i = 0; i < 2; ++i) b[i] = __builtin_bit_cast(bf16x8, operands[(4 + i) * 64 + lane]);
  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  out[static_cast<int64_t>(blockIdx.x) * 512 + threadIdx.x] = s;
}

}  // namespace

int launch_read_floor(const void* codes, int64_t K, int64_t N, int bits, void* out,
                      hipStream_t stream) {
  const int64_t sb = strip_bytes(K, bits);
  const int pieces = static_cast<int>(sb / 1024 / 8);  // 1 KiB pieces per wavefront
  if (pieces < 1) return WOL_ERR_BAD_SHAPE;
  read_floor_kernel<<<dim3(static_cast<unsigned>(N / kStripCols)), dim3(512), 0, stream>>>(
      static_cast<const uint8_t*>(codes), sb, pieces, static_cast<uint32_t*>(out));
  return hipGetLastError() == hipSuccess ? WOL_OK : WOL_ERR_HIP;
}

int launch_mfma_ceiling(const void* operands, int workgroups, int iters, float* out,
                        hipStream_t stream) {
  mfma_ceiling_kernel<<<dim3(static_cast<unsigned>(workgroups)), dim3(512), 0, stream>>>(
      static_cast<const u32x4*>(operands), iters, out);
  return hipGetLastError() == hipSuccess ? WOL_OK : WOL_ERR_HIP;
}

}  // namespace wol

extern "C" {

int wol_read_floor(const void* codes, int64_t K, int64_t N, int bits, void* out, void* stream) {
  if (bits != 8 && bits != 4) return WOL_ERR_BAD_BITS;
  if (K <= 0 || N <= 0 || K % 64 != 0 || N % 16 != 0 || K > (int64_t{1} << 24) || N > (int64_t{1} << 24))
    return WOL_ERR_BAD_SHAPE;
  if (K * bits % (8 * 1024 * 8 / 16) != 0) return WOL_ERR_BAD_SHAPE;  // whole 1 KiB pieces per wavefront
  if (codes == nullptr || out == nullptr) return WOL_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(codes) & 15u) != 0) return WOL_ERR_ALIGNMENT;
  return wol::launch_read_floor(codes, K, N, bits, out, static_cast<hipStream_t>(stream));
}

int wol_mfma_ceiling(const void* operands, int workgroups, int iters, float* out, void* stream) {
  if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 24)) return WOL_ERR_BAD_SHAPE;
  if (operands == nullptr || out == nullptr) return WOL_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(operands) & 15u) != 0) return WOL_ERR_ALIGNMENT;
  return wol::launch_mfma_ceiling(operands, workgroups, iters, out, static_cast<hipStream_t>(stream));
}

int wol_decode_phases(const void* x, const void* codes, const void* scale, int64_t K, int64_t N, int group_size,
                      void* out, unsigned long long* phases, size_t phases_bytes, void* stream) {
  if (K != 4096 || N <= 0 || N % 16 != 0 || N > (1 << 24) || (group_size != 64 && group_size != 128))
    return WOL_ERR_BAD_SHAPE;
  if (x == nullptr || codes == nullptr || scale == nullptr || out == nullptr || phases == nullptr) return WOL_ERR_NULL_POINTER;
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(codes) | reinterpret_cast<uintptr_t>(scale) |
        reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(phases)) & 15u) != 0)
    return WOL_ERR_ALIGNMENT;
  if (phases_bytes < static_cast<size_t>(N / 16) * WOL_DECODE_PHASES_PER_WORKGROUP * 8) return WOL_ERR_WORKSPACE;
  return wol::launch_decode_phases(x, codes, scale, K, N, group_size, out, phases, static_cast<hipStream_t>(stream));
}

int wol_prefill_phases(const void* x, const void* codes, const void* scale, int64_t M, int64_t K, int64_t N,
                       void* out, unsigned long long* phases, size_t phases_bytes, void* stream) {
  if (M <= 0 || N <= 0 || M % 256 != 0 || N % 256 != 0 || K % 64 != 0 || K < 192 || M > (1 << 20) || N > (1 << 20) ||
      K > (1 << 20))
    return WOL_ERR_BAD_SHAPE;
  if (x == nullptr || codes == nullptr || scale == nullptr || out == nullptr || phases == nullptr) return WOL_ERR_NULL_POINTER;
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(codes) | reinterpret_cast<uintptr_t>(scale) |
        reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(phases)) & 15u) != 0)
    return WOL_ERR_ALIGNMENT;
  if (phases_bytes < static_cast<size_t>(M / 256) * static_cast<size_t>(N / 256) * WOL_PREFILL_PHASES_PER_WORKGROUP * 8)
    return WOL_ERR_WORKSPACE;
  return wol::launch_prefill_phases(x, codes, scale, M, K, N, out, phases, static_cast<hipStream_t>(stream));
}

int wol_mfma_probe(int variant, const void* operands, size_t operand_bytes, int workgroups, int iters, float* out,
                   void* stream) {
  if (variant < 0 || variant >= WOL_MFMA_PROBE_VARIANTS) return WOL_ERR_BAD_SHAPE;
  if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 24)) return WOL_ERR_BAD_SHAPE;
  if (operands == nullptr || out == nullptr) return WOL_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(operands) & 15u) != 0) return WOL_ERR_ALIGNMENT;
  if (operand_bytes < WOL_MFMA_PROBE_OPERAND_BYTES) return WOL_ERR_WORKSPACE;  // the variants with loads read this much
  return wol::launch_mfma_probe(variant, operands, workgroups, iters, out, static_cast<hipStream_t>(stream));
}

}  // extern "C"
