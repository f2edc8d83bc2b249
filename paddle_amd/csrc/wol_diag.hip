// Diagnostic kernel: reads a packed weight with the launch shape of the
// one-row streaming kernel (one workgroup of 8 wavefronts per 16-column strip,
// every wavefront loading its 1/8 of the strip's k range with 16-byte
// non-temporal loads, all requested before the first use) and does nothing
// else.  Its time is the floor any decode kernel of that shape has on a given
// machine: launch, first-byte latency and the HBM stream, without a single
// MFMA, scale or activation.
#include "wol_common.h"

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

}  // namespace wol
