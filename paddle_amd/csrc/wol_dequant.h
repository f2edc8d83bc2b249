// Offset dequantisation shared by the linear kernels: the stored code turns
// into a bf16/fp16 bit pattern with one or two bit operations, at the price of
// a constant offset that the consumer cancels with one more MFMA against a
// constant B operand (every product and the cancelling term are exact, the
// fp32 accumulation absorbs both).
#pragma once

#include "wol_common.h"

namespace wol {

// Codes of one k step (8 per lane) -> four dwords of T pairs holding
// code + offset exactly, and the B operand that cancels the offset.
//   int4/bf16: nibble | 0x4300      = 128 + (code + 8)      offset 136
//   int4/fp16: nibble<<4 | 0x5400   = 64 + (code + 8)       offset 72
//   int8/bf16: float(byte) high half = code + 128           offset 128
//   int8/fp16: byte | 0x6400        = 1024 + (code + 128)   offset 1152
template <int DT, int BITS>
struct Dequant;

// (v & mask) | magic.  magic arrives in a VGPR whose value the compiler cannot
// see, which lets it pick the three-operand v_and_or_b32 (mask on the scalar
// bus) instead of two instructions with literals.  Written as plain C so the
// compiler's MFMA hazard tracking sees every register it touches.
__device__ inline uint32_t and_or(uint32_t v, uint32_t mask, uint32_t magic) {
  return (v & mask) | magic;
}

template <>
struct Dequant<WOL_DTYPE_BF16, 4> {
  static constexpr uint32_t kCancel = 0xC308C308u;  // -136, -136
  static constexpr float kOffset = 136.0f;
  static constexpr uint32_t kMagic = 0x43004300u;
  __device__ static inline u32x4 run(const uint32_t* w, uint32_t magic) {
    const uint32_t v = w[0];
    u32x4 o;
    o.x = and_or(v, 0x000F000Fu, magic);
    o.y = and_or(v >> 4, 0x000F000Fu, magic);
    o.z = and_or(v >> 8, 0x000F000Fu, magic);
    o.w = and_or(v >> 12, 0x000F000Fu, magic);
    return o;
  }
};

template <>
struct Dequant<WOL_DTYPE_F16, 4> {
  static constexpr uint32_t kCancel = 0xD480D480u;  // -72, -72
  static constexpr float kOffset = 72.0f;
  static constexpr uint32_t kMagic = 0x54005400u;
  __device__ static inline u32x4 run(const uint32_t* w, uint32_t magic) {
    const uint32_t v = w[0];
    u32x4 o;
    o.x = and_or(v << 4, 0x00F000F0u, magic);
    o.y = and_or(v, 0x00F000F0u, magic);
    o.z = and_or(v >> 4, 0x00F000F0u, magic);
    o.w = and_or(v >> 8, 0x00F000F0u, magic);
    return o;
  }
};

template <>
struct Dequant<WOL_DTYPE_BF16, 8> {
  static constexpr uint32_t kCancel = 0xC300C300u;  // -128, -128
  static constexpr float kOffset = 128.0f;
  static constexpr uint32_t kMagic = 0u;
  __device__ static inline uint32_t pair(uint32_t lo_byte_val, uint32_t hi_byte_val) {
    // high halves of two fp32 values side by side (both are exact in bf16)
    return __builtin_amdgcn_perm(__float_as_uint(static_cast<float>(hi_byte_val)),
                                 __float_as_uint(static_cast<float>(lo_byte_val)), 0x07060302u);
  }
  __device__ static inline u32x4 run(const uint32_t* w, uint32_t) {
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
  static constexpr float kOffset = 1152.0f;
  static constexpr uint32_t kMagic = 0x64646464u;
  __device__ static inline u32x4 run(const uint32_t* w, uint32_t magic) {
    u32x4 o;
    o.x = __builtin_amdgcn_perm(w[0], magic, 0x00050004u);
    o.y = __builtin_amdgcn_perm(w[0], magic, 0x00070006u);
    o.z = __builtin_amdgcn_perm(w[1], magic, 0x00050004u);
    o.w = __builtin_amdgcn_perm(w[1], magic, 0x00070006u);
    return o;
  }
};

}  // namespace wol
