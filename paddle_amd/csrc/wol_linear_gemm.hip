// weight_only_linear for large M (prefill): MFMA GEMMs.
//
// gemm_dma_kernel is the kernel that runs whenever K is made of whole k tiles
// (64 k for int8, 128 k for int4): a workgroup of WM x WN wavefronts computes a
// BM x BN tile of the output from TM x TN blocks of v_mfma_f32_32x32x16 per
// wavefront.  Both operands travel global -> LDS with direct-to-LDS loads,
// two or three k tiles deep; the packed weights land as they lie in memory and
// are dequantised in registers to exact signed bf16/fp16 integers on their way
// into the B operand; scales are applied to fp32 accumulators -- in the
// epilogue (per-channel) or once per group -- so code * scale is never rounded
// to T.  For few rows K is cut into runs across workgroups whose fp32 partial
// sums reduce_partials_kernel adds.  Workgroups are numbered so that each XCD
// (one L2 each) works on a compact block of neighbouring tiles.
//
// gemm_kernel (v_mfma_f32_16x16x32, activations staged through registers into
// padded LDS rows, weights loaded straight into B-fragment order) takes the
// remaining K: those that end in a partial k tile.
#include <atomic>

#include "wol_common.h"
#include "wol_dequant.h"

#include <climits>
#include <type_traits>

namespace wol {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
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
  __device__ static inline float sbyte(uint32_t v, int i) {
    return static_cast<float>(static_cast<int>(static_cast<int8_t>((v >> (8 * i)) & 0xFFu)));
  }
  __device__ static inline u32x4 run(const uint32_t* w) {
    // stored byte = code + 128; flipping the top bit gives the two's complement code
    const uint32_t a = w[0] ^ 0x80808080u, b = w[1] ^ 0x80808080u;
    u32x4 o;
    o.x = pack_bf16_hi(sbyte(a, 0), sbyte(a, 1));
    o.y = pack_bf16_hi(sbyte(a, 2), sbyte(a, 3));
    o.z = pack_bf16_hi(sbyte(b, 0), sbyte(b, 1));
    o.w = pack_bf16_hi(sbyte(b, 2), sbyte(b, 3));
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

// Workgroup -> output tile.  Hardware deals consecutive workgroup ids to the
// 8 XCDs in turn; give XCD x the ids that form a compact block of tiles so
// that its L2 sees every A row block and B column block of that block once.
__device__ inline void tile_of_block(int id, int nbx, int nby, int* bx, int* by) {
  const int total = nbx * nby;
  constexpr int kXcd = 8;
  int t = id;
  if (total % kXcd == 0) {
    const int per = total / kXcd;
    t = (id % kXcd) * per + id / kXcd;
  }
  // walk the tiles in column-major panels of 8 row blocks so neighbours share B
  *by = t % nby;
  *bx = t / nby;
}

// The same with a two-dimensional split: the 8 XCDs form a grid of rg x 8/rg
// and each owns nby/rg row blocks x nbx/(8/rg) column blocks, the shape that
// makes the sum of the A rows and B columns an L2 has to fetch smallest
// (plan_xcd_rows on the host).  rg == 0: plain order.
// rg < 0 (the grouped GEMM over experts; nby a multiple of 8 * -rg): runs of
// -rg consecutive row tiles -- one expert's, when the experts have about that
// many -- go to one XCD with all their column tiles, column tile by column
// tile, so that the row tiles of an expert meet its weights in one L2 while
// they are there, and no other XCD fetches them.
__device__ inline void tile_of_block_2d(int id, int nbx, int nby, int rg, int* bx, int* by) {
  if (rg == 0) {
    *by = id % nby;
    *bx = id / nby;
    return;
  }
  constexpr int kXcd = 8;
  if (rg < 0) {
    const int tpe = -rg, x = id % kXcd, i = id / kXcd;
    const int per = tpe * nbx, gi = i / per, w = i % per;
    *by = (gi * kXcd + x) * tpe + w % tpe;
    *bx = w / tpe;
    return;
  }
  const int x = id % kXcd, i = id / kXcd;
  const int r = nby / rg, c = nbx / (kXcd / rg);
  *by = (x % rg) * r + i % r;
  *bx = (x / rg) * c + i / r;
}

template <int DT, int BITS, bool GROUPED, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ codes,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ scale, void* __restrict__ out,
    int M, int K, int N, int gshift, int out_f32, int nbx, int nby, int act) {
  constexpr int NT = 64 * WM * WN;
  constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
  constexpr int TK = BITS == 8 ? 64 : 128;     // k per 16-byte lane load
  constexpr int kDw = BITS == 8 ? 2 : 1;       // dwords per k step
  constexpr int kRow = TK + 8;                 // padded LDS row, in elements
  constexpr int kChunks = BM * (TK / 8) / NT;  // 16-byte pieces of the A tile per thread
  static_assert(BM * (TK / 8) % NT == 0, "A tile must split evenly over the threads");
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // 2 x BM x kRow

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int j = lane & 15, kb = lane >> 4;
  int bx, by;
  tile_of_block(blockIdx.x, nbx, nby, &bx, &by);
  const int m0 = by * BM;
  const int strip0 = bx * (BN / 16) + wn * TN;
  const int nstrips = N / kStripCols;

  // this thread's pieces of the A tile: row r, 8 elements at column 8*cc
  const uint16_t* aptr[kChunks];
  int aoff[kChunks];
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int id = tid + c * NT, r = id / (TK / 8), cc = id % (TK / 8);
    int m = m0 + r;
    m = m < M ? m : M - 1;  // rows past M are computed on valid data and never stored
    aptr[c] = x + static_cast<int64_t>(m) * K + cc * 8;
    aoff[c] = r * kRow + cc * 8;
  }
  // this lane's 16 bytes of every strip of the wavefront
  const uint8_t* bptr[TN];
#pragma unroll
  for (int s = 0; s < TN; ++s) {
    const int st = strip0 + s < nstrips ? strip0 + s : nstrips - 1;  // past N: valid data, never stored
    bptr[s] = codes + static_cast<int64_t>(st) * strip_bytes(K, BITS) + lane * 16;
  }

  f32x4 tot[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b) tot[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int nfull = K / TK;
  const int niter = nfull + ((K % TK) ? 1 : 0);
  u32x4 areg[kChunks];
  u32x4 wcur[TN], wnext[TN];

  auto load_a = [&](int it) {
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
      // the int4 half tile at the end of K has only TK/2 columns
      const bool ok = it < nfull || (aoff[c] % kRow) < TK / 2;
      areg[c] = ok ? *reinterpret_cast<const u32x4*>(aptr[c] + it * TK) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int c = 0; c < kChunks; ++c)
      *reinterpret_cast<u32x4*>(&lds[buf * BM * kRow + aoff[c]]) = areg[c];
  };
  auto load_b = [&](u32x4 (&w)[TN], int it) {
#pragma unroll
    for (int s = 0; s < TN; ++s) {
      if (it < nfull) {
        w[s] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(bptr[s] + it * 1024));
      } else {  // 8 bytes per lane in the half tile
        const u32x2 q = *reinterpret_cast<const u32x2*>(bptr[s] - lane * 8 + nfull * 1024);
        w[s] = u32x4{q.x, q.y, 0u, 0u};
      }
    }
  };

  load_a(0);
  load_b(wcur, 0);
  store_a(0);
  __syncthreads();

  for (int it = 0; it < niter; ++it) {
    const bool more = it + 1 < niter;
    if (more) {
      load_a(it + 1);
      load_b(wnext, it + 1);
    }
    const uint16_t* As = lds + (it & 1) * BM * kRow;
    const int nsub = (it < nfull ? TK : TK / 2) / 64;
#pragma unroll
    for (int sb = 0; sb < TK / 64; ++sb) {
      if (sb >= nsub) break;
      f32x4 part[GROUPED ? TM : 1][GROUPED ? TN : 1];
      if (GROUPED) {
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
          for (int b = 0; b < TN; ++b) part[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const int step = sb * 2 + st;
        u32x4 bfrag[TN];
#pragma unroll
        for (int s = 0; s < TN; ++s) {
          const uint32_t w[4] = {wcur[s].x, wcur[s].y, wcur[s].z, wcur[s].w};
          bfrag[s] = DequantExact<DT, BITS>::run(&w[step * kDw]);
        }
#pragma unroll
        for (int a = 0; a < TM; ++a) {
          const int row = (wm * TM + a) * 16 + j;
          const u32x4 af = *reinterpret_cast<const u32x4*>(&As[row * kRow + step * 32 + kb * 8]);
#pragma unroll
          for (int s = 0; s < TN; ++s) {
            if (GROUPED) part[a][s] = mfma16<DT>(af, bfrag[s], part[a][s]);
            else tot[a][s] = mfma16<DT>(af, bfrag[s], tot[a][s]);
          }
        }
      }
      if (GROUPED) {
        const int g = (it * TK + sb * 64) >> gshift;
#pragma unroll
        for (int s = 0; s < TN; ++s) {
          const int st = strip0 + s < nstrips ? strip0 + s : nstrips - 1;
          const float sc = to_f32<DT>(scale[static_cast<int64_t>(g) * N + st * 16 + j]);
#pragma unroll
          for (int a = 0; a < TM; ++a) tot[a][s] += part[a][s] * sc;
        }
      }
    }
    if (more) store_a((it + 1) & 1);
    __syncthreads();
    if (more) {
#pragma unroll
      for (int s = 0; s < TN; ++s) wcur[s] = wnext[s];
    }
  }

  // ---- epilogue: scale, bias, cast; 16-row slabs leave through LDS ----
  float sc[TN], bv[TN];
#pragma unroll
  for (int s = 0; s < TN; ++s) {
    const int st = strip0 + s < nstrips ? strip0 + s : nstrips - 1;
    const int n = st * 16 + j;
    sc[s] = GROUPED ? 1.0f : to_f32<DT>(scale[n]);
    bv[s] = bias != nullptr ? to_f32<DT>(bias[n]) : 0.0f;
  }
  if (out_f32) {
#pragma unroll
    for (int s = 0; s < TN; ++s) {
      if (strip0 + s >= nstrips) continue;
      const int n = (strip0 + s) * 16 + j;
#pragma unroll
      for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = m0 + (wm * TM + a) * 16 + kb * 4 + r;
          if (m < M) static_cast<float*>(out)[static_cast<int64_t>(m) * N + n] = act_apply(tot[a][s][r] * sc[s] + bv[s], act);
        }
    }
    return;
  }
  constexpr int kSlabRow = TN * 16 + 8;              // padded, in elements
  uint16_t* slab = lds + wave * 16 * kSlabRow;       // private to the wavefront (A buffers are free now)
  static_assert(WM * WN * 16 * kSlabRow <= 2 * BM * kRow, "slabs must fit in the A buffers");
  constexpr int kPieces = 16 * (TN * 16 / 8);        // 16-byte pieces of a slab
#pragma unroll
  for (int a = 0; a < TM; ++a) {
#pragma unroll
    for (int s = 0; s < TN; ++s)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        slab[(kb * 4 + r) * kSlabRow + s * 16 + j] = cast_out<DT>(act_apply(tot[a][s][r] * sc[s] + bv[s], act));
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = lane; p < kPieces; p += 64) {
      const int r = p / (TN * 2), c = p % (TN * 2);   // row of the slab, 8-column piece
      const int m = m0 + (wm * TM + a) * 16 + r;
      const int n = strip0 * 16 + c * 8;
      const u32x4 v = *reinterpret_cast<const u32x4*>(&slab[r * kSlabRow + c * 8]);
      if (m < M && n < N)
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(out) + static_cast<int64_t>(m) * N + n) = v;
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// s_waitcnt that only bounds the number of outstanding vector-memory loads.
template <int N_>
__device__ inline void wait_vmcnt() {
  // gfx9 encoding: vmcnt = [15:14][3:0], expcnt = [6:4], lgkmcnt = [11:8]
  __builtin_amdgcn_s_waitcnt((N_ & 0xF) | ((N_ >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// XOR applied to the 16-byte piece index of an A row in LDS (C pieces per
// row).  A lane group reads the same piece of 16 consecutive rows; the XOR
// spreads those reads over the banks whether the LDS serves 8 or 16 lanes of
// a 128-bit read per cycle.
template <int C>
__device__ inline int a_swizzle(int row) {
  if (C == 8) return (row & 7) ^ ((row >> 3) & 1);  // 128-byte rows
  return row & (C - 1);                             // 256-byte rows
}

typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int DT>
__device__ inline f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if (DT == WOL_DTYPE_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// acc + the sum of the eight T values of an operand fragment, in fp32 (four
// packed dot products against (1, 1)).
template <int DT>
__device__ inline float sum8(u32x4 v, float acc) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (DT == WOL_DTYPE_BF16)
      acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w[i]), __builtin_bit_cast(bf16x2, 0x3F803F80u), acc, false);
    else
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, w[i]), __builtin_bit_cast(h16x2, 0x3C003C00u), acc, false);
  }
  return acc;
}

// What one launch of the fast kernel works on.
struct DmaParams {
  const uint16_t* x;
  const uint8_t* codes;
  const uint16_t* bias;
  const uint16_t* scale;
  void* out;                    // T or fp32 [M, N]; with nsplit > 1 fp32 partial sums
                                // [nsplit][M][columns of the launch]
  int M, K, N;
  int out_f32;
  int strip_lo, strip_hi;       // the launch covers the 16-column strips [strip_lo, strip_hi)
  int nbx, nby;                 // output tiles of the launch
  int nsplit, tiles_per_split;  // K is cut into nsplit runs of k tiles, one workgroup each
  int xcd_rows;                 // row groups of the XCD grid (tile_of_block), 0 = plain order
  int act;                      // WOL_ACT_NONE or WOL_ACT_GELU, applied where the final sum is formed
  // Grouped launch (mixture of experts): row tile `by` of the launch is entry
  // `by` of this table -- {expert, first row, rows} -- written on the device by
  // moe_plan_kernel; an expert's rows use that expert's weights, scales and
  // bias (consecutive tensors, the strides below apart).  Null: one problem.
  const int* moe_table;
  int64_t moe_codes_stride;     // bytes between two experts' packed weights
  int moe_rows;                 // rows of the whole grouped problem (the partial sums' row count)
  // STAMP instantiation only: six cycle counts per wavefront, [workgroup][wavefront][8] (see wol_prefill_phases)
  unsigned long long* stamps;
};

// One entry of the row-tile table of a grouped launch.
struct MoeTile {
  int expert;  // -1: the tile is not used
  int row0;    // first row of the tile in the permuted input
  int rows;    // rows of the tile that exist (1 .. tile height)
  int pad;
};

// Fast path: K a multiple of the tile depth.
//
// v_mfma_f32_32x32x16 is the instruction that reaches the matrix cores' full
// rate on gfx950 (the 16x16x32 form issues at half of it), so the wavefront
// tile is built from 32 x 32 blocks: TM x TN of them.  Both operands travel
// global -> LDS with direct-to-LDS loads (no registers, no LDS store
// instructions), STAGES k tiles deep: while tile `it` is consumed the loads of
// tiles it+1 (and, with three stages, it+2) are in flight.  A lands in LDS as unpadded rows whose
// 16-byte pieces are XOR-swizzled by row so a lane group's fragment reads
// fall into distinct banks.  The raw packed B tiles land exactly as they lie
// in memory (16-column strips in 16x16x32 order); a 32x32x16 B operand is
// assembled by letting lane l = 32*b + 16*sp + j read the 16 bytes that lane
// j + 16*(2h + b) of strip sp owns: MFMA (step, h) then contracts over
// k = 32*step + 16*h + 8*b + i, and the A fragment for it is simply piece
// 4*step + 2*h + b of the row.
//
// G = 0: per-channel scales, applied in the epilogue.  G = 64 or 128:
// group-wise scales; the MFMAs of a group accumulate into `part`, which is
// folded into the running sum with the group's scale (an fp32 FMA per
// accumulator element), so code * scale is never rounded to T.
//
// OFFS selects the offset dequantiser: a fraction of the VALU work, and the
// constant offset of every code is taken out again as -offset * (sum of the
// row's activations).  OFFS = 1 forms that sum with one more MFMA per A
// fragment and slice against a constant B operand (into `canc`, added when
// the scale is applied) -- the right trade when M is small: the matrix pipe
// idles, the VALU does not.  OFFS = 2 forms it with four packed dot products
// per A fragment (a lane adds up the eight activations of its fragment; the
// two lanes that share a row meet in the epilogue), which costs no MFMA and
// no accumulators and is what lets int4 weights under bf16 activations take
// the largest tile; per-channel scales only.
//
// With nsplit > 1 a workgroup covers only a run of k tiles and leaves its
// fp32 sums (scaled, without bias) in a partial buffer; reduce_partials_kernel
// adds the runs.  That is what fills the CUs when M is small.
//
// SWI != 0: swiglu in the epilogue (TN = 2, per-channel scales).  The weight is
// a gate | up projection, [K, N] with the gate in columns 0 .. N/2-1; block 0
// of every wavefront then takes 32 gate columns and block 1 the 32 up columns
// N/2 further on, so that silu(gate) * up is formed lane by lane from the two
// accumulators and only [M, N/2] leaves the kernel.  SWI = 1 applies it to the
// fp32 sums (wol_linear_fused); SWI = 2 first rounds both sums to T, as a
// separate fc1 output would have been (the mixture-of-experts FFN).
//
// RESC (group-wise scales): one set of accumulators instead of two.  The
// running sums are kept in units of the current group's scale: where a group
// starts they are multiplied by (previous unit / new unit) and the group's
// MFMAs then accumulate straight into them; the epilogue multiplies by the last
// unit.  Every rescaling rounds the sums once (2^-24 relative, a few dozen
// times per output element), code * scale is still never rounded to T, and
// the registers of the second accumulator set are free for the largest tile.
// The unit of a column follows its group scale but never falls more than 2^64
// below the largest scale the column has had so far (a group that small
// weighs nothing next to the others in fp32), so the sums cannot overflow
// however the scales of a column differ.
//
// STAMP (a diagnostic instantiation, never on a product path): every wavefront
// reads the cycle counter at kernel entry, around the two waits of every k
// tile (for its own tile loads, then for the workgroup) and around the
// epilogue, and leaves the sums in p.stamps.  The reads sit where the
// wavefront has just waited for all its LDS traffic anyway.
template <int DT, int BITS, int G, int OFFS, int WM, int WN, int TM, int TN, int STAGES, int SWI = 0, bool RESC = false,
          bool STAMP = false>
__global__ __launch_bounds__(64 * WM * WN) void gemm_dma_kernel(const DmaParams p) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  constexpr int NW = WM * WN;
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int TK = BITS == 8 ? 64 : 128;       // k per 16-byte lane load of B
  constexpr int kDw = BITS == 8 ? 2 : 1;         // dwords per 8 codes
  constexpr int C = TK / 8;                      // 16-byte pieces per A row
  constexpr int kABytes = BM * TK * 2;           // one A tile
  constexpr int kBBytes = (BN / 16) * 1024;      // one raw B tile (all strips of the workgroup)
  constexpr int kSBytes = G == 0 ? 0 : NW * 256;  // the tile's group scales: 128 values per wavefront
  constexpr int kStage = kABytes + kBBytes + kSBytes;
  constexpr int kStages = STAGES;  // k tiles resident or in flight
  static_assert(kStages == 2 || kStages == 3, "two or three stages");
  constexpr int kALoads = kABytes / 1024 / NW;   // wave-level loads (1 KiB each) per wavefront
  constexpr int kBLoads = BN / 16 / NW;
  static_assert(kABytes / 1024 % NW == 0 && kALoads >= 1, "A tile must split evenly over the wavefronts");
  static_assert(BN / 16 % NW == 0 && kBLoads >= 1, "B tile must split evenly over the wavefronts");
  constexpr int Q = TK / 16;  // 16-k slices (one MFMA per 32x32 block each) per tile
  // group-wise scales: a fold every kFold slices, kGT folds (groups or halves of one) per tile
  constexpr int kFoldK = G == 0 ? TK : (G < TK ? G : TK);
  constexpr int kFold = kFoldK / 16;
  constexpr int kGT = TK / kFoldK;
  constexpr int kGShift = G == 128 ? 7 : 6;
  static_assert(kGT * BN <= NW * 128, "the tile's scales must fit the wavefronts' 4-byte loads");
  // direct-to-LDS loads every lane issues per stage.  They are the only vector
  // memory loads of the main loop, so they complete in issue order and
  // s_waitcnt vmcnt(n) can tell which stages have landed.
  constexpr int kPerStage = kALoads + kBLoads + (G == 0 ? 0 : 1);
  static_assert(Q >= 2 && (Q - 2) % kFold != 0 && (Q - 2) % kFold != kFold - 1,
                "the slice that holds the barrier neither starts nor ends a group");
  static_assert(SWI == 0 || ((TN == 2 || (TN == 1 && WN % 2 == 0)) && (G == 0 || RESC)),
                "the swiglu epilogue pairs the two blocks of a wavefront, or two neighbouring wavefronts");
  // SWI with one block per wavefront: wavefront columns 2i and 2i+1 hold the gate and the up block of
  // the same 32 output columns, and the up wavefront hands its sums over through LDS in the epilogue
  constexpr bool kPair = SWI != 0 && TN == 1;
  static_assert(OFFS != 2 || G == 0, "row sums by dot products are taken out once, in the epilogue");
  static_assert(!RESC || (G != 0 && OFFS == 0), "rescaled sums are for group-wise scales and the exact dequantisers");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned long long st_entry = 0, st_prev = 0, st_work = 0, st_loads = 0, st_bar = 0, st_loop0 = 0;
  if (STAMP) st_entry = __builtin_readcyclecounter();

  const uint16_t* __restrict__ x = p.x;
  const uint16_t* __restrict__ scale = p.scale;
  const uint16_t* __restrict__ bias = p.bias;
  const uint8_t* __restrict__ codes = p.codes;
  void* outp = p.out;
  int M = p.M;
  const int K = p.K, N = p.N;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int j = lane & 15, sp = (lane >> 4) & 1, b = lane >> 5, r32 = lane & 31;
  const int ntiles = p.nbx * p.nby;
  const int split = blockIdx.x / ntiles;
  int bx, by;
  tile_of_block_2d(blockIdx.x - split * ntiles, p.nbx, p.nby, p.xcd_rows, &bx, &by);
  int m0 = by * BM;
  if (p.moe_table != nullptr) {
    // this row tile belongs to one expert: shift every base to that expert and
    // to the tile's first row, and let M be the rows that exist
    const MoeTile t = reinterpret_cast<const MoeTile*>(p.moe_table)[by];
    if (t.expert < 0) return;
    x += static_cast<int64_t>(t.row0) * K;
    if (p.nsplit > 1) outp = static_cast<float*>(outp) + static_cast<int64_t>(t.row0) * N;  // partial sums
    else outp = static_cast<uint16_t*>(outp) + static_cast<int64_t>(t.row0) * (SWI ? N / 2 : N);
    codes += static_cast<int64_t>(t.expert) * p.moe_codes_stride;
    scale += static_cast<int64_t>(t.expert) * N;
    if (bias != nullptr) bias += static_cast<int64_t>(t.expert) * N;
    M = t.rows;
    m0 = 0;
  }
  // SWI: a workgroup takes BN / 2 gate columns and the BN / 2 up columns that go with them
  const int strip_blk = p.strip_lo + bx * (SWI ? BN / 32 : BN / 16);
  const int nstrips = p.strip_hi;
  const int n_hi = p.strip_hi * kStripCols;
  const int up_strips = N / 2 / kStripCols;  // SWI: strips between a gate column and its up column
  // this workgroup's run of k tiles
  const int t0 = split * p.tiles_per_split;
  const int niter = (K / TK - t0) < p.tiles_per_split ? (K / TK - t0) : p.tiles_per_split;
  auto tile_index = [&](int it) {  // past the end of the run: the last tile again
    return it < niter ? it : niter - 1;
  };

  // global source of this lane for each of its A loads: LDS piece q holds row
  // q / C, piece (q % C) ^ swizzle(row) of the tile
  const uint16_t* asrc[kALoads];
#pragma unroll
  for (int c = 0; c < kALoads; ++c) {
    const int q = (c * NW + wave) * 64 + lane;
    const int row = q / C, slot = q % C;
    const int cc = slot ^ a_swizzle<C>(row);
    int m = m0 + row;
    m = m < M ? m : M - 1;  // rows past M are computed on valid data and never stored
    asrc[c] = x + static_cast<int64_t>(m) * K + static_cast<int64_t>(t0) * TK + cc * 8;
  }
  const uint8_t* bsrc[kBLoads];
#pragma unroll
  for (int c = 0; c < kBLoads; ++c) {
    int st = strip_blk + c * NW + wave;
    if (SWI) {
      // LDS slot L of the B tile serves wavefront column L / 4, block (L / 2) % 2, half L % 2
      const int L = c * NW + wave;
      st = strip_blk + (L / 4) * 2 + L % 2;
    }
    st = st < nstrips ? st : nstrips - 1;  // past the last column: valid data, never stored
    if (SWI && ((c * NW + wave) / 2) % 2 == 1) st += up_strips;  // block 1: the up columns
    bsrc[c] = codes + static_cast<int64_t>(st) * strip_bytes(K, BITS) +
              static_cast<int64_t>(t0) * 1024 + lane * 16;
  }
  const int swz = a_swizzle<C>(lane & 15);  // fragment rows are 32*t + r32; the swizzle has period 16

  // Group scales travel with the tile: value v = 2 * (64 * wave + lane) of the
  // flattened [kGT][BN] block of the tile's scale rows, two values per lane.
  const int sval = 2 * (wave * 64 + lane) < kGT * BN ? 2 * (wave * 64 + lane) : 0;
  const int sfold = sval / BN;
  int scol = strip_blk * kStripCols + sval % BN;
  if (SWI) {
    // position p of the tile's columns is column p % 32 of block (p / 32) % 2 of wavefront column p / 64:
    // the gate columns of that wavefront column, or the up columns N / 2 further on
    const int pcol = sval % BN;
    scol = (strip_blk + (pcol / 64) * 2) * kStripCols + pcol % 32;
    scol = scol < n_hi ? scol : n_hi - 2;
    scol += ((pcol / 32) % 2) * (N / 2);
  }
  scol = scol < (SWI ? N : n_hi) ? scol : n_hi - 2;  // past the last column: valid data, never used
  // Loads lo .. hi-1 of tile `it` into its stage; a stage's loads are numbered
  // [scales,] A loads, B loads.
  auto issue_range = [&](int it, int lo, int hi) {
    const int t = tile_index(it);  // past the end: reload the last tile into a spare stage
    unsigned char* stage = smem + (it % kStages) * kStage;
    constexpr int kS = G == 0 ? 0 : 1;
    if (G != 0 && lo == 0 && hi > 0) {
      const int64_t row = (static_cast<int64_t>(t0 + t) * TK + sfold * kFoldK) >> kGShift;
      __builtin_amdgcn_global_load_lds(scale + row * N + scol,
                                       (lds_ptr_t)(stage + kABytes + kBBytes + wave * 256), 4, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < kALoads; ++c)
      if (kS + c >= lo && kS + c < hi)
        __builtin_amdgcn_global_load_lds(asrc[c] + t * TK, (lds_ptr_t)(stage + (c * NW + wave) * 1024), 16, 0, 0);
#pragma unroll
    for (int c = 0; c < kBLoads; ++c)
      if (kS + kALoads + c >= lo && kS + kALoads + c < hi)
        __builtin_amdgcn_global_load_lds(bsrc[c] + t * 1024,
                                         (lds_ptr_t)(stage + kABytes + (c * NW + wave) * 1024), 16, 0, 0);
  };
  auto issue = [&](int it) { issue_range(it, 0, kPerStage); };
  // With three stages the loads of tile it+3 may be issued anywhere between the
  // barrier of tile `it` (which frees their stage) and the barrier of tile it+1,
  // and still have a whole tile period to land.  They are spread over that
  // period, a few per slice: issued in one burst right behind the barrier, the
  // loads of all wavefronts meet in the one load path of the CU at the same
  // moment, and a wavefront that waits there issues no MFMA.  Segment 0 is the
  // half slice behind the barrier, segment 1 the last slice of the tile,
  // segments 2 .. Q-1 the slices 0 .. Q-3 of the next tile.  Two stages leave
  // no such freedom: everything goes out behind the barrier.
  constexpr bool kSpread = kStages == 3;
  auto seg_lo = [](int s) { return kSpread ? (s * kPerStage + Q - 1) / Q : (s > 0 ? kPerStage : 0); };
  auto seg_n = [&](int s) { return seg_lo(s + 1) - seg_lo(s); };

  // columns of this lane's accumulators: block c of the wavefront, column r32
  const int col0 = (strip_blk + (kPair ? wn / 2 : wn) * (SWI ? 1 : TN) * 2) * 16;
  int ncol[TN];
#pragma unroll
  for (int c = 0; c < TN; ++c) {
    const int n = col0 + c * 32 + r32;
    ncol[c] = n < n_hi ? n : n_hi - 1;
    if (SWI && c == 1) ncol[c] = ncol[0] + N / 2;
  }
  if (kPair && wn % 2 == 1) ncol[0] += N / 2;
  // this lane's scales of the tile in `stage`, out of LDS
  auto read_scales = [&](const unsigned char* stage, uint16_t (&dst)[kGT > 0 ? kGT : 1][TN]) {
    if (G != 0) {
#pragma unroll
      for (int f = 0; f < kGT; ++f)
#pragma unroll
        for (int c = 0; c < TN; ++c)
          dst[f][c] = *reinterpret_cast<const uint16_t*>(
              stage + kABytes + kBBytes + (f * BN + (wn * TN + c) * 32 + r32) * 2);
    }
  };

  f32x16 tot[TM][TN];
  f32x16 part[G != 0 && !RESC ? TM : 1][G != 0 && !RESC ? TN : 1];
  float unit[TN], mrun[TN];  // RESC: what one unit of this lane's sums of block c is worth; the largest scale so far
#pragma unroll
  for (int c = 0; c < TN; ++c) unit[c] = mrun[c] = 0.0f;
  f32x16 canc[OFFS == 1 ? TM : 1];
  float rsum[OFFS == 2 ? TM : 1];  // this lane's share of the sum of the activations of row r32 of block a
#pragma unroll
  for (int a = 0; a < TM; ++a) {
#pragma unroll
    for (int c = 0; c < TN; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) tot[a][c][r] = 0.0f;
    if (OFFS == 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) canc[a][r] = 0.0f;
    }
    if (OFFS == 2) rsum[a] = 0.0f;
  }
  uint32_t magic = Dequant<DT, BITS>::kMagic;
  asm volatile("" : "+v"(magic));  // keep the constant in a VGPR

  // byte offsets inside a stage that do not change from tile to tile
  const int a_row_off = (wm * TM * 32 + r32) * (TK * 2);
  const int b_off = kABytes + (wn * TN * 2 + sp) * 1024 + (j + 16 * b) * 16;
  constexpr int kValuPerMfma = ((OFFS == 2 ? 4 * TN + 4 * TM : (BITS == 8 ? 16 : 12) * TN) + TM * TN - 1) / (TM * TN) + 2;
  constexpr int kValuRescale = RESC ? 16 : 0;  // more per MFMA in the slice that starts a group
  constexpr int kHalf = (TM * TN + 1) / 2;  // MFMAs of a slice issued before the barrier
  // (With one workgroup per CU, wavefronts w and w + 4 share a SIMD and the older one wins every
  // arbitration: it finishes a k tile in two thirds of the tile's time and waits out the rest at the
  // barrier.  Handing the priority back and forth with s_setprio evens their arrival out and makes the
  // kernel 3 % slower: the tile's period follows the sum of their work, and the switches add to it.)

  // The wavefront's pipeline registers: raw codes of the current and the next
  // tile, and two sets of operands -- the one the MFMAs of slice q use and the
  // one being prepared for slice q+1 (A fragments read from LDS, B fragments
  // dequantised).
  u32x4 braw[2][TN][2];
  uint16_t sraw[kGT > 0 ? kGT : 1][TN];
  u32x4 af[2][TM];
  u32x4 bf[2][TN];
  auto read_b = [&](const unsigned char* stage, u32x4 (&dst)[TN][2]) {
#pragma unroll
    for (int c = 0; c < TN; ++c)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        dst[c][h] = *reinterpret_cast<const u32x4*>(stage + b_off + c * 2048 + h * 512);
  };
  auto read_a = [&](const unsigned char* stage, u32x4 (&dst)[TM], int q) {
#pragma unroll
    for (int a = 0; a < TM; ++a) {
      const int slot = (2 * q + b) ^ swz;
      dst[a] = *reinterpret_cast<const u32x4*>(stage + a_row_off + a * 32 * (TK * 2) + slot * 16);
    }
  };
  auto dequant = [&](u32x4 (&dst)[TN], const u32x4 (&raw)[TN][2], int q) {
    const int step = q / 2, h = q % 2;
#pragma unroll
    for (int c = 0; c < TN; ++c) {
      const uint32_t w4[4] = {raw[c][h].x, raw[c][h].y, raw[c][h].z, raw[c][h].w};
      if (OFFS) dst[c] = Dequant<DT, BITS>::run(&w4[step * kDw], magic);
      else dst[c] = DequantExact<DT, BITS>::run(&w4[step * kDw]);
    }
  };
  // MFMAs lo .. hi-1 (numbered a * TN + c) of slice q
  // gstart: the tile starts a group (a group of 128 spans two int8 tiles: the second one of a pair does not)
  auto mfmas = [&](const u32x4 (&a4)[TM], const u32x4 (&b4)[TN], int q, int lo, int hi, bool gstart = true) {
    const bool first = q % kFold == 0 && (!RESC || gstart);
    f32x16 zero;
#pragma unroll
    for (int r = 0; r < 16; ++r) zero[r] = 0.0f;
    float rho[TN];
    if (RESC && first) {
#pragma unroll
      for (int c = 0; c < TN; ++c) {
        const float s = to_f32<DT>(sraw[q / kFold][c]);
        mrun[c] = fmaxf(mrun[c], s);
        const float u0 = fmaxf(s, mrun[c] * 0x1p-64f);
        // a scale of zero before any other (or one in the denormal range, which the reciprocal below
        // does not take): the unit stays what it is
        const float u = u0 < 0x1p-126f ? unit[c] : u0;
        // what was summed under a unit of zero (groups whose scale is zero may hold any codes) counts
        // for nothing; inside a group, and from a group to one of the same scale, nothing changes
        rho[c] = unit[c] == 0.0f ? 0.0f : (u == unit[c] ? 1.0f : unit[c] * __builtin_amdgcn_rcpf(u));
        unit[c] = u;
      }
    }
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int c = 0; c < TN; ++c)
        if (a * TN + c >= lo && a * TN + c < hi) {
          if (OFFS == 2 && c == 0) {
            rsum[a] = sum8<DT>(a4[a], rsum[a]);
            // pinned to this slice: left alone the compiler sinks the sums of a
            // whole tile behind the loop's branch and keeps every fragment alive for them
            asm volatile("" : "+v"(rsum[a]));
          }
          if (OFFS == 1 && c == 0) {
            const u32x4 cb = {Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel,
                              Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel};
            canc[a] = mfma32<DT>(a4[a], cb, (G != 0 && first) ? zero : canc[a]);
          }
          if (RESC && first) {
            f32x16 t = tot[a][c];
#pragma unroll
            for (int r = 0; r < 16; ++r) t[r] *= rho[c];
            tot[a][c] = mfma32<DT>(a4[a], b4[c], t);
          } else if (G == 0 || RESC) {
            tot[a][c] = mfma32<DT>(a4[a], b4[c], tot[a][c]);
          } else if (first) {
            part[a][c] = mfma32<DT>(a4[a], b4[c], zero);
          } else {
            part[a][c] = mfma32<DT>(a4[a], b4[c], part[a][c]);
          }
        }
  };
  // after the last slice of a group: tot += part * scale
  auto fold = [&](const uint16_t (&sr)[kGT > 0 ? kGT : 1][TN], int q) {
    if (G != 0 && !RESC && q % kFold == kFold - 1) {
#pragma unroll
      for (int c = 0; c < TN; ++c) {
        const float sc = to_f32<DT>(sr[q / kFold][c]);
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            tot[a][c][r] = fmaf(OFFS == 1 ? part[a][c][r] + canc[a][r] : part[a][c][r], sc, tot[a][c][r]);
      }
    }
  };

  issue(0);
  issue(1);
  if (kStages == 3) issue_range(2, 0, seg_lo(2));  // the rest of tile 2 goes out during tile 0
  wait_vmcnt<(kStages - 2) * kPerStage + (kStages == 3 ? (2 * kPerStage + Q - 1) / Q : kPerStage)>();  // tile 0 has landed
  __builtin_amdgcn_s_barrier();
  if (STAMP) st_loop0 = st_prev = __builtin_readcyclecounter();
  read_b(smem, braw[0]);
  read_a(smem, af[0], 0);
  dequant(bf[0], braw[0], 0);
  // Every slice runs its MFMAs with the preparation of the next slice's
  // operands (A fragments read from LDS, B fragments dequantised) spread
  // between them, so that the VALU work executes in the shadow of the matrix
  // pipe.  The workgroup barrier that hands the stage of tile `it` over to
  // tile it+3 sits in the middle of the last but one slice, once the
  // wavefront has fetched its last operands of the tile; the raw codes of tile
  // it+1 are read right behind it and have a whole slice to arrive.
  auto tile = [&](auto odd_tile, int it, u32x4 (&raw)[TN][2], u32x4 (&raw_next)[TN][2]) {
    // RESC with groups of two tiles: the run starts on a group (launch_dma sees to it), so odd tiles continue one
    constexpr bool gstart = !(RESC && G > TK && decltype(odd_tile)::value);
    const unsigned char* stage = smem + (it % kStages) * kStage;
    const unsigned char* next = smem + ((it + 1) % kStages) * kStage;
    read_scales(stage, sraw);  // before the stage is handed over
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      if (q != Q - 2) {
        const bool last = q == Q - 1;
        // this slice's share of the tile loads (segment 1 of tile it+3, or segment q+2 of tile it+2)
        const int seg = last ? 1 : q + 2;
        if (kSpread) issue_range(last ? it + kStages : it + kStages - 1, seg_lo(seg), seg_lo(seg + 1));
        read_a(last ? next : stage, af[(q + 1) & 1], last ? 0 : q + 1);
        dequant(bf[(q + 1) & 1], last ? raw_next : raw, last ? 0 : q + 1);
        mfmas(af[q & 1], bf[q & 1], q, 0, TM * TN, gstart);
#pragma unroll
        for (int i = 0; i < TM * TN; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                   // one MFMA
          if (i < TM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);       // one LDS read
          if (kSpread && i % 2 == 1 && i / 2 < seg_n(seg)) {
            __builtin_amdgcn_sched_group_barrier(0x004, 2, 0);                 // its LDS address into m0
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                 // one tile load
          }
          if (RESC && gstart && q % kFold == 0) __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma + kValuRescale, 0);
          else __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma, 0);  // VALU
        }
        __builtin_amdgcn_sched_barrier(0);
        fold(sraw, q);
      } else {
        read_a(stage, af[(q + 1) & 1], q + 1);
        mfmas(af[q & 1], bf[q & 1], q, 0, kHalf);
#pragma unroll
        for (int i = 0; i < kHalf; ++i) {
          if (2 * i < TM) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // this wavefront needs nothing more from the tile's stage; once every
        // wavefront is there, tile it+1 (landed by now) may be read and the
        // stage refilled with tile it+3
        __builtin_amdgcn_s_waitcnt(0x0070 | (0xF << 0) | (3 << 14));  // lgkmcnt(0)
        unsigned long long st_a = 0, st_b = 0;
        if (STAMP) st_a = __builtin_readcyclecounter();
        wait_vmcnt<(kStages - 2) * kPerStage>();
        if (STAMP) st_b = __builtin_readcyclecounter();
        __builtin_amdgcn_s_barrier();
        if (STAMP) {
          const unsigned long long st_c = __builtin_readcyclecounter();
          st_work += st_a - st_prev;
          st_loads += st_b - st_a;
          st_bar += st_c - st_b;
          st_prev = st_c;
        }
        issue_range(it + kStages, 0, seg_lo(1));
        read_b(next, raw_next);
        dequant(bf[(q + 1) & 1], raw, q + 1);
        mfmas(af[q & 1], bf[q & 1], q, kHalf, TM * TN);
#pragma unroll
        for (int i = 0; i < TM * TN - kHalf + 1; ++i) {
          if (i < TM * TN - kHalf) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (i < 2 * TN) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (kSpread && i < seg_n(0)) {
            __builtin_amdgcn_sched_group_barrier(0x004, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x002, 2 * kValuPerMfma, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  for (int it = 0; it < niter; it += 2) {
    tile(std::false_type(), it, braw[0], braw[1]);
    if (it + 1 < niter) tile(std::true_type(), it + 1, braw[1], braw[0]);
  }
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();  // the spare loads are done and every wavefront has stopped reading
  unsigned long long st_loop1 = 0;
  if (STAMP) st_loop1 = __builtin_readcyclecounter();
  // the stamps leave at the end of the epilogue (lane 0 of every wavefront)
  auto leave_stamps = [&]() {
    if (STAMP && lane == 0 && p.stamps != nullptr) {
      unsigned long long* o = p.stamps + (static_cast<size_t>(blockIdx.x) * NW + wave) * 8;
      const unsigned long long st_end = __builtin_readcyclecounter();
      o[0] = st_loop0 - st_entry;   // entry to the first tile's barrier
      o[1] = st_work;               // between the barriers: MFMAs and everything issued among them
      o[2] = st_loads;              // waiting for this wavefront's own tile loads
      o[3] = st_bar;                // waiting for the other wavefronts
      o[4] = st_loop1 - st_prev;    // the last tile's tail and the closing barrier
      o[5] = st_end - st_loop1;     // epilogue
      o[6] = st_end - st_entry;     // all of it
      o[7] = static_cast<unsigned long long>(niter);
    }
  };

  // ---- epilogue: scale, bias, cast; 32-row slabs leave through LDS as 16-byte stores ----
  // accumulator element r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its block
  float sc[TN], bv[TN];
#pragma unroll
  for (int c = 0; c < TN; ++c) {
    sc[c] = RESC ? unit[c] : (G == 0 ? to_f32<DT>(scale[ncol[c]]) : 1.0f);
    bv[c] = (bias != nullptr && p.nsplit == 1) ? to_f32<DT>(bias[ncol[c]]) : 0.0f;
  }
  if (OFFS == 1 && G == 0) {
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int c = 0; c < TN; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) tot[a][c][r] += canc[a][r];
  }
  if (OFFS == 2) {
    // Row sums: lanes l and l + 32 hold the two halves of row r32's sum.  They
    // are added and parked in LDS (the stages are free now), from where a lane
    // takes the sums of the sixteen rows its accumulators belong to.
    constexpr int kRsOff = kStages * kStage - NW * TM * 32 * 4;  // the end of the stages; the slabs use their start
    static_assert(kRsOff >= NW * 32 * ((SWI ? 1 : TN) * 32 + 8) * 2, "row sums and slabs must not overlap");
    float* rsl = reinterpret_cast<float*>(smem + kRsOff) + wave * TM * 32;
#pragma unroll
    for (int a = 0; a < TM; ++a) {
      const float other = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(((lane ^ 32) << 2), __builtin_bit_cast(int, rsum[a])));
      if (b == 0) rsl[a * 32 + r32] = rsum[a] + other;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 rv = *reinterpret_cast<const f32x4*>(&rsl[a * 32 + 8 * q4 + 4 * b]);
#pragma unroll
        for (int c = 0; c < TN; ++c)
#pragma unroll
          for (int e = 0; e < 4; ++e) tot[a][c][4 * q4 + e] = fmaf(-Dequant<DT, BITS>::kOffset, rv[e], tot[a][c][4 * q4 + e]);
      }
    __builtin_amdgcn_wave_barrier();
  }
  if (p.out_f32 || p.nsplit > 1) {
    // fp32 results (verification mode) or partial sums of this run of k tiles: plain stores
    // partial sums are kept compact: row length = the columns of this launch
    const int64_t ld = p.nsplit > 1 ? static_cast<int64_t>(p.strip_hi - p.strip_lo) * kStripCols : N;
    const int ncol0 = p.nsplit > 1 ? p.strip_lo * kStripCols : 0;
    const int64_t run_rows = p.moe_table != nullptr ? p.moe_rows : M;  // rows of one run's partial sums
    float* outf = static_cast<float*>(outp) + (p.nsplit > 1 ? static_cast<int64_t>(split) * run_rows * ld : 0);
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int c = 0; c < TN; ++c) {
        const int n = col0 + c * 32 + r32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + (wm * TM + a) * 32 + 8 * (r / 4) + 4 * b + r % 4;
          if (m < M && n < n_hi) {
            const float v = tot[a][c][r] * sc[c] + bv[c];  // a partial sum when K is cut into runs
            outf[static_cast<int64_t>(m) * ld + (n - ncol0)] = p.nsplit > 1 ? v : act_apply(v, p.act);
          }
        }
      }
    return;
  }
  uint16_t* out = static_cast<uint16_t*>(outp);
  constexpr int kOutBlocks = SWI ? 1 : TN;        // 32-column blocks a wavefront writes
  constexpr int kSlabRow = kOutBlocks * 32 + 8;   // padded, in elements
  static_assert(NW * 32 * kSlabRow * 2 <= kStages * kStage, "slabs must fit in the stage buffers");
  uint16_t* slab = reinterpret_cast<uint16_t*>(smem) + wave * 32 * kSlabRow;
  constexpr int kPieces = 32 * (kOutBlocks * 32 / 8);
  const int ld_out = SWI ? N / 2 : N;             // row length of the output
  if constexpr (kPair) {
    // behind the slabs: one block of fp32 sums per pair of wavefronts
    constexpr int kXOff = (NW * 32 * kSlabRow * 2 + 255) / 256 * 256;
    static_assert(kXOff + NW / 2 * 4096 <= kStages * kStage, "slabs and handed-over sums must fit in the stage buffers");
    float* xbuf = reinterpret_cast<float*>(smem + kXOff) + (wave / 2) * 1024;
#pragma unroll
    for (int a = 0; a < TM; ++a) {
      if (wn % 2 == 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) xbuf[r * 64 + lane] = tot[a][0][r] * sc[0] + bv[0];
      }
      __syncthreads();
      if (wn % 2 == 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float g = tot[a][0][r] * sc[0] + bv[0], u = xbuf[r * 64 + lane];
          if (SWI == 2) {
            g = to_f32<DT>(cast_out<DT>(g));
            u = to_f32<DT>(cast_out<DT>(u));
          }
          slab[(8 * (r / 4) + 4 * b + r % 4) * kSlabRow + r32] = cast_out<DT>(act_swiglu(g, u));
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int q = lane; q < kPieces; q += 64) {
          const int r = q / 4, cc = q % 4;
          const int m = m0 + (wm * TM + a) * 32 + r;
          const int n = col0 + cc * 8;
          const u32x4 v = *reinterpret_cast<const u32x4*>(&slab[r * kSlabRow + cc * 8]);
          if (m < M && n < n_hi) *reinterpret_cast<u32x4*>(out + static_cast<int64_t>(m) * ld_out + n) = v;
        }
      }
      __syncthreads();  // the handed-over sums have been read
    }
    return;
  }
#pragma unroll
  for (int a = 0; a < TM; ++a) {
    if (SWI) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float g = tot[a][0][r] * sc[0] + bv[0], u = tot[a][TN - 1][r] * sc[TN - 1] + bv[TN - 1];
        if (SWI == 2) {  // as if fc1 had been written out in T and read back
          g = to_f32<DT>(cast_out<DT>(g));
          u = to_f32<DT>(cast_out<DT>(u));
        }
        slab[(8 * (r / 4) + 4 * b + r % 4) * kSlabRow + r32] = cast_out<DT>(act_swiglu(g, u));
      }
    } else {
#pragma unroll
      for (int c = 0; c < TN; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          slab[(8 * (r / 4) + 4 * b + r % 4) * kSlabRow + c * 32 + r32] =
              cast_out<DT>(act_apply(tot[a][c][r] * sc[c] + bv[c], p.act));
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = lane; q < kPieces; q += 64) {
      const int r = q / (kOutBlocks * 4), cc = q % (kOutBlocks * 4);
      const int m = m0 + (wm * TM + a) * 32 + r;
      const int n = col0 + cc * 8;
      const u32x4 v = *reinterpret_cast<const u32x4*>(&slab[r * kSlabRow + cc * 8]);
      if (m < M && n < n_hi) *reinterpret_cast<u32x4*>(out + static_cast<int64_t>(m) * ld_out + n) = v;
    }
    __builtin_amdgcn_wave_barrier();
  }
  leave_stamps();
#endif
}

// out[m, col0 + c] = T( sum over the runs of part[run][m][c] + bias[col0 + c] ) for the ncols
// columns from col0 on; four columns per thread; total = M * ncols.  valid_rows (may be null):
// rows from *valid_rows on were never computed and are left alone.
template <int DT>
__global__ __launch_bounds__(256) void reduce_partials_kernel(
    const float* __restrict__ part, int nsplit, const uint16_t* __restrict__ bias,
    void* __restrict__ out, int out_f32, int64_t total, int N, int col0, int ncols, int act,
    const int64_t* __restrict__ valid_rows = nullptr) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  if (valid_rows != nullptr && i / ncols >= *valid_rows) return;
  const int64_t o = i / ncols * N + col0 + i % ncols;  // position in out
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  // W loads in flight at a time (past the last run: the last run again, not
  // added), added in run order: one trip to memory for up to W runs
  auto add_runs = [&](auto width) {
    constexpr int W = decltype(width)::value;
    for (int r0 = 0; r0 < nsplit; r0 += W) {
      f32x4 v[W];
#pragma unroll
      for (int u = 0; u < W; ++u) {
        const int r = r0 + u < nsplit ? r0 + u : nsplit - 1;
        v[u] = *reinterpret_cast<const f32x4*>(part + r * total + i);
      }
#pragma unroll
      for (int u = 0; u < W; ++u)
        if (r0 + u < nsplit) {
#pragma unroll
          for (int e = 0; e < 4; ++e) s[e] += v[u][e];
        }
    }
  };
  if (nsplit <= 4) add_runs(std::integral_constant<int, 4>());
  else add_runs(std::integral_constant<int, 8>());
  if (bias != nullptr) {
    const int n = col0 + static_cast<int>(i % ncols);
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] += to_f32<DT>(bias[n + e]);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) s[e] = act_apply(s[e], act);
  if (out_f32) {
    *reinterpret_cast<f32x4*>(static_cast<float*>(out) + o) = s;
  } else {
    u32x2 v;
    v.x = cast_out<DT>(s[0]) | (static_cast<uint32_t>(cast_out<DT>(s[1])) << 16);
    v.y = cast_out<DT>(s[2]) | (static_cast<uint32_t>(cast_out<DT>(s[3])) << 16);
    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + o) = v;
  }
}

// The same for a gate|up projection: out[m, c] = T(silu(g) * u) with g and u the sums (plus bias)
// of columns c and N/2 + c; out is [M, N/2], four columns per thread, total = M * N / 2,
// N % 8 == 0.  The runs are [run][M][N].
template <int DT>
__global__ __launch_bounds__(256) void reduce_partials_swiglu_kernel(
    const float* __restrict__ part, int nsplit, const uint16_t* __restrict__ bias,
    void* __restrict__ out, int out_f32, int64_t total, int N) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  const int half = N / 2;
  const int64_t m = i / half;
  const int c = static_cast<int>(i % half);
  const int64_t run = total * 2;
  f32x4 s[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int r0 = 0; r0 < nsplit; r0 += 4) {
    f32x4 v[4][2];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int r = r0 + u < nsplit ? r0 + u : nsplit - 1;
#pragma unroll
      for (int h = 0; h < 2; ++h) v[u][h] = *reinterpret_cast<const f32x4*>(part + r * run + m * N + h * half + c);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (r0 + u < nsplit) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int e = 0; e < 4; ++e) s[h][e] += v[u][h][e];
      }
  }
  if (bias != nullptr) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 4; ++e) s[h][e] += to_f32<DT>(bias[h * half + c + e]);
  }
  f32x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = act_swiglu(s[0][e], s[1][e]);
  if (out_f32) {
    *reinterpret_cast<f32x4*>(static_cast<float*>(out) + i) = o;
  } else {
    u32x2 v;
    v.x = cast_out<DT>(o[0]) | (static_cast<uint32_t>(cast_out<DT>(o[1])) << 16);
    v.y = cast_out<DT>(o[2]) | (static_cast<uint32_t>(cast_out<DT>(o[3])) << 16);
    *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + i) = v;
  }
}

struct Args {
  const void* x; const void* codes; const void* bias; const void* scale; void* out;
  int M, K, N, gshift, out_f32;
  void* ws; size_t ws_bytes;  // scratch for split-K partial sums, may be null
  hipStream_t stream;
  int act;
};

// Raises a kernel's dynamic LDS limit once per device (the attribute belongs to
// the device's copy of the function); safe to call from several threads.
inline void allow_lds(const void* kern, size_t lds, std::atomic<uint32_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const uint32_t bit = 1u << (dev & 31);
  if (done.load(std::memory_order_acquire) & bit) return;
  (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  done.fetch_or(bit, std::memory_order_release);
}

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

template <int DT, int BITS, bool GROUPED, int WM, int WN, int TM, int TN>
void launch_one(const Args& a) {
  constexpr int BM = WM * TM * 16, BN = WN * TN * 16, TK = BITS == 8 ? 64 : 128;
  const int nbx = (a.N + BN - 1) / BN, nby = (a.M + BM - 1) / BM;
  const size_t lds = 2 * static_cast<size_t>(BM) * (TK + 8) * sizeof(uint16_t);
  auto kern = gemm_kernel<DT, BITS, GROUPED, WM, WN, TM, TN>;
  static std::atomic<uint32_t> configured{0};  // per instantiation
  allow_lds(reinterpret_cast<const void*>(kern), lds, configured);
  kern<<<dim3(static_cast<unsigned>(nbx * nby)), dim3(64 * WM * WN), lds, a.stream>>>(
      static_cast<const uint16_t*>(a.x), static_cast<const uint8_t*>(a.codes),
      static_cast<const uint16_t*>(a.bias), static_cast<const uint16_t*>(a.scale), a.out, a.M, a.K,
      a.N, a.gshift, a.out_f32, nbx, nby, a.act);
}

// Row groups rg of the XCD grid for tile_of_block_2d: among the divisors of 8
// that split both tile counts evenly, the one with the least bytes per XCD and
// k step, rows * a_bytes + columns * b_bytes (bytes of one row block / column
// block per k).  0 when the tiles do not divide over the XCDs.
inline int plan_xcd_rows(int nbx, int nby, int a_bytes, int b_bytes) {
  int best = 0;
  int64_t best_cost = INT64_MAX;
  for (int rg = 1; rg <= 8; rg *= 2) {
    const int cg = 8 / rg;
    if (nby % rg != 0 || nbx % cg != 0) continue;
    const int64_t cost = static_cast<int64_t>(nby / rg) * a_bytes + static_cast<int64_t>(nbx / cg) * b_bytes;
    if (cost < best_cost) { best_cost = cost; best = rg; }
  }
  return best;
}

template <int BITS, int G, int WM, int WN, int TM, int TN, int STAGES = 3>
constexpr size_t dma_lds_bytes() {
  return STAGES * (static_cast<size_t>(WM * TM * 32) * (BITS == 8 ? 64 : 128) * 2 +
              (WN * TN * 32 / 16) * 1024 + (G == 0 ? 0 : WM * WN * 256));
}

// Launches the fast kernel on the columns of strips [strip_lo, strip_hi), K
// cut into nsplit runs (nsplit > 1 needs a.ws: nsplit x M x columns floats).
// SWI != 0 (swiglu epilogue): the strips are those of the gate half, [0, N / 32), a.out is [M, N / 2].
template <int DT, int BITS, int G, int OFFS, int WM, int WN, int TM, int TN, int STAGES = 3, int SWI = 0, bool RESC = false>
void launch_dma(const Args& a, int strip_lo, int strip_hi, int nsplit) {
  constexpr int BM = WM * TM * 32, BN = (SWI ? TN * WN * 16 : TN * WN * 32), TK = BITS == 8 ? 64 : 128;  // BN: output columns
  if (strip_hi <= strip_lo) return;
  if (SWI) nsplit = 1;
  constexpr size_t lds = dma_lds_bytes<BITS, G, WM, WN, TM, TN, STAGES>();
  auto kern = gemm_dma_kernel<DT, BITS, G, OFFS, WM, WN, TM, TN, STAGES, SWI, RESC>;
  static std::atomic<uint32_t> configured{0};  // per instantiation
  allow_lds(reinterpret_cast<const void*>(kern), lds, configured);
  const int ncols = (strip_hi - strip_lo) * kStripCols;
  if (nsplit > 1 && (a.ws == nullptr ||
                     a.ws_bytes < static_cast<size_t>(nsplit) * a.M * ncols * sizeof(float)))
    nsplit = 1;  // never write past the scratch buffer
  DmaParams p;
  p.x = static_cast<const uint16_t*>(a.x);
  p.codes = static_cast<const uint8_t*>(a.codes);
  p.bias = static_cast<const uint16_t*>(a.bias);
  p.scale = static_cast<const uint16_t*>(a.scale);
  p.out = nsplit > 1 ? a.ws : a.out;
  p.M = a.M; p.K = a.K; p.N = a.N;
  p.out_f32 = a.out_f32;
  p.strip_lo = strip_lo; p.strip_hi = strip_hi;
  p.nbx = ((strip_hi - strip_lo) * kStripCols + BN - 1) / BN;
  p.nby = (a.M + BM - 1) / BM;
  const int tiles = a.K / TK;
  p.tiles_per_split = (tiles + nsplit - 1) / nsplit;
  if (RESC && G > TK) p.tiles_per_split = (p.tiles_per_split + 1) & ~1;  // every run starts on a group of two tiles
  p.nsplit = (tiles + p.tiles_per_split - 1) / p.tiles_per_split;
  p.xcd_rows = plan_xcd_rows(p.nbx, p.nby, BM * 2, WN * TN * 32 * BITS / 8);
  p.act = a.act;
  p.moe_table = nullptr;
  p.moe_codes_stride = 0;
  p.moe_rows = 0;
  p.stamps = nullptr;
  kern<<<dim3(static_cast<unsigned>(p.nbx * p.nby * p.nsplit)), dim3(64 * WM * WN), lds, a.stream>>>(p);
  if (nsplit > 1) {
    const int64_t total = static_cast<int64_t>(a.M) * ncols;
    if (!SWI && a.act == WOL_ACT_SWIGLU) {
      // a gate|up projection whose runs cover all of N (the small-M configurations): the kernel
      // that adds the runs forms silu(gate) * up, out is [M, N / 2]
      reduce_partials_swiglu_kernel<DT><<<dim3(static_cast<unsigned>((total / 8 + 255) / 256)), dim3(256), 0, a.stream>>>(
          static_cast<const float*>(a.ws), p.nsplit, p.bias, a.out, a.out_f32, total / 2, a.N);
      return;
    }
    reduce_partials_kernel<DT><<<dim3(static_cast<unsigned>((total / 4 + 255) / 256)), dim3(256), 0, a.stream>>>(
        static_cast<const float*>(a.ws), p.nsplit, p.bias, a.out, a.out_f32, total, a.N,
        strip_lo * kStripCols, ncols, a.act);
  }
}

// The half-size tile of the int8 paths: 256 x 128 (four A blocks
// share each dequantised B block: less VALU work per MFMA, 9 % faster than
// 128 x 256 at M = 512) unless its 256-row blocks would pad M much further
// than 128-row blocks do.
inline bool tall_half_tile(int M) {
  const int pad256 = (M + 255) / 256 * 256, pad128 = (M + 127) / 128 * 128;
  return pad256 * 100 <= pad128 * 108;
}

// Number of 256-column tiles given to the 256-row kernel; the remaining
// columns run with 128-row tiles.  Cost model: a workgroup owns its CU, so a
// launch takes ceil(tiles / CUs) tile times; a half-size tile costs kSmall of a
// full one (a little more than half).
inline int plan_big_columns(int M, int N, bool tall_ok = true) {
  const int cus = num_cus();
  constexpr double kSmall = 0.55;
  const int nbx = (N + 255) / 256, nby_big = (M + 255) / 256, nby_small = (M + 127) / 128;
  const bool tall = tall_ok && tall_half_tile(M);  // half tiles of 256 x 128 instead of 128 x 256
  int best = nbx;
  double best_t = 1e30;
  for (int c = nbx; c >= 0; --c) {
    const int small = tall ? 2 * (nbx - c) * nby_big : (nbx - c) * nby_small;
    const double t = static_cast<double>((c * nby_big + cus - 1) / cus) +
                     kSmall * static_cast<double>((small + cus - 1) / cus);
    if (t < best_t - 1e-9) { best_t = t; best = c; }
  }
  return best;
}

// Rows up to which the small-M configurations (one row block of 32 or 64
// rows, K split across workgroups) are used.  They run two stages deep
// instead of three: the smaller LDS footprint lets a third (32 rows, and
// int8) or second (64 rows, int4) workgroup share the CU, which hides more
// latency than the third stage did.
constexpr int kSkinnyMaxM = 64;

// How a small-M problem is cut up.  A workgroup takes 256 columns, or 512
// (two 32-column blocks per wavefront: half the activation bytes out of L2
// and half the A-fragment reads out of LDS per MFMA, for twice the weight
// bytes per k tile), and K is split into runs: at most 16, of at least 4 k
// tiles, and no more than the scratch buffer holds.  Of all such pairs the one
// with the lowest estimated time is taken.  The estimate, in k-tile times of a
// 256-column workgroup:
//   ceil(workgroups / CUs) x (tiles per run + 8) x (1.3 if 512 columns)
//     + runs x M x N / 300000
// The workgroups of a CU share its load path, so what counts is how many
// the fullest CU gets, not how many are resident; the 8 is a workgroup's
// start (the first tile's latency) and end (writing the partial sums); the
// last term is the traffic of the partial sums, which every run writes and
// the reduction reads.  The three constants are fitted to three sweeps, on
// three machines, over every admissible pair on 160 problems (4096 <= K, N <=
// 28672; 17, 32, 48, 64 rows; int4 and int8, with and without groups),
// scoring a pair by the slowest of its three times: launches with more
// workgroups than CUs but fewer than resident slots vary by up to 30 %
// between machines, launches of at most one workgroup per CU by 3 %.  The
// choice is 1.8 % slower than the best pair on average and 14 % at worst; the
// rule it replaces (width by N and K alone, rounds by resident slots, no
// traffic term) was 9.6 % and 29 % off.  int4 with group size 64 and 64-row
// tiles does not fit the registers at 512 columns.
struct SkinnyPlan {
  bool wide;  // 512 columns per workgroup instead of 256
  int ns;     // K runs
};
inline SkinnyPlan plan_skinny(int M, int K, int N, int bits, int group, size_t ws_bytes) {
  const int tk = bits == 8 ? 64 : 128, tiles = K / tk;
  const int cus = num_cus();
  const size_t per_run = static_cast<size_t>(M) * N * sizeof(float);
  const double traffic = static_cast<double>(M) * N / 300000.0;
  SkinnyPlan best{false, 1};
  double best_cost = 1e300;
  for (int wide = 0; wide < 2; ++wide) {
    if (wide && bits == 4 && group == 64 && M > 32) continue;
    const int cols = wide ? 512 : 256;
    const int64_t nbx = (N + cols - 1) / cols;
    for (int ns = 1; ns <= 16; ++ns) {
      const int tps = (tiles + ns - 1) / ns;
      const int eff = (tiles + tps - 1) / tps;
      if (eff != ns || (ns > 1 && tps < 4)) continue;
      if (ns > 1 && per_run * ns > ws_bytes) continue;
      const int64_t rounds = (nbx * ns + cus - 1) / cus;
      const double cost = static_cast<double>(rounds) * (tps + 8) * (wide ? 1.3 : 1.0) +
                          (ns > 1 ? ns * traffic : 0.0) + 1e-6 * ns;  // the last term prefers fewer runs on ties
      if (cost < best_cost) { best_cost = cost; best = SkinnyPlan{wide != 0, ns}; }
    }
  }
  return best;
}

// Tile of the configuration launch_fast gives the columns that do not get
// 256 x 256 tiles (above 64 rows), and the first strip of those columns.
inline void half_tile_config(int M, int N, int bits, int group, int* bm, int* bn, int* strip_lo) {
  *strip_lo = 0;
  // 256 x 256 tiles on whole rounds of the CUs (int4 with group-wise scales has none:
  // two stages of its 128-deep tiles and their scales do not fit the LDS)
  if (group == 0 || bits == 8) {
    const int c = plan_big_columns(M, N, bits == 8) * 16, nstrips = N / kStripCols;
    *strip_lo = c < nstrips ? c : nstrips;
  }
  if (bits == 8 || group != 0) {
    *bm = tall_half_tile(M) ? 256 : 128;
    *bn = tall_half_tile(M) ? 128 : 256;
  } else {
    *bm = 128;
    *bn = 256;
  }
}

// How a half-size configuration (one workgroup per CU) covers ncols columns:
// the column tiles of whole rounds of the CUs run as they are; the tiles of
// the last, partial round leave CUs idle for a whole tile time, so K is cut
// into as many runs as fit the idle CUs (2..4, each at least 8 k tiles long,
// and only if the scratch buffer holds ns x M x columns floats).  The extra
// traffic is worth it below half occupancy.  full_tiles = 0 with ns = 1 means
// one plain launch over everything.
struct TailPlan {
  int full_tiles;  // column tiles launched without a K split
  int ns;          // K runs of the remaining column tiles
};
inline TailPlan plan_tail(int M, int K, int ncols, int bm, int bn, int tk, size_t ws_bytes) {
  const int cus = num_cus(), tiles = K / tk;
  const int nbx = (ncols + bn - 1) / bn, nby = (M + bm - 1) / bm;
  const int blocks = nbx * nby;
  if (blocks == 0) return {0, 1};
  const int full = blocks > cus ? (blocks / cus) * cus / nby : 0;
  const int rest = (nbx - full) * nby;
  if (rest == 0) return {0, 1};
  const size_t rest_cols = static_cast<size_t>(ncols) - static_cast<size_t>(full) * bn;
  int ns = cus / rest;
  ns = ns > 4 ? 4 : ns;
  while (ns > 1 && (tiles / ns < 8 || static_cast<size_t>(ns) * M * rest_cols * sizeof(float) > ws_bytes)) --ns;
  if (ns <= 1) return {0, 1};
  return {full, ns};
}

template <int DT, int BITS, int G>
void launch_fast(const Args& a) {
  const int nstrips = a.N / kStripCols;
  if (a.M <= kSkinnyMaxM) {
    const SkinnyPlan sp = plan_skinny(a.M, a.K, a.N, BITS, G, a.ws != nullptr ? a.ws_bytes : 0);
    const bool wide = sp.wide;
    const int ns = sp.ns;
    if constexpr (BITS == 4) {
      if (a.M <= 32) {
        if (wide) launch_dma<DT, BITS, G, true, 1, 8, 1, 2, 2>(a, 0, nstrips, ns);
        else launch_dma<DT, BITS, G, true, 1, 8, 1, 1, 2>(a, 0, nstrips, ns);
        return;
      }
    }
    if constexpr (!(BITS == 4 && G == 64)) {
      if (wide) { launch_dma<DT, BITS, G, false, 1, 8, 2, 2, 2>(a, 0, nstrips, ns); return; }
    }
    launch_dma<DT, BITS, G, false, 1, 8, 2, 1, 2>(a, 0, nstrips, ns);
    return;
  }
  constexpr int TK = BITS == 8 ? 64 : 128;
  int bm = 0, bn = 0, lo = 0;
  half_tile_config(a.M, a.N, BITS, G, &bm, &bn, &lo);
  const TailPlan t = plan_tail(a.M, a.K, (nstrips - lo) * kStripCols, bm, bn, TK, a.ws != nullptr ? a.ws_bytes : 0);
  const int mid = lo + t.full_tiles * (bn / kStripCols);  // strips [lo, mid) unsplit, [mid, nstrips) in t.ns runs
  // launches a half-size configuration on both parts
#define WOL_HALF(...)                                              \
  do {                                                             \
    launch_dma<DT, BITS, G, __VA_ARGS__>(a, lo, mid, 1);           \
    launch_dma<DT, BITS, G, __VA_ARGS__>(a, mid, nstrips, t.ns);   \
  } while (0)
  if constexpr (BITS == 8 && G == 0) {
    // 256 x 256 x 64 tiles (144 KiB of LDS, one workgroup per CU) for as many
    // column tiles as fill whole rounds of the CUs; the rest, which would
    // leave CUs idle for a whole tile time, goes to half-size tiles.
    launch_dma<DT, BITS, G, false, 2, 4, 4, 2>(a, 0, lo, 1);
    if (bm == 256) WOL_HALF(false, 2, 4, 4, 1);
    else WOL_HALF(false, 2, 4, 2, 2);
  } else if constexpr (BITS == 8) {
    // group-wise scales: the sums are kept in units of the current group's
    // scale (RESC), so one set of accumulators serves and the tiles are those
    // of the per-channel weights
    launch_dma<DT, BITS, G, 0, 2, 4, 4, 2, 3, 0, true>(a, 0, lo, 1);
    if (bm == 256) WOL_HALF(0, 2, 4, 4, 1, 3, 0, true);
    else WOL_HALF(0, 2, 4, 2, 2, 3, 0, true);
  } else if constexpr (G != 0) {
    // int4 with group-wise scales: the same, on 256 x 128 tiles where the rows
    // fill them (four A blocks share every dequantised B block, and the exact
    // int4 dequantiser is the expensive part), 128 x 256 otherwise
    if (bm == 256) WOL_HALF(0, 2, 4, 4, 1, 2, 0, true);
    else WOL_HALF(0, 2, 4, 2, 2, 2, 0, true);
  } else if constexpr (DT == WOL_DTYPE_BF16) {
    // the exact int4 -> bf16 dequantiser costs 32 VALU instructions per 8
    // codes; the offset form is faster: with row sums by dot products on the
    // 256 x 256 tile (two stages of 64 + 16 KiB fill the LDS), with one
    // cancelling MFMA per A block on the 128 x 256 tiles of the remainder
    launch_dma<DT, BITS, G, 2, 2, 4, 4, 2, 2>(a, 0, lo, 1);
    WOL_HALF(true, 2, 4, 2, 2);
  } else {
    launch_dma<DT, BITS, G, 0, 2, 4, 4, 2, 2>(a, 0, lo, 1);
    WOL_HALF(false, 2, 4, 2, 2);
  }
#undef WOL_HALF
}

// Row-tile table of a grouped launch with tiles of `bm` rows.  cum[e] is the
// number of rows of experts 0 .. e (the inclusive running total that the
// reference's moe_dispatch returns as token_nums_per_expert,
// paddle/phi/kernels/fusion/cutlass/moe_dispatch.cu:174-182): expert e owns
// rows cum[e-1] .. cum[e]-1 and ceil(rows / bm) tiles.  One workgroup; the
// table has max_tiles entries, unused ones marked -1.
__global__ __launch_bounds__(256) void moe_plan_kernel(const int64_t* __restrict__ cum, int num_experts, int bm,
                                                       int max_tiles, int64_t rows, MoeTile* __restrict__ table) {
  __shared__ int first_tile[1025];  // exclusive running total of tiles, by expert
  __shared__ int row_end[1025];     // end of expert e's rows is row_end[e + 1]; row_end[0] = 0
  for (int i = threadIdx.x; i < max_tiles; i += 256) table[i] = MoeTile{-1, 0, 0, 0};
  if (threadIdx.x == 0) {
    // The running totals come from the device and are not trusted: each is
    // clamped to [previous total, rows], so an expert's count is never negative
    // and no tile reaches past the last row of the input.
    int acc = 0;
    int64_t prev = 0;
    row_end[0] = 0;
    for (int e = 0; e < num_experts; ++e) {
      first_tile[e] = acc;
      int64_t end = cum[e];
      end = end < prev ? prev : (end > rows ? rows : end);
      acc += static_cast<int>((end - prev + bm - 1) / bm);
      prev = end;
      row_end[e + 1] = static_cast<int>(end);
    }
    first_tile[num_experts] = acc;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < num_experts; e += 256) {
    const int r0 = row_end[e], r1 = row_end[e + 1];
    const int t0 = first_tile[e], nt = first_tile[e + 1] - t0;
    for (int t = 0; t < nt && t0 + t < max_tiles; ++t) {
      const int row = r0 + t * bm;
      const int left = r1 - row;
      table[t0 + t] = MoeTile{e, row, left < bm ? left : bm, 0};
    }
  }
}

// Rows of a grouped launch's tiles, by the average number of rows per expert
// (the host knows the total only; the per-expert counts stay on the device):
// 128 x 256 tiles, or the small-M configurations' 64 x 256 (32 x 256 for int4)
// when the experts have few rows each -- a decode step of a mixture of
// experts -- where the large tile would do up to eight times the MFMA work
// and hold one workgroup per CU where three fit.
// From 512 rows per expert on, the 256 x 256 tile of the ungrouped prefill
// launch (more MFMAs per dequantised fragment; a partial last tile per expert
// then weighs little).
inline int moe_tile_rows(int64_t rows, int num_experts, int bits) {
  const int64_t avg = rows / (num_experts > 0 ? num_experts : 1);
  if (avg <= 32 && bits == 4) return 32;
  if (avg <= 64) return 64;
  if (avg >= 512) return 256;
  return 128;
}

// What a grouped launch needs besides the problem: the row-tile table, and
// for K runs (ns > 1; bias must be null, the runs' sums have no expert) the
// scratch for ns x rows x N floats and the device word that holds the number
// of rows that belong to an expert.
struct MoeLaunch {
  const int* table;
  int max_tiles, bm, ns;
  int64_t rows;
  float* partial;
  const int64_t* valid_rows;
  int tiles_per_expert = 0;  // > 0: row tiles an expert has on average; its tiles then share an XCD (max_tiles a multiple of 8 x this)
};

// One grouped GEMM: every expert's rows against that expert's weights, tiles
// of WM * TM * 32 rows x 256 columns, per-channel scales, out [rows, N] T.
// SWI = 2: the swiglu of the fc1 output is formed in the epilogue and out is
// [rows, N / 2] (the configurations with two blocks per wavefront).
template <int DT, int BITS, int OFFS, int WM, int WN, int TM, int TN, int STAGES, int SWI = 0>
void launch_moe_gemm_cfg(const void* x, const MoeLaunch& ml, const void* codes, const void* bias,
                         const void* scale, int64_t K, int64_t N, void* out, hipStream_t stream) {
  const int* table = ml.table;
  const int max_tiles = ml.max_tiles;
  constexpr int BN = (SWI ? 1 : TN) * WN * 32;  // output columns of a tile
  constexpr size_t lds = dma_lds_bytes<BITS, 0, WM, WN, TM, TN, STAGES>();
  auto kern = gemm_dma_kernel<DT, BITS, 0, OFFS, WM, WN, TM, TN, STAGES, SWI>;
  static std::atomic<uint32_t> configured{0};
  allow_lds(reinterpret_cast<const void*>(kern), lds, configured);
  DmaParams p;
  p.x = static_cast<const uint16_t*>(x);
  p.codes = static_cast<const uint8_t*>(codes);
  p.bias = static_cast<const uint16_t*>(bias);
  p.scale = static_cast<const uint16_t*>(scale);
  const int tiles = static_cast<int>(K / (BITS == 8 ? 64 : 128));
  const int ns = !SWI && bias == nullptr && ml.partial != nullptr ? ml.ns : 1;
  p.M = WM * TM * 32; p.K = static_cast<int>(K); p.N = static_cast<int>(N);
  p.out_f32 = 0;
  const int64_t out_cols = SWI ? N / 2 : N;
  p.strip_lo = 0; p.strip_hi = static_cast<int>(out_cols / kStripCols);
  p.nbx = static_cast<int>((out_cols + BN - 1) / BN);
  p.nby = max_tiles;
  p.xcd_rows = 0;
  if (ml.tiles_per_expert > 0 && max_tiles % (8 * ml.tiles_per_expert) == 0) p.xcd_rows = -ml.tiles_per_expert;
  p.tiles_per_split = (tiles + ns - 1) / ns;
  p.nsplit = (tiles + p.tiles_per_split - 1) / p.tiles_per_split;
  p.out = p.nsplit > 1 ? static_cast<void*>(ml.partial) : out;
  p.act = WOL_ACT_NONE;
  p.moe_table = table;
  p.moe_codes_stride = K * N * BITS / 8;
  p.moe_rows = static_cast<int>(ml.rows);
  p.stamps = nullptr;
  kern<<<dim3(static_cast<unsigned>(p.nbx * p.nby * p.nsplit)), dim3(64 * WM * WN), lds, stream>>>(p);
  if (p.nsplit > 1) {
    const int64_t total = ml.rows * N;
    reduce_partials_kernel<DT><<<dim3(static_cast<unsigned>((total / 4 + 255) / 256)), dim3(256), 0, stream>>>(
        ml.partial, p.nsplit, nullptr, out, 0, total, static_cast<int>(N), 0, static_cast<int>(N), WOL_ACT_NONE,
        ml.valid_rows);
  }
}

// Whether the grouped GEMM with tiles of bm rows forms the swiglu of its output itself.
inline bool moe_fuses_swiglu(int bm) { return bm >= 128; }

// ml.bm: the tile rows the table was built for (moe_tile_rows).  swiglu: out is
// [rows, N / 2], the swiglu of the product (only where moe_fuses_swiglu(ml.bm)).
template <int DT, int BITS>
void launch_moe_gemm(const void* x, const MoeLaunch& ml, const void* codes, const void* bias,
                     const void* scale, int64_t K, int64_t N, void* out, hipStream_t stream, bool swiglu = false) {
  constexpr bool kOffs = BITS == 4 && DT == WOL_DTYPE_BF16;  // as the ungrouped launch chooses
  constexpr int kBigOffs = kOffs ? 2 : 0;           // the 256-row tile: row sums by dot products
  constexpr int kBigStages = BITS == 8 ? 3 : 2;     // 128-deep int4 tiles: two stages fill the LDS
  if (swiglu) {
    if (ml.bm == 256)
      launch_moe_gemm_cfg<DT, BITS, kBigOffs, 2, 4, 4, 2, kBigStages, 2>(x, ml, codes, bias, scale, K, N, out, stream);
    else
      launch_moe_gemm_cfg<DT, BITS, kOffs, 2, 4, 2, 2, 3, 2>(x, ml, codes, bias, scale, K, N, out, stream);
    return;
  }
  if constexpr (BITS == 4) {
    if (ml.bm == 32) {
      launch_moe_gemm_cfg<DT, 4, true, 1, 8, 1, 1, 2>(x, ml, codes, bias, scale, K, N, out, stream);
      return;
    }
  }
  if (ml.bm == 256) {
    launch_moe_gemm_cfg<DT, BITS, kBigOffs, 2, 4, 4, 2, kBigStages>(x, ml, codes, bias, scale, K, N, out, stream);
    return;
  }
  if (ml.bm == 64)
    launch_moe_gemm_cfg<DT, BITS, false, 1, 8, 2, 1, 2>(x, ml, codes, bias, scale, K, N, out, stream);
  else
    launch_moe_gemm_cfg<DT, BITS, kOffs, 2, 4, 2, 2, 3>(x, ml, codes, bias, scale, K, N, out, stream);
}

// K runs of a grouped launch with small tiles: as many as bring the workgroups
// (column tiles x row tiles x runs) to the CU count, at most 4, each of at
// least 8 k tiles.  The large tile is not split.
inline int moe_runs(int64_t K, int64_t N, int bits, int bm, int max_tiles) {
  if (bm >= 128) return 1;
  const int64_t tiles = K / (bits == 8 ? 64 : 128), wgs = (N + 255) / 256 * max_tiles;
  int ns = static_cast<int>((num_cus() + wgs - 1) / wgs);
  ns = ns > 4 ? 4 : ns;
  while (ns > 1 && tiles / ns < 8) --ns;
  return ns < 1 ? 1 : ns;
}
constexpr int kMoeMaxRuns = 4;

template <int DT, int BITS>
void launch_cfg(const Args& a) {
  constexpr int TK = BITS == 8 ? 64 : 128;
  if (a.K % TK == 0 && a.K / TK >= 2) {
    if (a.gshift < 0) launch_fast<DT, BITS, 0>(a);
    else if (a.gshift == 6) launch_fast<DT, BITS, 64>(a);
    else launch_fast<DT, BITS, 128>(a);
    return;
  }
  if (a.gshift >= 0) {
    launch_one<DT, BITS, true, 2, 4, 8, 2>(a);   // 256 x 128, partial accumulators per group
  } else {
    launch_one<DT, BITS, false, 2, 4, 8, 4>(a);  // 256 x 256
  }
}

}  // namespace

int launch_reduce_partials(const float* part, int nsplit, const void* bias, int dtype, void* out,
                           bool out_f32, int64_t M, int64_t N, int act, hipStream_t stream) {
  if (act == WOL_ACT_SWIGLU) {  // out is [M, N/2]
    if (N % 8 != 0) return WOL_ERR_BAD_SHAPE;
    const int64_t total = M * N / 2;
    const dim3 grid(static_cast<unsigned>((total / 4 + 255) / 256)), block(256);
    if (dtype == WOL_DTYPE_BF16)
      reduce_partials_swiglu_kernel<WOL_DTYPE_BF16><<<grid, block, 0, stream>>>(
          part, nsplit, static_cast<const uint16_t*>(bias), out, out_f32 ? 1 : 0, total, static_cast<int>(N));
    else
      reduce_partials_swiglu_kernel<WOL_DTYPE_F16><<<grid, block, 0, stream>>>(
          part, nsplit, static_cast<const uint16_t*>(bias), out, out_f32 ? 1 : 0, total, static_cast<int>(N));
    return check_launch();
  }
  const int64_t total = M * N;
  const dim3 grid(static_cast<unsigned>((total / 4 + 255) / 256)), block(256);
  if (dtype == WOL_DTYPE_BF16)
    reduce_partials_kernel<WOL_DTYPE_BF16><<<grid, block, 0, stream>>>(
        part, nsplit, static_cast<const uint16_t*>(bias), out, out_f32 ? 1 : 0, total, static_cast<int>(N), 0,
        static_cast<int>(N), act);
  else
    reduce_partials_kernel<WOL_DTYPE_F16><<<grid, block, 0, stream>>>(
        part, nsplit, static_cast<const uint16_t*>(bias), out, out_f32 ? 1 : 0, total, static_cast<int>(N), 0,
        static_cast<int>(N), act);
  return check_launch();
}

size_t linear_gemm_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  const int tk = bits == 8 ? 64 : 128;
  if (K % tk != 0 || K / tk < 2) return 0;
  if (M > kSkinnyMaxM) {
    int bm = 0, bn = 0, lo = 0;
    const int g = group_size > 0 ? group_size : 0;
    half_tile_config(static_cast<int>(M), static_cast<int>(N), bits, g, &bm, &bn, &lo);
    const int ncols = static_cast<int>(N) - lo * kStripCols;
    const TailPlan t = plan_tail(static_cast<int>(M), static_cast<int>(K), ncols, bm, bn, tk, SIZE_MAX);
    return t.ns > 1 ? static_cast<size_t>(t.ns) * M * (ncols - t.full_tiles * bn) * sizeof(float) : 0;
  }
  const int ns = plan_skinny(static_cast<int>(M), static_cast<int>(K), static_cast<int>(N), bits,
                             group_size > 0 ? group_size : 0, SIZE_MAX).ns;
  return ns > 1 ? static_cast<size_t>(ns) * M * N * sizeof(float) : 0;
}

void describe_linear_gemm(int64_t M, int64_t K, int64_t N, int bits, int group_size, size_t ws_bytes,
                          char* buf, size_t n) {
  const int tk = bits == 8 ? 64 : 128;
  const int g = group_size > 0 ? group_size : 0;
  if (K % tk != 0 || K / tk < 2) {
    snprintf(buf, n, "wol::gemm_kernel (register-staged v_mfma_f32_16x16x32, 256 x %d tiles)", g ? 128 : 256);
    return;
  }
  if (M <= kSkinnyMaxM) {
    const SkinnyPlan sp = plan_skinny(static_cast<int>(M), static_cast<int>(K), static_cast<int>(N), bits, g, ws_bytes);
    const bool wide = sp.wide;
    const int ns = sp.ns;
    snprintf(buf, n, "wol::gemm_dma_kernel: %d rows x %d columns per workgroup, K in %d run(s)%s",
             bits == 4 && M <= 32 ? 32 : 64, wide ? 512 : 256, ns, ns > 1 ? " + reduce_partials_kernel" : "");
    return;
  }
  int bm = 0, bn = 0, lo = 0;
  half_tile_config(static_cast<int>(M), static_cast<int>(N), bits, g, &bm, &bn, &lo);
  const int nstrips = static_cast<int>(N / kStripCols);
  const TailPlan t = plan_tail(static_cast<int>(M), static_cast<int>(K), (nstrips - lo) * kStripCols, bm, bn, tk, ws_bytes);
  const int mid = lo + t.full_tiles * (bn / kStripCols);
  int len = 0;
  len += snprintf(buf + len, n - len, "wol::gemm_dma_kernel (v_mfma_f32_32x32x16):");
  if (lo > 0 && len < static_cast<int>(n))
    len += snprintf(buf + len, n - len, " 256x256 tiles on columns [0,%d)", lo * kStripCols);
  if (mid > lo && len < static_cast<int>(n))
    len += snprintf(buf + len, n - len, " %dx%d tiles on [%d,%d)", bm, bn, lo * kStripCols, mid * kStripCols);
  if (nstrips > mid && len < static_cast<int>(n))
    len += snprintf(buf + len, n - len, " %dx%d tiles on [%d,%d)%s", bm, bn, mid * kStripCols, nstrips * kStripCols,
                    t.ns > 1 ? " with K in runs + reduce_partials_kernel" : "");
}

// swiglu of a gate | up projection inside the GEMM's epilogue: the tiles with two
// blocks per wavefront, above the small-M configurations.
// Up to 64 rows: where K is cut into runs, in the kernel that adds them.
bool linear_gemm_fuses_swiglu(int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  const int tk = bits == 8 ? 64 : 128;
  if (K % tk != 0 || K / tk < 2 || N % 32 != 0) return false;
  if (M > kSkinnyMaxM) return true;
  return plan_skinny(static_cast<int>(M), static_cast<int>(K), static_cast<int>(N), bits,
                     group_size > 0 ? group_size : 0, SIZE_MAX).ns > 1;
}

namespace {
// out [M, N / 2] = T(swiglu(x . W + bias)) in one launch
template <int DT, int BITS, int G>
void launch_swiglu_gemm(const Args& a) {
  const int gate_strips = a.N / 2 / kStripCols;
  if constexpr (G != 0) {
    // group-wise scales: the tiles with two blocks per wavefront and rescaled sums
    if constexpr (BITS == 8) {
      if (a.M >= 192) launch_dma<DT, 8, G, 0, 2, 4, 4, 2, 3, 1, true>(a, 0, gate_strips, 1);
      else launch_dma<DT, 8, G, 0, 2, 4, 2, 2, 3, 1, true>(a, 0, gate_strips, 1);
    } else {
      // (256 x 128 tiles: gate and up blocks in neighbouring wavefronts)
      if (tall_half_tile(a.M)) launch_dma<DT, 4, G, 0, 2, 4, 4, 1, 2, 1, true>(a, 0, gate_strips, 1);
      else launch_dma<DT, 4, G, 0, 2, 4, 2, 2, 2, 1, true>(a, 0, gate_strips, 1);
    }
  } else if constexpr (BITS == 8) {
    if (a.M >= 192) launch_dma<DT, 8, 0, false, 2, 4, 4, 2, 3, 1>(a, 0, gate_strips, 1);
    else launch_dma<DT, 8, 0, false, 2, 4, 2, 2, 3, 1>(a, 0, gate_strips, 1);
  } else {
    if (a.M >= 192) launch_dma<DT, 4, 0, DT == WOL_DTYPE_BF16 ? 2 : 0, 2, 4, 4, 2, 2, 1>(a, 0, gate_strips, 1);
    else launch_dma<DT, 4, 0, DT == WOL_DTYPE_BF16 ? 1 : 0, 2, 4, 2, 2, 3, 1>(a, 0, gate_strips, 1);
  }
}
template <int DT, int BITS>
void launch_swiglu_gemm_g(const Args& a) {
  if (a.gshift < 0) launch_swiglu_gemm<DT, BITS, 0>(a);
  else if (a.gshift == 6) launch_swiglu_gemm<DT, BITS, 64>(a);
  else launch_swiglu_gemm<DT, BITS, 128>(a);
}
}  // namespace

// f.act == WOL_ACT_SWIGLU (only where linear_gemm_fuses_swiglu): out is [M, N / 2] T.
int launch_linear_gemm(const void* x, const void* codes, const void* bias, const void* scale,
                       int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                       void* out, bool out_f32, void* workspace, size_t workspace_bytes,
                       hipStream_t stream, const Fuse& f) {
  const int gshift = group_size == 64 ? 6 : (group_size == 128 ? 7 : -1);
  const Args a{x, codes, bias, scale, out, static_cast<int>(M), static_cast<int>(K),
               static_cast<int>(N), gshift, out_f32 ? 1 : 0, workspace, workspace_bytes, stream, f.act};
  if (f.act == WOL_ACT_SWIGLU && M <= kSkinnyMaxM) {
    // the runs of K must be the ones the plan was made with: all of the scratch is required
    if (out_f32 || !linear_gemm_fuses_swiglu(M, K, N, bits, group_size)) return WOL_ERR_BAD_SHAPE;
    if (workspace == nullptr || workspace_bytes < linear_gemm_workspace(M, K, N, bits, group_size)) return WOL_ERR_WORKSPACE;
  } else if (f.act == WOL_ACT_SWIGLU) {
    if (out_f32 || !linear_gemm_fuses_swiglu(M, K, N, bits, group_size)) return WOL_ERR_BAD_SHAPE;
    if (dtype == WOL_DTYPE_BF16) {
      if (bits == 8) launch_swiglu_gemm_g<WOL_DTYPE_BF16, 8>(a); else launch_swiglu_gemm_g<WOL_DTYPE_BF16, 4>(a);
    } else {
      if (bits == 8) launch_swiglu_gemm_g<WOL_DTYPE_F16, 8>(a); else launch_swiglu_gemm_g<WOL_DTYPE_F16, 4>(a);
    }
    return check_launch();
  }
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) launch_cfg<WOL_DTYPE_BF16, 8>(a); else launch_cfg<WOL_DTYPE_BF16, 4>(a);
  } else {
    if (bits == 8) launch_cfg<WOL_DTYPE_F16, 8>(a); else launch_cfg<WOL_DTYPE_F16, 4>(a);
  }
  return check_launch();
}

// ---- mixture-of-experts FFN ---------------------------------------------------
static size_t moe_up(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

// Entries of the row-tile table for tiles of bm rows: every expert may end in
// a partial tile.
static int moe_max_tiles(int64_t rows, int num_experts, int bm) {
  return static_cast<int>((rows + bm - 1) / bm) + num_experts;
}

// Scratch: [row-tile table][fc1 output rows x inter T][activation rows x inter/2 T]
// [fp32 sums of the second GEMM's K runs, rows x hidden each, when the tiles are small]
size_t moe_ffn_workspace(int64_t rows, int64_t hidden, int64_t inter, int num_experts) {
  // (the table at its longest: 32-row tiles; the runs' sums whenever either bit width would use small tiles)
  const bool small = moe_tile_rows(rows, num_experts, 4) < 128;
  return moe_up(static_cast<size_t>(moe_max_tiles(rows, num_experts, 32)) * sizeof(MoeTile)) +
         moe_up(static_cast<size_t>(rows) * inter * 2) + moe_up(static_cast<size_t>(rows) * (inter / 2) * 2) +
         (small ? moe_up(static_cast<size_t>(kMoeMaxRuns) * rows * hidden * sizeof(float)) : 0);
}

int launch_moe_ffn(const void* x, const int64_t* rows_before_expert, const void* ffn1_codes,
                   const void* ffn1_bias, const void* ffn1_scale, const void* ffn2_codes,
                   const void* ffn2_scale, int dtype, int64_t rows, int64_t hidden, int64_t inter,
                   int num_experts, int bits, void* out, void* workspace, hipStream_t stream) {
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  const int bm = moe_tile_rows(rows, num_experts, bits);
  int max_tiles = moe_max_tiles(rows, num_experts, bm);
  // large tiles (one workgroup per CU): an expert's row tiles and all their column tiles on one XCD.  The
  // table (sized for 32-row tiles) has room for the padding of its length to a multiple of 8 experts' tiles.
  int tpe = 0;
  if (bm >= 128) {
    tpe = static_cast<int>((rows / (num_experts > 0 ? num_experts : 1) + bm - 1) / bm);
    tpe = tpe < 1 ? 1 : tpe;
    const int padded = (max_tiles + 8 * tpe - 1) / (8 * tpe) * (8 * tpe);
    if (padded <= moe_max_tiles(rows, num_experts, 32)) max_tiles = padded; else tpe = 0;
  }
  MoeTile* table = reinterpret_cast<MoeTile*>(ws);
  unsigned char* fc1 = ws + moe_up(static_cast<size_t>(moe_max_tiles(rows, num_experts, 32)) * sizeof(MoeTile));
  unsigned char* act = fc1 + moe_up(static_cast<size_t>(rows) * inter * 2);
  float* partial = reinterpret_cast<float*>(act + moe_up(static_cast<size_t>(rows) * (inter / 2) * 2));
  // the second GEMM has hidden / 256 column tiles only: K (= inter / 2) in runs when the tiles are small
  const MoeLaunch l1{reinterpret_cast<const int*>(table), max_tiles, bm, 1, rows, nullptr, nullptr, tpe};
  const MoeLaunch l2{reinterpret_cast<const int*>(table), max_tiles, bm, moe_runs(inter / 2, hidden, bits, bm, max_tiles),
                     rows, bm < 128 ? partial : nullptr, rows_before_expert + (num_experts - 1), tpe};
  moe_plan_kernel<<<dim3(1), dim3(256), 0, stream>>>(rows_before_expert, num_experts, bm, max_tiles, rows, table);
#define WOL_MOE(DT, B)                                                                                        \
  do {                                                                                                        \
    if (moe_fuses_swiglu(bm)) {                                                                               \
      launch_moe_gemm<DT, B>(x, l1, ffn1_codes, ffn1_bias, ffn1_scale, hidden, inter, act, stream, true);     \
    } else {                                                                                                  \
      launch_moe_gemm<DT, B>(x, l1, ffn1_codes, ffn1_bias, ffn1_scale, hidden, inter, fc1, stream);           \
      const int rc = launch_swiglu_t(fc1, dtype, rows, inter, act, stream);                                   \
      if (rc != WOL_OK) return rc;                                                                            \
    }                                                                                                         \
    launch_moe_gemm<DT, B>(act, l2, ffn2_codes, nullptr, ffn2_scale, inter / 2, hidden, out, stream); \
  } while (0)
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) WOL_MOE(WOL_DTYPE_BF16, 8); else WOL_MOE(WOL_DTYPE_BF16, 4);
  } else {
    if (bits == 8) WOL_MOE(WOL_DTYPE_F16, 8); else WOL_MOE(WOL_DTYPE_F16, 4);
  }
#undef WOL_MOE
  return check_launch();
}

// ---- the prefill kernel's inner loop, one ingredient at a time (wol_mfma_probe) ----
namespace {

// The register tile and instruction mix of gemm_dma_kernel's 256 x 256
// configuration (4 x 2 blocks of v_mfma_f32_32x32x16 per wavefront, k tiles of
// four slices) with its ingredients switched on one by one, and no global
// memory traffic other than what LOADS adds:
//   DQ     B fragments dequantised per slice (int8 -> bf16, exact) out of raw
//          codes read from LDS once per tile (0 or 2)
//   NA     A fragments read from LDS per slice (0 or 4)
//   BAR    one workgroup barrier per tile
//   LOADS  six direct-to-LDS loads (1 KiB each) per wavefront and tile out of
//          a 25 MB region of `ops`, two stages, waited for before the barrier
//   M16    v_mfma_f32_16x16x32 on 8 x 4 blocks instead (the same flops)
template <bool M16, int DQ, int NA, bool BAR, bool LOADS>
__global__ __launch_bounds__(512) void mfma_probe_kernel(const u32x4* __restrict__ ops, int iters,
                                                         float* __restrict__ out) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 6144; i += 512) reinterpret_cast<u32x4*>(smem)[i] = ops[i & 511];  // 96 KiB of operand pattern
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned char* base = smem + (wave & 3) * 4096 + lane * 16;
  float total = 0.0f;
  if constexpr (!M16) {
    f32x16 acc[4][2];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][c][r] = 0.0f;
    u32x4 af[2][4], bf[2][2], raw[2][2];
#pragma unroll
    for (int a = 0; a < 4; ++a) af[0][a] = af[1][a] = *reinterpret_cast<const u32x4*>(base + a * 1024);
#pragma unroll
    for (int c = 0; c < 2; ++c) bf[0][c] = bf[1][c] = *reinterpret_cast<const u32x4*>(base + 16384 + c * 1024);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int h = 0; h < 2; ++h) raw[c][h] = *reinterpret_cast<const u32x4*>(base + 32768 + (c * 2 + h) * 1024);
    for (int it = 0; it < iters; ++it) {
      const unsigned char* tb = base + ((it & 3) << 14);
      if (DQ > 0) {
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int h = 0; h < 2; ++h) raw[c][h] = *reinterpret_cast<const u32x4*>(tb + (c * 2 + h) * 1024 + 8192);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (NA > 0) {
#pragma unroll
          for (int a = 0; a < NA; ++a)
            af[(q + 1) & 1][a] = *reinterpret_cast<const u32x4*>(tb + ((q * 4 + a) & 7) * 1024);
        }
        if (DQ > 0) {
          const int step = ((q + 1) & 3) / 2, h = (q + 1) % 2;
#pragma unroll
          for (int c = 0; c < DQ; ++c) {
            const uint32_t w4[4] = {raw[c][h].x, raw[c][h].y, raw[c][h].z, raw[c][h].w};
            bf[(q + 1) & 1][c] = DequantExact<WOL_DTYPE_BF16, 8>::run(&w4[step * 2]);
          }
        }
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int c = 0; c < 2; ++c) acc[a][c] = mfma32<WOL_DTYPE_BF16>(af[q & 1][a], bf[q & 1][c], acc[a][c]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (i < NA) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (DQ > 0) __builtin_amdgcn_sched_group_barrier(0x002, (14 * DQ + 7) / 8 + 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (LOADS) {
        wait_vmcnt<6>();
        __builtin_amdgcn_s_barrier();
        unsigned char* stage = smem + 65536 + (it & 1) * 49152;
        const unsigned char* g = reinterpret_cast<const unsigned char*>(ops) +
                                 ((static_cast<int>(blockIdx.x) & 63) * 8 + (it & 7)) * 49152;
#pragma unroll
        for (int c = 0; c < 6; ++c)
          __builtin_amdgcn_global_load_lds(g + (c * 8 + wave) * 1024 + lane * 16,
                                           (lds_ptr_t)(stage + (c * 8 + wave) * 1024), 16, 0, 0);
      } else if (BAR) {
        __builtin_amdgcn_s_barrier();
      }
    }
    if (LOADS) wait_vmcnt<0>();
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[a][c][r];
  } else {
    f32x4 acc[8][4];
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[a][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 af[2][8], bf[2][4], raw[4];
#pragma unroll
    for (int a = 0; a < 8; ++a) af[0][a] = af[1][a] = *reinterpret_cast<const u32x4*>(base + a * 1024);
#pragma unroll
    for (int c = 0; c < 4; ++c) bf[0][c] = bf[1][c] = *reinterpret_cast<const u32x4*>(base + 16384 + c * 1024);
#pragma unroll
    for (int c = 0; c < 4; ++c) raw[c] = *reinterpret_cast<const u32x4*>(base + 32768 + c * 1024);
    for (int it = 0; it < iters; ++it) {
      const unsigned char* tb = base + ((it & 3) << 14);
      if (DQ > 0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) raw[c] = *reinterpret_cast<const u32x4*>(tb + c * 1024 + 8192);
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        if (NA > 0) {
#pragma unroll
          for (int a = 0; a < 2 * NA; ++a)
            af[(st + 1) & 1][a] = *reinterpret_cast<const u32x4*>(tb + ((st * 8 + a) & 7) * 1024);
        }
        if (DQ > 0) {
#pragma unroll
          for (int c = 0; c < 2 * DQ; ++c) {
            const uint32_t w4[4] = {raw[c].x, raw[c].y, raw[c].z, raw[c].w};
            bf[(st + 1) & 1][c] = DequantExact<WOL_DTYPE_BF16, 8>::run(&w4[((st + 1) & 1) * 2]);
          }
        }
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[a][c] = mfma16<WOL_DTYPE_BF16>(af[st & 1][a], bf[st & 1][c], acc[a][c]);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (i < 2 * NA) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (DQ > 0) __builtin_amdgcn_sched_group_barrier(0x002, (14 * 2 * DQ + 31) / 32 + 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (BAR) __builtin_amdgcn_s_barrier();
    }
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) total += acc[a][c][r];
  }
  out[static_cast<int64_t>(blockIdx.x) * 512 + tid] = total;
#endif
}

template <bool M16, int DQ, int NA, bool BAR, bool LOADS>
void launch_probe(const void* ops, int wgs, int iters, float* out, hipStream_t s) {
  auto kern = mfma_probe_kernel<M16, DQ, NA, BAR, LOADS>;
  static std::atomic<uint32_t> configured{0};
  const size_t lds = LOADS ? 160 * 1024 : 96 * 1024;  // one workgroup per CU either way
  allow_lds(reinterpret_cast<const void*>(kern), lds, configured);
  kern<<<dim3(static_cast<unsigned>(wgs)), dim3(512), lds, s>>>(static_cast<const u32x4*>(ops), iters, out);
}

}  // namespace

// The prefill GEMM's 256 x 256 int8 per-channel bf16 launch with cycle stamps
// (M and N multiples of 256, K a multiple of 64 and at least 192): out [M, N]
// bf16, stamps [(M / 256) * (N / 256)][8 wavefronts][8] counts.
int launch_prefill_phases(const void* x, const void* codes, const void* scale, int64_t M, int64_t K, int64_t N,
                          void* out, unsigned long long* stamps, hipStream_t stream) {
  constexpr int WM = 2, WN = 4, TM = 4, TN = 2, STAGES = 3;
  constexpr size_t lds = dma_lds_bytes<8, 0, WM, WN, TM, TN, STAGES>();
  auto kern = gemm_dma_kernel<WOL_DTYPE_BF16, 8, 0, 0, WM, WN, TM, TN, STAGES, 0, false, true>;
  static std::atomic<uint32_t> configured{0};
  allow_lds(reinterpret_cast<const void*>(kern), lds, configured);
  DmaParams p;
  p.x = static_cast<const uint16_t*>(x);
  p.codes = static_cast<const uint8_t*>(codes);
  p.bias = nullptr;
  p.scale = static_cast<const uint16_t*>(scale);
  p.out = out;
  p.M = static_cast<int>(M); p.K = static_cast<int>(K); p.N = static_cast<int>(N);
  p.out_f32 = 0;
  p.strip_lo = 0; p.strip_hi = static_cast<int>(N / kStripCols);
  p.nbx = static_cast<int>(N / 256);
  p.nby = static_cast<int>(M / 256);
  p.tiles_per_split = static_cast<int>(K / 64);
  p.nsplit = 1;
  p.xcd_rows = plan_xcd_rows(p.nbx, p.nby, 256 * 2, 256);
  p.act = WOL_ACT_NONE;
  p.moe_table = nullptr;
  p.moe_codes_stride = 0;
  p.moe_rows = 0;
  p.stamps = stamps;
  kern<<<dim3(static_cast<unsigned>(p.nbx * p.nby)), dim3(64 * WM * WN), lds, stream>>>(p);
  return check_launch();
}

int launch_mfma_probe(int variant, const void* ops, int workgroups, int iters, float* out, hipStream_t stream) {
  switch (variant) {
    case 0: launch_probe<false, 0, 0, false, false>(ops, workgroups, iters, out, stream); break;
    case 1: launch_probe<false, 2, 0, false, false>(ops, workgroups, iters, out, stream); break;
    case 2: launch_probe<false, 0, 4, false, false>(ops, workgroups, iters, out, stream); break;
    case 3: launch_probe<false, 2, 4, false, false>(ops, workgroups, iters, out, stream); break;
    case 4: launch_probe<false, 2, 4, true, false>(ops, workgroups, iters, out, stream); break;
    case 5: launch_probe<false, 2, 4, true, true>(ops, workgroups, iters, out, stream); break;
    case 6: launch_probe<false, 0, 0, true, true>(ops, workgroups, iters, out, stream); break;
    case 7: launch_probe<true, 0, 0, false, false>(ops, workgroups, iters, out, stream); break;
    case 8: launch_probe<true, 2, 4, true, false>(ops, workgroups, iters, out, stream); break;
    default: return WOL_ERR_BAD_SHAPE;
  }
  return check_launch();
}

}  // namespace wol
