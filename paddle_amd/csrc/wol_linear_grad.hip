// x_grad of weight_only_linear straight from the packed codes:
//   x_grad[M, K] = out_grad[M, N] . dequant(W)[K, N]^T
// (what paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu:27-72
// computes by dequantising the whole weight to T and calling a library GEMM).
//
// Arithmetic.  The contraction runs over n on v_mfma_f32_32x32x16_f16 with fp32
// accumulation, for both element types T:
//   c[n]    = the power of two that brings max_g |scale[g, n]| into [2^7, 2^8)
//   s'[g,n] = scale[g, n] * 2^c[n]                 (exact: a T value fits fp16)
//   B[n,k]  = fp16(code[k, n] * s'[g(k), n])       one rounding, 11 bits
//   e[m]    = the power of two that brings max_n |out_grad[m, n]| * 2^-c[n]
//             into [2^14, 2^15)
//   A[m,n]  = fp16(out_grad[m, n] * 2^(e[m] - c[n]))  (exact unless the value
//             lies more than 2^-29 below the row's largest: then it is tiny)
//   x_grad[m,k] = T( 2^-e[m] * sum_n A[m,n] * B[n,k] )
// so code * scale is rounded once, to 11 significant bits, whatever T is; it is
// never rounded to T.  fp16 is used for bfloat16 tensors as well: a bfloat16
// product code * scale would keep 8 bits.
//
// Three launches (two with per-channel scales, where the first rides along
// with the second):
//   grad_scales_kernel   c[n] and s' (fp16 bits) from the scale tensor
//   grad_prepare_kernel  e[m] and A, one workgroup per row of out_grad
//   grad_gemm_kernel     the product
//
// grad_gemm_kernel.  A workgroup of 8 wavefronts (2 along m, 4 along k) owns an
// output tile of 64*TM rows by 128*TB columns and walks N in chunks of 64.
// The packed layout keeps, per lane, eight consecutive k of one column n: the
// transpose of what an MFMA operand wants for a contraction over n (eight
// consecutive n of one k).  The weight therefore takes a detour through LDS:
// a wavefront loads its share of the chunk's codes (a unit: 64 k of one
// 16-column strip, 16 codes per lane), turns them into fp16 pairs (k, k+1),
// trades halves with the neighbouring lane (one DPP move and one byte
// permute) so that a dword holds columns (n, n+1) of one k, and stores dwords
// into a [k][64 n] tile whose 16-byte pieces are XOR-swizzled such that both
// these stores and the 128-bit operand reads are free of bank conflicts.
// out_grad's tile goes global -> LDS with direct-to-LDS loads, as in the
// forward GEMM.  Two stages: while chunk `it` is multiplied, chunk it+1 is
// loaded, converted and stored; one workgroup barrier per chunk.
#include <atomic>

#include "wol_common.h"

namespace wol {
namespace {

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr int kChunk = 64;  // n per step of the contraction

inline int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// ---- preparation ---------------------------------------------------------

// c for a column whose largest scale magnitude is mx.
__device__ inline int column_exponent(float mx) {
  if (!(mx > 0.0f && mx < __builtin_inff())) return 0;
  int e;
  (void)frexpf(mx, &e);  // mx = f * 2^e, f in [0.5, 1)
  const int c = 8 - e;
  return c > 120 ? 120 : (c < -120 ? -120 : c);  // fits a byte; scales below 2^-112 lose their normalisation
}

// One thread per column n: c[n] and s'[g, n] for every group g.
template <int DT>
__global__ __launch_bounds__(256) void grad_scales_kernel(const uint16_t* __restrict__ scale, int groups,
                                                          int N, uint16_t* __restrict__ sp,
                                                          int* __restrict__ cexp) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float mx = 0.0f;
  for (int g = 0; g < groups; ++g) mx = fmaxf(mx, fabsf(to_f32<DT>(scale[static_cast<int64_t>(g) * N + n])));
  const int c = column_exponent(mx);
  cexp[n] = c;
  for (int g = 0; g < groups; ++g) {
    const float s = to_f32<DT>(scale[static_cast<int64_t>(g) * N + n]);
    sp[static_cast<int64_t>(g) * N + n] = f32_to_f16_rne(ldexpf(s, c));
  }
}

// One workgroup per row m of out_grad: e[m], A[m, :] (row length npad, zeros
// behind column N) and rowf[m] = 2^-e[m].  The row stays in registers between
// the two passes when it has at most kKeep * 2048 elements.
// ONE: per-channel scales.  c[n] then follows from scale[n] alone and is
// computed on the spot (no grad_scales_kernel launch, no c array); workgroup 0
// also writes s'.
template <int DT, bool ONE>
__global__ __launch_bounds__(256) void grad_prepare_kernel(const uint16_t* __restrict__ dout,
                                                           const int* __restrict__ cexp,
                                                           const uint16_t* __restrict__ scale,
                                                           uint16_t* __restrict__ sp, int N, int npad,
                                                           uint16_t* __restrict__ a, float* __restrict__ rowf) {
  constexpr int kKeep = 4;
  __shared__ float red[4];
  const int m = blockIdx.x;
  const uint16_t* row = dout + static_cast<int64_t>(m) * N;
  const bool keep = N <= kKeep * 256 * 8;
  // the eight c of columns n0 .. n0+7
  auto load_c = [&](int n0, int (&c)[8]) {
    if (ONE) {
      const u32x4 sv = *reinterpret_cast<const u32x4*>(scale + n0);
      const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
      for (int i = 0; i < 8; ++i)
        c[i] = column_exponent(fabsf(to_f32<DT>(static_cast<uint16_t>(sw[i / 2] >> (16 * (i % 2))))));
      if (m == 0) {
        uint32_t r[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float lo = ldexpf(to_f32<DT>(static_cast<uint16_t>(sw[i] & 0xFFFFu)), c[2 * i]);
          const float hi = ldexpf(to_f32<DT>(static_cast<uint16_t>(sw[i] >> 16)), c[2 * i + 1]);
          r[i] = static_cast<uint32_t>(f32_to_f16_rne(lo)) | (static_cast<uint32_t>(f32_to_f16_rne(hi)) << 16);
        }
        *reinterpret_cast<u32x4*>(sp + n0) = u32x4{r[0], r[1], r[2], r[3]};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) c[i] = cexp[n0 + i];
    }
  };
  u32x4 held[kKeep];
  int8_t heldc[kKeep][8];
  float mx = 0.0f;
  auto scan = [&](int n0, int slot) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(row + n0);
    int c[8];
    load_c(n0, c);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint16_t h = static_cast<uint16_t>(w[i / 2] >> (16 * (i % 2)));
      mx = fmaxf(mx, ldexpf(fabsf(to_f32<DT>(h)), -c[i]));
    }
    if (slot >= 0) {
      held[slot] = v;
#pragma unroll
      for (int i = 0; i < 8; ++i) heldc[slot][i] = static_cast<int8_t>(c[i]);
    }
  };
  if (keep) {
#pragma unroll
    for (int t = 0; t < kKeep; ++t) {
      const int n0 = (t * 256 + static_cast<int>(threadIdx.x)) * 8;
      if (n0 < N) scan(n0, t);
    }
  } else {
    for (int n0 = threadIdx.x * 8; n0 < N; n0 += 256 * 8) scan(n0, -1);  // N is a multiple of 16
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  int em = 0;
  if (mx > 0.0f && mx < __builtin_inff()) {
    int e;
    (void)frexpf(mx, &e);
    em = 15 - e;
    em = em > 100 ? 100 : (em < -100 ? -100 : em);
  }
  if (threadIdx.x == 0) rowf[m] = ldexpf(1.0f, -em);
  uint16_t* arow = a + static_cast<int64_t>(m) * npad;
  auto emit = [&](int n0, const u32x4& v, const int (&c)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = ldexpf(to_f32<DT>(static_cast<uint16_t>(w[i] & 0xFFFFu)), em - c[2 * i]);
      const float hi = ldexpf(to_f32<DT>(static_cast<uint16_t>(w[i] >> 16)), em - c[2 * i + 1]);
      r[i] = static_cast<uint32_t>(f32_to_f16_rne(lo)) | (static_cast<uint32_t>(f32_to_f16_rne(hi)) << 16);
    }
    *reinterpret_cast<u32x4*>(arow + n0) = u32x4{r[0], r[1], r[2], r[3]};
  };
  if (keep) {
#pragma unroll
    for (int t = 0; t < kKeep; ++t) {
      const int n0 = (t * 256 + static_cast<int>(threadIdx.x)) * 8;
      if (n0 < N) {
        int c[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) c[i] = heldc[t][i];
        emit(n0, held[t], c);
      } else if (n0 < npad) {
        *reinterpret_cast<u32x4*>(arow + n0) = u32x4{0u, 0u, 0u, 0u};
      }
    }
    // padding columns beyond what the kept slots cover (npad - N < 64)
    for (int n0 = (kKeep * 256 + static_cast<int>(threadIdx.x)) * 8; n0 < npad; n0 += 256 * 8)
      *reinterpret_cast<u32x4*>(arow + n0) = u32x4{0u, 0u, 0u, 0u};
  } else {
    for (int n0 = threadIdx.x * 8; n0 < npad; n0 += 256 * 8) {
      if (n0 < N) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + n0);
        int c[8];
        load_c(n0, c);
        emit(n0, v, c);
      } else {
        *reinterpret_cast<u32x4*>(arow + n0) = u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
}

// ---- the product ---------------------------------------------------------

struct GradParams {
  const uint16_t* a;     // [M, npad] fp16
  const uint8_t* codes;  // GFX950 layout of the [K, N] weight
  const uint16_t* sp;    // [groups, N] fp16
  const float* rowf;     // [M]
  void* out;             // [M, K] T, or float when out_f32
  int out_f32;
  int M, K, N, npad;
  int gshift;            // log2(group size), -1: one scale row
  int nbm, nbk;          // output tiles along m and k
  int nsplit, chunks_per_split;  // N is cut into nsplit runs of chunks, one workgroup each
  float* partial;        // nsplit > 1: [nsplit][M][K] sums (times 2^-e[m]) of the runs
};

// Every load (direct-to-LDS ones included) and LDS store of the wavefront has
// completed, then the workgroup meets.
__device__ inline void sync_stage() {
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __syncthreads();
}

// XOR applied to the 16-byte piece index of a row of out_grad's tile (rows of
// 128 bytes): a lane group reads the same piece of 16 consecutive rows.
__device__ inline int a_swizzle(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// The same for the weight tile, rows k of 128 bytes: a linear map of the low
// five bits of k to a 3-bit piece XOR, chosen so that no access of the kernel
// has a bank conflict whether the LDS serves 128 or 256 bytes per cycle:
//   * 128-bit operand reads: 8 (16) consecutive rows, the same logical piece ->
//     8 distinct pieces (and 16 distinct piece/row-parity pairs);
//   * the dword stores of one instruction: rows i + 8*kb + (j & 1), pieces
//     2*strip + j/8 -> the 8 combinations of (j & 1, kb & 1, j / 8) (128 bytes
//     per cycle: half a wavefront) and of (kb, j / 8) per row parity (256) all
//     land in different pieces.
__device__ inline int b_swizzle(int k) {
  const int k0 = k & 1, k1 = (k >> 1) & 1, k2 = (k >> 2) & 1, k3 = (k >> 3) & 1, k4 = (k >> 4) & 1;
  return k1 | ((k0 ^ k2 ^ k4) << 1) | ((k2 ^ k3) << 2);
}

// s_waitcnt that only bounds the number of outstanding vector-memory loads.
template <int N_>
__device__ inline void wait_vmcnt() {
  // gfx9 encoding: vmcnt = [15:14][3:0], expcnt = [6:4], lgkmcnt = [11:8]
  __builtin_amdgcn_s_waitcnt((N_ & 0xF) | ((N_ >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// Two LDS stages of each tile.
template <int DT, int BITS, int TM, int TB>
__global__ __launch_bounds__(512) void grad_gemm_kernel(const GradParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NW = 8, WKW = 4;
  constexpr int BMR = 2 * TM * 32;    // rows of the output tile
  constexpr int BKC = WKW * TB * 32;  // columns (k) of the output tile
  constexpr int kABytes = BMR * 128, kBBytes = BKC * 128;
  constexpr int AS = 2;
  constexpr int kBBase = AS * kABytes;  // the weight stages lie behind out_grad's
  constexpr int kLds = AS * kABytes + 2 * kBBytes;
  constexpr int kALoads = BMR / 64;   // 1 KiB direct-to-LDS loads per wavefront
  constexpr int kUnits = TB;          // units (64 k of one strip) per wavefront and chunk
  constexpr int kCLoads = 2 * kUnits; // register loads per chunk: codes and scale of every unit
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WKW, wk = wave % WKW;
  const int j = lane & 15, kb = lane >> 4, b = lane >> 5, r32 = lane & 31;
  const int ntiles = p.nbm * p.nbk;
  const int split = blockIdx.x / ntiles, tile = blockIdx.x - split * ntiles;
  const int bm = tile % p.nbm, bk = tile / p.nbm;
  const int m0 = bm * BMR, k0 = bk * BKC;
  const int M = p.M, K = p.K, N = p.N;
  const int nstrips = N / kStripCols;
  // this workgroup's run of chunks
  const int cbase = split * p.chunks_per_split;
  const int niter = (p.npad / kChunk - cbase) < p.chunks_per_split ? (p.npad / kChunk - cbase) : p.chunks_per_split;

  // ---- out_grad's tile: sources of this lane's direct-to-LDS loads
  const uint16_t* asrc[kALoads];
#pragma unroll
  for (int c = 0; c < kALoads; ++c) {
    const int q = (c * NW + wave) * 64 + lane;
    const int row = q / 8, slot = q % 8;
    int m = m0 + row;
    m = m < M ? m : M - 1;  // rows past M: valid data, never stored
    asrc[c] = p.a + static_cast<int64_t>(m) * p.npad + (slot ^ a_swizzle(row)) * 8;
  }

  // ---- the weight units of this wavefront: unit u = wave * TB + c covers k
  // chunk u / 4 (64 k) of strip u % 4 of the n chunk
  int ustrip[kUnits];
  const uint8_t* ucode[kUnits];   // the lane's codes in strip 0
  const uint16_t* uscale[kUnits]; // the lane's scale in strip 0
  uint32_t ulds[kUnits];          // byte offset of the lane's first store inside a weight tile
#pragma unroll
  for (int c = 0; c < kUnits; ++c) {
    const int u = wave * TB + c;
    ustrip[c] = u % 4;
    const int ukc = u / 4;
    int kc = k0 / 64 + ukc;
    kc = kc < K / 64 ? kc : K / 64 - 1;  // columns past K: valid data, never stored
    int64_t off;
    if (BITS == 8) {
      off = static_cast<int64_t>(kc) * 1024 + lane * 16;
    } else {
      const int full = K / 128;  // a K that is 64 mod 128 ends with a half tile, 8 bytes per lane
      off = kc / 2 < full ? static_cast<int64_t>(kc / 2) * 1024 + lane * 16 + (kc % 2) * 8
                          : static_cast<int64_t>(full) * 1024 + lane * 8;
    }
    ucode[c] = p.codes + off;
    uscale[c] = p.sp + static_cast<int64_t>(p.gshift >= 0 ? (kc * 64) >> p.gshift : 0) * N + j;
    // pair pr of k step `step` goes to row 64*ukc + 32*step + 8*kb + 2*pr + (j & 1),
    // logical piece 2*strip + j / 8, dword (j / 2) % 4 of the piece
    const int row = 64 * ukc + 8 * kb + (j & 1);
    ulds[c] = static_cast<uint32_t>(row * 128 + ((j >> 1) & 3) * 4);
  }
  // the lane's part of the stores' swizzle (k = 8*kb + 2*pr + (j & 1): bits 0, 3
  // and 4 of k are the lane's, bits 1 and 2 the pair's)
  const int wpiece_lane = b_swizzle(8 * kb + (j & 1));
  const uint32_t xsel = (j & 1) ? 0x03020706u : 0x05040100u;  // see the trade below
  const int64_t sbytes = strip_bytes(K, BITS);

  // registers of one chunk's units
  struct Raw {
    uint32_t c[kUnits][BITS == 8 ? 4 : 2];
    uint16_t s[kUnits];
  };
  auto load_units = [&](int it, Raw& r) {
#pragma unroll
    for (int c = 0; c < kUnits; ++c) {
      int st = it * 4 + ustrip[c];
      st = st < nstrips ? st : nstrips - 1;  // past N: finite codes against zeros of out_grad's tile
      const uint8_t* src = ucode[c] + st * sbytes;
      r.s[c] = uscale[c][st * kStripCols];
      if (BITS == 8) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(src);
        r.c[c][0] = v.x; r.c[c][1] = v.y; r.c[c][2] = v.z; r.c[c][3] = v.w;
      } else {
        const u32x2 v = *reinterpret_cast<const u32x2*>(src);
        r.c[c][0] = v.x; r.c[c][1] = v.y;
      }
    }
  };
  // chunk `it` of out_grad's tile into stage it % AS; past the last chunk the
  // last one is fetched again (into a stage nobody reads any more)
  auto issue_a = [&](int it) {
    unsigned char* stage = smem + (it % AS) * kABytes;
    const int src = cbase + (it < niter ? it : niter - 1);
#pragma unroll
    for (int c = 0; c < kALoads; ++c)
      __builtin_amdgcn_global_load_lds(asrc[c] + src * kChunk, (lds_ptr_t)(stage + (c * NW + wave) * 1024), 16, 0, 0);
  };
  // Converts pairs (2*h, 2*h+1) of k step `step` of every unit and stores them
  // into the weight tile `tile`: a quarter of a chunk's conversion work.
  auto store_quarter = [&](unsigned char* tile, const Raw& r, int step, int h) {
#pragma unroll
    for (int c = 0; c < kUnits; ++c) {
      const _Float16 sh = __builtin_bit_cast(_Float16, r.s[c]);
      const f16x2 s2 = {sh, sh};
      const int piece0 = (2 * ustrip[c] + (j >> 3)) ^ wpiece_lane;
#pragma unroll
      for (int pr = 2 * h; pr < 2 * h + 2; ++pr) {
        // fp16 bits of (1024 + stored code) for k = 2*pr and 2*pr + 1 of the step
        uint32_t bits2;
        f16x2 off;
        if (BITS == 8) {
          const uint32_t d = r.c[c][2 * step + pr / 2];
          // bytes (2*(pr%2), 2*(pr%2)+1) into the low bytes of the halves, 0x64 above them
          bits2 = __builtin_amdgcn_perm(0x64646464u, d, (pr % 2) ? 0x04030402u : 0x04010400u);
          off = f16x2{static_cast<_Float16>(-1152.0f), static_cast<_Float16>(-1152.0f)};
        } else {
          bits2 = ((r.c[c][step] >> (4 * pr)) & 0x000F000Fu) | 0x64006400u;
          off = f16x2{static_cast<_Float16>(-1032.0f), static_cast<_Float16>(-1032.0f)};
        }
        // exact code, then one rounding in the product with s'
        const f16x2 w2 = (__builtin_bit_cast(f16x2, bits2) + off) * s2;
        // trade halves with the neighbouring lane (column n ^ 1): even lanes end
        // up with row k (columns n, n+1), odd lanes with row k+1 (columns n-1, n)
        const uint32_t mine = __builtin_bit_cast(uint32_t, w2);
        int fresh;
        asm volatile("" : "=v"(fresh));  // an undefined register for the lanes DPP does not write (none)
        const uint32_t other = static_cast<uint32_t>(
            __builtin_amdgcn_update_dpp(fresh, static_cast<int>(mine), 0xB1, 0xF, 0xF, false));
        const uint32_t d = __builtin_amdgcn_perm(other, mine, xsel);
        // the swizzle is linear: the pair's part is that of k = 2*pr
        const int piece = piece0 ^ b_swizzle(2 * pr);
        *reinterpret_cast<uint32_t*>(tile + ulds[c] + (32 * step + 2 * pr) * 128 + piece * 16) = d;
      }
    }
  };

  f32x16 acc[TM][TB];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int c = 0; c < TB; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][c][r] = 0.0f;

  // operand reads: rows 32*t + r32 of a tile; the swizzles have period 16 (out_grad) and 32 (weight)
  const int a_off = (wm * TM * 32 + r32) * 128;
  const int a_swz = a_swizzle(r32 & 15);
  const int b_off = (wk * TB * 32 + r32) * 128;
  const int b_swz = b_swizzle(r32);
  auto read_frags = [&](const unsigned char* at, const unsigned char* bt, u32x4 (&af)[TM], u32x4 (&bf)[TB], int q) {
#pragma unroll
    for (int a = 0; a < TM; ++a)
      af[a] = *reinterpret_cast<const u32x4*>(at + a_off + a * 32 * 128 + (((2 * q + b) ^ a_swz) * 16));
#pragma unroll
    for (int c = 0; c < TB; ++c)
      bf[c] = *reinterpret_cast<const u32x4*>(bt + b_off + c * 32 * 128 + (((2 * q + b) ^ b_swz) * 16));
  };
  auto chunk_of = [&](int it) { return cbase + (it < niter ? it : niter - 1); };  // past the end: the last chunk again
  auto mfmas = [&](const u32x4 (&af)[TM], const u32x4 (&bf)[TB]) {
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int c = 0; c < TB; ++c)
        acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, af[a]),
                                                           __builtin_bit_cast(f16x8, bf[c]), acc[a][c], 0, 0, 0);
  };

  // Schedule.  A chunk is four slices of 16 n; operand fragments are read two
  // slices ahead of their MFMAs, and the one workgroup barrier of a chunk sits
  // in its middle:
  //   first half of chunk it:   MFMAs of slices 0, 1; fragments of slices 2, 3
  //                             are read; the codes of chunk it+1 (in registers
  //                             since the middle of chunk it-1) are converted
  //                             and stored into the other weight tile
  //   middle:                   wait for out_grad's tile of chunk it+1 and for
  //                             the stores; barrier.  Nobody reads the tiles of
  //                             chunk it any more (their last fragments are in
  //                             registers), so out_grad's tile of chunk it+2
  //                             is requested into the stage of chunk it, and
  //                             the codes of chunk it+3 into the registers
  //                             just converted
  //   second half:              MFMAs of slices 2, 3 while the fragments of
  //                             slices 0, 1 of chunk it+1 are read
  // so neither the barrier nor the LDS latency stands between two MFMAs, and
  // two stages of each tile suffice.  Loads past the last chunk repeat it into
  // places nobody reads any more.
  // (With eight MFMAs per slice one slice of lead covers the LDS latency, and
  // four sets of fragments would not fit the registers: kDeep = false reads
  // one slice ahead and requests slice 3 just before the barrier.)
  constexpr bool kDeep = TM * TB < 8;
  Raw raw[2];
  u32x4 af[kDeep ? 4 : 2][TM], bf[kDeep ? 4 : 2][TB];  // kDeep: the fragments of slice q live in af[q], bf[q]
  issue_a(0);
  load_units(chunk_of(0), raw[0]);
  issue_a(1);
  load_units(chunk_of(1), raw[1]);
#pragma unroll
  for (int q = 0; q < 4; ++q) store_quarter(smem + kBBase, raw[0], q / 2, q % 2);
  load_units(chunk_of(2), raw[0]);
  wait_vmcnt<0>();
  __builtin_amdgcn_s_waitcnt(0x0070 | (0xF << 0) | (3 << 14));  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  read_frags(smem, smem + kBBase, af[0], bf[0], 0);
  if (kDeep) read_frags(smem, smem + kBBase, af[1], bf[1], 1);

  // conv: the codes of chunk it+1; refilled with those of chunk it+3
  auto chunk = [&](int it, Raw& conv) {
    const unsigned char* at = smem + (it & 1) * kABytes;
    const unsigned char* bt = smem + kBBase + (it & 1) * kBBytes;
    const unsigned char* an = smem + ((it + 1) & 1) * kABytes;
    unsigned char* bn = smem + kBBase + ((it + 1) & 1) * kBBytes;
    if (kDeep) {
      read_frags(at, bt, af[2], bf[2], 2);
      mfmas(af[0], bf[0]);
      store_quarter(bn, conv, 0, 0);
      store_quarter(bn, conv, 0, 1);
      read_frags(at, bt, af[3], bf[3], 3);
      mfmas(af[1], bf[1]);
      store_quarter(bn, conv, 1, 0);
      store_quarter(bn, conv, 1, 1);
    } else {
      read_frags(at, bt, af[1], bf[1], 1);
      mfmas(af[0], bf[0]);
      store_quarter(bn, conv, 0, 0);
      store_quarter(bn, conv, 0, 1);
      __builtin_amdgcn_sched_barrier(0);
      read_frags(at, bt, af[0], bf[0], 2);
      mfmas(af[1], bf[1]);
      store_quarter(bn, conv, 1, 0);
      store_quarter(bn, conv, 1, 1);
      __builtin_amdgcn_sched_barrier(0);
      read_frags(at, bt, af[1], bf[1], 3);
    }
    __builtin_amdgcn_sched_barrier(0);
    // out_grad's tile of chunk it+1 has landed (the codes requested with it may
    // still fly), this wavefront's stores and fragment reads are done
    wait_vmcnt<kCLoads>();
    __builtin_amdgcn_s_waitcnt(0x0070 | (0xF << 0) | (3 << 14));  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    issue_a(it + 2);
    load_units(chunk_of(it + 3), conv);
    __builtin_amdgcn_sched_barrier(0);
    if (kDeep) {
      read_frags(an, bn, af[0], bf[0], 0);
      mfmas(af[2], bf[2]);
      read_frags(an, bn, af[1], bf[1], 1);
      mfmas(af[3], bf[3]);
    } else {
      mfmas(af[0], bf[0]);
      __builtin_amdgcn_sched_barrier(0);
      read_frags(an, bn, af[0], bf[0], 0);
      mfmas(af[1], bf[1]);
    }
  };
  for (int it = 0; it < niter; it += 2) {
    chunk(it, raw[1]);
    if (it + 1 < niter) chunk(it + 1, raw[0]);
  }
  wait_vmcnt<0>();
  __builtin_amdgcn_s_waitcnt(0x0070 | (0xF << 0) | (3 << 14));  // the fragments read ahead have arrived
  __builtin_amdgcn_s_barrier();  // the spare loads are done and every wavefront has stopped reading

  // ---- epilogue: 2^-e[m], cast, 32-row slabs leave through LDS as 16-byte stores
  // accumulator element r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its block
  const int col0 = k0 + wk * TB * 32;
  if (p.out_f32 || p.nsplit > 1) {  // fp32 results (verification mode) or the sums of this run: plain stores
    float* outf = p.nsplit > 1 ? p.partial + static_cast<int64_t>(split) * M * K : static_cast<float*>(p.out);
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
      for (int c = 0; c < TB; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + (wm * TM + a) * 32 + 8 * (r / 4) + 4 * b + r % 4;
          const int k = col0 + c * 32 + r32;
          if (m < M && k < K) outf[static_cast<int64_t>(m) * K + k] = acc[a][c][r] * p.rowf[m];
        }
    return;
  }
  uint16_t* out = static_cast<uint16_t*>(p.out);
  constexpr int kSlabRow = TB * 32 + 8;  // padded, in elements
  static_assert(NW * 32 * kSlabRow * 2 <= kLds, "slabs must fit in the stage buffers");
  uint16_t* slab = reinterpret_cast<uint16_t*>(smem) + wave * 32 * kSlabRow;
  constexpr int kPieces = 32 * (TB * 32 / 8);
#pragma unroll
  for (int a = 0; a < TM; ++a) {
    float rf[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      int m = m0 + (wm * TM + a) * 32 + 8 * (r / 4) + 4 * b + r % 4;
      m = m < M ? m : M - 1;
      rf[r] = p.rowf[m];
    }
#pragma unroll
    for (int c = 0; c < TB; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        slab[(8 * (r / 4) + 4 * b + r % 4) * kSlabRow + c * 32 + r32] = cast_out<DT>(acc[a][c][r] * rf[r]);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = lane; q < kPieces; q += 64) {
      const int r = q / (TB * 4), cc = q % (TB * 4);
      const int m = m0 + (wm * TM + a) * 32 + r;
      const int k = col0 + cc * 8;
      const u32x4 v = *reinterpret_cast<const u32x4*>(&slab[r * kSlabRow + cc * 8]);
      if (m < M && k < K) *reinterpret_cast<u32x4*>(out + static_cast<int64_t>(m) * K + k) = v;
    }
    __builtin_amdgcn_wave_barrier();
  }
#endif
}

// out[i] = T(sum over the runs of part[run][i]) (or the fp32 sum), eight elements per thread.
template <int DT>
__global__ __launch_bounds__(256) void reduce_runs_kernel(const float* __restrict__ part, int runs, int64_t total,
                                                          void* __restrict__ out, int out_f32) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 8;  // total is a multiple of 64
  if (i >= total) return;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = 0.0f;
  for (int r = 0; r < runs; ++r) {  // in run order: the result does not depend on timing
    const float* src = part + static_cast<int64_t>(r) * total + i;
    const f32x4v a = *reinterpret_cast<const f32x4v*>(src), b2 = *reinterpret_cast<const f32x4v*>(src + 4);
    v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w;
    v[4] += b2.x; v[5] += b2.y; v[6] += b2.z; v[7] += b2.w;
  }
  if (out_f32) {
    float* o = static_cast<float*>(out) + i;
    *reinterpret_cast<f32x4v*>(o) = f32x4v{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4v*>(o + 4) = f32x4v{v[4], v[5], v[6], v[7]};
  } else {
    uint32_t r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      r[e] = static_cast<uint32_t>(cast_out<DT>(v[2 * e])) | (static_cast<uint32_t>(cast_out<DT>(v[2 * e + 1])) << 16);
    *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(out) + i) = u32x4{r[0], r[1], r[2], r[3]};
  }
}

template <int DT, int BITS, int TM, int TB>
void launch_cfg(const GradParams& p0, hipStream_t stream) {
  GradParams p = p0;
  constexpr int BMR = 2 * TM * 32, BKC = 4 * TB * 32;
  p.nbm = (p.M + BMR - 1) / BMR;
  p.nbk = (p.K + BKC - 1) / BKC;
  const size_t lds = static_cast<size_t>(2 * BMR + 2 * BKC) * 128;
  auto kern = grad_gemm_kernel<DT, BITS, TM, TB>;
  // more than 64 KiB of LDS must be allowed once per device
  static std::atomic<uint32_t> done{0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const uint32_t bit = 1u << (dev & 31);
  if (!(done.load(std::memory_order_acquire) & bit)) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds));
    done.fetch_or(bit, std::memory_order_release);
  }
  // Few tiles: N is cut into runs so that the CUs fill (a chunk costs a workgroup
  // about the same time whatever the tile, so a run of half the chunks takes
  // half as long); the runs' fp32 sums meet in reduce_runs_kernel.
  const int tiles = p.nbm * p.nbk, chunks = p.npad / kChunk;
  int ns = 1;
  if (p.partial != nullptr) {
    while (ns < 4 && tiles * ns * 2 <= 256 && chunks / (ns * 2) >= 8) ns *= 2;
  }
  p.chunks_per_split = (chunks + ns - 1) / ns;
  p.nsplit = (chunks + p.chunks_per_split - 1) / p.chunks_per_split;
  kern<<<dim3(static_cast<unsigned>(tiles * p.nsplit)), dim3(512), lds, stream>>>(p);
  if (p.nsplit > 1) {
    const int64_t total = static_cast<int64_t>(p.M) * p.K;
    reduce_runs_kernel<DT><<<dim3(static_cast<unsigned>((total / 8 + 255) / 256)), dim3(256), 0, stream>>>(
        p.partial, p.nsplit, total, p.out, p.out_f32);
  }
}

// Tile choice.  Every element of the weight is converted once per row tile, so
// tall tiles are preferred; a tile count of at least 7/8 of the CUs (256) keeps
// the device busy.
void pick_tile(int64_t M, int64_t K, int* tm, int* tb) {
  auto count = [&](int t_m, int t_b) {
    return ((M + 64 * t_m - 1) / (64 * t_m)) * ((K + 128 * t_b - 1) / (128 * t_b));
  };
  if (count(4, 2) >= 224) { *tm = 4; *tb = 2; return; }
  if (count(4, 1) >= 224) { *tm = 4; *tb = 1; return; }
  if (count(2, 2) >= 224) { *tm = 2; *tb = 2; return; }
  *tm = 2; *tb = 1;
}

template <int DT, int BITS>
void launch_gemm(const GradParams& p, hipStream_t stream) {
  int tm, tb;
  pick_tile(p.M, p.K, &tm, &tb);
  if (tm == 4 && tb == 2) launch_cfg<DT, BITS, 4, 2>(p, stream);
  else if (tm == 4) launch_cfg<DT, BITS, 4, 1>(p, stream);
  else if (tb == 2) launch_cfg<DT, BITS, 2, 2>(p, stream);
  else launch_cfg<DT, BITS, 2, 1>(p, stream);
}

struct Layout {
  size_t sp, cexp, rowf, a, partial, total;
  int64_t npad, groups;
};

// Runs of N the GEMM may use for a problem (the scratch is sized for it).
int max_runs(int64_t M, int64_t K) {
  int tm, tb;
  pick_tile(M, K, &tm, &tb);
  const int64_t tiles = ((M + 64 * tm - 1) / (64 * tm)) * ((K + 128 * tb - 1) / (128 * tb));
  return tiles * 2 <= 256 ? (tiles * 4 <= 256 ? 4 : 2) : 1;
}

Layout layout_of(int64_t M, int64_t K, int64_t N, int group_size) {
  Layout l;
  l.npad = round_up(N, kChunk);
  l.groups = group_size > 0 ? (K + group_size - 1) / group_size : 1;  // a K of 64 still has one group of 128
  l.sp = 0;
  l.cexp = round_up(static_cast<size_t>(l.groups) * N * 2, 256);
  l.rowf = l.cexp + round_up(static_cast<size_t>(N) * 4, 256);
  l.a = l.rowf + round_up(static_cast<size_t>(M) * 4, 256);
  l.partial = l.a + round_up(static_cast<size_t>(M) * l.npad * 2, 256);
  const int runs = max_runs(M, K);
  l.total = l.partial + (runs > 1 ? round_up(static_cast<size_t>(runs) * M * K * 4, 256) : 0);
  return l;
}

}  // namespace

size_t linear_grad_workspace(int64_t M, int64_t K, int64_t N, int group_size) {
  return layout_of(M, K, N, group_size).total;
}

void describe_linear_grad(int64_t M, int64_t K, int64_t N, char* buf, size_t n) {
  int tm, tb;
  pick_tile(M, K, &tm, &tb);
  const int64_t tiles = ((M + 64 * tm - 1) / (64 * tm)) * ((K + 128 * tb - 1) / (128 * tb));
  const int64_t chunks = round_up(N, kChunk) / kChunk;
  int ns = 1;
  while (ns < 4 && tiles * ns * 2 <= 256 && chunks / (ns * 2) >= 8) ns *= 2;
  snprintf(buf, n, "wol::grad_gemm_kernel: %d rows x %d columns (k) per workgroup, N in chunks of %d%s",
           64 * tm, 128 * tb, kChunk, ns == 1 ? "" : (ns == 2 ? ", in 2 runs + reduce_runs_kernel" : ", in 4 runs + reduce_runs_kernel"));
}

int launch_linear_grad(const void* out_grad, const void* codes, const void* scale, int dtype, int64_t M,
                       int64_t K, int64_t N, int bits, int group_size, void* x_grad, bool out_f32,
                       void* workspace, hipStream_t stream) {
  const Layout l = layout_of(M, K, N, group_size);
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  uint16_t* sp = reinterpret_cast<uint16_t*>(ws + l.sp);
  int* cexp = reinterpret_cast<int*>(ws + l.cexp);
  float* rowf = reinterpret_cast<float*>(ws + l.rowf);
  uint16_t* a = reinterpret_cast<uint16_t*>(ws + l.a);
  const uint16_t* sc = static_cast<const uint16_t*>(scale);
  const uint16_t* dout = static_cast<const uint16_t*>(out_grad);
  const dim3 sgrid(static_cast<unsigned>((N + 255) / 256)), pgrid(static_cast<unsigned>(M));
  const int n32 = static_cast<int>(N), np32 = static_cast<int>(l.npad);
  const bool one = l.groups == 1;  // per-channel: the scale preparation rides along with the rows
  if (dtype == WOL_DTYPE_BF16) {
    if (one) {
      grad_prepare_kernel<WOL_DTYPE_BF16, true><<<pgrid, 256, 0, stream>>>(dout, cexp, sc, sp, n32, np32, a, rowf);
    } else {
      grad_scales_kernel<WOL_DTYPE_BF16><<<sgrid, 256, 0, stream>>>(sc, static_cast<int>(l.groups), n32, sp, cexp);
      grad_prepare_kernel<WOL_DTYPE_BF16, false><<<pgrid, 256, 0, stream>>>(dout, cexp, sc, sp, n32, np32, a, rowf);
    }
  } else {
    if (one) {
      grad_prepare_kernel<WOL_DTYPE_F16, true><<<pgrid, 256, 0, stream>>>(dout, cexp, sc, sp, n32, np32, a, rowf);
    } else {
      grad_scales_kernel<WOL_DTYPE_F16><<<sgrid, 256, 0, stream>>>(sc, static_cast<int>(l.groups), n32, sp, cexp);
      grad_prepare_kernel<WOL_DTYPE_F16, false><<<pgrid, 256, 0, stream>>>(dout, cexp, sc, sp, n32, np32, a, rowf);
    }
  }
  GradParams p;
  p.a = a;
  p.codes = static_cast<const uint8_t*>(codes);
  p.sp = sp;
  p.rowf = rowf;
  p.out = x_grad;
  p.out_f32 = out_f32 ? 1 : 0;
  p.M = static_cast<int>(M);
  p.K = static_cast<int>(K);
  p.N = static_cast<int>(N);
  p.npad = static_cast<int>(l.npad);
  p.gshift = group_size == 64 ? 6 : (group_size == 128 ? 7 : -1);
  p.nbm = p.nbk = 0;
  p.nsplit = 1;
  p.chunks_per_split = 0;
  p.partial = max_runs(M, K) > 1 ? reinterpret_cast<float*>(ws + l.partial) : nullptr;
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) launch_gemm<WOL_DTYPE_BF16, 8>(p, stream); else launch_gemm<WOL_DTYPE_BF16, 4>(p, stream);
  } else {
    if (bits == 8) launch_gemm<WOL_DTYPE_F16, 8>(p, stream); else launch_gemm<WOL_DTYPE_F16, 4>(p, stream);
  }
  return check_launch();
}

}  // namespace wol
