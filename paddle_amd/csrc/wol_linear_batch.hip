// weight_only_linear for a small batch of rows (2 <= M <= 16, up to 32 in the
// K-split form): the decode kernel for batched serving.
//
// What limits the one-row kernel's launch shape (a workgroup per 16-column
// strip) at several rows is the activations: every workgroup needs all of x,
// 16 rows x K, and with one workgroup per strip that is N/16 copies of x out
// of L2 -- four times the weight bytes at 16 rows of int4.  Here the grid is
// at most one workgroup per CU and a workgroup owns a contiguous run of strips
// (N/16 / 256 of them), so x is fetched once per CU.
//
// A workgroup has 16 wavefronts that split K evenly between them (K = 2048,
// 4096 or 8192: every wavefront owns the same whole number of 1 KiB weight
// tiles of each strip), and the A fragments of a wavefront's run of k (16 rows
// x 32 k each, 16 bytes per lane; 32 registers at K = 4096, 64 at 8192) are
// loaded once and stay in registers for every strip of the workgroup -- the
// registers are the staging buffer for x, nothing of it passes through LDS.
// The wavefront's work is a list of items (a strip's tiles of the run, or half
// of them) in strip order.  Weight tiles live in a register ring of D items:
// the ring is filled before the first use, and a slot is refilled with the
// item D places further on as soon as it has been consumed.  All loads are
// unconditional instructions (past the last item they are buffer loads beyond
// the end of their descriptor, which fetch nothing), which is what lets the
// compiler wait for exactly the tile it needs while the younger loads stay in
// flight.
//
// Arithmetic: as in the one-row kernel the codes become T bit patterns
// (code + offset, exact) and v_mfma_f32_16x16x32 does the multiply and the
// reduction over k.  The MFMAs of one chain (a tile, or a scale group inside
// it: at most 128 k) accumulate in place, starting from the chain's cancelling
// term mfma(A, constant B); those terms depend on the wavefront's A fragments
// only and, where 16 registers hold them, are computed once for all strips.  Only a
// chain's result is added to the running fp32 sums (times the group scale
// when scales are group-wise).  Nothing is rounded to T before the final cast.
//
// The wavefronts never wait for each other while they stream: every
// wavefront leaves its partial sums of every strip in LDS (16 KiB per strip),
// and one barrier at the end of a run of up to seven strips precedes the
// reduction (in wavefront order: deterministic), scale, bias, cast and store.
// The per-channel scales and the bias of a run are parked in LDS at its start;
// group-wise scales travel with their weight tiles, one 2-byte load per lane
// and group.
//
// A second form of the kernel (SPLIT) cuts K into runs across workgroups as
// well: workgroup b works on run b % runs of strip set b / runs, a run being
// 16 wavefronts x 128 or 256 k, and the runs' fp32 sums meet in a scratch
// buffer that reduce_partials_kernel (wol_linear_gemm.hip) adds up.  That
// serves any K of whole weight tiles, keeps the activations a workgroup fetches
// down to K / runs when the strips are few, and -- with two 16-row operands
// per wavefront (MT = 2) -- takes up to 32 rows.
#include <atomic>

#include "wol_common.h"
#include "wol_dequant.h"

namespace wol {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  if (DT == WOL_DTYPE_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

constexpr int kBatchWaves = 16;
constexpr int kBatchRun = 7;  // strips whose partial sums (16 KiB each per 16 rows) share the LDS

struct BatchParams {
  const uint16_t* x;
  const uint8_t* codes;
  const uint16_t* bias;
  const uint16_t* scale;
  void* out;
  int M, K, N;
  int gshift;   // log2(group size), -1 per-channel
  int out_f32;
  int strips_q, strips_r;  // strips (SWI: pairs of strips) per workgroup: N / 16 = grid * strips_q + strips_r
  const uint16_t* pre;     // [K] per-channel scales of the activations, or null
  int act;                 // WOL_ACT_NONE or WOL_ACT_GELU
  // K cut into runs across workgroups (SPLIT): workgroup b takes run b % nseg
  // of strip set b / nseg and leaves its scaled fp32 sums in ws[run][M][N]
  int nseg;
  int ntiles;              // K / tile depth
  float* ws;
};

// G: 0 per-channel, else the group size.  TPW: weight tiles (1 KiB, 64 or 128
// k) of a strip that belong to one wavefront: K = 16 * TPW * tile depth
// exactly, so that every wavefront runs the same instruction stream and every
// load below is unconditional -- the compiler then knows at each use how many
// younger loads may still be in flight (s_waitcnt vmcnt(n) with n > 0); a load
// under a condition would make every later wait a wait for all loads.
// IT: tiles per item, D: items in the ring (a multiple of TPW / IT).
// PRE: the activations are multiplied by p.pre (each product rounded to T as
// apply_per_channel_scale rounds it) once, in the registers they stay in.
// MT: 16-row operands (M <= 16 * MT); every dequantised B fragment feeds MT
// MFMAs.
// SPLIT: K is cut into p.nseg runs of 16 * TPW tiles across workgroups, the
// last of which may reach past K: a wavefront's tiles past the end have zero
// activations and fetch nothing.  The sums of a run go to p.ws and a second
// kernel adds the runs (bias and activation function there).  This is what
// serves any K made of whole tiles, and what keeps x down to K / nseg per CU
// when the strips are few.
// SWI: the weight is a gate|up projection and the kernel writes
// silu(gate) * up, [M, N/2].  The unit of work is then a pair of strips, gate
// strip u and up strip u + N/32: a workgroup owns a contiguous range of pairs,
// a run holds up to three of them with the strips in the order gate, up, gate,
// up ..., and the end of a run combines the two sums of every output element.
template <int DT, int BITS, int G, int TPW, int IT, int D, bool PRE, int MT, bool SPLIT, bool SWI>
__global__ __launch_bounds__(kBatchWaves * 64) void batch_kernel(const BatchParams p) {
  constexpr int WK = kBatchWaves;
  constexpr int TK = BITS == 8 ? 64 : 128;   // k per 1 KiB weight tile
  constexpr int SPT = TK / 32;               // k steps per tile
  constexpr int kDw = BITS == 8 ? 2 : 1;     // dwords per k step and lane
  constexpr int P = TPW / IT;                // items per strip
  static_assert(TPW % IT == 0 && D % P == 0, "ring slot d always holds part d % P of a strip");
  constexpr int CK = G == 0 ? TK : (G < TK ? G : TK);  // k per chain
  constexpr int CPT = TK / CK;               // chains per tile
  constexpr int SPC = SPT / CPT;             // k steps per chain
  constexpr int NS = G == 0 ? 1 : IT * CPT;  // group scales per item and lane
  constexpr bool kKeepCancel = MT * TPW * SPT <= 8 && MT * TPW * CPT <= 4;  // cancelling terms computed once and kept
                                                                         // where 32 registers of A leave 16 for them
  static_assert(!(PRE && (SPLIT || MT > 1)), "the fused activation scales exist for the one-run, 16-row form");
  static_assert(!(SWI && (SPLIT || MT > 1 || PRE)), "the gate|up form exists for the one-run, 16-row form without activation scales");
  constexpr int SPU = SWI ? 2 : 1;  // strips per unit of the workgroup's range
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, kb = lane >> 4;
  const int K = p.K, N = p.N, M = p.M;
  // this workgroup's strips; this wavefront's tiles are t0 .. t0 + TPW - 1 of each
  const int seg = SPLIT ? static_cast<int>(blockIdx.x) % p.nseg : 0;
  const int bid = SPLIT ? static_cast<int>(blockIdx.x) / p.nseg : static_cast<int>(blockIdx.x);
  const int s0 = bid * p.strips_q + (bid < p.strips_r ? bid : p.strips_r);
  const int s1 = s0 + p.strips_q + (bid < p.strips_r ? 1 : 0);
  const int t0 = (seg * WK + wave) * TPW;
  const int ntiles = p.ntiles;
  const int64_t sbytes = strip_bytes(K, BITS);

  uint32_t magic = Dequant<DT, BITS>::kMagic;
  asm volatile("" : "+v"(magic));  // keep the constant in a VGPR
  const u32x4 cancel = {Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel,
                        Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel};

  // A fragment of k step `step`: lane (kb, j) holds row j, k = 32 * step + 8 * kb .. + 7.
  // Only the lanes of rows that exist load anything (the texture unit spends
  // its cycles per active lane: at 4 rows the fragments cost a quarter of what
  // 16 rows cost); the other rows hold whatever the registers held (rows of an MFMA result do
  // not mix) and are never stored.
  u32x4 A[MT][TPW * SPT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = mt * 16 + j;
    const uint16_t* xrow = p.x + static_cast<int64_t>(row < M ? row : 0) * K + t0 * TK + 8 * kb;
#pragma unroll
    for (int s = 0; s < TPW * SPT; ++s) asm volatile("" : "=v"(A[mt][s]));  // any value will do in the rows past M
    if (SPLIT) {
      // tiles past the end of K: zero activations in every lane, so that what
      // the weight registers of such a tile hold (zeros) never counts
#pragma unroll
      for (int s = 0; s < TPW * SPT; ++s)
        if (t0 + s / SPT >= ntiles) A[mt][s] = u32x4{0u, 0u, 0u, 0u};
    }
    if (row < M) {
#pragma unroll
      for (int s = 0; s < TPW * SPT; ++s)
        if (!SPLIT || t0 + s / SPT < ntiles) A[mt][s] = *reinterpret_cast<const u32x4*>(xrow + s * 32);
    }
  }
  // The activation scales of the wavefront's k (the same for every row): lane
  // 4 * s + kb holds the eight scales that go with A[s] in lane group kb, one
  // 16-byte load for the whole run; they are handed out by lane permutes later.
  u32x4 PS = {0u, 0u, 0u, 0u};
  if (PRE) PS = *reinterpret_cast<const u32x4*>(p.pre + t0 * TK + (lane % (TPW * SPT * 4)) * 8);

  u32x4 W[D][IT];
  uint16_t S[D][NS];
  // part `part` (IT tiles) of this wavefront's share of strip `strip`.  The
  // tiles come through a buffer descriptor that spans the strips of the run
  // (at most 7 x 128 KiB): with real == false the offset lies past its end,
  // and such a load returns zeros without touching memory -- the instruction
  // stays unconditional, the traffic does not.
  const int lane_off = t0 * 1024 + lane * 16;
  auto load_item = [&](__amdgpu_buffer_rsrc_t rsrc, int strip, int strip_of_run, int part, bool real,
                       u32x4 (&w)[IT], uint16_t (&sc)[NS]) {
    if (G != 0) {  // the item's group scales travel with it (past the last item: the last strip's again)
#pragma unroll
      for (int q = 0; q < NS; ++q) {
        int k0 = (t0 + part * IT) * TK + q * CK;
        if (SPLIT) k0 = k0 < K ? k0 : K - CK;  // a tile past K: any scale that exists (it meets zeros)
        sc[q] = p.scale[static_cast<int64_t>(k0 >> p.gshift) * N + strip * kStripCols + j];
      }
    }
    const int soff = real ? strip_of_run * static_cast<int>(sbytes) + part * IT * 1024 : 0x7FFF0000;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      const int off = !SPLIT || t0 + part * IT + i < ntiles ? soff : 0x7FFF0000;
      // non-temporal: the weights pass through once and must not push the scales and the other workgroups'
      // activations out of the caches (3 to 10 % of the kernel's time at 8 and 16 rows)
      w[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off + off + i * 1024, 0, 2));
    }
  };

  f32x4 ccs[MT][kKeepCancel ? TPW * CPT : 1];  // the cancelling term of every chain of the wavefront's run
  bool have_cc = false;
  // the per-channel scales (first row of the scale tensor) and the bias behind
  // bounded descriptors, for the staging loads
  const __amdgpu_buffer_rsrc_t scale_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.scale), 0, N * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t bias_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.bias != nullptr ? p.bias : p.scale), 0, N * 2, 0x00020000);

  constexpr int kRun = kBatchRun / MT / SPU;  // units (strips, or pairs of them) whose partial sums share the LDS
  const int up0 = N / kStripCols / 2;         // SWI: the first up strip
  for (int sr = s0; sr < s1; sr += kRun) {
    const int cnt = s1 - sr < kRun ? s1 - sr : kRun;  // units of this run
    const int nstr = cnt * SPU;                       // strips of this run
    const int nitems = nstr * P;  // item it: strip it / P of the run, part it % P

    const int ncols = nstr * kStripCols;
    float* red = reinterpret_cast<float*>(smem);                                // [nstr][WK][MT * 4][64]
    uint16_t* lsc = reinterpret_cast<uint16_t*>(smem + nstr * WK * MT * 1024);  // [ncols] per-channel scales
    uint16_t* lbi = lsc + ncols;                                          // [ncols] bias
    // strip sl of the run is strip run_strip(sl) of the weight
    auto run_strip = [&](int sl) { return SWI ? sr + (sl >> 1) + (sl & 1) * up0 : sr + sl; };

    // What the end of the run needs -- per-channel scales and bias of its
    // columns -- is requested first (one load each by the first threads; the
    // others read past the end of the descriptor: nothing) and parked in LDS
    // once the weight ring has been requested as well.
    int boff = static_cast<int>(threadIdx.x) < ncols ? (sr * kStripCols + static_cast<int>(threadIdx.x)) * 2 : 0x7FFFFFF0;
    if constexpr (SWI) {
      if (static_cast<int>(threadIdx.x) < ncols)
        boff = (run_strip(static_cast<int>(threadIdx.x) / kStripCols) * kStripCols +
                static_cast<int>(threadIdx.x) % kStripCols) * 2;
    }
    const uint16_t sstage = __builtin_amdgcn_raw_buffer_load_b16(scale_rsrc, boff, 0, 0);
    const uint16_t bstage = __builtin_amdgcn_raw_buffer_load_b16(bias_rsrc, boff, 0, 0);

    // fill the ring; slots past the last item load nothing
    // (SWI: from the run's first gate strip to its last up strip, half the
    // weight further on: the host keeps that below 2 GiB)
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.codes + sr * sbytes), 0, ((SWI ? up0 : 0) + cnt) * static_cast<int>(sbytes), 0x00020000);
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int sl = d / P < nstr ? d / P : nstr - 1;
      if constexpr (SWI)
        load_item(wrsrc, run_strip(sl), (sl >> 1) + (sl & 1) * up0, d % P, d < nitems, W[d], S[d]);
      else
        load_item(wrsrc, sr + sl, d / P, d % P, d < nitems, W[d], S[d]);
    }

    // the staged values have arrived before the ring (they were requested first)
    if (static_cast<int>(threadIdx.x) < ncols) {
      lsc[threadIdx.x] = sstage;
      lbi[threadIdx.x] = bstage;
    }

    if (PRE && !have_cc) {  // once, after the first ring has been requested
#pragma unroll
      for (int s = 0; s < TPW * SPT; ++s) {
        const int src = (4 * s + kb) * 4;  // byte address of the source lane for ds_bpermute
        u32x4 ps;
        ps.x = __builtin_amdgcn_ds_bpermute(src, PS.x);
        ps.y = __builtin_amdgcn_ds_bpermute(src, PS.y);
        ps.z = __builtin_amdgcn_ds_bpermute(src, PS.z);
        ps.w = __builtin_amdgcn_ds_bpermute(src, PS.w);
        A[0][s] = prescale_frag<DT>(A[0][s], ps);
      }
    }
    if (kKeepCancel && !have_cc) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < TPW * CPT; ++c) {
          f32x4 cc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < SPC; ++s) cc = mfma16<DT>(A[mt][c * SPC + s], cancel, cc);
          ccs[mt][c] = cc;
        }
    }
    have_cc = true;
    f32x4 tot[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) tot[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = 0; base < nitems; base += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int part = d % P;  // static: D is a multiple of P and base a multiple of D
        const int it = base + d;
        const int sl = it / P;   // strip of the run
        if (it < nitems) {
#pragma unroll
          for (int i = 0; i < IT; ++i) {
            const uint32_t w4[4] = {W[d][i].x, W[d][i].y, W[d][i].z, W[d][i].w};
#pragma unroll
            for (int ch = 0; ch < CPT; ++ch) {
              const int a0 = ((part * IT + i) * CPT + ch) * SPC;  // first A fragment of the chain
              f32x4 acc[MT];
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) {
                if (kKeepCancel) {
                  acc[mt] = ccs[mt][(part * IT + i) * CPT + ch];
                } else {
                  acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                  for (int s = 0; s < SPC; ++s) acc[mt] = mfma16<DT>(A[mt][a0 + s], cancel, acc[mt]);
                }
              }
#pragma unroll
              for (int s = 0; s < SPC; ++s) {
                const u32x4 b = Dequant<DT, BITS>::run(&w4[(ch * SPC + s) * kDw], magic);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt] = mfma16<DT>(A[mt][a0 + s], b, acc[mt]);
              }
              if (G != 0) {
                const float sc = to_f32<DT>(S[d][i * CPT + ch]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                  for (int r = 0; r < 4; ++r) tot[mt][r] = fmaf(acc[mt][r], sc, tot[mt][r]);
              } else {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                  for (int r = 0; r < 4; ++r) tot[mt][r] += acc[mt][r];
              }
            }
          }
          if (part == P - 1) {  // the strip is complete for this wavefront
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
              for (int r = 0; r < 4; ++r) red[((sl * WK + wave) * MT * 4 + mt * 4 + r) * 64 + lane] = tot[mt][r];
              tot[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
          }
        }
        // the slot is free: refill it with the item D places further on (if there is one)
        const int nsl = (it + D) / P < nstr ? (it + D) / P : nstr - 1;
        if constexpr (SWI)
          load_item(wrsrc, run_strip(nsl), (nsl >> 1) + (nsl & 1) * up0, part, it + D < nitems, W[d], S[d]);
        else
          load_item(wrsrc, sr + nsl, (it + D) / P, part, it + D < nitems, W[d], S[d]);
      }
    }

    // ---- the run is done: partial sums of the 16 wavefronts meet in LDS ----
    __syncthreads();
    if constexpr (SWI) {
      // (the ring's registers are named before the sums here, see the end of the run: they are free for the epilogue)
#pragma unroll
      for (int d = 0; d < D; ++d) {
#pragma unroll
        for (int i = 0; i < IT; ++i) asm volatile("" ::"v"(W[d][i]));
#pragma unroll
        for (int q = 0; q < NS; ++q) asm volatile("" ::"v"(S[d][q]));
      }
      const int e = threadIdx.x;  // at most 3 pairs x 256 elements
      if (e < cnt * 256) {
        // e = (pair of the run * 4 + r) * 64 + lane of the MFMA result
        const int u = e >> 8, rr = (e >> 6) & 3, l = e & 63;
        const int m = 4 * (l >> 4) + rr;
        if (m < M) {
          float v[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < WK; ++w) s += red[(((2 * u + h) * WK + w) * 4 + rr) * 64 + l];
            const int cl = (2 * u + h) * kStripCols + (l & 15);
            const float ep_scale = G == 0 ? to_f32<DT>(lsc[cl]) : 1.0f;
            const float ep_bias = p.bias != nullptr ? to_f32<DT>(lbi[cl]) : 0.0f;
            v[h] = s * ep_scale + ep_bias;
          }
          const float s = act_swiglu(v[0], v[1]);
          const int64_t o = static_cast<int64_t>(m) * (N / 2) + (sr + u) * kStripCols + (l & 15);
          if (p.out_f32)
            static_cast<float*>(p.out)[o] = s;
          else
            static_cast<uint16_t*>(p.out)[o] = cast_out<DT>(s);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < (SWI ? 0 : 2); ++q) {
      const int e = threadIdx.x + q * WK * 64;
      if (e < cnt * MT * 256) {
        // e = ((strip of the run * MT + mt) * 4 + r) * 64 + lane of the MFMA result
        const int sl = e / (MT * 256), rr = (e >> 6) % (MT * 4), l = e & 63;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < WK; ++w) s += red[((sl * WK + w) * MT * 4 + rr) * 64 + l];
        const int m = (rr >> 2) * 16 + 4 * (l >> 4) + (rr & 3);
        if (m < M) {
          const int cl = sl * kStripCols + (l & 15);
          const float ep_scale = G == 0 ? to_f32<DT>(lsc[cl]) : 1.0f;
          const int64_t o = static_cast<int64_t>(m) * N + (sr + sl) * kStripCols + (l & 15);
          if (SPLIT) {
            p.ws[static_cast<int64_t>(seg) * M * N + o] = s * ep_scale;
            continue;
          }
          const float ep_bias = p.bias != nullptr ? to_f32<DT>(lbi[cl]) : 0.0f;
          s = act_apply(s * ep_scale + ep_bias, p.act);
          if (p.out_f32)
            static_cast<float*>(p.out)[o] = s;
          else
            static_cast<uint16_t*>(p.out)[o] = cast_out<DT>(s);
        }
      }
    }
    // Name the ring's registers: the loads past the last item (which fetch
    // nothing) are then known to have completed here, and the next run starts
    // with a load queue whose content the compiler knows exactly -- otherwise
    // the first loads of a run would wait for older ones they do not depend on.
    if constexpr (!SWI) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
#pragma unroll
        for (int i = 0; i < IT; ++i) asm volatile("" ::"v"(W[d][i]));
#pragma unroll
        for (int q = 0; q < NS; ++q) asm volatile("" ::"v"(S[d][q]));
      }
    }
    if (sr + kRun < s1) __syncthreads();  // the next run overwrites the partial sums
  }
}

struct Args {
  const void* x; const void* codes; const void* bias; const void* scale; void* out;
  int M, K, N, gshift, out_f32; hipStream_t stream;
  const void* pre; int act;
  int nseg; float* ws;  // K runs across workgroups and where their sums go (nseg = 1: none)
  bool swi = false;     // gate|up projection: write silu(gate) * up (the one-run form)
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

// Raises a kernel's dynamic LDS limit once per device.
inline void allow_lds(const void* kern, size_t lds, std::atomic<uint32_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const uint32_t bit = 1u << (dev & 31);
  if (done.load(std::memory_order_acquire) & bit) return;
  (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  done.fetch_or(bit, std::memory_order_release);
}

// LDS of a launch: partial sums, scales and bias of the longest run of strips.
// sets: strip sets (workgroups, or workgroups / K runs); mt: 16-row operands.
// swi: the sets are sets of strip pairs.
inline size_t batch_lds(int64_t N, int sets, int mt, bool swi = false) {
  const int spu = swi ? 2 : 1;
  const int64_t units = N / kStripCols / spu;
  int64_t per_wg = (units + sets - 1) / sets;
  if (per_wg > kBatchRun / mt / spu) per_wg = kBatchRun / mt / spu;
  per_wg *= spu;  // strips
  return static_cast<size_t>(per_wg * kBatchWaves * mt * 1024 + 2 * per_wg * kStripCols * 2);
}

// grid: strip sets; with SPLIT every set is worked on by a.nseg workgroups
template <int DT, int BITS, int G, int TPW, int IT, int D, bool PRE, int MT = 1, bool SPLIT = false, bool SWI = false>
void launch_pre(const Args& a, int grid) {
  const size_t lds = batch_lds(a.N, grid, MT, SWI);
  auto kern = batch_kernel<DT, BITS, G, TPW, IT, D, PRE, MT, SPLIT, SWI>;
  static std::atomic<uint32_t> configured{0};  // per instantiation
  allow_lds(reinterpret_cast<const void*>(kern), 160 * 1024, configured);
  BatchParams p;
  p.x = static_cast<const uint16_t*>(a.x);
  p.codes = static_cast<const uint8_t*>(a.codes);
  p.bias = static_cast<const uint16_t*>(a.bias);
  p.scale = static_cast<const uint16_t*>(a.scale);
  p.out = a.out;
  p.M = a.M; p.K = a.K; p.N = a.N;
  p.gshift = a.gshift;
  p.out_f32 = a.out_f32;
  p.strips_q = a.N / kStripCols / (SWI ? 2 : 1) / grid;
  p.strips_r = a.N / kStripCols / (SWI ? 2 : 1) % grid;
  p.pre = PRE ? static_cast<const uint16_t*>(a.pre) : nullptr;
  p.act = a.act;
  p.nseg = SPLIT ? a.nseg : 1;
  p.ntiles = a.K / (BITS == 8 ? 64 : 128);
  p.ws = a.ws;
  kern<<<dim3(static_cast<unsigned>(grid * p.nseg)), dim3(kBatchWaves * 64), lds, a.stream>>>(p);
}

// The fused activation scales are built where the registers allow: A
// fragments of 32 registers or fewer (K <= 4096), except int8 codes with
// group-wise scales at K = 4096.
constexpr bool pre_fits(int bits, int group, int k_steps_per_wave) {
  return k_steps_per_wave <= 8 && !(bits == 8 && group != 0 && k_steps_per_wave == 8);
}

template <int DT, int BITS, int G, int TPW, int IT, int D>
void launch_one(const Args& a, int grid) {
  if constexpr (pre_fits(BITS, G, TPW * (BITS == 8 ? 2 : 4))) {
    if (a.pre != nullptr) {  // (never together with the gate|up form: launch_linear_batch refuses)
      launch_pre<DT, BITS, G, TPW, IT, D, true>(a, grid);
      return;
    }
  }
  if (a.swi) launch_pre<DT, BITS, G, TPW, IT, D, false, 1, false, true>(a, grid);
  else launch_pre<DT, BITS, G, TPW, IT, D, false>(a, grid);
}

// tpw = K / (16 * tile depth): 1, 2 or 4.  Items and ring depths by what the
// 128 registers of a 16-wavefront workgroup hold next to the A fragments
// (16 registers per tile of the run): an item of IT tiles is 4 * IT registers.
template <int DT, int BITS, int G>
void launch_cfg(const Args& a, int grid, int tpw) {
  if constexpr (BITS == 4) {
    if (tpw == 1) launch_one<DT, 4, G, 1, 1, 4>(a, grid);        // K = 2048
    else if (tpw == 2) launch_one<DT, 4, G, 2, 2, 3>(a, grid);   // K = 4096
    else if constexpr (G != 64) launch_one<DT, 4, G, 4, 2, 2>(a, grid);  // K = 8192
  } else {
    if (tpw == 2) launch_one<DT, 8, G, 2, 2, 3>(a, grid);        // K = 2048
    else if (tpw == 4) launch_one<DT, 8, G, 4, 4, 2>(a, grid);   // K = 4096
  }
}

template <int DT, int BITS>
void launch_g(const Args& a, int grid, int tpw) {
  if (a.gshift < 0) launch_cfg<DT, BITS, 0>(a, grid, tpw);
  else if (a.gshift == 6) launch_cfg<DT, BITS, 64>(a, grid, tpw);
  else launch_cfg<DT, BITS, 128>(a, grid, tpw);
}

// The K-split form.  k2: a wavefront's run is 256 k long (two int4 tiles,
// four int8 tiles) instead of 128; the items and ring depths are those of the
// one-run form with the same run.  Up to 16 rows, or up to 32 as two 16-row
// operands -- those with the short run only: 64 registers of A fragments
// leave no room for the ring.
template <int DT, int BITS, int G, int MT>
void launch_split_cfg(const Args& a, int sets, bool k2) {
  if constexpr (MT == 1) {
    if (k2) {
      if constexpr (BITS == 4) launch_pre<DT, 4, G, 2, 2, 3, false, 1, true>(a, sets);
      else launch_pre<DT, 8, G, 4, 4, 2, false, 1, true>(a, sets);
      return;
    }
  }
  if constexpr (BITS == 4) launch_pre<DT, 4, G, 1, 1, 4, false, MT, true>(a, sets);
  else launch_pre<DT, 8, G, 2, 2, 3, false, MT, true>(a, sets);
}

template <int DT, int BITS>
void launch_split_g(const Args& a, int sets, bool k2) {
  if (a.M <= 16) {
    if (a.gshift < 0) launch_split_cfg<DT, BITS, 0, 1>(a, sets, k2);
    else if (a.gshift == 6) launch_split_cfg<DT, BITS, 64, 1>(a, sets, k2);
    else launch_split_cfg<DT, BITS, 128, 1>(a, sets, k2);
  } else {
    if (a.gshift < 0) launch_split_cfg<DT, BITS, 0, 2>(a, sets, k2);
    else if (a.gshift == 6) launch_split_cfg<DT, BITS, 64, 2>(a, sets, k2);
    else launch_split_cfg<DT, BITS, 128, 2>(a, sets, k2);
  }
}

}  // namespace

// K must split into the same number of whole weight tiles for each of the 16
// wavefronts, and that number must be one the kernel is built for: K = 2048
// or 4096, and K = 8192 with int4 codes unless their groups are 64 long (64
// registers of A fragments leave no room for more).
bool linear_batch_supports(int64_t M, int64_t K, int bits, int group_size) {
  if (M < 1 || M > 16) return false;
  if (K == 2048 || K == 4096) return true;
  return K == 8192 && bits == 4 && group_size != 64;
}

int linear_batch_cus() { return num_cus(); }

// The one-run form writes silu(gate) * up of a gate|up projection itself when
// the halves are whole strips and a run's gate and up strips lie within 2 GiB
// of each other (no activation scales in the same call).
bool linear_batch_fuses_swiglu(int64_t K, int64_t N, int bits) {
  return N % (2 * kStripCols) == 0 && (N / kStripCols / 2 + kBatchRun) * strip_bytes(K, bits) < (int64_t{1} << 31);
}

// Whether launch_linear_batch applies a Fuse::pre_scale itself for this K.
bool linear_batch_fuses_pre_scale(int64_t K, int bits, int group_size) {
  return pre_fits(bits, group_size > 0 ? group_size : 0, static_cast<int>(K / 32 / kBatchWaves));
}

// Grid (workgroups: one per CU, fewer when there are fewer strips) and the
// weight tiles of a strip per wavefront.
// swi: the unit a workgroup owns is a pair of strips.
void plan_linear_batch(int64_t K, int64_t N, int bits, int* grid, int* tpw, bool swi) {
  const int64_t nstrips = N / kStripCols / (swi ? 2 : 1);
  const int cus = num_cus();
  *grid = static_cast<int>(nstrips < cus ? nstrips : cus);
  *tpw = static_cast<int>(K / (bits == 8 ? 64 : 128) / kBatchWaves);
}

int launch_linear_batch(const void* x, const void* codes, const void* bias, const void* scale,
                        int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                        void* out, bool out_f32, hipStream_t stream, const Fuse& f) {
  const int gshift = group_size == 64 ? 6 : (group_size == 128 ? 7 : -1);
  int grid = 1, tpw = 1;
  const bool swi = f.act == WOL_ACT_SWIGLU;
  if (swi && (!linear_batch_fuses_swiglu(K, N, bits) || f.pre_scale != nullptr)) return WOL_ERR_BAD_SHAPE;
  plan_linear_batch(K, N, bits, &grid, &tpw, swi);
  const Args a{x, codes, bias, scale, out, static_cast<int>(M), static_cast<int>(K),
               static_cast<int>(N), gshift, out_f32 ? 1 : 0, stream,
               linear_batch_fuses_pre_scale(K, bits, group_size) ? f.pre_scale : nullptr,
               swi ? WOL_ACT_NONE : f.act, 1, nullptr, swi};
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) launch_g<WOL_DTYPE_BF16, 8>(a, grid, tpw); else launch_g<WOL_DTYPE_BF16, 4>(a, grid, tpw);
  } else {
    if (bits == 8) launch_g<WOL_DTYPE_F16, 8>(a, grid, tpw); else launch_g<WOL_DTYPE_F16, 4>(a, grid, tpw);
  }
  return check_launch();
}

// The K-split form takes up to 32 rows and any K made of at least 16 whole
// weight tiles (128 k for int4, 64 k for int8).
bool linear_batch_split_supports(int64_t M, int64_t K, int bits, int group_size) {
  (void)group_size;
  const int64_t tk = bits == 8 ? 64 : 128;
  return M >= 1 && M <= 32 && K % tk == 0 && K / tk >= 16;
}

// How the K-split form cuts a problem: k2 (256 k per wavefront and run
// instead of 128), the number of runs and the number of strip sets (each set
// is worked on by one workgroup per run; sets x runs is about the CU count).
// The longer run halves the partial sums and doubles the activations a
// workgroup holds: measured faster from seven short runs on (K >= 13824 for
// int4), slower below.  Two 16-row operands leave registers for the short run
// only.
void plan_linear_batch_split(int64_t M, int64_t K, int64_t N, int bits, int group_size, bool* k2,
                             int* nseg, int* sets) {
  (void)group_size;
  const int64_t tk = bits == 8 ? 64 : 128, tiles = K / tk;
  const int64_t nstrips = N / kStripCols;
  const int cus = num_cus();
  const int64_t per_run_short = kBatchWaves * (128 / tk);
  *k2 = M <= 16 && (tiles + per_run_short - 1) / per_run_short >= 7;
  const int64_t per_run = *k2 ? 2 * per_run_short : per_run_short;
  *nseg = static_cast<int>((tiles + per_run - 1) / per_run);
  int64_t v = cus / *nseg;
  if (v < 1) v = 1;
  *sets = static_cast<int>(v < nstrips ? v : nstrips);
}

size_t linear_batch_split_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  if (!linear_batch_split_supports(M, K, bits, group_size)) return 0;
  bool k2 = false;
  int nseg = 1, sets = 1;
  plan_linear_batch_split(M, K, N, bits, group_size, &k2, &nseg, &sets);
  return static_cast<size_t>(nseg) * M * N * sizeof(float);
}

void describe_linear_batch_split(int64_t M, int64_t K, int64_t N, int bits, int group_size, char* buf, size_t n) {
  bool k2 = false;
  int nseg = 1, sets = 1;
  plan_linear_batch_split(M, K, N, bits, group_size, &k2, &nseg, &sets);
  snprintf(buf, n, "wol::batch_kernel: %d strip sets x %d K runs of %d k, %d-row operands x %d + reduce_partials_kernel",
           sets, nseg, kBatchWaves * (k2 ? 256 : 128), 16, M > 16 ? 2 : 1);
}

// ws: nseg x M x N floats (linear_batch_split_workspace).  No fused pre-scale.
int launch_linear_batch_split(const void* x, const void* codes, const void* bias, const void* scale,
                              int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                              void* out, bool out_f32, void* ws, size_t ws_bytes, hipStream_t stream,
                              const Fuse& f) {
  if (!linear_batch_split_supports(M, K, bits, group_size) || f.pre_scale != nullptr) return WOL_ERR_BAD_SHAPE;
  if (ws == nullptr || ws_bytes < linear_batch_split_workspace(M, K, N, bits, group_size)) return WOL_ERR_WORKSPACE;
  const int gshift = group_size == 64 ? 6 : (group_size == 128 ? 7 : -1);
  bool k2 = false;
  int nseg = 1, sets = 1;
  plan_linear_batch_split(M, K, N, bits, group_size, &k2, &nseg, &sets);
  const Args a{x, codes, nullptr, scale, nullptr, static_cast<int>(M), static_cast<int>(K),
               static_cast<int>(N), gshift, 0, stream, nullptr, WOL_ACT_NONE, nseg, static_cast<float*>(ws)};
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) launch_split_g<WOL_DTYPE_BF16, 8>(a, sets, k2); else launch_split_g<WOL_DTYPE_BF16, 4>(a, sets, k2);
  } else {
    if (bits == 8) launch_split_g<WOL_DTYPE_F16, 8>(a, sets, k2); else launch_split_g<WOL_DTYPE_F16, 4>(a, sets, k2);
  }
  if (const int rc = check_launch(); rc != WOL_OK) return rc;
  return launch_reduce_partials(static_cast<const float*>(ws), nseg, bias, dtype, out, out_f32, M, N, f.act, stream);
}

}  // namespace wol
