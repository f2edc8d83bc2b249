// weight_only_linear for small M (decode): a bandwidth-bound kernel that
// streams the GFX950-packed weight once with 128-bit loads and feeds it to
// the matrix cores.
//
// One workgroup owns one strip of 16 output columns; its WK wavefronts split
// K between them.  A wavefront loads 16 bytes per lane (1 KiB per load, fully
// coalesced, one tile of 64 or 128 k), turns the biased codes into bf16/fp16
// bit patterns with AND-OR / byte-permute tricks (the code plus a constant
// offset, exact), and issues v_mfma_f32_16x16x32 with the activations as the
// A operand -- the MFMA does the multiply and the reduction over k across
// lanes.  The constant offset is removed by a second MFMA of the same A
// against a constant B, exact in fp32 up to the accumulator's rounding; the
// accumulator restarts every k step so the cancelling terms stay small.
// Scales multiply the fp32 partial sums, never the weights, so nothing is
// rounded to T before the final cast.
//
// Small M does not fill the 16 rows of the A operand, and rows of the result
// are independent of each other, so the spare rows carry other k steps: with
// MP = M rounded up to a power of two, one 16-byte-per-lane load of x (1 KiB,
// coalesced) fills row group `slot` with the activations of k step `slot`,
// S = 16/MP steps at once.  The MFMA of step s against that operand produces
// the wanted dot products in row group s and unrelated finite sums elsewhere;
// a per-lane select keeps only row group s.  For M = 1 this is one x load per
// 512 k instead of sixteen.  Rows beyond M may hold anything (they are never
// stored), so no operand is ever zero-filled.
// Partial sums of row groups and of the WK wavefronts meet in LDS in a fixed
// order.
#include "wol_common.h"
#include "wol_dequant.h"

// The instantiations are split over two translation units by activation
// type, so that they compile side by side: this file is the bf16 half and
// holds the host-side planning; wol_linear_stream_f16.hip includes it with
// WOL_STREAM_F16_TU defined and yields the fp16 half only.
namespace wol {

// What a launch needs, whichever half runs it.
struct StreamArgs {
  const void* x; const void* codes; const void* bias; const void* scale; void* out;
  int M, K, N, gshift, out_f32, tn; hipStream_t stream;
  const void* pre; int act;  // act: none or gelu; the gate|up form is chosen by the caller of the half
};
// The fp16 half (wol_linear_stream_f16.hip): swi = the gate|up form, wk = wavefronts of the workgroup.
void launch_linear_stream_f16(const StreamArgs& a, int bits, bool swi, int wk, int nu);

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
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

// Sum of v over the four lane groups (lanes l, l^16, l^32, l^48), in every lane.
__device__ inline float sum_lane_groups(float v, bool x16, bool x32) {
  if (x32) {
    const auto p = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(p[0]) + __uint_as_float(p[1]);
  }
  if (x16) {
    const auto q = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(q[0]) + __uint_as_float(q[1]);
  }
  return v;
}

// Which block of strips a workgroup takes.  Workgroups are dealt to the 8 XCDs
// round-robin by their linear id, and every XCD has an L2 of its own.  Four
// neighbouring strips share each 128-byte line of the scales, the bias and the
// output (16 columns of 2 bytes per strip): in linear order the four would sit
// on four XCDs and each L2 would fetch the line for itself, four times the
// scales' bytes from HBM.  Every round of 32 workgroups therefore takes 32
// consecutive blocks with four neighbours per XCD; what is left over after the
// last whole round keeps the linear order.
__device__ inline int block_of_workgroup(int b, int nblocks) {
  if (b >= (nblocks & ~31)) return b;
  const int r = b & 31;
  return (b & ~31) + (r & 7) * 4 + (r >> 3);
}

// The same for the kernels whose workgroups are all resident at once (every
// load issued at once, 257 to 1024 workgroups on 256 CUs): there workgroups b, b + 256, b + 512, b + 768 run on one CU (read back
// from HW_REG_HW_ID: always so), and giving them neighbouring strips lets the
// CU's L1 fetch a line of scales once for all of them as well -- the gathers
// of the later workgroups meet the first one's outstanding miss.  CU slot
// c = b % 256 sits on XCD c % 8; slots are numbered XCD by XCD so that the
// strips of neighbouring slots still meet in one L2, and the slots the last,
// partial round reaches (c < nblocks % 256) own one strip more.  Written
// without a branch: both numberings are a few scalar instructions, and a
// branch here cost the launches that keep the other numbering 1 %.
__device__ inline int block_of_resident_workgroup(int b, int nblocks) {
  const int r5 = b & 31;
  const int by_xcd = b >= (nblocks & ~31) ? b : (b & ~31) + (r5 & 7) * 4 + (r5 >> 3);
  const int q = nblocks >> 8, rem = nblocks & 255;
  const int c = b & 255, r = b >> 8;
  const int x = c & 7, i = c >> 3;
  const int a = rem >> 3, t = rem & 7;
  const int more = a + (x < t ? 1 : 0);  // slots of this XCD with one strip more
  const int by_cu = (x * 32 + i) * q + a * x + (x < t ? x : t) + (i < more ? i : more) + r;
  return nblocks > 256 && nblocks <= 1024 ? by_cu : by_xcd;
}

// NU > 0: every wavefront owns exactly NU units and issues all their loads at
// once (the whole problem is in flight from the first cycle; used when K is
// small enough).  NU == 0: a wavefront walks its share of the units with the
// loads of the next units (one to three, by register budget) in flight while
// it consumes the current one.
//
// TN strips (16 columns each) share one workgroup and with it every load of
// the activations: the activation traffic out of L2, which grows with M, drops
// by TN.
//
// PRE: the activations are multiplied by a per-channel scale vector on their
// way into the A operand, each product rounded to T as
// apply_per_channel_scale rounds it (built for one row only; other row counts
// get the scaled activations from a pass of that kernel).
//
// SWI: the weight is a gate|up projection and the kernel writes
// silu(gate) * up, [M, N/2].  The first half of the workgroup's wavefronts
// works on gate strip b, the second half on up strip b + N/32, each half
// splitting K as a whole workgroup does otherwise; the two sums of an output
// element meet in the epilogue, which is the only place that differs.
//
// STAMP (a diagnostic instantiation, never on a product path; NU > 0 only):
// every wavefront reads the clocks at entry, once its loads are issued, once
// they have all landed (an explicit wait the product kernel does not have),
// after its arithmetic, after the workgroup's barrier and at the end, and
// leaves them in `stamps` (wol_decode_phases).
template <int DT, int BITS, int MP, int MT, int WK, int NU, int TN, bool GROUPED, bool PRE, bool SWI, bool STAMP = false>
struct StreamKernel {
  static_assert(MT == 1 || MP == 16, "several M tiles only with full 16-row operands");
  static_assert(!SWI || (TN == 1 && MT == 1 && WK >= 2), "the gate|up form pairs two single strips");
  static constexpr int kWS = SWI ? WK / 2 : WK;       // wavefronts that share a strip
  static constexpr int kS = 16 / MP;                  // k steps sharing one A operand
  static constexpr int kSPT = BITS == 8 ? 2 : 4;      // k steps per 16-byte weight tile
  static constexpr int kDw = BITS == 8 ? 2 : 1;       // dwords per k step
  static constexpr int kU = kS > kSPT ? kS : kSPT;    // k steps per unit of work
  static constexpr int kNT = kU / kSPT;               // weight tiles per unit
  static constexpr int kNA = kU / kS;                 // A operands per unit
  static constexpr int kRowsPerGroup = MP < 4 ? 4 / MP : 1;  // row groups inside one lane group
  static constexpr int kClasses = kS / kRowsPerGroup;        // lane groups that receive results
  static constexpr int kLive = MP == 1 ? 1 : (MP == 2 ? 2 : 4);  // accumulators left after folding
  // Group-wise scales a lane loads per unit.  With MP < 16 a lane keeps only
  // the steps of its own class (all others land in sums that are discarded),
  // kRowsPerGroup consecutive steps per A operand, and two consecutive steps
  // (64 k) always share a group: one load per pair.  MP = 16 keeps every step.
  static constexpr int kPairs = kRowsPerGroup >= 2 ? kRowsPerGroup / 2 : 1;
  static constexpr int kNS = MP == 16 ? kU / 2 : kNA * kPairs;
  // Walking wavefronts: K's whole weight tiles may end with a partial unit when
  // a unit spans several tiles (otherwise they divide into whole units).
  static constexpr bool kPartial = NU == 0 && kU > kSPT;
  // Walking wavefronts: units in the ring, from the registers one unit takes.
  // The ring stays within 64 registers: 16 wavefronts leave 128 each, and a
  // narrower workgroup that needs more than 128 loses its neighbour on the CU.
  static constexpr int kUnitRegs = 4 * (TN * kNT + kNA * MT + (PRE ? kNA : 0)) + (GROUPED ? TN * kNS : 0);
  static constexpr int kD = 64 / kUnitRegs < 2 ? 2 : (64 / kUnitRegs > 4 ? 4 : 64 / kUnitRegs);

  const uint16_t* x;
  const uint16_t* scale;
  const uint16_t* pre;  // [K] per-channel scales of the activations (PRE)
  unsigned long long* stamps = nullptr;  // STAMP: [workgroup][wavefront][8]
  int act;              // WOL_ACT_NONE or WOL_ACT_GELU
  int M, K, N;
  int gshift;  // log2(group_size) when GROUPED
  int vsteps;  // k steps that lie in whole 16-byte weight tiles (all but an int4 half tile)
  int lane, j, kb;
  int n[TN];  // this lane's column in each strip (clamped to the last valid one)
  uint32_t magic;
  // totc[mt][c] gathers the steps whose results belong to lane group c (for
  // MP = 8: lane groups 2c, 2c+1); lanes outside that group accumulate sums
  // that are discarded when the classes are merged at the end.
  f32x4 totc[TN][MT][kClasses];

  // Everything one unit of work (kU k steps of this strip) reads from memory.
  struct Unit {
    u32x4 wv[TN][kNT];
    u32x4 av[kNA][MT];
    u32x4 pv[PRE ? kNA : 1];  // the activation scales of the same k as av
    uint16_t sraw[TN][kNS];
  };

  // A operand whose row group `slot` holds k step (step0 + slot); with
  // spread == false every row group holds step0.
  // tail: the unit is the partial one that ends K.
  __device__ inline u32x4 load_a(int mt, int step0, bool spread, bool tail = false) const {
    int m = mt * 16 + (j % MP);
    if (MP > 1 || MT > 1) m = m < M ? m : M - 1;  // rows past M are never stored
    int step = step0 + (spread ? j / MP : 0);
    if (tail) {
      // steps past the end read the
      // last valid one (never past the row) and count as zero
      const bool valid = step < vsteps;
      step = valid ? step : vsteps - 1;
      const u32x4 v = *reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(m) * K + step * 32 + 8 * kb);
      return valid ? v : u32x4{0u, 0u, 0u, 0u};
    }
    return *reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(m) * K + step * 32 + 8 * kb);
  }

  // The activation scales that go with load_a(., step0, spread, tail): the same
  // k for every row.
  __device__ inline u32x4 load_pre(int step0, bool spread, bool tail = false) const {
    int step = step0 + (spread ? j / MP : 0);
    if (tail) step = step < vsteps ? step : vsteps - 1;
    return *reinterpret_cast<const u32x4*>(pre + step * 32 + 8 * kb);
  }

  __device__ inline uint16_t load_scale_raw(int step, int t) const {
    const uint16_t* row = scale + static_cast<int64_t>((step * 32) >> gshift) * N;
    return row[n[t]];
  }

  // Index into Unit::sraw of the scale that step s of a unit uses.
  __device__ static constexpr int scale_slot(int s) {
    return MP == 16 ? s / 2 : (s / kS) * kPairs + ((s % kS) % kRowsPerGroup) / 2;
  }

  // The small loads (activations, scales) go first: the memory system returns
  // loads in order, so the first weight tile can be consumed while the later
  // ones are still on their way.
  // Walking wavefronts load through buffer descriptors: `wr` ends with the
  // wavefront's share of the strip, `xr` covers the activations.  A unit past
  // the share (u > ulast) is requested like any other, from offsets beyond the
  // descriptors: it costs no traffic and arrives as zeros, and with a zero A
  // operand every sum it is added to stays exactly as it was.  Its scales repeat
  // those of unit `ulast`.  Nothing in the walk is loaded under a condition, so
  // the compiler counts precisely how many loads may still be in flight when a
  // unit is consumed.
  __device__ inline void load_unit_walk(Unit& d, const __amdgpu_buffer_rsrc_t (&wr)[TN],
                                        __amdgpu_buffer_rsrc_t xr, int u, int ulast) const {
    const bool real = u <= ulast;
    const int step0 = (real ? u : ulast) * kU;
    constexpr uint32_t kNowhere = 0xC0000000u;  // beyond every descriptor (activations end below 2^31 bytes)
#pragma unroll
    for (int a = 0; a < kNA; ++a)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        int m = mt * 16 + (j % MP);
        if (MP > 1 || MT > 1) m = m < M ? m : M - 1;
        const uint32_t off = static_cast<uint32_t>(m) * static_cast<uint32_t>(K) * 2u +
                             static_cast<uint32_t>(step0 + a * kS + j / MP) * 64u + 16u * kb;
        d.av[a][mt] = __builtin_bit_cast(
            u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, static_cast<int>(real ? off : kNowhere), 0, 0));
      }
    if (PRE) {
#pragma unroll
      for (int a = 0; a < kNA; ++a) d.pv[a] = load_pre(step0 + a * kS, true);
    }
    if (GROUPED) {
      const int mine = MP == 8 ? (kb >> 1) : kb;
#pragma unroll
      for (int p = 0; p < kNS; ++p) {
        const int step = MP == 16 ? step0 + 2 * p
                                  : step0 + (p / kPairs) * kS + mine * kRowsPerGroup + 2 * (p % kPairs);
#pragma unroll
        for (int t = 0; t < TN; ++t) d.sraw[t][p] = load_scale_raw(step, t);
      }
    }
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int i = 0; i < kNT; ++i) {
        // the whole offset in the vector operand: that is the one the
        // hardware checks against the descriptor's size
        const uint32_t off = real ? static_cast<uint32_t>(u * kNT + i) * 1024u + 16u * lane : kNowhere;
        d.wv[t][i] = __builtin_bit_cast(
            u32x4, __builtin_amdgcn_raw_buffer_load_b128(wr[t], static_cast<int>(off), 0, 2));
      }
  }

  __device__ inline void load_unit(Unit& d, const u32x4* const (&tp)[TN], int u, bool tail = false) const {
    const int step0 = u * kU;
#pragma unroll
    for (int a = 0; a < kNA; ++a)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) d.av[a][mt] = load_a(mt, step0 + a * kS, true, tail);
    if (PRE) {
#pragma unroll
      for (int a = 0; a < kNA; ++a) d.pv[a] = load_pre(step0 + a * kS, true, tail);
    }
    if (GROUPED) {
      const int mine = MP == 8 ? (kb >> 1) : kb;
#pragma unroll
      for (int p = 0; p < kNS; ++p) {
        const int step = MP == 16 ? step0 + 2 * p
                                  : step0 + (p / kPairs) * kS + mine * kRowsPerGroup + 2 * (p % kPairs);
        const int sstep = tail ? (step < vsteps ? step : vsteps - 1) : step;
#pragma unroll
        for (int t = 0; t < TN; ++t) d.sraw[t][p] = load_scale_raw(sstep, t);
      }
    }
    if (NU > 0) __builtin_amdgcn_sched_barrier(0);  // keep the compiler from moving them behind the weights
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int i = 0; i < kNT; ++i) {
        int tile = step0 / kSPT + i;
        if (tail) tile = tile < vsteps / kSPT ? tile : vsteps / kSPT - 1;
        d.wv[t][i] = __builtin_nontemporal_load(tp[t] + tile * 64);
      }
  }

  // mfma(A, constant B): the term that removes the dequantiser's offset.  It
  // depends on A only, so it is computed once per A operand and used as the
  // accumulator input of every step that shares the operand.
  __device__ inline f32x4 cancel_term(u32x4 a) const {
    const u32x4 cancel = {Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel,
                          Dequant<DT, BITS>::kCancel, Dequant<DT, BITS>::kCancel};
    return mfma16<DT>(a, cancel, f32x4{0.f, 0.f, 0.f, 0.f});
  }

  // One k step: dequantise, one MFMA per M tile, add the rows of row group
  // `slot` to that group's class.
  __device__ inline void step_mfma(const uint32_t* w, const u32x4 (&a)[MT], const f32x4 (&cc)[MT],
                                   int slot, float sc, int t) {
    const u32x4 b = Dequant<DT, BITS>::run(w, magic);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const f32x4 acc = mfma16<DT>(a[mt], b, cc[mt]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool rsel = MP >= 4 ? true : (r / MP == slot % kRowsPerGroup);
        if (rsel) {
          const float v = totc[t][mt][slot / kRowsPerGroup][r];
          totc[t][mt][slot / kRowsPerGroup][r] = GROUPED ? fmaf(acc[r], sc, v) : v + acc[r];
        }
      }
    }
  }

  __device__ inline void compute_unit(const Unit& d) {
    f32x4 cc[kNA][MT];
    u32x4 av[kNA][MT];
#pragma unroll
    for (int a = 0; a < kNA; ++a)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        av[a][mt] = PRE ? prescale_frag<DT>(d.av[a][mt], d.pv[a]) : d.av[a][mt];
        cc[a][mt] = cancel_term(av[a][mt]);
      }
#pragma unroll
    for (int s = 0; s < kU; ++s)
#pragma unroll
      for (int t = 0; t < TN; ++t) {
        const u32x4 v = d.wv[t][s / kSPT];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        const float sc = GROUPED ? to_f32<DT>(d.sraw[t][scale_slot(s)]) : 1.0f;
        step_mfma(w + (s % kSPT) * kDw, av[s / kS], cc[s / kS], s % kS, sc, t);
      }
  }

  __device__ inline void run(const uint8_t* codes, const uint16_t* bias, void* out, int out_f32,
                             float* red) {
    unsigned long long st_rt0 = 0, st_c0 = 0, st_ca = 0, st_c1 = 0, st_c2 = 0, st_c3 = 0, st_c4 = 0;
    if (STAMP) {
      st_rt0 = __builtin_amdgcn_s_memrealtime();
      st_c0 = __builtin_readcyclecounter();
    }
    lane = threadIdx.x & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = SWI ? wave_all % kWS : wave_all;  // its place among the wavefronts of its strip
    j = lane & 15;
    kb = lane >> 4;
    const int nstrips = N / kStripCols;
    const int bid = NU > 0 ? block_of_resident_workgroup(static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x))
                           : block_of_workgroup(static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x));
    const uint8_t* strip[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      int tn = bid * TN + t;
      if (SWI) tn += (wave_all / kWS) * (nstrips / 2);  // the up strip of the same output columns
      tn = tn < nstrips ? tn : nstrips - 1;  // a strip past the end repeats the last one and is not stored
      n[t] = tn * kStripCols + j;
      strip[t] = codes + static_cast<int64_t>(tn) * strip_bytes(K, BITS);
    }
    magic = Dequant<DT, BITS>::kMagic;
    asm volatile("" : "+v"(magic));  // keep the constant in a VGPR
    if (STAMP) {
      asm volatile("" ::"s"(strip[0]), "s"(scale), "s"(x));  // the kernel's arguments have arrived
      st_ca = __builtin_readcyclecounter();
    }
    const int nsteps = K / 32;
    vsteps = BITS == 4 ? (K / 128) * 4 : nsteps;
    const int nunits = (NU > 0 ? nsteps : vsteps) / kU;  // whole units
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < kClasses; ++c) totc[t][mt][c] = f32x4{0.f, 0.f, 0.f, 0.f};

    // what the epilogue needs from memory, requested before the long loads:
    // thread t always stores column t % 16 of the strip
    // (raw bits; they are converted where they are used, after the long loads)
    // (SWI: the gate column's and, in slot 1, the up column's)
    constexpr int kEp = SWI ? 2 : TN;
    uint16_t ep_sraw[kEp], ep_braw[kEp];
    const u32x4* tp[TN];
#pragma unroll
    for (int t = 0; t < kEp; ++t) {
      const int col = SWI ? bid * kStripCols + j + t * (N / 2) : n[t];
      // group-wise scales have been applied step by step; and most linears
      // of a decoder carry no bias: neither load is issued then (a load of two
      // bytes per lane occupies the CU's memory pipeline like any other)
      ep_sraw[t] = 0;
      ep_braw[t] = 0;
      if (!GROUPED) ep_sraw[t] = scale[col];
      if (bias != nullptr) ep_braw[t] = bias[col];
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) tp[t] = reinterpret_cast<const u32x4*>(strip[t]) + lane;
    if (NU > 0) {
      Unit d[NU > 0 ? NU : 1];
#pragma unroll
      for (int i = 0; i < NU; ++i) load_unit(d[i], tp, wave * NU + i);
      __builtin_amdgcn_sched_barrier(0);  // every load is in flight before the first wait
      if (STAMP) {
        st_c1 = __builtin_readcyclecounter();
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): every load has landed
        st_c2 = __builtin_readcyclecounter();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < NU; ++i) compute_unit(d[i]);
    } else {
      const int u0 = nunits * wave / kWS, u1 = nunits * (wave + 1) / kWS;
      // the partial unit that ends K goes to wavefront 0 (the floor split
      // gives it the fewest whole units), ahead of its walk
      const bool tail = kPartial && wave == 0 && nunits * kU < vsteps;
      if (u0 < u1 || tail) {
        int u = u0;
        if (tail) {
          Unit dt;
          load_unit(dt, tp, nunits, true);
          compute_unit(dt);
        }
        if (u0 < u1) {
          __amdgpu_buffer_rsrc_t wr[TN];
#pragma unroll
          for (int t = 0; t < TN; ++t)
            wr[t] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(strip[t]), 0, u1 * kNT * 1024,
                                                      0x00020000);
          const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
              const_cast<uint16_t*>(x), 0, static_cast<int>(static_cast<uint32_t>(M) * static_cast<uint32_t>(K) * 2u),
              0x00020000);
          // A ring of kD units, kD - 1 of them on their way while one is
          // consumed: what hides the memory latency is the number of bytes in
          // flight, and a unit is small when the operand has many rows.  The
          // barriers keep every load ahead of the arithmetic that follows it
          // in program order.
          Unit d[kD];
#pragma unroll
          for (int i = 0; i < kD - 1; ++i) load_unit_walk(d[i], wr, xr, u + i, u1 - 1);
          for (; u + kD <= u1; u += kD) {
#pragma unroll
            for (int i = 0; i < kD; ++i) {
              load_unit_walk(d[(i + kD - 1) % kD], wr, xr, u + i + kD - 1, u1 - 1);
              __builtin_amdgcn_sched_barrier(0);
              compute_unit(d[i]);
              __builtin_amdgcn_sched_barrier(0);
            }
          }
          // fewer than kD units are left, all of them requested already
#pragma unroll
          for (int i = 0; i < kD - 1; ++i) {
            if (u + i < u1) compute_unit(d[i]);
          }
        }
      }
      if (BITS == 4 && wave == 0) {
        // the half tile that ends a K that is 64 mod 128: two k steps, 8 bytes
        // of codes per lane.  Every row group carries the same step, row
        // group 0 is kept.
        for (int step = vsteps; step < nsteps; step += 2) {
          u32x4 a[2][MT];
          f32x4 cc[2][MT];
#pragma unroll
          for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              a[st][mt] = load_a(mt, step + st, false);
              if (PRE) a[st][mt] = prescale_frag<DT>(a[st][mt], load_pre(step + st, false));
              cc[st][mt] = cancel_term(a[st][mt]);
            }
#pragma unroll
          for (int t = 0; t < TN; ++t) {
            const u32x2 v = *reinterpret_cast<const u32x2*>(strip[t] + (K / 128) * 1024 + lane * 8);
            const uint32_t w[4] = {v.x, v.y, 0, 0};
            const float sc = GROUPED ? to_f32<DT>(load_scale_raw(step, t)) : 1.0f;
#pragma unroll
            for (int st = 0; st < 2; ++st) step_mfma(w + st * kDw, a[st], cc[st], 0, sc, t);
          }
        }
      }
    }

    // The epilogue's operands were requested first and have arrived by now;
    // naming them here keeps the compiler from sinking those loads (and the
    // reads of the kernel arguments) into the tail of the kernel.
#pragma unroll
    for (int t = 0; t < kEp; ++t) asm volatile("" ::"v"(ep_sraw[t]), "v"(ep_braw[t]));
    asm volatile("" ::"s"(out), "s"(out_f32));

#pragma unroll
    for (int t = 0; t < TN; ++t) {
      // Merge the classes: every lane keeps the class of its own lane group.
      f32x4 tot[MT];
      {
        const int mine = MP == 8 ? (kb >> 1) : kb;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          tot[mt] = totc[t][mt][0];
#pragma unroll
          for (int c = 1; c < kClasses; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) tot[mt][r] = mine == c ? totc[t][mt][c][r] : tot[mt][r];
        }
      }
      // Fold the kS row groups that carried the same output row: registers
      // first (MP < 4 keeps several row groups in one lane), then across the
      // lane groups.  Afterwards rows 0 .. MP-1 hold the wavefront's sums.
      if (MP == 1) {
        tot[0][0] = (tot[0][0] + tot[0][1]) + (tot[0][2] + tot[0][3]);
      } else if (MP == 2) {
        tot[0][0] += tot[0][2];
        tot[0][1] += tot[0][3];
      }
      if (MP <= 8) {
#pragma unroll
        for (int r = 0; r < kLive; ++r) tot[0][r] = sum_lane_groups(tot[0][r], MP <= 4, true);
      }
      // Meet in LDS: red[strip][wave][mt][r][lane], summed over wavefronts in order.
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < kLive; ++r)
          red[(((t * WK + wave_all) * MT + mt) * 4 + r) * 64 + lane] = tot[mt][r];
    }
    if (STAMP) st_c3 = __builtin_readcyclecounter();
    __syncthreads();
    if (STAMP) st_c4 = __builtin_readcyclecounter();
    auto leave_stamps = [&]() {
      if (STAMP && lane == 0 && stamps != nullptr) {
        unsigned long long* o = stamps + (static_cast<size_t>(blockIdx.x) * WK + wave_all) * 8;
        const unsigned long long c5 = __builtin_readcyclecounter();
        o[0] = st_rt0;                             // entry, constant-rate clock (100 MHz)
        o[1] = __builtin_amdgcn_s_memrealtime();   // end, the same clock
        o[2] = st_ca - st_c0;                      // entry until the kernel's arguments are in registers
        o[3] = st_c1 - st_ca;                      // addresses, every load issued
        o[4] = st_c2 - st_c1;                      // waiting for the loads
        o[5] = st_c3 - st_c2;                      // dequantisation, MFMAs, folding, sums into LDS
        o[6] = st_c4 - st_c3;                      // waiting for the workgroup's other wavefronts
        o[7] = c5 - st_c4;                         // adding the wavefronts' sums, scale, store
      }
    };
    const int rows = M < 16 * MT ? M : 16 * MT;
    if (SWI) {
      float ep_scale[2], ep_bias[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        ep_scale[h] = GROUPED ? 1.0f : to_f32<DT>(ep_sraw[h]);
        ep_bias[h] = bias != nullptr ? to_f32<DT>(ep_braw[h]) : 0.0f;
      }
      for (int idx = threadIdx.x; idx < rows * 16; idx += WK * 64) {
        const int m = idx / 16, nl = idx % 16;  // nl == j
        float v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float s = 0.0f;
#pragma unroll
          for (int w = 0; w < kWS; ++w) s += red[((h * kWS + w) * 4 + (m % 4)) * 64 + (m / 4) * 16 + nl];
          v[h] = s * ep_scale[h] + ep_bias[h];
        }
        const float s = act_swiglu(v[0], v[1]);
        const int64_t o = static_cast<int64_t>(m) * (N / 2) + bid * kStripCols + nl;
        if (out_f32)
          static_cast<float*>(out)[o] = s;
        else
          static_cast<uint16_t*>(out)[o] = cast_out<DT>(s);
      }
      return;
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      if (bid * TN + t >= nstrips) break;  // the repeated last strip
      const float ep_scale = GROUPED ? 1.0f : to_f32<DT>(ep_sraw[t]);
      const float ep_bias = bias != nullptr ? to_f32<DT>(ep_braw[t]) : 0.0f;
      for (int idx = threadIdx.x; idx < rows * 16; idx += WK * 64) {
        const int m = idx / 16, nl = idx % 16;  // nl == j: the stride of idx is a multiple of 16
        const int mt = m / 16, row = m % 16;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < WK; ++w)
          s += red[(((t * WK + w) * MT + mt) * 4 + (row % 4)) * 64 + (row / 4) * 16 + nl];
        s = act_apply(s * ep_scale + ep_bias, act);
        const int64_t o = static_cast<int64_t>(m) * N + n[t];
        if (out_f32)
          static_cast<float*>(out)[o] = s;
        else
          static_cast<uint16_t*>(out)[o] = cast_out<DT>(s);
      }
    }
    leave_stamps();
  }
};

template <int DT, int BITS, int MP, int MT, int WK, int NU, int TN, bool GROUPED, bool PRE, bool SWI>
__global__ __launch_bounds__(WK * 64) void stream_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ codes,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ scale, void* __restrict__ out,
    int M, int K, int N, int gshift, int out_f32, const uint16_t* __restrict__ pre, int act) {
  extern __shared__ float red[];
  StreamKernel<DT, BITS, MP, MT, WK, NU, TN, GROUPED, PRE, SWI> k;
  k.x = x;
  k.scale = scale;
  k.pre = pre;
  k.act = act;
  k.M = M;
  k.K = K;
  k.N = N;
  k.gshift = gshift;
  k.run(codes, bias, out, out_f32, red);
}

using Args = StreamArgs;

// The headline decode kernel (one row, int4, group-wise scales, 8 wavefronts, one unit each) with stamps.
template <int DT>
__global__ __launch_bounds__(512) void stream_phases_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ codes, const uint16_t* __restrict__ scale,
    void* __restrict__ out, int K, int N, int gshift, unsigned long long* __restrict__ stamps) {
  extern __shared__ float red[];
  StreamKernel<DT, 4, 1, 1, 8, 1, 1, true, false, false, true> k;
  k.x = x;
  k.scale = scale;
  k.pre = nullptr;
  k.stamps = stamps;
  k.act = WOL_ACT_NONE;
  k.M = 1;
  k.K = K;
  k.N = N;
  k.gshift = gshift;
  k.run(codes, nullptr, out, 0, red);
}

template <int DT, int BITS, int MP, int MT, int WK, int NU, int TN, bool SWI = false>
void launch_tn(const Args& a) {
  const size_t lds = static_cast<size_t>(TN) * WK * MT * 256 * sizeof(float);
  const dim3 grid(static_cast<unsigned>(SWI ? a.N / kStripCols / 2 : (a.N / kStripCols + TN - 1) / TN)), block(WK * 64);
  const uint16_t* x = static_cast<const uint16_t*>(a.x);
  const uint8_t* codes = static_cast<const uint8_t*>(a.codes);
  const uint16_t* bias = static_cast<const uint16_t*>(a.bias);
  const uint16_t* scale = static_cast<const uint16_t*>(a.scale);
  const uint16_t* pre = static_cast<const uint16_t*>(a.pre);
  if constexpr (MP == 1) {  // the fused activation scales exist for one row
    if (pre != nullptr) {
      if (a.gshift >= 0)
        stream_kernel<DT, BITS, MP, MT, WK, NU, TN, true, true, SWI><<<grid, block, lds, a.stream>>>(
            x, codes, bias, scale, a.out, a.M, a.K, a.N, a.gshift, a.out_f32, pre, a.act);
      else
        stream_kernel<DT, BITS, MP, MT, WK, NU, TN, false, true, SWI><<<grid, block, lds, a.stream>>>(
            x, codes, bias, scale, a.out, a.M, a.K, a.N, a.gshift, a.out_f32, pre, a.act);
      return;
    }
  }
  if (a.gshift >= 0)
    stream_kernel<DT, BITS, MP, MT, WK, NU, TN, true, false, SWI><<<grid, block, lds, a.stream>>>(
        x, codes, bias, scale, a.out, a.M, a.K, a.N, a.gshift, a.out_f32, nullptr, a.act);
  else
    stream_kernel<DT, BITS, MP, MT, WK, NU, TN, false, false, SWI><<<grid, block, lds, a.stream>>>(
        x, codes, bias, scale, a.out, a.M, a.K, a.N, a.gshift, a.out_f32, nullptr, a.act);
}

// Two strips per workgroup exist for the operand shapes whose activation
// traffic matters and whose registers allow it (8 to 16 rows).
template <int DT, int BITS, int MP, int MT, int WK, int NU>
void launch_one(const Args& a) {
  if constexpr (MP >= 8 && MT == 1) {
    if (a.tn == 2) {
      launch_tn<DT, BITS, MP, MT, WK, NU, 2>(a);
      return;
    }
  }
  launch_tn<DT, BITS, MP, MT, WK, NU, 1>(a);
}

// wk in {1,2,4,8,16}; nu == 1 selects the all-loads-at-once variant (exactly
// one unit per wavefront), anything else the walking variant.
template <int DT, int BITS, int MP, int MT>
void launch_wk(const Args& a, int wk, int nu) {
  constexpr int kMaxWk = MT <= 2 ? 16 : 8;  // LDS for the cross-wavefront sums
  if constexpr ((MP == 4 || MP == 8) && MT == 1) {
    // several units per wavefront, still all in flight at once (8 wavefronts)
    if (nu == 2) { launch_one<DT, BITS, MP, MT, 8, 2>(a); return; }
    if (nu == 4 && wk >= 16) { launch_one<DT, BITS, MP, MT, 16, 4>(a); return; }
    if (nu == 4) { launch_one<DT, BITS, MP, MT, 8, 4>(a); return; }
  }
  if (nu == 1) {
    if (wk >= 16 && kMaxWk == 16) launch_one<DT, BITS, MP, MT, kMaxWk, 1>(a);
    else if (wk >= 8) launch_one<DT, BITS, MP, MT, 8, 1>(a);
    else if (wk >= 4) launch_one<DT, BITS, MP, MT, 4, 1>(a);
    else if (wk >= 2) launch_one<DT, BITS, MP, MT, 2, 1>(a);
    else launch_one<DT, BITS, MP, MT, 1, 1>(a);
  } else {
    // 16 wavefronts (1024 threads) leave 128 registers each: enough for the
    // ring of units of 2 to 8 rows (and of one row of int4), not for the others
    if constexpr ((MP >= 2 && MP <= 8) || (MP == 1 && BITS == 4)) {
      if (wk >= 16) { launch_one<DT, BITS, MP, MT, 16, 0>(a); return; }
    }
    if (wk >= 8) launch_one<DT, BITS, MP, MT, 8, 0>(a);
    else if (wk >= 4) launch_one<DT, BITS, MP, MT, 4, 0>(a);
    else if (wk >= 2) launch_one<DT, BITS, MP, MT, 2, 0>(a);
    else launch_one<DT, BITS, MP, MT, 1, 0>(a);
  }
}

// The gate|up form: `total` wavefronts per workgroup, half of them per strip.
template <int DT, int BITS, int MP>
void launch_wk_swi(const Args& a, int total, int nu) {
  if constexpr (MP == 4 || MP == 8) {
    if (nu == 2) { launch_tn<DT, BITS, MP, 1, 16, 2, 1, true>(a); return; }
    if (nu == 4) { launch_tn<DT, BITS, MP, 1, 16, 4, 1, true>(a); return; }
  }
  if (nu == 1) {
    if (total >= 16) launch_tn<DT, BITS, MP, 1, 16, 1, 1, true>(a);
    else if (total >= 8) launch_tn<DT, BITS, MP, 1, 8, 1, 1, true>(a);
    else if (total >= 4) launch_tn<DT, BITS, MP, 1, 4, 1, 1, true>(a);
    else launch_tn<DT, BITS, MP, 1, 2, 1, 1, true>(a);
  } else {
    if constexpr ((MP >= 2 && MP <= 8) || (MP == 1 && BITS == 4)) {
      if (total >= 16) { launch_tn<DT, BITS, MP, 1, 16, 0, 1, true>(a); return; }
    }
    if (total >= 8) launch_tn<DT, BITS, MP, 1, 8, 0, 1, true>(a);
    else if (total >= 4) launch_tn<DT, BITS, MP, 1, 4, 0, 1, true>(a);
    else launch_tn<DT, BITS, MP, 1, 2, 0, 1, true>(a);
  }
}

template <int DT, int BITS>
void launch_m_swi(const Args& a, int total, int nu) {
  if (a.M <= 1) launch_wk_swi<DT, BITS, 1>(a, total, nu);
  else if (a.M <= 2) launch_wk_swi<DT, BITS, 2>(a, total, nu);
  else if (a.M <= 4) launch_wk_swi<DT, BITS, 4>(a, total, nu);
  else if (a.M <= 8) launch_wk_swi<DT, BITS, 8>(a, total, nu);
  else launch_wk_swi<DT, BITS, 16>(a, total, nu);
}

template <int DT, int BITS>
void launch_m(const Args& a, int wk, int nu) {
  if (a.M <= 1) launch_wk<DT, BITS, 1, 1>(a, wk, nu);
  else if (a.M <= 2) launch_wk<DT, BITS, 2, 1>(a, wk, nu);
  else if (a.M <= 4) launch_wk<DT, BITS, 4, 1>(a, wk, nu);
  else if (a.M <= 8) launch_wk<DT, BITS, 8, 1>(a, wk, nu);
  else if (a.M <= 16) launch_wk<DT, BITS, 16, 1>(a, wk, nu);
  else if (a.M <= 32) launch_wk<DT, BITS, 16, 2>(a, wk, nu);
  else if (a.M <= 48) launch_wk<DT, BITS, 16, 3>(a, wk, nu);
  else launch_wk<DT, BITS, 16, 4>(a, wk, nu);
}

}  // namespace

#if !defined(WOL_STREAM_F16_TU)
// bf16 activations, int4 codes with group-wise scales, K = 4096 (eight wavefronts with one unit of 512 k
// each, every load issued at once: the kernel wol_linear takes for the benchmark's headline shape).
int launch_decode_phases(const void* x, const void* codes, const void* scale, int64_t K, int64_t N, int group_size,
                         void* out, unsigned long long* stamps, hipStream_t stream) {
  if (K != 4096 || (group_size != 64 && group_size != 128) || N % kStripCols != 0) return WOL_ERR_BAD_SHAPE;
  const dim3 grid(static_cast<unsigned>(N / kStripCols)), block(512);
  const size_t lds = static_cast<size_t>(8) * 256 * sizeof(float);
  stream_phases_kernel<WOL_DTYPE_BF16><<<grid, block, lds, stream>>>(
      static_cast<const uint16_t*>(x), static_cast<const uint8_t*>(codes), static_cast<const uint16_t*>(scale), out,
      static_cast<int>(K), static_cast<int>(N), group_size == 64 ? 6 : 7, stamps);
  return check_launch();
}
#endif

#if defined(WOL_STREAM_F16_TU)
void launch_linear_stream_f16(const StreamArgs& a, int bits, bool swi, int wk, int nu) {
  if (swi) {
    if (bits == 8) launch_m_swi<WOL_DTYPE_F16, 8>(a, wk, nu); else launch_m_swi<WOL_DTYPE_F16, 4>(a, wk, nu);
  } else {
    if (bits == 8) launch_m<WOL_DTYPE_F16, 8>(a, wk, nu); else launch_m<WOL_DTYPE_F16, 4>(a, wk, nu);
  }
}
#else
// Work split.  A unit is kU k steps of one strip.  When the unit count per
// strip is a power of two up to 16, each wavefront takes exactly one unit and
// issues all its loads at once: with one or two rows whatever the number of
// strips (workgroups beyond the ~8 192 wavefronts the chip holds start as
// earlier ones end; measured against the walk at 896 to 2 560 strips, K = 4096
// and 8192: 6 to 12 % faster), with more rows while every wavefront is
// resident at once (~6 per SIMD on 1024 SIMDs).  With 3 to 8 rows and 16 or 32
// units per strip eight wavefronts take two or four units each, all loads
// again issued at once, at any number of strips (7 to 17 % faster than the
// walk from 1 024 strips on; with 64 units sixteen wavefronts take four each,
// up to 1 536 strips).  Otherwise wavefronts walk their units with up
// to three more in flight, and WK follows a budget of resident wavefronts that
// shrinks with the row count.
static void pick_split(int64_t M, int64_t K, int64_t N, int bits, int* wk, int* nu, int* tn) {
  int mp = 1;
  while (mp < 16 && mp < M) mp *= 2;
  *tn = stream_strips_per_workgroup(M, N, bits);
  const int64_t strips = (N / kStripCols + *tn - 1) / *tn;  // workgroups
  const int s = 16 / mp, spt = bits == 8 ? 2 : 4;
  const int ku = s > spt ? s : spt;
  const int64_t nsteps = K / 32, nunits = nsteps / ku;
  const int maxwk = M <= 32 ? 16 : 8;
  if (nunits * ku == nsteps && nunits <= maxwk && (nunits & (nunits - 1)) == 0 &&
      (mp <= 2 || strips * nunits <= 6144)) {
    *wk = static_cast<int>(nunits);
    *nu = 1;
    return;
  }
  // 3 to 8 rows: units are short (4 k steps), so a strip has many of them;
  // eight wavefronts with two or four units each still keep everything in flight
  if (mp >= 4 && mp <= 8 && nunits * ku == nsteps && (nunits == 16 || nunits == 32)) {
    *wk = 8;
    *nu = static_cast<int>(nunits / 8);
    return;
  }
  // 64 units per strip (K = 8192, and K = 4096 on int8 at 5 to 8 rows): sixteen
  // wavefronts with four units each, 5 to 11 % faster than the walk up to
  // 1 376 strips; at 1 792 the walk is faster
  if (mp >= 4 && mp <= 8 && nunits * ku == nsteps && nunits == 64 && strips <= 1536) {
    *wk = 16;
    *nu = 4;
    return;
  }
  // measured: one or two rows want up to ~8 wavefronts per SIMD, full 16-row
  // operands (more registers and LDS per wavefront) only one or two
  const int64_t budget = mp <= 2 ? 8192 : (mp <= 8 ? 4096 : 2048);
  int w = 1;
  const int maxwalk = (mp >= 2 && mp <= 8) || (mp == 1 && bits == 4) ? 16 : 8;
  // at least four units per wavefront, unless the strips leave CUs (256) with
  // one workgroup at most: then only a wider workgroup puts more wavefronts on a SIMD
  const int minu = strips <= 256 ? 1 : 4;
  while (w < maxwalk && strips * w * 2 <= budget && w * minu <= nunits) w *= 2;
  *wk = w;
  *nu = 0;
}

bool linear_stream_loads_at_once(int64_t M, int64_t K, int64_t N, int bits) {
  int wk = 1, nu = 0, tn = 1;
  pick_split(M, K, N, bits, &wk, &nu, &tn);
  return nu > 0;
}

void describe_linear_stream(int64_t M, int64_t K, int64_t N, int bits, int group_size, char* buf, size_t n) {
  int wk = 1, nu = 0, tn = 1;
  pick_split(M, K, N, bits, &wk, &nu, &tn);
  int mp = 1;
  while (mp < 16 && mp < M) mp *= 2;
  snprintf(buf, n, "wol::stream_kernel: %lld workgroups of %d wavefronts, %d strip(s) each, %d-row operands x %d, %s",
           static_cast<long long>((N / kStripCols + tn - 1) / tn), wk, tn, mp, static_cast<int>((M + 15) / 16),
           nu > 0 ? "all loads of a wavefront issued at once" : "wavefronts walk their units through a ring of loads");
  (void)group_size;
}

// Up to 16 rows of a gate|up projection (N a multiple of 32) leave the kernel as
// silu(gate) * up.
bool linear_stream_fuses_swiglu(int64_t M, int64_t N) { return M >= 1 && M <= 16 && N % 32 == 0; }

// f.pre_scale is honoured for one row only (the caller scales the activations
// itself otherwise); f.act may be none, gelu or -- where
// linear_stream_fuses_swiglu says so -- swiglu (out is then [M, N/2]).
int launch_linear_stream(const void* x, const void* codes, const void* bias, const void* scale,
                         int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                         void* out, bool out_f32, hipStream_t stream, const Fuse& f) {
  const int gshift = group_size == 64 ? 6 : (group_size == 128 ? 7 : -1);
  int wk = 1, nu = 0, tn = 1;
  pick_split(M, K, N, bits, &wk, &nu, &tn);
  const bool swi = f.act == WOL_ACT_SWIGLU;
  if (swi && !linear_stream_fuses_swiglu(M, N)) return WOL_ERR_BAD_SHAPE;
  const Args a{x, codes, bias, scale, out, static_cast<int>(M), static_cast<int>(K),
               static_cast<int>(N), gshift, out_f32 ? 1 : 0, tn, stream, M == 1 ? f.pre_scale : nullptr,
               swi ? WOL_ACT_NONE : f.act};
  if (swi) {
    // the split of one strip, twice in a workgroup; where that is more
    // wavefronts than a workgroup holds, the halves walk their units instead
    int mp = 1;
    while (mp < 16 && mp < M) mp *= 2;
    const int walk_max = (mp >= 2 && mp <= 8) || (mp == 1 && bits == 4) ? 16 : 8;
    int total = 2 * wk;
    if (nu == 1 && total > 16) nu = 0;
    if (nu == 4 && wk == 16) nu = 0;  // 64 units per strip: twice sixteen wavefronts
    if (nu == 2 || nu == 4) total = 16;
    if (nu == 0 && total > walk_max) total = walk_max;
    if (dtype == WOL_DTYPE_BF16) {
      if (bits == 8) launch_m_swi<WOL_DTYPE_BF16, 8>(a, total, nu); else launch_m_swi<WOL_DTYPE_BF16, 4>(a, total, nu);
    } else {
      launch_linear_stream_f16(a, bits, true, total, nu);
    }
    return check_launch();
  }
  if (dtype == WOL_DTYPE_BF16) {
    if (bits == 8) launch_m<WOL_DTYPE_BF16, 8>(a, wk, nu); else launch_m<WOL_DTYPE_BF16, 4>(a, wk, nu);
  } else {
    launch_linear_stream_f16(a, bits, false, wk, nu);
  }
  return check_launch();
}
#endif  // WOL_STREAM_F16_TU

}  // namespace wol
