/*
 * wol_diag.h -- measurement aids exported by libwol_gfx950.so.  None of them
 * has a counterpart in the reference and none is part of the operator
 * boundary (that is wol_c_api.h): they exist so that a benchmark can time the
 * machine's own ceilings beside the kernels, in the same process and on the
 * same buffers.  Same conventions as wol_c_api.h: device pointers owned by
 * the caller, work enqueued on `stream`, a wol_status returned.
 */
#ifndef WOL_DIAG_H_
#define WOL_DIAG_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Reads a GFX950-layout
 * weight with the launch shape of the one-row decode kernel (one workgroup of
 * eight wavefronts per 16-column strip, 16-byte non-temporal loads, all of a
 * wavefront's loads requested at once) and computes nothing.  Its duration is
 * the floor a decode call of that shape has on the machine at hand; bench.py
 * reports it beside the decode time.  out receives N/16*8 uint32 (an XOR of
 * what each wavefront read).  K*bits/8*16 must be a multiple of 8 KiB.
 */
int wol_read_floor(const void* codes, int64_t K, int64_t N, int bits, void* out,
                   void* stream);

/*
 * A register-only loop of v_mfma_f32_32x32x16_bf16 on the caller's operands:
 * every wavefront of a grid that fills the chip (one workgroup of 8
 * wavefronts per CU slot, `workgroups` of them) loads 2 x 4 operand fragments
 * from `operands` (at least 8 KiB of bf16 data; use random values, the clock
 * follows the switching activity of the data) once and then issues
 * `iters` x 8 MFMAs into eight independent accumulator blocks, with no memory
 * traffic inside the loop.  out receives one float per thread (keeps the
 * accumulators alive).  The launch performs
 *     workgroups * 8 * iters * 8 * 2 * 32 * 32 * 16   floating-point operations;
 * divided by its duration this is the rate the matrix pipes sustain on the
 * machine at hand with nothing else in their way -- the ceiling a GEMM kernel
 * is measured against beside the published peak.
 */
int wol_mfma_ceiling(const void* operands, int workgroups, int iters, float* out,
                     void* stream);

/*
 * The inner loop of the prefill GEMM's 256 x 256 tile with its ingredients
 * switched on one at a time, for a bottom-up account of where the matrix
 * pipes' time goes: same register tile (4 x 2 blocks of 32 x 32 per
 * wavefront, 8 wavefronts per workgroup, one workgroup per CU), same
 * instruction mix per k tile, no global traffic unless the variant says so.
 *   0  MFMAs only (what wol_mfma_ceiling measures)
 *   1  + the int8 -> bf16 dequantisation of two B fragments per slice
 *   2  + four A fragments read from LDS per slice
 *   3  + both
 *   4  + both and one workgroup barrier per k tile
 *   5  + both, the barrier and six direct-to-LDS loads (1 KiB each) per
 *        wavefront and k tile
 *   6  MFMAs, the barrier and the loads only
 *   7  v_mfma_f32_16x16x32 on 8 x 4 blocks, MFMAs only
 *   8  the same with dequantisation, A reads and barrier
 * operands: random bf16 data, at least WOL_MFMA_PROBE_OPERAND_BYTES of it
 * (operand_bytes says how much).  A launch performs
 *     workgroups * 8 * iters * 1048576 floating-point operations.
 * out receives one float per thread (workgroups * 512).
 */
#define WOL_MFMA_PROBE_VARIANTS 9
#define WOL_MFMA_PROBE_OPERAND_BYTES (64 * 8 * 49152 + 65536)
int wol_mfma_probe(int variant, const void* operands, size_t operand_bytes,
                   int workgroups, int iters, float* out, void* stream);

/*
 * Where the wavefronts of the decode GEMV spend their time: runs the kernel
 * wol_linear takes for one row of bf16 activations on int4 codes with
 * group-wise scales at K = 4096 (the benchmark's headline shape: a workgroup
 * of 8 wavefronts per 16-column strip, every load of a wavefront issued at
 * once) on an instantiation that reads the clocks as it goes.  out: [1, N]
 * bf16, bit for bit what wol_linear writes.  phases: for workgroup w (of
 * N / 16) and wavefront v (of 8), eight 64-bit values at
 * phases[(w * 8 + v) * 8 ...]:
 *   0  entry, 1  end: the constant-rate clock (100 MHz, common to the device)
 *   2  entry until the kernel's arguments are in registers, shader cycles
 *   3  addresses, every load issued
 *   4  waiting until every load has landed (an explicit wait the product
 *      kernel does not have: it starts on the first tile as it arrives)
 *   5  dequantisation, MFMAs, folding, partial sums into LDS
 *   6  waiting at the workgroup barrier
 *   7  adding the wavefronts' sums, scale, store
 * Values 2 to 7 add up to the wavefront's life in shader cycles.
 */
#define WOL_DECODE_PHASES_PER_WORKGROUP 64 /* values: 8 wavefronts x 8 */
int wol_decode_phases(const void* x, const void* codes, const void* scale,
                      int64_t K, int64_t N, int group_size, void* out,
                      unsigned long long* phases, size_t phases_bytes,
                      void* stream);

/*
 * Where the wavefronts of the prefill GEMM spend their cycles: runs the
 * 256 x 256 launch of wol_linear (bf16 activations, int8 codes with
 * per-channel scales, GFX950 layout; M and N multiples of 256, K a multiple
 * of 64 and at least 192; no bias) on an instantiation of the same kernel that
 * reads the shader's cycle counter at kernel entry, around the two waits of
 * every k tile and around the epilogue.  out: [M, N] bf16, bit for bit what
 * wol_linear writes.  phases: for workgroup w (of (M / 256) * (N / 256)) and
 * wavefront v (of 8), eight 64-bit counts at phases[(w * 8 + v) * 8 ...]:
 *   0  kernel entry to the first k tile's barrier (addresses, first loads)
 *   1  between the barriers of the k loop: MFMAs and whatever is issued among
 *      them (fragment reads, dequantisation, tile loads) and stalls on it
 *   2  waiting for this wavefront's own direct-to-LDS loads of the next tile
 *   3  waiting at the workgroup barrier for the other wavefronts
 *   4  the last tile's tail and the closing barrier
 *   5  epilogue (scale, cast, store)
 *   6  entry to end
 *   7  k tiles (K / 64)
 * Every stamp costs a scalar memory round trip (three per k tile), so the
 * stamped kernel runs a few per cent longer than the product's.
 */
#define WOL_PREFILL_PHASES_PER_WORKGROUP 64 /* counts: 8 wavefronts x 8 */
int wol_prefill_phases(const void* x, const void* codes, const void* scale,
                       int64_t M, int64_t K, int64_t N, void* out,
                       unsigned long long* phases, size_t phases_bytes,
                       void* stream);

/*
 * Writes into buf (NUL-terminated, at most buf_bytes) one line naming the
 * kernel and launch shape wol_linear takes for a problem when it is handed
 * workspace_bytes of scratch.  No device work.  For benchmarks and dispatch
 * tests.
 */
int wol_linear_plan(int64_t M, int64_t K, int64_t N, int bits, int group_size,
                    size_t workspace_bytes, char* buf, size_t buf_bytes);

/* The same for wol_linear_grad: the tile of its MFMA kernel. */
int wol_linear_grad_plan(int64_t M, int64_t K, int64_t N, char* buf,
                         size_t buf_bytes);

#ifdef __cplusplus
}
#endif
#endif /* WOL_DIAG_H_ */
