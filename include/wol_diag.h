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
