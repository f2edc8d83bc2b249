/*
 * wol_c_api.h -- C ABI of the MI355X (gfx950) weight-only quantized linear
 * library (libwol_gfx950.so).
 *
 * These entry points are what Paddle's three PHI GPU kernels for this path
 * call once their bodies are replaced:
 *
 *   wol_quantize    <- phi::WeightQuantizeKernel<T, GPUContext>
 *                      paddle/phi/kernels/weight_quantize_kernel.h:21-28,
 *                      paddle/phi/kernels/gpu/weight_quantize_kernel.cu:25-115
 *                      (arithmetic: the CPU kernel's,
 *                      paddle/phi/kernels/impl/weight_quantize_kernel_impl.h:45-183)
 *   wol_dequantize  <- phi::WeightDequantizeKernel<T, GPUContext>
 *                      paddle/phi/kernels/weight_dequantize_kernel.h:21-28,
 *                      paddle/phi/kernels/gpu/weight_dequantize_kernel.cu:440-475
 *   wol_linear      <- phi::WeightOnlyLinearKernel<T, GPUContext>
 *                      paddle/phi/kernels/weight_only_linear_kernel.h:21-30,
 *                      paddle/phi/kernels/gpu/weight_only_linear_kernel.cu:26-201
 *
 * Conventions
 *   - Plain pointers and sizes only.  Every pointer is DEVICE memory owned by
 *     the caller; the library never allocates, frees or synchronises.  All
 *     work is enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     null stream), the way the reference enqueues on dev_ctx.stream().
 *   - K = in_features, N = out_features, M = tokens (x.numel() / K).
 *   - dtype is the activation / scale / bias / output type T.
 *   - Every function returns a wol_status; 0 is success.  Nothing throws.
 *     Argument errors mirror the reference's InferMeta checks
 *     (paddle/phi/infermeta/unary.cc:5946-6011, binary.cc:4499-4570,
 *     multiary.cc:5495-5575); the PHI glue turns a non-zero status into
 *     PADDLE_THROW(InvalidArgument / External).
 *   - Thread-safe and re-entrant: no mutable global state.
 *   - WOL_LOG=1 in the environment makes wol_linear, wol_linear_fused and
 *     wol_linear_grad write one line per call to stderr (the problem and the
 *     kernel taken), the way the reference's VLOG lines name the GEMV/GEMM
 *     branch (gpu/weight_only_linear_kernel.cu:60-200).  Read once per process.
 *   - WOL_ROCTX=1 in the environment wraps every compute call in a roctx
 *     range named after its entry point (for rocprofv3 --marker-trace); the
 *     marker library is looked up with dlopen, there is no link dependency.
 *     Read once per process.
 */
#ifndef WOL_C_API_H_
#define WOL_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* T: the two types the reference registers (gpu/weight_quantize_kernel.cu:118-123). */
#define WOL_DTYPE_F16 0
#define WOL_DTYPE_BF16 1

/* float -> T flavour used for the SCALE (the codes are computed against the
 * rounded scale, impl/weight_quantize_kernel_impl.h:55,92-94).
 * RNE   : bf16 of CPU/CUDA builds (paddle/phi/common/bfloat16.h:61-88), fp16 of
 *         F16C and device builds (paddle/phi/common/float16.h:107-119).
 * TRUNC : bf16 of HIP builds (bfloat16.h:103-110), fp16 of a host build
 *         without F16C (float16.h:121-139). */
#define WOL_ROUND_RNE 0
#define WOL_ROUND_TRUNC 1

/* Weight tensor layouts.  All hold the same K*N*bits/8 bytes.
 * CANONICAL  : the reference's codes before any layout step: [K,N] int8, or
 *              [K,N/2] bytes with column 2j in the low nibble (two's
 *              complement nibbles) -- the x_int buffer of
 *              paddle/phi/kernels/cpu/weight_quantize_kernel.cc:95-107.
 * PADDLE_HIP : what a PADDLE_WITH_HIP build returns (:113-125): CANONICAL
 *              transposed bytewise to [N,K] / [N/2,K], int4 nibbles stored +8.
 * GFX950     : this library's streaming layout (see wol_layout_version). */
#define WOL_LAYOUT_CANONICAL 0
#define WOL_LAYOUT_PADDLE_HIP 1
#define WOL_LAYOUT_GFX950 2

typedef enum wol_status {
  WOL_OK = 0,
  WOL_ERR_NULL_POINTER = 1,   /* a required pointer is NULL                     */
  WOL_ERR_BAD_DTYPE = 2,      /* dtype not F16/BF16                             */
  WOL_ERR_BAD_BITS = 3,       /* bits not 8/4 (weight_dtype not int8/int4)      */
  WOL_ERR_BAD_GROUP_SIZE = 4, /* group_size not -1/64/128                       */
  WOL_ERR_BAD_SHAPE = 5,      /* K % 64, N % 16, M < 0, a size above 2^24, ...   */
  WOL_ERR_BAD_LAYOUT = 6,     /* unknown layout id                              */
  WOL_ERR_BAD_ROUND_MODE = 7,
  WOL_ERR_WORKSPACE = 8,      /* workspace NULL or smaller than the query says  */
  WOL_ERR_ALIGNMENT = 9,      /* a pointer is not 16-byte aligned               */
  WOL_ERR_HIP = 10,           /* a HIP launch failed; see hipGetLastError       */
  WOL_ERR_NO_DEVICE = 11      /* valid arguments, but the current device is not
                                 a gfx950 (checked once per device)             */
} wol_status;

/* Human-readable text for a status (static storage). */
const char* wol_status_str(int status);

/* Version tag of the GFX950 layout.  A checkpoint that stores packed weights
 * should store this beside them; a different value means "repack". */
int wol_layout_version(void);

/* Bytes of device scratch wol_quantize needs (per-channel abs-max uses an
 * fp32 [N] buffer; group-wise needs none).  Returns 0 for invalid arguments. */
size_t wol_quantize_workspace(int64_t K, int64_t N, int bits, int group_size);

/*
 * weight_quantize.  w: [K,N] T row-major.  Computes, bit-exactly as the
 * reference's CPU kernel does,
 *     scale[gk,n] = cast_T( max_k |w[k,n]| / bound ),  bound = 127 | 7
 *     code[k,n]   = clip( round_half_away( float(w) / float(scale) ) )
 * and writes the codes in `layout` (GFX950 for wol_linear) into codes_out
 * (K*N*bits/8 bytes; reported to Paddle as [N,K] int8 or [N/2,K] int8,
 * paddle/phi/infermeta/unary.cc:5994-6005) and scale_out ([N] or
 * [ceil(K/g),N] T, :5985-5992).
 * Requires K % 64 == 0, N % 16 == 0, group_size in {-1,64,128}.
 */
int wol_quantize(const void* w, int dtype, int64_t K, int64_t N, int bits,
                 int group_size, int round_mode, int layout, void* codes_out,
                 void* scale_out, void* workspace, size_t workspace_bytes,
                 void* stream);

/*
 * wol_quantize for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same arithmetic, arguments and
 * results as wol_quantize, but without the workspace: the per-channel abs-max
 * buffer is a static device array inside the library (256 KiB on every GPU
 * the library runs on, held until the process ends), so per-channel
 * quantisation (group_size -1) is limited to N <= 65536 and returns
 * WOL_ERR_BAD_SHAPE beyond that; group-wise quantisation uses no scratch and
 * has no extra limit.  The call allocates and frees nothing.  All calls on one
 * GPU share that GPU's array: per-channel calls that overlap on one GPU (two
 * streams, two threads) race and must be serialised by the caller.
 * The first call on a device looks up that device's properties and the
 * address of its copy of the array; make one call outside of any stream
 * capture (any size) before capturing calls on that device.
 */
int wol_quantize_static(const void* w, int dtype, int64_t K, int64_t N, int bits,
                        int group_size, int round_mode, int layout,
                        void* codes_out, void* scale_out, void* stream);

/*
 * weight_quantize with algo = "llm.int8" (cpu/weight_quantize_kernel.cc:163-166,
 * quant_compute<..., int8_t, 8, float>): int8 codes computed against the
 * unrounded fp32 scale amax/127, which is also what is returned.
 * scale_out: [N] or [ceil(K/g), N] float.  The reference returns the codes as
 * [N,K] (a plain byte transpose, :108-111): that is WOL_LAYOUT_PADDLE_HIP.
 * These tensors feed llm_int8_linear, not wol_linear (whose scales are T).
 * Workspace as for wol_quantize with bits = 8.
 */
int wol_quantize_llm_int8(const void* w, int dtype, int64_t K, int64_t N,
                          int group_size, int layout, void* codes_out,
                          float* scale_out, void* workspace,
                          size_t workspace_bytes, void* stream);

/*
 * weight_dequantize.  out_KN[k,n] = cast_T( float(code[k,n]) * float(scale) ),
 * written directly as [K,N] row-major T (the reference writes [N,K] and then
 * transposes, gpu/weight_dequantize_kernel.cu:464-470).  `layout` names the
 * layout of `codes`.  The final cast is round-to-nearest-even.
 */
int wol_dequantize(const void* codes, int layout, const void* scale, int dtype,
                   int64_t K, int64_t N, int bits, int group_size,
                   void* out_KN, void* stream);

/* Bytes of device scratch wol_linear can use for this problem (may be 0).  The
 * scratch is optional: without it (NULL or fewer bytes) the result is the
 * same to fp32 summation order and only the speed of small-M problems drops,
 * because K can no longer be split across workgroups.  Must be 16-byte aligned.
 * wol_linear takes the same kernel with exactly this many bytes as with any
 * larger buffer. */
size_t wol_linear_workspace(int64_t M, int64_t K, int64_t N, int bits,
                            int group_size);

/*
 * weight_only_linear.  out[M,N] = x[M,K] . dequant(W)[K,N] (+ bias[N]),
 * fp32 accumulation, one round-to-nearest-even cast to T at the end.
 * codes must be in GFX950 layout.  bias may be NULL.
 * scale: [N] T (group_size -1) or [ceil(K/g),N] T, as wol_quantize wrote it.
 * M <= 16 takes a decode (HBM-bound) kernel -- the batched one, which fetches
 * the activations once per workgroup, where it applies (2 to 16 rows, K =
 * 2048/4096/8192, at least 2.5 16-column strips per CU), else the streaming
 * one --, M > 64 the MFMA GEMM, and in between the streaming kernel or the
 * GEMM, whichever a cost model predicts to be faster.  Where the workspace
 * allows and it is measured faster (10 to 32 rows on some shapes), the
 * batched kernel with K cut into runs across workgroups runs instead.  The
 * reference's split is M <= 3 (gpu/weight_only_linear_kernel.cu:60-61).
 * code * scale is never rounded to T in any kernel (the reference's GEMM
 * rounds the scaled weight to T, cutlass_extensions/gemm/warp/
 * mma_tensorop_dequantizer.h:155-195): per-channel scales multiply the fp32
 * sums; group-wise scales multiply each group's fp32 sum up to 64 rows, and
 * above 64 rows the running sums are kept in units of the current group's
 * scale and rescaled from group to group (one fp32 rounding of the sums per
 * group; a column's unit never falls more than 2^64 below its largest scale,
 * so no ratio of scales overflows).
 * x, codes, scale, out and (when given) bias must be 16-byte aligned: the
 * kernels read and write 16 bytes at a time, the output rows included
 * (WOL_ERR_ALIGNMENT otherwise).
 */
int wol_linear(const void* x, const void* codes, const void* bias,
               const void* scale, int dtype, int64_t M, int64_t K, int64_t N,
               int bits, int group_size, void* out, void* workspace,
               size_t workspace_bytes, void* stream);

/* Same as wol_linear but writes the fp32 accumulators (plus bias) instead of
 * casting to T: out_f32 is [M,N] float.  Used to check the arithmetic without
 * the final rounding. */
int wol_linear_f32(const void* x, const void* codes, const void* bias,
                   const void* scale, int dtype, int64_t M, int64_t K,
                   int64_t N, int bits, int group_size, float* out_f32,
                   void* workspace, size_t workspace_bytes, void* stream);

/* Activation fused behind the linear by wol_linear_fused.  The reference's
 * GEMV takes act_method "None" or "gelu"
 * (paddle/phi/kernels/funcs/weight_only_gemv.h:33, gelu formula
 * funcs/weight_only_gemv.cu:147-157, applied to accumulator + bias in float,
 * :1045-1046); swiglu is what its MoE FFN runs on the output of the first
 * linear (paddle/phi/kernels/fusion/cutlass/moe_ffn.cu:133-139). */
#define WOL_ACT_NONE 0
#define WOL_ACT_GELU 1   /* v * 0.5 * (1 + tanh(0.7978845608 * (v + 0.044715 v^3)))      */
#define WOL_ACT_SWIGLU 2 /* out[m, n] = silu(v[m, n]) * v[m, n + N/2], n < N/2: out is
                            [M, N/2]; needs N % 32 == 0                                */

/*
 * weight_only_linear with what usually stands on either side of it folded in:
 *   x' = T(x * pre_scale)            apply_per_channel_scale, when pre_scale != NULL
 *                                    (paddle/phi/kernels/gpu/apply_per_channel_scale_kernel.cu:93-126:
 *                                    each product rounded once to T, bit for bit
 *                                    what wol_apply_per_channel_scale writes)
 *   v  = x' . dequant(W) + bias      fp32 accumulation, as wol_linear
 *   out = T(act(v))                  act applied to the fp32 sum, one rounding
 * pre_scale: [K] T.  out: [M, N] T, or [M, N/2] T for WOL_ACT_SWIGLU.
 * The decode kernels (up to 16 rows) apply pre_scale while they load the
 * activations and gelu or swiglu in their epilogues (with K cut into runs: in
 * the kernel that adds the runs); the MFMA GEMM applies gelu in its epilogue,
 * swiglu too with per-channel scales above 64 rows, and takes pre-scaled
 * activations -- and the swiglu of its other forms -- through the workspace
 * (one element-wise pass each, inside this call).  The workspace is therefore
 * required whenever wol_linear_fused_workspace() is non-zero.
 */
size_t wol_linear_fused_workspace(int64_t M, int64_t K, int64_t N, int bits,
                                  int group_size, int has_pre_scale, int act);
int wol_linear_fused(const void* x, const void* pre_scale, const void* codes,
                     const void* bias, const void* scale, int dtype, int64_t M,
                     int64_t K, int64_t N, int bits, int group_size, int act,
                     void* out, void* workspace, size_t workspace_bytes,
                     void* stream);

/*
 * Replaces WeightOnlyLinearGradKernel<T, GPUContext>
 * (paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu:27-72; op
 * paddle/phi/ops/yaml/backward.yaml:3651-3661): the only gradient of
 * weight_only_linear,
 *   x_grad[M, K] = out_grad[M, N] . dequant(W)[K, N]^T.
 * The reference dequantises the whole weight to T and calls a library GEMM
 * (per-channel scales only, :38-49).  Here one MFMA kernel contracts over n
 * straight from the packed codes, for every group size; code * scale is
 * rounded once to 11 significant bits (fp16 operands for both T, powers of two
 * taken out per column and per row and put back exactly), never to T, and
 * the sums are kept in fp32.  No bias and no activations are involved (x is
 * no_need_buffer in the reference).
 * codes: GFX950 layout.  scale: as for wol_linear.  The workspace holds the
 * scaled out_grad and scales (and, for M <= 512 or so, the sums of the runs N
 * is cut into); wol_linear_grad_workspace() bytes are required.  out_grad,
 * codes, scale, x_grad and the workspace must be 16-byte aligned.
 */
size_t wol_linear_grad_workspace(int64_t M, int64_t K, int64_t N, int bits,
                                 int group_size);
int wol_linear_grad(const void* out_grad, const void* codes, const void* scale,
                    int dtype, int64_t M, int64_t K, int64_t N, int bits,
                    int group_size, void* x_grad, void* workspace,
                    size_t workspace_bytes, void* stream);

/* Same as wol_linear_grad but writes the fp32 sums (times 2^-e[m]) instead of
 * casting to T: x_grad_f32 is [M,K] float.  Used to check the arithmetic
 * without the final rounding. */
int wol_linear_grad_f32(const void* out_grad, const void* codes,
                        const void* scale, int dtype, int64_t M, int64_t K,
                        int64_t N, int bits, int group_size, float* x_grad_f32,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * Replaces MoeFFNKernel<T, GPUContext> for quant_method "weight_only_int8" /
 * "weight_only_int4" (paddle/phi/kernels/fusion/cutlass/moe_ffn.cu:36-183,
 * whose CUTLASS grouped GEMMs :74-154 have no ROCm build): the expert FFN of a
 * mixture-of-experts layer on tokens already permuted into expert order,
 *   fc1  = permute_input . dequant(ffn1_weight[e]) + ffn1_bias[e]     [rows, inter]  T
 *   act  = T( silu(fc1[:, :inter/2]) * fc1[:, inter/2:] )            [rows, inter/2] (swiglu, :133-139)
 *   out  = act . dequant(ffn2_weight[e])                              [rows, hidden] T
 * where e is the expert of the row.  token_nums_per_expert: [num_experts]
 * int64 on the device, holding what the reference's moe_dispatch writes there
 * -- the running total of rows up to and including each expert
 * (fusion/cutlass/moe_dispatch.cu:174-182, moe/fused_moe_op.h:896-908), so
 * expert e owns rows [t[e-1], t[e]) and t[num_experts-1] <= rows.  It is read
 * on the device only: nothing returns to the host.
 * Weights: num_experts consecutive tensors as wol_quantize writes them
 * (GFX950 layout, per-channel scales): ffn1_weight [E] x (K = hidden,
 * N = inter), ffn1_scale [E, inter] T, ffn1_bias [E, inter] T or NULL,
 * ffn2_weight [E] x (K = inter/2, N = hidden), ffn2_scale [E, hidden] T.
 * Each of the two products is ONE grouped launch (tiles looked up in a
 * row-tile table that a one-workgroup kernel derives from
 * token_nums_per_expert: 128 x 256, or 64 x 256 / 32 x 256 when rows /
 * num_experts is at most 64 / 32, in which case the second product may run
 * with K cut into runs and a kernel that adds them); the swiglu between them
 * is an element-wise pass.
 * Requires hidden % 128 == 0, inter % 256 == 0, num_experts <= 1024; the
 * workspace (wol_moe_ffn_workspace bytes, 16-byte aligned) holds the table,
 * the two intermediate tensors and the runs' sums.
 */
size_t wol_moe_ffn_workspace(int64_t rows, int64_t hidden, int64_t inter,
                             int num_experts);
int wol_moe_ffn(const void* permute_input, const int64_t* token_nums_per_expert,
                const void* ffn1_weight, const void* ffn1_bias,
                const void* ffn1_scale, const void* ffn2_weight,
                const void* ffn2_scale, int dtype, int64_t rows, int64_t hidden,
                int64_t inter, int num_experts, int bits, void* ffn_out,
                void* workspace, size_t workspace_bytes, void* stream);

/* Kernel choice of wol_linear_on. */
enum wol_kernel {
  WOL_KERNEL_AUTO = 0,   /* what wol_linear does                                */
  WOL_KERNEL_STREAM = 1, /* the streaming kernel (a workgroup per 16 columns);
                            M <= 64 only                                        */
  WOL_KERNEL_GEMM = 2,   /* the MFMA GEMM                                       */
  WOL_KERNEL_BATCH = 3,  /* the batched decode kernel (a workgroup per CU, the
                            activations fetched once per workgroup); M <= 16
                            and K = 2048 or 4096 (8192 for int4 with group_size
                            -1 or 128) only                                     */
  WOL_KERNEL_BATCH_SPLIT = 4 /* the same kernel with K cut into runs across
                            workgroups, the runs' sums added by a second
                            kernel; M <= 32, K at least 16 whole weight tiles
                            (128 k for int4, 64 k for int8); needs the
                            workspace wol_linear_workspace_for reports        */
};

/*
 * wol_linear / wol_linear_f32 with the kernel choice pinned: out is [M,N] T
 * (out_is_f32 == 0) or float.  No counterpart in the reference; it exists so
 * that both kernels can be timed and verified on the same problem.
 * wol_linear_workspace_for is the matching scratch query.
 */
size_t wol_linear_workspace_for(int64_t M, int64_t K, int64_t N, int bits,
                                int group_size, int kernel);
int wol_linear_on(const void* x, const void* codes, const void* bias,
                  const void* scale, int dtype, int64_t M, int64_t K, int64_t N,
                  int bits, int group_size, void* out, int out_is_f32,
                  int kernel, void* workspace, size_t workspace_bytes,
                  void* stream);

/*
 * Re-lays a code tensor between layouts (any pair of the three).  It is a
 * pure, invertible permutation (plus the documented nibble/byte bias of the
 * target layout), which is what makes the packed weights checkpointable and
 * comparable with the reference's codes.
 */
int wol_repack(const void* codes_in, int layout_in, void* codes_out,
               int layout_out, int64_t K, int64_t N, int bits, void* stream);

/*
 * wol_repack on HOST memory (no device work, no stream): the same re-layout
 * done by the calling thread.  It is what a CPU weight_quantize kernel calls to
 * hand out GFX950 weights -- the reference's CPU kernel ends in a layout step
 * of its own (a byte transpose on HIP builds,
 * paddle/phi/kernels/cpu/weight_quantize_kernel.cc:113-125) which this call
 * replaces with layout_in = WOL_LAYOUT_CANONICAL, layout_out = WOL_LAYOUT_GFX950
 * -- and what a loader uses for checkpoints that hold the reference's layout.
 * codes_in and codes_out must not overlap.
 */
int wol_repack_host(const void* codes_in, int layout_in, void* codes_out,
                    int layout_out, int64_t K, int64_t N, int bits);

/*
 * Host-side index helper (no device work): byte offset of element (k, n) in a
 * code tensor of the given layout, and through *nibble_shift which nibble of
 * that byte holds it (0 or 4; always 0 for int8).  Returns -1 for arguments
 * outside the contract.  For tools that read or write packed checkpoints; it
 * has no counterpart in the reference, whose layouts are implicit in its
 * kernels (paddle/phi/kernels/impl/weight_quantize_kernel_impl.h:185-441).
 */
int64_t wol_code_offset(int layout, int64_t K, int64_t N, int bits, int64_t k,
                        int64_t n, int* nibble_shift);

/*
 * Replaces ApplyPerChannelScaleKernel<T, GPUContext>
 * (paddle/phi/kernels/gpu/apply_per_channel_scale_kernel.cu:146-190, device
 * kernel :93-126; shape contract ApplyPerChannelScaleInferMeta,
 * paddle/phi/infermeta/binary.cc:3452-3481): the pre-quant smoothing of the
 * activations in front of weight_only_linear,
 *   out[r, c] = T( x[r, c] * scales[c] ),  one multiply rounded once (RNE).
 * x and out are [rows, cols] T row-major, scales is [cols] T; out may be x.
 * Any cols; rows and cols at most 2^24.  16-byte accesses are used when cols
 * is a multiple of 8 and the three pointers are 16-byte aligned (the file it
 * replaces supports only that case).  A NaN product is a NaN of unspecified
 * payload.
 */
int wol_apply_per_channel_scale(const void* x, const void* scales, int dtype,
                                int64_t rows, int64_t cols, void* out,
                                void* stream);

/*
 * Replaces LLMInt8LinearKernel<T, GPUContext>
 * (paddle/phi/kernels/gpu/llm_int8_linear_kernel.cu:29-79, the stages of
 * paddle/phi/kernels/impl/llm_int8_matmul_kernel_impl.h:560-690; shape
 * contract LLMInt8LinearInferMeta, paddle/phi/infermeta/multiary.cc:3792-3837).
 *   x [M,K] T; weight [N,K] int8 and weight_scale [N] float as
 *   weight_quantize(algo="llm.int8") returns them (wol_quantize_llm_int8 with
 *   WOL_LAYOUT_PADDLE_HIP, group_size -1); bias [N] T or NULL; out [M,N] T.
 *   Column k is an outlier when any |x[m,k]| > T(threshold).
 *   range[m]  = max_k |x[m,k]| over the elements not above the threshold
 *   qx[m,k]   = 0 in outlier columns, else clip(round(x * 127 * (1 / range[m])), -127, 127)
 *   acc[m,n]  = sum_k qx[m,k] * weight[n,k]                         (int32, exact)
 *   sub[m,n]  = T( sum over outlier k, ascending, of x[m,k] * T(weight[n,k] * weight_scale[n]) )  (fp32 sum)
 *   out[m,n]  = T( sub + T(acc * range[m] * weight_scale[n] / 127) ), then T(out + bias[n])
 * The reference reads the weight of the outlier columns through the index
 * permutation of another layout (impl/llm_int8_matmul_kernel_impl.h:351-362)
 * than the one its quantiser writes; this library indexes weight[n,k] plainly,
 * as the operator's description and the reference's own test
 * (test/quantization/test_llm_int8_linear.py:84-111) have it.
 * Requires K % 64 == 0, K <= 131072 and N % 16 == 0 (what weight_quantize
 * accepts; beyond K = 133152 the int32 sums of 127 * 127 products could wrap,
 * which the reference's int32 GEMM does silently); x,
 * weight, weight_scale, out and workspace 16-byte aligned; out must not
 * overlap an input (with many outlier columns their product waits in out
 * until it is merged).  The workspace is
 * required (wol_llm_int8_linear_workspace bytes); it holds the row ranges,
 * the outlier mask and list, the activation codes and, for few rows, the int32
 * sums of the runs K is cut into.  Nothing returns to the host: the reference's device-to-host copy of
 * the outlier count has no counterpart here.
 */
size_t wol_llm_int8_linear_workspace(int64_t M, int64_t K, int64_t N);
int wol_llm_int8_linear(const void* x, const void* weight, const void* bias,
                        const float* weight_scale, float threshold, int dtype,
                        int64_t M, int64_t K, int64_t N, void* out,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Where the intermediate results of wol_llm_int8_linear lie in its workspace
 * after a call, as byte offsets: [0] range (float [M]), [1] outlier mask
 * (bit k % 32 of int32 word k / 32), [2] outlier count (int32), [3] outlier
 * columns (int32, ascending), [4] activation codes (int8 [M,K]), [5] int32
 * sums, one [M,N] slab per K run, or -1 when the GEMM writes the output
 * itself; [6] is the number of K runs (not an offset).  offsets has room for
 * seven values.  For tests that compare the stages with the reference's; no
 * counterpart there. */
int wol_llm_int8_linear_stage_offsets(int64_t M, int64_t K, int64_t N,
                                      int64_t* offsets);

#ifdef __cplusplus
}
#endif
#endif /* WOL_C_API_H_ */
