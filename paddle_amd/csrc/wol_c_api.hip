// extern "C" entry points of libwol_gfx950.so: argument validation (the
// shape/dtype contract of the reference's InferMeta functions), kernel
// selection, nothing else.  See include/wol_c_api.h for the contract.
#include <atomic>
#include <cstring>

#include <dlfcn.h>
#include <stdlib.h>

#include "wol_common.h"
#include "wol_diag.h"

namespace {

// WOL_OK when the current device is a gfx950, WOL_ERR_NO_DEVICE otherwise (no
// device at all, or one this library holds no code object for).  The answer
// is looked up once per device.
int require_gfx950() {
  static std::atomic<int> known[64];  // 0 = not looked up, 1 = gfx950, 2 = something else
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return WOL_ERR_NO_DEVICE;
  }
  if (dev < 0 || dev >= 64) return WOL_ERR_NO_DEVICE;
  int k = known[dev].load(std::memory_order_acquire);
  if (k == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
      (void)hipGetLastError();
      return WOL_ERR_NO_DEVICE;
    }
    k = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
    known[dev].store(k, std::memory_order_release);
  }
  return k == 1 ? WOL_OK : WOL_ERR_NO_DEVICE;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// paddle/phi/infermeta/unary.cc:5961-5983 (weight_quantize) and
// multiary.cc:5503-5560 (weight_only_linear): K % 64, N % 16, group size.
int check_problem(int dtype, int64_t K, int64_t N, int bits, int group_size) {
  if (dtype != WOL_DTYPE_F16 && dtype != WOL_DTYPE_BF16) return WOL_ERR_BAD_DTYPE;
  if (bits != 8 && bits != 4) return WOL_ERR_BAD_BITS;
  if (!(group_size == -1 || group_size == 64 || group_size == 128)) return WOL_ERR_BAD_GROUP_SIZE;
  if (K <= 0 || N <= 0 || K % 64 != 0 || N % 16 != 0) return WOL_ERR_BAD_SHAPE;
  // byte offsets inside a tensor are kept in int64; row, column and k-tile
  // indices (and a k tile's byte offset inside a strip, K * 16) in int32
  if (K > (int64_t{1} << 24) || N > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  return WOL_OK;
}

bool layout_ok(int layout) {
  return layout == WOL_LAYOUT_CANONICAL || layout == WOL_LAYOUT_PADDLE_HIP ||
         layout == WOL_LAYOUT_GFX950;
}

// The streaming kernel takes M <= 64 (four 16-row MFMA tiles).  It streams
// the weights best, but every 16-column strip re-reads its activations from
// L2; the MFMA GEMM shares them through LDS at the price of a second launch
// that adds the K runs.  Up to 16 rows the streaming kernel won every shape
// measured against the GEMM (K and N from 4096 to 28672, both bit widths; the
// batched decode kernel, where it applies, is chosen before either, see
// use_batch); from 17 to 64 rows
// the cheaper of the two by a linear cost model runs (microseconds, least
// squares of the relative error over 648 measurements on MI355X: 18 shapes
// with K, N from 2048 to 28672, four weight formats, nine row counts; the
// streaming kernel only where K is a power of two -- elsewhere its wavefronts
// walk their units instead of loading them at once and the GEMM won every
// case.  The choice costs 0.2 % of the total time of those cases against
// always taking the faster kernel, 23 % in the worst case).
constexpr int64_t kStreamMaxM = 64;
constexpr int64_t kStreamAlwaysM = 16;

bool gemm_fast_path(int64_t K, int bits) {
  const int64_t tk = bits == 8 ? 64 : 128;
  return K % tk == 0 && K / tk >= 2;
}

// have_ws: the caller's scratch buffer holds what the GEMM asks for on this problem
bool use_stream(int64_t M, int64_t K, int64_t N, int bits, bool have_ws) {
  if (M > kStreamMaxM) return false;
  if (M <= kStreamAlwaysM || !gemm_fast_path(K, bits)) return true;
  const double w = static_cast<double>(K) * N * bits / 8.0 * 1e-6;  // weight MB
  // activation MB the strips re-read out of L2: the rows that exist, and the
  // 16-row operands they are padded to (padding rows repeat the last row)
  const double a = static_cast<double>(N / 16) * M * K * 2.0 * 1e-6;
  const double a_pad = static_cast<double>(N / 16) * ((M + 15) / 16 * 16) * K * 2.0 * 1e-6;
  const double t_stream = 2.908 + 0.0305 * w + 0.0914 * a + 0.0238 * a_pad;
  // two launches; K runs of a few k tiles each; fp32 partial sums written and
  // read back (M * N); MFMA work of the 32- or 64-row tile
  const double tile_rows = bits == 4 && M <= 32 ? 32.0 : 64.0;
  if (!have_ws) {
    // without scratch every workgroup walks all of K: measured 0.75 us per k
    // tile (1.17 us for 64 rows of int4), one workgroup per 256 columns
    const double tiles = static_cast<double>(K / (bits == 8 ? 64 : 128));
    const double rounds = static_cast<double>((N / 256 + 511) / 512);  // two workgroups fit a CU
    return t_stream <= 3.0 + tiles * (bits == 4 && M > 32 ? 1.17 : 0.75) * rounds;
  }
  if ((K & (K - 1)) != 0) return false;
  const double t_gemm = 10.232 + (bits == 8 ? 0.0622 : 0.0445) * w + 2.047 * (M * N * 1e-6) +
                        2.2896 * (tile_rows * N * K * 1e-9);
  return t_stream <= t_gemm;
}

// The batched decode kernel (a workgroup per CU that owns N / 16 / CUs strips
// and fetches the activations once for all of them) against the streaming
// kernel (a workgroup per strip): measured on MI355X over K = 2048, 4096 and
// 8192, N from 4096 to 28672, both bit widths, it wins from 2.5 strips per CU
// on when the streaming kernel's activation reads weigh in -- 5 rows and more
// (16-row and 8-row operands) -- by up to 30 %; for 3 and 4 rows from 3.5
// strips per CU on, for 2 rows from 2.5 (int4) or 5 (int8).  With exactly two
// strips per CU (N = 8192 on 256 CUs) and with one the streaming kernel has
// the shorter critical path at every row count (by 2 to 40 %).
bool use_batch(int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  if (M < 2 || M > 16 || !wol::linear_batch_supports(M, K, bits, group_size)) return false;
  const double per_cu = static_cast<double>(N / wol::kStripCols) / wol::linear_batch_cus();
  // 2 to 4 rows where the streaming kernel issues all loads of a wavefront at
  // once (K = 2048 and 4096, 2 to 7 strips per CU): it is 3 to 20 % faster
  // than this kernel except on int4 at K >= 4096 from 5 strips per CU on
  // (4 to 9 % slower there)
  if (M <= 4 && wol::linear_stream_loads_at_once(M, K, N, bits)) return bits == 4 && K >= 4096 && per_cu >= 5.0;
  // the same for 5 to 8 rows on int8 (K = 2048: 3 to 12 % at every width; K = 4096: 1 to 11 % below 5 strips per CU)
  if (M <= 8 && bits == 8 && wol::linear_stream_loads_at_once(M, K, N, bits)) return K >= 4096 && per_cu >= 5.0;
  if (M == 3 || M == 4) return per_cu >= 3.5;
  if (M == 2) return per_cu >= (bits == 4 ? 2.5 : 5.0);
  return per_cu >= 2.5;
}

// The batched decode kernel with K cut into runs across workgroups (two
// launches: the runs, then their sum) against whatever the rules above would
// take.  Measured on MI355X over 18 shapes (K, N from 2048 to 28672, also the
// ones that are not powers of two), both bit widths, 2 to 32 rows:
//  * up to 16 rows it wins where the streaming kernel is at its worst -- 10
//    rows and more (the activation reads of a workgroup per strip weigh in),
//    a K the one-launch batched kernel is not built for, and strips that
//    leave the CUs a ragged last round (N / 16 / CUs is 1.1 or more below
//    its ceiling: N = 5120 ... 7168 on 256 CUs), by 10 to 49 %; int4 with
//    K >= 14336 from 12 rows on also with whole rounds (9 to 18 %), and with
//    K >= 11008 at 16 rows (4 to 13 %);
//  * from 17 to 32 rows (two 16-row operands) it beats the better of the
//    streaming kernel and the MFMA GEMM on int8 weights of 20 MB and more by
//    5 to 20 %, and on int4 weights of 10 to 34 MB by up to 17 %.
// Elsewhere the second launch (3 us) costs more than the split gains.
// ws_bytes: the caller's scratch.
bool use_batch_split(int64_t M, int64_t K, int64_t N, int bits, int group_size, size_t ws_bytes) {
  if (M < 2 || !wol::linear_batch_split_supports(M, K, bits, group_size)) return false;
  if (ws_bytes < wol::linear_batch_split_workspace(M, K, N, bits, group_size)) return false;
  const double w = static_cast<double>(K) * N * bits / 8.0 * 1e-6;  // weight MB
  if (M > 16) return bits == 4 ? (w >= 10.0 && w <= 34.0) : w >= 20.0;
  const int64_t cus = wol::linear_batch_cus(), nstrips = N / wol::kStripCols;
  if (M < 10 || nstrips > 2 * cus || wol::linear_batch_supports(M, K, bits, group_size)) return false;
  const double rounds = static_cast<double>(nstrips) / cus;
  const double ragged = static_cast<double>((nstrips + cus - 1) / cus) / rounds;
  if (ragged >= 1.1) return true;
  return bits == 4 && ((M >= 12 && K >= 14336) || (M >= 16 && K >= 11008));
}

// kernel: a wol_kernel; AUTO resolves by M and the cost model.  Returns the
// wol_kernel that runs.  ws_bytes: the caller's scratch (SIZE_MAX: as much as
// any kernel asks for).
int resolve_kernel(int kernel, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                   size_t ws_bytes = SIZE_MAX) {
  if (kernel != WOL_KERNEL_AUTO) return kernel;
  if (use_batch_split(M, K, N, bits, group_size, ws_bytes)) return WOL_KERNEL_BATCH_SPLIT;
  if (use_batch(M, K, N, bits, group_size)) return WOL_KERNEL_BATCH;
  // With ample scratch first: if the streaming kernel wins there it is taken
  // whatever the caller brought (wol_linear_workspace then reports 0 bytes, and
  // a caller who passes exactly that gets the same kernel).  Only a GEMM that
  // cannot have its K runs is compared again, as the unsplit GEMM it becomes.
  if (use_stream(M, K, N, bits, true)) return WOL_KERNEL_STREAM;
  if (ws_bytes >= wol::linear_gemm_workspace(M, K, N, bits, group_size)) return WOL_KERNEL_GEMM;
  return use_stream(M, K, N, bits, false) ? WOL_KERNEL_STREAM : WOL_KERNEL_GEMM;
}

const char* kernel_name(int which) {
  switch (which) {
    case WOL_KERNEL_BATCH: return "batch";
    case WOL_KERNEL_BATCH_SPLIT: return "batch (K split)";
    case WOL_KERNEL_STREAM: return "stream";
    default: return "gemm";
  }
}

// WOL_LOG=1 in the environment: every compute call writes one line to stderr
// (entry point, problem, the kernel taken).  Read once.
bool log_enabled() {
  static const bool on = [] {
    const char* e = getenv("WOL_LOG");
    return e != nullptr && e[0] != '\0' && e[0] != '0';
  }();
  return on;
}

// WOL_ROCTX=1 in the environment: every compute call of the C ABI is wrapped
// in a roctx range named after its entry point, so that a rocprofv3
// --marker-trace shows which launches belong to which call.  The marker
// library is looked up at run time (no link dependency); without it, or
// without the variable, a range costs one load of a static flag.
struct RoctxApi {
  int (*push)(const char*) = nullptr;
  int (*pop)() = nullptr;
};
const RoctxApi& roctx_api() {
  static const RoctxApi api = [] {
    RoctxApi a;
    const char* e = getenv("WOL_ROCTX");
    if (e == nullptr || e[0] == '\0' || e[0] == '0') return a;
    void* h = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_GLOBAL);
    if (h == nullptr) h = dlopen("libroctx64.so", RTLD_NOW | RTLD_GLOBAL);
    if (h == nullptr) return a;
    a.push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
    a.pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
    if (a.push == nullptr || a.pop == nullptr) a = RoctxApi();
    return a;
  }();
  return api;
}
struct Range {
  explicit Range(const char* name) : on(roctx_api().push != nullptr) {
    if (on) roctx_api().push(name);
  }
  ~Range() {
    if (on) roctx_api().pop();
  }
  Range(const Range&) = delete;
  Range& operator=(const Range&) = delete;
  bool on;
};

// Whether kernel `which` forms the swiglu of a gate|up projection in its own epilogue.
bool kernel_fuses_swiglu(int which, int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  if (which == WOL_KERNEL_GEMM) return wol::linear_gemm_fuses_swiglu(M, K, N, bits, group_size);
  if (which == WOL_KERNEL_STREAM) return wol::linear_stream_fuses_swiglu(M, N);
  if (which == WOL_KERNEL_BATCH) return wol::linear_batch_fuses_swiglu(K, N, bits);
  if (which == WOL_KERNEL_BATCH_SPLIT) return N % 32 == 0;  // in the kernel that adds the runs
  return false;
}

int linear_impl(const void* x, const void* codes, const void* bias, const void* scale, int dtype,
                int64_t M, int64_t K, int64_t N, int bits, int group_size, void* out, bool out_f32,
                int kernel, void* workspace, size_t workspace_bytes, void* stream,
                const wol::Fuse& fuse = wol::Fuse()) {
  const Range range("wol_linear");
  const int rc = check_problem(dtype, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (M < 0 || M > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  if (kernel != WOL_KERNEL_AUTO && kernel != WOL_KERNEL_STREAM && kernel != WOL_KERNEL_GEMM &&
      kernel != WOL_KERNEL_BATCH && kernel != WOL_KERNEL_BATCH_SPLIT)
    return WOL_ERR_BAD_SHAPE;
  if (kernel == WOL_KERNEL_STREAM && M > kStreamMaxM) return WOL_ERR_BAD_SHAPE;
  if (kernel == WOL_KERNEL_BATCH && M > 0 && !wol::linear_batch_supports(M, K, bits, group_size)) return WOL_ERR_BAD_SHAPE;
  if (kernel == WOL_KERNEL_BATCH_SPLIT && M > 0 &&
      (!wol::linear_batch_split_supports(M, K, bits, group_size) || fuse.pre_scale != nullptr))
    return WOL_ERR_BAD_SHAPE;
  if (M == 0) return WOL_OK;  // empty batch: nothing to write
  if (x == nullptr || codes == nullptr || scale == nullptr || out == nullptr)
    return WOL_ERR_NULL_POINTER;
  // the kernels read and write 16 bytes at a time (the output rows included)
  if (!aligned16(x) || !aligned16(codes) || !aligned16(scale) || !aligned16(out) || !aligned16(bias))
    return WOL_ERR_ALIGNMENT;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (workspace == nullptr || !aligned16(workspace)) workspace_bytes = 0;  // optional: only speeds up
  int which = resolve_kernel(kernel, M, K, N, bits, group_size, workspace_bytes);
  if (which == WOL_KERNEL_BATCH_SPLIT && kernel == WOL_KERNEL_AUTO && fuse.pre_scale != nullptr)
    which = resolve_kernel(kernel, M, K, N, bits, group_size, 0);  // that kernel applies no pre-scale
  if (fuse.act == WOL_ACT_SWIGLU && !kernel_fuses_swiglu(which, M, K, N, bits, group_size)) return WOL_ERR_BAD_SHAPE;
  if (log_enabled())
    fprintf(stderr, "[wol] linear M=%lld K=%lld N=%lld int%d group=%d %s%s%s act=%d -> %s kernel\n",
            static_cast<long long>(M), static_cast<long long>(K), static_cast<long long>(N), bits, group_size,
            dtype == WOL_DTYPE_BF16 ? "bf16" : "f16", bias != nullptr ? " bias" : "",
            fuse.pre_scale != nullptr ? " pre_scale" : "", fuse.act,
            kernel_name(which));
  if (which == WOL_KERNEL_BATCH_SPLIT)
    return wol::launch_linear_batch_split(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out,
                                          out_f32, workspace, workspace_bytes, s, fuse);
  if (which == WOL_KERNEL_BATCH)
    return wol::launch_linear_batch(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out,
                                    out_f32, s, fuse);
  if (which == WOL_KERNEL_STREAM)
    return wol::launch_linear_stream(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out,
                                     out_f32, s, fuse);
  return wol::launch_linear_gemm(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out,
                                 out_f32, workspace, workspace_bytes, s, fuse);
}

}  // namespace

extern "C" {

const char* wol_status_str(int status) {
  switch (status) {
    case WOL_OK: return "ok";
    case WOL_ERR_NULL_POINTER: return "a required pointer is NULL";
    case WOL_ERR_BAD_DTYPE: return "dtype must be float16 (0) or bfloat16 (1)";
    case WOL_ERR_BAD_BITS: return "weight_dtype must be int8 or int4";
    case WOL_ERR_BAD_GROUP_SIZE: return "group_size must be -1, 64 or 128";
    case WOL_ERR_BAD_SHAPE:
      return "shape outside the contract (K divisible by 64, N divisible by 16, sizes positive and at most 2^24)";
    case WOL_ERR_BAD_LAYOUT: return "unknown weight layout";
    case WOL_ERR_BAD_ROUND_MODE: return "round_mode must be RNE (0) or TRUNC (1)";
    case WOL_ERR_WORKSPACE: return "workspace missing or too small";
    case WOL_ERR_ALIGNMENT: return "pointer not 16-byte aligned";
    case WOL_ERR_HIP: return "HIP launch failed";
    case WOL_ERR_NO_DEVICE: return "the current device is not a gfx950 (or there is no device)";
    default: return "unknown status";
  }
}

int wol_layout_version(void) { return wol::kLayoutVersion; }

size_t wol_quantize_workspace(int64_t K, int64_t N, int bits, int group_size) {
  if (check_problem(WOL_DTYPE_F16, K, N, bits, group_size) != WOL_OK) return 0;
  return group_size == -1 ? static_cast<size_t>(N) * sizeof(uint32_t) : 0;
}

int wol_quantize(const void* w, int dtype, int64_t K, int64_t N, int bits, int group_size,
                 int round_mode, int layout, void* codes_out, void* scale_out, void* workspace,
                 size_t workspace_bytes, void* stream) {
  const Range range("wol_quantize");
  const int rc = check_problem(dtype, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (round_mode != WOL_ROUND_RNE && round_mode != WOL_ROUND_TRUNC) return WOL_ERR_BAD_ROUND_MODE;
  if (!layout_ok(layout)) return WOL_ERR_BAD_LAYOUT;
  if (w == nullptr || codes_out == nullptr || scale_out == nullptr) return WOL_ERR_NULL_POINTER;
  if (!aligned16(w) || !aligned16(codes_out)) return WOL_ERR_ALIGNMENT;
  const size_t need = wol_quantize_workspace(K, N, bits, group_size);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need)) return WOL_ERR_WORKSPACE;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_quantize(w, dtype, K, N, bits, group_size, round_mode, layout, codes_out,
                              scale_out, false, workspace, static_cast<hipStream_t>(stream));
}

int wol_quantize_static(const void* w, int dtype, int64_t K, int64_t N, int bits, int group_size,
                        int round_mode, int layout, void* codes_out, void* scale_out, void* stream) {
  const Range range("wol_quantize_static");
  const int rc = check_problem(dtype, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (round_mode != WOL_ROUND_RNE && round_mode != WOL_ROUND_TRUNC) return WOL_ERR_BAD_ROUND_MODE;
  if (!layout_ok(layout)) return WOL_ERR_BAD_LAYOUT;
  if (group_size == -1 && N > wol::kQuantizeStaticMaxN) return WOL_ERR_BAD_SHAPE;
  if (w == nullptr || codes_out == nullptr || scale_out == nullptr) return WOL_ERR_NULL_POINTER;
  if (!aligned16(w) || !aligned16(codes_out)) return WOL_ERR_ALIGNMENT;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_quantize_static(w, dtype, K, N, bits, group_size, round_mode, layout, codes_out,
                                     scale_out, static_cast<hipStream_t>(stream));
}

int wol_quantize_llm_int8(const void* w, int dtype, int64_t K, int64_t N, int group_size,
                          int layout, void* codes_out, float* scale_out, void* workspace,
                          size_t workspace_bytes, void* stream) {
  const Range range("wol_quantize_llm_int8");
  const int rc = check_problem(dtype, K, N, 8, group_size);
  if (rc != WOL_OK) return rc;
  if (!layout_ok(layout)) return WOL_ERR_BAD_LAYOUT;
  if (w == nullptr || codes_out == nullptr || scale_out == nullptr) return WOL_ERR_NULL_POINTER;
  if (!aligned16(w) || !aligned16(codes_out)) return WOL_ERR_ALIGNMENT;
  const size_t need = wol_quantize_workspace(K, N, 8, group_size);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need)) return WOL_ERR_WORKSPACE;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_quantize(w, dtype, K, N, 8, group_size, WOL_ROUND_RNE, layout, codes_out,
                              scale_out, true, workspace, static_cast<hipStream_t>(stream));
}

int wol_dequantize(const void* codes, int layout, const void* scale, int dtype, int64_t K,
                   int64_t N, int bits, int group_size, void* out_KN, void* stream) {
  const Range range("wol_dequantize");
  const int rc = check_problem(dtype, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (!layout_ok(layout)) return WOL_ERR_BAD_LAYOUT;
  if (codes == nullptr || scale == nullptr || out_KN == nullptr) return WOL_ERR_NULL_POINTER;
  if (!aligned16(scale) || !aligned16(out_KN)) return WOL_ERR_ALIGNMENT;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_dequantize(codes, layout, scale, dtype, K, N, bits, group_size, out_KN,
                                static_cast<hipStream_t>(stream));
}

size_t wol_linear_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  return wol_linear_workspace_for(M, K, N, bits, group_size, WOL_KERNEL_AUTO);
}

size_t wol_linear_workspace_for(int64_t M, int64_t K, int64_t N, int bits, int group_size,
                                int kernel) {
  if (check_problem(WOL_DTYPE_F16, K, N, bits, group_size) != WOL_OK || M <= 0) return 0;
  if (kernel == WOL_KERNEL_STREAM && M > kStreamMaxM) return 0;
  const int which = resolve_kernel(kernel, M, K, N, bits, group_size);
  if (which == WOL_KERNEL_BATCH_SPLIT) return wol::linear_batch_split_workspace(M, K, N, bits, group_size);
  if (which != WOL_KERNEL_GEMM) return 0;  // partial sums stay on chip
  return wol::linear_gemm_workspace(M, K, N, bits, group_size);
}

int wol_linear(const void* x, const void* codes, const void* bias, const void* scale, int dtype,
               int64_t M, int64_t K, int64_t N, int bits, int group_size, void* out,
               void* workspace, size_t workspace_bytes, void* stream) {
  return linear_impl(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out, false,
                     WOL_KERNEL_AUTO, workspace, workspace_bytes, stream);
}

int wol_linear_f32(const void* x, const void* codes, const void* bias, const void* scale,
                   int dtype, int64_t M, int64_t K, int64_t N, int bits, int group_size,
                   float* out_f32, void* workspace, size_t workspace_bytes, void* stream) {
  return linear_impl(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out_f32, true,
                     WOL_KERNEL_AUTO, workspace, workspace_bytes, stream);
}

namespace {

// How wol_linear_fused lays a call out: which parts the linear kernel applies
// itself and what goes through the workspace ([the linear's own scratch]
// [pre-scaled activations M x K T] [fp32 sums M x N]).
struct FusedPlan {
  bool prepass;          // the activations are scaled by a pass of the prescale kernel
  bool swiglu_pass;      // the linear writes fp32 sums, a pass turns them into T(swiglu)
  size_t linear_ws, x_off, sums_off, total;
};

FusedPlan plan_fused(int64_t M, int64_t K, int64_t N, int bits, int group_size, bool has_pre, int act) {
  FusedPlan f{};
  const size_t lws = wol_linear_workspace(M, K, N, bits, group_size);
  // a call with activation scales never takes the K-split batched kernel
  const int which = resolve_kernel(WOL_KERNEL_AUTO, M, K, N, bits, group_size, has_pre ? 0 : SIZE_MAX);
  const bool fused_pre = (which == WOL_KERNEL_BATCH && wol::linear_batch_fuses_pre_scale(K, bits, group_size)) ||
                         (which == WOL_KERNEL_STREAM && M == 1);
  f.prepass = has_pre && !fused_pre;
  // the decode kernels and the GEMM's large tiles form the swiglu in their epilogue; elsewhere it is a pass over fp32 sums
  // (the batched kernel applies activation scales or forms the swiglu, not both)
  f.swiglu_pass = act == WOL_ACT_SWIGLU && !(kernel_fuses_swiglu(which, M, K, N, bits, group_size) &&
                                             !(which == WOL_KERNEL_BATCH && has_pre && fused_pre));
  auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
  f.linear_ws = lws;
  f.x_off = up(lws);
  f.sums_off = f.x_off + (f.prepass ? up(static_cast<size_t>(M) * K * 2) : 0);
  f.total = f.sums_off + (f.swiglu_pass ? up(static_cast<size_t>(M) * N * 4) : 0);
  if (!f.prepass && !f.swiglu_pass) f.total = lws;
  return f;
}

}  // namespace

size_t wol_linear_fused_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size,
                                  int has_pre_scale, int act) {
  if (check_problem(WOL_DTYPE_F16, K, N, bits, group_size) != WOL_OK || M <= 0) return 0;
  if (act != WOL_ACT_NONE && act != WOL_ACT_GELU && act != WOL_ACT_SWIGLU) return 0;
  return plan_fused(M, K, N, bits, group_size, has_pre_scale != 0, act).total;
}

int wol_linear_fused(const void* x, const void* pre_scale, const void* codes, const void* bias,
                     const void* scale, int dtype, int64_t M, int64_t K, int64_t N, int bits,
                     int group_size, int act, void* out, void* workspace, size_t workspace_bytes,
                     void* stream) {
  const Range range("wol_linear_fused");
  const int rc = check_problem(dtype, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (M < 0 || M > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  if (act != WOL_ACT_NONE && act != WOL_ACT_GELU && act != WOL_ACT_SWIGLU) return WOL_ERR_BAD_SHAPE;
  if (act == WOL_ACT_SWIGLU && N % 32 != 0) return WOL_ERR_BAD_SHAPE;
  if (M == 0) return WOL_OK;
  if (x == nullptr || codes == nullptr || scale == nullptr || out == nullptr) return WOL_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(codes) || !aligned16(scale) || !aligned16(out) || !aligned16(bias))
    return WOL_ERR_ALIGNMENT;
  if (pre_scale != nullptr && !aligned16(pre_scale)) return WOL_ERR_ALIGNMENT;
  const FusedPlan f = plan_fused(M, K, N, bits, group_size, pre_scale != nullptr, act);
  // (a swiglu formed inside the kernel: the kernel must be the one the plan was made for, scratch included)
  if (f.prepass || f.swiglu_pass || (act == WOL_ACT_SWIGLU && f.total > 0)) {
    if (workspace == nullptr || workspace_bytes < f.total) return WOL_ERR_WORKSPACE;
    if (!aligned16(workspace)) return WOL_ERR_ALIGNMENT;
  }
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  hipStream_t s = static_cast<hipStream_t>(stream);
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  wol::Fuse fuse;
  fuse.act = act == WOL_ACT_GELU || (act == WOL_ACT_SWIGLU && !f.swiglu_pass) ? act : WOL_ACT_NONE;
  const void* xin = x;
  if (f.prepass) {
    const int prc = wol::launch_prescale(x, pre_scale, dtype, M, K, ws + f.x_off, s);
    if (prc != WOL_OK) return prc;
    xin = ws + f.x_off;
  } else {
    fuse.pre_scale = pre_scale;
  }
  // without extra passes the caller's scratch is the linear's as it is (it stays optional)
  const bool passes = f.prepass || f.swiglu_pass;
  void* lws = passes ? (f.linear_ws > 0 ? ws : nullptr) : workspace;
  const size_t lws_bytes = passes ? f.linear_ws : workspace_bytes;
  if (!f.swiglu_pass)
    return linear_impl(xin, codes, bias, scale, dtype, M, K, N, bits, group_size, out, false, WOL_KERNEL_AUTO,
                       lws, lws_bytes, stream, fuse);
  float* sums = reinterpret_cast<float*>(ws + f.sums_off);
  const int lrc = linear_impl(xin, codes, bias, scale, dtype, M, K, N, bits, group_size, sums, true,
                              WOL_KERNEL_AUTO, lws, lws_bytes, stream, fuse);
  if (lrc != WOL_OK) return lrc;
  return wol::launch_swiglu_f32(sums, dtype, M, N, out, s);
}

size_t wol_linear_grad_workspace(int64_t M, int64_t K, int64_t N, int bits, int group_size) {
  if (check_problem(WOL_DTYPE_F16, K, N, bits, group_size) != WOL_OK || M <= 0 || M > (int64_t{1} << 24)) return 0;
  return wol::linear_grad_workspace(M, K, N, group_size);
}

namespace {
int linear_grad_impl(const void* out_grad, const void* codes, const void* scale, int dtype, int64_t M,
                     int64_t K, int64_t N, int bits, int group_size, void* x_grad, bool out_f32,
                     void* workspace, size_t workspace_bytes, void* stream) {
  const Range range("wol_linear_grad");
  const int rc = check_problem(dtype, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (M < 0 || M > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  if (M == 0) return WOL_OK;
  if (out_grad == nullptr || codes == nullptr || scale == nullptr || x_grad == nullptr) return WOL_ERR_NULL_POINTER;
  if (!aligned16(out_grad) || !aligned16(codes) || !aligned16(scale) || !aligned16(x_grad)) return WOL_ERR_ALIGNMENT;
  if (workspace == nullptr || workspace_bytes < wol::linear_grad_workspace(M, K, N, group_size))
    return WOL_ERR_WORKSPACE;
  if (!aligned16(workspace)) return WOL_ERR_ALIGNMENT;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  if (log_enabled())
    fprintf(stderr, "[wol] linear_grad M=%lld K=%lld N=%lld int%d group=%d %s\n", static_cast<long long>(M),
            static_cast<long long>(K), static_cast<long long>(N), bits, group_size,
            dtype == WOL_DTYPE_BF16 ? "bf16" : "f16");
  return wol::launch_linear_grad(out_grad, codes, scale, dtype, M, K, N, bits, group_size, x_grad, out_f32,
                                 workspace, static_cast<hipStream_t>(stream));
}
}  // namespace

int wol_linear_grad(const void* out_grad, const void* codes, const void* scale, int dtype, int64_t M,
                    int64_t K, int64_t N, int bits, int group_size, void* x_grad, void* workspace,
                    size_t workspace_bytes, void* stream) {
  return linear_grad_impl(out_grad, codes, scale, dtype, M, K, N, bits, group_size, x_grad, false, workspace,
                          workspace_bytes, stream);
}

int wol_linear_grad_f32(const void* out_grad, const void* codes, const void* scale, int dtype, int64_t M,
                        int64_t K, int64_t N, int bits, int group_size, float* x_grad_f32, void* workspace,
                        size_t workspace_bytes, void* stream) {
  return linear_grad_impl(out_grad, codes, scale, dtype, M, K, N, bits, group_size, x_grad_f32, true, workspace,
                          workspace_bytes, stream);
}

namespace {
int check_moe(int64_t rows, int64_t hidden, int64_t inter, int num_experts) {
  if (rows < 0 || rows > (int64_t{1} << 24) || hidden <= 0 || inter <= 0) return WOL_ERR_BAD_SHAPE;
  if (hidden % 128 != 0 || inter % 256 != 0 || hidden > (int64_t{1} << 24) || inter > (int64_t{1} << 24))
    return WOL_ERR_BAD_SHAPE;
  if (hidden < 256 || inter < 512) return WOL_ERR_BAD_SHAPE;  // at least two k tiles in both products
  if (num_experts <= 0 || num_experts > 1024) return WOL_ERR_BAD_SHAPE;
  return WOL_OK;
}
}  // namespace

size_t wol_moe_ffn_workspace(int64_t rows, int64_t hidden, int64_t inter, int num_experts) {
  if (check_moe(rows, hidden, inter, num_experts) != WOL_OK || rows == 0) return 0;
  return wol::moe_ffn_workspace(rows, hidden, inter, num_experts);
}

int wol_moe_ffn(const void* permute_input, const int64_t* token_nums_per_expert, const void* ffn1_weight,
                const void* ffn1_bias, const void* ffn1_scale, const void* ffn2_weight, const void* ffn2_scale,
                int dtype, int64_t rows, int64_t hidden, int64_t inter, int num_experts, int bits, void* ffn_out,
                void* workspace, size_t workspace_bytes, void* stream) {
  const Range range("wol_moe_ffn");
  if (dtype != WOL_DTYPE_F16 && dtype != WOL_DTYPE_BF16) return WOL_ERR_BAD_DTYPE;
  if (bits != 8 && bits != 4) return WOL_ERR_BAD_BITS;
  const int rc = check_moe(rows, hidden, inter, num_experts);
  if (rc != WOL_OK) return rc;
  if (rows == 0) return WOL_OK;
  if (permute_input == nullptr || token_nums_per_expert == nullptr || ffn1_weight == nullptr ||
      ffn1_scale == nullptr || ffn2_weight == nullptr || ffn2_scale == nullptr || ffn_out == nullptr)
    return WOL_ERR_NULL_POINTER;
  if (!aligned16(permute_input) || !aligned16(ffn1_weight) || !aligned16(ffn2_weight) || !aligned16(ffn1_scale) ||
      !aligned16(ffn2_scale) || !aligned16(ffn_out))
    return WOL_ERR_ALIGNMENT;
  if (workspace == nullptr || workspace_bytes < wol::moe_ffn_workspace(rows, hidden, inter, num_experts))
    return WOL_ERR_WORKSPACE;
  if (!aligned16(workspace)) return WOL_ERR_ALIGNMENT;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_moe_ffn(permute_input, token_nums_per_expert, ffn1_weight, ffn1_bias, ffn1_scale, ffn2_weight,
                             ffn2_scale, dtype, rows, hidden, inter, num_experts, bits, ffn_out, workspace,
                             static_cast<hipStream_t>(stream));
}

int wol_linear_on(const void* x, const void* codes, const void* bias, const void* scale, int dtype,
                  int64_t M, int64_t K, int64_t N, int bits, int group_size, void* out,
                  int out_is_f32, int kernel, void* workspace, size_t workspace_bytes,
                  void* stream) {
  return linear_impl(x, codes, bias, scale, dtype, M, K, N, bits, group_size, out,
                     out_is_f32 != 0, kernel, workspace, workspace_bytes, stream);
}

int wol_repack(const void* codes_in, int layout_in, void* codes_out, int layout_out, int64_t K,
               int64_t N, int bits, void* stream) {
  const Range range("wol_repack");
  const int rc = check_problem(WOL_DTYPE_F16, K, N, bits, -1);
  if (rc != WOL_OK) return rc;
  if (!layout_ok(layout_in) || !layout_ok(layout_out)) return WOL_ERR_BAD_LAYOUT;
  if (codes_in == nullptr || codes_out == nullptr) return WOL_ERR_NULL_POINTER;
  if (codes_in == codes_out) return WOL_ERR_BAD_LAYOUT;  // not in place
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_repack(codes_in, layout_in, codes_out, layout_out, K, N, bits,
                            static_cast<hipStream_t>(stream));
}

int wol_repack_host(const void* codes_in, int layout_in, void* codes_out, int layout_out, int64_t K,
                    int64_t N, int bits) {
  const int rc = check_problem(WOL_DTYPE_F16, K, N, bits, -1);
  if (rc != WOL_OK) return rc;
  if (!layout_ok(layout_in) || !layout_ok(layout_out)) return WOL_ERR_BAD_LAYOUT;
  if (codes_in == nullptr || codes_out == nullptr) return WOL_ERR_NULL_POINTER;
  if (codes_in == codes_out) return WOL_ERR_BAD_LAYOUT;  // not in place
  const uint8_t* in = static_cast<const uint8_t*>(codes_in);
  uint8_t* out = static_cast<uint8_t*>(codes_out);
  if (bits == 4) std::memset(out, 0, static_cast<size_t>(K) * N / 2);  // nibbles are ORed in
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n) {
      int si = 0, so = 0;
      const int64_t oi = wol::code_offset(layout_in, K, N, bits, k, n, &si);
      const int64_t oo = wol::code_offset(layout_out, K, N, bits, k, n, &so);
      const int q = wol::decode_code(layout_in, bits, in[oi] >> si);
      const int v = wol::encode_code(layout_out, bits, q);
      if (bits == 8) out[oo] = static_cast<uint8_t>(v);
      else out[oo] = static_cast<uint8_t>(out[oo] | (v << so));
    }
  return WOL_OK;
}

int64_t wol_code_offset(int layout, int64_t K, int64_t N, int bits, int64_t k, int64_t n,
                        int* nibble_shift) {
  if (check_problem(WOL_DTYPE_F16, K, N, bits, -1) != WOL_OK || !layout_ok(layout)) return -1;
  if (k < 0 || k >= K || n < 0 || n >= N) return -1;
  int shift = 0;
  const int64_t off = wol::code_offset(layout, K, N, bits, k, n, &shift);
  if (nibble_shift != nullptr) *nibble_shift = shift;
  return off;
}

int wol_apply_per_channel_scale(const void* x, const void* scales, int dtype, int64_t rows,
                                int64_t cols, void* out, void* stream) {
  const Range range("wol_apply_per_channel_scale");
  if (dtype != WOL_DTYPE_F16 && dtype != WOL_DTYPE_BF16) return WOL_ERR_BAD_DTYPE;
  if (rows < 0 || cols <= 0 || rows > (int64_t{1} << 24) || cols > (int64_t{1} << 24))
    return WOL_ERR_BAD_SHAPE;
  if (rows == 0) return WOL_OK;
  if (x == nullptr || scales == nullptr || out == nullptr) return WOL_ERR_NULL_POINTER;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_prescale(x, scales, dtype, rows, cols, out, static_cast<hipStream_t>(stream));
}

// int32 accumulation: |sum| <= K * 127 * 127 must stay below 2^31, i.e.
// K <= 133152 (the reference's cublasLt int32 GEMM has the same limit without
// checking it); the outlier mask of a call (K / 32 words) also sits in LDS
constexpr int64_t kLlmInt8MaxK = 131072;

size_t wol_llm_int8_linear_workspace(int64_t M, int64_t K, int64_t N) {
  if (check_problem(WOL_DTYPE_F16, K, N, 8, -1) != WOL_OK || M <= 0 || M > (int64_t{1} << 24)) return 0;
  if (K > kLlmInt8MaxK) return 0;
  return wol::llm_int8_workspace(M, K, N);
}

int wol_llm_int8_linear_stage_offsets(int64_t M, int64_t K, int64_t N, int64_t* offsets) {
  if (offsets == nullptr) return WOL_ERR_NULL_POINTER;
  if (check_problem(WOL_DTYPE_F16, K, N, 8, -1) != WOL_OK || M <= 0 || M > (int64_t{1} << 24) || K > kLlmInt8MaxK)
    return WOL_ERR_BAD_SHAPE;
  wol::llm_int8_workspace_offsets(M, K, N, offsets);
  return WOL_OK;
}

int wol_llm_int8_linear(const void* x, const void* weight, const void* bias, const float* weight_scale,
                        float threshold, int dtype, int64_t M, int64_t K, int64_t N, void* out,
                        void* workspace, size_t workspace_bytes, void* stream) {
  const Range range("wol_llm_int8_linear");
  const int rc = check_problem(dtype, K, N, 8, -1);
  if (rc != WOL_OK) return rc;
  if (M < 0 || M > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  if (M * N > (int64_t{1} << 40) || K > kLlmInt8MaxK) return WOL_ERR_BAD_SHAPE;  // tile counts in int32; mask in LDS
  if (M == 0) return WOL_OK;  // empty batch: nothing to write
  if (x == nullptr || weight == nullptr || weight_scale == nullptr || out == nullptr)
    return WOL_ERR_NULL_POINTER;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(weight_scale) || !aligned16(out))
    return WOL_ERR_ALIGNMENT;
  if (workspace == nullptr || workspace_bytes < wol::llm_int8_workspace(M, K, N)) return WOL_ERR_WORKSPACE;
  if (!aligned16(workspace)) return WOL_ERR_ALIGNMENT;
  if (const int dv = require_gfx950(); dv != WOL_OK) return dv;
  return wol::launch_llm_int8_linear(x, weight, bias, weight_scale, threshold, dtype, M, K, N, out, workspace,
                                     static_cast<hipStream_t>(stream));
}

int wol_linear_grad_plan(int64_t M, int64_t K, int64_t N, char* buf, size_t buf_bytes) {
  if (buf == nullptr || buf_bytes == 0) return WOL_ERR_NULL_POINTER;
  const int rc = check_problem(WOL_DTYPE_F16, K, N, 8, -1);
  if (rc != WOL_OK) return rc;
  if (M <= 0 || M > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  wol::describe_linear_grad(M, K, N, buf, buf_bytes);
  return WOL_OK;
}

int wol_linear_plan(int64_t M, int64_t K, int64_t N, int bits, int group_size, size_t workspace_bytes,
                    char* buf, size_t buf_bytes) {
  if (buf == nullptr || buf_bytes == 0) return WOL_ERR_NULL_POINTER;
  const int rc = check_problem(WOL_DTYPE_F16, K, N, bits, group_size);
  if (rc != WOL_OK) return rc;
  if (M <= 0 || M > (int64_t{1} << 24)) return WOL_ERR_BAD_SHAPE;
  const int which = resolve_kernel(WOL_KERNEL_AUTO, M, K, N, bits, group_size, workspace_bytes);
  if (which == WOL_KERNEL_BATCH_SPLIT) {
    wol::describe_linear_batch_split(M, K, N, bits, group_size, buf, buf_bytes);
  } else if (which == WOL_KERNEL_BATCH) {
    int grid = 1, tpw = 1;
    wol::plan_linear_batch(K, N, bits, &grid, &tpw);
    snprintf(buf, buf_bytes, "wol::batch_kernel: %d workgroups of 16 wavefronts, %lld or %lld strips each, "
             "activations resident in registers (%d weight tiles of a strip per wavefront)",
             grid, static_cast<long long>(N / 16 / grid), static_cast<long long>((N / 16 + grid - 1) / grid), tpw);
  } else if (which == WOL_KERNEL_STREAM) {
    wol::describe_linear_stream(M, K, N, bits, group_size, buf, buf_bytes);
  } else {
    wol::describe_linear_gemm(M, K, N, bits, group_size, workspace_bytes, buf, buf_bytes);
  }
  return WOL_OK;
}

}  // extern "C"
