// Drop-in replacement of paddle/phi/kernels/gpu/weight_quantize_kernel.cu for
// gfx950.  Same template signature (paddle/phi/kernels/weight_quantize_kernel.h:
// 21-28) and registration (gpu/weight_quantize_kernel.cu:118-123).  Unlike the
// file it replaces, it produces the CPU kernel's codes and scales bit for bit,
// supports group_size 64/128, int4 and the 'llm.int8' flavour on the device,
// and launches on dev_ctx.stream() rather than the null stream.
#include "paddle/phi/kernels/weight_quantize_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
#include "wol_phi_common.h"

namespace phi {

template <typename T, typename Context>
void WeightQuantizeKernel(const Context& dev_ctx,
                          const DenseTensor& x,
                          const std::string& algo,
                          const int32_t arch,  // ignored on AMD, as in the reference's HIP build
                          const int32_t group_size,
                          DenseTensor* out,
                          DenseTensor* scale) {
  PADDLE_ENFORCE_EQ(algo == "weight_only_int8" || algo == "weight_only_int4" || algo == "llm.int8",
                    true,
                    common::errors::Unimplemented(
                        "The algo must be in ['weight_only_int8', 'weight_only_int4', "
                        "'llm.int8'], but got[%s]",
                        algo));
  const bool llm = algo == "llm.int8";
  const int bits = llm ? 8 : wol_glue::Bits(algo, "weight_quantize");
  const auto dims = x.dims();
  const int64_t K = dims[0], N = dims[1];
  dev_ctx.template Alloc<int8_t>(out);   // [N, K] or [N/2, K], set by WeightQuantizeInferMeta
  DenseTensor workspace;
  const size_t ws_bytes = wol_quantize_workspace(K, N, bits, group_size);
  void* ws = nullptr;
  if (ws_bytes > 0) {
    workspace.Resize({static_cast<int64_t>(ws_bytes)});
    ws = dev_ctx.template Alloc<uint8_t>(&workspace);
  }
  if (llm) {
    // fp32 scales and the plain [N, K] transpose, as the reference returns them
    // for this algo (cpu/weight_quantize_kernel.cc:108-111, :163-166)
    dev_ctx.template Alloc<float>(scale);
    wol_glue::Check(wol_quantize_llm_int8(x.data<T>(),
                                          wol_glue::DTypeTag<T>::value,
                                          K,
                                          N,
                                          group_size,
                                          WOL_LAYOUT_PADDLE_HIP,
                                          out->data<int8_t>(),
                                          scale->data<float>(),
                                          ws,
                                          ws_bytes,
                                          dev_ctx.stream()),
                    "weight_quantize");
    return;
  }
  dev_ctx.template Alloc<T>(scale);      // [N] or [ceil(K/group_size), N]
  wol_glue::Check(wol_quantize(x.data<T>(),
                               wol_glue::DTypeTag<T>::value,
                               K,
                               N,
                               bits,
                               group_size,
                               WOL_ROUND_RNE,
                               WOL_LAYOUT_GFX950,
                               out->data<int8_t>(),
                               scale->data<T>(),
                               ws,
                               ws_bytes,
                               dev_ctx.stream()),
                  "weight_quantize");
}

}  // namespace phi

PD_REGISTER_KERNEL(weight_quantize,
                   GPU,
                   ALL_LAYOUT,
                   phi::WeightQuantizeKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
