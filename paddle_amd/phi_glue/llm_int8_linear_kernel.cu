// Drop-in replacement of paddle/phi/kernels/gpu/llm_int8_linear_kernel.cu for
// gfx950.  Same template signature (paddle/phi/kernels/llm_int8_linear_kernel.h)
// and registration (gpu/llm_int8_linear_kernel.cu:81-86).  The file it replaces
// throws Unimplemented outside CUDA >= 11.2 (:58-61); this one computes on
// MI355X.  The bias is added inside the library call (the reference runs
// phi::AddKernel afterwards, :55-57: the same T addition).
#include "paddle/phi/kernels/llm_int8_linear_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
#include "wol_phi_common.h"

namespace phi {

template <typename T, typename Context>
void LLMInt8LinearKernel(const Context& dev_ctx,
                         const DenseTensor& x,
                         const DenseTensor& weight,
                         const paddle::optional<DenseTensor>& bias,
                         const DenseTensor& weight_scale,
                         const float threshold,
                         DenseTensor* out) {
  dev_ctx.template Alloc<T>(out);
  const auto w_dims = weight.dims();
  const int64_t k = w_dims[1];  // gpu/llm_int8_linear_kernel.cu:39-41
  const int64_t n = w_dims[0];
  const int64_t m = x.numel() / k;
  if (m == 0) return;
  // scratch: row ranges, outlier mask and list, activation codes, partial sums;
  // the reference allocates the same kinds of temporaries inside LLMGemm
  // (impl/llm_int8_matmul_kernel_impl.h:572-579, :610-616, :657-659)
  DenseTensor workspace;
  const size_t ws_bytes = wol_llm_int8_linear_workspace(m, k, n);
  PADDLE_ENFORCE_GT(ws_bytes,
                    0UL,
                    common::errors::InvalidArgument(
                        "llm_int8_linear: the weight must be [N, K] with K divisible by 64 and N by 16 "
                        "(what weight_quantize(algo='llm.int8') returns), but got [%d, %d]",
                        n,
                        k));
  workspace.Resize({static_cast<int64_t>(ws_bytes)});
  dev_ctx.template Alloc<uint8_t>(&workspace);
  wol_glue::Check(wol_llm_int8_linear(x.data<T>(),
                                      weight.data<int8_t>(),
                                      bias ? bias.get().data<T>() : nullptr,
                                      weight_scale.data<float>(),
                                      threshold,
                                      wol_glue::DTypeTag<T>::value,
                                      m,
                                      k,
                                      n,
                                      out->data<T>(),
                                      workspace.data<uint8_t>(),
                                      ws_bytes,
                                      dev_ctx.stream()),
                  "llm_int8_linear");
}

}  // namespace phi

PD_REGISTER_KERNEL(llm_int8_linear,
                   GPU,
                   ALL_LAYOUT,
                   phi::LLMInt8LinearKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
