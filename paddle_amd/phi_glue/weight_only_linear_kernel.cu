// Drop-in replacement of paddle/phi/kernels/gpu/weight_only_linear_kernel.cu for
// gfx950.  Same template signature (paddle/phi/kernels/weight_only_linear_kernel.h:
// 21-30) and registration (gpu/weight_only_linear_kernel.cu:204-209).  The file
// it replaces throws "Please compile with cutlass" on ROCm.
#include "paddle/phi/kernels/weight_only_linear_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
#include "wol_phi_common.h"

namespace phi {

template <typename T, typename Context>
void WeightOnlyLinearKernel(const Context& dev_ctx,
                            const DenseTensor& x,
                            const DenseTensor& weight,
                            const paddle::optional<DenseTensor>& bias,
                            const DenseTensor& weight_scale,
                            const std::string& weight_dtype,
                            const int32_t arch,  // ignored on AMD
                            const int32_t group_size,
                            DenseTensor* out) {
  const int bits = wol_glue::Bits(weight_dtype, "weight_only_linear");
  dev_ctx.template Alloc<T>(out);
  // n, k, m as the reference derives them (gpu/weight_only_linear_kernel.cu:56-58)
  const int64_t n = group_size > 0 ? weight_scale.dims()[1] : weight_scale.dims()[0];
  const int64_t k = weight.dims()[1];
  const int64_t m = x.numel() / k;
  DenseTensor workspace;
  const size_t ws_bytes = wol_linear_workspace(m, k, n, bits, group_size);
  void* ws = nullptr;
  if (ws_bytes > 0) {
    workspace.Resize({static_cast<int64_t>(ws_bytes)});
    ws = dev_ctx.template Alloc<uint8_t>(&workspace);
  }
  wol_glue::Check(wol_linear(x.data<T>(),
                             weight.data<int8_t>(),
                             bias ? bias.get().data<T>() : nullptr,
                             weight_scale.data<T>(),
                             wol_glue::DTypeTag<T>::value,
                             m,
                             k,
                             n,
                             bits,
                             group_size,
                             out->data<T>(),
                             ws,
                             ws_bytes,
                             dev_ctx.stream()),
                  "weight_only_linear");
}

}  // namespace phi

PD_REGISTER_KERNEL(weight_only_linear,
                   GPU,
                   ALL_LAYOUT,
                   phi::WeightOnlyLinearKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
