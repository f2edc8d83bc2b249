// Drop-in replacement of paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu
// for gfx950.  Same template signature (paddle/phi/kernels/
// weight_only_linear_grad_kernel.h) and registration (gpu/
// weight_only_linear_grad_kernel.cu:76-81), same composition as the reference
// (:52-69): dequantise the weight to T, then the framework's MatmulKernel.  The
// dequantised weight comes out as [K, N] here (the reference's functor yields
// [N, K]), hence transpose_y.  Group-wise scales and int4 work as well; the
// reference's arch 80/86 and per-channel checks have nothing to guard on AMD.
#include "paddle/phi/kernels/weight_only_linear_grad_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
#include "paddle/phi/kernels/matmul_kernel.h"
#include "wol_phi_common.h"

namespace phi {

template <typename T, typename Context>
void WeightOnlyLinearGradKernel(const Context& dev_ctx,
                                const DenseTensor& x,
                                const DenseTensor& weight,
                                const paddle::optional<DenseTensor>& bias,
                                const DenseTensor& weight_scale,
                                const DenseTensor& out_grad,
                                const std::string& weight_dtype,
                                const int32_t arch,  // ignored on AMD
                                const int32_t group_size,
                                DenseTensor* x_grad) {
  const int bits = wol_glue::Bits(weight_dtype, "weight_only_linear_grad");
  const int64_t n = group_size > 0 ? weight_scale.dims()[1] : weight_scale.dims()[0];
  const int64_t k = weight.dims()[1];
  dev_ctx.template Alloc<T>(x_grad);
  DenseTensor weight_dequantized;
  weight_dequantized.Resize({k, n});
  dev_ctx.template Alloc<T>(&weight_dequantized);
  wol_glue::Check(wol_dequantize(weight.data<int8_t>(),
                                 WOL_LAYOUT_GFX950,
                                 weight_scale.data<T>(),
                                 wol_glue::DTypeTag<T>::value,
                                 k,
                                 n,
                                 bits,
                                 group_size,
                                 weight_dequantized.data<T>(),
                                 dev_ctx.stream()),
                  "weight_only_linear_grad");
  // x_grad[..., K] = out_grad[..., N] . W_dq[K, N]^T
  MatmulKernel<T, Context>(dev_ctx, out_grad, weight_dequantized, false, true, x_grad);
}

}  // namespace phi

PD_REGISTER_KERNEL(weight_only_linear_grad,
                   GPU,
                   ALL_LAYOUT,
                   phi::WeightOnlyLinearGradKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
