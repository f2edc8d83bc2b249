// Drop-in replacement of paddle/phi/kernels/gpu/weight_only_linear_grad_kernel.cu
// for gfx950.  Same template signature (paddle/phi/kernels/
// weight_only_linear_grad_kernel.h) and registration (gpu/
// weight_only_linear_grad_kernel.cu:76-81).  The reference dequantises the
// whole weight to T and calls the framework's MatmulKernel (:52-69); here
// wol_linear_grad contracts out_grad with the packed codes directly, so no
// dequantised copy of the weight exists and no library GEMM is involved.
// Group-wise scales and int4 work as well; the reference's arch 80/86 and
// per-channel checks (:38-49) have nothing to guard on AMD.  x only gives the
// shape of x_grad (no_need_buffer, backward.yaml:3651-3661); bias gets no gradient.
#include "paddle/phi/kernels/weight_only_linear_grad_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
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
  const int64_t m = out_grad.numel() / n;
  dev_ctx.template Alloc<T>(x_grad);
  if (m == 0) return;
  DenseTensor workspace;
  const size_t ws_bytes = wol_linear_grad_workspace(m, k, n, bits, group_size);
  workspace.Resize({static_cast<int64_t>(ws_bytes)});
  void* ws = dev_ctx.template Alloc<uint8_t>(&workspace);
  // x_grad[..., K] = out_grad[..., N] . dequant(W)[K, N]^T
  wol_glue::Check(wol_linear_grad(out_grad.data<T>(),
                                  weight.data<int8_t>(),
                                  weight_scale.data<T>(),
                                  wol_glue::DTypeTag<T>::value,
                                  m,
                                  k,
                                  n,
                                  bits,
                                  group_size,
                                  x_grad->data<T>(),
                                  ws,
                                  ws_bytes,
                                  dev_ctx.stream()),
                  "weight_only_linear_grad");
}

}  // namespace phi

PD_REGISTER_KERNEL(weight_only_linear_grad,
                   GPU,
                   ALL_LAYOUT,
                   phi::WeightOnlyLinearGradKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
