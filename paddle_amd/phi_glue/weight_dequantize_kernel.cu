// Drop-in replacement of paddle/phi/kernels/gpu/weight_dequantize_kernel.cu for
// gfx950.  Same template signature (paddle/phi/kernels/weight_dequantize_kernel.h:
// 21-28) and registration (gpu/weight_dequantize_kernel.cu:479-484).  Writes the
// [K, N] result directly; the file it replaces writes [N, K] and transposes.
#include "paddle/phi/kernels/weight_dequantize_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
#include "wol_phi_common.h"

namespace phi {

template <typename T, typename Context>
void WeightDequantizeKernel(const Context& dev_ctx,
                            const DenseTensor& x,
                            const DenseTensor& scale,
                            const std::string& algo,
                            DataType out_dtype,
                            int32_t group_size,
                            DenseTensor* out) {
  const int bits = wol_glue::Bits(algo, "weight_dequantize");
  const auto out_dims = out->dims();  // [K, N] from WeightDequantizeInferMeta
  dev_ctx.template Alloc<T>(out);
  wol_glue::Check(wol_dequantize(x.data<int8_t>(),
                                 WOL_LAYOUT_GFX950,
                                 scale.data<T>(),
                                 wol_glue::DTypeTag<T>::value,
                                 out_dims[0],
                                 out_dims[1],
                                 bits,
                                 group_size,
                                 out->data<T>(),
                                 dev_ctx.stream()),
                  "weight_dequantize");
}

}  // namespace phi

PD_REGISTER_KERNEL(weight_dequantize,
                   GPU,
                   ALL_LAYOUT,
                   phi::WeightDequantizeKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
