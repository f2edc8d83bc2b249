// Drop-in replacement of paddle/phi/kernels/gpu/apply_per_channel_scale_kernel.cu
// for gfx950.  Same template signature
// (paddle/phi/kernels/apply_per_channel_scale_kernel.h) and registration
// (gpu/apply_per_channel_scale_kernel.cu:201-206).  The file it replaces has a
// body only in CUDA builds and is left out of ROCm builds
// (paddle/phi/kernels/CMakeLists.txt:233); this one is compiled in both.
#include "paddle/phi/kernels/apply_per_channel_scale_kernel.h"

#include "paddle/phi/core/kernel_registry.h"
#include "wol_phi_common.h"

namespace phi {

template <typename T, typename Context>
void ApplyPerChannelScaleKernel(const Context& dev_ctx,
                                const DenseTensor& x,
                                const DenseTensor& scales,
                                DenseTensor* out) {
  const int64_t rows = x.dims()[0];  // rank 2 by ApplyPerChannelScaleInferMeta
  const int64_t cols = x.dims()[1];
  dev_ctx.template Alloc<T>(out);
  wol_glue::Check(wol_apply_per_channel_scale(x.data<T>(),
                                              scales.data<T>(),
                                              wol_glue::DTypeTag<T>::value,
                                              rows,
                                              cols,
                                              out->data<T>(),
                                              dev_ctx.stream()),
                  "apply_per_channel_scale");
}

}  // namespace phi

PD_REGISTER_KERNEL(apply_per_channel_scale,
                   GPU,
                   ALL_LAYOUT,
                   phi::ApplyPerChannelScaleKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
