// Replacement of paddle/phi/kernels/fusion/cutlass/moe_ffn.cu for gfx950 and the
// weight-only quant methods.  Same template signature (:36-45) and registration
// (:189-199).  The file it replaces is built on CUTLASS grouped GEMMs (:74-183)
// and is not compiled on ROCm; quant_method "None" (dense experts) stays with
// whatever the build provides and is refused here.
#include "paddle/phi/core/kernel_registry.h"
#include "wol_phi_common.h"

namespace phi {
namespace fusion {

template <typename T, typename Context>
void MoeFFNKernel(const Context& ctx,
                  const DenseTensor& permute_input,
                  const DenseTensor& token_nums_per_expert,
                  const DenseTensor& ffn1_weight,
                  const DenseTensor& ffn2_weight,
                  const paddle::optional<DenseTensor>& ffn1_bias,
                  const paddle::optional<DenseTensor>& ffn1_scale,
                  const paddle::optional<DenseTensor>& ffn2_scale,
                  const std::string& quant_method,
                  DenseTensor* ffn_out) {
  ffn_out->Resize(permute_input.dims());
  T* out = ctx.template Alloc<T>(ffn_out);
  const int bits = wol_glue::Bits(quant_method, "moe_ffn");
  PADDLE_ENFORCE_EQ(ffn1_scale && ffn2_scale,
                    true,
                    common::errors::InvalidArgument(
                        "moe_ffn: ffn1_scale and ffn2_scale are required for %s", quant_method));
  // dims as the reference reads them (:70-76): experts stacked along dim 0;
  // the weights are the per-expert outputs of weight_quantize, [E, inter(/2), hidden]
  const int64_t rows = permute_input.dims()[0];
  const int64_t hidden = permute_input.dims()[1];
  const int num_experts = static_cast<int>(ffn1_weight.dims()[0]);
  const int64_t inter = ffn1_scale.get().dims()[1];
  DenseTensor workspace;
  const size_t ws_bytes = wol_moe_ffn_workspace(rows, hidden, inter, num_experts);
  void* ws = nullptr;
  if (ws_bytes > 0) {
    workspace.Resize({static_cast<int64_t>(ws_bytes)});
    ws = ctx.template Alloc<uint8_t>(&workspace);
  }
  wol_glue::Check(wol_moe_ffn(permute_input.data<T>(),
                              token_nums_per_expert.data<int64_t>(),
                              ffn1_weight.data<int8_t>(),
                              ffn1_bias ? ffn1_bias.get().data<T>() : nullptr,
                              ffn1_scale.get().data<T>(),
                              ffn2_weight.data<int8_t>(),
                              ffn2_scale.get().data<T>(),
                              wol_glue::DTypeTag<T>::value,
                              rows,
                              hidden,
                              inter,
                              num_experts,
                              bits,
                              out,
                              ws,
                              ws_bytes,
                              ctx.stream()),
                  "moe_ffn");
}

}  // namespace fusion
}  // namespace phi

PD_REGISTER_KERNEL(moe_ffn,
                   GPU,
                   ALL_LAYOUT,
                   phi::fusion::MoeFFNKernel,
                   phi::dtype::float16,
                   phi::dtype::bfloat16) {}
