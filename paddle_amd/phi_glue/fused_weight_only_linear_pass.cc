// Replacement of paddle/fluid/pir/transforms/gpu/fused_weight_only_linear_pass.cc
// for ROCm builds that carry the gfx950 weight-only kernels.
//
// What the pass does is unchanged: a matmul (optionally followed by an add of a
// 1-D bias, on either side) whose second operand is a persistable fp16/bf16
// [K, N] weight with K % 64 == 0 and N % 16 == 0 becomes
// weight_quantize(w) + weight_only_linear(x, qw, bias, scale).  What differs
// from the file it replaces:
//   * the gate.  The reference asks for an NVIDIA SM version, which is -1
//     without CUDA + CUTLASS (:30-37), and CanApplyOn then refuses every
//     program (:312-318).  Here a HIP build always applies: the gfx950 kernels
//     ignore `arch`, so a fixed tag is written into the attribute.
//   * int4.  The reference routes the weight device -> host -> CPU
//     weight_quantize -> device because its GPU weight_quantize has no int4
//     (:111-136, :241-264).  The gfx950 weight_quantize quantises int4 on the
//     device, so both algos take the same three ops.
//   * group-wise scales.  The pass attribute "weight_only_group_size" (-1, 64
//     or 128; default -1) is handed to both ops (:142, :154 fix it to -1);
//     weights whose K is not a multiple of the group size are left alone.
#include "paddle/fluid/pir/transforms/gpu/fused_weight_only_linear_pass.h"

#include <memory>
#include <string>
#include <utility>

#include "paddle/fluid/pir/dialect/operator/ir/pd_op.h"
#include "paddle/fluid/pir/drr/include/drr_pattern_base.h"
#include "paddle/fluid/pir/utils/general_functions.h"
#include "paddle/pir/include/pass/pass.h"
#include "paddle/pir/include/pass/pass_registry.h"

namespace {

// This file replaces the reference's pass in a ROCm build that links the
// gfx950 kernels; it is not meant for any other build.

// Value of the ops' `arch` attribute.  The gfx950 kernels do not read it; 80
// keeps every arch check above them (Python wrapper, InferMeta) quiet.
int ArchTag() { return 80; }

bool ArchSupported(int arch) { return arch > 0; }

enum class BiasSide { kNone, kAfterMatmul, kBeforeMatmul };  // add(matmul, b) or add(b, matmul)

struct RewriteOptions {
  std::string algo;    // weight_only_int8 | weight_only_int4
  int group_size;      // -1 | 64 | 128
  int arch;
};

// One pattern for the three shapes of the source graph.
class WeightOnlyLinearRewrite : public paddle::drr::DrrPatternBase {
 public:
  WeightOnlyLinearRewrite(BiasSide side, RewriteOptions opt) : side_(side), opt_(std::move(opt)) {}

  std::string name() const override {
    return side_ == BiasSide::kNone ? "WeightOnlyLinearRewriteNoBias" : "WeightOnlyLinearRewriteWithBias";
  }

  // the bias forms must win over the bare matmul they contain
  uint32_t benefit() const override { return side_ == BiasSide::kNone ? 1 : 2; }

  void operator()(paddle::drr::DrrPatternContext *ctx) const override {
    auto src = ctx->SourcePattern();
    const auto &mm = src.Op(paddle::dialect::MatmulOp::name(),
                            {{"transpose_x", src.Attr("tx")}, {"transpose_y", src.Attr("ty")}});
    src.Tensor("mm_out") = mm(src.Tensor("x"), src.Tensor("w"));
    const char *result = "mm_out";
    if (side_ != BiasSide::kNone) {
      const auto &add = src.Op(paddle::dialect::AddOp::name());
      src.Tensor("sum") = side_ == BiasSide::kAfterMatmul ? add(src.Tensor("mm_out"), src.Tensor("bias"))
                                                          : add(src.Tensor("bias"), src.Tensor("mm_out"));
      result = "sum";
    }

    const bool with_bias = side_ != BiasSide::kNone;
    const int group = opt_.group_size;
    src.AddConstraint([with_bias, group](const paddle::drr::MatchContext &m) -> bool {
      if (m.Attr<bool>("tx") || m.Attr<bool>("ty")) return false;
      if (!pir::ValueIsPersistable(m.Tensor("w"))) return false;
      const auto wt = pir::GetDataTypeFromValue(m.Tensor("w"));
      if (!wt.isa<pir::Float16Type>() && !wt.isa<pir::BFloat16Type>()) return false;
      const auto w = pir::GetShapeFromValue(m.Tensor("w"));
      const auto x = pir::GetShapeFromValue(m.Tensor("x"));
      if (w.size() != 2 || x.size() < 2) return false;
      if (with_bias && pir::GetShapeFromValue(m.Tensor("bias")).size() != 1) return false;
      const int64_t K = w[0], N = w[1];
      if (K % 64 != 0 || N % 16 != 0 || x.back() != K) return false;
      if (group > 0 && K % group != 0) return false;
      return true;
    });

    auto res = src.ResultPattern();
    const auto &quantize = res.Op(paddle::dialect::WeightQuantizeOp::name(),
                                  {{"algo", res.StrAttr(opt_.algo)},
                                   {"arch", res.Int32Attr(opt_.arch)},
                                   {"group_size", res.Int32Attr(opt_.group_size)}});
    quantize({&res.Tensor("w")}, {&res.Tensor("qweight"), &res.Tensor("qscale")});
    const auto &linear =
        res.Op(paddle::dialect::WeightOnlyLinearOp::name(),
               {{"weight_dtype", res.StrAttr(opt_.algo == "weight_only_int4" ? "int4" : "int8")},
                {"arch", res.Int32Attr(opt_.arch)},
                {"group_size", res.Int32Attr(opt_.group_size)}});
    linear({&res.Tensor("x"),
            &res.Tensor("qweight"),
            with_bias ? &res.Tensor("bias") : &res.InputNoneTensor(),
            &res.Tensor("qscale")},
           {&res.Tensor(result)});
  }

 private:
  BiasSide side_;
  RewriteOptions opt_;
};

class FusedWeightOnlyLinearPass : public pir::PatternRewritePass {
 public:
  FusedWeightOnlyLinearPass() : pir::PatternRewritePass("fused_weight_only_linear_pass", 4), arch_(ArchTag()) {}

  pir::RewritePatternSet InitializePatterns(pir::IrContext *context) override {
    RewriteOptions opt{"weight_only_int8", -1, arch_};
    if (Has("weight_only_algo")) opt.algo = Get<std::string>("weight_only_algo");
    if (Has("weight_only_group_size")) opt.group_size = Get<int>("weight_only_group_size");
    PADDLE_ENFORCE_EQ(opt.algo == "weight_only_int8" || opt.algo == "weight_only_int4",
                      true,
                      common::errors::InvalidArgument("fused_weight_only_linear_pass only support "
                                                      "weight_only_int8 or weight_only_int4, but get %s.",
                                                      opt.algo));
    PADDLE_ENFORCE_EQ(opt.group_size == -1 || opt.group_size == 64 || opt.group_size == 128,
                      true,
                      common::errors::InvalidArgument("fused_weight_only_linear_pass: weight_only_group_size "
                                                      "must be -1, 64 or 128, but get %d.",
                                                      opt.group_size));
    pir::RewritePatternSet patterns(context);
    for (BiasSide side : {BiasSide::kAfterMatmul, BiasSide::kBeforeMatmul, BiasSide::kNone})
      patterns.Add(paddle::drr::Create<WeightOnlyLinearRewrite>(context, side, opt));
    return patterns;
  }

  pir::GreedyRewriteConfig InitializeConfig() override {
    pir::GreedyRewriteConfig config;
    config.use_top_down_traversal = false;  // users (the add) are visited before the matmul they consume
    config.max_iterations = 10;
    return config;
  }

  bool CanApplyOn(pir::Operation *op) const override { return ArchSupported(arch_) && op->num_regions() > 0; }

 private:
  int arch_;
};

}  // namespace

namespace pir {
std::unique_ptr<Pass> CreateFusedWeightOnlyLinearPass() { return std::make_unique<FusedWeightOnlyLinearPass>(); }
}  // namespace pir

REGISTER_IR_PASS(fused_weight_only_linear_pass, FusedWeightOnlyLinearPass);
