// Shared helpers of the PHI glue: dtype tag, status -> PADDLE_THROW.
#pragma once

#include "paddle/phi/backends/gpu/gpu_context.h"
#include "paddle/phi/common/bfloat16.h"
#include "paddle/phi/common/float16.h"
#include "paddle/phi/core/dense_tensor.h"
#include "paddle/phi/core/enforce.h"
#include "wol_c_api.h"

namespace phi {
namespace wol_glue {

template <typename T>
struct DTypeTag;
template <>
struct DTypeTag<phi::dtype::float16> {
  static constexpr int value = WOL_DTYPE_F16;
};
template <>
struct DTypeTag<phi::dtype::bfloat16> {
  static constexpr int value = WOL_DTYPE_BF16;
};

// Argument errors become InvalidArgument (what the reference's InferMeta and
// kernels raise for the same conditions); launch failures become External.
inline void Check(int status, const char* op) {
  if (status == WOL_OK) return;
  if (status >= WOL_ERR_NULL_POINTER && status <= WOL_ERR_ALIGNMENT) {
    PADDLE_THROW(common::errors::InvalidArgument("%s: %s", op, wol_status_str(status)));
  }
  PADDLE_THROW(common::errors::External("%s: %s", op, wol_status_str(status)));
}

inline int Bits(const std::string& algo_or_dtype, const char* op) {
  if (algo_or_dtype == "weight_only_int8" || algo_or_dtype == "int8") return 8;
  if (algo_or_dtype == "weight_only_int4" || algo_or_dtype == "int4") return 4;
  PADDLE_THROW(common::errors::InvalidArgument(
      "%s: the algo must be 'weight_only_int8' or 'weight_only_int4' (weight_dtype 'int8' or "
      "'int4'), but got[%s]",
      op,
      algo_or_dtype));
}

}  // namespace wol_glue
}  // namespace phi
