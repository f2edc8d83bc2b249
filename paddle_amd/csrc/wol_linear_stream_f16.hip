// The fp16 half of the streaming kernel's instantiations: the same source as
// wol_linear_stream.hip, which with this macro defines launch_linear_stream_f16
// and nothing of the host-side planning.
#define WOL_STREAM_F16_TU 1
#include "wol_linear_stream.hip"
