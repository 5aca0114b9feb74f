// Fused one-workgroup-per-row kernel instantiated for one element type.
#include "fused_row_launch.h"

namespace atk {
namespace fused {
ATK_INSTANTIATE_FUSED(ATK_F32)
}  // namespace fused
}  // namespace atk

ATK_TRACE_READER(atk_trace_fused_row_f32)  // (nothing, unless the library is built for the phase timelines)
