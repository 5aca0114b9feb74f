// Streaming stage-1 kernels instantiated for one element type.
#include "stage1_stream_launch.h"

namespace atk {
namespace stream {
ATK_INSTANTIATE_STREAM(ATK_F16)
}  // namespace stream
}  // namespace atk

ATK_TRACE_READER(atk_trace_stage1_stream_f16)  // (nothing, unless the library is built for the phase timelines)
