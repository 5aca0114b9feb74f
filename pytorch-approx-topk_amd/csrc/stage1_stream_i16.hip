// Streaming stage-1 kernels instantiated for one element type.
#include "stage1_stream_launch.h"

namespace atk {
namespace stream {
ATK_INSTANTIATE_STREAM(ATK_I16)
}  // namespace stream
}  // namespace atk
