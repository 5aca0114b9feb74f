// Contiguous-layout stage-1 kernel instantiated for one element type.
#include "stage1_contig_launch.h"

namespace atk {
namespace contig {
ATK_INSTANTIATE_CONTIG(ATK_F16)
}  // namespace contig
}  // namespace atk
