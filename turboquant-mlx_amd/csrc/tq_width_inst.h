// Explicit instantiations of the matrix-core launchers for the width TQ_WIDTH_HERE (1, 2 or 4 bits; the 3-bit ones
// are instantiated beside the host code of the entry points).  Included by tq_width1.hip, tq_width2.hip and
// tq_width4.hip, one translation unit per width so that they compile in parallel.
#include "tq_split_mfma.h"

namespace tqm {
template void launch_vonly_tiles<TQ_WIDTH_HERE>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
TQ_PACKED_LAUNCHERS(, TQ_WIDTH_HERE)
template void launch_split_tiles<TQ_WIDTH_HERE>(int, dim3, const SplitArgs&, const Codebook&, hipStream_t);
}  // namespace tqm
