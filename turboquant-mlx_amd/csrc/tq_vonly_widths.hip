// The matrix-core tile pass of the V-only decode step for values of 1, 2 and 4 bits (the 3-bit instantiation
// lives beside the host code in tq_attn.hip): a translation unit of its own so that the widths compile in parallel.
#define TQ_VONLY_OTHER_WIDTHS_HERE
#include "tq_decode_mfma.h"

namespace tqm {
template void launch_vonly_tiles<1>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
template void launch_vonly_tiles<2>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
template void launch_vonly_tiles<4>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
}  // namespace tqm
