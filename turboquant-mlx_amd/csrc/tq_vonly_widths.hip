// The matrix-core tile passes over packed VALUES of 1, 2 and 4 bits -- the V-only decode step and the given-weights
// pass of sparse_v_matvec / the thresholded step -- (the 3-bit instantiations live beside the host code in
// tq_attn.hip): a translation unit of its own so that the widths compile in parallel.
#define TQ_VONLY_OTHER_WIDTHS_HERE
#include "tq_packed_mfma.h"

namespace tqm {
template void launch_vonly_tiles<1>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
template void launch_vonly_tiles<2>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
template void launch_vonly_tiles<4>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
template void launch_given_tiles<1>(int, dim3, const PackedArgs&, const Codebook&, const Codebook&, hipStream_t);
template void launch_given_tiles<2>(int, dim3, const PackedArgs&, const Codebook&, const Codebook&, hipStream_t);
template void launch_given_tiles<4>(int, dim3, const PackedArgs&, const Codebook&, const Codebook&, hipStream_t);
}  // namespace tqm
