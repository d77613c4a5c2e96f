// kvc_fused_mfma_v96.hip -- the matrix-core V kernel for one query head per KV head and tiles that may straddle two
// heads (head_dim no multiple of 64, e.g. 96), softmax on the fly: <1, 4, ROUNDED> of kvc_fused_mfma_impl.h, compiled by
// itself.  Beside the kernel's other instances the register allocator needs 77 vector registers for it (six waves per
// SIMD) and spills 13 when held to the 72 of seven waves; by itself it fits 72 without a spill.
#include "kvc_fused_mfma_impl.h"

template __global__ void kvc_fused_mfma_kernel<1, 4, true>(KvcFusedArgs);
template __global__ void kvc_fused_mfma_kernel<1, 4, false>(KvcFusedArgs);
