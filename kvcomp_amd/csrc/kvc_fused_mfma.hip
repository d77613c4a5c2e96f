// kvc_fused_mfma.hip -- launchers of the matrix-core fused decode + matvec kernels (kvc_fused_mfma_impl.h) and all of
// their instances but the ones that have a translation unit of their own (kvc_fused_mfma_v96.hip).
#include "kvc_fused_mfma_impl.h"

// compiled in kvc_fused_mfma_v96.hip
extern template __global__ void kvc_fused_mfma_kernel<1, 4, true>(KvcFusedArgs);
extern template __global__ void kvc_fused_mfma_kernel<1, 4, false>(KvcFusedArgs);

template <int REP, bool ROUNDED>
static void kvc_launch_mfma_kind(int kind, const KvcFusedArgs &a, dim3 grid, size_t lds, hipStream_t stream)
{
    if (kind == 0) hipLaunchKernelGGL((kvc_fused_mfma_kernel<REP, 0, ROUNDED>), grid, dim3(KVC_WG), lds, stream, a);
    else if (kind == 1) hipLaunchKernelGGL((kvc_fused_mfma_kernel<REP, 1, ROUNDED>), grid, dim3(KVC_WG), lds, stream, a);
    else if (kind == 2) hipLaunchKernelGGL((kvc_fused_mfma_kernel<REP, 2, ROUNDED>), grid, dim3(KVC_WG), lds, stream, a);
    else if (kind == 3) hipLaunchKernelGGL((kvc_fused_mfma_kernel<REP, 3, ROUNDED>), grid, dim3(KVC_WG), lds, stream, a);
    else hipLaunchKernelGGL((kvc_fused_mfma_kernel<REP, 4, ROUNDED>), grid, dim3(KVC_WG), lds, stream, a);
}

void kvc_launch_fused_mfma(int rep, int kind, bool rounded, const KvcFusedArgs &a, dim3 grid, size_t lds, hipStream_t stream)
{
#define KVC_MFMA_REP(R)                                                         \
    if (rounded) kvc_launch_mfma_kind<R, true>(kind, a, grid, lds, stream);     \
    else kvc_launch_mfma_kind<R, false>(kind, a, grid, lds, stream)
    switch (rep) {
        case 1: KVC_MFMA_REP(1); break;
        case 2: KVC_MFMA_REP(2); break;
        case 4: KVC_MFMA_REP(4); break;
        default: KVC_MFMA_REP(8); break;
    }
#undef KVC_MFMA_REP
}
