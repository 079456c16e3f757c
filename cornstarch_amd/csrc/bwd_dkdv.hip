// Backward of bitfield-masked attention: delta pre-pass and the dK/dV instantiations for sequences of up to 131072
// rows, with their dispatch.
#include "bwd_kernels.h"

namespace bam {

int launch_bwd_dkdv_long(const AttnParams& p, int dtype, hipStream_t stream);  // bwd_long.hip

template <typename T, int D>
static int launch_pre_t(const AttnParams& p, hipStream_t stream) {
    const int64_t threads = (int64_t)p.B * p.Sq * p.Hq * (D / 8);
    const int64_t blocks = (threads + 255) / 256;
    hipLaunchKernelGGL((bwd_preprocess_kernel<T, D>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}
template <typename T, int D>
static int launch_dkdv_t(const AttnParams& p, hipStream_t stream) {
    return p.bias != nullptr ? launch_dkdv_b<T, D, true, false>(p, stream) : launch_dkdv_b<T, D, false, false>(p, stream);
}

int launch_bwd_preprocess(const AttnParams& p, int dtype, hipStream_t stream) { BAM_DISPATCH(launch_pre_t) }
int launch_bwd_dkdv(const AttnParams& p, int dtype, hipStream_t stream) {
    if (p.Sq > MAX_SLICE_LIST * 32) return launch_bwd_dkdv_long(p, dtype, stream);
    BAM_DISPATCH(launch_dkdv_t)
}

}  // namespace bam
