// Backward of bitfield-masked attention: dQ from the dS blocks the dK/dV kernel stored (head dim 128).
#include "bwd_dq_saved.h"

namespace bam {

template <typename T, int D>
static int launch_dq_saved_t(const AttnParams& p, hipStream_t stream) {
    const int blocks = p.num_m * p.B * p.Hq;
    hipLaunchKernelGGL((bwd_dq_saved_kernel<T, D>), dim3(blocks), dim3(DQS_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

int launch_bwd_dq_saved(const AttnParams& p, int dtype, hipStream_t stream) {
    return dtype == 1 ? launch_dq_saved_t<BF16, 128>(p, stream) : launch_dq_saved_t<F16, 128>(p, stream);
}

}  // namespace bam
