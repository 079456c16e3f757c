// Backward of bitfield-masked attention: the dK/dV and dQ instantiations that walk sequences beyond 131072 tokens in
// several passes.
#include "bwd_kernels.h"

namespace bam {

template <typename T, int D>
static int launch_dkdv_long_t(const AttnParams& p, hipStream_t stream) {
    return p.bias != nullptr ? launch_dkdv_b<T, D, true, true>(p, stream) : launch_dkdv_b<T, D, false, true>(p, stream);
}
template <typename T, int D>
static int launch_dq_long_t(const AttnParams& p, hipStream_t stream) {
    return p.bias != nullptr ? launch_dq_b<T, D, true, true>(p, stream) : launch_dq_b<T, D, false, true>(p, stream);
}

int launch_bwd_dkdv_long(const AttnParams& p, int dtype, hipStream_t stream) { BAM_DISPATCH(launch_dkdv_long_t) }
int launch_bwd_dq_long(const AttnParams& p, int dtype, hipStream_t stream) { BAM_DISPATCH(launch_dq_long_t) }

}  // namespace bam
