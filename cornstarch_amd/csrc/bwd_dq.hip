// Backward of bitfield-masked attention: the dQ instantiations for sequences of up to 131072 keys, and the dispatch.
#include "bwd_kernels.h"

namespace bam {

int launch_bwd_dq_long(const AttnParams& p, int dtype, hipStream_t stream);  // bwd_long.hip

template <typename T, int D>
static int launch_dq_t(const AttnParams& p, hipStream_t stream) {
    return p.bias != nullptr ? launch_dq_b<T, D, true, false>(p, stream) : launch_dq_b<T, D, false, false>(p, stream);
}

int launch_bwd_dq(const AttnParams& p, int dtype, hipStream_t stream) {
    if (p.Sk > MAX_LIST * DQ_KT) return launch_bwd_dq_long(p, dtype, stream);
    BAM_DISPATCH(launch_dq_t)
}

}  // namespace bam
