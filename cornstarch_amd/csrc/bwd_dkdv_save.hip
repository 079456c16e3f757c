// Backward of bitfield-masked attention: the dK/dV instantiations that also store dS for the dQ kernel of
// bwd_dq_saved.h (head dim 128, sequences of up to 131072 rows, plan required).
#include "bwd_kernels.h"

namespace bam {

template <typename T, int D>
static int launch_dkdv_save_t(const AttnParams& p, hipStream_t stream) {
    return p.bias != nullptr ? launch_dkdv_save_b<T, D, true>(p, stream) : launch_dkdv_save_b<T, D, false>(p, stream);
}

int launch_bwd_dkdv_save(const AttnParams& p, int dtype, hipStream_t stream) {
    // (at head dim 64 the stores cost dK/dV more than the dQ kernel saves: half the arithmetic per stored byte)
    return dtype == 1 ? launch_dkdv_save_t<BF16, 128>(p, stream) : launch_dkdv_save_t<F16, 128>(p, stream);
}

}  // namespace bam
