// Forward of bitfield-masked attention: the instantiations for sequences of up to 131072 keys, and the dispatch.
#include "fwd_kernel.h"

namespace bam {

int launch_fwd_long(const AttnParams& p, int dtype, hipStream_t stream);  // fwd_long.hip

int launch_fwd(const AttnParams& p, int dtype, hipStream_t stream) {
    if (p.Sk > MAX_LIST * FWD_KT) return launch_fwd_long(p, dtype, stream);
    return launch_fwd_all<false>(p, dtype, stream);
}

}  // namespace bam
