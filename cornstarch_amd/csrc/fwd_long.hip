// Forward of bitfield-masked attention: the instantiations that walk sequences beyond 131072 keys in several passes.
#include "fwd_kernel.h"

namespace bam {

int launch_fwd_long(const AttnParams& p, int dtype, hipStream_t stream) { return launch_fwd_all<true>(p, dtype, stream); }

}  // namespace bam
