"""``cornstarch.kernel.bitfield_attention`` is ``cornstarch_amd.kernel.bitfield_attention``: the very same module object, so
class-level state (flag cache, registered adapters) is shared whichever name a caller imports."""

import sys

from cornstarch_amd.kernel import bitfield_attention as _impl

sys.modules[__name__] = _impl
