"""``cornstarch.kernel.attention`` is ``cornstarch_amd.kernel.attention``: the very same module object, so
class-level state (flag cache, registered adapters) is shared whichever name a caller imports."""

import sys

from cornstarch_amd.kernel import attention as _impl

sys.modules[__name__] = _impl
