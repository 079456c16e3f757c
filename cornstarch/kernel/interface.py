"""``cornstarch.kernel.interface`` is ``cornstarch_amd.kernel.interface``: the very same module object, so
class-level state (flag cache, registered adapters) is shared whichever name a caller imports."""

import sys

from cornstarch_amd.kernel import interface as _impl

sys.modules[__name__] = _impl
