"""``cornstarch`` import path for the MI355X kernels.

The reference's callers import the attention kernels as ``cornstarch.kernel.bitfield_attention``,
``cornstarch.kernel.attention`` and ``cornstarch.kernel.interface`` (e.g.
cornstarch/shardformer/layers/utils.py:11-12, cornstarch/shardformer/modeling/llama.py:31,
cornstarch/models/multimodal_language_model/modeling_multimodal_language_model.py:37).  This package serves
exactly those three modules from ``cornstarch_amd.kernel`` and nothing else.  When a Cornstarch checkout or
install sits further down ``sys.path``, its directories are appended to this package's search path, so every
other subpackage (``cornstarch.shardformer``, ``cornstarch.models``, ...) still resolves there, while
``cornstarch.kernel`` resolves here.
"""

import os as _os
import sys as _sys

__version__ = "0.0.5+mi355x"

_here = _os.path.dirname(_os.path.abspath(__file__))
for _entry in list(_sys.path):
    _cand = _os.path.join(_os.path.abspath(_entry or "."), "cornstarch")
    if _cand != _here and _cand not in __path__ and _os.path.isfile(_os.path.join(_cand, "__init__.py")):
        __path__.append(_cand)
