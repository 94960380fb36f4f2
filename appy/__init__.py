"""``import appy`` resolves to :mod:`appy_amd`, so programs written for the
reference package (``import appy`` / ``@appy.jit``) run unchanged."""
import sys as _sys

import appy_amd as _impl

_sys.modules[__name__] = _impl
