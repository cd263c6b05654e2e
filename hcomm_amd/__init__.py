"""hcomm_amd - MI355X-native local copy / reduce engine behind HCOMM's collective schedules.

The product is ``hcomm_amd/csrc/libhcomm_gfx.so`` (C host code + hand-written gfx950 kernels, C ABI declared
in ``include/hcomm_gfx.h``).  This package is the thin Python mirror of that ABI used by the tests and the
benchmark: same function names, argument meaning and return codes as the reference's operator interface
(``include/hcomm_primitives.h``, ``include/hcomm_res.h`` in the reference tree).
"""
from .api import *  # noqa: F401,F403
from .api import __all__  # noqa: F401
