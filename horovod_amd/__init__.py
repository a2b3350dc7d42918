"""MI355X (gfx950) implementation of Horovod's single-GPU gradient hot path.

The product is the C-ABI shared library ``horovod_amd/lib/libhvdhip.so``
(declared in ``include/hvdhip.h``).  This package only loads it and wraps its
handles for tests and benchmarks; there is no CPU fallback: if the library is
missing, loading raises.
"""
from ._lib import (  # noqa: F401
    DTYPE, HvdHipError, dtype_size, lib, lib_path, check,
)
from .host import AdasumPlan, FusionPlan, Stream, Timer  # noqa: F401
