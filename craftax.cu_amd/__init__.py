"""MI355X (gfx950) implementation of craftax.cu's batched policy path.

The product is libcfpolicy.so (hand-written HIP behind the C ABI of
include/cfp.h); this package is the thin host-side mirror of the reference's
CuPolicy call surface used by the tests and the benchmark.  Importing it loads
the shared library and fails if it has not been built.
"""
from . import _lib
from . import policy
from .policy import Policy, Trainer, lib
from . import env
from .env import Env

lib()  # fail at import time, not at first use, when the HIP library is missing

__all__ = ["Policy", "Trainer", "Env", "policy", "env", "lib", "_lib"]
