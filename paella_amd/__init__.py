"""paella_amd -- MI355X-native serving hot path of Paella/LLIS (host-side Python bindings).

The product is the set of shared libraries under paella_amd/lib (built from paella_amd/csrc by
`make -C paella_amd/csrc`) and the executables under paella_amd/bin.  This package only binds their
C-ABI (include/*.h) through ctypes for tests and benches; there is no CPU fallback anywhere: a missing
library or a missing GPU is an error.
"""
from . import _abi  # noqa: F401
