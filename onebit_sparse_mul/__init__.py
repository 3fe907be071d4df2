"""Drop-in import name of the reference package: `import onebit_sparse_mul` resolves to onebitsparsemul_amd.

Also makes `import onebit_sparse_cuda` resolve to the compiled binding built in onebitsparsemul_amd/."""
import sys

import onebitsparsemul_amd as _impl
from onebitsparsemul_amd import *  # noqa: F401,F403
from onebitsparsemul_amd import _semi_structured_conversions

sys.modules[__name__ + "._semi_structured_conversions"] = _semi_structured_conversions


def _alias_binding():
    try:
        from onebitsparsemul_amd import onebit_sparse_cuda
    except ImportError:
        return
    sys.modules.setdefault("onebit_sparse_cuda", onebit_sparse_cuda)


_alias_binding()
__all__ = list(_impl.__all__)
