"""bittorch_amd: MI355X (gfx950) ternary-linear backend with BitTorch's Python API.

``import bittorch_amd as bittorch`` gives the same ``nn`` / ``ops`` / ``quant``
surface as the reference package; the device work runs in hand-written HIP
kernels behind a C-ABI library (``_hip/libbittorch_hip.so``).
"""

__version__ = "0.2.0"

import torch  # noqa: F401  (loads the ROCm runtime libraries the HIP library links to)

from . import nn, ops, quant, utils  # noqa: E402

try:
    from . import _C  # noqa: F401,E402
    _HAS_CUDA_EXT = True
except ImportError:
    _HAS_CUDA_EXT = False


def has_cuda_ext() -> bool:
    """True when the HIP library is built and loadable (name kept from the reference).  A process that imported the
    package before the library was built finds it here on the next call."""
    global _HAS_CUDA_EXT
    if not _HAS_CUDA_EXT:
        try:
            from . import _C  # noqa: F401
            _HAS_CUDA_EXT = True
        except ImportError:
            pass
    return _HAS_CUDA_EXT
