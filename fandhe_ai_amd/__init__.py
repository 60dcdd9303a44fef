"""MI355X-native quantized decode path behind the reference's backend interface.

``fandhe_ai_amd.backend`` mirrors the reference's ``BackendOps`` / ``MemoryOps``
surface for ``Device::Rocm``; ``fandhe_ai_amd.capi`` is the ctypes view of the C
ABI (include/fandhe_rocm.h) in ``lib/libfandhe_rocm.so``.
"""
from . import capi  # noqa: F401  (raises if the HIP library is not built)
from .backend import *  # noqa: F401,F403
from .paged_cache import BlockTable, PagedKvCache, PagedKvCacheConfig  # noqa: F401,E402
from .decoder import Decoder  # noqa: F401,E402
from . import safetensors_io  # noqa: F401,E402
from . import scheduler  # noqa: F401,E402
