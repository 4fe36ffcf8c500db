"""MI355X-native DFlash speculative-verify kernels behind the reference's own API.

``DFlashKernels`` / ``DFlashKernelRegistry`` mirror Sources/DFlash/DFlashKernels.swift and
DFlashKernelProvider.swift; the caches mirror Sources/DFlash/RecurrentRollbackCache.swift;
``DFlashRuntime`` and the engines mirror the accept/rollback part of
Sources/DFlash/DFlashRuntime.swift and DFlashEngine.swift.  All compute happens in
``lib/libdflash_hip.so`` (hand-written HIP for gfx950); there is no fallback path.
"""

from ._lib import DFlashError, DFlashUnsupported, LIB_PATH  # noqa: F401
from .dflash_kernels import (DFlashKernelProvider, DFlashKernelRegistry, DFlashKernels,  # noqa: F401
                             DFlashKernelsInstance)
from .rollback_cache import (KVCacheSimple, MambaCache, MambaSnapshotCache,  # noqa: F401
                             RecurrentRollbackCache)
from .runtime import (AcceptResult, DFlashEngine, DFlashRuntime, FullAttentionEngine,  # noqa: F401
                      HybridGDNEngine, committed_segment, verify_ids_for_block)
