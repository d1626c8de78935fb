"""pegaflow_amd — MI355X-native implementation of PegaFlow's layer-wise KV
block transfer path (GPU paged KV cache <-> pinned host pool, by block ID).

Everything that moves bytes runs in ``libpegahip.so`` (hand-written gfx950 HIP
kernels + HIP runtime calls behind a C ABI, ``include/pegahip.h``).  This
package is the host-side mirror of the reference's interfaces for the path.
Importing submodules that touch the library raises if it has not been built.
"""

from .connector import (  # noqa: F401
    KVCacheRegistrationInfo,
    assemble_layer_saves,
    block_shard,
    derive_namespace,
    infer_kv_cache_registration,
    reconcile_hybrid_hit,
    register_kv_caches,
    registration_tensor,
    resolve_transfer_backend,
    storage_group_ids,
)

__all__ = [
    "KVCacheRegistrationInfo",
    "assemble_layer_saves",
    "block_shard",
    "derive_namespace",
    "infer_kv_cache_registration",
    "reconcile_hybrid_hit",
    "register_kv_caches",
    "registration_tensor",
    "resolve_transfer_backend",
    "storage_group_ids",
]
__version__ = "0.1.0"
