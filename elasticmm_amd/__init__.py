"""elasticmm_amd — MI355X-native KV-cache data movement for ElasticMM.

The package holds exactly one hot path: pack / unpack / reshape_and_cache /
copy_blocks (+ the ragged vision-embedding concat) as hand-written gfx950 HIP
kernels behind a C ABI (``include/emm_kv.h``, built into ``libemm_kv.so``), and
the Python surface of the reference worker on top of it.

  build            compile the HIP library in-tree (hipcc, gfx950)
  _lib             ctypes loader; raises if the library is missing
  kv_ops           tensor-level operators (pack, unpack, copy_blocks, append, ...)
  cache_ops        vLLM-shaped ``reshape_and_cache_flash`` / ``copy_blocks``
  worker           ``KVWorker``: the data-path methods of the reference's V0Worker
  pool_transfer    gather/scatter on the legacy monolithic 6-D pool and the vision block pool
  block_manager    host-side free-list block tables (index producer)
  kv_transfer      ``KVTransferManager`` / ``KVMigrationManager``: the callers that move requests between workers
"""
from .build import build_library, library_path  # noqa: F401

__all__ = ["build_library", "library_path"]
