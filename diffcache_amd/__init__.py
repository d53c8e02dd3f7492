"""diffcache_amd: the decode-time retrieval path of DiffCache on one MI355X.

``DiffCache`` keeps the reference's KV-cache operator API
(src/diffcache/kvcache/diffcache.py), ``DiffCacheHIP`` mirrors its native data
layer (diffcache_cpu/src/lib.rs ``DiffCacheCPU``); both run on hand-written HIP
kernels behind the C ABI of ``include/diffcache_hip.h``.  Importing the package
needs the built ``libdiffcache_hip.so`` (``python diffcache_amd/build.py``).
"""
from . import _hip
from .data_layer import DiffCacheHIP, init_metrics, metrics
from .kvcache import DiffCache

__all__ = ["DiffCache", "DiffCacheHIP", "init_metrics", "metrics", "_hip"]
