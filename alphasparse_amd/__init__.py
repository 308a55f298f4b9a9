"""alphasparse_amd: MI355X-native SpMV format-and-kernel generator (host-side Python mirror).

The product is the C++/HIP library ``libalphasparse_amd.so``; this package only binds its
C ABI so that tests and benchmarks read like the upstream drivers."""
from . import _capi as capi  # noqa: F401
from ._capi import AlphaSparseError  # noqa: F401
from .matrix import Matrix  # noqa: F401
from .builder import Builder, DeviceArray, Stream, device_count, device_facts, device_memory_free_bytes, kernel_cache_stats, template_is_supported  # noqa: F401
from .search import find_best_graph, part_execute_code_builder, execute_code_builder  # noqa: F401
