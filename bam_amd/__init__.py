"""MI355X-native GPU-side storage-access path (page cache + NVMe queues on gfx950).

The device path lives in ``libbam_amd.so`` (hand-written HIP, built in-tree by
``bam_amd/csrc/Makefile``) and is reached through its C-ABI (``include/bam_amd.h``).
This package is the Python host-side mirror of the reference's host objects
(Controller, page_cache_t, range_t, array_t) on top of that ABI.  There is no
CPU fallback: without the built library every call raises.
"""
from ._lib import load, load_host, LibraryMissing  # noqa: F401
from .host import Target, Controller, PageCache, Range, Array, Range32, Array32, sssp, sssp_float, vectoradd, BamError  # noqa: F401
from . import gen  # noqa: F401
