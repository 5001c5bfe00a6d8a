"""MI355X-native single-shot all-reduce / all-gather over virtual ranks.

The product is the C ABI in ``include/vrank_allreduce.h`` (built into
``libvrank_allreduce.so`` from ``csrc/``) and the C++ host header
``include/vrank/allreduce.hpp``.  This package is the Python-side binding of that
C ABI (ctypes) used by the tests and the benchmark.
"""
from .binding import (  # noqa: F401
    ALGOS,
    TRANSPORT_DEFAULT,
    TRANSPORT_DIRECT,
    TRANSPORT_WIRE,
    VRError,
    VirtualRanks,
    algo_id,
    build_library,
    check_allreduce,
    launch_geometry,
    direct_launch_plan,
    lib,
    library_path,
    parse_nelems,
)
