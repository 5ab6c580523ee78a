"""Import seam `core.moe_cuda_wrapper`.

The reference model does `from core.moe_cuda_wrapper import MoECUDAOps`
(Src/Main_Scripts/core/model.py:78-84); the capacity layer of that module is
exported under its reference name as well.
"""
from adaptivetrainingsystem_amd import _lib
from adaptivetrainingsystem_amd.layers import CapacityMoEFFNLayer as MoEFFNLayer  # noqa: F401
from adaptivetrainingsystem_amd.layers import MoECUDAOps  # noqa: F401
from adaptivetrainingsystem_amd.profiling import (  # noqa: F401  (moe_cuda_wrapper.py:76-159, 599-611)
    MoEPerformanceMonitor,
    enable_performance_monitor,
    get_performance_summary,
    print_performance_summary,
    reset_performance_monitor,
    timer_context,
)

CUDA_OPS_AVAILABLE = _lib.is_built()
