"""beam -- MI355X (gfx950) gemmrc kernels behind a ctypes binding of libbeam_hip.so.

Counterpart of the reference's python/beam package (python/beam/__init__.py:1-5): the same
operator names and keyword arguments, working on torch tensors or on beam.DeviceArray buffers.
"""
from ._C import (  # noqa: F401
    BeamError,
    DeviceArray,
    TileConfig,
    custom_gemmrc_128x128,
    custom_gemmrc_128x256,
    custom_gemmrc_256x128,
    cutlass_gemmrc,
    cutlass_gemmrc_spec,
    cutlass_gemmrc_splitk,
    cutlass_gemmrc_splitk_spec,
    cutlass_parallel_gemmrc_lnr,
    device_info,
    gemmrc,
    gemmrc_ln,
    gemmrc_spec,
    gemmrc_splitk,
    gemmrc_splitk_spec,
    list_configs,
    library_path,
    matmul,
    parallel_gemmrc_silu,
    silu,
)
from .tuner import Operator, OperatorTuner  # noqa: F401
