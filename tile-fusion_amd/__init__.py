"""tile-fusion for MI355X: Python plumbing over libtilefusion_hip (ctypes).

The product is the C-ABI library built from ``csrc/`` (see ``include/tilefusion_hip.h``)
and the C++ header ``include/tile-fusion.h``.  This package only loads the library,
wraps its handles, and generates the synthetic workloads the benchmark is quoted on.
The directory name is not a Python identifier; import it with
``importlib.import_module("tile-fusion_amd")``.
"""
from .binding import (  # noqa: F401
    TileFusionError, lib, lib_path, device_init, device_synchronize, CsrMatrix, DenseMatrix,
    FusedSchedule, inspector, spmm_spmm, gemm_spmm, spmm, gemm, Stream, Event,
    OP_SPMM_SPMM, OP_GEMM_SPMM, ACCUMULATE, SECOND_STREAM, RELU, gcn_two_layers, spmm_spmm_noalloc, noalloc_scratch_bytes,
    pattern_hash, read_matrix, read_dense, reorder_rcm, reorder_partition, permute_csr, calibrate_issue,
)
from . import workloads  # noqa: F401
