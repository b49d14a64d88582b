"""MI355X-native Sparse DNN Graph Challenge inference (host-side Python view of the C ABI).

The product is the C-ABI library ``libspdnn.so`` (include/spdnn.h) and the ``spdnn_network``
driver built from ``csrc/``; this package is a thin ctypes front end used by the tests and the
benchmark.  It never falls back to a CPU path: without the built library it raises.
"""
from .binding import (  # noqa: F401
    KERNEL_AUTO, KERNEL_BAND, KERNEL_BLOCK, KERNEL_GATHER, KERNEL_TILED, LayerPlan, Network, RunResult, SpdnnError,
    device_alloc_calls, device_info, device_memory, hash_reorder, lib_path, load_library, measure_copy_bandwidth, reference_bias,
    read_features_tsv, synth_features_host, synth_layer_csr, weight_file_name,
)
from .build import build  # noqa: F401
