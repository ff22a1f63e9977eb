"""MI355X-native quantized matmul backend for orangu-server's `Backend` seam.

The product is the C-ABI shared library (``include/orangu_mi355x.h``) built from
``orangu_amd/csrc``.  This package holds the build script and a thin ctypes mirror of the
reference's ``Backend`` trait used by tests and the benchmark.
"""
from .capi import LIB_PATH, OgmError, load_library  # noqa: F401
from .backend import LlamaDecoder, Mi355xBackend, MatmulOp, QuantMatrix  # noqa: F401

GGML_TYPE_Q8_0 = 8
GGML_TYPE_Q4_0 = 2
GGML_TYPE_Q5_0 = 6
GGML_TYPE_IQ4_NL = 20
GGML_TYPE_Q3_K = 11
GGML_TYPE_Q4_K = 12
GGML_TYPE_Q5_K = 13
GGML_TYPE_Q6_K = 14
