"""nuvec_amd — MI355X (gfx950) backend for nuvec's quantized-matmul path.

`libnuvec_hip.so` (C ABI in include/nuvec_hip.h) holds the kernels; `ops` mirrors nuvec's
public `quantize`, `dequantize`, `quantized_matmul` and `gather_qmm`.
"""
from .ops import (GatherQmm, InvalidArgument, Quant, QuantMode, Quantized, Unsupported, dequantize, gather_qmm,  # noqa: F401
                  quantize, quantized_matmul, sorted_offsets)
