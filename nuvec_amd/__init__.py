"""nuvec_amd — MI355X (gfx950) backend for nuvec's quantized-matmul path.

`libnuvec_hip.so` (C ABI in include/nuvec_hip.h) holds the kernels; `ops` mirrors nuvec's
public `quantize`, `dequantize`, `quantized_matmul` and `gather_qmm`, and the row lookup of
nuvec-nn's `QuantizedEmbedding` as `embedding`; `moe_order`, `moe_route` and `weighted_sum` are the glue of
nuvec-lm's mixture-of-experts blocks around the gathered products; `formats` and `checkpoint` turn checkpoint files
into `Quantized` operands in device memory.
"""
from .ops import (GatherQmm, InvalidArgument, Quant, QuantMode, Quantized, Unsupported, dequantize, embedding,  # noqa: F401
                  gather_qmm, gather_qmm_glu, gather_qmm_grouped, gather_qqmm, glu, moe_order, pair_rows, moe_route, qqmm, quantize, quantize_dequantize,
                  quantized_matmul, quantized_matmul_glu, quantized_matmul_route, sorted_offsets, weighted_sum)
