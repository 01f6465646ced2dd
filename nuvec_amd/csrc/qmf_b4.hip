// The few-row matrix-core kernel for affine 4-bit codes (see qmf_kernel.h).
#include "qmf_kernel.h"

namespace nvq {

int32_t launch_qmf_b4(const ProductArgs &a, hipStream_t s) { return qmf::run_dtype<4, false>(a, s); }

}  // namespace nvq
