// The few-row matrix-core kernel for affine 2-bit codes (see qmf_kernel.h).
#include "qmf_kernel.h"

namespace nvq {

int32_t launch_qmf_b2(const ProductArgs &a, hipStream_t s) { return qmf::run_dtype<2, false>(a, s); }

}  // namespace nvq
