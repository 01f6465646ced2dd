// The few-row matrix-core kernel for affine 6-bit codes (see qmf_kernel.h).
#include "qmf_kernel.h"

namespace nvq {

int32_t launch_qmf_b6(const ProductArgs &a, hipStream_t s) { return qmf::run_dtype<6, false>(a, s); }

}  // namespace nvq
