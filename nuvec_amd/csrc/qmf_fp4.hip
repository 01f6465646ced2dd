// The few-row matrix-core kernel for MXFP4 codes (see qmf_kernel.h).
#include "qmf_kernel.h"

namespace nvq {

int32_t launch_qmf_fp4(const ProductArgs &a, hipStream_t s) { return qmf::run_dtype<4, true>(a, s); }

}  // namespace nvq
