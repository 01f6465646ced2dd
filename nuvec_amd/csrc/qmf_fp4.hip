// The few-row and the grouped matrix-core kernels for MXFP4 codes (qmf_kernel.h, qmg_kernel.h).
#include "qmg_kernel.h"

namespace nvq {

int32_t launch_qmf_fp4(const ProductArgs &a, hipStream_t s) {
    return a.offsets != nullptr ? qmg::run_dtype<4, true>(a, s) : qmf::run_dtype<4, true>(a, s);
}

}  // namespace nvq
