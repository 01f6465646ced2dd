// The few-row, grouped and tiled matrix-core kernels for affine 1-bit codes (qmf_kernel.h, qmg_kernel.h,
// qmm_kernel.h).
#include "qmg_kernel.h"
#include "qmm_kernel.h"

namespace nvq {

int32_t launch_qmf_b1(const ProductArgs &a, hipStream_t s) {
    return a.offsets != nullptr ? qmg::run_dtype<1, false>(a, s) : qmf::run_dtype<1, false>(a, s);
}

int32_t launch_qmm_b1(const ProductArgs &a, void *workspace, hipStream_t s) { return qmm::run_dtype<1, false>(a, workspace, s); }

}  // namespace nvq
