// The few-row, grouped and tiled matrix-core kernels for affine 5-bit codes (qmf_kernel.h, qmg_kernel.h,
// qmm_kernel.h).
#include "qmg_kernel.h"
#include "qmm_kernel.h"

namespace nvq {

int32_t launch_qmf_b5(const ProductArgs &a, hipStream_t s) {
    return a.offsets != nullptr ? qmg::run_dtype<5, false>(a, s) : qmf::run_dtype<5, false>(a, s);
}

int32_t launch_qmm_b5(const ProductArgs &a, void *workspace, hipStream_t s) { return qmm::run_dtype<5, false>(a, workspace, s); }

}  // namespace nvq
