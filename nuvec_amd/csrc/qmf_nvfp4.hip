// The few-row, grouped and tiled matrix-core kernels for NVFP4 codes (a global scale folded into the group scales) (qmf_kernel.h, qmg_kernel.h,
// qmm_kernel.h).
#include "qmg_kernel.h"
#include "qmm_kernel.h"

namespace nvq {

int32_t launch_qmf_nvfp4(const ProductArgs &a, hipStream_t s) {
    return a.offsets != nullptr ? qmg::run_dtype<4, qmf::kNvfp4>(a, s) : qmf::run_dtype<4, qmf::kNvfp4>(a, s);
}

int32_t launch_qmm_nvfp4(const ProductArgs &a, void *workspace, hipStream_t s) { return qmm::run_dtype<4, qmf::kNvfp4>(a, workspace, s); }

}  // namespace nvq
