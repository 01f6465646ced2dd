// The few-row, grouped and tiled matrix-core kernels for MXFP8 codes (qmf_kernel.h, qmg_kernel.h, qmm_kernel.h).
#include "qmg_kernel.h"
#include "qmm_kernel.h"

namespace nvq {

int32_t launch_qmf_fp8(const ProductArgs &a, hipStream_t s) {
    return a.offsets != nullptr ? qmg::run_dtype<8, qmf::kMxfp8>(a, s) : qmf::run_dtype<8, qmf::kMxfp8>(a, s);
}

int32_t launch_qmm_fp8(const ProductArgs &a, void *workspace, hipStream_t s) { return qmm::run_dtype<8, qmf::kMxfp8>(a, workspace, s); }

}  // namespace nvq
