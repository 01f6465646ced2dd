// Routing of the tiled matrix-core kernel (qmm_kernel.h): which products it takes and the per-width entry
// points.
#include "qmm_kernel.h"

namespace nvq {

// Whether the tiled kernel takes this product: a block format or affine 1 to 6 or 8 bits, bf16 or f16, whole
// steps of 64 values, and a batch that is a single stride per operand (or no batch).
bool qmm_supported(const ProductArgs &a) {
    if (a.dtype != NVQ_BF16 && a.dtype != NVQ_F16) return false;
    if (a.mode == NVQ_AFFINE) {
        if (a.bits < 1 || a.bits > 8 || a.bits == 7) return false;
    }  // (NVFP4 with a global scale: the scaled weights are rounded to the element type like the affine ones)
    if (a.rhs != nullptr) return false;
    if (a.batch > 1 && a.batch_ndim != 1) return false;
    return a.batch <= 65535 && a.k >= qmm::BK && a.k % qmm::BK == 0;
}

// With its better tile and, for a single product, its better split of K (the caller is expected to bring the
// workspace the size query names).
double qmm_estimate_us(const ProductArgs &a) {
    double us = 0.0;
    qmm::k_splits(a, compute_units(), nullptr, &us);
    return us;
}

size_t qmm_workspace_bytes(const ProductArgs &a) {
    const int splits = qmm::k_splits(a, compute_units());
    return splits > 1 ? (size_t)splits * (size_t)a.m * (size_t)a.n * sizeof(float) : 0;
}

int32_t launch_qmm(const ProductArgs &a, void *workspace, hipStream_t s) {
    if (a.mode == NVQ_MXFP4) return launch_qmm_fp4(a, workspace, s);
    if (a.mode == NVQ_MXFP8) return launch_qmm_fp8(a, workspace, s);
    if (a.mode == NVQ_NVFP4) return launch_qmm_nvfp4(a, workspace, s);
    switch (a.bits) {
    case 1: return launch_qmm_b1(a, workspace, s);
    case 2: return launch_qmm_b2(a, workspace, s);
    case 3: return launch_qmm_b3(a, workspace, s);
    case 4: return launch_qmm_b4(a, workspace, s);
    case 5: return launch_qmm_b5(a, workspace, s);
    case 6: return launch_qmm_b6(a, workspace, s);
    default: return launch_qmm_b8(a, workspace, s);
    }
}

}  // namespace nvq
