// Routing of the few-row and the grouped matrix-core kernels (qmf_kernel.h, qmg_kernel.h): which products
// they take and the per-width entry points.
#include "qmg_kernel.h"

namespace nvq {

// Whether the few-row matrix-core kernel takes this product: a block format or affine 1 to 6 or 8 bits, bf16 or
// f16, whole steps of 64 values (whole windows of 128 for 1, 3 and 5 bits, whose 16-byte chunks straddle steps),
// a scale table that fits in LDS, and either no batch, a batch with one stride per operand, gathered pairs,
// or the grouped gather.
bool qmf_supported(const ProductArgs &a) {
    if (a.dtype != NVQ_BF16 && a.dtype != NVQ_F16) return false;
    if (a.k < 64 || a.k % 64 != 0) return false;
    size_t lds = 0;
    if (a.mode == NVQ_MXFP4 || a.mode == NVQ_NVFP4) {
        lds = qmf::lds_needed<4>(a);
    } else if (a.mode == NVQ_MXFP8) {
        lds = qmf::lds_needed<8>(a);
    } else if (a.mode == NVQ_AFFINE) {
        switch (a.bits) {
        case 1: lds = qmf::lds_needed<1>(a); break;
        case 2: lds = qmf::lds_needed<2>(a); break;
        case 3: lds = qmf::lds_needed<3>(a); break;
        case 4: lds = qmf::lds_needed<4>(a); break;
        case 5: lds = qmf::lds_needed<5>(a); break;
        case 6: lds = qmf::lds_needed<6>(a); break;
        case 8: lds = qmf::lds_needed<8>(a); break;
        default: return false;
        }
        if (a.bits % 2 != 0 && a.k % 128 != 0) return false;
    } else {
        return false;
    }
    if (a.offsets != nullptr)  // the grouped kernel: one row of x per pair, its scale table within its LDS budget
        return a.m == 1 && a.experts <= 65535 && !a.exact_weights && qmg::table_bytes(a) <= (size_t)qmg::kTableMaxBytes;
    if (lds > (size_t)qmf::kLdsLimit) return false;
    if (a.rhs != nullptr) return a.batch <= 65535 && (a.m + 31) / 32 <= 65535;  // gathered pairs, one per grid z
    return (a.batch == 1 || a.batch_ndim == 1) && a.batch <= 65535 && (a.m + 31) / 32 <= 65535;
}

int32_t launch_qmf(const ProductArgs &a, hipStream_t s) {
    if (a.mode == NVQ_MXFP4) return launch_qmf_fp4(a, s);
    if (a.mode == NVQ_MXFP8) return launch_qmf_fp8(a, s);
    if (a.mode == NVQ_NVFP4) return launch_qmf_nvfp4(a, s);
    switch (a.bits) {
    case 1: return launch_qmf_b1(a, s);
    case 2: return launch_qmf_b2(a, s);
    case 3: return launch_qmf_b3(a, s);
    case 4: return launch_qmf_b4(a, s);
    case 5: return launch_qmf_b5(a, s);
    case 6: return launch_qmf_b6(a, s);
    default: return launch_qmf_b8(a, s);
    }
}

}  // namespace nvq
