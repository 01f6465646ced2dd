// Index helpers of the gathered products (reference: crates/nuvec-core/src/kernels.rs:873-892,
// crates/nuvec-kernels/src/metal/gather_gemm.metal:436-457).
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

// offsets[row, g] = first position of `indices[row, :]` whose value is not below g
// (a lower bound by binary search; the row is sorted by the caller's contract).
__global__ void sorted_offsets_kernel(const uint32_t *__restrict__ indices, int64_t rows, int64_t m, int32_t groups,
                                      int32_t *__restrict__ offsets) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= rows * groups) return;
    const int64_t r = t / groups;
    const uint32_t g = (uint32_t)(t % groups);
    const uint32_t *row = indices + r * m;
    int64_t lo = 0, hi = m;
    while (lo < hi) {
        const int64_t mid = lo + (hi - lo) / 2;
        if (row[mid] < g) lo = mid + 1; else hi = mid;
    }
    offsets[t] = (int32_t)lo;
}

__global__ void fill_zero_kernel(uint16_t *p, int64_t halves) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < halves) p[t] = 0;
}

}  // namespace

int32_t launch_sorted_offsets(const uint32_t *indices, int64_t rows, int64_t m, int32_t groups, int32_t *offsets,
                              hipStream_t s) {
    const int64_t n = rows * groups;
    hipLaunchKernelGGL(sorted_offsets_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, indices, rows, m, groups, offsets);
    NVQ_LAUNCH_CHECK("sorted_offsets");
    return NVQ_OK;
}

// Zero-fills `bytes` (even: element sizes are 2 or 4) with a kernel, so that a caller capturing
// the stream into a graph records no memset node.
int32_t launch_fill_zero(void *p, int64_t bytes, hipStream_t s) {
    const int64_t halves = bytes / 2;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((halves + 255) / 256)), dim3(256), 0, s, (uint16_t *)p, halves);
    NVQ_LAUNCH_CHECK("fill_zero");
    return NVQ_OK;
}

}  // namespace nvq
