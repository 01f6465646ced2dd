// Calibration kernels for the measurement harness: what this box delivers to a kernel that only reads memory, and to
// one that only issues matrix instructions.  They take no part in any product.
#include "nvq_device.h"
#include "nvq_internal.h"
#include "qmf_kernel.h"

namespace nvq {
namespace {

// Thread t of block b reads the 16-byte pieces b * 1024 + t and b * 1024 + 512 + t (non-temporal, as the decode kernel
// reads its codes): with N / 8 blocks this is the decode kernel's grid and its bytes of packed codes, nothing else.
__global__ void __launch_bounds__(512) read_kernel(const uint4 *__restrict__ p, uint32_t *sink) {
    const uint4 *q = p + (size_t)blockIdx.x * 1024 + threadIdx.x;
    const uint4 a = stream_load(q), b = stream_load(q + 512);
    const uint32_t v = (a.x ^ a.y ^ a.z ^ a.w) + (b.x ^ b.y ^ b.z ^ b.w);
    if (v == 0x9E3779B9u && sink != nullptr) sink[0] = v;  // keeps the loads; practically never taken
}

// Eight independent accumulator tiles per wavefront, `iters` rounds of one v_mfma_f32_32x32x16_bf16 each, operands
// constant: the matrix pipe with nothing else to do.
__global__ void __launch_bounds__(256) mfma_kernel(int iters, float *sink) {
    using qmf::floatx16_t;
    floatx16_t acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
    const uint32_t one = 0x3F803F80u + (threadIdx.x & 1);
    const uint4 a = make_uint4(one, one, one, one), b = make_uint4(one, one, one, one ^ 1u);
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = qmf::Ops<bf16_t>::mfma(a, b, acc[i]);
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) sum += acc[i][e];
    if (sum == 12345.678f && sink != nullptr) sink[0] = sum;
}

}  // namespace

int32_t launch_calibrate(int32_t kind, const void *buffer, int64_t bytes, int32_t iters, void *sink, int64_t *work, hipStream_t s) {
    if (kind == NVQ_CALIBRATE_READ) {
        const int64_t blocks = bytes / 16384;
        if (buffer == nullptr || blocks <= 0 || blocks > 0x7FFFFFFF || bytes % 16384 != 0)
            return fail(NVQ_INVALID_ARGUMENT, "calibrate: the read takes a buffer of a multiple of 16384 bytes");
        hipLaunchKernelGGL(read_kernel, dim3((unsigned)blocks), dim3(512), 0, s, (const uint4 *)buffer, (uint32_t *)sink);
        NVQ_LAUNCH_CHECK("calibrate read");
        if (work != nullptr) *work = bytes;
        return NVQ_OK;
    }
    if (kind == NVQ_CALIBRATE_MFMA) {
        if (iters <= 0) return fail(NVQ_INVALID_ARGUMENT, "calibrate: iters must be positive");
        const int blocks = 2 * compute_units();  // two wavefronts per SIMD
        hipLaunchKernelGGL(mfma_kernel, dim3((unsigned)blocks), dim3(256), 0, s, iters, (float *)sink);
        NVQ_LAUNCH_CHECK("calibrate mfma");
        if (work != nullptr) *work = (int64_t)blocks * 4 * iters * 8 * (2LL * 32 * 32 * 16);
        return NVQ_OK;
    }
    return fail(NVQ_INVALID_ARGUMENT, "calibrate: unknown kind %d", kind);
}

}  // namespace nvq
