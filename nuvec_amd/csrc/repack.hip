// Hugging Face integer packings (AutoAWQ's GEMM layout, GPTQ v1 / v2) into MLX's affine layout, bit for bit
// nuvec-lm's conversion at load (reference: crates/nuvec-lm/src/quant.rs:35-196): packed codes
// [out, in * bits / 32] with value i of a row at bit i * bits, scales [out, groups] (a transpose) and
// biases = -(zero) * scale, the product in float32, rounded once more to the scales' type.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

// AWQ's order of the eight 4-bit values in a word: value c of a group of eight outputs sits in nibble
// order[c] (quant.rs:35-37).
__device__ __forceinline__ uint32_t awq_shift(uint32_t c) { return 4u * ((0x73625140u >> (4u * c)) & 0xFu); }

// One thread per output word (o, iw): per_word = 32 / bits codes of inputs iw * per_word ..
// GPTQ keeps exactly these codes, in this order, in word [iw, o] of qweight [in * bits / 32, out]: a transpose.
// AWQ keeps input i's codes of eight neighbouring outputs in word [i, o / 8], in AWQ's nibble order.
template <bool AWQ>
__global__ void repack_codes_kernel(const uint32_t *__restrict__ qweight, int64_t in_words, int64_t outputs, int32_t bits,
                                    uint32_t *__restrict__ packed) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= in_words * outputs) return;
    // consecutive threads take consecutive outputs (coalesced reads); the writes of a wavefront go to 64 rows
    const int64_t iw = t / outputs, o = t % outputs;
    uint32_t word;
    if constexpr (AWQ) {
        const int64_t cols = outputs / 8;
        const uint32_t shift = awq_shift((uint32_t)(o % 8));
        word = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) word |= ((qweight[(iw * 8 + j) * cols + o / 8] >> shift) & 0xFu) << (4 * j);
    } else {
        word = qweight[iw * outputs + o];
    }
    packed[o * in_words + iw] = word;
}

// One thread per (group g, output o): scales [groups, out] -> [out, groups]; bias from the zero.
template <typename T, int FORMAT>  // FORMAT 0: AWQ, 1: GPTQ v1 (zeros stored minus one), 2: GPTQ v2
__global__ void repack_scales_kernel(const uint32_t *__restrict__ qzeros, const T *__restrict__ scales, int64_t groups,
                                     int64_t outputs, int32_t bits, T *__restrict__ scales_out, T *__restrict__ biases_out) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= groups * outputs) return;
    const int64_t g = t / outputs, o = t % outputs;
    const int64_t per_word = 32 / bits;
    float zero;
    if (qzeros == nullptr) {
        zero = (float)(1u << (bits - 1));  // symmetric (quant.rs:140)
    } else {
        const int64_t zcols = (outputs + per_word - 1) / per_word;
        const uint32_t w = qzeros[g * zcols + o / per_word];
        const uint32_t shift = FORMAT == 0 ? awq_shift((uint32_t)(o % per_word)) : (uint32_t)(bits * (o % per_word));
        zero = (float)(((w >> shift) & ((1u << bits) - 1u)) + (FORMAT == 1 ? 1u : 0u));
    }
    const float s = Elem<T>::load(scales, t);
    Elem<T>::store(scales_out, o * groups + g, s);
    // -(zero) * scale: the product rounded to float32, then the store's rounding to T, as the reference's two
    // steps.  The product passes through an opaque register so that the compiler cannot fuse it with the
    // conversion (one rounding instead of two, and a +0.0 addend that turns the -0.0 of a zero of 0 into +0.0);
    // the sign is flipped on the bits.
    float product = zero * s;
    asm volatile("" : "+v"(product));
    Elem<T>::store(biases_out, o * groups + g, u2f(f2u(product) ^ 0x80000000u));
}

template <typename T>
int32_t run_scales(int32_t format, const uint32_t *qzeros, const void *scales, int64_t groups, int64_t outputs, int32_t bits,
                   void *scales_out, void *biases_out, hipStream_t s) {
    const int64_t n = groups * outputs;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (format == 0)
        hipLaunchKernelGGL((repack_scales_kernel<T, 0>), grid, block, 0, s, qzeros, (const T *)scales, groups, outputs, bits, (T *)scales_out, (T *)biases_out);
    else if (format == 1)
        hipLaunchKernelGGL((repack_scales_kernel<T, 1>), grid, block, 0, s, qzeros, (const T *)scales, groups, outputs, bits, (T *)scales_out, (T *)biases_out);
    else
        hipLaunchKernelGGL((repack_scales_kernel<T, 2>), grid, block, 0, s, qzeros, (const T *)scales, groups, outputs, bits, (T *)scales_out, (T *)biases_out);
    NVQ_LAUNCH_CHECK("convert_packed");
    return NVQ_OK;
}

}  // namespace

int32_t launch_convert_packed(int32_t format, int32_t bits, int32_t dtype, const uint32_t *qweight, const uint32_t *qzeros,
                              const void *scales, int64_t inputs, int64_t outputs, int64_t groups, uint32_t *packed,
                              void *scales_out, void *biases_out, hipStream_t s) {
    const int64_t in_words = inputs * bits / 32, n = in_words * outputs;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (format == 0)
        hipLaunchKernelGGL(repack_codes_kernel<true>, grid, block, 0, s, qweight, in_words, outputs, bits, packed);
    else
        hipLaunchKernelGGL(repack_codes_kernel<false>, grid, block, 0, s, qweight, in_words, outputs, bits, packed);
    NVQ_LAUNCH_CHECK("convert_packed");
    switch (dtype) {
    case NVQ_F32: return run_scales<float>(format, qzeros, scales, groups, outputs, bits, scales_out, biases_out, s);
    case NVQ_BF16: return run_scales<bf16_t>(format, qzeros, scales, groups, outputs, bits, scales_out, biases_out, s);
    default: return run_scales<f16_t>(format, qzeros, scales, groups, outputs, bits, scales_out, biases_out, s);
    }
}

}  // namespace nvq
