// MXFP4 quantize / dequantize for gfx950 (E2M1 values, groups of 32, E8M0 scales), bit for
// bit nuvec's CPU arithmetic (reference: crates/nuvec-core/src/kernels.rs:906-1009,
// crates/nuvec-core/src/fp8.rs:47-129).
//
// A lane owns 8 consecutive values = one uint32 of packed nibbles (value i in bits 4i..4i+3,
// low nibble first); a group of 32 values is 4 adjacent lanes.  The reference flushes float32
// subnormals explicitly at every step (it reproduces a device that flushes them); gfx950 keeps
// subnormals, so the same explicit flushes are applied here.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

constexpr int kBlock = 256;

template <typename T>
__device__ __forceinline__ void load8(const T *w, int64_t base, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = Elem<T>::load(w, base + i);
}

// kernels.rs:914-971 with group 32, 4 bits, no global scale.
template <typename T>
__global__ void __launch_bounds__(kBlock)
mxfp4_quantize_kernel(const T *__restrict__ w, int64_t chunks, uint32_t *__restrict__ packed,
                      uint8_t *__restrict__ scales) {
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const bool active = chunk < chunks;  // chunks % 4 == 0: a group is wholly in or out of range
    float v[8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        v[i] = active ? ftz(Elem<T>::load(w, chunk * 8 + i)) : 0.0f;
        amax = fmaxf(amax, fabsf(v[i]));  // NaN is ignored, as Rust's f32::max
    }
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    if (!active) return;
    const float scale = ftz(amax / 6.0f);
    const uint32_t code = e8m0_round_up_code(scale);
    const float decoded = ftz(e8m0_to_f32(code));
    const float inverse = decoded == 0.0f ? 0.0f : ftz(1.0f / decoded);
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float scaled = canonical(ftz(v[i] * inverse));
        word |= e2m1_from_f32(scaled) << (4 * i);
    }
    packed[chunk] = word;
    if ((chunk & 3) == 0) scales[chunk >> 2] = (uint8_t)code;
}

// kernels.rs:976-1009 with group 32, 4 bits, no global scale.
template <typename T>
__global__ void __launch_bounds__(kBlock)
mxfp4_dequantize_kernel(const uint32_t *__restrict__ packed, const uint8_t *__restrict__ scales,
                        int64_t chunks, T *__restrict__ out) {
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (chunk >= chunks) return;
    const uint32_t word = packed[chunk];
    const float scale = ftz(e8m0_to_f32(scales[chunk >> 2]));
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float value = e2m1_to_f32((word >> (4 * i)) & 0xFu);
        Elem<T>::store(out, chunk * 8 + i, canonical(ftz(scale * value)));
    }
}

template <typename T>
int32_t quantize_t(const void *w, int64_t n, void *packed, void *scales, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((mxfp4_quantize_kernel<T>), dim3(blocks), dim3(kBlock), 0, s, (const T *)w, chunks,
                       (uint32_t *)packed, (uint8_t *)scales);
    NVQ_LAUNCH_CHECK("mxfp4_quantize");
    return NVQ_OK;
}
template <typename T>
int32_t dequantize_t(const void *packed, const void *scales, int64_t n, void *out, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((mxfp4_dequantize_kernel<T>), dim3(blocks), dim3(kBlock), 0, s, (const uint32_t *)packed,
                       (const uint8_t *)scales, chunks, (T *)out);
    NVQ_LAUNCH_CHECK("mxfp4_dequantize");
    return NVQ_OK;
}

}  // namespace

int32_t launch_fp_quantize(int32_t mode, int32_t dtype, const void *w, int64_t n, void *packed, void *scales,
                           hipStream_t s) {
    if (mode != NVQ_MXFP4) return fail(NVQ_UNSUPPORTED, "quantize: no gfx950 kernel for mode %s yet", mode_name(mode));
    switch (dtype) {
    case NVQ_F32: return quantize_t<float>(w, n, packed, scales, s);
    case NVQ_BF16: return quantize_t<bf16_t>(w, n, packed, scales, s);
    default: return quantize_t<f16_t>(w, n, packed, scales, s);
    }
}

int32_t launch_fp_dequantize(int32_t mode, int32_t out_dtype, const void *packed, const void *scales, int64_t n,
                             void *out, hipStream_t s) {
    if (mode != NVQ_MXFP4) return fail(NVQ_UNSUPPORTED, "dequantize: no gfx950 kernel for mode %s yet", mode_name(mode));
    switch (out_dtype) {
    case NVQ_F32: return dequantize_t<float>(packed, scales, n, out, s);
    case NVQ_BF16: return dequantize_t<bf16_t>(packed, scales, n, out, s);
    default: return dequantize_t<f16_t>(packed, scales, n, out, s);
    }
}

}  // namespace nvq
