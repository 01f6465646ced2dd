// Floating-point block formats for gfx950, bit for bit nuvec's CPU arithmetic (reference:
// crates/nuvec-core/src/kernels.rs:906-1009, crates/nuvec-core/src/fp8.rs:11-129), without a global scale:
//   MXFP4: E2M1 values, groups of 32, E8M0 scales (the group maximum over 6, rounded up to a power of two);
//   MXFP8: E4M3 values, groups of 32, E8M0 scales (the maximum over 448, rounded up);
//   NVFP4: E2M1 values, groups of 16, E4M3 scales (the maximum over 6, rounded to nearest).
//
// A lane owns 8 consecutive values = one (4-bit) or two (8-bit) uint32 of packed codes, value i in bits
// i*bits of the stream; a group is 4 (2 for NVFP4) adjacent lanes.  The reference flushes float32
// subnormals explicitly at every step (it reproduces a device that flushes them); gfx950 keeps
// subnormals, so the same explicit flushes are applied here.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

constexpr int kBlock = 256;

template <int MODE> struct Format;
template <> struct Format<NVQ_MXFP4> { static constexpr int lanes = 4, bits = 4; static constexpr float max_element = 6.0f; static constexpr bool mx = true; };
template <> struct Format<NVQ_MXFP8> { static constexpr int lanes = 4, bits = 8; static constexpr float max_element = 448.0f; static constexpr bool mx = true; };
template <> struct Format<NVQ_NVFP4> { static constexpr int lanes = 2, bits = 4; static constexpr float max_element = 6.0f; static constexpr bool mx = false; };

// kernels.rs:914-971 without a global scale.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock)
fp_quantize_kernel(const T *__restrict__ w, int64_t chunks, uint32_t *__restrict__ packed, uint8_t *__restrict__ scales) {
    using F = Format<MODE>;
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const bool active = chunk < chunks;  // chunks is a multiple of the lanes per group: a group is wholly in or out of range
    float v[8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        v[i] = active ? ftz(Elem<T>::load(w, chunk * 8 + i)) : 0.0f;
        amax = fmaxf(amax, fabsf(v[i]));  // NaN is ignored, as Rust's f32::max
    }
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    if constexpr (F::lanes == 4) amax = fmaxf(amax, __shfl_xor(amax, 2));
    if (!active) return;
    const float scale = ftz(amax / F::max_element);
    uint32_t code;
    float decoded;
    if constexpr (F::mx) {
        code = e8m0_round_up_code(scale);
        decoded = e8m0_to_f32(code);
    } else {
        code = e4m3_from_f32(scale);
        decoded = e4m3_to_f32(code);
    }
    decoded = ftz(decoded);
    const float inverse = decoded == 0.0f ? 0.0f : ftz(1.0f / decoded);
    if constexpr (F::bits == 4) {
        uint32_t word = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) word |= e2m1_from_f32(canonical(ftz(v[i] * inverse))) << (4 * i);
        packed[chunk] = word;
    } else {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo |= e4m3_from_f32(canonical(ftz(v[i] * inverse))) << (8 * i);
            hi |= e4m3_from_f32(canonical(ftz(v[4 + i] * inverse))) << (8 * i);
        }
        reinterpret_cast<uint2 *>(packed)[chunk] = make_uint2(lo, hi);
    }
    if (chunk % F::lanes == 0) scales[chunk / F::lanes] = (uint8_t)code;
}

// kernels.rs:976-1009 without a global scale.  With `ids`, output row r is table row ids[r] (`row_chunks` chunks
// per row, ids clamped to `table_rows`): the rows of a quantized embedding.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock)
fp_dequantize_kernel(const uint32_t *__restrict__ packed, const uint8_t *__restrict__ scales, int64_t chunks, T *__restrict__ out,
                     const uint32_t *__restrict__ ids, int64_t row_chunks, int64_t table_rows) {
    using F = Format<MODE>;
    const int64_t out_chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (out_chunk >= chunks) return;
    int64_t chunk = out_chunk;
    if (ids != nullptr) {
        const int64_t r = out_chunk / row_chunks;
        const int64_t row = min((int64_t)ids[r], table_rows - 1);
        chunk = row * row_chunks + (out_chunk - r * row_chunks);
    }
    const uint32_t sc = scales[chunk / F::lanes];
    const float scale = ftz(F::mx ? e8m0_to_f32(sc) : e4m3_to_f32(sc));
    if constexpr (F::bits == 4) {
        const uint32_t word = packed[chunk];
#pragma unroll
        for (int i = 0; i < 8; i++)
            Elem<T>::store(out, out_chunk * 8 + i, canonical(ftz(scale * e2m1_to_f32((word >> (4 * i)) & 0xFu))));
    } else {
        const uint2 words = reinterpret_cast<const uint2 *>(packed)[chunk];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            Elem<T>::store(out, out_chunk * 8 + i, canonical(ftz(scale * e4m3_to_f32((words.x >> (8 * i)) & 0xFFu))));
            Elem<T>::store(out, out_chunk * 8 + 4 + i, canonical(ftz(scale * e4m3_to_f32((words.y >> (8 * i)) & 0xFFu))));
        }
    }
}

template <typename T, int MODE>
int32_t quantize_t(const void *w, int64_t n, void *packed, void *scales, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((fp_quantize_kernel<T, MODE>), dim3(blocks), dim3(kBlock), 0, s, (const T *)w, chunks,
                       (uint32_t *)packed, (uint8_t *)scales);
    NVQ_LAUNCH_CHECK("fp_quantize");
    return NVQ_OK;
}
template <typename T, int MODE>
int32_t dequantize_t(const void *packed, const void *scales, int64_t n, void *out, const uint32_t *ids, int64_t cols,
                     int64_t table_rows, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((fp_dequantize_kernel<T, MODE>), dim3(blocks), dim3(kBlock), 0, s, (const uint32_t *)packed,
                       (const uint8_t *)scales, chunks, (T *)out, ids, cols / 8, table_rows);
    NVQ_LAUNCH_CHECK("fp_dequantize");
    return NVQ_OK;
}

template <typename T>
int32_t quantize_mode(int32_t mode, const void *w, int64_t n, void *packed, void *scales, hipStream_t s) {
    switch (mode) {
    case NVQ_MXFP4: return quantize_t<T, NVQ_MXFP4>(w, n, packed, scales, s);
    case NVQ_MXFP8: return quantize_t<T, NVQ_MXFP8>(w, n, packed, scales, s);
    case NVQ_NVFP4: return quantize_t<T, NVQ_NVFP4>(w, n, packed, scales, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "quantize: mode %s is not a floating-point block format", mode_name(mode));
    }
}
template <typename T>
int32_t dequantize_mode(int32_t mode, const void *packed, const void *scales, int64_t n, void *out, const uint32_t *ids,
                        int64_t cols, int64_t table_rows, hipStream_t s) {
    switch (mode) {
    case NVQ_MXFP4: return dequantize_t<T, NVQ_MXFP4>(packed, scales, n, out, ids, cols, table_rows, s);
    case NVQ_MXFP8: return dequantize_t<T, NVQ_MXFP8>(packed, scales, n, out, ids, cols, table_rows, s);
    case NVQ_NVFP4: return dequantize_t<T, NVQ_NVFP4>(packed, scales, n, out, ids, cols, table_rows, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "dequantize: mode %s is not a floating-point block format", mode_name(mode));
    }
}

}  // namespace

int32_t launch_fp_quantize(int32_t mode, int32_t dtype, const void *w, int64_t n, void *packed, void *scales,
                           hipStream_t s) {
    switch (dtype) {
    case NVQ_F32: return quantize_mode<float>(mode, w, n, packed, scales, s);
    case NVQ_BF16: return quantize_mode<bf16_t>(mode, w, n, packed, scales, s);
    default: return quantize_mode<f16_t>(mode, w, n, packed, scales, s);
    }
}

int32_t launch_fp_dequantize(int32_t mode, int32_t out_dtype, const void *packed, const void *scales, int64_t n,
                             void *out, const uint32_t *ids, int64_t cols, int64_t table_rows, hipStream_t s) {
    switch (out_dtype) {
    case NVQ_F32: return dequantize_mode<float>(mode, packed, scales, n, out, ids, cols, table_rows, s);
    case NVQ_BF16: return dequantize_mode<bf16_t>(mode, packed, scales, n, out, ids, cols, table_rows, s);
    default: return dequantize_mode<f16_t>(mode, packed, scales, n, out, ids, cols, table_rows, s);
    }
}

}  // namespace nvq
