// Affine quantize / dequantize for gfx950, bit for bit nuvec's CPU arithmetic
// (reference: crates/nuvec-core/src/kernels.rs:774-859).
//
// Both kernels are streaming: a lane owns 8 consecutive values, which is exactly `bits`
// bytes of the packed little-endian bit stream (value i at bit i*bits), so a lane's codes
// never share a byte with its neighbour's.  A quantization group of 32/64/128 values is
// 4/8/16 adjacent lanes of one wavefront; its extremes are folded with lane shuffles.
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
template <>
__device__ __forceinline__ void load8<float>(const float *w, int64_t base, float (&v)[8]) {
    const float4 *p = reinterpret_cast<const float4 *>(w + base);  // base % 8 == 0, w 16-byte aligned
    float4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t *w, int64_t base, float (&v)[8]) {
    uint4 q = *reinterpret_cast<const uint4 *>(w + base);
    uint32_t r[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[2 * i] = u2f(r[i] << 16);
        v[2 * i + 1] = u2f(r[i] & 0xFFFF0000u);
    }
}

template <>
__device__ __forceinline__ void load8<f16_t>(const f16_t *w, int64_t base, float (&v)[8]) {
    uint4 q = *reinterpret_cast<const uint4 *>(w + base);
    f16_t h[8];
    __builtin_memcpy(h, &q, 16);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = (float)h[i];
}

// Rounds 8 float32 values to T (they are already exact T values here) and stores them with
// 16-byte stores.
template <typename T>
__device__ __forceinline__ void store8(T *out, int64_t base, const float (&v)[8]);
template <>
__device__ __forceinline__ void store8<float>(float *out, int64_t base, const float (&v)[8]) {
    float4 *p = reinterpret_cast<float4 *>(out + base);
    p[0] = make_float4(v[0], v[1], v[2], v[3]);
    p[1] = make_float4(v[4], v[5], v[6], v[7]);
}
template <>
__device__ __forceinline__ void store8<bf16_t>(bf16_t *out, int64_t base, const float (&v)[8]) {
    uint32_t r[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        r[i] = (uint32_t)f32_to_bf16_bits(v[2 * i]) | ((uint32_t)f32_to_bf16_bits(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4 *>(out + base) = make_uint4(r[0], r[1], r[2], r[3]);
}
template <>
__device__ __forceinline__ void store8<f16_t>(f16_t *out, int64_t base, const float (&v)[8]) {
    f16_t h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = (f16_t)v[i];
    uint4 q;
    __builtin_memcpy(&q, h, 16);
    *reinterpret_cast<uint4 *>(out + base) = q;
}

// Stores the low `BITS` bytes of `stream` at `bytes + BITS*chunk` with the widest stores the
// alignment allows.
template <int BITS>
__device__ __forceinline__ void store_codes(uint8_t *bytes, int64_t chunk, uint64_t stream) {
    uint8_t *p = bytes + chunk * BITS;
    if constexpr (BITS == 8) {
        *reinterpret_cast<uint2 *>(p) = make_uint2((uint32_t)stream, (uint32_t)(stream >> 32));
    } else if constexpr (BITS == 4) {
        *reinterpret_cast<uint32_t *>(p) = (uint32_t)stream;
    } else if constexpr (BITS == 2) {
        *reinterpret_cast<uint16_t *>(p) = (uint16_t)stream;
    } else if constexpr (BITS == 6) {
        uint16_t *h = reinterpret_cast<uint16_t *>(p);
        h[0] = (uint16_t)stream; h[1] = (uint16_t)(stream >> 16); h[2] = (uint16_t)(stream >> 32);
    } else {
#pragma unroll
        for (int b = 0; b < BITS; b++) p[b] = (uint8_t)(stream >> (8 * b));
    }
}

template <int BITS>
__device__ __forceinline__ uint64_t load_codes(const uint8_t *bytes, int64_t chunk) {
    const uint8_t *p = bytes + chunk * BITS;
    if constexpr (BITS == 8) {
        uint2 q = *reinterpret_cast<const uint2 *>(p);
        return (uint64_t)q.x | ((uint64_t)q.y << 32);
    } else if constexpr (BITS == 4) {
        return *reinterpret_cast<const uint32_t *>(p);
    } else if constexpr (BITS == 2) {
        return *reinterpret_cast<const uint16_t *>(p);
    } else if constexpr (BITS == 6) {
        const uint16_t *h = reinterpret_cast<const uint16_t *>(p);
        return (uint64_t)h[0] | ((uint64_t)h[1] << 16) | ((uint64_t)h[2] << 32);
    } else {
        uint64_t s = 0;
#pragma unroll
        for (int b = 0; b < BITS; b++) s |= (uint64_t)p[b] << (8 * b);
        return s;
    }
}

// kernels.rs:774-831.  `chunks` = n_values / 8; `lanes` = group / 8 (4, 8 or 16).
template <typename T, int BITS>
__global__ void __launch_bounds__(kBlock)
affine_quantize_kernel(const T *__restrict__ w, int64_t chunks, int lanes, uint8_t *__restrict__ packed,
                       T *__restrict__ scales, T *__restrict__ biases) {
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    // chunks is a multiple of `lanes` and the block size is a multiple of 16: a group's lanes
    // are all in range or all out of range, so the shuffles below never mix the two.
    const bool active = chunk < chunks;
    float v[8];
    if (active) {
        load8<T>(w, chunk * 8, v);
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = 0.0f;
    }
    // f32 extremes of the group: min/max ignore NaN and order -0 below +0, so the fold's
    // order does not matter (the reference folds from +Inf / -Inf in index order).
    float lo = INFINITY, hi = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; i++) { lo = rs_min(lo, v[i]); hi = rs_max(hi, v[i]); }
    for (int d = 1; d < lanes; d <<= 1) {
        lo = rs_min(lo, __shfl_xor(lo, d));
        hi = rs_max(hi, __shfl_xor(hi, d));
    }
    const float n_bins = (float)((1u << BITS) - 1u);
    const float eps = 1e-7f;
    float scale, bias;
    if constexpr (BITS == 1) {
        scale = rs_max(hi - lo, eps);
        bias = lo;
    } else {
        const bool wide = fabsf(lo) > fabsf(hi);
        scale = rs_max((hi - lo) / n_bins, eps);
        scale = wide ? scale : -scale;
        const float edge = wide ? lo : hi;
        const float q0 = rintf(edge / scale);
        if (q0 == 0.0f) {
            bias = 0.0f;
        } else {
            scale = edge / q0;
            bias = edge;
        }
    }
    if (!active) return;
    // code = rint((v - bias) / scale) with the correctly rounded quotient.  Eight divisions per lane are the
    // bulk of this kernel's arithmetic, and only the rounded integer is needed: (v - bias) * (1 / scale) is
    // within 2^-23 relative of the quotient, so both round to the same integer unless they lie that close to
    // a half; those few values (and odd scales) take the division.
    const float inv = 1.0f / scale;
    const float mag = fabsf(scale);
    const bool plain = mag > 1e-30f && mag < 1e30f;  // finite, normal, with a finite normal reciprocal
    uint64_t stream = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float d = v[i] - bias;
        float t = d * inv;
        const float u = fabsf(t);
        const float frac = u - floorf(u);
        if (!plain || !(fabsf(frac - 0.5f) > 4e-7f * u)) t = d / scale;  // also NaN and infinities
        float q = rintf(t);
        q = fminf(fmaxf(q, 0.0f), n_bins);  // NaN -> 0, as Rust's clamp followed by `as u32`
        stream |= (uint64_t)(uint32_t)q << (i * BITS);
    }
    store_codes<BITS>(packed, chunk, stream);
    if (chunk % lanes == 0) {
        const int64_t g = chunk / lanes;
        Elem<T>::store(scales, g, scale);
        Elem<T>::store(biases, g, bias);
    }
}

// kernels.rs:835-859: round(round(code * scale) + bias), both roundings in T.  With `ids`, output row r is
// table row ids[r] (the rows of a quantized embedding, crates/nuvec-nn/src/layers.rs:245-255): `row_chunks` chunks
// per row, ids clamped to the table's `table_rows`.
template <typename T, int BITS>
__global__ void __launch_bounds__(kBlock)
affine_dequantize_kernel(const uint8_t *__restrict__ packed, const T *__restrict__ scales,
                         const T *__restrict__ biases, int64_t chunks, int lanes, T *__restrict__ out,
                         const uint32_t *__restrict__ ids, int64_t row_chunks, int64_t table_rows) {
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (chunk >= chunks) return;
    int64_t src = chunk;
    if (ids != nullptr) {
        const int64_t r = chunk / row_chunks;
        const int64_t row = min((int64_t)ids[r], table_rows - 1);
        src = row * row_chunks + (chunk - r * row_chunks);
    }
    const uint64_t stream = load_codes<BITS>(packed, src);
    const int64_t g = src / lanes;
    const float s = Elem<T>::load(scales, g), b = Elem<T>::load(biases, g);
    constexpr uint32_t mask = (1u << BITS) - 1u;
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float c = (float)((uint32_t)(stream >> (i * BITS)) & mask);
        r[i] = Elem<T>::add(Elem<T>::mul(c, s), b);
    }
    store8<T>(out, chunk * 8, r);
}

template <typename T, int BITS>
int32_t quantize_t(int group, const void *w, int64_t n, void *packed, void *scales, void *biases, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((affine_quantize_kernel<T, BITS>), dim3(blocks), dim3(kBlock), 0, s, (const T *)w, chunks,
                       group / 8, (uint8_t *)packed, (T *)scales, (T *)biases);
    NVQ_LAUNCH_CHECK("affine_quantize");
    return NVQ_OK;
}
template <typename T, int BITS>
int32_t dequantize_t(int group, const void *packed, const void *scales, const void *biases, int64_t n, void *out,
                     const uint32_t *ids, int64_t cols, int64_t table_rows, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((affine_dequantize_kernel<T, BITS>), dim3(blocks), dim3(kBlock), 0, s,
                       (const uint8_t *)packed, (const T *)scales, (const T *)biases, chunks, group / 8, (T *)out, ids, cols / 8,
                       table_rows);
    NVQ_LAUNCH_CHECK("affine_dequantize");
    return NVQ_OK;
}

#define NVQ_BITS_SWITCH(bits, CALL)                                      \
    switch (bits) {                                                      \
    case 1: return CALL(1);                                              \
    case 2: return CALL(2);                                              \
    case 3: return CALL(3);                                              \
    case 4: return CALL(4);                                              \
    case 5: return CALL(5);                                              \
    case 6: return CALL(6);                                              \
    case 8: return CALL(8);                                              \
    default: return fail(NVQ_INVALID_ARGUMENT, "%d bits are not supported", bits); \
    }

}  // namespace

int32_t launch_affine_quantize(int32_t dtype, int group, int bits, const void *w, int64_t n, void *packed,
                               void *scales, void *biases, hipStream_t s) {
#define Q_F32(B) quantize_t<float, B>(group, w, n, packed, scales, biases, s)
#define Q_BF16(B) quantize_t<bf16_t, B>(group, w, n, packed, scales, biases, s)
#define Q_F16(B) quantize_t<f16_t, B>(group, w, n, packed, scales, biases, s)
    if (dtype == NVQ_F32) { NVQ_BITS_SWITCH(bits, Q_F32) }
    if (dtype == NVQ_BF16) { NVQ_BITS_SWITCH(bits, Q_BF16) }
    NVQ_BITS_SWITCH(bits, Q_F16)
}

int32_t launch_affine_dequantize(int32_t dtype, int group, int bits, const void *packed, const void *scales,
                                 const void *biases, int64_t n, void *out, const uint32_t *ids, int64_t cols,
                                 int64_t table_rows, hipStream_t s) {
#define D_F32(B) dequantize_t<float, B>(group, packed, scales, biases, n, out, ids, cols, table_rows, s)
#define D_BF16(B) dequantize_t<bf16_t, B>(group, packed, scales, biases, n, out, ids, cols, table_rows, s)
#define D_F16(B) dequantize_t<f16_t, B>(group, packed, scales, biases, n, out, ids, cols, table_rows, s)
    if (dtype == NVQ_F32) { NVQ_BITS_SWITCH(bits, D_F32) }
    if (dtype == NVQ_BF16) { NVQ_BITS_SWITCH(bits, D_BF16) }
    NVQ_BITS_SWITCH(bits, D_F16)
}

}  // namespace nvq
