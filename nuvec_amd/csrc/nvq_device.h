// Device-side scalar helpers: element types, exact conversions, the small float codecs.
// Everything here is written so that the bits equal nuvec's CPU arithmetic
// (reference: crates/nuvec-core/src/cast.rs:49-98, crates/nuvec-core/src/fp8.rs:11-129).
// The library is compiled with floating-point contraction off: a fused multiply-add appears
// only where it is written.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nuvec_hip.h"

namespace nvq {

struct bf16_t { uint16_t bits; };   // bfloat16 storage
typedef _Float16 f16_t;             // IEEE half: native arithmetic, round to nearest even

__device__ __forceinline__ uint32_t f2u(float x) { return __float_as_uint(x); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// bf16 <- f32: round to nearest even; a NaN keeps its high bits and is quieted (the `half` crate's
// bf16::from_f32, which cast.rs:85-98 calls).  gfx950's conversion instruction does exactly this: it was compared
// with the integer formulation ((u >> 16) | 0x40 for a NaN, else u >> 16 plus one when bit 15 and any of bits
// 16, 14..0 are set) on all 2^32 inputs.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }
// Two roundings in one instruction: `lo` in the low half of the word.
__device__ __forceinline__ uint32_t f32_to_bf16_pair(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

// Data that is read or written once (weights of a product, the streams of quantize and dequantize): non-temporal
// accesses keep it from displacing what is reused (x, scales, tables) in the caches.
typedef uint32_t stream_u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t stream_u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 stream_load(const uint4 *p) {
    const stream_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const stream_u32x4_t *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 stream_load(const uint2 *p) {
    const stream_u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const stream_u32x2_t *>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t stream_load(const uint32_t *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void stream_store(uint4 *p, uint4 v) {
    const stream_u32x4_t q = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(q, reinterpret_cast<stream_u32x4_t *>(p));
}
__device__ __forceinline__ void stream_store(uint2 *p, uint2 v) {
    const stream_u32x2_t q = {v.x, v.y};
    __builtin_nontemporal_store(q, reinterpret_cast<stream_u32x2_t *>(p));
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int code = 11;
    __device__ static __forceinline__ float load(const float *p, int64_t i) { return p[i]; }
    __device__ static __forceinline__ void store(float *p, int64_t i, float v) { p[i] = v; }
    // round(a*b) and round(a+b) in the element type
    __device__ static __forceinline__ float mul(float a, float b) { return a * b; }
    __device__ static __forceinline__ float add(float a, float b) { return a + b; }
};
template <> struct Elem<bf16_t> {
    static constexpr int code = 10;
    __device__ static __forceinline__ float load(const bf16_t *p, int64_t i) { return bf16_bits_to_f32(p[i].bits); }
    __device__ static __forceinline__ void store(bf16_t *p, int64_t i, float v) { p[i].bits = f32_to_bf16_bits(v); }
    __device__ static __forceinline__ float mul(float a, float b) { return bf16_bits_to_f32(f32_to_bf16_bits(a * b)); }
    __device__ static __forceinline__ float add(float a, float b) { return bf16_bits_to_f32(f32_to_bf16_bits(a + b)); }
};
template <> struct Elem<f16_t> {
    static constexpr int code = 9;
    __device__ static __forceinline__ float load(const f16_t *p, int64_t i) { return (float)p[i]; }
    __device__ static __forceinline__ void store(f16_t *p, int64_t i, float v) { p[i] = (f16_t)v; }
    // Both operands are exact halves: native half arithmetic rounds the exact result once.
    __device__ static __forceinline__ float mul(float a, float b) { return (float)((f16_t)a * (f16_t)b); }
    __device__ static __forceinline__ float add(float a, float b) { return (float)((f16_t)a + (f16_t)b); }
};

// A product's value for column n with the layer's bias, as QuantizedLinear::forward computes it
// (crates/nuvec-nn/src/layers.rs:155-162: the product, rounded to the element type, then a separate addition, rounded
// again).  The result is exact in the element type, so storing it rounds nothing.
template <typename T>
__device__ __forceinline__ float add_row_bias(const void *row_bias, float v, int64_t n) {
    return row_bias == nullptr ? v : Elem<T>::add(Elem<T>::mul(v, 1.0f), Elem<T>::load((const T *)row_bias, n));
}

// Rust's f32::min / f32::max as the reference's hosts evaluate them: the other operand
// when one is NaN, and -0 ordered below +0.
__device__ __forceinline__ float rs_min(float a, float b) {
    float m = fminf(a, b);
    if (a == 0.0f && b == 0.0f) m = u2f(f2u(a) | f2u(b));
    return m;
}
__device__ __forceinline__ float rs_max(float a, float b) {
    float m = fmaxf(a, b);
    if (a == 0.0f && b == 0.0f) m = u2f(f2u(a) & f2u(b));
    return m;
}

// fp8.rs:103-112: a float32 subnormal becomes a zero of its sign.
__device__ __forceinline__ float ftz(float x) {
    uint32_t u = f2u(x);
    return ((u & 0x7F800000u) == 0u) ? u2f(u & 0x80000000u) : x;
}
// fp8.rs:114-118
__device__ __forceinline__ float canonical(float x) { return x != x ? u2f(0x7FC00000u) : x; }

// fp8.rs:47-73
__device__ __forceinline__ uint32_t e2m1_from_f32(float x) {
    if (x != x) return 0x7u;
    uint32_t sign = (f2u(x) >> 28) & 0x8u;
    float a = fabsf(x);
    uint32_t code = a > 5.0f ? 7u : a >= 3.5f ? 6u : a > 2.5f ? 5u : a >= 1.75f ? 4u
                  : a > 1.25f ? 3u : a >= 0.75f ? 2u : a > 0.25f ? 1u : 0u;
    return code | sign;
}
// fp8.rs:75-80: 0, 0.5, 1, 1.5, 2, 3, 4, 6 and their negatives
__device__ __forceinline__ float e2m1_to_f32(uint32_t code) {
    uint32_t m = code & 7u;
    // magnitudes as float32 bit patterns, built from the code: m < 2 -> m/2; else 2^((m>>1)-1) * (1 + (m&1)/2)
    float v = m == 0u ? 0.0f : m == 1u ? 0.5f : u2f(((126u + (m >> 1)) << 23) | ((m & 1u) << 22));
    return (code & 8u) ? -v : v;
}
// fp8.rs:16-37: float32 -> E4M3 (FN variant: no infinities, 0x7F is NaN), round to nearest even, saturating
// to 0x7E (448); NaN goes to 0x7E too, as everything at or above the limit does after the sign is removed.
__device__ __forceinline__ uint32_t e4m3_from_f32(float x) {
    constexpr uint32_t kMax = 543u << 21, kDenorm = 141u << 23;
    uint32_t bits = f2u(x);
    const uint32_t sign = bits & 0x80000000u;
    bits ^= sign;
    uint32_t code;
    if (bits >= kMax) {
        code = 0x7Eu;
    } else if (bits < (121u << 23)) {
        code = (f2u(u2f(bits) + u2f(kDenorm)) - kDenorm) & 0xFFu;
    } else {
        const uint32_t odd = (bits >> 20) & 1u;
        bits += ((uint32_t)(7 - 127) << 23) + 0x7FFFFu;
        bits += odd;
        code = (bits >> 20) & 0xFFu;
    }
    return code | (sign >> 24);
}
// fp8.rs:39-45: the code's bits placed in a half and scaled by 256 (exact)
__device__ __forceinline__ float e4m3_to_f32(uint32_t code) {
    const uint32_t v = code & 127u;
    const uint16_t u = (uint16_t)((v << 7) | (((v + 1u) >> 7) << 14) | ((code >> 7) << 15));
    return (float)__builtin_bit_cast(_Float16, u) * 256.0f;
}
// fp8.rs:95-102
__device__ __forceinline__ float e8m0_to_f32(uint32_t code) {
    return code == 0u ? u2f(0x400000u) : u2f(code << 23);
}
// e8m0_from_f32(mx_scale_round_up(x)) for x = ftz(amax / max_element) >= 0 (fp8.rs:82-93,
// 120-129 as composed at kernels.rs:940-943): the smallest power of two not below x, i.e.
// exponent field + (mantissa != 0), at most 254; 0 for zero; 0xFF for +Inf.
__device__ __forceinline__ uint32_t e8m0_round_up_code(float x) {
    uint32_t u = f2u(x);
    if (u >= 0x7F800000u) return 0xFFu;
    if (u == 0u) return 0u;
    uint32_t c = (u >> 23) + ((u & 0x7FFFFFu) != 0u);
    return c > 254u ? 254u : c;
}

// ---- The gated activations of the experts' MLPs (crates/nuvec-nn/src/lib.rs:343-357, 513-519, 564-570, 581-590), every
// operation rounded to the element type as the reference's element-wise graphs evaluate them.
// kernels.rs:1539-1543
__device__ __forceinline__ float sigmoid_f32(float x) {
    const float a = fabsf(x);
    const float y = 1.0f / (1.0f + expf(a));
    return x < 0.0f ? y : 1.0f - y;
}

// kernels.rs:1367-1368: a NaN operand gives NaN
__device__ __forceinline__ float nan_min(float a, float b) { return (a != a || b != b) ? u2f(0x7FC00000u) : fminf(a, b); }
__device__ __forceinline__ float nan_max(float a, float b) { return (a != a || b != b) ? u2f(0x7FC00000u) : fmaxf(a, b); }

template <typename T>
__device__ __forceinline__ float rounded(float v) { return Elem<T>::mul(v, 1.0f); }

// `alpha` and `limit` are values of the activations' type (lib.rs:505-507: weak scalars): rounded first.
template <typename T, int ACT>
__device__ __forceinline__ float glu(float gate, float up, float alpha, float limit) {
    alpha = rounded<T>(alpha), limit = rounded<T>(limit);
    if constexpr (ACT == NVQ_GLU_SWIGLU) {
        const float s = rounded<T>(sigmoid_f32(gate));
        return Elem<T>::mul(Elem<T>::mul(gate, s), up);  // lib.rs:343-345, 516-517
    } else if constexpr (ACT == NVQ_GLU_SWIGLU_OAI) {
        // lib.rs:565-570
        const float g = nan_min(gate, limit);
        const float x = nan_min(nan_max(up, -limit), limit);
        const float s = rounded<T>(sigmoid_f32(Elem<T>::mul(alpha, g)));
        return Elem<T>::mul(Elem<T>::add(x, 1.0f), Elem<T>::mul(g, s));
    } else {
        // lib.rs:350-357, 583-590: gate^3 is one power (powf in float32, kernels.rs:1375, 1594), rounded once; the
        // constants are weak scalars of the activations' type.  The cube of a 16-bit element is exact in two float32
        // products but for the last rounding; a float32 gate is cubed in float64 and rounded once.
        float cube;
        if constexpr (sizeof(T) == 4) cube = (float)((double)gate * (double)gate * (double)gate);
        else cube = rounded<T>((gate * gate) * gate);
        const float inner = Elem<T>::mul(Elem<T>::add(gate, Elem<T>::mul(cube, rounded<T>(0.044715f))), rounded<T>(0.7978845608028654f));
        const float t = rounded<T>(tanhf(inner));
        return Elem<T>::mul(Elem<T>::mul(Elem<T>::mul(gate, 0.5f), Elem<T>::add(t, 1.0f)), up);
    }
}


}  // namespace nvq
