// Pieces the decode kernels share: batch offsets, the magic-number pair constants, the 16x16x32 matrix instruction.
#pragma once
#include "nvq_device.h"
#include "nvq_internal.h"
#include "qmf_kernel.h"  // matrix-instruction operand types

namespace nvq {
namespace {

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

// Element offsets of batch `z` for x, w (in packed dwords), scales/biases and y.
struct BatchOffsets { int64_t x, w, s, y, bias; };  // elements of x, dwords of w, scales, elements of y, of the row bias

__device__ __forceinline__ BatchOffsets batch_offsets(const ProductArgs &a, int64_t z, int64_t kwords, int64_t kgroups) {
    BatchOffsets o{0, 0, 0, z * a.m * a.n, 0};
    if (a.rhs != nullptr) {  // gathered pairs
        // An index outside its operand is the caller's error; it is clamped so that it cannot
        // fault the device.
        const int64_t l = min((int64_t)a.lhs[z], a.x_batches - 1), r = min((int64_t)a.rhs[z], a.experts - 1);
        o.x = l * a.m * a.k;
        o.w = r * a.n * kwords;
        o.s = r * a.n * kgroups;
        if (a.row_bias_per_expert) o.bias = r * a.n;
        if (a.out_rows != nullptr) o.y = min((int64_t)a.out_rows[z], a.batch - 1) * a.m * a.n;
        return o;
    }
    if (a.batch_ndim == 0) return o;
    int64_t rest = z;
#pragma unroll
    for (int d = NVQ_MAX_BATCH_DIMS - 1; d >= 0; d--) {  // constant indices: the arrays stay in kernel arguments
        if (d < a.batch_ndim) {
            const int64_t i = rest % a.batch_shape[d];
            rest /= a.batch_shape[d];
            o.x += i * a.x_strides[d];
            o.w += i * a.w_strides[d];
            o.s += i * a.s_strides[d];
        }
    }
    return o;
}


// Two codes become two element-type values in one instruction: code c in the low mantissa
// bits of the constant 128 (bf16, 0x4300) or 1024 (f16, 0x6400) is exactly 128 + c or 1024 + c.
// `v_dot2_f32_{bf16,f16}` then accumulates x0*(B + c0) + x1*(B + c1) in float32, and the
// offset is removed with the group's sum of x:  sum x*c = dot - B * sum x.
template <typename T> struct Pair;
template <> struct Pair<bf16_t> {
    static constexpr uint32_t magic = 0x43004300u;
    static constexpr float base = 128.0f;
    __device__ static __forceinline__ float dot2(uint32_t x, uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, x), __builtin_bit_cast(bf16x2_t, w), acc, false);
    }
    __device__ static __forceinline__ float lo(uint32_t p) { return u2f(p << 16); }
    __device__ static __forceinline__ float hi(uint32_t p) { return u2f(p & 0xFFFF0000u); }
};
template <> struct Pair<f16_t> {
    static constexpr uint32_t magic = 0x64006400u;
    static constexpr float base = 1024.0f;
    __device__ static __forceinline__ float dot2(uint32_t x, uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, x), __builtin_bit_cast(f16x2_t, w), acc, false);
    }
    __device__ static __forceinline__ float lo(uint32_t p) { return (float)__builtin_bit_cast(f16x2_t, p)[0]; }
    __device__ static __forceinline__ float hi(uint32_t p) { return (float)__builtin_bit_cast(f16x2_t, p)[1]; }
};

template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
    __device__ static __forceinline__ floatx4_t run(uint4 a, uint4 b, floatx4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(qmf::bf16x8_t, a), __builtin_bit_cast(qmf::bf16x8_t, b), c, 0, 0, 0);
    }
};
template <> struct Mfma16<f16_t> {
    __device__ static __forceinline__ floatx4_t run(uint4 a, uint4 b, floatx4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(qmf::f16x8_t, a), __builtin_bit_cast(qmf::f16x8_t, b), c, 0, 0, 0);
    }
};

}  // namespace
}  // namespace nvq
