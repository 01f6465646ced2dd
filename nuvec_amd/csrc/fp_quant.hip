// Floating-point block formats for gfx950, bit for bit nuvec's CPU arithmetic (reference:
// crates/nuvec-core/src/kernels.rs:906-1009, crates/nuvec-core/src/fp8.rs:11-129), without a global scale:
//   MXFP4: E2M1 values, groups of 32, E8M0 scales (the group maximum over 6, rounded up to a power of two);
//   MXFP8: E4M3 values, groups of 32, E8M0 scales (the maximum over 448, rounded up);
//   NVFP4: E2M1 values, groups of 16, E4M3 scales (the maximum over 6, rounded to nearest).
//
// A lane owns 8 consecutive values = one (4-bit) or two (8-bit) uint32 of packed codes, value i in bits
// i*bits of the stream; a group is 4 (2 for NVFP4) adjacent lanes, a quad or half a quad.  The reference flushes
// float32 subnormals explicitly at every step (it reproduces a device that flushes them); gfx950 keeps
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

// ---- the formats' conversion instructions ----
//
// gfx950 converts pairs of float32 / bfloat16 / half values to E2M1 or E4M3 codes divided by a power-of-two scale
// (v_cvt_scalef32_pk_fp4_*, v_cvt_scalef32_pk_fp8_*), and pairs of E2M1 codes back, in one instruction.  Compared
// with the integer formulation of the reference's arithmetic (flush, multiply by the reciprocal, flush, encode)
// on every float32, bfloat16 and half input, they give the same codes whenever
//   - the value is not a NaN (the instruction keeps a NaN's sign, the reference encodes the canonical NaN),
//   - the E8M0 scale code is in [4, 253] for E2M1 and [12, 253] for E4M3 (below, a subnormal input that the reference
//     flushes still rounds to a nonzero code; 254 has a subnormal reciprocal, which the reference flushes),
//   - the quotient does not exceed the format's largest value (E4M3 only: the instruction then gives the NaN code,
//     the reference saturates), which a group's own scale guarantees;
// and the decoding instructions give the reference's products for scale codes in [2, 254] (below, the reference
// flushes subnormal products; 255 is an infinite scale).  Groups outside these conditions take the integer
// formulation, so every input gives the reference's bits.

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef short s16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int kSwap1 = 0xB1, kSwap2 = 0x4E;  // quad permutations: the lane `lane ^ 1`, `lane ^ 2`
template <int CTRL> __device__ __forceinline__ uint32_t quad_swap(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, CTRL, 0xF, 0xF, true);
}

// A lane's 8 values as loaded: 4 words of pairs (16-bit types) or 8 words (float32).
template <typename T> struct Raw { uint32_t w[sizeof(T) * 2]; };

template <typename T> __device__ __forceinline__ Raw<T> load_raw(const T *w, int64_t chunk) {
    Raw<T> r;
    const uint4 *p = reinterpret_cast<const uint4 *>(w + chunk * 8);
    const uint4 a = stream_load(p);
    r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
    if constexpr (sizeof(T) == 4) {
        const uint4 b = stream_load(p + 1);
        r.w[4] = b.x; r.w[5] = b.y; r.w[6] = b.z; r.w[7] = b.w;
    }
    return r;
}
template <typename T> __device__ __forceinline__ void widen_raw(const Raw<T> &r, float (&v)[8]) {
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = u2f(r.w[i]);
    } else if constexpr (Elem<T>::code == 10) {
#pragma unroll
        for (int i = 0; i < 4; i++) { v[2 * i] = u2f(r.w[i] << 16); v[2 * i + 1] = u2f(r.w[i] & 0xFFFF0000u); }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const f16x2_t h = __builtin_bit_cast(f16x2_t, r.w[i]);
            v[2 * i] = (float)h.x; v[2 * i + 1] = (float)h.y;
        }
    }
}
// The float32 bits of the largest magnitude among the lane's values, by integer comparison of the magnitude bits:
// a NaN compares above infinity, so the result says whether the lane holds one.
template <typename T> __device__ __forceinline__ uint32_t magnitude_bits(const Raw<T> &r) {
    if constexpr (sizeof(T) == 4) {
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) m = max(m, r.w[i] & 0x7FFFFFFFu);
        return m;
    } else {
        u16x2_t m = {0, 0};
#pragma unroll
        for (int i = 0; i < 4; i++) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2_t, r.w[i] & 0x7FFF7FFFu));
        const uint32_t top = max((uint32_t)m.x, (uint32_t)m.y);
        if constexpr (Elem<T>::code == 10) return top << 16;
        else return f2u((float)__builtin_bit_cast(_Float16, (uint16_t)top));  // exact; a half NaN stays a NaN
    }
}
// Codes of the pair `pair` of the lane's values, divided by the scale whose exponent field `scale` carries.
template <typename T> __device__ __forceinline__ uint32_t fp4_pair(uint32_t word, const Raw<T> &r, int pair, float scale, int byte) {
    // `byte` must be a constant in the callers' unrolled loops
    if constexpr (sizeof(T) == 4) {
        switch (byte) {
        case 0: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, u2f(r.w[2 * pair]), u2f(r.w[2 * pair + 1]), scale, 0);
        case 1: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, u2f(r.w[2 * pair]), u2f(r.w[2 * pair + 1]), scale, 1);
        case 2: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, u2f(r.w[2 * pair]), u2f(r.w[2 * pair + 1]), scale, 2);
        default: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(word, u2f(r.w[2 * pair]), u2f(r.w[2 * pair + 1]), scale, 3);
        }
    } else if constexpr (Elem<T>::code == 10) {
        const bf16x2_t v = __builtin_bit_cast(bf16x2_t, r.w[pair]);
        switch (byte) {
        case 0: return __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(word, v, scale, 0);
        case 1: return __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(word, v, scale, 1);
        case 2: return __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(word, v, scale, 2);
        default: return __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(word, v, scale, 3);
        }
    } else {
        const f16x2_t v = __builtin_bit_cast(f16x2_t, r.w[pair]);
        switch (byte) {
        case 0: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(word, v, scale, 0);
        case 1: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(word, v, scale, 1);
        case 2: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(word, v, scale, 2);
        default: return __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(word, v, scale, 3);
        }
    }
}
template <typename T> __device__ __forceinline__ s16x2_t fp8_pair(s16x2_t word, const Raw<T> &r, int pair, float scale, bool high) {
    if constexpr (sizeof(T) == 4) {
        return high ? __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(word, u2f(r.w[2 * pair]), u2f(r.w[2 * pair + 1]), scale, true)
                    : __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(word, u2f(r.w[2 * pair]), u2f(r.w[2 * pair + 1]), scale, false);
    } else if constexpr (Elem<T>::code == 10) {
        const bf16x2_t v = __builtin_bit_cast(bf16x2_t, r.w[pair]);
        return high ? __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(word, v, scale, true) : __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(word, v, scale, false);
    } else {
        const f16x2_t v = __builtin_bit_cast(f16x2_t, r.w[pair]);
        return high ? __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(word, v, scale, true) : __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(word, v, scale, false);
    }
}

// kernels.rs:914-971 without a global scale.
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock)
fp_quantize_kernel(const T *__restrict__ w, int64_t chunks, uint32_t *__restrict__ packed, uint8_t *__restrict__ scales,
                   const float *__restrict__ global_scale) {
    using F = Format<MODE>;
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    // chunks is a multiple of the lanes per group and so is the block: a group is wholly in or out of range
    if (chunk >= chunks) return;
    const Raw<T> raw = load_raw<T>(w, chunk);
    if constexpr (F::mx) {
        // The group's scale code straight from the bits of its largest magnitude m * 2^e: the reference's
        // round_up(ftz(amax / max_element)) has the exponent of the quotient plus one unless the quotient is a
        // power of two, i.e. e - 2 + (m > 1.5) for 6 = 1.5 * 2^2 and e - 8 + (m > 1.75) for 448 = 1.75 * 2^8.
        constexpr uint32_t kCarry = F::bits == 4 ? 0x3FFFFFu : 0x1FFFFFu, kShift = F::bits == 4 ? 2u : 8u;
        constexpr uint32_t kLowest = F::bits == 4 ? 4u : 12u;
        uint32_t top = magnitude_bits<T>(raw);
        top = max(top, quad_swap<kSwap1>(top));
        top = max(top, quad_swap<kSwap2>(top));
        const uint32_t code = ((top + kCarry) >> 23) - kShift;
        if (top < 0x7F800000u && code - kLowest <= 253u - kLowest) {
            const float scale = u2f(code << 23);
            if constexpr (F::bits == 4) {
                uint32_t word = 0;
#pragma unroll
                for (int i = 0; i < 4; i++) word = fp4_pair<T>(word, raw, i, scale, i);
                __builtin_nontemporal_store(word, packed + chunk);
            } else {
                s16x2_t lo = {0, 0}, hi = {0, 0};
                lo = fp8_pair<T>(lo, raw, 0, scale, false); lo = fp8_pair<T>(lo, raw, 1, scale, true);
                hi = fp8_pair<T>(hi, raw, 2, scale, false); hi = fp8_pair<T>(hi, raw, 3, scale, true);
                stream_store(reinterpret_cast<uint2 *>(packed) + chunk, make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)));
            }
            if ((chunk & 3) == 0) scales[chunk >> 2] = (uint8_t)code;
            return;
        }
    }
    // The reference's arithmetic step by step: every group of NVFP4 (its scale is no power of two), and the groups
    // of the MX formats with a NaN, an infinity, or a scale at either end of the range.  The lanes of a group are
    // all here or none is.
    float v[8];
    widen_raw<T>(raw, v);
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        v[i] = ftz(v[i]);
        amax = fmaxf(amax, fabsf(v[i]));  // NaN is ignored, as Rust's f32::max
    }
    amax = fmaxf(amax, u2f(quad_swap<kSwap1>(f2u(amax))));
    if constexpr (F::lanes == 4) amax = fmaxf(amax, u2f(quad_swap<kSwap2>(f2u(amax))));
    float scale = ftz(amax / F::max_element);
    // NVFP4's global scale g (kernels.rs:933, 941-943, 957-961): the group scales are relative to g / (448 * 6).
    float scale_enc = 1.0f;
    if constexpr (!F::mx) {
        if (global_scale != nullptr) {
            scale_enc = ftz(448.0f * 6.0f / *global_scale);
            scale = ftz(scale * scale_enc);
        }
    }
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
    const float inverse = decoded == 0.0f ? 0.0f : ftz(scale_enc / decoded);
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

// Eight decoded values of a lane, stored with 16-byte stores.
template <typename T> __device__ __forceinline__ void store_values(T *out, int64_t base, const float (&v)[8]) {
    if constexpr (sizeof(T) == 4) {
        float4 *p = reinterpret_cast<float4 *>(out + base);
        p[0] = make_float4(v[0], v[1], v[2], v[3]);
        p[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        uint32_t r[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if constexpr (Elem<T>::code == 10) {
                r[i] = f32_to_bf16_pair(v[2 * i], v[2 * i + 1]);
            } else {
                const f16x2_t h = {(_Float16)v[2 * i], (_Float16)v[2 * i + 1]};
                r[i] = __builtin_bit_cast(uint32_t, h);
            }
        }
        stream_store(reinterpret_cast<uint4 *>(out + base), make_uint4(r[0], r[1], r[2], r[3]));
    }
}

// kernels.rs:1011-1065 (MLX's fp_quantize_dequantize, the activations of `qqmm`): per group the scale as the quantizer
// encodes it, each value (scale / scale_enc) * float(code) in float32 and one rounding to the input's type.  The
// reference's arithmetic step by step (the scaled conversions would need the same edge handling as the quantizer for
// what is a small operand: the activations of one product).
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock)
fp_quantize_dequantize_kernel(const T *__restrict__ w, int64_t chunks, T *__restrict__ out, const float *__restrict__ global_scale) {
    using F = Format<MODE>;
    const int64_t chunk = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (chunk >= chunks) return;  // a group is wholly in or out of range
    const Raw<T> raw = load_raw<T>(w, chunk);
    float v[8];
    widen_raw<T>(raw, v);
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        v[i] = ftz(v[i]);
        amax = fmaxf(amax, fabsf(v[i]));
    }
    amax = fmaxf(amax, u2f(quad_swap<kSwap1>(f2u(amax))));
    if constexpr (F::lanes == 4) amax = fmaxf(amax, u2f(quad_swap<kSwap2>(f2u(amax))));
    float scale = ftz(amax / F::max_element);
    const bool scaled = global_scale != nullptr;
    const float scale_enc = scaled ? ftz(448.0f * 6.0f / *global_scale) : 1.0f;
    if (scaled) scale = ftz(scale * scale_enc);
    float decoded;
    if (F::mx && !scaled) decoded = e8m0_to_f32(e8m0_round_up_code(scale));
    else decoded = e4m3_to_f32(e4m3_from_f32(scale));
    decoded = ftz(decoded);
    const float enc_b = decoded == 0.0f ? 0.0f : ftz(scale_enc / decoded);
    const float dec = ftz(decoded / scale_enc);
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float t = canonical(ftz(v[i] * enc_b));
        const float value = F::bits == 8 ? e4m3_to_f32(e4m3_from_f32(t)) : e2m1_to_f32(e2m1_from_f32(t));
        r[i] = canonical(ftz(dec * value));
    }
    store_values<T>(out, chunk * 8, r);
}

// kernels.rs:976-1009.  With `ids`, output row r is table row ids[r] (`row_chunks` chunks per row, ids clamped to
// `table_rows`): the rows of a quantized embedding.  A thread owns kUnroll chunks a block apart and requests the
// codes and scales of all of them before it converts the first: a wavefront that moved one chunk per lane had too
// few bytes in flight to cover the memory latency (4.1 TB/s at C5's weights).
constexpr int kUnroll = 4;
template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock)
fp_dequantize_kernel(const uint32_t *__restrict__ packed, const uint8_t *__restrict__ scales, uint32_t chunks, T *__restrict__ out,
                     const uint32_t *__restrict__ ids, uint32_t row_chunks, int64_t table_rows, const float *__restrict__ global_scale) {
    using F = Format<MODE>;
    const uint32_t first = blockIdx.x * (kBlock * kUnroll) + threadIdx.x;  // fewer than 2^29: an operand has fewer than 2^32 elements
    uint32_t code_lo[kUnroll], code_hi[kUnroll], sc_[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint32_t at = first + u * kBlock;
        const uint32_t oc = at < chunks ? at : chunks - 1;  // past the end: the last chunk again, never stored
        int64_t chunk = oc;
        if (ids != nullptr) {
            const uint32_t r = oc / row_chunks;
            const int64_t row = min((int64_t)ids[r], table_rows - 1);
            chunk = row * row_chunks + (oc - r * row_chunks);
        }
        sc_[u] = scales[chunk / F::lanes];
        if constexpr (F::bits == 4) {
            code_lo[u] = stream_load(packed + chunk);
            code_hi[u] = 0u;
        } else {
            const uint2 words = stream_load(reinterpret_cast<const uint2 *>(packed) + chunk);
            code_lo[u] = words.x;
            code_hi[u] = words.y;
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint32_t out_chunk = first + u * kBlock;
        if (out_chunk >= chunks) continue;
        const uint32_t sc = sc_[u], word = code_lo[u];
        const int64_t base = (int64_t)out_chunk * 8;
        if constexpr (MODE == NVQ_MXFP4) {
            if (sc - 2u <= 252u) {  // one instruction per pair of codes
                const float scale = u2f(sc << 23);
                if constexpr (sizeof(T) == 4) {
                    const f32x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, scale, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, scale, 1),
                                  c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, scale, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, scale, 3);
                    float4 *p = reinterpret_cast<float4 *>(out + base);
                    p[0] = make_float4(a.x, a.y, b.x, b.y);
                    p[1] = make_float4(c.x, c.y, d.x, d.y);
                } else if constexpr (Elem<T>::code == 10) {
                    const bf16x2_t a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 0), b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 1),
                                   c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 2), d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 3);
                    stream_store(reinterpret_cast<uint4 *>(out + base), make_uint4(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                                                                                   __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, d)));
                } else {
                    const f16x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, scale, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, scale, 1),
                                  c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, scale, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, scale, 3);
                    stream_store(reinterpret_cast<uint4 *>(out + base), make_uint4(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                                                                                   __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, d)));
                }
                continue;
            }
        }
        float scale = ftz(F::mx ? e8m0_to_f32(sc) : e4m3_to_f32(sc));
        if constexpr (!F::mx) {  // NVFP4's global scale (kernels.rs:992, 996-998)
            if (global_scale != nullptr) scale = ftz(scale * ftz(*global_scale / (448.0f * 6.0f)));
        }
        float v[8];
        if constexpr (F::bits == 4) {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = canonical(ftz(scale * e2m1_to_f32((word >> (4 * i)) & 0xFu)));
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                v[i] = canonical(ftz(scale * e4m3_to_f32((code_lo[u] >> (8 * i)) & 0xFFu)));
                v[4 + i] = canonical(ftz(scale * e4m3_to_f32((code_hi[u] >> (8 * i)) & 0xFFu)));
            }
        }
        store_values<T>(out, base, v);
    }
}

// float32 out: a lane's eight values would leave as two 16-byte stores 32 bytes apart.  Here a lane takes four values, one
// half of a chunk, of two chunks that lie 32 chunks apart, so that each of a wavefront's two stores writes 1 KB of
// consecutive bytes, non-temporally; the two lanes of a chunk read the same codes and scale.  A value's arithmetic is
// that of the kernel above (MXFP4 [4096,4096]: 21.1 us with the eight-value lanes).
template <int MODE>
__global__ void __launch_bounds__(kBlock)
fp_dequantize_f32_kernel(const uint32_t *__restrict__ packed, const uint8_t *__restrict__ scales, uint32_t chunks, float *__restrict__ out,
                         const uint32_t *__restrict__ ids, uint32_t row_chunks, int64_t table_rows, const float *__restrict__ global_scale) {
    using F = Format<MODE>;
    const uint32_t lane = threadIdx.x & 63u, half = lane & 1u;
    const uint32_t first = blockIdx.x * kBlock + (threadIdx.x & ~63u);  // the wavefront's 64 chunks
    uint32_t word_[2], sc_[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t at = first + 32 * j + (lane >> 1);
        const uint32_t oc = at < chunks ? at : chunks - 1;  // past the end: the last chunk again, never stored
        int64_t chunk = oc;
        if (ids != nullptr) {
            const uint32_t r = oc / row_chunks;
            const int64_t row = min((int64_t)ids[r], table_rows - 1);
            chunk = row * row_chunks + (oc - r * row_chunks);
        }
        sc_[j] = scales[chunk / F::lanes];
        // the half's four codes: the low or high 16 bits of the chunk's word, or one of its two words
        if constexpr (F::bits == 4) word_[j] = stream_load(packed + chunk) >> (16 * half);
        else word_[j] = stream_load(packed + 2 * chunk + half);
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t out_chunk = first + 32 * j + (lane >> 1);
        if (out_chunk >= chunks) continue;
        const uint32_t sc = sc_[j], word = word_[j];
        float v[4];
        bool done = false;
        if constexpr (MODE == NVQ_MXFP4) {
            if (sc - 2u <= 252u) {  // one instruction per pair of codes
                const float scale = u2f(sc << 23);
                const f32x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, scale, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, scale, 1);
                v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
                done = true;
            }
        }
        if (!done) {
            float scale = ftz(F::mx ? e8m0_to_f32(sc) : e4m3_to_f32(sc));
            if constexpr (!F::mx) {  // NVFP4's global scale (kernels.rs:992, 996-998)
                if (global_scale != nullptr) scale = ftz(scale * ftz(*global_scale / (448.0f * 6.0f)));
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
                v[i] = canonical(ftz(scale * (F::bits == 4 ? e2m1_to_f32((word >> (4 * i)) & 0xFu) : e4m3_to_f32((word >> (8 * i)) & 0xFFu))));
        }
        stream_store(reinterpret_cast<uint4 *>(out + (int64_t)out_chunk * 8 + half * 4), make_uint4(f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])));
    }
}

template <typename T, int MODE>
int32_t quantize_t(const void *w, int64_t n, void *packed, void *scales, const float *global_scale, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((fp_quantize_kernel<T, MODE>), dim3(blocks), dim3(kBlock), 0, s, (const T *)w, chunks,
                       (uint32_t *)packed, (uint8_t *)scales, global_scale);
    NVQ_LAUNCH_CHECK("fp_quantize");
    return NVQ_OK;
}
template <typename T, int MODE>
int32_t dequantize_t(const void *packed, const void *scales, int64_t n, void *out, const uint32_t *ids, int64_t cols,
                     int64_t table_rows, const float *global_scale, hipStream_t s) {
    const int64_t chunks = n / 8;
    if constexpr (std::is_same<T, float>::value) {
        hipLaunchKernelGGL((fp_dequantize_f32_kernel<MODE>), dim3((unsigned)((chunks + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, (const uint32_t *)packed,
                           (const uint8_t *)scales, (uint32_t)chunks, (float *)out, ids, (uint32_t)(cols / 8), table_rows, global_scale);
        NVQ_LAUNCH_CHECK("fp_dequantize");
        return NVQ_OK;
    }
    const unsigned blocks = (unsigned)((chunks + kBlock * kUnroll - 1) / (kBlock * kUnroll));
    hipLaunchKernelGGL((fp_dequantize_kernel<T, MODE>), dim3(blocks), dim3(kBlock), 0, s, (const uint32_t *)packed,
                       (const uint8_t *)scales, (uint32_t)chunks, (T *)out, ids, (uint32_t)(cols / 8), table_rows, global_scale);
    NVQ_LAUNCH_CHECK("fp_dequantize");
    return NVQ_OK;
}

template <typename T, int MODE>
int32_t quantize_dequantize_t(const void *w, int64_t n, void *out, const float *g, hipStream_t s) {
    const int64_t chunks = n / 8;
    const unsigned blocks = (unsigned)((chunks + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((fp_quantize_dequantize_kernel<T, MODE>), dim3(blocks), dim3(kBlock), 0, s, (const T *)w, chunks, (T *)out, g);
    NVQ_LAUNCH_CHECK("fp_quantize_dequantize");
    return NVQ_OK;
}
template <typename T>
int32_t quantize_dequantize_mode(int32_t mode, const void *w, int64_t n, void *out, const float *g, hipStream_t s) {
    switch (mode) {
    case NVQ_MXFP4: return quantize_dequantize_t<T, NVQ_MXFP4>(w, n, out, g, s);
    case NVQ_MXFP8: return quantize_dequantize_t<T, NVQ_MXFP8>(w, n, out, g, s);
    case NVQ_NVFP4: return quantize_dequantize_t<T, NVQ_NVFP4>(w, n, out, g, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "quantize_dequantize: mode %s is not a floating-point block format", mode_name(mode));
    }
}
template <typename T>
int32_t quantize_mode(int32_t mode, const void *w, int64_t n, void *packed, void *scales, const float *g, hipStream_t s) {
    switch (mode) {
    case NVQ_MXFP4: return quantize_t<T, NVQ_MXFP4>(w, n, packed, scales, g, s);
    case NVQ_MXFP8: return quantize_t<T, NVQ_MXFP8>(w, n, packed, scales, g, s);
    case NVQ_NVFP4: return quantize_t<T, NVQ_NVFP4>(w, n, packed, scales, g, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "quantize: mode %s is not a floating-point block format", mode_name(mode));
    }
}
template <typename T>
int32_t dequantize_mode(int32_t mode, const void *packed, const void *scales, int64_t n, void *out, const uint32_t *ids,
                        int64_t cols, int64_t table_rows, const float *g, hipStream_t s) {
    switch (mode) {
    case NVQ_MXFP4: return dequantize_t<T, NVQ_MXFP4>(packed, scales, n, out, ids, cols, table_rows, g, s);
    case NVQ_MXFP8: return dequantize_t<T, NVQ_MXFP8>(packed, scales, n, out, ids, cols, table_rows, g, s);
    case NVQ_NVFP4: return dequantize_t<T, NVQ_NVFP4>(packed, scales, n, out, ids, cols, table_rows, g, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "dequantize: mode %s is not a floating-point block format", mode_name(mode));
    }
}

}  // namespace

int32_t launch_fp_quantize(int32_t mode, int32_t dtype, const void *w, int64_t n, void *packed, void *scales,
                           const float *g, hipStream_t s) {
    switch (dtype) {
    case NVQ_F32: return quantize_mode<float>(mode, w, n, packed, scales, g, s);
    case NVQ_BF16: return quantize_mode<bf16_t>(mode, w, n, packed, scales, g, s);
    default: return quantize_mode<f16_t>(mode, w, n, packed, scales, g, s);
    }
}

int32_t launch_fp_quantize_dequantize(int32_t mode, int32_t dtype, const void *w, int64_t n, void *out, const float *g, hipStream_t s) {
    switch (dtype) {
    case NVQ_F32: return quantize_dequantize_mode<float>(mode, w, n, out, g, s);
    case NVQ_BF16: return quantize_dequantize_mode<bf16_t>(mode, w, n, out, g, s);
    default: return quantize_dequantize_mode<f16_t>(mode, w, n, out, g, s);
    }
}

int32_t launch_fp_dequantize(int32_t mode, int32_t out_dtype, const void *packed, const void *scales, int64_t n,
                             void *out, const uint32_t *ids, int64_t cols, int64_t table_rows, const float *g, hipStream_t s) {
    switch (out_dtype) {
    case NVQ_F32: return dequantize_mode<float>(mode, packed, scales, n, out, ids, cols, table_rows, g, s);
    case NVQ_BF16: return dequantize_mode<bf16_t>(mode, packed, scales, n, out, ids, cols, table_rows, g, s);
    default: return dequantize_mode<f16_t>(mode, packed, scales, n, out, ids, cols, table_rows, g, s);
    }
}

}  // namespace nvq
