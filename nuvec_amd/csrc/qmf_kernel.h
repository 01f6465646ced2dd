// Few-row quantized products on the gfx950 matrix cores: y[m, n] = x[m, :] . dequantize(w[n, :]) for up to
// 32 rows of x per pass.  Values follow nuvec's CPU product (reference:
// crates/nuvec-core/src/kernels.rs:1091-1142) within the stated tolerance.  (The grouped gathered product
// of mixture-of-experts layers has its own kernel, qmg_kernel.h, which shares the code expansion below.)
//
// This header holds the kernel template; qmf_b*.hip instantiate it per code width (affine 2, 3, 4, 6, 8 bits
// and MXFP4) so that the widths compile in parallel.
//
// The weights are the large operand and each weight is decoded exactly once per pass.  The kernel is bound
// by the memory instructions it issues, so everything is arranged to issue few, wide, coalesced ones:
//   * a block of eight wavefronts owns 32 RG weight rows (RG = 1 or 2 groups of 32) and splits K into
//     contiguous ranges, one per wavefront.  A wavefront takes its range in windows of two steps
//     (128 values = 16 BITS bytes of every row, i.e. BITS chunks of 16 bytes): its loads, each a wavefront of
//     consecutive chunks, fetch a window into registers several windows ahead; the window then goes through
//     a private piece of LDS (chunks XOR-swizzled by row where BITS is a power of two) to reach the matrix
//     operand layout, in which a lane (row n = lane % 32, half h = lane / 32) holds the 32 codes (BITS
//     dwords) of its half of a step for every row group;
//   * the scales and biases of the block's rows are one contiguous piece of memory: it is copied once,
//     coalesced, into an LDS table (rows padded against bank conflicts), and read from there;
//   * the pieces of x are shared by the row groups, and a pass of at most 8 (16) rows of x packs four
//     (two) of a step's pieces into one load: lane (row r = l % XR, slot q = l / XR) of a half loads the
//     pieces q NL .. q NL + NL - 1 (NL = XR / 8), the matrix instruction of piece kk takes that register with the
//     lanes of other slots cleared, so row r + XR q of the accumulator holds the share of piece kk and the
//     shares are added when the tile is written.
// Codes are expanded into matrix operands in registers (affine: code -> float -> fma -> packed convert;
// MXFP4: one scaled FP4 -> element-type conversion per two codes).  The K order inside a step is permuted
// consistently for both operands (piece kk of half h holds values 32 h + 8 kk .. + 8 of the step).  The
// wavefronts' partial tiles are summed through LDS in a fixed order, so results do not depend on scheduling.
#pragma once

#include "nvq_device.h"
#include "nvq_internal.h"

#include <type_traits>
#include <utility>

namespace nvq {
namespace qmf {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2v_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
// The FP4 template parameter of the kernels below names the code format: 0 affine integers with a scale and a bias per
// group, 1 MXFP4 (E2M1 codes, an E8M0 scale per 32), 2 MXFP8 (E4M3 codes, an E8M0 scale per 32), 3 NVFP4 (E2M1 codes, an
// E4M3 scale per 16, times the factor of a global scale where the product has one).  Every weight of the block formats
// is exact in bfloat16 and float16 (at most six significant bits times a power of two) but for NVFP4 with a global
// scale, whose weights are rounded once to the element type like the affine ones.
constexpr int kAffine = 0, kMxfp4 = 1, kMxfp8 = 2, kNvfp4 = 3;
typedef float floatx16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef u32x4_t u32x4_a4_t __attribute__((aligned(4)));  // 16 bytes in memory at any dword

constexpr int kWaves = 8;  // wavefronts per block, each with its own range of K
constexpr int kThreads = 64 * kWaves;
constexpr int kLdsLimit = 160 * 1024;

// Sizes that follow from the code width and the rows per block; shared by the kernel and its launcher.
template <int BITS, int RG>
struct Geometry {
    static constexpr int kRows = 32 * RG;                  // weight rows per block = columns of y
    static constexpr int kChunks = kRows * BITS;           // 16-byte chunks of one window
    static constexpr int kLoads = (kChunks + 63) / 64;     // loads per lane and window
    static constexpr int kDepth = kLoads <= 4 ? 4 : 2;     // windows of weights in flight per lane
    static constexpr int kRowBytes = 16 * BITS;            // of one row in a window
    static constexpr int kStageBytes = kChunks * 16;       // one window of one wavefront
    static constexpr int kPartialBytes = 4 * RG * 16 * 64 * 4;  // four wavefronts' tiles
    static constexpr int kFixedLdsBytes = kPartialBytes + kWaves * kStageBytes;
    static constexpr bool kPow2 = (BITS & (BITS - 1)) == 0;
    // 16-byte chunk c of row `row` sits at chunk position c ^ swizzle(row)
    __host__ __device__ static constexpr int swizzle(int row) { return kPow2 ? (row / (BITS >= 16 ? 1 : 16 / BITS)) % BITS : 0; }
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant in the body
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Byte B of `v` as a float (v_cvt_f32_ubyteB).  `opaque` hides how a word was masked, so that the compiler keeps
// the byte conversions instead of re-deriving bit-field extracts from the mask.
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}
template <int B>
__device__ __forceinline__ float ubyte_to_float(uint32_t v) {
    return (float)((v >> (8 * B)) & 0xFFu);
}

template <typename T> struct Ops;
template <> struct Ops<bf16_t> {
    __device__ static __forceinline__ floatx16_t mfma(uint4 a, uint4 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
        const floatx2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2v_t));
    }
    // The two E2M1 codes of byte B of `word` times `scale`, as two elements (low nibble first).
    template <int B> __device__ static __forceinline__ uint32_t fp4_pair(uint32_t word, float scale) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, B));
    }
    // The two E4M3 codes of the low or high half of `word` times the power of two `scale`.
    template <bool HIGH> __device__ static __forceinline__ uint32_t fp8_pair(uint32_t word, float scale) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(word, scale, HIGH));
    }
    // The codes of a group for the scaled conversions above, which take the exponent field of `scale` alone: an E8M0
    // scale of 2^-127 is zero once flushed (crates/nuvec-core/src/fp8.rs:95-112) but reads as 2^-127 there, and bf16
    // holds 448 x 2^-127, so such a group's codes become code 0 (+0 in E2M1 and in E4M3).
    __device__ static __forceinline__ uint32_t mx_codes(uint32_t word, float scale) { return scale != 0.0f ? word : 0u; }
};
template <> struct Ops<f16_t> {
    __device__ static __forceinline__ floatx16_t mfma(uint4 a, uint4 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
        const floatx2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2v_t));
    }
    template <int B> __device__ static __forceinline__ uint32_t fp4_pair(uint32_t word, float scale) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, scale, B));
    }
    template <bool HIGH> __device__ static __forceinline__ uint32_t fp8_pair(uint32_t word, float scale) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(word, scale, HIGH));
    }
    // (448 x 2^-127 is far below half of f16's smallest subnormal: the conversion itself gives the zero of a flushed scale)
    __device__ static __forceinline__ uint32_t mx_codes(uint32_t word, float) { return word; }
};

// Low / high 16 bits of a word as element-type values.
template <typename T> __device__ __forceinline__ float half_lo(uint32_t p);
template <typename T> __device__ __forceinline__ float half_hi(uint32_t p);
template <> __device__ __forceinline__ float half_lo<bf16_t>(uint32_t p) { return u2f(p << 16); }
template <> __device__ __forceinline__ float half_hi<bf16_t>(uint32_t p) { return u2f(p & 0xFFFF0000u); }
template <> __device__ __forceinline__ float half_lo<f16_t>(uint32_t p) { return (float)__builtin_bit_cast(f16x2v_t, p)[0]; }
template <> __device__ __forceinline__ float half_hi<f16_t>(uint32_t p) { return (float)__builtin_bit_cast(f16x2v_t, p)[1]; }

// Two dequantized affine weights as the element type holds them.  As the reference's device kernels: one rounding of
// fma(code, scale, bias).  EXACT: the CPU's two roundings, round(round(code * scale) + bias)
// (crates/nuvec-core/src/kernels.rs:835-859; code * scale is exact in float32 and the sum of two elements rounds to
// the element type as from the exact sum), so that the weights are bit for bit those nuvec's CPU product multiplies.
template <typename T, bool EXACT>
__device__ __forceinline__ uint32_t affine_pair(float c0, float c1, float s, float b) {
    if constexpr (!EXACT) {
        return Ops<T>::pack(__builtin_fmaf(c0, s, b), __builtin_fmaf(c1, s, b));
    } else {
        const uint32_t p = Ops<T>::pack(c0 * s, c1 * s);
        return Ops<T>::pack(half_lo<T>(p) + b, half_hi<T>(p) + b);
    }
}

// The two E2M1 codes of byte B of `word` times any `scale` (NVFP4: the scale is no power of two, so the scaled
// conversion, which takes the scale's exponent only, does not apply): decoded to float, multiplied, packed.
template <typename T, int B>
__device__ __forceinline__ uint32_t fp4_pair_times(uint32_t word, float scale) {
    const floatx2_t v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, B);
    return Ops<T>::pack(v.x * scale, v.y * scale);
}

// NVFP4 with a global scale g (reference: crates/nuvec-core/src/kernels.rs:992-998): every group scale becomes
// ftz(scale * ftz(g / (448 * 6))); a gather has one g per expert (quantized.rs:620-636).  Without one the factor is 1,
// which changes no bit of a scale.
__device__ __forceinline__ float nvfp4_factor(const ProductArgs &a, int64_t expert) {
    if (a.global_scale == nullptr) return 1.0f;
    const int64_t e = a.rhs != nullptr ? (expert < a.experts ? expert : a.experts - 1) : 0;
    return ftz(a.global_scale[e] / (448.0f * 6.0f));
}
__device__ __forceinline__ float nvfp4_scale(uint32_t code, float factor) { return ftz(ftz(e4m3_to_f32(code)) * factor); }

// Code J of a lane's 32 codes (BITS dwords, value i in bits i BITS .. of the stream) as a float.
template <int BITS, int J>
__device__ __forceinline__ float code_to_float(const uint32_t (&dw)[BITS]) {
    constexpr int bit = J * BITS, d = bit / 32, s = bit % 32;
    constexpr uint32_t mask = (1u << BITS) - 1u;
    if constexpr (BITS == 8) {
        return ubyte_to_float<s / 8>(dw[d]);
    } else if constexpr (s + BITS <= 32) {
        return (float)((dw[d] >> s) & mask);
    } else {
        return (float)(((dw[d] >> s) | (dw[d + 1] << (32 - s))) & mask);
    }
}

// Piece KK (eight codes, stream order) of a lane's 32 codes as one matrix operand.
template <typename T, int BITS, int FP4, int KK, bool EXACT = false>
__device__ __forceinline__ uint4 expand_piece(const uint32_t (&dw)[BITS], float s, float b) {
    uint4 r;
    if constexpr (FP4 == kMxfp8) {
        const uint32_t w0 = Ops<T>::mx_codes(dw[2 * KK], s), w1 = Ops<T>::mx_codes(dw[2 * KK + 1], s);
        r.x = Ops<T>::template fp8_pair<false>(w0, s);
        r.y = Ops<T>::template fp8_pair<true>(w0, s);
        r.z = Ops<T>::template fp8_pair<false>(w1, s);
        r.w = Ops<T>::template fp8_pair<true>(w1, s);
    } else if constexpr (FP4 == kNvfp4) {
        const uint32_t word = dw[KK];
        r.x = fp4_pair_times<T, 0>(word, s);
        r.y = fp4_pair_times<T, 1>(word, s);
        r.z = fp4_pair_times<T, 2>(word, s);
        r.w = fp4_pair_times<T, 3>(word, s);
    } else if constexpr (FP4) {
        const uint32_t word = Ops<T>::mx_codes(dw[KK], s);
        r.x = Ops<T>::template fp4_pair<0>(word, s);
        r.y = Ops<T>::template fp4_pair<1>(word, s);
        r.z = Ops<T>::template fp4_pair<2>(word, s);
        r.w = Ops<T>::template fp4_pair<3>(word, s);
    } else if constexpr (BITS == 4) {
        const uint32_t word = dw[KK];
        const uint32_t even = opaque(word & 0x0F0F0F0Fu), odd = opaque((word >> 4) & 0x0F0F0F0Fu);
        r.x = affine_pair<T, EXACT>(ubyte_to_float<0>(even), ubyte_to_float<0>(odd), s, b);
        r.y = affine_pair<T, EXACT>(ubyte_to_float<1>(even), ubyte_to_float<1>(odd), s, b);
        r.z = affine_pair<T, EXACT>(ubyte_to_float<2>(even), ubyte_to_float<2>(odd), s, b);
        r.w = affine_pair<T, EXACT>(ubyte_to_float<3>(even), ubyte_to_float<3>(odd), s, b);
    } else {
        constexpr int J = 8 * KK;
        r.x = affine_pair<T, EXACT>(code_to_float<BITS, J + 0>(dw), code_to_float<BITS, J + 1>(dw), s, b);
        r.y = affine_pair<T, EXACT>(code_to_float<BITS, J + 2>(dw), code_to_float<BITS, J + 3>(dw), s, b);
        r.z = affine_pair<T, EXACT>(code_to_float<BITS, J + 4>(dw), code_to_float<BITS, J + 5>(dw), s, b);
        r.w = affine_pair<T, EXACT>(code_to_float<BITS, J + 6>(dw), code_to_float<BITS, J + 7>(dw), s, b);
    }
    return r;
}

// The LDS table of scales (or biases) of a block's rows keeps the memory order [row][group] with rows padded
// to an odd number of dwords, so that the coalesced copy in writes neighbouring addresses and lanes reading
// one group of consecutive rows fall on different banks.
__host__ __device__ inline int table_stride(int kgroups, int elem_bytes) { return 4 * (((kgroups * elem_bytes + 3) / 4) | 1); }

// Copies `count` elements (whole rows of `kgroups`) starting at `src` into the table: aligned 16-byte pieces,
// each thread scattering its piece's elements; bytes of a piece outside the rows are dropped.
template <typename S, int THREADS>
__device__ __forceinline__ void fill_table(unsigned char *table, const S *src, int count, int kgroups, int stride, int tid) {
    constexpr int kPer = 16 / (int)sizeof(S);
    const int skew = (int)((uintptr_t)src & 15) / (int)sizeof(S);  // elements before src in its first piece
    const uint4 *pieces = reinterpret_cast<const uint4 *>(src - skew);
    const int n_pieces = (skew + count + kPer - 1) / kPer;
    for (int p = tid; p < n_pieces; p += THREADS) {
        const uint4 v = pieces[p];
        S elems[kPer];
        __builtin_memcpy(elems, &v, 16);
        int idx = p * kPer - skew;  // element index of elems[0] within the block's rows
        int row = idx >= 0 ? idx / kgroups : 0, g = idx >= 0 ? idx - row * kgroups : 0;
#pragma unroll
        for (int e = 0; e < kPer; e++, idx++) {
            if (idx >= 0 && idx < count) {
                *reinterpret_cast<S *>(table + row * stride + g * (int)sizeof(S)) = elems[e];
                if (++g == kgroups) g = 0, row++;
            }
        }
    }
}

// blockIdx.z is a batch with one stride per operand, or a gathered pair; blockIdx.y a pass of 32 rows.
// EXACT (affine codes): the weights as nuvec's CPU product holds them (affine_pair).
template <typename T, int BITS, int FP4, int RG, bool EXACT = false>
__global__ void __launch_bounds__(kThreads) qmf_kernel(const ProductArgs a) {
    using G = Geometry<BITS, RG>;
    constexpr int kRows = G::kRows, kDepth = G::kDepth, kLoads = G::kLoads;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    float *partial = reinterpret_cast<float *>(lds);  // [4][RG][values][64]
    using S = std::conditional_t<FP4 != 0, uint8_t, T>;    // stored scale type
    unsigned char *table_s = lds + G::kFixedLdsBytes;  // scales [rows][groups, padded]; the biases follow
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, l32 = lane & 31;
    const int K = (int)a.k, N = (int)a.n;
    const int gshift = FP4 == kNvfp4 ? 4 : FP4 ? 5 : (a.group == 32 ? 5 : a.group == 64 ? 6 : 7);
    const int kgroups = K >> gshift;
    const int64_t row_bytes = (int64_t)(K >> 3) * BITS;  // of one packed weight row
    const int tstride = table_stride(kgroups, (int)sizeof(S));
    unsigned char *table_b = table_s + kRows * tstride;
    const int n0 = blockIdx.x * kRows;

    int row_begin, row_end;  // rows of x (and of y) this block multiplies
    int64_t xo = 0, wo = 0, so = 0, yo = 0, bo = 0;
    row_begin = blockIdx.y * 32;
    row_end = row_begin + 32 < (int)a.m ? row_begin + 32 : (int)a.m;
    if (a.rhs != nullptr) {  // gathered pairs: pair z takes x batch lhs[z] and weight matrix rhs[z]
        // An index outside its operand is the caller's error; it is clamped so that it cannot fault the device.
        const int64_t l = min((int64_t)a.lhs[blockIdx.z], a.x_batches - 1), r = min((int64_t)a.rhs[blockIdx.z], a.experts - 1);
        xo = l * a.m * K;
        wo = r * N * row_bytes;
        so = r * N * kgroups;
        if (a.row_bias_per_expert) bo = r * N;
        yo = (a.out_rows != nullptr ? min((int64_t)a.out_rows[blockIdx.z], a.batch - 1) : (int64_t)blockIdx.z) * a.m * N;
    } else if (a.batch_ndim > 0) {
        xo = (int64_t)blockIdx.z * a.x_strides[0];
        wo = (int64_t)blockIdx.z * a.w_strides[0] * 4;  // the stride counts packed words
        so = (int64_t)blockIdx.z * a.s_strides[0];
        yo = (int64_t)blockIdx.z * a.m * N;
    }
    const T *x = (const T *)a.x + xo;
    T *y = (T *)a.y + yo;

    // K in steps of 64 values, split over the wavefronts in windows of two steps.
    const int steps = K >> 6;
    const int windows = (steps + 1) >> 1;
    const int s_begin = 2 * (windows * wave / kWaves);
    const int s_end = 2 * (windows * (wave + 1) / kWaves) < steps ? 2 * (windows * (wave + 1) / kWaves) : steps;

    // Window loads: load j of this lane is chunk q = 64 j + lane of the window, i.e. chunk q % BITS of
    // row q / BITS.  Chunks of the window's second step begin at BITS / 2 (a window that ends the range
    // early exists only for even BITS; its lanes fetch the first step again).
    const unsigned char *wload[kLoads];
    int wstore[kLoads];  // byte offset of the chunk within the wavefront's stage
    bool second[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        const int q = 64 * j + lane, qc = q < G::kChunks ? q : G::kChunks - 1;
        const int row = qc / BITS, c = qc % BITS;
        const int n = n0 + row < N ? n0 + row : N - 1;  // tail rows are computed, not stored
        wload[j] = (const unsigned char *)a.w + wo + (int64_t)n * row_bytes + 16 * c;
        wstore[j] = row * G::kRowBytes + 16 * (c ^ G::swizzle(row));
        second[j] = 2 * c >= BITS;
    }
    // Every load of the K loop is issued on every path, so that the number of loads in flight is known where
    // a window is consumed and the wait leaves the younger windows' loads outstanding.  A window past the
    // range loads the first 16 bytes of the weights instead (one address for all lanes).
    auto load_window = [&](int step, u32x4_t (&w)[kLoads]) {
        const bool real = step < s_end, half = step + 1 >= s_end;
#pragma unroll
        for (int j = 0; j < kLoads; j++) {
            const int off = step * 8 * BITS - ((half && second[j]) ? 8 * BITS : 0);
            const unsigned char *src = real ? wload[j] + off : (const unsigned char *)a.w;
            w[j] = *reinterpret_cast<const u32x4_a4_t *>(src);
        }
    };
    unsigned char *stage = lds + G::kPartialBytes + wave * G::kStageBytes;
    // Operand reads: the BITS dwords of half h of step t of row l32 (row group 0), in pieces that do not
    // straddle a chunk.
    constexpr int kPiece = BITS % 4 == 0 ? 4 : BITS % 2 == 0 ? 2 : 1;  // dwords per LDS read
    constexpr int kPieces = BITS / kPiece;
    int wread[2][kPieces];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int p = 0; p < kPieces; p++) {
            const int byte = (2 * t + h) * 4 * BITS + 4 * kPiece * p;  // within the row
            wread[t][p] = l32 * G::kRowBytes + 16 * ((byte >> 4) ^ G::swizzle(l32)) + (byte & 15);
        }
    static_assert(G::swizzle(32) == 0 && G::swizzle(33) == G::swizzle(1), "row groups share the swizzle of their rows");

    const float factor = FP4 == kNvfp4 ? nvfp4_factor(a, a.rhs != nullptr ? (int64_t)a.rhs[blockIdx.z] : 0) : 1.0f;
    // The scale (NVFP4: the two scales, one per 16 values) and bias of this lane's 32 values of a step.
    auto load_scales = [&](int step, float (&scale)[RG][2], float (&bias)[RG]) {
        const int g = (step * 64 + 32 * h) >> gshift;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const int at = (32 * rg + l32) * tstride + g * (int)sizeof(S);
            const S *sp = reinterpret_cast<const S *>(table_s + at), *bp = reinterpret_cast<const S *>(table_b + at);
            if constexpr (FP4 == kNvfp4) {
                scale[rg][0] = nvfp4_scale(sp[0], factor);
                scale[rg][1] = nvfp4_scale(sp[1], factor);
                bias[rg] = 0.0f;
            } else if constexpr (FP4) {
                scale[rg][0] = scale[rg][1] = ftz(e8m0_to_f32(*sp));
                bias[rg] = 0.0f;
            } else {
                scale[rg][0] = scale[rg][1] = Elem<T>::load(sp, 0);
                bias[rg] = Elem<T>::load(bp, 0);
            }
        }
    };

    {
        // The scales (and biases) of rows n0 .. n0 + kRows - 1 are contiguous in memory.
        const int valid_rows = N - n0 < kRows ? N - n0 : kRows;
        fill_table<S, kThreads>(table_s, (const S *)a.scales + so + (int64_t)n0 * kgroups, valid_rows * kgroups, kgroups, tstride, tid);
        if constexpr (!FP4)
            fill_table<S, kThreads>(table_b, (const S *)a.biases + so + (int64_t)n0 * kgroups, valid_rows * kgroups, kgroups, tstride, tid);
    }

    // One pass over at most XR rows of x (XR = 8, 16 or 32).
    auto run_pass = [&](auto xr_tag, int pass, int rows) {
        constexpr int XR = decltype(xr_tag)::value;
        constexpr int NL = XR / 8;        // loads of x per step
        constexpr int XD = (32 / XR) < kDepth ? (32 / XR) : kDepth;  // windows of x in flight (kDepth is a multiple of it)
        constexpr int NV = XR / 2;        // values of the tile per lane and row group once the slots are added
        const int r = l32 % XR, slot = l32 / XR;
        const bool live = r < rows;  // this lane's row of x exists
        const int64_t xr = pass + (live ? r : 0);  // x row of this lane
        const T *xrow = x + xr * K + 32 * h + 8 * NL * slot;  // piece kk of half h covers k0 + 32 h + 8 kk .. + 8

        floatx16_t acc[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[rg][e] = 0.0f;

        u32x4_t ring[kDepth][kLoads] = {};  // windows in flight
        uint4 xring[XD][2][NL] = {};        // x pieces, XD windows ahead (they come from the cache)
        // Lanes without a row of x read the pass's first row: their tile rows are never stored.
        auto load_x = [&](int step, uint4 (&xf)[2][NL]) {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int sc = step + t < s_end ? step + t : (step < s_end ? step : s_begin);
#pragma unroll
                for (int j = 0; j < NL; j++) xf[t][j] = *reinterpret_cast<const uint4 *>(xrow + sc * 64 + 8 * j);
            }
        };
        static_for<kDepth>([&](auto d_tag) {
            constexpr int d = decltype(d_tag)::value;
            load_window(s_begin + 2 * d, ring[d]);
            if constexpr (d < XD) load_x(s_begin + 2 * d, xring[d]);
        });
        __syncthreads();  // first pass: the table is written; later passes: nothing pending

        for (int s0 = s_begin; s0 < s_end; s0 += 2 * kDepth) {
            static_for<kDepth>([&](auto d_tag) {
                constexpr int d = decltype(d_tag)::value;
                const int step = s0 + 2 * d;
                // through LDS into the operand layout; the wavefront's LDS accesses execute in order
                asm volatile("" ::: "memory");
#pragma unroll
                for (int j = 0; j < kLoads; j++)
                    if (G::kChunks % 64 == 0 || 64 * j + lane < G::kChunks) *reinterpret_cast<u32x4_t *>(stage + wstore[j]) = ring[d][j];
                load_window(step + 2 * kDepth, ring[d]);  // the registers are free again: refill them
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");
                uint32_t codes[2][RG][BITS];
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int rg = 0; rg < RG; rg++)
#pragma unroll
                        for (int p = 0; p < kPieces; p++) {
                            const unsigned char *src = stage + wread[t][p] + rg * 32 * G::kRowBytes;
                            if constexpr (kPiece == 4) {
                                const u32x4_t v = *reinterpret_cast<const u32x4_t *>(src);
                                codes[t][rg][4 * p] = v.x, codes[t][rg][4 * p + 1] = v.y, codes[t][rg][4 * p + 2] = v.z, codes[t][rg][4 * p + 3] = v.w;
                            } else if constexpr (kPiece == 2) {
                                const u32x2_t v = *reinterpret_cast<const u32x2_t *>(src);
                                codes[t][rg][2 * p] = v.x, codes[t][rg][2 * p + 1] = v.y;
                            } else {
                                codes[t][rg][p] = *reinterpret_cast<const uint32_t *>(src);
                            }
                        }
                asm volatile("" ::: "memory");
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    if (step + t < s_end) {
                        float scale[RG][2], bias[RG];
                        load_scales(step + t, scale, bias);
                        static_for<4>([&](auto kk_tag) {
                            constexpr int kk = decltype(kk_tag)::value;
                            uint4 xa = xring[d % XD][t][kk % NL];
                            if constexpr (XR < 32) {
                                const bool mine = slot == kk / NL;
                                xa.x = mine ? xa.x : 0u, xa.y = mine ? xa.y : 0u, xa.z = mine ? xa.z : 0u, xa.w = mine ? xa.w : 0u;
                            }
#pragma unroll
                            for (int rg = 0; rg < RG; rg++)
                                acc[rg] = Ops<T>::mfma(xa, expand_piece<T, BITS, FP4, kk, EXACT>(codes[t][rg], scale[rg][kk >> 1], bias[rg]), acc[rg]);
                        });
                    }
                }
                // x of this window is used up: refill its registers (only now, so that the same registers serve
                // and no copy, which would have to wait for the data, is needed at the loop's end)
                load_x(step + 2 * XD, xring[d % XD]);
            });
        }

        // Accumulator element e of lane l is tile row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32; tile rows
        // r, r + XR, ... are the slots' shares of row r of x.
        float vals[RG][NV];
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
#pragma unroll
            for (int v = 0; v < NV; v++) {
                float sum = acc[rg][v];
#pragma unroll
                for (int q = 1; q < 32 / XR; q++) sum += acc[rg][v + NV * q];
                vals[rg][v] = sum;
            }
        // Sum the wavefronts' partial tiles in a fixed order: the upper four hand theirs to the lower four,
        // whose tiles are then added in wavefront order.
        auto slot_of = [&](int w, int rg, int v) -> float * { return partial + ((w * RG + rg) * NV + v) * 64; };
        if (wave >= 4) {
#pragma unroll
            for (int rg = 0; rg < RG; rg++)
#pragma unroll
                for (int v = 0; v < NV; v++) slot_of(wave - 4, rg, v)[lane] = vals[rg][v];
        }
        __syncthreads();
        if (wave < 4) {
#pragma unroll
            for (int rg = 0; rg < RG; rg++)
#pragma unroll
                for (int v = 0; v < NV; v++) vals[rg][v] += slot_of(wave, rg, v)[lane];
        }
        __syncthreads();
        if (wave < 4) {
#pragma unroll
            for (int rg = 0; rg < RG; rg++)
#pragma unroll
                for (int v = 0; v < NV; v++) slot_of(wave, rg, v)[lane] = vals[rg][v];
        }
        __syncthreads();
        for (int idx = tid; idx < RG * NV * 64; idx += kThreads) {
            const int l = idx & 63, v = (idx >> 6) % NV, rg = idx / (64 * NV);
            const float sum = ((slot_of(0, rg, v)[l] + slot_of(1, rg, v)[l]) + slot_of(2, rg, v)[l]) + slot_of(3, rg, v)[l];
            const int m = 8 * (v >> 2) + 4 * (l >> 5) + (v & 3), col = n0 + 32 * rg + (l & 31);
            if (m < rows && col < N) Elem<T>::store(y, (int64_t)(pass + m) * N + col, add_row_bias<T>(a.row_bias, sum, bo + col));
        }
        __syncthreads();
    };

    for (int pass = row_begin; pass < row_end; pass += 32) {
        const int rows = row_end - pass < 32 ? row_end - pass : 32;
        if (rows <= 8) run_pass(std::integral_constant<int, 8>{}, pass, rows);
        else if (rows <= 16) run_pass(std::integral_constant<int, 16>{}, pass, rows);
        else run_pass(std::integral_constant<int, 32>{}, pass, rows);
    }
}

// Bytes of the LDS table of scales (and biases) for `rows` weight rows.
inline size_t table_bytes(const ProductArgs &a, int rows) {
    const bool block = a.mode != NVQ_AFFINE;  // one-byte scale codes, no biases
    const int64_t bytes = (int64_t)rows * table_stride((int)(a.k / a.group), block ? 1 : 2) * (block ? 1 : 2);
    return (size_t)((bytes + 15) & ~(int64_t)15);
}

// Groups of 32 weight rows per block: two, unless that leaves most compute units without a block.
inline int row_groups(const ProductArgs &a) {
    const int64_t blocks = ((a.n + 63) / 64) * ((a.m + 31) / 32) * a.batch;
    return blocks >= 192 ? 2 : 1;
}

template <typename T, int BITS, int FP4, int RG, bool EXACT = false>
int32_t run_variant(const ProductArgs &a, hipStream_t s) {
    using G = Geometry<BITS, RG>;
    static std::atomic<bool> configured = false;
    auto kernel = qmf_kernel<T, BITS, FP4, RG, EXACT>;
    if (!configured) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
        configured = true;
    }
    const size_t lds_bytes = G::kFixedLdsBytes + table_bytes(a, G::kRows);
    if (lds_bytes > (size_t)kLdsLimit) return fail(NVQ_UNSUPPORTED, "quantized_matmul: K = %lld needs a %zu-byte LDS table", (long long)a.k, lds_bytes);
    const unsigned gx = (unsigned)((a.n + G::kRows - 1) / G::kRows);
    const dim3 grid(gx, (unsigned)((a.m + 31) / 32), (unsigned)a.batch);
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds_bytes, s, a);
    NVQ_LAUNCH_CHECK("qmf");
    return NVQ_OK;
}

template <typename T, int BITS, int FP4>
int32_t run_width(const ProductArgs &a, hipStream_t s) {
    if constexpr (FP4 == kAffine)
        if (a.exact_weights) return run_variant<T, BITS, FP4, 1, true>(a, s);  // (rows of few outputs: 32 weight rows per block)
    return row_groups(a) == 2 ? run_variant<T, BITS, FP4, 2>(a, s) : run_variant<T, BITS, FP4, 1>(a, s);
}

template <int BITS, int FP4>
int32_t run_dtype(const ProductArgs &a, hipStream_t s) {
    return a.dtype == NVQ_BF16 ? run_width<bf16_t, BITS, FP4>(a, s) : run_width<f16_t, BITS, FP4>(a, s);
}

// LDS bytes of the variant `launch_qmf` would pick (for `qmf_supported`).
template <int BITS>
inline size_t lds_needed(const ProductArgs &a) {
    return row_groups(a) == 2 && !a.exact_weights ? Geometry<BITS, 2>::kFixedLdsBytes + table_bytes(a, 64) : Geometry<BITS, 1>::kFixedLdsBytes + table_bytes(a, 32);
}

}  // namespace qmf

// One per code width, each in its own translation unit.
int32_t launch_qmf_fp8(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_nvfp4(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b2(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b1(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b3(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b5(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b4(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b6(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_b8(const ProductArgs &a, hipStream_t s);
int32_t launch_qmf_fp4(const ProductArgs &a, hipStream_t s);

}  // namespace nvq
