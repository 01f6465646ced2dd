// Few-row quantized products on the gfx950 matrix cores: y[m, n] = x[m, :] . dequantize(w[n, :]) for up to
// 32 rows of x per pass, and the grouped (sorted) gathered product of mixture-of-experts layers, where
// each expert's rows are such a product against that expert's weights.  Values follow nuvec's CPU product
// (reference: crates/nuvec-core/src/kernels.rs:1091-1142, crates/nuvec-core/src/quantized.rs:679-719) within
// the stated tolerance; the grouped route is the counterpart of the reference's `gather_qmm_rhs`
// (crates/nuvec-kernels/src/metal/quantized.h:3301-3449, schedule at 2866-2906).
//
// The weights are the large operand and each weight is decoded exactly once, whatever the number of rows:
// a block of four wavefronts owns 32 weight rows and splits K into four contiguous ranges, one per
// wavefront.  Per step of 64 values a lane (row n = lane % 32, half h = lane / 32) loads the 16 bytes of
// packed codes of its half-group straight into registers (four steps ahead, to keep HBM busy), expands them
// into four matrix operands (affine: v_cvt_f32_ubyte + fma + packed convert; MXFP4: one scaled
// FP4 -> element-type conversion per two codes) and issues four 32x32x16 matrix instructions against the
// matching 16-byte pieces of x.  The K order inside a step is permuted consistently for both operands
// (operand kk of half h is packed word 4 h + kk).  The four partial 32 x 32 tiles are summed through LDS in
// a fixed order, so results do not depend on scheduling.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2v_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));

constexpr int kWaves = 4, kThreads = kWaves * 64;
constexpr int kRows = 32;   // weight rows per block = columns of y
constexpr int kDepth = 4;   // steps of weights in flight per lane
constexpr int kXDepth = 2;  // steps of x in flight per lane (kDepth is a multiple of it)

template <int B>
__device__ __forceinline__ float ubyte_to_float(uint32_t v) {
    float f;
    if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
    return f;
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
};

// What a lane holds of one step: its 32 codes and the float scale (and bias) of their group.
struct StepData {
    uint4 codes;
    float scale, bias;
};

// Eight codes of one packed word as one matrix operand (8 elements, stream order).
template <typename T, bool FP4>
__device__ __forceinline__ uint4 expand8(uint32_t word, float s, float b) {
    uint4 r;
    if constexpr (FP4) {
        r.x = Ops<T>::template fp4_pair<0>(word, s);
        r.y = Ops<T>::template fp4_pair<1>(word, s);
        r.z = Ops<T>::template fp4_pair<2>(word, s);
        r.w = Ops<T>::template fp4_pair<3>(word, s);
    } else {
        const uint32_t even = word & 0x0F0F0F0Fu, odd = (word >> 4) & 0x0F0F0F0Fu;
        r.x = Ops<T>::pack(__builtin_fmaf(ubyte_to_float<0>(even), s, b), __builtin_fmaf(ubyte_to_float<0>(odd), s, b));
        r.y = Ops<T>::pack(__builtin_fmaf(ubyte_to_float<1>(even), s, b), __builtin_fmaf(ubyte_to_float<1>(odd), s, b));
        r.z = Ops<T>::pack(__builtin_fmaf(ubyte_to_float<2>(even), s, b), __builtin_fmaf(ubyte_to_float<2>(odd), s, b));
        r.w = Ops<T>::pack(__builtin_fmaf(ubyte_to_float<3>(even), s, b), __builtin_fmaf(ubyte_to_float<3>(odd), s, b));
    }
    return r;
}

// GROUPED: blockIdx.z is an expert; its rows of x / y are [offsets[z], offsets[z+1]) (the last expert ends at
// `pairs`), taken in passes of 32.  Otherwise blockIdx.z is a batch with one stride per operand and
// blockIdx.y a pass of 32 rows.
template <typename T, bool FP4, bool GROUPED>
__global__ void __launch_bounds__(kThreads) qmf_kernel(const ProductArgs a) {
    __shared__ float partial[kWaves][16][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, l32 = lane & 31;
    const int K = (int)a.k, N = (int)a.n;
    const int gshift = FP4 ? 5 : (a.group == 32 ? 5 : a.group == 64 ? 6 : 7);
    const int kwords = K >> 3, kgroups = K >> gshift;
    const int n0 = blockIdx.x * kRows;
    const int n = n0 + l32 < N ? n0 + l32 : N - 1;  // tail rows are computed, not stored

    int row_begin, row_end;  // rows of x (and of y) this block multiplies
    int64_t xo = 0, wo = 0, so = 0, yo = 0;
    if constexpr (GROUPED) {
        const int e = blockIdx.z;
        row_begin = a.offsets[e];
        row_end = e + 1 < (int)a.experts ? a.offsets[e + 1] : (int)a.batch;
        if (row_begin >= row_end) return;  // the whole block: no barrier has been reached
        wo = (int64_t)e * N * kwords;
        so = (int64_t)e * N * kgroups;
    } else {
        row_begin = blockIdx.y * 32;
        row_end = row_begin + 32 < (int)a.m ? row_begin + 32 : (int)a.m;
        if (a.batch_ndim > 0) {
            xo = (int64_t)blockIdx.z * a.x_strides[0];
            wo = (int64_t)blockIdx.z * a.w_strides[0];
            so = (int64_t)blockIdx.z * a.s_strides[0];
            yo = (int64_t)blockIdx.z * a.m * N;
        }
    }
    const T *x = (const T *)a.x + xo;
    const uint32_t *wrow = (const uint32_t *)a.w + wo + (int64_t)n * kwords + 4 * h;
    const uint8_t *s8 = (const uint8_t *)a.scales + so + (int64_t)n * kgroups;
    const T *sT = (const T *)a.scales + so + (int64_t)n * kgroups, *bT = (const T *)a.biases + so + (int64_t)n * kgroups;
    T *y = (T *)a.y + yo;

    const int steps = K >> 6;  // K is a multiple of 64 (checked on the host)
    const int s_begin = steps * wave / kWaves, s_end = steps * (wave + 1) / kWaves;

    auto load_step = [&](int step) -> StepData {
        StepData d;
        const int sc = step < s_end ? step : s_end - 1;  // past the range: a harmless reload
        d.codes = *reinterpret_cast<const uint4 *>(wrow + sc * 8);
        const int g = (sc * 64 + 32 * h) >> gshift;
        if constexpr (FP4) {
            d.scale = ftz(e8m0_to_f32(s8[g]));
            d.bias = 0.0f;
        } else {
            d.scale = Elem<T>::load(sT, g);
            d.bias = Elem<T>::load(bT, g);
        }
        return d;
    };

    for (int pass = row_begin; pass < row_end; pass += 32) {
        const int rows = row_end - pass < 32 ? row_end - pass : 32;
        const bool live = l32 < rows;  // this lane's row of x exists
        // x row of this lane; in the grouped route rows are gathered through lhs (arange for sorted gathers)
        int64_t xr = pass + (live ? l32 : 0);
        if constexpr (GROUPED) xr = a.lhs != nullptr ? (int64_t)a.lhs[xr] : xr;
        const T *xrow = x + xr * K + 32 * h;  // operand kk of half h covers k0 + 8 (4 h + kk) .. + 8

        floatx16_t acc;
#pragma unroll
        for (int e = 0; e < 16; e++) acc[e] = 0.0f;

        if (s_begin < s_end) {
            StepData ring[kDepth];
            uint4 xring[kXDepth][4];  // x pieces, kXDepth steps ahead (they come from the cache)
            auto load_x = [&](int step, uint4 (&xf)[4]) {
                const int sc = step < s_end ? step : s_end - 1;
#pragma unroll
                for (int kk = 0; kk < 4; kk++)
                    xf[kk] = live ? *reinterpret_cast<const uint4 *>(xrow + sc * 64 + 8 * kk) : make_uint4(0, 0, 0, 0);
            };
#pragma unroll
            for (int d = 0; d < kXDepth; d++) load_x(s_begin + d, xring[d]);
#pragma unroll
            for (int d = 0; d < kDepth; d++) ring[d] = load_step(s_begin + d);
            for (int s0 = s_begin; s0 < s_end; s0 += kDepth) {
#pragma unroll
                for (int d = 0; d < kDepth; d++) {
                    const int step = s0 + d;
                    const StepData cur = ring[d];
                    uint4 xf[4];
#pragma unroll
                    for (int kk = 0; kk < 4; kk++) xf[kk] = xring[d % kXDepth][kk];
                    ring[d] = load_step(step + kDepth);
                    load_x(step + kXDepth, xring[d % kXDepth]);
                    if (step < s_end) {
                        const uint32_t words[4] = {cur.codes.x, cur.codes.y, cur.codes.z, cur.codes.w};
#pragma unroll
                        for (int kk = 0; kk < 4; kk++) acc = Ops<T>::mfma(xf[kk], expand8<T, FP4>(words[kk], cur.scale, cur.bias), acc);
                    }
                }
            }
        }
        // Sum the four wavefronts' partial tiles in wavefront order.
#pragma unroll
        for (int e = 0; e < 16; e++) partial[wave][e][lane] = acc[e];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + i * kThreads, e = idx >> 6, l = idx & 63;
            const float v = ((partial[0][e][l] + partial[1][e][l]) + partial[2][e][l]) + partial[3][e][l];
            // accumulator element e of lane l is row 8 (e / 4) + 4 (l / 32) + e % 4 (a row of x), column l % 32
            const int m = 8 * (e >> 2) + 4 * (l >> 5) + (e & 3), col = n0 + (l & 31);
            if (m < rows && col < N) Elem<T>::store(y, (int64_t)(pass + m) * N + col, v);
        }
        __syncthreads();
    }
}

template <typename T, bool FP4>
int32_t run_qmf(const ProductArgs &a, hipStream_t s) {
    const unsigned gx = (unsigned)((a.n + kRows - 1) / kRows);
    if (a.offsets != nullptr) {
        hipLaunchKernelGGL((qmf_kernel<T, FP4, true>), dim3(gx, 1, (unsigned)a.experts), dim3(kThreads), 0, s, a);
    } else {
        hipLaunchKernelGGL((qmf_kernel<T, FP4, false>), dim3(gx, (unsigned)((a.m + 31) / 32), (unsigned)a.batch), dim3(kThreads), 0, s, a);
    }
    NVQ_LAUNCH_CHECK("qmf");
    return NVQ_OK;
}

}  // namespace

// Whether the few-row matrix-core kernel takes this product: 4-bit affine or MXFP4, bf16 or f16, whole
// steps of 64 values, and either no batch, a batch with one stride per operand, or the grouped gather.
bool qmf_supported(const ProductArgs &a) {
    if (!(a.mode == NVQ_MXFP4 || (a.mode == NVQ_AFFINE && a.bits == 4))) return false;
    if (a.dtype != NVQ_BF16 && a.dtype != NVQ_F16) return false;
    if (a.k < 64 || a.k % 64 != 0) return false;
    if (a.offsets != nullptr) return a.m == 1 && a.experts <= 65535;
    if (a.rhs != nullptr) return false;
    return (a.batch == 1 || a.batch_ndim == 1) && a.batch <= 65535 && (a.m + 31) / 32 <= 65535;
}

int32_t launch_qmf(const ProductArgs &a, hipStream_t s) {
    if (a.mode == NVQ_MXFP4) return a.dtype == NVQ_BF16 ? run_qmf<bf16_t, true>(a, s) : run_qmf<f16_t, true>(a, s);
    return a.dtype == NVQ_BF16 ? run_qmf<bf16_t, false>(a, s) : run_qmf<f16_t, false>(a, s);
}

}  // namespace nvq
