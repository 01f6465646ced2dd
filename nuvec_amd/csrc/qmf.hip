// Few-row quantized products on the gfx950 matrix cores: y[m, n] = x[m, :] . dequantize(w[n, :]) for up to
// 32 rows of x per pass, and the grouped (sorted) gathered product of mixture-of-experts layers, where
// each expert's rows are such a product against that expert's weights.  Values follow nuvec's CPU product
// (reference: crates/nuvec-core/src/kernels.rs:1091-1142, crates/nuvec-core/src/quantized.rs:679-719) within
// the stated tolerance; the grouped route is the counterpart of the reference's `gather_qmm_rhs`
// (crates/nuvec-kernels/src/metal/quantized.h:3301-3449, schedule at 2866-2906).
//
// The weights are the large operand and each weight is decoded exactly once per pass.  The kernel is bound
// by the memory instructions it issues, not by arithmetic, so everything is arranged to issue few, wide,
// coalesced ones:
//   * a block of eight wavefronts owns 64 weight rows and splits K into contiguous ranges, one per wavefront.
//     A wavefront takes its range in windows of two steps (128 values = 64 bytes of every row): four loads,
//     each 16 rows x 64 contiguous bytes, fetch a window into registers three windows ahead; the window then
//     goes through a private 4 KB piece of LDS (16-byte slots XOR-swizzled by row) to reach the matrix
//     operand layout, in which a lane (row n = lane % 32, half h = lane / 32) holds the 32 codes of its half
//     of a step for either group of 32 rows;
//   * the scales and biases of the block's 64 rows are one contiguous piece of memory: it is copied once,
//     coalesced, into an LDS table laid out [group][row], and read from there;
//   * the pieces of x are shared by both row groups, and a pass of at most 8 (16) rows of x packs four
//     (two) of a step's pieces into one load: lane (row r = l % XR, slot q = l / XR) of a half loads the
//     pieces q NL .. q NL + NL - 1 (NL = XR / 8), the matrix instruction of piece kk takes that register with the
//     lanes of other slots cleared, so row r + XR q of the accumulator holds the share of piece kk and the
//     shares are added when the tile is written.
// Codes are expanded into matrix operands in registers (affine: v_cvt_f32_ubyte + fma + packed convert;
// MXFP4: one scaled FP4 -> element-type conversion per two codes).  The K order inside a step is permuted
// consistently for both operands (piece kk of half h is packed word 4 h + kk).  The wavefronts' partial tiles
// are summed through LDS in a fixed order, so results do not depend on scheduling.
#include "nvq_device.h"
#include "nvq_internal.h"

#include <type_traits>
#include <utility>

namespace nvq {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2v_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kRowGroups = 2;             // groups of 32 weight rows per block
constexpr int kRows = 32 * kRowGroups;    // weight rows per block = columns of y
constexpr int kWaves = 8;                 // wavefronts per block, each with its own range of K
constexpr int kThreads = 64 * kWaves;
constexpr int kDepth = 4;                 // windows (of two steps) of weights in flight per lane
constexpr int kPartialBytes = 4 * kRowGroups * 16 * 64 * 4;  // four wavefronts' tiles
constexpr int kStageBytes = kRows * 64;   // one window of one wavefront
constexpr int kFixedLdsBytes = kPartialBytes + kWaves * kStageBytes;
constexpr int kTableMaxBytes = 64 * 1024; // scales + biases of the block's rows; larger tables are not staged

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant in the body
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

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
// `pairs`), taken in passes of up to 32.  Otherwise blockIdx.z is a batch with one stride per operand and
// blockIdx.y a pass of 32 rows.  TABLE: scales and biases go through the LDS table.
template <typename T, bool FP4, bool GROUPED, bool TABLE>
__global__ void __launch_bounds__(kThreads) qmf_kernel(const ProductArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    float *partial = reinterpret_cast<float *>(lds);  // [4][kRowGroups][values][64]
    using S = std::conditional_t<FP4, uint8_t, T>;    // stored scale type
    S *table_s = reinterpret_cast<S *>(lds + kFixedLdsBytes);  // [group][64 rows]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, l32 = lane & 31;
    const int K = (int)a.k, N = (int)a.n;
    const int gshift = FP4 ? 5 : (a.group == 32 ? 5 : a.group == 64 ? 6 : 7);
    const int kwords = K >> 3, kgroups = K >> gshift;
    S *table_b = table_s + kRows * kgroups;
    const int n0 = blockIdx.x * kRows;

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
    T *y = (T *)a.y + yo;
    const S *srow[kRowGroups], *brow[kRowGroups];  // used when the table is not staged
#pragma unroll
    for (int rg = 0; rg < kRowGroups; rg++) {
        const int n = n0 + 32 * rg + l32 < N ? n0 + 32 * rg + l32 : N - 1;  // tail rows are computed, not stored
        srow[rg] = (const S *)a.scales + so + (int64_t)n * kgroups;
        brow[rg] = (const S *)a.biases + so + (int64_t)n * kgroups;
    }

    const int steps = K >> 6;  // K is a multiple of 64 (checked on the host)
    const int s_begin = steps * wave / kWaves, s_end = steps * (wave + 1) / kWaves;

    // Window loads: piece j of this lane is 16 bytes of row 16 j + lane / 4, chunk c = lane % 4 of the window's
    // 64 bytes (chunk 2 t + h' = half h' of step t).
    const int lrow = lane >> 2, chunk = lane & 3;
    const uint32_t *wload[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int n = n0 + 16 * j + lrow < N ? n0 + 16 * j + lrow : N - 1;
        wload[j] = (const uint32_t *)a.w + wo + (int64_t)n * kwords + 4 * chunk;
    }
    auto load_window = [&](int step, u32x4_t (&w)[4]) {
        // the second step of a window may lie past the range: its lanes fetch the first step again
        const int word = (chunk >= 2 && step + 1 >= s_end) ? step * 8 - 8 : step * 8;
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = *reinterpret_cast<const u32x4_t *>(wload[j] + word);
    };
    // The wavefront's piece of LDS holds [64 rows][4 slots of 16 bytes]; chunk c of row n sits in slot
    // c ^ ((n / 4) % 4), which spreads both the stores and the operand loads over all banks.
    unsigned char *stage = lds + kPartialBytes + wave * kStageBytes;
    u32x4_t *stage_store = reinterpret_cast<u32x4_t *>(stage + lrow * 64 + 16 * (chunk ^ ((lrow >> 2) & 3)));
    const u32x4_t *stage_load[2];  // step t of the window, row group 0
#pragma unroll
    for (int t = 0; t < 2; t++) stage_load[t] = reinterpret_cast<const u32x4_t *>(stage + l32 * 64 + 16 * ((2 * t + h) ^ ((l32 >> 2) & 3)));

    auto load_scales = [&](int step, float (&scale)[kRowGroups], float (&bias)[kRowGroups]) {
        const int g = (step * 64 + 32 * h) >> gshift;
#pragma unroll
        for (int rg = 0; rg < kRowGroups; rg++) {
            const S *sp = TABLE ? table_s + g * kRows + 32 * rg + l32 : srow[rg] + g;
            const S *bp = TABLE ? table_b + g * kRows + 32 * rg + l32 : brow[rg] + g;
            if constexpr (FP4) {
                scale[rg] = ftz(e8m0_to_f32(*sp));
                bias[rg] = 0.0f;
            } else {
                scale[rg] = Elem<T>::load(sp, 0);
                bias[rg] = Elem<T>::load(bp, 0);
            }
        }
    };

    if constexpr (TABLE) {
        // The scales (and biases) of rows n0 .. n0 + 63 are contiguous: copy them in aligned 16-byte pieces
        // and scatter the elements to [group][row].  Bytes of a piece outside the rows are dropped.
        constexpr int kPer = 16 / (int)sizeof(S);
        const int valid_rows = N - n0 < kRows ? N - n0 : kRows;
        const int count = valid_rows * kgroups;
        const int tensors = FP4 ? 1 : 2;
        for (int t = 0; t < tensors; t++) {
            const S *src = (t == 0 ? (const S *)a.scales : (const S *)a.biases) + so + (int64_t)n0 * kgroups;
            S *dst = t == 0 ? table_s : table_b;
            const int skew = (int)((uintptr_t)src & 15) / (int)sizeof(S);  // elements before src in its first piece
            const uint4 *pieces = reinterpret_cast<const uint4 *>(src - skew);
            const int n_pieces = (skew + count + kPer - 1) / kPer;
            for (int p = tid; p < n_pieces; p += kThreads) {
                const uint4 v = pieces[p];
                S elems[kPer];
                __builtin_memcpy(elems, &v, 16);
                int idx = p * kPer - skew;  // element index of elems[0] within the block's rows
                int row = idx >= 0 ? idx / kgroups : 0, g = idx >= 0 ? idx - row * kgroups : 0;
#pragma unroll
                for (int e = 0; e < kPer; e++, idx++) {
                    if (idx >= 0 && idx < count) {
                        dst[g * kRows + row] = elems[e];
                        if (++g == kgroups) g = 0, row++;
                    }
                }
            }
        }
    }

    // One pass over at most XR rows of x (XR = 8, 16 or 32).
    auto run_pass = [&](auto xr_tag, int pass, int rows) {
        constexpr int XR = decltype(xr_tag)::value;
        constexpr int NL = XR / 8;        // loads of x per step
        constexpr int XD = 32 / XR;         // windows of x in flight per lane (kDepth is a multiple of it)
        constexpr int NV = XR / 2;        // values of the tile per lane and row group once the slots are added
        const int r = l32 % XR, slot = l32 / XR;
        const bool live = r < rows;  // this lane's row of x exists
        // x row of this lane; in the grouped route rows are gathered through lhs (arange for sorted gathers)
        int64_t xr = pass + (live ? r : 0);
        if constexpr (GROUPED) xr = a.lhs != nullptr ? (int64_t)a.lhs[xr] : xr;
        const T *xrow = x + xr * K + 32 * h + 8 * NL * slot;  // piece kk of half h covers k0 + 8 (4 h + kk) .. + 8

        floatx16_t acc[kRowGroups];
#pragma unroll
        for (int rg = 0; rg < kRowGroups; rg++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[rg][e] = 0.0f;

        u32x4_t ring[kDepth][4] = {};  // windows in flight: piece j belongs to row 16 j + lane / 4
        uint4 xring[XD][2][NL] = {};  // x pieces, XD windows ahead (they come from the cache)
        auto load_x = [&](int step, uint4 (&xf)[2][NL]) {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int sc = step + t < s_end ? step + t : step;
#pragma unroll
                for (int j = 0; j < NL; j++)
                    xf[t][j] = live ? *reinterpret_cast<const uint4 *>(xrow + sc * 64 + 8 * j) : make_uint4(0, 0, 0, 0);
            }
        };
        static_for<kDepth>([&](auto d_tag) {
            constexpr int d = decltype(d_tag)::value;
            if (s_begin + 2 * d < s_end) {
                load_window(s_begin + 2 * d, ring[d]);
                if constexpr (d < XD) load_x(s_begin + 2 * d, xring[d]);
            }
        });
        if constexpr (TABLE) __syncthreads();  // first pass: the table is written; later passes: nothing pending

        for (int s0 = s_begin; s0 < s_end; s0 += 2 * kDepth) {
            static_for<kDepth>([&](auto d_tag) {
                constexpr int d = decltype(d_tag)::value;
                const int step = s0 + 2 * d;
                if (step < s_end) {
                    // through LDS into the operand layout; the wavefront's LDS accesses execute in order
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int j = 0; j < 4; j++) stage_store[j * 64] = ring[d][j];
                    __builtin_amdgcn_wave_barrier();
                    asm volatile("" ::: "memory");
                    u32x4_t codes[2][kRowGroups];
#pragma unroll
                    for (int t = 0; t < 2; t++)
#pragma unroll
                        for (int rg = 0; rg < kRowGroups; rg++) codes[t][rg] = stage_load[t][rg * 128];
                    asm volatile("" ::: "memory");
                    uint4 xf[2][NL];
#pragma unroll
                    for (int t = 0; t < 2; t++)
#pragma unroll
                        for (int j = 0; j < NL; j++) xf[t][j] = xring[d % XD][t][j];
                    if (step + 2 * kDepth < s_end) load_window(step + 2 * kDepth, ring[d]);
                    if (step + 2 * XD < s_end) load_x(step + 2 * XD, xring[d % XD]);
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        if (step + t < s_end) {
                            float scale[kRowGroups], bias[kRowGroups];
                            load_scales(step + t, scale, bias);
#pragma unroll
                            for (int kk = 0; kk < 4; kk++) {
                                uint4 xa = xf[t][kk % NL];
                                if constexpr (XR < 32) {
                                    const bool mine = slot == kk / NL;
                                    xa.x = mine ? xa.x : 0u, xa.y = mine ? xa.y : 0u, xa.z = mine ? xa.z : 0u, xa.w = mine ? xa.w : 0u;
                                }
#pragma unroll
                                for (int rg = 0; rg < kRowGroups; rg++) {
                                    const u32x4_t cw = codes[t][rg];
                                    const uint32_t word = kk == 0 ? cw.x : kk == 1 ? cw.y : kk == 2 ? cw.z : cw.w;
                                    acc[rg] = Ops<T>::mfma(xa, expand8<T, FP4>(word, scale[rg], bias[rg]), acc[rg]);
                                }
                            }
                        }
                    }
                }
            });
        }

        // Accumulator element e of lane l is tile row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32; tile rows
        // r, r + XR, ... are the slots' shares of row r of x.
        float vals[kRowGroups][NV];
#pragma unroll
        for (int rg = 0; rg < kRowGroups; rg++)
#pragma unroll
            for (int v = 0; v < NV; v++) {
                float sum = acc[rg][v];
#pragma unroll
                for (int q = 1; q < 32 / XR; q++) sum += acc[rg][v + NV * q];
                vals[rg][v] = sum;
            }
        // Sum the wavefronts' partial tiles in a fixed order: the upper four hand theirs to the lower four,
        // whose tiles are then added in wavefront order.
        auto slot_of = [&](int w, int rg, int v) -> float * { return partial + ((w * kRowGroups + rg) * NV + v) * 64; };
        if (wave >= 4) {
#pragma unroll
            for (int rg = 0; rg < kRowGroups; rg++)
#pragma unroll
                for (int v = 0; v < NV; v++) slot_of(wave - 4, rg, v)[lane] = vals[rg][v];
        }
        __syncthreads();
        if (wave < 4) {
#pragma unroll
            for (int rg = 0; rg < kRowGroups; rg++)
#pragma unroll
                for (int v = 0; v < NV; v++) vals[rg][v] += slot_of(wave, rg, v)[lane];
        }
        __syncthreads();
        if (wave < 4) {
#pragma unroll
            for (int rg = 0; rg < kRowGroups; rg++)
#pragma unroll
                for (int v = 0; v < NV; v++) slot_of(wave, rg, v)[lane] = vals[rg][v];
        }
        __syncthreads();
        for (int idx = tid; idx < kRowGroups * NV * 64; idx += kThreads) {
            const int l = idx & 63, v = (idx >> 6) % NV, rg = idx / (64 * NV);
            const float sum = ((slot_of(0, rg, v)[l] + slot_of(1, rg, v)[l]) + slot_of(2, rg, v)[l]) + slot_of(3, rg, v)[l];
            const int m = 8 * (v >> 2) + 4 * (l >> 5) + (v & 3), col = n0 + 32 * rg + (l & 31);
            if (m < rows && col < N) Elem<T>::store(y, (int64_t)(pass + m) * N + col, sum);
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

// Bytes of the LDS table for this product, or 0 when it is not staged (too large).
size_t table_bytes(const ProductArgs &a) {
    const int64_t group = a.mode == NVQ_MXFP4 ? 32 : a.group;
    const int64_t bytes = a.mode == NVQ_MXFP4 ? kRows * (a.k / group) : 2 * kRows * (a.k / group) * 2;
    return bytes <= kTableMaxBytes ? (size_t)((bytes + 15) & ~(int64_t)15) : 0;
}

template <typename T, bool FP4, bool GROUPED, bool TABLE>
int32_t run_qmf_variant(const ProductArgs &a, size_t lds_bytes, hipStream_t s) {
    static bool configured = false;
    auto kernel = qmf_kernel<T, FP4, GROUPED, TABLE>;
    if (!configured) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        kFixedLdsBytes + kTableMaxBytes));
        configured = true;
    }
    const unsigned gx = (unsigned)((a.n + kRows - 1) / kRows);
    const dim3 grid = GROUPED ? dim3(gx, 1, (unsigned)a.experts) : dim3(gx, (unsigned)((a.m + 31) / 32), (unsigned)a.batch);
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds_bytes, s, a);
    NVQ_LAUNCH_CHECK("qmf");
    return NVQ_OK;
}

template <typename T, bool FP4>
int32_t run_qmf(const ProductArgs &a, hipStream_t s) {
    const size_t table = table_bytes(a);
    const size_t lds_bytes = kFixedLdsBytes + table;
    if (a.offsets != nullptr)
        return table ? run_qmf_variant<T, FP4, true, true>(a, lds_bytes, s) : run_qmf_variant<T, FP4, true, false>(a, lds_bytes, s);
    return table ? run_qmf_variant<T, FP4, false, true>(a, lds_bytes, s) : run_qmf_variant<T, FP4, false, false>(a, lds_bytes, s);
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
