// Tiled quantized products y[M,N] = x[M,K] . dequantize(w[N,K])^T on the gfx950 matrix cores: the
// prefill-shaped path.  Values follow nuvec's CPU product (reference:
// crates/nuvec-core/src/kernels.rs:1091-1142) within the stated tolerance; as in the reference's
// device kernels the weight tile is dequantized into on-chip memory in the element type and the
// products accumulate in float32 (crates/nuvec-kernels/src/metal/quantized.h:583-817, 1358-1485).
//
// One block of 512 threads (eight wavefronts, 2 x 4, each 128 x 64 of y) owns a BM x BN = 256 x 256 tile
// and walks K in steps of BK = 64.  Per step and block:
//   * x tile   256 x 64 elements (32 KB): copied global -> registers -> LDS, 16 bytes per access;
//   * w tile   256 rows x 32 packed bytes: thread t owns half a row (32 codes, inside one quantization
//              group): codes -> float (v_cvt_f32_ubyte) -> fma(code, scale, bias) -> packed element type
//              -> 64 B of LDS;
//   * 32 MFMA 32x32x16 per wavefront (4 x 2 accumulator tiles of 32 x 32, 128 accumulator registers).
// LDS rows are 128 B (64 elements) with the 16-byte chunk index XOR-ed with (row & 7), which makes the
// 16-byte fragment reads of the matrix instruction and the tile writes bank-conflict free.
//
// Overlap.  Each SIMD holds two wavefronts of the block.  LDS tiles are double-buffered and there is
// one barrier per step; inside a step wavefronts 0-3 first dequantize step s+1 into the other buffer
// and then run the matrix instructions of step s, while wavefronts 4-7 do the two phases in the
// opposite order.  So on every SIMD one wavefront issues matrix instructions while the other issues
// the conversion arithmetic, and the two pipes work at the same time.
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

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 512;
constexpr int kRowBytes = BK * 2;                       // 128 B per LDS row
constexpr int kTileBytes = (BM + BN) * kRowBytes;       // one stage: x tile then w tile
constexpr int kLdsBytes = 2 * kTileBytes;               // 128 KB

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    __device__ static __forceinline__ floatx16_t mfma(uint4 a, uint4 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) {  // round to nearest even
        const floatx2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2v_t));
    }
};
template <> struct Mma<f16_t> {
    __device__ static __forceinline__ floatx16_t mfma(uint4 a, uint4 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
        const floatx2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2v_t));
    }
};

// Byte offset of 16-byte chunk `chunk` (0..7) of LDS row `row`.
__device__ __forceinline__ int lds_offset(int row, int chunk) { return row * kRowBytes + ((chunk ^ (row & 7)) << 4); }

// Eight 4-bit codes of `word` (value i in bits 4i..4i+3) as fma(code, s, b), packed to the element
// type in stream order.
template <typename T>
__device__ __forceinline__ uint4 dequant8(uint32_t word, float s, float b) {
    const uint32_t even = word & 0x0F0F0F0Fu, odd = (word >> 4) & 0x0F0F0F0Fu;  // codes 0,2,4,6 and 1,3,5,7
    float e[4], o[4];
    e[0] = (float)(even & 0xFFu); e[1] = (float)((even >> 8) & 0xFFu); e[2] = (float)((even >> 16) & 0xFFu); e[3] = (float)(even >> 24);
    o[0] = (float)(odd & 0xFFu);  o[1] = (float)((odd >> 8) & 0xFFu);  o[2] = (float)((odd >> 16) & 0xFFu);  o[3] = (float)(odd >> 24);
    uint4 r;
    r.x = Mma<T>::pack(__builtin_fmaf(e[0], s, b), __builtin_fmaf(o[0], s, b));
    r.y = Mma<T>::pack(__builtin_fmaf(e[1], s, b), __builtin_fmaf(o[1], s, b));
    r.z = Mma<T>::pack(__builtin_fmaf(e[2], s, b), __builtin_fmaf(o[2], s, b));
    r.w = Mma<T>::pack(__builtin_fmaf(e[3], s, b), __builtin_fmaf(o[3], s, b));
    return r;
}

template <typename T, bool BATCHED>
__global__ void __launch_bounds__(kThreads) qmm4_kernel(const ProductArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave >> 2) & 1, wn = wave & 3;  // wavefront grid 2 x 4: 128 x 64 each
    const bool convert_first = wave < 4;            // the two wavefronts of a SIMD run the phases in opposite order
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = a.group == 32 ? 5 : a.group == 64 ? 6 : 7;
    const int kwords = K >> 3, kgroups = K >> gshift;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    int64_t bx = 0, bw = 0, bs = 0, by = 0;
    if constexpr (BATCHED) {  // a batch with one stride per operand
        bx = (int64_t)blockIdx.z * a.x_strides[0];
        bw = (int64_t)blockIdx.z * a.w_strides[0];
        bs = (int64_t)blockIdx.z * a.s_strides[0];
        by = (int64_t)blockIdx.z * M * N;
    }
    const T *x = (const T *)a.x + bx;
    const uint32_t *w = (const uint32_t *)a.w + bw;
    const T *scales = (const T *)a.scales + bs, *biases = (const T *)a.biases + bs;
    T *y = (T *)a.y + by;

    // Global-load assignment.  x: 8 chunks of 16 B per row; thread t copies chunk t%8 of rows t/8 + 64 i.
    const int xc = tid & 7, xr = tid >> 3;
    const T *xrow[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = m0 + xr + 64 * i;
        xrow[i] = x + (int64_t)(row < M ? row : M - 1) * K + xc * 8;  // tail rows are computed, not stored
    }
    // w: thread t owns half h = t%2 (32 codes = 16 packed bytes) of tile row t/2.
    const int wr = tid >> 1, wh = tid & 1;
    const int wrow = n0 + wr < N ? n0 + wr : N - 1;
    const uint32_t *wp = w + (int64_t)wrow * kwords;
    const T *sp = scales + (int64_t)wrow * kgroups, *bp = biases + (int64_t)wrow * kgroups;

    floatx16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    uint4 xg[4], wg;
    float sc, bi;
    auto load_step = [&](int k0) {
        const bool xlive = k0 + xc * 8 < K;  // K is a multiple of 32: a chunk of 8 is whole or absent
#pragma unroll
        for (int i = 0; i < 4; i++) xg[i] = xlive ? *reinterpret_cast<const uint4 *>(xrow[i] + k0) : make_uint4(0, 0, 0, 0);
        const int kh = k0 + 32 * wh < K ? k0 + 32 * wh : K - 32;  // an absent half reads valid data; its x is zero
        wg = *reinterpret_cast<const uint4 *>(wp + (kh >> 3));
        sc = Elem<T>::load(sp, kh >> gshift);
        bi = Elem<T>::load(bp, kh >> gshift);
    };
    auto store_step = [&](int stage) {
        unsigned char *xs = lds + stage * kTileBytes, *ws = xs + BM * kRowBytes;
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<uint4 *>(xs + lds_offset(xr + 64 * i, xc)) = xg[i];
        const uint32_t d[4] = {wg.x, wg.y, wg.z, wg.w};
#pragma unroll
        for (int j = 0; j < 4; j++) *reinterpret_cast<uint4 *>(ws + lds_offset(wr, 4 * wh + j)) = dequant8<T>(d[j], sc, bi);
    };
    auto mma_step = [&](int stage) {
        const unsigned char *xs = lds + stage * kTileBytes, *ws = xs + BM * kRowBytes;
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
            uint4 af[4], bf[2];
            const int chunk = 2 * kk + (lane >> 5);
#pragma unroll
            for (int i = 0; i < 4; i++) af[i] = *reinterpret_cast<const uint4 *>(xs + lds_offset(wm * 128 + i * 32 + (lane & 31), chunk));
#pragma unroll
            for (int j = 0; j < 2; j++) bf[j] = *reinterpret_cast<const uint4 *>(ws + lds_offset(wn * 64 + j * 32 + (lane & 31), chunk));
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = Mma<T>::mfma(af[i], bf[j], acc[i][j]);
        }
    };

    const int steps = (K + BK - 1) / BK;
    load_step(0);
    store_step(0);
    if (steps > 1) load_step(BK);  // the registers now hold step 1
    __syncthreads();
    // Two half-steps per step, a barrier after the second.  In step s every wavefront converts step
    // s+1 into the other LDS stage and multiplies step s, in the order its group prescribes; one copy
    // of each phase's code serves both groups.
    for (int half = 0; half < 2 * steps; half++) {
        const int step = half >> 1, stage = step & 1;
        const bool convert = ((half & 1) == 0) == convert_first;
        if (convert) {
            if (step + 1 < steps) store_step(stage ^ 1);
            if (step + 2 < steps) load_step((step + 2) * BK);
        } else {
            mma_step(stage);
        }
        if (half & 1) __syncthreads();
    }

    // Epilogue: accumulator element e of a 32 x 32 tile is row 8 (e / 4) + 4 (lane / 32) + e % 4, column lane % 32.
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * 128 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (row < M && col < N) Elem<T>::store(y, (int64_t)row * N + col, acc[i][j][e]);
            }
        }
}

template <typename T>
int32_t run_qmm4(const ProductArgs &a, hipStream_t s) {
    static bool configured[2] = {false, false};
    const bool batched = a.batch > 1;
    auto kernel = batched ? qmm4_kernel<T, true> : qmm4_kernel<T, false>;
    if (!configured[batched]) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
        configured[batched] = true;
    }
    dim3 grid((unsigned)((a.n + BN - 1) / BN), (unsigned)((a.m + BM - 1) / BM), (unsigned)a.batch);
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), kLdsBytes, s, a);
    NVQ_LAUNCH_CHECK("qmm4");
    return NVQ_OK;
}

}  // namespace

// Whether the tiled kernel takes this product: affine 4-bit, bf16 or f16, and a batch that is a
// single stride per operand (or no batch).
bool qmm_supported(const ProductArgs &a) {
    if (a.mode != NVQ_AFFINE || a.bits != 4 || (a.dtype != NVQ_BF16 && a.dtype != NVQ_F16)) return false;
    if (a.rhs != nullptr) return false;
    if (a.batch > 1 && a.batch_ndim != 1) return false;
    return a.batch <= 65535 && a.k >= 32;
}

int32_t launch_qmm(const ProductArgs &a, hipStream_t s) {
    return a.dtype == NVQ_BF16 ? run_qmm4<bf16_t>(a, s) : run_qmm4<f16_t>(a, s);
}

}  // namespace nvq
