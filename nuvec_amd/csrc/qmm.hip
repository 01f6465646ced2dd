// Tiled quantized products y[M,N] = x[M,K] . dequantize(w[N,K])^T on the gfx950 matrix cores: the
// prefill-shaped path.  Values follow nuvec's CPU product (reference:
// crates/nuvec-core/src/kernels.rs:1091-1142) within the stated tolerance; as in the reference's
// device kernels the weights are dequantized on chip in the element type (one rounding of
// fma(code, scale, bias)) and the products accumulate in float32
// (crates/nuvec-kernels/src/metal/quantized.h:583-817, 1358-1485).
//
// One block of 512 threads (eight wavefronts, 2 x 4, each 128 x 64 of y) owns a BM x BN = 256 x 256 tile
// and walks K in steps of BK = 64 through a ring of three LDS stages.  A stage holds
//   * the x tile, 256 rows x 128 B, 16-byte chunk index XOR-ed with (row & 7) so that the 16-byte
//     fragment reads of the matrix instruction are bank-conflict free, and
//   * the w tile still packed, 256 rows x 32 B (a quarter of the bytes of a dequantized tile).
// Both arrive by direct global-to-LDS loads (no registers, no copy instructions); the loads of step
// s+2 are issued before the matrix work of step s, and there is one barrier per step.  Scales and
// biases are staged per 256 values of K (four steps) in a small double-buffered LDS table.
// A wavefront dequantizes its own weight fragments right before use: per step and lane two 16-byte
// LDS reads bring the 64 codes of its two columns; 8 codes -> float (v_cvt_f32_ubyte) ->
// fma(code, scale, bias) -> packed element type make one matrix operand.  With two wavefronts per
// SIMD the conversion arithmetic of one runs under the matrix instructions of the other.
// The K order inside a step is permuted (fragment kk of lane half h is packed word 4 h + kk) so that
// a lane's four weight words are one contiguous 16 bytes; x fragments follow the same order.
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
constexpr int kStages = 3;
constexpr int kRowBytes = BK * 2;                    // 128 B per x row in LDS
constexpr int kXBytes = BM * kRowBytes;              // 32 KB
constexpr int kWBytes = BN * (BK / 2);               // 8 KB of packed codes
constexpr int kStageBytes = kXBytes + kWBytes;       // 40 KB
constexpr int kPeriod = 256;                         // values of K per scale/bias table
constexpr int kSbBytes = (kPeriod / 32) * BN * 4;    // one table: up to 8 groups x 256 rows x (scale, bias)
constexpr int kLdsBytes = kStages * kStageBytes + 2 * kSbBytes;  // 136 KB

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    __device__ static __forceinline__ floatx16_t mfma(uint4 a, uint4 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) {  // round to nearest even
        const floatx2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2v_t));
    }
    __device__ static __forceinline__ float lo(uint32_t p) { return u2f(p << 16); }
    __device__ static __forceinline__ float hi(uint32_t p) { return u2f(p & 0xFFFF0000u); }
};
template <> struct Mma<f16_t> {
    __device__ static __forceinline__ floatx16_t mfma(uint4 a, uint4 b, floatx16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack(float lo, float hi) {
        const floatx2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2v_t));
    }
    __device__ static __forceinline__ float lo(uint32_t p) { return (float)__builtin_bit_cast(f16x2v_t, p)[0]; }
    __device__ static __forceinline__ float hi(uint32_t p) { return (float)__builtin_bit_cast(f16x2v_t, p)[1]; }
};

// Byte offset of 16-byte chunk `chunk` (0..7) of LDS row `row`.
__device__ __forceinline__ int lds_offset(int row, int chunk) { return row * kRowBytes + ((chunk ^ (row & 7)) << 4); }

// Byte `B` of `v` as float: one instruction (the compiler otherwise extracts the byte first).
template <int B>
__device__ __forceinline__ float ubyte_to_float(uint32_t v) {
    float f;
    if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
    else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
    return f;
}

// Eight 4-bit codes of `word` (value i in bits 4i..4i+3) as fma(code, s, b), packed to the element
// type in stream order.
template <typename T>
__device__ __forceinline__ uint4 dequant8(uint32_t word, float s, float b) {
    const uint32_t even = word & 0x0F0F0F0Fu, odd = (word >> 4) & 0x0F0F0F0Fu;  // codes 0,2,4,6 and 1,3,5,7
    uint4 r;
    r.x = Mma<T>::pack(__builtin_fmaf(ubyte_to_float<0>(even), s, b), __builtin_fmaf(ubyte_to_float<0>(odd), s, b));
    r.y = Mma<T>::pack(__builtin_fmaf(ubyte_to_float<1>(even), s, b), __builtin_fmaf(ubyte_to_float<1>(odd), s, b));
    r.z = Mma<T>::pack(__builtin_fmaf(ubyte_to_float<2>(even), s, b), __builtin_fmaf(ubyte_to_float<2>(odd), s, b));
    r.w = Mma<T>::pack(__builtin_fmaf(ubyte_to_float<3>(even), s, b), __builtin_fmaf(ubyte_to_float<3>(odd), s, b));
    return r;
}

// 16 bytes per lane from global memory straight into LDS: lane l of the wavefront writes
// lds_base + 16 l.  Issued as assembly so that the compiler keeps no account of it: the waits are
// placed by hand (dma_wait), which is what lets the loads of later steps stay in flight across
// the LDS reads of the current one.
__device__ __forceinline__ void dma16(const void *src, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_base), "v"(src) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait() {  // all but the N most recent vector-memory loads of this lane are complete
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <typename T, bool BATCHED>
__global__ void __launch_bounds__(kThreads) qmm4_kernel(const ProductArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    uint32_t *sb_table = reinterpret_cast<uint32_t *>(lds + kStages * kStageBytes);  // [2][group][row]: scale | bias << 16
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave >> 2) & 1, wn = wave & 3;  // wavefront grid 2 x 4: 128 x 64 each
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = a.group == 32 ? 5 : a.group == 64 ? 6 : 7;
    const int kwords = K >> 3, kgroups = K >> gshift;
    const int gper = kPeriod >> gshift;  // groups per table: 8, 4 or 2
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

    // Direct-to-LDS assignment.  x: instruction i of wavefront v fills the 64 consecutive 16-byte
    // slots starting at slot i*512 + v*64; slot S is row S/8, position S%8, and holds chunk
    // position ^ (row & 7) of that row.  w: slot v*64 + l is half l%2 of row (v*64 + l)/2.
    const T *xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int slot = i * 512 + wave * 64 + lane, row = slot >> 3, chunk = (slot & 7) ^ (row & 7);
        const int grow = m0 + row < M ? m0 + row : M - 1;  // tail rows are computed, not stored
        xsrc[i] = x + (int64_t)grow * K + chunk * 8;
    }
    const int wslot = wave * 64 + lane;
    const int wrow = n0 + (wslot >> 1) < N ? n0 + (wslot >> 1) : N - 1;
    const uint32_t *wsrc = w + (int64_t)wrow * kwords + (wslot & 1) * 4;
    const int steps = K / BK;  // K is a multiple of 64 (checked on the host)
    // Load `part` (0..3: x, 4: w) of `step`; five parts per step and lane.
    auto issue_part = [&](int step, int part) {
        const int k0 = (step < steps ? step : steps - 1) * BK;  // past the end: a harmless reload, keeps the wait counts uniform
        const uint32_t base = lds0 + (step % kStages) * kStageBytes;
        if (part < 4) dma16(xsrc[part] + k0, base + (part * 512 + wave * 64) * 16);
        else dma16(wsrc + (k0 >> 3), base + kXBytes + wave * 64 * 16);
    };
    auto issue = [&](int step) {
#pragma unroll
        for (int part = 0; part < 5; part++) issue_part(step, part);
    };

    // Scale/bias tables: thread t < 256 owns tile row t.
    const int srow = n0 + (tid & 255) < N ? n0 + (tid & 255) : N - 1;
    const T *sp = scales + (int64_t)srow * kgroups, *bp = biases + (int64_t)srow * kgroups;
    T sreg[8], breg[8];
    auto sb_load = [&](int period) {
        if (tid < 256) {
#pragma unroll
            for (int g = 0; g < 8; g++)
                if (g < gper) {
                    const int gi = period * gper + g < kgroups ? period * gper + g : kgroups - 1;
                    sreg[g] = sp[gi];
                    breg[g] = bp[gi];
                }
        }
    };
    auto sb_store = [&](int period) {
        if (tid < 256) {
            uint32_t *t = sb_table + (period & 1) * (kSbBytes / 4);
#pragma unroll
            for (int g = 0; g < 8; g++)
                if (g < gper) {
                    uint16_t sbits, bbits;
                    __builtin_memcpy(&sbits, &sreg[g], 2);
                    __builtin_memcpy(&bbits, &breg[g], 2);
                    t[g * BN + tid] = (uint32_t)sbits | ((uint32_t)bbits << 16);
                }
        }
    };

    floatx16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    const int h = lane >> 5, l32 = lane & 31;
    issue(0);
    issue(1);
    sb_load(0);
    sb_store(0);
    for (int step = 0; step < steps; step++) {
        dma_wait<5>();    // this lane's loads of `step` have landed (those of step + 1 may be in flight)
        __syncthreads();  // ... and everyone's; everyone is also done reading the stage refilled next
        // The table of the next 256 values of K is loaded two steps ahead and written one step ahead.
        // Its loads go before this step's direct-to-LDS loads so that the wait above never covers them.
        if ((step & 3) == 1 && step + 3 < steps) sb_load((step + 3) >> 2);
        issue_part(step + 2, 4);  // the remaining four parts are spread over the matrix work below
        const unsigned char *xs = lds + (step % kStages) * kStageBytes, *ws = xs + kXBytes;
        const uint32_t *sbt = sb_table + ((step >> 2) & 1) * (kSbBytes / 4) + ((((step & 3) * BK + 32 * h) >> gshift) * BN);
        uint4 raw[2];
        float sc[2], bi[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = wn * 64 + j * 32 + l32;
            raw[j] = *reinterpret_cast<const uint4 *>(ws + col * 32 + h * 16);
            const uint32_t sbv = sbt[col];
            sc[j] = Mma<T>::lo(sbv);
            bi[j] = Mma<T>::hi(sbv);
        }
        // x fragments are read one substep ahead of the matrix instructions that use them.
        uint4 af[2][4];
#pragma unroll
        for (int i = 0; i < 4; i++) af[0][i] = *reinterpret_cast<const uint4 *>(xs + lds_offset(wm * 128 + i * 32 + l32, 4 * h));
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            uint4 bf[2];
            if (kk < 3) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    af[(kk + 1) & 1][i] = *reinterpret_cast<const uint4 *>(xs + lds_offset(wm * 128 + i * 32 + l32, 4 * h + kk + 1));
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint32_t word = kk == 0 ? raw[j].x : kk == 1 ? raw[j].y : kk == 2 ? raw[j].z : raw[j].w;
                bf[j] = dequant8<T>(word, sc[j], bi[j]);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = Mma<T>::mfma(af[kk & 1][i], bf[j], acc[i][j]);
            issue_part(step + 2, kk);
        }
        if ((step & 3) == 2 && step + 2 < steps) sb_store((step + 2) >> 2);
    }
    dma_wait<0>();

    // Epilogue: accumulator element e of a 32 x 32 tile is row 8 (e / 4) + 4 (lane / 32) + e % 4, column lane % 32.
    // The 32 lanes of a half-wavefront store 32 consecutive elements of one row.
    const bool full = m0 + BM <= M && n0 + BN <= N;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n0 + wn * 64 + j * 32 + l32;
            const int row0 = m0 + wm * 128 + i * 32 + 4 * h;
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const uint32_t pair = Mma<T>::pack(acc[i][j][e], acc[i][j][e + 1]);  // rounded to nearest even
                const int row = row0 + 8 * (e >> 2) + (e & 3);
                uint16_t *out = reinterpret_cast<uint16_t *>(y) + (int64_t)row * N + col;
                if (full || (row < M && col < N)) out[0] = (uint16_t)pair;
                if (full || (row + 1 < M && col < N)) out[N] = (uint16_t)(pair >> 16);
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
    return a.batch <= 65535 && a.k >= BK && a.k % BK == 0;
}

int32_t launch_qmm(const ProductArgs &a, hipStream_t s) {
    return a.dtype == NVQ_BF16 ? run_qmm4<bf16_t>(a, s) : run_qmm4<f16_t>(a, s);
}

}  // namespace nvq
