// Tiled quantized products y[M,N] = x[M,K] . dequantize(w[N,K])^T on the gfx950 matrix cores: the
// prefill-shaped path, for affine 2, 3, 4, 6 and 8-bit codes and MXFP4 (this header holds the kernel template;
// the per-width translation units instantiate it).  Values follow nuvec's CPU product (reference:
// crates/nuvec-core/src/kernels.rs:1091-1142) within the stated tolerance; as in the reference's
// device kernels the weights are dequantized on chip in the element type (one rounding of
// fma(code, scale, bias)) and the products accumulate in float32
// (crates/nuvec-kernels/src/metal/quantized.h:583-817, 1358-1485).
//
// One block of 512 threads (eight wavefronts, 2 x 4, each 128 x 64 of y) owns a BM x BN = 256 x 256 tile
// and walks K in steps of BK = 64 through a ring of three LDS stages (products whose 256 x 256 tiles would not
// fill the chip take 128 x 128 tiles of four wavefronts, two blocks per compute unit).  A stage holds
//   * the x tile, 256 rows x 128 B, 16-byte chunk index XOR-ed with (row & 7) so that the 16-byte
//     fragment reads of the matrix instruction are bank-conflict free, and
//   * the w tile still packed, 256 rows x 8 BITS bytes: lane (row, half) of the loading threads owns the BITS
//     dwords of its 32 codes and brings them in one or two pieces (16, 12 or 4 bytes each), each piece of all
//     lanes forming one region of the stage (16 bytes per lane, 4 for single dwords).
// Both arrive by direct global-to-LDS loads (no registers, no copy instructions); the loads of step
// s+2 are issued before the matrix work of step s, and there is one barrier per step.  Scales and
// biases are staged per 256 values of K (four steps) in a small double-buffered LDS table.
// A wavefront dequantizes its own weight fragments right before use: per step and lane the LDS reads
// bring the 64 codes of its two columns; 8 codes -> float -> fma(code, scale, bias) -> packed element type
// (MXFP4: scaled FP4 conversions) make one matrix operand.  With two wavefronts per
// SIMD the conversion arithmetic of one runs under the matrix instructions of the other.
// The K order inside a step is permuted (fragment kk of lane half h is packed word 4 h + kk) so that
// a lane's four weight words are one contiguous 16 bytes; x fragments follow the same order.
#pragma once

#include "qmf_kernel.h"

#include <math.h>

namespace nvq {
namespace qmm {

using namespace qmf;  // element operations and code expansion

constexpr int BK = 64;
constexpr int kStages = 3;
constexpr int kRowBytes = BK * 2;   // 128 B per x row in LDS
constexpr int kPeriod = 256;        // values of K per scale/bias table

// A block's tile: WM x WN wavefronts, each TI x TJ matrix tiles of 32 x 32.  The number of threads equals
// twice the weight rows (one loading lane per row half) and the x tile takes four 16-byte pieces per thread.
template <int WM_, int WN_, int TI_, int TJ_>
struct Tile {
    static constexpr int WM = WM_, WN = WN_, TI = TI_, TJ = TJ_;
    static constexpr int BM = WM * TI * 32, BN = WN * TJ * 32;
    static constexpr int kThreads = WM * WN * 64;
    static constexpr int kXBytes = BM * kRowBytes;
    static constexpr int kSbBytes = (kPeriod / 32) * BN * 4;  // one table: up to 8 groups x BN rows x (scale, bias)
    static_assert(kThreads == 2 * BN && BM * 8 == 4 * kThreads, "the loading assignment below assumes these");
};
using BigTile = Tile<2, 4, 4, 2>;    // 256 x 256, 512 threads
using SmallTile = Tile<2, 2, 2, 2>;  // 128 x 128, 256 threads: for products whose big tiles would not fill the chip

// How a lane's BITS dwords travel into LDS: one or two pieces of 4, 3 or 1 dwords.
template <int BITS> struct Pieces;
template <> struct Pieces<2> { static constexpr int count = 2, dwords = 1; };
template <> struct Pieces<3> { static constexpr int count = 1, dwords = 3; };
template <> struct Pieces<4> { static constexpr int count = 1, dwords = 4; };
template <> struct Pieces<6> { static constexpr int count = 2, dwords = 3; };
template <> struct Pieces<8> { static constexpr int count = 2, dwords = 4; };

template <int BITS, class TL>
struct Geometry {
    // a 12-byte piece lands at 16 bytes per lane, like a 16-byte one (its fourth dword is not written)
    static constexpr int kPieceBytes = Pieces<BITS>::dwords == 1 ? 4 : 16;  // of LDS per lane and piece
    static constexpr int kRegionBytes = TL::kThreads * kPieceBytes;     // one piece of every loading lane
    static constexpr int kWBytes = Pieces<BITS>::count * kRegionBytes;  // packed codes of one step
    static constexpr int kStageBytes = TL::kXBytes + kWBytes;
    static constexpr int kLdsBytes = kStages * kStageBytes + 2 * TL::kSbBytes;  // big tile: 136 KB at 4 bits, 160 KB at 8
    static constexpr int kParts = 4 + Pieces<BITS>::count;              // direct-to-LDS loads per step and lane
};

// Byte offset of 16-byte chunk `chunk` (0..7) of LDS row `row`.
__device__ __forceinline__ int lds_offset(int row, int chunk) { return row * kRowBytes + ((chunk ^ (row & 7)) << 4); }

// Low / high 16 bits of a table entry as element-type values.
template <typename T> __device__ __forceinline__ float half_lo(uint32_t p);
template <typename T> __device__ __forceinline__ float half_hi(uint32_t p);
template <> __device__ __forceinline__ float half_lo<bf16_t>(uint32_t p) { return u2f(p << 16); }
template <> __device__ __forceinline__ float half_hi<bf16_t>(uint32_t p) { return u2f(p & 0xFFFF0000u); }
template <> __device__ __forceinline__ float half_lo<f16_t>(uint32_t p) { return (float)__builtin_bit_cast(f16x2v_t, p)[0]; }
template <> __device__ __forceinline__ float half_hi<f16_t>(uint32_t p) { return (float)__builtin_bit_cast(f16x2v_t, p)[1]; }

// DWORDS x 4 bytes per lane from global memory straight into LDS: lane l of the wavefront writes
// lds_base + 16 l (4 l for a single dword).  Issued as assembly so that the compiler keeps no account of it: the waits are
// placed by hand (dma_wait), which is what lets the loads of later steps stay in flight across
// the LDS reads of the current one.
template <int DWORDS>
__device__ __forceinline__ void dma(const void *src, uint32_t lds_base) {
    if constexpr (DWORDS == 4)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_base), "v"(src) : "memory", "m0");
    else if constexpr (DWORDS == 3)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx3 %1, off" : : "s"(lds_base), "v"(src) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(lds_base), "v"(src) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait() {  // all but the N most recent vector-memory loads of this lane are complete
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <typename T, int BITS, bool FP4, bool BATCHED, class TL>
__global__ void __launch_bounds__(TL::kThreads) qmm_kernel(const ProductArgs a) {
    using G = Geometry<BITS, TL>;
    constexpr int BM = TL::BM, BN = TL::BN, kThreads = TL::kThreads, kXBytes = TL::kXBytes, kSbBytes = TL::kSbBytes;
    constexpr int TI = TL::TI, TJ = TL::TJ;
    using P = Pieces<BITS>;
    using S = std::conditional_t<FP4, uint8_t, T>;  // stored scale type
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    uint32_t *sb_table = reinterpret_cast<uint32_t *>(lds + kStages * G::kStageBytes);  // [2][group][row]: scale | bias << 16
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / TL::WN, wn = wave % TL::WN;  // wavefront grid WM x WN: 32 TI x 32 TJ each
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = FP4 ? 5 : (a.group == 32 ? 5 : a.group == 64 ? 6 : 7);
    const int row_dwords = (K >> 5) * BITS, kgroups = K >> gshift;
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
    const S *scales = (const S *)a.scales + bs, *biases = (const S *)a.biases + bs;
    T *y = (T *)a.y + by;

    // Direct-to-LDS assignment.  x: instruction i of wavefront v fills the 64 consecutive 16-byte
    // slots starting at slot i*512 + v*64; slot S is row S/8, position S%8, and holds chunk
    // position ^ (row & 7) of that row.  w: loading lane v*64 + l is half l%2 of row (v*64 + l)/2 and owns the
    // BITS dwords of that half's 32 codes.
    const T *xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int slot = i * kThreads + wave * 64 + lane, row = slot >> 3, chunk = (slot & 7) ^ (row & 7);
        const int grow = m0 + row < M ? m0 + row : M - 1;  // tail rows are computed, not stored
        xsrc[i] = x + (int64_t)grow * K + chunk * 8;
    }
    const int wslot = wave * 64 + lane;
    const int wrow = n0 + (wslot >> 1) < N ? n0 + (wslot >> 1) : N - 1;
    const uint32_t *wsrc = w + (int64_t)wrow * row_dwords + (wslot & 1) * BITS;
    const int steps = K / BK;  // K is a multiple of 64 (checked on the host)
    // Load `part` (0..3: x, 4..: the pieces of w) of `step`.
    auto issue_part = [&](int step, int part) {
        const int sc = step < steps ? step : steps - 1;  // past the end: a harmless reload, keeps the wait counts uniform
        const uint32_t base = lds0 + (step % kStages) * G::kStageBytes;
        if (part < 4) {
            dma<4>(xsrc[part] + sc * BK, base + (part * kThreads + wave * 64) * 16);
        } else {
            const int piece = part - 4;
            dma<P::dwords>(wsrc + sc * 2 * BITS + piece * P::dwords, base + kXBytes + piece * G::kRegionBytes + wave * 64 * G::kPieceBytes);
        }
    };
    auto issue = [&](int step) {
#pragma unroll
        for (int part = 0; part < G::kParts; part++) issue_part(step, part);
    };

    // Scale/bias tables: thread t < BN owns tile row t.
    const int srow = n0 + (tid % BN) < N ? n0 + (tid % BN) : N - 1;
    const S *sp = scales + (int64_t)srow * kgroups, *bp = biases + (int64_t)srow * kgroups;
    S sreg[8], breg[8];
    auto sb_load = [&](int period) {
        if (tid < BN) {
#pragma unroll
            for (int g = 0; g < 8; g++)
                if (g < gper) {
                    const int gi = period * gper + g < kgroups ? period * gper + g : kgroups - 1;
                    sreg[g] = sp[gi];
                    if constexpr (!FP4) breg[g] = bp[gi];
                }
        }
    };
    auto sb_store = [&](int period) {
        if (tid < BN) {
            uint32_t *t = sb_table + (period & 1) * (kSbBytes / 4);
#pragma unroll
            for (int g = 0; g < 8; g++)
                if (g < gper) {
                    if constexpr (FP4) {
                        t[g * BN + tid] = (uint32_t)sreg[g];
                    } else {
                        uint16_t sbits, bbits;
                        __builtin_memcpy(&sbits, &sreg[g], 2);
                        __builtin_memcpy(&bbits, &breg[g], 2);
                        t[g * BN + tid] = (uint32_t)sbits | ((uint32_t)bbits << 16);
                    }
                }
        }
    };

    floatx16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    const int h = lane >> 5, l32 = lane & 31;
    issue(0);
    issue(1);
    sb_load(0);
    sb_store(0);
    for (int step = 0; step < steps; step++) {
        dma_wait<G::kParts>();  // this lane's loads of `step` have landed (those of step + 1 may be in flight)
        __syncthreads();        // ... and everyone's; everyone is also done reading the stage refilled next
        // The table of the next 256 values of K is loaded two steps ahead and written one step ahead.
        // Its loads go before this step's direct-to-LDS loads so that the wait above never covers them.
        if ((step & 3) == 1 && step + 3 < steps) sb_load((step + 3) >> 2);
#pragma unroll
        for (int part = 4; part < G::kParts; part++) issue_part(step + 2, part);  // the x parts are spread over the matrix work below
        const unsigned char *xs = lds + (step % kStages) * G::kStageBytes, *ws = xs + kXBytes;
        const uint32_t *sbt = sb_table + ((step >> 2) & 1) * (kSbBytes / 4) + ((((step & 3) * BK + 32 * h) >> gshift) * BN);
        uint32_t raw[TJ][BITS];
        float sc[TJ], bi[TJ];
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = wn * (32 * TJ) + j * 32 + l32;
#pragma unroll
            for (int piece = 0; piece < P::count; piece++) {
                const unsigned char *src = ws + piece * G::kRegionBytes + (col * 2 + h) * G::kPieceBytes;
                if constexpr (P::dwords == 4) {
                    const u32x4_t v = *reinterpret_cast<const u32x4_t *>(src);
                    raw[j][4 * piece] = v.x, raw[j][4 * piece + 1] = v.y, raw[j][4 * piece + 2] = v.z, raw[j][4 * piece + 3] = v.w;
                } else {
#pragma unroll
                    for (int d = 0; d < P::dwords; d++) raw[j][P::dwords * piece + d] = reinterpret_cast<const uint32_t *>(src)[d];
                }
            }
            const uint32_t sbv = sbt[col];
            if constexpr (FP4) {
                sc[j] = ftz(e8m0_to_f32((uint8_t)sbv));
                bi[j] = 0.0f;
            } else {
                sc[j] = half_lo<T>(sbv);
                bi[j] = half_hi<T>(sbv);
            }
        }
        // x fragments are read one substep ahead of the matrix instructions that use them.
        uint4 af[2][TI];
#pragma unroll
        for (int i = 0; i < TI; i++) af[0][i] = *reinterpret_cast<const uint4 *>(xs + lds_offset(wm * (32 * TI) + i * 32 + l32, 4 * h));
        static_for<4>([&](auto kk_tag) {
            constexpr int kk = decltype(kk_tag)::value;
            uint4 bf[TJ];
            if constexpr (kk < 3) {
#pragma unroll
                for (int i = 0; i < TI; i++)
                    af[(kk + 1) & 1][i] = *reinterpret_cast<const uint4 *>(xs + lds_offset(wm * (32 * TI) + i * 32 + l32, 4 * h + kk + 1));
            }
#pragma unroll
            for (int j = 0; j < TJ; j++) bf[j] = expand_piece<T, BITS, FP4, kk>(raw[j], sc[j], bi[j]);
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++) acc[i][j] = Ops<T>::mfma(af[kk & 1][i], bf[j], acc[i][j]);
            issue_part(step + 2, kk);
        });
        if ((step & 3) == 2 && step + 2 < steps) sb_store((step + 2) >> 2);
    }
    dma_wait<0>();

    // Epilogue: accumulator element e of a 32 x 32 tile is row 8 (e / 4) + 4 (lane / 32) + e % 4, column lane % 32.
    // The 32 lanes of a half-wavefront store 32 consecutive elements of one row.
    const bool full = m0 + BM <= M && n0 + BN <= N;
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn * (32 * TJ) + j * 32 + l32;
            const int row0 = m0 + wm * (32 * TI) + i * 32 + 4 * h;
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const uint32_t pair = Ops<T>::pack(acc[i][j][e], acc[i][j][e + 1]);  // rounded to nearest even
                const int row = row0 + 8 * (e >> 2) + (e & 3);
                uint16_t *out = reinterpret_cast<uint16_t *>(y) + (int64_t)row * N + col;
                if (full || (row < M && col < N)) out[0] = (uint16_t)pair;
                if (full || (row + 1 < M && col < N)) out[N] = (uint16_t)(pair >> 16);
            }
        }
}

// Estimated microseconds of the tiled kernel with tile TL on `cus` compute units, from its measured behaviour:
// about 1.7 us (big tile, one block per compute unit) or 1.0 us (small tile, two blocks) per step of 64 values
// and round of tiles.
template <class TL>
inline double estimate_us(const ProductArgs &a, int cus) {
    const double tiles = (double)((a.m + TL::BM - 1) / TL::BM) * (double)((a.n + TL::BN - 1) / TL::BN) * (double)a.batch;
    const bool big = TL::BM == 256;
    const double rounds = ceil(tiles / ((double)cus * (big ? 1.0 : 2.0)));
    return rounds * (double)(a.k / BK) * (big ? 1.7 : 1.0);
}
inline bool small_tile_is_faster(const ProductArgs &a, int cus) { return estimate_us<SmallTile>(a, cus) < estimate_us<BigTile>(a, cus); }

template <typename T, int BITS, bool FP4, class TL>
int32_t run_tile(const ProductArgs &a, hipStream_t s) {
    using G = Geometry<BITS, TL>;
    static bool configured[2] = {false, false};
    const bool batched = a.batch > 1;
    auto kernel = batched ? qmm_kernel<T, BITS, FP4, true, TL> : qmm_kernel<T, BITS, FP4, false, TL>;
    if (!configured[batched]) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, G::kLdsBytes));
        configured[batched] = true;
    }
    dim3 grid((unsigned)((a.n + TL::BN - 1) / TL::BN), (unsigned)((a.m + TL::BM - 1) / TL::BM), (unsigned)a.batch);
    hipLaunchKernelGGL(kernel, grid, dim3(TL::kThreads), G::kLdsBytes, s, a);
    NVQ_LAUNCH_CHECK("qmm");
    return NVQ_OK;
}

template <typename T, int BITS, bool FP4>
int32_t run(const ProductArgs &a, hipStream_t s) {
    return small_tile_is_faster(a, compute_units()) ? run_tile<T, BITS, FP4, SmallTile>(a, s) : run_tile<T, BITS, FP4, BigTile>(a, s);
}

template <int BITS, bool FP4>
int32_t run_dtype(const ProductArgs &a, hipStream_t s) {
    return a.dtype == NVQ_BF16 ? run<bf16_t, BITS, FP4>(a, s) : run<f16_t, BITS, FP4>(a, s);
}

}  // namespace qmm

// One per code width, each in its own translation unit.
int32_t launch_qmm_b2(const ProductArgs &a, hipStream_t s);
int32_t launch_qmm_b3(const ProductArgs &a, hipStream_t s);
int32_t launch_qmm_b4(const ProductArgs &a, hipStream_t s);
int32_t launch_qmm_b6(const ProductArgs &a, hipStream_t s);
int32_t launch_qmm_b8(const ProductArgs &a, hipStream_t s);
int32_t launch_qmm_fp4(const ProductArgs &a, hipStream_t s);

}  // namespace nvq
