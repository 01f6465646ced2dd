// Tiled quantized products y[M,N] = x[M,K] . dequantize(w[N,K])^T on the gfx950 matrix cores: the
// prefill-shaped path, for affine 1- to 6- and 8-bit codes and the block formats (this header holds the kernel template;
// the per-width translation units instantiate it).  Values follow nuvec's CPU product (reference:
// crates/nuvec-core/src/kernels.rs:1091-1142) within the stated tolerance; as in the reference's
// device kernels the weights are dequantized on chip in the element type (one rounding of
// fma(code, scale, bias)) and the products accumulate in float32
// (crates/nuvec-kernels/src/metal/quantized.h:583-817, 1358-1485).
//
// One block of 256 threads (four wavefronts, one per SIMD, each 256 x 64 of y in 256 accumulator registers) owns a
// BM x BN = 256 x 256 tile and walks K in steps of BK = 64 through a ring of three LDS stages (products whose
// 256 x 256 tiles would not fill the chip take 128 x 128 tiles of 2 x 2 wavefronts, two blocks per compute unit).
// A wavefront covers all rows of the tile, so every weight is expanded once per block.  A stage holds
//   * the x tile, 256 rows x 128 B, 16-byte chunk index XOR-ed with (row >> 1) & 7 so that the 16-byte
//     fragment reads of the matrix instruction are free of conflicts on the 64 LDS banks, and
//   * the w tile still packed, 256 rows x 8 BITS bytes: loading slot (row, half) owns the BITS dwords of its 32
//     codes and brings them in one or two pieces (16, 12 or 4 bytes each), each piece of all slots forming one
//     region of the stage (16 bytes per slot, 4 for single dwords).
// Both arrive by direct global-to-LDS loads (no registers, no copy instructions) whose addresses are a scalar
// base per step plus a constant per-lane offset; the loads of step s+2 are issued during step s, and there is one
// barrier per step.  Scales and biases of four groups at a time (two of 128) travel the same way, one 16-bit
// element per lane and load, into a double-buffered table.
// The K loop is a written software pipeline.  A wavefront issues little more than one instruction per five cycles,
// so whatever is not a matrix instruction has to fit under one: after each of a substep's sixteen matrix
// instructions comes one item of side work for the next substep (the read of one x fragment, or two codes ->
// float -> fma(code, scale, bias) -> packed element type; MXFP4: scaled FP4 conversions), kept in that order with
// scheduling barriers.  The step's last substep first waits for the next stage (and everyone's), then prepares
// the next step's first operands under its own matrix instructions.
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

// A block's tile: WM x WN wavefronts, each TI x TJ matrix tiles of 32 x 32.  Per step a thread brings kXParts
// 16-byte pieces of the x tile and the codes of kWSlots weight row halves (32 codes each).
template <int WM_, int WN_, int TI_, int TJ_>
struct Tile {
    static constexpr int WM = WM_, WN = WN_, TI = TI_, TJ = TJ_;
    static constexpr int BM = WM * TI * 32, BN = WN * TJ * 32;
    static constexpr int kThreads = WM * WN * 64;
    static constexpr int kXBytes = BM * kRowBytes;
    static constexpr int kSbBytes = 2 * 4 * BN * 4;  // one table: (scales, biases) x 4 groups x BN rows, a dword each
    static constexpr int kXParts = BM * 8 / kThreads, kWSlots = 2 * BN / kThreads;
    static constexpr int kWavesPerSimd = TI * TJ >= 16 ? 1 : 2;  // by the accumulators: 256 or 128 registers of the 512
    static_assert(kXParts % 4 == 0 && kXParts * kThreads == BM * 8 && kWSlots * kThreads == 2 * BN && BN <= kThreads,
                  "the loading assignment below assumes these");
};
using BigTile = Tile<1, 4, 8, 2>;    // 256 x 256, 256 threads: one wavefront per SIMD owns 256 x 64, no code is expanded twice
using SmallTile = Tile<2, 2, 2, 2>;  // 128 x 128, 256 threads, two blocks per compute unit: for products whose big tiles would not fill the chip

// How a lane's BITS dwords travel into LDS: one or two pieces of 4, 3 or 1 dwords.
template <int BITS> struct Pieces;
template <> struct Pieces<1> { static constexpr int count = 1, dwords = 1; };
template <> struct Pieces<2> { static constexpr int count = 2, dwords = 1; };
template <> struct Pieces<3> { static constexpr int count = 1, dwords = 3; };
template <> struct Pieces<4> { static constexpr int count = 1, dwords = 4; };
template <> struct Pieces<5> { static constexpr int count = 5, dwords = 1; };
template <> struct Pieces<6> { static constexpr int count = 2, dwords = 3; };
template <> struct Pieces<8> { static constexpr int count = 2, dwords = 4; };

template <int BITS, class TL>
struct Geometry {
    // a 12-byte piece lands at 16 bytes per lane, like a 16-byte one (its fourth dword is not written)
    static constexpr int kPieceBytes = Pieces<BITS>::dwords == 1 ? 4 : 16;  // of LDS per lane and piece
    static constexpr int kRegionBytes = 2 * TL::BN * kPieceBytes;       // one piece of every row half
    static constexpr int kWBytes = Pieces<BITS>::count * kRegionBytes;  // packed codes of one step
    static constexpr int kStageBytes = TL::kXBytes + kWBytes;
    static constexpr int kLdsBytes = kStages * kStageBytes + 2 * TL::kSbBytes;  // big tile: 136 KB at 4 bits, 160 KB at 8
    static constexpr int kParts = TL::kXParts + TL::kWSlots * Pieces<BITS>::count;  // direct-to-LDS loads per step and lane
};

// Byte offset of 16-byte chunk `chunk` (0..7) of LDS row `row`.  The LDS has 64 banks of 4 bytes: sixteen
// consecutive rows reading the same chunk fall on sixteen different 16-byte bank groups (the row's parity picks
// the half, the swizzle the group within it).
__device__ __forceinline__ int swizzle(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int lds_offset(int row, int chunk) { return row * kRowBytes + ((chunk ^ swizzle(row)) << 4); }

// DWORDS x 4 bytes per lane from global memory straight into LDS: lane l of the wavefront reads base + offset
// (a wavefront-uniform base, so the per-step address arithmetic is scalar) and writes lds_base + 16 l (4 l for
// a single dword).  Issued as assembly so that the compiler keeps no account of it: the waits are placed by hand
// (dma_wait), which is what lets the loads of later steps stay in flight across the LDS reads of the current one.
template <int DWORDS>
__device__ __forceinline__ void dma(const void *base, uint32_t offset, uint32_t lds_base) {
    if constexpr (DWORDS == 4)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
    else if constexpr (DWORDS == 3)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx3 %1, %2" : : "s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait() {  // all but the N most recent vector-memory loads of this lane are complete
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
// One 16-bit (or 8-bit) element per lane, zero-extended to the dword at lds_base + 4 l.
template <int BYTES>
__device__ __forceinline__ void dma_element(const void *base, uint32_t offset, uint32_t lds_base) {
    if constexpr (BYTES == 2)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2" : : "s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ubyte %1, %2" : : "s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
}
// Nothing moves across this point when the compiler orders the instructions: the interleaving of matrix
// instructions, LDS reads and code expansion below is the written one.
__device__ __forceinline__ void pin() { __builtin_amdgcn_sched_barrier(0); }
// A use of `v` at this point: what computes it stays in this block of the loop instead of sinking into the block
// of its first real use, where nothing would run beside it.
__device__ __forceinline__ void keep(const uint4 &v) { asm volatile("" : : "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w)); }

// Dword D (two elements) of piece KK of a lane's 32 codes: expand_piece, one register at a time.
template <typename T, int BITS, int FP4, int KK, int D, bool EXACT = false>
__device__ __forceinline__ uint32_t expand_dword(const uint32_t (&dw)[BITS], float s, float b) {
    if constexpr (FP4 == kMxfp8) {
        return Ops<T>::template fp8_pair<(D & 1) != 0>(Ops<T>::mx_codes(dw[2 * KK + D / 2], s), s);
    } else if constexpr (FP4 == kNvfp4) {
        return fp4_pair_times<T, D>(dw[KK], s);
    } else if constexpr (FP4) {
        return Ops<T>::template fp4_pair<D>(Ops<T>::mx_codes(dw[KK], s), s);
    } else if constexpr (BITS == 4) {
        const uint32_t word = dw[KK];
        const uint32_t even = opaque(word & 0x0F0F0F0Fu), odd = opaque((word >> 4) & 0x0F0F0F0Fu);
        return affine_pair<T, EXACT>(ubyte_to_float<D>(even), ubyte_to_float<D>(odd), s, b);
    } else {
        constexpr int J = 8 * KK + 2 * D;
        return affine_pair<T, EXACT>(code_to_float<BITS, J>(dw), code_to_float<BITS, J + 1>(dw), s, b);
    }
}

// EXACT (affine codes): the weights as nuvec's CPU product holds them (affine_pair).
template <typename T, int BITS, int FP4, bool BATCHED, class TL, bool EXACT = false>
__global__ void __launch_bounds__(TL::kThreads) __attribute__((amdgpu_waves_per_eu(TL::kWavesPerSimd, TL::kWavesPerSimd)))
qmm_kernel(const ProductArgs a) {
    using G = Geometry<BITS, TL>;
    constexpr int BM = TL::BM, BN = TL::BN, kThreads = TL::kThreads, kXBytes = TL::kXBytes, kSbBytes = TL::kSbBytes;
    constexpr int TI = TL::TI, TJ = TL::TJ;
    using P = Pieces<BITS>;
    using S = std::conditional_t<FP4 != 0, uint8_t, T>;  // stored scale type
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    // Scale and bias tables, two buffers of [scale | bias][group 0..3][row] dwords (the element in the low bits).
    const uint32_t *sb_table = reinterpret_cast<const uint32_t *>(lds + kStages * G::kStageBytes);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / TL::WN, wn = wave % TL::WN;  // wavefront grid WM x WN: 32 TI x 32 TJ each
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = FP4 == kNvfp4 ? 4 : FP4 ? 5 : (a.group == 32 ? 5 : a.group == 64 ? 6 : 7);
    const int row_dwords = (K >> 5) * BITS, kgroups = K >> gshift;
    // A table covers a period of 4 groups (2 of 128; NVFP4, which has no biases: 8 of 16): two steps for groups of 16
    // and 32, else four.
    constexpr int kTableGroups = FP4 == kNvfp4 ? 8 : 4;
    const int pshift = gshift <= 5 ? 1 : 2, psteps = 1 << pshift;
    const int gper = (psteps * BK) >> gshift;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    // A single product may split K over grid z (few tiles, long K): this block takes the steps
    // [step0, step0 + steps) and leaves float32 partial sums for a second kernel.
    int step0 = 0, steps = K / BK;  // K is a multiple of 64 (checked on the host)
    if constexpr (!BATCHED) {
        if (a.k_splits > 1) {
            step0 = blockIdx.z * a.k_split_steps;  // whole table periods
            steps = steps - step0 < a.k_split_steps ? steps - step0 : a.k_split_steps;
            if (steps <= 0) return;  // (the host sizes the grid so that every split has a step)
        }
    }
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
    // slots starting at slot i*kThreads + v*64; slot S is row S/8, position S%8, and holds chunk
    // position ^ swizzle(row) of that row.  w: loading slot S is half S%2 of row S/2 and owns the BITS dwords of that
    // half's 32 codes.  Addresses are a block-uniform base (advanced per step with scalar arithmetic) plus a
    // per-lane byte offset that never changes.
    constexpr int XP = TL::kXParts, WS = TL::kWSlots;
    const char *xbase = reinterpret_cast<const char *>(x + (int64_t)m0 * K + (int64_t)step0 * BK);
    const char *wbase = reinterpret_cast<const char *>(w + (int64_t)n0 * row_dwords + (int64_t)step0 * 2 * BITS);
    uint32_t xoff[XP], woff[WS];
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const int slot = i * kThreads + wave * 64 + lane, row = slot >> 3, chunk = (slot & 7) ^ swizzle(row);
        const int r = m0 + row < M ? row : M - 1 - m0;  // tail rows are computed, not stored
        xoff[i] = ((uint32_t)r * (uint32_t)K + chunk * 8) * 2;
    }
#pragma unroll
    for (int j = 0; j < WS; j++) {
        const int slot = j * kThreads + wave * 64 + lane;
        const int r = n0 + (slot >> 1) < N ? (slot >> 1) : N - 1 - n0;
        woff[j] = ((uint32_t)r * (uint32_t)row_dwords + (slot & 1) * BITS) * 4;
    }
    // The loads of one step: its global bases (a step past the end reloads the last one, harmlessly, which keeps
    // the wait counts uniform) and the LDS address of this wavefront's lane 0 in the step's stage.
    struct Loads {
        const char *x, *w[P::count];
        uint32_t lds;
    };
    const uint32_t lds_wave = lds0 + wave * 64 * 16;
    auto loads_of = [&](int step, int stage) {
        const int sc = step < steps ? step : steps - 1;
        Loads l;
        l.x = xbase + sc * (BK * 2);
#pragma unroll
        for (int piece = 0; piece < P::count; piece++) l.w[piece] = wbase + sc * (2 * BITS * 4) + piece * (P::dwords * 4);
        l.lds = lds_wave + stage * G::kStageBytes;
        // computed here once, in scalar registers, not again at every load
        asm volatile("" : "+s"(l.x), "+s"(l.lds));
#pragma unroll
        for (int piece = 0; piece < P::count; piece++) asm volatile("" : "+s"(l.w[piece]));
        return l;
    };
    // Load `part` (0..XP-1: x, then the pieces of each weight slot).
    auto issue_part = [&](const Loads &l, auto part_tag) {
        constexpr int part = decltype(part_tag)::value;
        if constexpr (part < XP) {
            dma<4>(l.x, xoff[part], l.lds + part * kThreads * 16);
        } else {
            constexpr int j = (part - XP) / P::count, piece = (part - XP) % P::count;
            // the wavefront's share of a weight region starts at wave * 64 pieces, not wave * 64 * 16 bytes
            constexpr int off = kXBytes + piece * G::kRegionBytes + j * kThreads * G::kPieceBytes;
            dma<P::dwords>(l.w[piece], woff[j], l.lds + off - (G::kPieceBytes == 16 ? 0 : wave * 64 * 12));
        }
    };
    auto issue_parts = [&](const Loads &l, auto first_tag, auto count_tag) {
        static_for<decltype(count_tag)::value>([&](auto i) { issue_part(l, std::integral_constant<int, decltype(first_tag)::value + decltype(i)::value>{}); });
    };
    // The table of period `period`: every wavefront brings kTableLoads times 64 consecutive rows of one group's
    // scales or biases (groups past the row's last one repeat it: they are never read).
    constexpr int kKinds = FP4 ? 1 : 2, kTableLoads = kKinds * kTableGroups * BN / kThreads;
    const int trow = n0 + tid % BN < N ? tid % BN : N - 1 - n0;
    const uint32_t toff = (uint32_t)trow * (uint32_t)kgroups * (uint32_t)sizeof(S);
    const int g0 = (step0 * BK) >> gshift, groups_left = kgroups - g0;  // this block's first group
    const char *sbase = reinterpret_cast<const char *>(scales + (int64_t)n0 * kgroups + g0);
    const char *bbase = reinterpret_cast<const char *>(biases + (int64_t)n0 * kgroups + g0);
    auto issue_table = [&](int period) {
        const uint32_t tbase = lds0 + kStages * G::kStageBytes + (period & 1) * kSbBytes;
#pragma unroll
        for (int i = 0; i < kTableLoads; i++) {
            const int entry = i * kThreads + wave * 64;  // of this wavefront's first lane: [kind][group][row]
            const int kind = entry / (kTableGroups * BN), g = (entry / BN) % kTableGroups;
            const int gi = period * gper + g < groups_left ? period * gper + g : groups_left - 1;
            dma_element<sizeof(S)>((kind ? bbase : sbase) + gi * (int)sizeof(S), toff, tbase + entry * 4);
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
    uint32_t raw[TJ][BITS], sraw[TJ], braw[TJ];  // codes and table entries as read: converted where first used (NVFP4: braw is the second scale)
    float sc[TJ][2], bi[TJ];
    uint4 af[2][TI], bf[2][TJ];
    // The packed codes, scales and biases of this lane's TJ columns for `step` (its stage and table are visible).
    auto read_codes = [&](int step, int stage) {
        const unsigned char *ws = lds + stage * G::kStageBytes + kXBytes;
        const uint32_t *sbt = sb_table + ((step >> pshift) & 1) * (kSbBytes / 4) + ((((step & (psteps - 1)) * BK + 32 * h) >> gshift) * BN);
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
            sraw[j] = sbt[col];
            if constexpr (!FP4) braw[j] = sbt[4 * BN + col];
            if constexpr (FP4 == kNvfp4) braw[j] = sbt[BN + col];  // the lane's second group of 16
        }
    };
    const float factor = FP4 == kNvfp4 ? nvfp4_factor(a, 0) : 1.0f;  // (one matrix, or a batch that shares the scale)
    auto convert_scales = [&](int j) {
        if constexpr (FP4 == kNvfp4) {
            sc[j][0] = nvfp4_scale((uint8_t)sraw[j], factor);
            sc[j][1] = nvfp4_scale((uint8_t)braw[j], factor);
            bi[j] = 0.0f;
        } else if constexpr (FP4) {
            sc[j][0] = sc[j][1] = ftz(e8m0_to_f32((uint8_t)sraw[j]));
            bi[j] = 0.0f;
        } else {
            sc[j][0] = sc[j][1] = half_lo<T>(sraw[j]);
            bi[j] = half_lo<T>(braw[j]);
        }
    };
    // x fragment i of substep kk of the step in `stage`.
    auto read_x = [&](int stage, int kk, int i) {
        return *reinterpret_cast<const uint4 *>(lds + stage * G::kStageBytes + lds_offset(wm * (32 * TI) + i * 32 + l32, 4 * h + kk));
    };
    // The side work that prepares substep (step, KK) into buffer (KK & 1), in items: first x fragment reads and
    // expanded dwords alternate, then what is left of either.  Item t of kItems.
    // Substep 0 of the next step takes all reads first: its codes were only just requested.
    constexpr int kItems = TI + 4 * TJ, kPairs = TI < 4 * TJ ? TI : 4 * TJ;
    auto side_item = [&](int stage, auto kk_tag, auto t_tag) {
        constexpr int KK = decltype(kk_tag)::value, t = decltype(t_tag)::value;
        constexpr bool alternate = KK != 0 && t < 2 * kPairs;
        constexpr bool is_read = KK == 0 ? t < TI : (alternate ? t % 2 == 0 : TI > 4 * TJ);
        constexpr int index = KK == 0 ? (t < TI ? t : t - TI) : (alternate ? t / 2 : t - kPairs);
        if constexpr (is_read) {
            af[KK & 1][index] = read_x(stage, KK, index);
        } else {
            constexpr int j = index / 4, d = index % 4;
            if constexpr (KK == 0 && d == 0) convert_scales(j);
            const uint32_t v = expand_dword<T, BITS, FP4, KK, d, EXACT>(raw[j], sc[j][KK >> 1], bi[j]);
            if constexpr (d == 0) bf[KK & 1][j].x = v;
            else if constexpr (d == 1) bf[KK & 1][j].y = v;
            else if constexpr (d == 2) bf[KK & 1][j].z = v;
            else bf[KK & 1][j].w = v;
        }
    };

    // Prologue: tables, two steps of loads in flight, the first substep's operands.
    issue_table(0);
    if (psteps == 2) issue_table(1);
    using c0 = std::integral_constant<int, 0>;
    issue_parts(loads_of(0, 0), c0{}, std::integral_constant<int, G::kParts>{});
    issue_parts(loads_of(1, 1), c0{}, std::integral_constant<int, G::kParts>{});
    dma_wait<G::kParts>();
    __syncthreads();
    read_codes(0, 0);
    static_for<kItems>([&](auto t) { side_item(0, c0{}, t); });

    constexpr int kMfmas = TI * TJ;
    int stage = 0;  // step % kStages
    for (int step = 0; step < steps; step++) {
        // Entering: stage `step` is visible to everyone, this lane holds its codes, and buffer 0 holds substep 0.
        const int stage1 = stage == kStages - 1 ? 0 : stage + 1, stage2 = stage1 == kStages - 1 ? 0 : stage1 + 1;
        const Loads next2 = loads_of(step + 2, stage2);
        issue_parts(next2, std::integral_constant<int, XP>{}, std::integral_constant<int, G::kParts - XP>{});  // w first; x is spread below
        static_for<4>([&](auto kk_tag) {
            constexpr int kk = decltype(kk_tag)::value;
            constexpr int next = (kk + 1) & 3;
            using next_tag = std::integral_constant<int, next>;
            if constexpr (kk == 3) {
                // The step's last substep also turns to the next step: its stage must have landed for everyone
                // (and everyone is done reading the stage that the next loads refill), then its codes and first
                // operands are read and expanded under this substep's matrix instructions.
                issue_parts(next2, std::integral_constant<int, 3 * (XP / 4)>{}, std::integral_constant<int, XP - 3 * (XP / 4)>{});
                // (a table issued after the previous step's barrier is older than those loads: it is waited for too,
                // a step after its issue rather than two)
                dma_wait<G::kParts>();
                __syncthreads();
                if (((step + 3) & (psteps - 1)) == 0 && step + 3 < steps) issue_table((step + 3) >> pshift);
                read_codes(step + 1, stage1);
                pin();
            }
            static_for<kMfmas>([&](auto q_tag) {
                constexpr int q = decltype(q_tag)::value, i = q % TI, j = q / TI;
                acc[i][j] = Ops<T>::mfma(af[kk & 1][i], bf[kk & 1][j], acc[i][j]);
                static_for<kItems>([&](auto t_tag) {
                    constexpr int t = decltype(t_tag)::value;
                    if constexpr (t >= q * kItems / kMfmas && t < (q + 1) * kItems / kMfmas) side_item(kk == 3 ? stage1 : stage, next_tag{}, t_tag);
                });
                pin();
            });
            if constexpr (kk < 3) issue_parts(next2, std::integral_constant<int, kk * (XP / 4)>{}, std::integral_constant<int, XP / 4>{});
            if constexpr (kk >= 2) {  // the blocks of the loop end after substeps 2 and 3
#pragma unroll
                for (int j = 0; j < TJ; j++) keep(bf[next & 1][j]);
            }
        });
        stage = stage1;
    }
    dma_wait<0>();

    // Epilogue: accumulator element e of a 32 x 32 tile is row 8 (e / 4) + 4 (lane / 32) + e % 4, column lane % 32.
    // The 32 lanes of a half-wavefront store 32 consecutive elements of one row.
    auto store_tile = [&](auto whole_tag) {
        constexpr bool whole = decltype(whole_tag)::value;  // the tile lies inside y: no element is tested
        uint16_t *out0 = reinterpret_cast<uint16_t *>(y) + (int64_t)(m0 + wm * (32 * TI) + 4 * h) * N + n0 + wn * (32 * TJ) + l32;
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const int col = n0 + wn * (32 * TJ) + j * 32 + l32;
                const int row0 = m0 + wm * (32 * TI) + i * 32 + 4 * h;
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    const uint32_t pair = Ops<T>::pack(add_row_bias<T>(a.row_bias, acc[i][j][e], col),
                                                       add_row_bias<T>(a.row_bias, acc[i][j][e + 1], col));  // rounded to nearest even
                    const int r = i * 32 + 8 * (e >> 2) + (e & 3);
                    uint16_t *out = out0 + (int64_t)r * N + j * 32;
                    if (whole || (row0 + r - i * 32 < M && col < N)) out[0] = (uint16_t)pair;
                    if (whole || (row0 + r - i * 32 + 1 < M && col < N)) out[N] = (uint16_t)(pair >> 16);
                }
            }
    };
    if constexpr (!BATCHED) {
        if (a.k_splits > 1) {  // float32 partial sums [split][M][N]
            float *out0 = a.partials + ((int64_t)blockIdx.z * M + m0 + wm * (32 * TI) + 4 * h) * N + n0 + wn * (32 * TJ) + l32;
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    const int col = n0 + wn * (32 * TJ) + j * 32 + l32;
                    const int row0 = m0 + wm * (32 * TI) + i * 32 + 4 * h;
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        const int r = 8 * (e >> 2) + (e & 3);
                        if (row0 + r < M && col < N) out0[(int64_t)(i * 32 + r) * N + j * 32] = acc[i][j][e];
                    }
                }
            return;
        }
    }
    if (m0 + BM <= M && n0 + BN <= N) store_tile(std::true_type{});
    else store_tile(std::false_type{});
}

// y = the splits' partial sums added in split order, rounded once.
template <typename T>
__global__ void __launch_bounds__(256) qmm_reduce_kernel(const float *__restrict__ partials, T *__restrict__ y, int splits, int64_t total,
                                                         const void *row_bias, int64_t n) {
    const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (idx >= total) return;
    if (idx + 4 <= total) {
        float4 sum = *reinterpret_cast<const float4 *>(partials + idx);
        int s = 1;
        for (; s + 4 <= splits; s += 4) {  // four loads under way at a time; the additions keep the splits' order
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const float4 *>(partials + (s + u) * total + idx);
#pragma unroll
            for (int u = 0; u < 4; u++) sum.x += v[u].x, sum.y += v[u].y, sum.z += v[u].z, sum.w += v[u].w;
        }
        for (; s < splits; s++) {
            const float4 v = *reinterpret_cast<const float4 *>(partials + s * total + idx);
            sum.x += v.x, sum.y += v.y, sum.z += v.z, sum.w += v.w;
        }
        const float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
        for (int j = 0; j < 4; j++) Elem<T>::store(y, idx + j, add_row_bias<T>(row_bias, v[j], (idx + j) % n));
    } else {
        for (int64_t i = idx; i < total; i++) {
            float sum = 0.0f;
            for (int s = 0; s < splits; s++) sum += partials[s * total + i];
            Elem<T>::store(y, i, add_row_bias<T>(row_bias, sum, i % n));
        }
    }
}

// Tile choice and the split of K over the grid: the host rules of nvq_splits.h, here bound to this kernel's constants.
static_assert(BK == splits::kQmmStep && BigTile::BM == splits::kQmmBigTile && BigTile::BN == splits::kQmmBigTile &&
              SmallTile::BM == splits::kQmmSmallTile && SmallTile::BN == splits::kQmmSmallTile, "nvq_splits.h describes these tiles");
inline splits::Product split_product(const ProductArgs &a) {
    return splits::Product{a.m, a.n, a.k, a.batch, a.row_exact != 0, a.exact_weights != 0};
}
inline bool small_tile_is_faster(const ProductArgs &a, int cus) { return splits::qmm_small_tile_is_faster(split_product(a), cus); }
// How many ways a single product splits K over the grid (1: no split), the steps of a split, the estimated duration.
inline int k_splits(const ProductArgs &a, int cus, int *steps_per_split = nullptr, double *estimate = nullptr) {
    const splits::Plan p = splits::qmm_plan(split_product(a), cus);
    if (steps_per_split != nullptr) *steps_per_split = (int)p.per_split;
    if (estimate != nullptr) *estimate = p.estimate_us;
    return p.splits;
}

template <typename T, int BITS, int FP4, class TL, bool EXACT = false>
int32_t run_tile(ProductArgs a, void *workspace, hipStream_t s) {
    using G = Geometry<BITS, TL>;
    static std::atomic<bool> configured[2] = {false, false};
    const bool batched = a.batch > 1;
    auto kernel = batched ? qmm_kernel<T, BITS, FP4, true, TL, EXACT> : qmm_kernel<T, BITS, FP4, false, TL, EXACT>;
    if (!configured[batched]) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, G::kLdsBytes));
        configured[batched] = true;
    }
    int per = 0;
    const int splits = workspace != nullptr ? k_splits(a, compute_units(), &per) : 1;
    if (splits > 1 && (int64_t)(splits - 1) * per >= a.k / BK)  // (a block of such a split would leave its partial sums unwritten)
        return fail(NVQ_BACKEND, "quantized_matmul: %d splits of %d steps leave one without a step of K = %lld", splits, per, (long long)a.k);
    a.k_splits = splits;
    a.k_split_steps = per;
    a.partials = splits > 1 ? static_cast<float *>(workspace) : nullptr;
    dim3 grid((unsigned)((a.n + TL::BN - 1) / TL::BN), (unsigned)((a.m + TL::BM - 1) / TL::BM), (unsigned)(batched ? a.batch : splits));
    hipLaunchKernelGGL(kernel, grid, dim3(TL::kThreads), G::kLdsBytes, s, a);
    NVQ_LAUNCH_CHECK("qmm");
    if (splits > 1) {
        const int64_t total = a.m * a.n;
        hipLaunchKernelGGL((qmm_reduce_kernel<T>), dim3((unsigned)((total / 4 + 256) / 256)), dim3(256), 0, s, a.partials, (T *)a.y, splits, total, a.row_bias, a.n);
        NVQ_LAUNCH_CHECK("qmm_reduce");
    }
    return NVQ_OK;
}

template <typename T, int BITS, int FP4>
int32_t run(const ProductArgs &a, void *workspace, hipStream_t s) {
    if constexpr (FP4 == kAffine)
        if (a.exact_weights) return run_tile<T, BITS, FP4, SmallTile, true>(a, workspace, s);  // (rows of few outputs: the small tile)
    return small_tile_is_faster(a, compute_units()) ? run_tile<T, BITS, FP4, SmallTile>(a, workspace, s)
                                                    : run_tile<T, BITS, FP4, BigTile>(a, workspace, s);
}

template <int BITS, int FP4>
int32_t run_dtype(const ProductArgs &a, void *workspace, hipStream_t s) {
    return a.dtype == NVQ_BF16 ? run<bf16_t, BITS, FP4>(a, workspace, s) : run<f16_t, BITS, FP4>(a, workspace, s);
}

}  // namespace qmm

// One per code width, each in its own translation unit.
int32_t launch_qmm_b2(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_b1(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_b3(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_b5(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_b4(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_b6(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_b8(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_fp4(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_fp8(const ProductArgs &a, void *workspace, hipStream_t s);
int32_t launch_qmm_nvfp4(const ProductArgs &a, void *workspace, hipStream_t s);

}  // namespace nvq
