// The grouped (sorted) gathered product of mixture-of-experts layers on the gfx950 matrix cores: the rows of
// x that belong to expert e, [offsets[e], offsets[e+1]), times that expert's weights, every weight decoded
// once per pass of 64 rows.  Counterpart of the reference's `gather_qmm_rhs`
// (crates/nuvec-kernels/src/metal/quantized.h:3301-3449, schedule at 2866-2906); values follow nuvec's CPU
// product (crates/nuvec-core/src/quantized.rs:679-719, crates/nuvec-core/src/kernels.rs:1091-1142) within the
// stated tolerance.
//
// Experts give the launch its parallelism, so a block does not split K: a block of four wavefronts owns
// 128 weight rows of one expert (32 per wavefront) and all wavefronts walk K together in windows of 128
// values.  Per window
//   * the block's 256 threads bring the x tile (up to 64 rows x 256 bytes, rows gathered through lhs) with
//     four coalesced 16-byte loads each, one window ahead, into one of two LDS stages (chunks XOR-swizzled
//     by row), from which every wavefront reads its matrix operands (one or two tiles of 32 rows): x leaves
//     the cache once per 128 weight rows;
//   * each wavefront fetches its own 32 weight rows of the window (16 BITS bytes per row) with coalesced
//     loads into registers several windows ahead and passes them through a private piece of LDS into the
//     operand layout, exactly as the few-row kernel does (qmf_kernel.h), and expands them in registers;
//   * scales (and biases) of the block's rows come from an LDS table filled once per block.
// A wavefront owns its 32 x 32 tiles of y outright, so nothing is reduced across wavefronts.
#pragma once

#include "qmf_kernel.h"

namespace nvq {
namespace qmg {

using namespace qmf;  // element operations, code expansion, static_for

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr int kRows = 32 * kWaves;            // weight rows per block
constexpr int kPassRows = 64;                 // rows of x per pass: two tiles of 32
constexpr int kXStageBytes = kPassRows * 256;  // one window of x: 64 rows x 128 values
constexpr int kTableMaxBytes = 48 * 1024;

template <int BITS>
struct Geometry {
    static constexpr int kChunks = 32 * BITS;              // 16-byte chunks of one wavefront's window
    static constexpr int kLoads = (kChunks + 63) / 64;     // loads per lane and window
    static constexpr int kDepth = 2;                       // windows of weights in flight per lane
    static constexpr int kRowBytes = 16 * BITS;            // of one row in a window
    static constexpr int kStageBytes = kChunks * 16;       // one window of one wavefront
    static constexpr int kFixedLdsBytes = 2 * kXStageBytes + kWaves * kStageBytes;
    static constexpr bool kPow2 = (BITS & (BITS - 1)) == 0;
    __host__ __device__ static constexpr int swizzle(int row) { return kPow2 ? (row / (BITS >= 16 ? 1 : 16 / BITS)) % BITS : 0; }
};

// GLU: the gated activation of the experts' MLPs as the epilogue (a.glu).  The weights then hold the gate and the up
// projection in alternating runs of 64 rows, so that a block's wavefronts 0 and 1 own 64 columns of the gate product
// and wavefronts 2 and 3 the same 64 columns of the up product, lane for lane: after a pass the latter leave their
// values (rounded as the product's output, the expert's bias added) in LDS, the former combine them with their own
// and write y [rows, N / 2].
template <typename T, int BITS, int FP4, bool GLU = false>
// Three blocks per compute unit (three wavefronts per SIMD): the registers are capped for that, and the LDS of a
// block (two x stages, the weight stages, the table) fits three times.
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3))) qmg_kernel(const ProductArgs a) {
    using G = Geometry<BITS>;
    constexpr int kDepth = G::kDepth, kLoads = G::kLoads;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    using S = std::conditional_t<FP4 != 0, uint8_t, T>;  // stored scale type
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
    // Work items are (pass of up to 64 rows of an expert, 128 weight rows): every item costs the same whatever the
    // experts' loads, and an expert with many rows has its passes side by side.  The passes are counted from the
    // offsets by every wavefront on its own (lane l owns a run of experts; a prefix sum over the lanes), and the block
    // finds the expert and the pass of its item there.  Blocks are handed to the 8 XCDs in turn, each with an L2 of
    // its own: block p takes item (p % 8) * ceil(items / 8) + p / 8 of the pass-major list, so that the blocks of a
    // pass, which read the same rows of x and neighbouring pieces of the same cache lines of weights, sit on one XCD.
    const int tiles = (N + kRows - 1) / kRows, experts = (int)a.experts;
    const int run = (experts + 63) >> 6, e_first = lane * run;
    // Rows [begin, end) of expert ei, as the offsets give them; offsets that do not ascend within the rows are the
    // caller's error and are clamped so that they cannot fault the device.
    auto rows_of = [&](int ei, int &begin, int &end) {
        const int rows_all = (int)a.batch;
        begin = min(max(a.offsets[ei], 0), rows_all);
        end = ei + 1 < experts ? min(max(a.offsets[ei + 1], begin), rows_all) : rows_all;
    };
    constexpr int kKept = 4;  // experts of a lane whose offsets stay in registers for the walk below (all of them up to 256 experts)
    int kept_begin[kKept], kept_end[kKept];
    int mine = 0;  // passes of this lane's experts
#pragma unroll
    for (int i = 0; i < kKept; i++) {
        const int ei = e_first + i;
        kept_begin[i] = kept_end[i] = 0;
        if (i < run && ei < experts) rows_of(ei, kept_begin[i], kept_end[i]);
        mine += (kept_end[i] - kept_begin[i] + kPassRows - 1) / kPassRows;
    }
    for (int i = kKept; i < run; i++) {
        const int ei = e_first + i;
        if (ei < experts) {
            int begin, end;
            rows_of(ei, begin, end);
            mine += (end - begin + kPassRows - 1) / kPassRows;
        }
    }
    int upto = mine;  // inclusive prefix over the lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int v = __shfl_up(upto, o);
        if (lane >= o) upto += v;
    }
    const int passes = __shfl(upto, 63);
    const int items = tiles * passes, per = (items + 7) >> 3;
    const int slot = (int)(blockIdx.x >> 3), item = (int)(blockIdx.x & 7) * per + slot;
    if (slot >= per || item >= items) return;  // the whole block: no barrier has been reached
    const int n0 = (item % tiles) * kRows, target = item / tiles;
    // the lane whose experts hold pass `target` walks them; every lane takes its answer
    const int owner = __builtin_ctzll(__ballot(upto > target));
    int found_e = 0, found_begin = 0, found_end = 0;
    if (lane == owner) {
        int before = upto - mine;
        bool found = false;
        auto look = [&](int ei, int begin, int end) {
            const int count = (end - begin + kPassRows - 1) / kPassRows;
            if (!found && target < before + count) {
                found = true;
                found_e = ei, found_begin = begin + (target - before) * kPassRows;
                found_end = found_begin + kPassRows < end ? found_begin + kPassRows : end;
            }
            if (!found) before += count;
        };
#pragma unroll
        for (int i = 0; i < kKept; i++) look(e_first + i, kept_begin[i], kept_end[i]);  // (an expert past the lane's run holds no pass)
        for (int i = kKept; i < run && !found; i++) {
            const int ei = e_first + i;
            if (ei >= experts) break;
            int begin, end;
            rows_of(ei, begin, end);
            look(ei, begin, end);
        }
    }
    const int e = __builtin_amdgcn_readfirstlane(__shfl(found_e, owner));
    const int row_begin = __builtin_amdgcn_readfirstlane(__shfl(found_begin, owner));
    const int row_end = __builtin_amdgcn_readfirstlane(__shfl(found_end, owner));
    if (row_begin >= row_end) return;  // the whole block: no barrier has been reached
    const int64_t wo = (int64_t)e * N * row_bytes, so = (int64_t)e * N * kgroups;
    const T *x = (const T *)a.x;
    T *y = (T *)a.y;

    const int steps = K >> 6;             // K is a multiple of 64 (checked on the host)
    const int windows = (steps + 1) >> 1;  // the last window may hold one step

    // Weight window loads of this wavefront: load j of a lane is chunk q = 64 j + lane, i.e. chunk q % BITS of
    // row q / BITS of the wavefront's 32 rows.  Chunks of the window's second step begin at BITS / 2 (a window
    // of one step exists only for even BITS; its lanes fetch the first step again).
    const unsigned char *wload[kLoads];
    int wstore[kLoads];
    bool second[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; j++) {
        const int q = 64 * j + lane, qc = q < G::kChunks ? q : G::kChunks - 1;
        const int row = qc / BITS, c = qc % BITS;
        const int n = n0 + 32 * wave + row < N ? n0 + 32 * wave + row : N - 1;  // tail rows are computed, not stored
        wload[j] = (const unsigned char *)a.w + wo + (int64_t)n * row_bytes + 16 * c;
        wstore[j] = row * G::kRowBytes + 16 * (c ^ G::swizzle(row));
        second[j] = 2 * c >= BITS;
    }
    // Every load of the K loop is issued on every path (a window past the end loads one 16-byte piece, the
    // same for all lanes), so that the waits can leave the younger windows' loads in flight.
    auto load_window = [&](int win, u32x4_t (&w)[kLoads]) {
        const bool real = win < windows, half = 2 * win + 1 >= steps;
#pragma unroll
        for (int j = 0; j < kLoads; j++) {
            const int off = win * 16 * BITS - ((half && second[j]) ? 8 * BITS : 0);
            const unsigned char *src = real ? wload[j] + off : (const unsigned char *)a.w;
            w[j] = *reinterpret_cast<const u32x4_a4_t *>(src);
        }
    };
    unsigned char *stage = lds + 2 * kXStageBytes + wave * G::kStageBytes;
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

    // The first windows of weights are requested before anything waits: they depend on nothing but the block's place.
    u32x4_t ring[kDepth][kLoads];  // weight windows in flight
    static_for<kDepth>([&](auto d_tag) {
        constexpr int d = decltype(d_tag)::value;
        load_window(d, ring[d]);
    });
    __builtin_amdgcn_sched_barrier(0);

    const float factor = FP4 == kNvfp4 && a.global_scale != nullptr ? ftz(a.global_scale[e] / (448.0f * 6.0f)) : 1.0f;  // (one per expert)
    // The scale (NVFP4: the two scales, one per 16 values) and bias of this lane's 32 values of a step.
    auto load_scales = [&](int step, float (&scale)[2], float &bias) {
        const int g = (step * 64 + 32 * h) >> gshift;
        const int at = (32 * wave + l32) * tstride + g * (int)sizeof(S);
        const S *sp = reinterpret_cast<const S *>(table_s + at), *bp = reinterpret_cast<const S *>(table_b + at);
        if constexpr (FP4 == kNvfp4) {
            scale[0] = nvfp4_scale(sp[0], factor);
            scale[1] = nvfp4_scale(sp[1], factor);
            bias = 0.0f;
        } else if constexpr (FP4) {
            scale[0] = scale[1] = ftz(e8m0_to_f32(*sp));
            bias = 0.0f;
        } else {
            scale[0] = scale[1] = Elem<T>::load(sp, 0);
            bias = Elem<T>::load(bp, 0);
        }
    };

    {
        // The scales (and biases) of rows n0 .. n0 + 127 are contiguous in memory.
        const int valid_rows = N - n0 < kRows ? N - n0 : kRows;
        fill_table<S, kThreads>(table_s, (const S *)a.scales + so + (int64_t)n0 * kgroups, valid_rows * kgroups, kgroups, tstride, tid);
        if constexpr (!FP4)
            fill_table<S, kThreads>(table_b, (const S *)a.biases + so + (int64_t)n0 * kgroups, valid_rows * kgroups, kgroups, tstride, tid);
    }

    // x tile loads: thread t brings chunks t + 256 i (i < 4) of a window's 1024 (chunk q: row q / 16, 16-byte
    // piece q % 16); piece c of row r is stored at position c ^ (r % 16).  The operand of piece kk of step t
    // for lane (row r = lane % 32, half h) of tile u is piece 8 t + 4 h + kk of row 32 u + r.
    const int xc = tid & 15;
    int xstore[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (tid >> 4) + 16 * i;
        xstore[i] = r * 256 + 16 * (xc ^ (r & 15));
    }
    int xread[2][4];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int kk = 0; kk < 4; kk++) xread[t][kk] = l32 * 256 + 16 * ((8 * t + 4 * h + kk) ^ (l32 & 15));

    for (int pass = row_begin; pass < row_end; pass += kPassRows) {
        const int rows = row_end - pass < kPassRows ? row_end - pass : kPassRows;
        const bool two = rows > 32;  // the pass has a second tile of rows
        // rows of x behind this thread's four chunks, gathered through lhs; a row past the pass reads the
        // start of x (its tile row is never stored)
        const T *xsrc[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int r = (tid >> 4) + 16 * i;
            int64_t g = pass + (r < rows ? r : 0);
            if (a.lhs != nullptr) g = min((int64_t)a.lhs[g], a.x_batches - 1);  // an index beyond x is the caller's error: clamped
            xsrc[i] = x + (r < rows ? g * K : 0) + 8 * xc;
        }
        auto load_x = [&](int win, u32x4_t (&xq)[4]) {
            // a window of one step has no second half: those chunks (pieces 8..15) fetch the first half again
            const int k0 = win < windows ? win * 128 - ((2 * win + 1 >= steps && xc >= 8) ? 64 : 0) : 0;
            // chunks 2 and 3 are rows 32..63: fetched only when the pass has a second tile (the loads are issued
            // either way, so that the waits see the same number of them: a tile-less one reads the start of x)
#pragma unroll
            for (int i = 0; i < 4; i++) xq[i] = *reinterpret_cast<const u32x4_t *>(i < 2 || two ? xsrc[i] + k0 : x);
        };
        auto store_x = [&](int win, const u32x4_t (&xq)[4]) {
            unsigned char *dst = lds + (win & 1) * kXStageBytes;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (i < 2 || two) *reinterpret_cast<u32x4_t *>(dst + xstore[i]) = xq[i];
        };

        floatx16_t acc[2];
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int el = 0; el < 16; el++) acc[u][el] = 0.0f;

        u32x4_t xq[2][4];                   // x chunks of the next two windows
        load_x(0, xq[0]);
        load_x(1, xq[1]);
        if (pass != row_begin) {  // (the first pass found its windows on the way already)
            static_for<kDepth>([&](auto d_tag) {
                constexpr int d = decltype(d_tag)::value;
                load_window(d, ring[d]);
            });
        }
        store_x(0, xq[0]);
        load_x(2, xq[0]);
        __syncthreads();  // window 0 of x is in LDS (first pass: the table too)

        for (int w0 = 0; w0 < windows; w0 += kDepth) {
            static_for<kDepth>([&](auto d_tag) {
                constexpr int d = decltype(d_tag)::value;
                const int win = w0 + d;
                // weights through LDS into the operand layout; the wavefront's LDS accesses execute in order
                asm volatile("" ::: "memory");
#pragma unroll
                for (int j = 0; j < kLoads; j++)
                    if (G::kChunks % 64 == 0 || 64 * j + lane < G::kChunks) *reinterpret_cast<u32x4_t *>(stage + wstore[j]) = ring[d][j];
                load_window(win + kDepth, ring[d]);  // the registers are free again: refill them
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");
                uint32_t codes[2][BITS];
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int p = 0; p < kPieces; p++) {
                        const unsigned char *src = stage + wread[t][p];
                        if constexpr (kPiece == 4) {
                            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(src);
                            codes[t][4 * p] = v.x, codes[t][4 * p + 1] = v.y, codes[t][4 * p + 2] = v.z, codes[t][4 * p + 3] = v.w;
                        } else if constexpr (kPiece == 2) {
                            const u32x2_t v = *reinterpret_cast<const u32x2_t *>(src);
                            codes[t][2 * p] = v.x, codes[t][2 * p + 1] = v.y;
                        } else {
                            codes[t][p] = *reinterpret_cast<const uint32_t *>(src);
                        }
                    }
                asm volatile("" ::: "memory");
                if (win < windows) {
                    // All x operands of a tile are requested before the first matrix instruction needs one (LDS
                    // answers in order), so the window pays the LDS latency once, not once per instruction.  A
                    // window of one step reads its absent second step too (stale but valid LDS) and skips its
                    // matrix instructions.
                    const unsigned char *xs = lds + (win & 1) * kXStageBytes;
                    const bool second_step = 2 * win + 1 < steps;
                    uint4 xf[2][4], wb[2][4];
#pragma unroll
                    for (int t = 0; t < 2; t++)
#pragma unroll
                        for (int kk = 0; kk < 4; kk++) xf[t][kk] = *reinterpret_cast<const uint4 *>(xs + xread[t][kk]);
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        float scale[2], bias;
                        load_scales(2 * win + (t == 0 || second_step ? t : 0), scale, bias);
                        static_for<4>([&](auto kk_tag) {
                            constexpr int kk = decltype(kk_tag)::value;
                            wb[t][kk] = expand_piece<T, BITS, FP4, kk>(codes[t], scale[kk >> 1], bias);
                        });
                    }
#pragma unroll
                    for (int t = 0; t < 2; t++)
                        if (t == 0 || second_step) {
#pragma unroll
                            for (int kk = 0; kk < 4; kk++) acc[0] = Ops<T>::mfma(xf[t][kk], wb[t][kk], acc[0]);
                        }
                    if (two) {
#pragma unroll
                        for (int t = 0; t < 2; t++)
#pragma unroll
                            for (int kk = 0; kk < 4; kk++) xf[t][kk] = *reinterpret_cast<const uint4 *>(xs + 32 * 256 + xread[t][kk]);
#pragma unroll
                        for (int t = 0; t < 2; t++)
                            if (t == 0 || second_step) {
#pragma unroll
                                for (int kk = 0; kk < 4; kk++) acc[1] = Ops<T>::mfma(xf[t][kk], wb[t][kk], acc[1]);
                            }
                    }
                }
                // the next window of x goes into the other stage (last read one window ago, before the previous
                // barrier); its registers then take the window after the next
                store_x(win + 1, xq[(d + 1) & 1]);
                load_x(win + 3, xq[(d + 1) & 1]);
                __syncthreads();
            });
        }

        // Accumulator element el of lane l is tile row 8 (el / 4) + 4 (l / 32) + el % 4 (a row of x), column l % 32.
        const int col = n0 + 32 * wave + l32;
        // A scattered product writes sorted row r where the caller wants it (its pair's place): lane l fetches the
        // place of the pass's row l (one load per wavefront) and the stores read it across lanes.
        uint32_t place = pass + lane;
        if (a.out_rows != nullptr) place = (uint32_t)min((int64_t)a.out_rows[pass + (lane < rows ? lane : 0)], a.batch - 1);
        if constexpr (GLU) {
            // (N is whole blocks here: checked on the host.)  The x stages are free: the loop ended with a barrier.
            float *exchange = reinterpret_cast<float *>(lds) + ((wave & 1) * 32) * 64 + lane;  // [wavefront pair][value][lane]
            const float bias = a.expert_bias != nullptr ? Elem<T>::load((const T *)a.expert_bias, (int64_t)e * N + col) : 0.0f;
            auto value = [&](int u, int el) {  // the product as its output holds it, then the separate rounded addition
                const float v = rounded<T>(acc[u][el]);
                return a.expert_bias != nullptr ? Elem<T>::add(v, bias) : v;
            };
            if (wave >= 2) {
#pragma unroll
                for (int u = 0; u < 2; u++)
#pragma unroll
                    for (int el = 0; el < 16; el++)
                        if (u == 0 || two) exchange[(16 * u + el) * 64] = value(u, el);
            }
            __syncthreads();
            if (wave < 2) {
                const int H = N >> 1, hcol = (n0 >> 1) + 32 * wave + l32;
#pragma unroll
                for (int u = 0; u < 2; u++)
#pragma unroll
                    for (int el = 0; el < 16; el++) {
                        const int m0 = 32 * u + 8 * (el >> 2) + (el & 3), m = m0 + 4 * h;
                        const uint32_t lo = __builtin_amdgcn_readlane(place, m0), hi = __builtin_amdgcn_readlane(place, m0 + 4);
                        if (m < rows) {
                            const float g = value(u, el), up = exchange[(16 * u + el) * 64];
                            const float out = a.glu == 1 + NVQ_GLU_SWIGLU       ? glu<T, NVQ_GLU_SWIGLU>(g, up, a.glu_alpha, a.glu_limit)
                                              : a.glu == 1 + NVQ_GLU_SWIGLU_OAI ? glu<T, NVQ_GLU_SWIGLU_OAI>(g, up, a.glu_alpha, a.glu_limit)
                                                                                : glu<T, NVQ_GLU_GEGLU>(g, up, a.glu_alpha, a.glu_limit);
                            Elem<T>::store(y, (int64_t)(h ? hi : lo) * H + hcol, out);
                        }
                    }
            }
            __syncthreads();  // the next pass stores x where the values were exchanged
            continue;
        }
        // The expert's bias (crates/nuvec-lm/src/model.rs:2139-2143): added to the product as its output holds it, a
        // separate rounded addition.
        const bool biased = a.expert_bias != nullptr;
        const float bias = biased && col < N ? Elem<T>::load((const T *)a.expert_bias, (int64_t)e * N + col) : 0.0f;
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int el = 0; el < 16; el++) {
                const int m0 = 32 * u + 8 * (el >> 2) + (el & 3), m = m0 + 4 * h;
                const uint32_t lo = __builtin_amdgcn_readlane(place, m0), hi = __builtin_amdgcn_readlane(place, m0 + 4);
                const float v = biased ? Elem<T>::add(rounded<T>(acc[u][el]), bias) : acc[u][el];
                if (m < rows && col < N) Elem<T>::store(y, (int64_t)(h ? hi : lo) * N + col, v);
            }
    }
}

// Bytes of the LDS table of scales (and biases) for the block's rows.
inline size_t table_bytes(const ProductArgs &a) { return qmf::table_bytes(a, kRows); }

template <typename T, int BITS, int FP4, bool GLU>
int32_t run_kernel(const ProductArgs &a, hipStream_t s) {
    using G = Geometry<BITS>;
    static std::atomic<bool> configured = false;
    auto kernel = qmg_kernel<T, BITS, FP4, GLU>;
    const size_t lds_bytes = G::kFixedLdsBytes + table_bytes(a);
    if (!configured) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        G::kFixedLdsBytes + kTableMaxBytes));
        configured = true;
    }
    // every expert with rows adds at most one partial pass: blocks for that many items, the rest leave at once
    const int64_t passes = a.batch / kPassRows + (a.experts < a.batch ? a.experts : a.batch);
    const int64_t items = (a.n + kRows - 1) / kRows * passes;
    const dim3 grid((unsigned)((items + 7) / 8 * 8));
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds_bytes, s, a);
    NVQ_LAUNCH_CHECK("qmg");
    return NVQ_OK;
}

template <typename T, int BITS, int FP4>
int32_t run(const ProductArgs &a, hipStream_t s) {
    if (a.glu == 0) return run_kernel<T, BITS, FP4, false>(a, s);
    if (a.n % kRows != 0) return fail(NVQ_UNSUPPORTED, "gather_qmm: the gated epilogue takes gate and up rows in whole runs of 64");
    return run_kernel<T, BITS, FP4, true>(a, s);
}

template <int BITS, int FP4>
int32_t run_dtype(const ProductArgs &a, hipStream_t s) {
    return a.dtype == NVQ_BF16 ? run<bf16_t, BITS, FP4>(a, s) : run<f16_t, BITS, FP4>(a, s);
}

}  // namespace qmg
}  // namespace nvq
