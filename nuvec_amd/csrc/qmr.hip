// Batched decode: passes of up to 64 rows of x (16 or 32 where x has no more) times 4- or 8-bit affine weights stored [N, K],
// bf16 / f16, on the 16x16x32 matrix instruction with every weight fetched and dequantized once per pass.  The regime
// between the few-row kernels (up to 16 rows a pass: more rows are passes that read the weights again) and the tiled
// kernel (tiles of 128 or 256 rows of x, whose step costs the same however few rows it multiplies).  The reference routes
// these row counts to its tiled kernel (crates/nuvec-core/src/gpu.rs:6975-7060,
// crates/nuvec-kernels/src/metal/quantized.h:1358-1485); values follow nuvec's CPU product
// (crates/nuvec-core/src/kernels.rs:1091-1142) as the tiled kernel's do: a weight is one rounding of
// fma(code, scale, bias) to the element type.
//
// A block of four wavefronts owns 16 WT weight rows (64, or 128 where the weight has more rows than one round of 64-row
// blocks covers: x is then read half as often per weight) and all rows of the pass; its wavefronts split K: wavefront v takes
// the chunks of 512 values v, v + 4, ...  Nothing is shared between them until their partial tiles are added, so the
// loop has no block barrier.  A wavefront walks its chunks in windows of 128 values:
//   * weights: lane (row n = lane % 16, quarter q = lane / 16) loads the 32 codes [32 q, 32 q + 32) of the window of its
//     row of each of the WT tiles (BITS dwords: a wavefront's load is 16 runs of 16 BITS bytes), two windows ahead,
//     straight into registers; matrix instruction s of a window takes codes [8 s, 8 s + 8) of every quarter;
//   * scales and biases: a lane's 32 codes lie in one group.  The scales and biases of a chunk's groups of the block's
//     weight rows are a table in the wavefront's own LDS (a lane brings a weight row's 512 / GROUP values with one load
//     for the scales and one for the biases, a chunk ahead), and a lane reads its 16-bit pair per tile and window there.
//     Fetched per lane and window from memory they were 8 of a window's 28 requests, each of 64 two-byte pieces
//     (W[14336,4096] at 64 rows 24.0 -> 20.5 us, W[151936,4096] 209 -> 156); passes of 64 rows on 128-row blocks of groups of
//     32, whose table does not fit beside x, still fetch them so;
//   * x: the window of the pass's rows (16 XT rows of 256 bytes) is loaded coalesced (a load is four whole rows) three
//     windows ahead, written to the wavefront's own LDS a window before its use (rows 272 bytes apart: the 16-byte
//     operand reads of sixteen rows fall on all 64 banks) and read from there in the instruction's operand layout;
//   * a window's XT x WT accumulators run over all of the wavefront's K: each dequantized weight operand feeds XT matrix
//     instructions, each x operand WT; the operands of a step are expanded under the matrix instructions of the step
//     before it.
// Every block reads all of x (from the L2): 2 x 16 XT K bytes against the 8 WT K bytes of its weights; a window takes
// the time of its requests, not of its arithmetic (measured: 20 us at K = 4096 for any N up to 16384, one round of
// blocks).
#include "qmv_common.h"

namespace nvq {
namespace {

constexpr int kQmrWaves = 4;                       // wavefronts of a block: the splits of K
constexpr int kQmrWindow = 128;                    // values of K per window
constexpr int kQmrChunk = 4 * kQmrWindow;          // values of K per turn of the loop
constexpr int kQmrRowBytes = 2 * kQmrWindow + 16;  // a row of a window of x in LDS

template <int XT> constexpr int qmr_buffer_bytes() { return 16 * XT * kQmrRowBytes; }
// A wavefront's table of the scales and biases of a chunk (its weight rows' groups of 512 values, 16 bits each), where
// it fits beside the buffers of x; 0: the lanes fetch them from memory window by window.
template <int XT, int WT, int GROUP> constexpr int qmr_table_bytes() {
    constexpr int bytes = 2 * 16 * WT * (kQmrChunk / GROUP) * 2;
    return 2 * qmr_buffer_bytes<XT>() + bytes <= 160 * 1024 / kQmrWaves ? bytes : 0;  // (all but passes of 64 rows on 128 weight rows in groups of 32)
}
template <int XT, int WT, int GROUP> constexpr int qmr_wave_bytes() { return 2 * qmr_buffer_bytes<XT>() + qmr_table_bytes<XT, WT, GROUP>(); }
template <int XT, int WT, int GROUP> constexpr size_t qmr_lds_bytes() { return (size_t)kQmrWaves * qmr_wave_bytes<XT, WT, GROUP>(); }

// The table of scales is written in dwords and read 16 bits at a time: types that may alias, so that the reads stay
// behind the writes.
typedef uint32_t __attribute__((may_alias)) qmr_word_t;
typedef uint16_t __attribute__((may_alias)) qmr_half_t;

// BITS dwords from p (whole dwords; the widest loads the alignment of every window allows).
template <int BITS>
__device__ __forceinline__ void qmr_load_codes(const uint32_t *p, uint32_t (&out)[BITS]) {
    if constexpr (BITS % 4 == 0) {
#pragma unroll
        for (int i = 0; i < BITS / 4; i++) {
            const uint4 v = *reinterpret_cast<const uint4 *>(p + 4 * i);
            out[4 * i] = v.x, out[4 * i + 1] = v.y, out[4 * i + 2] = v.z, out[4 * i + 3] = v.w;
        }
    } else if constexpr (BITS % 2 == 0) {
#pragma unroll
        for (int i = 0; i < BITS / 2; i++) {
            const uint2 v = *reinterpret_cast<const uint2 *>(p + 2 * i);
            out[2 * i] = v.x, out[2 * i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < BITS; i++) out[i] = p[i];
    }
}

template <typename T, int BITS, int GROUP, int XT, int WT, bool EXACT>
__global__ void __launch_bounds__(64 * kQmrWaves) qmr_kernel(const ProductArgs a) {
    constexpr int kRows = 16 * XT, kCols = 16 * WT;
    constexpr int kXLoads = 4 * XT;                   // loads of a window of x per lane: four rows of 256 bytes each
    constexpr int kBuf = qmr_buffer_bytes<XT>();
    constexpr int kWaveBytes = qmr_wave_bytes<XT, WT, GROUP>();
    constexpr int kTabRow = kQmrChunk / GROUP * 2;    // bytes of a weight row's scales (or biases) of a chunk
    constexpr bool kTable = qmr_table_bytes<XT, WT, GROUP>() != 0;
    constexpr int kOutStride = kCols + 4;             // floats between two rows of a wavefront's partial tile
    // Eight tiles of weight rows fill the registers: their weights are requested one window ahead instead of two and
    // expanded in the step that multiplies them.
    constexpr int kWeightsAhead = WT >= 8 || BITS >= 8 ? 1 : 2;  // (8-bit codes: a window of them is twice the registers)
    constexpr int kXSets = WT >= 8 ? 1 : 2;           // windows of x on their way in registers
    constexpr bool kAhead = WT < 8;
    static_assert(kRows * kOutStride * 4 <= 2 * kBuf, "the partial tile reuses the wavefront's x buffers");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, q = lane >> 4;
    const int M = (int)a.m, N = (int)a.n, K = (int)a.k;
    const int kwords = K / 32 * BITS, kgroups = K / GROUP;
    const int m0 = blockIdx.y * kRows, n0 = blockIdx.x * kCols;
    const int chunks = K / kQmrChunk;
    const int turns = chunks > wave ? (chunks - wave + kQmrWaves - 1) / kQmrWaves : 0;  // chunks of this wavefront
    unsigned char *mine = lds + wave * kWaveBytes;
    unsigned char *table = mine + 2 * kBuf;  // [scales, biases][weight row of the block][group of the chunk]

    // k of window `widx` of this wavefront; windows past its last one (and a wavefront without chunks) fetch a window
    // that exists, and nothing of it is used: no test around the loads.
    auto k_of = [&](int widx) {
        int chunk = wave + kQmrWaves * (widx >> 2);
        chunk = chunk < chunks ? chunk : chunks - 1;
        return chunk * kQmrChunk + (widx & 3) * kQmrWindow;
    };

    // x: load j of a window brings rows 4 j .. 4 j + 3 of the pass, lane L the piece L % 16 of row 4 j + L / 16.
    const T *xbase = (const T *)a.x + (int64_t)m0 * K + 8 * (lane & 15);
    const int xrows = M - m0;  // rows of this pass that exist; the others read the last one and are never stored
    const int xrow = lane >> 4;
    const int xdst = (lane >> 4) * kQmrRowBytes + (lane & 15) * 16;   // + 4 j rows
    const int xsrc = nl * kQmrRowBytes + 64 * q;                      // + 16 t rows + 16 s
    // w, scales, biases: this lane's row of each tile (rows past N read row N - 1)
    const uint32_t *wbase = (const uint32_t *)a.w;
    const uint16_t *sbase = (const uint16_t *)a.scales, *bbase = (const uint16_t *)a.biases;
    const int nrow = n0 + nl, wlane = q * BITS;  // (the tiles' offsets are computed at the loads: sixteen registers fewer)

    qmf::u32x4_t xg[kXSets][kXLoads];  // (a native vector: arrays of it stay in registers)
    uint32_t wq[4][WT][BITS], sq[4][WT], bq[4][WT];
    auto load_x = [&](int widx, auto buffer_tag, auto first_tag, auto count_tag) __attribute__((always_inline)) {
        constexpr int set = kXSets == 2 ? decltype(buffer_tag)::value : 0, first = decltype(first_tag)::value, count = decltype(count_tag)::value;
        const T *src = xbase + k_of(widx);
#pragma unroll
        for (int j = first; j < first + count; j++) {
            const int r = 4 * j + xrow;
            xg[set][j] = *reinterpret_cast<const qmf::u32x4_t *>(src + (r < xrows ? r : xrows - 1) * K);
        }
    };
    auto store_x = [&](auto buffer_tag, auto first_tag, auto count_tag) __attribute__((always_inline)) {
        constexpr int buffer = decltype(buffer_tag)::value, first = decltype(first_tag)::value, count = decltype(count_tag)::value;
        constexpr int set = kXSets == 2 ? buffer : 0;
        unsigned char *dst = mine + buffer * kBuf + xdst;
#pragma unroll
        for (int j = first; j < first + count; j++) {
            // x on its way lives in the accumulation registers (loads and LDS writes take them), which the loop leaves free
            asm("" : "+a"(xg[set][j]));
            *reinterpret_cast<qmf::u32x4_t *>(dst + 4 * j * kQmrRowBytes) = xg[set][j];
        }
    };
    // The codes of a window and, per tile, the scale and bias of the group this lane's 32 codes lie in: from the
    // wavefront's table of the chunk, or from memory.
    auto load_codes = [&](int widx, auto set_tag) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value;
        const uint32_t *src = wbase + k_of(widx) / 32 * BITS;
#pragma unroll
        for (int wt = 0; wt < WT; wt++) {
            const int n = nrow + 16 * wt < N ? nrow + 16 * wt : N - 1;
            qmr_load_codes<BITS>(src + n * kwords + wlane, wq[set][wt]);
        }
    };
    auto load_groups = [&](int widx, auto set_tag) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value;
        const unsigned char *src = table + nl * kTabRow + ((widx & 3) * kQmrWindow + 32 * q) / GROUP * 2;
#pragma unroll
        for (int wt = 0; wt < WT; wt++) {
            sq[set][wt] = *reinterpret_cast<const qmr_half_t *>(src + 16 * wt * kTabRow);
            bq[set][wt] = *reinterpret_cast<const qmr_half_t *>(src + (kCols + 16 * wt) * kTabRow);
        }
    };
    auto load_w = [&](int widx, auto set_tag) __attribute__((always_inline)) {
        if constexpr (kTable) {
            load_codes(widx, set_tag);
            load_groups(widx, set_tag);
        } else {  // (one walk over the tiles: a row's offset serves its codes, scale and bias)
            constexpr int set = decltype(set_tag)::value;
            const int k0 = k_of(widx);
            const uint32_t *src = wbase + k0 / 32 * BITS;
            const int g = (k0 + 32 * q) / GROUP;
#pragma unroll
            for (int wt = 0; wt < WT; wt++) {
                const int n = nrow + 16 * wt < N ? nrow + 16 * wt : N - 1;
                qmr_load_codes<BITS>(src + n * kwords + wlane, wq[set][wt]);
                sq[set][wt] = sbase[n * kgroups + g];
                bq[set][wt] = bbase[n * kgroups + g];
            }
        }
    };
    // The table of a chunk: lane L brings the scales and the biases of the chunk's groups of weight rows L, L + 64, ...
    // of the block (kTabRow bytes each), a chunk ahead; they go to LDS once the last window of the chunk before has
    // read its own (the wavefront's LDS accesses execute in order: no barrier).
    constexpr int kTabRows = kCols / 64, kTabWords = kTabRow / 4;
    uint32_t tq[kTable ? 2 * kTabRows * kTabWords : 1];
    auto table_load = [&](int turn) __attribute__((always_inline)) {
        if constexpr (kTable) {
            int chunk = wave + kQmrWaves * turn;
            chunk = chunk < chunks ? chunk : chunks - 1;
#pragma unroll
            for (int r = 0; r < kTabRows; r++) {
                const int n = n0 + lane + 64 * r < N ? n0 + lane + 64 * r : N - 1;
                const int at = n * kgroups + chunk * (kQmrChunk / GROUP);
                qmr_load_codes<kTabWords>(reinterpret_cast<const uint32_t *>(sbase + at), reinterpret_cast<uint32_t (&)[kTabWords]>(tq[(2 * r) * kTabWords]));
                qmr_load_codes<kTabWords>(reinterpret_cast<const uint32_t *>(bbase + at), reinterpret_cast<uint32_t (&)[kTabWords]>(tq[(2 * r + 1) * kTabWords]));
            }
        }
    };
    auto table_store = [&]() __attribute__((always_inline)) {
        if constexpr (kTable) {
#pragma unroll
            for (int r = 0; r < kTabRows; r++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    qmr_word_t *dst = reinterpret_cast<qmr_word_t *>(table + (h * kCols + lane + 64 * r) * kTabRow);
#pragma unroll
                    for (int i = 0; i < kTabWords; i++) dst[i] = tq[(2 * r + h) * kTabWords + i];
                }
        }
    };

    floatx4_t acc[XT][WT];
#pragma unroll
    for (int t = 0; t < XT; t++)
#pragma unroll
        for (int wt = 0; wt < WT; wt++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[t][wt][e] = 0.0f;

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using IAll = std::integral_constant<int, kXLoads>;
    using IPart = std::integral_constant<int, XT>;  // a quarter of a window's loads

    // Prologue: x of window 0 to LDS; x of windows 1 and 2 and the weights of windows 0 and 1 on their way.  Every load is
    // requested two windows before its use: requests return in order, so the shortest lead is everyone's.
    table_load(0);
    load_x(0, I0{}, I0{}, IAll{});
    if constexpr (kTable) load_codes(0, I0{}); else load_w(0, I0{});
    if constexpr (kXSets == 2) load_x(1, I1{}, I0{}, IAll{});
    if constexpr (kWeightsAhead == 2) {
        if constexpr (kTable) load_codes(1, I1{}); else load_w(1, I1{});
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kTable) {
        table_store();
        load_groups(0, I0{});
        if constexpr (kWeightsAhead == 2) load_groups(1, I1{});
    }
    store_x(I0{}, I0{}, IAll{});
    load_x(kXSets, I0{}, I0{}, IAll{});
    __builtin_amdgcn_sched_barrier(0);

    // The weight operands of a step are expanded during the matrix instructions of the step before it (they run on
    // their own pipe): set s % 2 of `wo` holds step s of a window.
    uint4 wo[kAhead ? 2 : 1][WT];
    float sc[WT], bi[WT];
    auto expand = [&](auto j_tag, auto s_tag, auto wt_tag) __attribute__((always_inline)) {
        constexpr int j = decltype(j_tag)::value, s = decltype(s_tag)::value, wt = decltype(wt_tag)::value;
        if constexpr (s == 0) sc[wt] = Pair<T>::lo(sq[j][wt]), bi[wt] = Pair<T>::lo(bq[j][wt]);  // (the window's last expansion is behind)
        wo[kAhead ? s & 1 : 0][wt] = qmf::expand_piece<T, BITS, qmf::kAffine, s, EXACT>(wq[j][wt], sc[wt], bi[wt]);
    };
    if constexpr (kAhead) qmf::static_for<WT>([&](auto wt_tag) { expand(I0{}, I0{}, wt_tag); });

#pragma unroll 1
    for (int turn = 0; turn < turns; turn++) {
        qmf::static_for<4>([&](auto j_tag) {
            constexpr int j = decltype(j_tag)::value;
            const int widx = 4 * turn + j;
            const unsigned char *src = mine + (j & 1) * kBuf + xsrc;
            qmf::static_for<4>([&](auto s_tag) {
                constexpr int s = decltype(s_tag)::value;
                using First = std::integral_constant<int, s * XT>;
                // a quarter of the next window of x goes to LDS and its registers take the window two after that one
                using Next = std::integral_constant<int, (j + 1) & 1>;
                store_x(Next{}, First{}, IPart{});
                load_x(widx + 1 + kXSets, Next{}, First{}, IPart{});
                if constexpr (s == 0) {
                    // (the first window ahead that lies in the next chunk finds that chunk's table)
                    if constexpr (j == 4 - kWeightsAhead) table_store();
                    load_w(widx + kWeightsAhead, std::integral_constant<int, (j + kWeightsAhead) & 3>{});
                    if constexpr (j == 0) table_load(turn + 1);
                }
                __builtin_amdgcn_sched_barrier(0);  // (the requests keep this order: the waits count them)
                qmf::u32x4_t xo[XT];
#pragma unroll
                for (int t = 0; t < XT; t++) xo[t] = *reinterpret_cast<const qmf::u32x4_t *>(src + 16 * t * kQmrRowBytes + 16 * s);
                using NextJ = std::integral_constant<int, s == 3 ? (j + 1) & 3 : j>;
                using NextS = std::integral_constant<int, (s + 1) & 3>;
                qmf::static_for<WT>([&](auto wt_tag) {
                    constexpr int wt = decltype(wt_tag)::value;
                    if constexpr (!kAhead) expand(j_tag, s_tag, wt_tag);
#pragma unroll
                    for (int t = 0; t < XT; t++) acc[t][wt] = Mfma16<T>::run(__builtin_bit_cast(uint4, xo[t]), wo[kAhead ? s & 1 : 0][wt], acc[t][wt]);
                    if constexpr (kAhead) expand(NextJ{}, NextS{}, wt_tag);
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    }

    // The wavefronts' partial tiles, added in a fixed order.  Accumulator element e of lane (n, q) is row 4 q + e of its
    // tile of x rows and column n of its tile of weight rows.  A wavefront writes into its own buffers, after its own
    // reads of them (its LDS accesses execute in order) and once its last requests for x, which nothing uses, have left
    // its registers.
    float *part = reinterpret_cast<float *>(mine);
#pragma unroll
    for (int t = 0; t < XT; t++)
#pragma unroll
        for (int wt = 0; wt < WT; wt++)
#pragma unroll
            for (int e = 0; e < 4; e++) part[(16 * t + 4 * q + e) * kOutStride + 16 * wt + nl] = acc[t][wt][e];
    __syncthreads();
    T *y = (T *)a.y;
    constexpr int kItems = kRows * kCols / 8;  // eight neighbouring columns of a row each
    const bool whole = N % 8 == 0;
    for (int item = tid; item < kItems; item += 64 * kQmrWaves) {
        const int r = item / (kCols / 8), c = 8 * (item % (kCols / 8));
        const int row = m0 + r, col = n0 + c;
        if (row >= M || col >= N) continue;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kQmrWaves; wv++) {
            const floatx4_t *p = reinterpret_cast<const floatx4_t *>(lds + wv * kWaveBytes + (r * kOutStride + c) * 4);
            const floatx4_t lo = p[0], hi = p[1];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] += lo[e], v[4 + e] += hi[e];
        }
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = add_row_bias<T>(a.row_bias, v[e], col + e < N ? col + e : col);
        T *dst = y + (int64_t)row * N + col;
        if (whole) {
            uint4 o;
            o.x = qmf::Ops<T>::pack(v[0], v[1]), o.y = qmf::Ops<T>::pack(v[2], v[3]);
            o.z = qmf::Ops<T>::pack(v[4], v[5]), o.w = qmf::Ops<T>::pack(v[6], v[7]);
            *reinterpret_cast<uint4 *>(dst) = o;
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (col + e < N) Elem<T>::store(dst, e, v[e]);
        }
    }
}

template <typename T, int BITS, int GROUP, int XT, int WT, bool EXACT>
int32_t run_sized(const ProductArgs &a, hipStream_t s) {
    const dim3 grid((unsigned)((a.n + 16 * WT - 1) / (16 * WT)), (unsigned)((a.m + 16 * XT - 1) / (16 * XT)));
    auto kernel = qmr_kernel<T, BITS, GROUP, XT, WT, EXACT>;
    constexpr size_t lds_bytes = qmr_lds_bytes<XT, WT, GROUP>();
    static std::atomic<bool> configured{false};
    if (lds_bytes > 64 * 1024 && !configured.load()) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        configured.store(true);
    }
    hipLaunchKernelGGL(kernel, grid, dim3(64 * kQmrWaves), lds_bytes, s, a);
    NVQ_LAUNCH_CHECK("qmr");
    return NVQ_OK;
}

template <typename T, int BITS, int GROUP>
int32_t run_shape(const ProductArgs &a, hipStream_t s, bool tall) {
    // Up to 16 and up to 32 rows of x: passes of 16 and of 32 rows, which read a quarter and half as much of x per weight.
    if constexpr (BITS == 4) {
        if (a.m <= 16) return tall ? run_sized<T, BITS, GROUP, 1, 8, false>(a, s) : run_sized<T, BITS, GROUP, 1, 4, false>(a, s);
        if (a.m <= 32) return tall ? run_sized<T, BITS, GROUP, 2, 8, false>(a, s) : run_sized<T, BITS, GROUP, 2, 4, false>(a, s);
        return tall ? run_sized<T, BITS, GROUP, 4, 8, false>(a, s) : run_sized<T, BITS, GROUP, 4, 4, false>(a, s);
    } else {  // (8-bit codes: blocks of 64 weight rows only, the registers hold no more)
        if (a.m <= 16) return run_sized<T, BITS, GROUP, 1, 4, false>(a, s);
        if (a.m <= 32) return run_sized<T, BITS, GROUP, 2, 4, false>(a, s);
        return run_sized<T, BITS, GROUP, 4, 4, false>(a, s);
    }
}

template <typename T, int BITS>
int32_t run_group(const ProductArgs &a, hipStream_t s) {
    // More weight rows than one round of 64-row blocks covers: blocks of 128 rows, which read x half as often per weight
    // (us, 64 rows of x: W[28672,4096] 47.9 -> 43.3, W[32768,4096] 50.8 -> 42.5, W[65536,4096] 98.5 -> 88.7, W[28672,8192] 87.3 ->
    // 79.4; a single round of them is slower, W[14336,4096] 25.2 -> 40.4).
    const bool tall = a.n > 64 * (int64_t)compute_units();
    switch (a.group) {
    case 32: return run_shape<T, BITS, 32>(a, s, tall);
    case 64: return run_shape<T, BITS, 64>(a, s, tall);
    default: return run_shape<T, BITS, 128>(a, s, tall);
    }
}

}  // namespace

// Whether the kernel takes the product (the routes decide by its shape whether it should): a single product of bf16 / f16
// rows and 4- or 8-bit affine codes whose weights take one rounding, K in chunks of 512, every operand 16-byte aligned,
// offsets within 32 bits.
bool qmr_supported(const ProductArgs &a) {
    if (a.dtype == NVQ_F32 || a.mode != NVQ_AFFINE || (a.bits != 4 && a.bits != 8) || a.row_exact || a.exact_weights) return false;
    if (a.group != 32 && a.group != 64 && a.group != 128) return false;
    if (a.batch != 1 || a.batch_ndim != 0 || a.rhs != nullptr || a.lhs != nullptr || a.offsets != nullptr || a.glu != 0) return false;
    if (a.k < kQmrChunk || a.k % kQmrChunk != 0 || a.k > (1 << 24) || a.m < 1 || (a.m + 15) / 16 > 65535) return false;
    if (a.n * (a.k / 32 * a.bits) >= (1LL << 31)) return false;
    return ((uintptr_t)a.scales | (uintptr_t)a.biases | (uintptr_t)a.w | (uintptr_t)a.x | (uintptr_t)a.y) % 16 == 0;
}

int32_t launch_qmr(const ProductArgs &a, hipStream_t s) {
    if (!qmr_supported(a)) return fail(NVQ_UNSUPPORTED, "quantized_matmul: the batched-decode kernel does not take this product");
    if (a.bits == 8) return a.dtype == NVQ_BF16 ? run_group<bf16_t, 8>(a, s) : run_group<f16_t, 8>(a, s);
    return a.dtype == NVQ_BF16 ? run_group<bf16_t, 4>(a, s) : run_group<f16_t, 4>(a, s);
}


}  // namespace nvq
