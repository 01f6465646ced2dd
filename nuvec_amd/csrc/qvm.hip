// Products with the weights stored [K, N] (transpose = false): y[m, n] = sum_k x[m, k] * dequantize(w[k, n]),
// the reference's `qvm` / `qmm_n` routes (crates/nuvec-core/src/gpu.rs:6934-7168; values as
// crates/nuvec-core/src/kernels.rs:1091-1142 within the stated tolerance).  Every mode, width and element type.
//
// Weight rows run along N here, so the reduction walks rows: a lane owns 32 consecutive outputs (the BITS
// dwords of its codes in every row, one quantization group - two for NVFP4 - per row) and a wavefront 2048
// of them; the wavefront's loads of a row are one contiguous piece.  Per row a lane loads its codes and
// its scale and bias, takes x[m, k] (the same for all lanes) and accumulates x*scale*code and x*bias in
// float32, the next row's loads in flight.  K is split over the grid so that small products still fill
// the chip: each split writes float32 partial sums to the caller's workspace and a second kernel adds them
// in split order (deterministic), rounding once.
#include "nvq_device.h"
#include "nvq_internal.h"
#include "qmf_kernel.h"

namespace nvq {

bool qvm_takes_tiled(const ProductArgs &a);

namespace {

template <int BITS>
__device__ __forceinline__ void load_words(const uint32_t *p, uint32_t (&d)[BITS]) {
    if constexpr (BITS == 4) {
        const uint4 q = *reinterpret_cast<const uint4 *>(p);
        d[0] = q.x; d[1] = q.y; d[2] = q.z; d[3] = q.w;
    } else if constexpr (BITS == 8) {
        const uint4 q0 = reinterpret_cast<const uint4 *>(p)[0], q1 = reinterpret_cast<const uint4 *>(p)[1];
        d[0] = q0.x; d[1] = q0.y; d[2] = q0.z; d[3] = q0.w;
        d[4] = q1.x; d[5] = q1.y; d[6] = q1.z; d[7] = q1.w;
    } else if constexpr (BITS == 2) {
        const uint2 q = *reinterpret_cast<const uint2 *>(p);
        d[0] = q.x; d[1] = q.y;
    } else {
#pragma unroll
        for (int i = 0; i < BITS; i++) d[i] = p[i];
    }
}

// Code `i` (0..31) of the lane's BITS dwords: value i sits at bit i*BITS of the stream (kernels.rs:749-756).
template <int BITS>
__device__ __forceinline__ uint32_t code_at(const uint32_t (&d)[BITS], int i) {
    constexpr uint32_t mask = (1u << BITS) - 1u;
    const int bit = i * BITS, word = bit >> 5, sh = bit & 31;
    uint32_t v = d[word] >> sh;
    if (sh + BITS > 32) v |= d[word + 1] << (32 - sh);
    return v & mask;
}

struct Offsets { int64_t x, w, s, y; };

// Element offsets of batch `z` for x, w (packed dwords), scales/biases and y (in units of M*N).
__device__ __forceinline__ Offsets batch_offsets(const ProductArgs &a, int64_t z) {
    Offsets o{0, 0, 0, z};
    if (a.rhs != nullptr) {  // gathered pairs; an index outside its operand is the caller's error and is clamped
        const int64_t l = min((int64_t)a.lhs[z], a.x_batches - 1), r = min((int64_t)a.rhs[z], a.experts - 1);
        o.x = l * a.m * a.k;
        o.w = r * a.k * (a.n * a.bits / 32);
        o.s = r * a.k * (a.n / a.group);
        return o;
    }
    if (a.batch_ndim == 0) return o;
    int64_t rest = z;
#pragma unroll
    for (int d = NVQ_MAX_BATCH_DIMS - 1; d >= 0; d--) {
        if (d < a.batch_ndim) {
            const int64_t i = rest % a.batch_shape[d];
            rest /= a.batch_shape[d];
            o.x += i * a.x_strides[d];
            o.w += i * a.w_strides[d];
            o.s += i * a.s_strides[d];
        }
    }
    return o;
}

// MODE: NVQ_AFFINE, NVQ_MXFP4, NVQ_MXFP8 or NVQ_NVFP4.  grid = (ceil(N / 2048), splits, batch * passes of RM rows).
// A block's kQvmWaves wavefronts own the same 2048 columns and consecutive pieces of the split's rows of w; their sums
// meet in LDS in wavefront order, so that the grid's splits (and the reduction kernel's serial additions) stay few
// while enough wavefronts stream the weights.
constexpr int kQvmWaves = 8;
template <typename T, int BITS, int MODE, int RM, bool EXACT = false>
__global__ void __launch_bounds__(64 * kQvmWaves) qvm_kernel(const ProductArgs a, int splits, float *partial) {
    constexpr bool kAffine = MODE == NVQ_AFFINE;
    constexpr int kHalves = MODE == NVQ_NVFP4 ? 2 : 1;  // groups per lane
    __shared__ float sums[kQvmWaves - 1][32][64];  // [wavefront - 1][column of the lane][lane]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = kAffine ? (a.group == 32 ? 5 : a.group == 64 ? 6 : 7) : (MODE == NVQ_NVFP4 ? 4 : 5);
    const int passes = (M + RM - 1) / RM;
    const int bz = blockIdx.z / passes, m0 = (blockIdx.z % passes) * RM;
    const int n0 = (blockIdx.x * 64 + lane) * 32;
    const bool live = n0 < N;  // a lane's 32 outputs are all there or all absent, but for NVFP4's N % 32 == 16:
    const bool whole = MODE != NVQ_NVFP4 || n0 + 32 <= N;  // the last lane then owns one group of 16
    const int nc = live ? n0 : 0;
    const int row_dwords = (N * BITS) >> 5, ngroups = N >> gshift;
    const Offsets o = batch_offsets(a, bz);
    const T *x = (const T *)a.x + o.x;
    const uint32_t *w = (const uint32_t *)a.w + o.w + (nc >> 5) * BITS;
    const int64_t s_at = o.s + (nc >> gshift);
    const int per = (K + splits - 1) / splits;
    const int s_begin = blockIdx.y * per, s_end = s_begin + per < K ? s_begin + per : K;  // the split's rows of w
    const int sub = (s_end - s_begin + kQvmWaves - 1) / kQvmWaves;                          // ... and the wavefront's
    const int k_begin = s_begin + wave * sub < s_end ? s_begin + wave * sub : s_end, k_end = k_begin + sub < s_end ? k_begin + sub : s_end;
    constexpr bool exact = kAffine && EXACT;  // the weights as the CPU holds them (rows of few outputs)

    float acc[RM][32], accb[RM];
#pragma unroll
    for (int i = 0; i < RM; i++) {
        accb[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; j++) acc[i][j] = 0.0f;
    }

    struct Row {
        uint32_t d[BITS];
        float s[kHalves], b;
        float x[RM];
    };
    auto load_row = [&](int k, Row &r) {
        const int kc = k < k_end ? k : k_end - 1;  // past the range: a harmless reload
        if constexpr (MODE == NVQ_NVFP4) {  // an absent second group reads the first again; its outputs are not stored
            const uint2 *p = reinterpret_cast<const uint2 *>(w + (int64_t)kc * row_dwords);
            const uint2 lo = p[0], hi = p[whole ? 1 : 0];
            r.d[0] = lo.x; r.d[1] = lo.y; r.d[2] = hi.x; r.d[3] = hi.y;
        } else {
            load_words<BITS>(w + (int64_t)kc * row_dwords, r.d);
        }
        r.b = 0.0f;
        if constexpr (kAffine) {
            r.s[0] = Elem<T>::load((const T *)a.scales, s_at + (int64_t)kc * ngroups);
            r.b = Elem<T>::load((const T *)a.biases, s_at + (int64_t)kc * ngroups);
        } else {
            const uint8_t *sp = (const uint8_t *)a.scales + s_at + (int64_t)kc * ngroups;
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) r.s[hf] = ftz(MODE == NVQ_NVFP4 ? e4m3_to_f32(sp[whole ? hf : 0]) : e8m0_to_f32(sp[hf]));
        }
#pragma unroll
        for (int i = 0; i < RM; i++) r.x[i] = m0 + i < M ? Elem<T>::load(x, (int64_t)(m0 + i) * K + kc) : 0.0f;
    };

    if (k_begin < k_end) {
        // D rows of the weights in flight per lane: a wavefront's row is 1 KB (4 bits), and a split's few wavefronts
        // need tens of KB each under way to cover the memory latency
        constexpr int D = RM == 1 ? 8 : 4;
        Row ring[D];
#pragma unroll
        for (int d = 0; d < D; d++) load_row(k_begin + d, ring[d]);
        for (int k = k_begin; k < k_end; k += D) {
#pragma unroll
            for (int d = 0; d < D; d++) {
                const Row r = ring[d];
                load_row(k + d + D, ring[d]);
                if (k + d < k_end) {
                    float xs[RM][kHalves];
#pragma unroll
                    for (int i = 0; i < RM; i++) {
#pragma unroll
                        for (int hf = 0; hf < kHalves; hf++) xs[i][hf] = exact ? r.x[i] : r.x[i] * r.s[hf];
                        if (!exact) accb[i] = __builtin_fmaf(r.x[i], r.b, accb[i]);
                    }
#pragma unroll
                    for (int j = 0; j < 32; j++) {
                        const uint32_t c = code_at<BITS>(r.d, j);
                        float v = kAffine ? (float)c : (MODE == NVQ_MXFP8 ? e4m3_to_f32(c) : e2m1_to_f32(c));
                        if constexpr (kAffine)
                            if (exact) v = Elem<T>::add(Elem<T>::mul(v, r.s[0]), r.b);  // the weight as the CPU holds it (kernels.rs:835-859)
#pragma unroll
                        for (int i = 0; i < RM; i++) acc[i][j] = __builtin_fmaf(xs[i][j * kHalves / 32], v, acc[i][j]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RM; i++) {
        if (i > 0) __syncthreads();  // the previous row's sums are read
        if (wave > 0) {
#pragma unroll
            for (int j = 0; j < 32; j++) sums[wave - 1][j][lane] = acc[i][j] + accb[i];
        }
        __syncthreads();
        if (wave > 0) continue;
#pragma unroll
        for (int j = 0; j < 32; j++) {
            float v = acc[i][j] + accb[i];
#pragma unroll
            for (int wv = 0; wv < kQvmWaves - 1; wv++) v += sums[wv][j][lane];
            acc[i][j] = v;
        }
        accb[i] = 0.0f;
        if (!live || m0 + i >= M) continue;
        if (splits == 1) {
            T *out = (T *)a.y + (o.y * M + m0 + i) * N + n0;
#pragma unroll
            for (int j = 0; j < 32; j++)
                if (j < 16 || whole) Elem<T>::store(out, j, add_row_bias<T>(a.row_bias, acc[i][j] + accb[i], n0 + j));
        } else {
            float *out = partial + (((int64_t)bz * splits + blockIdx.y) * M + m0 + i) * N + n0;
#pragma unroll
            for (int j = 0; j < 32; j++)
                if (j < 16 || whole) out[j] = acc[i][j] + accb[i];
        }
    }
}

// y[b, m, n] = the splits' partial sums added in split order, rounded once.
template <typename T>
__global__ void __launch_bounds__(256) qvm_reduce_kernel(const float *partial, T *y, int splits, int64_t per_batch, int64_t total,
                                                         const void *row_bias, int64_t n) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t b = idx / per_batch, rest = idx - b * per_batch;
    const float *p = partial + b * splits * per_batch + rest;
    float sum = 0.0f;
    int s = 0;
    for (; s + 8 <= splits; s += 8) {  // eight loads under way at a time; the additions keep the splits' order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = p[(int64_t)(s + u) * per_batch];
#pragma unroll
        for (int u = 0; u < 8; u++) sum += v[u];
    }
    for (; s < splits; s++) sum += p[(int64_t)s * per_batch];
    Elem<T>::store(y, idx, add_row_bias<T>(row_bias, sum, idx % n));
}


// ---- Many rows of x: the same product on the matrix cores ---------------------------------------------------------
// A block of four wavefronts (2 x 2, each 64 x 64 of y as 2 x 2 tiles of the 32x32x16 instruction; for up to 32 rows of
// x 1 x 4 wavefronts of one tile each, see Shape) owns 128 x 128 of y and walks K in steps of 64 rows of w through two
// LDS stages, one barrier per step, two blocks per compute unit.
// The matrix instruction wants eight consecutive k per lane and column, the storage gives eight consecutive columns
// per row and word, so the weights are turned on the way into LDS: thread (q = t / 16, c = t % 16) loads the codes of
// columns 8 c .. 8 c + 7 of rows 4 q .. 4 q + 3 of the step (one word per row at 4 bits: sixteen lanes cover the
// row's 64 bytes) two steps ahead, expands each row with its scale and bias to the element type (one rounding of
// fma(code, scale, bias), as the tiled kernel of the transposed storage) between the matrix instructions of the
// running step, swaps the 4 x 8 block in registers (one byte permute per output word) and writes, per column, its
// four k as one 8-byte piece.  x travels through registers into the other half of the stage.
// LDS layouts, both in 16-byte slots of eight k: x row r, slot ch at r * 8 + (ch ^ (r >> 1) % 8); w column n, slot ch
// at (n / 16 * 8 + ch) * 16 + (n + n / 16 + 8 (ch / 4)) % 16.  Sixteen lanes reading one slot index of consecutive
// rows (columns) touch sixteen different bank groups in either layout, and so do the writes of sixteen lanes whose
// columns are eight apart (the rotation by n / 16).  A substep of the matrix instructions takes slot ks for the
// lanes' lower half and slot 4 + ks for the upper one, which the layouts keep in different banks.
// Products of few tiles split K over the grid (float32 partial sums in the caller's workspace, added in split order
// by the reduction kernel above); without a workspace K is not split.
namespace qmn {

using namespace qmf;

constexpr int BN = 128, BK = 64, kThreads = 256;
constexpr int kWBytes = BN * BK * 2;

// The four wavefronts of a block as WM x (4 / WM), each TI x TJ tiles of 32 x 32: 128 x 128 of y per block (two blocks
// per compute unit), or 32 x 128 for up to 32 rows of x (one tile per wavefront, four blocks per compute unit, all of
// a step's operands read at once).
template <int WM_, int TI_, int TJ_, int BLOCKS_>
struct Shape {
    static constexpr int WM = WM_, WN = 4 / WM_, TI = TI_, TJ = TJ_, kBlocksPerCu = BLOCKS_;
    static constexpr int BM = WM * TI * 32;
    static constexpr int kXParts = BM * 8 / kThreads;  // 16-byte pieces of a step of x per thread
    static constexpr int kXBytes = BM * BK * 2, kStageBytes = kXBytes + kWBytes;
    static_assert(WN * TJ * 32 == BN && kXParts * kThreads == BM * 8, "the loading assignment below assumes these");
};
using Tile128 = Shape<2, 2, 2, 2>;
using Tile32 = Shape<1, 1, 1, 4>;

__device__ __forceinline__ int x_slot(int row, int ch) { return (row * 8 + (ch ^ ((row >> 1) & 7))) * 16; }
__device__ __forceinline__ int w_slot(int n, int ch) { return (((n >> 4) * 8 + ch) * 16 + ((n + (n >> 4) + 2 * (ch & 4)) & 15)) * 16; }

// The codes of eight columns of one row: BITS bytes.
template <int BITS>
__device__ __forceinline__ void load_run(const unsigned char *p, uint32_t (&d)[BITS]) {
#pragma unroll
    for (int i = 0; i < BITS; i++) d[i] = 0;
    if constexpr (BITS == 8) {
        const uint2 v = *reinterpret_cast<const uint2 *>(p);
        d[0] = v.x, d[1] = v.y;
    } else if constexpr (BITS == 4) {
        d[0] = *reinterpret_cast<const uint32_t *>(p);
    } else if constexpr (BITS == 2) {
        d[0] = *reinterpret_cast<const uint16_t *>(p);
    } else {  // 1, 3, 5 and 6 bits: a run is BITS bytes at any byte offset of the row
#pragma unroll
        for (int i = 0; i < BITS; i++) d[i >> 2] |= (uint32_t)p[i] << (8 * (i & 3));
    }
}

// EXACT (affine codes): the weights as nuvec's CPU product holds them (qmf::affine_pair).
template <typename T, int BITS, int FP4, bool EXACT, class TL>
__global__ void __launch_bounds__(kThreads, TL::kBlocksPerCu) qmn_kernel(const ProductArgs a, int splits, float *partial) {
    using S = std::conditional_t<FP4 != 0, uint8_t, T>;  // stored scale type
    constexpr int BM = TL::BM, TI = TL::TI, TJ = TL::TJ, kXParts = TL::kXParts, kXBytes = TL::kXBytes, kStageBytes = TL::kStageBytes;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kStageBytes];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / TL::WN, wn = wave % TL::WN, h = lane >> 5, l32 = lane & 31;
    const int K = (int)a.k, N = (int)a.n;
    const int gshift = FP4 == kNvfp4 ? 4 : FP4 ? 5 : (a.group == 32 ? 5 : a.group == 64 ? 6 : 7);
    const int ngroups = N >> gshift;
    const int64_t row_bytes = ((int64_t)N * BITS) >> 3;
    const int ntiles = (N + BN - 1) / BN;
    const bool grouped = a.offsets != nullptr;
    int M = (int)a.m, m0, n0, pair0 = 0;
    Offsets o;
    if (grouped) {
        // Rows of one row of x each, sorted by expert: expert e's rows of x are the pairs [offsets[e], offsets[e + 1]),
        // taken through `lhs`.  The grid holds ceil(pairs / BM) + experts tiles of rows (every expert adds at most one
        // partial tile) times the column tiles, in launch order tile of rows by tile of rows (so the work goes round the
        // XCDs); a block finds its tile's expert by walking the offsets, and the tiles past the last expert's leave.
        const int tile = (int)blockIdx.x / ntiles;
        int e = 0, first = 0, rows = 0;
        for (; e < (int)a.experts; e++) {
            // (offsets that do not ascend within the pairs are the caller's error: clamped, so that they cannot fault the device)
            pair0 = min(max(a.offsets[e], 0), (int)a.batch);
            rows = (e + 1 < (int)a.experts ? min(max(a.offsets[e + 1], pair0), (int)a.batch) : (int)a.batch) - pair0;
            const int tiles = (rows + BM - 1) / BM;
            if (tile < first + tiles) break;
            first += tiles;
        }
        if (e == (int)a.experts) return;  // the whole block, before any barrier
        M = rows;
        m0 = (tile - first) * BM, n0 = ((int)blockIdx.x % ntiles) * BN;
        o = Offsets{0, (int64_t)e * K * (N * BITS / 32), (int64_t)e * K * ngroups, 0};
    } else {
        // Blocks are handed to the 8 XCDs (an L2 each) in turn: block p takes item (p % 8) * ceil(items / 8) + p / 8 of the
        // tile list, whose order walks bands of 8 tiles of rows column tile by column tile, so that an XCD's 64 resident
        // blocks are 8 x 8 tiles that share 8 tiles of x and 8 of w.
        const int mtiles = (M + BM - 1) / BM, items = mtiles * ntiles, per = (items + 7) >> 3;
        const int item = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
        if (item >= items) return;  // the whole block, before any barrier
        const int band = item / (8 * ntiles), in_band = item - band * 8 * ntiles;
        const int band_rows = mtiles - 8 * band < 8 ? mtiles - 8 * band : 8;
        m0 = (8 * band + in_band % band_rows) * BM, n0 = (in_band / band_rows) * BN;
        o = batch_offsets(a, blockIdx.y);
    }
    const T *x = (const T *)a.x + o.x;

    // Addresses are a base that is the same for the whole block (scalar registers, advanced per step by scalar
    // arithmetic) plus a 32-bit offset per lane that never changes.
    // This thread's part of a step of w: columns n0 + 8 c .. + 7 (a run past N reads the block's first run; its
    // columns are not stored), rows 4 q .. 4 q + 3.
    const int c = tid & 15, q = tid >> 4;
    const int run = n0 + 8 * c < N ? 8 * c : 0;  // within the tile
    const unsigned char *wbase = (const unsigned char *)a.w + o.w * 4 + (((int64_t)n0 * BITS) >> 3);
    const S *sbase = (const S *)a.scales + o.s + (n0 >> gshift);
    const S *bbase = (const S *)a.biases + o.s + (n0 >> gshift);
    const uint32_t woff = (uint32_t)(4 * q) * (uint32_t)row_bytes + (uint32_t)((run * BITS) >> 3);
    const uint32_t soff = ((uint32_t)(4 * q * ngroups) + (uint32_t)(((n0 + run) >> gshift) - (n0 >> gshift))) * (uint32_t)sizeof(S);
    int wdst[8];
#pragma unroll
    for (int j = 0; j < 8; j++) wdst[j] = kXBytes + w_slot(8 * c + j, q >> 1) + 8 * (q & 1);
    // This thread's part of a step of x: 16-byte pieces t + 256 i (piece p: row p / 8, slot p % 8).
    const unsigned char *xbase = (const unsigned char *)(x + (grouped ? 0 : (int64_t)m0 * K));
    uint32_t xoff[kXParts];
    int xdst[kXParts];
#pragma unroll
    for (int i = 0; i < kXParts; i++) {
        const int p = tid + 256 * i, r = p >> 3, ch = p & 7;
        const int row = m0 + r < M ? r : M - 1 - m0;  // rows past M are computed, not stored
        // grouped: the row of x of pair pair0 + m0 + row (an index outside x is the caller's error and is clamped)
        const uint32_t xrow = grouped ? (uint32_t)min((int64_t)a.lhs[pair0 + m0 + row], a.x_batches - 1) : (uint32_t)row;
        xoff[i] = (xrow * (uint32_t)K + 8u * ch) * 2u;
        xdst[i] = x_slot(r, ch);
    }

    struct Regs {
        u32x4_t x[kXParts];
        uint32_t w[4][BITS];
        S s[4], b[4];
    };
    auto load = [&](int step, Regs &r) {
        const int64_t k0 = (int64_t)step * BK;
        const unsigned char *xs = xbase + k0 * 2;
#pragma unroll
        for (int i = 0; i < kXParts; i++) r.x[i] = *reinterpret_cast<const u32x4_t *>(xs + xoff[i]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            load_run<BITS>(wbase + (k0 + i) * row_bytes + woff, r.w[i]);
            const int64_t srow = (k0 + i) * ngroups * (int64_t)sizeof(S);
            r.s[i] = *reinterpret_cast<const S *>((const unsigned char *)sbase + srow + soff);
            if constexpr (!FP4) r.b[i] = *reinterpret_cast<const S *>((const unsigned char *)bbase + srow + soff);
        }
    };
    // Row I of the thread's block of a step: eight columns, two per word, in the element type.
    auto row = [&](const Regs &r, auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        const S sv = r.s[i], bv = r.b[i];
        float scale, bias = 0.0f;
        if constexpr (FP4 == kNvfp4) scale = ftz(e4m3_to_f32(sv));
        else if constexpr (FP4) scale = ftz(e8m0_to_f32(sv));
        else scale = Elem<T>::load(&sv, 0), bias = Elem<T>::load(&bv, 0);
        return expand_piece<T, BITS, FP4, 0, EXACT>(r.w[i], scale, bias);
    };
    // The four expanded rows turned (columns 2 d: the words' low halves, 2 d + 1: the high halves; rows (0, 1) and (2, 3)
    // as two words each) and written to a stage together with the thread's pieces of x.
    auto store = [&](int stage_at, const Regs &r, const uint4 &v0, const uint4 &v1, const uint4 &v2, const uint4 &v3) {
        unsigned char *stage = lds + stage_at * kStageBytes;
#pragma unroll
        for (int i = 0; i < kXParts; i++) *reinterpret_cast<u32x4_t *>(stage + xdst[i]) = r.x[i];
        auto turn = [&](uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, int even_at, int odd_at) {
            const uint2 even = {__builtin_amdgcn_perm(a1, a0, 0x05040100u), __builtin_amdgcn_perm(a3, a2, 0x05040100u)};
            const uint2 odd = {__builtin_amdgcn_perm(a1, a0, 0x07060302u), __builtin_amdgcn_perm(a3, a2, 0x07060302u)};
            *reinterpret_cast<uint2 *>(stage + even_at) = even;
            *reinterpret_cast<uint2 *>(stage + odd_at) = odd;
        };
        turn(v0.x, v1.x, v2.x, v3.x, wdst[0], wdst[1]);
        turn(v0.y, v1.y, v2.y, v3.y, wdst[2], wdst[3]);
        turn(v0.z, v1.z, v2.z, v3.z, wdst[4], wdst[5]);
        turn(v0.w, v1.w, v2.w, v3.w, wdst[6], wdst[7]);
    };

    int xread[TI], wread[TJ];  // of the first slot of the lane's half; the others are an XOR (x) or a constant (w) away
#pragma unroll
    for (int t = 0; t < TI; t++) xread[t] = (32 * TI * wm + 32 * t + l32) * 128;
#pragma unroll
    for (int t = 0; t < TJ; t++) wread[t] = kXBytes + w_slot(32 * TJ * wn + 32 * t + l32, 4 * h);
    const int xswz = ((l32 >> 1) & 7) ^ (4 * h);  // (the tile bases are multiples of 16 rows) slot s of the lane's half: s ^ xswz

    floatx16_t acc[TI][TJ];
#pragma unroll
    for (int ti = 0; ti < TI; ti++)
#pragma unroll
        for (int tj = 0; tj < TJ; tj++)
#pragma unroll
            for (int el = 0; el < 16; el++) acc[ti][tj][el] = 0.0f;

    // This block's steps of K (all of them without a split), loaded two steps ahead into two sets of registers.
    const int all_steps = K / BK, per_split = (all_steps + splits - 1) / splits;
    const int first = (int)blockIdx.z * per_split, steps = all_steps - first < per_split ? all_steps - first : per_split;
    if (steps <= 0) return;  // (the host gives every split a step; the whole block leaves, before any barrier)
    const int last = first + steps - 1;
    auto at = [&](int step) { return step < last ? step : last; };  // a step past the end loads the last one again
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    Regs ra, rb;
    load(first, ra);
    load(at(first + 1), rb);
    store(0, ra, row(ra, I0{}), row(ra, I1{}), row(ra, I2{}), row(ra, I3{}));
    load(at(first + 2), ra);
    __syncthreads();
    // One step.  Its four substeps of 16 k each read their operands from the stage a substep ahead and run four
    // matrix instructions, between which one row of the next step's registers is expanded (register work only: the
    // order of LDS reads and writes stays the written one, reads first).  Then the expanded block is turned and
    // written to the other stage (last read a step ago, before the barrier) and the registers take the step after
    // the next but one.  Nothing branches (a step past the end is stored and never read).
    auto step = [&](int stage_at, Regs &next, int refill) {
        const unsigned char *stage = lds + stage_at * kStageBytes;
        uint4 v[4];
        // substep ks takes the eight k of slot ks for the lanes' lower half and of slot 4 + ks for the upper one (any
        // order of k serves as long as x and w agree): the two halves then never meet in a bank
        constexpr bool kAllAtOnce = TI * TJ == 1;  // one tile per wavefront: the registers hold the operands of all four substeps
        uint4 xa[kAllAtOnce ? 4 : 1][TI], wb[kAllAtOnce ? 4 : 1][TJ];
        auto fragments = [&](int ks) {
#pragma unroll
            for (int t = 0; t < TI; t++) xa[kAllAtOnce ? ks : 0][t] = *reinterpret_cast<const uint4 *>(stage + xread[t] + ((ks ^ xswz) << 4));
#pragma unroll
            for (int t = 0; t < TJ; t++) wb[kAllAtOnce ? ks : 0][t] = *reinterpret_cast<const uint4 *>(stage + wread[t] + ks * 256);
        };
        if constexpr (kAllAtOnce) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++) fragments(ks);
        }
        static_for<4>([&](auto ks_tag) {
            constexpr int ks = decltype(ks_tag)::value;
            if constexpr (!kAllAtOnce) fragments(ks);
#pragma unroll
            for (int ti = 0; ti < TI; ti++)
#pragma unroll
                for (int tj = 0; tj < TJ; tj++) acc[ti][tj] = Ops<T>::mfma(xa[kAllAtOnce ? ks : 0][ti], wb[kAllAtOnce ? ks : 0][tj], acc[ti][tj]);
            v[ks] = row(next, ks_tag);
            if constexpr (!kAllAtOnce) __builtin_amdgcn_sched_group_barrier(0x100, TI + TJ, 0);
#pragma unroll
            for (int i = 0; i < TI * TJ; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        store(stage_at ^ 1, next, v[0], v[1], v[2], v[3]);
        load(at(refill), next);
        __syncthreads();
    };
    for (int s = 0; s < steps; s += 2) {
        step(0, rb, first + s + 3);
        if (s + 1 >= steps) break;
        step(1, ra, first + s + 4);
    }

    // Accumulator element el of lane l is tile row 8 (el / 4) + 4 (l / 32) + el % 4 (a row of x), column l % 32.
    T *y = (T *)a.y + (grouped ? (int64_t)pair0 * N : o.y * M * N);
    float *part = partial + ((int64_t)blockIdx.y * splits + blockIdx.z) * M * N;  // (used with a split only; never grouped)
    const bool biased = a.row_bias != nullptr;
#pragma unroll
    for (int tj = 0; tj < TJ; tj++) {
        const int col = n0 + 32 * TJ * wn + 32 * tj + l32;
        if (col >= N) continue;
        const float bias = biased && splits == 1 ? Elem<T>::load((const T *)a.row_bias, col) : 0.0f;
#pragma unroll
        for (int ti = 0; ti < TI; ti++)
#pragma unroll
            for (int el = 0; el < 16; el++) {
                const int m = m0 + 32 * TI * wm + 32 * ti + 8 * (el >> 2) + 4 * h + (el & 3);
                if (m >= M) continue;
                const float v = acc[ti][tj][el];
                if (splits > 1) part[(int64_t)m * N + col] = v;
                else Elem<T>::store(y, (int64_t)m * N + col, biased ? Elem<T>::add(Elem<T>::mul(v, 1.0f), bias) : v);  // as add_row_bias
            }
    }
}

inline bool few_rows(const ProductArgs &a) { return a.m <= Tile32::BM; }

// Splits of K for a product whose tiles do not fill the chip: the host rule of nvq_splits.h, bound to these tiles.
static_assert(BK == splits::kQmnStep && BN == splits::kQmnTileCols && Tile32::BM == splits::kQmnFewRows &&
              Tile128::BM == splits::kQmnManyRows && Tile32::kBlocksPerCu == splits::kQmnFewBlocksPerCu &&
              Tile128::kBlocksPerCu == splits::kQmnManyBlocksPerCu, "nvq_splits.h describes these tiles");
inline splits::Product split_product(const ProductArgs &a) {
    return splits::Product{a.m, a.n, a.k, a.batch, a.row_exact != 0, a.exact_weights != 0};
}
template <class TL>
int splits_of_shape(const ProductArgs &a) {
    return splits::qmn_plan(split_product(a), compute_units(), TL::BM == Tile32::BM).splits;
}
inline int splits_of(const ProductArgs &a) { return few_rows(a) ? splits_of_shape<Tile32>(a) : splits_of_shape<Tile128>(a); }

template <typename T, int BITS, int FP4, class TL>
int32_t run_shape(const ProductArgs &a, float *workspace, hipStream_t s) {
    const bool grouped = a.offsets != nullptr;  // ceil(pairs / BM) + experts tiles of rows: every expert adds at most one partial tile
    const int splits = workspace != nullptr && !grouped ? splits_of_shape<TL>(a) : 1;  // without a workspace K is not split
    const int64_t row_tiles = grouped ? (a.batch + TL::BM - 1) / TL::BM + a.experts : (a.m + TL::BM - 1) / TL::BM;
    const int64_t tiles = row_tiles * ((a.n + BN - 1) / BN);
    const dim3 grid((unsigned)(grouped ? tiles : (tiles + 7) / 8 * 8), (unsigned)(grouped ? 1 : a.batch), (unsigned)splits);
    {  // (the kernel's split of the steps; a block of a split without a step would leave its partial sums unwritten)
        const int64_t steps = a.k / BK, per_split = (steps + splits - 1) / splits;
        if (splits > 1 && (int64_t)(splits - 1) * per_split >= steps)
            return fail(NVQ_BACKEND, "quantized_matmul: %d splits leave one without a step of K = %lld", splits, (long long)a.k);
    }
    if (FP4 == kAffine && a.exact_weights) hipLaunchKernelGGL((qmn_kernel<T, BITS, FP4, FP4 == kAffine, TL>), grid, dim3(kThreads), 0, s, a, splits, workspace);
    else hipLaunchKernelGGL((qmn_kernel<T, BITS, FP4, false, TL>), grid, dim3(kThreads), 0, s, a, splits, workspace);
    NVQ_LAUNCH_CHECK("qmn");
    if (splits > 1) {
        const int64_t per_batch = a.m * a.n, total = a.batch * per_batch;
        hipLaunchKernelGGL((qvm_reduce_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const float *)workspace,
                           (T *)a.y, splits, per_batch, total, a.row_bias, a.n);
        NVQ_LAUNCH_CHECK("qvm_reduce");
    }
    return NVQ_OK;
}

template <typename T, int BITS, int FP4>
int32_t run(const ProductArgs &a, float *workspace, hipStream_t s) {
    // (grouped: the tile of 32 rows up to 64 rows per expert on average)
    const bool few = a.offsets != nullptr ? a.batch <= 2 * (int64_t)Tile32::BM * a.experts : few_rows(a);
    return few ? run_shape<T, BITS, FP4, Tile32>(a, workspace, s) : run_shape<T, BITS, FP4, Tile128>(a, workspace, s);
}

template <typename T>
int32_t run_typed(const ProductArgs &a, float *ws, hipStream_t s) {
    switch (a.mode) {
    case NVQ_MXFP4: return run<T, 4, kMxfp4>(a, ws, s);
    case NVQ_MXFP8: return run<T, 8, kMxfp8>(a, ws, s);
    case NVQ_NVFP4: return run<T, 4, kNvfp4>(a, ws, s);
    default: break;
    }
    switch (a.bits) {
    case 1: return run<T, 1, kAffine>(a, ws, s);
    case 2: return run<T, 2, kAffine>(a, ws, s);
    case 3: return run<T, 3, kAffine>(a, ws, s);
    case 4: return run<T, 4, kAffine>(a, ws, s);
    case 5: return run<T, 5, kAffine>(a, ws, s);
    case 6: return run<T, 6, kAffine>(a, ws, s);
    default: return run<T, 8, kAffine>(a, ws, s);
    }
}

}  // namespace qmn

template <typename T, int BITS, int MODE>
int32_t run_qvm(const ProductArgs &a, void *workspace, hipStream_t s) {
    const int splits = qvm_splits(a);
    if (splits > 1 && workspace == nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "quantized_matmul: this product needs its %zu-byte workspace", qvm_workspace_bytes(a));
    const unsigned tiles = (unsigned)((a.n + 2047) / 2048);
    const int rm = a.m == 1 ? 1 : 4;
    const int64_t z = a.batch * ((a.m + rm - 1) / rm);
    if (z > 65535) return fail(NVQ_UNSUPPORTED, "quantized_matmul: %lld row passes exceed the grid limit", (long long)z);
    const dim3 grid(tiles, (unsigned)splits, (unsigned)z);
    constexpr bool kCanBeExact = MODE == NVQ_AFFINE && !std::is_same<T, float>::value;
    if (kCanBeExact && a.exact_weights) {
        if (rm == 1) hipLaunchKernelGGL((qvm_kernel<T, BITS, MODE, 1, kCanBeExact>), grid, dim3(64 * kQvmWaves), 0, s, a, splits, (float *)workspace);
        else hipLaunchKernelGGL((qvm_kernel<T, BITS, MODE, 4, kCanBeExact>), grid, dim3(64 * kQvmWaves), 0, s, a, splits, (float *)workspace);
    } else if (rm == 1) {
        hipLaunchKernelGGL((qvm_kernel<T, BITS, MODE, 1>), grid, dim3(64 * kQvmWaves), 0, s, a, splits, (float *)workspace);
    } else {
        hipLaunchKernelGGL((qvm_kernel<T, BITS, MODE, 4>), grid, dim3(64 * kQvmWaves), 0, s, a, splits, (float *)workspace);
    }
    NVQ_LAUNCH_CHECK("qvm");
    if (splits > 1) {
        const int64_t per_batch = a.m * a.n, total = a.batch * per_batch;
        hipLaunchKernelGGL((qvm_reduce_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const float *)workspace,
                           (T *)a.y, splits, per_batch, total, a.row_bias, a.n);
        NVQ_LAUNCH_CHECK("qvm_reduce");
    }
    return NVQ_OK;
}

template <typename T>
int32_t run_qvm_typed(const ProductArgs &a, void *workspace, hipStream_t s) {
    switch (a.mode) {
    case NVQ_MXFP4: return run_qvm<T, 4, NVQ_MXFP4>(a, workspace, s);
    case NVQ_MXFP8: return run_qvm<T, 8, NVQ_MXFP8>(a, workspace, s);
    case NVQ_NVFP4: return run_qvm<T, 4, NVQ_NVFP4>(a, workspace, s);
    default: break;
    }
    switch (a.bits) {
    case 1: return run_qvm<T, 1, NVQ_AFFINE>(a, workspace, s);
    case 2: return run_qvm<T, 2, NVQ_AFFINE>(a, workspace, s);
    case 3: return run_qvm<T, 3, NVQ_AFFINE>(a, workspace, s);
    case 4: return run_qvm<T, 4, NVQ_AFFINE>(a, workspace, s);
    case 5: return run_qvm<T, 5, NVQ_AFFINE>(a, workspace, s);
    case 6: return run_qvm<T, 6, NVQ_AFFINE>(a, workspace, s);
    case 8: return run_qvm<T, 8, NVQ_AFFINE>(a, workspace, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "quantized_matmul: %d bits are not supported", a.bits);
    }
}

}  // namespace

// Splits of K of the vector kernel: the host rule of nvq_splits.h.
static_assert(kQvmWaves == splits::kQvmWaves, "nvq_splits.h describes this block");
int qvm_splits(const ProductArgs &a) {
    return splits::qvm_plan(splits::Product{a.m, a.n, a.k, a.batch, a.row_exact != 0, a.exact_weights != 0}, compute_units()).splits;
}

size_t qvm_workspace_bytes(const ProductArgs &a) {
    if (qvm_takes_tiled(a)) {
        const int splits = qmn::splits_of(a);
        return splits > 1 ? (size_t)splits * (size_t)a.batch * (size_t)a.m * (size_t)a.n * sizeof(float) : 0;
    }
    const int splits = qvm_splits(a);
    return splits > 1 ? (size_t)splits * (size_t)a.batch * (size_t)a.m * (size_t)a.n * sizeof(float) : 0;
}

// (With eight wavefronts a block, eight rows of w in flight per lane and at most 32 splits the vector kernel above went,
// at bf16 4-bit g64 and one row of x, kernel and reduction: w[4096,14336] 67 -> 23 us, w[14336,4096] 143 -> 52 us,
// w[4096,4096] 65 -> 19 us; the matrix-core kernel: 23 / 26 / 12 us, and flat up to 16 rows where this one adds 8 us a row.)
// The matrix-core kernel takes the 16-bit products whose codes come in whole runs of eight columns (every affine width,
// the block formats without a global scale) and whose K is whole steps of 64, whatever the rows of x: measured
// against the vector kernel above (bf16, 4-bit g64, both with their split of K and its reduction, us per call of the
// Python wrapper) w[4096,14336] 1 row 42 / 55, 8 rows 42 / 91, 32 rows 45 / 246, 512 rows 128 / 1890; w[14336,4096]
// 1 row 35 / 131; w[1024,1024] 1 row 24 / 24, 32 rows 24 / 37; MXFP4 w[4096,4096] 1 row 22 / 94, 128 rows 26 / 588.
bool qvm_takes_tiled(const ProductArgs &a) {
    if (a.dtype == NVQ_F32 || a.row_exact || a.global_scale != nullptr || a.m < 1) return false;
    // 1, 3, 5 and 6 bits: a run of eight codes is 1, 3, 5 or 6 bytes, fetched byte by byte.  bf16, us, vector kernel ->
    // this one: w[4096,4096] 3 bits at 1 / 16 / 512 rows 17.9 / 31.6 / 961 -> 14.9 / 13.4 / 52.5; w[4096,14336] 6 bits at
    // 2 / 16 / 512 rows 32.0 / 152 / 2324 -> 29.5 / 31.8 / 115; only a single row against many columns stays behind
    // (w[4096,14336] 3 bits 18.7 against 23.4, 6 bits 24.6 against 29.3).
    if (a.mode == NVQ_AFFINE && !(a.bits == 2 || a.bits == 4 || a.bits == 8) && a.m == 1 && a.offsets == nullptr && a.n > 8192) return false;
    if (a.k < qmn::BK || a.k % qmn::BK != 0 || (a.batch > 65535 && a.offsets == nullptr)) return false;
    for (int d = 0; d < a.batch_ndim; d++)
        if (a.x_strides[d] % 8 != 0 || a.w_strides[d] % 4 != 0) return false;  // 16-byte pieces of x, 8-byte runs of codes
    return ((uintptr_t)a.w | (uintptr_t)a.x) % 16 == 0;
}

// Whether the tiled kernel takes the pairs of a gather sorted by expert as groups (`a.offsets` set, one row of x per
// pair): each expert's weights are then read once per tile of its rows instead of once per pair.
bool qvm_takes_grouped(const ProductArgs &a) {
    if (a.offsets == nullptr || a.m != 1 || a.rhs == nullptr || a.exact_weights || a.row_bias != nullptr) return false;
    if (a.experts > 4096 || a.x_batches * a.k >= (1LL << 31) || a.batch >= (1LL << 30)) return false;  // (a block walks the offsets)
    return qvm_takes_tiled(a);
}

const char *qvm_kernel_name(const ProductArgs &a) { return qvm_takes_tiled(a) ? "qmn_kernel" : "qvm_kernel"; }

int32_t launch_qvm(const ProductArgs &a, void *workspace, hipStream_t s) {
    if (qvm_takes_tiled(a))
        return a.dtype == NVQ_BF16 ? qmn::run_typed<bf16_t>(a, (float *)workspace, s) : qmn::run_typed<f16_t>(a, (float *)workspace, s);
    switch (a.dtype) {
    case NVQ_F32: return run_qvm_typed<float>(a, workspace, s);
    case NVQ_BF16: return run_qvm_typed<bf16_t>(a, workspace, s);
    default: return run_qvm_typed<f16_t>(a, workspace, s);
    }
}

}  // namespace nvq
