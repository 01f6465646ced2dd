// float32 products of many rows on the matrix cores: y[M,N] = x[M,K] . dequantize(w[N,K])^T for x, scales and biases in
// float32 and affine codes of every width or a block format (MXFP4, MXFP8, NVFP4), on v_mfma_f32_32x32x2_f32.  The reference instantiates its tiled kernels
// for float as for the half types (crates/nuvec-kernels/src/metal/quantized.metal:40-70, kernel
// crates/nuvec-kernels/src/metal/quantized.h:1358-1485); values follow nuvec's CPU product
// (crates/nuvec-core/src/kernels.rs:1091-1142): the weights are dequantized in float32 exactly as the CPU does,
// round(round(code * scale) + bias) (kernels.rs:835-859; a block format's weight is its decoded code times its group's
// decoded scale, NVFP4's scale first times ftz(g / 2688) where a global scale g is given, kernels.rs:992-998), and the
// products accumulate in float32.
//
// A block of four wavefronts owns a 64 x 64 tile of y (2 x 2 wavefronts, one 32 x 32 matrix tile each) and walks K in
// steps of 64 values.  The x tile of a step (64 rows x 256 bytes) goes through LDS, double buffered, rows 272 bytes
// apart so that the 16-byte operand reads of sixteen rows fall on all 64 banks; the step after the next is requested
// into registers while the current one is multiplied.  A lane (column n = lane % 32, half h = lane / 32) fetches the 32
// codes [32 h, 32 h + 32) of its weight row itself (BITS dwords: always whole dwords, one group) and dequantizes one
// weight per matrix instruction, which takes 64 cycles: the vector work hides under it.  Instruction j of a step
// multiplies the values k = 32 h + j of the step in both operands.  Four blocks share a compute unit (35 KB of LDS
// each), so sixteen wavefronts hide each other's waits without a deeper pipeline.
#include "nvq_device.h"
#include "nvq_internal.h"
#include "qmf_kernel.h"

namespace nvq {
namespace {

using qmf::code_to_float;
using qmf::floatx16_t;
using qmf::static_for;

typedef float f32x4_t __attribute__((ext_vector_type(4)));  // (a native vector: arrays of it stay in registers)

constexpr int kTile = 64;                 // rows of x and weight rows of a block
constexpr int kStep = 64;                 // values of K per step
constexpr int kRowFloats = kStep + 4;     // an x row of a step in LDS: 272 bytes

// MODE: NVQ_AFFINE, NVQ_MXFP4, NVQ_MXFP8 or NVQ_NVFP4 (BITS is 4 or 8 for the block formats).
template <int BITS, int MODE>
__global__ void __launch_bounds__(256) qmm_f32_kernel(const ProductArgs a) {
    constexpr bool kAffine = MODE == NVQ_AFFINE;
    constexpr int kHalves = MODE == NVQ_NVFP4 ? 2 : 1;  // groups in a lane's 32 values
    __shared__ __attribute__((aligned(16))) float xs[2][kTile * kRowFloats];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, h = lane >> 5, l32 = lane & 31;
    const int M = (int)a.m, N = (int)a.n, K = (int)a.k;
    const int gshift = kAffine ? (a.group == 32 ? 5 : a.group == 64 ? 6 : 7) : (MODE == NVQ_NVFP4 ? 4 : 5);
    const int kgroups = K >> gshift, row_dwords = (K >> 5) * BITS, steps = K / kStep;
    const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
    const float *x = (const float *)a.x;
    float *y = (float *)a.y;

    // x: the tile of a step is 1024 pieces of four values; thread t brings pieces t + 256 i (row p / 16, piece p % 16).
    // Rows past M read row M - 1 and are never stored.
    const float *xsrc[4];
    int xdst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int p = tid + 256 * i, r = p >> 4, c = p & 15;
        const int row = m0 + r < M ? m0 + r : M - 1;
        xsrc[i] = x + (int64_t)row * K + 4 * c;
        xdst[i] = r * kRowFloats + 4 * c;
    }
    // w: this lane's weight row (a row past N reads row N - 1) and its half of a step's codes
    const int n = n0 + 32 * wn + l32 < N ? n0 + 32 * wn + l32 : N - 1;
    const uint32_t *wp = (const uint32_t *)a.w + (int64_t)n * row_dwords + h * BITS;
    const float *sp = (const float *)a.scales + (int64_t)n * kgroups, *bp = (const float *)a.biases + (int64_t)n * kgroups;  // affine
    const uint8_t *cp = (const uint8_t *)a.scales + (int64_t)n * kgroups;                                                    // block formats: one byte a group
    float inv_enc = 1.0f;
    bool scaled = false;
    if constexpr (MODE == NVQ_NVFP4) {
        if (a.global_scale != nullptr) inv_enc = ftz(a.global_scale[0] / (448.0f * 6.0f)), scaled = true;
    }

    // The operands of two steps in registers, used in turn (set p holds the even or the odd steps), so that none is
    // copied while its loads are under way.
    f32x4_t xq[2][4];
    uint32_t cq[2][BITS];
    float sq[2], bq[2];
    uint32_t rq[2][kHalves];  // block formats: the scale codes
    auto request = [&](int step, auto p_tag) __attribute__((always_inline)) {
        constexpr int p = decltype(p_tag)::value;
        const int sc = step < steps ? step : steps - 1;  // (a step past the end fetches the last one again: no test around the loads)
#pragma unroll
        for (int i = 0; i < 4; i++) xq[p][i] = *reinterpret_cast<const f32x4_t *>(xsrc[i] + sc * kStep);
#pragma unroll
        for (int d = 0; d < BITS; d++) cq[p][d] = wp[sc * 2 * BITS + d];
        const int g = (sc * kStep + 32 * h) >> gshift;
        if constexpr (kAffine) {
            sq[p] = sp[g];
            bq[p] = bp[g];
        } else {
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) rq[p][hf] = cp[g + hf];
        }
    };

    // Four accumulators take the instructions of a step in turn: a matrix instruction waits for the one before it on the
    // same accumulator.  They are added once, at the end.
    floatx16_t acc[4];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[0][e] = acc[1][e] = acc[2][e] = acc[3][e] = 0.0f;

    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    auto multiply = [&](int step, auto p_tag, auto other_tag) __attribute__((always_inline)) {
        constexpr int p = decltype(p_tag)::value;
        float *stage = xs[p];
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<f32x4_t *>(stage + xdst[i]) = xq[p][i];
        request(step + 1, other_tag);
        // One barrier per step: the stage written now was last read two steps ago, before every wavefront's previous barrier.
        // Only the LDS writes are waited for: __syncthreads() would also wait for the loads just requested, a round trip
        // to memory per step.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        const float *xrow = stage + (32 * wm + l32) * kRowFloats + 32 * h;
        f32x4_t xa[8];
#pragma unroll
        for (int q = 0; q < 8; q++) xa[q] = *reinterpret_cast<const f32x4_t *>(xrow + 4 * q);
        float scale[kHalves], bias = 0.0f;
        if constexpr (kAffine) {
            scale[0] = sq[p], bias = bq[p];
        } else {
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) {
                scale[hf] = ftz(MODE == NVQ_NVFP4 ? e4m3_to_f32(rq[p][hf]) : e8m0_to_f32(rq[p][hf]));
                if (scaled) scale[hf] = ftz(scale[hf] * inv_enc);
            }
        }
        static_for<32>([&](auto j_tag) {
            constexpr int j = decltype(j_tag)::value;
            float wv;
            if constexpr (kAffine) {
                wv = code_to_float<BITS, j>(cq[p]) * scale[0] + bias;  // two roundings, as the CPU's weight
            } else {
                constexpr int per = 32 / BITS;
                const uint32_t c = (cq[p][j / per] >> (BITS * (j % per))) & ((1u << BITS) - 1u);
                wv = (MODE == NVQ_MXFP8 ? e4m3_to_f32(c) : e2m1_to_f32(c)) * scale[kHalves == 2 ? j / 16 : 0];
            }
            const float xv = xa[j >> 2][j & 3];
            acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(xv, wv, acc[j & 3], 0, 0, 0);
        });
    };
    request(0, P0{});
    int step = 0;
    for (; step + 2 <= steps; step += 2) {
        multiply(step, P0{}, P1{});
        multiply(step + 1, P1{}, P0{});
    }
    if (step < steps) multiply(step, P0{}, P1{});
#pragma unroll
    for (int e = 0; e < 16; e++) acc[0][e] = (acc[0][e] + acc[1][e]) + (acc[2][e] + acc[3][e]);

    // Accumulator element e of lane l is tile row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32.
    const int col = n0 + 32 * wn + l32;
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int row = m0 + 32 * wm + 8 * (e >> 2) + 4 * h + (e & 3);
        if (row < M && col < N) y[(int64_t)row * N + col] = add_row_bias<float>(a.row_bias, acc[0][e], col);
    }
}

template <int BITS, int MODE = NVQ_AFFINE>
int32_t run(const ProductArgs &a, hipStream_t s) {
    const dim3 grid((unsigned)((a.n + kTile - 1) / kTile), (unsigned)((a.m + kTile - 1) / kTile));
    hipLaunchKernelGGL((qmm_f32_kernel<BITS, MODE>), grid, dim3(256), 0, s, a);
    NVQ_LAUNCH_CHECK("qmm_f32");
    return NVQ_OK;
}

}  // namespace

// What the kernel takes: one product (no batch, no gathered pairs, no gated epilogue, not row-exact) of float32 x against
// affine or block-format weights stored [N, K] with K in whole steps of 64, where it is estimated faster than the vector kernel, which
// walks the weights once per four rows of x.  Measured, 4-bit g64, us, vector kernel -> this one: W[4096,4096] at 64 /
// 128 / 512 / 2048 rows 130 / 245 / 969 / 3850 -> 105 / 107 / 178 / 629 (109 TFLOP/s at 2048 rows); W[14336,4096] at 16 /
// 64 / 512 / 2048 rows 112 / 427 / 3366 / 13444 -> 106 / 106 / 540 / 2042 (118 TFLOP/s); a step of 64 values costs a block
// 1.64 us alone on a compute unit and 1.25 us per block that shares it, a pass of the vector kernel 1 us per 2.2 M weights.
bool qmm_f32_takes(const ProductArgs &a) {
    if (a.dtype != NVQ_F32 || a.row_exact) return false;
    if (a.batch != 1 || a.batch_ndim != 0 || a.rhs != nullptr || a.lhs != nullptr || a.glu != 0) return false;
    if (a.k < kStep || a.k % kStep != 0 || (a.mode == NVQ_AFFINE && a.group != 32 && a.group != 64 && a.group != 128)) return false;
    if (a.m < 8 || a.m > 65535 * (int64_t)kTile || a.n > 0x7FFFFFFF / 64 || (uintptr_t)a.x % 16 != 0) return false;
    // Both kernels as timed on 1078 products (fourteen weight shapes, seven formats, 8 to 512 rows): this one a step of 64
    // values at 1.64 us for a lone block and 1.25 us per block sharing a compute unit, the block formats 1.7 times that;
    // the vector kernel a pass of four rows at 1 us per 2.06 M weights with K counted in its steps of 2048 values (a row
    // of 512 costs a whole step: W[32768,512] at 8 rows 68.6 us there against 25.4 here), the block formats 2.05 times
    // that.  Choosing by them is 0.2 % above always taking the faster kernel, 1.4 x at worst.
    const bool block_format = a.mode != NVQ_AFFINE;
    const double tiles = (double)((a.m + kTile - 1) / kTile) * (double)((a.n + kTile - 1) / kTile);
    const double per_unit = 1.25 * tiles / compute_units();
    const double here = (double)(a.k / kStep) * (per_unit > 1.64 ? per_unit : 1.64) * (block_format ? 1.7 : 1.0);
    const double k_steps = (double)((a.k + 2047) / 2048) * 2048.0;
    const double there = (double)((a.m + 3) / 4) * (double)a.n * k_steps / 2.2e6 * (block_format ? 2.05 : 1.07);
    return here < there;
}

int32_t launch_qmm_f32(const ProductArgs &a, hipStream_t s) {
    if (!qmm_f32_takes(a)) return fail(NVQ_UNSUPPORTED, "quantized_matmul: the float32 matrix-core kernel does not take this product");
    if (a.mode == NVQ_MXFP4) return run<4, NVQ_MXFP4>(a, s);
    if (a.mode == NVQ_MXFP8) return run<8, NVQ_MXFP8>(a, s);
    if (a.mode == NVQ_NVFP4) return run<4, NVQ_NVFP4>(a, s);
    switch (a.bits) {
    case 1: return run<1>(a, s);
    case 2: return run<2>(a, s);
    case 3: return run<3>(a, s);
    case 4: return run<4>(a, s);
    case 5: return run<5>(a, s);
    case 6: return run<6>(a, s);
    case 8: return run<8>(a, s);
    default: return fail(NVQ_INVALID_ARGUMENT, "quantized_matmul: %d bits are not supported", a.bits);
    }
}

}  // namespace nvq
