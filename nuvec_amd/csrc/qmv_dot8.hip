// One row of x against 4-bit affine weights, bf16 / f16, K in whole chunks of 2048 up to 14336: the decode product y[1,N] = x . dequantize(w)^T
// with the integer dot-product instruction.  Values follow nuvec's CPU product (reference:
// crates/nuvec-core/src/kernels.rs:1091-1142) within the stated tolerance, in the factored form of the reference's device
// kernels, scale * sum(x * code) + bias * sum(x) per group (crates/nuvec-kernels/src/metal/quantized.h:247-360, 876-988).
//
// Why integers.  The decode kernel that turns a code into an element of the activation type spends eleven vector
// instructions per eight weights (three shifts, four mask-and-or, four two-element dot products); at W[14336,4096] that is
// 3.5 us of issue time on every SIMD, which the 4.7 us of memory time does not hide.  Here x is made fixed point once per
// block: a lane's slice of 32 values shares the exponent e of its largest magnitude, and every value becomes the 16-bit
// integer round(x * 2^(14-e)) + 32768, whose four nibbles are spread over four operand dwords in the order of the codes.
// v_dot8_u32_u4 then multiplies eight packed codes, exactly as they lie in memory, with eight nibbles of x: five
// instructions per eight weights (four limbs and the codes' own sum, which removes the offset), no expansion at all:
//     sum code * x  =  2^(e-14) * (sum_j 16^j dot8(codes, limb_j) - 32768 * dot8(codes, ones)).
// The integer sums are exact; x is rounded to 2^-15 of its slice's largest binade, far below the element type's own step
// for every value that matters to the sum.  A slice that holds an infinity or a NaN gives NaN.
//
// Work split.  A block of eight wavefronts owns 8 R consecutive weight rows (R chosen on the host so that the blocks
// about fill the chip once); wavefront v takes rows v, v + 8, ... of them, lane l the values [32 l, 32 l + 32) of each
// chunk of 2048, i.e. one 16-byte load per chunk: a wavefront-wide load reads 1 KB of consecutive bytes.  The block
// requests x first, then the first rows' weights, turns x into limbs (LDS, one barrier) while those are on their way and
// keeps the limbs in registers for all of its rows; from then on every wavefront requests two rows ahead of the one it
// works on and shares nothing, so the loads never wait for arithmetic.  The R row sums of a wavefront are folded across its
// lanes in one pass (half-wavefront and 16-lane-row swaps, then moves inside a row).
//
// Several rows of x.  A block may carry the limbs of up to four rows of x (MX; 16 registers per lane, row and chunk) and
// multiply every weight row with each of them: the codes, their sum and the scale and bias are fetched once.  The rows
// share nothing else, so each has the bits of its one-row product whatever MX is: a row-exact product of many rows walks
// the weights once per four rows, and two to four ordinary rows take one pass.
#include <type_traits>
#include <utility>

#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

constexpr int kWaves = 8;       // wavefronts of a block
constexpr int kLimbBits = 16;   // x in fixed point: four nibbles, offset 2^15

template <int... I, class F>
__device__ __forceinline__ void static_for_each(std::integer_sequence<int, I...>, F &&f) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) { static_for_each(std::make_integer_sequence<int, N>{}, f); }

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_max(uint32_t v) {
    return max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true));
}
// Lanes 32..63 of `a` change places with lanes 0..31 of `b`; the odd rows of 16 lanes of `a` with the even rows of `b`.
// Written as assembly: the compiler's builtins return only the first of the two results.  The idle cycles on either side
// keep the instructions clear of their neighbours' results, which the compiler does not track through assembly.
__device__ __forceinline__ void swap_halves(float &a, float &b) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void swap_rows(float &a, float &b) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b)); }

template <typename T> __device__ __forceinline__ float pair_lo(uint32_t p);
template <typename T> __device__ __forceinline__ float pair_hi(uint32_t p);
template <> __device__ __forceinline__ float pair_lo<bf16_t>(uint32_t p) { return u2f(p << 16); }
template <> __device__ __forceinline__ float pair_hi<bf16_t>(uint32_t p) { return u2f(p & 0xFFFF0000u); }
template <> __device__ __forceinline__ float pair_lo<f16_t>(uint32_t p) { return (float)__builtin_bit_cast(f16_t, (uint16_t)p); }
template <> __device__ __forceinline__ float pair_hi<f16_t>(uint32_t p) { return (float)__builtin_bit_cast(f16_t, (uint16_t)(p >> 16)); }

// Eight values of x (a 16-byte piece, as loaded) -> their four limb dwords, the scale that undoes the fixed point, and
// their sum.  The exponent is shared by the four pieces of a slice, which sit in adjacent lanes.
template <typename T>
__device__ __forceinline__ void to_limbs(const uint4 piece, uint4 &limbs, float &down, float &sum) {
    const uint32_t q[4] = {piece.x, piece.y, piece.z, piece.w};
    float xv[8];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        xv[i] = (i & 1) ? pair_hi<T>(q[i >> 1]) : pair_lo<T>(q[i >> 1]);
        m = max(m, f2u(xv[i]) & 0x7FFFFFFFu);
    }
    m = dpp_max<0xB1>(m);  // quad_perm [1,0,3,2]
    m = dpp_max<0x4E>(m);  // quad_perm [2,3,0,1]
    int e = (int)(m >> 23);                  // biased exponent of the slice's largest magnitude
    e = e < kLimbBits ? kLimbBits : e;       // (tiny slices: the scale below stays a normal number)
    const float up = u2f((uint32_t)(127 + 127 + kLimbBits - 2 - e) << 23);  // 2^(14 - (e - 127)): |x| * up < 2^15
    down = e == 255 ? u2f(0x7FC00000u) : u2f((uint32_t)(e - (kLimbBits - 2)) << 23);
    uint32_t v[8];
    sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        sum += xv[i];
        // 1.5 * 2^23 + 2^15 + x * up: the low 16 bits of the result are round(x * up) + 32768 (ties to even)
        v[i] = f2u(__builtin_fmaf(xv[i], up, 12582912.0f + 32768.0f));
    }
    sum = dpp_add<0xB1>(sum);
    sum = dpp_add<0x4E>(sum);
    // the low bytes of v0..v3 and v4..v7, then their second bytes
    const uint32_t la = __builtin_amdgcn_perm(__builtin_amdgcn_perm(v[3], v[2], 0x0C0C0400u) << 16, __builtin_amdgcn_perm(v[1], v[0], 0x0C0C0400u), 0x07060100u);
    const uint32_t lb = __builtin_amdgcn_perm(__builtin_amdgcn_perm(v[7], v[6], 0x0C0C0400u) << 16, __builtin_amdgcn_perm(v[5], v[4], 0x0C0C0400u), 0x07060100u);
    const uint32_t ha = __builtin_amdgcn_perm(__builtin_amdgcn_perm(v[3], v[2], 0x0C0C0501u) << 16, __builtin_amdgcn_perm(v[1], v[0], 0x0C0C0501u), 0x07060100u);
    const uint32_t hb = __builtin_amdgcn_perm(__builtin_amdgcn_perm(v[7], v[6], 0x0C0C0501u) << 16, __builtin_amdgcn_perm(v[5], v[4], 0x0C0C0501u), 0x07060100u);
    // the low nibbles of the eight bytes of (a, b), packed into eight nibbles
    auto squeeze = [](uint32_t ea, uint32_t eb) {
        const uint32_t ta = ea | (ea >> 4), tb = eb | (eb >> 4);
        return __builtin_amdgcn_perm(tb, ta, 0x06040200u);
    };
    const uint32_t k = 0x0F0F0F0Fu;
    limbs.x = squeeze(la & k, lb & k);
    limbs.y = squeeze((la >> 4) & k, (lb >> 4) & k);
    limbs.z = squeeze(ha & k, hb & k);
    limbs.w = squeeze((ha >> 4) & k, (hb >> 4) & k);
}

// S: chunks of 2048 values of K.  R: weight rows per wavefront.  MX: rows of x per block.
// Grid: (blocks of 8 R weight rows, groups of MX rows of x).
template <typename T, int S, int R, int MX>
__global__ void __launch_bounds__(kWaves * 64) qmv4_dot8_kernel(const ProductArgs a) {
    static_assert(R >= 1 && R <= 8 && S >= 1 && S <= 7 && MX >= 1 && MX <= 4, "one batched reduction of up to eight rows per row of x");
    // Rows whose loads run ahead of the arithmetic: two; one where a row is 4 KB and more per wavefront (a row ahead then
    // already keeps 8 x 4 KB per compute unit under way, and the registers hold the limbs of a long x).
    constexpr int kAhead = S >= 4 ? 1 : 2;
    constexpr int kRowPieces = S * 256;                    // 16-byte pieces of a row of x
    constexpr int kPieces = MX * kRowPieces;
    constexpr int kPerThread = (kPieces + 511) / 512;
    constexpr int kRowQuads = S * 64;                      // 16-byte pieces of a row of codes
    __shared__ uint4 x_limbs[MX][S][4][64];                // [row][chunk][dword t of the slice][lane]: limbs 0..3 of values 8 t .. 8 t + 7
    __shared__ float2 x_meta[MX][S][64];                   // [row][chunk][lane]: (2^(e-14), sum of the slice's x)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N = (int)a.n, M = (int)a.m;
    const int gshift = a.group == 32 ? 5 : a.group == 64 ? 6 : 7;
    const int kgroups = (S * 2048) >> gshift;
    const int m0 = blockIdx.y * MX;                        // this block's first row of x
    const T *x = (const T *)a.x;
    T *y = (T *)a.y;
    const T *scales = (const T *)a.scales, *biases = (const T *)a.biases;

    // x first: it is needed first (a row past M reads row M - 1 and is not stored)
    uint4 xg[kPerThread];
#pragma unroll
    for (int p = 0; p < kPerThread; p++) {
        const int piece = tid + p * 512, pc = piece < kPieces ? piece : kPieces - 1;
        const int mr = m0 + pc / kRowPieces < M ? m0 + pc / kRowPieces : M - 1;
        xg[p] = reinterpret_cast<const uint4 *>(x + (int64_t)mr * (S * 2048))[pc % kRowPieces];
    }
    __builtin_amdgcn_sched_barrier(0);
    // Row j of this wavefront: its codes (one 16-byte load per chunk, read once: non-temporal), and the scale and bias of
    // the lane's slice of each chunk.  Rows past N read row N - 1 and are not stored.
    const int row0 = blockIdx.x * (kWaves * R) + wave;
    uint4 wq[R][S];
    T sr[R][S], br[R][S];
    auto request = [&](auto jt) {
        constexpr int j = decltype(jt)::value;
        if constexpr (j < R) {
            const int row = row0 + j * kWaves < N ? row0 + j * kWaves : N - 1;
            const uint4 *p = reinterpret_cast<const uint4 *>(a.w) + (int64_t)row * kRowQuads + lane;
            const int64_t g = (int64_t)row * kgroups + ((32 * lane) >> gshift);
#pragma unroll
            for (int u = 0; u < S; u++) wq[j][u] = stream_load(p + 64 * u);
#pragma unroll
            for (int u = 0; u < S; u++) sr[j][u] = scales[g + ((2048 * u) >> gshift)], br[j][u] = biases[g + ((2048 * u) >> gshift)];
            __builtin_amdgcn_sched_barrier(0);  // rows are requested in the order they are used
        }
    };
    static_for<kAhead>(request);

    // x -> limbs, through LDS to the lanes that use them
#pragma unroll
    for (int p = 0; p < kPerThread; p++) {
        const int piece = tid + p * 512;
        uint4 limbs;
        float down, sum;
        to_limbs<T>(xg[p], limbs, down, sum);
        if (piece < kPieces) {
            const int mr = piece / kRowPieces, q = piece % kRowPieces;
            x_limbs[mr][q >> 8][q & 3][(q & 255) >> 2] = limbs;
            if ((q & 3) == 0) x_meta[mr][q >> 8][(q & 255) >> 2] = make_float2(down, sum);
        }
    }
    __syncthreads();
    uint4 xr[MX][S][4];
    float2 xm[MX][S];
#pragma unroll
    for (int mr = 0; mr < MX; mr++)
#pragma unroll
        for (int u = 0; u < S; u++) {
#pragma unroll
            for (int t = 0; t < 4; t++) xr[mr][u][t] = x_limbs[mr][u][t][lane];
            xm[mr][u] = x_meta[mr][u][lane];
        }
    uint32_t ones;
    asm volatile("s_mov_b32 %0, 0x11111111" : "=s"(ones));  // (held in a scalar register: a literal would be re-materialised per use)

    float sums[MX][8];
#pragma unroll
    for (int mr = 0; mr < MX; mr++)
#pragma unroll
        for (int j = 0; j < 8; j++) sums[mr][j] = 0.0f;
    auto row = [&](auto jt) {
        constexpr int j = decltype(jt)::value;
        request(std::integral_constant<int, j + kAhead>{});
        float acc[MX];
#pragma unroll
        for (int mr = 0; mr < MX; mr++) acc[mr] = 0.0f;
#pragma unroll
        for (int u = 0; u < S; u++) {
            const uint32_t d[4] = {wq[j][u].x, wq[j][u].y, wq[j][u].z, wq[j][u].w};
            uint32_t cs = 0;
#pragma unroll
            for (int t = 0; t < 4; t++) cs = __builtin_amdgcn_udot8(d[t], ones, cs, false);
            const float sc = Elem<T>::load(&sr[j][u], 0), bi = Elem<T>::load(&br[j][u], 0);
#pragma unroll
            for (int mr = 0; mr < MX; mr++) {
                uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    a0 = __builtin_amdgcn_udot8(d[t], xr[mr][u][t].x, a0, false);
                    a1 = __builtin_amdgcn_udot8(d[t], xr[mr][u][t].y, a1, false);
                    a2 = __builtin_amdgcn_udot8(d[t], xr[mr][u][t].z, a2, false);
                    a3 = __builtin_amdgcn_udot8(d[t], xr[mr][u][t].w, a3, false);
                }
                uint32_t h = (a3 << 4) + a2;
                h = (h << 4) + a1;
                h = (h << 4) + a0;
                const int total = (int)h - (int)(cs << (kLimbBits - 1));  // sum code * round(x * up): below 2^25 in magnitude
                acc[mr] = __builtin_fmaf(sc * xm[mr][u].x, (float)total, __builtin_fmaf(bi, xm[mr][u].y, acc[mr]));
            }
        }
#pragma unroll
        for (int mr = 0; mr < MX; mr++) sums[mr][j] = acc[mr];
    };
    static_for<R>(row);

    // Eight rows' sums at once, per row of x: after the two swaps and the select, lane l carries row (l >> 3) & 7, and
    // three moves inside its eight lanes finish the sum.
#pragma unroll
    for (int mr = 0; mr < MX; mr++) {
        float s4[4], s2[2];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float p = sums[mr][j], q = sums[mr][j + 4];
            swap_halves(p, q);
            s4[j] = p + q;
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            float p = s4[j], q = s4[j + 2];
            swap_rows(p, q);
            s2[j] = p + q;
        }
        const float u0 = dpp_add<0x128>(s2[0]), u1 = dpp_add<0x128>(s2[1]);  // row_ror:8
        float total = (lane & 8) ? u1 : u0;
        total = dpp_add<0x141>(total);  // row_half_mirror
        total = dpp_add<0xB1>(total);   // quad_perm [1,0,3,2]
        total = dpp_add<0x4E>(total);   // quad_perm [2,3,0,1]
        const int j = (lane >> 3) & 7, n = row0 + j * kWaves;
        if ((lane & 7) == 0 && j < R && n < N && m0 + mr < M)
            Elem<T>::store(y, (int64_t)(m0 + mr) * N + n, add_row_bias<T>(a.row_bias, total, n));
    }
}

template <typename T, int S, int MX>
int32_t run_rows(const ProductArgs &a, int r, hipStream_t s) {
    const dim3 grid((unsigned)((a.n + kWaves * r - 1) / (kWaves * r)), (unsigned)((a.m + MX - 1) / MX)), block(kWaves * 64);
    switch (r) {
    case 1: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 1, MX>), grid, block, 0, s, a); break;
    case 2: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 2, MX>), grid, block, 0, s, a); break;
    case 3: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 3, MX>), grid, block, 0, s, a); break;
    case 4: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 4, MX>), grid, block, 0, s, a); break;
    case 5: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 5, MX>), grid, block, 0, s, a); break;
    case 6: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 6, MX>), grid, block, 0, s, a); break;
    case 7: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 7, MX>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((qmv4_dot8_kernel<T, S, 8, MX>), grid, block, 0, s, a); break;
    }
    NVQ_LAUNCH_CHECK("qmv4_dot8");
    return NVQ_OK;
}
template <typename T, int S>
int32_t run_x_rows(const ProductArgs &a, int r, hipStream_t s) {
    const int mx = a.m >= 4 ? 4 : (int)a.m;  // rows of x per block (more rows: groups of four)
    return mx == 1 ? run_rows<T, S, 1>(a, r, s) : mx == 2 ? run_rows<T, S, 2>(a, r, s) : mx == 3 ? run_rows<T, S, 3>(a, r, s) : run_rows<T, S, 4>(a, r, s);
}

}  // namespace

// Rows per wavefront: the fewest with which the blocks fit the chip at once (one block per compute unit), at most eight.
int qmv_dot8_rows_per_wave(int64_t n, int cus) {
    const int64_t r = (n + (int64_t)kWaves * cus - 1) / ((int64_t)kWaves * cus);
    return r < 1 ? 1 : r > 8 ? 8 : (int)r;
}

// What the kernel takes: single products (no batch, no gathered pairs, no gated epilogue) of 4-bit affine weights stored
// [N, K] with K = 2048, 4096 (several rows of x) or 6144 .. 14336 (one row), bf16 / f16, 1024 outputs and more (rows of fewer outputs materialise the CPU's weights
// elsewhere), operands 16-byte aligned.  One row of x (two against 8192 weight rows and more) in one pass over the
// weights, or the rows of a row-exact product four per pass: every row has the bits of its one-row product either way.
bool qmv_dot8_takes(const ProductArgs &a) {
    if (a.mode != NVQ_AFFINE || a.bits != 4 || (a.dtype != NVQ_BF16 && a.dtype != NVQ_F16)) return false;
    if (a.batch != 1 || a.batch_ndim != 0 || a.rhs != nullptr || a.lhs != nullptr || a.glu != 0 || a.exact_weights) return false;
    // K in whole chunks of 2048 up to 14336 (us against the float decode kernel: W[4096,14336] 8.85 -> 8.26, W[14336,8192]
    // 13.6 -> 12.1, W[8192,6144] 7.9 -> 6.3; at K = 16384 the limbs no longer fit the registers: 10.5 -> 12.4, not taken)
    if (a.k < 2048 || a.k > 14336 || a.k % 2048 != 0) return false;
    if (a.k > 4096 && a.m != 1) return false;  // (the limbs of one long row of x fill the registers)
    if (a.group != 32 && a.group != 64 && a.group != 128) return false;
    if (a.n < 1024 || a.n > 0x7FFFFFFF / 128 || a.m < 1 || a.m > 65535) return false;
    // two rows where the matrix is large (W[14336,4096]: 8.7 us against 9.8 on the 16x16x32 decode kernel; three and four rows
    // cost 1.7 us each here and stay there: 10.4 / 12.3 against 9.8 / 9.9 us); a row-exact product any number, four per pass
    if (!(a.m == 1 || (a.m == 2 && a.n >= 8192) || a.row_exact)) return false;  // up to four rows in one pass; a row-exact product any number, four per pass
    return ((uintptr_t)a.w | (uintptr_t)a.x) % 16 == 0;
}

template <typename T>
int32_t run_chunks(const ProductArgs &a, int r, hipStream_t s) {
    switch (a.k / 2048) {
    case 1: return run_x_rows<T, 1>(a, r, s);
    case 2: return run_x_rows<T, 2>(a, r, s);
    // longer rows (K = 6144 .. 14336): one row of x per pass
    case 3: return run_rows<T, 3, 1>(a, r, s);
    case 4: return run_rows<T, 4, 1>(a, r, s);
    case 5: return run_rows<T, 5, 1>(a, r, s);
    case 6: return run_rows<T, 6, 1>(a, r, s);
    default: return run_rows<T, 7, 1>(a, r, s);
    }
}

int32_t launch_qmv_dot8(const ProductArgs &a, hipStream_t s) {
    if (!qmv_dot8_takes(a)) return fail(NVQ_UNSUPPORTED, "quantized_matmul: the integer decode kernel does not take this product");
    const int r = qmv_dot8_rows_per_wave(a.n, compute_units());
    return a.dtype == NVQ_BF16 ? run_chunks<bf16_t>(a, r, s) : run_chunks<f16_t>(a, r, s);
}

}  // namespace nvq
