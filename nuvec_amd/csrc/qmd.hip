// Few rows of x (passes of up to 16) times affine weights of 2, 3, 4, 5, 6 or 8 bits in groups of 32, 64 or 128, bf16 / f16,
// on the 16x16x32 matrix instruction with the weights loaded straight into the instruction's operand layout: the
// counterpart of the reference's few-row matrix-unit kernel affine_qmv_mma (crates/nuvec-kernels/src/metal/quantized.h:1722-1905:
// 1 to 16 rows, 4 and 8 bits, groups of 32, 64 and 128; routed at crates/nuvec-core/src/gpu.rs:6978-7024), here also
// for 2, 3, 5 and 6 bits.
//
// A block of W wavefronts owns 16 RT weight rows and walks K in chunks of W slices of 512 values; wavefront v owns
// slice v of the chunk.  A slice is cut into spans of 4 C values.  Lane (column n = lane % 16, quarter q = lane / 16)
// loads the C codes [C q, C q + C) of each span of its weight row — C BITS / 32 whole dwords, straight from memory into
// registers, no weight passes through the LDS — and matrix instruction j of the span takes the eight codes
// [8 j, 8 j + 8) of every quarter's chunk, i.e. the values {C q + 8 j .. + 7 : q = 0..3} of the span.
//   * C = GROUP / 4 where that is whole dwords: a span is one group, every instruction stays inside it.
//   * otherwise C = 32: a span of 128 values holds 128 / GROUP groups, each made of whole quarters; group g gets an
//     accumulator of its own whose x operand is zero in the quarters of the other groups.
// The vector units only turn codes into elements: code c becomes B + c (B = 128 in bf16, 1024 in f16) by or-ing it
// into the mantissa of the constant (8-bit codes in bf16, which has no room for them there, by conversion: B = 0).
// The 16 tile rows are 16 rows of x; per group the accumulator P and the group's sums of x (X: the same x operands
// against a weight operand of ones) give    y += scale (P - B X) + bias X.
// x is staged per wavefront in LDS, in the pair order the expansion produces; a wavefront reads only what it
// staged itself, so no block barrier is needed before the final sum of the wavefronts' partial rows.
#include "qmv_common.h"

namespace nvq {
namespace {

constexpr int kQmdSlice = 512;                 // values of K per wavefront and chunk
constexpr int kQmdPieces = kQmdSlice / 8;      // 16-byte pieces of a row of x in a slice
constexpr int kQmdRowPieces = kQmdPieces + 1;  // pieces between two rows of a slice of x: one apart in bank space
constexpr int kQmdSlices = 8;                  // slices of a block: what the LDS holds of 16 rows of x is 4096 values of K

// Codes per lane and span: 32 (a span of 128 values: a lane's load is 4 BITS bytes, a wavefront's 64 BITS / 8 bytes of
// each of 16 rows) for groups of 64 and 128, 16 for groups of 32 (where that is whole dwords).  Measured at
// W[14336,4096], 4 bits, groups of 64: 13.6 us with 16 codes (loads of 8 bytes a lane), 11.2 us with 32.
template <int MODE, int BITS, int GROUP> constexpr int qmd_chunk() {
    if (MODE != NVQ_AFFINE) return BITS == 8 ? 16 : 32;  // the block formats: 16 bytes of codes a lane (one or two groups)
    constexpr int want = GROUP == 32 ? 16 : 32;
    return (want * BITS) % 32 == 0 ? want : 32;
}

// Whether code c enters the operand as B + c by or-ing it into the constant's mantissa.
template <typename T, int BITS> constexpr bool qmd_magic() { return !(BITS == 8 && std::is_same<T, bf16_t>::value); }

// The eight values of a piece of x in the order of the expansion's pairs: (0,4)(1,5)(2,6)(3,7) for 2, 3 and 4 bits,
// (0,2)(1,3)(4,6)(5,7) for 5, 6 and 8 bits.
template <int BITS>
__device__ __forceinline__ uint4 qmd_pair_order(const uint4 q) {
    uint4 pr;
    if constexpr (BITS == 8 || BITS == 6 || BITS == 5) {
        pr.x = __builtin_amdgcn_perm(q.y, q.x, 0x05040100u);
        pr.y = __builtin_amdgcn_perm(q.y, q.x, 0x07060302u);
        pr.z = __builtin_amdgcn_perm(q.w, q.z, 0x05040100u);
        pr.w = __builtin_amdgcn_perm(q.w, q.z, 0x07060302u);
    } else {
        pr.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);
        pr.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);
        pr.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);
        pr.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);
    }
    return pr;
}

// The LEN bits (up to 32) from bit OFF of the lane's chunk, in the low bits of the result (the bits above them are the
// chunk's next ones or zeros).
template <int OFF, int LEN, int DW>
__device__ __forceinline__ uint32_t qmd_bits(const uint32_t (&dw)[DW]) {
    constexpr int i = OFF / 32, sh = OFF % 32;
    if constexpr (sh == 0) return dw[i];
    else if constexpr (sh + LEN <= 32) return dw[i] >> sh;
    else return __builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh);
}

// The weight operand of matrix instruction J from the lane's chunk of a span (DW dwords).  Written in C so that the
// compiler sees the writes that feed the matrix instruction.
template <typename T, int BITS, int DW, int J>
__device__ __forceinline__ uint4 qmd_operand(const uint32_t (&dw)[DW], uint32_t mask, uint32_t magic) {
    uint4 b;
    if constexpr (BITS == 4) {
        const uint32_t d = dw[J];
        b.x = (d & mask) | magic;
        b.y = ((d >> 4) & mask) | magic;
        b.z = ((d >> 8) & mask) | magic;
        b.w = ((d >> 12) & mask) | magic;
    } else if constexpr (BITS == 8) {
        const uint32_t d0 = dw[2 * J], d1 = dw[2 * J + 1];
        if constexpr (qmd_magic<T, BITS>()) {
            b.x = (d0 & mask) | magic;
            b.y = ((d0 >> 8) & mask) | magic;
            b.z = (d1 & mask) | magic;
            b.w = ((d1 >> 8) & mask) | magic;
        } else {
            b.x = qmf::Ops<T>::pack(qmf::ubyte_to_float<0>(d0), qmf::ubyte_to_float<2>(d0));
            b.y = qmf::Ops<T>::pack(qmf::ubyte_to_float<1>(d0), qmf::ubyte_to_float<3>(d0));
            b.z = qmf::Ops<T>::pack(qmf::ubyte_to_float<0>(d1), qmf::ubyte_to_float<2>(d1));
            b.w = qmf::Ops<T>::pack(qmf::ubyte_to_float<1>(d1), qmf::ubyte_to_float<3>(d1));
        }
    } else if constexpr (BITS == 3) {
        // 24 bits from bit 24 J of the chunk; codes 0..3 stay in the low half, codes 4..7 move to the high half
        uint32_t v;
        if constexpr (J == 0) v = dw[0];
        else if constexpr (J == 1) v = __builtin_amdgcn_alignbit(dw[1], dw[0], 24);
        else if constexpr (J == 2) v = __builtin_amdgcn_alignbit(dw[2], dw[1], 16);
        else v = dw[2] >> 8;
        const uint32_t z = (v & 0xFFFu) | ((v << 4) & 0x0FFF0000u);
        b.x = (z & mask) | magic;
        b.y = ((z >> 3) & mask) | magic;
        b.z = ((z >> 6) & mask) | magic;
        b.w = ((z >> 9) & mask) | magic;
    } else if constexpr (BITS == 6 || BITS == 5) {
        // four codes (24 or 20 bits) at a time: codes 0, 1 stay in the low half, codes 2, 3 move to the high half
        constexpr uint32_t kLow = (1u << (2 * BITS)) - 1;
        const uint32_t va = qmd_bits<8 * BITS * J, 4 * BITS>(dw), vb = qmd_bits<8 * BITS * J + 4 * BITS, 4 * BITS>(dw);
        const uint32_t za = (va & kLow) | ((va << (16 - 2 * BITS)) & (kLow << 16)), zb = (vb & kLow) | ((vb << (16 - 2 * BITS)) & (kLow << 16));
        b.x = (za & mask) | magic;
        b.y = ((za >> BITS) & mask) | magic;
        b.z = (zb & mask) | magic;
        b.w = ((zb >> BITS) & mask) | magic;
    } else {
        static_assert(BITS == 2, "2, 3, 4, 5, 6 and 8 bits");
        const uint32_t v = dw[J >> 1] >> (16 * (J & 1));
        const uint32_t z = (v & 0xFFu) | ((v << 8) & 0x00FF0000u);
        b.x = (z & mask) | magic;
        b.y = ((z >> 2) & mask) | magic;
        b.z = ((z >> 4) & mask) | magic;
        b.w = ((z >> 6) & mask) | magic;
    }
    return b;
}

template <int DW> struct QmdWords;
template <> struct QmdWords<1> { typedef uint32_t type; };
template <> struct QmdWords<2> { typedef uint2 type; };
template <> struct QmdWords<3> { struct __attribute__((aligned(4))) type { uint32_t x, y, z; }; };
template <> struct QmdWords<4> { typedef uint4 type; };
template <> struct QmdWords<5> { struct __attribute__((aligned(4))) type { uint32_t x, y, z, w, v; }; };
template <> struct QmdWords<6> { struct __attribute__((aligned(4))) type { uint32_t x, y, z, w, v, u; }; };

// DW dwords from p (whole-dword aligned; 16-byte aligned where DW is 4 or 8).
template <int DW>
__device__ __forceinline__ void qmd_load(const uint32_t *p, uint32_t (&out)[DW]) {
    if constexpr (DW == 8) {
        const uint4 a = *reinterpret_cast<const uint4 *>(p), b = *reinterpret_cast<const uint4 *>(p + 4);
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
    } else {
        const typename QmdWords<DW>::type v = *reinterpret_cast<const typename QmdWords<DW>::type *>(p);
        __builtin_memcpy(out, &v, sizeof(v));
    }
}

// LDS of a block: per wavefront its rows of x, a piece of zeros and the sums of x over the groups of its slice
// ([group][16 rows] float32); the wavefronts' partial rows, twice (the block
// walks its tiles with one barrier each: a tile's sums are read while the next tile's are written).
// LDS of a block, per wavefront: its slice of the rows of x and a piece of zeros; the sums of x over the groups of the
// slice ([group][quarter] x 4 rows, float32); its partial rows — twice where the block walks several tiles (one barrier
// each: a tile's sums are read while the next tile's are written).
template <int RM, int RT, int GROUP>
__host__ __device__ constexpr size_t qmd_lds_bytes(int slices, bool chunked, bool sums) {
    return (size_t)slices * ((RM * kQmdRowPieces + 1) * 16 + (sums ? (kQmdSlice / GROUP) * 64 : 0) + (chunked ? 1 : 2) * (size_t)RT * RM * 16 * 4);
}

// CHUNKED: K is longer than the block's wavefronts cover at once; the block owns one group of RT tiles of weight rows
// and walks K in chunks, staging x anew for each.  Otherwise x is staged once and the block walks `tiles` groups of
// tiles, the weights of a group requested one step ahead.
//
// The block formats (MXFP4, MXFP8, NVFP4 with or without a global scale) take the same walk with less arithmetic: the scaled
// conversion instructions give the dequantized elements themselves (exact: a code times a power of two; NVFP4's E4M3
// scale by one multiplication in float32), so the accumulators run over all of K and there are no sums of x.
template <typename T, int MODE, int BITS, int GROUP, int RM, int RT, bool CHUNKED>
__global__ void __launch_bounds__(64 * kQmdSlices) qmd_kernel(const ProductArgs a, const int tiles) {
    constexpr bool kBlock = MODE != NVQ_AFFINE;
    constexpr int C = qmd_chunk<MODE, BITS, GROUP>(), kSpan = 4 * C, kSpans = kQmdSlice / kSpan, J = C / 8;
    constexpr int NG = kBlock ? 1 : kSpan / GROUP;  // groups (accumulators) per span: 1, 2 or 4
    constexpr int DW = C * BITS / 32;            // dwords of codes per lane and span
    constexpr int SG = kQmdSlice / GROUP;        // groups per slice: a lane holds their scales (and biases)
    constexpr int SW = kBlock ? SG / 4 : SG / 2; // dwords of scales of a slice (one byte a group in the block formats)
    static_assert(kBlock || (NG >= 1 && NG <= 4 && NG * GROUP == kSpan && J >= 1), "a span is one, two or four whole groups");
    const int slices = __builtin_amdgcn_readfirstlane(blockDim.x >> 6);  // one wavefront per slice
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int chunk_k = slices * kQmdSlice;
    const int steps = CHUNKED ? K / chunk_k : tiles;
    const int kwords = K * BITS / 32, kgroups = K / GROUP;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slice = wave;
    const int nl = lane & 15, kq = lane >> 4;
    uint4 *xs = reinterpret_cast<uint4 *>(lds) + slice * (RM * kQmdRowPieces + 1);  // this slice's rows of x, then a piece of zeros
    floatx4_t *xsum = reinterpret_cast<floatx4_t *>(lds + (size_t)slices * (RM * kQmdRowPieces + 1) * 16) + wave * SG * 4;  // [SG][4 quarters] (affine)
    float *partial = reinterpret_cast<float *>(lds + (size_t)slices * ((RM * kQmdRowPieces + 1) * 16 + (kBlock ? 0 : SG * 64)));  // [2][RT][slices][RM][16] (chunked: one)
    const int m0 = blockIdx.y * RM;
    const bool batched = !(a.batch == 1 && a.rhs == nullptr);
    const BatchOffsets o = batched ? batch_offsets(a, blockIdx.z, kwords, kgroups) : BatchOffsets{0, 0, 0, 0, 0};
    const float factor = MODE == NVQ_NVFP4 ? qmf::nvfp4_factor(a, a.rhs != nullptr ? (int64_t)a.rhs[blockIdx.z] : 0) : 1.0f;
    const T *x = (const T *)a.x + o.x;
    const uint32_t *w = (const uint32_t *)a.w + o.w;
    using S = std::conditional_t<kBlock, uint8_t, T>;  // a scale: the element type, or one byte (E8M0; NVFP4: E4M3)
    const S *scales = (const S *)a.scales + o.s, *biases = kBlock ? nullptr : (const S *)a.biases + o.s;
    T *y = (T *)a.y + o.y;
    constexpr uint32_t ones = std::is_same<T, bf16_t>::value ? 0x3F803F80u : 0x3C003C00u;
    constexpr float base = qmd_magic<T, BITS>() ? Pair<T>::base : 0.0f;
    uint32_t mask, magic;
    asm volatile("s_mov_b32 %0, %1" : "=s"(mask) : "i"(BITS == 8 ? 0x00FF00FF : BITS == 6 ? 0x003F003F : BITS == 5 ? 0x001F001F : BITS == 4 ? 0x000F000F : BITS == 3 ? 0x00070007 : 0x00030003));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(Pair<T>::magic));

    if (lane == 0) xs[RM * kQmdRowPieces] = make_uint4(0, 0, 0, 0);
    // x operands: tile row nl is row nl of the pass; rows beyond RM read the piece of zeros
    const int a_zero = RM * kQmdRowPieces;
    const int a_live = nl < RM ? nl * kQmdRowPieces + J * kq : a_zero;
    const int a_step = nl < RM ? 1 : 0;
    const uint4 b_ones = make_uint4(ones, ones, ones, ones);

    // What a step reads from memory: the codes, scales and biases of RT tiles of weight rows for this wavefront's slice.
    struct Tile {
        uint32_t w[RT][kSpans][DW];
        uint32_t s[RT][SW], b[RT][kBlock ? 1 : SW];
    };
    // The group of RT tiles this wavefront takes in a step.
    auto group_of = [&](int step) { return CHUNKED ? (int)blockIdx.x : (int)blockIdx.x * tiles + step; };
    // Every step's loads are issued on every path (a conditional load makes the compiler wait for all loads at every
    // use); a step past the end reads the start of the weights in every lane, and nothing of it is used.
    auto fetch = [&](Tile &t, int step) {
        const bool real = step < steps;
        const int group = group_of(step);
        const int k0 = (CHUNKED ? step * chunk_k : 0) + slice * kQmdSlice;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const int n = (group * RT + rt) * 16 + nl, row = n < N ? n : N - 1;  // tail rows are computed, not stored
            const uint32_t *wp = real ? w + (int64_t)row * kwords + (k0 + C * kq) * BITS / 32 : w;
            const int stride = real ? kSpan * BITS / 32 : 0;
#pragma unroll
            for (int sp = 0; sp < kSpans; sp++) qmd_load<DW>(wp + sp * stride, t.w[rt][sp]);
            const int64_t g0 = real ? (int64_t)row * kgroups + k0 / GROUP : 0;
            qmd_load<SW>(reinterpret_cast<const uint32_t *>(scales + g0), t.s[rt]);
            if constexpr (!kBlock) qmd_load<SW>(reinterpret_cast<const uint32_t *>(biases + g0), t.b[rt]);
        }
    };
    // x of a step: a row of the slice is one 16-byte piece per lane.  A wavefront reads only what it staged itself, and
    // its LDS accesses execute in order: no block barrier.
    auto stage_x = [&](int step) {
        const int k0 = (CHUNKED ? step * chunk_k : 0) + slice * kQmdSlice;
        uint4 xq[RM];
#pragma unroll
        for (int i = 0; i < RM; i++)
            xq[i] = m0 + i < M ? *reinterpret_cast<const uint4 *>(x + (int64_t)(m0 + i) * K + k0 + 8 * lane) : make_uint4(0, 0, 0, 0);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < RM; i++) xs[i * kQmdRowPieces + lane] = kBlock ? xq[i] : qmd_pair_order<BITS>(xq[i]);  // (the conversions give the elements in order)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };
    // The sums X of the slice's groups: the x operands against a weight operand of ones give them in the accumulator
    // layout of P (the same values in the 16 lanes of a quarter); they wait in the LDS for the tiles.
    auto sums = [&]() {
        if constexpr (kBlock) return;
#pragma unroll
        for (int sp = 0; sp < kSpans; sp++)
#pragma unroll
            for (int g = 0; g < NG; g++) {
                floatx4_t acc;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] = 0.0f;
                const bool mine = NG == 1 || (C * kq) / GROUP == g;
                const uint4 *xa = xs + (mine ? a_live + (sp * 4 * J) * a_step : a_zero);
                const int step = mine ? a_step : 0;
#pragma unroll
                for (int j = 0; j < J; j++) acc = Mfma16<T>::run(xa[j * step], b_ones, acc);
                if (nl == 0) xsum[(sp * NG + g) * 4 + kq] = acc;
            }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };
    floatx4_t part[RT];
    auto clear = [&]() {
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int e = 0; e < 4; e++) part[rt][e] = 0.0f;
    };
    auto compute = [&](const Tile &t) {
        if constexpr (kBlock) {
            // Byte g of the slice's scales is group g; the lane's chunk of span sp lies in group (sp kSpan + C q) / GROUP
            // (NVFP4: and in the next one).
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                floatx4_t even = part[rt], odd;
#pragma unroll
                for (int e = 0; e < 4; e++) odd[e] = 0.0f;
#pragma unroll
                for (int sp = 0; sp < kSpans; sp++) {
                    const int g = (sp * kSpan) / GROUP + (C * kq) / GROUP;  // (sp kSpan / GROUP is a compile-time constant)
                    const uint32_t word = MODE == NVQ_NVFP4 ? (kq < 2 ? t.s[rt][2 * sp] : t.s[rt][2 * sp + 1])
                                          : MODE == NVQ_MXFP8 ? t.s[rt][sp / 2] : t.s[rt][sp];
                    float sc0, sc1;
                    if constexpr (MODE == NVQ_NVFP4) {
                        const uint32_t two = word >> (16 * (kq & 1));
                        sc0 = qmf::nvfp4_scale(two & 255u, factor), sc1 = qmf::nvfp4_scale((two >> 8) & 255u, factor);
                    } else {
                        sc0 = sc1 = ftz(e8m0_to_f32((word >> (8 * (g & 3))) & 255u));
                    }
                    const uint4 *xa = xs + a_live + (sp * 4 * J) * a_step;
#pragma unroll
                    for (int j = 0; j < J; j++) {
                        uint4 b;
                        if constexpr (MODE == NVQ_MXFP8) {
                            const uint32_t w0 = qmf::Ops<T>::mx_codes(t.w[rt][sp][2 * j], sc0), w1 = qmf::Ops<T>::mx_codes(t.w[rt][sp][2 * j + 1], sc0);
                            b.x = qmf::Ops<T>::template fp8_pair<false>(w0, sc0);
                            b.y = qmf::Ops<T>::template fp8_pair<true>(w0, sc0);
                            b.z = qmf::Ops<T>::template fp8_pair<false>(w1, sc0);
                            b.w = qmf::Ops<T>::template fp8_pair<true>(w1, sc0);
                        } else if constexpr (MODE == NVQ_MXFP4) {
                            const uint32_t w0 = qmf::Ops<T>::mx_codes(t.w[rt][sp][j], sc0);
                            b.x = qmf::Ops<T>::template fp4_pair<0>(w0, sc0);
                            b.y = qmf::Ops<T>::template fp4_pair<1>(w0, sc0);
                            b.z = qmf::Ops<T>::template fp4_pair<2>(w0, sc0);
                            b.w = qmf::Ops<T>::template fp4_pair<3>(w0, sc0);
                        } else {
                            const uint32_t w0 = t.w[rt][sp][j];
                            const float sc = j < 2 ? sc0 : sc1;  // codes 0..15 of the chunk, 16..31
                            b.x = qmf::fp4_pair_times<T, 0>(w0, sc);
                            b.y = qmf::fp4_pair_times<T, 1>(w0, sc);
                            b.z = qmf::fp4_pair_times<T, 2>(w0, sc);
                            b.w = qmf::fp4_pair_times<T, 3>(w0, sc);
                        }
                        if (j & 1) odd = Mfma16<T>::run(xa[j * a_step], b, odd);
                        else even = Mfma16<T>::run(xa[j * a_step], b, even);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; e++) part[rt][e] = even[e] + odd[e];
            }
            return;
        }
#pragma unroll
        for (int sp = 0; sp < kSpans; sp++) {
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                uint4 b[J];
#pragma unroll
                for (int j = 0; j < J; j++) {
                    if constexpr (J == 1) b[j] = qmd_operand<T, BITS, DW, 0>(t.w[rt][sp], mask, magic);
                    else if constexpr (J == 2) b[j] = j == 0 ? qmd_operand<T, BITS, DW, 0>(t.w[rt][sp], mask, magic) : qmd_operand<T, BITS, DW, 1>(t.w[rt][sp], mask, magic);
                    else
                        b[j] = j == 0   ? qmd_operand<T, BITS, DW, 0>(t.w[rt][sp], mask, magic)
                               : j == 1 ? qmd_operand<T, BITS, DW, 1>(t.w[rt][sp], mask, magic)
                               : j == 2 ? qmd_operand<T, BITS, DW, 2>(t.w[rt][sp], mask, magic)
                                        : qmd_operand<T, BITS, DW, 3>(t.w[rt][sp], mask, magic);
                }
#pragma unroll
                for (int g = 0; g < NG; g++) {
                    floatx4_t acc;
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[e] = 0.0f;
                    const bool mine = NG == 1 || (C * kq) / GROUP == g;
                    const uint4 *xa = xs + (mine ? a_live + (sp * 4 * J) * a_step : a_zero);
                    const int step = mine ? a_step : 0;
#pragma unroll
                    for (int j = 0; j < J; j++) acc = Mfma16<T>::run(xa[j * step], b[j], acc);
                    // y += scale (P - B X) + bias X for the lane's four rows of x
                    const int gi = sp * NG + g;
                    const uint32_t sw = t.s[rt][gi >> 1], bw = t.b[rt][gi >> 1];
                    const float sc = (gi & 1) ? Pair<T>::hi(sw) : Pair<T>::lo(sw), bi = (gi & 1) ? Pair<T>::hi(bw) : Pair<T>::lo(bw);
                    const float bb = base != 0.0f ? __builtin_fmaf(-base, sc, bi) : bi;
                    const floatx4_t xsg = xsum[gi * 4 + kq];
#pragma unroll
                    for (int e = 0; e < 4; e++) part[rt][e] = __builtin_fmaf(sc, acc[e], __builtin_fmaf(bb, xsg[e], part[rt][e]));
                }
            }
        }
    };
    // The wavefronts' partial rows added in a fixed order and stored.  Accumulator element e of lane
    // (n, q) is row 4 q + e of the pass.  Consecutive calls alternate between two buffers, so one barrier a call is
    // enough: a buffer is written again only after the barrier of the call in between, which every thread reaches
    // after it has read the buffer.
    auto finish = [&](int step) {
        float *buf = partial + (step & 1) * (RT * slices * RM * 16);
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (4 * kq + e < RM) buf[((rt * slices + slice) * RM + 4 * kq + e) * 16 + nl] = part[rt][e];
        __syncthreads();
        for (int out = tid; out < RT * RM * 16; out += (int)blockDim.x) {
            const int rt = out / (RM * 16), m = (out >> 4) % RM, n = out & 15;
            const float *src = buf + ((rt * slices) * RM + m) * 16 + n;
            float v = 0.0f;
#pragma unroll 4
            for (int wv = 0; wv < slices; wv++) v += src[wv * RM * 16];
            const int col = (group_of(step) * RT + rt) * 16 + n;
            if (m0 + m < M && col < N) Elem<T>::store(y, (int64_t)(m0 + m) * N + col, add_row_bias<T>(a.row_bias, v, o.bias + col));
        }
    };

    // x first, then the weights: requests return in the order they were made, and x queued behind the weights of every
    // wavefront of the compute unit would arrive last.
    clear();
    if constexpr (CHUNKED) {
        Tile t;
#pragma unroll 1
        for (int step = 0; step < steps; step++) {
            stage_x(step);  // after the last chunk's reads (same wavefront: in order)
            fetch(t, step);
            sums();
            compute(t);
        }
        finish(0);
    } else {
        stage_x(0);
        Tile ta, tb;
        fetch(ta, 0);
        sums();
#pragma unroll 1
        for (int step = 0; step < steps; step += 2) {
            fetch(tb, step + 1);
            compute(ta);
            finish(step);
            clear();
            fetch(ta, step + 2);  // the registers are free again
            if (step + 1 < steps) {
                compute(tb);
                finish(step + 1);
                clear();
            }
        }
    }
}

// Slices of a block: one per 512 values of K, the largest divisor of K / 512 up to 8 (what the LDS holds of x).
inline int qmd_slices(int64_t k) {
    const int all = (int)(k / kQmdSlice);
    for (int wv = all < kQmdSlices ? all : kQmdSlices; wv >= 1; wv--)
        if (all % wv == 0) return wv;
    return 1;
}

template <typename T, int MODE, int BITS, int GROUP, int RM, int RT>
int32_t run_qmd_sized(const ProductArgs &a, hipStream_t s) {
    const int slices = qmd_slices(a.k);
    const bool chunked = a.k > (int64_t)slices * kQmdSlice;
    const size_t lds_bytes = qmd_lds_bytes<RM, RT, GROUP>(slices, chunked, MODE == NVQ_AFFINE);
    // Groups of RT tiles of 16 weight rows; a block that stages x once walks several where there are more blocks than
    // compute units, so that x is staged less often and the blocks are one round on the chip.  Measured at
    // W[14336,4096], 3 bits, 16 rows of x: 21.8 / 14.3 / 11.8 / 18.3 us with 1 / 2 / 4 / 8 groups a block.
    const int64_t groups = (a.n + 16 * RT - 1) / (16 * RT), passes = (a.m + RM - 1) / RM;
    int tiles = 1;
    if (!chunked) {
        // rounds of blocks on the chip x (staging of x: about 2.5 us, plus 1.5 us a group walked)
        const int64_t slots = compute_units();
        double best = 0.0;
        for (int t = 1; t <= 8; t++) {
            const int64_t blocks = (groups + t - 1) / t * passes * a.batch;
            const double cost = (double)((blocks + slots - 1) / slots) * (2.5 + 1.5 * t);
            if (t == 1 || cost < best) best = cost, tiles = t;
        }
    }
    const dim3 grid((unsigned)((groups + tiles - 1) / tiles), (unsigned)passes, (unsigned)a.batch);
    void (*kernel)(const ProductArgs, int);
    if constexpr (RT == 1) kernel = chunked ? qmd_kernel<T, MODE, BITS, GROUP, RM, RT, true> : qmd_kernel<T, MODE, BITS, GROUP, RM, RT, false>;
    else kernel = qmd_kernel<T, MODE, BITS, GROUP, RM, RT, true>;  // (two tiles a wavefront: only where K is walked in chunks)
    static std::atomic<bool> configured[2] = {false, false};
    if (lds_bytes > 64 * 1024 && !configured[chunked]) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        configured[chunked] = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(slices * 64), lds_bytes, s, a, tiles);
    NVQ_LAUNCH_CHECK("qmd");
    return NVQ_OK;
}

template <typename T, int MODE, int BITS, int GROUP>
int32_t run_qmd_rows(const ProductArgs &a, hipStream_t s) {
    const bool chunked = a.k > (int64_t)qmd_slices(a.k) * kQmdSlice;
    if (chunked) {
        // A long K (walked in chunks, x staged per chunk): two tiles of weight rows per wavefront halve the staging
        // where there are weight rows enough to fill the chip with such blocks.
        const bool two = a.n * a.batch >= 8192;
        if (a.m <= 8) return two ? run_qmd_sized<T, MODE, BITS, GROUP, 8, 2>(a, s) : run_qmd_sized<T, MODE, BITS, GROUP, 8, 1>(a, s);
        return two ? run_qmd_sized<T, MODE, BITS, GROUP, 16, 2>(a, s) : run_qmd_sized<T, MODE, BITS, GROUP, 16, 1>(a, s);
    }
    return a.m <= 8 ? run_qmd_sized<T, MODE, BITS, GROUP, 8, 1>(a, s) : run_qmd_sized<T, MODE, BITS, GROUP, 16, 1>(a, s);
}

template <typename T, int BITS>
int32_t run_qmd_group(const ProductArgs &a, hipStream_t s) {
    if constexpr (BITS == 4 || BITS == 6 || BITS == 8) {
        if (a.group == 32) return run_qmd_rows<T, NVQ_AFFINE, BITS, 32>(a, s);
    }
    return a.group == 64 ? run_qmd_rows<T, NVQ_AFFINE, BITS, 64>(a, s) : run_qmd_rows<T, NVQ_AFFINE, BITS, 128>(a, s);
}

template <typename T>
int32_t run_qmd(const ProductArgs &a, hipStream_t s) {
    if (a.mode == NVQ_MXFP4) return run_qmd_rows<T, NVQ_MXFP4, 4, 32>(a, s);
    if (a.mode == NVQ_MXFP8) return run_qmd_rows<T, NVQ_MXFP8, 8, 32>(a, s);
    if (a.mode == NVQ_NVFP4) return run_qmd_rows<T, NVQ_NVFP4, 4, 16>(a, s);
    switch (a.bits) {
    case 2: return run_qmd_group<T, 2>(a, s);
    case 3: return run_qmd_group<T, 3>(a, s);
    case 4: return run_qmd_group<T, 4>(a, s);
    case 5: return run_qmd_group<T, 5>(a, s);
    case 6: return run_qmd_group<T, 6>(a, s);
    default: return run_qmd_group<T, 8>(a, s);
    }
}

}  // namespace

// Whether the kernel takes the product: bf16 / f16, affine 2, 3, 4, 5, 6 or 8 bits, K in slices of 512, 16-byte aligned
// scale and bias rows (a lane reads the scales of its slice with vector loads).
bool qmd_supported(const ProductArgs &a) {
    if (a.dtype == NVQ_F32 || a.row_exact || a.exact_weights) return false;  // (the factored form never materialises a weight)
    if (a.mode == NVQ_AFFINE) {
        if (!(a.bits == 2 || a.bits == 3 || a.bits == 4 || a.bits == 5 || a.bits == 6 || a.bits == 8)) return false;
        if (!(a.group == 64 || a.group == 128 || (a.group == 32 && (a.bits == 4 || a.bits == 6 || a.bits == 8)))) return false;  // 2, 3 and 5 bits in groups of 32: four groups per span
    }
    if (a.k < kQmdSlice || a.k % kQmdSlice != 0 || a.m < 1) return false;
    if ((a.m + 15) / 16 > 65535 || a.batch > 65535) return false;
    return ((uintptr_t)a.scales | (uintptr_t)(a.mode == NVQ_AFFINE ? a.biases : nullptr) | (uintptr_t)a.w | (uintptr_t)a.x) % 16 == 0;
}

int32_t launch_qmd(const ProductArgs &a, hipStream_t s) {
    if (!qmd_supported(a)) return fail(NVQ_UNSUPPORTED, "quantized_matmul: the few-row matrix-core kernel does not take this product");
    return a.dtype == NVQ_BF16 ? run_qmd<bf16_t>(a, s) : run_qmd<f16_t>(a, s);
}

}  // namespace nvq
