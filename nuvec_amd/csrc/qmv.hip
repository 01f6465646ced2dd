// Few-row quantized products y = x . dequantize(w)^T for gfx950: the decode-shaped path.
// Values follow nuvec's CPU product (reference: crates/nuvec-core/src/kernels.rs:1091-1142)
// within the stated tolerance; the factored form per group,
//     scale * sum(x * code) + bias * sum(x),
// is the one the reference's device kernels use (crates/nuvec-kernels/src/metal/quantized.h:247-360).
//
// Work split.  A wavefront owns RN consecutive weight rows and walks K in steps of 2048
// values; inside a step lane l owns the 32 values [32 l, 32 l + 32), which are `bits`
// consecutive dwords of the packed row (one 128-bit load at 4 bits) and lie inside one
// quantization group (groups are 32, 64 or 128 values).  A wavefront-wide load therefore
// reads 64*4*bits contiguous bytes of one row.  The x slice of the step is decoded once and
// reused for the RN rows; the RN*RM partial sums stay in registers and are folded across
// the wavefront once, at the end.  No LDS and no barriers: HBM latency is covered by the RN
// independent row loads each lane has in flight.
#include "nvq_device.h"
#include "nvq_internal.h"
#include "qmf_kernel.h"  // matrix-instruction wrappers
#include "qmv_common.h"

namespace nvq {
namespace {

constexpr int kStep = 64 * 32;        // values of K per wavefront step

// v + (v moved across lanes by a DPP control); lanes the control does not feed add 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, true);
    return v + __int_as_float(moved);
}

// Sum over the wavefront in VALU data-parallel-primitive steps (no LDS traffic): shifts by
// 1, 2, 4, 8 inside each row of 16 lanes, then the row totals carried into the next rows.
// The total is valid in lane 63 only.
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v = dpp_add<0x111, 0xF>(v);  // row_shr:1
    v = dpp_add<0x112, 0xF>(v);  // row_shr:2
    v = dpp_add<0x114, 0xF>(v);  // row_shr:4
    v = dpp_add<0x118, 0xF>(v);  // row_shr:8
    v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

// (a & mask) | magic in one instruction.  The mask travels in a scalar register and the
// constant in a vector register: a three-operand VALU instruction of this ISA takes no
// literal and at most one scalar operand, so the compiler would otherwise emit an AND and an OR.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask_sgpr, uint32_t magic_vgpr) {
    uint32_t d;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask_sgpr), "v"(magic_vgpr));
    return d;
}

// Loads the lane's `BITS` dwords of a packed row.
template <int BITS>
__device__ __forceinline__ void load_words(const uint32_t *p, uint32_t (&d)[BITS]) {
    if constexpr (BITS == 4) {
        const uint4 q = stream_load(reinterpret_cast<const uint4 *>(p));
        d[0] = q.x; d[1] = q.y; d[2] = q.z; d[3] = q.w;
    } else if constexpr (BITS == 8) {
        const uint4 q0 = stream_load(reinterpret_cast<const uint4 *>(p)), q1 = stream_load(reinterpret_cast<const uint4 *>(p) + 1);
        d[0] = q0.x; d[1] = q0.y; d[2] = q0.z; d[3] = q0.w;
        d[4] = q1.x; d[5] = q1.y; d[6] = q1.z; d[7] = q1.w;
    } else if constexpr (BITS == 2) {
        const uint2 q = stream_load(reinterpret_cast<const uint2 *>(p));
        d[0] = q.x; d[1] = q.y;
    } else {
#pragma unroll
        for (int i = 0; i < BITS; i++) d[i] = stream_load(p + i);
    }
}

// Code `i` (0..31) of the lane's BITS dwords: value i sits at bit i*BITS of the stream
// (reference: kernels.rs:749-756).
template <int BITS>
__device__ __forceinline__ uint32_t code_at(const uint32_t (&d)[BITS], int i) {
    constexpr uint32_t mask = (1u << BITS) - 1u;
    const int bit = i * BITS, word = bit >> 5, sh = bit & 31;
    uint32_t v = d[word] >> sh;
    if (sh + BITS > 32) v |= d[word + 1] << (32 - sh);
    return v & mask;
}

// ── general kernel: any bit width, any element type, affine or a floating-point block format ──
// A block of eight wavefronts shares the x slice of one K step (2048 values) through LDS, converted to
// float32 once and laid out [piece][lane] so that a lane's eight 16-byte reads of its 32 values are free of
// bank conflicts, together with the sums of the 32-value slices (the bias term).  A wavefront owns one
// weight row: per step a lane loads the BITS dwords of its 32 codes (the wavefront's loads are one
// contiguous piece of the row), extracts them at compile-time bit positions, converts and accumulates in
// float32.  Every load of a step is issued before the first use.  MODE: NVQ_AFFINE, or NVQ_MXFP4 /
// NVQ_MXFP8 / NVQ_NVFP4 (E2M1 or E4M3 values; E8M0 scales per 32 or E4M3 scales per 16 values, a lane's
// slice then spanning two groups).
// EXACT (affine codes, 16-bit elements): every weight is materialised as nuvec's CPU product holds it, round(round(code *
// scale) + bias) in the element type (kernels.rs:835-859), instead of the factored float32 form.
template <typename T, int BITS, int MODE, int RM, bool EXACT = false>
__global__ void __launch_bounds__(512) qmv_lds_kernel(const ProductArgs a) {
    constexpr int kBlockWaves = 8;
    constexpr int kPer = 4;  // values of one x row per thread and step: 2048 / 512
    constexpr bool kAffine = MODE == NVQ_AFFINE;
    constexpr int kHalves = MODE == NVQ_NVFP4 ? 2 : 1;  // groups per lane slice
    __shared__ float4 x_vals[RM][8][64];  // [row][piece][lane]: values 4 piece .. + 4 of the lane's 32
    __shared__ float x_sums[RM][64];      // [row][lane]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = kAffine ? (a.group == 32 ? 5 : a.group == 64 ? 6 : 7) : (MODE == NVQ_NVFP4 ? 4 : 5);
    const int n = __builtin_amdgcn_readfirstlane(blockIdx.x * kBlockWaves + wave);
    const int nc = n < N ? n : N - 1;  // tail rows are computed, not stored
    const int m0 = blockIdx.y * RM;
    const int row_dwords = (K * BITS) >> 5, kgroups = K >> gshift;  // NVFP4 rows may end in half a slice (K % 32 == 16)
    const BatchOffsets o = batch_offsets(a, blockIdx.z, row_dwords, kgroups);
    const T *x = (const T *)a.x + o.x;
    const uint32_t *wrow = (const uint32_t *)a.w + o.w + (int64_t)nc * row_dwords;
    T *y = (T *)a.y + o.y;

    float acc[RM];
#pragma unroll
    for (int i = 0; i < RM; i++) acc[i] = 0.0f;

    // Everything a step reads from memory: the thread's four values of each x row (one vector load), the lane's codes
    // and its group's scale and bias as stored.  The next step's are requested before the current step is computed, so
    // a product of two steps (K = 4096) pays the memory latency once.
    using S = std::conditional_t<kAffine, T, uint8_t>;
    struct Step {
        float xin[RM][kPer];
        uint32_t d[BITS];
        S sc[kHalves], bi;
    };
    auto fetch = [&](int k0) {
        Step st;
        const int kx = k0 + tid * kPer;
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const bool have = kx < K && m0 + i < M;
            const T *px = x + (have ? (int64_t)(m0 + i) * K + kx : 0);  // K is a multiple of 16 and x 16-byte aligned
            if constexpr (sizeof(T) == 4) {
                const float4 v = *reinterpret_cast<const float4 *>(px);
                st.xin[i][0] = have ? v.x : 0.0f; st.xin[i][1] = have ? v.y : 0.0f;
                st.xin[i][2] = have ? v.z : 0.0f; st.xin[i][3] = have ? v.w : 0.0f;
            } else {
                const uint2 v = *reinterpret_cast<const uint2 *>(px);
                T e[4];
                __builtin_memcpy(e, &v, 8);
#pragma unroll
                for (int j = 0; j < kPer; j++) st.xin[i][j] = have ? Elem<T>::load(e, j) : 0.0f;
            }
        }
        const int kb = k0 + lane * 32;
        const int kc = kb < K ? kb : 0;  // an absent slice reads valid memory; its x is zero
        // NVFP4: a row of K % 32 == 16 values ends in a slice of one group; its absent half reads the present one
        // again (codes and scale) and meets x = 0
        const bool second = MODE != NVQ_NVFP4 || kc + 16 < K;
        if constexpr (MODE == NVQ_NVFP4) {
            const uint2 *p = reinterpret_cast<const uint2 *>(wrow + (kc >> 3));
            const uint2 lo = stream_load(p), hi = stream_load(p + (second ? 1 : 0));
            st.d[0] = lo.x; st.d[1] = lo.y; st.d[2] = hi.x; st.d[3] = hi.y;
        } else {
            load_words<BITS>(wrow + (kc >> 5) * BITS, st.d);
        }
        const int64_t g = (int64_t)nc * kgroups + (kc >> gshift);
        if constexpr (kAffine) {
            st.sc[0] = ((const T *)a.scales + o.s)[g];
            st.bi = ((const T *)a.biases + o.s)[g];
        } else {
            const uint8_t *sp = (const uint8_t *)a.scales + o.s + g;
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) st.sc[hf] = sp[second ? hf : 0];
            st.bi = 0;
        }
        return st;
    };
    constexpr bool exact = EXACT;
    float inv_enc = 1.0f;
    bool scaled = false;
    if constexpr (MODE == NVQ_NVFP4) {
        // kernels.rs:992-998: a global scale g turns every group scale into ftz(scale * ftz(g / (448 * 6)));
        // a gather has one g per expert (quantized.rs:620-636)
        if (a.global_scale != nullptr) {
            const float g = a.global_scale[a.rhs != nullptr ? min((int64_t)a.rhs[blockIdx.z], a.experts - 1) : 0];
            inv_enc = ftz(g / (448.0f * 6.0f));
            scaled = true;
        }
    }

    Step cur = fetch(0);
    for (int k0 = 0; k0 < K; k0 += kStep) {
        const Step nxt = fetch(k0 + kStep);  // past the end: valid addresses, nothing of it is used
        const auto &xin = cur.xin;
        const auto &d = cur.d;
        float sc[kHalves], bi = 0.0f;
        if constexpr (kAffine) {
            sc[0] = Elem<T>::load(&cur.sc[0], 0);
            bi = Elem<T>::load(&cur.bi, 0);
        } else {
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) {
                sc[hf] = ftz(MODE == NVQ_NVFP4 ? e4m3_to_f32(cur.sc[hf]) : e8m0_to_f32(cur.sc[hf]));
                if (scaled) sc[hf] = ftz(sc[hf] * inv_enc);
            }
        }
        if (k0 != 0) __syncthreads();  // the previous step's readers are done with the LDS
#pragma unroll
        for (int i = 0; i < RM; i++) {
            // thread t holds values 4 t .. 4 t + 3 of the step: piece t % 8 of lane t / 8
            x_vals[i][tid & 7][tid >> 3] = make_float4(xin[i][0], xin[i][1], xin[i][2], xin[i][3]);
            float sum = (xin[i][0] + xin[i][1]) + (xin[i][2] + xin[i][3]);
            sum += __shfl_xor(sum, 1);  // the eight pieces of a lane's slice sit in adjacent threads
            sum += __shfl_xor(sum, 2);
            sum += __shfl_xor(sum, 4);
            if ((tid & 7) == 0) x_sums[i][tid >> 3] = sum;
        }
        __syncthreads();
        float dot[RM][kHalves];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) dot[i][hf] = 0.0f;
#pragma unroll
        for (int p = 0; p < 8; p++) {
            constexpr int kPiecesPerHalf = 8 / kHalves;
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t c = code_at<BITS>(d, 4 * p + j);
                v[j] = kAffine ? (float)c : (MODE == NVQ_MXFP8 ? e4m3_to_f32(c) : e2m1_to_f32(c));
                if constexpr (exact) v[j] = Elem<T>::add(Elem<T>::mul(v[j], sc[0]), bi);  // the weight as the CPU holds it
            }
#pragma unroll
            for (int i = 0; i < RM; i++) {
                const float4 xv = x_vals[i][p][lane];
                float t = dot[i][p / kPiecesPerHalf];
                t = __builtin_fmaf(xv.x, v[0], t);
                t = __builtin_fmaf(xv.y, v[1], t);
                t = __builtin_fmaf(xv.z, v[2], t);
                t = __builtin_fmaf(xv.w, v[3], t);
                dot[i][p / kPiecesPerHalf] = t;
            }
        }
#pragma unroll
        for (int i = 0; i < RM; i++) {
            if constexpr (kAffine) {
                acc[i] = exact ? acc[i] + dot[i][0] : __builtin_fmaf(sc[0], dot[i][0], __builtin_fmaf(bi, x_sums[i][lane], acc[i]));
            } else {
#pragma unroll
                for (int hf = 0; hf < kHalves; hf++) acc[i] = __builtin_fmaf(sc[hf], dot[i][hf], acc[i]);
            }
        }
        cur = nxt;
    }
#pragma unroll
    for (int i = 0; i < RM; i++) {
        const float v = wave_sum_lane63(acc[i]);
        if (lane == 63 && n < N && m0 + i < M) Elem<T>::store(y, (int64_t)(m0 + i) * N + n, add_row_bias<T>(a.row_bias, v, o.bias + n));
    }
}

// What a lane of the decode kernels reads of the scales of its 32 values: the element (affine), NVFP4's two bytes at
// once, or one byte.
constexpr int kAffine8 = 64;  // as a MODE of the decode kernels: affine codes of 8 bits (NVQ_AFFINE there means 4 bits)
constexpr int kAffine3 = 65;  // ... and of 3 bits: a lane's 32 codes are three dwords, carried in a uint4
constexpr int kAffine6 = 66;  // ... of 6 bits: six dwords, three to a uint4
constexpr int kAffine5 = 67;  // ... of 5 bits: five dwords, three and two
constexpr int kAffine2 = 68;  // ... of 2 bits: two dwords
constexpr bool is_affine_mode(int mode) { return mode == NVQ_AFFINE || mode == kAffine8 || mode == kAffine3 || mode == kAffine6 || mode == kAffine5 || mode == kAffine2; }
constexpr int slice_quads(int mode) { return mode == NVQ_MXFP8 || mode == kAffine8 || mode == kAffine6 || mode == kAffine5 ? 2 : 1; }  // uint4 that carry a lane's 32 codes
template <typename T, int MODE> struct SliceScale { using type = std::conditional_t<is_affine_mode(MODE), T, std::conditional_t<MODE == NVQ_NVFP4, uint16_t, uint8_t>>; };

// A lane's slice of 32 values of one weight row against the same slice of RM rows of x (xp: the four pieces of eight
// values as pairs, in the expansion's pair order for affine codes and in memory order for the block formats; xs: the
// slices' sums, affine only), added to acc.  Affine: scale * (dot - B * sum x) + bias * sum x with the codes entered as
// B + c.  Block formats: the conversion instructions give the code values, the group's float32 scale (NVFP4: two
// groups) multiplies the group's sum.
template <typename T, int RM, int MODE>
__device__ __forceinline__ void slice_dot(const uint4 (&wq)[slice_quads(MODE)], typename SliceScale<T, MODE>::type sraw, T braw,
                                          const uint4 (&xp)[RM][4], const float (&xs)[RM], float factor, uint32_t mask, uint32_t magic,
                                          float (&acc)[RM]) {
    constexpr int BITS = MODE == NVQ_MXFP8 || MODE == kAffine8 ? 8 : 4;
    constexpr int kHalves = MODE == NVQ_NVFP4 ? 2 : 1;
    if constexpr (MODE == kAffine8) {
        // 8-bit codes: converted (a bf16 mantissa has no room for them), paired in memory order; the slice is inside one
        // group (groups of 32 and more): scale * dot + bias * sum x
        float dot[RM][2];
#pragma unroll
        for (int i = 0; i < RM; i++) dot[i][0] = dot[i][1] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint4 q = wq[j >> 1];
            const uint32_t d0 = (j & 1) ? q.z : q.x, d1 = (j & 1) ? q.w : q.y;
            const uint32_t p0 = qmf::Ops<T>::pack(qmf::ubyte_to_float<0>(d0), qmf::ubyte_to_float<1>(d0));
            const uint32_t p1 = qmf::Ops<T>::pack(qmf::ubyte_to_float<2>(d0), qmf::ubyte_to_float<3>(d0));
            const uint32_t p2 = qmf::Ops<T>::pack(qmf::ubyte_to_float<0>(d1), qmf::ubyte_to_float<1>(d1));
            const uint32_t p3 = qmf::Ops<T>::pack(qmf::ubyte_to_float<2>(d1), qmf::ubyte_to_float<3>(d1));
#pragma unroll
            for (int i = 0; i < RM; i++) {
                dot[i][0] = Pair<T>::dot2(xp[i][j].x, p0, dot[i][0]);
                dot[i][1] = Pair<T>::dot2(xp[i][j].y, p1, dot[i][1]);
                dot[i][0] = Pair<T>::dot2(xp[i][j].z, p2, dot[i][0]);
                dot[i][1] = Pair<T>::dot2(xp[i][j].w, p3, dot[i][1]);
            }
        }
        const float sc = Elem<T>::load(&sraw, 0), bi = Elem<T>::load(&braw, 0);
#pragma unroll
        for (int i = 0; i < RM; i++) acc[i] = __builtin_fmaf(sc, dot[i][0] + dot[i][1], __builtin_fmaf(bi, xs[i], acc[i]));
    } else if constexpr (MODE == kAffine3) {
        // 3-bit codes: piece j is the 24 bits from bit 24 j of the lane's 96; codes 0..3 stay in the low half, codes 4..7
        // move to the high half, and the pairs (c0, c4) (c1, c5) (c2, c6) (c3, c7) enter as B + c like the 4-bit ones
        const uint32_t d0 = wq[0].x, d1 = wq[0].y, d2 = wq[0].z;
        const uint32_t piece[4] = {d0, __builtin_amdgcn_alignbit(d1, d0, 24), __builtin_amdgcn_alignbit(d2, d1, 16), d2 >> 8};
        float dot[RM][4];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int t = 0; t < 4; t++) dot[i][t] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t z = (piece[j] & 0xFFFu) | ((piece[j] << 4) & 0x0FFF0000u);
            const uint32_t p0 = and_or(z, mask, magic), p1 = and_or(z >> 3, mask, magic);
            const uint32_t p2 = and_or(z >> 6, mask, magic), p3 = and_or(z >> 9, mask, magic);
#pragma unroll
            for (int i = 0; i < RM; i++) {
                dot[i][0] = Pair<T>::dot2(xp[i][j].x, p0, dot[i][0]);
                dot[i][1] = Pair<T>::dot2(xp[i][j].y, p1, dot[i][1]);
                dot[i][2] = Pair<T>::dot2(xp[i][j].z, p2, dot[i][2]);
                dot[i][3] = Pair<T>::dot2(xp[i][j].w, p3, dot[i][3]);
            }
        }
        const float sc = Elem<T>::load(&sraw, 0), bi = Elem<T>::load(&braw, 0);
        const float bb = __builtin_fmaf(-Pair<T>::base, sc, bi);
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const float dsum = (dot[i][0] + dot[i][1]) + (dot[i][2] + dot[i][3]);
            acc[i] = __builtin_fmaf(sc, dsum, __builtin_fmaf(bb, xs[i], acc[i]));
        }
    } else if constexpr (MODE == kAffine2) {
        // 2-bit codes: piece j is the 16 bits from bit 16 j of the lane's 64; codes 0..3 stay in the low half, codes 4..7
        // move to the high half, and the pairs (c0, c4) (c1, c5) (c2, c6) (c3, c7) enter as B + c like the 4-bit ones
        const uint32_t d[2] = {wq[0].x, wq[0].y};
        float dot[RM][4];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int t = 0; t < 4; t++) dot[i][t] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t v = d[j >> 1] >> (16 * (j & 1));
            const uint32_t z = (v & 0xFFu) | ((v << 8) & 0x00FF0000u);
            const uint32_t p0 = and_or(z, mask, magic), p1 = and_or(z >> 2, mask, magic);
            const uint32_t p2 = and_or(z >> 4, mask, magic), p3 = and_or(z >> 6, mask, magic);
#pragma unroll
            for (int i = 0; i < RM; i++) {
                dot[i][0] = Pair<T>::dot2(xp[i][j].x, p0, dot[i][0]);
                dot[i][1] = Pair<T>::dot2(xp[i][j].y, p1, dot[i][1]);
                dot[i][2] = Pair<T>::dot2(xp[i][j].z, p2, dot[i][2]);
                dot[i][3] = Pair<T>::dot2(xp[i][j].w, p3, dot[i][3]);
            }
        }
        const float sc = Elem<T>::load(&sraw, 0), bi = Elem<T>::load(&braw, 0);
        const float bb = __builtin_fmaf(-Pair<T>::base, sc, bi);
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const float dsum = (dot[i][0] + dot[i][1]) + (dot[i][2] + dot[i][3]);
            acc[i] = __builtin_fmaf(sc, dsum, __builtin_fmaf(bb, xs[i], acc[i]));
        }
    } else if constexpr (MODE == kAffine6 || MODE == kAffine5) {
        // 6- and 5-bit codes: piece t is the four codes (24 or 20 bits) from bit 24 t or 20 t of the lane's 192 or 160;
        // its codes 0, 1 stay in the low half, 2, 3 move to the high half, and the pairs (c0, c2) (c1, c3) enter as B + c
        constexpr int W = MODE == kAffine6 ? 6 : 5;
        const uint32_t d0 = wq[0].x, d1 = wq[0].y, d2 = wq[0].z, d3 = wq[1].x, d4 = wq[1].y, d5 = wq[1].z;
        uint32_t piece[8];
        if constexpr (W == 6) {
            piece[0] = d0, piece[1] = __builtin_amdgcn_alignbit(d1, d0, 24), piece[2] = __builtin_amdgcn_alignbit(d2, d1, 16), piece[3] = d2 >> 8;
            piece[4] = d3, piece[5] = __builtin_amdgcn_alignbit(d4, d3, 24), piece[6] = __builtin_amdgcn_alignbit(d5, d4, 16), piece[7] = d5 >> 8;
        } else {
            piece[0] = d0, piece[1] = __builtin_amdgcn_alignbit(d1, d0, 20), piece[2] = __builtin_amdgcn_alignbit(d2, d1, 8), piece[3] = __builtin_amdgcn_alignbit(d2, d1, 28);
            piece[4] = __builtin_amdgcn_alignbit(d3, d2, 16), piece[5] = d3 >> 4, piece[6] = __builtin_amdgcn_alignbit(d4, d3, 24), piece[7] = d4 >> 12;
        }
        constexpr uint32_t kLow = (1u << (2 * W)) - 1;
        float dot[RM][4];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int t = 0; t < 4; t++) dot[i][t] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t za = (piece[2 * j] & kLow) | ((piece[2 * j] << (16 - 2 * W)) & (kLow << 16));
            const uint32_t zb = (piece[2 * j + 1] & kLow) | ((piece[2 * j + 1] << (16 - 2 * W)) & (kLow << 16));
            const uint32_t p0 = and_or(za, mask, magic), p1 = and_or(za >> W, mask, magic);
            const uint32_t p2 = and_or(zb, mask, magic), p3 = and_or(zb >> W, mask, magic);
#pragma unroll
            for (int i = 0; i < RM; i++) {
                dot[i][0] = Pair<T>::dot2(xp[i][j].x, p0, dot[i][0]);
                dot[i][1] = Pair<T>::dot2(xp[i][j].y, p1, dot[i][1]);
                dot[i][2] = Pair<T>::dot2(xp[i][j].z, p2, dot[i][2]);
                dot[i][3] = Pair<T>::dot2(xp[i][j].w, p3, dot[i][3]);
            }
        }
        const float sc = Elem<T>::load(&sraw, 0), bi = Elem<T>::load(&braw, 0);
        const float bb = __builtin_fmaf(-Pair<T>::base, sc, bi);
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const float dsum = (dot[i][0] + dot[i][1]) + (dot[i][2] + dot[i][3]);
            acc[i] = __builtin_fmaf(sc, dsum, __builtin_fmaf(bb, xs[i], acc[i]));
        }
    } else if constexpr (MODE == NVQ_AFFINE) {
        const uint32_t d[4] = {wq[0].x, wq[0].y, wq[0].z, wq[0].w};
        float dot[RM][4];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int t = 0; t < 4; t++) dot[i][t] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t p0 = and_or(d[j], mask, magic), p1 = and_or(d[j] >> 4, mask, magic);
            const uint32_t p2 = and_or(d[j] >> 8, mask, magic), p3 = and_or(d[j] >> 12, mask, magic);
#pragma unroll
            for (int i = 0; i < RM; i++) {
                dot[i][0] = Pair<T>::dot2(xp[i][j].x, p0, dot[i][0]);
                dot[i][1] = Pair<T>::dot2(xp[i][j].y, p1, dot[i][1]);
                dot[i][2] = Pair<T>::dot2(xp[i][j].z, p2, dot[i][2]);
                dot[i][3] = Pair<T>::dot2(xp[i][j].w, p3, dot[i][3]);
            }
        }
        const float sc = Elem<T>::load(&sraw, 0), bi = Elem<T>::load(&braw, 0);
        const float bb = __builtin_fmaf(-Pair<T>::base, sc, bi);
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const float dsum = (dot[i][0] + dot[i][1]) + (dot[i][2] + dot[i][3]);
            acc[i] = __builtin_fmaf(sc, dsum, __builtin_fmaf(bb, xs[i], acc[i]));
        }
    } else {
        // piece j of the lane's slice: eight values, the pairs of xp[i][j] in memory order
        float dot[RM][kHalves][2];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int hf = 0; hf < kHalves; hf++) dot[i][hf][0] = dot[i][hf][1] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            constexpr int kPiecesPerHalf = 4 / kHalves;
            const int hf = j / kPiecesPerHalf;
            uint32_t p0, p1, p2, p3;
            if constexpr (BITS == 4) {
                const uint4 q = wq[0];
                const uint32_t d = j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w;
                p0 = qmf::Ops<T>::template fp4_pair<0>(d, 1.0f);
                p1 = qmf::Ops<T>::template fp4_pair<1>(d, 1.0f);
                p2 = qmf::Ops<T>::template fp4_pair<2>(d, 1.0f);
                p3 = qmf::Ops<T>::template fp4_pair<3>(d, 1.0f);
            } else {
                const uint4 q = wq[j >> 1];
                const uint32_t d0 = (j & 1) ? q.z : q.x, d1 = (j & 1) ? q.w : q.y;
                p0 = qmf::Ops<T>::template fp8_pair<false>(d0, 1.0f);
                p1 = qmf::Ops<T>::template fp8_pair<true>(d0, 1.0f);
                p2 = qmf::Ops<T>::template fp8_pair<false>(d1, 1.0f);
                p3 = qmf::Ops<T>::template fp8_pair<true>(d1, 1.0f);
            }
#pragma unroll
            for (int i = 0; i < RM; i++) {
                dot[i][hf][0] = Pair<T>::dot2(xp[i][j].x, p0, dot[i][hf][0]);
                dot[i][hf][1] = Pair<T>::dot2(xp[i][j].y, p1, dot[i][hf][1]);
                dot[i][hf][0] = Pair<T>::dot2(xp[i][j].z, p2, dot[i][hf][0]);
                dot[i][hf][1] = Pair<T>::dot2(xp[i][j].w, p3, dot[i][hf][1]);
            }
        }
        float sc[2];
        if constexpr (MODE == NVQ_NVFP4) {
            // both E4M3 scales by one conversion (every E4M3 value is a normal float32 or zero); times the
            // global scale's factor as crates/nuvec-core/src/kernels.rs:992-998
            const auto two = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8((uint32_t)sraw, 1.0f, false);
            sc[0] = ftz(two[0] * factor), sc[1] = ftz(two[1] * factor);
        } else {
            sc[0] = sc[1] = ftz(e8m0_to_f32(sraw));
        }
#pragma unroll
        for (int hf = 0; hf < kHalves; hf++)
#pragma unroll
            for (int i = 0; i < RM; i++) acc[i] = __builtin_fmaf(sc[hf], dot[i][hf][0] + dot[i][hf][1], acc[i]);
    }
}

// ── 4-bit affine and the block formats, bf16 / f16, one to four rows of x: the decode kernel ───────────
// A block of WAVES wavefronts shares the x slice of one K step (4096 values) through LDS, stored
// once in the pair order the codes need (affine: together with the sums of its 32-value slices), so the
// per-row work of a wavefront is only: two 128-bit weight loads per lane (four for 8-bit codes), the code
// expansion, the packed dot products and one data-parallel-primitive reduction.  Every load of a step is
// issued before the first use; blocks are small (WAVES*RN weight rows) so that tens of
// thousands of independent loads are in flight on the chip.
// MODE: NVQ_AFFINE (4 bits: a code enters as B + c through the constant's mantissa, and the factored form
// scale (dot - B sum x) + bias sum x never materialises a weight), or NVQ_MXFP4 / NVQ_NVFP4 / NVQ_MXFP8: the
// conversion instructions give the code values as element pairs (every E2M1 and E4M3 value is exact in bf16 and f16),
// in memory order, and a lane's 32 values are one group (NVFP4: two), whose float32 scale multiplies the group's sum.
// kAffine2 / kAffine3 / kAffine5 / kAffine6 / kAffine8: affine codes of those widths (2, 3, 5, 6 or 8 dwords a lane; see slice_dot).
// GLU (the pairs of a gather whose weights hold the experts' gate and up projections in alternating runs of 64 rows,
// RN = 2): a wavefront takes output column c of [pairs, N / 2], i.e. weight rows 128 (c / 64) + c % 64 (gate) and that
// + 64 (up), and stores the gated activation of the two rounded products (each with its expert's bias first), bit for
// bit what the product followed by the activation kernel gives.
template <typename T, int RM, int RN, int WAVES, bool BATCHED, int MODE = NVQ_AFFINE, bool GLU = false>
__global__ void __launch_bounds__(WAVES * 64) qmv4_lds_kernel(const ProductArgs a) {
    constexpr int kThreads = WAVES * 64;
    constexpr int kXPerThread = 512 / kThreads;  // 128-bit pieces of one x row per thread and step
    static_assert(512 % kThreads == 0, "a step of x must split evenly over the block");
    constexpr bool kAffine = is_affine_mode(MODE);
    constexpr int BITS = MODE == NVQ_MXFP8 || MODE == kAffine8 ? 8 : MODE == kAffine3 ? 3 : MODE == kAffine6 ? 6 : MODE == kAffine5 ? 5 : MODE == kAffine2 ? 2 : 4;
    constexpr int kQuads = slice_quads(MODE);           // loads of a lane's 32 codes (16 bytes each; 3, 5 and 6 bits: 12 and 8)
    constexpr int kHalves = MODE == NVQ_NVFP4 ? 2 : 1;  // groups per lane slice
    __shared__ uint4 x_pairs[RM][2][4][64];               // [row][chunk][word][lane]: 4 pairs of eight values
    __shared__ float x_sums[kAffine ? RM : 1][2][64];     // [row][chunk][lane]: sum of the lane's 32 values (affine)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Sizes fit 32 bits (checked on the host); only row bases are 64-bit, and they are uniform.
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = kAffine ? (a.group == 32 ? 5 : a.group == 64 ? 6 : 7) : (MODE == NVQ_NVFP4 ? 4 : 5);
    static_assert(!GLU || (RN == 2 && BATCHED), "the gated epilogue: a gate and an up row per wavefront, pairs of a gather");
    const int column = __builtin_amdgcn_readfirstlane(blockIdx.x * WAVES + wave);  // (GLU: of the output)
    const int n0 = GLU ? 128 * (column >> 6) + (column & 63) : column * RN;
    constexpr int kRowStep = GLU ? 64 : 1;  // between a wavefront's rows
    const int m0 = blockIdx.y * RM;
    const int kwords = (K * BITS) >> 5, kgroups = K >> gshift;
    // The single-product instantiation carries no batch arithmetic at all.
    const BatchOffsets o = BATCHED ? batch_offsets(a, blockIdx.z, kwords, kgroups) : BatchOffsets{0, 0, 0, 0, 0};
    const T *x = (const T *)a.x + o.x;
    const uint32_t *w = (const uint32_t *)a.w + o.w;
    using S = std::conditional_t<kAffine, T, uint8_t>;  // a scale as stored: the element type, or one byte (E8M0; NVFP4: E4M3)
    const S *scales = (const S *)a.scales + o.s, *biases = kAffine ? (const S *)a.biases + o.s : nullptr;
    T *y = (T *)a.y + o.y;
    constexpr uint32_t ones = std::is_same<T, bf16_t>::value ? 0x3F803F80u : 0x3C003C00u;
    uint32_t mask, magic;
    asm volatile("s_mov_b32 %0, %1" : "=s"(mask) : "i"(BITS == 3 ? 0x00070007 : BITS == 6 ? 0x003F003F : BITS == 5 ? 0x001F001F : BITS == 2 ? 0x00030003 : 0x000F000F));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(Pair<T>::magic));
    float factor = 1.0f;
    if constexpr (MODE == NVQ_NVFP4) factor = qmf::nvfp4_factor(a, BATCHED && a.rhs != nullptr ? (int64_t)a.rhs[blockIdx.z] : 0);

    float acc[RN][RM];
#pragma unroll
    for (int r = 0; r < RN; r++)
#pragma unroll
        for (int i = 0; i < RM; i++) acc[r][i] = 0.0f;

    for (int k0 = 0; k0 < K; k0 += 2 * kStep) {
        // x first: it is needed first and arrives from the cache.
        uint4 xg[RM][kXPerThread];
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int p = 0; p < kXPerThread; p++) {
                const int kx = k0 + (tid + p * kThreads) * 8;
                xg[i][p] = (kx < K && m0 + i < M) ? *reinterpret_cast<const uint4 *>(x + (int64_t)(m0 + i) * K + kx)
                                                      : make_uint4(0, 0, 0, 0);  // absent x: contributes nothing
            }
        uint4 wq[2][RN][kQuads];
        using SR = typename SliceScale<T, MODE>::type;
        SR sraw[2][RN];
        T braw[2][RN];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int kb = k0 + u * kStep + lane * 32;
            const int kc = kb < K ? kb : 0;  // an absent slice reads valid memory; its x is zero
#pragma unroll
            for (int r = 0; r < RN; r++) {
                const int n = n0 + r * kRowStep < N ? n0 + r * kRowStep : N - 1;  // tail rows are computed, not stored
                // the codes are read once: a non-temporal load keeps them from displacing x and the scales in the caches
                // (8.1 -> 7.8 us at W[14336,4096]; the scales, shared by neighbouring lanes and rows, lose by it)
                if constexpr (BITS == 2) {  // two dwords (rows are whole multiples of 8 bytes: K % 32 == 0)
                    const uint2 v = stream_load(reinterpret_cast<const uint2 *>(w + (int64_t)n * kwords + (kc >> 5) * 2));
                    wq[u][r][0] = make_uint4(v.x, v.y, 0u, 0u);
                } else if constexpr (BITS == 3) {  // three dwords, dword-aligned
                    typedef uint32_t u32x3_a4_t __attribute__((ext_vector_type(3), aligned(4)));
                    const u32x3_a4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x3_a4_t *>(w + (int64_t)n * kwords + (kc >> 5) * 3));
                    wq[u][r][0] = make_uint4(v.x, v.y, v.z, 0u);
                } else if constexpr (BITS == 6 || BITS == 5) {  // three dwords and three (5 bits: two), dword-aligned
                    typedef uint32_t u32x3_a4_t __attribute__((ext_vector_type(3), aligned(4)));
                    typedef uint32_t u32x2_a4_t __attribute__((ext_vector_type(2), aligned(4)));
                    const uint32_t *pw = w + (int64_t)n * kwords + (kc >> 5) * BITS;
                    const u32x3_a4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x3_a4_t *>(pw));
                    wq[u][r][0] = make_uint4(v.x, v.y, v.z, 0u);
                    if constexpr (BITS == 6) {
                        const u32x3_a4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x3_a4_t *>(pw + 3));
                        wq[u][r][1] = make_uint4(t.x, t.y, t.z, 0u);
                    } else {
                        const u32x2_a4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x2_a4_t *>(pw + 3));
                        wq[u][r][1] = make_uint4(t.x, t.y, 0u, 0u);
                    }
                } else {
                    const uint4 *pw = reinterpret_cast<const uint4 *>(w + (int64_t)n * kwords + (kc >> 5) * BITS);
#pragma unroll
                    for (int c = 0; c < kQuads; c++) wq[u][r][c] = stream_load(pw + c);
                }
                sraw[u][r] = *reinterpret_cast<const SR *>(scales + (int64_t)n * kgroups + (kc >> gshift));
                if constexpr (kAffine) braw[u][r] = (biases + (int64_t)n * kgroups)[kc >> gshift];
                else braw[u][r] = T{};
            }
        }
        if (k0 != 0) __syncthreads();  // the previous step's readers are done with the LDS
#pragma unroll
        for (int i = 0; i < RM; i++)
#pragma unroll
            for (int p = 0; p < kXPerThread; p++) {
                const int idx = tid + p * kThreads;  // 128-bit piece: chunk idx/256, lane (idx%256)/4, word idx%4
                const uint4 q = xg[i][p];            // q.x = (x0,x1) q.y = (x2,x3) q.z = (x4,x5) q.w = (x6,x7)
                if constexpr (kAffine) {
                    uint4 pr = q;
                    if constexpr (MODE == kAffine6 || MODE == kAffine5) {
                        pr.x = __builtin_amdgcn_perm(q.y, q.x, 0x05040100u);  // (x0, x2)
                        pr.y = __builtin_amdgcn_perm(q.y, q.x, 0x07060302u);  // (x1, x3)
                        pr.z = __builtin_amdgcn_perm(q.w, q.z, 0x05040100u);  // (x4, x6)
                        pr.w = __builtin_amdgcn_perm(q.w, q.z, 0x07060302u);  // (x5, x7)
                    } else if constexpr (MODE != kAffine8) {  // (8-bit codes are converted in memory order)
                        pr.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);  // (x0, x4)
                        pr.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);  // (x1, x5)
                        pr.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);  // (x2, x6)
                        pr.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);  // (x3, x7)
                    }
                    x_pairs[i][idx >> 8][idx & 3][(idx & 255) >> 2] = pr;
                    float sum = Pair<T>::dot2(pr.x, ones, 0.0f);
                    sum = Pair<T>::dot2(pr.y, ones, sum);
                    sum = Pair<T>::dot2(pr.z, ones, sum);
                    sum = Pair<T>::dot2(pr.w, ones, sum);
                    sum += __shfl_xor(sum, 1);  // the four pieces of a lane's slice sit in adjacent threads
                    sum += __shfl_xor(sum, 2);
                    if ((idx & 3) == 0) x_sums[i][idx >> 8][(idx & 255) >> 2] = sum;
                } else {
                    x_pairs[i][idx >> 8][idx & 3][(idx & 255) >> 2] = q;  // (the conversions give the code values in memory order)
                }
            }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 2; u++) {
            uint4 xp[RM][4];
            float xs[RM];
#pragma unroll
            for (int i = 0; i < RM; i++) {
#pragma unroll
                for (int j = 0; j < 4; j++) xp[i][j] = x_pairs[i][u][j][lane];
                if constexpr (kAffine) xs[i] = x_sums[i][u][lane];
                else xs[i] = 0.0f;
            }
#pragma unroll
            for (int r = 0; r < RN; r++) slice_dot<T, RM, MODE>(wq[u][r], sraw[u][r], braw[u][r], xp, xs, factor, mask, magic, acc[r]);
        }
    }
    if constexpr (GLU) {
        const int H = N >> 1;
        T *out = (T *)a.y + (int64_t)blockIdx.z * M * H;  // (no scattered rows on this route)
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const float g = wave_sum_lane63(acc[0][i]), u = wave_sum_lane63(acc[1][i]);
            if (lane == 63 && column < H && m0 + i < M) {
                // the products as their outputs hold them, the expert's bias by a separate rounded addition
                const float gate = add_row_bias<T>(a.row_bias, rounded<T>(g), o.bias + n0), up = add_row_bias<T>(a.row_bias, rounded<T>(u), o.bias + n0 + 64);
                const float v = a.glu == 1 + NVQ_GLU_SWIGLU       ? glu<T, NVQ_GLU_SWIGLU>(gate, up, a.glu_alpha, a.glu_limit)
                                : a.glu == 1 + NVQ_GLU_SWIGLU_OAI ? glu<T, NVQ_GLU_SWIGLU_OAI>(gate, up, a.glu_alpha, a.glu_limit)
                                                                  : glu<T, NVQ_GLU_GEGLU>(gate, up, a.glu_alpha, a.glu_limit);
                Elem<T>::store(out, (int64_t)(m0 + i) * H + column, v);
            }
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < RN; r++)
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const float v = wave_sum_lane63(acc[r][i]);
            if (lane == 63 && n0 + r < N && m0 + i < M) Elem<T>::store(y, (int64_t)(m0 + i) * N + n0 + r, add_row_bias<T>(a.row_bias, v, o.bias + n0 + r));
        }
}



// ── The same for short rows: K up to 2048 ──────────────────────────────────────────────────────────────
// The decode kernel above gives a weight row to a wavefront, 32 values a lane: a row of K < 2048 values leaves lanes
// (and the second of its two loads) without work.  Here a row takes L lanes, L the power of two that covers K / 32
// (2 to 64), so a wavefront holds 64 / L rows at once and two such sets in flight; x (all of K) is staged once per
// block, and the L partial sums of a row are added with a butterfly of cross-lane moves inside its L lanes.
template <typename T, int RM, int L, bool BATCHED, int MODE>
__global__ void __launch_bounds__(512) qmv4_short_kernel(const ProductArgs a) {
    constexpr int kWaves = 8;
    constexpr int kSub = 64 / L;                 // rows of a wavefront's set
    constexpr int kRowsPerWave = 2 * kSub, kRowsPerBlock = kWaves * kRowsPerWave;
    constexpr bool kAffine = MODE == NVQ_AFFINE;
    constexpr int BITS = MODE == NVQ_MXFP8 ? 8 : 4;
    constexpr int kQuads = BITS / 4;
    __shared__ uint4 x_pairs[RM][4][L];              // [row][word][slice]: 4 pairs of eight values
    __shared__ float x_sums[kAffine ? RM : 1][L];    // [row][slice]: sum of the slice's 32 values (affine)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane / L, kl = lane % L;
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    const int gshift = kAffine ? (a.group == 32 ? 5 : a.group == 64 ? 6 : 7) : (MODE == NVQ_NVFP4 ? 4 : 5);
    const int n_base = (blockIdx.x * kWaves + wave) * kRowsPerWave + sub;
    const int m0 = blockIdx.y * RM;
    const int kwords = (K * BITS) >> 5, kgroups = K >> gshift;
    const BatchOffsets o = BATCHED ? batch_offsets(a, blockIdx.z, kwords, kgroups) : BatchOffsets{0, 0, 0, 0, 0};
    const T *x = (const T *)a.x + o.x;
    const uint32_t *w = (const uint32_t *)a.w + o.w;
    using S = std::conditional_t<kAffine, T, uint8_t>;
    using SR = typename SliceScale<T, MODE>::type;
    const S *scales = (const S *)a.scales + o.s, *biases = kAffine ? (const S *)a.biases + o.s : nullptr;
    T *y = (T *)a.y + o.y;
    constexpr uint32_t ones = std::is_same<T, bf16_t>::value ? 0x3F803F80u : 0x3C003C00u;
    uint32_t mask, magic;
    asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(mask));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(Pair<T>::magic));
    float factor = 1.0f;
    if constexpr (MODE == NVQ_NVFP4) factor = qmf::nvfp4_factor(a, BATCHED && a.rhs != nullptr ? (int64_t)a.rhs[blockIdx.z] : 0);

    // x first: thread t < 4 L holds piece t (eight values) of every row of x; pieces past K are zero
    uint4 xg[RM];
#pragma unroll
    for (int i = 0; i < RM; i++)
        xg[i] = (tid * 8 < K && m0 + i < M) ? *reinterpret_cast<const uint4 *>(x + (int64_t)(m0 + i) * K + tid * 8) : make_uint4(0, 0, 0, 0);
    const int kc = kl * 32 < K ? kl * 32 : 0;  // an absent slice reads valid memory; its x is zero
    uint4 wq[2][kQuads];
    SR sraw[2];
    T braw[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int n = n_base + u * kSub < N ? n_base + u * kSub : N - 1;  // tail rows are computed, not stored
        const uint4 *pw = reinterpret_cast<const uint4 *>(w + (int64_t)n * kwords + (kc >> 5) * BITS);
#pragma unroll
        for (int c = 0; c < kQuads; c++) wq[u][c] = stream_load(pw + c);
        sraw[u] = *reinterpret_cast<const SR *>(scales + (int64_t)n * kgroups + (kc >> gshift));
        if constexpr (kAffine) braw[u] = (biases + (int64_t)n * kgroups)[kc >> gshift];
        else braw[u] = T{};
    }
    if (tid < 4 * L) {
#pragma unroll
        for (int i = 0; i < RM; i++) {
            const uint4 q = xg[i];  // q.x = (x0,x1) q.y = (x2,x3) q.z = (x4,x5) q.w = (x6,x7)
            if constexpr (kAffine) {
                uint4 pr;
                pr.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);  // (x0, x4)
                pr.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);  // (x1, x5)
                pr.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);  // (x2, x6)
                pr.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);  // (x3, x7)
                x_pairs[i][tid & 3][tid >> 2] = pr;
                float sum = Pair<T>::dot2(pr.x, ones, 0.0f);
                sum = Pair<T>::dot2(pr.y, ones, sum);
                sum = Pair<T>::dot2(pr.z, ones, sum);
                sum = Pair<T>::dot2(pr.w, ones, sum);
                sum += __shfl_xor(sum, 1);  // the four pieces of a slice sit in adjacent threads
                sum += __shfl_xor(sum, 2);
                if ((tid & 3) == 0) x_sums[i][tid >> 2] = sum;
            } else {
                x_pairs[i][tid & 3][tid >> 2] = q;
            }
        }
    }
    __syncthreads();
    uint4 xp[RM][4];
    float xs[RM];
#pragma unroll
    for (int i = 0; i < RM; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) xp[i][j] = x_pairs[i][j][kl];
        if constexpr (kAffine) xs[i] = x_sums[i][kl];
        else xs[i] = 0.0f;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        float acc[RM];
#pragma unroll
        for (int i = 0; i < RM; i++) acc[i] = 0.0f;
        slice_dot<T, RM, MODE>(wq[u], sraw[u], braw[u], xp, xs, factor, mask, magic, acc);
        const int n = n_base + u * kSub;
#pragma unroll
        for (int i = 0; i < RM; i++) {
            float v = acc[i];
#pragma unroll
            for (int off = 1; off < L; off <<= 1) v += __shfl_xor(v, off);  // (inside the row's L lanes)
            if (kl == 0 && n < N && m0 + i < M) Elem<T>::store(y, (int64_t)(m0 + i) * N + n, add_row_bias<T>(a.row_bias, v, o.bias + n));
        }
    }
}

// ── 4-bit affine, bf16 / f16, up to four rows of x, groups of 64 or 128: decode on the matrix cores ──────
// The vector units only turn nibbles into elements (one v_and_or_b32 per two codes, the magic-number form
// above); multiplying and summing is left to v_mfma_f32_32x32x16, whose 32 tile rows carry the (up to four)
// rows of x and zeros.  A block of eight wavefronts owns 32 weight rows; wavefront v owns the K slice
// [v K/8, (v+1) K/8) of them.  Lane (column c = lane % 32, half h = lane / 32) loads, per group of 64 values,
// the 16 bytes of its row's codes [64 g + 32 h, + 32): its four dwords are the B operands of four matrix
// instructions whose 16 values of K are {8 j .. 8 j + 7} of both halves, all inside the group, so a group's
// products land in a fresh accumulator P and the factored form of the vector kernel applies per group:
//     y += scale * (P - B * X) + bias * X,   X = sum of the group's x,  B = 128 (bf16) or 1024 (f16).
// Only tile rows 0..RM-1 are live: one to four fused multiply-adds per group and lane instead of sixteen.
// x is staged once per block in LDS in the pair order of the nibbles ((x0,x4),(x1,x5),(x2,x6),(x3,x7) per
// eight values) with the sums X of its 64-value spans; the lanes of dead tile rows read row 0 again.  The wavefronts' partial rows are added in wavefront order.
using qmf::floatx16_t;
using qmf::u32x4_t;
constexpr int kMmWaves = 8, kMmRows = 32, kMmChunk = 256;  // values of K per register chunk (four groups of 64)
constexpr int kMmStageBytes = kMmRows * kMmChunk / 2;        // one chunk of a wavefront's 32 rows: 4 KB

// Bytes between the rows of the block's scale (or bias) table: the row's groups plus eight, so that the 8-byte
// reads of 32 consecutive rows fall on different banks.
__host__ __device__ constexpr int mm_table_stride(int64_t kgroups) { return (int)kgroups * 2 + 8; }

template <int RM>
__host__ __device__ constexpr size_t mm_lds_bytes(int64_t k) {
    return (size_t)RM * k * 2 + (size_t)RM * (k >> 6) * 4 + (size_t)kMmWaves * RM * kMmRows * 4 + (size_t)kMmWaves * kMmStageBytes +
           2 * (size_t)kMmRows * mm_table_stride(k >> 6);
}

template <typename T, int RM, bool G128, bool BATCHED>
__global__ void __launch_bounds__(kMmWaves * 64) qmv4_mfma_kernel(const ProductArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, c = lane & 31;
    const int K = (int)a.k, N = (int)a.n, M = (int)a.m;
    constexpr int gshift = G128 ? 7 : 6;
    const int kwords = K >> 3, kgroups = K >> gshift, kchunks = K >> 3;  // dwords, groups, 16-byte x chunks per row
    const int n0 = blockIdx.x * kMmRows, m0 = blockIdx.y * RM;
    const BatchOffsets o = BATCHED ? batch_offsets(a, blockIdx.z, kwords, kgroups) : BatchOffsets{0, 0, 0, 0, 0};
    const T *x = (const T *)a.x + o.x;
    const uint32_t *w = (const uint32_t *)a.w + o.w;
    const T *scales = (const T *)a.scales + o.s, *biases = (const T *)a.biases + o.s;
    T *y = (T *)a.y + o.y;
    uint4 *xs = reinterpret_cast<uint4 *>(lds);                                      // [RM][K / 8]
    float *xsum = reinterpret_cast<float *>(lds + (size_t)RM * K * 2);               // [RM][K / 64]
    float *partial = xsum + RM * (K >> 6);                                           // [waves][RM][32]
    constexpr uint32_t ones = std::is_same<T, bf16_t>::value ? 0x3F803F80u : 0x3C003C00u;
    uint32_t mask, magic;
    asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(mask));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(Pair<T>::magic));

    // This lane's weights, scales and biases: chunk q of the wavefront's slice holds four groups of 64.
    const int kslice = K >> 3, k_wave = wave * kslice, chunks = kslice / kMmChunk;
    struct Chunk {
        u32x4_t w[4];
    };
    // The chunk's codes are fetched coalesced: load t of lane l is the 16-byte piece l % 8 of row 8 t + l / 8 of
    // the wavefront's 32 rows (128 contiguous bytes per row and load), and travels through a private piece of LDS
    // into the operand layout (piece p of row r sits at position p ^ ((r / 2) % 8): the lanes of a read, which
    // take one piece of 32 different rows 128 bytes apart, then spread over the 64 banks).
    // Every load is issued on every path (a chunk past the slice reads the slice's first one again).
    const int lrow = lane >> 3, lpiece = lane & 7;
    const uint4 *wl[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int r = n0 + 8 * t + lrow < N ? n0 + 8 * t + lrow : N - 1;  // tail rows are computed, not stored
        wl[t] = reinterpret_cast<const uint4 *>(w + (int64_t)r * kwords) + (k_wave >> 5) + lpiece;
    }
    auto load_chunk = [&](int q, Chunk &ch) {
        const int qc = q < chunks ? q : 0;
#pragma unroll
        for (int t = 0; t < 4; t++) ch.w[t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(wl[t] + 8 * qc));
    };
    const int tstride = mm_table_stride(K >> 6);
    unsigned char *table_s = reinterpret_cast<unsigned char *>(partial + kMmWaves * RM * kMmRows), *table_b = table_s + kMmRows * tstride;
    unsigned char *stage = table_b + kMmRows * tstride + wave * kMmStageBytes;
    int wstore[4], wread[4];
#pragma unroll
    for (int t = 0; t < 4; t++) wstore[t] = (8 * t + lrow) * 128 + 16 * (lpiece ^ (((8 * t + lrow) >> 1) & 7));
#pragma unroll
    for (int g = 0; g < 4; g++) wread[g] = c * 128 + 16 * ((2 * g + h) ^ ((c >> 1) & 7));
    // x first: it is needed first and arrives from the cache; the weights' loads follow, so that the wait for x
    // leaves them in flight.  (Every thread has a chunk in the first round: K / 8 >= 256 and whole wavefronts.)
    auto load_x = [&](int idx, int i) {
        return m0 + i < M && idx < kchunks ? *reinterpret_cast<const uint4 *>(x + (int64_t)(m0 + i) * K + 8 * idx) : make_uint4(0, 0, 0, 0);
    };
    uint4 xq[RM];
#pragma unroll
    for (int i = 0; i < RM; i++) xq[i] = load_x(tid, i);
    // The scales and biases of the block's 32 rows are contiguous in memory: 8-byte pieces, coalesced, the
    // scales by the lower half of the threads and the biases by the upper (first round in registers, as x).
    const int row_pieces = kgroups >> 2, table_pieces = kMmRows * row_pieces;  // 8-byte pieces (4 groups each)
    const int valid_pieces = (N - n0 < kMmRows ? N - n0 : kMmRows) * row_pieces;
    const int tp = tid & 255;
    const T *tsrc = (tid < 256 ? scales : biases) + (int64_t)n0 * kgroups;
    unsigned char *tdst = tid < 256 ? table_s : table_b;
    auto load_t = [&](int piece) { return piece < valid_pieces ? reinterpret_cast<const uint2 *>(tsrc)[piece] : make_uint2(0, 0); };
    const uint2 tq[2] = {load_t(tp), load_t(tp + 256)};  // two rounds cover K <= 4096
    Chunk ring[2];
    load_chunk(0, ring[0]);
    load_chunk(1, ring[1]);

    // x into LDS: pair order and span sums.  The first round's x is in registers already; later rounds
    // (K > 4096) load theirs here.
    auto stage_x = [&](int idx, int i, uint4 q) {
        uint4 pr;
        pr.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);  // (x0, x4)
        pr.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);  // (x1, x5)
        pr.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);  // (x2, x6)
        pr.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);  // (x3, x7)
        xs[i * kchunks + idx] = pr;
        float sum = Pair<T>::dot2(pr.x, ones, 0.0f);
        sum = Pair<T>::dot2(pr.y, ones, sum);
        sum = Pair<T>::dot2(pr.z, ones, sum);
        sum = Pair<T>::dot2(pr.w, ones, sum);
        sum += __shfl_xor(sum, 1);  // the eight chunks of a span of 64 sit in adjacent threads
        sum += __shfl_xor(sum, 2);
        sum += __shfl_xor(sum, 4);
        if ((idx & 7) == 0) xsum[i * (K >> 6) + (idx >> 3)] = sum;
    };
    if (tid < kchunks) {
#pragma unroll
        for (int i = 0; i < RM; i++) stage_x(tid, i, xq[i]);
    }
    auto store_t = [&](int piece, uint2 v) {
        if (piece < table_pieces) *reinterpret_cast<uint2 *>(tdst + (piece / row_pieces) * tstride + (piece % row_pieces) * 8) = v;
    };
    store_t(tp, tq[0]);
    store_t(tp + 256, tq[1]);
    for (int piece = tp + 512; piece < table_pieces; piece += 256) store_t(piece, load_t(piece));
    for (int idx = tid + kMmWaves * 64; idx < kchunks; idx += kMmWaves * 64) {
#pragma unroll
        for (int i = 0; i < RM; i++) stage_x(idx, i, load_x(idx, i));
    }
    __syncthreads();

    // A operands: tile row c is row c of x; chunk (k_wave + 64 g + 32 h) / 8 + j.  Tile rows RM.. are never looked
    // at, so their lanes read row 0 again (one address: a broadcast).
    const uint4 *xa = xs + (c < RM ? c : 0) * kchunks + ((k_wave + 32 * h) >> 3);
    const float *xsp = xsum + (k_wave >> 6);
    float yacc[RM];
#pragma unroll
    for (int i = 0; i < RM; i++) yacc[i] = 0.0f;
    floatx16_t zero;
#pragma unroll
    for (int e = 0; e < 16; e++) zero[e] = 0.0f;

    for (int q0 = 0; q0 < chunks; q0 += 2) {
        qmf::static_for<2>([&](auto d_tag) {
            constexpr int d = decltype(d_tag)::value;
            const int q = q0 + d;
            if (q < chunks) {
                // the chunk's codes through LDS into the operand layout; the wavefront's LDS accesses execute in order
                asm volatile("" ::: "memory");
#pragma unroll
                for (int t = 0; t < 4; t++) *reinterpret_cast<u32x4_t *>(stage + wstore[t]) = ring[d].w[t];
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");
                u32x4_t codes[4];
#pragma unroll
                for (int g = 0; g < 4; g++) codes[g] = *reinterpret_cast<const u32x4_t *>(stage + wread[g]);
                // the chunk's four (two of 128) scales and biases of this lane's row
                T cs[4], cb[4];
                {
                    const int at = c * tstride + ((k_wave + kMmChunk * q) >> gshift) * 2;
                    if constexpr (G128) {
                        const uint32_t sv = *reinterpret_cast<const uint32_t *>(table_s + at), bv = *reinterpret_cast<const uint32_t *>(table_b + at);
                        __builtin_memcpy(cs, &sv, 4);
                        __builtin_memcpy(cb, &bv, 4);
                    } else {
                        const uint2 sv = *reinterpret_cast<const uint2 *>(table_s + at), bv = *reinterpret_cast<const uint2 *>(table_b + at);
                        __builtin_memcpy(cs, &sv, 8);
                        __builtin_memcpy(cb, &bv, 8);
                    }
                }
                asm volatile("" ::: "memory");
                // two groups at a time, so that consecutive matrix instructions do not depend on each other
#pragma unroll
                for (int g0 = 0; g0 < 4; g0 += 2) {
                    floatx16_t P[2] = {zero, zero};
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int u = 0; u < 2; u++) {
                            const uint32_t dw = codes[g0 + u][j];
                            uint4 b;
                            // written in C (the constants sit in registers, so each line is one v_and_or_b32): the
                            // compiler must see these writes to keep the matrix instruction's operand hazards
                            b.x = (dw & mask) | magic;
                            b.y = ((dw >> 4) & mask) | magic;
                            b.z = ((dw >> 8) & mask) | magic;
                            b.w = ((dw >> 12) & mask) | magic;
                            P[u] = qmf::Ops<T>::mfma(xa[32 * q + 8 * (g0 + u) + j], b, P[u]);
                        }
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        const int g = g0 + u, sg = G128 ? g >> 1 : g;
                        const float sc = Elem<T>::load(&cs[sg], 0), bi = Elem<T>::load(&cb[sg], 0);
                        const float bb = __builtin_fmaf(-Pair<T>::base, sc, bi);
#pragma unroll
                        for (int i = 0; i < RM; i++) yacc[i] = __builtin_fmaf(sc, P[u][i], __builtin_fmaf(bb, xsp[i * (K >> 6) + 4 * q + g], yacc[i]));
                    }
                }
            }
            load_chunk(q + 2, ring[d]);  // the registers are free again
        });
    }

    // Tile rows 0..RM-1 live in lanes 0..31 (accumulator element e of lane l is row 8 (e / 4) + 4 (l / 32) + e % 4).
    if (h == 0) {
#pragma unroll
        for (int i = 0; i < RM; i++) partial[(wave * RM + i) * kMmRows + c] = yacc[i];
    }
    __syncthreads();
    if (tid < RM * kMmRows) {
        const int i = tid / kMmRows, col = tid % kMmRows;
        float v = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kMmWaves; wv++) v += partial[(wv * RM + i) * kMmRows + col];
        if (m0 + i < M && n0 + col < N) Elem<T>::store(y, (int64_t)(m0 + i) * N + n0 + col, add_row_bias<T>(a.row_bias, v, o.bias + n0 + col));
    }
}

// ── 4-bit affine, bf16 / f16, up to eight rows of x, groups of 64, K = 512 W <= 8192: decode on the 16x16x32 matrix instruction ──
// The vector units only turn nibbles into elements (the magic-number form above: three shifts and four
// v_and_or_b32 per packed word); v_mfma_f32_16x16x32 multiplies and sums.  A block of W = K / 512 wavefronts owns
// 16 RT weight rows; wavefront v owns the K slice [512 v, 512 v + 512) of them, NW = 4 windows of 128 values.  Lane
// (column n = lane % 16, quarter q = lane / 16) loads the 16 bytes [32 q, 32 q + 32) of each window of its row,
// straight into the B operand layout: word j of the load feeds matrix instruction j of the window, whose 32
// values of K are {32 q + 8 j .. + 7}, q = 0..3, so no weight passes through the LDS.  The 16 tile rows carry
// rows of x times groups: tile row kGpt m + g holds row m of x restricted to group g of the phase (half s = g % 2
// of window g / 2: the operand is zero in the lanes of the other half and in the other windows), so an
// accumulator collects the plain sums P of kGpt groups for 16 / kGpt rows of x separately and is read once per
// phase:   y += scale * (P - B * X) + bias * X,   X = sum of the group's x,  B = 128 (bf16) or 1024 (f16).
// One row of x: all eight groups of the slice in one accumulator; eight rows: one window (two groups) per phase.
// X comes from the same operands of x against a weight operand of ones, once per wavefront.
// x is staged once per block in LDS in the pair order of the nibbles; dead tile rows read a zero piece (one
// address: a broadcast).  The wavefronts' partial rows are added in a fixed order.
constexpr int kD16Rows = 16, kD16Slice = 512;  // weight rows of a tile; values of K per wavefront (a block has K / 512 wavefronts)

// Rows of x a tile carries (RM rounded up to a power of two), the groups of the slice it carries for each
// (kGpt), and the rows of x one lane's four accumulator elements belong to.
template <int RM> constexpr int d16_rows_pow2() { return RM <= 1 ? 1 : RM <= 2 ? 2 : RM <= 4 ? 4 : 8; }
template <int RM, int NW> constexpr int d16_gpt() { return 16 / d16_rows_pow2<RM>() < 2 * NW ? 16 / d16_rows_pow2<RM>() : 2 * NW; }
template <int RM, int NW> constexpr int d16_mpl() { return d16_gpt<RM, NW>() >= 4 ? 1 : 4 / d16_gpt<RM, NW>(); }

// LDS of a block: x in pair order, 64 bytes of zeros per wavefront, the wavefronts' partial rows.
template <int RM, int NW, int RT>
__host__ __device__ constexpr size_t d16_lds_bytes(int waves) {
    return (size_t)RM * (waves * 128 * NW * 2 + 16) + 64 * waves + (size_t)RT * waves * d16_mpl<RM, NW>() * 64 * 4;
}

template <typename T, int RM, int NW, int RT, bool BATCHED, bool CHUNKED>
__global__ void __launch_bounds__(1024) qmv4_mm16_kernel(const ProductArgs a) {
    constexpr int kSlice = 128 * NW, kSliceGroups = 2 * NW;
    static_assert(kSlice == kD16Slice, "the host sizes the block by the slice");
    const int waves = __builtin_amdgcn_readfirstlane(blockDim.x >> 6);
    // The block walks K in chunks of one slice per wavefront (a single chunk up to K = 8192).
    const int K = (int)a.k, chunk_k = waves * kSlice, chunks = CHUNKED ? K / chunk_k : 1;  // one chunk: no loop is compiled
    const int kPieces = chunk_k >> 3, kGroups = K >> 6;  // 16-byte pieces of x per row and chunk; groups per weight row
    constexpr int kGpt = d16_gpt<RM, NW>();          // groups per tile and row of x: 2, 4, 8 or 16
    constexpr int kPhases = kSliceGroups / kGpt;     // accumulators a slice goes through, one after the other
    constexpr int kMpl = d16_mpl<RM, NW>();          // rows of x per lane of the accumulator
    static_assert(RM <= 8 && kSliceGroups % kGpt == 0 && kSliceGroups <= 8, "the slice must split into whole tiles");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    // Rows of x lie one 16-byte piece more than their length apart: the lanes of an operand read take the same piece
    // of up to eight rows, which then fall on different banks.
    const int kRowPieces = kPieces + 1;
    uint4 *xs = reinterpret_cast<uint4 *>(lds);                                       // [RM][kRowPieces] + 4 pieces of zeros per wavefront
    float *partial = reinterpret_cast<float *>(lds + (size_t)RM * kRowPieces * 16 + 64 * waves);                                       // [RT][waves][kMpl][64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, kq = lane >> 4;
    const int N = (int)a.n, M = (int)a.m;
    const int kwords = K >> 3;
    const int n0 = blockIdx.x * kD16Rows * RT, m0 = blockIdx.y * RM;
    const BatchOffsets o = BATCHED ? batch_offsets(a, blockIdx.z, kwords, kGroups) : BatchOffsets{0, 0, 0, 0, 0};
    const T *x = (const T *)a.x + o.x;
    const uint32_t *w = (const uint32_t *)a.w + o.w;
    const T *scales = (const T *)a.scales + o.s, *biases = (const T *)a.biases + o.s;
    T *y = (T *)a.y + o.y;
    constexpr uint32_t ones = std::is_same<T, bf16_t>::value ? 0x3F803F80u : 0x3C003C00u;
    uint32_t mask, magic;
    asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(mask));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(Pair<T>::magic));

    if (lane < 4) xs[RM * kRowPieces + 4 * wave + lane] = make_uint4(0, 0, 0, 0);
    const int me = (4 * kq) / kGpt;  // the first row of x among this lane's accumulator elements
    float part[RT][kMpl];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int u = 0; u < kMpl; u++) part[rt][u] = 0.0f;
#pragma unroll 1
    for (int c = 0; c < chunks; c++) {
    // x first: a row of the chunk is one 16-byte piece per thread.
    uint4 xq[RM];
#pragma unroll
    for (int i = 0; i < RM; i++)
        xq[i] = m0 + i < M ? *reinterpret_cast<const uint4 *>(x + (int64_t)(m0 + i) * K + 8 * (c * kPieces + tid)) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < RM; i++) {
            const uint4 q = xq[i];
            uint4 pr;
            pr.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);  // (x0, x4)
            pr.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);  // (x1, x5)
            pr.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);  // (x2, x6)
            pr.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);  // (x3, x7)
            xs[i * kRowPieces + tid] = pr;
        }
    // The weights are asked for once x is on its way into the LDS: requests return in the order they were made, and
    // x queued behind the weights of every wavefront of the compute unit would arrive last.
    uint4 wq[RT][NW];
    int rows[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        rows[rt] = n0 + 16 * rt + nl < N ? n0 + 16 * rt + nl : N - 1;  // tail rows are computed, not stored
        const uint4 *wp = reinterpret_cast<const uint4 *>(w + (int64_t)rows[rt] * kwords) + ((c * chunk_k + wave * kSlice + 32 * kq) >> 5);
#pragma unroll
        for (int d = 0; d < NW; d++) wq[rt][d] = wp[4 * d];
    }
    // Accumulator element j of this lane is tile row t = 4 q + j: row t / kGpt of x, group t % kGpt of the phase.
    // The lane's scales and biases: the slice's groups (tiles of up to four groups: every lane uses them all), or
    // the four groups of the lane's half of a tile of eight.
    constexpr int kScaleWords = kGpt >= 8 ? 2 : kSliceGroups / 2;  // dwords of scales a lane holds
    const int gl0 = kGpt >= 8 ? (4 * kq) % kGpt : 0;
    uint32_t sraw[RT][kScaleWords], braw[RT][kScaleWords];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const int g0 = (c * chunk_k >> 6) + wave * kSliceGroups + gl0;
        const T *sp = scales + (int64_t)rows[rt] * kGroups + g0, *bp = biases + (int64_t)rows[rt] * kGroups + g0;
        if constexpr (kScaleWords == 4) {
            const uint4 sv = *reinterpret_cast<const uint4 *>(sp), bv = *reinterpret_cast<const uint4 *>(bp);
            sraw[rt][0] = sv.x; sraw[rt][1] = sv.y; sraw[rt][2] = sv.z; sraw[rt][3] = sv.w;
            braw[rt][0] = bv.x; braw[rt][1] = bv.y; braw[rt][2] = bv.z; braw[rt][3] = bv.w;
        } else {
            const uint2 sv = *reinterpret_cast<const uint2 *>(sp), bv = *reinterpret_cast<const uint2 *>(bp);
            sraw[rt][0] = sv.x; sraw[rt][1] = sv.y;
            braw[rt][0] = bv.x; braw[rt][1] = bv.y;
        }
    }

    // A thread stages piece tid of every row of x, which lies in the K slice of its own wavefront, and a wavefront
    // reads no other slice (nor another's zeros): its LDS accesses execute in order, so no block barrier is needed.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");

    // A operands: tile row nl = row nl / kGpt of x, group nl % kGpt of the phase: window (nl % kGpt) / 2 of the
    // phase, from the lanes of half nl % 2 only.
    const int ma = nl / kGpt, da = (nl % kGpt) >> 1, sa = nl & 1;
    const bool alive = (kq >> 1) == sa && ma < RM;
    const int a_live = ma * kRowPieces + ((wave * kSlice) >> 3) + 4 * kq, a_zero = RM * kRowPieces + 4 * wave;
    // The sums X of the groups come from the matrix cores as well: the same x operands against a weight operand of
    // ones, once per wavefront, land in the accumulator layout of P.
    const uint4 b_ones = make_uint4(ones, ones, ones, ones);
    floatx4_t accx[kPhases];
#pragma unroll
    for (int ph = 0; ph < kPhases; ph++)
#pragma unroll
        for (int e = 0; e < 4; e++) accx[ph][e] = 0.0f;
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
#pragma unroll
    for (int ph = 0; ph < kPhases; ph++) {
        floatx4_t acc;
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] = 0.0f;
#pragma unroll
        for (int dd = 0; dd < kGpt / 2; dd++) {
            const int d = ph * (kGpt / 2) + dd;
            const uint4 *xa = xs + ((alive && da == dd) ? a_live + 16 * d : a_zero);
            const uint32_t dws[4] = {wq[rt][d].x, wq[rt][d].y, wq[rt][d].z, wq[rt][d].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t dw = dws[j];
                uint4 b;
                // written in C (the constants sit in registers, so each line is one v_and_or_b32): the compiler
                // must see these writes to keep the matrix instruction's operand hazards
                b.x = (dw & mask) | magic;
                b.y = ((dw >> 4) & mask) | magic;
                b.z = ((dw >> 8) & mask) | magic;
                b.w = ((dw >> 12) & mask) | magic;
                acc = Mfma16<T>::run(xa[j], b, acc);
                if (rt == 0) accx[ph] = Mfma16<T>::run(xa[j], b_ones, accx[ph]);
            }
        }
        // y += scale * (P - B X) + bias * X for the lane's four (row of x, group) pairs
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int u = kGpt >= 4 ? 0 : j / kGpt;                  // which of the lane's rows of x
            const int gi = kGpt >= 8 ? j : ph * kGpt + j % kGpt;     // index among the lane's scales
            const uint32_t sw = sraw[rt][gi >> 1], bw = braw[rt][gi >> 1];
            const float sc = (gi & 1) ? Pair<T>::hi(sw) : Pair<T>::lo(sw), bi = (gi & 1) ? Pair<T>::hi(bw) : Pair<T>::lo(bw);
            const float bb = __builtin_fmaf(-Pair<T>::base, sc, bi);
            part[rt][u] = __builtin_fmaf(sc, acc[j], __builtin_fmaf(bb, accx[ph][j], part[rt][u]));
        }
    }
    if constexpr (!CHUNKED) {  // a single chunk: the tile's partial rows leave the registers right away
#pragma unroll
        for (int u = 0; u < kMpl; u++) partial[((rt * waves + wave) * kMpl + u) * 64 + lane] = me + u < RM ? part[rt][u] : 0.0f;
    }
    }
    asm volatile("" ::: "memory");  // the next chunk's x is written after this chunk's reads (same wavefront: in order)
    }
    if constexpr (CHUNKED) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int u = 0; u < kMpl; u++) partial[((rt * waves + wave) * kMpl + u) * 64 + lane] = me + u < RM ? part[rt][u] : 0.0f;
    }
    __syncthreads();
    for (int out = tid; out < RT * RM * 16; out += (int)blockDim.x) {
        const int rt = out / (RM * 16), m = (out >> 4) % RM, n = out & 15;
        // Row m of x is tile rows kGpt m .. kGpt m + kGpt - 1: element u of the lanes of kQ quarters from q0 on.
        constexpr int kQ = kGpt >= 4 ? kGpt / 4 : 1;
        const int q0 = (m * kGpt) >> 2, u = kGpt >= 4 ? 0 : ((m * kGpt) & 3) / kGpt;
        const float *src = partial + (rt * waves * kMpl + u) * 64 + 16 * q0 + n;
        float v = 0.0f;
#pragma unroll 4
        for (int wv = 0; wv < waves; wv++)
#pragma unroll
            for (int q = 0; q < kQ; q++) v += src[wv * kMpl * 64 + 16 * q];
        if (m0 + m < M && n0 + 16 * rt + n < N) Elem<T>::store(y, (int64_t)(m0 + m) * N + n0 + 16 * rt + n, add_row_bias<T>(a.row_bias, v, o.bias + n0 + 16 * rt + n));
    }
}

// Wavefronts of a block: one per 512 values of K up to 8192; beyond, the largest divisor of K / 512 up to 16 (the
// block then walks K in chunks of that many slices).
inline int d16_waves(int64_t k) {
    const int slices = (int)(k / kD16Slice);
    for (int wv = slices < 16 ? slices : 16; wv >= 1; wv--)
        if (slices % wv == 0) return wv;
    return 1;
}

// Whether the 16x16x32 decode kernel takes the product: one to eight rows of x, groups of 64, K a multiple of 512
// (a wavefront per 512 values) up to 8192, 16-byte aligned scale and bias rows.  Measured against the vector kernel
// and the 32x32x16 kernels (us per launch at 1 / 2 / 4 / 8 rows, old -> new):
//   W[8192,1024]   4.2 /  5.6 /  8.6 /  7.0 ->  3.3 /  3.4 /  3.7 /  4.1     W[32768,2048] 11.8 / 15.8 / 16.2 / 21.9 ->  8.8 /  9.2 /  9.3 / 10.0
//   W[6144,3072]   4.3 /  5.0 /  7.4 /  8.7 ->  5.1 /  5.5 /  5.6 /  6.5     W[18944,3584]  8.9 / 11.7 / 18.2 / 30.1 ->  9.2 / 10.0 / 11.5 / 12.7
//   W[14336,4096]  7.9 /  9.7 / 12.8 / 17.3 ->  9.2 /  9.4 /  9.9 / 10.4     W[4096,4096]   3.9 /  4.2 /  7.2 /  9.9 ->  4.6 /  5.0 /  5.1 /  5.3
//   W[13824,5120] 11.5 / 15.2 / 24.9 / 21.9 -> 10.3 / 11.7 / 11.8 / 14.0     W[8192,7168]   8.3 / 10.8 / 16.8 / 14.9 ->  8.6 /  9.0 /  9.4 / 10.1
//   W[8192,8192]   8.6 / 11.1 / 13.5 / 16.5 -> 10.3 / 11.0 / 11.0 / 11.6     W[28672,8192] 23.9 / 32.4 / 45.5 / 52.0 -> 27.2 / 30.8 / 34.2 / 38.1
// Three rows and more: always.  Two rows: not for 2048 < K <= 4096 with fewer than 8192 weight rows.  One row: only
// where the vector kernel's steps of 4096 values fit K badly (K <= 2048, 4096 < K <= 6144).
inline bool d16_takes(const ProductArgs &a) {
    if (a.mode != NVQ_AFFINE || a.bits != 4 || a.dtype == NVQ_F32 || a.group != 64 || a.exact_weights) return false;
    if (a.k % kD16Slice != 0 || a.k < 2 * kD16Slice || (a.k > 16 * kD16Slice && d16_waves(a.k) < 7)) return false;
    if (a.m < 1 || a.m > 8 || (a.k > 16 * kD16Slice && a.m < 3)) return false;
    if (a.m == 2 && a.k > 2048 && a.k <= 4096 && a.n < 8192) return false;
    if (a.m == 1 && !(a.k <= 2048 || (a.k > 4096 && a.k <= 6144))) return false;
    return ((uintptr_t)a.scales | (uintptr_t)a.biases) % 16 == 0;
}

template <typename T, int RM, int NW, int RT>
int32_t run_d16_sized(const ProductArgs &a, hipStream_t s) {
    const int waves = d16_waves(a.k);
    const size_t lds_bytes = d16_lds_bytes<RM, NW, RT>(waves);
    dim3 grid((unsigned)((a.n + kD16Rows * RT - 1) / (kD16Rows * RT)), (unsigned)((a.m + RM - 1) / RM), (unsigned)a.batch);
    const bool batched = !(a.batch == 1 && a.rhs == nullptr);
    const bool chunked = a.k > (int64_t)waves * kD16Slice;
    void (*kernel)(const ProductArgs);
    if constexpr (RM >= 4) {  // K beyond 8192 is taken from three rows on
        kernel = chunked ? (batched ? qmv4_mm16_kernel<T, RM, NW, RT, true, true> : qmv4_mm16_kernel<T, RM, NW, RT, false, true>)
                         : (batched ? qmv4_mm16_kernel<T, RM, NW, RT, true, false> : qmv4_mm16_kernel<T, RM, NW, RT, false, false>);
    } else {
        kernel = batched ? qmv4_mm16_kernel<T, RM, NW, RT, true, false> : qmv4_mm16_kernel<T, RM, NW, RT, false, false>;
    }
    static std::atomic<bool> configured[2][2] = {{false, false}, {false, false}};
    if (lds_bytes > 64 * 1024 && !configured[batched][chunked]) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        configured[batched][chunked] = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(waves * 64), lds_bytes, s, a);
    NVQ_LAUNCH_CHECK("qmv4_mm16");
    return NVQ_OK;
}

template <typename T>
int32_t run_d16(const ProductArgs &a, hipStream_t s) {
    if (a.m == 1) return run_d16_sized<T, 1, 4, 1>(a, s);
    if (a.m == 2) return run_d16_sized<T, 2, 4, 1>(a, s);
    // Two tiles of weight rows per block halve the staging of x; with fewer than 8192 weight rows the blocks of one
    // tile are needed to fill the chip.
    const bool two = a.n >= 8192;
    if (a.m <= 4) return two ? run_d16_sized<T, 4, 4, 2>(a, s) : run_d16_sized<T, 4, 4, 1>(a, s);
    return two ? run_d16_sized<T, 8, 4, 2>(a, s) : run_d16_sized<T, 8, 4, 1>(a, s);
}

// Whether the matrix-core decode kernel takes the product: groups of 64 or 128, K in whole chunks per wavefront,
// the staged x within the LDS.
template <int RM>
bool mfma_decode_takes(const ProductArgs &a) {
    return (a.group == 64 || a.group == 128) && a.k % (kMmWaves * kMmChunk) == 0 && mm_lds_bytes<RM>(a.k) <= 160 * 1024;
}

template <typename T, int RM>
int32_t run_mfma4(const ProductArgs &a, hipStream_t s) {
    const size_t lds_bytes = mm_lds_bytes<RM>(a.k);
    dim3 grid((unsigned)((a.n + kMmRows - 1) / kMmRows), (unsigned)((a.m + RM - 1) / RM), (unsigned)a.batch);
    const bool batched = !(a.batch == 1 && a.rhs == nullptr), g128 = a.group == 128;
    void (*kernel)(const ProductArgs) = g128 ? (batched ? qmv4_mfma_kernel<T, RM, true, true> : qmv4_mfma_kernel<T, RM, true, false>)
                                             : (batched ? qmv4_mfma_kernel<T, RM, false, true> : qmv4_mfma_kernel<T, RM, false, false>);
    static std::atomic<bool> configured[2][2] = {{false, false}, {false, false}};
    if (!configured[g128][batched]) {
        NVQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        configured[g128][batched] = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(kMmWaves * 64), lds_bytes, s, a);
    NVQ_LAUNCH_CHECK("qmv4_mfma");
    return NVQ_OK;
}

template <typename T, int RM, int RN, int WAVES, int MODE = NVQ_AFFINE>
int32_t run_lds4(const ProductArgs &a, hipStream_t s) {
    const int64_t rows = (int64_t)WAVES * RN;
    dim3 grid((unsigned)((a.n + rows - 1) / rows), (unsigned)((a.m + RM - 1) / RM), (unsigned)a.batch);
    if (a.batch == 1 && a.rhs == nullptr)
        hipLaunchKernelGGL((qmv4_lds_kernel<T, RM, RN, WAVES, false, MODE>), grid, dim3(WAVES * 64), 0, s, a);
    else
        hipLaunchKernelGGL((qmv4_lds_kernel<T, RM, RN, WAVES, true, MODE>), grid, dim3(WAVES * 64), 0, s, a);
    NVQ_LAUNCH_CHECK("qmv4_lds");
    return NVQ_OK;
}

// The pairs of a gather with the gated activation as the epilogue: whether the decode kernel takes them (4-bit affine
// codes that are never materialised, or a block format; bf16 / f16; up to four rows of x per pair; K in whole slices;
// the two projections' rows in whole runs of 64) ...
bool glu_pairs_take(const ProductArgs &a) {  // (also a single product, without pairs: batch 1)
    if ((a.rhs == nullptr && a.batch != 1) || a.dtype == NVQ_F32 || a.row_exact || a.exact_weights || a.out_rows != nullptr) return false;
    if (a.m < 1 || a.m > 4 || a.k % 32 != 0 || a.n % 128 != 0 || ((uintptr_t)a.w | (uintptr_t)a.x) % 16 != 0) return false;
    if (a.mode == NVQ_AFFINE) return a.bits == 4;
    return a.mode != NVQ_NVFP4 || (uintptr_t)a.scales % 2 == 0;
}

// ... and their launch: a wavefront per output column.
template <typename T, int MODE>
int32_t run_glu_pairs_mode(const ProductArgs &a, hipStream_t s) {
    const int rm = a.m == 1 ? 1 : a.m == 2 ? 2 : 4;
    const dim3 grid((unsigned)((a.n / 2 + 7) / 8), (unsigned)((a.m + rm - 1) / rm), (unsigned)a.batch);
    void (*kernel)(const ProductArgs) = rm == 1   ? qmv4_lds_kernel<T, 1, 2, 8, true, MODE, true>
                                        : rm == 2 ? qmv4_lds_kernel<T, 2, 2, 8, true, MODE, true>
                                                  : qmv4_lds_kernel<T, 4, 2, 8, true, MODE, true>;
    hipLaunchKernelGGL(kernel, grid, dim3(512), 0, s, a);
    NVQ_LAUNCH_CHECK("qmv4_lds with the gated epilogue");
    return NVQ_OK;
}

template <typename T>
int32_t run_glu_pairs(const ProductArgs &a, hipStream_t s) {
    switch (a.mode) {
    case NVQ_MXFP4: return run_glu_pairs_mode<T, NVQ_MXFP4>(a, s);
    case NVQ_MXFP8: return run_glu_pairs_mode<T, NVQ_MXFP8>(a, s);
    case NVQ_NVFP4: return run_glu_pairs_mode<T, NVQ_NVFP4>(a, s);
    default: return run_glu_pairs_mode<T, NVQ_AFFINE>(a, s);
    }
}

// Whether the decode kernel takes a product of a block format: bf16 / f16, up to kBlockDecodeRows rows of x, whole
// slices of 32 values (NVFP4 rows may end in half a slice: those stay on the general kernel).  Row-exact products
// stay on the general kernel at every row count.
// Measured against the few-row matrix-core kernels (us per launch at 1 / 2 / 3 / 4 rows, bf16; theirs -> this one):
//   MXFP4 W[14336,4096] 10.2 / 10.3 / 10.3 / 10.3 ->  7.5 /  8.8 / 10.2 / 12.6     W[2880,2880] 5.9 / 6.0 / 6.0 / 6.0 -> 3.7 / 4.2 / 4.8 / 5.4
//   MXFP4 W[4096,14336] 10.5 / 11.0 / 11.1 / 11.1 ->  8.3 / 10.4 / 12.3 / 14.8     W[4096,4096] 5.2 / 5.3 / 5.3 / 5.4 -> 4.2 / 4.5 / 5.0 / 5.7
//   NVFP4 W[14336,4096] 13.0 / 13.1 / 13.1 / 13.2 ->  8.9 / 10.3 / 12.3 / 13.9     W[2880,2880] 7.9 / 8.1 / 8.2 / 8.3 -> 4.0 / 4.6 / 5.3 / 6.0
//   MXFP8 W[14336,4096] 16.8 / 16.0 / 16.1 / 16.1 -> 13.6 / 14.3 / 14.7 / 16.0     W[4096,14336] 16.8 / 16.2 / 16.3 / 16.1 -> 14.6 / 15.5 / 16.6 / 18.8
// One and two rows: always.  Three rows (MXFP8: and four): up to K = 4096.  Up to four rows where the kernel that
// loads the weights straight into operand layout does not take the product (K in slices of 512).
inline bool block_decode_takes(const ProductArgs &a) {
    if (a.mode == NVQ_AFFINE || a.dtype == NVQ_F32 || a.row_exact) return false;
    if (a.m < 1 || a.m > 4 || a.k % 32 != 0 || (uintptr_t)a.w % 16 != 0 || (uintptr_t)a.x % 16 != 0) return false;
    if (a.mode == NVQ_NVFP4 && (uintptr_t)a.scales % 2 != 0) return false;  // (a lane reads its two scales at once)
    if (a.m <= 2 || !qmd_supported(a)) return true;
    return a.k <= 4096 && (a.m == 3 || a.mode == NVQ_MXFP8);
}

// Whether the short-row decode kernel takes the product: the pairs of a gather (the experts of decoded tokens, whose
// down projections have short rows) with 4-bit affine codes (never materialised: not with exact weights) or a block
// format the decode kernel takes, bf16 / f16, up to four rows of x, K up to 2048 in whole slices.  Measured, 32 pairs of
// one row against the kernels above (us): 4-bit g64 W[2048,512] 28.8 -> 8.5, W[2048,768] 29.0 -> 12.1, W[4096,1408]
// 54.5 -> 34.9; MXFP4 W[2048,768] 24.8 -> 11.3, W[2048,1024] 24.7 -> 11.9, W[2048,2048] 25.4 -> 19.8, W[4096,1408]
// 46.1 -> 32.3; MXFP8 W[2048,1024] 25.6 -> 18.0.  Where the 16x16x32 decode kernel takes affine pairs it stays ahead
// (W[2048,1024] 11.2 against 12.7, W[2048,2048] 16.5 against 21.4), and single products gain nothing (a launch either way).
// Single products take it too where a row is at most 512 values (the reference's qmv_quad shapes, K = 64 and 128,
// crates/nuvec-kernels/src/metal/quantized.h:819-874, and up to 16 lanes a row): a wavefront per row leaves 48 to 62
// of its lanes idle there (us, one / four rows of x, 4-bit g64 bf16: W[32768,128] 10.9 / 24.8, W[131072,128] 38.7 / 90.2
// on the decode kernel).
inline bool short_decode_takes(const ProductArgs &a) {
    if (a.dtype == NVQ_F32 || a.row_exact || a.k > 2048 || a.k % 32 != 0 || a.m < 1 || a.m > 4) return false;
    if (a.rhs == nullptr && (a.k > 512 || a.batch != 1 || a.batch_ndim != 0 || a.glu != 0)) return false;
    if (a.mode != NVQ_AFFINE) return block_decode_takes(a);
    return a.bits == 4 && !a.exact_weights && !d16_takes(a) && (uintptr_t)a.w % 16 == 0 && (uintptr_t)a.x % 16 == 0;
}

template <typename T, int MODE, int L>
int32_t run_short_lanes(const ProductArgs &a, hipStream_t s) {
    constexpr int kRowsPerBlock = 8 * 2 * (64 / L);
    const int rm = a.m == 1 ? 1 : a.m == 2 ? 2 : 4;
    const dim3 grid((unsigned)((a.n + kRowsPerBlock - 1) / kRowsPerBlock), (unsigned)((a.m + rm - 1) / rm), (unsigned)a.batch);
    void (*kernel)(const ProductArgs) = rm == 1   ? qmv4_short_kernel<T, 1, L, true, MODE>
                                        : rm == 2 ? qmv4_short_kernel<T, 2, L, true, MODE>
                                                  : qmv4_short_kernel<T, 4, L, true, MODE>;
    hipLaunchKernelGGL(kernel, grid, dim3(512), 0, s, a);
    NVQ_LAUNCH_CHECK("qmv4_short");
    return NVQ_OK;
}

template <typename T, int MODE>
int32_t run_short(const ProductArgs &a, hipStream_t s) {
    const int slices = (int)(a.k / 32);
    if (slices <= 2) return run_short_lanes<T, MODE, 2>(a, s);
    if (slices <= 4) return run_short_lanes<T, MODE, 4>(a, s);
    if (slices <= 8) return run_short_lanes<T, MODE, 8>(a, s);
    if (slices <= 16) return run_short_lanes<T, MODE, 16>(a, s);
    if (slices <= 32) return run_short_lanes<T, MODE, 32>(a, s);
    return run_short_lanes<T, MODE, 64>(a, s);
}

// Whether the decode kernel takes a few rows against 8-bit affine codes: up to three, four with groups of 32 (against
// the kernel that loads the weights straight into operand layout, 2 / 3 / 4 rows, us: W[4096,4096] g32 9.6 / 9.6 / 9.7 ->
// 6.4 / 7.0 / 7.3, g64 8.2 / 8.2 / 8.2 -> 6.3 / 6.9 / 7.2; W[14336,4096] g32 20.6 / 20.5 / 20.7 -> 14.7 / 17.1 / 17.6, g64
// 17.8 / 17.7 / 17.8 -> 15.5 / 16.9 / 17.9; W[4096,14336] g64 19.7 / 19.8 / 20.0 -> 17.0 / 20.3 / 21.3).
inline bool decode8_takes(const ProductArgs &a) {
    return a.mode == NVQ_AFFINE && a.bits == 8 && a.dtype != NVQ_F32 && a.m >= 1 && a.m <= (a.group == 32 ? 4 : 3) && !a.exact_weights && !a.row_exact && a.k % 32 == 0 &&
           ((uintptr_t)a.w | (uintptr_t)a.x) % 16 == 0;
}

// ... and one or two rows against 3-bit ones (two rows: W[4096,4096] 5.95 -> 4.78 us, W[4096,14336] 15.7 -> 12.8 us,
// W[14336,4096] 11.2 -> 11.3 us; three rows and more are the other kernel's: 5.8 against 6.2, 11.1 against 14.4).
// ... and up to four rows against 6- and 5-bit ones (us, against the general kernel at one row and the matrix-core kernel
// of few rows beyond: 6 bits W[4096,4096] g64 1 / 2 / 3 / 4 rows 6.5 / 11.9 / 12.0 / 12.1 -> 4.9 / 5.6 / 6.4 / 7.7, W[14336,4096]
// 14.5 / 20.6 / 20.8 / 20.8 -> 11.2 / 13.5 / 14.9 / 17.5, W[4096,14336] g128 14.7 / 24.8 / 25.0 / 25.2 -> 14.1 / 15.3 / 18.3 / 20.4;
// 5 bits W[4096,4096] 6.2 / 11.9 / 12.0 / 12.0 -> 4.7 / 5.3 / 6.5 / 7.5, W[14336,4096] 13.3 / 19.4 / 19.5 / 19.5 -> 10.2 / 12.5 / 14.2 /
// 16.8.  Rows of K = 2048 and less leave lanes idle: W[8192,2048] 6 bits 2 / 4 rows 8.7 / 8.7 -> 7.3 / 10.3, W[16384,1024]
// 9.2 / 9.2 -> 10.8 / 16.8, so the callers send those only with one row, or two at K = 2048.)
// ... and one or two rows against 2-bit ones (us, against the kernel that loads the weights straight into operand layout:
// W[4096,4096] g64 1 / 2 rows 5.3 / 5.3 -> 3.9 / 4.5, W[14336,4096] 10.1 / 10.1 -> 7.8 / 10.0, W[4096,14336] g128 one row
// 12.3 -> 9.1, W[2880,2880] g32 one row 7.7 -> 3.8; three rows and more are the other kernel's: 10.1 against 12.2).
inline bool decode2_takes(const ProductArgs &a) {
    return a.mode == NVQ_AFFINE && a.bits == 2 && a.dtype != NVQ_F32 && a.m >= 1 && a.m <= 2 && !a.exact_weights && !a.row_exact && a.k % 32 == 0 &&
           ((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 8 == 0);
}

inline bool decode56_takes(const ProductArgs &a) {
    return a.mode == NVQ_AFFINE && (a.bits == 6 || a.bits == 5) && a.dtype != NVQ_F32 && a.m >= 1 && a.m <= 4 && !a.exact_weights && !a.row_exact &&
           a.k % 32 == 0 && (uintptr_t)a.x % 16 == 0;
}

inline bool decode3_takes(const ProductArgs &a) {
    return a.mode == NVQ_AFFINE && a.bits == 3 && a.dtype != NVQ_F32 && a.m >= 1 && a.m <= 2 && !a.exact_weights && !a.row_exact && a.k % 32 == 0 &&
           (uintptr_t)a.x % 16 == 0;
}

template <typename T, int MODE>
int32_t run_block_decode(const ProductArgs &a, hipStream_t s) {
    if (a.m == 1) return run_lds4<T, 1, 1, 8, MODE>(a, s);
    if (a.m == 2) return run_lds4<T, 2, 1, 8, MODE>(a, s);
    if (a.m == 3) return run_lds4<T, 3, 1, 8, MODE>(a, s);
    return run_lds4<T, 4, 1, 8, MODE>(a, s);
}

template <typename T, int BITS, int MODE>
int32_t run_general(const ProductArgs &a, hipStream_t s) {
    const unsigned gx = (unsigned)((a.n + 7) / 8);
    constexpr bool kCanBeExact = MODE == NVQ_AFFINE && !std::is_same<T, float>::value;
    if ((a.m + 3) / 4 > 65535) return fail(NVQ_UNSUPPORTED, "quantized_matmul: %lld rows exceed the grid limit", (long long)a.m);
    const dim3 grid(gx, a.m == 1 ? 1u : (unsigned)((a.m + 3) / 4), (unsigned)a.batch);  // one row, or passes of four rows over grid.y
    if (kCanBeExact && a.exact_weights) {
        if (a.m == 1) hipLaunchKernelGGL((qmv_lds_kernel<T, BITS, MODE, 1, kCanBeExact>), grid, dim3(512), 0, s, a);
        else hipLaunchKernelGGL((qmv_lds_kernel<T, BITS, MODE, 4, kCanBeExact>), grid, dim3(512), 0, s, a);
    } else if (a.m == 1) {
        hipLaunchKernelGGL((qmv_lds_kernel<T, BITS, MODE, 1>), grid, dim3(512), 0, s, a);
    } else {
        hipLaunchKernelGGL((qmv_lds_kernel<T, BITS, MODE, 4>), grid, dim3(512), 0, s, a);
    }
    NVQ_LAUNCH_CHECK("qmv");
    return NVQ_OK;
}

template <typename T>
int32_t run_typed(const ProductArgs &a, hipStream_t s) {
    if constexpr (!std::is_same<T, float>::value) {
        if (short_decode_takes(a)) {
            if (a.mode == NVQ_MXFP4) return run_short<T, NVQ_MXFP4>(a, s);
            if (a.mode == NVQ_MXFP8) return run_short<T, NVQ_MXFP8>(a, s);
            if (a.mode == NVQ_NVFP4) return run_short<T, NVQ_NVFP4>(a, s);
            return run_short<T, NVQ_AFFINE>(a, s);
        }
        if (block_decode_takes(a)) {
            if (a.mode == NVQ_MXFP4) return run_block_decode<T, NVQ_MXFP4>(a, s);
            if (a.mode == NVQ_MXFP8) return run_block_decode<T, NVQ_MXFP8>(a, s);
            return run_block_decode<T, NVQ_NVFP4>(a, s);
        }
    }
    if (a.mode == NVQ_MXFP4) return run_general<T, 4, NVQ_MXFP4>(a, s);
    if (a.mode == NVQ_MXFP8) return run_general<T, 8, NVQ_MXFP8>(a, s);
    if (a.mode == NVQ_NVFP4) return run_general<T, 4, NVQ_NVFP4>(a, s);
    if constexpr (!std::is_same<T, float>::value) {
        // A single row against 8-bit codes (groups of 32 and more hold a lane's 32 values): the decode kernel.  Against
        // the general kernel below (us): W[4096,4096] g32 6.90 -> 5.80, g64 6.68 -> 5.35; W[14336,4096] g64 15.87 ->
        // 14.25; W[2880,2880] g32 5.99 -> 4.80; W[4096,14336] g128 15.69 -> 15.62.
        if (decode8_takes(a)) return a.m == 1 ? run_lds4<T, 1, 1, 8, kAffine8>(a, s) : a.m == 2 ? run_lds4<T, 2, 1, 8, kAffine8>(a, s) : run_lds4<T, 4, 1, 8, kAffine8>(a, s);
        // (3 bits, against the general kernel: W[4096,4096] g64 5.47 -> 4.01, W[14336,4096] 12.2 -> 8.2, W[2880,2880] g32 5.39 -> 3.78)
        if (decode3_takes(a)) return a.m == 1 ? run_lds4<T, 1, 1, 8, kAffine3>(a, s) : a.m == 2 ? run_lds4<T, 2, 1, 8, kAffine3>(a, s) : run_lds4<T, 4, 1, 8, kAffine3>(a, s);
        if (decode2_takes(a)) return run_block_decode<T, kAffine2>(a, s);
        if (decode56_takes(a)) {
            if (a.bits == 6) return run_block_decode<T, kAffine6>(a, s);
            return run_block_decode<T, kAffine5>(a, s);
        }
        if (a.bits == 4 && !a.exact_weights) {  // (the decode kernels never materialise a weight)
            // One row (or row-exact rows) against K = 2048 / 4096: the integer dot-product kernel (W[14336,4096]: 7.8 -> 6.8 us).
            if (qmv_dot8_takes(a)) return launch_qmv_dot8(a, s);
            // Four rows at a time run faster on the matrix cores (measured at W[14336,4096]: 14.0 against 15.3 us);
            // one to three rows stay on the vector kernel, whose blocks are smaller and start sooner (7.8 against
            // 10.4 us at one row).
            // Row-exact products stay on the vector kernel at every row count: a row's arithmetic there does not depend
            // on the rows that share its pass.
            if (!a.row_exact && d16_takes(a)) return run_d16<T>(a, s);  // 9.8 / 10.6 / 12.1 us at 2 / 4 / 8 rows of W[14336,4096] (vector and 32x32x16 kernels: 10.0 / 12.7 / 17.3)
            if (!a.row_exact && a.m >= 4 && mfma_decode_takes<4>(a)) return run_mfma4<T, 4>(a, s);  // more rows: passes of four over grid.y
            if (a.m == 1) return run_lds4<T, 1, 1, 8>(a, s);
            if (a.m == 2) return run_lds4<T, 2, 1, 8>(a, s);
            if (a.m == 3) return run_lds4<T, 3, 1, 8>(a, s);
            return run_lds4<T, 4, 1, 8>(a, s);  // more rows: passes of four over grid.y
        }
    }
#define NVQ_GENERIC(B) run_general<T, B, NVQ_AFFINE>(a, s)
    switch (a.bits) {
    case 1: return NVQ_GENERIC(1);
    case 2: return NVQ_GENERIC(2);
    case 3: return NVQ_GENERIC(3);
    case 4: return NVQ_GENERIC(4);
    case 5: return NVQ_GENERIC(5);
    case 6: return NVQ_GENERIC(6);
    case 8: return NVQ_GENERIC(8);
    default: return fail(NVQ_INVALID_ARGUMENT, "quantized_matmul: %d bits are not supported", a.bits);
    }
#undef NVQ_GENERIC
}

}  // namespace

bool qmv_d16_takes(const ProductArgs &a) { return !a.row_exact && d16_takes(a); }
bool qmv_block_decode_takes(const ProductArgs &a) { return block_decode_takes(a); }
bool qmv_decode_takes_width(const ProductArgs &a) { return decode8_takes(a) || decode3_takes(a) || decode56_takes(a) || decode2_takes(a); }

// Mirrors run_typed.
const char *qmv_kernel_name(const ProductArgs &a) {
    if (a.mode == NVQ_AFFINE && a.bits == 4 && a.dtype != NVQ_F32 && !a.exact_weights) {
        if (short_decode_takes(a)) return "qmv4_short_kernel";
        if (qmv_dot8_takes(a)) return "qmv4_dot8_kernel";
        if (!a.row_exact && d16_takes(a)) return "qmv4_mm16_kernel";
        if (!a.row_exact && a.m >= 4 && mfma_decode_takes<4>(a)) return "qmv4_mfma_kernel";
        return "qmv4_lds_kernel";
    }
    if (short_decode_takes(a)) return "qmv4_short_kernel";
    if (block_decode_takes(a) || decode8_takes(a) || decode3_takes(a) || decode56_takes(a) || decode2_takes(a)) return "qmv4_lds_kernel";
    return "qmv_lds_kernel";
}

bool qmv_glu_pairs_take(const ProductArgs &a) { return glu_pairs_take(a); }

int32_t launch_qmv_glu_pairs(const ProductArgs &a, hipStream_t s) {
    if (!glu_pairs_take(a) || a.glu == 0) return fail(NVQ_UNSUPPORTED, "gather_qmm: the decode kernel does not take these pairs with the gated epilogue");
    if (a.batch > 65535) return fail(NVQ_UNSUPPORTED, "gather_qmm: %lld pairs exceed the grid limit", (long long)a.batch);
    return a.dtype == NVQ_BF16 ? run_glu_pairs<bf16_t>(a, s) : run_glu_pairs<f16_t>(a, s);
}

int32_t launch_qmv(const ProductArgs &a, hipStream_t s) {
    if (a.batch > 65535) return fail(NVQ_UNSUPPORTED, "quantized_matmul: %lld batches exceed the grid limit", (long long)a.batch);
    switch (a.dtype) {
    case NVQ_F32: return run_typed<float>(a, s);
    case NVQ_BF16: return run_typed<bf16_t>(a, s);
    default: return run_typed<f16_t>(a, s);
    }
}

}  // namespace nvq
