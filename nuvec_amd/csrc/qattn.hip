// Attention of one query row per head over an affine-quantized key / value cache, in one kernel: the counterpart of
// the reference's FastOp::QuantizedAttention kernel (crates/nuvec-core/src/fast.rs:694-718; its fit rule
// crates/nuvec-core/src/fast/imp.rs:3944-3992; launch crates/nuvec-core/src/gpu.rs:4969-5040):
//     out[b, h, :] = softmax(scale * q[b, h, :] . K[b, h / rep]^T [, sink[h]]) . V[b, h / rep]
// with K and V stored packed (codes [B, Hkv, S, D bits / 32], scales and biases [B, Hkv, S, D / group]).  The codes are
// dequantized in registers and never rounded; products and sums are float32 (the reference's kernel likewise: "within
// the float bound of the dequantized attention").
//
// A block of four wavefronts owns one (batch, query head).  A row of the cache is D bits / 8 bytes = CH chunks of 16
// bytes (3 bits: of 12 bytes, 32 codes); lane l of a wavefront takes chunk l % CH of key l / CH of the wavefront's
// current tile of 64 / CH keys, so a wavefront-wide load reads 1 KB (768 bytes) of consecutive rows.  Per key the lanes of a row form the score from their partial
// dot products (factored: scale * sum(q * code) + bias * sum(q) per chunk) with cross-lane adds, every lane keeps an
// online softmax (running maximum, denominator) for the keys it has seen and accumulates its chunk of the output in
// the same factored form; at the end the (64 / CH) x 4 partial states are merged through LDS.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
int attention_splits(const nvq_attention_desc &d);
namespace {

constexpr int kAttnWaves = 4;

// A lane's chunk of a row: 16 bytes (BITS 4: 32 codes, 8: 16 codes), or the 12 bytes that hold 32 codes of 3 bits.
template <int BITS> struct Chunk { uint32_t w[BITS == 3 ? 3 : 4]; };

template <int BITS>
__device__ __forceinline__ Chunk<BITS> load_chunk(const uint32_t *p) {
    Chunk<BITS> c;
    if constexpr (BITS == 3) {
        c.w[0] = p[0], c.w[1] = p[1], c.w[2] = p[2];  // (rows of 3-bit codes are whole dwords: 4-byte aligned)
    } else {
        const uint4 v = *reinterpret_cast<const uint4 *>(p);
        c.w[0] = v.x, c.w[1] = v.y, c.w[2] = v.z, c.w[3] = v.w;
    }
    return c;
}

// Code i of a chunk as a float (i is a constant after unrolling).
template <int BITS>
__device__ __forceinline__ float chunk_code(const Chunk<BITS> &c, int i) {
    if constexpr (BITS == 4) {
        return (float)((c.w[i >> 3] >> (4 * (i & 7))) & 15u);
    } else if constexpr (BITS == 8) {
        return (float)((c.w[i >> 2] >> (8 * (i & 3))) & 255u);
    } else {
        const int bit = 3 * i, dw = bit >> 5, sh = bit & 31;
        const uint32_t v = sh <= 29 ? c.w[dw] >> sh : (c.w[dw] >> sh) | (c.w[dw + 1] << (32 - sh));
        return (float)(v & 7u);
    }
}

// softmax's last step: the weighted sum over a maximum `top` and its denominator, with the head's sink if it has one.
__device__ __forceinline__ float attention_finish(float sum, float denom, float top, float sink, bool has_sink) {
    if (!has_sink) return sum / denom;
    const float t2 = fmaxf(top, sink), f = __expf(top - t2);
    return sum * f / (denom * f + __expf(sink - t2));
}

// Keys of one split of the positions: whole tiles of the block (64 keys at most), so that no tile is shared.
__host__ __device__ inline int attention_split_keys(int64_t positions, int splits) {
    const int64_t per = (positions + splits - 1) / splits;
    return (int)((per + 63) / 64 * 64);
}

template <typename T, int BITS, int D>
__global__ void __launch_bounds__(64 * kAttnWaves) qattn_kernel(const nvq_attention_desc d, const T *__restrict__ q, const uint32_t *__restrict__ kw,
                                                               const T *__restrict__ ks, const T *__restrict__ kb,
                                                               const uint32_t *__restrict__ vw, const T *__restrict__ vs,
                                                               const T *__restrict__ vb, const T *__restrict__ sinks, T *__restrict__ out,
                                                               float *__restrict__ partials) {
    constexpr int CPL = BITS == 3 ? 32 : 128 / BITS;  // codes (values of D) per lane
    constexpr int CW = CPL * BITS / 32;               // dwords of a lane's chunk
    constexpr int CH = D / CPL;            // lanes per key: 2, 4 or 8
    constexpr int KPT = 64 / CH;           // keys per wavefront tile
    constexpr int kSlots = KPT * kAttnWaves;
    __shared__ float part[kSlots][D + 1];  // the slots' partial outputs, already scaled to the block's maximum
    __shared__ float slot_m[kSlots], slot_l[kSlots];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane % CH, j = lane / CH;
    const int h = blockIdx.x, b = blockIdx.y;
    const int rep = d.query_heads / d.key_heads, hk = h / rep;
    const int S = d.positions, groups = D / d.group_size;
    const int gi = (c * CPL) / d.group_size;  // this lane's group of a row (a chunk lies inside one group: group >= 32 >= CPL)
    const int64_t row0 = ((int64_t)b * d.key_heads + hk) * S;
    const int splits = gridDim.z, per = attention_split_keys(S, splits);
    const int s_begin = blockIdx.z * per, s_end = s_begin + per < S ? s_begin + per : S;

    // the lane's CPL values of the query, scaled; their sum (the bias term of the factored score)
    float qv[CPL], qsum = 0.0f;
    const T *qrow = q + ((int64_t)b * d.query_heads + h) * D + c * CPL;
#pragma unroll
    for (int i = 0; i < CPL; i++) {
        qv[i] = d.scale * Elem<T>::load(qrow, i);
        qsum += qv[i];
    }
    float m = -INFINITY, l = 0.0f, acc[CPL], accb = 0.0f;
#pragma unroll
    for (int i = 0; i < CPL; i++) acc[i] = 0.0f;

    // One tile of keys: everything it reads from memory.  The next tile is requested before the current one is computed.
    struct Tile {
        Chunk<BITS> kc, vc;
        T sk, bk, sv, bv;
    };
    auto fetch = [&](int s0) {
        const int s = s0 + j;
        const int64_t r = row0 + (s < s_end ? s : S - 1);  // a key past the end reads the last one and is given no weight
        Tile t;
        t.kc = load_chunk<BITS>(kw + (r * CH + c) * CW), t.vc = load_chunk<BITS>(vw + (r * CH + c) * CW);
        t.sk = ks[r * groups + gi], t.bk = kb[r * groups + gi], t.sv = vs[r * groups + gi], t.bv = vb[r * groups + gi];
        return t;
    };
    Tile cur = fetch(s_begin + wave * KPT);
    for (int s0 = s_begin + wave * KPT; s0 < s_end; s0 += kAttnWaves * KPT) {
        const Tile nxt = fetch(s0 + kAttnWaves * KPT);  // (past the end: valid addresses, nothing of it is used)
        const bool live = s0 + j < s_end;
        const float sk = Elem<T>::load(&cur.sk, 0), bk = Elem<T>::load(&cur.bk, 0);
        const float sv = Elem<T>::load(&cur.sv, 0), bv = Elem<T>::load(&cur.bv, 0);
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < CPL; i++) dot = __builtin_fmaf(qv[i], chunk_code<BITS>(cur.kc, i), dot);
        float score = __builtin_fmaf(sk, dot, bk * qsum);
#pragma unroll
        for (int o = 1; o < CH; o <<= 1) score += __shfl_xor(score, o);  // the lanes of a key sit side by side
        if (!live) score = -INFINITY;
        const float m_new = fmaxf(m, score);
        // (a slot that has seen no live key keeps m = -inf: its weights are zero, not NaN)
        const float corr = m_new == -INFINITY ? 1.0f : __expf(m - m_new), p = m_new == -INFINITY ? 0.0f : __expf(score - m_new);
        m = m_new;
        l = __builtin_fmaf(l, corr, p);
        const float pv = p * sv;
        accb = __builtin_fmaf(accb, corr, p * bv);
#pragma unroll
        for (int i = 0; i < CPL; i++) acc[i] = __builtin_fmaf(acc[i], corr, pv * chunk_code<BITS>(cur.vc, i));
        cur = nxt;
    }

    // merge: the block's maximum, every slot scaled to it, the slots added up
    const int slot = wave * KPT + j;
    if (c == 0) slot_m[slot] = m;
    __syncthreads();
    float top = -INFINITY;
    for (int t = 0; t < kSlots; t++) top = fmaxf(top, slot_m[t]);
    const float w = m == -INFINITY ? 0.0f : __expf(m - top);
    if (c == 0) slot_l[slot] = l * w;
#pragma unroll
    for (int i = 0; i < CPL; i++) part[slot][c * CPL + i] = (acc[i] + accb) * w;
    __syncthreads();
    if (tid < D) {
        float denom = 0.0f, sum = 0.0f;
        for (int t = 0; t < kSlots; t++) {
            denom += slot_l[t];
            sum += part[t][tid];
        }
        const int64_t head = (int64_t)b * d.query_heads + h;
        if (splits == 1) {
            const bool has_sink = sinks != nullptr;
            Elem<T>::store(out, head * D + tid, attention_finish(sum, denom, top, has_sink ? Elem<T>::load(sinks, h) : 0.0f, has_sink));
        } else {  // this split's state: maximum, denominator, weighted sum
            float *dst = partials + (head * splits + blockIdx.z) * (D + 2);
            if (tid == 0) dst[0] = top, dst[1] = denom;
            dst[2 + tid] = sum;
        }
    }
}

// The splits of one (batch, head) merged: block = D threads.
template <typename T, int D>
__global__ void __launch_bounds__(D) qattn_merge_kernel(const nvq_attention_desc d, const float *__restrict__ partials, int splits,
                                                        const T *__restrict__ sinks, T *__restrict__ out) {
    const int64_t head = (int64_t)blockIdx.y * d.query_heads + blockIdx.x;
    const float *src = partials + head * splits * (D + 2);
    float top = -INFINITY;
    for (int z = 0; z < splits; z++) top = fmaxf(top, src[z * (D + 2)]);
    float denom = 0.0f, sum = 0.0f;
    for (int z = 0; z < splits; z++) {
        const float mz = src[z * (D + 2)], w = mz == -INFINITY ? 0.0f : __expf(mz - top);
        denom = __builtin_fmaf(src[z * (D + 2) + 1], w, denom);
        sum = __builtin_fmaf(src[z * (D + 2) + 2 + threadIdx.x], w, sum);
    }
    const bool has_sink = sinks != nullptr;
    Elem<T>::store(out, head * D + threadIdx.x,
                   attention_finish(sum, denom, top, has_sink ? Elem<T>::load(sinks, blockIdx.x) : 0.0f, has_sink));
}

template <typename T, int BITS, int D>
int32_t run_attention_sized(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb, const void *vw,
                            const void *vs, const void *vb, const void *sinks, void *out, void *workspace, hipStream_t s) {
    const int splits = workspace != nullptr ? attention_splits(d) : 1;
    const dim3 grid((unsigned)d.query_heads, (unsigned)d.batch, (unsigned)splits), block(64 * kAttnWaves);
    hipLaunchKernelGGL((qattn_kernel<T, BITS, D>), grid, block, 0, s, d, (const T *)q, (const uint32_t *)kw, (const T *)ks, (const T *)kb,
                       (const uint32_t *)vw, (const T *)vs, (const T *)vb, (const T *)sinks, (T *)out, (float *)workspace);
    NVQ_LAUNCH_CHECK("quantized_attention");
    if (splits > 1) {
        hipLaunchKernelGGL((qattn_merge_kernel<T, D>), dim3((unsigned)d.query_heads, (unsigned)d.batch), dim3(D), 0, s, d,
                           (const float *)workspace, splits, (const T *)sinks, (T *)out);
        NVQ_LAUNCH_CHECK("quantized_attention merge");
    }
    return NVQ_OK;
}

template <typename T, int BITS>
int32_t run_attention(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb, const void *vw,
                      const void *vs, const void *vb, const void *sinks, void *out, void *workspace, hipStream_t s) {
    return d.head_dim == 64 ? run_attention_sized<T, BITS, 64>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s)
                            : run_attention_sized<T, BITS, 128>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s);
}

template <typename T>
int32_t run_attention_bits(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb, const void *vw,
                           const void *vs, const void *vb, const void *sinks, void *out, void *workspace, hipStream_t s) {
    return d.bits == 4   ? run_attention<T, 4>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s)
           : d.bits == 3 ? run_attention<T, 3>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s)
                         : run_attention<T, 8>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s);
}

}  // namespace

// Splits of the positions over the grid: about two blocks per compute unit, at least 256 keys a split, at most 64 splits.
int attention_splits(const nvq_attention_desc &d) {
    const int64_t heads = d.batch * d.query_heads;
    if (heads <= 0 || d.positions < 512) return 1;
    int64_t want = (2 * (int64_t)compute_units() + heads - 1) / heads;
    const int64_t most = d.positions / 256;
    want = want > most ? most : want;
    want = want > 64 ? 64 : want;
    if (want < 2) return 1;
    const int per = attention_split_keys(d.positions, (int)want);  // whole tiles: fewer splits may cover the positions
    return (int)((d.positions + per - 1) / per);
}

size_t attention_workspace_bytes(const nvq_attention_desc &d) {
    const int splits = attention_splits(d);
    return splits > 1 ? (size_t)d.batch * (size_t)d.query_heads * (size_t)splits * (size_t)(d.head_dim + 2) * sizeof(float) : 0;
}

int32_t launch_quantized_attention(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb,
                                   const void *vw, const void *vs, const void *vb, const void *sinks, void *out, void *workspace,
                                   hipStream_t s) {
    switch (d.dtype) {
    case NVQ_F32: return run_attention_bits<float>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s);
    case NVQ_BF16: return run_attention_bits<bf16_t>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s);
    default: return run_attention_bits<f16_t>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, workspace, s);
    }
}

}  // namespace nvq
