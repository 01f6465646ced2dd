// Attention of one query row per head over an affine-quantized key / value cache, in one kernel: the counterpart of
// the reference's FastOp::QuantizedAttention kernel (crates/nuvec-core/src/fast.rs:694-718; its fit rule
// crates/nuvec-core/src/fast/imp.rs:3944-3992; launch crates/nuvec-core/src/gpu.rs:4969-5040):
//     out[b, h, :] = softmax(scale * q[b, h, :] . K[b, h / rep]^T [, sink[h]]) . V[b, h / rep]
// with K and V stored packed (codes [B, Hkv, S, D bits / 32], scales and biases [B, Hkv, S, D / group]).  The codes are
// dequantized in registers and never rounded; products and sums are float32 (the reference's kernel likewise: "within
// the float bound of the dequantized attention").
//
// A block of four wavefronts owns one (batch, query head).  A row of the cache is D bits / 8 bytes = CH chunks of 16
// bytes; lane l of a wavefront takes chunk l % CH of key l / CH of the wavefront's current tile of 64 / CH keys, so a
// wavefront-wide load reads 1 KB of consecutive rows.  Per key the lanes of a row form the score from their partial
// dot products (factored: scale * sum(q * code) + bias * sum(q) per chunk) with cross-lane adds, every lane keeps an
// online softmax (running maximum, denominator) for the keys it has seen and accumulates its chunk of the output in
// the same factored form; at the end the (64 / CH) x 4 partial states are merged through LDS.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

constexpr int kAttnWaves = 4;

// Code i of a 16-byte chunk (BITS 4: 32 codes, 8: 16 codes) as a float.
template <int BITS>
__device__ __forceinline__ float chunk_code(const uint4 &c, int i) {
    const uint32_t w[4] = {c.x, c.y, c.z, c.w};
    if constexpr (BITS == 4) return (float)((w[i >> 3] >> (4 * (i & 7))) & 15u);
    else return (float)((w[i >> 2] >> (8 * (i & 3))) & 255u);
}

template <typename T, int BITS, int D>
__global__ void __launch_bounds__(64 * kAttnWaves) qattn_kernel(const nvq_attention_desc d, const T *__restrict__ q, const uint4 *__restrict__ kw,
                                                               const T *__restrict__ ks, const T *__restrict__ kb,
                                                               const uint4 *__restrict__ vw, const T *__restrict__ vs,
                                                               const T *__restrict__ vb, const T *__restrict__ sinks, T *__restrict__ out) {
    constexpr int CPL = 128 / BITS;        // codes (values of D) per lane
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

    for (int s0 = wave * KPT; s0 < S; s0 += kAttnWaves * KPT) {
        const int s = s0 + j;
        const bool live = s < S;
        const int64_t r = row0 + (live ? s : S - 1);  // a key past the end reads the last one and is given no weight
        const uint4 kc = kw[r * CH + c], vc = vw[r * CH + c];
        const float sk = Elem<T>::load(ks, r * groups + gi), bk = Elem<T>::load(kb, r * groups + gi);
        const float sv = Elem<T>::load(vs, r * groups + gi), bv = Elem<T>::load(vb, r * groups + gi);
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < CPL; i++) dot = __builtin_fmaf(qv[i], chunk_code<BITS>(kc, i), dot);
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
        for (int i = 0; i < CPL; i++) acc[i] = __builtin_fmaf(acc[i], corr, pv * chunk_code<BITS>(vc, i));
    }

    // merge: the block's maximum, every slot scaled to it, the slots added up
    const int slot = wave * KPT + j;
    if (c == 0) slot_m[slot] = m;
    __syncthreads();
    float top = -INFINITY;
    for (int t = 0; t < kSlots; t++) top = fmaxf(top, slot_m[t]);
    const float sink = sinks != nullptr ? Elem<T>::load(sinks, h) : -INFINITY;
    top = fmaxf(top, sink);
    const float w = m == -INFINITY ? 0.0f : __expf(m - top);
    if (c == 0) slot_l[slot] = l * w;
#pragma unroll
    for (int i = 0; i < CPL; i++) part[slot][c * CPL + i] = (acc[i] + accb) * w;
    __syncthreads();
    if (tid < D) {
        float denom = sinks != nullptr ? __expf(sink - top) : 0.0f, sum = 0.0f;
        for (int t = 0; t < kSlots; t++) {
            denom += slot_l[t];
            sum += part[t][tid];
        }
        Elem<T>::store(out, ((int64_t)b * d.query_heads + h) * D + tid, sum / denom);
    }
}

template <typename T, int BITS>
int32_t run_attention(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb, const void *vw,
                      const void *vs, const void *vb, const void *sinks, void *out, hipStream_t s) {
    const dim3 grid((unsigned)d.query_heads, (unsigned)d.batch), block(64 * kAttnWaves);
    if (d.head_dim == 64)
        hipLaunchKernelGGL((qattn_kernel<T, BITS, 64>), grid, block, 0, s, d, (const T *)q, (const uint4 *)kw, (const T *)ks, (const T *)kb,
                           (const uint4 *)vw, (const T *)vs, (const T *)vb, (const T *)sinks, (T *)out);
    else
        hipLaunchKernelGGL((qattn_kernel<T, BITS, 128>), grid, block, 0, s, d, (const T *)q, (const uint4 *)kw, (const T *)ks, (const T *)kb,
                           (const uint4 *)vw, (const T *)vs, (const T *)vb, (const T *)sinks, (T *)out);
    NVQ_LAUNCH_CHECK("quantized_attention");
    return NVQ_OK;
}

template <typename T>
int32_t run_attention_bits(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb, const void *vw,
                           const void *vs, const void *vb, const void *sinks, void *out, hipStream_t s) {
    return d.bits == 4 ? run_attention<T, 4>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, s)
                       : run_attention<T, 8>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, s);
}

}  // namespace

int32_t launch_quantized_attention(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb,
                                   const void *vw, const void *vs, const void *vb, const void *sinks, void *out, hipStream_t s) {
    switch (d.dtype) {
    case NVQ_F32: return run_attention_bits<float>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, s);
    case NVQ_BF16: return run_attention_bits<bf16_t>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, s);
    default: return run_attention_bits<f16_t>(d, q, kw, ks, kb, vw, vs, vb, sinks, out, s);
    }
}

}  // namespace nvq
