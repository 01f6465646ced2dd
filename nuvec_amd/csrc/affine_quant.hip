// Affine quantize / dequantize for gfx950, bit for bit nuvec's CPU arithmetic
// (reference: crates/nuvec-core/src/kernels.rs:774-859).
//
// Both kernels are streaming: a lane owns 8 consecutive values, which is exactly `bits`
// bytes of the packed little-endian bit stream (value i at bit i*bits), so a lane's codes
// never share a byte with its neighbour's.  A quantization group of 32/64/128 values is
// 4/8/16 adjacent lanes of one wavefront; its extremes are folded with lane shuffles.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

constexpr int kBlock = 256;

template <typename T>
__device__ __forceinline__ void load8(const T *w, int64_t base, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = Elem<T>::load(w, base + i);
}
template <>
__device__ __forceinline__ void load8<float>(const float *w, int64_t base, float (&v)[8]) {
    const float4 *p = reinterpret_cast<const float4 *>(w + base);  // base % 8 == 0, w 16-byte aligned
    float4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t *w, int64_t base, float (&v)[8]) {
    uint4 q = *reinterpret_cast<const uint4 *>(w + base);
    uint32_t r[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[2 * i] = u2f(r[i] << 16);
        v[2 * i + 1] = u2f(r[i] & 0xFFFF0000u);
    }
}

template <>
__device__ __forceinline__ void load8<f16_t>(const f16_t *w, int64_t base, float (&v)[8]) {
    uint4 q = *reinterpret_cast<const uint4 *>(w + base);
    f16_t h[8];
    __builtin_memcpy(h, &q, 16);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = (float)h[i];
}

// Rounds 8 float32 values to T (they are already exact T values here) and stores them with
// 16-byte stores.
template <typename T>
__device__ __forceinline__ void store8(T *out, int64_t base, const float (&v)[8]);
template <>
__device__ __forceinline__ void store8<float>(float *out, int64_t base, const float (&v)[8]) {
    float4 *p = reinterpret_cast<float4 *>(out + base);
    p[0] = make_float4(v[0], v[1], v[2], v[3]);
    p[1] = make_float4(v[4], v[5], v[6], v[7]);
}
template <>
__device__ __forceinline__ void store8<bf16_t>(bf16_t *out, int64_t base, const float (&v)[8]) {
    uint32_t r[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        r[i] = f32_to_bf16_pair(v[2 * i], v[2 * i + 1]);
    stream_store(reinterpret_cast<uint4 *>(out + base), make_uint4(r[0], r[1], r[2], r[3]));
}
template <>
__device__ __forceinline__ void store8<f16_t>(f16_t *out, int64_t base, const float (&v)[8]) {
    f16_t h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = (f16_t)v[i];
    uint4 q;
    __builtin_memcpy(&q, h, 16);
    stream_store(reinterpret_cast<uint4 *>(out + base), q);
}

// Stores the low `BITS` bytes of `stream` at `bytes + BITS*chunk` with the widest stores the
// alignment allows.
template <int BITS>
__device__ __forceinline__ void store_codes(uint8_t *bytes, int64_t chunk, uint64_t stream) {
    uint8_t *p = bytes + chunk * BITS;
    if constexpr (BITS == 8) {
        *reinterpret_cast<uint2 *>(p) = make_uint2((uint32_t)stream, (uint32_t)(stream >> 32));
    } else if constexpr (BITS == 4) {
        *reinterpret_cast<uint32_t *>(p) = (uint32_t)stream;
    } else if constexpr (BITS == 2) {
        *reinterpret_cast<uint16_t *>(p) = (uint16_t)stream;
    } else if constexpr (BITS == 6) {
        uint16_t *h = reinterpret_cast<uint16_t *>(p);
        h[0] = (uint16_t)stream; h[1] = (uint16_t)(stream >> 16); h[2] = (uint16_t)(stream >> 32);
    } else {
#pragma unroll
        for (int b = 0; b < BITS; b++) p[b] = (uint8_t)(stream >> (8 * b));
    }
}

template <int BITS>
__device__ __forceinline__ uint64_t load_codes(const uint8_t *bytes, int64_t chunk) {
    const uint8_t *p = bytes + chunk * BITS;
    if constexpr (BITS == 8) {
        uint2 q = stream_load(reinterpret_cast<const uint2 *>(p));
        return (uint64_t)q.x | ((uint64_t)q.y << 32);
    } else if constexpr (BITS == 4) {
        return stream_load(reinterpret_cast<const uint32_t *>(p));
    } else if constexpr (BITS == 2) {
        return *reinterpret_cast<const uint16_t *>(p);
    } else if constexpr (BITS == 6) {
        const uint16_t *h = reinterpret_cast<const uint16_t *>(p);
        return (uint64_t)h[0] | ((uint64_t)h[1] << 16) | ((uint64_t)h[2] << 32);
    } else {
        uint64_t s = 0;
#pragma unroll
        for (int b = 0; b < BITS; b++) s |= (uint64_t)p[b] << (8 * b);
        return s;
    }
}

// ---- quantize ----
//
// A lane owns 32 consecutive values (a whole group of 32, half a group of 64, a quarter of a group of 128), so
// the group's extremes need at most two lane exchanges and the scale arithmetic (four divisions) is done once per
// 32 values.  A wavefront fetches its 64 x 32 values with coalesced 16-byte loads and turns them through a private
// LDS stage into one row per lane; the swizzle keeps both the 16-byte writes and the 16-byte reads free of bank
// conflicts on the 64 banks (a row is 4 or 8 pieces; 16 consecutive lanes must touch 16 different piece slots).
template <int P> __device__ __forceinline__ int stage_slot(int row, int piece) {
    if constexpr (P == 4) return row * 4 + (piece ^ ((row >> 2) & 3));
    else return row * 8 + (piece ^ ((row >> 1) & 7));
}

// The lane's 32 values as float32.  A signalling NaN is quieted (hardware min/max would return it, a quiet one
// they skip, as the reference's f32::min/max skip every NaN).
template <typename T> __device__ __forceinline__ void widen(const uint4 *in, float (&v)[32]);
template <> __device__ __forceinline__ void widen<float>(const uint4 *in, float (&v)[32]) {
#pragma unroll
    for (int p = 0; p < 8; p++) {
        v[4 * p] = u2f(in[p].x); v[4 * p + 1] = u2f(in[p].y); v[4 * p + 2] = u2f(in[p].z); v[4 * p + 3] = u2f(in[p].w);
    }
}
template <> __device__ __forceinline__ void widen<bf16_t>(const uint4 *in, float (&v)[32]) {
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const uint32_t r[4] = {in[p].x, in[p].y, in[p].z, in[p].w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[8 * p + 2 * i] = u2f(r[i] << 16);
            v[8 * p + 2 * i + 1] = u2f(r[i] & 0xFFFF0000u);
        }
    }
}
template <> __device__ __forceinline__ void widen<f16_t>(const uint4 *in, float (&v)[32]) {
#pragma unroll
    for (int p = 0; p < 4; p++) {
        f16_t h[8];
        __builtin_memcpy(h, &in[p], 16);
#pragma unroll
        for (int i = 0; i < 8; i++) v[8 * p + i] = (float)h[i];
    }
}

// The value of the lane `lane ^ 1` (kSwap1) or `lane ^ 2` (kSwap2): a move inside the quad, no LDS.
constexpr int kSwap1 = 0xB1, kSwap2 = 0x4E;
template <int CTRL> __device__ __forceinline__ float quad_swap(float x) {
    return u2f((uint32_t)__builtin_amdgcn_mov_dpp((int)f2u(x), CTRL, 0xF, 0xF, true));
}

// Packs 32 codes into BITS words of the little-endian bit stream.  `raw[i]` is the code plus JUNK (the bits of
// the float 1.5 * 2^23 when the code sits in a float's low mantissa bits); where a word holds whole codes the junk
// is summed along and taken off once per word, so a code costs one shift-and-add.
template <int BITS, uint32_t JUNK>
__device__ __forceinline__ void pack_words(const uint32_t (&raw)[32], uint32_t (&words)[BITS]) {
    if constexpr (32 % BITS == 0) {
        constexpr int kPer = 32 / BITS;
        uint64_t ones = 0;
        for (int i = 0; i < kPer; i++) ones += (uint64_t)1 << (BITS * i);
        const uint32_t junk = (uint32_t)((uint64_t)JUNK * ones);
#pragma unroll
        for (int k = 0; k < BITS; k++) {
            uint32_t acc = raw[k * kPer + kPer - 1];
#pragma unroll
            for (int i = kPer - 2; i >= 0; i--) acc = (acc << BITS) + raw[k * kPer + i];
            words[k] = acc - junk;
        }
    } else {
#pragma unroll
        for (int k = 0; k < BITS; k++) words[k] = 0u;
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const uint32_t code = raw[i] - JUNK;
            const int k = (i * BITS) / 32, shift = (i * BITS) % 32;
            words[k] |= code << shift;
            if (shift + BITS > 32) words[k + 1] |= code >> (32 - shift);
        }
    }
}

// kernels.rs:774-831.  `rows` = n_values / 32; a group is `1 << lanes_log2` adjacent lanes (1, 2 or 4).
template <typename T, int BITS>
__global__ void __launch_bounds__(kBlock)
affine_quantize_kernel(const T *__restrict__ w, int64_t rows, int lanes_log2, uint32_t *__restrict__ packed,
                       T *__restrict__ scales, T *__restrict__ biases) {
    constexpr int P = 32 * (int)sizeof(T) / 16;  // 16-byte pieces of a lane's row
    __shared__ uint4 stages[kBlock / 64][64 * P];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row0 = ((int64_t)blockIdx.x * (kBlock / 64) + wave) * 64;
    if (row0 >= rows) return;  // the whole wavefront; nothing below synchronizes across wavefronts
    uint4 *stage = stages[wave];
    const uint4 *src = reinterpret_cast<const uint4 *>(w) + row0 * P;
    const int64_t last = (rows - row0) * P - 1;  // beyond the end the last piece is read again and never used
    uint4 in[P];
#pragma unroll
    for (int j = 0; j < P; j++) in[j] = stream_load(src + min((int64_t)(j * 64 + lane), last));
#pragma unroll
    for (int j = 0; j < P; j++) {
        const int c = j * 64 + lane;
        stage[stage_slot<P>(c / P, c % P)] = in[j];
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = 0; p < P; p++) in[p] = stage[stage_slot<P>(lane, p)];
    float v[32];
    widen<T>(in, v);
#pragma unroll
    for (int i = 0; i < 32; i++) v[i] = __builtin_canonicalizef(v[i]);

    // f32 extremes of the group: the hardware's min/max skip NaN and order -0 below +0, as the reference's fold
    // from +Inf / -Inf does on its hosts, so the order of the fold does not matter.
    float lo = INFINITY, hi = -INFINITY;
#pragma unroll
    for (int i = 0; i < 32; i++) { lo = __builtin_fminf(lo, v[i]); hi = __builtin_fmaxf(hi, v[i]); }
    if (lanes_log2 >= 1) {
        lo = __builtin_fminf(lo, quad_swap<kSwap1>(lo));
        hi = __builtin_fmaxf(hi, quad_swap<kSwap1>(hi));
    }
    if (lanes_log2 >= 2) {
        lo = __builtin_fminf(lo, quad_swap<kSwap2>(lo));
        hi = __builtin_fmaxf(hi, quad_swap<kSwap2>(hi));
    }
    constexpr float n_bins = (float)((1u << BITS) - 1u);
    const float eps = 1e-7f;
    float scale, bias;
    if constexpr (BITS == 1) {
        scale = __builtin_fmaxf(hi - lo, eps);
        bias = lo;
    } else {
        const bool wide = fabsf(lo) > fabsf(hi);
        scale = __builtin_fmaxf((hi - lo) / n_bins, eps);
        scale = wide ? scale : -scale;
        const float edge = wide ? lo : hi;
        const float q0 = rintf(edge / scale);
        if (q0 == 0.0f) {
            bias = 0.0f;
        } else {
            scale = edge / q0;
            bias = edge;
        }
    }
    // code = clamp(rint((v - bias) / scale)) with the correctly rounded quotient.  Thirty-two divisions would be the
    // bulk of the kernel; with y = 1 / scale (correctly rounded, once per lane) the quotient of d by scale is
    // t0 = d * y, then twice t <- fma(fma(-scale, t, d), y, t): the first step leaves t within a rounding of the
    // quotient and the second is then the correctly rounded quotient itself (Markstein's theorem, the same
    // scheme the compiler's own division expands to, with a better reciprocal).  It needs scale, y and the
    // remainders in the normal range: other groups (tiny or huge scales, infinite values) take the divisions.
    // Adding 1.5 * 2^23 rounds to the nearest integer, ties to even, and leaves it in the low mantissa bits.
    constexpr float kMagic = 12582912.0f;
    const float y = 1.0f / scale;
    const float mag = fabsf(scale);
    const bool plain = mag > 1e-20f && mag < 1e20f && (hi - lo) * fabsf(y) < 1024.0f;
    uint32_t raw[32], words[BITS];
#pragma unroll
    for (int i = 0; i < 32; i++) {
        const float d = v[i] - bias;
        float t = d * y;
        t = __builtin_fmaf(__builtin_fmaf(-scale, t, d), y, t);
        t = __builtin_fmaf(__builtin_fmaf(-scale, t, d), y, t);
        raw[i] = f2u(__builtin_amdgcn_fmed3f(t + kMagic, kMagic, kMagic + n_bins));  // NaN -> the smallest: code 0
    }
    pack_words<BITS, 0x4B400000u>(raw, words);
    if (!plain) {
#pragma unroll
        for (int i = 0; i < 32; i++) {
            float q = rintf((v[i] - bias) / scale);
            q = fminf(fmaxf(q, 0.0f), n_bins);  // NaN -> 0, as Rust's clamp followed by `as u32`
            raw[i] = (uint32_t)q;
        }
        pack_words<BITS, 0u>(raw, words);
    }
    const int64_t row = row0 + lane;
    if (row >= rows) return;
    if constexpr (BITS == 4) {
        stream_store(reinterpret_cast<uint4 *>(packed + row * 4), make_uint4(words[0], words[1], words[2], words[3]));
    } else if constexpr (BITS == 8) {
        stream_store(reinterpret_cast<uint4 *>(packed + row * 8), make_uint4(words[0], words[1], words[2], words[3]));
        stream_store(reinterpret_cast<uint4 *>(packed + row * 8) + 1, make_uint4(words[4], words[5], words[6], words[7]));
    } else {
        struct Words { uint32_t w[BITS]; } out;
#pragma unroll
        for (int k = 0; k < BITS; k++) out.w[k] = words[k];
        *reinterpret_cast<Words *>(packed + row * BITS) = out;
    }
    if ((lane & ((1 << lanes_log2) - 1)) == 0) {
        const int64_t g = row >> lanes_log2;
        Elem<T>::store(scales, g, scale);
        Elem<T>::store(biases, g, bias);
    }
}

// kernels.rs:835-859: round(round(code * scale) + bias), both roundings in T.  With `ids`, output row r is
// table row ids[r] (the rows of a quantized embedding, crates/nuvec-nn/src/layers.rs:245-255): `row_chunks` chunks
// per row, ids clamped to the table's `table_rows`.
// Chunks per thread, a block apart: all their loads are requested before the first conversion.  (The 16-bit types;
// float32 has the kernel below.)
template <typename T> constexpr int kUnrollOf = sizeof(T) == 4 ? 1 : 4;
template <typename T, int BITS>
__global__ void __launch_bounds__(kBlock)
affine_dequantize_kernel(const uint8_t *__restrict__ packed, const T *__restrict__ scales,
                         const T *__restrict__ biases, uint32_t chunks, int lanes_log2, T *__restrict__ out,
                         const uint32_t *__restrict__ ids, uint32_t row_chunks, int64_t table_rows) {
    constexpr int kUnroll = kUnrollOf<T>;
    const uint32_t first = blockIdx.x * (kBlock * kUnroll) + threadIdx.x;  // fewer than 2^29: an operand has fewer than 2^32 elements
    uint64_t stream_[kUnroll];
    T s_[kUnroll], b_[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint32_t at = first + u * kBlock;
        const uint32_t chunk = at < chunks ? at : chunks - 1;  // past the end: the last chunk again, never stored
        int64_t src = chunk;
        if (ids != nullptr) {
            const uint32_t r = chunk / row_chunks;
            const int64_t row = min((int64_t)ids[r], table_rows - 1);
            src = row * row_chunks + (chunk - r * row_chunks);
        }
        stream_[u] = load_codes<BITS>(packed, src);
        const int64_t g = src >> lanes_log2;
        s_[u] = scales[g];
        b_[u] = biases[g];
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const uint32_t chunk = first + u * kBlock;
        if (chunk >= chunks) continue;
        const uint64_t stream = stream_[u];
        const float s = Elem<T>::load(&s_[u], 0), b = Elem<T>::load(&b_[u], 0);
        constexpr uint32_t mask = (1u << BITS) - 1u;
        float c[8];
#pragma unroll
        for (int i = 0; i < 8; i++) c[i] = (float)((uint32_t)(stream >> (i * BITS)) & mask);
        if constexpr (sizeof(T) == 2 && Elem<T>::code == 10) {
            // bfloat16: the two roundings of a pair of values are one conversion instruction each.
            uint32_t r[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t p = f32_to_bf16_pair(c[2 * i] * s, c[2 * i + 1] * s);
                r[i] = f32_to_bf16_pair(u2f(p << 16) + b, u2f(p & 0xFFFF0000u) + b);
            }
            stream_store(reinterpret_cast<uint4 *>(out + (int64_t)chunk * 8), make_uint4(r[0], r[1], r[2], r[3]));
        } else {
            float r[8];
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = Elem<T>::add(Elem<T>::mul(c[i], s), b);
            store8<T>(out, (int64_t)chunk * 8, r);
        }
    }
}

// float32 out: a lane's eight values would leave as two 16-byte stores 32 bytes apart.  Here a lane takes four values, one
// half of a chunk, of two chunks that lie 32 chunks apart, so that each of a wavefront's two stores writes 1 KB of
// consecutive bytes; the two lanes of a chunk read the same codes, scale and bias.  The arithmetic of a value is the same.
// [4096,4096] at 4 bits in groups of 64: 18.9 us with the eight-value lanes, 16.3 us with these stores, 12.0-15.1 us with
// them non-temporal; 3 bits in groups of 128: 20.8 -> 11.8 us.
template <int BITS>
__global__ void __launch_bounds__(kBlock)
affine_dequantize_f32_kernel(const uint8_t *__restrict__ packed, const float *__restrict__ scales, const float *__restrict__ biases,
                             uint32_t chunks, int lanes_log2, float *__restrict__ out, const uint32_t *__restrict__ ids,
                             uint32_t row_chunks, int64_t table_rows) {
    const uint32_t lane = threadIdx.x & 63u, half = lane & 1u;
    const uint32_t base = blockIdx.x * kBlock + (threadIdx.x & ~63u);  // the wavefront's 64 chunks
    uint64_t stream_[2];
    float s_[2], b_[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t at = base + 32 * j + (lane >> 1);
        const uint32_t chunk = at < chunks ? at : chunks - 1;  // past the end: the last chunk again, never stored
        int64_t src = chunk;
        if (ids != nullptr) {
            const uint32_t r = chunk / row_chunks;
            const int64_t row = min((int64_t)ids[r], table_rows - 1);
            src = row * row_chunks + (chunk - r * row_chunks);
        }
        stream_[j] = load_codes<BITS>(packed, src) >> (half * 4 * BITS);
        const int64_t g = src >> lanes_log2;
        s_[j] = scales[g];
        b_[j] = biases[g];
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t chunk = base + 32 * j + (lane >> 1);
        if (chunk >= chunks) continue;
        constexpr uint32_t mask = (1u << BITS) - 1u;
        float r[4];
#pragma unroll
        for (int i = 0; i < 4; i++) r[i] = Elem<float>::add(Elem<float>::mul((float)((uint32_t)(stream_[j] >> (i * BITS)) & mask), s_[j]), b_[j]);
        // written once and not read here again: a non-temporal store
        stream_store(reinterpret_cast<uint4 *>(out + (int64_t)chunk * 8 + half * 4), make_uint4(f2u(r[0]), f2u(r[1]), f2u(r[2]), f2u(r[3])));
    }
}

template <typename T, int BITS>
int32_t quantize_t(int group, const void *w, int64_t n, void *packed, void *scales, void *biases, hipStream_t s) {
    const int64_t rows = n / 32;  // a lane's 32 values; the group is 1, 2 or 4 of them
    const unsigned blocks = (unsigned)((rows + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((affine_quantize_kernel<T, BITS>), dim3(blocks), dim3(kBlock), 0, s, (const T *)w, rows,
                       group == 32 ? 0 : group == 64 ? 1 : 2, (uint32_t *)packed, (T *)scales, (T *)biases);
    NVQ_LAUNCH_CHECK("affine_quantize");
    return NVQ_OK;
}
template <typename T, int BITS>
int32_t dequantize_t(int group, const void *packed, const void *scales, const void *biases, int64_t n, void *out,
                     const uint32_t *ids, int64_t cols, int64_t table_rows, hipStream_t s) {
    const int64_t chunks = n / 8;
    if constexpr (std::is_same<T, float>::value) {
        hipLaunchKernelGGL((affine_dequantize_f32_kernel<BITS>), dim3((unsigned)((chunks + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                           (const uint8_t *)packed, (const float *)scales, (const float *)biases, (uint32_t)chunks,
                           group == 32 ? 2 : group == 64 ? 3 : 4, (float *)out, ids, (uint32_t)(cols / 8), table_rows);
        NVQ_LAUNCH_CHECK("affine_dequantize");
        return NVQ_OK;
    }
    const unsigned blocks = (unsigned)((chunks + kBlock * kUnrollOf<T> - 1) / (kBlock * kUnrollOf<T>));
    hipLaunchKernelGGL((affine_dequantize_kernel<T, BITS>), dim3(blocks), dim3(kBlock), 0, s,
                       (const uint8_t *)packed, (const T *)scales, (const T *)biases, (uint32_t)chunks,
                       group == 32 ? 2 : group == 64 ? 3 : 4, (T *)out, ids, (uint32_t)(cols / 8), table_rows);
    NVQ_LAUNCH_CHECK("affine_dequantize");
    return NVQ_OK;
}

#define NVQ_BITS_SWITCH(bits, CALL)                                      \
    switch (bits) {                                                      \
    case 1: return CALL(1);                                              \
    case 2: return CALL(2);                                              \
    case 3: return CALL(3);                                              \
    case 4: return CALL(4);                                              \
    case 5: return CALL(5);                                              \
    case 6: return CALL(6);                                              \
    case 8: return CALL(8);                                              \
    default: return fail(NVQ_INVALID_ARGUMENT, "%d bits are not supported", bits); \
    }

}  // namespace

int32_t launch_affine_quantize(int32_t dtype, int group, int bits, const void *w, int64_t n, void *packed,
                               void *scales, void *biases, hipStream_t s) {
#define Q_F32(B) quantize_t<float, B>(group, w, n, packed, scales, biases, s)
#define Q_BF16(B) quantize_t<bf16_t, B>(group, w, n, packed, scales, biases, s)
#define Q_F16(B) quantize_t<f16_t, B>(group, w, n, packed, scales, biases, s)
    if (dtype == NVQ_F32) { NVQ_BITS_SWITCH(bits, Q_F32) }
    if (dtype == NVQ_BF16) { NVQ_BITS_SWITCH(bits, Q_BF16) }
    NVQ_BITS_SWITCH(bits, Q_F16)
}

int32_t launch_affine_dequantize(int32_t dtype, int group, int bits, const void *packed, const void *scales,
                                 const void *biases, int64_t n, void *out, const uint32_t *ids, int64_t cols,
                                 int64_t table_rows, hipStream_t s) {
#define D_F32(B) dequantize_t<float, B>(group, packed, scales, biases, n, out, ids, cols, table_rows, s)
#define D_BF16(B) dequantize_t<bf16_t, B>(group, packed, scales, biases, n, out, ids, cols, table_rows, s)
#define D_F16(B) dequantize_t<f16_t, B>(group, packed, scales, biases, n, out, ids, cols, table_rows, s)
    if (dtype == NVQ_F32) { NVQ_BITS_SWITCH(bits, D_F32) }
    if (dtype == NVQ_BF16) { NVQ_BITS_SWITCH(bits, D_BF16) }
    NVQ_BITS_SWITCH(bits, D_F16)
}

}  // namespace nvq
