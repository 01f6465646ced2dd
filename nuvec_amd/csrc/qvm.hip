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

namespace nvq {
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
template <typename T, int BITS, int MODE, int RM>
__global__ void __launch_bounds__(64) qvm_kernel(const ProductArgs a, int splits, float *partial) {
    constexpr bool kAffine = MODE == NVQ_AFFINE;
    constexpr int kHalves = MODE == NVQ_NVFP4 ? 2 : 1;  // groups per lane
    const int lane = threadIdx.x;
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
    const int k_begin = blockIdx.y * per, k_end = k_begin + per < K ? k_begin + per : K;

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
        Row ring[2];
        load_row(k_begin, ring[0]);
        for (int k = k_begin; k < k_end; k += 2) {
#pragma unroll
            for (int d = 0; d < 2; d++) {
                load_row(k + d + 1, ring[(d + 1) & 1]);
                const Row &r = ring[d];
                if (k + d < k_end) {
                    float xs[RM][kHalves];
#pragma unroll
                    for (int i = 0; i < RM; i++) {
#pragma unroll
                        for (int hf = 0; hf < kHalves; hf++) xs[i][hf] = r.x[i] * r.s[hf];
                        accb[i] = __builtin_fmaf(r.x[i], r.b, accb[i]);
                    }
#pragma unroll
                    for (int j = 0; j < 32; j++) {
                        const uint32_t c = code_at<BITS>(r.d, j);
                        const float v = kAffine ? (float)c : (MODE == NVQ_MXFP8 ? e4m3_to_f32(c) : e2m1_to_f32(c));
#pragma unroll
                        for (int i = 0; i < RM; i++) acc[i][j] = __builtin_fmaf(xs[i][j * kHalves / 32], v, acc[i][j]);
                    }
                }
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int i = 0; i < RM; i++) {
        if (m0 + i >= M) break;
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
    float sum = 0.0f;
    for (int s = 0; s < splits; s++) sum += partial[(b * splits + s) * per_batch + rest];
    Elem<T>::store(y, idx, add_row_bias<T>(row_bias, sum, idx % n));
}

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
    if (rm == 1) hipLaunchKernelGGL((qvm_kernel<T, BITS, MODE, 1>), grid, dim3(64), 0, s, a, splits, (float *)workspace);
    else hipLaunchKernelGGL((qvm_kernel<T, BITS, MODE, 4>), grid, dim3(64), 0, s, a, splits, (float *)workspace);
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

// Splits of K: enough blocks for about four wavefronts per compute unit, at least 32 rows per split.
int qvm_splits(const ProductArgs &a) {
    const int rm = a.m == 1 ? 1 : 4;
    // row-exact: the split is the one-row product's, whatever the rows and batches, so that every row keeps its bits
    const int64_t base = ((a.n + 2047) / 2048) * (a.row_exact ? 1 : a.batch * ((a.m + rm - 1) / rm));
    const int64_t want = ((int64_t)compute_units() * 4 + base - 1) / base;
    const int64_t most = a.k / 32 > 1 ? a.k / 32 : 1;
    const int64_t splits = want < 1 ? 1 : (want > most ? most : want);
    return (int)(splits > 1024 ? 1024 : splits);
}

size_t qvm_workspace_bytes(const ProductArgs &a) {
    const int splits = qvm_splits(a);
    return splits > 1 ? (size_t)splits * (size_t)a.batch * (size_t)a.m * (size_t)a.n * sizeof(float) : 0;
}

int32_t launch_qvm(const ProductArgs &a, void *workspace, hipStream_t s) {
    switch (a.dtype) {
    case NVQ_F32: return run_qvm_typed<float>(a, workspace, s);
    case NVQ_BF16: return run_qvm_typed<bf16_t>(a, workspace, s);
    default: return run_qvm_typed<f16_t>(a, workspace, s);
    }
}

}  // namespace nvq
