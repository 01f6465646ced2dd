// Index helpers of the gathered products (reference: crates/nuvec-core/src/kernels.rs:873-892,
// crates/nuvec-kernels/src/metal/gather_gemm.metal:436-457).
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

// offsets[row, g] = first position of `indices[row, :]` whose value is not below g
// (a lower bound by binary search; the row is sorted by the caller's contract).
__global__ void sorted_offsets_kernel(const uint32_t *__restrict__ indices, int64_t rows, int64_t m, int32_t groups,
                                      int32_t *__restrict__ offsets) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= rows * groups) return;
    const int64_t r = t / groups;
    const uint32_t g = (uint32_t)(t % groups);
    const uint32_t *row = indices + r * m;
    int64_t lo = 0, hi = m;
    while (lo < hi) {
        const int64_t mid = lo + (hi - lo) / 2;
        if (row[mid] < g) lo = mid + 1; else hi = mid;
    }
    offsets[t] = (int32_t)lo;
}

// The pairs (token, choice) of a mixture-of-experts layer ordered by expert, stably: what SwitchGlu::forward gets
// from `argsort` of the flattened expert ids, its inverse, and `sorted_offsets` of the sorted ids
// (crates/nuvec-lm/src/model.rs:2193-2210), in one block.  A counting sort: a histogram of the ids in LDS, an
// exclusive scan over the experts (the offsets), then the pairs placed chunk by chunk in pair order; inside a
// chunk a pair's rank among the equal ids before it comes from wavefront ballots (lanes before it in its own
// wavefront) plus the counts of the wavefronts before its own.
constexpr int kOrderThreads = 1024, kOrderWaves = kOrderThreads / 64;

// Places the pairs [chunk, chunk + 1024) of the block stably: `next[e]` is where expert e's next pair goes (advanced by
// the chunk's count); `wave_count` is scratch [wavefronts][experts].  A pair's rank among the equal ids before it in
// the chunk comes from wavefront ballots (lanes before it in its own wavefront) plus the counts of the wavefronts
// before its own.
__device__ __forceinline__ void place_chunk(const uint32_t *__restrict__ ids, int64_t pairs, int32_t experts, int64_t chunk,
                                            int32_t *next, int32_t *wave_count, uint32_t *__restrict__ order,
                                            uint32_t *__restrict__ restore, uint32_t *__restrict__ sorted_ids) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < kOrderWaves * experts; i += kOrderThreads) wave_count[i] = 0;
    __syncthreads();
    const int64_t p = chunk + tid;
    const bool live = p < pairs;
    const uint32_t e = live ? min(ids[p], (uint32_t)(experts - 1)) : 0u;  // an id beyond the experts is clamped
    // Rank among the lanes of this wavefront with the same id: one ballot per distinct id.
    int rank = 0;
    uint64_t todo = __ballot(live);
    while (todo != 0) {
        const int leader = __ffsll((long long)todo) - 1;
        const uint32_t e0 = __shfl(e, leader);
        const uint64_t same = __ballot(live && e == e0);
        if (live && e == e0) {
            rank = __popcll(same & ((1ull << lane) - 1ull));
            if (lane == leader) wave_count[wave * experts + e0] = __popcll(same);
        }
        todo &= ~same;
    }
    __syncthreads();
    if (live) {
        int before = 0;
        for (int w = 0; w < wave; w++) before += wave_count[w * experts + e];
        const uint32_t at = (uint32_t)(next[e] + before + rank);
        order[at] = (uint32_t)p;
        restore[p] = at;
        sorted_ids[at] = e;
    }
    __syncthreads();
    for (int ee = tid; ee < experts; ee += kOrderThreads) {
        int total = 0;
        for (int w = 0; w < kOrderWaves; w++) total += wave_count[w * experts + ee];
        next[ee] += total;
    }
    __syncthreads();
}

__global__ void __launch_bounds__(kOrderThreads)
moe_order_kernel(const uint32_t *__restrict__ ids, int64_t pairs, int32_t experts, uint32_t *__restrict__ order,
                 uint32_t *__restrict__ restore, uint32_t *__restrict__ sorted_ids, int32_t *__restrict__ offsets) {
    extern __shared__ int32_t lds_i[];
    int32_t *next = lds_i;                       // [experts]: histogram, then where each expert's next pair goes
    int32_t *wave_count = lds_i + experts;       // [waves][experts]: this chunk's pairs per wavefront and expert
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < experts; e += kOrderThreads) next[e] = 0;
    __syncthreads();
    for (int64_t p = tid; p < pairs; p += kOrderThreads) atomicAdd(&next[min(ids[p], (uint32_t)(experts - 1))], 1);
    __syncthreads();
    // Exclusive scan by one wavefront, 64 experts at a time.
    if (wave == 0) {
        int32_t carry = 0;
        for (int base = 0; base < experts; base += 64) {
            const int e = base + lane;
            const int32_t count = e < experts ? next[e] : 0;
            int32_t incl = count;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int32_t up = __shfl_up(incl, d);
                if (lane >= d) incl += up;
            }
            if (e < experts) {
                next[e] = carry + incl - count;
                offsets[e] = carry + incl - count;
            }
            carry += __shfl(incl, 63);
        }
    }
    __syncthreads();
    for (int64_t chunk = 0; chunk < pairs; chunk += kOrderThreads) place_chunk(ids, pairs, experts, chunk, next, wave_count, order, restore, sorted_ids);
}

// The same ordering for many pairs, over the whole chip in three steps: every block counts the ids of its chunk of
// 1024 pairs; one block turns the counts into the experts' offsets and, per chunk and expert, the position of the
// chunk's first such pair (chunks in order: the sort stays stable); every block places its chunk.
__global__ void __launch_bounds__(kOrderThreads)
moe_count_kernel(const uint32_t *__restrict__ ids, int64_t pairs, int32_t experts, int32_t *__restrict__ counts) {
    extern __shared__ int32_t lds_i[];
    const int tid = threadIdx.x;
    for (int e = tid; e < experts; e += kOrderThreads) lds_i[e] = 0;
    __syncthreads();
    const int64_t p = (int64_t)blockIdx.x * kOrderThreads + tid;
    if (p < pairs) atomicAdd(&lds_i[min(ids[p], (uint32_t)(experts - 1))], 1);
    __syncthreads();
    for (int e = tid; e < experts; e += kOrderThreads) counts[(int64_t)blockIdx.x * experts + e] = lds_i[e];
}

__global__ void __launch_bounds__(kOrderThreads)
moe_scan_kernel(int32_t *__restrict__ counts, int32_t chunks, int32_t experts, int32_t *__restrict__ offsets) {
    extern __shared__ int32_t lds_i[];  // [experts]: totals, then offsets
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < experts; e += kOrderThreads) {
        int32_t total = 0;
        for (int c = 0; c < chunks; c++) total += counts[(int64_t)c * experts + e];
        lds_i[e] = total;
    }
    __syncthreads();
    if (wave == 0) {  // exclusive scan over the experts, 64 at a time
        int32_t carry = 0;
        for (int base = 0; base < experts; base += 64) {
            const int e = base + lane;
            const int32_t count = e < experts ? lds_i[e] : 0;
            int32_t incl = count;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int32_t up = __shfl_up(incl, d);
                if (lane >= d) incl += up;
            }
            if (e < experts) {
                lds_i[e] = carry + incl - count;
                offsets[e] = carry + incl - count;
            }
            carry += __shfl(incl, 63);
        }
    }
    __syncthreads();
    for (int e = tid; e < experts; e += kOrderThreads) {
        int32_t at = lds_i[e];
        for (int c = 0; c < chunks; c++) {
            const int32_t n = counts[(int64_t)c * experts + e];
            counts[(int64_t)c * experts + e] = at;
            at += n;
        }
    }
}

__global__ void __launch_bounds__(kOrderThreads)
moe_place_kernel(const uint32_t *__restrict__ ids, int64_t pairs, int32_t experts, const int32_t *__restrict__ starts,
                 uint32_t *__restrict__ order, uint32_t *__restrict__ restore, uint32_t *__restrict__ sorted_ids) {
    extern __shared__ int32_t lds_i[];
    int32_t *next = lds_i, *wave_count = lds_i + experts;
    for (int e = threadIdx.x; e < experts; e += kOrderThreads) next[e] = starts[(int64_t)blockIdx.x * experts + e];
    __syncthreads();
    place_chunk(ids, pairs, experts, (int64_t)blockIdx.x * kOrderThreads, next, wave_count, order, restore, sorted_ids);
}

// round(a / b) in the element type.  The float32 quotient is correctly rounded and float32 carries more than twice
// the element types' digits, so rounding it again gives the correctly rounded quotient of the element type.
template <typename T> __device__ __forceinline__ float elem_div(float a, float b) {
    if constexpr (sizeof(T) == 4) return a / b;
    else if constexpr (Elem<T>::code == 10) return bf16_bits_to_f32(f32_to_bf16_bits(a / b));
    else return (float)(f16_t)(a / b);
}

// The order of the reference's sort: NaN last for float32 and half; bfloat16 compares plainly, as its sort does
// (crates/nuvec-kernels/src/metal/moe.metal:19-31).
template <typename T> __device__ __forceinline__ bool route_less(float a, float b) {
    if constexpr (Elem<T>::code != 10) {
        const bool an = a != a, bn = b != b;
        if (an | bn) return (!an) & bn;
    }
    return a < b;
}

// fast::moe_route (crates/nuvec-kernels/src/metal/moe.metal:33-88): per row of `n` probabilities the k largest in
// the stable ascending order, their values and, with `normalize`, those divided by their sum (summed in the
// element type, in order).  One block per row, one thread per expert: an expert's position in the sorted row is
// the number of experts sorting before it.
template <typename T>
__global__ void __launch_bounds__(1024) moe_route_kernel(const T *__restrict__ probs, uint32_t *__restrict__ indices,
                                                         T *__restrict__ scores, int n, int k, int normalize) {
    __shared__ float p[1024], top[1024];
    __shared__ float total;
    const int e = threadIdx.x;
    const int64_t row = blockIdx.x;
    probs += row * n;
    indices += row * k;
    scores += row * k;
    if (e < n) p[e] = Elem<T>::load(probs, e);
    __syncthreads();
    if (e < n) {
        const float v = p[e];
        int rank = 0;
        for (int j = 0; j < n; j++) {
            const float u = p[j];
            rank += (route_less<T>(u, v) || (!route_less<T>(v, u) && j < e)) ? 1 : 0;
        }
        const int slot = rank - (n - k);
        if (slot >= 0) {
            indices[slot] = (uint32_t)e;
            top[slot] = v;
        }
    }
    __syncthreads();
    if (normalize) {
        if (e == 0) {
            float sum = 0.0f;
            for (int j = 0; j < k; j++) sum = Elem<T>::add(top[j], sum);
            total = sum;
        }
        __syncthreads();
        if (e < k) Elem<T>::store(scores, e, elem_div<T>(top[e], total));
    } else if (e < k) {
        Elem<T>::store(scores, e, top[e]);
    }
}

// fast::weighted_sum (moe.metal:90-118): out[r, c] = sum over j of x[r, j, c] * w[r, j], every product and every
// addition rounded to the element type: min(k, 8) partial sums of every min(k, 8)-th product (one partial sum when
// D = 1), added in order.  One thread per output element.
template <typename T>
__global__ void __launch_bounds__(256) weighted_sum_kernel(const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ out,
                                                           int64_t rows, int k, int64_t d) {
    const int64_t at = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= rows * d) return;
    const int64_t r = at / d, c = at - r * d;
    x += r * k * d + c;
    w += r * k;
    const int lanes = d == 1 ? 1 : (k < 8 ? k : 8);
    float sum = 0.0f;
    for (int y = 0; y < lanes; y++) {
        float t = 0.0f;
        for (int j = y; j < k; j += lanes) t = Elem<T>::add(Elem<T>::mul(Elem<T>::load(x, (int64_t)j * d), Elem<T>::load(w, j)), t);
        sum = y == 0 ? t : Elem<T>::add(t, sum);
    }
    Elem<T>::store(out, at, sum);
}

__global__ void fill_zero_kernel(uint16_t *p, int64_t halves) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < halves) p[t] = 0;
}

}  // namespace

int32_t launch_sorted_offsets(const uint32_t *indices, int64_t rows, int64_t m, int32_t groups, int32_t *offsets,
                              hipStream_t s) {
    const int64_t n = rows * groups;
    hipLaunchKernelGGL(sorted_offsets_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, indices, rows, m, groups, offsets);
    NVQ_LAUNCH_CHECK("sorted_offsets");
    return NVQ_OK;
}

size_t moe_order_lds_bytes(int32_t experts) { return (size_t)(1 + kOrderWaves) * experts * sizeof(int32_t); }

// Above this many pairs the ordering runs over the whole chip (three launches) when the caller gave the workspace.
constexpr int64_t kOrderOneBlock = 2048;
size_t moe_order_workspace_bytes(int64_t pairs, int32_t experts) {
    if (pairs <= kOrderOneBlock) return 0;
    return (size_t)((pairs + kOrderThreads - 1) / kOrderThreads) * (size_t)experts * sizeof(int32_t);
}

int32_t launch_moe_order(const uint32_t *ids, int64_t pairs, int32_t experts, uint32_t *order, uint32_t *restore,
                         uint32_t *sorted_ids, int32_t *offsets, void *workspace, hipStream_t s) {
    if (workspace == nullptr || pairs <= kOrderOneBlock) {
        hipLaunchKernelGGL(moe_order_kernel, dim3(1), dim3(kOrderThreads), moe_order_lds_bytes(experts), s, ids, pairs, experts, order,
                           restore, sorted_ids, offsets);
        NVQ_LAUNCH_CHECK("moe_order");
        return NVQ_OK;
    }
    const unsigned chunks = (unsigned)((pairs + kOrderThreads - 1) / kOrderThreads);
    int32_t *counts = (int32_t *)workspace;
    hipLaunchKernelGGL(moe_count_kernel, dim3(chunks), dim3(kOrderThreads), (size_t)experts * sizeof(int32_t), s, ids, pairs, experts, counts);
    NVQ_LAUNCH_CHECK("moe_order (count)");
    hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(kOrderThreads), (size_t)experts * sizeof(int32_t), s, counts, (int32_t)chunks, experts, offsets);
    NVQ_LAUNCH_CHECK("moe_order (scan)");
    hipLaunchKernelGGL(moe_place_kernel, dim3(chunks), dim3(kOrderThreads), moe_order_lds_bytes(experts), s, ids, pairs, experts, counts, order,
                       restore, sorted_ids);
    NVQ_LAUNCH_CHECK("moe_order (place)");
    return NVQ_OK;
}

int32_t launch_moe_route(int32_t dtype, const void *probs, int64_t rows, int32_t experts, int32_t k, int32_t normalize,
                         uint32_t *indices, void *scores, hipStream_t s) {
    const dim3 grid((unsigned)rows), block((unsigned)((experts + 63) / 64 * 64));
    if (dtype == NVQ_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, grid, block, 0, s, (const float *)probs, indices, (float *)scores, experts, k, normalize);
    else if (dtype == NVQ_BF16)
        hipLaunchKernelGGL(moe_route_kernel<bf16_t>, grid, block, 0, s, (const bf16_t *)probs, indices, (bf16_t *)scores, experts, k, normalize);
    else
        hipLaunchKernelGGL(moe_route_kernel<f16_t>, grid, block, 0, s, (const f16_t *)probs, indices, (f16_t *)scores, experts, k, normalize);
    NVQ_LAUNCH_CHECK("moe_route");
    return NVQ_OK;
}

int32_t launch_weighted_sum(int32_t dtype, const void *x, const void *w, int64_t rows, int32_t k, int64_t d, void *out, hipStream_t s) {
    const dim3 grid((unsigned)((rows * d + 255) / 256)), block(256);
    if (dtype == NVQ_F32)
        hipLaunchKernelGGL(weighted_sum_kernel<float>, grid, block, 0, s, (const float *)x, (const float *)w, (float *)out, rows, k, d);
    else if (dtype == NVQ_BF16)
        hipLaunchKernelGGL(weighted_sum_kernel<bf16_t>, grid, block, 0, s, (const bf16_t *)x, (const bf16_t *)w, (bf16_t *)out, rows, k, d);
    else
        hipLaunchKernelGGL(weighted_sum_kernel<f16_t>, grid, block, 0, s, (const f16_t *)x, (const f16_t *)w, (f16_t *)out, rows, k, d);
    NVQ_LAUNCH_CHECK("weighted_sum");
    return NVQ_OK;
}

// Zero-fills `bytes` (even: element sizes are 2 or 4) with a kernel, so that a caller capturing
// the stream into a graph records no memset node.
int32_t launch_fill_zero(void *p, int64_t bytes, hipStream_t s) {
    const int64_t halves = bytes / 2;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((halves + 255) / 256)), dim3(256), 0, s, (uint16_t *)p, halves);
    NVQ_LAUNCH_CHECK("fill_zero");
    return NVQ_OK;
}

}  // namespace nvq
