// The gated activation between the experts' up / gate products and their down product, in one pass over the two
// products: each row's expert's bias added to either (the reference's `SwitchProjection::forward`,
// crates/nuvec-lm/src/model.rs:2139-2143: `y + bias[indices]`), then SwiGLU or gpt-oss's clamped SwiGLU
// (`SwitchGlu::through`, model.rs:2157-2170; crates/nuvec-nn/src/lib.rs:513-519 `silu(gate) * x` with
// `silu(x) = x * sigmoid(x)` lib.rs:343-345, and lib.rs:564-570).  The reference evaluates the graph one operation
// at a time, each result an array of the activations' type (crates/nuvec-core/src/fused.rs:190-215), so every
// operation below rounds to that type; sigmoid is kernels.rs:1539-1543 in float32.
#include "nvq_device.h"
#include "nvq_internal.h"

namespace nvq {
namespace {

// One thread per output element; consecutive threads take consecutive columns of a row.
template <typename T, int ACT>
__global__ void __launch_bounds__(256) glu_kernel(const T *__restrict__ gate, const T *__restrict__ up, const T *__restrict__ gate_bias,
                                                  const T *__restrict__ up_bias, const int32_t *__restrict__ ids, T *__restrict__ out,
                                                  int64_t rows, int64_t hidden, int64_t gate_stride, int64_t up_stride, int64_t experts,
                                                  float alpha, float limit) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * hidden) return;
    const int64_t r = idx / hidden, c = idx - r * hidden;
    float g = Elem<T>::load(gate, r * gate_stride + c), u = Elem<T>::load(up, r * up_stride + c);
    if (gate_bias != nullptr) {
        int64_t e = ids[r];  // an id outside the biases is the caller's error: clamped
        e = e < 0 ? 0 : (e >= experts ? experts - 1 : e);
        g = Elem<T>::add(g, Elem<T>::load(gate_bias, e * hidden + c));
        u = Elem<T>::add(u, Elem<T>::load(up_bias, e * hidden + c));
    }
    Elem<T>::store(out, idx, glu<T, ACT>(g, u, alpha, limit));
}

template <typename T>
int32_t run_glu(const nvq_glu_desc &d, const void *gate, const void *up, const void *gate_bias, const void *up_bias, const int32_t *ids,
                void *out, hipStream_t s) {
    const int64_t total = d.rows * d.hidden;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    const float alpha = d.alpha, limit = d.limit;
    if (d.activation == NVQ_GLU_SWIGLU)
        hipLaunchKernelGGL((glu_kernel<T, NVQ_GLU_SWIGLU>), grid, block, 0, s, (const T *)gate, (const T *)up, (const T *)gate_bias,
                           (const T *)up_bias, ids, (T *)out, d.rows, d.hidden, d.gate_stride, d.up_stride, d.experts, alpha, limit);
    else if (d.activation == NVQ_GLU_SWIGLU_OAI)
        hipLaunchKernelGGL((glu_kernel<T, NVQ_GLU_SWIGLU_OAI>), grid, block, 0, s, (const T *)gate, (const T *)up, (const T *)gate_bias,
                           (const T *)up_bias, ids, (T *)out, d.rows, d.hidden, d.gate_stride, d.up_stride, d.experts, alpha, limit);
    else
        hipLaunchKernelGGL((glu_kernel<T, NVQ_GLU_GEGLU>), grid, block, 0, s, (const T *)gate, (const T *)up, (const T *)gate_bias,
                           (const T *)up_bias, ids, (T *)out, d.rows, d.hidden, d.gate_stride, d.up_stride, d.experts, alpha, limit);
    NVQ_LAUNCH_CHECK("glu");
    return NVQ_OK;
}

}  // namespace

int32_t launch_glu(const nvq_glu_desc &d, const void *gate, const void *up, const void *gate_bias, const void *up_bias,
                   const int32_t *ids, void *out, hipStream_t s) {
    switch (d.dtype) {
    case NVQ_F32: return run_glu<float>(d, gate, up, gate_bias, up_bias, ids, out, s);
    case NVQ_BF16: return run_glu<bf16_t>(d, gate, up, gate_bias, up_bias, ids, out, s);
    default: return run_glu<f16_t>(d, gate, up, gate_bias, up_bias, ids, out, s);
    }
}

}  // namespace nvq
