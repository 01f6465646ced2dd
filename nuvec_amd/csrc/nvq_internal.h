// Internal declarations shared by the host entry points and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "nuvec_hip.h"
#include "nvq_splits.h"

namespace nvq {

// ── errors ──────────────────────────────────────────────────────────────────────────
// Records `status` and a printf-style message for the calling thread; returns `status`.
int32_t fail(int32_t status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define NVQ_HIP_TRY(expr)                                                                      \
    do {                                                                                       \
        hipError_t nvq_e_ = (expr);                                                            \
        if (nvq_e_ != hipSuccess)                                                              \
            return ::nvq::fail(nvq_e_ == hipErrorOutOfMemory ? NVQ_OUT_OF_MEMORY : NVQ_BACKEND, \
                               "%s: %s", #expr, hipGetErrorString(nvq_e_));                    \
    } while (0)

// Launch check: a bad configuration is reported by the launch itself.
#define NVQ_LAUNCH_CHECK(what)                                                                  \
    do {                                                                                        \
        hipError_t nvq_e_ = hipGetLastError();                                                  \
        if (nvq_e_ != hipSuccess)                                                               \
            return ::nvq::fail(NVQ_BACKEND, "%s launch: %s", what, hipGetErrorString(nvq_e_));   \
    } while (0)

int32_t require_device();          // NVQ_OK once nvq_init succeeded
int32_t compute_units();           // of the bound device
int32_t check_quant(const nvq_quant *q, const char *op);
inline bool float_dtype(int32_t d) { return d == NVQ_F16 || d == NVQ_BF16 || d == NVQ_F32; }
inline int dtype_size(int32_t d) { return d == NVQ_F32 ? 4 : (d == NVQ_U8 ? 1 : (d == NVQ_U32 || d == NVQ_I32 ? 4 : 2)); }
const char *dtype_name(int32_t d);
const char *mode_name(int32_t m);

// ── kernel launchers (each validates nothing: the entry points did) ─────────────────────
int32_t launch_affine_quantize(int32_t dtype, int group, int bits, const void *w, int64_t n_values,
                               void *packed, void *scales, void *biases, hipStream_t s);
// `ids` non-NULL: output row r is table row ids[r] (rows of `cols` values, ids clamped to `table_rows`).
int32_t launch_affine_dequantize(int32_t dtype, int group, int bits, const void *packed, const void *scales,
                                 const void *biases, int64_t n_values, void *out, const uint32_t *ids, int64_t cols,
                                 int64_t table_rows, hipStream_t s);
// `global_scale`: NULL, or NVFP4's one float32 value on the device
int32_t launch_fp_quantize(int32_t mode, int32_t dtype, const void *w, int64_t n_values, void *packed,
                           void *scales, const float *global_scale, hipStream_t s);
int32_t launch_fp_quantize_dequantize(int32_t mode, int32_t dtype, const void *w, int64_t n_values, void *out,
                                      const float *global_scale, hipStream_t s);
int32_t launch_fp_dequantize(int32_t mode, int32_t out_dtype, const void *packed, const void *scales,
                             int64_t n_values, void *out, const uint32_t *ids, int64_t cols, int64_t table_rows,
                             const float *global_scale, hipStream_t s);
int32_t launch_sorted_offsets(const uint32_t *indices, int64_t rows, int64_t m, int32_t groups,
                              int32_t *offsets, hipStream_t s);
// Hugging Face integer packings into the affine layout (repack.hip).  format 0: AWQ, 1: GPTQ v1, 2: GPTQ v2.
int32_t launch_convert_packed(int32_t format, int32_t bits, int32_t dtype, const uint32_t *qweight, const uint32_t *qzeros,
                              const void *scales, int64_t inputs, int64_t outputs, int64_t groups, uint32_t *packed,
                              void *scales_out, void *biases_out, hipStream_t s);
size_t moe_order_lds_bytes(int32_t experts);
int32_t launch_moe_route(int32_t dtype, const void *probs, int64_t rows, int32_t experts, int32_t k, int32_t normalize,
                         uint32_t *indices, void *scores, hipStream_t s);
int32_t launch_glu(const nvq_glu_desc &d, const void *gate, const void *up, const void *gate_bias, const void *up_bias,
                   const int32_t *ids, void *out, hipStream_t s);
int32_t launch_weighted_sum(int32_t dtype, const void *x, const void *w, int64_t rows, int32_t k, int64_t d, void *out, hipStream_t s);
size_t moe_order_workspace_bytes(int64_t pairs, int32_t experts);
int32_t launch_moe_order(const uint32_t *ids, int64_t pairs, int32_t experts, uint32_t *order, uint32_t *restore,
                         uint32_t *sorted_ids, int32_t *offsets, void *workspace, hipStream_t s);

// One transposed product per batch/pair.  `lhs`/`rhs` NULL = batch strides from `desc`.
struct ProductArgs {
    const void *x, *w, *scales, *biases;
    void *y;
    int32_t mode, group, bits, dtype;
    int64_t m, n, k;
    int64_t batch;                  // grid z
    int32_t batch_ndim;             // 0: single product
    int64_t batch_shape[NVQ_MAX_BATCH_DIMS];
    int64_t x_strides[NVQ_MAX_BATCH_DIMS], w_strides[NVQ_MAX_BATCH_DIMS], s_strides[NVQ_MAX_BATCH_DIMS];
    const uint32_t *lhs, *rhs;      // gather: batch z reads x batch lhs[z] and weight batch rhs[z]
    int64_t x_batches, experts;     // gather: index bounds (an index beyond them is clamped)
    const int32_t *offsets;         // grouped gather: rows of expert e are [offsets[e], offsets[e+1]) of `batch` rows
    int32_t k_splits, k_split_steps;  // tiled kernel: K split over grid z (0 or 1: no split), steps of 64 values per split
    float *partials;                // tiled kernel with a split: float32 [k_splits][m][n], summed by a second kernel
    const float *global_scale;      // NVFP4: NULL, one float32 value, or one per expert of a gather (weights stored [N, K] only)
    const uint32_t *out_rows;       // gather with the weights stored [N, K]: pair z writes block out_rows[z] of y (NULL: block z)
    const void *row_bias;           // NULL, or one value of the element type per column of y, added to the rounded product
                                    // (QuantizedLinear's bias)
    int32_t row_bias_per_expert;    // gathered pairs: `row_bias` is [experts, n] and pair z takes row rhs[z] (SwitchProjection's bias)
    int32_t row_exact;              // every row takes the arithmetic of its one-row product: the vector kernels only, K split
                                    // (weights stored [K, N]) by the weight's shape alone
    // Affine codes, 16-bit elements, rows of few outputs: the kernels materialise the weights with the CPU's two roundings
    // (round(round(code * scale) + bias), kernels.rs:835-859) instead of one; the routes keep such products off the
    // kernels that never materialise a weight.
    int32_t exact_weights;
    // Grouped gather with the gated activation as its epilogue (0: none, else 1 + NVQ_GLU_*): w holds the gate and up
    // projections in alternating runs of 64 rows, y is [batch, n / 2]; expert_bias (NULL or [experts, n], rows as w) is
    // added to the rounded products first.
    int32_t glu;
    float glu_alpha, glu_limit;
    const void *expert_bias;
};
int32_t launch_qmv(const ProductArgs &a, hipStream_t s);
const char *qmv_kernel_name(const ProductArgs &a);  // which of the vector / decode kernels launch_qmv runs for `a`
// Whether the 16x16x32 matrix-core decode kernel takes the product (4-bit affine, groups of 64, K = 4096).
bool qmv_d16_takes(const ProductArgs &a);
// The integer dot-product decode kernel: one row of x (or the rows of a row-exact product) against 4-bit affine weights.
bool qmv_dot8_takes(const ProductArgs &a);
int32_t launch_qmv_dot8(const ProductArgs &a, hipStream_t s);
int qmv_dot8_rows_per_wave(int64_t n, int cus);  // rows a wavefront takes, by the weight's rows and the chip's compute units
bool qmv_glu_pairs_take(const ProductArgs &a);      // whether the decode kernel takes unsorted pairs with the gated epilogue
int32_t launch_qmv_glu_pairs(const ProductArgs &a, hipStream_t s);
bool qmv_block_decode_takes(const ProductArgs &a);  // whether the decode kernel takes a product of a block format
bool qmv_decode_takes_width(const ProductArgs &a);  // whether the decode kernel takes these few rows of 3- or 8-bit affine codes
// The 16x16x32 matrix-core kernel for passes of up to 16 rows of x (affine 2, 3, 4 and 8 bits, every group size).
bool qmd_supported(const ProductArgs &a);
int32_t launch_qmd(const ProductArgs &a, hipStream_t s);
// The tiled matrix-core kernel (many rows of x); `qmm_supported` says whether it takes `a`.
bool qmm_supported(const ProductArgs &a);
size_t qmm_workspace_bytes(const ProductArgs &a);  // float32 partial sums when K is split over the grid, else 0
int32_t launch_qmm(const ProductArgs &a, void *workspace, hipStream_t s);  // workspace NULL: no split
double qmm_estimate_us(const ProductArgs &a);  // estimated duration of the tiled kernel with its better tile
// float32 products of many rows on v_mfma_f32_32x32x2_f32 (affine codes, weights stored [N, K]).
bool qmm_f32_takes(const ProductArgs &a);
int32_t launch_qmm_f32(const ProductArgs &a, hipStream_t s);
// Batched decode: passes of up to 64 rows of x (5 to 128 rows routed there, where it measured faster), every weight fetched and dequantized once per pass (4- and 8-bit affine codes).
bool qmr_supported(const ProductArgs &a);
int32_t launch_qmr(const ProductArgs &a, hipStream_t s);
// The few-row matrix-core kernel (up to 32 rows of x per pass; also the grouped gathered product).
bool qmf_supported(const ProductArgs &a);
int32_t launch_qmf(const ProductArgs &a, hipStream_t s);
int32_t launch_fill_zero(void *p, int64_t bytes, hipStream_t s);
int32_t launch_quantized_attention(const nvq_attention_desc &d, const void *q, const void *kw, const void *ks, const void *kb,
                                   const void *vw, const void *vs, const void *vb, const void *sinks, void *out, void *workspace,
                                   hipStream_t s);
size_t attention_workspace_bytes(const nvq_attention_desc &d);  // float32 states of the splits of the positions, or 0
int32_t launch_calibrate(int32_t kind, const void *buffer, int64_t bytes, int32_t iters, void *sink, int64_t *work, hipStream_t s);
// Products with the weights stored [K, N] (transpose = false); K is split over the grid through a float32 workspace.
int qvm_splits(const ProductArgs &a);
size_t qvm_workspace_bytes(const ProductArgs &a);
int32_t launch_qvm(const ProductArgs &a, void *workspace, hipStream_t s);
bool qvm_takes_grouped(const ProductArgs &a);  // whether sorted pairs of one row each run as groups on the matrix-core kernel
const char *qvm_kernel_name(const ProductArgs &a);  // the matrix-core kernel (many rows of x) or the vector kernel

}  // namespace nvq
