/*
 * nuvec_hip.h — C ABI of the MI355X (gfx950) backend for nuvec's quantized-matmul path.
 *
 * This is the surface a `hip` arm of nuvec's device boundary binds: the counterpart of
 * `GpuEval::{supports, run}` for the five primitives of the path
 * (reference: crates/nuvec-core/src/gpu.rs:1571-1799; the stub with the same surface is
 * gpu.rs:154-281).  Every entry point cites the reference routine it replaces.
 *
 * Conventions (they mirror what the reference's boundary already does):
 *  - Plain C: pointers, sizes and small POD structs.  No exceptions or panics cross it;
 *    every call returns an `nvq_status` and `nvq_last_error()` holds the message of the
 *    calling thread's last failure (nuvec maps it to `Error::Backend`, error.rs:29-34).
 *  - Ownership: the caller allocates every operand, output and workspace with the exact
 *    byte size and owns them (gpu.rs:1696, 6256-6258).  These entry points allocate nothing
 *    and free nothing.
 *  - Pointers are device pointers of the device given to `nvq_init` (any memory the HIP
 *    runtime can read from a kernel).  Operands are row-contiguous in their last two
 *    dimensions; batch dimensions are described by element strides (gpu.rs:7042-7051).
 *  - Asynchrony: a call validates on the host, enqueues kernels on `stream` (a `hipStream_t`
 *    passed as `void*`; NULL is the default stream) and returns.  Completion is the caller's
 *    stream or event synchronisation (the reference's `run` likewise only encodes,
 *    gpu.rs:1-11).  Empty products never reach the backend (gpu.rs:1640,1665,1667); here they
 *    return NVQ_OK without launching.
 *  - Re-entrant: no mutable global state besides a once-initialised device record.
 *  - dtype codes are nuvec's fixture order (crates/nuvec-core/tests/common/fixture.rs:15-30).
 *  - Packed layout is MLX's: per row a little-endian bit stream, value i at bit i*bits,
 *    stored as uint32 (crates/nuvec-core/src/kernels.rs:749-756, 808-817).
 */
#ifndef NUVEC_HIP_H
#define NUVEC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NVQ_MAX_BATCH_DIMS 6

#if defined(__GNUC__)
#define NVQ_API __attribute__((visibility("default")))
#else
#define NVQ_API
#endif

typedef enum nvq_status {
    NVQ_OK = 0,
    NVQ_INVALID_ARGUMENT = 1, /* Error::InvalidArgument / shape / dtype mismatch (error.rs) */
    NVQ_UNSUPPORTED = 2,      /* `supports()` would be false: the caller falls back to its CPU path */
    NVQ_OUT_OF_MEMORY = 3,    /* Error::OutOfMemory */
    NVQ_BACKEND = 4,          /* Error::Backend: a HIP call failed */
    NVQ_NO_DEVICE = 5         /* Error::UnsupportedDevice */
} nvq_status;

typedef enum nvq_dtype {
    NVQ_U8 = 1, NVQ_U32 = 3, NVQ_I32 = 7, NVQ_F16 = 9, NVQ_BF16 = 10, NVQ_F32 = 11
} nvq_dtype;

/* QuantMode (crates/nuvec-core/src/quantized.rs:22-35). */
typedef enum nvq_mode { NVQ_AFFINE = 0, NVQ_MXFP4 = 1, NVQ_MXFP8 = 2, NVQ_NVFP4 = 3 } nvq_mode;

/* Quant (quantized.rs:93-101). */
typedef struct nvq_quant {
    int32_t mode;       /* nvq_mode */
    int32_t group_size; /* affine 32/64/128; mxfp4, mxfp8 32; nvfp4 16 */
    int32_t bits;       /* affine 1-6 or 8; mxfp4, nvfp4 4; mxfp8 8 */
} nvq_quant;

typedef struct nvq_device_info {
    int32_t device;
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t lds_bytes_per_block;
    int64_t global_memory_bytes;
    char arch[64]; /* e.g. "gfx950:sramecc+:xnack-" */
    char name[128];
} nvq_device_info;

/* Primitive::QuantizedMatmul operands (crates/nuvec-core/src/primitive.rs:466-494) as the
 * device routine receives them (gpu.rs:6934-7060):
 *   x       dtype  [batch..., m, k]
 *   w       u32    [batch..., n, k*bits/32]   (transpose)  or [batch..., k, n*bits/32]
 *   scales  dtype  [batch..., n, k/group]     (affine)     or u8 for the fp modes
 *   biases  dtype  like scales (affine), NULL for the fp modes
 *   y       dtype  [batch..., m, n], row-contiguous
 * `batch_shape` is the output's batch shape; each operand's batch strides are in elements
 * of that operand (0 = broadcast).  With a 2-D `w` and row-contiguous `x` the caller folds
 * all leading rows into `m` and passes batch_ndim = 0 (the reference's "flat" rule,
 * gpu.rs:6948-6950); `item_rows` then carries x's second-to-last dimension, which is what
 * routing between the few-row and the tiled kernels looks at (gpu.rs:6975-6981). */
typedef struct nvq_qmm_desc {
    nvq_quant quant;
    int32_t dtype;     /* NVQ_F16 / NVQ_BF16 / NVQ_F32: x, y and (affine) scales, biases */
    int32_t transpose; /* 1: y = x . dequantize(w)^T  (MLX's default) */
    int32_t row_exact; /* Primitive::QuantizedMatmul::row_exact (primitive.rs:491-493; lib.rs:159-193): a product of up to
                          8 rows per item gives each row the bits of its one-row product (itself computed with the flag
                          set): it runs on the vector kernels, whose per-row arithmetic does not depend on the rows
                          that share a pass, and an untransposed product splits K by the weight's shape alone
                          (gpu.rs:6956-6981) */
    int32_t rows;      /* Primitive::QuantizedMatmul::rows (primitive.rs:489-490): every row count takes the
                          matrix-vector kernels, rows independent as above (qqmm's products) */
    int64_t m, n, k;
    int64_t item_rows; /* 0 = m */
    int32_t batch_ndim;
    int64_t batch_shape[NVQ_MAX_BATCH_DIMS];
    int64_t x_strides[NVQ_MAX_BATCH_DIMS];
    int64_t w_strides[NVQ_MAX_BATCH_DIMS];
    int64_t s_strides[NVQ_MAX_BATCH_DIMS]; /* scales and biases share a shape and strides */
} nvq_qmm_desc;

/* FastOp::GatherQmm operands (crates/nuvec-core/src/quantized.rs:539-587, gpu.rs:7174-7294):
 *   x [x_batches, m, k]; w [experts, n, k*bits/32] (transpose); scales/biases [experts, n, k/group];
 *   lhs, rhs u32[pairs]; y [pairs, m, n] = x[lhs[i]] . dequantize(w[rhs[i]])^T.
 * `offsets` (i32[experts], from nvq_sorted_offsets) is given when the caller took the grouped
 * route: rhs sorted, lhs = arange, m == 1 (quantized.rs:646-651, 772-782). */
typedef struct nvq_gather_desc {
    nvq_quant quant;
    int32_t dtype;
    int32_t transpose;
    int32_t row_exact; /* crate::row_exact() at the gather (gpu.rs:7325-7340): every pair on the vector kernels, so that a
                          pair has the bits of its one-row product, sorted or not; the caller's grouped rule
                          (nvq_gather_grouped) then asks for 65 rows before it passes `offsets` */
    int32_t reserved;  /* 0 */
    int64_t m, n, k;
    int64_t pairs;
    int64_t x_batches;
    int64_t experts;
} nvq_gather_desc;

/* FastOp::QuantizedAttention (crates/nuvec-core/src/fast.rs:694-718; fit rule fast/imp.rs:3944-3992): one query row per
 * head over an affine-quantized key / value cache.
 *   q dtype [batch, query_heads, 1, head_dim];  k_w, v_w u32 [batch, key_heads, positions, head_dim*bits/32];
 *   k_s, k_b, v_s, v_b dtype [batch, key_heads, positions, head_dim/group_size];  sinks dtype [query_heads] or NULL;
 *   out dtype [batch, query_heads, 1, head_dim], all contiguous. */
typedef struct nvq_attention_desc {
    int32_t dtype;      /* NVQ_F16 / NVQ_BF16 / NVQ_F32: q, scales, biases, sinks, out */
    int32_t bits;       /* 3, 4 or 8 (3 bits: a row's chunks of 32 codes are 12 bytes, rows 4-byte aligned) */
    int32_t group_size; /* 32, 64 or 128, dividing head_dim */
    int32_t head_dim;   /* 64 or 128 */
    int64_t batch, query_heads, key_heads, positions;
    float scale;
} nvq_attention_desc;

/* ── runtime ─────────────────────────────────────────────────────────────────────── */

/* Binds the library to HIP device `device` (idempotent; the process-wide device record,
 * as `Device::shared()`, crates/nuvec-gpu/src/cuda/device.rs:79-82).  NVQ_NO_DEVICE when
 * there is no gfx950 device: `GpuEval::available` (gpu.rs:1571-1573) is then false. */
NVQ_API int32_t nvq_init(int32_t device);
NVQ_API int32_t nvq_get_device_info(nvq_device_info *info);
/* The calling thread's last error message ("" if none).  Valid until its next failing call. */
NVQ_API const char *nvq_last_error(void);
NVQ_API const char *nvq_version(void);

/* No counterpart in the reference: two calibration kernels for the measurement harness, so that a benchmark can state
 * what this machine gives a kernel that does nothing but read memory or nothing but issue matrix instructions.
 *   NVQ_CALIBRATE_READ: every byte of `buffer` (`bytes`, a multiple of 16384) is read once with non-temporal 16-byte
 *     loads, 32 bytes per thread in blocks of 512 threads (bytes = N * K / 2 gives the decode kernel's grid);
 *   NVQ_CALIBRATE_MFMA: two wavefronts per SIMD issue `iters` rounds of eight independent v_mfma_f32_32x32x16_bf16.
 * `*work` (host, may be NULL) receives the bytes read or the floating-point operations of the launch; `sink` (device,
 * may be NULL) exists so that the compiler keeps the work. */
#define NVQ_CALIBRATE_READ 0
#define NVQ_CALIBRATE_MFMA 1
NVQ_API int32_t nvq_calibrate(int32_t kind, const void *buffer, int64_t bytes, int32_t iters, void *sink, int64_t *work,
                      void *stream);

/* ── validation mirrors (usable without a device) ────────────────────────────────── */

/* Quant::checked (quantized.rs:133-168): NVQ_OK or NVQ_INVALID_ARGUMENT with the
 * reference's message, prefixed by `op`. */
NVQ_API int32_t nvq_quant_check(const nvq_quant *quant, const char *op);

/* GatherQmm::groups / grouped (quantized.rs:724-735): 1 if a sorted gather of `rows` index
 * rows over `experts` weight batches takes the grouped kernel. */
NVQ_API int32_t nvq_gather_grouped(int64_t rows, int64_t experts, int32_t row_exact);

/* GpuEval::supports for Primitive::QuantizedMatmul (gpu.rs:1665): 1 if nvq_quantized_matmul
 * has a kernel for `desc`, else 0 (the caller then runs its CPU path, eval.rs:738-748). */
NVQ_API int32_t nvq_quantized_matmul_supported(const nvq_qmm_desc *desc);

/* ── the path ────────────────────────────────────────────────────────────────────── */

/* GpuEval::quantize / fp_quantize (gpu.rs:6247-6275, 6302-6324); arithmetic of
 * kernels::quantize / fp_quantize (kernels.rs:774-831, 914-971), bit for bit.
 *   w       dtype [rows, cols] row-contiguous (leading dims folded into rows), cols % group == 0
 *   packed  u32   [rows, cols*bits/32]
 *   scales  dtype [rows, cols/group] (affine) or u8 (fp modes)
 *   biases  dtype [rows, cols/group] (affine), NULL for the fp modes */
NVQ_API int32_t nvq_quantize(const nvq_quant *quant, int32_t dtype, const void *w, int64_t rows, int64_t cols,
                     void *packed, void *scales, void *biases, void *stream);

/* GpuEval::dequantize / fp_dequantize (gpu.rs:6905-6930, 6879-6902) with the CPU's
 * arithmetic (kernels.rs:835-859: two roundings in the scales' dtype; 976-1009), bit for bit.
 *   affine: `dtype` is the dtype of scales, biases and out.
 *   fp modes: `dtype` is the output dtype (f16, bf16 or f32); scales are u8, biases NULL.
 *   out dtype [rows, cols]. */
NVQ_API int32_t nvq_dequantize(const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales,
                       const void *biases, int64_t rows, int64_t cols, void *out, void *stream);

/* The rows of a quantized table dequantized: output row r is table row ids[r], bit for bit
 * nvq_dequantize of the taken rows (QuantizedEmbedding::forward, crates/nuvec-nn/src/layers.rs:245-255:
 * `take` of weight, scales and biases along axis 0, then `dequantize`).  Fused so that the taken packed
 * rows are never materialised.
 *   packed u32 [table_rows, cols*bits/32]; scales / biases [table_rows, cols/group]; ids u32 [count]
 *   (an id beyond the table is the caller's error and is clamped); out dtype [count, cols]. */
NVQ_API int32_t nvq_dequantize_rows(const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales,
                            const void *biases, int64_t table_rows, int64_t cols, const uint32_t *ids, int64_t count,
                            void *out, void *stream);

/* Bytes of scratch nvq_quantized_matmul needs for `desc` (split-K partials; the reference
 * allocates them on its side of the boundary, gpu.rs:7562).  0 = none; nonzero for products whose K is
 * split over the grid (float32 partial sums): transpose = 0, and transpose = 1 products of many rows with few
 * output tiles and a long K (the counterpart of the reference's qmm_t_splitk, gpu.rs:7507-7590).  A transposed
 * product given no workspace runs unsplit. */
/* The kernel a product of this descriptor runs on with operands aligned as hipMalloc aligns them ("qmm_kernel",
 * "qmf_kernel", "qmd_kernel", "qmv4_lds_kernel", ...), from the same routing code as the launch; NULL with
 * nvq_last_error for a descriptor the launch would refuse.  The reference names its kernels by route as well
 * (gpu.rs:7022, "nuvec_affine_qmv_mma_..."; its tests check the names, crates/nuvec-core/tests/quantized.rs:843-861).
 * Needs nvq_init. */
NVQ_API const char *nvq_quantized_matmul_route(const nvq_qmm_desc *desc);
NVQ_API size_t nvq_quantized_matmul_workspace_bytes(const nvq_qmm_desc *desc);

/* GpuEval::quantized_matmul / fp_quantized_matmul (gpu.rs:6934-7168, 6336-6577); values of
 * kernels::quantized_matmul (kernels.rs:1091-1142) within the stated tolerance.
 * `workspace` may be NULL when nvq_quantized_matmul_workspace_bytes(desc) == 0 (and for transposed products). */
NVQ_API int32_t nvq_quantized_matmul(const nvq_qmm_desc *desc, const void *x, const void *w, const void *scales,
                             const void *biases, void *y, void *workspace, void *stream);

/* QuantizedLinear::forward (crates/nuvec-nn/src/layers.rs:155-162): `x . dequantize(w)^T + bias` in one launch.  The
 * reference records the product and a separate addition; here the product kernels' epilogues add `bias` (element type
 * `desc->dtype`, one value per column of y, [n]) to the product already rounded to the element type and round again, so
 * the result has the bits of the two operations.  `bias` NULL: nvq_quantized_matmul.  A bias of another element type is
 * the caller's promotion (it then adds separately, as the reference does). */
NVQ_API int32_t nvq_quantized_linear(const nvq_qmm_desc *desc, const void *x, const void *w, const void *scales,
                             const void *biases, const void *bias, void *y, void *workspace, void *stream);

/* No counterpart in the reference: nvq_quantized_matmul for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc) and so cannot bring the workspace.  Same operands,
 * same routing and bit for bit the same results as nvq_quantized_matmul given the workspace its size query names; the
 * partial sums of a split K go to a scratch array inside the library (NVQ_STATIC_SCRATCH_BYTES of device memory, held
 * by every device the library is loaded on until the process ends).  A product whose partial sums need more is refused
 * with NVQ_UNSUPPORTED.  The call allocates and frees nothing.  All calls on a device share the one array (nothing in
 * it needs clearing: every partial sum a call reads it has written first), so calls that overlap in time on one device,
 * from several streams or threads, race: serialise them, or use nvq_quantized_matmul with a workspace per stream. */
#define NVQ_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)
NVQ_API int32_t nvq_quantized_matmul_static(const nvq_qmm_desc *desc, const void *x, const void *w, const void *scales,
                                    const void *biases, void *y, void *stream);

/* GpuEval::quantized_attention (gpu.rs:4969-5040): softmax(scale * q . K^T [, sinks]) . V in one kernel, the codes
 * dequantized in registers (never rounded), float32 products and sums; within the float bound of the dequantized
 * attention, as the reference's kernel.  Caches of 3, 4 and 8 bits are taken.  What the fit rule excludes (several query
 * rows, a mask, other head sizes or widths, query heads that are not 1, 2, 4 or 8 per key head, more than 65535 batches or
 * 2^31 cache values) answers NVQ_UNSUPPORTED: the caller then records the
 * composition of two quantized products and a softmax, as the reference does (fast/imp.rs:3996-4035).
 * With the workspace the size query names (float32 states of the splits: maximum, denominator and weighted sum per
 * split and head) the positions are split over the grid and a second kernel merges the splits; with NULL one block
 * walks all positions of a head. */
NVQ_API size_t nvq_quantized_attention_workspace_bytes(const nvq_attention_desc *desc);
NVQ_API int32_t nvq_quantized_attention(const nvq_attention_desc *desc, const void *q, const void *k_w, const void *k_s,
                                const void *k_b, const void *v_w, const void *v_s, const void *v_b, const void *sinks,
                                void *out, void *workspace, void *stream);

/* GpuEval::sorted_offsets (gpu.rs:6732-6756); kernels::sorted_offsets (kernels.rs:873-892):
 * per row of `indices` u32[rows, m], offsets[row, g] = first position whose value is >= g. */
NVQ_API int32_t nvq_sorted_offsets(const uint32_t *indices, int64_t rows, int64_t m, int32_t groups,
                           int32_t *offsets, void *stream);

/* One layer of a Hugging Face AWQ / GPTQ checkpoint as nuvec's affine layout, as the loader converts it
 * (crates/nuvec-lm/src/quant.rs:35-196, crates/nuvec-lm/src/config.rs:30-48).
 *   qweight i32/u32 [rows, cols]: AWQ [in, out / 8] (4 bits, AWQ's nibble order), GPTQ [in * bits / 32, out];
 *   qzeros likewise along the outputs, [groups, ceil(out * bits / 32)], or NULL (zero = 2^(bits - 1));
 *   scales dtype [groups, out].
 * Outputs: weight u32 [out, in * bits / 32]; scales_out, biases_out dtype [out, groups] with
 * bias = -(zero) * scale (GPTQ v1 stores each zero minus one).  A `g_idx` must be the identity grouping: the
 * caller checks it, as the reference does (quant.rs:104-118). */
#define NVQ_PACKED_AWQ 0
#define NVQ_PACKED_GPTQ_V1 1
#define NVQ_PACKED_GPTQ_V2 2
NVQ_API int32_t nvq_convert_packed(int32_t format, const nvq_quant *quant, int32_t dtype, const uint32_t *qweight,
                           const uint32_t *qzeros, const void *scales, int64_t rows, int64_t cols, uint32_t *weight,
                           void *scales_out, void *biases_out, void *stream);

/* The pairs of a mixture-of-experts layer ordered by expert: what SwitchGlu::forward computes with `argsort`
 * of the flattened expert ids, `argsort` of that (the inverse) and `sorted_offsets`
 * (crates/nuvec-lm/src/model.rs:2193-2210), as one stable counting sort.
 *   ids u32[pairs] (an id beyond `experts` is the caller's error and is clamped);
 *   order u32[pairs]: the pair at each sorted position, ties in pair order;  restore u32[pairs]: its inverse;
 *   sorted_ids u32[pairs] = ids[order];  offsets i32[experts]: where each expert's pairs start. */
NVQ_API int32_t nvq_moe_order(const uint32_t *ids, int64_t pairs, int32_t experts, uint32_t *order, uint32_t *restore,
                      uint32_t *sorted_ids, int32_t *offsets, void *workspace, void *stream);
/* Bytes of `workspace` (per-chunk counters) with which the ordering of many pairs runs over the whole chip in three
 * launches; 0 for few pairs, and with a NULL workspace one block orders them all. */
NVQ_API size_t nvq_moe_order_workspace_bytes(int64_t pairs, int32_t experts);

/* NVFP4 with a global scale (MLX's `quantize(..., global_scale=)`; ops.rs `quantize_scaled`, quantized.rs:972-1005,
 * kernels.rs:914-1009 with `g`; validated as primitive.rs:1378-1395: NVFP4 only): `global_scale` points at one
 * float32 value on the device; the group scales are relative to it, g / (448 * 6).  No biases in this mode. */
NVQ_API int32_t nvq_quantize_scaled(const nvq_quant *quant, int32_t dtype, const void *w, int64_t rows, int64_t cols,
                            const float *global_scale, void *packed, void *scales, void *stream);
NVQ_API int32_t nvq_dequantize_scaled(const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales,
                              const float *global_scale, int64_t rows, int64_t cols, void *out, void *stream);
/* quantized.rs:469-491: x [M, K] times transposed w [N, K'] (no batch); any other shape the reference itself
 * dequantizes and multiplies densely (NVQ_UNSUPPORTED here). */
NVQ_API int32_t nvq_quantized_matmul_scaled(const nvq_qmm_desc *desc, const void *x, const void *w, const void *scales,
                                    const float *global_scale, void *y, void *workspace, void *stream);
/* quantized.rs:620-636, 677-719: one global scale per expert, float32 [experts]. */
NVQ_API int32_t nvq_gather_qmm_scaled(const nvq_gather_desc *desc, const void *x, const void *w, const void *scales,
                              const float *global_scales, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                              void *y, void *workspace, void *stream);
/* The gathered product with its result rows put where the caller wants them: pair z (sorted position z of a grouped
 * product) writes block out_rows[z] of y [pairs, M, N] (u32[pairs], a permutation; an index beyond `pairs` is the
 * caller's error and is clamped).  With out_rows = the `order` of nvq_moe_order the ordered down projection of
 * SwitchGlu::forward lands in pair order and the inverse permutation `take(out, inverse)` of
 * crates/nuvec-lm/src/model.rs:2205-2210 is never run.  `biases` / `global_scales` as the mode needs them (either
 * may be NULL).  Weights stored [N, K] only (transpose = 1); else NVQ_UNSUPPORTED. */
NVQ_API int32_t nvq_gather_qmm_scatter(const nvq_gather_desc *desc, const void *x, const void *w, const void *scales,
                               const void *biases, const float *global_scales, const uint32_t *lhs, const uint32_t *rhs,
                               const int32_t *offsets, const uint32_t *out_rows, void *y, void *workspace, void *stream);

/* FastOp::QuantizeDequantize (crates/nuvec-core/src/products.rs:307-315, kernels.rs:1011-1065; MLX's
 * fp_quantize_dequantize): x through its quantization in a floating-point mode, i.e. the values the codes represent,
 * in x's dtype: the activations of `qqmm` / `gather_qqmm` (products.rs:333-470), which then take
 * nvq_quantized_matmul(_scaled) / nvq_gather_qmm(_scaled).  `global_scale`: NULL, or NVFP4's one float32 value. */
NVQ_API int32_t nvq_quantize_dequantize(const nvq_quant *quant, int32_t dtype, const void *x, int64_t rows, int64_t cols,
                                const float *global_scale, void *out, void *stream);

/* fast::moe_route (crates/nuvec-core/src/fast.rs:740-746, fast/imp.rs:2652-2673; kernel
 * crates/nuvec-kernels/src/metal/moe.metal:33-88): per row of `experts` router probabilities the k largest in the
 * stable ascending order of the sort (NaN last for float32 and half), i.e. the last k of `argsort`, their values
 * and, with `normalize`, those divided by their sum (summed in `dtype`, in order).
 *   probs dtype[rows, experts] (contiguous);  indices u32[rows, k];  scores dtype[rows, k].
 * Up to 1024 experts and, with `normalize`, k <= 64 (beyond, the reference composes argpartition / take / sum /
 * divide itself: NVQ_UNSUPPORTED). */
NVQ_API int32_t nvq_moe_route(int32_t dtype, const void *probs, int64_t rows, int32_t experts, int32_t k, int32_t normalize,
                      uint32_t *indices, void *scores, void *stream);

/* fast::weighted_sum (fast/imp.rs:2731-2747; kernel moe.metal:90-118): out[r, c] = sum_j x[r, j, c] * w[r, j], the
 * experts' outputs weighted by the router's scores, every product and addition rounded to `dtype` in the kernel's
 * order (min(k, 8) interleaved partial sums, added in order).
 *   x dtype[rows, k, d];  w dtype[rows, k];  out dtype[rows, d];  1 <= k < 32 (beyond: NVQ_UNSUPPORTED). */
NVQ_API int32_t nvq_weighted_sum(int32_t dtype, const void *x, const void *w, int64_t rows, int32_t k, int64_t d, void *out,
                         void *stream);

/* The experts' gated activation between their gate / up products and their down product (`SwitchGlu::through`,
 * crates/nuvec-lm/src/model.rs:2157-2170), with each row's expert's bias added to either product first
 * (`SwitchProjection::forward`, model.rs:2139-2143): out[r, c] = act(gate[r, c] + gate_bias[ids[r], c],
 * up[r, c] + up_bias[ids[r], c]), every operation rounded to `dtype` in the reference's order.
 *   NVQ_GLU_SWIGLU      gate * sigmoid(gate) * up                     (crates/nuvec-nn/src/lib.rs:343-345, 513-519)
 *   NVQ_GLU_SWIGLU_OAI  (clip(up, -limit, limit) + 1) * g * sigmoid(alpha * g), g = min(gate, limit)   (lib.rs:564-570)
 *   NVQ_GLU_GEGLU       0.5 gate (1 + tanh(sqrt(2 / pi) (gate + 0.044715 gate^3))) * up: Gemma's, with the tanh
 *                       approximation of GELU as MLX's `gelu_approx`                                     (lib.rs:347-357, 581-590)
 *   gate, up dtype[rows, hidden] with `gate_stride` / `up_stride` elements between rows (so the two halves of one
 *   product [rows, 2 * hidden] of fused gate / up weights serve);  out dtype[rows, hidden];  gate_bias, up_bias
 *   dtype[experts, hidden], both or neither, with ids i32[rows] (an id outside is clamped). */
enum { NVQ_GLU_SWIGLU = 0, NVQ_GLU_SWIGLU_OAI = 1, NVQ_GLU_GEGLU = 2 };
typedef struct nvq_glu_desc {
    int32_t dtype;       /* NVQ_F32, NVQ_F16 or NVQ_BF16 */
    int32_t activation;  /* NVQ_GLU_* */
    float alpha, limit;  /* NVQ_GLU_SWIGLU_OAI (gpt-oss: 1.702 and 7) */
    int64_t rows, hidden;
    int64_t gate_stride, up_stride;
    int64_t experts;     /* rows of the biases; 0 without */
} nvq_glu_desc;
NVQ_API int32_t nvq_glu(const nvq_glu_desc *desc, const void *gate, const void *up, const void *gate_bias, const void *up_bias,
                const int32_t *ids, void *out, void *stream);

/* nvq_gather_qmm_scatter with each row's expert's bias added in the kernel's epilogue (`SwitchProjection::forward`,
 * crates/nuvec-lm/src/model.rs:2139-2143: `y + bias[indices]`): y[z] = round(round(x[lhs[z]] . w[rhs[z]]^T) +
 * expert_bias[rhs[z]]), bit for bit the product followed by the separate addition, on the grouped route and on the
 * routes of one product per pair alike.  expert_bias dtype[experts, n] or NULL; out_rows and global_scales may be
 * NULL.  Weights stored [N, K] only (transpose = 1); else NVQ_UNSUPPORTED (the caller then adds the bias after
 * nvq_gather_qmm). */
NVQ_API int32_t nvq_gather_qmm_expert_bias(const nvq_gather_desc *desc, const void *x, const void *w, const void *scales,
                                   const void *biases, const float *global_scales, const uint32_t *lhs, const uint32_t *rhs,
                                   const int32_t *offsets, const uint32_t *out_rows, const void *expert_bias, void *y,
                                   void *workspace, void *stream);

/* `Mlp::forward` up to its down projection (crates/nuvec-lm/src/model.rs:2066-2074: `swiglu(gate(x), up(x))`, Gemma's
 * `geglu`) for up to four rows of x in one kernel: w, scales, biases (and bias, dtype[n] or NULL: the two
 * projections' biases, layers.rs:155-162) hold the gate and up projections in alternating runs of 64 rows as for
 * nvq_gather_qmm_glu, desc->n is their total, y dtype[m, n / 2] = act(x . gate^T + bias_gate, x . up^T + bias_up) with
 * the products rounded to `dtype` first: bit for bit nvq_quantized_linear on the decode kernel followed by nvq_glu.
 * NVQ_UNSUPPORTED beyond four rows, for float32, batches, untransposed weights and affine widths other than 4 bits
 * (the caller then composes the products and nvq_glu). */
NVQ_API int32_t nvq_quantized_matmul_glu(const nvq_qmm_desc *desc, int32_t activation, float alpha, float limit, const void *x,
                                 const void *w, const void *scales, const void *biases, const void *bias, void *y, void *stream);

/* The grouped gathered product of the experts' gate and up projections with the gated activation as its epilogue:
 * `SwitchGlu::through` up to its down projection (crates/nuvec-lm/src/model.rs:2157-2169) in one kernel.  w, scales,
 * biases and expert_bias hold both projections in alternating runs of 64 rows (rows 128 b .. 128 b + 63: rows
 * 64 b .. of the gate projection, rows 128 b + 64 .. 128 b + 127: the same rows of the up projection), desc->n is
 * their total (a multiple of 128), desc->m is 1, rows sorted by expert with `offsets` as for nvq_gather_qmm.
 *   y dtype[pairs, n / 2] = act(x[lhs] . gate^T + bias_gate[rhs], x[lhs] . up^T + bias_up[rhs]), the products rounded
 *   to `dtype` as nvq_gather_qmm returns them, then nvq_glu's arithmetic: bit for bit that composition.
 *   expert_bias dtype[experts, n] or NULL.  With offsets = NULL the pairs are unsorted (the experts of decoded tokens,
 *   up to four rows of x each: desc->m) and run on the decode kernel with the same epilogue: y dtype[pairs, m, n / 2].
 *   NVQ_UNSUPPORTED where the grouped matrix-core kernel (the decode kernel) does not take the product (the caller
 *   then composes nvq_gather_qmm and nvq_glu). */
NVQ_API int32_t nvq_gather_qmm_glu(const nvq_gather_desc *desc, int32_t activation, float alpha, float limit, const void *x,
                           const void *w, const void *scales, const void *biases, const uint32_t *lhs, const uint32_t *rhs,
                           const int32_t *offsets, const void *expert_bias, void *y, void *stream);

/* Bytes of float32 partial sums nvq_gather_qmm wants in `workspace`: with the weights stored [K, N] (transpose = 0) K is
 * split over the grid (the reference's split-K scratch, gpu.rs:7562); 0 for transposed weights. */
NVQ_API size_t nvq_gather_qmm_workspace_bytes(const nvq_gather_desc *desc);

/* GpuEval::gather_qmm / fp_gather_qmm (gpu.rs:7174-7294, 6758-6876); values of the gathered
 * products of quantized::gather_qmm_graph (quantized.rs:679-719), both weight orientations.
 * `offsets` NULL = one product per pair; non-NULL = grouped route (see nvq_gather_desc; transposed weights only). */
NVQ_API int32_t nvq_gather_qmm(const nvq_gather_desc *desc, const void *x, const void *w, const void *scales,
                       const void *biases, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                       void *y, void *workspace, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* NUVEC_HIP_H */
