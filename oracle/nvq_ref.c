/*
 * nvq_ref — CPU restatement of nuvec's quantized-matmul path.
 *
 * TEST INFRASTRUCTURE.  This file is the parity oracle: tests, the smoke check
 * and the `cpu_baseline` leg of the benchmark load it as the checker (or as the
 * timed CPU baseline).  Nothing on the product path links, loads or calls it.
 *
 * Every function follows the reference's CPU implementation, cited per
 * function as path:line under the reference checkout:
 *
 *   crates/nuvec-core/src/kernels.rs   746-859   affine code/quantize/dequantize
 *                                      873-892   sorted_offsets
 *                                      906-1009  fp_quantize / fp_dequantize
 *                                      1087-1142 quantized_matmul
 *   crates/nuvec-core/src/fp8.rs       11-129    E4M3 / E2M1 / E8M0 codecs, ftz
 *   crates/nuvec-core/src/cast.rs      49-98     rounding paths of f16 / bf16
 *   crates/nuvec-cpu/src/few_rows.rs   57-224    fixed-order products (M <= 16)
 *   crates/nuvec-cpu/src/matmul.rs     101-251   product dispatch
 *   crates/nuvec-core/src/quantized.rs 679-719   gather_qmm as gathered products
 *
 * Parity status per function (what pins it is listed in tests/test_oracle_*.py):
 *   affine quantize, code packing, affine dequantize (both roundings), MXFP4/
 *   MXFP8/NVFP4 codecs, fp_quantize, fp_dequantize, sorted_offsets: pinned
 *   bit-exactly by the reference's recorded golden vectors and known answers.
 *   products with M <= 16 (few_rows order): restated from source; no reference
 *   vector holds their exact bits, so they are pinned by the recorded MLX
 *   outputs within the reference's own bounds, by the few_rows invariants and
 *   by an exact rational/f64 dot product — *bit-level parity unpinned*.
 *   products with M > 16: the reference calls the un-vendored `gemm` 0.19 crate
 *   (Cargo.lock:720-722); its accumulation order is not restated.  The oracle
 *   accumulates the f32 products in f64 and rounds once — *parity unpinned at
 *   the bit level*, tolerance only.
 *   NaN payload bits of half/bf16 conversions (`half` 2.7.1): unpinned.
 *
 * Build: gcc -O3 -march=x86-64-v3 -ffp-contract=off -fopenmp -shared -fPIC
 * (contraction off: a fused multiply-add appears only where the reference
 * writes `mul_add`, as an explicit fmaf).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define NVQ_EXPORT __attribute__((visibility("default")))

enum { NVQ_F16 = 9, NVQ_BF16 = 10, NVQ_F32 = 11 };               /* fixture.rs:15-30 */
enum { NVQ_AFFINE = 0, NVQ_MXFP4 = 1, NVQ_MXFP8 = 2, NVQ_NVFP4 = 3 }; /* quantized.rs:22-35 */

/* ── scalar conversions (cast.rs:49-98 and the `half` crate they call) ───────────── */

static inline uint32_t f32_bits(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float bits_f32(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* `bf16::from_f32`: round to nearest even; a NaN keeps its high bits and is quieted. */
static inline uint16_t f32_to_bf16(float x) {
    uint32_t u = f32_bits(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t round_bit = 0x8000u;
    if ((u & round_bit) && (u & (3 * round_bit - 1))) return (uint16_t)((u >> 16) + 1);
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    if (exp == 0x1F) return bits_f32(sign | 0x7F800000u | (man << 13));
    if (exp == 0) {
        float v = (float)man * 0x1p-24f; /* subnormal or zero: exact */
        return bits_f32(f32_bits(v) | sign);
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* `f16::from_f64`, correctly rounded to nearest even (the reference's hosts convert in
 * hardware; cast.rs:67-83 goes f64 -> f16 directly, without a float32 step). */
static inline uint16_t f64_to_f16(double x) {
    uint64_t u; memcpy(&u, &x, 8);
    uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    double a = fabs(x);
    if (a != a) return (uint16_t)(sign | 0x7E00u);
    if (a >= 65520.0) return (uint16_t)(sign | 0x7C00u);
    if (a < 0x1p-14) { /* subnormal range: units of 2^-24 (rint: ties to even) */
        return (uint16_t)(sign | (uint16_t)rint(a * 0x1p24));
    }
    int e;
    (void)frexp(a, &e);            /* a = m * 2^e, m in [0.5, 1) */
    int exp = e - 1;               /* a in [2^exp, 2^(exp+1)) */
    double q = rint(ldexp(a, 10 - exp)); /* in [1024, 2048] */
    if (q >= 2048.0) { q = 1024.0; exp += 1; }
    if (exp > 15) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | (uint16_t)((exp + 15) << 10) | ((uint16_t)q - 1024u));
}

/* `round_to::<T>(f64)` (kernels.rs:766-769): f16 directly, bf16 through float32, f32 `as`. */
static inline void store_rounded(void *out, int64_t i, int dtype, double v) {
    switch (dtype) {
    case NVQ_F16: ((uint16_t *)out)[i] = f64_to_f16(v); break;
    case NVQ_BF16: ((uint16_t *)out)[i] = f32_to_bf16((float)v); break;
    default: ((float *)out)[i] = (float)v; break;
    }
}

static inline float load_f32(const void *p, int64_t i, int dtype) {
    switch (dtype) {
    case NVQ_F16: return f16_to_f32(((const uint16_t *)p)[i]);
    case NVQ_BF16: return bf16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}

static inline int dtype_size(int dtype) { return dtype == NVQ_F32 ? 4 : 2; }
static inline int dtype_ok(int dtype) { return dtype == NVQ_F16 || dtype == NVQ_BF16 || dtype == NVQ_F32; }

/* Rust's `f32::min` / `f32::max`: the other operand when one is NaN.  For zeros of either
 * sign the reference's hosts (aarch64 fminnm/fmaxnm) order -0 below +0. */
static inline float rs_min(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    if (a == 0.0f && b == 0.0f) return signbit(a) ? a : b;
    return a < b ? a : b;
}
static inline float rs_max(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    if (a == 0.0f && b == 0.0f) return signbit(a) ? b : a;
    return a > b ? a : b;
}

/* Rust's saturating `f32 as u32` after `clamp(0, n_bins)` (NaN stays NaN and casts to 0). */
static inline uint32_t clamp_code(float q, float n_bins) {
    if (q != q) return 0;
    if (q < 0.0f) q = 0.0f;
    if (q > n_bins) q = n_bins;
    return (uint32_t)q;
}

/* ── affine (kernels.rs:746-859) ─────────────────────────────────────────────────── */

/* kernels.rs:749-756: code `i` of a little-endian stream of `bits`-bit values. */
NVQ_EXPORT uint32_t nvq_ref_code(const uint8_t *bytes, int64_t i, int bits) {
    int64_t byte = i * bits / 8;
    int shift = (int)(i * bits % 8);
    uint32_t v = (uint32_t)bytes[byte] >> shift;
    if (shift + bits > 8) v |= (uint32_t)bytes[byte + 1] << (8 - shift);
    return v & ((1u << bits) - 1u);
}

static int affine_ok(int group, int bits) { /* quantized.rs:136-148 */
    return (group == 32 || group == 64 || group == 128) && ((bits >= 1 && bits <= 6) || bits == 8);
}

/* kernels.rs:774-831.  `n` values (a multiple of `group`), any leading shape flattened:
 * the bit stream runs over the whole flattened array.  Outputs: packed u32[n*bits/32],
 * scales and biases `dtype`[n/group]. */
NVQ_EXPORT int nvq_ref_affine_quantize(const void *w, int dtype, int64_t n, int group, int bits,
                                       uint32_t *packed, void *scales, void *biases) {
    if (!dtype_ok(dtype) || !affine_ok(group, bits) || n % group) return 1;
    uint8_t *bytes = (uint8_t *)packed;
    memset(bytes, 0, (size_t)(n * bits / 32) * 4);
    const float n_bins = (float)((1u << bits) - 1u);
    const float eps = 1e-7f;
    for (int64_t g = 0; g < n / group; g++) {
        float lo = INFINITY, hi = -INFINITY;
        for (int j = 0; j < group; j++) {
            float v = load_f32(w, g * group + j, dtype);
            lo = rs_min(lo, v);
            hi = rs_max(hi, v);
        }
        float scale, bias;
        if (bits == 1) {
            scale = rs_max(hi - lo, eps);
            bias = lo;
        } else {
            int wide = fabsf(lo) > fabsf(hi);
            scale = rs_max((hi - lo) / n_bins, eps);
            scale = wide ? scale : -scale;
            float edge = wide ? lo : hi;
            float q0 = rintf(edge / scale);
            if (q0 == 0.0f) {
                bias = 0.0f;
            } else {
                scale = edge / q0;
                bias = edge;
            }
        }
        for (int j = 0; j < group; j++) {
            float v = load_f32(w, g * group + j, dtype);
            uint32_t q = clamp_code(rintf((v - bias) / scale), n_bins);
            int64_t bit = (g * group + j) * bits;
            int64_t byte = bit / 8;
            int shift = (int)(bit % 8);
            uint32_t wide = q << shift;
            bytes[byte] |= (uint8_t)wide;
            if (shift + bits > 8) bytes[byte + 1] |= (uint8_t)(wide >> 8);
        }
        store_rounded(scales, g, dtype, (double)scale);
        store_rounded(biases, g, dtype, (double)bias);
    }
    return 0;
}

/* kernels.rs:835-859: `round(round(code*scale) + bias)`, each rounding to the scales' dtype.
 * `n` = number of values (packed holds n*bits/32 words). */
NVQ_EXPORT int nvq_ref_affine_dequantize(const uint32_t *packed, const void *scales, const void *biases,
                                         int dtype, int64_t n, int group, int bits, void *out) {
    if (!dtype_ok(dtype) || !affine_ok(group, bits) || n % group) return 1;
    const uint8_t *bytes = (const uint8_t *)packed;
    for (int64_t i = 0; i < n; i++) {
        int64_t g = i / group;
        double s = (double)load_f32(scales, g, dtype), b = (double)load_f32(biases, g, dtype);
        double c = (double)nvq_ref_code(bytes, i, bits);
        double product;
        switch (dtype) { /* the product rounded to T, read back */
        case NVQ_F16: product = (double)f16_to_f32(f64_to_f16(c * s)); break;
        case NVQ_BF16: product = (double)bf16_to_f32(f32_to_bf16((float)(c * s))); break;
        default: product = (double)(float)(c * s); break;
        }
        store_rounded(out, i, dtype, product + b);
    }
    return 0;
}

/* The device-side variant the reference's recorded GPU vectors hold (one rounding of
 * `fma(code, scale, bias)` in float32; crates/nuvec-kernels/src/metal/quantized.h:2701-2772).
 * Not what the CPU computes and not what the HIP backend ships: it exists so that the 54
 * recorded `affine-dequantize-*` device vectors pin the code extraction a second time. */
NVQ_EXPORT int nvq_ref_affine_dequantize_fma(const uint32_t *packed, const void *scales, const void *biases,
                                             int dtype, int64_t n, int group, int bits, void *out) {
    if (!dtype_ok(dtype) || !affine_ok(group, bits) || n % group) return 1;
    const uint8_t *bytes = (const uint8_t *)packed;
    for (int64_t i = 0; i < n; i++) {
        int64_t g = i / group;
        float s = load_f32(scales, g, dtype), b = load_f32(biases, g, dtype);
        float v = fmaf((float)nvq_ref_code(bytes, i, bits), s, b);
        store_rounded(out, i, dtype, (double)v);
    }
    return 0;
}

/* ── 8- and 4-bit float codecs (fp8.rs:11-129) ───────────────────────────────────── */

#define E4M3_MAX 448.0f
#define E2M1_MAX 6.0f

NVQ_EXPORT float nvq_ref_ftz(float x) { /* fp8.rs:103-112 */
    uint32_t u = f32_bits(x);
    if ((u & 0x7F800000u) == 0 && (u & 0x007FFFFFu) != 0) return bits_f32(u & 0x80000000u);
    return x;
}

NVQ_EXPORT float nvq_ref_canonical(float x) { /* fp8.rs:114-118 */
    return x != x ? bits_f32(0x7FC00000u) : x;
}

NVQ_EXPORT uint8_t nvq_ref_e4m3_from_f32(float x) { /* fp8.rs:16-37 */
    const uint32_t FP8_MAX = 543u << 21, DENORM_MASK = 141u << 23;
    uint32_t bits = f32_bits(x);
    uint32_t sign = bits & 0x80000000u;
    bits ^= sign;
    uint8_t code;
    if (bits >= FP8_MAX) {
        code = 0x7E;
    } else if (bits < (121u << 23)) {
        float sum = bits_f32(bits) + bits_f32(DENORM_MASK);
        code = (uint8_t)(f32_bits(sum) - DENORM_MASK);
    } else {
        uint32_t odd = (bits >> 20) & 1u;
        bits += ((uint32_t)(7 - 127) << 23) + 0x7FFFFu;
        bits += odd;
        code = (uint8_t)(bits >> 20);
    }
    return (uint8_t)(code | (uint8_t)(sign >> 24));
}

NVQ_EXPORT float nvq_ref_e4m3_to_f32(uint8_t code) { /* fp8.rs:39-45 */
    uint16_t v = code & 127u;
    uint16_t sign = (uint16_t)((code >> 7) << 15);
    uint16_t u = (uint16_t)((v << 7) | (((v + 1u) >> 7) << 14) | sign);
    /* f16::from_f32(f16(u) * 256): exact (a power-of-two scaling inside the half range). */
    return f16_to_f32(f64_to_f16((double)(f16_to_f32(u) * 256.0f)));
}

NVQ_EXPORT uint8_t nvq_ref_e2m1_from_f32(float x) { /* fp8.rs:47-73 */
    if (x != x) return 0x7;
    uint8_t sign = signbit(x) ? 0x8 : 0x0;
    float a = fabsf(x);
    uint8_t code = a > 5.0f ? 7 : a >= 3.5f ? 6 : a > 2.5f ? 5 : a >= 1.75f ? 4
                 : a > 1.25f ? 3 : a >= 0.75f ? 2 : a > 0.25f ? 1 : 0;
    return (uint8_t)(code | sign);
}

NVQ_EXPORT float nvq_ref_e2m1_to_f32(uint8_t code) { /* fp8.rs:75-80 */
    static const float VALUES[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float m = VALUES[code & 7];
    return (code & 8) ? -m : m;
}

NVQ_EXPORT uint8_t nvq_ref_e8m0_from_f32(float x) { /* fp8.rs:82-93 */
    if (!isfinite(x)) return 0xFF;
    if (x < 0.0f) return 0x00;
    float r = roundf(log2f(x)); /* halves away from zero; log2(0) = -inf saturates below */
    int n = r != r ? 0 : r <= -127.0f ? -127 : r >= 127.0f ? 127 : (int)r;
    return (uint8_t)(n + 127);
}

NVQ_EXPORT float nvq_ref_e8m0_to_f32(uint8_t code) { /* fp8.rs:95-102 */
    return code == 0 ? bits_f32(0x400000u) : bits_f32((uint32_t)code << 23);
}

NVQ_EXPORT float nvq_ref_mx_scale_round_up(float x) { /* fp8.rs:120-129 */
    uint8_t code = nvq_ref_e8m0_from_f32(x);
    if (code < 0xFE && nvq_ref_ftz(nvq_ref_e8m0_to_f32(code)) < x) code += 1;
    return nvq_ref_e8m0_to_f32(code);
}

static int fp_mode_ok(int mode, int *group, int *bits) { /* quantized.rs:48-56 */
    switch (mode) {
    case NVQ_MXFP4: *group = 32; *bits = 4; return 1;
    case NVQ_MXFP8: *group = 32; *bits = 8; return 1;
    case NVQ_NVFP4: *group = 16; *bits = 4; return 1;
    default: return 0;
    }
}

/* kernels.rs:914-971.  `g` NULL = no global scale; otherwise the NVFP4 global scale: group scales are
 * relative to g / (448 * 6).  Outputs: packed u32[n*bits/32], scales u8[n/group]. */
static int fp_quantize_impl(const void *w, int dtype, int64_t n, int mode, const float *g,
                            uint32_t *packed, uint8_t *scales) {
    int group, bits;
    if (!dtype_ok(dtype) || !fp_mode_ok(mode, &group, &bits) || n % group) return 1;
    uint8_t *bytes = (uint8_t *)packed;
    const int mx = group == 32;
    const float max_element = bits == 4 ? E2M1_MAX : E4M3_MAX;
    const float scale_enc = g ? nvq_ref_ftz(E4M3_MAX * E2M1_MAX / *g) : 1.0f;
    for (int64_t gi = 0; gi < n / group; gi++) {
        float amax = 0.0f;
        for (int j = 0; j < group; j++)
            amax = rs_max(amax, fabsf(nvq_ref_ftz(load_f32(w, gi * group + j, dtype))));
        float scale = nvq_ref_ftz(amax / max_element);
        if (g) scale = nvq_ref_ftz(scale * scale_enc);
        uint8_t code;
        float decoded;
        if (mx && !g) {
            code = nvq_ref_e8m0_from_f32(nvq_ref_mx_scale_round_up(scale));
            decoded = nvq_ref_e8m0_to_f32(code);
        } else {
            code = nvq_ref_e4m3_from_f32(scale);
            decoded = nvq_ref_e4m3_to_f32(code);
        }
        scales[gi] = code;
        decoded = nvq_ref_ftz(decoded);
        float inverse = decoded == 0.0f ? 0.0f : nvq_ref_ftz(scale_enc / decoded);
        for (int j = 0; j < group; j++) {
            int64_t i = gi * group + j;
            float v = nvq_ref_ftz(load_f32(w, i, dtype));
            float scaled = nvq_ref_canonical(nvq_ref_ftz(v * inverse));
            if (bits == 8) {
                bytes[i] = nvq_ref_e4m3_from_f32(scaled);
            } else {
                uint8_t nibble = nvq_ref_e2m1_from_f32(scaled);
                if (i % 2 == 0) bytes[i / 2] = nibble;
                else bytes[i / 2] |= (uint8_t)(nibble << 4);
            }
        }
    }
    return 0;
}
NVQ_EXPORT int nvq_ref_fp_quantize(const void *w, int dtype, int64_t n, int mode,
                                   uint32_t *packed, uint8_t *scales) {
    return fp_quantize_impl(w, dtype, n, mode, NULL, packed, scales);
}
NVQ_EXPORT int nvq_ref_fp_quantize_scaled(const void *w, int dtype, int64_t n, int mode, float g,
                                          uint32_t *packed, uint8_t *scales) {
    return fp_quantize_impl(w, dtype, n, mode, &g, packed, scales);
}

static inline float fp_value(const uint8_t *codes, const uint8_t *s, int64_t i, int group, int bits, const float *inv_enc) {
    /* kernels.rs:994-1005; `inv_enc` NULL = no global scale, else ftz(g / (448 * 6)) */
    uint8_t sc = s[i / group];
    float scale = nvq_ref_ftz(group == 32 ? nvq_ref_e8m0_to_f32(sc) : nvq_ref_e4m3_to_f32(sc));
    if (inv_enc) scale = nvq_ref_ftz(scale * *inv_enc);
    float value = bits == 8 ? nvq_ref_e4m3_to_f32(codes[i])
                            : nvq_ref_e2m1_to_f32((uint8_t)((codes[i / 2] >> (4 * (i % 2))) & 0xF));
    return nvq_ref_canonical(nvq_ref_ftz(scale * value));
}

/* kernels.rs:976-1009. */
static int fp_dequantize_impl(const uint32_t *packed, const uint8_t *scales, int64_t n, int mode,
                              int out_dtype, const float *g, void *out) {
    int group, bits;
    if (!dtype_ok(out_dtype) || !fp_mode_ok(mode, &group, &bits) || n % group) return 1;
    const uint8_t *codes = (const uint8_t *)packed;
    float inv = g ? nvq_ref_ftz(*g / (E4M3_MAX * E2M1_MAX)) : 0.0f;
    for (int64_t i = 0; i < n; i++)
        store_rounded(out, i, out_dtype, (double)fp_value(codes, scales, i, group, bits, g ? &inv : NULL));
    return 0;
}
NVQ_EXPORT int nvq_ref_fp_dequantize(const uint32_t *packed, const uint8_t *scales, int64_t n, int mode,
                                     int out_dtype, void *out) {
    return fp_dequantize_impl(packed, scales, n, mode, out_dtype, NULL, out);
}
NVQ_EXPORT int nvq_ref_fp_dequantize_scaled(const uint32_t *packed, const uint8_t *scales, int64_t n, int mode,
                                            int out_dtype, float g, void *out) {
    return fp_dequantize_impl(packed, scales, n, mode, out_dtype, &g, out);
}

/* kernels.rs:1011-1065 (MLX's fp_quantize_dequantize, qqmm's activations): per group the scale as the quantizer
 * encodes it, the values (scale / scale_enc) * float(code) in float32, one rounding to the input's dtype.
 * `g` NULL = no global scale. */
static int fp_quantize_dequantize_impl(const void *w, int dtype, int64_t n, int mode, const float *g, void *out) {
    int group, bits;
    if (!dtype_ok(dtype) || !fp_mode_ok(mode, &group, &bits) || n % group) return 1;
    const int mx = group == 32;
    const float max_element = bits == 4 ? E2M1_MAX : E4M3_MAX;
    const float scale_enc = g ? nvq_ref_ftz(E4M3_MAX * E2M1_MAX / *g) : 1.0f;
    for (int64_t gi = 0; gi < n / group; gi++) {
        float amax = 0.0f;
        for (int j = 0; j < group; j++)
            amax = rs_max(amax, fabsf(nvq_ref_ftz(load_f32(w, gi * group + j, dtype))));
        float scale = nvq_ref_ftz(amax / max_element);
        if (g) scale = nvq_ref_ftz(scale * scale_enc);
        float decoded = nvq_ref_ftz(mx && !g ? nvq_ref_e8m0_to_f32(nvq_ref_e8m0_from_f32(nvq_ref_mx_scale_round_up(scale)))
                                              : nvq_ref_e4m3_to_f32(nvq_ref_e4m3_from_f32(scale)));
        float enc_b = decoded == 0.0f ? 0.0f : nvq_ref_ftz(scale_enc / decoded);
        float dec = nvq_ref_ftz(decoded / scale_enc);
        for (int j = 0; j < group; j++) {
            int64_t i = gi * group + j;
            float scaled = nvq_ref_canonical(nvq_ref_ftz(nvq_ref_ftz(load_f32(w, i, dtype)) * enc_b));
            float value = bits == 8 ? nvq_ref_e4m3_to_f32(nvq_ref_e4m3_from_f32(scaled))
                                    : nvq_ref_e2m1_to_f32(nvq_ref_e2m1_from_f32(scaled));
            store_rounded(out, i, dtype, (double)nvq_ref_canonical(nvq_ref_ftz(dec * value)));
        }
    }
    return 0;
}
NVQ_EXPORT int nvq_ref_fp_quantize_dequantize(const void *w, int dtype, int64_t n, int mode, void *out) {
    return fp_quantize_dequantize_impl(w, dtype, n, mode, NULL, out);
}
NVQ_EXPORT int nvq_ref_fp_quantize_dequantize_scaled(const void *w, int dtype, int64_t n, int mode, float g, void *out) {
    return fp_quantize_dequantize_impl(w, dtype, n, mode, &g, out);
}

/* ── sorted offsets (kernels.rs:873-892) ─────────────────────────────────────────── */

NVQ_EXPORT int nvq_ref_sorted_offsets(const uint32_t *indices, int64_t rows, int64_t m, int32_t groups,
                                      int32_t *out) {
    for (int64_t r = 0; r < rows; r++) {
        const uint32_t *row = indices + r * m;
        for (int32_t g = 0; g < groups; g++) {
            /* partition_point(|i| i < g): binary search for the first index not below g */
            int64_t lo = 0, hi = m;
            while (lo < hi) {
                int64_t mid = lo + (hi - lo) / 2;
                if ((int64_t)row[mid] < (int64_t)g) lo = mid + 1; else hi = mid;
            }
            out[r * groups + g] = (int32_t)lo;
        }
    }
    return 0;
}

/* ── products (kernels.rs:1087-1142, few_rows.rs:57-224, matmul.rs:119-152) ───────── */

/* few_rows.rs:57-61,188-224: term p goes to partial p mod 8 by a fused multiply-add from +0,
 * in increasing p; the partials are combined by one fixed tree. */
static inline float dot_few_rows(const float *x, const float *w, int64_t ws, int64_t k) {
    float s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t full = k / 8 * 8;
    if (ws == 1) {
        for (int64_t q = 0; q < full; q += 8)
            for (int l = 0; l < 8; l++) s[l] = fmaf(x[q + l], w[q + l], s[l]);
        for (int64_t p = full; p < k; p++) s[p - full] = fmaf(x[p], w[p], s[p - full]);
    } else {
        for (int64_t p = 0; p < k; p++) s[p % 8] = fmaf(x[p], w[p * ws], s[p % 8]);
    }
    return ((s[0] + s[4]) + (s[2] + s[6])) + ((s[1] + s[5]) + (s[3] + s[7]));
}

/* More than 16 rows: the reference hands the product to the `gemm` crate, whose order is
 * not restated; f32 products accumulated in f64, rounded once (parity unpinned, see top). */
static inline float dot_many_rows(const float *x, const float *w, int64_t ws, int64_t k) {
    double acc = 0.0;
    for (int64_t p = 0; p < k; p++) acc += (double)(x[p] * w[p * ws]);
    return (float)acc;
}

NVQ_EXPORT float nvq_ref_dot_few_rows(const float *x, const float *w, int64_t w_stride, int64_t k) {
    return dot_few_rows(x, w, w_stride, k);
}

/* The dense matrix of one weight batch in float32, exactly as the product sees it:
 * affine = kernels.rs:835-859 in the scales' dtype then widened (kernels.rs:716-742,
 * matmul.rs:161-203); fp modes = kernels.rs:1105 (float32 directly). */
static int dense_f32(int mode, int group, int bits, int dtype, const uint32_t *w, const void *scales,
                     const void *biases, int64_t n_values, float *dense) {
    if (mode == NVQ_AFFINE) {
        if (dtype == NVQ_F32)
            return nvq_ref_affine_dequantize(w, scales, biases, dtype, n_values, group, bits, dense);
        uint16_t *tmp = (uint16_t *)malloc((size_t)n_values * 2);
        if (!tmp) return 2;
        int rc = nvq_ref_affine_dequantize(w, scales, biases, dtype, n_values, group, bits, tmp);
        for (int64_t i = 0; i < n_values && !rc; i++) dense[i] = load_f32(tmp, i, dtype);
        free(tmp);
        return rc;
    }
    return nvq_ref_fp_dequantize(w, (const uint8_t *)scales, n_values, mode, NVQ_F32, dense);
}

/* y[M,N] = x[M,K] . dense^T (transpose) or x . dense, rounded once to `dtype`
 * (kernels.rs:1112-1142).  `dense` is [N,K] if transpose else [K,N].  Columns in blocks of
 * 64 across threads (few_rows.rs:116-126); the bits do not depend on the threading. */
static void product_rows(int dtype, int transpose, int64_t M, int64_t N, int64_t K, const float *x32,
                         const float *dense, void *y, int threads) {
    const int64_t blocks = (N + 63) / 64;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (int64_t blk = 0; blk < blocks; blk++) {
        int64_t j1 = blk * 64 + 64 < N ? blk * 64 + 64 : N;
        for (int64_t j = blk * 64; j < j1; j++) {
            const float *col = transpose ? dense + j * K : dense + j;
            int64_t ws = transpose ? 1 : N;
            for (int64_t i = 0; i < M; i++) {
                float v = M <= 16 ? dot_few_rows(x32 + i * K, col, ws, K)
                                  : dot_many_rows(x32 + i * K, col, ws, K);
                store_rounded(y, i * N + j, dtype, (double)v);
            }
        }
    }
}

/* kernels.rs:1091-1142.  x is [batch, M, K] in `dtype`; w is [w_batch, N, K*bits/32]
 * (transpose) or [w_batch, K, N*bits/32]; `w_batch` is 1 (shared by every batch of x) or
 * `batch`.  scales/biases: `dtype` for affine, uint8 / NULL for the fp modes.  Each batch is
 * its own M-row product (kernels.rs:1145-1149 loops the batches).  K == 0 gives zeros
 * (matmul.rs:237-240). */
/* x[M,K] times an already dequantized float32 matrix (`dense` [N,K] if transpose else [K,N]), rounded once to
 * `dtype`: the product step of kernels.rs:1112-1142 on its own, for weights dequantized with a global scale. */
NVQ_EXPORT int nvq_ref_dense_matmul(int dtype, int transpose, int64_t M, int64_t N, int64_t K, const void *x,
                                    const float *dense, void *y, int threads) {
    if (!dtype_ok(dtype)) return 1;
    float *x32 = (float *)malloc((size_t)(M * K) * 4 + 4);
    if (!x32) return 2;
    for (int64_t i = 0; i < M * K; i++) x32[i] = load_f32(x, i, dtype);
    product_rows(dtype, transpose, M, N, K, x32, dense, y, threads < 1 ? 1 : threads);
    free(x32);
    return 0;
}

NVQ_EXPORT int nvq_ref_quantized_matmul(int mode, int group, int bits, int dtype, int transpose,
                                        int64_t batch, int64_t M, int64_t N, int64_t K, int64_t w_batch,
                                        const void *x, const uint32_t *w, const void *scales,
                                        const void *biases, void *y, int threads) {
    if (!dtype_ok(dtype)) return 1;
    if (mode == NVQ_AFFINE) {
        if (!affine_ok(group, bits) || !biases) return 1;
    } else {
        int g2, b2;
        if (!fp_mode_ok(mode, &g2, &b2) || g2 != group || b2 != bits || biases) return 1;
    }
    if (w_batch != 1 && w_batch != batch) return 1;
    if (batch == 0 || M == 0 || N == 0) return 0;
    if (K == 0) { memset(y, 0, (size_t)(batch * M * N) * dtype_size(dtype)); return 0; }
    int64_t cols = transpose ? K : N; /* values per packed row */
    int64_t rows = transpose ? N : K;
    if (cols % group) return 1;
    int64_t n_values = rows * cols, n_groups = n_values / group;
    float *dense = (float *)malloc((size_t)n_values * 4);
    float *x32 = (float *)malloc((size_t)(M * K) * 4);
    if (!dense || !x32) { free(dense); free(x32); return 2; }
    if (threads < 1) threads = 1;
    int rc = 0;
    for (int64_t b = 0; b < batch && !rc; b++) {
        if (b == 0 || w_batch != 1) {
            int64_t wb = w_batch == 1 ? 0 : b;
            int ssz = mode == NVQ_AFFINE ? dtype_size(dtype) : 1;
            rc = dense_f32(mode, group, bits, dtype, w + wb * (n_values * bits / 32),
                           (const char *)scales + wb * n_groups * ssz,
                           biases ? (const char *)biases + wb * n_groups * ssz : NULL, n_values, dense);
            if (rc) break;
        }
        for (int64_t i = 0; i < M * K; i++) x32[i] = load_f32(x, b * M * K + i, dtype);
        product_rows(dtype, transpose, M, N, K, x32, dense, (char *)y + b * M * N * dtype_size(dtype), threads);
    }
    free(dense);
    free(x32);
    return rc;
}

/* quantized.rs:679-719: output batch i = x[lhs[i]] . dequantize(w[rhs[i]])^T, each pair an
 * M-row product of its own.  The reference gathers the operands and runs one batched product;
 * rows of different pairs never mix, so dequantizing each selected expert once and walking
 * its pairs gives the same bits without materialising the gathered weights. */
NVQ_EXPORT int nvq_ref_gather_qmm(int mode, int group, int bits, int dtype, int transpose, int64_t pairs,
                                  int64_t M, int64_t N, int64_t K, int64_t x_batches, int64_t experts,
                                  const void *x, const uint32_t *w, const void *scales, const void *biases,
                                  const uint32_t *lhs, const uint32_t *rhs, void *y, int threads) {
    if (!dtype_ok(dtype)) return 1;
    if (mode == NVQ_AFFINE) {
        if (!affine_ok(group, bits) || !biases) return 1;
    } else {
        int g2, b2;
        if (!fp_mode_ok(mode, &g2, &b2) || g2 != group || b2 != bits || biases) return 1;
    }
    if (pairs == 0 || M == 0 || N == 0) return 0;
    if (K == 0) { memset(y, 0, (size_t)(pairs * M * N) * dtype_size(dtype)); return 0; }
    for (int64_t i = 0; i < pairs; i++)
        if ((int64_t)lhs[i] >= x_batches || (int64_t)rhs[i] >= experts) return 1;
    int64_t cols = transpose ? K : N, rows = transpose ? N : K;
    if (cols % group) return 1;
    int64_t n_values = rows * cols, n_groups = n_values / group;
    float *dense = (float *)malloc((size_t)n_values * 4);
    float *x32 = (float *)malloc((size_t)(M * K) * 4);
    if (!dense || !x32) { free(dense); free(x32); return 2; }
    if (threads < 1) threads = 1;
    int ssz = mode == NVQ_AFFINE ? dtype_size(dtype) : 1;
    int rc = 0;
    for (int64_t e = 0; e < experts && !rc; e++) {
        int have = 0;
        for (int64_t i = 0; i < pairs && !rc; i++) {
            if ((int64_t)rhs[i] != e) continue;
            if (!have) {
                rc = dense_f32(mode, group, bits, dtype, w + e * (n_values * bits / 32),
                               (const char *)scales + e * n_groups * ssz,
                               biases ? (const char *)biases + e * n_groups * ssz : NULL, n_values, dense);
                if (rc) break;
                have = 1;
            }
            for (int64_t t = 0; t < M * K; t++) x32[t] = load_f32(x, (int64_t)lhs[i] * M * K + t, dtype);
            product_rows(dtype, transpose, M, N, K, x32, dense, (char *)y + i * M * N * dtype_size(dtype), threads);
        }
    }
    free(dense);
    free(x32);
    return rc;
}

/* Selected outputs of a transposed product, for shapes whose whole product is out of reach
 * of a CPU test: y_sample[t] = element (rows[t], cols[t]) of x[M,K] . dequantize(w[N,..])^T,
 * computed exactly as nvq_ref_quantized_matmul would. */
NVQ_EXPORT int nvq_ref_quantized_matmul_sample(int mode, int group, int bits, int dtype, int64_t M,
                                               int64_t N, int64_t K, const void *x, const uint32_t *w,
                                               const void *scales, const void *biases, int64_t samples,
                                               const int64_t *rows, const int64_t *cols, void *y_sample) {
    if (!dtype_ok(dtype) || K % group) return 1;
    float *dense = (float *)malloc((size_t)K * 4), *x32 = (float *)malloc((size_t)K * 4);
    if (!dense || !x32) { free(dense); free(x32); return 2; }
    int ssz = mode == NVQ_AFFINE ? dtype_size(dtype) : 1;
    int rc = 0;
    for (int64_t t = 0; t < samples && !rc; t++) {
        int64_t i = rows[t], j = cols[t];
        if (i < 0 || i >= M || j < 0 || j >= N) { rc = 1; break; }
        rc = dense_f32(mode, group, bits, dtype, w + j * (K * bits / 32),
                       (const char *)scales + j * (K / group) * ssz,
                       biases ? (const char *)biases + j * (K / group) * ssz : NULL, K, dense);
        if (rc) break;
        for (int64_t p = 0; p < K; p++) x32[p] = load_f32(x, i * K + p, dtype);
        float v = M <= 16 ? dot_few_rows(x32, dense, 1, K) : dot_many_rows(x32, dense, 1, K);
        store_rounded(y_sample, t, dtype, (double)v);
    }
    free(dense);
    free(x32);
    return rc;
}

NVQ_EXPORT int nvq_ref_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
