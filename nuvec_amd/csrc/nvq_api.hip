// Host side of the C ABI: device record, error reporting, the reference's argument checks and
// the routing from an operation to a gfx950 kernel.
//
// Validation restates nuvec's record-time checks so that a caller binding this library gets the
// same refusals with the same wording (reference: crates/nuvec-core/src/quantized.rs:133-168,
// 363-379; crates/nuvec-core/src/primitive.rs:1223-1320, 1412-1460).
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "nvq_internal.h"

#include <math.h>

namespace nvq {

// Scratch for nvq_quantized_matmul_static, the entry point for callers that cannot allocate: the float32 partial sums of
// a product whose K is split over the grid.  Every device the library is loaded on holds its own copy of the array at its
// own address; host code never passes the array's name to a kernel, only the address hipGetSymbolAddress reported
// for the bound device (g_scratch).
static __device__ __align__(256) unsigned char scratch[NVQ_STATIC_SCRATCH_BYTES];

namespace {
thread_local char g_error[512] = "";
constexpr int kMaxDevices = 64;
void *g_scratch[kMaxDevices] = {};  // device address of `scratch` per device, written under the device record's mutex

// Written under the mutex by nvq_init; `ready`, `device` and `units` are read without it on every call.
struct DeviceRecord {
    std::mutex mutex;
    std::atomic<bool> ready{false};
    std::atomic<int> device{-1};
    std::atomic<int> units{0};
    hipDeviceProp_t prop;
} g_device;

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
}  // namespace

int32_t fail(int32_t status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return status;
}

const char *dtype_name(int32_t d) {
    switch (d) {
    case NVQ_U8: return "uint8";
    case NVQ_U32: return "uint32";
    case NVQ_I32: return "int32";
    case NVQ_F16: return "float16";
    case NVQ_BF16: return "bfloat16";
    case NVQ_F32: return "float32";
    default: return "unknown";
    }
}

const char *mode_name(int32_t m) {
    switch (m) {
    case NVQ_AFFINE: return "affine";
    case NVQ_MXFP4: return "mxfp4";
    case NVQ_MXFP8: return "mxfp8";
    case NVQ_NVFP4: return "nvfp4";
    default: return "unknown";
    }
}

// The bound device must also be the calling thread's current one: kernels launch on the current device, and the
// caller's stream and buffers belong to the device it bound.
int32_t require_device() {
    if (!g_device.ready.load(std::memory_order_acquire)) return fail(NVQ_NO_DEVICE, "no device bound: call nvq_init first");
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess) {
        (void)hipGetLastError();
        return fail(NVQ_NO_DEVICE, "no current HIP device");
    }
    const int bound = g_device.device.load(std::memory_order_relaxed);
    if (current != bound)
        return fail(NVQ_INVALID_ARGUMENT, "the calling thread's current device is %d but the library is bound to device %d", current, bound);
    return NVQ_OK;
}

int32_t compute_units() { return g_device.ready.load(std::memory_order_acquire) ? g_device.units.load(std::memory_order_relaxed) : 0; }

// Quant::checked (quantized.rs:133-168), messages included.
int32_t check_quant(const nvq_quant *q, const char *op) {
    if (q == nullptr) return fail(NVQ_INVALID_ARGUMENT, "%s: null quant", op);
    const int g = q->group_size, b = q->bits;
    if (q->mode == NVQ_AFFINE) {
        if (!(g == 32 || g == 64 || g == 128))
            return fail(NVQ_INVALID_ARGUMENT, "%s: group size %d is not supported (32, 64 or 128)", op, g);
        if (!((b >= 1 && b <= 6) || b == 8))
            return fail(NVQ_INVALID_ARGUMENT, "%s: %d bits are not supported (1, 2, 3, 4, 5, 6 or 8)", op, b);
        return NVQ_OK;
    }
    int eg, eb;
    switch (q->mode) {
    case NVQ_MXFP4: eg = 32; eb = 4; break;
    case NVQ_MXFP8: eg = 32; eb = 8; break;
    case NVQ_NVFP4: eg = 16; eb = 4; break;
    default: return fail(NVQ_INVALID_ARGUMENT, "%s: invalid quantization mode %d (affine, mxfp4, mxfp8 or nvfp4)", op, q->mode);
    }
    if (g != eg)
        return fail(NVQ_INVALID_ARGUMENT, "%s: %s quantization requires group size %d but got %d", op, mode_name(q->mode), eg, g);
    if (b != eb)
        return fail(NVQ_INVALID_ARGUMENT, "%s: %s quantization requires bits to be %d but got %d", op, mode_name(q->mode), eb, b);
    return NVQ_OK;
}

namespace {

// check_groups (quantized.rs:363-379) as far as pointers can tell: affine needs biases, the
// floating-point modes must not have them.
int32_t check_groups(const char *op, int32_t mode, const void *biases) {
    if (mode == NVQ_AFFINE && biases == nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "%s: biases must be provided for affine quantization", op);
    if (mode != NVQ_AFFINE && biases != nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "%s: biases must be null for quantization mode '%s'", op, mode_name(mode));
    return NVQ_OK;
}

int32_t check_float(const char *op, int32_t dtype) {
    if (!float_dtype(dtype)) return fail(NVQ_INVALID_ARGUMENT, "%s: unsupported dtype %s", op, dtype_name(dtype));
    return NVQ_OK;
}

// The kernels use 16-byte vector accesses on x, the packed weights, y and the workspace; allocations from
// hipMalloc (and any sub-buffer at a multiple of 16 bytes) satisfy this.  Scales and biases are read at element
// granularity (the kernels that fetch them in wider pieces start at the enclosing aligned piece), so they need
// only the alignment of their element type.
int32_t check_aligned(const char *op, const char *what, const void *p, size_t to = 16) {
    if (p != nullptr && !aligned(p, to))
        return fail(NVQ_UNSUPPORTED, "%s: %s is not %zu-byte aligned", op, what, to);
    return NVQ_OK;
}

int32_t check_groups_aligned(const char *op, const nvq_quant &q, int32_t dtype, const void *scales, const void *biases) {
    const size_t to = q.mode == NVQ_AFFINE ? (size_t)dtype_size(dtype) : 1;
    int32_t rc = check_aligned(op, "scales", scales, to);
    return rc != NVQ_OK ? rc : check_aligned(op, "biases", biases, to);
}

#define NVQ_TRY(expr)                     \
    do {                                  \
        int32_t nvq_rc_ = (expr);         \
        if (nvq_rc_ != NVQ_OK) return nvq_rc_; \
    } while (0)

// The product's argument checks (primitive.rs:1279-1320 after quantized_columns,
// primitive.rs:1412-1460): K must be whole groups and whole packed words.
int32_t check_product_dims(const char *op, const nvq_quant &q, int32_t transpose, int64_t m, int64_t n, int64_t k) {
    if (m < 0 || n < 0 || k < 0) return fail(NVQ_INVALID_ARGUMENT, "%s: negative dimension", op);
    const int64_t cols = transpose ? k : n;  // values per packed row
    if (cols % q.group_size != 0 || (cols * q.bits) % 32 != 0)
        return fail(NVQ_INVALID_ARGUMENT,
                    "%s: packed weights [.., %lld] and scales [.., %lld] do not match group size %d and %d bits", op,
                    (long long)(cols * q.bits / 32), (long long)(cols / q.group_size), q.group_size, q.bits);
    if (m >= (1LL << 31) || n >= (1LL << 31) || k >= (1LL << 31))
        return fail(NVQ_UNSUPPORTED, "%s: dimensions beyond 2^31", op);
    return NVQ_OK;
}

}  // namespace
}  // namespace nvq

using namespace nvq;

// Whether the tiled kernel beats the passes of the few-row kernel, from their measured behaviour: the few-row kernel
// runs a block (one per compute unit) per pass of 32 rows and 64 weight rows - 32 weight rows where that leaves fewer
// than 192 blocks (qmf::row_groups).  Both kernels were timed on 1236 products (fifteen weight shapes from W[4096,128]
// to W[16384,2048] and W[4096,14336], seven formats, bf16 and f16, 24 to 1024 rows of x) and fitted by least squares:
// a round of the few-row kernel's blocks costs a fixed part (the tables of scales, the sum of eight wavefronts' partial
// tiles) and a part per value of K, more of both with the CPU's weights; the tiled kernel takes its estimate of the
// steps and of the second kernel that adds the splits of K, scaled (MXFP4 expands cheaply, the CPU's weights dearly),
// plus a fixed part.  The fits are off by 9 to 14 % on average; choosing by them costs 1.7 % against always taking
// the faster kernel, 30 % at worst (the rule before them, a round at 5 us per 1024 values of K against the bare
// estimate: 6.3 % and 2.5 x - W[4096,1024] at 256 rows 47.4 us on the few-row kernel against 19.8).  The counterpart
// of the reference's device-specific `qmv_batch_limit` (crates/nuvec-core/src/gpu.rs:1506-1538).
static bool tiled_is_faster(const nvq::ProductArgs &a) {
    const double passes = (double)((a.m + 31) / 32) * (double)a.batch, k = (double)a.k;
    const double blocks64 = passes * (double)((a.n + 63) / 64);
    const bool wide = blocks64 >= 192.0, exact = a.exact_weights != 0, fp4 = a.mode == NVQ_MXFP4;
    const double blocks = wide ? blocks64 : passes * (double)((a.n + 31) / 32);
    const double round_us = wide ? (exact ? 13.5 + 4.4e-3 * k : 7.4 + (fp4 ? 2.16e-3 : 2.45e-3) * k)
                                 : (exact ? 8.0 + 2.0e-3 * k : 6.0 + 2.05e-3 * k);
    const double few_us = ceil(blocks / fmax(1.0, (double)nvq::compute_units())) * round_us;
    const double steps_us = nvq::qmm_estimate_us(a);
    const double tiled_us = exact ? 1.8 + 1.26 * steps_us : fp4 ? 3.2 + 0.73 * steps_us : 3.4 + steps_us;
    return fmax(7.0, tiled_us) < few_us;  // (its fastest launches, at K = 128, take 6 to 7.4 us)
}

// Whether the 16x16x32 kernel with directly loaded weight operands takes a few-row product, from its measured times
// against the kernels it replaces (bf16, us per launch, new / old):
//   3 bits g64   W[4096,4096]  2 rows 6.0 / 10.5, 16 rows 6.9 / 11.5;  W[14336,4096] 16 rows 11.9 / 19.9;  W[151936,1024] 4 rows 22.6 / 72.8
//   8 bits g32   W[4096,4096] 16 rows 11.1 / 12.9;  W[4096,14336] 8 rows 23.6 / 28.1;  W[151936,1024] 8 rows 47.8 / 74.5
//   4 bits g64   W[14336,4096] 12 rows 12.8 / 17.5;  W[32768,2048] 16 rows 13.3 / 26.0  (up to 8 rows the 4-bit decode kernels are ahead: 13.1 / 11.1)
//   4 bits g128  W[14336,4096]  4 rows 10.4 / 13.5, 8 rows 10.8 / 16.4;  W[151936,1024] 1 row 19.9 / 50.1
// One row stays on the vector kernels except for very tall matrices.  More than 16 rows are passes of 16 that read
// the weights again (from the caches, if the matrix is small enough): measured up to 192 rows at five shapes, e.g.
// 4 bits g64 W[4096,4096] 64 rows 11.8 / 14.6, 96 rows 18.2 / 18.6; W[14336,4096] 64 rows 33.7 / 35.3, 96 rows 49.3 / 33.9;
// W[1024,4096] 128 rows 8.2 / 15.5; 8 bits g32 W[4096,4096] 32 rows 13.0 / 16.9, 48 rows 19.5 / 17.1.  The rule below is
// passes x megabytes of weights, fitted to those tables.
// Whether a few-row product stays on the decode kernels of the vector units (per-row work there is cheaper than a
// matrix-core kernel's full dequantization up to these row counts).
// A few rows of 3-, 5-, 6- or 8-bit codes that the decode kernel's variants take ahead of the matrix-core kernels: K
// beyond 2048 (shorter rows leave its lanes idle), for 5 and 6 bits also two rows at K = 2048.
static bool wide_decode_takes(const nvq::ProductArgs &a) {
    return (a.k > 2048 || (a.k == 2048 && a.m <= 2 && (a.bits == 5 || a.bits == 6))) && nvq::qmv_decode_takes_width(a);
}

static bool takes_decode(const nvq::ProductArgs &a) {
    if (a.dtype == NVQ_F32) return false;
    if (a.mode != NVQ_AFFINE) return nvq::qmv_block_decode_takes(a);
    if (a.bits == 4) return a.m <= 4 || nvq::qmv_d16_takes(a);
    if (a.bits == 2) return nvq::qmv_decode_takes_width(a) && (a.m == 1 || a.k > 2048);
    return a.bits >= 3 && (a.m == 1 || wide_decode_takes(a));
}

static bool takes_few_rows_direct(const nvq::ProductArgs &a) {
    if (!nvq::qmd_supported(a)) return false;
    if (a.mode != NVQ_AFFINE && nvq::qmv_block_decode_takes(a)) return false;  // one or two rows (some more): the decode kernel of the vector units
    const int64_t rows = a.n * a.batch;
    // The kernel's block is one wavefront per 512 values of K, up to eight - the largest divisor of K / 512 where K is
    // longer and walked in chunks.  Short blocks against many weight rows lose: W[32768,512] (one wavefront) 2 to 4 rows
    // of 4-bit codes in groups of 32 15 us against 5 - 7 on the short-row decode kernel, 10 to 16 rows 17 - 20 against
    // 13 - 14 on the few-row kernel; K = 6144 (six wavefronts, two chunks) at 10 to 16 rows 16 - 22 against 13 - 17.
    if (a.mode == NVQ_AFFINE && a.k < 1024 && rows >= 16384) return false;  // (MXFP4 there: 8.4 - 8.8 us at 4 to 8 rows against 10.4 - 11.2)
    if (a.k > 4096) {
        const int64_t all = a.k / 512;
        int64_t slices = 8;
        while (all % slices != 0) slices--;
        if (slices < 7) return false;
    }
    // The block formats (bf16, new / the few-row kernel of the 32x32x16 instruction): MXFP4 W[14336,4096] 1 row 11.1 / 13.4,
    // 16 rows 11.3 / 14.6; W[4096,4096] 1 row 5.4 / 6.9, 32 rows 7.0 / 14.2; NVFP4 W[14336,4096] 1 row 13.2 / 17.7;
    // MXFP8 W[4096,14336] 16 rows 18.8 / 29.4: every row count up to 16, 32 where K or the matrix is short.
    if (a.mode != NVQ_AFFINE && a.m <= 32) return a.m <= 16 || a.k <= 4096 || rows <= 4096;
    if (a.m > 16) {
        // (5 and 6 bits: the passes' never-rounded weights put one of 139360 half-precision outputs of a 130-row product of
        // 6-bit codes in groups of 128 at 1.06 x the bar against the CPU's doubly rounded ones; the tiles round once)
        if (a.k > 4096 || a.m > 192 || a.bits == 5 || a.bits == 6) return false;  // (a long K is walked in chunks with x staged per chunk and pass)
        // (W[32768,512] at 17 to 192 rows: 17 - 22 us against 11.3 - 13 on the tiles)
        const double passes = (double)((a.m + 15) / 16), mb = (double)rows * (double)a.k * a.bits / 8.0 / 1048576.0;
        // Timed against the better of the other two kernels on 462 products (us, this kernel / the other): MXFP4
        // W[4096,4096] at 64 rows 9.0 / 13.4, W[16384,2048] at 64 rows 0.73 of the other, W[11008,4096] at 48 rows 0.93, at
        // 80 rows 1.11; NVFP4 W[4096,4096] at 64 rows 0.87, at 96 rows 1.08; 4 bits in groups of 32 W[11008,4096] at 17 to
        // 32 rows 0.74, W[14336,4096] 1.24 - 1.31.
        if (a.mode != NVQ_AFFINE) return passes * mb <= (a.mode == NVQ_MXFP4 ? 64.0 : 48.0);
        if (a.bits == 8) return passes * mb <= (a.group == 32 ? 34.0 : 40.0);
        if (a.group == 32) return passes * mb <= 45.0;
        return passes * mb <= 50.0 || (passes <= 4.0 && mb <= 32.0);
    }
    // One or two rows of 3-bit, up to three or four of 8-bit codes with K beyond 2048: the decode kernel of the vector units (3 bits, us: W[4096,4096]
    // g128 4.91 -> 4.07, W[14336,4096] g128 9.16 -> 7.75, W[32768,4096] g64 20.1 -> 15.0; with K up to 2048 and many
    // weight rows this kernel stays ahead: W[65536,2048] 17.7 against 24.6).
    if (a.bits != 4 && a.bits != 2 && wide_decode_takes(a)) return false;
    switch (a.bits) {
    case 2: return !(nvq::qmv_decode_takes_width(a) && (a.m == 1 || a.k > 2048));
    case 5:  // beside the decode kernel's rows, against the few-row kernel of the 32x32x16 instruction (us): 6 bits W[4096,4096] g64
    case 6:  // 5 / 16 rows 12.2 / 12.4 -> 7.8 / 8.7, W[14336,4096] 8 / 16 rows 21.2 / 21.9 -> 16.6 / 17.2, W[4096,14336] g128 16 rows
             // 31.0 -> 20.0, W[8192,2048] 4 / 16 rows 8.8 / 10.6 -> 6.4 / 7.2, W[2048,1024] 3 / 16 rows 6.4 / 9.2 -> 4.4 / 5.1; 32 / 64 rows of
             // W[4096,4096] stay on the tiles (16.9 / 18.2 against 10.5 / 15.5: see above); 5 bits alike
        return a.m >= 2;
    case 3: return a.group == 128 || a.m >= 2 || rows >= 16384;
    case 8: return a.m >= 2 || rows >= (a.group == 128 ? 32768 : 65536);
    default:  // 4 bits: beside the 4-bit decode kernels
        if (a.group == 64) return a.m > 8 || (a.m > 4 && !nvq::qmv_d16_takes(a));
        if (a.group == 128) return a.m >= 3 || rows >= 32768;
        return a.m >= 5 || (rows >= 32768 && a.m >= 2) || rows >= 65536;
    }
}

// Whether a product of 4- or 8-bit affine codes takes the batched-decode kernel.  4 bits: 17 to 64 rows of x (passes of 32 rows up to 32, of 64 beyond)
// against 8192 weight rows or more, where its one pass over the weights beats the passes of 16 rows of the few-row
// kernels and the tiles of the tiled one.  The bounds are those of 702 products timed on both sides (4 bits, K 512 to
// 16384, 8192 to 151936 weight rows, 17 to 128 rows, the three group sizes, bf16 and f16): without the kernel they take
// 18.8 % more time than always the faster of the two, with this rule 0.2 % (worst 1.22 x).  us, this kernel / the other:
// W[14336,4096] 17 / 32 / 33 / 64 rows 13.8 / 14.1 / 18.8 / 19.2 against 16.4 / 17.5 / 28.8 / 32.9; W[16384,1024] 32 rows
// 0.53 x, W[32768,4096] 64 rows 32.7 / 52.7, W[11008,8192] in groups of 32 at 32 rows 23.6 / 44.8, W[32768,14336] 64 rows
// 0.57 x.  It loses, and is not taken: under 11008 weight rows from K = 3072 (one round of 128 blocks: W[8192,4096] 1.2 x at
// 32 rows), groups of 128 below K = 4096 (W[8192,2048] 1.26 x: the few-row kernel's per-group work is small there), K = 512
// beyond 16384 weight rows and K = 1024 beyond 32768 (65536 from 33 rows) - one or two of the block's four wavefronts
// have a chunk of K -, and from 65 rows (two passes: W[14336,4096] 34.4 against 31.7 on the tiles) but for fewer than 11008
// weight rows at K <= 4096 (W[8192,2048] at 128 rows 12.4 / 17.6).
// Up to 16 rows (a pass of 16), timed the same way on 420 products of 5 to 16 rows (8.2 % -> 0.6 %): from 9 rows against
// 11008 weight rows or more at K <= 1024 (W[14336,512] at 16 rows 7.0 against 10.2 us, W[65536,512] 11.7 / 27.2,
// W[32768,1024] 10.6 / 15.6), at K <= 2048 up to 16384 weight rows (W[14336,2048] 7.7 / 9.3) and from K = 8192
// (W[14336,8192] 19.9 / 25.9, W[32768,14336] 67.5 / 95.9) - at K = 4096 the direct few-row kernel's slices fit and it is
// level or ahead, and groups of 128 cost it little below K = 8192; from 5 rows at K = 512 against 14336 weight rows or
// more (W[65536,512] at 8 rows 11.8 / 25.3) and, in groups of 32, at K >= 4096 against 11008 to 16384 or from 28672 weight rows
// (W[14336,4096] at 8 rows 12.7 / 15.5, W[11008,8192] 20.8 / 31.6, W[32768,4096] at 16 rows 25.0 / 30.0, W[28672,8192] 46.2 /
// 72.0; between 16384 and 28672 weight rows the 128-row blocks leave compute units idle: W[20480,4096] 20.8 / 19.2).
static bool takes_batched_decode(const nvq::ProductArgs &a) {
    if (a.m < 5 || a.m > 128 || a.n < 8192 || !nvq::qmr_supported(a)) return false;
    // 8-bit codes (blocks of 64 weight rows only; a window of codes one window ahead): 418 products of 8 to 128 rows timed
    // on both sides, 19.5 % -> 0.5 %.  W[14336,4096] at 16 / 32 / 64 rows 13.6-15.6 / 17.9 / 23.2 us against 15.0 / 20.3 /
    // 38.3; W[11008,8192] in groups of 32 at 32 rows 32.0 / 53.6; W[32768,4096] at 64 rows 51 / 61-62.
    if (a.bits == 8) {
        if (a.m < 8 || a.k < 1024) return false;  // (fewer rows and shorter K were not timed)
        if (a.m > 64) return a.n < 11008;
        if (a.m <= 16) return a.n >= 11008 && (a.k >= 8192 || a.n <= 16384 || (a.k <= 1024 && a.n <= 32768));
        return !(a.k <= 1024 && a.n >= 28672 && a.m >= 33);
    }
    if (a.m <= 16) {
        if (a.group == 32) return a.k >= 4096 && a.n >= 11008 && (a.n <= 16384 || a.n >= 28672);
        if (a.m <= 8) return a.k < 1024 && a.n >= 14336;
        if (a.n < 11008 || (a.group == 128 && a.k < 8192)) return false;
        if (a.k <= 1024 || a.k >= 8192) return true;
        return a.k <= 2048 && a.n <= 16384;
    }
    if (a.m > 64) return a.n < 11008 && a.k <= 4096;
    if (a.group == 128) return a.k >= 4096 && a.n >= 11008;
    if (a.k >= 3072) return a.n >= 11008;
    if (a.k >= 2048) return true;
    if (a.k >= 1024) return a.n <= (a.m <= 32 ? 32768 : 65536);
    return a.n <= 16384;
}

// The kernels' view of a product descriptor.
// Which half-precision affine products materialise the CPU's weights, round(round(code * scale) + bias)
// (kernels.rs:835-859), bit for bit, instead of the one rounding of fma(code, scale, bias) the device kernels give a
// weight.  The CPU's first rounding is a noise of about 0.7 % of a bfloat16 weight; over a product it is the same
// fraction of an output's deviation, and the worst of M x N outputs against the bar of a product (1e-2 of a row's
// largest output) grows with the rows of x and falls with the outputs of a row: measured over 100 seeds each, one-
// rounding products of 130 rows and 1024..2048 outputs exceed the bar for one seed in five, of 12 rows for none, of
// 2048 rows and 14336 outputs stay at 0.8 of it.  So: every row of fewer than 1024 outputs, and bfloat16 products of
// more than 16 rows up to 8192 outputs (float16 stays under 0.65 of its bar from 1024 outputs on).  With the CPU's
// weights only the order of the float32 sums differs: at most one rounding step of an output, 0.78 of the bar.
static bool wants_exact_weights(int32_t mode, int32_t dtype, int64_t n, int64_t m) {
    if (mode != NVQ_AFFINE || dtype == NVQ_F32) return false;
    return n < 1024 || (dtype == NVQ_BF16 && m > 16 && n < 8192);
}

static nvq::ProductArgs product_args(const nvq_qmm_desc *d, int64_t batch) {
    nvq::ProductArgs a{};
    a.mode = d->quant.mode; a.group = d->quant.group_size; a.bits = d->quant.bits; a.dtype = d->dtype;
    a.m = d->m; a.n = d->n; a.k = d->k;
    a.batch = batch;
    // Row-exact products of up to ROW_INDEPENDENT_ROWS = 8 rows per item, and products built with `rows` (every row
    // count on the matrix-vector kernels), give each row the bits of its one-row product (lib.rs:159-193,
    // gpu.rs:6956-6981, primitive.rs:489-493).
    const int64_t item = d->item_rows > 0 ? d->item_rows : d->m;
    a.row_exact = d->rows != 0 || (d->row_exact != 0 && item <= 8);
    a.exact_weights = wants_exact_weights(d->quant.mode, d->dtype, d->n, a.row_exact ? 1 : d->m);  // (row-exact: one-row products)
    // Batch dimensions that one stride per operand describes together are merged (dimension i with i + 1 where every
    // operand's stride of i is its stride of i + 1 times the extent of i + 1; extents of 1 vanish): a [B, H] batch of
    // dense operands is one dimension, which the matrix-core kernels take.
    int nd = 0;
    for (int i = 0; i < d->batch_ndim; i++) {
        if (d->batch_shape[i] == 1) continue;
        const int64_t e = d->batch_shape[i], xs = d->x_strides[i], ws = d->w_strides[i], ss = d->s_strides[i];
        if (nd > 0 && a.x_strides[nd - 1] == xs * e && a.w_strides[nd - 1] == ws * e && a.s_strides[nd - 1] == ss * e) {
            a.batch_shape[nd - 1] *= e;
            a.x_strides[nd - 1] = xs, a.w_strides[nd - 1] = ws, a.s_strides[nd - 1] = ss;
        } else {
            a.batch_shape[nd] = e, a.x_strides[nd] = xs, a.w_strides[nd] = ws, a.s_strides[nd] = ss;
            nd++;
        }
    }
    a.batch_ndim = nd;
    return a;
}

extern "C" {

const char *nvq_last_error(void) { return g_error; }

const char *nvq_version(void) { return "nuvec-hip 0.1.0 (gfx950)"; }

int32_t nvq_init(int32_t device) {
    std::lock_guard<std::mutex> lock(g_device.mutex);
    if (g_device.ready && g_device.device == device) return NVQ_OK;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(NVQ_NO_DEVICE, "no HIP device is visible");
    }
    if (device < 0 || device >= count) return fail(NVQ_NO_DEVICE, "device %d of %d does not exist", device, count);
    hipDeviceProp_t prop;
    NVQ_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(NVQ_NO_DEVICE, "device %d is %s: this library holds gfx950 code only", device, prop.gcnArchName);
    if (device >= kMaxDevices) return fail(NVQ_NO_DEVICE, "device %d: at most %d devices", device, kMaxDevices);
    if (g_scratch[device] == nullptr) {  // once per device, with that device current
        int current = -1;
        NVQ_HIP_TRY(hipGetDevice(&current));
        if (current != device) NVQ_HIP_TRY(hipSetDevice(device));
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (current != device) (void)hipSetDevice(current);
        if (e != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            return fail(NVQ_BACKEND, "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
        }
        g_scratch[device] = ptr;
    }
    g_device.prop = prop;
    g_device.device.store(device, std::memory_order_relaxed);
    g_device.units.store(prop.multiProcessorCount, std::memory_order_relaxed);
    g_device.ready.store(true, std::memory_order_release);
    return NVQ_OK;
}

int32_t nvq_get_device_info(nvq_device_info *info) {
    if (info == nullptr) return fail(NVQ_INVALID_ARGUMENT, "device_info: null output");
    NVQ_TRY(require_device());
    std::lock_guard<std::mutex> lock(g_device.mutex);
    memset(info, 0, sizeof *info);
    info->device = g_device.device;
    info->compute_units = g_device.prop.multiProcessorCount;
    info->wavefront_size = g_device.prop.warpSize;
    info->lds_bytes_per_block = (int32_t)g_device.prop.sharedMemPerBlock;
    info->global_memory_bytes = (int64_t)g_device.prop.totalGlobalMem;
    snprintf(info->arch, sizeof info->arch, "%s", g_device.prop.gcnArchName);
    snprintf(info->name, sizeof info->name, "%s", g_device.prop.name);
    return NVQ_OK;
}

int32_t nvq_calibrate(int32_t kind, const void *buffer, int64_t bytes, int32_t iters, void *sink, int64_t *work, void *stream) {
    NVQ_TRY(require_device());
    return launch_calibrate(kind, buffer, bytes, iters, sink, work, (hipStream_t)stream);
}

int32_t nvq_quant_check(const nvq_quant *quant, const char *op) { return check_quant(quant, op ? op : "quant"); }

// quantized.rs:724-735 (`ROW_TOKENS` = ROW_INDEPENDENT_ROWS * 8 = 64: crates/nuvec-core/src/lib.rs).
int32_t nvq_gather_grouped(int64_t rows, int64_t experts, int32_t row_exact) {
    const int64_t least = row_exact ? 65 : 16;
    return rows >= least && rows / (experts > 1 ? experts : 1) >= 4;
}

// primitive.rs:1378-1395 (MLX's validate_global_scale): NVFP4 only.
static int32_t check_global_scale(const char *op, const nvq_quant *quant, const float *global_scale) {
    if (global_scale == nullptr) return fail(NVQ_INVALID_ARGUMENT, "%s: null global scale", op);
    if (quant->mode != NVQ_NVFP4)
        return fail(NVQ_INVALID_ARGUMENT, "%s: a global scale is only supported for nvfp4, got %s", op, mode_name(quant->mode));
    return NVQ_OK;
}

static int32_t quantize_any(const nvq_quant *quant, int32_t dtype, const void *w, int64_t rows, int64_t cols, void *packed,
                            void *scales, void *biases, const float *global_scale, void *stream) {
    NVQ_TRY(check_quant(quant, "quantize"));
    // primitive.rs:1234-1243
    if (!float_dtype(dtype)) return fail(NVQ_INVALID_ARGUMENT, "quantize: unsupported dtype %s", dtype_name(dtype));
    if (rows < 0 || cols < 0 || cols % quant->group_size != 0)
        return fail(NVQ_INVALID_ARGUMENT,
                    "quantize: needs at least 2 dimensions with the last divisible by the group size %d, got shape [%lld, %lld]",
                    quant->group_size, (long long)rows, (long long)cols);
    NVQ_TRY(check_groups("quantize", quant->mode, quant->mode == NVQ_AFFINE ? biases : nullptr));
    if (quant->mode != NVQ_AFFINE && biases != nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "quantize: biases must be null for quantization mode '%s'", mode_name(quant->mode));
    if (rows == 0 || cols == 0) return NVQ_OK;
    if (w == nullptr || packed == nullptr || scales == nullptr) return fail(NVQ_INVALID_ARGUMENT, "quantize: null operand");
    NVQ_TRY(require_device());
    NVQ_TRY(check_aligned("quantize", "w", w));
    NVQ_TRY(check_aligned("quantize", "packed", packed));
    NVQ_TRY(check_groups_aligned("quantize", *quant, dtype, scales, biases));
    const int64_t n = rows * cols;
    if (n >= (1LL << 32)) return fail(NVQ_INVALID_ARGUMENT, "quantize: %lld elements; an operand holds fewer than 2^32", (long long)n);
    if (quant->mode == NVQ_AFFINE)
        return launch_affine_quantize(dtype, quant->group_size, quant->bits, w, n, packed, scales, biases, (hipStream_t)stream);
    return launch_fp_quantize(quant->mode, dtype, w, n, packed, scales, global_scale, (hipStream_t)stream);
}

int32_t nvq_quantize(const nvq_quant *quant, int32_t dtype, const void *w, int64_t rows, int64_t cols, void *packed,
                     void *scales, void *biases, void *stream) {
    return quantize_any(quant, dtype, w, rows, cols, packed, scales, biases, nullptr, stream);
}

int32_t nvq_quantize_scaled(const nvq_quant *quant, int32_t dtype, const void *w, int64_t rows, int64_t cols,
                            const float *global_scale, void *packed, void *scales, void *stream) {
    NVQ_TRY(check_quant(quant, "quantize"));
    NVQ_TRY(check_global_scale("quantize", quant, global_scale));
    return quantize_any(quant, dtype, w, rows, cols, packed, scales, nullptr, global_scale, stream);
}

int32_t nvq_quantize_dequantize(const nvq_quant *quant, int32_t dtype, const void *x, int64_t rows, int64_t cols,
                                const float *global_scale, void *out, void *stream) {
    NVQ_TRY(check_quant(quant, "quantize_dequantize"));
    if (quant->mode == NVQ_AFFINE)  // products.rs:263-289: qqmm quantizes in a floating-point mode
        return fail(NVQ_INVALID_ARGUMENT, "quantize_dequantize: mode affine is not a floating-point block format");
    if (global_scale != nullptr) NVQ_TRY(check_global_scale("quantize_dequantize", quant, global_scale));
    if (!float_dtype(dtype)) return fail(NVQ_INVALID_ARGUMENT, "quantize_dequantize: unsupported dtype %s", dtype_name(dtype));
    if (rows < 0 || cols < 0 || cols % quant->group_size != 0)
        return fail(NVQ_INVALID_ARGUMENT, "quantize_dequantize: the last dimension %lld is not whole groups of %d", (long long)cols,
                    quant->group_size);
    if (rows == 0 || cols == 0) return NVQ_OK;
    if (x == nullptr || out == nullptr) return fail(NVQ_INVALID_ARGUMENT, "quantize_dequantize: null operand");
    if (rows * cols >= (1LL << 32)) return fail(NVQ_INVALID_ARGUMENT, "quantize_dequantize: an operand holds fewer than 2^32 elements");
    NVQ_TRY(require_device());
    NVQ_TRY(check_aligned("quantize_dequantize", "x", x));
    NVQ_TRY(check_aligned("quantize_dequantize", "out", out));
    return launch_fp_quantize_dequantize(quant->mode, dtype, x, rows * cols, out, global_scale, (hipStream_t)stream);
}

// Shared by nvq_dequantize and nvq_dequantize_rows: `count` output rows, each table row ids[r] (or row r).
static int32_t dequantize_any(const char *op, const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales,
                              const void *biases, int64_t table_rows, int64_t cols, const uint32_t *ids, int64_t count,
                              void *out, void *stream, const float *global_scale = nullptr) {
    NVQ_TRY(check_quant(quant, op));
    NVQ_TRY(check_groups(op, quant->mode, biases));
    // primitive.rs:1272-1276
    if (!float_dtype(dtype)) return fail(NVQ_INVALID_ARGUMENT, "%s: unsupported dtype %s", op, dtype_name(dtype));
    if (table_rows < 0 || count < 0 || cols < 0 || cols % quant->group_size != 0 || (cols * quant->bits) % 32 != 0)
        return fail(NVQ_INVALID_ARGUMENT,
                    "%s: packed weights [%lld, %lld] and scales [%lld, %lld] do not match group size %d and %d bits", op,
                    (long long)table_rows, (long long)(cols * quant->bits / 32), (long long)table_rows,
                    (long long)(cols / quant->group_size), quant->group_size, quant->bits);
    if (count == 0 || cols == 0) return NVQ_OK;
    if (table_rows == 0) return fail(NVQ_INVALID_ARGUMENT, "%s: rows of an empty table", op);
    if (packed == nullptr || scales == nullptr || out == nullptr) return fail(NVQ_INVALID_ARGUMENT, "%s: null operand", op);
    NVQ_TRY(require_device());
    NVQ_TRY(check_aligned(op, "packed", packed));
    NVQ_TRY(check_aligned(op, "out", out));
    NVQ_TRY(check_groups_aligned(op, *quant, dtype, scales, biases));
    const int64_t n = count * cols;
    if (n >= (1LL << 32) || table_rows * cols >= (1LL << 32))  // gpu.rs:1582-1590
        return fail(NVQ_INVALID_ARGUMENT, "%s: %lld elements; an operand holds fewer than 2^32", op, (long long)n);
    if (quant->mode == NVQ_AFFINE)
        return launch_affine_dequantize(dtype, quant->group_size, quant->bits, packed, scales, biases, n, out, ids, cols,
                                        table_rows, (hipStream_t)stream);
    return launch_fp_dequantize(quant->mode, dtype, packed, scales, n, out, ids, cols, table_rows, global_scale, (hipStream_t)stream);
}

int32_t nvq_dequantize(const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales, const void *biases,
                       int64_t rows, int64_t cols, void *out, void *stream) {
    return dequantize_any("dequantize", quant, dtype, packed, scales, biases, rows, cols, nullptr, rows, out, stream);
}

int32_t nvq_dequantize_scaled(const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales,
                              const float *global_scale, int64_t rows, int64_t cols, void *out, void *stream) {
    NVQ_TRY(check_quant(quant, "dequantize"));
    NVQ_TRY(check_global_scale("dequantize", quant, global_scale));
    return dequantize_any("dequantize", quant, dtype, packed, scales, nullptr, rows, cols, nullptr, rows, out, stream, global_scale);
}

int32_t nvq_dequantize_rows(const nvq_quant *quant, int32_t dtype, const void *packed, const void *scales, const void *biases,
                            int64_t table_rows, int64_t cols, const uint32_t *ids, int64_t count, void *out, void *stream) {
    if (ids == nullptr && count > 0) return fail(NVQ_INVALID_ARGUMENT, "dequantize_rows: null ids");
    return dequantize_any("dequantize_rows", quant, dtype, packed, scales, biases, table_rows, cols, ids, count, out, stream);
}

static int32_t check_qmm(const nvq_qmm_desc *d, const char *op) {
    if (d == nullptr) return fail(NVQ_INVALID_ARGUMENT, "%s: null descriptor", op);
    NVQ_TRY(check_quant(&d->quant, op));
    NVQ_TRY(check_float(op, d->dtype));
    NVQ_TRY(check_product_dims(op, d->quant, d->transpose, d->m, d->n, d->k));
    if (d->batch_ndim < 0 || d->batch_ndim > NVQ_MAX_BATCH_DIMS)
        return fail(NVQ_INVALID_ARGUMENT, "%s: %d batch dimensions (at most %d)", op, d->batch_ndim, NVQ_MAX_BATCH_DIMS);
    for (int i = 0; i < d->batch_ndim; i++)
        if (d->batch_shape[i] < 0 || d->x_strides[i] < 0 || d->w_strides[i] < 0 || d->s_strides[i] < 0)
            return fail(NVQ_INVALID_ARGUMENT, "%s: negative batch shape or stride", op);
    return NVQ_OK;
}

// The limits of the launch grids, the same ones the launch meets: batches and passes of rows travel in grid y and z
// (at most 65535 each).  Every mode, width, element type and both orientations have a kernel: the matrix-core kernels
// take affine and MXFP4 transposed, the general kernels the rest.
static int32_t check_grid(const nvq_qmm_desc *d) {
    int64_t batch = 1;
    for (int i = 0; i < d->batch_ndim; i++) batch *= d->batch_shape[i];
    if (batch == 0 || d->m == 0 || d->n == 0 || d->k == 0) return NVQ_OK;
    if (batch > 65535) return fail(NVQ_UNSUPPORTED, "quantized_matmul: %lld batches exceed the grid limit", (long long)batch);
    const int64_t passes = (d->m + 3) / 4;  // the vector kernels take four rows of x per pass
    if (!d->transpose) {
        if (batch * (d->m == 1 ? 1 : passes) > 65535)
            return fail(NVQ_UNSUPPORTED, "quantized_matmul: %lld row passes exceed the grid limit", (long long)(batch * passes));
        return NVQ_OK;
    }
    const ProductArgs a = product_args(d, batch);
    const int64_t item = d->item_rows > 0 ? d->item_rows : d->m;
    if (!a.row_exact && item > 32 && qmm_supported(a)) return NVQ_OK;  // tiled: rows travel in grid x
    if (passes > 65535) return fail(NVQ_UNSUPPORTED, "quantized_matmul: %lld rows exceed the grid limit", (long long)d->m);
    return NVQ_OK;
}

int32_t nvq_quantized_matmul_supported(const nvq_qmm_desc *d) {
    if (check_qmm(d, "quantized_matmul") != NVQ_OK) return 0;
    return check_grid(d) == NVQ_OK;
}

// Whether a transposed product goes to the tiled kernel: routed by one item's rows, as the reference does
// (gpu.rs:6975-6981), where its tiles cost less than the passes of the few-row kernel.
static bool takes_tiled(const nvq_qmm_desc *d, const ProductArgs &a) {
    const int64_t item = d->item_rows > 0 ? d->item_rows : d->m;
    return item > 16 && qmm_supported(a) && (!qmf_supported(a) || tiled_is_faster(a));
}

// The kernel family of a product (the counterpart of the routing in GpuEval::quantized_matmul, gpu.rs:6934-7168).
enum class Route { kUntransposed, kVector, kTiled, kTiledF32, kBatchedDecode, kFewRowsDirect, kFewRows };
static Route pick_route(const nvq_qmm_desc *d, const ProductArgs &a);

size_t nvq_quantized_matmul_workspace_bytes(const nvq_qmm_desc *d) {
    if (check_qmm(d, "quantized_matmul") != NVQ_OK) return 0;
    int64_t batch = 1;
    for (int i = 0; i < d->batch_ndim; i++) batch *= d->batch_shape[i];
    if (batch == 0 || d->m == 0 || d->n == 0 || d->k == 0 || require_device() != NVQ_OK) return 0;
    const ProductArgs a = product_args(d, batch);
    // float32 partial sums of the splits of K: weights stored [K, N], or few tiles of a long K
    if (!d->transpose) return qvm_workspace_bytes(a);
    return pick_route(d, a) == Route::kTiled ? qmm_workspace_bytes(a) : 0;
}

static Route pick_route(const nvq_qmm_desc *d, const ProductArgs &a) {
    if (!d->transpose) return Route::kUntransposed;        // weights stored [K, N]
    if (a.row_exact) return Route::kVector;                // the vector kernels: a row's bits do not depend on its neighbours
    if (qmm_f32_takes(a)) return Route::kTiledF32;         // float32, many rows: the float32 matrix instruction
    if (takes_batched_decode(a)) return Route::kBatchedDecode;
    if (takes_few_rows_direct(a)) return Route::kFewRowsDirect;  // (also passes of 16 rows of small matrices, ahead of the tiles)
    if (takes_tiled(d, a)) return Route::kTiled;
    // Up to four rows of 4-bit affine weights (up to eight where the 16x16x32 decode kernel takes the product): the
    // decode kernels (per-row work on the vector units, which is cheaper than the matrix-core kernel's full
    // dequantization up to there).  A single row of the other affine widths from 3 bits, and the few rows the decode
    // kernel's 3-, 5-, 6- and 8-bit variants take (wide_decode_takes): the vector kernels too (a row of 3-bit codes at
    // 4096 x 4096: 4.0 us against 10.1 us on the matrix cores, of 8-bit codes in groups of 32 5.8 against 11.7 us).
    // Other few-row products share one weight decode on the matrix cores where those kernels take them.
    // The CPU's weights (rows of fewer than 1024 outputs) at up to 16 rows: the vector kernel's passes of four rows are
    // ahead of the few-row kernel's exact variant on matrices this small (us: W[768,2048] 2 to 8 rows 4.6 - 4.9 against
    // 7.4 - 8.4, W[512,4096] 16 rows 7.8 / 10.7, W[640,8192] 12 rows 13 / 17, 16 rows 21 / 18).
    if (a.exact_weights && a.m <= 16 && a.m * a.k <= 12 * 8192) return Route::kVector;
    if (!takes_decode(a) && qmf_supported(a)) return Route::kFewRows;
    // Five rows and more that neither few-row kernel takes (1, 3 and 5 bits with K off whole windows of 128): the tiles
    // where the vector kernel's passes of four rows add up (3 bits, W[11008,2880]: 5 / 16 rows 42 / 82 us there, 23 here;
    // W[2880,2880]: 5 to 8 rows, two passes of four, 14 against 16, 12 rows 21 against 16.)
    if (!takes_decode(a) && a.m >= 5 && (double)((a.m + 3) / 4) * (double)a.n * (double)a.k * (double)a.batch >= 20.0e6 && qmm_supported(a))
        return Route::kTiled;
    return Route::kVector;
}

static int32_t quantized_matmul_any(const nvq_qmm_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                                    const float *global_scale, void *y, void *workspace, void *stream, const void *row_bias = nullptr) {
    NVQ_TRY(check_qmm(d, "quantized_matmul"));
    NVQ_TRY(check_groups("quantized_matmul", d->quant.mode, biases));
    int64_t batch = 1;
    for (int i = 0; i < d->batch_ndim; i++) batch *= d->batch_shape[i];
    if (batch == 0 || d->m == 0 || d->n == 0) return NVQ_OK;
    if (x == nullptr || w == nullptr || scales == nullptr || y == nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "quantized_matmul: null operand");
    NVQ_TRY(require_device());
    NVQ_TRY(check_grid(d));
    NVQ_TRY(check_aligned("quantized_matmul", "x", x));
    NVQ_TRY(check_aligned("quantized_matmul", "w", w));
    NVQ_TRY(check_aligned("quantized_matmul", "y", y));
    NVQ_TRY(check_aligned("quantized_matmul", "workspace", workspace));
    NVQ_TRY(check_groups_aligned("quantized_matmul", d->quant, d->dtype, scales, biases));
    if (d->k == 0) {  // an empty reduction is zero (crates/nuvec-cpu/src/matmul.rs:237-240)
        return launch_fill_zero(y, batch * d->m * d->n * dtype_size(d->dtype), (hipStream_t)stream);
    }
    ProductArgs a = product_args(d, batch);
    a.x = x; a.w = w; a.scales = scales; a.biases = biases; a.y = y;
    a.global_scale = global_scale;
    a.row_bias = row_bias;
    switch (pick_route(d, a)) {
    case Route::kUntransposed: return launch_qvm(a, workspace, (hipStream_t)stream);
    case Route::kTiled: return launch_qmm(a, workspace, (hipStream_t)stream);  // without a workspace: K is not split
    case Route::kTiledF32: return launch_qmm_f32(a, (hipStream_t)stream);
    case Route::kBatchedDecode: return launch_qmr(a, (hipStream_t)stream);
    case Route::kFewRowsDirect: return launch_qmd(a, (hipStream_t)stream);
    case Route::kFewRows: return launch_qmf(a, (hipStream_t)stream);
    default: return launch_qmv(a, (hipStream_t)stream);
    }
}

const char *nvq_quantized_matmul_route(const nvq_qmm_desc *d) {
    if (check_qmm(d, "quantized_matmul") != NVQ_OK || check_grid(d) != NVQ_OK || require_device() != NVQ_OK) return nullptr;
    int64_t batch = 1;
    for (int i = 0; i < d->batch_ndim; i++) batch *= d->batch_shape[i];
    ProductArgs a = product_args(d, batch);
    a.x = a.w = a.scales = a.biases = reinterpret_cast<const void *>(uintptr_t{256});  // operands aligned as hipMalloc aligns them
    a.y = reinterpret_cast<void *>(uintptr_t{256});
    switch (pick_route(d, a)) {
    case Route::kUntransposed: return qvm_kernel_name(a);
    case Route::kTiled: return "qmm_kernel";
    case Route::kTiledF32: return "qmm_f32_kernel";
    case Route::kBatchedDecode: return "qmr_kernel";
    case Route::kFewRowsDirect: return "qmd_kernel";
    case Route::kFewRows: return "qmf_kernel";
    default: return qmv_kernel_name(a);
    }
}

int32_t nvq_quantized_matmul(const nvq_qmm_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                             void *y, void *workspace, void *stream) {
    return quantized_matmul_any(d, x, w, scales, biases, nullptr, y, workspace, stream);
}

int32_t nvq_quantized_linear(const nvq_qmm_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                             const void *bias, void *y, void *workspace, void *stream) {
    NVQ_TRY(check_qmm(d, "quantized_linear"));
    if (bias != nullptr && d->k == 0)  // an empty reduction is zero: the fill kernel has no bias epilogue
        return fail(NVQ_UNSUPPORTED, "quantized_linear: a bias over an empty reduction");
    NVQ_TRY(check_aligned("quantized_linear", "bias", bias, (size_t)dtype_size(d->dtype)));
    return quantized_matmul_any(d, x, w, scales, biases, nullptr, y, workspace, stream, bias);
}

// `Mlp::forward` up to its down projection (crates/nuvec-lm/src/model.rs:2066-2074) for a few rows of x: the gate and up
// products and the gated activation in one kernel.
int32_t nvq_quantized_matmul_glu(const nvq_qmm_desc *d, int32_t activation, float alpha, float limit, const void *x, const void *w,
                                 const void *scales, const void *biases, const void *bias, void *y, void *stream) {
    const char *op = "quantized_matmul";
    NVQ_TRY(check_qmm(d, op));
    NVQ_TRY(check_groups(op, d->quant.mode, biases));
    if (activation < NVQ_GLU_SWIGLU || activation > NVQ_GLU_GEGLU) return fail(NVQ_INVALID_ARGUMENT, "%s: unknown activation %d", op, activation);
    if (d->m == 0 || d->n == 0) return NVQ_OK;
    if (x == nullptr || w == nullptr || scales == nullptr || y == nullptr) return fail(NVQ_INVALID_ARGUMENT, "%s: null operand", op);
    if (!d->transpose || d->batch_ndim != 0 || d->k == 0 || d->n % 128 != 0 || d->row_exact || d->rows)
        return fail(NVQ_UNSUPPORTED, "%s: the gated epilogue takes x [M, K] times transposed weights whose gate and up rows alternate in runs of 64", op);
    if (wants_exact_weights(d->quant.mode, d->dtype, d->n / 2, d->m))
        return fail(NVQ_UNSUPPORTED, "%s: the gated epilogue takes affine projections of 1024 rows or more each", op);
    NVQ_TRY(require_device());
    NVQ_TRY(check_aligned(op, "x", x));
    NVQ_TRY(check_aligned(op, "w", w));
    NVQ_TRY(check_aligned(op, "y", y));
    NVQ_TRY(check_groups_aligned(op, d->quant, d->dtype, scales, biases));
    NVQ_TRY(check_aligned(op, "bias", bias, (size_t)dtype_size(d->dtype)));
    ProductArgs a{};
    a.x = x; a.w = w; a.scales = scales; a.biases = biases; a.y = y;
    a.mode = d->quant.mode; a.group = d->quant.group_size; a.bits = d->quant.bits; a.dtype = d->dtype;
    a.m = d->m; a.n = d->n; a.k = d->k;
    a.batch = 1;
    a.row_bias = bias;
    a.glu = 1 + activation; a.glu_alpha = alpha; a.glu_limit = limit;
    if (!qmv_glu_pairs_take(a)) return fail(NVQ_UNSUPPORTED, "%s: the decode kernel does not take this product with the gated epilogue", op);
    return launch_qmv_glu_pairs(a, (hipStream_t)stream);
}

int32_t nvq_quantized_matmul_static(const nvq_qmm_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                                    void *y, void *stream) {
    NVQ_TRY(check_qmm(d, "quantized_matmul"));
    const size_t need = nvq_quantized_matmul_workspace_bytes(d);  // 0 without a device: the launch below says so
    if (need > (size_t)NVQ_STATIC_SCRATCH_BYTES)
        return fail(NVQ_UNSUPPORTED, "quantized_matmul: this product splits K through %zu bytes of partial sums; the static scratch holds %d",
                    need, NVQ_STATIC_SCRATCH_BYTES);
    void *workspace = nullptr;
    if (need > 0) {
        NVQ_TRY(require_device());
        workspace = g_scratch[g_device.device.load(std::memory_order_relaxed)];
    }
    return quantized_matmul_any(d, x, w, scales, biases, nullptr, y, workspace, stream);
}

int32_t nvq_quantized_matmul_scaled(const nvq_qmm_desc *d, const void *x, const void *w, const void *scales,
                                    const float *global_scale, void *y, void *workspace, void *stream) {
    NVQ_TRY(check_qmm(d, "quantized_matmul"));
    NVQ_TRY(check_global_scale("quantized_matmul", &d->quant, global_scale));
    // quantized.rs:481-491: with a global scale only a transposed product of two matrices reaches a kernel; the
    // reference dequantizes and multiplies densely otherwise.
    if (!d->transpose || d->batch_ndim != 0)
        return fail(NVQ_UNSUPPORTED, "quantized_matmul: with a global scale only x [M, K] times transposed w [N, K'] has a kernel");
    return quantized_matmul_any(d, x, w, scales, nullptr, global_scale, y, workspace, stream);
}

// The argument checks and the fit rule of the fused attention kernel (fast/imp.rs:3944-3992, 4037-4075).
static int32_t check_attention(const nvq_attention_desc *d) {
    const char *op = "quantized_attention";
    if (d == nullptr) return fail(NVQ_INVALID_ARGUMENT, "%s: null descriptor", op);
    NVQ_TRY(check_float(op, d->dtype));
    const nvq_quant quant{NVQ_AFFINE, d->group_size, d->bits};
    NVQ_TRY(check_quant(&quant, op));
    if (d->batch < 0 || d->query_heads < 0 || d->key_heads < 0 || d->positions < 0 || d->head_dim < 0)
        return fail(NVQ_INVALID_ARGUMENT, "%s: negative size", op);
    if (d->key_heads == 0 || d->query_heads % d->key_heads != 0)
        return fail(NVQ_INVALID_ARGUMENT, "%s: %lld query heads over %lld key heads", op, (long long)d->query_heads, (long long)d->key_heads);
    const int64_t rep = d->query_heads / d->key_heads;
    if ((d->head_dim != 64 && d->head_dim != 128) || (d->bits != 3 && d->bits != 4 && d->bits != 8) || d->head_dim % d->group_size != 0 ||
        !(rep == 1 || rep == 2 || rep == 4 || rep == 8) || d->positions < 1 || d->batch > 65535 ||
        d->batch * d->key_heads * d->positions * d->head_dim >= (1LL << 31))
        return fail(NVQ_UNSUPPORTED, "%s: the kernel takes head sizes 64 and 128, 3, 4 or 8 bits, 1, 2, 4 or 8 query heads per key head", op);
    return NVQ_OK;
}

size_t nvq_quantized_attention_workspace_bytes(const nvq_attention_desc *d) {
    if (check_attention(d) != NVQ_OK || require_device() != NVQ_OK) return 0;
    return attention_workspace_bytes(*d);
}

int32_t nvq_quantized_attention(const nvq_attention_desc *d, const void *q, const void *k_w, const void *k_s, const void *k_b,
                                const void *v_w, const void *v_s, const void *v_b, const void *sinks, void *out, void *workspace,
                                void *stream) {
    const char *op = "quantized_attention";
    NVQ_TRY(check_attention(d));
    if (d->batch == 0 || d->query_heads == 0) return NVQ_OK;
    if (q == nullptr || k_w == nullptr || k_s == nullptr || k_b == nullptr || v_w == nullptr || v_s == nullptr || v_b == nullptr || out == nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "%s: null operand", op);
    NVQ_TRY(require_device());
    NVQ_TRY(check_aligned(op, "keys", k_w));
    NVQ_TRY(check_aligned(op, "values", v_w));
    NVQ_TRY(check_aligned(op, "workspace", workspace));
    return launch_quantized_attention(*d, q, k_w, k_s, k_b, v_w, v_s, v_b, sinks, out, workspace, (hipStream_t)stream);
}

int32_t nvq_sorted_offsets(const uint32_t *indices, int64_t rows, int64_t m, int32_t groups, int32_t *offsets, void *stream) {
    if (rows < 0 || m < 0 || groups < 0) return fail(NVQ_INVALID_ARGUMENT, "sorted_offsets: negative size");
    if (rows == 0 || groups == 0) return NVQ_OK;
    if (offsets == nullptr || (indices == nullptr && m > 0)) return fail(NVQ_INVALID_ARGUMENT, "sorted_offsets: null operand");
    NVQ_TRY(require_device());
    return launch_sorted_offsets(indices, rows, m, groups, offsets, (hipStream_t)stream);
}

// float32 partial sums when the weights are stored [K, N] and K is split over the grid; nothing otherwise.
size_t nvq_gather_qmm_workspace_bytes(const nvq_gather_desc *d) {
    if (d == nullptr || d->transpose || check_quant(&d->quant, "gather_qmm") != NVQ_OK) return 0;
    if (d->pairs <= 0 || d->m <= 0 || d->n <= 0 || d->k <= 0 || require_device() != NVQ_OK) return 0;
    ProductArgs a{};
    a.mode = d->quant.mode; a.group = d->quant.group_size; a.bits = d->quant.bits; a.dtype = d->dtype;
    a.m = d->m; a.n = d->n; a.k = d->k;
    a.batch = d->pairs;
    a.row_exact = d->row_exact != 0;
    return qvm_workspace_bytes(a);
}

int32_t nvq_convert_packed(int32_t format, const nvq_quant *quant, int32_t dtype, const uint32_t *qweight, const uint32_t *qzeros,
                           const void *scales, int64_t rows, int64_t cols, uint32_t *weight, void *scales_out, void *biases_out,
                           void *stream) {
    NVQ_TRY(check_quant(quant, "convert_packed"));
    NVQ_TRY(check_float("convert_packed", dtype));
    const int32_t bits = quant->bits;
    if (quant->mode != NVQ_AFFINE || format < NVQ_PACKED_AWQ || format > NVQ_PACKED_GPTQ_V2 ||
        (format == NVQ_PACKED_AWQ ? bits != 4 : (bits != 4 && bits != 8)))  // config.rs:1140-1168
        return fail(NVQ_INVALID_ARGUMENT, "convert_packed: format %d with %d bits (AWQ loads 4 bits, GPTQ 4 and 8)", format, bits);
    if (rows < 0 || cols < 0) return fail(NVQ_INVALID_ARGUMENT, "convert_packed: negative size");
    const int64_t per_word = 32 / bits;
    const int64_t inputs = format == NVQ_PACKED_AWQ ? rows : rows * per_word, outputs = format == NVQ_PACKED_AWQ ? cols * per_word : cols;
    if (inputs % quant->group_size != 0)  // quant.rs:96-103
        return fail(NVQ_INVALID_ARGUMENT, "convert_packed: %lld inputs do not match groups of %d", (long long)inputs, quant->group_size);
    if (inputs == 0 || outputs == 0) return NVQ_OK;
    if (qweight == nullptr || scales == nullptr || weight == nullptr || scales_out == nullptr || biases_out == nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "convert_packed: null operand");
    NVQ_TRY(require_device());
    return launch_convert_packed(format, bits, dtype, qweight, qzeros, scales, inputs, outputs, inputs / quant->group_size, weight,
                                 scales_out, biases_out, (hipStream_t)stream);
}

size_t nvq_moe_order_workspace_bytes(int64_t pairs, int32_t experts) {
    if (pairs <= 0 || experts <= 0) return 0;
    return moe_order_workspace_bytes(pairs, experts);
}

int32_t nvq_moe_order(const uint32_t *ids, int64_t pairs, int32_t experts, uint32_t *order, uint32_t *restore,
                      uint32_t *sorted_ids, int32_t *offsets, void *workspace, void *stream) {
    if (pairs < 0 || experts <= 0) return fail(NVQ_INVALID_ARGUMENT, "moe_order: %lld pairs, %d experts", (long long)pairs, experts);
    if (pairs > INT32_MAX) return fail(NVQ_INVALID_ARGUMENT, "moe_order: %lld pairs exceed 32-bit positions", (long long)pairs);
    if (moe_order_lds_bytes(experts) > 64 * 1024)
        return fail(NVQ_UNSUPPORTED, "moe_order: %d experts exceed the block's counters", experts);
    if (offsets == nullptr || (pairs > 0 && (ids == nullptr || order == nullptr || restore == nullptr || sorted_ids == nullptr)))
        return fail(NVQ_INVALID_ARGUMENT, "moe_order: null operand");
    NVQ_TRY(require_device());
    return launch_moe_order(ids, pairs, experts, order, restore, sorted_ids, offsets, workspace, (hipStream_t)stream);
}

int32_t nvq_moe_route(int32_t dtype, const void *probs, int64_t rows, int32_t experts, int32_t k, int32_t normalize,
                      uint32_t *indices, void *scores, void *stream) {
    // fast/imp.rs:2652-2673
    if (!float_dtype(dtype)) return fail(NVQ_INVALID_ARGUMENT, "moe_route: unsupported dtype %s", dtype_name(dtype));
    if (rows < 0 || experts < 0 || k < 1 || k > experts)
        return fail(NVQ_INVALID_ARGUMENT, "moe_route: k must be in 1..=%d for probabilities of shape [%lld, %d]", experts, (long long)rows, experts);
    if (experts > 1024 || (normalize && k > 64))
        return fail(NVQ_UNSUPPORTED, "moe_route: %d experts, k = %d: the kernel takes up to 1024 experts and sums up to 64 scores", experts, k);
    if (rows == 0) return NVQ_OK;
    if (rows > INT32_MAX) return fail(NVQ_INVALID_ARGUMENT, "moe_route: %lld rows", (long long)rows);
    if (probs == nullptr || indices == nullptr || scores == nullptr) return fail(NVQ_INVALID_ARGUMENT, "moe_route: null operand");
    NVQ_TRY(require_device());
    return launch_moe_route(dtype, probs, rows, experts, k, normalize != 0, indices, scores, (hipStream_t)stream);
}

int32_t nvq_weighted_sum(int32_t dtype, const void *x, const void *w, int64_t rows, int32_t k, int64_t d, void *out, void *stream) {
    // fast/imp.rs:2731-2747
    if (!float_dtype(dtype)) return fail(NVQ_INVALID_ARGUMENT, "weighted_sum: unsupported dtype %s", dtype_name(dtype));
    if (rows < 0 || k < 0 || d < 0) return fail(NVQ_INVALID_ARGUMENT, "weighted_sum: x must be [..., k, D] and w [..., k]");
    if (k < 1 || k >= 32) return fail(NVQ_UNSUPPORTED, "weighted_sum: k = %d: the kernel sums 1 to 31 weighted rows", k);
    if (rows == 0 || d == 0) return NVQ_OK;
    if (rows * d >= (1LL << 32) || rows * k * d >= (1LL << 32)) return fail(NVQ_INVALID_ARGUMENT, "weighted_sum: an operand holds fewer than 2^32 elements");
    if (x == nullptr || w == nullptr || out == nullptr) return fail(NVQ_INVALID_ARGUMENT, "weighted_sum: null operand");
    NVQ_TRY(require_device());
    return launch_weighted_sum(dtype, x, w, rows, k, d, out, (hipStream_t)stream);
}

int32_t nvq_glu(const nvq_glu_desc *d, const void *gate, const void *up, const void *gate_bias, const void *up_bias, const int32_t *ids,
                void *out, void *stream) {
    // model.rs:2139-2143, 2157-2170
    if (d == nullptr) return fail(NVQ_INVALID_ARGUMENT, "glu: null descriptor");
    if (!float_dtype(d->dtype)) return fail(NVQ_INVALID_ARGUMENT, "glu: unsupported dtype %s", dtype_name(d->dtype));
    if (d->activation < NVQ_GLU_SWIGLU || d->activation > NVQ_GLU_GEGLU)
        return fail(NVQ_INVALID_ARGUMENT, "glu: unknown activation %d", d->activation);
    if (d->rows < 0 || d->hidden < 0 || d->experts < 0) return fail(NVQ_INVALID_ARGUMENT, "glu: negative size");
    if (d->gate_stride < d->hidden || d->up_stride < d->hidden)
        return fail(NVQ_INVALID_ARGUMENT, "glu: a row stride (%lld, %lld) below the %lld columns", (long long)d->gate_stride,
                    (long long)d->up_stride, (long long)d->hidden);
    if ((gate_bias == nullptr) != (up_bias == nullptr)) return fail(NVQ_INVALID_ARGUMENT, "glu: one bias without the other");
    if (gate_bias != nullptr && (ids == nullptr || d->experts < 1)) return fail(NVQ_INVALID_ARGUMENT, "glu: biases need the rows' expert ids");
    if (d->rows == 0 || d->hidden == 0) return NVQ_OK;
    if (d->rows * d->hidden >= (1LL << 40)) return fail(NVQ_INVALID_ARGUMENT, "glu: more than 2^40 outputs");
    if (gate == nullptr || up == nullptr || out == nullptr) return fail(NVQ_INVALID_ARGUMENT, "glu: null operand");
    NVQ_TRY(require_device());
    return launch_glu(*d, gate, up, gate_bias, up_bias, ids, out, (hipStream_t)stream);
}

struct GluEpilogue {  // activation < 0: no activation, only the experts' bias
    int32_t activation;
    float alpha, limit;
    const void *expert_bias;
};

static int32_t gather_qmm_any(const nvq_gather_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                              const float *global_scale, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                              const uint32_t *out_rows, void *y, void *workspace, void *stream, const GluEpilogue *glu = nullptr) {
    if (d == nullptr) return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: null descriptor");
    NVQ_TRY(check_quant(&d->quant, "gather_qmm"));
    NVQ_TRY(check_groups("gather_qmm", d->quant.mode, biases));
    NVQ_TRY(check_float("gather_qmm", d->dtype));
    NVQ_TRY(check_product_dims("gather_qmm", d->quant, d->transpose, d->m, d->n, d->k));
    if (d->pairs < 0 || d->x_batches < 0 || d->experts < 0) return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: negative size");
    if (d->pairs == 0 || d->m == 0 || d->n == 0) return NVQ_OK;
    // Indices are clamped into [0, x_batches) and [0, experts) on the device: an empty operand leaves nothing to clamp to.
    if (d->x_batches < 1 || d->experts < 1)
        return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: %lld pairs index %lld batches of x and %lld experts", (long long)d->pairs,
                    (long long)d->x_batches, (long long)d->experts);
    if (x == nullptr || w == nullptr || scales == nullptr || y == nullptr || lhs == nullptr || rhs == nullptr)
        return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: null operand");
    NVQ_TRY(require_device());
    if (!d->transpose && global_scale != nullptr)
        return fail(NVQ_UNSUPPORTED, "gather_qmm: no gfx950 kernel for untransposed weights with a global scale");
    if (!d->transpose && out_rows != nullptr)
        return fail(NVQ_UNSUPPORTED, "gather_qmm: no gfx950 kernel for untransposed weights with scattered output rows");
    NVQ_TRY(check_aligned("gather_qmm", "x", x));
    NVQ_TRY(check_aligned("gather_qmm", "w", w));
    NVQ_TRY(check_aligned("gather_qmm", "y", y));
    NVQ_TRY(check_aligned("gather_qmm", "workspace", workspace));
    NVQ_TRY(check_groups_aligned("gather_qmm", d->quant, d->dtype, scales, biases));
    NVQ_TRY(check_aligned("gather_qmm", "lhs", lhs, 4));
    NVQ_TRY(check_aligned("gather_qmm", "rhs", rhs, 4));
    NVQ_TRY(check_aligned("gather_qmm", "offsets", offsets, 4));
    const void *expert_bias = nullptr;
    if (glu != nullptr && glu->activation < 0) {  // the experts' bias alone: the grouped kernel's epilogue
        expert_bias = glu->expert_bias;
        glu = nullptr;
        NVQ_TRY(check_aligned("gather_qmm", "expert bias", expert_bias, (size_t)dtype_size(d->dtype)));
        if (expert_bias != nullptr && (!d->transpose || d->k == 0))
            return fail(NVQ_UNSUPPORTED, "gather_qmm: the experts' bias takes transposed weights and a reduction that is not empty");
    }
    if (glu != nullptr) {
        if (glu->activation < NVQ_GLU_SWIGLU || glu->activation > NVQ_GLU_GEGLU)
            return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: unknown activation %d", glu->activation);
        if (!d->transpose || (offsets != nullptr && d->m != 1) || d->k == 0 || d->n % 128 != 0)
            return fail(NVQ_UNSUPPORTED, "gather_qmm: the gated epilogue belongs to products of transposed weights whose gate and up "
                                         "rows alternate in runs of 64 (sorted pairs: of one row each)");
    }
    if (d->k == 0) {
        return launch_fill_zero(y, d->pairs * d->m * d->n * dtype_size(d->dtype), (hipStream_t)stream);
    }
    ProductArgs a{};
    a.x = x; a.w = w; a.scales = scales; a.biases = biases; a.y = y;
    a.mode = d->quant.mode; a.group = d->quant.group_size; a.bits = d->quant.bits; a.dtype = d->dtype;
    a.m = d->m; a.n = d->n; a.k = d->k;
    a.batch = d->pairs;
    a.lhs = lhs; a.rhs = rhs;
    a.x_batches = d->x_batches; a.experts = d->experts;
    a.global_scale = global_scale;
    a.out_rows = out_rows;
    a.row_exact = d->row_exact != 0;
    a.exact_weights = wants_exact_weights(d->quant.mode, d->dtype, d->n, a.row_exact ? 1 : d->m);
    if (!d->transpose) {
        // Weights stored [K, N]: rows sorted by expert as groups on the matrix-core kernel (each expert's weights read once
        // per tile of its rows; the reference's grouped kernel of the block formats, gpu.rs:6786-6812), else one product
        // per pair.
        a.offsets = offsets;
        if (!qvm_takes_grouped(a)) a.offsets = nullptr;
        return launch_qvm(a, workspace, (hipStream_t)stream);
    }
    // Grouped route (rows sorted by expert, offsets given): each expert's rows against its weights, every
    // weight decoded once.  Otherwise one product per pair, on the kernel a single product of that many rows takes:
    // the few-row matrix-core kernels, or the decode kernels of the vector units (the experts of one decoded token are
    // pairs of one row each: 32 pairs against 4-bit W[14336,4096] 361 us on the few-row kernel, 221 us there).
    a.offsets = offsets;
    if (glu != nullptr) {
        // (projections of fewer rows take the exact-weights kernels as separate products: the epilogue form would differ)
        if (wants_exact_weights(d->quant.mode, d->dtype, d->n / 2, d->m))
            return fail(NVQ_UNSUPPORTED, "gather_qmm: the gated epilogue takes affine projections of 1024 rows or more each");
        a.exact_weights = 0;
        a.glu = 1 + glu->activation; a.glu_alpha = glu->alpha; a.glu_limit = glu->limit;
        if (offsets == nullptr) {  // unsorted pairs (the experts of decoded tokens): the decode kernel's epilogue
            a.row_bias = glu->expert_bias;
            a.row_bias_per_expert = 1;
            if (!qmv_glu_pairs_take(a)) return fail(NVQ_UNSUPPORTED, "gather_qmm: the decode kernel does not take these pairs with the gated epilogue");
            return launch_qmv_glu_pairs(a, (hipStream_t)stream);
        }
        a.expert_bias = glu->expert_bias;
        if (!qmf_supported(a)) return fail(NVQ_UNSUPPORTED, "gather_qmm: the grouped matrix-core kernel does not take this product");
        return launch_qmf(a, (hipStream_t)stream);
    }
    a.expert_bias = expert_bias;
    if (offsets != nullptr && qmf_supported(a)) return launch_qmf(a, (hipStream_t)stream);
    a.offsets = nullptr;
    if (expert_bias != nullptr) {  // one product per pair: the row-bias epilogue of those kernels, pair z taking row rhs[z]
        a.expert_bias = nullptr;
        a.row_bias = expert_bias;
        a.row_bias_per_expert = 1;
    }
    // Row-exact: every pair on the vector kernels, so that a pair has the bits of its one-row product whether the
    // gather is sorted or not and however many pairs it holds (the few-row contract of gpu.rs:7325-7340).
    if (!a.row_exact && takes_few_rows_direct(a)) return launch_qmd(a, (hipStream_t)stream);
    if (!a.row_exact && !takes_decode(a) && qmf_supported(a)) return launch_qmf(a, (hipStream_t)stream);
    return launch_qmv(a, (hipStream_t)stream);
}

int32_t nvq_gather_qmm(const nvq_gather_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                       const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets, void *y, void *workspace, void *stream) {
    return gather_qmm_any(d, x, w, scales, biases, nullptr, lhs, rhs, offsets, nullptr, y, workspace, stream);
}

int32_t nvq_gather_qmm_scaled(const nvq_gather_desc *d, const void *x, const void *w, const void *scales,
                              const float *global_scales, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                              void *y, void *workspace, void *stream) {
    if (d == nullptr) return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: null descriptor");
    NVQ_TRY(check_quant(&d->quant, "gather_qmm"));
    if (global_scales == nullptr) return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: null global scale");
    if (d->quant.mode != NVQ_NVFP4)  // quantized.rs:620-623
        return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: global scale is only supported for 'nvfp4' quantization mode");
    return gather_qmm_any(d, x, w, scales, nullptr, global_scales, lhs, rhs, offsets, nullptr, y, workspace, stream);
}

int32_t nvq_gather_qmm_scatter(const nvq_gather_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                               const float *global_scales, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                               const uint32_t *out_rows, void *y, void *workspace, void *stream) {
    if (out_rows == nullptr) return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: null output rows");
    if (global_scales != nullptr && d != nullptr && d->quant.mode != NVQ_NVFP4)  // quantized.rs:620-623
        return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: global scale is only supported for 'nvfp4' quantization mode");
    return gather_qmm_any(d, x, w, scales, biases, global_scales, lhs, rhs, offsets, out_rows, y, workspace, stream);
}

int32_t nvq_gather_qmm_expert_bias(const nvq_gather_desc *d, const void *x, const void *w, const void *scales, const void *biases,
                                   const float *global_scales, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                                   const uint32_t *out_rows, const void *expert_bias, void *y, void *workspace, void *stream) {
    if (d != nullptr && global_scales != nullptr && d->quant.mode != NVQ_NVFP4)  // quantized.rs:620-623
        return fail(NVQ_INVALID_ARGUMENT, "gather_qmm: global scale is only supported for 'nvfp4' quantization mode");
    const GluEpilogue only_bias{-1, 0.0f, 0.0f, expert_bias};
    return gather_qmm_any(d, x, w, scales, biases, global_scales, lhs, rhs, offsets, out_rows, y, workspace, stream, &only_bias);
}

int32_t nvq_gather_qmm_glu(const nvq_gather_desc *d, int32_t activation, float alpha, float limit, const void *x, const void *w,
                           const void *scales, const void *biases, const uint32_t *lhs, const uint32_t *rhs, const int32_t *offsets,
                           const void *expert_bias, void *y, void *stream) {
    const GluEpilogue glu{activation, alpha, limit, expert_bias};
    return gather_qmm_any(d, x, w, scales, biases, nullptr, lhs, rhs, offsets, nullptr, y, nullptr, stream, &glu);
}

}  // extern "C"
