// Host-only checks of the library's launch arithmetic, compiled and run by tests/test_host_checks.py with the host
// compiler (no GPU, no device code):
//   1. the rules that split K over the grid (nuvec_amd/csrc/nvq_splits.h), over a grid of shapes and chip sizes:
//      every split has a unit of K, the splits cover K, the kernels' own derivation of a split's length agrees with
//      the plan, the workspace is the [batch][splits][m][n] float32 array the kernels index, and the plan does not
//      depend on anything but the shape and the chip;
//   2. the mapping of a failing HIP call to the library's status codes (NVQ_HIP_TRY), which the reference has as
//      GpuError -> Error (crates/nuvec-gpu/src/gpu.rs:8289-8303): out of memory stays apart from every other failure.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "nvq_internal.h"

static int32_t g_status = -1;
static char g_message[512];
int32_t nvq::fail(int32_t status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_message, sizeof g_message, fmt, ap);
    va_end(ap);
    g_status = status;
    return status;
}

static int32_t wrapped(hipError_t e) {
    NVQ_HIP_TRY(e);
    return NVQ_OK;
}

static long g_failures = 0, g_plans = 0, g_split_plans = 0;
#define EXPECT(cond, ...)                                      \
    do {                                                       \
        if (!(cond)) {                                         \
            if (g_failures++ < 20) {                           \
                printf("FAILED %s: ", #cond);                  \
                printf(__VA_ARGS__);                           \
                printf("\n");                                  \
            }                                                  \
        }                                                      \
    } while (0)

using nvq::splits::Plan;
using nvq::splits::Product;

static void check_plan(const char *rule, const Plan &p, const Product &a, int cus, bool kernel_derives_length) {
    g_plans++;
    if (p.splits > 1) g_split_plans++;
    EXPECT(nvq::splits::every_split_has_a_unit(p), "%s m=%lld n=%lld k=%lld batch=%lld cus=%d: %d splits of %lld over %lld units", rule,
           (long long)a.m, (long long)a.n, (long long)a.k, (long long)a.batch, cus, p.splits, (long long)p.per_split, (long long)p.units);
    if (kernel_derives_length)  // qmn_kernel and qvm_kernel compute ceil(units / splits) themselves
        EXPECT((p.units + p.splits - 1) / p.splits == p.per_split, "%s m=%lld n=%lld k=%lld cus=%d: kernel takes %lld per split, plan %lld", rule,
               (long long)a.m, (long long)a.n, (long long)a.k, cus, (long long)((p.units + p.splits - 1) / p.splits), (long long)p.per_split);
    const size_t bytes = nvq::splits::workspace_bytes(p, a);
    // the last float a kernel writes: [batch - 1][splits - 1][m - 1][n - 1]
    const size_t last = ((((size_t)a.batch - 1) * p.splits + (p.splits - 1)) * a.m + (a.m - 1)) * a.n + (a.n - 1);
    if (p.splits > 1) EXPECT(bytes == (last + 1) * sizeof(float), "%s: workspace %zu bytes, last element %zu", rule, bytes, last);
    else EXPECT(bytes == 0, "%s: an unsplit product asks for %zu bytes", rule, bytes);
}

int main() {
    const int64_t ms[] = {1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 32, 33, 64, 100, 128, 129, 512, 2048, 5000};
    const int64_t ns[] = {8, 64, 128, 136, 1000, 1024, 2048, 2880, 4096, 14336, 50000};
    const int64_t steps64[] = {64, 128, 192, 256, 320, 448, 512, 576, 1024, 1088, 2880 / 64 * 64, 4096, 7168, 8192, 14336, 16384, 65536};
    const int64_t any_k[] = {1, 2, 3, 17, 64, 100, 127, 128, 129, 130, 255, 256, 257, 1000, 4096, 4097, 14336, 65537};
    const int64_t batches[] = {1, 2, 7, 64};
    const int cus_list[] = {1, 2, 8, 64, 104, 192, 256, 304, 1024};
    for (int64_t m : ms) for (int64_t n : ns) for (int64_t b : batches) for (int cus : cus_list) for (int flags = 0; flags < 4; flags++) {
        Product a{m, n, 0, b, (flags & 1) != 0, (flags & 2) != 0};
        for (int64_t k : steps64) {
            a.k = k;
            const Plan q = nvq::splits::qmm_plan(a, cus);
            check_plan("qmm", q, a, cus, false);
            EXPECT(b == 1 || q.splits == 1, "qmm splits a batch");
            EXPECT(q.splits == 1 || q.per_split % 4 == 0, "qmm m=%lld n=%lld k=%lld: a split of %lld steps is not whole table periods", (long long)m, (long long)n, (long long)k, (long long)q.per_split);
            EXPECT(q.splits <= 8, "qmm: %d splits", q.splits);
            for (int few = 0; few < 2; few++) {
                if (few && m > nvq::splits::kQmnFewRows) continue;
                const Plan r = nvq::splits::qmn_plan(a, cus, few != 0);
                check_plan("qmn", r, a, cus, true);
                EXPECT(r.splits <= 64, "qmn: %d splits", r.splits);
            }
        }
        for (int64_t k : any_k) {
            a.k = k;
            const Plan v = nvq::splits::qvm_plan(a, cus);
            check_plan("qvm", v, a, cus, true);
            EXPECT(v.splits <= 32, "qvm: %d splits", v.splits);
            if (a.row_exact) {  // the split of the one-row product, whatever the rows and batches
                Product one = a;
                one.m = 1, one.batch = 1;
                EXPECT(nvq::splits::qvm_plan(one, cus).splits == v.splits, "qvm row-exact m=%lld batch=%lld k=%lld: split differs from the one-row product's", (long long)m, (long long)b, (long long)k);
            }
        }
    }
    EXPECT(g_split_plans * 20 > g_plans, "only %ld of %ld plans split K: the grid of shapes does not exercise the rules", g_split_plans, g_plans);

    // a failing HIP call: out of memory keeps its own status, everything else is a backend failure, and the message
    // names the call and HIP's text
    EXPECT(wrapped(hipSuccess) == NVQ_OK && g_status == -1, "success reported as %d", g_status);
    EXPECT(wrapped(hipErrorOutOfMemory) == NVQ_OUT_OF_MEMORY && g_status == NVQ_OUT_OF_MEMORY, "out of memory reported as %d", g_status);
    EXPECT(strstr(g_message, "e: ") == g_message, "message '%s'", g_message);
    const hipError_t others[] = {hipErrorInvalidValue, hipErrorLaunchFailure, hipErrorIllegalAddress, hipErrorInvalidDevice, hipErrorNotReady, hipErrorUnknown};
    for (hipError_t e : others) {
        g_status = -1;
        EXPECT(wrapped(e) == NVQ_BACKEND && g_status == NVQ_BACKEND, "hip error %d reported as %d", (int)e, g_status);
    }
    printf("%ld plans checked, %ld of them split K, %ld failures\n", g_plans, g_split_plans, g_failures);
    return g_failures != 0;
}
