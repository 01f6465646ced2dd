// How the products that split K over the grid choose their splits: host arithmetic only (no HIP types), with the
// chip's compute units as a parameter, so that the same rules run in the launchers and in a CPU test of their
// invariants.  A split plan is what the launch, the kernel's indexing and the workspace query must agree on:
//   splits       blocks along the grid axis of K (1: no split, no workspace);
//   per_split    units of K per split, in the kernel's unit (steps of 64 values for the matrix-core kernels, rows of
//                the weight for the vector kernel); split i takes [i * per_split, min((i + 1) * per_split, units));
//   every split has at least one unit: (splits - 1) * per_split < units.
// The float32 partial sums are [batch][splits][m][n] (one batch for the tiled kernel of weights stored [N, K]).
#pragma once

#include <math.h>
#include <stddef.h>
#include <stdint.h>

namespace nvq {
namespace splits {

struct Product {
    int64_t m, n, k, batch;
    bool row_exact;      // every row takes the split of its one-row product
    bool exact_weights;  // the tiled kernel of weights stored [N, K]: the small tile
};

struct Plan {
    int splits;
    int64_t per_split;  // units per split
    int64_t units;      // all units of K
    double estimate_us; // of the kernel with this plan, where the rule estimates one (else 0)
};

inline bool every_split_has_a_unit(const Plan &p) {
    return p.splits >= 1 && p.per_split >= 1 && (int64_t)(p.splits - 1) * p.per_split < p.units &&
           (int64_t)p.splits * p.per_split >= p.units;
}
inline size_t workspace_bytes(const Plan &p, const Product &a) {
    return p.splits > 1 ? (size_t)p.splits * (size_t)a.batch * (size_t)a.m * (size_t)a.n * sizeof(float) : 0;
}

// ── the tiled kernel of weights stored [N, K] (qmm_kernel) ──────────────────────────────────────────────────────────
constexpr int kQmmStep = 64;                     // values of K per step
constexpr int kQmmBigTile = 256, kQmmSmallTile = 128;  // square tiles of y

// Estimated microseconds of `tiles` tiles walking `steps` steps on `cus` compute units, from the kernel's measured
// behaviour: about 1.7 us per step for the big tile (one block per compute unit); the small tile takes 0.8 us per
// step alone on a compute unit and 1.2 us when two share it.
inline double qmm_tiles_us(bool small, double tiles, double steps, int cus) {
    if (!small) return ceil(tiles / cus) * steps * 1.7;
    if (tiles <= cus) return steps * 0.8;
    return ceil(tiles / (2.0 * cus)) * steps * 1.2;
}
inline double qmm_estimate_us(bool small, const Product &a, int cus) {
    const int64_t t = small ? kQmmSmallTile : kQmmBigTile;
    const double tiles = (double)((a.m + t - 1) / t) * (double)((a.n + t - 1) / t) * (double)a.batch;
    return qmm_tiles_us(small, tiles, (double)(a.k / kQmmStep), cus);
}
inline bool qmm_small_tile_is_faster(const Product &a, int cus) {
    return a.exact_weights || qmm_estimate_us(true, a, cus) < qmm_estimate_us(false, a, cus);
}

// The splits fill the chip's block slots with its (few) tiles, and cost a second kernel that reads their float32
// partial sums (about 3 us to launch and 4 bytes per microsecond and compute unit... in all: 4 TB/s).  Each split has
// at least eight steps, in whole table periods (four steps); at most eight splits; a batch is never split.
inline Plan qmm_plan(const Product &a, int cus) {
    const int64_t steps = a.k / kQmmStep;
    const bool small = qmm_small_tile_is_faster(a, cus);
    Plan p{1, steps, steps, qmm_estimate_us(small, a, cus)};
    if (a.batch != 1) return p;
    const int64_t t = small ? kQmmSmallTile : kQmmBigTile;
    const double tiles = (double)(((a.m + t - 1) / t) * ((a.n + t - 1) / t));
    for (int want = 2; want <= 8 && want <= steps / 8; want++) {
        const int64_t per = (((steps + want - 1) / want) + 3) & ~(int64_t)3;  // whole table periods
        const int splits = (int)((steps + per - 1) / per);                    // every split has a step
        if (splits < 2) continue;
        const double reduce_us = 3.0 + ((double)splits * 4.0 + 2.0) * (double)a.m * (double)a.n * 2.0 / 4.0e6;  // written, then read
        const double us = qmm_tiles_us(small, tiles * splits, (double)per, cus) + reduce_us;
        if (us < 0.9 * p.estimate_us) p.estimate_us = us, p.splits = splits, p.per_split = per;
    }
    return p;
}

// ── the matrix-core kernel of weights stored [K, N] (qmn_kernel) ────────────────────────────────────────────────────
constexpr int kQmnStep = 64, kQmnTileCols = 128;
constexpr int kQmnFewRows = 32, kQmnManyRows = 128;          // rows of x per tile
constexpr int kQmnFewBlocksPerCu = 4, kQmnManyBlocksPerCu = 2;

// Splits of K for a product whose tiles do not fill the chip: the split with the least estimated time, counted as
// rounds of resident blocks x (3 us to start + 1.2 us per step of the longest split; 0.64 us per step of the 32-row
// tile) plus, with a split, the reduction: its launch, 0.38 us per split it adds up in turn and its float32 traffic at
// 4 TB/s (fitted to w[4096,4096] at 1 to 32 rows: 43 / 26 / 17 / 13 / 15 / 20 us with 1 / 2 / 4 / 8 / 16 / 32 splits).
inline Plan qmn_plan(const Product &a, int cus, bool few_rows) {
    const int64_t bm = few_rows ? kQmnFewRows : kQmnManyRows;
    const int64_t tiles = ((a.m + bm - 1) / bm) * ((a.n + kQmnTileCols - 1) / kQmnTileCols) * a.batch, steps = a.k / kQmnStep;
    const int64_t resident = (int64_t)(few_rows ? kQmnFewBlocksPerCu : kQmnManyBlocksPerCu) * cus;
    Plan p{1, steps < 1 ? 1 : steps, steps, 0.0};
    if (tiles >= resident || steps < 4) return p;
    const double step_us = few_rows ? 0.64 : 1.2;
    for (int64_t splits = 1; splits <= steps / 2 && splits <= 64; splits++) {
        const int64_t per_split = (steps + splits - 1) / splits;
        if ((steps + per_split - 1) / per_split != splits) continue;  // (another count gives the same longest split)
        const int64_t rounds = (tiles * splits + resident - 1) / resident;
        double us = (double)rounds * (3.0 + step_us * (double)per_split);
        if (splits > 1) us += 2.0 + 0.38 * (double)splits + (double)splits * (double)(a.batch * a.m * a.n) * 4.0 / 4.0e6;
        if (splits == 1 || us < p.estimate_us) p.estimate_us = us, p.splits = (int)splits, p.per_split = per_split;
    }
    return p;
}

// ── the vector kernel of weights stored [K, N] (qvm_kernel) ─────────────────────────────────────────────────────────
constexpr int kQvmWaves = 8, kQvmTileCols = 2048;

// About a block (of eight wavefronts) per compute unit, at least 16 rows of w per wavefront, at most 32 splits (the
// reduction kernel adds them one after the other).  The unit is a row of the weight.
inline Plan qvm_plan(const Product &a, int cus) {
    const int rm = a.m == 1 ? 1 : 4;
    // row-exact: the split is the one-row product's, whatever the rows and batches, so that every row keeps its bits
    const int64_t base = ((a.n + kQvmTileCols - 1) / kQvmTileCols) * (a.row_exact ? 1 : a.batch * ((a.m + rm - 1) / rm));
    const int64_t want = ((int64_t)cus + base - 1) / base;
    const int64_t most = a.k / (16 * kQvmWaves) > 1 ? a.k / (16 * kQvmWaves) : 1;
    int64_t splits = want < 1 ? 1 : (want > most ? most : want);
    if (splits > 32) splits = 32;
    int64_t per = (a.k + splits - 1) / splits;
    if (per < 1) per = 1;
    splits = (a.k + per - 1) / per;  // the count that this longest split gives: no split is left without a row
    if (splits < 1) splits = 1;
    return Plan{(int)splits, per, a.k, 0.0};
}

}  // namespace splits
}  // namespace nvq
