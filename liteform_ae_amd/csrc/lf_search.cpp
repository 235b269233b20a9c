// Host-side bucket-width search.
//
// Works on the per-class statistics produced by lf_bucket_stats and mirrors the
// reference's search state by state: modify_single_row_buckets (format_algos.py:928-954),
// move_width_one_bucket (903-923), move_largest_bucket (623-648), get_memory_cost
// (1035-1166), modify_bucket_widths (709-774), get_bucket_config (777-816).
//
// The reference keeps each partition's buckets in a Python dict whose iteration order is
// insertion order; the cost is a floating-point sum over that order, so the order is part
// of the result.  `Pool` below is that dict: a vector in insertion order, erase on delete,
// push_back on insert.  Column sets are not materialised: a bucket remembers which initial
// width classes were merged into it (a bitmask) and the size of its column set is read off
// the per-partition histogram of column class-masks.
//
// This file must be compiled without floating-point contraction (-ffp-contract=off) so the
// double arithmetic matches CPython's operation by operation.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#include "lf_internal.h"

namespace {

struct Bucket {
    int32_t width;
    int64_t num_rows;   // cost-model rows
    int64_t nnz;
    int64_t out_rows;   // len(row_indices)
    uint32_t classes;   // initial width classes merged into this bucket
};

struct Pool {
    std::vector<Bucket> items;  // insertion order

    Bucket* find(int32_t width) {
        for (auto& b : items)
            if (b.width == width) return &b;
        return nullptr;
    }
    void erase(int32_t width) {
        for (size_t i = 0; i < items.size(); ++i)
            if (items[i].width == width) {
                items.erase(items.begin() + i);
                return;
            }
    }
    int32_t max_width() const {
        int32_t m = 0;
        for (auto& b : items) m = std::max(m, b.width);
        return m;
    }
    std::vector<int32_t> sorted_widths() const {
        std::vector<int32_t> w;
        for (auto& b : items) w.push_back(b.width);
        std::sort(w.begin(), w.end());
        return w;
    }
};

// format_algos.py:623-648
void move_largest_bucket(Pool& pool, int32_t pre, int32_t neww) {
    Bucket src = *pool.find(pre);
    const int64_t moved = src.num_rows * (int64_t)(pre / neww);
    if (Bucket* dst = pool.find(neww)) {
        dst->num_rows += moved;
        dst->nnz += src.nnz;
        dst->out_rows += src.out_rows;
        dst->classes |= src.classes;
    } else {
        pool.items.push_back(Bucket{neww, moved, src.nnz, src.out_rows, src.classes});
    }
    pool.erase(pre);
}

int64_t column_set_size(const int64_t* hist, int nmask, uint32_t classes) {
    int64_t n = 0;
    for (int m = 1; m < nmask; ++m)
        if ((uint32_t)m & classes) n += hist[m];
    return n;
}

// format_algos.py:1035-1166, value of return_dict["cost"]
double reference_cost(const Pool& pool, const int64_t* hist, int nmask, int32_t feat, int32_t parts) {
    const int32_t max_w = pool.max_width();
    double cost = 0.0;
    for (const Bucket& b : pool.items) {
        const int64_t block = max_w / b.width;
        const int64_t padded = (b.num_rows + block - 1) / block * block;
        const int64_t c1 = 2 * padded * b.width;
        const int64_t c2 = column_set_size(hist, nmask, b.classes) * feat;
        const bool atomic = parts > 1 || b.width == max_w;
        double c3;
        if (atomic) {
            const double weight = (double)padded / (double)b.out_rows;
            c3 = weight * (double)b.out_rows;
            c3 = c3 * (double)feat;
        } else {
            c3 = (double)(b.out_rows * feat);
        }
        const double bucket_cost = (double)(c1 + c2) + c3;
        cost = cost + bucket_cost;
    }
    return cost;
}

// ---------------------------------------------------------------------------------------
// gfx950 model.  All constants below were measured on MI355X with this library's kernels
// (2.45M-row power-law graph, 500k x 2M skewed matrix, uniform-degree matrices of 17 / 33 /
// 130 / 520 entries per row; N = 32 .. 512, 1-4 column partitions, 1-8 feature windows).
//
// Fold chain.  The kernels walk only the valid slots of an ELL row (rounded up to the unroll
// of eight), so padding costs no gathers; what a state changes is
//   * the slots that are read and staged through LDS whole, padding included (buckets of up
//     to 64 slots; wider rows are streamed and only their valid slots are touched):
//     8 bytes per slot at the fabric rate plus kStagedSlotPs;
//   * the number of ELL rows - row id and meta, loop set-up, one store (or partial sum) per
//     row: row_ps(N) per row, dearer at small N where many short rows share a wavefront.
// A class folded into a narrower bucket takes ceil(average fill / width) ELL rows per source
// row.  Measured against this model: folding never gains more than 3 % (33 entries per row,
// N = 128: widths [16] 2.32 ms against [64] 2.38 ms, which the model reproduces), and the
// power-law and skewed benchmark matrices keep their initial power-of-two widths.
constexpr double kFabricBytesPerPs = 7.493;       // 7.49 TB/s: what the fabric moves at best
constexpr double kStagedSlotPs = 6.7;
constexpr int kStagedWidthMax = 64;

double row_ps(int feat) {
    if (feat <= 32) return 230.0;
    if (feat <= 64) return 70.0;
    if (feat <= 128) return 40.0;
    if (feat <= 256) return 60.0;
    return 90.0;
}

// st: this partition's initial statistics [LF_MAX_CLASSES][LF_STATS_FIELDS]
double gfx950_cost(const Pool& pool, const int64_t* st, int32_t feat) {
    double ps = 0.0;
    for (const Bucket& b : pool.items) {
        for (int k = 0; k < LF_MAX_CLASSES; ++k) {
            if (!(b.classes >> k & 1u)) continue;
            const double rows = (double)st[(size_t)k * LF_STATS_FIELDS + 2];
            const double nnz = (double)st[(size_t)k * LF_STATS_FIELDS + 1];
            if (rows <= 0) continue;
            const double per_row = std::ceil(nnz / rows / (double)b.width);
            const double ell = rows * std::max(1.0, per_row);
            const double slots = ell * (double)b.width;
            ps += ell * row_ps(feat);
            // wider rows are streamed: only their valid slots are read, the same in every state
            if (b.width <= kStagedWidthMax) ps += slots * (kStagedSlotPs + 8.0 / kFabricBytesPerPs);
        }
    }
    return ps;
}

double state_cost(int model, const Pool& pool, const int64_t* hist, int nmask, const int64_t* st, int32_t feat,
                  int32_t parts) {
    return model == LF_COST_GFX950 ? gfx950_cost(pool, st, feat) : reference_cost(pool, hist, nmask, feat, parts);
}

}  // namespace

extern "C" int lf_search_bucket_config(const int64_t* h_stats, const int64_t* h_colhist,
                                       int32_t num_parts, int32_t width_limit, int32_t cfg_feat_size,
                                       int32_t cfg_num_parts, int32_t cost_model, int32_t* h_widths,
                                       int32_t* h_nwidths, double* h_trace_cost, int32_t* h_trace_len) {
    LF_REQUIRE(h_stats && h_widths && h_nwidths, LF_ERR_INVALID, "null argument");
    LF_REQUIRE(h_colhist || cost_model == LF_COST_GFX950, LF_ERR_INVALID,
               "the reference cost model needs the column histogram (null argument)");
    LF_REQUIRE(num_parts >= 1, LF_ERR_INVALID, "num_parts must be >= 1 (got %d)", num_parts);
    LF_REQUIRE(lf::is_pow2(width_limit) && width_limit <= (1 << (LF_MAX_CLASSES - 1)), LF_ERR_INVALID,
               "width_limit must be a power of two <= %d (got %d)", 1 << (LF_MAX_CLASSES - 1), width_limit);
    LF_REQUIRE(cost_model == LF_COST_REFERENCE || cost_model == LF_COST_GFX950, LF_ERR_INVALID,
               "unknown cost model %d", cost_model);
    const int nclass = lf::ilog2(width_limit) + 1;
    const int nmask = 1 << LF_MAX_CLASSES;

    for (int p = 0; p < num_parts; ++p) {
        const int64_t* st = h_stats + (size_t)p * LF_MAX_CLASSES * LF_STATS_FIELDS;
        const int64_t* hist = h_colhist ? h_colhist + (size_t)p * nmask : nullptr;
        int32_t* out_w = h_widths + (size_t)p * LF_MAX_CLASSES;
        double* trace = h_trace_cost ? h_trace_cost + (size_t)p * (LF_MAX_CLASSES + 1) : nullptr;
        int ntrace = 0;

        // get_init_buckets' result for this partition: keys ascending (format_algos.py:897)
        Pool pool;
        for (int k = 0; k < nclass; ++k) {
            const int64_t* f = st + (size_t)k * LF_STATS_FIELDS;
            if (f[2] > 0) pool.items.push_back(Bucket{1 << k, f[0], f[1], f[2], 1u << k});
        }
        if (pool.items.empty()) {  // format_algos.py:796-799
            h_nwidths[p] = 0;
            if (h_trace_len) h_trace_len[p] = 0;
            continue;
        }

        // modify_single_row_buckets: key snapshot, widest first (format_algos.py:940-953)
        std::vector<int32_t> snapshot = pool.sorted_widths();
        std::reverse(snapshot.begin(), snapshot.end());
        for (int32_t width : snapshot) {
            Bucket* b = pool.find(width);
            if (!b || b->num_rows != 1) continue;
            if (width == 1) {
                // move_width_one_bucket (format_algos.py:914-923): the target is looked up in
                // the snapshot, which may name a width that was folded away already
                const int32_t max_width = snapshot.front();
                int32_t target = 2;
                while (target <= max_width &&
                       std::find(snapshot.begin(), snapshot.end(), target) == snapshot.end())
                    target *= 2;
                if (target > max_width)
                    return lf::fail(LF_ERR_TOO_SMALL,
                                    "The partition is too small, only having 1 non-zero element.");
                move_largest_bucket(pool, 1, target);
            } else {
                move_largest_bucket(pool, width, width / 2);
            }
        }

        // modify_bucket_widths (format_algos.py:727-774)
        double best_cost = state_cost(cost_model, pool, hist, nmask, st, cfg_feat_size, cfg_num_parts);
        std::vector<int32_t> best = pool.sorted_widths();
        if (trace) trace[ntrace] = best_cost;
        ++ntrace;
        int32_t pre = pool.max_width();
        int32_t neww = pre / 2;
        while (neww >= 1) {
            move_largest_bucket(pool, pre, neww);
            const double c = state_cost(cost_model, pool, hist, nmask, st, cfg_feat_size, cfg_num_parts);
            if (trace) trace[ntrace] = c;
            ++ntrace;
            if (c < best_cost) {
                best = pool.sorted_widths();
                best_cost = c;
            }
            pre = neww;
            neww /= 2;
        }
        h_nwidths[p] = (int32_t)best.size();
        for (size_t i = 0; i < best.size(); ++i) out_w[i] = best[i];
        if (h_trace_len) h_trace_len[p] = ntrace;
    }
    return LF_OK;
}

// ---------------------------------------------------------------------------------------
// Launch shape.  Predicted time of one product with `num_parts` column partitions and
// `n_windows` feature windows, from the partitions' bucket statistics alone.
//
// One launch (one partition, one window of n = feat / windows features) moves
//   gathers  nnz_p rows of g = n * sizeof(B) bytes each,
//   C        rows * n * 4 bytes written by partition 0, 8 bytes per feature and touched row
//            (read-modify-write) by every later partition,
//   slabs    8 bytes per slot and per ELL row.
// The part of B that one launch can touch is slice = (columns of the partition) * g bytes.
// Three levels serve the gathers:
//   * each XCD's 4 MB L2 holds a share h2 = kL2Share * 4 MB / slice of the slice (at most 1),
//     less the first touches, which every one of the eight L2s has to make itself
//     (8 / uses per row of B); hits never leave the XCD and cost bytes / kL2BytesPerPs;
//   * what misses crosses the fabric, which moves kFabricBytesPerPs at best;
//   * the 256 MB memory-side cache serves a share h = kMallShare * 256 MB / slice of that (at
//     most 1, less the first touches); the rest comes from HBM as scattered rows at
//     kHbmBytesPerPs.
// The launch takes the time of its L2 hits plus the longer of the fabric and the HBM time of
// everything else, times a penalty when a window reads 256 bytes or less out of a wider row
// (partial rows use HBM worse: x (1 + beta * log2(row bytes / g)^2), scaled by the share that
// no cache serves), plus a fixed cost: kLaunchMs for the first launch of a product,
// kNextLaunchMs for every further one.
//
// kFabricBytesPerPs .. kNotLastPartition were fitted on 150 measured shapes of matrices whose
// rows hold 4 - 33 entries on average (1 - 4 partitions); the L2 terms and the split launch cost
// on 198 shapes of three graphs with 28 - 490 entries per row and 1 - 32 partitions, for which
// the model without an L2 level picked one partition and lost 40 - 80 % against the fastest
// measured shape.  On three further matrices measured after that fit and never fitted to (195
// shapes) the pick is 8 % slower than the fastest measured shape on average, 17 % at worst:
// the model finds the regime (how many partitions make the slice fit an L2) but not always the
// best neighbour.  tests/golden/launch_shape_measurements.json holds the three sets.
constexpr double kHbmBytesPerPs = 5.528;
constexpr double kMallShare = 0.5534;
constexpr double kMallBytes = 256.0 * 1048576.0;
constexpr double kL2BytesPerPs = 28.0;
constexpr double kL2Share = 1.1;
constexpr double kL2Bytes = 4.0 * 1048576.0;
constexpr double kXcdCount = 8.0;
constexpr double kBeta256 = 0.02, kBeta128 = 0.04, kSmallGather = 1.053;
constexpr double kLaunchMs = 0.029, kNextLaunchMs = 0.012;
// A partition whose rows of C a later one adds to cannot stream its stores past the caches, and
// what it leaves there takes room from B (fitted: with it the model's pick is within 2.1 % of the
// fastest measured shape in every group, without it 3.3 % off for the 2.45M-row graph at N = 256).
constexpr double kNotLastPartition = 1.07;

extern "C" int lf_model_spmm_ms(const int64_t* h_stats, int32_t num_parts, int32_t n_windows, int64_t num_rows,
                                int64_t num_cols, int32_t feat_size, int32_t b_dtype, double* h_ms) {
    LF_REQUIRE(h_stats && h_ms, LF_ERR_INVALID, "null argument");
    LF_REQUIRE(num_parts >= 1 && n_windows >= 1 && num_rows >= 0 && num_cols >= 1, LF_ERR_INVALID, "bad shape");
    LF_REQUIRE(feat_size >= 1 && feat_size % n_windows == 0, LF_ERR_INVALID,
               "feat_size %d is not a multiple of %d windows", feat_size, n_windows);
    LF_REQUIRE(b_dtype == LF_DTYPE_F32 || b_dtype == LF_DTYPE_BF16, LF_ERR_INVALID, "unknown B dtype %d", b_dtype);
    const double elem = b_dtype == LF_DTYPE_BF16 ? 2.0 : 4.0;
    const double n = (double)feat_size / n_windows;
    const double g = n * elem, row_bytes = (double)feat_size * elem;
    const double lg = std::log2(row_bytes / g);
    const double beta = g < 256.0 ? kBeta128 : (g < 512.0 ? kBeta256 : 0.0);
    const double penalty = (1.0 + beta * lg * lg) * (g < 256.0 ? kSmallGather : 1.0);
    const double cols_p = (double)num_cols / num_parts;
    double ms = 0.0;
    for (int p = 0; p < num_parts; ++p) {
        const int64_t* st = h_stats + (size_t)p * LF_MAX_CLASSES * LF_STATS_FIELDS;
        double ell = 0, slots = 0, nnz = 0, touched = 0;
        for (int k = 0; k < LF_MAX_CLASSES; ++k) {
            const double cost_rows = (double)st[k * LF_STATS_FIELDS], distinct = (double)st[k * LF_STATS_FIELDS + 2];
            const double e = k + 1 < LF_MAX_CLASSES ? distinct : std::max(cost_rows, distinct);
            ell += e;
            slots += e * (double)(1 << k);
            nnz += (double)st[k * LF_STATS_FIELDS + 1];
            touched += distinct;
        }
        const double slice = cols_p * g;
        const double first = std::min(1.0, cols_p / std::max(nnz, 1.0));
        const double first_l2 = std::min(1.0, kXcdCount * cols_p / std::max(nnz, 1.0));
        const double h = std::min(1.0, kMallShare * kMallBytes / slice) * (1.0 - first);
        const double h2 = std::min(1.0, kL2Share * kL2Bytes / slice) * (1.0 - first_l2);
        const double cached = std::max(h, h2);
        const double pen = 1.0 + (penalty - 1.0) * (1.0 - cached);
        const double gather = nnz * g;
        const double other = (p == 0 ? (double)num_rows * n * 4.0 : touched * n * 8.0) + slots * 8.0 + ell * 8.0;
        const double l2_ps = h2 * gather / kL2BytesPerPs;
        const double fabric_ps = ((1.0 - h2) * gather + other) * pen / kFabricBytesPerPs;
        const double hbm_ps = ((1.0 - cached) * gather + other) * pen / kHbmBytesPerPs;
        ms += (l2_ps + std::max(fabric_ps, hbm_ps)) * 1e-9 * (p + 1 < num_parts ? kNotLastPartition : 1.0) + kNextLaunchMs;
    }
    *h_ms = ms * n_windows + (kLaunchMs - kNextLaunchMs);
    return LF_OK;
}
