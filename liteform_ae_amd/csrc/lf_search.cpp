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

// Cost of a state for the gfx950 kernels, in bytes of HBM-traffic equivalent.  The B gather
// (nnz * feat * sizeof(B)) and the C store are the same for every state of the fold chain, so
// only what a fold changes is priced:
//   * 8 bytes per slab slot (column + value are streamed once, padding included);
//   * kRowBytes per ELL row: 8 bytes of row id + meta, and the fixed work of starting a row
//     (descriptor reads, loop set-up, a sub-wave slot left idle on continuation rows).
// kRowBytes was fitted on MI355X: on the 2.45M-row power-law graph at N = 128 every extra
// million ELL rows costs 0.07-0.2 ms at ~6 TB/s, i.e. 400-1200 bytes each, while padded slots
// cost no more than their slab bytes because a padded slot re-reads a row that is already
// in flight.  With these weights a fold pays only when it removes far more padding than it
// adds rows, which on the benchmark workloads keeps the initial power-of-two widths.
constexpr double kSlotBytes = 8.0;
constexpr double kRowBytes = 600.0;

double gfx950_cost(const Pool& pool, const int64_t* hist, int nmask, int32_t feat, int32_t parts) {
    (void)hist;
    (void)nmask;
    (void)feat;
    (void)parts;
    double cost = 0.0;
    for (const Bucket& b : pool.items)
        cost += kSlotBytes * (double)b.num_rows * (double)b.width + kRowBytes * (double)b.num_rows;
    return cost;
}

double state_cost(int model, const Pool& pool, const int64_t* hist, int nmask, int32_t feat, int32_t parts) {
    return model == LF_COST_GFX950 ? gfx950_cost(pool, hist, nmask, feat, parts)
                                   : reference_cost(pool, hist, nmask, feat, parts);
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
        double best_cost = state_cost(cost_model, pool, hist, nmask, cfg_feat_size, cfg_num_parts);
        std::vector<int32_t> best = pool.sorted_widths();
        if (trace) trace[ntrace] = best_cost;
        ++ntrace;
        int32_t pre = pool.max_width();
        int32_t neww = pre / 2;
        while (neww >= 1) {
            move_largest_bucket(pool, pre, neww);
            const double c = state_cost(cost_model, pool, hist, nmask, cfg_feat_size, cfg_num_parts);
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
