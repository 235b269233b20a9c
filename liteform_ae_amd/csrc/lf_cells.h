// Cells: buckets of a structured matrix (stencil, banded, block-structured) rewritten at plan
// time as groups of up to 16 rows that lie close together in every direction of the
// underlying grid, with the union of their columns.  Host interface between the plan
// (lf_spmm.hip) and the cell code (lf_cells.hip).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

#include "lf_internal.h"

// One rewritten bucket, as the kernel reads it (device pointers).  A cell holds up to 16 rows.
struct LfCellBucket {
    long long n_cells;        // cells, empty ones included
    long long n_tiles;        // workgroups: four cells each
    const int32_t* eoff;      // [n_cells + 1] first merged entry of each cell (multiples of 8)
    const int32_t* ecol;      // [entries] column of each merged entry, ascending inside a cell; a cell's
                              // entries are padded to a multiple of 8 with its last column
    const float4* wq;         // [entries / 4][16] weights: for four consecutive entries and one row of
                              // the cell, the row's values at those columns (0 where it lacks one)
    const int32_t* rows;      // [n_cells * 16] source row of each cell row, -1 where a cell has fewer
    const uint8_t* euse;      // [entries] bit q: one of the cell's rows 4q .. 4q+3 holds the entry's column
};

namespace lf {

constexpr int kCellEntriesCap = 256;   // merged entries of one cell at most

// Tries to rewrite one bucket (ELL rows of `width` slots, one ELL row per source row) as cells.
// *accepted is false when the rows do not share enough columns or the structure does not fit
// the limits; then nothing is kept.  Device memory that the kernel needs goes to `owned`,
// plan-time scratch to `temp` (the caller frees both).  row_bytes: bytes of one row of B (it
// steers the order in which the cells are walked).  Synchronises the stream.
int cells_build(const lf_bucket_desc& b, const int32_t* d_meta, int64_t num_rows, int64_t row_bytes, hipStream_t s,
                std::vector<void*>* owned, std::vector<void*>* temp, LfCellBucket* out, bool* accepted);

// One launch over `n_buckets` rewritten buckets (d_buckets: device array).  fp32 B with 128 or
// 256 features per pass: one 16-byte load per lane, 32 or 64 lanes per row of B.
int cells_launch(const LfCellBucket* d_buckets, int n_buckets, int grid, int b_dtype, const void* B, float* C,
                 int feat, int ldb, int ldc, int accumulate, hipStream_t s);

}  // namespace lf
