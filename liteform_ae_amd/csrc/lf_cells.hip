// Cells: shared gathers for structured matrices on gfx950.
//
// In a stencil, banded or block-structured matrix the rows that are close together in the
// underlying grid hold mostly the same columns.  The reference's kernel reads a row of B once
// per stored entry whatever the structure (playground_pipline/format_algos.py:99-102 under the
// schedule of 508-533).  Here a bucket of such rows is rewritten at plan time as cells: up to
// 16 rows that are neighbours in up to three directions (consecutive rows, rows one grid line
// apart, rows one grid plane apart), with the union of their columns ("merged entries") and,
// per merged entry, one weight per row of the cell (0 where the row lacks the column).  One
// 64-lane wavefront owns a cell: it reads each row of B of the union once (16 bytes per lane)
// and adds weight x row to the accumulator rows that hold the column.  A 2 x 2 x 4 cell of a
// 27-point stencil reads 96 rows of B for 16 output rows, 6 per row, where row by row it would
// read 27 and four consecutive rows at a time 13.5.
//
// The update "rows += weights (x) one row of B" is a rank-1 update, and the matrix pipe has
// instructions for exactly that.  Written with vector FMAs a cell takes 18 FMAs and ~30 scalar
// mask tests per merged entry, and rocprofv3 counters showed the kernel bound by instruction
// issue (one instruction per ~4.7 cycles and SIMD, 0.88 ms for the 100^3 stencil at N = 256,
// 0.79 ms with the gathers taken out).  v_mfma_f32_16x16x1_4b_f32 - four 16 x 16 outer
// products per issue, all 16 rows at once - brought that to 0.645 ms with the matrix pipe busy
// 54 % of the time, most of it on zeros: a 27-point stencil fills 432 of a cell's 96 x 16
// weights.  The kernel now uses v_mfma_f32_4x4x1_16b_f32 - sixteen 4 x 4 outer products per
// issue, i.e. four rows x 64 lanes, a quarter of the pipe time - once per quarter of the cell
// (four rows that follow each other) that holds the column, and skips the quarters that do
// not: 192 of 384 (entry, quarter) pairs for the stencil, 0.63 ms with the same cells, 0.604
// with cells whose quarters are 2 x 2 x 1.  This is not a GEMM formulation: data layout,
// gathers and accumulation order are the plain path's, only the accumulate instruction
// differs, and a row that lacks a column its quarter holds adds 0 * B (as padded slots do).
//
// Which rows are neighbours is found from the matrix itself: in a sample of rows, the most
// frequent differences between two columns of one row are the row distances at which rows
// share columns (1, 100 and 10000 for a 27-point stencil on a 100^3 grid).  Rows are binned
// into cells by their coordinates along those strides; the rewrite is kept only when the
// cells' unions are at most 70 % of the gathers the plain path would issue.
//
// A row's terms are added in ascending column order, as in the plain path.
#include "lf_cells.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "lf_spmm_device.h"

namespace {

constexpr int kCellRows = 16;              // rows of a cell: the row dimension of the outer-product instruction
constexpr int kCellQuarters = kCellRows / 4;   // groups of four rows: the row dimension of the 4 x 4 outer-product instruction
constexpr int kCellBatch = 8;              // merged entries are padded to whole batches of this many
constexpr int kCellTileCells = 4;          // cells a workgroup is on at a time: one per wavefront (one or two
                                           // per workgroup measured 2 % slower)
#ifndef LF_CELLS_PER_WAVE
#define LF_CELLS_PER_WAVE 1
#endif
constexpr int kCellsPerWave = LF_CELLS_PER_WAVE;   // cells a wavefront walks one after the other (<= 15)
constexpr int kCellWidthMax = 64;          // widest bucket that is looked at
constexpr int kCellSampleRows = 64;        // rows looked at to find the strides
constexpr int kCellSampleCols = 32;        // ... and how many of each row's columns
constexpr int kCellMaxPercent = 70;        // merged entries / plain gathers at most, in percent
constexpr long long kL2BytesPerXcd = 4ll << 20;

// Where a row lies along the strides: cell = ((z / g2) * n1 + y / g1) * n0 + x / g0 with
// x = (r mod s2) / s1, y = (r mod s3) / s2, z = r / s3 (fewer terms with fewer strides).
struct CellGeom {
    int k;                     // strides in use: 1..3
    int g0, g1, g2;            // rows of a cell along each stride
    long long s1, s2, s3;
    long long n0, n1, n2;      // cells along x, y and z
    int yb;                    // three strides: cell rows along y that are swept through all z before the next ones
};

__device__ __forceinline__ long long cell_of(const CellGeom& q, long long r) {
    long long x, y = 0, z = 0;
    if (q.k == 1) {
        x = r / q.s1;
    } else if (q.k == 2) {
        x = (r % q.s2) / q.s1;
        y = r / q.s2;
    } else {
        x = (r % q.s2) / q.s1;
        y = (r % q.s3) / q.s2;
        z = r / q.s3;
    }
    const long long xc = x / q.g0, yc = y / q.g1, zc = z / q.g2;
    if (q.k == 3 && q.yb > 0) return (((yc / q.yb) * q.n2 + zc) * q.yb + yc % q.yb) * q.n0 + xc;
    return (zc * q.n1 + yc) * q.n0 + xc;
}

// sample[i] = {source row, valid slots, columns...} of every stride-th ELL row
__global__ void cell_sample_kernel(const int32_t* __restrict__ rows, const int32_t* __restrict__ cols,
                                   const int32_t* __restrict__ meta, long long n_rows, int log_w,
                                   long long stride, int n_samples, int n_cols, int32_t* __restrict__ out) {
    const int i = blockIdx.x;
    if (i >= n_samples) return;
    const long long e = (long long)i * stride;
    if (e >= n_rows) return;
    int32_t* o = out + (size_t)i * (n_cols + 2);
    const int len = meta[e] & (int)kMetaLenMask;
    if (threadIdx.x == 0) {
        o[0] = rows[e];
        o[1] = len;
    }
    for (int j = threadIdx.x; j < n_cols; j += blockDim.x) o[2 + j] = j < len ? cols[(e << log_w) + j] : -1;
}

// perm[cell * G + i] = the i-th ELL row that falls into the cell, in arrival order (the merge
// pass sorts them); flags[0] is raised when a cell receives more than G rows.
__global__ void __launch_bounds__(256)
cell_assign_kernel(const int32_t* __restrict__ rows, long long n_rows, CellGeom q, int G,
                   int32_t* __restrict__ cnt, int32_t* __restrict__ perm, int* __restrict__ flags) {
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n_rows) return;
    const long long c = cell_of(q, rows[e]);
    const int pos = atomicAdd(&cnt[c], 1);
    if (pos < G) perm[c * G + pos] = (int32_t)e;
    else flags[0] = 1;
}

// ascending sort inside every group of 16 lanes
__device__ __forceinline__ unsigned group16_sort_ascending(unsigned v, int lane) {
    for (int k = 2; k <= 16; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            const unsigned o = __shfl_xor(v, j);
            const bool up = (lane & k) == 0 || k == 16;
            const bool lower = (lane & j) == 0;
            v = (lower == up) ? min(v, o) : max(v, o);
        }
    return v;
}

struct CellMergeArgs {
    const int32_t* rows;       // the bucket's slab
    const int32_t* cols;
    const float* vals;
    const int32_t* meta;
    int log_w;
    long long n_cells;
    const int32_t* perm;       // [n_cells * 16] ELL rows of each cell in arrival order, -1 = none
    // counting pass
    int32_t* m_out;            // [n_cells] merged entries, rounded up to whole batches
    int32_t* cnt_out;          // [n_cells] merged entries, not rounded
    int32_t* plain_out;        // [n_cells] gathers of the plain path for the same rows
    // writing pass (ecol != nullptr)
    const int32_t* eoff;
    int32_t* ecol;
    float* wq;                 // float4 per (four consecutive entries, row): [entry / 4][16][entry % 4]
    int32_t* rows_out;         // [n_cells * 16]
    uint8_t* euse;             // [entries] which quarters of the cell (rows 4q .. 4q+3) hold the entry's column
};

// Four cells per 64-thread workgroup, one lane per row of a cell.  The rows' slots are staged
// in LDS; then the 16 (ascending) column lists of a cell are merged step by step: the smallest
// head column is the next merged entry, every row that holds it supplies its value and moves
// on, the others supply 0.  The counting pass only counts the steps; the writing pass stores
// columns and weights, and pads each cell to whole batches with its last column and zero
// weights.  No atomics on the output, so the cells do not depend on scheduling.
__global__ void __launch_bounds__(64)
cell_merge_kernel(CellMergeArgs a) {
    constexpr int G = kCellRows;
    // 64 rows of w slots: columns, and in the writing pass values behind them.  Sized by the
    // launch for the bucket's width and the pass: a single-wavefront workgroup with room for
    // the widest bucket (32 KB) left five wavefronts to a CU, and the step-by-step merge is
    // all latency (1M-row stencil: 0.83 ms per pass that way).
    extern __shared__ int32_t s_dyn[];
    const int lane = threadIdx.x, r = lane & 15;
    const long long cell = (long long)blockIdx.x * 4 + (lane >> 4);
    const bool live = cell < a.n_cells;
    const bool write = a.ecol != nullptr;
    const int w = 1 << a.log_w;
    // a lane's row sits at an odd stride: the merge reads s_c[lane * ws + pos] with pos much the
    // same in all lanes, which at stride w lands 32 lanes on one bank
    const int ws = w + 1;
    int32_t* s_c = s_dyn;
    float* s_v = reinterpret_cast<float*>(s_dyn + 64 * ws);

    unsigned e = 0x7FFFFFFFu;
    if (live) {
        const int32_t p = a.perm[cell * G + r];
        if (p >= 0) e = (unsigned)p;
    }
    e = group16_sort_ascending(e, lane);           // ELL rows ascend with the source rows
    const bool have = e != 0x7FFFFFFFu;
    if (write && live) a.rows_out[cell * G + r] = have ? a.rows[e] : -1;
    const int len = have ? (a.meta[e] & (int)kMetaLenMask) : 0;
    // every lane stages its own row, all loads in flight at once (slabs are 16-byte aligned, w >= 8)
    if (have) {
        const int4* src_c = reinterpret_cast<const int4*>(a.cols + ((long long)e << a.log_w));
        const float4* src_v = reinterpret_cast<const float4*>(a.vals + ((long long)e << a.log_w));
#pragma unroll 4
        for (int j = 0; j < len; j += 4) {
            const int4 c4 = src_c[j >> 2];
            int32_t* d = s_c + lane * ws + j;
            d[0] = c4.x; d[1] = c4.y; d[2] = c4.z; d[3] = c4.w;
            if (write) {
                const float4 v4 = src_v[j >> 2];
                float* dv = s_v + lane * ws + j;
                dv[0] = v4.x; dv[1] = v4.y; dv[2] = v4.z; dv[3] = v4.w;
            }
        }
    }
    __syncthreads();
    int plain = (len + kUnroll - 1) / kUnroll * kUnroll;
    for (int d = 8; d > 0; d >>= 1) plain += __shfl_xor(plain, d);
    const int eo = (write && live) ? a.eoff[cell] : 0;
    const int m8 = (write && live) ? a.eoff[cell + 1] - eo : 0;
    int pos = 0, cnt = 0, last_col = 0;
    int head = pos < len ? s_c[lane * ws] : 0x7FFFFFFF;
    float4* wq4 = reinterpret_cast<float4*>(a.wq);
    float pend[4] = {0.f, 0.f, 0.f, 0.f};          // this row's weights of the four entries being filled
    for (;;) {
        int cmin = head;
        for (int d = 8; d > 0; d >>= 1) cmin = min(cmin, __shfl_xor(cmin, d));
        const bool any = cmin != 0x7FFFFFFF;       // this group still has columns
        if (__ballot(any) == 0) break;
        const bool mine = any && head == cmin;
        const unsigned long long holders = __ballot(mine);
        if (write && any) {
            const float v = mine ? s_v[lane * ws + pos] : 0.f;
            pend[0] = (cnt & 3) == 0 ? v : pend[0];
            pend[1] = (cnt & 3) == 1 ? v : pend[1];
            pend[2] = (cnt & 3) == 2 ? v : pend[2];
            pend[3] = (cnt & 3) == 3 ? v : pend[3];
            if ((cnt & 3) == 3) wq4[(size_t)((eo + cnt) >> 2) * G + r] = make_float4(pend[0], pend[1], pend[2], pend[3]);
            if (r == 0) {
                a.ecol[eo + cnt] = cmin;
                const unsigned h16 = (unsigned)(holders >> (lane & 48)) & 0xFFFFu;
                a.euse[eo + cnt] = (uint8_t)(((h16 & 0x000Fu) ? 1 : 0) | ((h16 & 0x00F0u) ? 2 : 0) | ((h16 & 0x0F00u) ? 4 : 0) |
                                             ((h16 & 0xF000u) ? 8 : 0));
            }
        }
        if (mine) {
            ++pos;
            head = pos < len ? s_c[lane * ws + pos] : 0x7FFFFFFF;
        }
        if (any) {
            ++cnt;
            last_col = cmin;
        }
    }
    if (!live) return;
    if (!write) {
        if (r == 0) {
            const int rounded = (cnt + kCellBatch - 1) / kCellBatch * kCellBatch;
            a.m_out[cell] = rounded;
            a.cnt_out[cell] = cnt;
            a.plain_out[cell] = cnt > 0 ? plain : 0;
        }
        return;
    }
    for (int i = cnt; i < m8; ++i) {               // padding entries: the last column again, weight 0
        pend[i & 3] = 0.f;
        if ((i & 3) == 3) wq4[(size_t)((eo + i) >> 2) * G + r] = make_float4(pend[0], pend[1], pend[2], pend[3]);
        if (r == 0) {
            a.ecol[eo + i] = last_col;
            a.euse[eo + i] = 0;
        }
    }
}

// stats[0] merged entries (not rounded), [1] gathers of the plain path, [2] rounded entries,
// [3] most rounded entries of a cell.  (One atomic per workgroup: with one per cell in the merge
// kernel, 250,000 atomics on four addresses made the counting pass of a 1M-row stencil take
// 0.8 ms instead of 0.3.)
__global__ void __launch_bounds__(256)
cell_stats_kernel(const int32_t* __restrict__ cnt, const int32_t* __restrict__ plain, const int32_t* __restrict__ rounded,
                  long long n_cells, unsigned long long* __restrict__ stats) {
    __shared__ unsigned long long s_red[4][4];
    unsigned long long v[4] = {0, 0, 0, 0};
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n_cells; i += (long long)gridDim.x * blockDim.x) {
        v[0] += (unsigned long long)cnt[i];
        v[1] += (unsigned long long)plain[i];
        v[2] += (unsigned long long)rounded[i];
        v[3] = max(v[3], (unsigned long long)rounded[i]);
    }
    for (int d = 32; d > 0; d >>= 1) {
        v[0] += __shfl_xor(v[0], d);
        v[1] += __shfl_xor(v[1], d);
        v[2] += __shfl_xor(v[2], d);
        v[3] = max(v[3], __shfl_xor(v[3], d));
    }
    if ((threadIdx.x & 63) == 0)
        for (int k = 0; k < 4; ++k) s_red[k][threadIdx.x >> 6] = v[k];
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < 4; ++wv) {
            v[0] += s_red[0][wv];
            v[1] += s_red[1][wv];
            v[2] += s_red[2][wv];
            v[3] = max(v[3], s_red[3][wv]);
        }
        atomicAdd(&stats[0], v[0]);
        atomicAdd(&stats[1], v[1]);
        atomicAdd(&stats[2], v[2]);
        atomicMax(&stats[3], v[3]);
    }
}

// dynamic LDS of one cell_merge_kernel workgroup
size_t merge_lds(const CellMergeArgs& a) { return (size_t)64 * 4 * (((size_t)1 << a.log_w) + 1) * (a.ecol ? 2 : 1); }

__global__ void fill_i32_kernel(int32_t* __restrict__ p, long long n, int32_t value) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        p[i] = value;
}

typedef float floatx16 __attribute__((ext_vector_type(16)));
// read-only plan data addressed through the constant address space: loads at wavefront-uniform
// addresses then go through the scalar cache and are counted apart from the vector loads
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef const f32x4 __attribute__((address_space(1)))* GlobalFloat4Ptr;
typedef const i32x4 __attribute__((address_space(1)))* GlobalInt4Ptr;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1)))* GlobalU32x4Ptr;
typedef const uint32_t __attribute__((address_space(1)))* GlobalU32Ptr;
typedef const int __attribute__((address_space(1)))* GlobalIntPtr;

// 16 bytes of a row of B as VEC floats
template <typename BT> __device__ __forceinline__ void unpack_features(const u32x4& r, float (&f)[Dense<BT>::kVec]);
template <> __device__ __forceinline__ void unpack_features<float>(const u32x4& r, float (&f)[4]) {
    f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y); f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
}
template <> __device__ __forceinline__ void unpack_features<bf16_t>(const u32x4& r, float (&f)[8]) {
    f[0] = __uint_as_float(r.x << 16); f[1] = __uint_as_float(r.x & 0xFFFF0000u);
    f[2] = __uint_as_float(r.y << 16); f[3] = __uint_as_float(r.y & 0xFFFF0000u);
    f[4] = __uint_as_float(r.z << 16); f[5] = __uint_as_float(r.z & 0xFFFF0000u);
    f[6] = __uint_as_float(r.w << 16); f[7] = __uint_as_float(r.w & 0xFFFF0000u);
}

// acc[Q] += (weights of rows 4Q .. 4Q+3) (x) (this lane's features), unless no row of the quarter
// holds the column.  The instruction forms 16 outer products of 4 x 4, one per block of four
// lanes; with the broadcast field set, every block of a group of 2^CB takes its four weights
// from block Q of the group - lanes 4Q .. 4Q+3, which hold the weights of rows 4Q .. 4Q+3.
template <int CB, int Q, int VEC>
__device__ __forceinline__ void quarter_add(uint32_t quarters, float w, const float (&f)[VEC], f32x4 (&acc)[4][VEC]) {
    static_assert(kCellQuarters == 4, "one call per quarter");
    if (__builtin_expect((quarters & (1u << Q)) != 0, 1)) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[Q][c] = __builtin_amdgcn_mfma_f32_4x4x1f32(w, f[c], acc[Q][c], CB, Q, 0);
    }
}

// The SpMM kernel: one workgroup per four cells, one wavefront per cell, XCD-aware like the
// other kernels (workgroup i runs on XCD i % 8 and takes the i / 8-th tile of that XCD's
// contiguous share of every bucket).  Per merged entry a wavefront gathers one row of B (lane l
// holds features VEC*l .. VEC*l+VEC-1) and issues, per quarter that holds the column, VEC
// matrix instructions: instruction c takes the quarter's four weights and the c-th feature of
// every lane.  In accumulator [q][c], register i of lane l belongs to row 4q + i and feature
// VEC*l + c.
//
// Columns and weights of a cell are read once and are never in a cache, so every load of them
// waits out the full memory latency.  Fetched piecemeal next to the gathers they steer (four
// columns and one weight vector per half-batch) that latency was paid 24 times per cell, one
// after the other: 100^3 stencil at N = 256, 0.75 ms, and still 0.73 ms with every gather
// turned into a cache hit.  Here the whole cell's columns arrive with one load (lane l: entries
// 4l .. 4l+3; a cell has at most 256) and its weights with up to eight full-width loads that
// go to LDS; the loop takes columns out of registers (readlane) and weights out of LDS and
// only ever waits for gathers: 0.67 ms.  Entries are walked in half-batches of four with three
// in flight (two 4 % slower, four and five 7 - 8 % slower).  C is stored past the caches'
// retention (non-temporal: 0.765 -> 0.75 ms before the other changes), which leaves more of
// the L2 to B.
// What binds it now (100^3 stencil, N = 256, HIP events): with every gather turned into a cache
// hit it takes 0.54 ms, without the stores 0.53, with both 0.515 - a wavefront lives ~21 us, of
// which ~5 pass before its first matrix instruction (offsets, then columns and weights, then the
// first gathers) and ~3 in the stores, and two wavefronts per SIMD are what the registers allow.
// Measured against it: weights straight into LDS with global_load_lds (no staging registers,
// three wavefronts per SIMD) 0.75-0.85 ms; three or four wavefronts per SIMD by register limit
// 0.68 / 0.77 ms; a grid of resident workgroups that walk every 64th tile and load the next
// cell's columns and weights behind the last gathers of the current one (loads of a wavefront
// return in order, so earlier would stall the gathers) 0.70 ms; loads that bring the columns
// and weights of a tile 8 or 12 ahead into the L2 0.74 ms - an L1 keeps only so many reads
// under way (70 of 128 bytes on average here, 99 at most on any kernel of this library, by its
// latency counters; it is stalled on pending data 64 % of its cycles), and that, not the
// wavefront's own idle time, is what the loop runs out of.  The four wavefronts of a workgroup are on
// neighbouring cells, and the L1 already serves about a third of their gathers from lines a
// neighbour asked for (L1 accesses 8.0 GB, its read requests to the L2 4.4 GB); a barrier per
// turn that keeps the four in step adds 4 % to that and nothing to the time.
constexpr int kCellChunk = 128;            // merged entries whose weights a wavefront holds in LDS at a time
constexpr int kCellDepth = 3;              // half-batches of gathers in flight

//
// LPR lanes cover a row of B (64: 256 fp32 or 512 bf16 features per pass; 32 and 16: half and a
// quarter of that).  With LPR < 64 one gather instruction fetches the rows of E = 64 / LPR
// consecutive merged entries, one per group of LPR lanes, and the instruction's sixteen blocks
// fall to different entries: the blocks of lanes e * LPR .. (e + 1) * LPR - 1 belong to entry e
// and take their weights from block q of their own group.  The groups of lanes then hold E
// partial sums of every output element (entries e, e + E, e + 2E, ..., each in ascending column
// order), which are added in the order e = 0 .. E-1 before the store.
// 27-point stencil on 100^3, cells against four-row groups: fp32 N = 256 0.60 / 1.12 ms,
// N = 128 0.37 / 0.52 ms, N = 64 0.29 / 0.30 ms with the 16 x 16 instruction (a tie: not worth
// the rewrite, so 16 lanes per row are not launched); bf16 B doubles the matrix instructions per
// gathered byte and the accumulator registers (one wavefront per SIMD): N = 512 / 256 / 128
// 1.87 / 1.15 / 0.68 ms against 1.51 / 0.72 / 0.41 ms with the 16 x 16 instruction, so bf16
// operands stay with the row groups.
template <typename BT, int LPR>
__global__ void __launch_bounds__(64 * kCellTileCells)
spmm_cell_kernel(const LfCellBucket* __restrict__ buckets, int n_buckets, const void* __restrict__ B,
                 float* __restrict__ C, int feat, int ldb, int ldc, int accumulate) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int G = kCellRows;
    constexpr int E = 64 / LPR;                       // merged entries per gather instruction
    constexpr int H = E == 4 ? 2 : 4;                 // gather instructions per half-batch
    constexpr int HE = H * E;                         // merged entries per half-batch: 4 or 8
    constexpr int D = kCellDepth;
    constexpr int kBroadcast = E == 1 ? 4 : E == 2 ? 3 : 2;   // the weights of one block serve all 16 / 8 / 4 blocks of a group of LPR lanes
    constexpr int kLoads = kCellChunk * 4 / 64;       // full-width loads that bring a chunk's weights
    __shared__ f32x4 s_w[kCellTileCells][kCellChunk * 4];
    const int xcd = blockIdx.x % kXcds;
    long long v = blockIdx.x / kXcds;
    for (int bi = 0; bi < n_buckets; ++bi) {
        const LfCellBucket& b = buckets[bi];
        const long long lo = b.n_tiles * xcd / kXcds;
        const long long hi = b.n_tiles * (xcd + 1) / kXcds;
        if (v >= hi - lo) { v -= hi - lo; continue; }
        // everything that steers the walk is the same for all lanes of a wavefront
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int lane = threadIdx.x & 63;
        const int sub_of_lane = lane / LPR;
        // A wavefront walks kCellsPerWave cells one after the other (at each step the four
        // wavefronts of the workgroup are on four neighbouring cells).  One cell per wavefront
        // measured fastest (100^3 stencil, N = 256: 0.76 / 0.80 / 1.01 ms for 1 / 2 / 4 cells).
        const long long first = (lo + v) * (kCellTileCells * kCellsPerWave);
        int my_off = 0;
        if (first + lane <= b.n_cells) my_off = b.eoff[first + lane];
        else my_off = b.eoff[b.n_cells];
        f32x4* sw = s_w[wave];
        for (int step = 0; step < kCellsPerWave; ++step) {
        const int slot = step * kCellTileCells + wave;
        const long long cell = first + slot;
        if (cell >= b.n_cells) break;
        const int e0 = __builtin_amdgcn_readlane(my_off, slot);
        const int m = __builtin_amdgcn_readlane(my_off, slot + 1) - e0;           // a multiple of kCellBatch
        if (m == 0) continue;
        // (pointers read out of the bucket record are generic to the compiler; saying that they
        // are global memory keeps their loads off the LDS counter)
        const int my_row = reinterpret_cast<GlobalIntPtr>(reinterpret_cast<uintptr_t>(b.rows))[cell * G + (lane & 15)];
        const int cidx = min(4 * lane, m - 4);
        const i32x4 colv = *reinterpret_cast<GlobalInt4Ptr>(reinterpret_cast<uintptr_t>(b.ecol + e0 + cidx));
        const uint32_t usev = *reinterpret_cast<GlobalU32Ptr>(reinterpret_cast<uintptr_t>(b.euse + e0 + cidx));
        f32x4 acc[kCellQuarters][VEC];                    // [quarter of the cell][feature of this lane]: rows 4q .. 4q+3
#pragma unroll
        for (int q = 0; q < kCellQuarters; ++q)
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc[q][c] = f32x4{0.f, 0.f, 0.f, 0.f};
        // A gather is "row base (the same for all lanes, scalar registers) + 16 * lane": no
        // per-load address registers, and the 16 bytes stay packed until they are used.
        const char* b_bytes = reinterpret_cast<const char*>(B);
        const size_t row_bytes = (size_t)ldb * sizeof(BT);
        const uint32_t lane_off = (uint32_t)lane * 16u;
        for (int base = 0; base < m; base += kCellChunk) {
            const int mc = min(kCellChunk, m - base);
            // the chunk's weights, [mc / 4][16 rows] float4, are contiguous: lane l takes float4 l of every 64
            const GlobalFloat4Ptr wsrc = reinterpret_cast<GlobalFloat4Ptr>(reinterpret_cast<uintptr_t>(b.wq)) +
                                         (size_t)(e0 + base) * 4;
            f32x4 wreg[kLoads];
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                if (i * 64 < mc * 4) wreg[i] = __builtin_nontemporal_load(wsrc + min(i * 64 + lane, mc * 4 - 1));
            const int sub = lane / LPR;                           // which of the E entries of an instruction this lane gathers
            const uint32_t sub_off = (uint32_t)(lane % LPR) * 16u;
            auto issue = [&](int j, f32x4 (&w)[(HE + 3) / 4], u32x4 (&x)[H], uint32_t (&use)[(HE + 3) / 4], bool with_w) {
                // (no branch around the loads: the compiler counts outstanding loads per path)
                const int jj = j < mc ? j : mc - HE;              // past the end: the last half-batch again, unused
                const int q = (base + jj) >> 2;                   // jj is a multiple of 4: entry n sits in lane n / 4, component n % 4
                int c[HE];
#pragma unroll
                for (int t = 0; t < HE; t += 4) {
                    c[t] = __builtin_amdgcn_readlane(colv.x, q + t / 4);
                    c[t + 1] = __builtin_amdgcn_readlane(colv.y, q + t / 4);
                    c[t + 2] = __builtin_amdgcn_readlane(colv.z, q + t / 4);
                    c[t + 3] = __builtin_amdgcn_readlane(colv.w, q + t / 4);
                    use[t / 4] = __builtin_amdgcn_readlane(usev, q + t / 4);
                }
                if (with_w) {
#pragma unroll
                    for (int t = 0; t < (HE + 3) / 4; ++t) w[t] = sw[((jj >> 2) + t) * G + (lane & 15)];
                }
#pragma unroll
                for (int u = 0; u < H; ++u) {
                    if constexpr (E == 1) {
                        const char* row = b_bytes + (size_t)(uint32_t)c[u] * row_bytes;
                        x[u] = *reinterpret_cast<GlobalU32x4Ptr>(reinterpret_cast<uintptr_t>(row + lane_off));
                    } else {
                        int col = c[u * E];
#pragma unroll
                        for (int e = 1; e < E; ++e) col = sub == e ? c[u * E + e] : col;
                        const char* row = b_bytes + (size_t)(uint32_t)col * row_bytes;
                        x[u] = *reinterpret_cast<GlobalU32x4Ptr>(reinterpret_cast<uintptr_t>(row + sub_off));
                    }
                }
            };
            auto add_rows = [&](const f32x4 (&w)[(HE + 3) / 4], const u32x4 (&x)[H], const uint32_t (&use)[(HE + 3) / 4]) {
#pragma unroll
                for (int u = 0; u < H; ++u) {
                    // the weight of this lane's row at the entry this lane's block belongs to
                    float wu = w[(u * E) / 4][(u * E) % 4];
                    uint32_t quarters = use[(u * E) / 4] >> (8 * ((u * E) % 4));
#pragma unroll
                    for (int e = 1; e < E; ++e) {
                        wu = sub == e ? w[(u * E + e) / 4][(u * E + e) % 4] : wu;
                        quarters |= use[(u * E + e) / 4] >> (8 * ((u * E + e) % 4));
                    }
                    float f[VEC];
                    unpack_features<BT>(x[u], f);
                    // quarter q: rows 4q .. 4q+3 += their four weights (lanes 4q .. 4q+3 of every
                    // group of LPR lanes, handed to all blocks of the group) x this lane's features;
                    // skipped when none of the four rows holds the column (wavefront-uniform test)
                    quarter_add<kBroadcast, 0, VEC>(quarters, wu, f, acc);
                    quarter_add<kBroadcast, 1, VEC>(quarters, wu, f, acc);
                    quarter_add<kBroadcast, 2, VEC>(quarters, wu, f, acc);
                    quarter_add<kBroadcast, 3, VEC>(quarters, wu, f, acc);
                }
            };
            // The scheduling fences keep each group of loads ahead of the arithmetic of the
            // half-batches before it; left alone, the compiler sinks the loads to just before
            // their first use and every half-batch waits out the full memory latency.
            f32x4 wr[D][(HE + 3) / 4];
            u32x4 xr[D][H];
            uint32_t ur[D][(HE + 3) / 4];
            issue(0, wr[0], xr[0], ur[0], false);                 // the first gathers leave before the weights are in
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                if (i * 64 < mc * 4) sw[i * 64 + lane] = wreg[i];
            // one wavefront writes and reads this part of LDS, and LDS operations of a wavefront
            // complete in order: no barrier between the workgroup's wavefronts is needed
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int t = 0; t < (HE + 3) / 4; ++t) wr[0][t] = sw[t * G + (lane & 15)];
#pragma unroll
            for (int k = 1; k < D - 1; ++k) issue(k * HE, wr[k], xr[k], ur[k], true);
            for (int j = 0; j < mc; j += D * HE) {
#pragma unroll
                for (int k = 0; k < D; ++k) {
                    issue(j + (D - 1 + k) * HE, wr[(D - 1 + k) % D], xr[(D - 1 + k) % D], ur[(D - 1 + k) % D], true);
                    __builtin_amdgcn_sched_barrier(0);
                    if (k == 0 || j + k * HE < mc) add_rows(wr[k], xr[k], ur[k]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        // Register i of acc[q][c] is row 4q + i of the cell at feature VEC * (lane % LPR) + c: a row
        // leaves as one contiguous run of 16 bytes per lane.
        if constexpr (E == 1) {
#pragma unroll
            for (int q = 0; q < kCellQuarters; ++q) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = __builtin_amdgcn_readlane(my_row, 4 * q + i);
                    if (row < 0) continue;
                    float* dst = C + (size_t)row * ldc + VEC * lane;
#pragma unroll
                    for (int c0 = 0; c0 < VEC; c0 += 4) {
                        f32x4 o = {acc[q][c0][i], acc[q][c0 + 1][i], acc[q][c0 + 2][i], acc[q][c0 + 3][i]};
                        if (accumulate & kAccumulateC) o += *reinterpret_cast<const f32x4*>(dst + c0);
                        store_f32x4(dst + c0, o, accumulate & kStreamC);
                    }
                }
            }
        } else {
            // Two entries per gather instruction: lanes 0-31 hold the sums over the even entries,
            // lanes 32-63 those over the odd ones.  Rows i and i + 2 of a quarter trade halves
            // (one instruction swaps the upper half of one register with the lower half of
            // another), after which the lower lanes hold both parts of row i and the upper lanes
            // both parts of row i + 2; even entries are added first in either.
            static_assert(E == 2, "the halves of a wavefront are traded");
#pragma unroll
            for (int q = 0; q < kCellQuarters; ++q) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int row_lo = __builtin_amdgcn_readlane(my_row, 4 * q + i);
                    const int row_hi = __builtin_amdgcn_readlane(my_row, 4 * q + i + 2);
                    const int row = sub_of_lane ? row_hi : row_lo;
#pragma unroll
                    for (int c0 = 0; c0 < VEC; c0 += 4) {
                        f32x4 o;
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            const auto t = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[q][c0 + c][i]),
                                                                            __float_as_uint(acc[q][c0 + c][i + 2]), false, false);
                            o[c] = __uint_as_float(t[0]) + __uint_as_float(t[1]);
                        }
                        if (row < 0) continue;
                        float* dst = C + (size_t)row * ldc + VEC * (lane % LPR);
                        if (accumulate & kAccumulateC) o += *reinterpret_cast<const f32x4*>(dst + c0);
                        store_f32x4(dst + c0, o, accumulate & kStreamC);
                    }
                }
            }
        }
        }
        return;
    }
}

// Strides and cell shape from a sample of rows.  Returns false when nothing stands out.
bool detect_geometry(const std::vector<int32_t>& sample, int n_samples, int n_cols, int cell_rows,
                     int64_t num_rows, long long bucket_rows, long long row_bytes, CellGeom* out, long long* n_cells) {
    std::vector<long long> diffs;
    int rows_seen = 0;
    for (int i = 0; i < n_samples; ++i) {
        const int32_t* o = sample.data() + (size_t)i * (n_cols + 2);
        const int len = std::min<int>(o[1], n_cols);
        if (len < 2) continue;
        ++rows_seen;
        for (int x = 0; x < len; ++x)
            for (int y = x + 1; y < len; ++y) {
                const long long d = std::llabs((long long)o[2 + y] - (long long)o[2 + x]);
                if (d > 0) diffs.push_back(d);
            }
    }
    if (rows_seen == 0 || diffs.empty()) return false;
    std::sort(diffs.begin(), diffs.end());
    std::vector<std::pair<long long, int>> runs;      // (difference, how often)
    for (size_t i = 0; i < diffs.size();) {
        size_t j = i;
        while (j < diffs.size() && diffs[j] == diffs[i]) ++j;
        runs.emplace_back(diffs[i], (int)(j - i));
        i = j;
    }
    int top = 0;
    for (auto& r : runs) top = std::max(top, r.second);
    if (top < rows_seen) return false;               // no difference that most rows show
    std::vector<long long> cand;                     // ascending
    for (auto& r : runs)
        if ((long long)r.second * 4 >= (long long)top * 3) cand.push_back(r.first);
    if (cand.empty() || cand[0] != 1) return false;  // rows that share columns must include neighbours
    auto first_at_least = [&](long long lo) -> long long {
        for (long long c : cand)
            if (c >= lo) return c;
        return 0;
    };
    CellGeom q{};
    q.s1 = 1;
    // Three strides: 2 x 2 x 4.  Four rows that follow each other in a cell share the matrix
    // instruction, so the fewer columns such a quarter spans the fewer instructions are spent on
    // zeros: 2 x 2 x 1 quarters of a 27-point stencil use 48 of the cell's 96 columns, the 4 x 1 x 1
    // quarters of a 4 x 2 x 2 cell 54 (100^3 stencil, N = 256 / 128: 0.604 / 0.370 ms against
    // 0.627 / 0.398; 2 x 4 x 2: 0.606 / 0.380; flat cells - 4 x 4 x 1, 8 x 2 x 1 - 0.69 / 0.47).
    int g3[3] = {2, 2, cell_rows / 4};
    if (const char* env = getenv("LF_CELL_SHAPE")) {
        int e0 = 0, e1 = 0, e2 = 0;
        if (sscanf(env, "%d,%d,%d", &e0, &e1, &e2) == 3 && e0 > 0 && e1 > 0 && e2 > 0 && e0 * e1 * e2 == cell_rows) {
            g3[0] = e0; g3[1] = e1; g3[2] = e2;
        }
    }
    const int g2[2] = {4, cell_rows / 4};            // two strides: 4 x 4
    const long long s2_3 = first_at_least((long long)g3[0]);
    const long long s3_3 = s2_3 ? first_at_least(s2_3 * g3[1]) : 0;
    const long long s2_2 = first_at_least((long long)g2[0]);
    if (s2_3 && s3_3) {
        q.k = 3; q.g0 = g3[0]; q.g1 = g3[1]; q.g2 = g3[2]; q.s2 = s2_3; q.s3 = s3_3;
        q.n0 = lf::ceil_div(q.s2, q.g0);
        q.n1 = lf::ceil_div(lf::ceil_div(q.s3, q.s2), q.g1);
        q.n2 = lf::ceil_div(lf::ceil_div(num_rows, q.s3), q.g2);
        // Order of the cells: in plain (z, y, x) order the planes of B that two z-layers of
        // cells share come round again a whole layer later, long after they left the L2.  So
        // yb cell rows along y are swept through all z before the next ones, with yb the
        // largest count whose rows of B for one z-step - (yb * g1 + 2) grid lines of s2 / s1
        // rows in g2 + 2 planes - fit one XCD's 4 MB L2 (100^3 stencil, 1 KB rows, 4 x 2 x 2
        // cells: 4; measured L2 misses 28.4M / 40.8M / 30.7M / 22.2M / 24.4M for plain order /
        // 1 / 2 / 4 / 8).
        const long long line_bytes = (q.s2 / q.s1) * (long long)(q.g2 + 2) * row_bytes;
        const long long lines = line_bytes > 0 ? kL2BytesPerXcd / line_bytes : 0;
        long long yb = (lines - 2) / q.g1;
        if (lines >= 6) yb = std::max<long long>(yb, 3);          // (measured: 3 or 4 beat 2 where this estimate says 2)
        const char* env_yb = getenv("LF_CELL_YB");
        if (env_yb) yb = atoi(env_yb);
        q.yb = (yb >= 2 && yb < q.n1) ? (int)yb : 0;
        *n_cells = (q.yb > 0 ? lf::ceil_div(q.n1, q.yb) * q.yb : q.n1) * q.n0 * q.n2;
    } else if (s2_2) {
        q.k = 2; q.g0 = g2[0]; q.g1 = g2[1]; q.g2 = 1; q.s2 = s2_2; q.s3 = 1;
        q.n0 = lf::ceil_div(q.s2, q.g0);
        q.n1 = lf::ceil_div(lf::ceil_div(num_rows, q.s2), q.g1);
        *n_cells = q.n0 * q.n1;
    } else {
        q.k = 1; q.g0 = cell_rows; q.g1 = q.g2 = 1; q.s2 = q.s3 = 1;
        q.n0 = lf::ceil_div(num_rows, q.g0);
        q.n1 = 1;
        *n_cells = q.n0;
    }
    // cells that stay mostly empty (a bucket that holds few of the matrix's rows) are not worth it
    if (*n_cells > 2 * lf::ceil_div(bucket_rows, cell_rows) + 4096 || *n_cells * cell_rows >= (1ll << 31)) return false;
    *out = q;
    return true;
}

template <typename T> int cell_alloc(std::vector<void*>* keep, T** out, size_t count) {
    *out = nullptr;
    void* p = nullptr;
    LF_HIP(hipMalloc(&p, std::max<size_t>(count, 1) * sizeof(T)));
    keep->push_back(p);
    *out = (T*)p;
    return LF_OK;
}

}  // namespace

namespace lf {

int cells_build(const lf_bucket_desc& b, const int32_t* d_meta, int64_t num_rows, int64_t row_bytes, hipStream_t s,
                std::vector<void*>* owned, std::vector<void*>* temp, LfCellBucket* out, bool* accepted) {
    *accepted = false;
    constexpr int G = kCellRows;
    if (b.num_ell_rows < 1 || b.width < 4 || b.width > kCellWidthMax) return LF_OK;   // (rows are staged 16 bytes at a time)
    const int log_w = lf::ilog2(b.width);
    const long long R = b.num_ell_rows;

    // ---- strides from a sample of rows
    const int n_samples = (int)std::min<long long>(kCellSampleRows, R);
    const int n_cols = std::min<int>(kCellSampleCols, b.width);
    int32_t* d_sample = nullptr;
    if (int rc = cell_alloc(temp, &d_sample, (size_t)n_samples * (n_cols + 2))) return rc;
    cell_sample_kernel<<<n_samples, 64, 0, s>>>(b.d_rows, b.d_cols, d_meta, R, log_w, R / n_samples, n_samples, n_cols, d_sample);
    LF_HIP(hipGetLastError());
    std::vector<int32_t> h_sample((size_t)n_samples * (n_cols + 2));
    LF_HIP(hipMemcpyAsync(h_sample.data(), d_sample, h_sample.size() * 4, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    CellGeom geom{};
    long long n_cells = 0;
    if (!detect_geometry(h_sample, n_samples, n_cols, G, num_rows, R, row_bytes, &geom, &n_cells)) return LF_OK;

    // ---- rows into cells, then count what the merged cells would hold
    int32_t *d_cnt = nullptr, *d_perm = nullptr, *d_m = nullptr, *d_partial = nullptr;
    unsigned long long* d_stats = nullptr;      // four counters, then (at [6]) the overflow flag
    if (int rc = cell_alloc(temp, &d_cnt, (size_t)n_cells)) return rc;
    if (int rc = cell_alloc(temp, &d_perm, (size_t)n_cells * G)) return rc;
    if (int rc = cell_alloc(temp, &d_m, (size_t)n_cells)) return rc;
    if (int rc = cell_alloc(temp, &d_partial, (size_t)lf::ceil_div(n_cells, 1024) + 1)) return rc;
    if (int rc = cell_alloc(temp, &d_stats, 8)) return rc;
    int32_t *d_cnt_raw = nullptr, *d_plain = nullptr;
    if (int rc = cell_alloc(temp, &d_cnt_raw, (size_t)n_cells)) return rc;
    if (int rc = cell_alloc(temp, &d_plain, (size_t)n_cells)) return rc;
    const int fgrid = (int)std::min<long long>(lf::ceil_div(n_cells * G, 256), 4096);
    fill_i32_kernel<<<fgrid, 256, 0, s>>>(d_cnt, n_cells, 0);
    fill_i32_kernel<<<fgrid, 256, 0, s>>>(d_perm, n_cells * G, -1);
    fill_i32_kernel<<<1, 64, 0, s>>>((int32_t*)d_stats, 16, 0);
    LF_HIP(hipGetLastError());
    int* d_flags = (int*)(d_stats + 6);
    cell_assign_kernel<<<(int)lf::ceil_div(R, 256), 256, 0, s>>>(b.d_rows, R, geom, G, d_cnt, d_perm, d_flags);
    LF_HIP(hipGetLastError());
    CellMergeArgs ma{};
    ma.rows = b.d_rows;
    ma.cols = b.d_cols;
    ma.vals = b.d_vals;
    ma.meta = d_meta;
    ma.log_w = log_w;
    ma.n_cells = n_cells;
    ma.perm = d_perm;
    ma.m_out = d_m;
    ma.cnt_out = d_cnt_raw;
    ma.plain_out = d_plain;
    cell_merge_kernel<<<(unsigned)lf::ceil_div(n_cells, 4), 64, merge_lds(ma), s>>>(ma);
    LF_HIP(hipGetLastError());
    cell_stats_kernel<<<(int)std::min<long long>(lf::ceil_div(n_cells, 256), 256), 256, 0, s>>>(d_cnt_raw, d_plain, d_m, n_cells,
                                                                                                d_stats);
    LF_HIP(hipGetLastError());
    unsigned long long h_stats[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    LF_HIP(hipMemcpyAsync(h_stats, d_stats, sizeof(h_stats), hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    const unsigned long long entries = h_stats[0], plain = h_stats[1], rounded = h_stats[2];
    const int overflow = (int)(h_stats[6] & 0xFFFFFFFFull);
    if (overflow || entries == 0 || rounded >= (1ull << 31) || entries * 100 > plain * kCellMaxPercent ||
        h_stats[3] > (unsigned long long)kCellEntriesCap)
        return LF_OK;

    // ---- offsets and the cells themselves
    int32_t *d_eoff = nullptr, *d_ecol = nullptr, *d_rows_out = nullptr;
    float4* d_wq = nullptr;
    uint8_t* d_euse = nullptr;
    if (int rc = cell_alloc(owned, &d_euse, (size_t)rounded)) return rc;
    if (int rc = cell_alloc(owned, &d_eoff, (size_t)n_cells + 1)) return rc;
    if (int rc = cell_alloc(owned, &d_ecol, (size_t)rounded)) return rc;
    if (int rc = cell_alloc(owned, &d_wq, (size_t)rounded / 4 * G)) return rc;
    if (int rc = cell_alloc(owned, &d_rows_out, (size_t)n_cells * G)) return rc;
    LF_HIP(exclusive_scan_i32(d_m, n_cells, d_partial, d_eoff, s));
    ma.eoff = d_eoff;
    ma.ecol = d_ecol;
    ma.wq = reinterpret_cast<float*>(d_wq);
    ma.rows_out = d_rows_out;
    ma.euse = d_euse;
    cell_merge_kernel<<<(unsigned)lf::ceil_div(n_cells, 4), 64, merge_lds(ma), s>>>(ma);
    LF_HIP(hipGetLastError());
    out->n_cells = n_cells;
    out->n_tiles = lf::ceil_div(n_cells, kCellTileCells * kCellsPerWave);
    out->eoff = d_eoff;
    out->ecol = d_ecol;
    out->wq = d_wq;
    out->rows = d_rows_out;
    out->euse = d_euse;
    *accepted = true;
    return LF_OK;
}

int cells_launch(const LfCellBucket* d_buckets, int n_buckets, int grid, int b_dtype, const void* B, float* C,
                 int feat, int ldb, int ldc, int accumulate, hipStream_t s) {
    if (n_buckets <= 0 || grid <= 0) return LF_OK;
    LF_REQUIRE(b_dtype == LF_DTYPE_F32 && (feat == 256 || feat == 128), LF_ERR_UNSUPPORTED,
               "cells are built for 128 or 256 fp32 features per pass");
    const dim3 wg(64 * kCellTileCells);
    if (feat == 256) spmm_cell_kernel<float, 64><<<grid, wg, 0, s>>>(d_buckets, n_buckets, B, C, feat, ldb, ldc, accumulate);
    else spmm_cell_kernel<float, 32><<<grid, wg, 0, s>>>(d_buckets, n_buckets, B, C, feat, ldb, ldc, accumulate);
    LF_HIP(hipGetLastError());
    return LF_OK;
}

}  // namespace lf
