// Device side of format composition for gfx950: bucket statistics for the width search
// and the hyb (column partition x power-of-two ELL bucket) builder.
//
// Reference behaviour reproduced here:
//   get_init_buckets   playground_pipline/format_algos.py:819-900   (lf_bucket_stats)
//   build_hyb_format   playground_pipline/format_algos.py:226-385   (lf_hyb_plan / lf_hyb_build)
//
// The reference walks nonzeros one at a time on the host.  On the GPU the same result is
// obtained from per-(row, partition) segments: CSR is row-major with ascending columns,
// so the nonzeros of one segment are contiguous, every bucket receives whole segments in
// ascending row order, and a segment of `fill` entries occupies ceil(fill / W) consecutive
// ELL rows that carry the same row id, with (0, 0) padding only after its last entry.
// ELL-row offsets are therefore an exclusive scan, in row order, of per-segment ELL-row
// counts, taken separately for each bucket.  All counting uses integer arithmetic, so the
// output does not depend on scheduling.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <mutex>
#include <vector>

#include "lf_internal.h"

// Accumulators of lf_row_features_static: {min, max, sum, sum of squares}.  One copy of the
// array lives on every GPU the library runs on, for the life of the process.  Host code never
// uses the array's name as an address: static_scratch() below asks the runtime where the
// current device keeps it.
static __device__ __align__(256) unsigned long long lf_static_scratch[4];

namespace {

constexpr int kBlock = 256;          // rows per workgroup in the per-segment kernels
constexpr int kStatsGrid = 2048;     // workgroups per partition in the statistics pass at most
// meta word of an ELL row: bits 0..10 valid slots (1..1024); bits 11..30 a count: on the
// first ELL row of a source row's segment the number of ELL rows in the segment, on a
// continuation row its index inside the segment; bit 31 set on continuation rows.
constexpr int kMetaLenBits = 11;
constexpr int kMetaSegMax = (1 << (31 - kMetaLenBits)) - 1;
constexpr uint32_t kMetaCont = 0x80000000u;

__host__ __device__ inline int32_t make_meta(int len, int i, int n_ell) {
    return (int32_t)((uint32_t)len | ((uint32_t)(i == 0 ? n_ell : i) << kMetaLenBits) | (i == 0 ? 0u : kMetaCont));
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---------------------------------------------------------------------------- device utils
__device__ __forceinline__ int lower_bound_i32(const int32_t* __restrict__ a, int lo, int hi, int64_t key) {
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if ((int64_t)a[mid] < key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Segment (row r, partition p): offset of its first entry in the CSR arrays and its length.
// With one partition the segment is the row; otherwise boundaries were precomputed into
// bnd[(P + 1)][rows] (partition-major so that neighbouring threads read neighbouring words).
struct SegView {
    const int32_t* indptr;
    const int32_t* bnd;
    int64_t rows;
    int parts;
};

__device__ __forceinline__ void seg_range(const SegView& v, int64_t r, int p, int& start, int& fill) {
    if (v.parts == 1) {
        start = v.indptr[r];
        fill = v.indptr[r + 1] - start;
    } else {
        start = v.bnd[(int64_t)p * v.rows + r];
        fill = v.bnd[(int64_t)(p + 1) * v.rows + r] - start;
    }
}

__global__ void fill_u32_kernel(uint32_t* __restrict__ p, int64_t n, uint32_t value) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        p[i] = value;
}

hipError_t fill_u32(void* p, int64_t n_words, uint32_t value, hipStream_t s) {
    if (n_words <= 0) return hipSuccess;
    const int grid = (int)std::min<int64_t>((n_words + 255) / 256, 4096);
    fill_u32_kernel<<<grid, 256, 0, s>>>((uint32_t*)p, n_words, value);
    return hipGetLastError();
}

// bnd[p][r] = first CSR position of row r whose column is >= p * psize   (p = 0..P)
__global__ void seg_bounds_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices,
                                  int64_t rows, int parts, int64_t psize, int32_t* __restrict__ bnd) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const int lo = indptr[r], hi = indptr[r + 1];
    bnd[r] = lo;
    int cur = lo;
    for (int p = 1; p < parts; ++p) {
        cur = lower_bound_i32(indices, cur, hi, (int64_t)p * psize);
        bnd[(int64_t)p * rows + r] = cur;
    }
    bnd[(int64_t)parts * rows + r] = hi;
}

// deg[p][r] += 1 for every COO triplet (format_algos.py:846-849 counts raw triplets)
__global__ void coo_degree_kernel(const int32_t* __restrict__ row, const int32_t* __restrict__ col,
                                  int64_t nnz, int64_t rows, int64_t psize, int32_t* __restrict__ deg) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nnz;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t p = col[i] / psize;
        atomicAdd(&deg[p * rows + row[i]], 1);
    }
}

// out = {min, max, sum, sum of squares} of the row lengths; out[0] starts at ~0, the rest at 0
__global__ void __launch_bounds__(kBlock)
row_features_kernel(const int32_t* __restrict__ indptr, int64_t rows, unsigned long long* __restrict__ out) {
    __shared__ unsigned long long s_red[4][kBlock / 64];
    unsigned long long lo = ~0ull, hi = 0, sum = 0, sq = 0;
    for (int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (int64_t)gridDim.x * kBlock) {
        const unsigned long long d = (unsigned long long)(indptr[r + 1] - indptr[r]);
        lo = d < lo ? d : lo;
        hi = d > hi ? d : hi;
        sum += d;
        sq += d * d;
    }
    for (int d = 32; d > 0; d >>= 1) {
        const unsigned long long l2 = __shfl_xor(lo, d), h2 = __shfl_xor(hi, d);
        lo = l2 < lo ? l2 : lo;
        hi = h2 > hi ? h2 : hi;
        sum += __shfl_xor(sum, d);
        sq += __shfl_xor(sq, d);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { s_red[0][wave] = lo; s_red[1][wave] = hi; s_red[2][wave] = sum; s_red[3][wave] = sq; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / 64; ++w) {
            lo = s_red[0][w] < lo ? s_red[0][w] : lo;
            hi = s_red[1][w] > hi ? s_red[1][w] : hi;
            sum += s_red[2][w];
            sq += s_red[3][w];
        }
        atomicMin(&out[0], lo);
        atomicMax(&out[1], hi);
        atomicAdd(&out[2], sum);
        atomicAdd(&out[3], sq);
    }
}

// out[0] += entries of row r that also occur in row r - 1, out[1] += entries of row r, for every
// stride-th row r >= 1 (two-pointer walk over the two ascending column lists).  Only the first
// kOverlapEntries entries of either row are looked at: one thread walks a pair of rows, and a
// sample that lands on a row of 100,000 entries would otherwise take longer than composing the
// whole format (11 ms against 0.3 ms for a 500k x 2M matrix with 50 such rows).
constexpr int kOverlapEntries = 64;
__global__ void __launch_bounds__(kBlock)
row_overlap_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices, int64_t rows,
                   int64_t stride, unsigned long long* __restrict__ out) {
    unsigned long long both = 0, seen = 0;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;; i += (int64_t)gridDim.x * kBlock) {
        const int64_t r = 1 + i * stride;
        if (r >= rows) break;
        int a = indptr[r - 1], b = indptr[r];
        const int a_end = min(b, a + kOverlapEntries), b_end = min(indptr[r + 1], b + kOverlapEntries);
        seen += (unsigned long long)(b_end - b);
        while (a < a_end && b < b_end) {
            const int ca = indices[a], cb = indices[b];
            both += ca == cb;
            a += ca <= cb;
            b += cb <= ca;
        }
    }
    for (int d = 32; d > 0; d >>= 1) {
        both += __shfl_xor(both, d);
        seen += __shfl_xor(seen, d);
    }
    if ((threadIdx.x & 63) == 0 && seen) {
        atomicAdd(&out[0], both);
        atomicAdd(&out[1], seen);
    }
}

// Initial width class of a segment of `deg` entries: width = min(next_pow2(deg), limit),
// cost-model rows = max(1, next_pow2(deg) / limit)            (format_algos.py:875-882)
__device__ __forceinline__ void width_class(int deg, int kmax, int& k, int& cost_rows) {
    k = deg <= 1 ? 0 : 32 - __clz(deg - 1);
    cost_rows = 1;
    if (k > kmax) {
        cost_rows = 1 << (k - kmax);
        k = kmax;
    }
}

// One thread per (row, partition) segment for the counters; blockIdx.y is the partition.
//   stats[p][k] += {cost rows, nnz, 1}
//   plane[k][c]  = 1             for every column c of a segment of class k  (skipped when planes is null)
// Column sets are one byte per (class, column), written with plain stores after an "already
// set?" probe: no atomics, and a stale probe (another XCD's L2 still holds the old line) only
// repeats a store of the same value.  blockIdx.z is the class a workgroup marks: workgroups
// are handed out z last, so the launch works through one class (and partition) at a time.
// The columns of a class are walked by the whole workgroup over the concatenation of its
// segments among 256 rows (element -> segment by a binary search over LDS prefix sums), four
// independent elements per thread, so neither a long row nor the chain "index load -> probe"
// of one row serialises.  Measured for 81.6M nonzeros, 2.45M columns: one thread per row
// with a 32-bit mask per column and atomicOr 2.0 ms; workgroup walk with 16-bit masks and
// atomicOr 1.86 ms, of which the ~13M atomics take 1.2 ms (a mask copy per XCD makes it
// 3.1 ms: more atomics, and they cost the same wherever the line lives); byte planes with
// all classes in flight 1.47 ms; byte planes class by class 1.44 ms (0.38 ms walk, 0.27 ms
// probes, 0.8 ms stores).  The counters show one 64-byte line fetched per probe and one
// written per first-touch store (5.2 GB + 1.1 GB): the pass runs at the rate the fabric
// moves single lines, the planes do not stay in the L2s between probes.
constexpr int kMarkUnroll = 4;

__global__ void __launch_bounds__(kBlock)
bucket_stats_kernel(SegView v, const int32_t* __restrict__ indices, const int32_t* __restrict__ seg_deg,
                    int kmax, uint8_t* __restrict__ planes, int64_t cols,
                    unsigned long long* __restrict__ stats) {
    __shared__ unsigned long long s_stats[LF_MAX_CLASSES * LF_STATS_FIELDS];
    __shared__ int s_off[kBlock + 1];      // exclusive prefix of the lengths of this class's segments
    __shared__ int s_start[kBlock];
    __shared__ int s_wave[kBlock / 64];
    for (int i = threadIdx.x; i < LF_MAX_CLASSES * LF_STATS_FIELDS; i += kBlock) s_stats[i] = 0ull;
    __syncthreads();

    const int p = blockIdx.y;
    const int kz = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint8_t* plane = planes ? planes + (size_t)kz * (size_t)cols : nullptr;
    // a workgroup walks several blocks of rows, so that the global counters below see a few
    // thousand updates per launch and not one per 256 rows
    for (int64_t base = (int64_t)blockIdx.x * kBlock; base < v.rows; base += (int64_t)gridDim.x * kBlock) {
        const int64_t r = base + threadIdx.x;
        int start = 0, fill = 0, deg = 0;
        if (r < v.rows) {
            seg_range(v, r, p, start, fill);
            deg = seg_deg ? seg_deg[(int64_t)p * v.rows + r] : fill;
        }
        int k = -1;
        if (deg > 0) {
            int cost_rows;
            width_class(deg, kmax, k, cost_rows);
            if (kz == 0) {
                atomicAdd(&s_stats[k * LF_STATS_FIELDS + 0], (unsigned long long)cost_rows);
                atomicAdd(&s_stats[k * LF_STATS_FIELDS + 1], (unsigned long long)deg);
                atomicAdd(&s_stats[k * LF_STATS_FIELDS + 2], 1ull);
            }
        }
        if (plane == nullptr) continue;                // uniform over the launch

        const int x = k == kz ? fill : 0;
        if (!__syncthreads_or(x)) continue;            // no segment of this class among these rows
        int incl = x;
        for (int d = 1; d < 64; d <<= 1) {
            const int y = __shfl_up(incl, d);
            if (lane >= d) incl += y;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        int wave_off = 0;
        for (int wv = 0; wv < wave; ++wv) wave_off += s_wave[wv];
        s_off[threadIdx.x] = wave_off + incl - x;
        s_start[threadIdx.x] = start;
        if (threadIdx.x == kBlock - 1) s_off[kBlock] = wave_off + incl;
        __syncthreads();
        const int total = s_off[kBlock];
        for (int j0 = 0; j0 < total; j0 += kBlock * kMarkUnroll) {
            int c[kMarkUnroll];
            uint8_t seen[kMarkUnroll];
#pragma unroll
            for (int u = 0; u < kMarkUnroll; ++u) {
                const int j = j0 + u * kBlock + (int)threadIdx.x;
                c[u] = -1;
                if (j < total) {
                    int lo = 0, hi = kBlock - 1;       // last segment whose offset is <= j
#pragma unroll
                    for (int step = 0; step < 8; ++step) {
                        const int mid = (lo + hi + 1) >> 1;
                        if (s_off[mid] <= j) lo = mid; else hi = mid - 1;
                    }
                    c[u] = indices[s_start[lo] + (j - s_off[lo])];
                }
            }
#pragma unroll
            for (int u = 0; u < kMarkUnroll; ++u) seen[u] = c[u] >= 0 ? plane[c[u]] : (uint8_t)1;
#pragma unroll
            for (int u = 0; u < kMarkUnroll; ++u)
                if (seen[u] == 0) plane[c[u]] = 1;
        }
        __syncthreads();                               // the tables are rewritten by the next block of rows
    }
    if (kz != 0) return;
    __syncthreads();
    for (int i = threadIdx.x; i < LF_MAX_CLASSES * LF_STATS_FIELDS; i += kBlock)
        if (s_stats[i]) atomicAdd(&stats[(size_t)p * LF_MAX_CLASSES * LF_STATS_FIELDS + i], s_stats[i]);
}

// hist[p][mask] = number of columns of partition p whose set of classes is mask
__global__ void __launch_bounds__(kBlock)
colmask_hist_kernel(const uint8_t* __restrict__ planes, int num_classes, int64_t cols, int64_t psize,
                    unsigned long long* __restrict__ hist) {
    constexpr int kBins = 1 << LF_MAX_CLASSES;
    __shared__ uint32_t s_hist[kBins];
    for (int i = threadIdx.x; i < kBins; i += kBlock) s_hist[i] = 0;
    __syncthreads();
    const int p = blockIdx.y;
    const int64_t lo = (int64_t)p * psize;
    const int64_t hi = lo + psize < cols ? lo + psize : cols;
    for (int64_t c = lo + (int64_t)blockIdx.x * kBlock + threadIdx.x; c < hi;
         c += (int64_t)gridDim.x * kBlock) {
        uint32_t m = 0;
        for (int k = 0; k < num_classes; ++k) m |= planes[(size_t)k * (size_t)cols + c] ? 1u << k : 0u;
        atomicAdd(&s_hist[m], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kBins; i += kBlock)
        if (s_hist[i]) atomicAdd(&hist[(size_t)p * kBins + i], (unsigned long long)s_hist[i]);
}

// ---------------------------------------------------------------------------- hyb plan/build
// Width table on the device: wtab[p][0] = count, wtab[p][1 + b] = width, wtab[p][12] = index
// of the partition's first bucket in the flat (p, b) bucket order.
constexpr int kWtabStride = 16;

// Bucket of a segment: first width >= deg, else the widest (format_algos.py:275-279).
__device__ __forceinline__ int pick_bucket(const int32_t* __restrict__ w, int n, int deg) {
    int b = 0;
    while (b < n && w[1 + b] < deg) ++b;
    return b == n ? n - 1 : b;
}

// Per workgroup of kBlock rows and per bucket: number of ELL rows the block contributes.
// blockcnt[(bucket_base[p] + b) * nblk + blk]
__global__ void __launch_bounds__(kBlock)
hyb_count_kernel(SegView v, const int32_t* __restrict__ seg_deg, const int32_t* __restrict__ wtab,
                 int nblk, int32_t* __restrict__ blockcnt, int32_t* __restrict__ flags) {
    __shared__ int s_cnt[LF_MAX_CLASSES];
    if (threadIdx.x < LF_MAX_CLASSES) s_cnt[threadIdx.x] = 0;
    __syncthreads();
    const int p = blockIdx.y;
    const int32_t* w = wtab + p * kWtabStride;
    const int n = w[0];
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r < v.rows) {
        int start, fill;
        seg_range(v, r, p, start, fill);
        if (fill > 0) {
            if (n == 0) {
                atomicOr(&flags[0], 1);       // nonzeros in a partition without widths
            } else {
                const int deg = seg_deg ? seg_deg[(int64_t)p * v.rows + r] : fill;
                const int b = pick_bucket(w, n, deg);
                const int width = w[1 + b];
                const int n_ell = (fill + width - 1) / width;
                if (n_ell > kMetaSegMax) atomicOr(&flags[0], 2);
                atomicAdd(&s_cnt[b], n_ell);
            }
        }
    }
    __syncthreads();
    if ((int)threadIdx.x < n)
        blockcnt[(int64_t)(w[12] + threadIdx.x) * nblk + blockIdx.x] = s_cnt[threadIdx.x];
}

// Exclusive scan over blocks, one workgroup per bucket; totals[k] = ELL rows of bucket k.
__global__ void __launch_bounds__(1024)
hyb_scan_kernel(int32_t* __restrict__ blockcnt, int nblk, long long* __restrict__ totals) {
    __shared__ long long s_wave[16];
    __shared__ long long s_carry;
    int32_t* a = blockcnt + (int64_t)blockIdx.x * nblk;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    for (int base = 0; base < nblk; base += 1024) {
        const int i = base + threadIdx.x;
        const long long x = i < nblk ? a[i] : 0;
        long long incl = x;
        for (int d = 1; d < 64; d <<= 1) {
            const long long y = __shfl_up(incl, d);
            if (lane >= d) incl += y;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        long long wave_off = 0;
        for (int wv = 0; wv < wave; ++wv) wave_off += s_wave[wv];
        const long long carry = s_carry;
        if (i < nblk) a[i] = (int32_t)(carry + wave_off + incl - x);
        __syncthreads();
        if (threadIdx.x == 1023) s_carry = carry + wave_off + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = s_carry;
}

// Fills the slabs.  One workgroup per 256 source rows, four column partitions at a time.
//   * one thread per (row, partition) segment finds the segment's bucket and its first ELL
//     row (per-wavefront counts per bucket - bit counts, or a shuffle scan where segments
//     split - combined through LDS with a single barrier) and writes the rows / meta entries;
//   * the workgroup then walks the concatenation of the 256 segments, each padded to whole
//     ELL rows: consecutive threads take consecutive groups of four slots (group -> segment
//     by a binary search over LDS prefix sums), so the CSR entries are read in order and
//     each segment's ELL rows, which are consecutive in the slab, are written in order,
//     padding included, with 16-byte accesses wherever a group lies inside one row.
// Reading in row order matters: a source row is ~130 bytes at an arbitrary offset, and when
// the slabs were filled bucket by bucket every row cost two full cache lines (1.27 GB fetched
// for 0.65 GB of entries on an 81.6M-nonzero matrix).
struct BucketOffsets {
    long long slot_off;    // first slot of the bucket in the flat slab arrays
    long long row_off;     // first ELL row of the bucket in the flat row arrays
};

constexpr int kFillUnroll = 4;
constexpr int kPartGroup = 4;        // column partitions whose segments are walked together
// four consecutive 32-bit values at a 4-byte aligned address (one 16-byte load)
struct __attribute__((packed, aligned(4))) Packed4i { int x, y, z, w; };
struct __attribute__((packed, aligned(4))) Packed4f { float x, y, z, w; };

__global__ void __launch_bounds__(kBlock)
hyb_fill_kernel(SegView v, const int32_t* __restrict__ seg_deg, const int32_t* __restrict__ wtab,
                int nblk, const int32_t* __restrict__ blockoff, const BucketOffsets* __restrict__ offs,
                const int32_t* __restrict__ indices, const float* __restrict__ values,
                int32_t* __restrict__ out_rows, int32_t* __restrict__ out_meta,
                int32_t* __restrict__ out_cols, float* __restrict__ out_vals, float* __restrict__ out_mask) {
    // segment tables of the walk, entry t * pg + pp for row t and the pp-th partition of the
    // group of pg <= kPartGroup partitions in hand: row-major, so the walk reads each row's CSR
    // entries once and in order however many partitions cut it
    constexpr int kSegs = kBlock * kPartGroup;
    __shared__ int s_cnt[kBlock / 64][LF_MAX_CLASSES + 1];
    // exclusive prefix of the padded segment lengths; 32 bits are enough: a segment is padded
    // by less than 1024 slots and the matrix holds fewer than 2^31 entries
    __shared__ uint32_t s_off[kSegs + 1];
    __shared__ long long s_dst[kSegs];         // first slab slot of each segment
    __shared__ int s_start[kSegs];
    __shared__ int s_fill[kSegs];
    __shared__ uint32_t s_len[kSegs];
    __shared__ uint32_t s_wave[kBlock / 64];
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    for (int p0 = 0; p0 < v.parts; p0 += kPartGroup) {
        const int pg = min(kPartGroup, v.parts - p0);
        uint32_t vl[kPartGroup];
#pragma unroll
        for (int pp = 0; pp < kPartGroup; ++pp) {
            vl[pp] = 0;
            if (pp >= pg) continue;                    // uniform
            const int p = p0 + pp;
            const int32_t* w = wtab + p * kWtabStride;
            const int n = w[0];
            const int kbase = w[12];
            int start = 0, fill = 0, mine = -1, width = 1, n_ell = 0;
            if (r < v.rows && n > 0) {
                seg_range(v, r, p, start, fill);
                if (fill > 0) {
                    const int deg = seg_deg ? seg_deg[(int64_t)p * v.rows + r] : fill;
                    mine = pick_bucket(w, n, deg);
                    width = w[1 + mine];
                    n_ell = (fill + width - 1) / width;
                }
            }
            // ELL rows of the same bucket that precede this segment inside its wavefront.  Only
            // the widest bucket splits segments; where every segment is one ELL row a bit count
            // does it.
            int in_wave = 0;
            for (int b = 0; b < n; ++b) {
                const unsigned long long members = __ballot(mine == b);
                if (__ballot(mine == b && n_ell != 1) == 0) {
                    if (mine == b) in_wave = __popcll(members & ((1ull << lane) - 1ull));
                    if (lane == 0) s_cnt[wave][b] = __popcll(members);
                } else {
                    const int x = mine == b ? n_ell : 0;
                    int incl = x;
                    for (int d = 1; d < 64; d <<= 1) {
                        const int y = __shfl_up(incl, d);
                        if (lane >= d) incl += y;
                    }
                    if (mine == b) in_wave = incl - x;
                    if (lane == 63) s_cnt[wave][b] = incl;
                }
            }
            __syncthreads();
            long long first = 0;      // flat ELL-row index of this segment's first ELL row
            long long dst = 0;
            if (mine >= 0) {
                int wave_off = 0;
                for (int wv = 0; wv < wave; ++wv) wave_off += s_cnt[wv][mine];
                const BucketOffsets bo = offs[kbase + mine];
                const long long local = (long long)blockoff[(int64_t)(kbase + mine) * nblk + blockIdx.x] + wave_off + in_wave;
                first = bo.row_off + local;
                dst = bo.slot_off + local * width;
            }
            const uint32_t slen = (uint32_t)n_ell * (uint32_t)width;   // slots of the segment's ELL rows
            vl[pp] = (slen + 3u) & ~3u;
            const int idx = threadIdx.x * pg + pp;
            s_dst[idx] = dst;
            s_start[idx] = start;
            s_fill[idx] = fill;
            s_len[idx] = slen;

            const bool is_long = n_ell > 8;
            if (n_ell > 0 && !is_long) {
                for (int i = 0; i < n_ell; ++i) {
                    const int len = min(width, fill - i * width);
                    out_rows[first + i] = (int32_t)r;
                    out_meta[first + i] = make_meta(len, i, n_ell);
                }
            }
            unsigned long long pending = __ballot(is_long);
            while (pending) {
                const int src = __ffsll((long long)pending) - 1;
                pending &= pending - 1;
                const long long f0 = __shfl(first, src);
                const int fl = __shfl(fill, src);
                const int wd = __shfl(width, src);
                const int ne = __shfl(n_ell, src);
                const int rr = (int)((int64_t)blockIdx.x * kBlock + (wave << 6) + src);
                for (int i = lane; i < ne; i += 64) {
                    const int len = min(wd, fl - i * wd);
                    out_rows[f0 + i] = rr;
                    out_meta[f0 + i] = make_meta(len, i, ne);
                }
            }
            __syncthreads();          // s_cnt is rewritten for the next partition
        }

        // exclusive prefix of the padded lengths over (row, partition)
        uint32_t mine_total = 0;
#pragma unroll
        for (int pp = 0; pp < kPartGroup; ++pp) mine_total += vl[pp];
        uint32_t vincl = mine_total;
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t y = __shfl_up(vincl, d);
            if (lane >= d) vincl += y;
        }
        if (lane == 63) s_wave[wave] = vincl;
        __syncthreads();
        uint32_t voff = vincl - mine_total;
        for (int wv = 0; wv < wave; ++wv) voff += s_wave[wv];
#pragma unroll
        for (int pp = 0; pp < kPartGroup; ++pp) {
            if (pp < pg) s_off[threadIdx.x * pg + pp] = voff;
            voff += vl[pp];
        }
        if (threadIdx.x == kBlock - 1) s_off[kBlock * pg] = voff;
        __syncthreads();

        // groups of four consecutive slots; the prefix sums are multiples of four, so a group
        // never straddles two segments
        const int n_seg = kBlock * pg;
        const int steps = 8 + (pg > 1) + (pg > 2);       // ceil(log2(n_seg))
        const uint32_t total = s_off[n_seg];
        for (uint32_t j0 = 0; j0 < total; j0 += kBlock * kFillUnroll * 4) {
            long long at[kFillUnroll];
            int len[kFillUnroll];                     // slots of the group inside its segment (0: none)
            int4 c[kFillUnroll];
            float4 x[kFillUnroll], m[kFillUnroll];
#pragma unroll
            for (int u = 0; u < kFillUnroll; ++u) {
                const uint32_t j = j0 + (u * kBlock + threadIdx.x) * 4;
                at[u] = 0;
                len[u] = 0;
                c[u] = make_int4(0, 0, 0, 0);
                x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                m[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (j < total) {
                    int lo = 0, hi = n_seg - 1;        // last segment whose offset is <= j
                    for (int step = 0; step < steps; ++step) {
                        const int mid = (lo + hi + 1) >> 1;
                        if (s_off[mid] <= j) lo = mid; else hi = mid - 1;
                    }
                    const int q = (int)(j - s_off[lo]);
                    const int live = s_fill[lo] - q;  // entries of the source row from q on
                    at[u] = s_dst[lo] + q;
                    len[u] = min(4, (int)s_len[lo] - q);
                    const int src = s_start[lo] + q;
                    if (live >= 4) {
                        const Packed4i ci = *reinterpret_cast<const Packed4i*>(indices + src);
                        c[u] = make_int4(ci.x, ci.y, ci.z, ci.w);
                        if (values) {
                            const Packed4f xv = *reinterpret_cast<const Packed4f*>(values + src);
                            x[u] = make_float4(xv.x, xv.y, xv.z, xv.w);
                        } else {
                            x[u] = make_float4(1.f, 1.f, 1.f, 1.f);
                        }
                        m[u] = make_float4(1.f, 1.f, 1.f, 1.f);
                    } else {
                        if (live > 0) { c[u].x = indices[src];     x[u].x = values ? values[src] : 1.f;     m[u].x = 1.f; }
                        if (live > 1) { c[u].y = indices[src + 1]; x[u].y = values ? values[src + 1] : 1.f; m[u].y = 1.f; }
                        if (live > 2) { c[u].z = indices[src + 2]; x[u].z = values ? values[src + 2] : 1.f; m[u].z = 1.f; }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kFillUnroll; ++u) {
                if (len[u] == 4 && (at[u] & 3) == 0) {
                    *reinterpret_cast<int4*>(out_cols + at[u]) = c[u];
                    *reinterpret_cast<float4*>(out_vals + at[u]) = x[u];
                    if (out_mask) *reinterpret_cast<float4*>(out_mask + at[u]) = m[u];
                } else {
                    const int cc[4] = {c[u].x, c[u].y, c[u].z, c[u].w};
                    const float xx[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
                    const float mm[4] = {m[u].x, m[u].y, m[u].z, m[u].w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (i < len[u]) {
                            out_cols[at[u] + i] = cc[i];
                            out_vals[at[u] + i] = xx[i];
                            if (out_mask) out_mask[at[u] + i] = mm[i];
                        }
                    }
                }
            }
        }
        __syncthreads();          // the tables are rewritten for the next group of partitions
    }
}

// ---------------------------------------------------------------------------- host helpers
struct StatsLayout {
    size_t bnd, planes, stats, hist, total;
};

StatsLayout stats_layout(int64_t rows, int64_t cols, int parts) {
    StatsLayout L{};
    size_t off = 0;
    L.bnd = off;
    if (parts > 1) off += align_up((size_t)(parts + 1) * rows * 4, 256);
    L.planes = off;
    off += align_up((size_t)LF_MAX_CLASSES * (size_t)cols, 256);
    L.stats = off;
    off += align_up((size_t)parts * LF_MAX_CLASSES * LF_STATS_FIELDS * 8, 256);
    L.hist = off;
    off += align_up((size_t)parts * (1 << LF_MAX_CLASSES) * 8, 256);
    L.total = off;
    return L;
}

struct HybLayout {
    size_t bnd, wtab, flags, totals, row_off, scatter, blockcnt, total;
    int nblk;
};

HybLayout hyb_layout(int64_t rows, int parts, int total_buckets) {
    HybLayout L{};
    L.nblk = (int)((rows + kBlock - 1) / kBlock);
    if (L.nblk < 1) L.nblk = 1;
    size_t off = 0;
    L.bnd = off;
    if (parts > 1) off += align_up((size_t)(parts + 1) * rows * 4, 256);
    L.wtab = off;
    off += align_up((size_t)parts * kWtabStride * 4, 256);
    L.flags = off;
    off += 256;
    L.totals = off;
    off += align_up((size_t)std::max(total_buckets, 1) * 8, 256);
    L.row_off = off;
    off += align_up((size_t)std::max(total_buckets, 1) * 8, 256);
    L.scatter = off;
    off += align_up((size_t)std::max(total_buckets, 1) * sizeof(BucketOffsets), 256);
    L.blockcnt = off;
    off += align_up((size_t)std::max(total_buckets, 1) * L.nblk * 4, 256);
    L.total = off;
    return L;
}

// Flat slab layout shared by the builder and its callers: ELL rows of bucket k start at a
// multiple of 64 entries, its slots at a multiple of the scatter workgroup span (1024
// slots), so every slab is at least 256-byte aligned inside 256-byte aligned allocations.
constexpr int64_t kRowAlign = 64;
constexpr int64_t kSlotAlign = 1024;   // a bucket's slots start at a multiple of this in the flat slab arrays

void flat_layout(const int64_t* ell_rows, const int32_t* widths, int nb, int64_t* row_off,
                 int64_t* slot_off, int64_t* total_rows, int64_t* total_slots) {
    int64_t r = 0, s = 0;
    for (int k = 0; k < nb; ++k) {
        row_off[k] = r;
        slot_off[k] = s;
        r += (ell_rows[k] + kRowAlign - 1) / kRowAlign * kRowAlign;
        s += (ell_rows[k] * widths[k] + kSlotAlign - 1) / kSlotAlign * kSlotAlign;
    }
    *total_rows = r;
    *total_slots = s;
}

int check_common(const int32_t* d_indptr, const int32_t* d_indices, int64_t rows, int64_t cols, int parts) {
    LF_REQUIRE(d_indptr != nullptr, LF_ERR_INVALID, "indptr is null");
    LF_REQUIRE(rows >= 0 && cols >= 1, LF_ERR_INVALID, "bad shape %lld x %lld", (long long)rows, (long long)cols);
    LF_REQUIRE(rows < (1ll << 31) && cols < (1ll << 31), LF_ERR_UNSUPPORTED, "shape exceeds int32 indices");
    LF_REQUIRE(parts >= 1 && parts <= 65535, LF_ERR_INVALID, "num_parts must be in 1..65535 (got %d)", parts);
    (void)d_indices;
    return LF_OK;
}

int check_widths(int parts, const int32_t* flat, const int32_t* off) {
    LF_REQUIRE(flat && off, LF_ERR_INVALID, "width table is null");
    LF_REQUIRE(off[0] == 0, LF_ERR_INVALID, "widths_off[0] must be 0");
    for (int p = 0; p < parts; ++p) {
        const int n = off[p + 1] - off[p];
        LF_REQUIRE(n >= 0 && n <= LF_MAX_CLASSES, LF_ERR_INVALID,
                   "partition %d has %d widths (max %d)", p, n, LF_MAX_CLASSES);
        for (int b = 0; b < n; ++b) {
            const int w = flat[off[p] + b];
            LF_REQUIRE(lf::is_pow2(w) && w <= (1 << (LF_MAX_CLASSES - 1)), LF_ERR_INVALID,
                       "invalid padding for col_indices[%d][%d] and bucket_width=%d", p, b, w);
            LF_REQUIRE(b == 0 || flat[off[p] + b - 1] < w, LF_ERR_INVALID,
                       "widths of partition %d are not strictly ascending", p);
        }
    }
    return LF_OK;
}

}  // namespace

// ============================================================================ C ABI
extern "C" {

size_t lf_stats_workspace_bytes(int64_t num_rows, int64_t num_cols, int32_t num_parts) {
    if (num_rows < 0 || num_cols < 0 || num_parts < 1) return 0;
    return stats_layout(num_rows, num_cols, num_parts).total;
}

const int32_t* lf_stats_seg_bounds(const void* d_stats_workspace, int64_t num_rows, int32_t num_parts) {
    if (d_stats_workspace == nullptr || num_parts <= 1 || num_rows <= 0) return nullptr;
    return (const int32_t*)((const char*)d_stats_workspace + stats_layout(num_rows, 1, num_parts).bnd);
}

int lf_coo_degrees(const int32_t* d_coo_row, const int32_t* d_coo_col, int64_t nnz, int64_t num_rows,
                   int64_t num_cols, int32_t num_parts, int32_t* d_seg_deg, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(d_seg_deg, LF_ERR_INVALID, "seg_deg is null");
    LF_REQUIRE(nnz == 0 || (d_coo_row && d_coo_col), LF_ERR_INVALID, "COO arrays are null");
    LF_REQUIRE(num_parts >= 1 && num_cols >= 1, LF_ERR_INVALID, "bad num_parts / num_cols");
    const int64_t psize = lf::ceil_div(num_cols, num_parts);
    LF_HIP(fill_u32(d_seg_deg, (int64_t)num_parts * num_rows, 0u, s));
    if (nnz > 0) {
        const int grid = (int)std::min<int64_t>((nnz + 255) / 256, 65535);
        coo_degree_kernel<<<grid, 256, 0, s>>>(d_coo_row, d_coo_col, nnz, num_rows, psize, d_seg_deg);
        LF_HIP(hipGetLastError());
    }
    return LF_OK;
}

int lf_bucket_stats(const int32_t* d_indptr, const int32_t* d_indices, const int32_t* d_seg_deg,
                    int64_t num_rows, int64_t num_cols, int32_t num_parts, int32_t width_limit,
                    void* d_workspace, size_t workspace_bytes, int64_t* h_stats, int64_t* h_colhist,
                    lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    if (int rc = check_common(d_indptr, d_indices, num_rows, num_cols, num_parts)) return rc;
    LF_REQUIRE(h_stats, LF_ERR_INVALID, "h_stats is null");
    LF_REQUIRE(lf::is_pow2(width_limit) && width_limit <= (1 << (LF_MAX_CLASSES - 1)), LF_ERR_INVALID,
               "width_limit must be a power of two <= %d", 1 << (LF_MAX_CLASSES - 1));
    const StatsLayout L = stats_layout(num_rows, num_cols, num_parts);
    LF_REQUIRE(d_workspace && workspace_bytes >= L.total, LF_ERR_WORKSPACE,
               "workspace has %zu bytes, %zu needed", workspace_bytes, L.total);
    char* ws = (char*)d_workspace;
    int32_t* bnd = (int32_t*)(ws + L.bnd);
    uint8_t* planes = (uint8_t*)(ws + L.planes);
    unsigned long long* stats = (unsigned long long*)(ws + L.stats);
    unsigned long long* hist = (unsigned long long*)(ws + L.hist);
    const int64_t psize = lf::ceil_div(num_cols, num_parts);
    const size_t stats_bytes = (size_t)num_parts * LF_MAX_CLASSES * LF_STATS_FIELDS * 8;
    const size_t hist_bytes = (size_t)num_parts * (1 << LF_MAX_CLASSES) * 8;

    if (h_colhist)
        LF_HIP(fill_u32(planes, (L.total - L.planes) / 4, 0u, s));   // planes, stats and hist
    else
        LF_HIP(fill_u32(stats, (L.total - L.stats) / 4, 0u, s));
    if (num_rows > 0) {
        const int nblk = (int)((num_rows + kBlock - 1) / kBlock);
        if (num_parts > 1) {
            seg_bounds_kernel<<<nblk, kBlock, 0, s>>>(d_indptr, d_indices, num_rows, num_parts, psize, bnd);
            LF_HIP(hipGetLastError());
        }
        SegView v{d_indptr, bnd, num_rows, num_parts};
        const int num_classes = lf::ilog2(width_limit) + 1;
        bucket_stats_kernel<<<dim3(std::min(nblk, kStatsGrid), num_parts, h_colhist ? num_classes : 1), kBlock, 0, s>>>(
            v, d_indices, d_seg_deg, num_classes - 1, h_colhist ? planes : nullptr, num_cols, stats);
        LF_HIP(hipGetLastError());
        if (h_colhist) {
            const int hgrid = (int)std::min<int64_t>((psize + kBlock - 1) / kBlock, 1024);
            colmask_hist_kernel<<<dim3(hgrid, num_parts), kBlock, 0, s>>>(planes, num_classes, num_cols, psize, hist);
            LF_HIP(hipGetLastError());
        }
    }
    LF_HIP(hipMemcpyAsync(h_stats, stats, stats_bytes, hipMemcpyDeviceToHost, s));
    if (h_colhist) LF_HIP(hipMemcpyAsync(h_colhist, hist, hist_bytes, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    return LF_OK;
}

int lf_row_features(const int32_t* d_indptr, int64_t num_rows, void* d_scratch, int64_t* h_out,
                    lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(h_out, LF_ERR_INVALID, "h_out is null");
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31), LF_ERR_INVALID, "bad num_rows");
    h_out[0] = h_out[1] = h_out[2] = h_out[3] = 0;
    if (num_rows == 0) return LF_OK;
    LF_REQUIRE(d_indptr && d_scratch, LF_ERR_INVALID, "null argument");
    LF_REQUIRE((uintptr_t)d_scratch % 8 == 0, LF_ERR_INVALID, "scratch must be 8-byte aligned");
    unsigned long long* acc = (unsigned long long*)d_scratch;
    LF_HIP(fill_u32(acc, 2, 0xFFFFFFFFu, s));
    LF_HIP(fill_u32(acc + 1, 6, 0u, s));
    const int grid = (int)std::min<int64_t>((num_rows + kBlock - 1) / kBlock, 1024);
    row_features_kernel<<<grid, kBlock, 0, s>>>(d_indptr, num_rows, acc);
    LF_HIP(hipGetLastError());
    LF_HIP(hipMemcpyAsync(h_out, acc, 32, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    return LF_OK;
}

int lf_row_overlap(const int32_t* d_indptr, const int32_t* d_indices, int64_t num_rows, int64_t sample_stride,
                   void* d_scratch, int64_t* h_out, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(h_out, LF_ERR_INVALID, "h_out is null");
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && sample_stride >= 1, LF_ERR_INVALID, "bad num_rows / stride");
    h_out[0] = h_out[1] = 0;
    if (num_rows < 2) return LF_OK;
    LF_REQUIRE(d_indptr && d_indices && d_scratch, LF_ERR_INVALID, "null argument");
    LF_REQUIRE((uintptr_t)d_scratch % 8 == 0, LF_ERR_INVALID, "scratch must be 8-byte aligned");
    unsigned long long* acc = (unsigned long long*)d_scratch;
    LF_HIP(fill_u32(acc, 4, 0u, s));
    const int64_t samples = (num_rows - 1 + sample_stride - 1) / sample_stride;
    const int grid = (int)std::min<int64_t>((samples + kBlock - 1) / kBlock, 1024);
    row_overlap_kernel<<<grid, kBlock, 0, s>>>(d_indptr, d_indices, num_rows, sample_stride, acc);
    LF_HIP(hipGetLastError());
    LF_HIP(hipMemcpyAsync(h_out, acc, 16, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    return LF_OK;
}

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
unsigned long long* g_scratch_ptr[kMaxDevices];     // device address of lf_static_scratch, per device

// Address of the current device's copy of lf_static_scratch, looked up once per device.
int static_scratch(unsigned long long** out) {
    int dev = -1;
    LF_HIP(hipGetDevice(&dev));
    LF_REQUIRE(dev >= 0 && dev < kMaxDevices, LF_ERR_UNSUPPORTED, "device index %d is out of range", dev);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        LF_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(lf_static_scratch)));
        LF_REQUIRE(p != nullptr, LF_ERR_HIP, "hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = (unsigned long long*)p;
    }
    *out = g_scratch_ptr[dev];
    return LF_OK;
}

__global__ void copy_features_kernel(const unsigned long long* __restrict__ acc, int64_t* __restrict__ out) {
    if (threadIdx.x < 4) out[threadIdx.x] = (int64_t)acc[threadIdx.x];
}

}  // namespace

int lf_row_features_static(const int32_t* d_indptr, int64_t num_rows, int64_t* d_out, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(d_out, LF_ERR_INVALID, "d_out is null");
    LF_REQUIRE(num_rows >= 0, LF_ERR_INVALID, "bad num_rows");
    LF_REQUIRE(num_rows <= LF_ROW_FEATURES_STATIC_MAX_ROWS, LF_ERR_UNSUPPORTED,
               "lf_row_features_static handles at most %lld rows (got %lld)",
               (long long)LF_ROW_FEATURES_STATIC_MAX_ROWS, (long long)num_rows);
    LF_REQUIRE(num_rows == 0 || d_indptr, LF_ERR_INVALID, "indptr is null");
    LF_REQUIRE((uintptr_t)d_out % 8 == 0, LF_ERR_INVALID, "d_out must be 8-byte aligned");
    unsigned long long* acc = nullptr;
    if (int rc = static_scratch(&acc)) return rc;
    // the array keeps the last call's values: min starts at all ones, the rest at zero
    // (num_rows == 0: the minimum is cleared too, which gives {0, 0, 0, 0})
    LF_HIP(fill_u32(acc, 2, num_rows > 0 ? 0xFFFFFFFFu : 0u, s));
    LF_HIP(fill_u32(acc + 1, 6, 0u, s));
    if (num_rows > 0) {
        const int grid = (int)std::min<int64_t>((num_rows + kBlock - 1) / kBlock, 1024);
        row_features_kernel<<<grid, kBlock, 0, s>>>(d_indptr, num_rows, acc);
        LF_HIP(hipGetLastError());
    }
    copy_features_kernel<<<1, 64, 0, s>>>(acc, d_out);
    LF_HIP(hipGetLastError());
    return LF_OK;
}

size_t lf_hyb_workspace_bytes(int64_t num_rows, int32_t num_parts, int32_t total_buckets) {
    if (num_rows < 0 || num_parts < 1 || total_buckets < 0) return 0;
    return hyb_layout(num_rows, num_parts, total_buckets).total;
}

int lf_hyb_layout(const int64_t* h_ell_rows, const int32_t* h_widths_flat, int32_t total_buckets,
                  int64_t* h_row_off, int64_t* h_slot_off, int64_t* h_total_rows, int64_t* h_total_slots) {
    LF_REQUIRE(total_buckets >= 0, LF_ERR_INVALID, "negative bucket count");
    LF_REQUIRE(h_total_rows && h_total_slots, LF_ERR_INVALID, "null output");
    LF_REQUIRE(total_buckets == 0 || (h_ell_rows && h_widths_flat && h_row_off && h_slot_off), LF_ERR_INVALID,
               "null argument");
    flat_layout(h_ell_rows, h_widths_flat, total_buckets, h_row_off, h_slot_off, h_total_rows, h_total_slots);
    return LF_OK;
}

int lf_hyb_plan(const int32_t* d_indptr, const int32_t* d_indices, const int32_t* d_seg_deg,
                const int32_t* d_seg_bounds, int64_t num_rows, int64_t num_cols, int32_t num_parts, const int32_t* h_widths_flat,
                const int32_t* h_widths_off, void* d_workspace, size_t workspace_bytes,
                int64_t* h_ell_rows, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    if (int rc = check_common(d_indptr, d_indices, num_rows, num_cols, num_parts)) return rc;
    if (int rc = check_widths(num_parts, h_widths_flat, h_widths_off)) return rc;
    const int nb = h_widths_off[num_parts];
    LF_REQUIRE(h_ell_rows || nb == 0, LF_ERR_INVALID, "h_ell_rows is null");
    const HybLayout L = hyb_layout(num_rows, num_parts, nb);
    LF_REQUIRE(d_workspace && workspace_bytes >= L.total, LF_ERR_WORKSPACE,
               "workspace has %zu bytes, %zu needed", workspace_bytes, L.total);
    char* ws = (char*)d_workspace;
    int32_t* bnd = (int32_t*)(ws + L.bnd);
    int32_t* wtab = (int32_t*)(ws + L.wtab);
    int32_t* flags = (int32_t*)(ws + L.flags);
    long long* totals = (long long*)(ws + L.totals);
    int32_t* blockcnt = (int32_t*)(ws + L.blockcnt);
    const int64_t psize = lf::ceil_div(num_cols, num_parts);

    std::vector<int32_t> h_wtab((size_t)num_parts * kWtabStride, 0);
    for (int p = 0; p < num_parts; ++p) {
        const int n = h_widths_off[p + 1] - h_widths_off[p];
        h_wtab[(size_t)p * kWtabStride] = n;
        for (int b = 0; b < n; ++b) h_wtab[(size_t)p * kWtabStride + 1 + b] = h_widths_flat[h_widths_off[p] + b];
        h_wtab[(size_t)p * kWtabStride + 12] = h_widths_off[p];
    }
    LF_HIP(hipMemcpyAsync(wtab, h_wtab.data(), h_wtab.size() * 4, hipMemcpyHostToDevice, s));
    LF_HIP(hipStreamSynchronize(s));     // h_wtab is pageable and about to go out of scope
    LF_HIP(fill_u32(flags, 64, 0u, s));
    LF_HIP(fill_u32(totals, (int64_t)std::max(nb, 1) * 2, 0u, s));
    if (num_rows > 0) {
        if (num_parts > 1 && d_seg_bounds) {       // bounds already known (the statistics pass made them)
            LF_HIP(hipMemcpyAsync(bnd, d_seg_bounds, (size_t)(num_parts + 1) * num_rows * 4,
                                  hipMemcpyDeviceToDevice, s));
        } else if (num_parts > 1) {
            seg_bounds_kernel<<<L.nblk, kBlock, 0, s>>>(d_indptr, d_indices, num_rows, num_parts, psize, bnd);
            LF_HIP(hipGetLastError());
        }
        SegView v{d_indptr, bnd, num_rows, num_parts};
        hyb_count_kernel<<<dim3(L.nblk, num_parts), kBlock, 0, s>>>(v, d_seg_deg, wtab, L.nblk, blockcnt, flags);
        LF_HIP(hipGetLastError());
        if (nb > 0) {
            hyb_scan_kernel<<<nb, 1024, 0, s>>>(blockcnt, L.nblk, totals);
            LF_HIP(hipGetLastError());
        }
    }
    int32_t h_flags = 0;
    std::vector<long long> h_tot((size_t)std::max(nb, 1), 0);
    LF_HIP(hipMemcpyAsync(&h_flags, flags, 4, hipMemcpyDeviceToHost, s));
    if (nb > 0) LF_HIP(hipMemcpyAsync(h_tot.data(), totals, (size_t)nb * 8, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    if (h_flags & 1)
        return lf::fail(LF_ERR_CONFIG, "list index out of range: a partition with nonzeros has no bucket widths");
    if (h_flags & 2)
        return lf::fail(LF_ERR_UNSUPPORTED, "a row is split over more than %d ELL rows", kMetaSegMax);
    for (int k = 0; k < nb; ++k) h_ell_rows[k] = h_tot[k];
    return LF_OK;
}

int lf_hyb_build(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                 const int32_t* d_seg_deg, int64_t num_rows, int64_t num_cols, int32_t num_parts,
                 const int32_t* h_widths_flat, const int32_t* h_widths_off, const int64_t* h_ell_rows,
                 void* d_workspace, size_t workspace_bytes, int32_t* d_rows, int32_t* d_meta,
                 int32_t* d_cols, float* d_vals, float* d_mask, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    if (int rc = check_common(d_indptr, d_indices, num_rows, num_cols, num_parts)) return rc;
    if (int rc = check_widths(num_parts, h_widths_flat, h_widths_off)) return rc;
    const int nb = h_widths_off[num_parts];
    if (nb == 0 || num_rows == 0) return LF_OK;
    LF_REQUIRE(h_ell_rows, LF_ERR_INVALID, "h_ell_rows is null");
    int64_t total_rows = 0;
    for (int k = 0; k < nb; ++k) {
        LF_REQUIRE(h_ell_rows[k] >= 0, LF_ERR_INVALID, "negative ELL row count");
        total_rows += h_ell_rows[k];
    }
    if (total_rows == 0) return LF_OK;
    LF_REQUIRE(d_rows && d_meta && d_cols && d_vals && d_indices, LF_ERR_INVALID, "slab pointers are null");
    const HybLayout L = hyb_layout(num_rows, num_parts, nb);
    LF_REQUIRE(d_workspace && workspace_bytes >= L.total, LF_ERR_WORKSPACE,
               "workspace has %zu bytes, %zu needed", workspace_bytes, L.total);
    char* ws = (char*)d_workspace;
    int32_t* bnd = (int32_t*)(ws + L.bnd);
    int32_t* wtab = (int32_t*)(ws + L.wtab);
    BucketOffsets* offs = (BucketOffsets*)(ws + L.scatter);
    int32_t* blockoff = (int32_t*)(ws + L.blockcnt);

    std::vector<BucketOffsets> h_offs((size_t)nb);
    std::vector<int64_t> roff((size_t)nb), soff((size_t)nb);
    int64_t flat_rows, flat_slots;
    flat_layout(h_ell_rows, h_widths_flat, nb, roff.data(), soff.data(), &flat_rows, &flat_slots);
    for (int k = 0; k < nb; ++k) {
        h_offs[k].slot_off = soff[k];
        h_offs[k].row_off = roff[k];
    }
    LF_HIP(hipMemcpyAsync(offs, h_offs.data(), (size_t)nb * sizeof(BucketOffsets), hipMemcpyHostToDevice, s));
    LF_HIP(hipStreamSynchronize(s));     // the pageable source goes out of scope below

    SegView v{d_indptr, bnd, num_rows, num_parts};
    hyb_fill_kernel<<<L.nblk, kBlock, 0, s>>>(v, d_seg_deg, wtab, L.nblk, blockoff, offs, d_indices, d_values,
                                              d_rows, d_meta, d_cols, d_vals, d_mask);
    LF_HIP(hipGetLastError());
    return LF_OK;
}

}  // extern "C"
