// Fused hyb SpMM for gfx950 (MI355X):  C[rows][N] = A_hyb . B[cols][N], fp32 accumulate.
//
// Takes over the kernel that the reference generates through SparseTIR/TVM in
// bench_hyb_with_config (playground_pipline/format_algos.py:388-605): all (partition,
// bucket) ELL blocks of the hyb format are walked by one launch per column partition.
// The reference binds 32 threads to 32 features and 8 ELL rows to a thread block and uses
// atomicAdd where several ELL rows feed one output row (format_algos.py:508-533).  Here:
//
//   * a "sub-wave" of LPR lanes owns one ELL row at a time; each lane holds VEC consecutive
//     features (float4, or 8 x bf16 = 16 bytes), so one B row is read with one 16-byte load
//     per lane, coalesced along the feature dimension (N = 128 fp32 -> 32 lanes, two rows
//     per 64-lane wavefront);
//   * narrow buckets stage their (column, value) tile in LDS with coalesced 16-byte loads
//     and read it back as broadcasts; wide buckets and the widest bucket of a partition
//     (whose source rows may span several ELL rows) stream slots through wavefront
//     shuffles instead;
//   * a source row split over several ELL rows is summed by one owner; rows longer than
//     kCoopSlots are reduced by a whole workgroup, kChunkSlots at a time: a row that fits one
//     chunk is written directly, a longer one leaves one partial row per chunk and a small
//     second kernel adds the partials in chunk order;
//   * partitions run as consecutive launches: partition 0 stores every output row (rows it
//     does not touch are cleared by the same launch), later partitions add.  Nothing
//     depends on scheduling, so results are bit-reproducible, and there are no atomics.
//
// The workgroup -> tile mapping is XCD-aware: workgroup i runs on XCD i % 8, and each
// group of tiles is cut into 8 contiguous ranges, one per XCD, so that neighbouring ELL
// rows (which tend to share B rows in structured matrices) meet in the same L2.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "lf_cells.h"
#include "lf_internal.h"
#include "lf_spmm_device.h"

namespace {

// Sum of `total` consecutive slab slots starting at `base`, streamed by one sub-wave: each
// lane loads one (col, val), the sub-wave then walks them by shuffle.  Slots past `total`
// are replaced by (first column, 0) so that every gather is unconditional and in range.
template <int LPR, int CH, typename BT>
__device__ __forceinline__ void stream_slots(const int32_t* __restrict__ cols, const float* __restrict__ vals,
                                             long long base, int total, const void* B,
                                             const Lane<LPR, CH, Dense<BT>::kVec>& ln,
                                             Acc<CH, Dense<BT>::kVec>& acc) {
    constexpr int U = kUnroll < LPR ? kUnroll : LPR;
    if (total <= 0) return;
    const int c_first = cols[base];
    // the next batch of slots is requested before the current one is walked: a slab is read
    // once, so each of these loads waits out the full memory latency
    int next_c = ln.sl < total ? cols[base + ln.sl] : c_first;
    float next_v = ln.sl < total ? (vals ? vals[base + ln.sl] : 1.f) : 0.f;
    for (int off = 0; off < total; off += LPR) {
        const int my_c = next_c;
        const float my_v = next_v;
        const int idx = off + LPR + ln.sl;
        const bool have = idx < total;
        next_c = have ? cols[base + idx] : c_first;
        next_v = have ? (vals ? vals[base + idx] : 1.f) : 0.f;
        const int cnt = min(LPR, total - off);
        for (int j = 0; j < cnt; j += U) {
            int c[U];
            float v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                c[u] = __shfl(my_c, j + u, LPR);
                v[u] = __shfl(my_v, j + u, LPR);
            }
            gather_fma<U, LPR, CH, BT>(B, ln, c, v, acc);
        }
    }
}

// ------------------------------------------------------------------------------------
// Tile bodies.  s_pairs / s_rm point into the workgroup's LDS: tile_slots(LPR) (col, val)
// pairs followed by kTileRows (row, meta) entries.

// Narrow bucket: W slots per ELL row, rows independent (one ELL row per source row).
// RPI rows are processed together by a sub-wave so that kUnroll gathers are in flight
// even when W < kUnroll.
template <int W, int LPR, int CH, typename BT>
__device__ __forceinline__ void ell_tile_narrow(const int2* s_pairs, const int2* s_rm, int n,
                                                const LaunchArgs& a, int sw, int sl) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    constexpr int RPI = kUnroll / W;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    for (int r0 = sw * RPI; r0 < n; r0 += SW * RPI) {
        Acc<CH, VEC> acc[RPI];
        int c[kUnroll];
        float v[kUnroll];
#pragma unroll
        for (int q = 0; q < RPI; ++q) {
            acc[q].clear();
            const int r = min(r0 + q, n - 1);
            const int len = s_rm[r].y & kMetaLenMask;
            const int c0 = s_pairs[r * W].x;
#pragma unroll
            for (int j = 0; j < W; ++j) {
                const int2 cv = s_pairs[r * W + j];
                c[q * W + j] = j < len ? cv.x : c0;
                v[q * W + j] = __int_as_float(cv.y);
            }
        }
        {
            float x[kUnroll][CH][VEC];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int cc = 0; cc < CH; ++cc)
                    Dense<BT>::load(dense_row<BT>(a.B, ln, cc, c[u]), x[u][cc]);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int cc = 0; cc < CH; ++cc)
#pragma unroll
                    for (int i = 0; i < VEC; ++i)
                        acc[u / W].v[cc][i] = fmaf(v[u], x[u][cc][i], acc[u / W].v[cc][i]);
        }
#pragma unroll
        for (int q = 0; q < RPI; ++q)
            if (r0 + q < n) store_row<LPR, CH, VEC>(a.C, s_rm[r0 + q].x, ln, acc[q], a.accumulate);
    }
}

// U staged slots of an ELL row from position j; slots at or past `len` are padding and are
// redirected to the row's first column (their value is 0).
template <int U, int LPR, int CH, typename BT>
__device__ __forceinline__ void staged_group(const int2* rp, int j, int len, int c0, const void* B,
                                             const Lane<LPR, CH, Dense<BT>::kVec>& ln,
                                             Acc<CH, Dense<BT>::kVec>& acc) {
    int c[U];
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int2 cv = rp[j + u];
        c[u] = j + u < len ? cv.x : c0;
        v[u] = __int_as_float(cv.y);
    }
    gather_fma<U, LPR, CH, BT>(B, ln, c, v, acc);
}

// Bucket with W >= kUnroll (a multiple of it) staged in LDS: one ELL row per sub-wave at a time.
template <int LPR, int CH, typename BT>
__device__ __forceinline__ void ell_tile_wide(const int2* s_pairs, const int2* s_rm, int n, int log_w,
                                              const LaunchArgs& a, int sw, int sl) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    for (int r = sw; r < n; r += SW) {
        const int2 rm = s_rm[r];
        const int len = rm.y & kMetaLenMask;
        const int2* rp = s_pairs + (r << log_w);
        const int c0 = rp[0].x;
        Acc<CH, VEC> acc;
        acc.clear();
        // Whole groups of kUnroll slots, then a tail of kUnroll or kUnroll / 2 gathers.  The
        // short tail saves padding gathers (a 27-slot stencil row: 28 instead of 32); with
        // many rows per wavefront (small N) the extra branch costs more than it saves.
        constexpr bool kShortTail = LPR >= 32;
        if constexpr (kShortTail) {
            int j = 0;
            for (; j + kUnroll <= len; j += kUnroll) staged_group<kUnroll, LPR, CH, BT>(rp, j, len, c0, a.B, ln, acc);
            if (len > j && len - j <= kUnroll / 2) staged_group<kUnroll / 2, LPR, CH, BT>(rp, j, len, c0, a.B, ln, acc);
            else if (len > j) staged_group<kUnroll, LPR, CH, BT>(rp, j, len, c0, a.B, ln, acc);
        } else {
            for (int j = 0; j < len; j += kUnroll) staged_group<kUnroll, LPR, CH, BT>(rp, j, len, c0, a.B, ln, acc);
        }
        store_row<LPR, CH, VEC>(a.C, rm.x, ln, acc, a.accumulate);
    }
}

// Staged tile of a bucket whose source rows may span several consecutive ELL rows (the widest
// bucket of a partition): the first ELL row of a segment owns it.  The part of the segment
// inside the tile is read from LDS, a part that runs past the tile's end is streamed from
// global memory.  Continuation rows and rows that take the cooperative path are skipped.
template <int LPR, int CH, typename BT>
__device__ __forceinline__ void ell_tile_segments(const Group& g, long long e0, const int2* s_pairs,
                                                  const int2* s_rm, int n, const LaunchArgs& a, int* s_next,
                                                  int sl) {
    constexpr int VEC = Dense<BT>::kVec;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    const int log_w = g.log_w;
    // Segments differ in length and continuation rows carry no work, so the sub-waves take
    // the tile's ELL rows from a shared counter as they become free instead of by a fixed
    // stride.  Which sub-wave sums a row does not change the order of its additions.
    for (;;) {
        int r = 0;
        if (sl == 0) r = atomicAdd(s_next, 1);
        r = __shfl(r, 0, LPR);
        if (r >= n) break;
        const int2 rm = s_rm[r];
        if (rm.y < 0) continue;                                  // continuation row
        const int seg = (int)((uint32_t)rm.y >> kMetaLenBits);
        if (((long long)seg << log_w) > kCoopSlots) continue;   // reduced by a whole workgroup
        int total = rm.y & kMetaLenMask;
        if (seg > 1) {
            const int last = r + seg - 1;
            const int last_meta = last < n ? s_rm[last].y : g.meta[e0 + last];
            total = ((seg - 1) << log_w) + (last_meta & kMetaLenMask);
        }
        const int staged = min(total, (n - r) << log_w);
        const int2* rp = s_pairs + (r << log_w);
        const int c0 = rp[0].x;
        Acc<CH, VEC> acc;
        acc.clear();
        for (int j = 0; j < staged; j += kUnroll) {
            int c[kUnroll];
            float v[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const bool in = j + u < staged;
                const int2 cv = rp[in ? j + u : 0];
                c[u] = in ? cv.x : c0;
                v[u] = in ? __int_as_float(cv.y) : 0.f;
            }
            gather_fma<kUnroll, LPR, CH, BT>(a.B, ln, c, v, acc);
        }
        if (total > staged)
            stream_slots<LPR, CH, BT>(g.cols, g.vals, ((e0 + r) << log_w) + staged, total - staged, a.B, ln, acc);
        store_row<LPR, CH, VEC>(a.C, rm.x, ln, acc, a.accumulate);
    }
}

// The same bucket with the work spread evenly: every ELL row of the tile is summed by the
// sub-wave it falls to, a row that is only part of a segment leaves its sum in LDS, and after
// a barrier the first ELL row of each segment adds the sums of its rows in order.  With the
// variant above a tile of a folded configuration offers fewer segments than sub-waves at
// small N (about 20 for 32 at N = 32), and the lanes in flight bound the gather rate.
// Rows that continue a segment begun in an earlier tile are summed by that tile, as above.
template <int LPR, int CH, typename BT>
__device__ __forceinline__ void ell_tile_segments_balanced(const Group& g, long long e0, const int2* s_pairs,
                                                           const int2* s_rm, int n, const LaunchArgs& a,
                                                           float* s_part, int sw, int sl) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    const int log_w = g.log_w;
    for (int r = sw; r < n; r += SW) {
        const int2 rm = s_rm[r];
        const bool cont = rm.y < 0;
        const int head = cont ? r - (int)(((uint32_t)rm.y & 0x7FFFFFFFu) >> kMetaLenBits) : r;
        if (head < 0) continue;                                  // belongs to the previous tile's last segment
        const int seg = (int)((uint32_t)s_rm[head].y >> kMetaLenBits);
        if (((long long)seg << log_w) > kCoopSlots) continue;   // reduced by a whole workgroup
        const int len = rm.y & kMetaLenMask;
        const int2* rp = s_pairs + (r << log_w);
        const int c0 = rp[0].x;
        Acc<CH, VEC> acc;
        acc.clear();
        for (int j = 0; j < len; j += kUnroll) {
            int c[kUnroll];
            float v[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const bool in = j + u < len;          // W may be below kUnroll: stay inside the row
                const int2 cv = rp[in ? j + u : 0];
                c[u] = in ? cv.x : c0;
                v[u] = in ? __int_as_float(cv.y) : 0.f;
            }
            gather_fma<kUnroll, LPR, CH, BT>(a.B, ln, c, v, acc);
        }
        if (seg == 1) {
            store_row<LPR, CH, VEC>(a.C, rm.x, ln, acc, a.accumulate);
        } else {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                if (!ln.on[c]) continue;
                float* dst = s_part + r * a.feat + ln.f[c];
#pragma unroll
                for (int i = 0; i < VEC; i += 4)
                    *reinterpret_cast<float4*>(dst + i) =
                        make_float4(acc.v[c][i], acc.v[c][i + 1], acc.v[c][i + 2], acc.v[c][i + 3]);
            }
        }
    }
    __syncthreads();
    for (int r = sw; r < n; r += SW) {
        const int2 rm = s_rm[r];
        if (rm.y < 0) continue;
        const int seg = (int)((uint32_t)rm.y >> kMetaLenBits);
        if (seg == 1 || ((long long)seg << log_w) > kCoopSlots) continue;
        Acc<CH, VEC> acc;
        acc.clear();
        const int inside = min(seg, n - r);
        for (int k = 0; k < inside; ++k) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                if (!ln.on[c]) continue;
                const float* src = s_part + (r + k) * a.feat + ln.f[c];
#pragma unroll
                for (int i = 0; i < VEC; i += 4) {
                    const float4 x = *reinterpret_cast<const float4*>(src + i);
                    acc.v[c][i] += x.x; acc.v[c][i + 1] += x.y; acc.v[c][i + 2] += x.z; acc.v[c][i + 3] += x.w;
                }
            }
        }
        if (inside < seg) {                                      // the segment runs past the tile: stream the rest
            const int total = ((seg - 1) << log_w) + (g.meta[e0 + r + seg - 1] & kMetaLenMask);
            const int staged = inside << log_w;
            stream_slots<LPR, CH, BT>(g.cols, g.vals, ((e0 + r) << log_w) + staged, total - staged, a.B, ln, acc);
        }
        store_row<LPR, CH, VEC>(a.C, rm.x, ln, acc, a.accumulate);
    }
}

template <int LPR, int CH, typename BT>
__device__ __forceinline__ void run_ell_tile(const Group& g, long long tile, int2* s_pairs, int2* s_rm,
                                             int* s_next, float* s_part, const LaunchArgs& a) {
    const int tid = threadIdx.x;
    const long long e0 = tile * g.rows_per_tile;
    const int n = (int)min((long long)g.rows_per_tile, g.n_items - e0);
    const int n_slots = n << g.log_w;
    const long long s0 = e0 << g.log_w;
    for (int i = tid * 4; i < n_slots; i += kWG * 4) {
        if (i + 4 <= n_slots) {            // s0 and i are multiples of 4, slabs are 16-byte aligned
            const lf_i32x4 c = load_i32x4(g.cols + s0 + i, a.accumulate & kStreamSlabs);
            const lf_i32x4 v = load_i32x4(g.vals + s0 + i, a.accumulate & kStreamSlabs);
            s_pairs[i + 0] = make_int2(c.x, v.x);
            s_pairs[i + 1] = make_int2(c.y, v.y);
            s_pairs[i + 2] = make_int2(c.z, v.z);
            s_pairs[i + 3] = make_int2(c.w, v.w);
        } else {
            for (int k = i; k < n_slots; ++k)
                s_pairs[k] = make_int2(g.cols[s0 + k], __float_as_int(g.vals[s0 + k]));
        }
    }
    for (int i = tid; i < n; i += kWG) s_rm[i] = make_int2(g.rows[e0 + i], g.meta[e0 + i]);
    if (tid == 0) *s_next = 0;
    __syncthreads();
    const int sw = tid / LPR, sl = tid % LPR;
    if (g.type == kEllSeg) {
        if (g.balanced) ell_tile_segments_balanced<LPR, CH, BT>(g, e0, s_pairs, s_rm, n, a, s_part, sw, sl);
        else ell_tile_segments<LPR, CH, BT>(g, e0, s_pairs, s_rm, n, a, s_next, sl);
        return;
    }
    switch (g.log_w) {
        case 0: ell_tile_narrow<1, LPR, CH, BT>(s_pairs, s_rm, n, a, sw, sl); break;
        case 1: ell_tile_narrow<2, LPR, CH, BT>(s_pairs, s_rm, n, a, sw, sl); break;
        case 2: ell_tile_narrow<4, LPR, CH, BT>(s_pairs, s_rm, n, a, sw, sl); break;
        case 3:
            if constexpr (kUnroll > 8) ell_tile_narrow<8, LPR, CH, BT>(s_pairs, s_rm, n, a, sw, sl);
            else ell_tile_wide<LPR, CH, BT>(s_pairs, s_rm, n, g.log_w, a, sw, sl);
            break;
        default: ell_tile_wide<LPR, CH, BT>(s_pairs, s_rm, n, g.log_w, a, sw, sl); break;
    }
}

// Bucket whose source rows may span several ELL rows, or whose rows are too wide to stage:
// the first ELL row of a segment owns it and streams all of its slots; continuation rows
// and segments above kCoopSlots (handled as chunks) are skipped.
template <int LPR, int CH, typename BT>
__device__ __forceinline__ void run_seg_tile(const Group& g, long long tile, const LaunchArgs& a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const int tid = threadIdx.x;
    const int sw = tid / LPR, sl = tid % LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    const long long e0 = tile * g.rows_per_tile;
    const int n = (int)min((long long)g.rows_per_tile, g.n_items - e0);
    for (int r = sw; r < n; r += SW) {
        const long long e = e0 + r;
        const int m = g.meta[e];
        if (m < 0) continue;                                   // continuation row
        const int seg = (int)((uint32_t)m >> kMetaLenBits);
        if (((long long)seg << g.log_w) > kCoopSlots) continue;
        int total = m & kMetaLenMask;
        if (seg > 1) total = ((seg - 1) << g.log_w) + (g.meta[e + seg - 1] & kMetaLenMask);
        Acc<CH, VEC> acc;
        acc.clear();
        stream_slots<LPR, CH, BT>(g.cols, g.vals, e << g.log_w, total, a.B, ln, acc);
        store_row<LPR, CH, VEC>(a.C, g.rows[e], ln, acc, a.accumulate);
    }
}

template <int LPR, int CH, typename BT>
__device__ __forceinline__ void run_zero_tile(const Group& g, long long tile, const LaunchArgs& a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const int tid = threadIdx.x;
    const int sw = tid / LPR, sl = tid % LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    const long long e0 = tile * g.rows_per_tile;
    const int n = (int)min((long long)g.rows_per_tile, g.n_items - e0);
    Acc<CH, VEC> zero;
    zero.clear();
    for (int r = sw; r < n; r += SW) store_row<LPR, CH, VEC>(a.C, g.rows[e0 + r], ln, zero, a.accumulate & kStreamC);
}

// One chunk of a heavy source row: the workgroup's sub-waves take consecutive slices of
// the chunk, their sums are combined through LDS in sub-wave order.
template <int LPR, int CH, typename BT>
__device__ __forceinline__ void run_chunk_tile(const Group& g, long long tile, float* s_red,
                                               const LaunchArgs& a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const int tid = threadIdx.x;
    const int sw = tid / LPR, sl = tid % LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    const Chunk ck = g.chunks[tile];
    int per = (ck.n_slots + SW - 1) / SW;
    per = (per + LPR - 1) / LPR * LPR;
    const int lo = min(sw * per, ck.n_slots);
    const int hi = min(lo + per, ck.n_slots);
    Acc<CH, VEC> acc;
    acc.clear();
    stream_slots<LPR, CH, BT>(g.cols, g.vals, ck.slot_begin + lo, hi - lo, a.B, ln, acc);
    // s_red[sw][c][sl][i]
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < VEC; ++i) s_red[((sw * CH + c) * LPR + sl) * VEC + i] = acc.v[c][i];
    __syncthreads();
    if (sw == 0) {
        Acc<CH, VEC> sum;
        sum.clear();
#pragma unroll
        for (int c = 0; c < CH; ++c)
            for (int s = 0; s < SW; ++s)
#pragma unroll
                for (int i = 0; i < VEC; ++i) sum.v[c][i] += s_red[((s * CH + c) * LPR + sl) * VEC + i];
        if (ck.partial < 0) {
            store_row<LPR, CH, VEC>(a.C, ck.row, ln, sum, a.accumulate);
        } else {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                if (!ln.on[c]) continue;
                float* dst = a.partials + (size_t)ck.partial * a.feat + ln.f[c];
#pragma unroll
                for (int i = 0; i < VEC; i += 4)
                    *reinterpret_cast<float4*>(dst + i) =
                        make_float4(sum.v[c][i], sum.v[c][i + 1], sum.v[c][i + 2], sum.v[c][i + 3]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------
// The fused kernel: one workgroup per tile, all tile groups of one column partition in one
// launch.  Workgroup i runs on XCD i % 8 and takes entry i / 8 of that XCD's tile list: for
// every group the contiguous eighth of its tiles that belongs to the XCD, groups
// concatenated.  The hardware hands out workgroups in index order as slots free up, which
// keeps the tiles in flight on an XCD next to each other and balances the load; a resident
// grid that strides over the tiles measured 2-7 % slower on every workload.
template <int LPR, int CH, typename BT>
__global__ void __launch_bounds__(kWG)
spmm_partition_kernel(LaunchArgs a) {
    // one LDS buffer, used either as the staged tile ((col, val) pairs then (row, meta)
    // entries) or as the reduction scratch of a chunk tile (one accumulator per thread)
    constexpr int kTileSlots = tile_slots(LPR);
    constexpr int kStageBytes = (kTileSlots + kTileRows) * (int)sizeof(int2);
    constexpr int kReduceBytes = kWG * CH * Dense<BT>::kVec * (int)sizeof(float);
    __shared__ __align__(16) char s_raw[kStageBytes > kReduceBytes ? kStageBytes : kReduceBytes];
    int2* s_pairs = reinterpret_cast<int2*>(s_raw);
    int2* s_rm = s_pairs + kTileSlots;
    __shared__ int s_next;                     // next ELL row of a tile whose rows are taken dynamically
    extern __shared__ __align__(16) float s_dyn[];   // per-ELL-row sums of a balanced segment tile

    const int xcd = blockIdx.x % kXcds;
    long long v = blockIdx.x / kXcds;          // position in this XCD's tile list
    for (int gi = 0; gi < a.n_groups; ++gi) {
        const Group& g = a.groups[gi];         // uniform address: scalar loads
        const long long lo = g.n_tiles * xcd / kXcds;
        const long long hi = g.n_tiles * (xcd + 1) / kXcds;
        if (v < hi - lo) {
            const long long tile = lo + v;
            switch (g.type) {
                case kEll:
                case kEllSeg: run_ell_tile<LPR, CH, BT>(g, tile, s_pairs, s_rm, &s_next, s_dyn, a); break;
                case kSeg: run_seg_tile<LPR, CH, BT>(g, tile, a); break;
                case kZero: run_zero_tile<LPR, CH, BT>(g, tile, a); break;
                default: run_chunk_tile<LPR, CH, BT>(g, tile, reinterpret_cast<float*>(s_raw), a); break;
            }
            return;
        }
        v -= hi - lo;
    }
}

// Adds the partial rows of every heavy source row in chunk order and writes the row (rows with
// more than kWideFinalPartials partial rows are left to spmm_finalize_wide_kernel).
template <int LPR, int CH, typename BT>
__global__ void __launch_bounds__(kWG)
spmm_finalize_kernel(const HeavyRow* __restrict__ heavy, int n_heavy, LaunchArgs a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const int sw = threadIdx.x / LPR, sl = threadIdx.x % LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    for (int h = blockIdx.x * SW + sw; h < n_heavy; h += gridDim.x * SW) {
        const HeavyRow hr = heavy[h];
        if (hr.n_partials > kWideFinalPartials) continue;
        Acc<CH, VEC> acc;
        acc.clear();
        for (int k = 0; k < hr.n_partials; ++k) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                if (!ln.on[c]) continue;
                const float* src = a.partials + (size_t)(hr.partial_begin + k) * a.feat + ln.f[c];
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc.v[c][i] += src[i];
            }
        }
        store_row<LPR, CH, VEC>(a.C, hr.row, ln, acc, a.accumulate);
    }
}

// The same for rows with many partial rows (dense rows cut into short chunks): one workgroup per
// row, sub-wave s adds partial rows s, s + SW, s + 2 SW, ... four at a time, and the sub-waves'
// sums are added in sub-wave order - a fixed order, so the result does not depend on scheduling.
template <int LPR, int CH, typename BT>
__global__ void __launch_bounds__(kWG)
spmm_finalize_wide_kernel(const HeavyRow* __restrict__ heavy, int n_heavy, LaunchArgs a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    constexpr int U = 4;
    __shared__ float s_red[kWG * CH * VEC];
    const int sw = threadIdx.x / LPR, sl = threadIdx.x % LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    const int h = blockIdx.x;
    if (h >= n_heavy) return;
    const HeavyRow hr = heavy[h];
    if (hr.n_partials <= kWideFinalPartials) return;
    Acc<CH, VEC> acc;
    acc.clear();
    for (int k0 = sw; k0 < hr.n_partials; k0 += SW * U) {
        float x[U][CH][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = min(k0 + u * SW, hr.n_partials - 1);      // (clamped loads, masked below)
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const float* src = a.partials + (size_t)(hr.partial_begin + k) * a.feat + (ln.on[c] ? ln.f[c] : 0);
#pragma unroll
                for (int i = 0; i < VEC; i += 4) {
                    const float4 v = *reinterpret_cast<const float4*>(src + i);
                    x[u][c][i] = v.x; x[u][c][i + 1] = v.y; x[u][c][i + 2] = v.z; x[u][c][i + 3] = v.w;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k0 + u * SW >= hr.n_partials) break;
#pragma unroll
            for (int c = 0; c < CH; ++c)
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc.v[c][i] += x[u][c][i];
        }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < VEC; ++i) s_red[((sw * CH + c) * LPR + sl) * VEC + i] = acc.v[c][i];
    __syncthreads();
    if (sw == 0) {
        Acc<CH, VEC> sum;
        sum.clear();
#pragma unroll
        for (int c = 0; c < CH; ++c)
            for (int s2 = 0; s2 < SW; ++s2)
#pragma unroll
                for (int i = 0; i < VEC; ++i) sum.v[c][i] += s_red[((s2 * CH + c) * LPR + sl) * VEC + i];
        store_row<LPR, CH, VEC>(a.C, hr.row, ln, sum, a.accumulate);
    }
}

// ------------------------------------------------------------------------------------
// Row groups.  In a banded, stencil or block-structured matrix consecutive rows hold mostly
// the same columns; a bucket of such rows is rewritten at plan time as groups of four
// consecutive ELL rows with the union of their columns ("merged entries": column, four
// values, a 4-bit presence mask), and one gather of a B row then feeds up to four output
// rows.  The 27-point stencil needs 54 gathers per four rows instead of 4 x 28.  Only
// buckets whose merged entries are well below their slots take this path (measured at plan
// time); a matrix without shared columns never does.  Separate kernel, so that its registers
// (four accumulators) do not weigh on the main one.
constexpr int kGroupRows = 4;
#ifndef LF_MERGED_CAP
#define LF_MERGED_CAP 1024
#endif
constexpr int kMergedCap = LF_MERGED_CAP;   // merged entries staged per workgroup at most
constexpr int kMergedTileGroups = 64;  // row groups per tile at most
constexpr long long kRowGroupMinRows = 4096;   // smaller buckets are not worth the analysis
constexpr int kRowGroupSample = 4096;          // the decision looks at about this many groups of a bucket first
constexpr int kRowGroupMaxPercent = 70;        // merged entries / plain gathers at most, in percent
constexpr int kRowGroupSampleEntries = 24;     // merged entries of a group that the sampling pass looks at

struct MergedBucket {
    long long n_groups;        // row groups
    long long n_rows;          // ELL rows of the bucket (the last group may hold fewer than four)
    long long n_tiles;
    int groups_per_tile;
    int pad_;
    const int32_t* rows;       // [n_rows] source rows of the bucket
    const int32_t* goff;       // [n_groups + 1] first merged entry of each group
    const int32_t* ecol;       // [entries]
    const float4* eval;        // [entries] the four rows' values, 0 where a row lacks the column
    const uint8_t* emask;      // [entries] bit r: row r of the group holds the column
};

// Merges the (ascending) column lists of the rows of group g; calls emit(col, vals[4], mask)
// per merged entry when kEmit, and returns the number of merged entries.
template <bool kEmit, typename Emit>
__device__ __forceinline__ int merge_group(const int32_t* __restrict__ cols, const float* __restrict__ vals,
                                           const int32_t* __restrict__ meta, long long g, long long n_rows,
                                           int log_w, Emit emit, int max_entries = 0x7FFFFFFF,
                                           int* consumed = nullptr) {
    // Four columns (and values) of every row are held in registers and refilled with one
    // 16-byte load: a row starts at a multiple of its width (>= 8 slots), so the loads are
    // aligned, and the chain of dependent loads is a quarter as long.
    int len[kGroupRows], pos[kGroupRows];
    long long base[kGroupRows];
    int4 cbuf[kGroupRows];
    float4 vbuf[kGroupRows];
#pragma unroll
    for (int r = 0; r < kGroupRows; ++r) {
        const long long e = g * kGroupRows + r;
        len[r] = e < n_rows ? (meta[e] & (int)kMetaLenMask) : 0;
        base[r] = e << log_w;
        pos[r] = 0;
        cbuf[r] = make_int4(0, 0, 0, 0);
        vbuf[r] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (len[r] > 0) {
            cbuf[r] = *reinterpret_cast<const int4*>(cols + base[r]);
            if (kEmit) vbuf[r] = *reinterpret_cast<const float4*>(vals + base[r]);
        }
    }
    auto pick = [](const int4& q, int i) { return i == 0 ? q.x : i == 1 ? q.y : i == 2 ? q.z : q.w; };
    auto pickf = [](const float4& q, int i) { return i == 0 ? q.x : i == 1 ? q.y : i == 2 ? q.z : q.w; };
    int m = 0;
    for (;;) {
        int head[kGroupRows];
        int cmin = 0x7FFFFFFF;
#pragma unroll
        for (int r = 0; r < kGroupRows; ++r) {
            head[r] = pos[r] < len[r] ? pick(cbuf[r], pos[r] & 3) : 0x7FFFFFFF;
            cmin = min(cmin, head[r]);
        }
        if (cmin == 0x7FFFFFFF) break;
        float v[kGroupRows];
        uint32_t mask = 0;
#pragma unroll
        for (int r = 0; r < kGroupRows; ++r) {
            v[r] = 0.f;
            if (head[r] == cmin) {
                if (kEmit) v[r] = pickf(vbuf[r], pos[r] & 3);
                mask |= 1u << r;
                ++pos[r];
                if ((pos[r] & 3) == 0 && pos[r] < len[r]) {
                    cbuf[r] = *reinterpret_cast<const int4*>(cols + base[r] + pos[r]);
                    if (kEmit) vbuf[r] = *reinterpret_cast<const float4*>(vals + base[r] + pos[r]);
                }
            }
        }
        if (kEmit) emit(m, cmin, v, mask);
        if (++m >= max_entries) break;
    }
    if (consumed) *consumed = pos[0] + pos[1] + pos[2] + pos[3];
    return m;
}

// One candidate bucket of the row-group analysis.
struct RowGroupCand {
    const int32_t* cols;
    const int32_t* meta;
    long long n_rows;
    long long n_groups;
    int32_t* m_out;            // merged length of every group, or null
    int log_w;
    int stride;                // > 1: only every stride-th group is looked at (sampling)
};

// counters[3 * cand + ...]: [0] merged entries, [1] gathers of the plain path (row lengths
// rounded up to the unroll; when sampling, the slots that the merged entries consumed),
// [2] longest group.  blockIdx.y is the candidate.
__global__ void __launch_bounds__(256)
rowgroup_count_kernel(const RowGroupCand* __restrict__ cands, unsigned long long* __restrict__ counters) {
    const RowGroupCand cd = cands[blockIdx.y];
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long g = t * cd.stride;
    int m = 0, plain = 0;
    if (g < cd.n_groups) {
        if (cd.stride > 1) {
            // sampling: the first merged entries of the group against the slots they consume
            m = merge_group<false>(cd.cols, nullptr, cd.meta, g, cd.n_rows, cd.log_w,
                                   [](int, int, const float*, uint32_t) {}, kRowGroupSampleEntries, &plain);
        } else {
            m = merge_group<false>(cd.cols, nullptr, cd.meta, g, cd.n_rows, cd.log_w, [](int, int, const float*, uint32_t) {});
            for (int r = 0; r < kGroupRows; ++r) {
                const long long e = g * kGroupRows + r;
                if (e < cd.n_rows) plain += ((cd.meta[e] & (int)kMetaLenMask) + kUnroll - 1) / kUnroll * kUnroll;
            }
        }
        if (cd.m_out) cd.m_out[g] = m;
    }
    int sm = m, sp = plain, mx = m;
    for (int d = 32; d > 0; d >>= 1) {
        sm += __shfl_xor(sm, d);
        sp += __shfl_xor(sp, d);
        mx = max(mx, __shfl_xor(mx, d));
    }
    if ((threadIdx.x & 63) == 0 && sp > 0) {
        unsigned long long* c = counters + 3 * blockIdx.y;
        atomicAdd(&c[0], (unsigned long long)sm);
        atomicAdd(&c[1], (unsigned long long)sp);
        atomicMax(&c[2], (unsigned long long)mx);
    }
}

__global__ void __launch_bounds__(256)
rowgroup_fill_kernel(const int32_t* __restrict__ cols, const float* __restrict__ vals,
                     const int32_t* __restrict__ meta, long long n_rows, int log_w, long long n_groups,
                     const int32_t* __restrict__ goff, int32_t* __restrict__ ecol, float4* __restrict__ eval,
                     uint8_t* __restrict__ emask) {
    const long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_groups) return;
    const long long at = goff[g];
    merge_group<true>(cols, vals, meta, g, n_rows, log_w, [&](int j, int c, const float* v, uint32_t mask) {
        ecol[at + j] = c;
        eval[at + j] = make_float4(v[0], v[1], v[2], v[3]);
        emask[at + j] = (uint8_t)mask;
    });
}

// One workgroup per tile of row groups, XCD-aware like the main kernel.  CH == 1 only.
template <int LPR, typename BT>
__global__ void __launch_bounds__(kWG)
spmm_rowgroup_kernel(const MergedBucket* __restrict__ buckets, int n_buckets, LaunchArgs a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    constexpr int U = VEC == 4 ? 8 : 4;          // gathers in flight per sub-wave
    __shared__ float4 s_val[kMergedCap];
    __shared__ int s_col[kMergedCap];
    __shared__ int s_goff[kMergedTileGroups + 1];
    __shared__ uint8_t s_msk[kMergedCap];

    const int xcd = blockIdx.x % kXcds;
    long long v = blockIdx.x / kXcds;
    for (int bi = 0; bi < n_buckets; ++bi) {
        const MergedBucket& b = buckets[bi];
        const long long lo = b.n_tiles * xcd / kXcds;
        const long long hi = b.n_tiles * (xcd + 1) / kXcds;
        if (v >= hi - lo) { v -= hi - lo; continue; }
        const long long g0 = (lo + v) * b.groups_per_tile;
        const int n = (int)min((long long)b.groups_per_tile, b.n_groups - g0);
        const int tid = threadIdx.x;
        for (int i = tid; i <= n; i += kWG) s_goff[i] = b.goff[g0 + i];
        __syncthreads();
        const int sw = tid / LPR, sl = tid % LPR;
        const Lane<LPR, 1, VEC> ln(sl, a.feat, a.ldb, a.ldc);
        // The tile's groups are staged in rounds of as many whole groups as the buffer holds
        // (one group always fits: the plan checks the longest group against the capacity).
        for (int ga = 0; ga < n;) {
            const int base = s_goff[ga];
            int gb = ga + 1;
            while (gb < n && s_goff[gb + 1] - base <= kMergedCap) ++gb;      // uniform
            const int n_entries = s_goff[gb] - base;
            for (int i = tid; i < n_entries; i += kWG) {
                s_col[i] = b.ecol[base + i];
                s_val[i] = b.eval[base + i];
                s_msk[i] = b.emask[base + i];
            }
            __syncthreads();
            for (int gi = ga + sw; gi < gb; gi += SW) {
                const int e0 = s_goff[gi] - base;
                const int m = s_goff[gi + 1] - s_goff[gi];
                Acc<1, VEC> acc[kGroupRows];
#pragma unroll
                for (int r = 0; r < kGroupRows; ++r) acc[r].clear();
                for (int j = 0; j < m; j += U) {
                    int c[U];
                    float4 w[U];
                    uint32_t k[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const bool in = j + u < m;
                        const int idx = e0 + (in ? j + u : 0);   // past the end: the first column again, nothing added
                        c[u] = s_col[idx];
                        w[u] = in ? s_val[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
                        k[u] = in ? s_msk[idx] : 0u;
                    }
                    float x[U][VEC];
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        Dense<BT>::load(dense_row<BT>(a.B, ln, 0, c[u]), x[u]);
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const float wr[kGroupRows] = {w[u].x, w[u].y, w[u].z, w[u].w};
#pragma unroll
                        for (int r = 0; r < kGroupRows; ++r) {
                            if constexpr (LPR == 64) {
                                // one group per wavefront: rows without the column are skipped outright
                                if (__builtin_amdgcn_readfirstlane(k[u]) & (1u << r)) {
#pragma unroll
                                    for (int i = 0; i < VEC; ++i) acc[r].v[0][i] = fmaf(wr[r], x[u][i], acc[r].v[0][i]);
                                }
                            } else {
                                // several groups per wavefront: the value is 0 where the row lacks the
                                // column (like a padded slot, this adds 0 * B: only non-finite B differs)
#pragma unroll
                                for (int i = 0; i < VEC; ++i) acc[r].v[0][i] = fmaf(wr[r], x[u][i], acc[r].v[0][i]);
                            }
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < kGroupRows; ++r) {
                    const long long e = (g0 + gi) * kGroupRows + r;
                    if (e < b.n_rows) store_row<LPR, 1, VEC>(a.C, b.rows[e], ln, acc[r], a.accumulate);
                }
            }
            ga = gb;
            if (ga < n) __syncthreads();                 // the buffer is refilled
        }
        return;
    }
}

// Row-parallel CSR product: one sub-wave per row, entries streamed by shuffle.
template <int LPR, int CH, typename BT>
__global__ void __launch_bounds__(kWG)
csr_spmm_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices,
                const float* __restrict__ values, long long n_rows, LaunchArgs a) {
    constexpr int VEC = Dense<BT>::kVec;
    constexpr int SW = kWG / LPR;
    const int sw = threadIdx.x / LPR, sl = threadIdx.x % LPR;
    const Lane<LPR, CH, VEC> ln(sl, a.feat, a.ldb, a.ldc);
    for (long long r = (long long)blockIdx.x * SW + sw; r < n_rows; r += (long long)gridDim.x * SW) {
        const int lo = indptr[r], hi = indptr[r + 1];
        Acc<CH, VEC> acc;
        acc.clear();
        stream_slots<LPR, CH, BT>(indices, values, lo, hi - lo, a.B, ln, acc);
        store_row<LPR, CH, VEC>(a.C, (int)r, ln, acc, kStreamC);
    }
}

// ------------------------------------------------------------------------------------
// Plan-time kernels.

// Inclusive scans over a 256-thread workgroup: the largest value at or before a thread, the
// smallest value at or after it.  s_wave: 4 ints of LDS.
__device__ __forceinline__ int block_scan_max_fwd(int x, int* s_wave) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_up(x, d);
        if (lane >= d) x = max(x, y);
    }
    if (lane == 63) s_wave[wave] = x;
    __syncthreads();
    for (int w = 0; w < wave; ++w) x = max(x, s_wave[w]);
    __syncthreads();
    return x;
}

__device__ __forceinline__ int block_scan_min_bwd(int x, int* s_wave) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_down(x, d);
        if (lane + d < 64) x = min(x, y);
    }
    if (lane == 0) s_wave[wave] = x;
    __syncthreads();
    for (int w = wave + 1; w < 4; ++w) x = min(x, s_wave[w]);
    __syncthreads();
    return x;
}

// meta from rows / vals for slabs that come without one (the reference passes rows, cols and
// values only, format_algos.py:552-578): len = position of the last nonzero value + 1 (at
// least 1); a run of equal row ids is one segment.  Two passes, so that a long run costs a
// scan and not a walk per ELL row: the first notes, per block of 256 ELL rows, its first and
// its last segment head (an ELL row whose predecessor carries another row id); the second
// finds for every ELL row the head at or before it and, for a head, the next head.
__global__ void __launch_bounds__(256)
derive_heads_kernel(const int32_t* __restrict__ rows, long long n_rows, int32_t* __restrict__ blk_first,
                    int32_t* __restrict__ blk_last) {
    __shared__ int s_wave[4];
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool head = e < n_rows && (e == 0 || rows[e - 1] != rows[e]);
    const int last = block_scan_max_fwd(head ? (int)e : -1, s_wave);
    const int first = block_scan_min_bwd(head ? (int)e : 0x7FFFFFFF, s_wave);
    if (threadIdx.x == 255) blk_last[blockIdx.x] = last;
    if (threadIdx.x == 0) blk_first[blockIdx.x] = first;
}

// flags[3] is raised when a segment is longer than the meta word can say.
__global__ void __launch_bounds__(256)
derive_meta_kernel(const int32_t* __restrict__ rows, const float* __restrict__ vals, long long n_rows,
                   int log_w, const int32_t* __restrict__ blk_first, const int32_t* __restrict__ blk_last,
                   int n_blocks, int32_t* __restrict__ meta, int* __restrict__ flags) {
    __shared__ int s_wave[4];
    __shared__ int s_prev, s_next;
    if (threadIdx.x == 0) {                      // heads outside this block (block 0 starts with one)
        int b = (int)blockIdx.x - 1;
        while (b >= 0 && blk_last[b] < 0) --b;
        s_prev = b >= 0 ? blk_last[b] : 0;
        b = (int)blockIdx.x + 1;
        while (b < n_blocks && blk_first[b] == 0x7FFFFFFF) ++b;
        s_next = b < n_blocks ? blk_first[b] : (int)n_rows;
    }
    __syncthreads();
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool in = e < n_rows;
    const bool head = in && (e == 0 || rows[e - 1] != rows[e]);
    int prev = block_scan_max_fwd(head ? (int)e : -1, s_wave);
    // the next head strictly after e: the smallest head at or after the thread's successor
    __shared__ int s_at_or_after[257];
    s_at_or_after[threadIdx.x] = block_scan_min_bwd(head ? (int)e : 0x7FFFFFFF, s_wave);
    if (threadIdx.x == 0) s_at_or_after[256] = 0x7FFFFFFF;
    __syncthreads();
    int next = s_at_or_after[threadIdx.x + 1];
    if (!in) return;
    if (prev < 0) prev = s_prev;
    if (next == 0x7FFFFFFF) next = min(s_next, (int)n_rows);
    const int w = 1 << log_w;
    const float* rv = vals + (e << log_w);
    int len = 1;
    for (int j = w - 1; j > 0; --j)
        if (rv[j] != 0.f) { len = j + 1; break; }
    uint32_t field, cont = 0;
    if (head) {
        field = (uint32_t)(next - (int)e);
    } else {
        field = (uint32_t)((int)e - prev);
        cont = 0x80000000u;
    }
    if (field >= (1u << (31 - kMetaLenBits))) {
        flags[3] = 1;
        field = 1;                                 // keep the word well formed; the plan is refused
    }
    meta[e] = (int32_t)((uint32_t)len | (field << kMetaLenBits) | cont);
}

// Checks what the SpMM kernels take on trust from a bucket: source rows inside the matrix,
// column indices inside B, 1..W valid slots per ELL row, and segments (a head that announces
// n ELL rows followed by continuation rows 1..n-1 with the same row id) that are complete
// and stay inside the bucket.  flags[0] bad column, [1] bad row, [2] bad meta.
__global__ void __launch_bounds__(256)
validate_bucket_kernel(const int32_t* __restrict__ rows, const int32_t* __restrict__ meta,
                       const int32_t* __restrict__ cols, long long n_rows, int log_w,
                       long long num_rows, long long num_cols, int* __restrict__ flags) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    const long long t0 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    bool bad_col = false, bad_row = false, bad_meta = false;
    const long long n_slots = n_rows << log_w;
    for (long long i = t0 * 4; i < n_slots; i += stride * 4) {
        if (i + 4 <= n_slots) {
            const int4 c = *reinterpret_cast<const int4*>(cols + i);
            bad_col |= (unsigned)c.x >= (unsigned long long)num_cols || (unsigned)c.y >= (unsigned long long)num_cols ||
                       (unsigned)c.z >= (unsigned long long)num_cols || (unsigned)c.w >= (unsigned long long)num_cols;
        } else {
            for (long long k = i; k < n_slots; ++k) bad_col |= (unsigned)cols[k] >= (unsigned long long)num_cols;
        }
    }
    for (long long e = t0; e < n_rows; e += stride) {
        bad_row |= (unsigned)rows[e] >= (unsigned long long)num_rows;
        const int m = meta[e];
        const int len = m & (int)kMetaLenMask;
        bad_meta |= len < 1 || len > (1 << log_w);
        const long long field = (long long)(((uint32_t)m & 0x7FFFFFFFu) >> kMetaLenBits);
        // what the next ELL row must be: a continuation row with index `want`, or a head (0)
        long long want = 0;
        if (m >= 0) {
            bad_meta |= field < 1 || e + field > n_rows;
            want = field > 1 ? 1 : 0;
        } else {
            const long long h = e - field;
            if (field < 1 || h < 0) {
                bad_meta = true;
            } else {
                const int hm = meta[h];
                const long long n = (long long)((uint32_t)hm >> kMetaLenBits);
                bad_meta |= hm < 0 || field >= n || rows[h] != rows[e];
                want = field + 1 < n ? field + 1 : 0;
            }
        }
        if (e == 0) bad_meta |= m < 0;
        if (e + 1 < n_rows) {
            const int nm = meta[e + 1];
            const long long nf = (long long)(((uint32_t)nm & 0x7FFFFFFFu) >> kMetaLenBits);
            bad_meta |= want == 0 ? nm < 0 : (nm >= 0 || nf != want);
        } else {
            bad_meta |= want != 0;
        }
    }
    if (__ballot(bad_col) != 0 && (threadIdx.x & 63) == 0) flags[0] = 1;
    if (__ballot(bad_row) != 0 && (threadIdx.x & 63) == 0) flags[1] = 1;
    if (__ballot(bad_meta) != 0 && (threadIdx.x & 63) == 0) flags[2] = 1;
}

// Finds the source rows of a bucket that take the cooperative path (more than kCoopSlots
// slots) and cuts them into chunks.  Runs twice: with chunks == nullptr it only counts
// (counters[0] chunks, [1] rows with several chunks, [2] their partial rows, [3] "the bucket
// has rows spanning several ELL rows"); the second run fills the tables, taking ranges with
// the same counters.  Table order depends on scheduling, results do not: every row's
// partials are private and are summed in chunk order.
__global__ void __launch_bounds__(256)
plan_chunks_kernel(const int32_t* __restrict__ rows, const int32_t* __restrict__ meta,
                   const int32_t* __restrict__ cols, long long n_rows, int log_w, int* __restrict__ counters,
                   Chunk* __restrict__ chunks, HeavyRow* __restrict__ heavy,
                   int partial_base, int heavy_base, int chunk_slots, long long dense_min_slots) {
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = threadIdx.x & 63;
    int seg = 0, n_chunks = 0, cs = chunk_slots;
    long long total = 0;
    bool split = false, dense = false;
    if (e < n_rows) {
        const int m = meta[e];
        if (m < 0) {
            split = true;
        } else {
            seg = (int)((uint32_t)m >> kMetaLenBits);
            split = seg > 1;
            // The counting pass is enqueued together with the slab checks, before their verdict
            // has been read: a head that announces more ELL rows than the bucket holds (which the
            // checks flag and the plan is then refused) must not be followed past the array.
            if (((long long)seg << log_w) > kCoopSlots && e + seg <= n_rows) {
                total = ((long long)(seg - 1) << log_w) + (meta[e + seg - 1] & kMetaLenMask);
                dense = total >= dense_min_slots;
                if (dense) cs = kDenseChunkSlots;
                n_chunks = (int)((total + cs - 1) / cs);
            }
        }
    }
    if (__ballot(dense) != 0 && lane == 0) atomicOr(&counters[3], 2);
    if (__ballot(n_chunks > kWideFinalPartials) != 0 && lane == 0) atomicOr(&counters[3], 4);
    if (__ballot(split) != 0 && lane == 0) atomicOr(&counters[3], 1);
    // ranges of the tables: one atomic per counter and wavefront (a matrix of long rows has
    // a cooperative row in every lane)
    const bool several = n_chunks > 1;
    const int part = several ? n_chunks : 0;
    int incl_c = n_chunks, incl_p = part;
    for (int d = 1; d < 64; d <<= 1) {
        const int yc = __shfl_up(incl_c, d), yp = __shfl_up(incl_p, d);
        if (lane >= d) { incl_c += yc; incl_p += yp; }
    }
    const int tot_c = __shfl(incl_c, 63), tot_p = __shfl(incl_p, 63);
    if (tot_c == 0) return;
    const unsigned long long votes = __ballot(several);
    int base_c = 0, base_h = 0, base_p = 0;
    if (lane == 0) {
        base_c = atomicAdd(&counters[0], tot_c);
        if (votes) {
            base_h = atomicAdd(&counters[1], __popcll(votes));
            base_p = atomicAdd(&counters[2], tot_p);
        }
    }
    base_c = __shfl(base_c, 0);
    base_h = __shfl(base_h, 0);
    base_p = __shfl(base_p, 0);
    if (chunks == nullptr || n_chunks == 0) return;
    const int c0 = base_c + incl_c - n_chunks;
    const int h = base_h + __popcll(votes & ((1ull << lane) - 1ull));
    const int p0 = base_p + incl_p - part;
    const int row = rows[e];
    for (int i = 0; i < n_chunks; ++i) {
        const long long lo = (long long)i * cs;
        const long long hi = min(total, lo + cs);
        Chunk ck;
        ck.slot_begin = (e << log_w) + lo;
        ck.n_slots = (int)(hi - lo) | (dense ? kChunkDenseBit : 0);
        ck.partial = several ? partial_base + p0 + i : -1;
        ck.row = row;
        ck.first_col = cols[ck.slot_begin];
        chunks[c0 + i] = ck;
    }
    if (several) heavy[heavy_base + h] = HeavyRow{row, partial_base + p0, n_chunks, 0};
}

__global__ void mark_rows_kernel(const int32_t* __restrict__ rows, long long n, uint8_t* __restrict__ covered) {
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n) covered[rows[e]] = 1;
}

// Rows that no bucket of partition 0 writes: counted (list == nullptr) or listed.  Each
// wavefront owns a contiguous range of rows and each workgroup takes its slice of the list
// with a single atomic: one atomic per wavefront was 38K updates of one address for 2.45M
// rows, 0.3 ms per pass.
__global__ void __launch_bounds__(256)
collect_uncovered_kernel(const uint8_t* __restrict__ covered, long long n_rows,
                         int* __restrict__ count, int32_t* __restrict__ list) {
    __shared__ int s_total[4];
    __shared__ int s_base;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long per_wave = ((n_rows + (long long)gridDim.x * 4 - 1) / ((long long)gridDim.x * 4) + 63) / 64 * 64;
    const long long lo = ((long long)blockIdx.x * 4 + wave) * per_wave;
    const long long hi = lo + per_wave < n_rows ? lo + per_wave : n_rows;
    int total = 0;
    for (long long r0 = lo; r0 < hi; r0 += 64) {
        const long long r = r0 + lane;
        total += __popcll(__ballot(r < hi && !covered[r]));
    }
    if (lane == 0) s_total[wave] = total;
    __syncthreads();
    if (threadIdx.x == 0) {
        const int sum = s_total[0] + s_total[1] + s_total[2] + s_total[3];
        s_base = sum ? atomicAdd(count, sum) : 0;
    }
    __syncthreads();
    if (list == nullptr) return;
    int at = s_base;
    for (int w = 0; w < wave; ++w) at += s_total[w];
    for (long long r0 = lo; r0 < hi; r0 += 64) {
        const long long r = r0 + lane;
        const bool mine = r < hi && !covered[r];
        const unsigned long long votes = __ballot(mine);
        if (mine) list[at + __popcll(votes & ((1ull << lane) - 1ull))] = (int32_t)r;
        at += __popcll(votes);
    }
}

__global__ void fill_bytes_kernel(uint32_t* __restrict__ p, long long n_words, uint32_t value) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n_words;
         i += (long long)gridDim.x * blockDim.x)
        p[i] = value;
}

}  // namespace

// ====================================================================================
struct lf_spmm_plan {
    int feat = 0, b_dtype = 0, num_parts = 0;
    int64_t num_rows = 0, num_cols = 0;
    int lpr = 0, ch = 0;
    int windows = 1;                 // feature windows of `feat` features each that a run covers
    int device = 0, num_cus = 0, grid = 0;
    struct Launch {
        int group_begin = 0, n_groups = 0, grid = 0;
        int dyn_lds = 0;             // bytes of dynamic LDS (balanced segment tiles)
        int merged_begin = 0, n_merged = 0, merged_grid = 0;   // row-group buckets of this partition
        int cell_begin = 0, n_cell_buckets = 0, cell_grid = 0; // buckets rewritten as cells
        long long tiles = 0;
        int heavy_begin = 0, n_heavy = 0;
        bool stream_c = false;       // store C past the caches (when this is the run's last partition)
        bool wide_rows = false;      // some rows have more than kWideFinalPartials partial rows
    };
    std::vector<Launch> launches;
    bool stream_slabs = false;          // read the slabs non-temporally
    MergedBucket* d_merged = nullptr;   // row-group buckets, grouped by partition
    LfCellBucket* d_cells = nullptr;    // buckets rewritten as cells, grouped by partition
    std::vector<void*> owned;        // device allocations released by destroy
    std::vector<void*> temp;         // plan-time scratch, released when lf_spmm_create returns
    Group* d_groups = nullptr;
    HeavyRow* d_heavy = nullptr;
    float* d_partials = nullptr;
    int64_t info[LF_SPMM_INFO_FIELDS] = {0};
};

namespace {

template <typename T> int dev_alloc(lf_spmm_plan* p, T** out, size_t count, bool temporary = false) {
    *out = nullptr;
    if (count == 0) return LF_OK;
    void* ptr = nullptr;
    LF_HIP(hipMalloc(&ptr, count * sizeof(T)));
    (temporary ? p->temp : p->owned).push_back(ptr);
    *out = (T*)ptr;
    return LF_OK;
}

int free_temporaries(lf_spmm_plan* p) {
    int rc = LF_OK;
    for (void* ptr : p->temp)
        if (hipFree(ptr) != hipSuccess) rc = LF_ERR_HIP;
    p->temp.clear();
    return rc;
}

using KernelFn = void (*)(LaunchArgs);
using FinalFn = void (*)(const HeavyRow*, int, LaunchArgs);
using CsrFn = void (*)(const int32_t*, const int32_t*, const float*, long long, LaunchArgs);

using RowGroupFn = void (*)(const MergedBucket*, int, LaunchArgs);

struct KernelSet {
    KernelFn tiles = nullptr;
    FinalFn finalize = nullptr;
    FinalFn finalize_wide = nullptr;
    CsrFn csr = nullptr;
    RowGroupFn rowgroup = nullptr;   // one 16-byte chunk per lane only
};

template <int LPR, int CH> void pick_kernels(int dtype, KernelSet* k) {
    if constexpr (CH == 1) {
        if (dtype == LF_DTYPE_BF16) k->rowgroup = spmm_rowgroup_kernel<LPR, bf16_t>;
        else k->rowgroup = spmm_rowgroup_kernel<LPR, float>;
    }
    if (dtype == LF_DTYPE_BF16) {
        k->tiles = spmm_partition_kernel<LPR, CH, bf16_t>;
        k->finalize = spmm_finalize_kernel<LPR, CH, bf16_t>;
        k->finalize_wide = spmm_finalize_wide_kernel<LPR, CH, bf16_t>;
        k->csr = csr_spmm_kernel<LPR, CH, bf16_t>;
    } else {
        k->tiles = spmm_partition_kernel<LPR, CH, float>;
        k->finalize = spmm_finalize_kernel<LPR, CH, float>;
        k->finalize_wide = spmm_finalize_wide_kernel<LPR, CH, float>;
        k->csr = csr_spmm_kernel<LPR, CH, float>;
    }
}

int select_kernels(int lpr, int ch, int dtype, KernelSet* k) {
    if (ch == 1) {
        switch (lpr) {
            case 8: pick_kernels<8, 1>(dtype, k); break;
            case 16: pick_kernels<16, 1>(dtype, k); break;
            case 32: pick_kernels<32, 1>(dtype, k); break;
            case 64: pick_kernels<64, 1>(dtype, k); break;
        }
    } else if (lpr == 64 && ch == 2) {
        pick_kernels<64, 2>(dtype, k);
    } else if (lpr == 64 && ch == 4) {
        pick_kernels<64, 4>(dtype, k);
    }
    LF_REQUIRE(k->tiles != nullptr, LF_ERR_UNSUPPORTED, "no kernel for %d lanes x %d chunks", lpr, ch);
    return LF_OK;
}

int feature_shape(int feat, int dtype, int* lpr, int* ch) {
    const int vec = dtype == LF_DTYPE_BF16 ? 8 : 4;
    LF_REQUIRE(feat >= 32 && feat % 32 == 0, LF_ERR_UNSUPPORTED,
               "feat_size must be a positive multiple of 32 (got %d)", feat);
    LF_REQUIRE(feat <= 1024, LF_ERR_UNSUPPORTED, "feat_size above 1024 is not supported (got %d)", feat);
    const int lanes = feat / vec;
    int l = 8;
    while (l < lanes && l < 64) l <<= 1;
    int c = (lanes + l - 1) / l;
    if (c == 3) c = 4;
    LF_REQUIRE(c == 1 || c == 2 || c == 4, LF_ERR_UNSUPPORTED, "feat_size %d is not supported", feat);
    *lpr = l;
    *ch = c;
    return LF_OK;
}

}  // namespace

extern "C" {

int lf_spmm_destroy(lf_spmm_plan* plan) {
    if (!plan) return LF_OK;
    int rc = free_temporaries(plan);
    for (void* p : plan->owned)
        if (hipFree(p) != hipSuccess) rc = LF_ERR_HIP;
    delete plan;
    if (rc != LF_OK) return lf::fail(rc, "hipFree failed while destroying the plan");
    return LF_OK;
}

int lf_spmm_create(lf_spmm_plan** out_plan, const lf_bucket_desc* h_buckets, int32_t num_buckets,
                   int32_t num_parts, int64_t num_rows, int64_t num_cols, int32_t feat_size,
                   int32_t b_dtype, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(out_plan, LF_ERR_INVALID, "out_plan is null");
    *out_plan = nullptr;
    LF_REQUIRE(num_buckets >= 0 && (num_buckets == 0 || h_buckets), LF_ERR_INVALID, "bucket list is null");
    LF_REQUIRE(num_parts >= 1, LF_ERR_INVALID, "num_parts must be >= 1");
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && num_cols >= 1 && num_cols < (1ll << 31),
               LF_ERR_INVALID, "bad shape");
    LF_REQUIRE(b_dtype == LF_DTYPE_F32 || b_dtype == LF_DTYPE_BF16, LF_ERR_INVALID, "unknown B dtype %d", b_dtype);
    int lpr, ch;
    if (int rc = feature_shape(feat_size, b_dtype, &lpr, &ch)) return rc;
    const int sw = kWG / lpr;
    for (int k = 0; k < num_buckets; ++k) {
        const lf_bucket_desc& b = h_buckets[k];
        LF_REQUIRE(lf::is_pow2(b.width) && b.width <= 1024, LF_ERR_INVALID, "bucket %d: width %d", k, b.width);
        LF_REQUIRE(b.part >= 0 && b.part < num_parts, LF_ERR_INVALID, "bucket %d: partition %d", k, b.part);
        LF_REQUIRE(b.num_ell_rows >= 0 && b.num_ell_rows < (1ll << 31), LF_ERR_INVALID, "bucket %d: row count", k);
        LF_REQUIRE(k == 0 || h_buckets[k - 1].part <= b.part, LF_ERR_INVALID, "buckets must be ordered by partition");
        if (b.num_ell_rows > 0) {
            LF_REQUIRE(b.d_rows && b.d_cols && b.d_vals, LF_ERR_INVALID, "bucket %d: null slab", k);
            LF_REQUIRE(((uintptr_t)b.d_cols % 16 == 0) && ((uintptr_t)b.d_vals % 16 == 0), LF_ERR_INVALID,
                       "bucket %d: slabs must be 16-byte aligned", k);
        }
    }

    lf_spmm_plan* plan = new lf_spmm_plan();
    plan->feat = feat_size;
    plan->b_dtype = b_dtype;
    plan->num_parts = num_parts;
    plan->num_rows = num_rows;
    plan->num_cols = num_cols;
    plan->lpr = lpr;
    plan->ch = ch;
    auto bail = [&](int rc) {
        std::string keep = lf::last_error();
        lf_spmm_destroy(plan);
        lf::last_error() = keep;
        return rc;
    };
#define LF_TRY(expr)                        \
    do {                                    \
        int _rc = (expr);                   \
        if (_rc != LF_OK) return bail(_rc); \
    } while (0)
#define LF_TRY_HIP(call)                                                                          \
    do {                                                                                          \
        hipError_t _e = (call);                                                                   \
        if (_e != hipSuccess)                                                                     \
            return bail(lf::fail(LF_ERR_HIP, "%s failed: %s", #call, hipGetErrorString(_e)));     \
    } while (0)

    hipDeviceProp_t prop;
    LF_TRY_HIP(hipGetDevice(&plan->device));
    LF_TRY_HIP(hipGetDeviceProperties(&prop, plan->device));
    plan->num_cus = prop.multiProcessorCount;

    // ---- meta: derive where missing; count the chunks of rows that take the cooperative path.
    // Every bucket has its own four counters (plus one set for the rows to clear), so that
    // the counting pass, the filling pass and the coverage pass each cost one copy back and
    // one synchronisation for the whole plan, not one per bucket.
    std::vector<const int32_t*> meta((size_t)num_buckets, nullptr);
    const int n_counters = 4 * (num_buckets + 2);
    int* d_counters = nullptr;              // [4k .. 4k+3]: plan_chunks_kernel's counters of bucket k
    LF_TRY(dev_alloc(plan, &d_counters, (size_t)n_counters, true));
    int* d_zero_count = d_counters + 4 * num_buckets;
    int* d_flags = d_counters + 4 * (num_buckets + 1);   // validate_bucket_kernel, derive_meta_kernel
    std::vector<int> h_counters((size_t)n_counters, 0);
    std::vector<int> is_multi((size_t)num_buckets, 0), has_dense((size_t)num_buckets, 0), has_wide((size_t)num_buckets, 0);
    struct ChunkCount { int chunks = 0, heavy = 0, partials = 0; };
    std::vector<ChunkCount> counts((size_t)num_buckets);
    auto clear_counters = [&]() {
        fill_bytes_kernel<<<1, 64, 0, s>>>((uint32_t*)d_counters, n_counters, 0u);
        return hipGetLastError();
    };
    auto read_counters = [&]() {
        hipError_t e = hipMemcpyAsync(h_counters.data(), d_counters, (size_t)n_counters * 4, hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
        return e;
    };
    // Chunk size of the rows that a whole workgroup reduces.  Small matrices want many short
    // chunks (a 170k-row graph: 0.076 ms with 2048-slot chunks, 0.112 ms with 8192), large ones
    // fewer partial rows and a shorter second kernel (500k x 2M with 50 rows of 100k entries:
    // 1.56 -> 1.51 ms with 8192); the chunk tiles lead the launch, so their length hides behind
    // the rest of the work.
    long long total_slots = 0;
    for (int k = 0; k < num_buckets; ++k) total_slots += h_buckets[k].num_ell_rows * h_buckets[k].width;
    const int chunk_slots = total_slots >= kLargeMatrixSlots ? kChunkSlotsLarge : kChunkSlots;
    // Slabs of a large matrix are read past the caches' retention (2.45M-row graph 6.15 -> 6.09 ms,
    // 500k x 2M matrix 1.457 -> 1.443); those of a small one are worth keeping between products
    // (170k-row graph, 6 MB of slabs: 0.073 ms cached, 0.076 ms streamed).
    plan->stream_slabs = total_slots >= kLargeMatrixSlots;
    const char* env_dense = getenv("LF_DENSE_ROWS");       // "0": dense rows are chunked like the other long rows
    // (where the memory-side cache holds the partition's part of B anyway there is nothing to order)
    const long long cols_p = lf::ceil_div(num_cols, num_parts);
    const bool b_is_cached = cols_p * feat_size * (b_dtype == LF_DTYPE_BF16 ? 2 : 4) <= kDenseMinBBytes;
    const long long dense_min_slots = (env_dense && env_dense[0] == '0') || b_is_cached
                                          ? (1ll << 62)
                                          : std::max<long long>(kDenseRowMinSlots, cols_p / kDenseRowShare);
    auto launch_plan_chunks = [&](int k, Chunk* out, HeavyRow* hout, int partial_base, int heavy_base) {
        const lf_bucket_desc& b = h_buckets[k];
        const int grid = (int)((b.num_ell_rows + 255) / 256);
        plan_chunks_kernel<<<grid, 256, 0, s>>>(b.d_rows, meta[k], b.d_cols, b.num_ell_rows, lf::ilog2(b.width),
                                                d_counters + 4 * k, out, hout, partial_base, heavy_base, chunk_slots,
                                                dense_min_slots);
        return hipGetLastError();
    };
    LF_TRY_HIP(clear_counters());
    for (int k = 0; k < num_buckets; ++k) {
        const lf_bucket_desc& b = h_buckets[k];
        if (b.num_ell_rows == 0) continue;
        const int log_w = lf::ilog2(b.width);
        if (b.d_meta) {
            meta[k] = b.d_meta;
        } else {
            int32_t *m = nullptr, *blk_first = nullptr, *blk_last = nullptr;
            const int n_blocks = (int)((b.num_ell_rows + 255) / 256);
            LF_TRY(dev_alloc(plan, &m, (size_t)b.num_ell_rows));
            LF_TRY(dev_alloc(plan, &blk_first, (size_t)n_blocks, true));
            LF_TRY(dev_alloc(plan, &blk_last, (size_t)n_blocks, true));
            derive_heads_kernel<<<n_blocks, 256, 0, s>>>(b.d_rows, b.num_ell_rows, blk_first, blk_last);
            LF_TRY_HIP(hipGetLastError());
            derive_meta_kernel<<<n_blocks, 256, 0, s>>>(b.d_rows, b.d_vals, b.num_ell_rows, log_w, blk_first,
                                                        blk_last, n_blocks, m, d_flags);
            LF_TRY_HIP(hipGetLastError());
            meta[k] = m;
        }
        {
            const long long units = std::max<long long>(b.num_ell_rows, ((long long)b.num_ell_rows << log_w) / 4);
            const int vgrid = (int)std::min<long long>(lf::ceil_div(units, 256), 4096);
            validate_bucket_kernel<<<vgrid, 256, 0, s>>>(b.d_rows, meta[k], b.d_cols, b.num_ell_rows, log_w,
                                                         num_rows, num_cols, d_flags);
            LF_TRY_HIP(hipGetLastError());
        }
        LF_TRY_HIP(launch_plan_chunks(k, nullptr, nullptr, 0, 0));
    }
    LF_TRY_HIP(read_counters());
    {
        // nothing below (and no SpMM launch) may run on slabs that fail these checks: a column
        // or row index out of range would be an out-of-range gather or store
        const int* f = &h_counters[4 * (num_buckets + 1)];
        if (f[0]) return bail(lf::fail(LF_ERR_INVALID, "a bucket holds a column index outside [0, %lld)", (long long)num_cols));
        if (f[1]) return bail(lf::fail(LF_ERR_INVALID, "a bucket holds a row index outside [0, %lld)", (long long)num_rows));
        if (f[2]) return bail(lf::fail(LF_ERR_INVALID, "a bucket's meta array is inconsistent (valid slots outside 1..W, "
                                                        "or a segment that is incomplete or leaves the bucket)"));
        if (f[3]) return bail(lf::fail(LF_ERR_UNSUPPORTED, "a row is split over more than %d ELL rows", (1 << (31 - kMetaLenBits)) - 1));
    }
    for (int k = 0; k < num_buckets; ++k) {
        counts[k].chunks = h_counters[4 * k + 0];
        counts[k].heavy = h_counters[4 * k + 1];
        counts[k].partials = h_counters[4 * k + 2];
        is_multi[k] = h_counters[4 * k + 3] & 1;
        has_dense[k] = (h_counters[4 * k + 3] >> 1) & 1;
        has_wide[k] = (h_counters[4 * k + 3] >> 2) & 1;
    }

    // ---- chunk tables, heavy-row table (grouped by bucket, hence by partition) and partial rows
    std::vector<Chunk*> d_chunks((size_t)num_buckets, nullptr);
    std::vector<int> heavy_base((size_t)num_buckets + 1, 0), partial_base((size_t)num_buckets + 1, 0);
    std::vector<long long> chunk_base((size_t)num_buckets + 1, 0);
    for (int k = 0; k < num_buckets; ++k) {
        heavy_base[k + 1] = heavy_base[k] + counts[k].heavy;
        partial_base[k + 1] = partial_base[k] + counts[k].partials;
        chunk_base[k + 1] = chunk_base[k] + counts[k].chunks;
    }
    const int n_heavy_total = heavy_base[num_buckets];
    const int n_partials = partial_base[num_buckets];
    if (n_heavy_total > 0) {
        LF_TRY(dev_alloc(plan, &plan->d_heavy, (size_t)n_heavy_total));
        LF_TRY(dev_alloc(plan, &plan->d_partials, (size_t)n_partials * feat_size));
    }
    Chunk* d_chunks_all = nullptr;
    LF_TRY(dev_alloc(plan, &d_chunks_all, (size_t)chunk_base[num_buckets]));
    LF_TRY_HIP(clear_counters());
    for (int k = 0; k < num_buckets; ++k) {
        if (counts[k].chunks == 0) continue;
        d_chunks[k] = d_chunks_all + chunk_base[k];
        LF_TRY_HIP(launch_plan_chunks(k, d_chunks[k], plan->d_heavy, partial_base[k], heavy_base[k]));
    }

    // ---- rows that partition 0 does not write are cleared by its launch
    int32_t* d_zero_rows = nullptr;
    int n_zero = 0;
    uint8_t* d_cov = nullptr;
    const int rgrid = (int)std::min<int64_t>((num_rows + 255) / 256, 1024);
    if (num_rows > 0) {
        const size_t cov_words = ((size_t)num_rows + 3) / 4;
        uint32_t* cov = nullptr;
        LF_TRY(dev_alloc(plan, &cov, cov_words, true));
        d_cov = (uint8_t*)cov;
        fill_bytes_kernel<<<(int)std::min<size_t>((cov_words + 255) / 256, 4096), 256, 0, s>>>(cov, (long long)cov_words, 0u);
        LF_TRY_HIP(hipGetLastError());
        for (int k = 0; k < num_buckets; ++k) {
            const lf_bucket_desc& b = h_buckets[k];
            if (b.part != 0 || b.num_ell_rows == 0) continue;
            mark_rows_kernel<<<(int)((b.num_ell_rows + 255) / 256), 256, 0, s>>>(b.d_rows, b.num_ell_rows, d_cov);
            LF_TRY_HIP(hipGetLastError());
        }
        collect_uncovered_kernel<<<rgrid, 256, 0, s>>>(d_cov, num_rows, d_zero_count, nullptr);
        LF_TRY_HIP(hipGetLastError());
    }
    LF_TRY_HIP(read_counters());             // the filling pass must have taken the same ranges
    for (int k = 0; k < num_buckets; ++k) {
        if (counts[k].chunks == 0) continue;
        if (h_counters[4 * k] != counts[k].chunks || h_counters[4 * k + 1] != counts[k].heavy ||
            h_counters[4 * k + 2] != counts[k].partials)
            return bail(lf::fail(LF_ERR_INVALID, "bucket %d changed while the plan was being built", k));
        if (has_dense[k]) {
            // The chunks of dense rows go behind the others, in column order (ties: by row, so
            // the order is the same in every plan): some thousands of records, sorted on the host.
            std::vector<Chunk> h_chunks((size_t)counts[k].chunks);
            LF_TRY_HIP(hipMemcpyAsync(h_chunks.data(), d_chunks[k], h_chunks.size() * sizeof(Chunk), hipMemcpyDeviceToHost, s));
            LF_TRY_HIP(hipStreamSynchronize(s));
            const auto mid = std::stable_partition(h_chunks.begin(), h_chunks.end(),
                                                   [](const Chunk& x) { return (x.n_slots & kChunkDenseBit) == 0; });
            std::sort(mid, h_chunks.end(), [](const Chunk& x, const Chunk& y) {
                if (x.first_col != y.first_col) return x.first_col < y.first_col;
                if (x.row != y.row) return x.row < y.row;
                return x.slot_begin < y.slot_begin;
            });
            for (auto it = mid; it != h_chunks.end(); ++it) it->n_slots &= ~kChunkDenseBit;
            LF_TRY_HIP(hipMemcpyAsync(d_chunks[k], h_chunks.data(), h_chunks.size() * sizeof(Chunk), hipMemcpyHostToDevice, s));
            LF_TRY_HIP(hipStreamSynchronize(s));
        }
    }
    n_zero = h_counters[4 * num_buckets];
    if (n_zero > 0) {
        LF_TRY(dev_alloc(plan, &d_zero_rows, (size_t)n_zero));
        fill_bytes_kernel<<<1, 64, 0, s>>>((uint32_t*)d_zero_count, 4, 0u);
        collect_uncovered_kernel<<<rgrid, 256, 0, s>>>(d_cov, num_rows, d_zero_count, d_zero_rows);
        LF_TRY_HIP(hipGetLastError());
    }

    // ---- row groups: buckets whose consecutive rows share most of their columns
    std::vector<MergedBucket> merged;                      // in bucket (hence partition) order
    std::vector<int> merged_of((size_t)num_buckets, -1);
    std::vector<LfCellBucket> cells;                       // in bucket (hence partition) order
    std::vector<int> cell_of((size_t)num_buckets, -1);
    {
        const char* env = getenv("LF_ROW_GROUPS");
        std::vector<int> cand;
        for (int k = 0; k < num_buckets && ch == 1 && !(env && env[0] == '0'); ++k) {
            const lf_bucket_desc& b = h_buckets[k];
            if (b.num_ell_rows >= kRowGroupMinRows && b.width >= kUnroll && b.width <= 64 && !is_multi[k]) cand.push_back(k);
        }
        unsigned long long* d_rg = nullptr;                // three counters per candidate
        std::vector<unsigned long long> h_rg(cand.size() * 3, 0);
        RowGroupCand* d_cands = nullptr;
        auto count_pass = [&](const std::vector<int>& which, bool sample, std::vector<int32_t*>* m_arrays) -> int {
            std::vector<RowGroupCand> h_cands(which.size());
            long long most = 1;
            for (size_t i = 0; i < which.size(); ++i) {
                const lf_bucket_desc& b = h_buckets[which[i]];
                RowGroupCand& c = h_cands[i];
                c.cols = b.d_cols;
                c.meta = meta[which[i]];
                c.n_rows = b.num_ell_rows;
                c.n_groups = lf::ceil_div(b.num_ell_rows, kGroupRows);
                c.m_out = m_arrays ? (*m_arrays)[i] : nullptr;
                c.log_w = lf::ilog2(b.width);
                c.stride = sample ? (int)std::max<long long>(1, c.n_groups / kRowGroupSample) : 1;
                most = std::max<long long>(most, lf::ceil_div(c.n_groups, c.stride));
            }
            fill_bytes_kernel<<<1, 64, 0, s>>>((uint32_t*)d_rg, (long long)cand.size() * 6, 0u);
            LF_HIP(hipGetLastError());
            LF_HIP(hipMemcpyAsync(d_cands, h_cands.data(), h_cands.size() * sizeof(RowGroupCand), hipMemcpyHostToDevice, s));
            rowgroup_count_kernel<<<dim3((unsigned)lf::ceil_div(most, 256), (unsigned)which.size()), 256, 0, s>>>(d_cands, d_rg);
            LF_HIP(hipGetLastError());
            LF_HIP(hipMemcpyAsync(h_rg.data(), d_rg, which.size() * 24, hipMemcpyDeviceToHost, s));
            LF_HIP(hipStreamSynchronize(s));               // also keeps h_cands alive until the copy is done
            return LF_OK;
        };
        if (!cand.empty()) {
            LF_TRY(dev_alloc(plan, &d_rg, cand.size() * 3, true));
            LF_TRY(dev_alloc(plan, &d_cands, cand.size(), true));
            LF_TRY(count_pass(cand, true, nullptr));       // a sample of the groups decides
            std::vector<int> chosen;
            for (size_t i = 0; i < cand.size(); ++i)
                if (h_rg[3 * i + 1] > 0 && h_rg[3 * i] * 100 <= h_rg[3 * i + 1] * kRowGroupMaxPercent) chosen.push_back(cand[i]);
            // fp32 B, one 16-byte load per lane and 32 or 64 lanes per row of B (128 or 256
            // features per pass): the chosen buckets are rewritten as cells of rows that are
            // neighbours in up to three directions where that structure is found, else four
            // consecutive rows at a time (as are all other operand shapes: the cells measured
            // slower there).
            const bool cells_fit = (feat_size == 256 || feat_size == 128) && b_dtype == LF_DTYPE_F32;
            if (!chosen.empty() && cells_fit && !(env && env[0] == '4')) {
                std::vector<int> rest;
                for (int k : chosen) {
                    LfCellBucket cb{};
                    bool ok = false;
                    LF_TRY(lf::cells_build(h_buckets[k], meta[k], num_rows, (int64_t)feat_size * (b_dtype == LF_DTYPE_BF16 ? 2 : 4), s,
                                           &plan->owned, &plan->temp, &cb, &ok));
                    if (ok) {
                        cell_of[k] = (int)cells.size();
                        cells.push_back(cb);
                    } else {
                        rest.push_back(k);
                    }
                }
                chosen.swap(rest);
            }
            if (!chosen.empty()) {
                std::vector<int32_t*> m_arrays(chosen.size(), nullptr);
                for (size_t i = 0; i < chosen.size(); ++i)
                    LF_TRY(dev_alloc(plan, &m_arrays[i], (size_t)lf::ceil_div(h_buckets[chosen[i]].num_ell_rows, kGroupRows), true));
                LF_TRY(count_pass(chosen, false, &m_arrays));
                for (size_t i = 0; i < chosen.size(); ++i) {
                    const int k = chosen[i];
                    const lf_bucket_desc& b = h_buckets[k];
                    const unsigned long long entries = h_rg[3 * i], plain = h_rg[3 * i + 1], longest = h_rg[3 * i + 2];
                    if (entries == 0 || entries >= (1ull << 31) || longest > (unsigned long long)kMergedCap ||
                        entries * 100 > plain * kRowGroupMaxPercent)
                        continue;
                    MergedBucket mb{};
                    mb.n_rows = b.num_ell_rows;
                    mb.n_groups = lf::ceil_div(b.num_ell_rows, kGroupRows);
                    int32_t *goff = nullptr, *ecol = nullptr;
                    float4* eval = nullptr;
                    uint8_t* emask = nullptr;
                    LF_TRY(dev_alloc(plan, &goff, (size_t)mb.n_groups + 1));
                    LF_TRY(dev_alloc(plan, &ecol, (size_t)entries));
                    LF_TRY(dev_alloc(plan, &eval, (size_t)entries));
                    LF_TRY(dev_alloc(plan, &emask, (size_t)entries));
                    const int n_blocks = (int)lf::ceil_div(mb.n_groups, 1024);
                    int32_t* partial = nullptr;
                    LF_TRY(dev_alloc(plan, &partial, (size_t)n_blocks + 1, true));
                    LF_TRY_HIP(exclusive_scan_i32(m_arrays[i], mb.n_groups, partial, goff, s));
                    rowgroup_fill_kernel<<<(int)lf::ceil_div(mb.n_groups, 256), 256, 0, s>>>(
                        b.d_cols, b.d_vals, meta[k], b.num_ell_rows, lf::ilog2(b.width), mb.n_groups, goff, ecol, eval, emask);
                    LF_TRY_HIP(hipGetLastError());
                    // tile: one group per sub-wave (the tile is staged in rounds when its entries
                    // exceed the buffer), fewer when the bucket is small
                    const long long spread = lf::ceil_div(mb.n_groups, (long long)4 * plan->num_cus);
                    const long long per_tile = std::max<long long>(1, std::min<long long>(std::min(sw, kMergedTileGroups), spread));
                    mb.groups_per_tile = (int)per_tile;
                    mb.n_tiles = lf::ceil_div(mb.n_groups, per_tile);
                    mb.rows = b.d_rows;
                    mb.goff = goff;
                    mb.ecol = ecol;
                    mb.eval = eval;
                    mb.emask = emask;
                    merged_of[k] = (int)merged.size();
                    merged.push_back(mb);
                }
            }
        }
    }

    // ---- tile groups per launch: chunks first (longest), then buckets widest first, then clears
    std::vector<Group> groups;
    plan->launches.resize((size_t)num_parts);
    long long total_tiles = 0;
    for (int p = 0; p < num_parts; ++p) {
        lf_spmm_plan::Launch& L = plan->launches[p];
        L.group_begin = (int)groups.size();
        std::vector<int> mine;
        for (int k = 0; k < num_buckets; ++k)
            if (h_buckets[k].part == p && h_buckets[k].num_ell_rows > 0) mine.push_back(k);
        // Streaming stores leave the caches to B, but a launch whose rows are mostly short is
        // made of stores as much as of gathers and loses by them: 2.45M-row graph (33 entries per
        // row) 6.23 -> 6.13 ms, 500k x 2M matrix (most rows 2-4 entries) 1.46 -> 1.53 ms.
        long long rows_wide = 0, rows_all = 0;
        for (int k : mine) {
            rows_all += h_buckets[k].num_ell_rows;
            if (h_buckets[k].width >= kStreamMinWidth) rows_wide += h_buckets[k].num_ell_rows;
        }
        L.stream_c = rows_wide * 2 >= rows_all;
        for (int k : mine) L.wide_rows = L.wide_rows || has_wide[k];
        L.heavy_begin = mine.empty() ? 0 : heavy_base[mine.front()];
        L.n_heavy = mine.empty() ? 0 : heavy_base[mine.back() + 1] - L.heavy_begin;
        for (int k : mine) {
            if (counts[k].chunks == 0) continue;
            Group g{};
            g.type = kChunk;
            g.log_w = lf::ilog2(h_buckets[k].width);
            g.rows_per_tile = 1;
            g.cols = h_buckets[k].d_cols;
            g.vals = h_buckets[k].d_vals;
            g.n_items = g.n_tiles = counts[k].chunks;       // (those of dense rows last, in column order)
            g.chunks = d_chunks[k];
            groups.push_back(g);
        }
        std::sort(mine.begin(), mine.end(), [&](int x, int y) { return h_buckets[x].width > h_buckets[y].width; });
        for (int k : mine) {
            const lf_bucket_desc& b = h_buckets[k];
            if (b.width > kCoopSlots) continue;            // every row of this bucket is a chunk
            if (merged_of[k] >= 0 || cell_of[k] >= 0) continue;   // served by the row-group or the cell kernel
            Group g{};
            g.log_w = lf::ilog2(b.width);
            const int fit = tile_slots(lpr) >> g.log_w;     // ELL rows whose slots fit the LDS tile
            const bool staged = fit >= sw;
            g.type = staged ? (is_multi[k] ? kEllSeg : kEll) : kSeg;
            g.rows_per_tile = staged ? std::min(kTileRows, fit) : std::max(sw, fit);
            if (staged) {
                // a small bucket is cut into more, shorter tiles so that it still spreads over
                // the CUs: at least one pass of every sub-wave (8 rows at a time in the
                // narrow-bucket code), aiming at four tiles per CU
                const int unit = sw * (b.width < kUnroll ? kUnroll / b.width : 1);
                const long long want = lf::ceil_div(b.num_ell_rows, (long long)4 * plan->num_cus);
                const long long rows = std::max<long long>(unit, lf::ceil_div(want, (long long)unit) * unit);
                g.rows_per_tile = (int)std::min<long long>(g.rows_per_tile, rows);
            }
            if (g.type == kEllSeg) {
                const long long part_bytes = (long long)g.rows_per_tile * feat_size * 4;
                if (part_bytes <= kPartBytesMax) {
                    g.balanced = 1;
                    L.dyn_lds = std::max(L.dyn_lds, (int)part_bytes);
                }
            }
            g.n_items = b.num_ell_rows;
            g.n_tiles = lf::ceil_div(g.n_items, g.rows_per_tile);
            g.rows = b.d_rows;
            g.meta = meta[k];
            g.cols = b.d_cols;
            g.vals = b.d_vals;
            groups.push_back(g);
        }
        if (p == 0 && n_zero > 0) {
            Group g{};
            g.type = kZero;
            g.rows_per_tile = 1024;
            g.n_items = n_zero;
            g.n_tiles = lf::ceil_div(g.n_items, g.rows_per_tile);
            g.rows = d_zero_rows;
            groups.push_back(g);
        }
        L.n_groups = (int)groups.size() - L.group_begin;
        L.merged_begin = -1;
        for (int k : mine) {
            if (merged_of[k] < 0) continue;
            if (L.merged_begin < 0 || merged_of[k] < L.merged_begin) L.merged_begin = merged_of[k];
            ++L.n_merged;                                  // a partition's buckets are consecutive in `merged`
        }
        L.cell_begin = -1;
        for (int k : mine) {
            if (cell_of[k] < 0) continue;
            if (L.cell_begin < 0 || cell_of[k] < L.cell_begin) L.cell_begin = cell_of[k];
            ++L.n_cell_buckets;                            // a partition's buckets are consecutive in `cells`
        }
        if (L.n_cell_buckets > 0) {
            long long longest_c = 0;
            for (int x = 0; x < kXcds; ++x) {
                long long len = 0;
                for (int i = L.cell_begin; i < L.cell_begin + L.n_cell_buckets; ++i)
                    len += cells[i].n_tiles * (x + 1) / kXcds - cells[i].n_tiles * x / kXcds;
                longest_c = std::max(longest_c, len);
            }
            if (longest_c * kXcds >= (1ll << 31)) return bail(lf::fail(LF_ERR_UNSUPPORTED, "too many cell tiles"));
            L.cell_grid = (int)(longest_c * kXcds);
        }
        if (L.n_merged > 0) {
            long long longest_m = 0;
            for (int x = 0; x < kXcds; ++x) {
                long long len = 0;
                for (int i = L.merged_begin; i < L.merged_begin + L.n_merged; ++i)
                    len += merged[i].n_tiles * (x + 1) / kXcds - merged[i].n_tiles * x / kXcds;
                longest_m = std::max(longest_m, len);
            }
            if (longest_m * kXcds >= (1ll << 31)) return bail(lf::fail(LF_ERR_UNSUPPORTED, "too many row-group tiles"));
            L.merged_grid = (int)(longest_m * kXcds);
        }
        // grid: 8 x the longest per-XCD tile list
        long long longest = 0;
        for (int x = 0; x < kXcds; ++x) {
            long long len = 0;
            for (int gi = L.group_begin; gi < (int)groups.size(); ++gi)
                len += groups[gi].n_tiles * (x + 1) / kXcds - groups[gi].n_tiles * x / kXcds;
            longest = std::max(longest, len);
        }
        for (int gi = L.group_begin; gi < (int)groups.size(); ++gi) L.tiles += groups[gi].n_tiles;
        if (longest * kXcds >= (1ll << 31))
            return bail(lf::fail(LF_ERR_UNSUPPORTED, "partition %d needs too many tiles", p));
        L.grid = (int)(longest * kXcds);
        total_tiles += L.tiles;
    }
    if (!merged.empty()) {
        LF_TRY(dev_alloc(plan, &plan->d_merged, merged.size()));
        LF_TRY_HIP(hipMemcpy(plan->d_merged, merged.data(), merged.size() * sizeof(MergedBucket), hipMemcpyHostToDevice));
    }
    if (!cells.empty()) {
        LF_TRY(dev_alloc(plan, &plan->d_cells, cells.size()));
        LF_TRY_HIP(hipMemcpy(plan->d_cells, cells.data(), cells.size() * sizeof(LfCellBucket), hipMemcpyHostToDevice));
    }
    if (!groups.empty()) {
        LF_TRY(dev_alloc(plan, &plan->d_groups, groups.size()));
        LF_TRY_HIP(hipMemcpy(plan->d_groups, groups.data(), groups.size() * sizeof(Group), hipMemcpyHostToDevice));
    }

    KernelSet ks;
    LF_TRY(select_kernels(lpr, ch, b_dtype, &ks));
    int occ = 0;
    int dyn_lds = 0;
    plan->grid = 0;
    for (const auto& L : plan->launches) {
        plan->grid = std::max(plan->grid, L.grid);
        dyn_lds = std::max(dyn_lds, L.dyn_lds);
    }
    LF_TRY_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, ks.tiles, kWG, dyn_lds));

    plan->info[0] = total_tiles;
    plan->info[1] = plan->grid;
    plan->info[2] = num_parts;
    {
        hipFuncAttributes fa;
        LF_TRY_HIP(hipFuncGetAttributes(&fa, reinterpret_cast<const void*>(ks.tiles)));
        plan->info[3] = (int64_t)fa.sharedSizeBytes + dyn_lds;
    }
    plan->info[4] = n_heavy_total;
    plan->info[5] = n_partials;
    plan->info[6] = n_zero;
    (void)occ;
    plan->info[7] = (int64_t)(merged.size() + cells.size());
    plan->info[8] = (int64_t)cells.size();
    LF_TRY_HIP(hipStreamSynchronize(s));     // the tables are complete: the plan may run on any stream
    if (free_temporaries(plan) != LF_OK) return bail(lf::fail(LF_ERR_HIP, "hipFree failed on plan-time scratch"));
    *out_plan = plan;
    return LF_OK;
#undef LF_TRY
#undef LF_TRY_HIP
}

int lf_spmm_info(const lf_spmm_plan* plan, int64_t* h_info) {
    LF_REQUIRE(plan && h_info, LF_ERR_INVALID, "null argument");
    std::memcpy(h_info, plan->info, sizeof(plan->info));
    return LF_OK;
}

int lf_spmm_run(lf_spmm_plan* plan, const void* d_B, float* d_C, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(plan, LF_ERR_INVALID, "plan is null");
    if (plan->num_rows == 0) return LF_OK;
    LF_REQUIRE(d_B && d_C, LF_ERR_INVALID, "B or C is null");
    LF_REQUIRE((uintptr_t)d_B % 16 == 0 && (uintptr_t)d_C % 16 == 0, LF_ERR_INVALID, "B and C must be 16-byte aligned");
    KernelSet ks;
    if (int rc = select_kernels(plan->lpr, plan->ch, plan->b_dtype, &ks)) return rc;
    // One pass per feature window (all partitions inside), each on its own columns of B and C.
    const size_t b_elem = plan->b_dtype == LF_DTYPE_BF16 ? 2 : 4;
    const int ld = plan->feat * plan->windows;
    for (int w = 0; w < plan->windows; ++w) {
        for (int p = 0; p < plan->num_parts; ++p) {
            const lf_spmm_plan::Launch& L = plan->launches[p];
            if (L.n_groups == 0 && L.n_merged == 0 && L.n_cell_buckets == 0) continue;
            LaunchArgs a{};
            a.groups = plan->d_groups + L.group_begin;
            a.n_groups = L.n_groups;
            a.accumulate = (p > 0 ? kAccumulateC : 0) | (p + 1 == plan->num_parts && L.stream_c ? kStreamC : 0) |
                           (plan->stream_slabs ? kStreamSlabs : 0);
            a.feat = plan->feat;
            a.ldb = a.ldc = ld;
            a.B = (const char*)d_B + (size_t)w * plan->feat * b_elem;
            a.C = d_C + (size_t)w * plan->feat;
            a.partials = plan->d_partials;
            if (L.grid > 0) {
                ks.tiles<<<L.grid, kWG, L.dyn_lds, s>>>(a);
                LF_HIP(hipGetLastError());
            }
            if (L.n_merged > 0) {
                ks.rowgroup<<<L.merged_grid, kWG, 0, s>>>(plan->d_merged + L.merged_begin, L.n_merged, a);
                LF_HIP(hipGetLastError());
            }
            if (L.n_cell_buckets > 0) {
                if (int rc = lf::cells_launch(plan->d_cells + L.cell_begin, L.n_cell_buckets, L.cell_grid, plan->b_dtype,
                                              a.B, a.C, a.feat, a.ldb, a.ldc, a.accumulate, s))
                    return rc;
            }
            if (L.n_heavy > 0) {
                const int sw = kWG / plan->lpr;
                const int fgrid = std::min((L.n_heavy + sw - 1) / sw, 1024);
                ks.finalize<<<fgrid, kWG, 0, s>>>(plan->d_heavy + L.heavy_begin, L.n_heavy, a);
                LF_HIP(hipGetLastError());
                if (L.wide_rows) {
                    ks.finalize_wide<<<L.n_heavy, kWG, 0, s>>>(plan->d_heavy + L.heavy_begin, L.n_heavy, a);
                    LF_HIP(hipGetLastError());
                }
            }
        }
    }
    return LF_OK;
}

int lf_spmm_set_windows(lf_spmm_plan* plan, int32_t n_windows) {
    LF_REQUIRE(plan, LF_ERR_INVALID, "plan is null");
    LF_REQUIRE(n_windows >= 1 && (int64_t)n_windows * plan->feat <= (1 << 20), LF_ERR_INVALID,
               "bad number of feature windows (%d)", n_windows);
    plan->windows = n_windows;
    return LF_OK;
}

int lf_csr_spmm_trusted(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                        int64_t num_rows, int64_t num_cols, int32_t feat_size, int32_t b_dtype,
                        const void* d_B, float* d_C, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && num_cols >= 1, LF_ERR_INVALID, "bad shape");
    if (num_rows == 0) return LF_OK;
    LF_REQUIRE(d_indptr && d_B && d_C, LF_ERR_INVALID, "null argument");
    LF_REQUIRE(b_dtype == LF_DTYPE_F32 || b_dtype == LF_DTYPE_BF16, LF_ERR_INVALID, "unknown B dtype %d", b_dtype);
    LF_REQUIRE((uintptr_t)d_B % 16 == 0 && (uintptr_t)d_C % 16 == 0, LF_ERR_INVALID, "B and C must be 16-byte aligned");
    int lpr, ch;
    if (int rc = feature_shape(feat_size, b_dtype, &lpr, &ch)) return rc;
    KernelSet ks;
    if (int rc = select_kernels(lpr, ch, b_dtype, &ks)) return rc;
    LaunchArgs a{};
    a.feat = feat_size;
    a.ldb = a.ldc = feat_size;
    a.B = d_B;
    a.C = d_C;
    const int sw = kWG / lpr;
    const int grid = (int)std::min<long long>((num_rows + sw - 1) / sw, 1 << 20);
    ks.csr<<<grid, kWG, 0, s>>>(d_indptr, d_indices, d_values, num_rows, a);
    LF_HIP(hipGetLastError());
    return LF_OK;
}

int lf_csr_spmm(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                int64_t num_rows, int64_t num_cols, int64_t nnz, int32_t feat_size, int32_t b_dtype,
                const void* d_B, float* d_C, void* d_scratch, lf_stream_t stream) {
    // arguments first, so that a bad feature size or operand is reported without touching the GPU
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && num_cols >= 1, LF_ERR_INVALID, "bad shape");
    if (num_rows > 0) {
        LF_REQUIRE(d_indptr && d_B && d_C, LF_ERR_INVALID, "null argument");
        LF_REQUIRE(b_dtype == LF_DTYPE_F32 || b_dtype == LF_DTYPE_BF16, LF_ERR_INVALID, "unknown B dtype %d", b_dtype);
        int lpr, ch;
        if (int rc = feature_shape(feat_size, b_dtype, &lpr, &ch)) return rc;
    }
    // no gather before the index arrays have passed
    if (int rc = lf::csr_check(d_indptr, d_indices, nullptr, num_rows, num_cols, nnz, d_scratch, nullptr, "lf_csr_spmm",
                               (hipStream_t)stream))
        return rc;
    return lf_csr_spmm_trusted(d_indptr, d_indices, d_values, num_rows, num_cols, feat_size, b_dtype, d_B, d_C, stream);
}

int lf_spmm_time_ms(lf_spmm_plan* plan, const void* d_B, float* d_C, int32_t warmup, int32_t repeat,
                    void* d_flush, size_t flush_bytes, float* h_ms, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(plan && h_ms, LF_ERR_INVALID, "null argument");
    LF_REQUIRE(warmup >= 0 && repeat >= 1, LF_ERR_INVALID, "bad warmup/repeat");
    for (int i = 0; i < warmup; ++i)
        if (int rc = lf_spmm_run(plan, d_B, d_C, stream)) return rc;
    hipEvent_t t0, t1;
    LF_HIP(hipEventCreate(&t0));
    if (hipError_t e = hipEventCreate(&t1)) {
        (void)hipEventDestroy(t0);
        return lf::fail(LF_ERR_HIP, "hipEventCreate failed: %s", hipGetErrorString(e));
    }
    int rc = LF_OK;
    for (int i = 0; i < repeat && rc == LF_OK; ++i) {
        if (d_flush && flush_bytes >= 4) {
            const long long words = (long long)(flush_bytes / 4);
            fill_bytes_kernel<<<(int)std::min<long long>((words + 255) / 256, 8192), 256, 0, s>>>((uint32_t*)d_flush, words, (uint32_t)i);
        }
        hipError_t e = hipEventRecord(t0, s);
        if (e == hipSuccess) {
            rc = lf_spmm_run(plan, d_B, d_C, stream);
            if (rc != LF_OK) break;
            e = hipEventRecord(t1, s);
        }
        if (e == hipSuccess) e = hipEventSynchronize(t1);
        if (e == hipSuccess) e = hipEventElapsedTime(&h_ms[i], t0, t1);
        if (e != hipSuccess) rc = lf::fail(LF_ERR_HIP, "timing failed: %s", hipGetErrorString(e));
    }
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    return rc;
}

}  // extern "C"
