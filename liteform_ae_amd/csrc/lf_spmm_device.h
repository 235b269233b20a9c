// Device-side building blocks shared by the SpMM kernels of liblfhip.so: launch arguments,
// dense-operand access (one 16-byte load per lane), per-lane accumulators, row stores.
// Everything lives in an anonymous namespace: each translation unit gets its own copy.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "lf_internal.h"

namespace {

constexpr int kWG = 256;            // threads per workgroup (4 wavefronts)
#ifndef LF_TILE_SLOTS_PER_SUBWAVE
#define LF_TILE_SLOTS_PER_SUBWAVE 64
#endif
#ifndef LF_UNROLL
#define LF_UNROLL 8
#endif
#ifndef LF_TILE_MIN
#define LF_TILE_MIN 512
#endif
// (col, val) pairs staged in LDS per tile: a fixed amount of work per sub-wave, so narrow
// feature sizes (many sub-waves per workgroup) get larger tiles.  N = 128 -> 512 slots.
constexpr int tile_slots(int lpr) {
    const int n = LF_TILE_SLOTS_PER_SUBWAVE * (kWG / lpr);
    return n < LF_TILE_MIN ? LF_TILE_MIN : n;
}
constexpr int kTileRows = 512;      // ELL rows per tile at most (<= tile_slots)
#ifndef LF_COOP_SLOTS
#define LF_COOP_SLOTS 256
#endif
#ifndef LF_CHUNK_SLOTS
#define LF_CHUNK_SLOTS 2048
#endif
constexpr int kCoopSlots = LF_COOP_SLOTS;    // a source row with more slab slots is reduced by a whole workgroup
constexpr int kChunkSlots = LF_CHUNK_SLOTS;  // ... in chunks of this many slots (a whole number of ELL rows)
constexpr int kChunkSlotsLarge = 8192;       // ... or this many, in a matrix of at least kLargeMatrixSlots slots
constexpr long long kLargeMatrixSlots = 4ll << 20;
// Dense rows: a row holding at least 1/kDenseRowShare of its partition's columns.  Several of
// them read much the same rows of B, so they are cut into shorter chunks that are walked in
// column order: the chunks in flight then cover a window of B that the memory-side cache holds,
// and a row of B is fetched from HBM once for all of them.  500k x 2M matrix with 50 rows of
// 100,000 entries, bf16 N = 512, ms per product by chunk size (whole workgroup per chunk):
// 8192 unordered 1.46; ordered 8192 1.53, 4096 1.43, 2048 1.39, 1024 1.295, 512 1.30, 256 1.40,
// 128 1.70; a sub-wave per chunk: 512 1.40, 256 1.37, 128 1.34, 64 1.44.  (Short enough for
// the window to fit an XCD's L2 they would need far fewer chunks in flight than fill the GPU.)
constexpr int kDenseRowShare = 32;
constexpr int kDenseRowMinSlots = 4096;
constexpr long long kDenseMinBBytes = 128ll << 20;   // ... in a partition whose part of B is larger than this
constexpr int kDenseChunkSlots = 1024;
constexpr int kWideFinalPartials = 64;       // rows with more partial rows are added up by a whole workgroup
constexpr int kXcds = 8;
constexpr int kPartBytesMax = 16384;   // LDS for per-ELL-row sums of a balanced segment tile at most
constexpr int kUnroll = LF_UNROLL;  // B-row gathers in flight per sub-wave
constexpr uint32_t kMetaLenMask = 0x7FFu;
constexpr int kMetaLenBits = 11;

enum GroupType : int { kEll = 0, kSeg = 1, kZero = 2, kChunk = 3, kEllSeg = 4 };

constexpr int kChunkDenseBit = 1 << 30;       // in Chunk::n_slots while the plan is built: a piece of a dense row

struct Chunk {
    long long slot_begin;   // first slot, relative to the bucket's slab
    int n_slots;
    int partial;            // index of the partial row this chunk produces; < 0: the chunk is the
                            // whole source row and goes straight to C
    int row;                // source row
    int first_col;          // column of the chunk's first slot (chunks of dense rows are ordered by it)
};

struct HeavyRow {
    int row;
    int partial_begin;
    int n_partials;
    int pad_;
};

struct Group {
    int type;
    int log_w;
    int rows_per_tile;
    int balanced;                 // kEllSeg: per-ELL-row sums through LDS (needs rows_per_tile * N floats)
    long long n_items;            // ELL rows / rows to clear / chunks
    long long n_tiles;
    const int32_t* rows;          // kEll, kSeg: source rows; kZero: rows to clear
    const int32_t* meta;
    const int32_t* cols;
    const float* vals;
    const Chunk* chunks;          // kChunk
};

struct LaunchArgs {
    const Group* groups;
    int n_groups;
    int accumulate;               // bit 0: C += result instead of C = result; bit 1 (kStreamC): no later
                                  // launch of the run reads these rows of C again; bit 2 (kStreamSlabs):
                                  // the slabs are too large to be worth caching
    int feat;                     // N: features computed by the launch
    int ldb, ldc;                 // row strides of B and C in elements (N, or more for a feature window)
    int pad_;
    const void* B;
    float* C;
    float* partials;
};

// ------------------------------------------------------------------------------------
// Dense-operand access: VEC features per lane as one 16-byte load.
template <typename BT> struct Dense;

template <> struct Dense<float> {
    static constexpr int kVec = 4;
    static constexpr int kElemBytes = 4;
    __device__ static __forceinline__ void load(const char* at, float (&x)[4]) {
        const float4 v = *reinterpret_cast<const float4*>(at);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    }
};

struct bf16_t { uint16_t bits; };

template <> struct Dense<bf16_t> {
    static constexpr int kVec = 8;
    static constexpr int kElemBytes = 2;
    __device__ static __forceinline__ void load(const char* at, float (&x)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(at);
        x[0] = __uint_as_float(v.x << 16); x[1] = __uint_as_float(v.x & 0xFFFF0000u);
        x[2] = __uint_as_float(v.y << 16); x[3] = __uint_as_float(v.y & 0xFFFF0000u);
        x[4] = __uint_as_float(v.z << 16); x[5] = __uint_as_float(v.z & 0xFFFF0000u);
        x[6] = __uint_as_float(v.w << 16); x[7] = __uint_as_float(v.w & 0xFFFF0000u);
    }
};

// Accumulator of one sub-wave lane: CH chunks of VEC features.
template <int CH, int VEC> struct Acc {
    float v[CH][VEC];
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < VEC; ++i) v[c][i] = 0.f;
    }
};

// Position of a lane inside the feature dimension.
template <int LPR, int CH, int VEC> struct Lane {
    int sl;                 // lane inside the sub-wave
    int feat;               // N: features this launch computes
    int ldb, ldc;           // elements between consecutive rows of B and of C (>= N)
    int f[CH];              // first feature of each chunk (clamped to 0 when outside N)
    bool on[CH];
    __device__ __forceinline__ Lane(int sl_, int feat_, int ldb_, int ldc_)
        : sl(sl_), feat(feat_), ldb(ldb_), ldc(ldc_) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int f0 = (c * LPR + sl_) * VEC;
            on[c] = f0 < feat_;
            f[c] = on[c] ? f0 : 0;
        }
    }
};

// Where lane `ln` finds its 16 bytes of row `col` of B: the lane's own place in row 0 plus
// col * (bytes between rows) - one 32 x 32 -> 64-bit multiply-add per gather.  (Indexing in
// elements, with the row stride as a signed int, cost two 64-bit multiply-adds, two moves and a
// shift-add per gather: more vector instructions than the four FMAs the gather feeds.)
template <typename BT, int LPR, int CH>
__device__ __forceinline__ const char* dense_row(const void* B, const Lane<LPR, CH, Dense<BT>::kVec>& ln, int c,
                                                 int col) {
    const char* lane0 = reinterpret_cast<const char*>(B) + (size_t)ln.f[c] * Dense<BT>::kElemBytes;
    const uint32_t pitch = (uint32_t)ln.ldb * (uint32_t)Dense<BT>::kElemBytes;      // ldb <= 2^20
    return lane0 + (uint64_t)(uint32_t)col * pitch;
}

template <int U, int LPR, int CH, typename BT>
__device__ __forceinline__ void gather_fma(const void* B, const Lane<LPR, CH, Dense<BT>::kVec>& ln,
                                           const int (&col)[U], const float (&val)[U],
                                           Acc<CH, Dense<BT>::kVec>& acc) {
    constexpr int VEC = Dense<BT>::kVec;
    float x[U][CH][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int c = 0; c < CH; ++c)
            Dense<BT>::load(dense_row<BT>(B, ln, c, col[u]), x[u][c]);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc.v[c][i] = fmaf(val[u], x[u][c][i], acc.v[c][i]);
}

// flags: LaunchArgs::accumulate.  Rows that nothing reads again in this run are stored
// non-temporally where the launch's rows are mostly wide, which leaves the caches to B (2.45M-row
// graph, N = 128: 6.23 -> 6.13 ms); rows that a later column partition adds to stay cached
// (170k-row graph, two partitions: streaming them costs 7 %).
constexpr int kAccumulateC = 1, kStreamC = 2, kStreamSlabs = 4;
constexpr int kStreamMinWidth = 16;      // a launch streams C when at least half of its ELL rows are this wide
typedef float lf_f32x4 __attribute__((ext_vector_type(4)));

// 16 bytes to global memory, streamed or not by a run-time flag.  The streaming store goes
// through a global-memory pointer made from the address as an integer: with the same pointer in
// both branches the compiler folds the two stores into one ordinary store.
__device__ __forceinline__ void store_f32x4(float* dst, lf_f32x4 o, bool stream) {
    if (stream)
        __builtin_nontemporal_store(o, reinterpret_cast<lf_f32x4 __attribute__((address_space(1)))*>(reinterpret_cast<uintptr_t>(dst)));
    else
        *reinterpret_cast<lf_f32x4*>(dst) = o;
}

// 16 bytes of a slab, streamed or not (same construction as store_f32x4)
typedef int lf_i32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ lf_i32x4 load_i32x4(const void* src, bool stream) {
    if (stream)
        return __builtin_nontemporal_load(
            reinterpret_cast<const lf_i32x4 __attribute__((address_space(1)))*>(reinterpret_cast<uintptr_t>(src)));
    return *reinterpret_cast<const lf_i32x4*>(src);
}

template <int LPR, int CH, int VEC>
__device__ __forceinline__ void store_row(float* C, int row, const Lane<LPR, CH, VEC>& ln,
                                          const Acc<CH, VEC>& acc, int flags) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if (!ln.on[c]) continue;
        float* dst = C + (size_t)row * ln.ldc + ln.f[c];
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
            lf_f32x4 o = {acc.v[c][i], acc.v[c][i + 1], acc.v[c][i + 2], acc.v[c][i + 3]};
            if (flags & kAccumulateC) o += *reinterpret_cast<const lf_f32x4*>(dst + i);
            store_f32x4(dst + i, o, flags & kStreamC);
        }
    }
}

// goff[g] = exclusive prefix of m[g], goff[n_groups] = total, in three small launches:
// sums of blocks of 1024 groups, their exclusive scan by one workgroup (in place, total
// appended), then the scan inside every block.
__device__ __forceinline__ int block_inclusive_scan_1024(int x, int* s_wave) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = x;
    for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_up(incl, d);
        if (lane >= d) incl += y;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    for (int w = 0; w < wave; ++w) incl += s_wave[w];
    __syncthreads();
    return incl;
}

__global__ void __launch_bounds__(1024)
scan_blocksum_kernel(const int32_t* __restrict__ m, long long n_groups, int32_t* __restrict__ partial) {
    __shared__ int s_wave[16];
    const long long i = (long long)blockIdx.x * 1024 + threadIdx.x;
    const int incl = block_inclusive_scan_1024(i < n_groups ? m[i] : 0, s_wave);
    if (threadIdx.x == 1023) partial[blockIdx.x] = incl;
}

__global__ void __launch_bounds__(1024)
scan_partials_kernel(int32_t* __restrict__ partial, int n_blocks) {
    __shared__ int s_wave[16];
    __shared__ int s_carry;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    for (int base = 0; base < n_blocks; base += 1024) {
        const int i = base + threadIdx.x;
        const int x = i < n_blocks ? partial[i] : 0;
        const int incl = block_inclusive_scan_1024(x, s_wave);
        const int carry = s_carry;
        if (i < n_blocks) partial[i] = carry + incl - x;
        __syncthreads();
        if (threadIdx.x == 1023) s_carry = carry + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[n_blocks] = s_carry;
}

__global__ void __launch_bounds__(1024)
scan_blocks_kernel(const int32_t* __restrict__ m, long long n_groups, const int32_t* __restrict__ partial,
                     int n_blocks, int32_t* __restrict__ goff) {
    __shared__ int s_wave[16];
    const long long i = (long long)blockIdx.x * 1024 + threadIdx.x;
    const int x = i < n_groups ? m[i] : 0;
    const int incl = block_inclusive_scan_1024(x, s_wave);
    if (i < n_groups) goff[i] = partial[blockIdx.x] + incl - x;
    if (blockIdx.x == 0 && threadIdx.x == 0) goff[n_groups] = partial[n_blocks];
}

// off[i] = exclusive prefix of m[i] for i < n, off[n] = total, enqueued on `s`.  `partial`
// needs ceil(n / 1024) + 1 ints.
inline hipError_t exclusive_scan_i32(const int32_t* m, long long n, int32_t* partial, int32_t* off, hipStream_t s) {
    const int n_blocks = (int)((n + 1023) / 1024);
    if (n_blocks == 0) return hipSuccess;
    scan_blocksum_kernel<<<n_blocks, 1024, 0, s>>>(m, n, partial);
    scan_partials_kernel<<<1, 1024, 0, s>>>(partial, n_blocks);
    scan_blocks_kernel<<<n_blocks, 1024, 0, s>>>(m, n, partial, n_blocks, off);
    return hipGetLastError();
}

}  // namespace
