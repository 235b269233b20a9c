// Block-sparse (BSR, square blocks of 16, 32 or 64) fp16 SpMM on the gfx950 matrix cores:
//     Y[mb*BS][F] (fp16) = A_bsr (fp16 blocks) . X[nb*BS][F] (fp16),  fp32 accumulation.
//
// Takes over the kernel that bench_bsrmm builds through SparseTIR/TVM with fp16 WMMA
// 16x16x16 fragments (playground_pipline/format_algos.py:1182-1643; any block size that is a
// multiple of 16 there, format_algos.py:1581-1582; 32 is what the driver passes,
// proc05.spmm.end-to-end.py:205).  This is the one place of the library where dense-block
// matrix-core work is the right shape; it is still HBM-bound (2 KiB of A and 32 rows of X per
// 32x32xF block product: ~26 flop/byte at F = 128), so the kernels are organised around
// coalesced loads, not around MFMA occupancy.
//
// One workgroup (4 wavefronts) per (block row, 128-feature tile); wavefront w owns features
// [32w, 32w+32) of the tile.
//   * blocks of 32 and 64: one 32x32 fp32 accumulator tile per 32 rows of the block row
//     (v_mfma_f32_32x32x8_f16, BS / 8 K-steps per nonzero block);
//   * blocks of 16: two 16x16 accumulator tiles (v_mfma_f32_16x16x16_f16, one K-step per
//     nonzero block and tile).
// The X tile needs four consecutive k (= four different rows of X) per lane, so it is loaded
// row-wise with 16-byte accesses and transposed through LDS: stored as XT[feature][k], read
// back as one 8-byte access; the next block's tile is in flight during the matrix
// instructions (two LDS buffers).  A blocks of 16 rows are read straight from global memory in
// the MFMA A layout (lane: one row, four consecutive k - 512 contiguous bytes per block);
// larger blocks are staged through LDS with 16-byte loads.  The accumulators hold one feature and many rows
// per lane; the result goes back through LDS so that a lane stores 16 contiguous bytes of one
// row of Y instead of one 2-byte element per row.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <algorithm>

#include "lf_internal.h"

namespace {

constexpr int kFeatTile = 128;     // features per workgroup
constexpr int kWgBsr = 256;
constexpr int kYPad = 8;           // halves of padding per staged row of Y (keeps 16-byte reads aligned)

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// halves per XT row: BS + 4 keeps 8-byte reads aligned and spreads banks
template <int BS> constexpr int xt_stride() { return BS + 4; }
template <int BS> constexpr int lds_halves() {
    const int xt = 2 * kFeatTile * xt_stride<BS>();
    const int y = BS * (kFeatTile + kYPad);
    return xt > y ? xt : y;
}

// The staged tile of Y, rows x 128 features, to global memory: 16 bytes per lane, 16 rows per pass.
template <int BS>
__device__ __forceinline__ void store_y_tile(const _Float16* s_y, _Float16* __restrict__ Y, size_t row0, int f0, int feat) {
    const int tid = threadIdx.x;
    const int vec = tid & 15;                // features 8 * vec .. + 7 of the tile
    const int f = f0 + 8 * vec;
    if (f >= feat) return;                   // feat is a multiple of 8: a vector is inside or outside
#pragma unroll
    for (int r = tid >> 4; r < BS; r += kWgBsr / 16) {
        const uint4 v = *reinterpret_cast<const uint4*>(s_y + r * (kFeatTile + kYPad) + 8 * vec);
        *reinterpret_cast<uint4*>(Y + (row0 + r) * feat + f) = v;
    }
}

// Blocks of 32 (RH = 1) or 64 (RH = 2) rows and columns.  The A block goes through LDS as well:
// read straight from global memory in the MFMA layout, a lane's 8 bytes lie a whole block row
// (64 or 128 bytes) from its neighbour's, one cache line per lane or pair of lanes, and all four
// wavefronts fetch the same block (64 x 64 blocks, N = 128: 1.13 ms that way).
template <int BS>
__global__ void __launch_bounds__(kWgBsr)
bsr_spmm_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices,
                const _Float16* __restrict__ data, const _Float16* __restrict__ X,
                _Float16* __restrict__ Y, int feat) {
    constexpr int RH = BS / 32;              // 32-row halves of a block row
    constexpr int KP = xt_stride<BS>();
    constexpr int AP = BS + 4;               // halves per staged row of A
    constexpr int AV = BS * BS / 8 / kWgBsr > 0 ? BS * BS / 8 / kWgBsr : 1;   // 16-byte vectors of A per thread
    __shared__ __align__(16) _Float16 s_raw[lds_halves<BS>()];
    __shared__ __align__(16) _Float16 s_a[2][BS * AP];
    auto xt_buf = [&](int buf) { return s_raw + buf * kFeatTile * KP; };

    const int brow = blockIdx.x;
    const int f0 = blockIdx.y * kFeatTile;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int li = lane & 31, kq = lane >> 5;

    // cooperative X-tile load: thread t reads rows t/8 (+32) of the block, two 16-byte vectors each
    const int xr = tid >> 3;                 // 0..31: row inside the block (= k)
    const int xv = tid & 7;                  // vector 0..7 -> features 8*xv and 64 + 8*xv
    const bool in0 = f0 + 8 * xv < feat, in1 = f0 + 64 + 8 * xv < feat;
    // cooperative A-block load: 16-byte vectors in memory order (BS / 8 per row)
    const bool a_on = tid < BS * BS / 8;     // 32 x 32: the first 128 threads

    float16_t acc[RH];
#pragma unroll
    for (int h = 0; h < RH; ++h)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[h][v] = 0.f;

    const int jb = indptr[brow], je = indptr[brow + 1];
    uint4 x0[RH], x1[RH], av[AV];
    auto load_x = [&](int j) {
        const _Float16* src = X + ((size_t)indices[j] * BS + xr) * feat + f0 + 8 * xv;
#pragma unroll
        for (int h = 0; h < RH; ++h) {
            x0[h] = in0 ? *reinterpret_cast<const uint4*>(src + (size_t)32 * h * feat) : make_uint4(0, 0, 0, 0);
            x1[h] = in1 ? *reinterpret_cast<const uint4*>(src + (size_t)32 * h * feat + 64) : make_uint4(0, 0, 0, 0);
        }
        const uint4* asrc = reinterpret_cast<const uint4*>(data + (size_t)j * BS * BS);
#pragma unroll
        for (int i = 0; i < AV; ++i)
            if (a_on) av[i] = asrc[tid + i * kWgBsr];
    };
    auto store_lds = [&](int buf) {
        _Float16* dst = xt_buf(buf);
#pragma unroll
        for (int h = 0; h < RH; ++h) {
            const _Float16* h0 = reinterpret_cast<const _Float16*>(&x0[h]);
            const _Float16* h1 = reinterpret_cast<const _Float16*>(&x1[h]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                dst[(8 * xv + i) * KP + 32 * h + xr] = h0[i];
                dst[(64 + 8 * xv + i) * KP + 32 * h + xr] = h1[i];
            }
        }
#pragma unroll
        for (int i = 0; i < AV; ++i) {
            if (!a_on) continue;
            const int v = tid + i * kWgBsr;                  // vector v: row v / (BS / 8), halves 8 * (v % (BS / 8)) ..
            _Float16* d = s_a[buf] + (v / (BS / 8)) * AP + 8 * (v % (BS / 8));
            *reinterpret_cast<uint2*>(d) = make_uint2(av[i].x, av[i].y);           // (rows are 8-byte aligned: AP = BS + 4)
            *reinterpret_cast<uint2*>(d + 4) = make_uint2(av[i].z, av[i].w);
        }
    };

    if (jb < je) {
        load_x(jb);
        store_lds(0);
    }
    __syncthreads();
    for (int j = jb; j < je; ++j) {
        const int buf = (j - jb) & 1;
        if (j + 1 < je) load_x(j + 1);                       // next tiles in flight during the MFMAs
        const _Float16* ablk = s_a[buf] + li * AP + 4 * kq;
        const _Float16* xt = xt_buf(buf) + (32 * wave + li) * KP + 4 * kq;
#pragma unroll
        for (int s = 0; s < BS / 8; ++s) {
            const half4_t b = *reinterpret_cast<const half4_t*>(xt + 8 * s);
#pragma unroll
            for (int h = 0; h < RH; ++h) {
                const half4_t a = *reinterpret_cast<const half4_t*>(ablk + 32 * h * AP + 8 * s);
                acc[h] = __builtin_amdgcn_mfma_f32_32x32x8f16(a, b, acc[h], 0, 0, 0);
            }
        }
        if (j + 1 < je) store_lds(buf ^ 1);
        __syncthreads();
    }

    // D layout of the 32x32 MFMA: lane holds column li, rows 8*(v/4) + 4*kq + v%4.  (The last
    // barrier of the loop - or the one before it for an empty block row - has retired every read
    // of the X tiles, so the staging buffer can take their place.)
    _Float16* s_y = s_raw;
#pragma unroll
    for (int h = 0; h < RH; ++h)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 32 * h + 8 * (v >> 2) + 4 * kq + (v & 3);
            s_y[row * (kFeatTile + kYPad) + 32 * wave + li] = (_Float16)acc[h][v];
        }
    __syncthreads();
    store_y_tile<BS>(s_y, Y, (size_t)brow * BS, f0, feat);
}

// Blocks of 16 rows and columns: two 16x16 accumulator tiles per wavefront.
__global__ void __launch_bounds__(kWgBsr)
bsr16_spmm_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices,
                  const _Float16* __restrict__ data, const _Float16* __restrict__ X,
                  _Float16* __restrict__ Y, int feat) {
    constexpr int BS = 16;
    constexpr int KP = xt_stride<BS>();
    __shared__ __align__(16) _Float16 s_raw[lds_halves<BS>()];
    auto xt_buf = [&](int buf) { return s_raw + buf * kFeatTile * KP; };

    const int brow = blockIdx.x;
    const int f0 = blockIdx.y * kFeatTile;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int li = lane & 15, kq = lane >> 4;            // row (A) / column (B, D) and group of four k

    // cooperative X-tile load: thread t reads row t/16 of the block, one 16-byte vector
    const int xr = tid >> 4;                 // 0..15
    const int xv = tid & 15;                 // features 8*xv .. + 7
    const bool in0 = f0 + 8 * xv < feat;

    float4_t acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[t][v] = 0.f;

    const int jb = indptr[brow], je = indptr[brow + 1];
    uint4 x0 = make_uint4(0, 0, 0, 0);
    auto load_x = [&](int j) {
        const _Float16* src = X + ((size_t)indices[j] * BS + xr) * feat + f0 + 8 * xv;
        x0 = in0 ? *reinterpret_cast<const uint4*>(src) : make_uint4(0, 0, 0, 0);
    };
    auto store_xt = [&](int buf) {
        _Float16* dst = xt_buf(buf);
        const _Float16* h0 = reinterpret_cast<const _Float16*>(&x0);
#pragma unroll
        for (int i = 0; i < 8; ++i) dst[(8 * xv + i) * KP + xr] = h0[i];
    };

    if (jb < je) {
        load_x(jb);
        store_xt(0);
    }
    __syncthreads();
    for (int j = jb; j < je; ++j) {
        const int buf = (j - jb) & 1;
        if (j + 1 < je) load_x(j + 1);
        const half4_t a = *reinterpret_cast<const half4_t*>(data + (size_t)j * BS * BS + li * BS + 4 * kq);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const half4_t b = *reinterpret_cast<const half4_t*>(xt_buf(buf) + (32 * wave + 16 * t + li) * KP + 4 * kq);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, acc[t], 0, 0, 0);
        }
        if (j + 1 < je) store_xt(buf ^ 1);
        __syncthreads();
    }

    // D layout of the 16x16 MFMA: lane holds column li, rows 4*kq + v
    _Float16* s_y = s_raw;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v)
            s_y[(4 * kq + v) * (kFeatTile + kYPad) + 32 * wave + 16 * t + li] = (_Float16)acc[t][v];
    __syncthreads();
    store_y_tile<BS>(s_y, Y, (size_t)brow * BS, f0, feat);
}

}  // namespace

extern "C" {

int lf_bsr_spmm_trusted(const int32_t* d_indptr, const int32_t* d_indices, const void* d_data,
                        int64_t num_block_rows, int64_t num_block_cols, int32_t block_size,
                        int32_t feat_size, const void* d_X, void* d_Y, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(block_size == 16 || block_size == 32 || block_size == 64, LF_ERR_UNSUPPORTED,
               "blocks of 16, 32 or 64 rows and columns are supported (got %d)", block_size);
    LF_REQUIRE(num_block_rows >= 0 && num_block_rows < (1ll << 26) && num_block_cols >= 1 &&
                   num_block_cols < (1ll << 26), LF_ERR_INVALID, "bad block shape");
    LF_REQUIRE(feat_size >= 8 && feat_size % 8 == 0, LF_ERR_UNSUPPORTED,
               "feat_size must be a positive multiple of 8 (got %d)", feat_size);
    if (num_block_rows == 0) return LF_OK;
    LF_REQUIRE(d_indptr && d_X && d_Y, LF_ERR_INVALID, "null argument");
    LF_REQUIRE((uintptr_t)d_X % 16 == 0 && (uintptr_t)d_Y % 16 == 0 && (uintptr_t)d_data % 16 == 0, LF_ERR_INVALID,
               "X, Y and the block data must be 16-byte aligned");
    const dim3 grid((unsigned)num_block_rows, (unsigned)((feat_size + kFeatTile - 1) / kFeatTile));
    const _Float16* data = (const _Float16*)d_data;
    const _Float16* X = (const _Float16*)d_X;
    _Float16* Y = (_Float16*)d_Y;
    if (block_size == 16) bsr16_spmm_kernel<<<grid, kWgBsr, 0, s>>>(d_indptr, d_indices, data, X, Y, feat_size);
    else if (block_size == 32) bsr_spmm_kernel<32><<<grid, kWgBsr, 0, s>>>(d_indptr, d_indices, data, X, Y, feat_size);
    else bsr_spmm_kernel<64><<<grid, kWgBsr, 0, s>>>(d_indptr, d_indices, data, X, Y, feat_size);
    LF_HIP(hipGetLastError());
    return LF_OK;
}

int lf_bsr_spmm(const int32_t* d_indptr, const int32_t* d_indices, const void* d_data,
                int64_t num_block_rows, int64_t num_block_cols, int64_t nnz_blocks, int32_t block_size,
                int32_t feat_size, const void* d_X, void* d_Y, void* d_scratch, lf_stream_t stream) {
    LF_REQUIRE(block_size == 16 || block_size == 32 || block_size == 64, LF_ERR_UNSUPPORTED,
               "blocks of 16, 32 or 64 rows and columns are supported (got %d)", block_size);
    LF_REQUIRE(num_block_rows >= 0 && num_block_rows < (1ll << 26) && num_block_cols >= 1 &&
                   num_block_cols < (1ll << 26), LF_ERR_INVALID, "bad block shape");
    // no gather before the block index arrays have passed
    if (int rc = lf::csr_check(d_indptr, d_indices, nullptr, num_block_rows, num_block_cols, nnz_blocks, d_scratch, nullptr,
                               "lf_bsr_spmm", (hipStream_t)stream))
        return rc;
    return lf_bsr_spmm_trusted(d_indptr, d_indices, d_data, num_block_rows, num_block_cols, block_size, feat_size,
                               d_X, d_Y, stream);
}

}  // extern "C"
