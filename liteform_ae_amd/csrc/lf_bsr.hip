// Block-sparse (BSR, 32 x 32 blocks) fp16 SpMM on the gfx950 matrix cores:
//     Y[mb*32][F] (fp16) = A_bsr (fp16 blocks) . X[nb*32][F] (fp16),  fp32 accumulation.
//
// Takes over the kernel that bench_bsrmm builds through SparseTIR/TVM with fp16 WMMA
// 16x16x16 fragments (playground_pipline/format_algos.py:1182-1643; block size 32 is what
// the driver passes, proc05.spmm.end-to-end.py:205).  This is the one place of the library
// where dense-block matrix-core work is the right shape; it is still HBM-bound (2 KiB of A
// and 32 rows of X per 32x32xF block product: ~26 flop/byte at F = 128), so the kernel is
// organised around coalesced loads, not around MFMA occupancy.
//
// One workgroup (4 wavefronts) per (block row, 128-feature tile); wavefront w owns features
// [32w, 32w+32) of the tile and one 32x32 fp32 accumulator tile (v_mfma_f32_32x32x8_f16,
// four K-steps per nonzero block).  The A block is read straight from global memory in the
// MFMA A layout (lane: row l%32, four consecutive k).  The X tile needs four consecutive k
// (= four different rows of X) per lane, so it is loaded row-wise with 16-byte accesses and
// transposed through LDS: stored as XT[feature][k], read back as one 8-byte access.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <algorithm>

#include "lf_internal.h"

namespace {

constexpr int kBs = 32;            // block size
constexpr int kFeatTile = 128;     // features per workgroup
constexpr int kWgBsr = 256;
constexpr int kKPad = 36;          // halves per XT row: 32 + 4 keeps 8-byte reads aligned and spreads banks

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(kWgBsr)
bsr_spmm_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices,
                const _Float16* __restrict__ data, const _Float16* __restrict__ X,
                _Float16* __restrict__ Y, int feat) {
    __shared__ __align__(16) _Float16 s_xt[2][kFeatTile * kKPad];

    const int brow = blockIdx.x;
    const int f0 = blockIdx.y * kFeatTile;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int li = lane & 31, kq = lane >> 5;

    // cooperative X-tile load: thread t reads row t/8 of the block, two 16-byte vectors
    const int xr = tid >> 3;                 // 0..31: row inside the block (= k)
    const int xv = tid & 7;                  // vector 0..7 -> features 8*xv and 64 + 8*xv
    const bool in0 = f0 + 8 * xv < feat, in1 = f0 + 64 + 8 * xv < feat;

    float16_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;

    const int jb = indptr[brow], je = indptr[brow + 1];
    uint4 x0 = make_uint4(0, 0, 0, 0), x1 = make_uint4(0, 0, 0, 0);
    auto load_x = [&](int j) {
        const _Float16* src = X + ((size_t)indices[j] * kBs + xr) * feat + f0 + 8 * xv;
        x0 = in0 ? *reinterpret_cast<const uint4*>(src) : make_uint4(0, 0, 0, 0);
        x1 = in1 ? *reinterpret_cast<const uint4*>(src + 64) : make_uint4(0, 0, 0, 0);
    };
    auto store_xt = [&](int buf) {
        _Float16* dst = s_xt[buf];
        const _Float16* h0 = reinterpret_cast<const _Float16*>(&x0);
        const _Float16* h1 = reinterpret_cast<const _Float16*>(&x1);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            dst[(8 * xv + i) * kKPad + xr] = h0[i];
            dst[(64 + 8 * xv + i) * kKPad + xr] = h1[i];
        }
    };

    if (jb < je) {
        load_x(jb);
        store_xt(0);
    }
    __syncthreads();
    for (int j = jb; j < je; ++j) {
        const int buf = (j - jb) & 1;
        if (j + 1 < je) load_x(j + 1);                       // next tile in flight during the MFMAs
        const _Float16* ablk = data + (size_t)j * kBs * kBs + li * kBs + 4 * kq;
        const _Float16* xt = s_xt[buf] + (32 * wave + li) * kKPad + 4 * kq;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const half4_t a = *reinterpret_cast<const half4_t*>(ablk + 8 * s);
            const half4_t b = *reinterpret_cast<const half4_t*>(xt + 8 * s);
            acc = __builtin_amdgcn_mfma_f32_32x32x8f16(a, b, acc, 0, 0, 0);
        }
        if (j + 1 < je) store_xt(buf ^ 1);
        __syncthreads();
    }

    // D layout of the 32x32 MFMA: lane holds column li, rows 8*(v/4) + 4*kq + v%4
    const int col = f0 + 32 * wave + li;
    if (col < feat) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * kq + (v & 3);
            Y[((size_t)brow * kBs + row) * feat + col] = (_Float16)acc[v];
        }
    }
}

}  // namespace

extern "C" {

int lf_bsr_spmm_trusted(const int32_t* d_indptr, const int32_t* d_indices, const void* d_data,
                        int64_t num_block_rows, int64_t num_block_cols, int32_t block_size,
                        int32_t feat_size, const void* d_X, void* d_Y, lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(block_size == kBs, LF_ERR_UNSUPPORTED, "only 32 x 32 blocks are supported (got %d)", block_size);
    LF_REQUIRE(num_block_rows >= 0 && num_block_rows < (1ll << 26) && num_block_cols >= 1 &&
                   num_block_cols < (1ll << 26), LF_ERR_INVALID, "bad block shape");
    LF_REQUIRE(feat_size >= 8 && feat_size % 8 == 0, LF_ERR_UNSUPPORTED,
               "feat_size must be a positive multiple of 8 (got %d)", feat_size);
    if (num_block_rows == 0) return LF_OK;
    LF_REQUIRE(d_indptr && d_X && d_Y, LF_ERR_INVALID, "null argument");
    LF_REQUIRE((uintptr_t)d_X % 16 == 0 && (uintptr_t)d_Y % 2 == 0 && (uintptr_t)d_data % 8 == 0, LF_ERR_INVALID,
               "X must be 16-byte aligned and the block data 8-byte aligned");
    const dim3 grid((unsigned)num_block_rows, (unsigned)((feat_size + kFeatTile - 1) / kFeatTile));
    bsr_spmm_kernel<<<grid, kWgBsr, 0, s>>>(d_indptr, d_indices, (const _Float16*)d_data, (const _Float16*)d_X,
                                            (_Float16*)d_Y, feat_size);
    LF_HIP(hipGetLastError());
    return LF_OK;
}

int lf_bsr_spmm(const int32_t* d_indptr, const int32_t* d_indices, const void* d_data,
                int64_t num_block_rows, int64_t num_block_cols, int64_t nnz_blocks, int32_t block_size,
                int32_t feat_size, const void* d_X, void* d_Y, void* d_scratch, lf_stream_t stream) {
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
