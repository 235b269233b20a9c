// COO -> canonical CSR on the GPU: sort by (row, column), add up duplicate entries, build
// the row pointer.  This is what the reference's matrix container does on the host every
// time a CSR view is asked for (playground_pipline/format_matrix_market.py:74-76:
// scipy's coo.tocsr(), which sorts columns and sums duplicates); it is the step that feeds
// lf_bucket_stats / lf_hyb_build.  Sorting and the segmented sum are plain library
// primitives (rocPRIM radix sort and reduce-by-key on a 64-bit key row * cols + col); the
// kernels written here only pack / unpack keys and locate the row boundaries.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_reduce_by_key.hpp>
#include <rocprim/functional.hpp>

#include "lf_internal.h"

namespace {

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

__global__ void pack_keys_kernel(const int32_t* __restrict__ row, const int32_t* __restrict__ col,
                                 const float* __restrict__ val, long long nnz, long long cols,
                                 unsigned long long* __restrict__ keys, float* __restrict__ vals) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < nnz;
         i += (long long)gridDim.x * blockDim.x) {
        keys[i] = (unsigned long long)row[i] * (unsigned long long)cols + (unsigned long long)col[i];
        vals[i] = val ? val[i] : 1.0f;
    }
}

__global__ void unpack_cols_kernel(const unsigned long long* __restrict__ keys, const int* __restrict__ n_unique,
                                   long long cols, int32_t* __restrict__ indices) {
    const long long n = *n_unique;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (long long)gridDim.x * blockDim.x)
        indices[i] = (int32_t)(keys[i] % (unsigned long long)cols);
}

// indptr[r] = number of unique keys below r * cols (keys are sorted)
__global__ void row_pointer_kernel(const unsigned long long* __restrict__ keys, const int* __restrict__ n_unique,
                                   long long rows, long long cols, int32_t* __restrict__ indptr) {
    const long long r = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (r > rows) return;
    const unsigned long long bound = (unsigned long long)r * (unsigned long long)cols;
    long long lo = 0, hi = *n_unique;
    while (lo < hi) {
        const long long mid = (lo + hi) >> 1;
        if (keys[mid] < bound) lo = mid + 1; else hi = mid;
    }
    indptr[r] = (int32_t)lo;
}

struct IngestLayout {
    size_t keys_a, keys_b, vals_a, count, temp, temp_bytes, total;
};

hipError_t ingest_layout(long long nnz, int key_bits, IngestLayout* L) {
    size_t sort_bytes = 0, reduce_bytes = 0;
    unsigned long long* k = nullptr;
    float* v = nullptr;
    int* c = nullptr;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, sort_bytes, k, k, v, v, (size_t)nnz, 0u, (unsigned)key_bits);
    if (e != hipSuccess) return e;
    e = rocprim::reduce_by_key(nullptr, reduce_bytes, k, v, (size_t)nnz, k, v, c, rocprim::plus<float>(),
                               rocprim::equal_to<unsigned long long>());
    if (e != hipSuccess) return e;
    size_t off = 0;
    L->keys_a = off; off += align_up((size_t)nnz * 8, 256);
    L->keys_b = off; off += align_up((size_t)nnz * 8, 256);
    L->vals_a = off; off += align_up((size_t)nnz * 4, 256);
    L->count = off;  off += 256;
    L->temp = off;
    L->temp_bytes = std::max(sort_bytes, reduce_bytes);
    off += align_up(L->temp_bytes, 256);
    L->total = off;
    return hipSuccess;
}

int key_bits_for(long long rows, long long cols) {
    const unsigned long long top = (unsigned long long)rows * (unsigned long long)cols;
    int bits = 1;
    while (bits < 64 && (top >> bits) != 0) ++bits;
    return bits;
}

}  // namespace

extern "C" {

size_t lf_coo_to_csr_workspace_bytes(int64_t nnz, int64_t num_rows, int64_t num_cols) {
    if (nnz <= 0 || num_rows <= 0 || num_cols <= 0) return 256;
    IngestLayout L{};
    if (ingest_layout(nnz, key_bits_for(num_rows, num_cols), &L) != hipSuccess) return 0;
    return L.total;
}

int lf_coo_to_csr(const int32_t* d_coo_row, const int32_t* d_coo_col, const float* d_coo_val, int64_t nnz,
                  int64_t num_rows, int64_t num_cols, void* d_workspace, size_t workspace_bytes,
                  int32_t* d_indptr, int32_t* d_indices, float* d_values, int64_t* h_nnz_out,
                  lf_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && num_cols >= 1 && num_cols < (1ll << 31), LF_ERR_INVALID,
               "bad shape %lld x %lld", (long long)num_rows, (long long)num_cols);
    LF_REQUIRE(nnz >= 0 && nnz < (1ll << 31), LF_ERR_UNSUPPORTED, "nnz must be below 2^31");
    LF_REQUIRE(d_indptr && h_nnz_out, LF_ERR_INVALID, "null output");
    if (nnz == 0) {
        LF_HIP(hipMemsetAsync(d_indptr, 0, (size_t)(num_rows + 1) * 4, s));
        LF_HIP(hipStreamSynchronize(s));
        *h_nnz_out = 0;
        return LF_OK;
    }
    LF_REQUIRE(d_coo_row && d_coo_col && d_indices && d_values, LF_ERR_INVALID, "null argument");
    const int key_bits = key_bits_for(num_rows, num_cols);
    IngestLayout L{};
    LF_HIP(ingest_layout(nnz, key_bits, &L));
    LF_REQUIRE(d_workspace && workspace_bytes >= L.total, LF_ERR_WORKSPACE, "workspace has %zu bytes, %zu needed",
               workspace_bytes, L.total);
    char* ws = (char*)d_workspace;
    unsigned long long* keys_a = (unsigned long long*)(ws + L.keys_a);
    unsigned long long* keys_b = (unsigned long long*)(ws + L.keys_b);
    float* vals_a = (float*)(ws + L.vals_a);
    int* count = (int*)(ws + L.count);
    void* temp = ws + L.temp;
    size_t temp_bytes = L.temp_bytes;

    const int grid = (int)std::min<long long>((nnz + 255) / 256, 65535);
    pack_keys_kernel<<<grid, 256, 0, s>>>(d_coo_row, d_coo_col, d_coo_val, nnz, num_cols, keys_a, d_values);
    LF_HIP(hipGetLastError());
    // sorted keys -> keys_b, values in the same order -> vals_a
    LF_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys_a, keys_b, d_values, vals_a, (size_t)nnz, 0u,
                                     (unsigned)key_bits, s));
    // unique keys -> keys_a, summed values -> d_values, count
    temp_bytes = L.temp_bytes;
    LF_HIP(rocprim::reduce_by_key(temp, temp_bytes, keys_b, vals_a, (size_t)nnz, keys_a, d_values, count,
                                  rocprim::plus<float>(), rocprim::equal_to<unsigned long long>(), s));
    unpack_cols_kernel<<<grid, 256, 0, s>>>(keys_a, count, num_cols, d_indices);
    LF_HIP(hipGetLastError());
    row_pointer_kernel<<<(int)((num_rows + 1 + 255) / 256), 256, 0, s>>>(keys_a, count, num_rows, num_cols, d_indptr);
    LF_HIP(hipGetLastError());
    int h_count = 0;
    LF_HIP(hipMemcpyAsync(&h_count, count, 4, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    *h_nnz_out = h_count;
    return LF_OK;
}

}  // extern "C"
