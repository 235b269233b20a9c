// COO -> canonical CSR on the GPU: sort by (row, column), add up duplicate entries, build
// the row pointer.  This is what the reference's matrix container does on the host every
// time a CSR view is asked for (playground_pipline/format_matrix_market.py:74-76:
// scipy's coo.tocsr(), which sorts columns and sums duplicates); it is the step that feeds
// lf_bucket_stats / lf_hyb_build.  Sorting and the segmented sum are plain library
// primitives (rocPRIM radix sort and reduce-by-key on a 64-bit key row * cols + col); the
// kernels written here only pack / unpack keys and locate the row boundaries.
//
// Also here: the structural check of CSR arrays that come from a caller (lf_csr_check), which
// every entry point that gathers through caller-supplied CSR or BSR index arrays runs first,
// and which tells an already canonical CSR (the fast path: no sort) from one that has to go
// through the COO route.
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

// One pass over the row pointer and one over the column indices.  out[0] is raised for
// anything a gather must not meet: a row pointer that does not start at 0, decreases, or
// does not end at nnz, or a column outside [0, num_cols).  out[1] counts the positions i > 0
// with indices[i] <= indices[i - 1] ("descents"), out[2] the non-empty rows whose first
// entry is such a position: the columns of every row ascend strictly (sorted, no
// duplicates) exactly when the two counts are equal.  out[3] is raised when a value differs
// from 1 (values == nullptr: not looked at).
__global__ void __launch_bounds__(256)
csr_check_kernel(const int32_t* __restrict__ indptr, const int32_t* __restrict__ indices,
                 const float* __restrict__ values, long long rows, long long cols, long long nnz,
                 unsigned int* __restrict__ out) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    const long long t0 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    bool bad = false, not_one = false;
    unsigned int descents = 0, boundary = 0;
    for (long long r = t0; r < rows; r += stride) {
        const long long lo = indptr[r], hi = indptr[r + 1];
        bad |= lo < 0 || hi < lo || hi > nnz;
        if (r == 0) bad |= lo != 0;
        if (r == rows - 1) bad |= hi != nnz;
        if (hi > lo && lo > 0 && lo < nnz && indices[lo] <= indices[lo - 1]) ++boundary;
    }
    for (long long i = t0; i < nnz; i += stride) {
        const int c = indices[i];
        bad |= (unsigned long long)(unsigned int)c >= (unsigned long long)cols;
        if (i > 0 && c <= indices[i - 1]) ++descents;
        if (values) not_one |= values[i] != 1.0f;
    }
    for (int d = 32; d > 0; d >>= 1) {
        descents += __shfl_xor(descents, d);
        boundary += __shfl_xor(boundary, d);
    }
    const bool any_bad = __ballot(bad) != 0;
    const bool any_not_one = __ballot(not_one) != 0;
    if ((threadIdx.x & 63) == 0) {
        if (any_bad) out[0] = 1u;
        if (any_not_one) out[3] = 1u;
        if (descents) atomicAdd(&out[1], descents);
        if (boundary) atomicAdd(&out[2], boundary);
    }
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

namespace lf {

int csr_check(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values, int64_t num_rows,
              int64_t num_cols, int64_t nnz, void* d_scratch, int32_t* h_flags, const char* what, hipStream_t s) {
    LF_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && num_cols >= 1 && num_cols < (1ll << 31), LF_ERR_INVALID,
               "bad shape %lld x %lld", (long long)num_rows, (long long)num_cols);
    LF_REQUIRE(nnz >= 0 && nnz < (1ll << 31), LF_ERR_UNSUPPORTED, "nnz must be below 2^31");
    if (h_flags) *h_flags = LF_CSR_CANONICAL | (d_values ? LF_CSR_UNIT_VALUES : 0);
    if (num_rows == 0) {
        LF_REQUIRE(nnz == 0, LF_ERR_INVALID, "%s: a matrix without rows holds %lld entries", what, (long long)nnz);
        return LF_OK;
    }
    LF_REQUIRE(d_indptr && (nnz == 0 || d_indices), LF_ERR_INVALID, "%s: null index array", what);
    LF_REQUIRE(d_scratch && (uintptr_t)d_scratch % 4 == 0, LF_ERR_INVALID, "%s: the check needs 16 bytes of device scratch", what);
    unsigned int* out = (unsigned int*)d_scratch;
    LF_HIP(hipMemsetAsync(out, 0, 16, s));
    const long long units = std::max<long long>(num_rows, nnz);
    const int grid = (int)std::min<long long>((units + 255) / 256, 8192);
    csr_check_kernel<<<grid, 256, 0, s>>>(d_indptr, d_indices, d_values, num_rows, num_cols, nnz, out);
    LF_HIP(hipGetLastError());
    unsigned int h[4] = {0, 0, 0, 0};
    LF_HIP(hipMemcpyAsync(h, out, 16, hipMemcpyDeviceToHost, s));
    LF_HIP(hipStreamSynchronize(s));
    LF_REQUIRE(h[0] == 0, LF_ERR_INVALID,
               "%s: the row pointer is not a non-decreasing sequence from 0 to nnz = %lld, or an index lies outside [0, %lld)",
               what, (long long)nnz, (long long)num_cols);
    if (h_flags) *h_flags = (h[1] == h[2] ? LF_CSR_CANONICAL : 0) | (d_values && h[3] == 0 ? LF_CSR_UNIT_VALUES : 0);
    return LF_OK;
}

}  // namespace lf

extern "C" {

int lf_csr_check(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values, int64_t num_rows,
                 int64_t num_cols, int64_t nnz, void* d_scratch, int32_t* h_flags, lf_stream_t stream) {
    return lf::csr_check(d_indptr, d_indices, d_values, num_rows, num_cols, nnz, d_scratch, h_flags, "CSR arrays",
                         (hipStream_t)stream);
}

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
