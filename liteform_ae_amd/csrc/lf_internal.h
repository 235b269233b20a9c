// Shared helpers for liblfhip.so: error reporting and small integer utilities.
#pragma once
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "liteform_hip.h"

namespace lf {

// Thread-local message behind lf_last_error().
std::string& last_error();

int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
inline int ilog2(int64_t x) { return 63 - __builtin_clzll((unsigned long long)x); }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace lf

#ifdef __HIPCC__
#include <hip/hip_runtime.h>
namespace lf {
// Structural check of caller-supplied CSR (or BSR block) index arrays on the GPU, behind
// lf_csr_check and in front of lf_csr_spmm / lf_bsr_spmm; `what` names the arrays in the
// error message.  Synchronises `s`.
int csr_check(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values, int64_t num_rows,
              int64_t num_cols, int64_t nnz, void* d_scratch, int32_t* h_flags, const char* what, hipStream_t s);
}  // namespace lf
#endif

#define LF_REQUIRE(cond, status, ...)                  \
    do {                                               \
        if (!(cond)) return lf::fail(status, __VA_ARGS__); \
    } while (0)

#define LF_HIP(call)                                                                     \
    do {                                                                                 \
        hipError_t _e = (call);                                                          \
        if (_e != hipSuccess)                                                            \
            return lf::fail(LF_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(_e), \
                            __FILE__, __LINE__);                                         \
    } while (0)
