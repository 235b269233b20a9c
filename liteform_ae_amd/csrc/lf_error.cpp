// Error state and status strings of the C ABI.
#include "lf_internal.h"

namespace lf {

std::string& last_error() {
    static thread_local std::string msg;
    return msg;
}

int fail(int status, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return status;
}

}  // namespace lf

extern "C" {

int lf_version(void) { return LF_VERSION; }

const char* lf_last_error(void) { return lf::last_error().c_str(); }

const char* lf_status_string(int status) {
    switch (status) {
        case LF_OK: return "ok";
        case LF_ERR_INVALID: return "invalid argument";
        case LF_ERR_TOO_SMALL: return "partition holds a single nonzero";
        case LF_ERR_HIP: return "HIP runtime error";
        case LF_ERR_CONFIG: return "bucket widths do not fit the matrix";
        case LF_ERR_UNSUPPORTED: return "unsupported size or type";
        case LF_ERR_WORKSPACE: return "workspace too small";
        default: return "unknown status";
    }
}

}  // extern "C"
