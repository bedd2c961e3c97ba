// Status reporting and per-device kernel set-up of libtmq_hip.
#include "common.h"

#include <map>
#include <mutex>
#include <utility>

namespace tmq {
static thread_local int g_last_hip_error = 0;

int note_hip_error(hipError_t e) {
    g_last_hip_error = (int)e;
    return TMQ_ERR_LAUNCH;
}

int allow_dynamic_lds(const void *kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return TMQ_OK;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return note_hip_error(e);
    static std::mutex guard;
    static std::map<std::pair<const void *, int>, size_t> granted;   // (kernel, device) -> largest size opted in to
    std::lock_guard<std::mutex> lock(guard);
    size_t &have = granted[std::make_pair(kernel, dev)];
    if (have >= bytes) return TMQ_OK;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return note_hip_error(e);
    have = bytes;
    return TMQ_OK;
}
}  // namespace tmq

extern "C" {

int tmq_version(void) { return 100; /* 0.1.0 */ }

int tmq_last_hip_error(void) { return tmq::g_last_hip_error; }

const char *tmq_status_string(int status) {
    switch (status) {
        case TMQ_OK: return "ok";
        case TMQ_ERR_INVALID_ARG: return "invalid argument (null pointer, bad size, misaligned or inconsistent shape)";
        case TMQ_ERR_UNSUPPORTED: return "unsupported dtype or shape";
        case TMQ_ERR_LAUNCH: return "HIP launch or runtime error (see tmq_last_hip_error)";
        case TMQ_ERR_TOO_LARGE: return "tensor too large for the launch geometry";
        case TMQ_ERR_BAD_DATA: return "malformed stream or illegal ternary code";
        default: return "unknown status";
    }
}

}  // extern "C"
