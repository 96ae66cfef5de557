// Status text and error bookkeeping for the C ABI.
#include "common.h"

namespace rwkv {
thread_local int g_last_hip_error = 0;
}

extern "C" {

const char* rwkv_strerror(int status) {
    switch (status) {
        case RWKV_OK: return "ok";
        case RWKV_ERR_SHAPE: return "bad shape (dims must be positive, C == H*64, T a multiple of the chunk where required)";
        case RWKV_ERR_NULL: return "a required pointer is NULL";
        case RWKV_ERR_ALIGN: return "a pointer is not 16-byte aligned";
        case RWKV_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case RWKV_ERR_LAUNCH: return "HIP refused the kernel launch";
        default: return "unknown status";
    }
}

int rwkv_last_hip_error(void) { return rwkv::g_last_hip_error; }

int rwkv_abi_version(void) { return 3; }

}  // extern "C"
