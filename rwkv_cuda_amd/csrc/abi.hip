// Status text and error bookkeeping for the C ABI.
#include "common.h"

namespace rwkv {
thread_local int g_last_hip_error = 0;
}

namespace rwkv {
namespace {
// Streams for measuring what the memory system delivers (bench.py prices the kernels against them): 16 bytes per lane,
// grid-stride, reads with the non-temporal hint.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(1024) void hbm_read_stream(const u32x4_t* __restrict__ a, size_t n, u32x4_t* sink) {
    u32x4_t acc = {0u, 0u, 0u, 0u};
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        acc ^= __builtin_nontemporal_load(a + i);
    if (acc[0] == 0x9e3779b9u && acc[1] == 0x7f4a7c15u && acc[2] == 1u) sink[0] = acc;      // keeps the loads alive
}
__global__ __launch_bounds__(1024) void hbm_write_stream(u32x4_t* __restrict__ a, size_t n) {
    const u32x4_t v = {1u, 2u, 3u, 4u};
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x) a[i] = v;
}
__global__ __launch_bounds__(1024) void hbm_copy_stream(const u32x4_t* __restrict__ a, u32x4_t* __restrict__ b, size_t n) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * blockDim.x)
        b[i] = __builtin_nontemporal_load(a + i);
}
}  // namespace
}  // namespace rwkv

extern "C" {

// mode 0: read `bytes` from src; 1: write `bytes` to dst; 2: copy src to dst.  A measuring aid, no counterpart in the reference.
int rwkv_hbm_probe(void* stream, int mode, const void* src, void* dst, size_t bytes) {
    using namespace rwkv;
    if (bytes % 16 != 0 || (mode != 1 && (src == nullptr || !aligned16(src))) || (mode != 0 && (dst == nullptr || !aligned16(dst)))) return RWKV_ERR_SHAPE;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t n = bytes / 16;
    const dim3 grid(32768), block(1024);
    if (mode == 0) {
        if (dst == nullptr) return RWKV_ERR_NULL;
        hipLaunchKernelGGL(hbm_read_stream, grid, block, 0, st, static_cast<const u32x4_t*>(src), n, static_cast<u32x4_t*>(dst));
    } else if (mode == 1) hipLaunchKernelGGL(hbm_write_stream, grid, block, 0, st, static_cast<u32x4_t*>(dst), n);
    else if (mode == 2) hipLaunchKernelGGL(hbm_copy_stream, grid, block, 0, st, static_cast<const u32x4_t*>(src), static_cast<u32x4_t*>(dst), n);
    else return RWKV_ERR_SHAPE;
    return launch_status();
}

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

int rwkv_abi_version(void) { return RWKV_ABI_VERSION; }

}  // extern "C"
