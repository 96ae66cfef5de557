// depthwise_conv1d ("TimeX"): causal depthwise convolution with a full-length (T-tap) kernel
// per channel, fp32, gfx950.
//
//   x[b,c,t]  = eps + sum_{u<=t} wr[t-u] k[b,c,u]            wr[d] = w[c, T-1-d]
//   gk[b,c,u] =       sum_{t>=u} wr[t-u] g[b,c,t]
//   gw[b,c,T-1-d] =   sum_{u}    g[b,c,u+d] k[b,c,u]         (per batch; the wrapper sums over b)
//
// conv / corr kernels: one workgroup per (channel, group of BB batch rows).  The reversed
// kernel row wr (with four leading zeros, so taps of negative lag read 0 and the diagonal block
// needs no mask) and the BB input rows sit in LDS; a thread owns 4 consecutive outputs for all
// BB rows and walks the lags 4 at a time: two 16-byte LDS reads give the 7 taps it needs, one
// broadcast 16-byte read per row gives the inputs, 16 FMAs per row follow.
// gw kernel: one workgroup per (b,c) row; a thread owns 4 consecutive lags d.
#include "common.h"

namespace rwkv {
namespace {

constexpr int BB = 8;

// MIRROR = false: out[t] = eps + sum_{u<=t} wr[t-u] in[u]      (forward)
// MIRROR = true : out[u] =       sum_{t>=u} wr[t-u] in[t]      (gk)
template <bool MIRROR>
__global__ __launch_bounds__(1024) void timex_conv(const float* __restrict__ w, const float* __restrict__ in,
                                                  float* __restrict__ out, float eps, int B, int C, int T) {
    extern __shared__ float lds[];
    float* wr = lds;                 // [T + 4], wr[4 + d] = w[c][T-1-d], wr[0..3] = 0
    float* rows = lds + T + 4;       // [BB][T]
    const int c = blockIdx.x, b0 = blockIdx.y * BB, tid = threadIdx.x;
    const int nthr = T >> 2;

    for (int i = tid; i < 4; i += nthr) wr[i] = 0.f;
    for (int d = tid; d < T; d += nthr) wr[4 + d] = w[static_cast<size_t>(c) * T + (T - 1 - d)];
#pragma unroll
    for (int r = 0; r < BB; ++r) {
        const int b = b0 + r;
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
        if (b < B) x = *reinterpret_cast<const float4*>(in + (static_cast<size_t>(b) * C + c) * T + 4 * tid);
        *reinterpret_cast<float4*>(rows + r * T + 4 * tid) = x;
    }
    __syncthreads();

    const int o0 = 4 * tid;          // first output index of this thread
    float acc[BB][4];
#pragma unroll
    for (int r = 0; r < BB; ++r)
#pragma unroll
        for (int a = 0; a < 4; ++a) acc[r][a] = MIRROR ? 0.f : eps;

    const int lo = MIRROR ? o0 : 0, hi = MIRROR ? T - 4 : o0;
    for (int s4 = lo; s4 <= hi; s4 += 4) {
        const int d0 = MIRROR ? s4 - o0 : o0 - s4;                   // >= 0, multiple of 4
        const float4 wl = *reinterpret_cast<const float4*>(wr + d0);       // lags d0-4 .. d0-1
        const float4 wh = *reinterpret_cast<const float4*>(wr + d0 + 4);   // lags d0   .. d0+3
        const float wv[8] = {wl.x, wl.y, wl.z, wl.w, wh.x, wh.y, wh.z, wh.w};
#pragma unroll
        for (int r = 0; r < BB; ++r) {
            const float4 x4 = *reinterpret_cast<const float4*>(rows + r * T + s4);
            const float xv[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    // forward: lag = (o0+a) - (s4+e) = d0 + a - e;  mirror: lag = (s4+e) - (o0+a) = d0 + e - a
                    acc[r][a] = fmaf(wv[4 + (MIRROR ? e - a : a - e)], xv[e], acc[r][a]);
        }
    }
#pragma unroll
    for (int r = 0; r < BB; ++r) {
        const int b = b0 + r;
        if (b < B)
            *reinterpret_cast<float4*>(out + (static_cast<size_t>(b) * C + c) * T + o0) =
                make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
    }
}

// gw[row][T-1-d] = sum_u g[row][u+d] k[row][u]
__global__ __launch_bounds__(1024) void timex_gw(const float* __restrict__ k, const float* __restrict__ g,
                                                float* __restrict__ gw, int T) {
    extern __shared__ float lds[];
    float* ks = lds;                 // [T]
    float* gs = lds + T;             // [T + 4], four trailing zeros
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    *reinterpret_cast<float4*>(ks + 4 * tid) = *reinterpret_cast<const float4*>(k + row * T + 4 * tid);
    *reinterpret_cast<float4*>(gs + 4 * tid) = *reinterpret_cast<const float4*>(g + row * T + 4 * tid);
    for (int i = tid; i < 4; i += (T >> 2)) gs[T + i] = 0.f;
    __syncthreads();

    const int d0 = 4 * tid;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int u4 = 0; u4 + d0 < T; u4 += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(ks + u4);
        const float4 g0 = *reinterpret_cast<const float4*>(gs + u4 + d0);
        const float4 g1 = *reinterpret_cast<const float4*>(gs + u4 + d0 + 4);
        const float kv[4] = {k4.x, k4.y, k4.z, k4.w};
        const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[a] = fmaf(gv[e + a], kv[e], acc[a]);   // g[u4+e + d0+a] k[u4+e]
    }
    // lags d0..d0+3 live at taps T-1-d0 .. T-4-d0
    *reinterpret_cast<float4*>(gw + row * T + (T - 4 - d0)) = make_float4(acc[3], acc[2], acc[1], acc[0]);
}

constexpr int T_MAX = 4096;

int check_tx(int B, int C, int T) {
    if (B <= 0 || C <= 0 || T <= 0) return RWKV_ERR_SHAPE;
    if (T % 4 != 0 || T > T_MAX) return RWKV_ERR_SHAPE;
    if ((B + BB - 1) / BB > 65535) return RWKV_ERR_SHAPE;
    return RWKV_OK;
}

template <typename K> int raise_lds_limit(K kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return RWKV_OK;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
    if (e != hipSuccess) { g_last_hip_error = static_cast<int>(e); return RWKV_ERR_LAUNCH; }
    return RWKV_OK;
}

}  // namespace
}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_timex_forward(void* stream, const float* w, const float* k, float* x, float eps, int B, int C, int T) {
    if (int e = check_tx(B, C, T)) return e;
    if (int e = check_ptrs({w, k, x})) return e;
    const size_t lds = (static_cast<size_t>(BB + 1) * T + 4) * sizeof(float);
    if (int e = raise_lds_limit(timex_conv<false>, lds)) return e;
    hipLaunchKernelGGL(timex_conv<false>, dim3(C, (B + BB - 1) / BB), dim3(T / 4), lds,
                       static_cast<hipStream_t>(stream), w, k, x, eps, B, C, T);
    return launch_status();
}

int rwkv_timex_backward(void* stream, const float* w, const float* k, const float* gwk, float* gw, float* gk,
                        int B, int C, int T) {
    if (int e = check_tx(B, C, T)) return e;
    if (int e = check_ptrs({w, k, gwk, gw, gk})) return e;
    if (static_cast<long long>(B) * C > 0x7fffffffLL) return RWKV_ERR_SHAPE;
    const size_t lds = (static_cast<size_t>(BB + 1) * T + 4) * sizeof(float);
    if (int e = raise_lds_limit(timex_conv<true>, lds)) return e;
    hipLaunchKernelGGL(timex_conv<true>, dim3(C, (B + BB - 1) / BB), dim3(T / 4), lds,
                       static_cast<hipStream_t>(stream), w, gwk, gk, 0.0f, B, C, T);
    hipLaunchKernelGGL(timex_gw, dim3(B * C), dim3(T / 4), (2 * static_cast<size_t>(T) + 4) * sizeof(float),
                       static_cast<hipStream_t>(stream), k, gwk, gw, T);
    return launch_status();
}

}  // extern "C"
