// RWKV-4 wkv, fp32, gfx950.  One lane per (batch, channel); lanes of a wave are 64 consecutive
// channels so every step reads and writes 256 contiguous bytes per tensor.
//
//   y_t = (e^{o-no} p + e^{u+k_t-no} v_t) / (e^{o-no} q + e^{u+k_t-no}),  no = max(o, u+k_t)
//   (p,q,o) <- decay by w and add e^{k_t}(v_t, 1), renormalised to the new running maximum o.
// The backward is the two-sweep scheme of wkv/cuda/wkv_cuda_v2.cu:40-114; what the ascending
// sweep must hand to the descending one (y_t, z_t = 1/den_t, zexp_t) is parked in the gv and gk
// output buffers and in a caller-provided workspace instead of per-thread local arrays, so T is
// not limited.
#include <math.h>

#include "common.h"

namespace rwkv {
namespace {

constexpr int NT = 64;
constexpr float O_INIT = -65500.0f;

__global__ __launch_bounds__(NT) void wkv4_fwd(int BC, int T, int C, const float* __restrict__ w_,
                                              const float* __restrict__ u_, const float* __restrict__ k_,
                                              const float* __restrict__ v_, float* __restrict__ y_) {
    const int idx = blockIdx.x * NT + threadIdx.x;
    if (idx >= BC) return;
    const int b = idx / C, c = idx % C;
    const size_t off = static_cast<size_t>(b) * T * C + c;
    const float u = u_[c], w = w_[c];
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    float* __restrict__ y = y_ + off;
    float p = 0.f, q = 0.f, o = O_INIT;
#pragma unroll 4
    for (int t = 0; t < T; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii];
        float no = fmaxf(o, u + kt);
        float A = expf(o - no), Bq = expf(u + kt - no);
        y[ii] = (A * p + Bq * vt) / (A * q + Bq);
        no = fmaxf(w + o, kt);
        A = expf(w + o - no);
        Bq = expf(kt - no);
        p = A * p + Bq * vt;
        q = A * q + Bq;
        o = no;
    }
}

__global__ __launch_bounds__(NT) void wkv4_bwd(int BC, int T, int C, const float* __restrict__ w_,
                                              const float* __restrict__ u_, const float* __restrict__ k_,
                                              const float* __restrict__ v_, const float* __restrict__ gy_,
                                              float* __restrict__ gw_, float* __restrict__ gu_,
                                              float* __restrict__ gk_, float* __restrict__ gv_,
                                              float* __restrict__ ws_) {
    const int idx = blockIdx.x * NT + threadIdx.x;
    if (idx >= BC) return;
    const int b = idx / C, c = idx % C;
    const size_t off = static_cast<size_t>(b) * T * C + c;
    const float u = u_[c], w = w_[c];
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    const float* __restrict__ gy = gy_ + off;
    float* __restrict__ gk = gk_ + off;      // holds z_t until the descending sweep overwrites it
    float* __restrict__ gv = gv_ + off;      // holds y_t
    float* __restrict__ ze = ws_ + off;      // zexp_t

    float gw = 0.f, gu = 0.f, p = 0.f, q = 0.f, dpdw = 0.f, dqdw = 0.f, o = O_INIT;
#pragma unroll 4
    for (int t = 0; t < T; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii], gt = gy[ii];
        float no = fmaxf(o, kt + u);
        float A = expf(o - no), Bq = expf(kt + u - no);
        const float num = A * p + Bq * vt;
        const float iden = 1.0f / (A * q + Bq);
        const float y = num * iden;
        gv[ii] = y;
        gk[ii] = iden;
        ze[ii] = kt + u - no;
        gw += gt * (dpdw - dqdw * y) * iden * A;
        gu += gt * (vt - y) * Bq * iden;
        no = fmaxf(w + o, kt);
        A = expf(w + o - no);
        Bq = expf(kt - no);
        dpdw = A * (p + dpdw);
        dqdw = A * (q + dqdw);
        p = A * p + Bq * vt;
        q = A * q + Bq;
        o = no;
    }
    float gp = 0.f, gq = 0.f;
    o = O_INIT;
#pragma unroll 4
    for (int t = T - 1; t >= 0; --t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii], gt = gy[ii];
        const float y = gv[ii], z = gk[ii], zexp = ze[ii];
        float A = gt * z * expf(zexp);
        float Bq = expf(kt + o);
        gk[ii] = A * (vt - y) + Bq * (gp * vt + gq);
        gv[ii] = A + Bq * gp;
        const float no = fmaxf(w + o, zexp - kt - u);
        A = expf(w + o - no);
        Bq = gt * z * expf(zexp - kt - u - no);
        gp = A * gp + Bq;
        gq = A * gq - Bq * y;
        o = no;
    }
    // the caller's buffers are accumulated into, as the reference does (wkv_cuda_v2.cu:112-113)
    gw_[static_cast<size_t>(b) * C + c] += gw * w;
    gu_[static_cast<size_t>(b) * C + c] += gu;
}

int check4(int B, int T, int C) {
    if (B <= 0 || T <= 0 || C <= 0) return RWKV_ERR_SHAPE;
    if (static_cast<long long>(B) * C > 0x7fffffffLL) return RWKV_ERR_SHAPE;
    return RWKV_OK;
}

}  // namespace
}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_wkv4_forward(void* stream, int B, int T, int C, const float* w, const float* u, const float* k,
                      const float* v, float* y) {
    if (int e = check4(B, T, C)) return e;
    if (int e = check_ptrs({w, u, k, v, y})) return e;
    const int BC = B * C;
    hipLaunchKernelGGL(wkv4_fwd, dim3((BC + NT - 1) / NT), dim3(NT), 0, static_cast<hipStream_t>(stream),
                       BC, T, C, w, u, k, v, y);
    return launch_status();
}

size_t rwkv_wkv4_backward_workspace_bytes(int B, int T, int C) {
    if (check4(B, T, C) != RWKV_OK) return 0;
    return static_cast<size_t>(B) * T * C * sizeof(float);
}

int rwkv_wkv4_backward(void* stream, int B, int T, int C, const float* w, const float* u, const float* k,
                       const float* v, const float* gy, float* gw, float* gu, float* gk, float* gv,
                       void* workspace, size_t workspace_bytes) {
    if (int e = check4(B, T, C)) return e;
    if (int e = check_ptrs({w, u, k, v, gy, gw, gu, gk, gv})) return e;
    if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < rwkv_wkv4_backward_workspace_bytes(B, T, C))
        return RWKV_ERR_WORKSPACE;
    const int BC = B * C;
    hipLaunchKernelGGL(wkv4_bwd, dim3((BC + NT - 1) / NT), dim3(NT), 0, static_cast<hipStream_t>(stream),
                       BC, T, C, w, u, k, v, gy, gw, gu, gk, gv, static_cast<float*>(workspace));
    return launch_status();
}

}  // extern "C"
