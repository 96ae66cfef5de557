// Torch-side shim over the C ABI of librwkv_hip.so: the `forward` / `backward` functions that each *_op.cpp of
// BlinkDL/RWKV-CUDA exposes through PYBIND11_MODULE and TORCH_LIBRARY, with the reference's tensor signatures, so that a
// driver written against `ext.forward(...)` / `torch.ops.<lib>.forward(...)` runs unchanged.
//
//   TORCH_LIBRARY name        reference shim                                               pybind submodule
//   wkv                       wkv/cuda/wkv_op.cpp:6-21                                     wkv
//   timex                     depthwise_conv1d/cuda/timex_op.cpp:6-21                      timex
//   wkv5                      wkv5_bf16/cuda/wkv5_op.cpp:8-22 and wkv5/cuda/wkv5_op.cpp:6-20  wkv5   (dtype of r selects bf16 or fp32)
//   wkv5a                     wkv5a/cuda/wkv5a_op.cpp:9-25                                 wkv5a
//   wkv6                      wkv6/cuda/wkv6_op.cpp:8-22                                   wkv6
//   wkv6b                     wkv6_state/cuda/wkv6state_op.cpp:8-22                        wkv6state
//   rwkv7_clampw              rwkv7_fast_fused/cuda/rwkv7_clampw.cpp:12-29                 rwkv7_clampw
//   rwkv7_state_clampw        rwkv7_fast_fused/cuda/rwkv7_state_clampw.cpp:12-29           rwkv7_state_clampw
//   rwkv7_statepassing_clampw rwkv7_fast_fused/cuda/rwkv7_statepassing_clampw.cpp:12-29    rwkv7_statepassing_clampw
// (the reference builds the rwkv7 sources twice, with and without -D_FP32_; here the dtype of r selects the mode.)
//
// Differences from the reference shims: arguments are checked (device, dtype, contiguity, element counts) with
// TORCH_CHECK instead of being cast blindly; work is enqueued on the current HIP stream of the tensors' device instead of
// the legacy default stream; the scratch some backwards need is taken from torch's caching allocator here (the C ABI
// itself never allocates).  No arithmetic happens in this file.
#include <limits>
#include <initializer_list>
#include <utility>
#include <torch/extension.h>
// PyTorch on ROCm presents HIP devices under the device type "cuda"; these are its stream and guard for that arrangement
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "rwkv_hip.h"

namespace {

using torch::Tensor;

void* stream_of(const Tensor& t) { return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream()); }

void ok(int status, const char* what) {
    TORCH_CHECK(status == RWKV_OK, what, ": librwkv_hip status ", status, " (", rwkv_strerror(status), ")",
                status == RWKV_ERR_LAUNCH ? ", hipError " + std::to_string(rwkv_last_hip_error()) : std::string());
}

struct Checker {
    const Tensor& first;
    const char* op;
    void operator()(const Tensor& t, c10::ScalarType dt, int64_t numel, const char* name) const {
        TORCH_CHECK(t.is_cuda(), op, ": ", name, " must live on a HIP device (there is no CPU path)");
        TORCH_CHECK(t.device() == first.device(), op, ": ", name, " is on ", t.device(), ", expected ", first.device());
        TORCH_CHECK(t.scalar_type() == dt, op, ": ", name, " must be ", dt, ", got ", t.scalar_type());
        TORCH_CHECK(t.is_contiguous(), op, ": ", name, " must be contiguous");
        TORCH_CHECK(numel < 0 || t.numel() == numel, op, ": ", name, " has ", t.numel(), " elements, expected ", numel);
    }
};

// The C ABI takes its sizes as int: a value outside (0, INT_MAX] would be narrowed silently, and the workspace-size queries
// run before any tensor is checked against it.
void dims_ok(const char* op, std::initializer_list<std::pair<const char*, int64_t>> dims) {
    for (const auto& d : dims)
        TORCH_CHECK(d.second > 0 && d.second <= std::numeric_limits<int>::max(), op, ": ", d.first, " = ", d.second, " is outside 1 .. 2147483647");
}

template <typename T> T* ptr(const Tensor& t) { return static_cast<T*>(t.data_ptr()); }
rwkv_bf16* bp(const Tensor& t) { return static_cast<rwkv_bf16*>(t.data_ptr()); }
float* fp(const Tensor& t) { return static_cast<float*>(t.data_ptr()); }

Tensor scratch(const Tensor& like, size_t bytes) {
    return torch::empty({static_cast<int64_t>(bytes < 16 ? 16 : bytes)}, like.options().dtype(torch::kUInt8));
}

constexpr auto BF = torch::kBFloat16;
constexpr auto F32 = torch::kFloat32;

// --------------------------------------------------------------------------------------------- wkv (RWKV-4)
void wkv_forward(int64_t B, int64_t T, int64_t C, Tensor& w, Tensor& u, Tensor& k, Tensor& v, Tensor& y) {
    const Checker chk{k, "wkv.forward"};
    dims_ok("wkv.forward", {{"B", B}, {"T", T}, {"C", C}});
    chk(w, F32, C, "w"); chk(u, F32, C, "u"); chk(k, F32, B * T * C, "k"); chk(v, F32, B * T * C, "v"); chk(y, F32, B * T * C, "y");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(k.device());
    ok(rwkv_wkv4_forward(stream_of(k), B, T, C, fp(w), fp(u), fp(k), fp(v), fp(y)), "wkv.forward");
}
void wkv_backward(int64_t B, int64_t T, int64_t C, Tensor& w, Tensor& u, Tensor& k, Tensor& v, Tensor& gy, Tensor& gw,
                  Tensor& gu, Tensor& gk, Tensor& gv) {
    const Checker chk{k, "wkv.backward"};
    dims_ok("wkv.backward", {{"B", B}, {"T", T}, {"C", C}});
    chk(w, F32, C, "w"); chk(u, F32, C, "u"); chk(k, F32, B * T * C, "k"); chk(v, F32, B * T * C, "v"); chk(gy, F32, B * T * C, "gy");
    chk(gw, F32, B * C, "gw"); chk(gu, F32, B * C, "gu"); chk(gk, F32, B * T * C, "gk"); chk(gv, F32, B * T * C, "gv");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(k.device());
    const size_t n = rwkv_wkv4_backward_workspace_bytes(B, T, C);
    Tensor ws = scratch(k, n);
    ok(rwkv_wkv4_backward(stream_of(k), B, T, C, fp(w), fp(u), fp(k), fp(v), fp(gy), fp(gw), fp(gu), fp(gk), fp(gv), ws.data_ptr(), n),
       "wkv.backward");
}

// --------------------------------------------------------------------------------------------- timex (depthwise_conv1d)
void timex_forward(Tensor& w, const Tensor& k, Tensor& x, double eps, int64_t B, int64_t C, int64_t T) {
    const Checker chk{k, "timex.forward"};
    dims_ok("timex.forward", {{"B", B}, {"C", C}, {"T", T}});
    chk(w, F32, C * T, "w"); chk(k, F32, B * C * T, "k"); chk(x, F32, B * C * T, "x");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(k.device());
    ok(rwkv_timex_forward(stream_of(k), fp(w), fp(k), fp(x), static_cast<float>(eps), B, C, T), "timex.forward");
}
void timex_backward(Tensor& w, const Tensor& k, const Tensor& gwk, Tensor& gw, Tensor& gk, int64_t B, int64_t C, int64_t T) {
    const Checker chk{k, "timex.backward"};
    dims_ok("timex.backward", {{"B", B}, {"C", C}, {"T", T}});
    chk(w, F32, C * T, "w"); chk(k, F32, B * C * T, "k"); chk(gwk, F32, B * C * T, "gwk"); chk(gw, F32, B * C * T, "gw"); chk(gk, F32, B * C * T, "gk");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(k.device());
    ok(rwkv_timex_backward(stream_of(k), fp(w), fp(k), fp(gwk), fp(gw), fp(gk), B, C, T), "timex.backward");
}

// --------------------------------------------------------------------------------------------- wkv5 (bf16 or fp32 I/O)
void wkv5_forward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w, Tensor& u, Tensor& y) {
    const Checker chk{r, "wkv5.forward"};
    dims_ok("wkv5.forward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    const auto dt = r.scalar_type();
    TORCH_CHECK(dt == BF || dt == F32, "wkv5.forward: r must be bfloat16 or float32");
    chk(r, dt, B * T * C, "r"); chk(k, dt, B * T * C, "k"); chk(v, dt, B * T * C, "v"); chk(w, F32, C, "w"); chk(u, dt, C, "u"); chk(y, dt, B * T * C, "y");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) {
        // heads of 128 channels need scratch for the fp32 terms of their four heads of 64; every other size needs none
        const size_t n = rwkv_wkv5_forward_workspace_bytes(B, T, C, H);
        Tensor ws = scratch(r, n > 0 ? n : 16);
        ok(rwkv_wkv5_forward_ws(stream_of(r), B, T, C, H, bp(r), bp(k), bp(v), fp(w), bp(u), bp(y), ws.data_ptr(), n, 0u), "wkv5.forward");
    }
    else ok(rwkv_wkv5f32_forward(stream_of(r), B, T, C, H, fp(r), fp(k), fp(v), fp(w), fp(u), fp(y)), "wkv5.forward");
}
void wkv5_backward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w, Tensor& ww, Tensor& u,
                   Tensor& gy, Tensor& gr, Tensor& gk, Tensor& gv, Tensor& gw, Tensor& gu) {
    const Checker chk{r, "wkv5.backward"};
    dims_ok("wkv5.backward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    const auto dt = r.scalar_type();
    TORCH_CHECK(dt == BF || dt == F32, "wkv5.backward: r must be bfloat16 or float32");
    chk(r, dt, B * T * C, "r"); chk(k, dt, B * T * C, "k"); chk(v, dt, B * T * C, "v"); chk(w, F32, C, "w"); chk(ww, F32, C, "ww");
    chk(u, dt, C, "u"); chk(gy, dt, B * T * C, "gy"); chk(gr, dt, B * T * C, "gr"); chk(gk, dt, B * T * C, "gk"); chk(gv, dt, B * T * C, "gv");
    chk(gw, dt, B * C, "gw"); chk(gu, dt, B * C, "gu");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) {
        const size_t n = rwkv_wkv5_backward_workspace_bytes(B, T, C, H);
        TORCH_CHECK(n > 0, "wkv5.backward: bad shape (C must be a multiple of H, head size at most 128)");
        Tensor ws = scratch(r, n);
        ok(rwkv_wkv5_backward(stream_of(r), B, T, C, H, bp(r), bp(k), bp(v), fp(w), fp(ww), bp(u), bp(gy), bp(gr), bp(gk), bp(gv),
                              bp(gw), bp(gu), ws.data_ptr(), n), "wkv5.backward");
    } else {
        ok(rwkv_wkv5f32_backward(stream_of(r), B, T, C, H, fp(r), fp(k), fp(v), fp(w), fp(ww), fp(u), fp(gy), fp(gr), fp(gk), fp(gv),
                                 fp(gw), fp(gu)), "wkv5.backward");
    }
}

// --------------------------------------------------------------------------------------------- wkv5a (fp32)
void wkv5a_forward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w1, Tensor& u1, Tensor& w2,
                   Tensor& u2, Tensor& y) {
    const Checker chk{r, "wkv5a.forward"};
    dims_ok("wkv5a.forward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    chk(r, F32, B * T * C, "r"); chk(k, F32, B * T * C, "k"); chk(v, F32, B * T * C, "v"); chk(y, F32, B * T * C, "y");
    chk(w1, F32, C, "w1"); chk(u1, F32, C, "u1"); chk(w2, F32, C, "w2"); chk(u2, F32, C, "u2");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    ok(rwkv_wkv5a_forward(stream_of(r), B, T, C, H, fp(r), fp(k), fp(v), fp(w1), fp(u1), fp(w2), fp(u2), fp(y)), "wkv5a.forward");
}
void wkv5a_backward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w1, Tensor& ww1, Tensor& u1,
                    Tensor& w2, Tensor& ww2, Tensor& u2, Tensor& gy, Tensor& gr, Tensor& gk, Tensor& gv, Tensor& gw1, Tensor& gu1,
                    Tensor& gw2, Tensor& gu2) {
    const Checker chk{r, "wkv5a.backward"};
    dims_ok("wkv5a.backward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    chk(r, F32, B * T * C, "r"); chk(k, F32, B * T * C, "k"); chk(v, F32, B * T * C, "v"); chk(gy, F32, B * T * C, "gy");
    chk(gr, F32, B * T * C, "gr"); chk(gk, F32, B * T * C, "gk"); chk(gv, F32, B * T * C, "gv");
    for (const Tensor* t : {&w1, &ww1, &u1, &w2, &ww2, &u2}) chk(*t, F32, C, "a per-head parameter");
    for (const Tensor* t : {&gw1, &gu1, &gw2, &gu2}) chk(*t, F32, B * C, "a per-batch parameter gradient");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    ok(rwkv_wkv5a_backward(stream_of(r), B, T, C, H, fp(r), fp(k), fp(v), fp(w1), fp(ww1), fp(u1), fp(w2), fp(ww2), fp(u2), fp(gy),
                           fp(gr), fp(gk), fp(gv), fp(gw1), fp(gu1), fp(gw2), fp(gu2)), "wkv5a.backward");
}

// --------------------------------------------------------------------------------------------- wkv6 (fp32 ew)
void wkv6_forward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w, Tensor& u, Tensor& y) {
    const Checker chk{r, "wkv6.forward"};
    dims_ok("wkv6.forward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    chk(r, BF, B * T * C, "r"); chk(k, BF, B * T * C, "k"); chk(v, BF, B * T * C, "v"); chk(w, F32, B * T * C, "w"); chk(u, BF, C, "u");
    chk(y, BF, B * T * C, "y");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    ok(rwkv_wkv6_forward(stream_of(r), B, T, C, H, bp(r), bp(k), bp(v), fp(w), bp(u), bp(y)), "wkv6.forward");
}
void wkv6_backward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w, Tensor& u, Tensor& gy,
                   Tensor& gr, Tensor& gk, Tensor& gv, Tensor& gw, Tensor& gu) {
    const Checker chk{r, "wkv6.backward"};
    dims_ok("wkv6.backward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    chk(r, BF, B * T * C, "r"); chk(k, BF, B * T * C, "k"); chk(v, BF, B * T * C, "v"); chk(w, F32, B * T * C, "w"); chk(u, BF, C, "u");
    chk(gy, BF, B * T * C, "gy"); chk(gr, BF, B * T * C, "gr"); chk(gk, BF, B * T * C, "gk"); chk(gv, BF, B * T * C, "gv");
    chk(gw, BF, B * T * C, "gw"); chk(gu, BF, B * C, "gu");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    const size_t n = rwkv_wkv6_backward_workspace_bytes(B, T, C, H);
    TORCH_CHECK(n > 0, "wkv6.backward: bad shape (C must be a multiple of H, head size at most 128)");
    Tensor ws = scratch(r, n);
    ok(rwkv_wkv6_backward(stream_of(r), B, T, C, H, bp(r), bp(k), bp(v), fp(w), bp(u), bp(gy), bp(gr), bp(gk), bp(gv), bp(gw), bp(gu),
                          ws.data_ptr(), n), "wkv6.backward");
}

// --------------------------------------------------------------------------------------------- wkv6b (wkv6_state)
void wkv6b_forward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w, Tensor& u, Tensor& s, Tensor& y) {
    const Checker chk{r, "wkv6b.forward"};
    dims_ok("wkv6b.forward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    chk(r, BF, B * T * C, "r"); chk(k, BF, B * T * C, "k"); chk(v, BF, B * T * C, "v"); chk(w, BF, B * T * C, "w"); chk(u, BF, C, "u");
    chk(s, BF, B * C * (C / H), "s"); chk(y, BF, B * T * C, "y");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    ok(rwkv_wkv6state_forward(stream_of(r), B, T, C, H, bp(r), bp(k), bp(v), bp(w), bp(u), bp(s), bp(y)), "wkv6b.forward");
}
void wkv6b_backward(int64_t B, int64_t T, int64_t C, int64_t H, Tensor& r, Tensor& k, Tensor& v, Tensor& w, Tensor& u, Tensor& s,
                    Tensor& gy, Tensor& gr, Tensor& gk, Tensor& gv, Tensor& gw, Tensor& gu, Tensor& gs) {
    const Checker chk{r, "wkv6b.backward"};
    dims_ok("wkv6b.backward", {{"B", B}, {"T", T}, {"C", C}, {"H", H}});
    chk(r, BF, B * T * C, "r"); chk(k, BF, B * T * C, "k"); chk(v, BF, B * T * C, "v"); chk(w, BF, B * T * C, "w"); chk(u, BF, C, "u");
    chk(s, BF, B * C * (C / H), "s"); chk(gy, BF, B * T * C, "gy"); chk(gr, BF, B * T * C, "gr"); chk(gk, BF, B * T * C, "gk");
    chk(gv, BF, B * T * C, "gv"); chk(gw, BF, B * T * C, "gw"); chk(gu, BF, B * C, "gu"); chk(gs, BF, B * C * (C / H), "gs");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    const size_t n = rwkv_wkv6state_backward_workspace_bytes(B, T, C, H);
    TORCH_CHECK(n > 0, "wkv6b.backward: bad shape (C must be a multiple of H, head size at most 128)");
    Tensor ws = scratch(r, n);
    ok(rwkv_wkv6state_backward(stream_of(r), B, T, C, H, bp(r), bp(k), bp(v), bp(w), bp(u), bp(s), bp(gy), bp(gr), bp(gk), bp(gv),
                               bp(gw), bp(gu), bp(gs), ws.data_ptr(), n), "wkv6b.backward");
}

// --------------------------------------------------------------------------------------------- rwkv7 clamp-w, three flavours
struct Dims7 { int B, T, H; int64_t btc, state, ckpt; };
Dims7 dims7(const Tensor& r, const char* op) {
    TORCH_CHECK(r.dim() == 4 && r.size(3) == 64, op, ": r must be [B,T,H,64]");
    dims_ok(op, {{"B", r.size(0)}, {"T", r.size(1)}, {"H", r.size(2)}});
    Dims7 d;
    d.B = static_cast<int>(r.size(0)); d.T = static_cast<int>(r.size(1)); d.H = static_cast<int>(r.size(2));
    d.btc = r.numel(); d.state = static_cast<int64_t>(d.B) * d.H * 64 * 64; d.ckpt = d.state * (d.T / RWKV7_CHUNK_LEN);
    return d;
}
c10::ScalarType mode7(const Tensor& r, const char* op) {
    const auto dt = r.scalar_type();
    TORCH_CHECK(dt == BF || dt == F32, op, ": r must be bfloat16 (default build) or float32 (the -D_FP32_ build)");
    return dt;
}

void r7sp_forward(Tensor& s0, Tensor& r, Tensor& w, Tensor& k, Tensor& v, Tensor& a, Tensor& b, Tensor& y, Tensor& sT, Tensor& s, Tensor& sa) {
    const char* op = "rwkv7_statepassing_clampw.forward";
    const Checker chk{r, op};
    const auto dt = mode7(r, op);
    const Dims7 d = dims7(r, op);
    for (const Tensor* t : {&r, &w, &k, &v, &a, &b, &y}) chk(*t, dt, d.btc, "r/w/k/v/a/b/y");
    chk(s0, F32, d.state, "s0"); chk(sT, F32, d.state, "sT"); chk(s, F32, d.ckpt, "s"); chk(sa, F32, d.btc, "sa");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) ok(rwkv7_statepassing_forward(stream_of(r), d.B, d.T, d.H, fp(s0), bp(r), bp(w), bp(k), bp(v), bp(a), bp(b), bp(y), fp(sT), fp(s), fp(sa)), op);
    else ok(rwkv7_statepassing_forward_f32(stream_of(r), d.B, d.T, d.H, fp(s0), fp(r), fp(w), fp(k), fp(v), fp(a), fp(b), fp(y), fp(sT), fp(s), fp(sa)), op);
}
void r7sp_backward(Tensor& r, Tensor& w, Tensor& k, Tensor& v, Tensor& a, Tensor& b, Tensor& dy, Tensor& dsT, Tensor& s, Tensor& sa,
                   Tensor& ds0, Tensor& dr, Tensor& dw, Tensor& dk, Tensor& dv, Tensor& da, Tensor& db) {
    const char* op = "rwkv7_statepassing_clampw.backward";
    const Checker chk{r, op};
    const auto dt = mode7(r, op);
    const Dims7 d = dims7(r, op);
    for (const Tensor* t : {&r, &w, &k, &v, &a, &b, &dy, &dr, &dw, &dk, &dv, &da, &db}) chk(*t, dt, d.btc, "r/w/k/v/a/b/dy/dr/dw/dk/dv/da/db");
    chk(dsT, F32, d.state, "dsT"); chk(ds0, F32, d.state, "ds0"); chk(s, F32, d.ckpt, "s"); chk(sa, F32, d.btc, "sa");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) ok(rwkv7_statepassing_backward(stream_of(r), d.B, d.T, d.H, bp(r), bp(w), bp(k), bp(v), bp(a), bp(b), bp(dy), fp(dsT), fp(s), fp(sa),
                                                 fp(ds0), bp(dr), bp(dw), bp(dk), bp(dv), bp(da), bp(db)), op);
    else ok(rwkv7_statepassing_backward_f32(stream_of(r), d.B, d.T, d.H, fp(r), fp(w), fp(k), fp(v), fp(a), fp(b), fp(dy), fp(dsT), fp(s), fp(sa),
                                            fp(ds0), fp(dr), fp(dw), fp(dk), fp(dv), fp(da), fp(db)), op);
}

void r7s_forward(Tensor& s0, Tensor& r, Tensor& w, Tensor& k, Tensor& v, Tensor& a, Tensor& b, Tensor& y, Tensor& s, Tensor& sa) {
    const char* op = "rwkv7_state_clampw.forward";
    const Checker chk{r, op};
    const auto dt = mode7(r, op);
    const Dims7 d = dims7(r, op);
    for (const Tensor* t : {&r, &w, &k, &v, &a, &b, &y}) chk(*t, dt, d.btc, "r/w/k/v/a/b/y");
    chk(s0, F32, d.state, "s0"); chk(s, F32, d.ckpt, "s"); chk(sa, F32, d.btc, "sa");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) ok(rwkv7_state_forward(stream_of(r), d.B, d.T, d.H, fp(s0), bp(r), bp(w), bp(k), bp(v), bp(a), bp(b), bp(y), fp(s), fp(sa)), op);
    else ok(rwkv7_state_forward_f32(stream_of(r), d.B, d.T, d.H, fp(s0), fp(r), fp(w), fp(k), fp(v), fp(a), fp(b), fp(y), fp(s), fp(sa)), op);
}
void r7s_backward(Tensor& r, Tensor& w, Tensor& k, Tensor& v, Tensor& a, Tensor& b, Tensor& dy, Tensor& s, Tensor& sa, Tensor& ds0,
                  Tensor& dr, Tensor& dw, Tensor& dk, Tensor& dv, Tensor& da, Tensor& db) {
    const char* op = "rwkv7_state_clampw.backward";
    const Checker chk{r, op};
    const auto dt = mode7(r, op);
    const Dims7 d = dims7(r, op);
    for (const Tensor* t : {&r, &w, &k, &v, &a, &b, &dy, &dr, &dw, &dk, &dv, &da, &db}) chk(*t, dt, d.btc, "r/w/k/v/a/b/dy/dr/dw/dk/dv/da/db");
    chk(ds0, F32, d.state, "ds0"); chk(s, F32, d.ckpt, "s"); chk(sa, F32, d.btc, "sa");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) ok(rwkv7_state_backward(stream_of(r), d.B, d.T, d.H, bp(r), bp(w), bp(k), bp(v), bp(a), bp(b), bp(dy), fp(s), fp(sa), fp(ds0),
                                          bp(dr), bp(dw), bp(dk), bp(dv), bp(da), bp(db)), op);
    else ok(rwkv7_state_backward_f32(stream_of(r), d.B, d.T, d.H, fp(r), fp(w), fp(k), fp(v), fp(a), fp(b), fp(dy), fp(s), fp(sa), fp(ds0),
                                     fp(dr), fp(dw), fp(dk), fp(dv), fp(da), fp(db)), op);
}

void r7_forward(Tensor& r, Tensor& w, Tensor& k, Tensor& v, Tensor& a, Tensor& b, Tensor& y, Tensor& s, Tensor& sa) {
    const char* op = "rwkv7_clampw.forward";
    const Checker chk{r, op};
    const auto dt = mode7(r, op);
    const Dims7 d = dims7(r, op);
    for (const Tensor* t : {&r, &w, &k, &v, &a, &b, &y}) chk(*t, dt, d.btc, "r/w/k/v/a/b/y");
    chk(s, F32, d.ckpt, "s"); chk(sa, F32, d.btc, "sa");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) ok(rwkv7_forward(stream_of(r), d.B, d.T, d.H, bp(r), bp(w), bp(k), bp(v), bp(a), bp(b), bp(y), fp(s), fp(sa)), op);
    else ok(rwkv7_forward_f32(stream_of(r), d.B, d.T, d.H, fp(r), fp(w), fp(k), fp(v), fp(a), fp(b), fp(y), fp(s), fp(sa)), op);
}
void r7_backward(Tensor& r, Tensor& w, Tensor& k, Tensor& v, Tensor& a, Tensor& b, Tensor& dy, Tensor& s, Tensor& sa, Tensor& dr,
                 Tensor& dw, Tensor& dk, Tensor& dv, Tensor& da, Tensor& db) {
    const char* op = "rwkv7_clampw.backward";
    const Checker chk{r, op};
    const auto dt = mode7(r, op);
    const Dims7 d = dims7(r, op);
    for (const Tensor* t : {&r, &w, &k, &v, &a, &b, &dy, &dr, &dw, &dk, &dv, &da, &db}) chk(*t, dt, d.btc, "r/w/k/v/a/b/dy/dr/dw/dk/dv/da/db");
    chk(s, F32, d.ckpt, "s"); chk(sa, F32, d.btc, "sa");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(r.device());
    if (dt == BF) ok(rwkv7_backward(stream_of(r), d.B, d.T, d.H, bp(r), bp(w), bp(k), bp(v), bp(a), bp(b), bp(dy), fp(s), fp(sa),
                                    bp(dr), bp(dw), bp(dk), bp(dv), bp(da), bp(db)), op);
    else ok(rwkv7_backward_f32(stream_of(r), d.B, d.T, d.H, fp(r), fp(w), fp(k), fp(v), fp(a), fp(b), fp(dy), fp(s), fp(sa),
                               fp(dr), fp(dw), fp(dk), fp(dv), fp(da), fp(db)), op);
}

}  // namespace

// One Python extension module with a submodule per reference extension: `ext.wkv6state.forward(...)` is what
// `wkv6state_cuda.forward(...)` is in wkv6_state/run.py:77,103.
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    // the ABI this shim was compiled against; binding.load() compares it with the library's
    m.attr("abi_version") = RWKV_ABI_VERSION;
    auto sub = [&](const char* name, auto fwd, auto bwd) {
        auto s = m.def_submodule(name);
        s.def("forward", fwd);
        s.def("backward", bwd);
    };
    sub("wkv", &wkv_forward, &wkv_backward);
    sub("timex", &timex_forward, &timex_backward);
    sub("wkv5", &wkv5_forward, &wkv5_backward);
    sub("wkv5a", &wkv5a_forward, &wkv5a_backward);
    sub("wkv6", &wkv6_forward, &wkv6_backward);
    sub("wkv6state", &wkv6b_forward, &wkv6b_backward);
    sub("rwkv7_clampw", &r7_forward, &r7_backward);
    sub("rwkv7_state_clampw", &r7s_forward, &r7s_backward);
    sub("rwkv7_statepassing_clampw", &r7sp_forward, &r7sp_backward);
}

TORCH_LIBRARY(wkv, m) { m.def("forward", wkv_forward); m.def("backward", wkv_backward); }
TORCH_LIBRARY(timex, m) { m.def("forward", timex_forward); m.def("backward", timex_backward); }
TORCH_LIBRARY(wkv5, m) { m.def("forward", wkv5_forward); m.def("backward", wkv5_backward); }
TORCH_LIBRARY(wkv5a, m) { m.def("forward", wkv5a_forward); m.def("backward", wkv5a_backward); }
TORCH_LIBRARY(wkv6, m) { m.def("forward", wkv6_forward); m.def("backward", wkv6_backward); }
TORCH_LIBRARY(wkv6b, m) { m.def("forward", wkv6b_forward); m.def("backward", wkv6b_backward); }
TORCH_LIBRARY(rwkv7_clampw, m) { m.def("forward", r7_forward); m.def("backward", r7_backward); }
TORCH_LIBRARY(rwkv7_state_clampw, m) { m.def("forward", r7s_forward); m.def("backward", r7s_backward); }
TORCH_LIBRARY(rwkv7_statepassing_clampw, m) { m.def("forward", r7sp_forward); m.def("backward", r7sp_backward); }
