// RWKV-4 wkv, fp32, gfx950.
//
//   y_t = (e^{o-no} p + e^{u+k_t-no} v_t) / (e^{o-no} q + e^{u+k_t-no}),  no = max(o, u+k_t)
//   (p,q,o) <- decay by w and add e^{k_t}(v_t, 1), renormalised to the new running maximum o.
// The backward is the two-sweep scheme of wkv/cuda/wkv_cuda_v2.cu:40-114; what the ascending
// sweep must hand to the descending one (y_t, z_t = 1/den_t, zexp_t) is parked in the gv and gk
// output buffers and in a caller-provided workspace instead of per-thread local arrays, so T is
// not limited.
// Two forms of each kernel: the time-parallel one used by the entry points (segments of the time axis
// side by side, joined by a scan of their states) and the plain one lane per (batch, channel) form,
// whose lanes of a wave are 64 consecutive channels (256 contiguous bytes per tensor and step).
#include <math.h>

#include <atomic>

#include "common.h"

namespace rwkv {
namespace {

constexpr int NT = 64;
constexpr float O_INIT = -65500.0f;

// e^x in six instructions, good to about 1.5 ulp over the whole range (underflow gives 0; the arguments here are finite
// and their results never overflow; the reference builds its kernel with --use_fast_math, wkv/run.py:87): 2^(x log2 e) by the hardware's own exp2, plus the first-order correction for what
// the rounded product and the rounded constant lost.
DEVINL float exp32(float x) {
    constexpr float L2E_HI = 1.44269502e+00f, L2E_LO = 1.92596299e-08f, LN2 = 0.693147182f;
    const float t = x * L2E_HI;
    const float lo = fmaf(x, L2E_LO, fmaf(x, L2E_HI, -t));
    const float r = __builtin_amdgcn_exp2f(t);
    return fmaf(r, lo * LN2, r);
}

// 1 / d for the denominators here, which lie between 1 and T (the newest or the largest term of the sum has weight 1):
// the hardware reciprocal and one Newton step, three instructions instead of the ten of a division
DEVINL float recip(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return fmaf(fmaf(-d, r, 1.0f), r, r);
}

// e^{a - max(a,b)} and e^{b - max(a,b)}: one of the two is e^0, so one exponential serves both
struct ExpPair { float no, ea, eb; };
DEVINL ExpPair exp_pair(float a, float b) {
    const float e = exp32(-fabsf(a - b));
    const bool first = a >= b;
    return {fmaxf(a, b), first ? 1.0f : e, first ? e : 1.0f};
}

template <bool RAW>
__global__ __launch_bounds__(NT) void wkv4_fwd(int BC, int T, int C, const float* __restrict__ w_,
                                              const float* __restrict__ u_, const float* __restrict__ k_,
                                              const float* __restrict__ v_, float* __restrict__ y_) {
    const int idx = blockIdx.x * NT + threadIdx.x;
    if (idx >= BC) return;
    const int b = idx / C, c = idx % C;
    const size_t off = static_cast<size_t>(b) * T * C + c;
    const float u = u_[c], w = RAW ? -expf(w_[c]) : w_[c];           // RAW: the wrapper's w = -exp(w_raw) done here
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    float* __restrict__ y = y_ + off;
    float p = 0.f, q = 0.f, o = O_INIT;
#pragma unroll 4
    for (int t = 0; t < T; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii];
        ExpPair e = exp_pair(o, u + kt);
        float no = e.no, A = e.ea, Bq = e.eb;
        y[ii] = (A * p + Bq * vt) * recip(A * q + Bq);
        e = exp_pair(w + o, kt);
        no = e.no;
        A = e.ea;
        Bq = e.eb;
        p = A * p + Bq * vt;
        q = A * q + Bq;
        o = no;
    }
}

// ---------------------------------------------------------------------------------------------------- time-parallel form
// B*C scans of T dependent steps leave most of the chip idle (3072 lanes at B4 C768), so the time axis is cut into NSEG
// segments that run side by side: a workgroup takes CH channels of one batch row, thread (channel, segment).
//   1. every segment scans its own steps from the empty state: (p, q, o) of the segment alone;
//   2. a Kogge-Stone scan over the segments combines them: a state that is n steps older enters with its exponent
//      lowered by n w (the decay is the same at every step), so after log2(NSEG) rounds segment s knows the state in
//      front of its first step;
//   3. every segment repeats its steps from that state and writes the outputs.
// The formulas of a step are those of the sequential kernel; only the order in which partial sums meet differs.
constexpr int CH = 16, NSEG = 64, NTS = CH * NSEG;
struct State3 { float p, q, o; };

// a: the older state, exponent already lowered by the decay over the steps of b
DEVINL State3 combine(const State3 a, const State3 b) {
    const ExpPair e = exp_pair(a.o, b.o);
    const float no = e.no, ea = e.ea, eb = e.eb;
    return {ea * a.p + eb * b.p, ea * a.q + eb * b.q, no};
}

template <bool RAW>
__global__ __launch_bounds__(NTS) void wkv4_fwd_seg(int T, int C, int S, const float* __restrict__ w_,
                                                   const float* __restrict__ u_, const float* __restrict__ k_,
                                                   const float* __restrict__ v_, float* __restrict__ y_) {
    __shared__ State3 X[2][NSEG][CH];
    const int cl = threadIdx.x % CH, s = threadIdx.x / CH;
    const int c = blockIdx.x * CH + cl, b = blockIdx.y;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const size_t off = static_cast<size_t>(b) * T * C + cc;
    const float u = u_[cc], w = RAW ? -expf(w_[cc]) : w_[cc];        // RAW: the wrapper's w = -exp(w_raw) done here
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    float* __restrict__ y = y_ + off;
    const int t0 = min(s * S, T), t1 = min(t0 + S, T);

    State3 x = {0.f, 0.f, O_INIT};
    for (int t = t0; t < t1; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii];
        const ExpPair e = exp_pair(w + x.o, kt);
        const float no = e.no, A = e.ea, Bq = e.eb;
        x.p = A * x.p + Bq * vt;
        x.q = A * x.q + Bq;
        x.o = no;
    }
    // Inclusive scan.  Every span is taken as full segments of S steps: only the last live segment can be shorter, and
    // the prefixes that contain it are needed by nobody.
    X[0][s][cl] = x;
    __syncthreads();
    int cur = 0;
#pragma unroll
    for (int d = 1; d < NSEG; d *= 2) {
        State3 mine = X[cur][s][cl];
        if (s >= d) {
            State3 older = X[cur][s - d][cl];
            older.o += static_cast<float>(d * S) * w;
            mine = combine(older, mine);
        }
        X[cur ^ 1][s][cl] = mine;
        cur ^= 1;
        __syncthreads();
    }
    x = State3{0.f, 0.f, O_INIT};
    if (s > 0) x = X[cur][s - 1][cl];

    for (int t = t0; t < t1; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii];
        ExpPair e = exp_pair(x.o, u + kt);
        float no = e.no, A = e.ea, Bq = e.eb;
        if (live) y[ii] = (A * x.p + Bq * vt) * recip(A * x.q + Bq);
        e = exp_pair(w + x.o, kt);
        no = e.no;
        A = e.ea;
        Bq = e.eb;
        x.p = A * x.p + Bq * vt;
        x.q = A * x.q + Bq;
        x.o = no;
    }
}

template <bool RAW>
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
    const float u = u_[c], w = RAW ? -expf(w_[c]) : w_[c];           // RAW: the wrapper's w = -exp(w_raw) done here
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
        ExpPair e = exp_pair(o, kt + u);
        float no = e.no, A = e.ea, Bq = e.eb;
        const float num = A * p + Bq * vt;
        const float iden = recip(A * q + Bq);
        const float y = num * iden;
        gv[ii] = y;
        gk[ii] = iden;
        ze[ii] = kt + u - no;
        gw += gt * (dpdw - dqdw * y) * iden * A;
        gu += gt * (vt - y) * Bq * iden;
        e = exp_pair(w + o, kt);
        no = e.no;
        A = e.ea;
        Bq = e.eb;
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
        float A = gt * z * exp32(zexp);
        float Bq = exp32(kt + o);
        gk[ii] = A * (vt - y) + Bq * (gp * vt + gq);
        gv[ii] = A + Bq * gp;
        const ExpPair e2 = exp_pair(w + o, zexp - kt - u);
        const float no = e2.no;
        A = e2.ea;
        Bq = gt * z * e2.eb;
        gp = A * gp + Bq;
        gq = A * gq - Bq * y;
        o = no;
    }
    // the caller's buffers are accumulated into, as the reference does (wkv_cuda_v2.cu:112-113)
    if constexpr (RAW) {                            // per-batch partials in the library's own scratch: plain stores
        gw_[static_cast<size_t>(b) * C + c] = gw * w;
        gu_[static_cast<size_t>(b) * C + c] = gu;
    } else {
        gw_[static_cast<size_t>(b) * C + c] += gw * w;
        gu_[static_cast<size_t>(b) * C + c] += gu;
    }
}

// Backward in the same time-parallel form.  The ascending sweep also carries dp/dw and dq/dw; a state that is n steps
// older enters with (dp, dq) <- (n p + dp, n q + dq) besides the lowered exponent, since P_{t+n} = e^{n w} P_t + ...
// gives dP_{t+n}/dw = e^{n w} (n P_t + dP_t/dw) + ...  The descending sweep is a scan of the same kind run from the last
// segment to the first (only the last live segment can be shorter than S, and there it is always the older operand).
struct State5 { float p, q, dp, dq, o; };

DEVINL State5 combine(const State5 a, const State5 b) {
    const ExpPair e = exp_pair(a.o, b.o);
    const float no = e.no, ea = e.ea, eb = e.eb;
    return {ea * a.p + eb * b.p, ea * a.q + eb * b.q, ea * a.dp + eb * b.dp, ea * a.dq + eb * b.dq, no};
}

template <bool RAW>
__global__ __launch_bounds__(NTS) void wkv4_bwd_seg(int T, int C, int S, const float* __restrict__ w_,
                                                   const float* __restrict__ u_, const float* __restrict__ k_,
                                                   const float* __restrict__ v_, const float* __restrict__ gy_,
                                                   float* __restrict__ gw_, float* __restrict__ gu_,
                                                   float* __restrict__ gk_, float* __restrict__ gv_,
                                                   float* __restrict__ ws_) {
    __shared__ State5 X[2][NSEG][CH];
    const int cl = threadIdx.x % CH, s = threadIdx.x / CH;
    const int c = blockIdx.x * CH + cl, b = blockIdx.y;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const size_t off = static_cast<size_t>(b) * T * C + cc;
    const float u = u_[cc], w = RAW ? -expf(w_[cc]) : w_[cc];        // RAW: the wrapper's w = -exp(w_raw) done here
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    const float* __restrict__ gy = gy_ + off;
    float* __restrict__ gk = gk_ + off;      // holds z_t until the descending sweep overwrites it
    float* __restrict__ gv = gv_ + off;      // holds y_t
    float* __restrict__ ze = ws_ + off;      // zexp_t
    // lanes past C have no steps: they only keep the barriers company
    const int t0 = live ? min(s * S, T) : T, t1 = min(t0 + S, T);
    const float span = static_cast<float>(S);

    // ---- ascending: the segment alone
    State5 x = {0.f, 0.f, 0.f, 0.f, O_INIT};
    for (int t = t0; t < t1; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii];
        const ExpPair e = exp_pair(w + x.o, kt);
        const float no = e.no, A = e.ea, Bq = e.eb;
        x.dp = A * (x.p + x.dp);
        x.dq = A * (x.q + x.dq);
        x.p = A * x.p + Bq * vt;
        x.q = A * x.q + Bq;
        x.o = no;
    }
    X[0][s][cl] = x;
    __syncthreads();
    int cur = 0;
#pragma unroll
    for (int d = 1; d < NSEG; d *= 2) {
        State5 mine = X[cur][s][cl];
        if (s >= d) {
            State5 older = X[cur][s - d][cl];
            const float n = static_cast<float>(d) * span;
            older.dp += n * older.p;
            older.dq += n * older.q;
            older.o += n * w;
            mine = combine(older, mine);
        }
        X[cur ^ 1][s][cl] = mine;
        cur ^= 1;
        __syncthreads();
    }
    x = State5{0.f, 0.f, 0.f, 0.f, O_INIT};
    if (s > 0) x = X[cur][s - 1][cl];
    __syncthreads();                               // X is reused below

    // ---- ascending, from the true state: y, 1/den and zexp are parked for the descending sweep
    float gw = 0.f, gu = 0.f;
    for (int t = t0; t < t1; ++t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii], gt = gy[ii];
        ExpPair e = exp_pair(x.o, kt + u);
        float no = e.no, A = e.ea, Bq = e.eb;
        const float num = A * x.p + Bq * vt;
        const float iden = recip(A * x.q + Bq);
        const float y = num * iden;
        gv[ii] = y;
        gk[ii] = iden;
        ze[ii] = kt + u - no;
        gw += gt * (x.dp - x.dq * y) * iden * A;
        gu += gt * (vt - y) * Bq * iden;
        e = exp_pair(w + x.o, kt);
        no = e.no;
        A = e.ea;
        Bq = e.eb;
        x.dp = A * (x.p + x.dp);
        x.dq = A * (x.q + x.dq);
        x.p = A * x.p + Bq * vt;
        x.q = A * x.q + Bq;
        x.o = no;
    }

    // ---- descending: the segment alone (p, q stand for gp, gq)
    State3 g = {0.f, 0.f, O_INIT};
    for (int t = t1 - 1; t >= t0; --t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], gt = gy[ii];
        const float y = gv[ii], z = gk[ii], zexp = ze[ii];
        const ExpPair e = exp_pair(w + g.o, zexp - kt - u);
        const float no = e.no, A = e.ea, Bq = gt * z * e.eb;
        g.p = A * g.p + Bq;
        g.q = A * g.q - Bq * y;
        g.o = no;
    }
    State3 (*G)[NSEG][CH] = reinterpret_cast<State3 (*)[NSEG][CH]>(&X[0][0][0]);    // [2][NSEG][CH], inside X
    const int rs = NSEG - 1 - s;                   // position in the descending order
    G[0][rs][cl] = g;
    __syncthreads();
    cur = 0;
#pragma unroll
    for (int d = 1; d < NSEG; d *= 2) {
        State3 mine = G[cur][rs][cl];
        if (rs >= d) {
            State3 older = G[cur][rs - d][cl];
            older.o += static_cast<float>(d) * span * w;
            mine = combine(older, mine);
        }
        G[cur ^ 1][rs][cl] = mine;
        cur ^= 1;
        __syncthreads();
    }
    g = State3{0.f, 0.f, O_INIT};
    if (rs > 0) g = G[cur][rs - 1][cl];
    __syncthreads();

    // ---- descending, from the true state
    for (int t = t1 - 1; t >= t0; --t) {
        const size_t ii = static_cast<size_t>(t) * C;
        const float kt = k[ii], vt = v[ii], gt = gy[ii];
        const float y = gv[ii], z = gk[ii], zexp = ze[ii];
        float A = gt * z * exp32(zexp);
        float Bq = exp32(kt + g.o);
        gk[ii] = A * (vt - y) + Bq * (g.p * vt + g.q);
        gv[ii] = A + Bq * g.p;
        const ExpPair e2 = exp_pair(w + g.o, zexp - kt - u);
        const float no = e2.no;
        A = e2.ea;
        Bq = gt * z * e2.eb;
        g.p = A * g.p + Bq;
        g.q = A * g.q - Bq * y;
        g.o = no;
    }

    // ---- gw, gu: the segments' sums, added in time order
    float2* part = reinterpret_cast<float2*>(&X[0][0][0]);                         // [NSEG][CH]
    part[s * CH + cl] = make_float2(gw, gu);
    __syncthreads();
    if (s == 0 && live) {
        float a = 0.f, bsum = 0.f;
        for (int z = 0; z < NSEG; ++z) { a += part[z * CH + cl].x; bsum += part[z * CH + cl].y; }
        // the caller's buffers are accumulated into, as the reference does (wkv_cuda_v2.cu:112-113)
        if constexpr (RAW) {                        // per-batch partials in the library's own scratch: plain stores
            gw_[static_cast<size_t>(b) * C + c] = a * w;
            gu_[static_cast<size_t>(b) * C + c] = bsum;
        } else {
            gw_[static_cast<size_t>(b) * C + c] += a * w;
            gu_[static_cast<size_t>(b) * C + c] += bsum;
        }
    }
}

// ---------------------------------------------------------------------------------------- time-parallel, inputs in registers
// Up to NSEG * 16 = 1024 steps (the reference's own limit, wkv/run.py:149,153) a segment is at most 16 steps long,
// and a lane can hold its segment's k, v, gy and, in the backward, what the ascending sweep hands to the descending one
// (y_t, 1/den_t, zexp_t) in registers: every input is fetched once, all loads of a segment are in flight together
// instead of one dependent load per step and sweep, and the backward needs no workspace.  The arithmetic and its order
// are those of wkv4_fwd_seg / wkv4_bwd_seg, so the results are the same bit for bit.
//   CHR channels x NSEG segments per workgroup; SM = the most steps a segment may have (8 with 16 channels, 16 with 8).
// Workgroups are handed to the chip's 8 XCDs in turn, each with an L2 of its own, and a workgroup's 16 channels are half of
// a 128-byte line: numbered as launched, the two workgroups that share every line would sit on different XCDs and each
// L2 would fetch the whole line.  Workgroup x of XCD d takes piece d * (n / 8) + x instead, so neighbours share an L2.
DEVINL int paired_workgroup(int launched, int n) {
    return n % 16 == 0 ? (launched % 8) * (n / 8) + launched / 8 : launched;
}

template <bool RAW, int CHR, int SM>
__global__ __launch_bounds__(CHR * NSEG) void wkv4_fwd_reg(int T, int C, int S, const float* __restrict__ w_,
                                                          const float* __restrict__ u_, const float* __restrict__ k_,
                                                          const float* __restrict__ v_, float* __restrict__ y_) {
    __shared__ State3 X[2][NSEG][CHR];
    const int cl = threadIdx.x % CHR, s = threadIdx.x / CHR;
    const int q = paired_workgroup(blockIdx.x, gridDim.x), nx = (C + CHR - 1) / CHR;
    const int c = (q % nx) * CHR + cl, b = q / nx;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const float u = u_[cc], w = RAW ? -expf(w_[cc]) : w_[cc];        // RAW: the wrapper's w = -exp(w_raw) done here
    const int t0 = min(s * S, T), n = live ? min(t0 + S, T) - t0 : 0;
    const size_t off = (static_cast<size_t>(b) * T + t0) * C + cc;
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    float* __restrict__ y = y_ + off;

    float kk[SM], vv[SM];
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        kk[j] = 0.f; vv[j] = 0.f;
        if (j < n) { kk[j] = k[static_cast<size_t>(j) * C]; vv[j] = v[static_cast<size_t>(j) * C]; }
    }
    State3 x = {0.f, 0.f, O_INIT};
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        if (j < n) {
            const ExpPair e = exp_pair(w + x.o, kk[j]);
            const float no = e.no, A = e.ea, Bq = e.eb;
            x.p = A * x.p + Bq * vv[j];
            x.q = A * x.q + Bq;
            x.o = no;
        }
    }
    X[0][s][cl] = x;
    __syncthreads();
    int cur = 0;
#pragma unroll
    for (int d = 1; d < NSEG; d *= 2) {
        State3 mine = X[cur][s][cl];
        if (s >= d) {
            State3 older = X[cur][s - d][cl];
            older.o += static_cast<float>(d * S) * w;
            mine = combine(older, mine);
        }
        X[cur ^ 1][s][cl] = mine;
        cur ^= 1;
        __syncthreads();
    }
    x = State3{0.f, 0.f, O_INIT};
    if (s > 0) x = X[cur][s - 1][cl];
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        if (j < n) {
            ExpPair e = exp_pair(x.o, u + kk[j]);
            float no = e.no, A = e.ea, Bq = e.eb;
            y[static_cast<size_t>(j) * C] = (A * x.p + Bq * vv[j]) * recip(A * x.q + Bq);
            e = exp_pair(w + x.o, kk[j]);
            no = e.no;
            A = e.ea;
            Bq = e.eb;
            x.p = A * x.p + Bq * vv[j];
            x.q = A * x.q + Bq;
            x.o = no;
        }
    }
}

template <bool RAW, int CHR, int SM>
__global__ __launch_bounds__(CHR * NSEG) void wkv4_bwd_reg(int T, int C, int S, const float* __restrict__ w_,
                                                          const float* __restrict__ u_, const float* __restrict__ k_,
                                                          const float* __restrict__ v_, const float* __restrict__ gy_,
                                                          float* __restrict__ gw_, float* __restrict__ gu_,
                                                          float* __restrict__ gk_, float* __restrict__ gv_) {
    __shared__ State5 X[2][NSEG][CHR];
    const int cl = threadIdx.x % CHR, s = threadIdx.x / CHR;
    const int q = paired_workgroup(blockIdx.x, gridDim.x), nx = (C + CHR - 1) / CHR;
    const int c = (q % nx) * CHR + cl, b = q / nx;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const float u = u_[cc], w = RAW ? -expf(w_[cc]) : w_[cc];        // RAW: the wrapper's w = -exp(w_raw) done here
    // lanes past C have no steps: they only keep the barriers company
    const int t0 = min(s * S, T), n = live ? min(t0 + S, T) - t0 : 0;
    const size_t off = (static_cast<size_t>(b) * T + t0) * C + cc;
    const float* __restrict__ k = k_ + off;
    const float* __restrict__ v = v_ + off;
    const float* __restrict__ gy = gy_ + off;
    float* __restrict__ gk = gk_ + off;
    float* __restrict__ gv = gv_ + off;
    const float span = static_cast<float>(S);

    float kk[SM], vv[SM], gg[SM], yy[SM], zz[SM], ze[SM];
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        kk[j] = 0.f; vv[j] = 0.f; gg[j] = 0.f;
        if (j < n) {
            kk[j] = k[static_cast<size_t>(j) * C]; vv[j] = v[static_cast<size_t>(j) * C]; gg[j] = gy[static_cast<size_t>(j) * C];
        }
    }

    // ---- ascending: the segment alone
    State5 x = {0.f, 0.f, 0.f, 0.f, O_INIT};
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        if (j < n) {
            const ExpPair e = exp_pair(w + x.o, kk[j]);
            const float no = e.no, A = e.ea, Bq = e.eb;
            x.dp = A * (x.p + x.dp);
            x.dq = A * (x.q + x.dq);
            x.p = A * x.p + Bq * vv[j];
            x.q = A * x.q + Bq;
            x.o = no;
        }
    }
    X[0][s][cl] = x;
    __syncthreads();
    int cur = 0;
#pragma unroll
    for (int d = 1; d < NSEG; d *= 2) {
        State5 mine = X[cur][s][cl];
        if (s >= d) {
            State5 older = X[cur][s - d][cl];
            const float m = static_cast<float>(d) * span;
            older.dp += m * older.p;
            older.dq += m * older.q;
            older.o += m * w;
            mine = combine(older, mine);
        }
        X[cur ^ 1][s][cl] = mine;
        cur ^= 1;
        __syncthreads();
    }
    x = State5{0.f, 0.f, 0.f, 0.f, O_INIT};
    if (s > 0) x = X[cur][s - 1][cl];
    __syncthreads();                               // X is reused below

    // ---- ascending, from the true state: y, 1/den and zexp stay in registers for the descending sweep
    float gw = 0.f, gu = 0.f;
#pragma unroll
    for (int j = 0; j < SM; ++j) {
        yy[j] = 0.f; zz[j] = 0.f; ze[j] = 0.f;
        if (j < n) {
            const float kt = kk[j], vt = vv[j], gt = gg[j];
            ExpPair e = exp_pair(x.o, kt + u);
            float no = e.no, A = e.ea, Bq = e.eb;
            const float num = A * x.p + Bq * vt;
            const float iden = recip(A * x.q + Bq);
            const float y = num * iden;
            yy[j] = y;
            zz[j] = iden;
            ze[j] = kt + u - no;
            gw += gt * (x.dp - x.dq * y) * iden * A;
            gu += gt * (vt - y) * Bq * iden;
            e = exp_pair(w + x.o, kt);
            no = e.no;
            A = e.ea;
            Bq = e.eb;
            x.dp = A * (x.p + x.dp);
            x.dq = A * (x.q + x.dq);
            x.p = A * x.p + Bq * vt;
            x.q = A * x.q + Bq;
            x.o = no;
        }
    }

    // ---- descending: the segment alone (p, q stand for gp, gq)
    State3 g = {0.f, 0.f, O_INIT};
#pragma unroll
    for (int j = SM - 1; j >= 0; --j) {
        if (j < n) {
            const ExpPair e = exp_pair(w + g.o, ze[j] - kk[j] - u);
            const float no = e.no, A = e.ea, Bq = gg[j] * zz[j] * e.eb;
            g.p = A * g.p + Bq;
            g.q = A * g.q - Bq * yy[j];
            g.o = no;
        }
    }
    State3 (*G)[NSEG][CHR] = reinterpret_cast<State3 (*)[NSEG][CHR]>(&X[0][0][0]);  // [2][NSEG][CHR], inside X
    const int rs = NSEG - 1 - s;                   // position in the descending order
    G[0][rs][cl] = g;
    __syncthreads();
    cur = 0;
#pragma unroll
    for (int d = 1; d < NSEG; d *= 2) {
        State3 mine = G[cur][rs][cl];
        if (rs >= d) {
            State3 older = G[cur][rs - d][cl];
            older.o += static_cast<float>(d) * span * w;
            mine = combine(older, mine);
        }
        G[cur ^ 1][rs][cl] = mine;
        cur ^= 1;
        __syncthreads();
    }
    g = State3{0.f, 0.f, O_INIT};
    if (rs > 0) g = G[cur][rs - 1][cl];
    __syncthreads();

    // ---- descending, from the true state
#pragma unroll
    for (int j = SM - 1; j >= 0; --j) {
        if (j < n) {
            const float kt = kk[j], vt = vv[j], gt = gg[j];
            const float y = yy[j], z = zz[j], zexp = ze[j];
            float A = gt * z * exp32(zexp);
            float Bq = exp32(kt + g.o);
            gk[static_cast<size_t>(j) * C] = A * (vt - y) + Bq * (g.p * vt + g.q);
            gv[static_cast<size_t>(j) * C] = A + Bq * g.p;
            const ExpPair e2 = exp_pair(w + g.o, zexp - kt - u);
            const float no = e2.no;
            A = e2.ea;
            Bq = gt * z * e2.eb;
            g.p = A * g.p + Bq;
            g.q = A * g.q - Bq * y;
            g.o = no;
        }
    }

    // ---- gw, gu: the segments' sums, added in time order
    float2* part = reinterpret_cast<float2*>(&X[0][0][0]);                         // [NSEG][CHR]
    part[s * CHR + cl] = make_float2(gw, gu);
    __syncthreads();
    if (s == 0 && live) {
        float a = 0.f, bsum = 0.f;
        for (int z = 0; z < NSEG; ++z) { a += part[z * CHR + cl].x; bsum += part[z * CHR + cl].y; }
        // the caller's buffers are accumulated into, as the reference does (wkv_cuda_v2.cu:112-113)
        if constexpr (RAW) {                        // per-batch partials in the library's own scratch: plain stores
            gw_[static_cast<size_t>(b) * C + c] = a * w;
            gu_[static_cast<size_t>(b) * C + c] = bsum;
        } else {
            gw_[static_cast<size_t>(b) * C + c] += a * w;
            gu_[static_cast<size_t>(b) * C + c] += bsum;
        }
    }
}

// ------------------------------------------------------------------------------- longer sequences: blocks of 512 steps
// Beyond NSEG * 16 steps a workgroup walks over blocks of NSEG * 8 steps and hands the state from block to block: inside
// a block everything is as in the register kernels, and the state in front of a segment is the block's entering state,
// aged by the steps in between, combined with the segments of the block before it.  The backward first walks up with
// the ascending sweep's summaries only (k, v read, nothing written) to learn the state entering every block, keeps those
// in LDS, then walks down block by block doing both sweeps.  k and v are read twice, gy once, nothing is parked in memory.
constexpr int BLK_S = 8, BLK_T = NSEG * BLK_S, BLK_CH = 16;
constexpr int BLK_MAX = 64;            // blocks whose entering states fit in LDS: T <= 32768

DEVINL State3 aged(State3 a, float steps, float w) { a.o += steps * w; return a; }
DEVINL State5 aged(State5 a, float steps, float w) {
    a.dp += steps * a.p;
    a.dq += steps * a.q;
    a.o += steps * w;
    return a;
}

template <bool RAW>
__global__ __launch_bounds__(BLK_CH * NSEG) void wkv4_fwd_blk(int T, int C, const float* __restrict__ w_,
                                                             const float* __restrict__ u_, const float* __restrict__ k_,
                                                             const float* __restrict__ v_, float* __restrict__ y_) {
    __shared__ State3 X[2][NSEG][BLK_CH];
    const int cl = threadIdx.x % BLK_CH, s = threadIdx.x / BLK_CH;
    const int q = paired_workgroup(blockIdx.x, gridDim.x), nx = (C + BLK_CH - 1) / BLK_CH;
    const int c = (q % nx) * BLK_CH + cl, b = q / nx;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const float u = u_[cc], w = RAW ? -expf(w_[cc]) : w_[cc];        // RAW: the wrapper's w = -exp(w_raw) done here
    const int nblk = (T + BLK_T - 1) / BLK_T;
    State3 carry = {0.f, 0.f, O_INIT};             // the state entering the block; every lane of a channel holds it

    for (int blk = 0; blk < nblk; ++blk) {
        const int t0 = min(blk * BLK_T + s * BLK_S, T), n = live ? min(t0 + BLK_S, T) - t0 : 0;
        const size_t off = (static_cast<size_t>(b) * T + t0) * C + cc;
        const float* __restrict__ k = k_ + off;
        const float* __restrict__ v = v_ + off;
        float* __restrict__ y = y_ + off;
        float kk[BLK_S], vv[BLK_S];
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            kk[j] = 0.f; vv[j] = 0.f;
            if (j < n) { kk[j] = k[static_cast<size_t>(j) * C]; vv[j] = v[static_cast<size_t>(j) * C]; }
        }
        State3 x = {0.f, 0.f, O_INIT};
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            if (j < n) {
                const ExpPair e = exp_pair(w + x.o, kk[j]);
                x.p = e.ea * x.p + e.eb * vv[j];
                x.q = e.ea * x.q + e.eb;
                x.o = e.no;
            }
        }
        X[0][s][cl] = x;
        __syncthreads();
        int cur = 0;
#pragma unroll
        for (int d = 1; d < NSEG; d *= 2) {
            State3 mine = X[cur][s][cl];
            if (s >= d) mine = combine(aged(X[cur][s - d][cl], static_cast<float>(d * BLK_S), w), mine);
            X[cur ^ 1][s][cl] = mine;
            cur ^= 1;
            __syncthreads();
        }
        x = aged(carry, static_cast<float>(s * BLK_S), w);
        if (s > 0) x = combine(x, X[cur][s - 1][cl]);
        carry = combine(aged(carry, static_cast<float>(BLK_T), w), X[cur][NSEG - 1][cl]);
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            if (j < n) {
                ExpPair e = exp_pair(x.o, u + kk[j]);
                y[static_cast<size_t>(j) * C] = (e.ea * x.p + e.eb * vv[j]) * recip(e.ea * x.q + e.eb);
                e = exp_pair(w + x.o, kk[j]);
                x.p = e.ea * x.p + e.eb * vv[j];
                x.q = e.ea * x.q + e.eb;
                x.o = e.no;
            }
        }
        __syncthreads();                           // X is written again by the next block
    }
}

template <bool RAW>
__global__ __launch_bounds__(BLK_CH * NSEG) void wkv4_bwd_blk(int T, int C, const float* __restrict__ w_,
                                                             const float* __restrict__ u_, const float* __restrict__ k_,
                                                             const float* __restrict__ v_, const float* __restrict__ gy_,
                                                             float* __restrict__ gw_, float* __restrict__ gu_,
                                                             float* __restrict__ gk_, float* __restrict__ gv_) {
    __shared__ State5 X[2][NSEG][BLK_CH];
    __shared__ State5 ENTER[BLK_MAX][BLK_CH];      // the ascending sweep's state entering each block
    const int cl = threadIdx.x % BLK_CH, s = threadIdx.x / BLK_CH;
    const int q = paired_workgroup(blockIdx.x, gridDim.x), nx = (C + BLK_CH - 1) / BLK_CH;
    const int c = (q % nx) * BLK_CH + cl, b = q / nx;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const float u = u_[cc], w = RAW ? -expf(w_[cc]) : w_[cc];        // RAW: the wrapper's w = -exp(w_raw) done here
    const int nblk = (T + BLK_T - 1) / BLK_T;
    const size_t row = static_cast<size_t>(b) * T;

    // the segment alone, from the empty state, then the scan over the block's segments: X[cur] holds the inclusive prefixes
    auto summaries = [&](const float (&kk)[BLK_S], const float (&vv)[BLK_S], int n) -> int {
        State5 x = {0.f, 0.f, 0.f, 0.f, O_INIT};
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            if (j < n) {
                const ExpPair e = exp_pair(w + x.o, kk[j]);
                x.dp = e.ea * (x.p + x.dp);
                x.dq = e.ea * (x.q + x.dq);
                x.p = e.ea * x.p + e.eb * vv[j];
                x.q = e.ea * x.q + e.eb;
                x.o = e.no;
            }
        }
        X[0][s][cl] = x;
        __syncthreads();
        int cur = 0;
#pragma unroll
        for (int d = 1; d < NSEG; d *= 2) {
            State5 mine = X[cur][s][cl];
            if (s >= d) mine = combine(aged(X[cur][s - d][cl], static_cast<float>(d * BLK_S), w), mine);
            X[cur ^ 1][s][cl] = mine;
            cur ^= 1;
            __syncthreads();
        }
        return cur;
    };

    // ---- up: the state entering every block
    State5 carry = {0.f, 0.f, 0.f, 0.f, O_INIT};
    for (int blk = 0; blk < nblk; ++blk) {
        if (s == 0) ENTER[blk][cl] = carry;
        if (blk == nblk - 1) break;
        const int t0 = min(blk * BLK_T + s * BLK_S, T), n = live ? min(t0 + BLK_S, T) - t0 : 0;
        const size_t off = (row + t0) * C + cc;
        float kk[BLK_S], vv[BLK_S];
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            kk[j] = 0.f; vv[j] = 0.f;
            if (j < n) { kk[j] = k_[off + static_cast<size_t>(j) * C]; vv[j] = v_[off + static_cast<size_t>(j) * C]; }
        }
        const int cur = summaries(kk, vv, n);
        carry = combine(aged(carry, static_cast<float>(BLK_T), w), X[cur][NSEG - 1][cl]);
        __syncthreads();                           // X is written again by the next block
    }
    __syncthreads();

    // ---- down: both sweeps of a block, the descending sweep's state handed from block to block
    State3 gcarry = {0.f, 0.f, O_INIT};
    float gw = 0.f, gu = 0.f;
    const int rs = NSEG - 1 - s;                   // position in the descending order
    for (int blk = nblk - 1; blk >= 0; --blk) {
        const int t0 = min(blk * BLK_T + s * BLK_S, T), n = live ? min(t0 + BLK_S, T) - t0 : 0;
        const size_t off = (row + t0) * C + cc;
        float* __restrict__ gk = gk_ + off;
        float* __restrict__ gv = gv_ + off;
        float kk[BLK_S], vv[BLK_S], gg[BLK_S], yy[BLK_S], zz[BLK_S], ze[BLK_S];
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            kk[j] = 0.f; vv[j] = 0.f; gg[j] = 0.f;
            if (j < n) {
                kk[j] = k_[off + static_cast<size_t>(j) * C]; vv[j] = v_[off + static_cast<size_t>(j) * C];
                gg[j] = gy_[off + static_cast<size_t>(j) * C];
            }
        }
        int cur = summaries(kk, vv, n);
        State5 x = aged(ENTER[blk][cl], static_cast<float>(s * BLK_S), w);
        if (s > 0) x = combine(x, X[cur][s - 1][cl]);
        __syncthreads();                           // X is reused below

        // ascending, from the true state
#pragma unroll
        for (int j = 0; j < BLK_S; ++j) {
            yy[j] = 0.f; zz[j] = 0.f; ze[j] = 0.f;
            if (j < n) {
                const float kt = kk[j], vt = vv[j], gt = gg[j];
                ExpPair e = exp_pair(x.o, kt + u);
                const float num = e.ea * x.p + e.eb * vt;
                const float iden = recip(e.ea * x.q + e.eb);
                const float y = num * iden;
                yy[j] = y;
                zz[j] = iden;
                ze[j] = kt + u - e.no;
                gw += gt * (x.dp - x.dq * y) * iden * e.ea;
                gu += gt * (vt - y) * e.eb * iden;
                e = exp_pair(w + x.o, kt);
                x.dp = e.ea * (x.p + x.dp);
                x.dq = e.ea * (x.q + x.dq);
                x.p = e.ea * x.p + e.eb * vt;
                x.q = e.ea * x.q + e.eb;
                x.o = e.no;
            }
        }
        // descending: the segment alone (p, q stand for gp, gq)
        State3 g = {0.f, 0.f, O_INIT};
#pragma unroll
        for (int j = BLK_S - 1; j >= 0; --j) {
            if (j < n) {
                const ExpPair e = exp_pair(w + g.o, ze[j] - kk[j] - u);
                const float Bq = gg[j] * zz[j] * e.eb;
                g.p = e.ea * g.p + Bq;
                g.q = e.ea * g.q - Bq * yy[j];
                g.o = e.no;
            }
        }
        State3 (*G)[NSEG][BLK_CH] = reinterpret_cast<State3 (*)[NSEG][BLK_CH]>(&X[0][0][0]);    // [2][NSEG][BLK_CH], inside X
        G[0][rs][cl] = g;
        __syncthreads();
        cur = 0;
#pragma unroll
        for (int d = 1; d < NSEG; d *= 2) {
            State3 mine = G[cur][rs][cl];
            if (rs >= d) mine = combine(aged(G[cur][rs - d][cl], static_cast<float>(d * BLK_S), w), mine);
            G[cur ^ 1][rs][cl] = mine;
            cur ^= 1;
            __syncthreads();
        }
        g = aged(gcarry, static_cast<float>(rs * BLK_S), w);
        if (rs > 0) g = combine(g, G[cur][rs - 1][cl]);
        gcarry = combine(aged(gcarry, static_cast<float>(BLK_T), w), G[cur][NSEG - 1][cl]);
        __syncthreads();                           // X is written again by the next block

        // descending, from the true state
#pragma unroll
        for (int j = BLK_S - 1; j >= 0; --j) {
            if (j < n) {
                const float kt = kk[j], vt = vv[j], gt = gg[j];
                const float y = yy[j], z = zz[j], zexp = ze[j];
                const float A = gt * z * exp32(zexp);
                const float Bq = exp32(kt + g.o);
                gk[static_cast<size_t>(j) * C] = A * (vt - y) + Bq * (g.p * vt + g.q);
                gv[static_cast<size_t>(j) * C] = A + Bq * g.p;
                const ExpPair e = exp_pair(w + g.o, zexp - kt - u);
                const float B2 = gt * z * e.eb;
                g.p = e.ea * g.p + B2;
                g.q = e.ea * g.q - B2 * y;
                g.o = e.no;
            }
        }
    }

    // ---- gw, gu: the segments' sums, added in time order
    float2* part = reinterpret_cast<float2*>(&X[0][0][0]);                         // [NSEG][BLK_CH]
    part[s * BLK_CH + cl] = make_float2(gw, gu);
    __syncthreads();
    if (s == 0 && live) {
        float a = 0.f, bsum = 0.f;
        for (int z = 0; z < NSEG; ++z) { a += part[z * BLK_CH + cl].x; bsum += part[z * BLK_CH + cl].y; }
        // the caller's buffers are accumulated into, as the reference does (wkv_cuda_v2.cu:112-113)
        if constexpr (RAW) {                        // per-batch partials in the library's own scratch: plain stores
            gw_[static_cast<size_t>(b) * C + c] = a * w;
            gu_[static_cast<size_t>(b) * C + c] = bsum;
        } else {
            gw_[static_cast<size_t>(b) * C + c] += a * w;
            gu_[static_cast<size_t>(b) * C + c] += bsum;
        }
    }
}

// out[c] = sum_b part[b][c]: the wrapper's torch.sum(gw, dim=0) (wkv/run.py:115-116), in a fixed order: four lanes per
// channel take every fourth batch row each, and their sums are added in lane order
__global__ __launch_bounds__(256) void wkv4_batch_sum(int B, int C, const float* __restrict__ pw, const float* __restrict__ pu,
                                                      float* __restrict__ gw, float* __restrict__ gu) {
    __shared__ float2 part[4][64];
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6, c = blockIdx.x * 64 + cl;
    float a = 0.f, b2 = 0.f;
    if (c < C)
        for (int b = q; b < B; b += 4) { a += pw[static_cast<size_t>(b) * C + c]; b2 += pu[static_cast<size_t>(b) * C + c]; }
    part[q][cl] = make_float2(a, b2);
    __syncthreads();
    if (q == 0 && c < C) {
        const float2 x0 = part[0][cl], x1 = part[1][cl], x2 = part[2][cl], x3 = part[3][cl];
        gw[c] = ((x0.x + x1.x) + x2.x) + x3.x;
        gu[c] = ((x0.y + x1.y) + x2.y) + x3.y;
    }
}

// Which form runs: one lane per scan beyond the grid's y range, inputs in registers while a segment has at most 16
// steps, blocks of 512 steps with the state handed on up to 32768 steps, and beyond that the form that parks the ascending
// sweep's results in memory.
template <bool RAW, int CHR, int SM, typename... Ptrs>
void launch4_fwd_reg(hipStream_t st, int B, int T, int C, int S, Ptrs... p) {
    hipLaunchKernelGGL((wkv4_fwd_reg<RAW, CHR, SM>), dim3(((C + CHR - 1) / CHR) * B), dim3(CHR * NSEG), 0, st, T, C, S, p...);
}
template <bool RAW, int CHR, int SM, typename... Ptrs>
void launch4_bwd_reg(hipStream_t st, int B, int T, int C, int S, Ptrs... p) {
    hipLaunchKernelGGL((wkv4_bwd_reg<RAW, CHR, SM>), dim3(((C + CHR - 1) / CHR) * B), dim3(CHR * NSEG), 0, st, T, C, S, p...);
}

template <bool RAW>
void launch4_fwd(hipStream_t st, int B, int T, int C, const float* w, const float* u, const float* k, const float* v, float* y) {
    const int S = (T + NSEG - 1) / NSEG;
    if (B > 65535) {
        const int BC = B * C;
        hipLaunchKernelGGL((wkv4_fwd<RAW>), dim3((BC + NT - 1) / NT), dim3(NT), 0, st, BC, T, C, w, u, k, v, y);
    } else if (S <= 8) {
        launch4_fwd_reg<RAW, 16, 8>(st, B, T, C, S, w, u, k, v, y);
    } else if (S <= 16) {
        launch4_fwd_reg<RAW, 8, 16>(st, B, T, C, S, w, u, k, v, y);
    } else if (T <= BLK_T * BLK_MAX) {
        hipLaunchKernelGGL((wkv4_fwd_blk<RAW>), dim3(((C + BLK_CH - 1) / BLK_CH) * B), dim3(BLK_CH * NSEG), 0, st, T, C, w, u, k, v, y);
    } else {
        hipLaunchKernelGGL((wkv4_fwd_seg<RAW>), dim3((C + CH - 1) / CH, B), dim3(NTS), 0, st, T, C, S, w, u, k, v, y);
    }
}

template <bool RAW>
void launch4_bwd(hipStream_t st, int B, int T, int C, const float* w, const float* u, const float* k, const float* v,
                 const float* gy, float* gw, float* gu, float* gk, float* gv, float* ze) {
    const int S = (T + NSEG - 1) / NSEG;
    if (B > 65535) {
        const int BC = B * C;
        hipLaunchKernelGGL((wkv4_bwd<RAW>), dim3((BC + NT - 1) / NT), dim3(NT), 0, st, BC, T, C, w, u, k, v, gy, gw, gu, gk, gv, ze);
    } else if (S <= 8) {
        launch4_bwd_reg<RAW, 16, 8>(st, B, T, C, S, w, u, k, v, gy, gw, gu, gk, gv);
    } else if (S <= 16) {
        launch4_bwd_reg<RAW, 8, 16>(st, B, T, C, S, w, u, k, v, gy, gw, gu, gk, gv);
    } else if (T <= BLK_T * BLK_MAX) {
        hipLaunchKernelGGL((wkv4_bwd_blk<RAW>), dim3(((C + BLK_CH - 1) / BLK_CH) * B), dim3(BLK_CH * NSEG), 0, st, T, C, w, u, k, v, gy, gw, gu, gk, gv);
    } else {
        hipLaunchKernelGGL((wkv4_bwd_seg<RAW>), dim3((C + CH - 1) / CH, B), dim3(NTS), 0, st, T, C, S, w, u, k, v, gy, gw, gu, gk, gv, ze);
    }
}

// the forms of launch4_bwd that take the workspace `ze` (the plain kernel and the one for very long sequences)
bool bwd_uses_workspace(int B, int T) {
    const int S = (T + NSEG - 1) / NSEG;
    return B > 65535 || (S > 16 && T > BLK_T * BLK_MAX);
}

int check4(int B, int T, int C) {
    if (B <= 0 || T <= 0 || C <= 0) return RWKV_ERR_SHAPE;
    if (static_cast<long long>(B) * C > 0x7fffffffLL) return RWKV_ERR_SHAPE;
    return RWKV_OK;
}

// Scratch of the entry point that allocates nothing: the backward's per-step intermediates (B*T*C floats) live in this
// file-scope device array instead of a caller's workspace.  Each GPU the library runs on holds its own copy, at its own
// address, until the process ends.  `scratch` itself is only a host-side handle: the device address comes from
// hipGetSymbolAddress, once per device, and that address is what the kernels receive.
constexpr size_t NOALLOC_MAX_FLOATS = size_t(1) << 21;           // 8 MiB: B*T*C <= 2 097 152 (B4 T512 C768 needs 1 572 864)
static __device__ __align__(256) float scratch[NOALLOC_MAX_FLOATS];
constexpr int MAX_DEVICES = 64;
std::atomic<float*> g_scratch_ptr[MAX_DEVICES];                  // written once per device; every writer stores the same value

int scratch_of_current_device(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return RWKV_ERR_LAUNCH;
    float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        void* sym = nullptr;
        const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (e != hipSuccess || sym == nullptr) { g_last_hip_error = static_cast<int>(e); return RWKV_ERR_LAUNCH; }
        p = static_cast<float*>(sym);
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
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
    launch4_fwd<false>(static_cast<hipStream_t>(stream), B, T, C, w, u, k, v, y);
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
    launch4_bwd<false>(static_cast<hipStream_t>(stream), B, T, C, w, u, k, v, gy, gw, gu, gk, gv, static_cast<float*>(workspace));
    return launch_status();
}

// ---- the whole of WKV.forward / WKV.backward (wkv/run.py:89-117) behind two entry points: raw w, summed gw and gu
int rwkv_wkv4raw_forward(void* stream, int B, int T, int C, const float* w_raw, const float* u, const float* k,
                         const float* v, float* y) {
    if (int e = check4(B, T, C)) return e;
    if (int e = check_ptrs({w_raw, u, k, v, y})) return e;
    launch4_fwd<true>(static_cast<hipStream_t>(stream), B, T, C, w_raw, u, k, v, y);
    return launch_status();
}

size_t rwkv_wkv4raw_backward_workspace_bytes(int B, int T, int C) {
    if (check4(B, T, C) != RWKV_OK) return 0;
    return (static_cast<size_t>(B) * T * C + 2 * static_cast<size_t>(B) * C) * sizeof(float);
}

int rwkv_wkv4raw_backward(void* stream, int B, int T, int C, const float* w_raw, const float* u, const float* k,
                          const float* v, const float* gy, float* gw, float* gu, float* gk, float* gv,
                          void* workspace, size_t workspace_bytes) {
    if (int e = check4(B, T, C)) return e;
    if (int e = check_ptrs({w_raw, u, k, v, gy, gw, gu, gk, gv})) return e;
    if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < rwkv_wkv4raw_backward_workspace_bytes(B, T, C))
        return RWKV_ERR_WORKSPACE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    float* ze = static_cast<float*>(workspace);
    float* pw = ze + static_cast<size_t>(B) * T * C;
    float* pu = pw + static_cast<size_t>(B) * C;
    launch4_bwd<true>(st, B, T, C, w_raw, u, k, v, gy, pw, pu, gk, gv, ze);
    hipLaunchKernelGGL(wkv4_batch_sum, dim3((C + 63) / 64), dim3(256), 0, st, B, C, pw, pu, gw, gu);
    return launch_status();
}

size_t rwkv_wkv4_backward_noalloc_max_elems(void) { return NOALLOC_MAX_FLOATS; }

int rwkv_wkv4_backward_noalloc(void* stream, int B, int T, int C, const float* w, const float* u, const float* k,
                               const float* v, const float* gy, float* gw, float* gu, float* gk, float* gv) {
    if (int e = check4(B, T, C)) return e;
    if (int e = check_ptrs({w, u, k, v, gy, gw, gu, gk, gv})) return e;
    float* ws = nullptr;
    // The kernels for T up to 32768 keep their intermediates in registers and LDS; only the plain kernel (B above 65535)
    // and the one for longer sequences write B T C floats to a workspace, and only those shapes are bounded by the scratch.
    if (bwd_uses_workspace(B, T)) {
        if (static_cast<unsigned long long>(B) * T * C > NOALLOC_MAX_FLOATS) return RWKV_ERR_WORKSPACE;
        // every element of the scratch that the kernels read they have written earlier in the same launch: nothing to clear
        if (int e = scratch_of_current_device(&ws)) return e;
    }
    launch4_bwd<false>(static_cast<hipStream_t>(stream), B, T, C, w, u, k, v, gy, gw, gu, gk, gv, ws);
    return launch_status();
}

}  // extern "C"
