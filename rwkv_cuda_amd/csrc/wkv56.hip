// wkv5 / wkv6 / wkv6_state for gfx950: sequential-in-time sweeps with the 64x64 state in VGPRs.
//
// One workgroup (8 waves) per (batch, head).  The state S[i][j] (i = value channel, j = key
// channel) is tiled 16 elements per lane in one of two ways:
//   shape F  lane = i, wave q holds j in [8q,8q+8)   out[i] = sum_j a[j] S[i][j];  S = S w[j] + b[j] x[i]
//   shape G  lane = j, wave q holds i in [8q,8q+8)   out[j] = sum_i a[i] S[i][j];  S = S w[j] + x[i] b[j]
// Vectors indexed by the in-register axis are kept one element per lane, replicated in every
// 16-lane DPP row, and enter the FMAs through row_newbcast, so a step is 3 VALU ops per state
// element and four LDS reads per lane.  Inputs are staged through LDS as fp32 in chunks of
// TC time steps (16-byte global loads, issued one chunk ahead); the four waves' partial sums
// are combined once per chunk, where the outputs are rounded to bf16 and stored 16 bytes
// at a time.
//
// Passes (what the reference does in wkv5_cuda_v1b.cu / wkv6_cuda_v1.cu / wkv6state_cuda_v1a.cu):
//   FWD  shape F, t up,   a=r b=k x=v    y_t[i]  = sum_j r(S + u k v)                 S_0 = s0
//   GR   shape G, t up,   a=gy x=v b=k   gr_t[j] = sum_i gy S + u k (v.gy);  gu;  r*dr' -> workspace
//   GK   shape G, t down, a=v x=gy b=r   gk_t[j] = sum_i v dS + u r (v.gy);  gw;  gs = dS_0
//   GV   shape F, t down, a=k b=r x=gy   gv_t[i] = sum_j k dS + gy sum_j(u r k)
// The decay gradient needs no third recurrence: with P_t[j] = sum_i dS_t[i,j] S_t[i,j],
//   G_t = w_t * sum_i dS_{t+1} S_t = P_{t+1} - k_t dk'_t,   P_t = G_t + r_t dr'_t,   P_T = 0,
// where dr', dk' are the bonus-free parts of gr, gk; gw_raw = -exp(w_raw) * G.
//
// The same kernels with fp32 loads and stores (F32) are the fp32 wkv5 op (wkv5/cuda/wkv5_op.cpp); there GR carries
// Q = dS/dw and makes gw itself, without the P recurrence and its workspace.  With TWO they are wkv5a
// (wkv5a_cuda_v1a2.cu): decay w1[j] w2[i] and bonus u1[j] + u2[i] per state element.
#include "common.h"

namespace rwkv {
namespace {

constexpr int N = 64;            // head size
constexpr int TC = 32;           // time steps per staged chunk
constexpr int NW = 8;            // waves per workgroup: two per SIMD (one wave per SIMD issues VALU ~3x slower)
constexpr int NT = NW * 64;
constexpr int JW = N / NW;       // state elements per lane
constexpr int NSTAGE = TC * N / 8;   // threads that stage / finish a chunk (8 elements each)
static_assert(JW <= 16 && (JW & (JW - 1)) == 0, "row broadcast: the state elements of a lane must fit one 16-lane row");
static_assert(NSTAGE <= NT && NSTAGE % 64 == 0, "staging threads are whole waves");

enum { P_FWD = 0, P_GR = 1, P_GK = 2, P_GV = 3 };
enum { W_HEAD = 0, W_EW = 1, W_RAW = 2 };   // wkv5 (eew[H,N] fp32) / wkv6 (ew fp32 [B,T,C]) / wkv6_state (raw bf16)

// Element pointers are typed for the bf16 ops; the fp32 wkv5 op stores float pointers in the same fields and its
// kernels (F32 = true) read them back as such through load8 / store8 / load1 / store1 below.
struct Args {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0, *gy;
    const void* w;        // W_HEAD: const float* eew[H*N]; W_EW: const float* ew[B*T*C]; W_RAW: const uint16_t* raw
    const float* ew_head; // W_HEAD, GK only: -exp(w_raw) [H*N]
    uint16_t *y, *gr, *gk, *gv, *gw, *gu, *gs;
    // two-sided decay and bonus (wkv5a): decay w[j] * w2[i], bonus u[j] + u2[i], i = value channel
    const float *w2, *ew2_head;
    const uint16_t* u2;
    uint16_t *gw2, *gu2;
    float* rdr;           // workspace [B,T,C] fp32: r * dr'
};

template <int PASS> struct Smem {
    static constexpr bool kBwd = PASS != P_FWD;
    static constexpr bool kGK = PASS == P_GK;
    float r[TC][N];
    float k[TC][N];
    float v[(PASS == P_GV) ? 1 : TC][N];
    float g[kBwd ? TC : 1][N];
    float w[TC][N];
    float f[kGK ? TC : 1][N];      // d(log decay)/d(w_raw) * ... : the factor that turns G into gw
    float rdr[kGK ? TC : 1][N];
    float part[NW][TC][N];
    float dot[TC];
    float u[N];
    float dot2[TC], dot3[TC];      // two-sided mode only
    float u2[N], w2[N];
};

// eight consecutive elements as they come from memory: bf16 in one 16-byte load, fp32 in two
template <bool F32> struct Raw8;
template <> struct Raw8<false> { uint4 q; };
template <> struct Raw8<true> { float4 a, b; };

template <bool F32> DEVINL Raw8<F32> load8(const uint16_t* p, size_t off, bool ok) {
    Raw8<F32> x;
    if constexpr (F32) {
        const float* f = reinterpret_cast<const float*>(p) + off;
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        x.a = ok ? *reinterpret_cast<const float4*>(f) : z;
        x.b = ok ? *reinterpret_cast<const float4*>(f + 4) : z;
    } else {
        x.q = ok ? *reinterpret_cast<const uint4*>(p + off) : make_uint4(0, 0, 0, 0);
    }
    return x;
}
template <bool F32> DEVINL void widen8(const Raw8<F32>& x, float (&f)[8]) {
    if constexpr (F32) {
        f[0] = x.a.x; f[1] = x.a.y; f[2] = x.a.z; f[3] = x.a.w; f[4] = x.b.x; f[5] = x.b.y; f[6] = x.b.z; f[7] = x.b.w;
    } else {
        unpack8(x.q, f);
    }
}
template <bool F32> DEVINL void store8(uint16_t* p, size_t off, const float (&f)[8]) {
    if constexpr (F32) {
        float* d = reinterpret_cast<float*>(p) + off;
        *reinterpret_cast<float4*>(d) = make_float4(f[0], f[1], f[2], f[3]);
        *reinterpret_cast<float4*>(d + 4) = make_float4(f[4], f[5], f[6], f[7]);
    } else {
        *reinterpret_cast<uint4*>(p + off) = pack8(f);
    }
}
template <bool F32> DEVINL float load1(const uint16_t* p, size_t i) {
    if constexpr (F32) return reinterpret_cast<const float*>(p)[i];
    else return bf2f(p[i]);
}
template <bool F32> DEVINL void store1(uint16_t* p, size_t i, float x) {
    if constexpr (F32) reinterpret_cast<float*>(p)[i] = x;
    else p[i] = f2bf(x);
}

template <bool F32> struct Staged {
    Raw8<F32> r, k, v, g;
    uint4 w0, w1;
    float4 rdr0, rdr1;
};

template <int PASS, int WMODE, bool F32>
DEVINL void prefetch(Staged<F32>& p, const Args& a, size_t base, int c0, int st, int sj) {
    const int t = c0 + st;
    const bool ok = t < a.T;
    const size_t off = base + static_cast<size_t>(t) * a.C + sj;
    const uint4 z = make_uint4(0, 0, 0, 0);
    p.r = load8<F32>(a.r, off, ok);
    p.k = load8<F32>(a.k, off, ok);
    if constexpr (PASS != P_GV) p.v = load8<F32>(a.v, off, ok);
    if constexpr (PASS != P_FWD) p.g = load8<F32>(a.gy, off, ok);
    if constexpr (WMODE == W_RAW) {
        p.w0 = ok ? *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.w) + off) : z;
    } else if constexpr (WMODE == W_EW) {
        const float* w = static_cast<const float*>(a.w) + off;
        p.w0 = ok ? *reinterpret_cast<const uint4*>(w) : z;
        p.w1 = ok ? *reinterpret_cast<const uint4*>(w + 4) : z;
    }
    if constexpr (PASS == P_GK && !F32) {
        const float4 zf = make_float4(0.f, 0.f, 0.f, 0.f);
        p.rdr0 = ok ? *reinterpret_cast<const float4*>(a.rdr + off) : zf;
        p.rdr1 = ok ? *reinterpret_cast<const float4*>(a.rdr + off + 4) : zf;
    }
}

DEVINL void st8(float* dst, const float (&f)[8]) {
    *reinterpret_cast<float4*>(dst) = make_float4(f[0], f[1], f[2], f[3]);
    *reinterpret_cast<float4*>(dst + 4) = make_float4(f[4], f[5], f[6], f[7]);
}
DEVINL void ld8f(const float* src, float (&f)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(src);
    const float4 b = *reinterpret_cast<const float4*>(src + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}

// registers -> LDS (fp32), plus the per-step scalar `dot`
template <int PASS, int WMODE, bool F32, bool TWO>
DEVINL void commit(Smem<PASS>& S, const Staged<F32>& p, const Args& a, int c0, int st, int sj) {
    const bool ok = (c0 + st) < a.T;
    float fr[8], fk[8], fv[8], fg[8];
    widen8<F32>(p.r, fr);
    widen8<F32>(p.k, fk);
    st8(&S.r[st][sj], fr);
    st8(&S.k[st][sj], fk);
    if constexpr (PASS != P_GV) { widen8<F32>(p.v, fv); st8(&S.v[st][sj], fv); }
    if constexpr (PASS != P_FWD) { widen8<F32>(p.g, fg); st8(&S.g[st][sj], fg); }
    if constexpr (WMODE != W_HEAD) {
        float fw[8], dec[8];
        if constexpr (WMODE == W_RAW) {
            unpack8(p.w0, fw);
#pragma unroll
            for (int e = 0; e < 8; ++e) fw[e] = -__expf(fw[e]);       // d(log decay): -exp(w_raw)
        } else {
            fw[0] = __uint_as_float(p.w0.x); fw[1] = __uint_as_float(p.w0.y);
            fw[2] = __uint_as_float(p.w0.z); fw[3] = __uint_as_float(p.w0.w);
            fw[4] = __uint_as_float(p.w1.x); fw[5] = __uint_as_float(p.w1.y);
            fw[6] = __uint_as_float(p.w1.z); fw[7] = __uint_as_float(p.w1.w);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) dec[e] = ok ? __expf(fw[e]) : 1.0f;  // rows past T leave the state alone
        st8(&S.w[st][sj], dec);
        if constexpr (PASS == P_GK) {
            // the factor of the decay gradient; zero once the decay is below e^-30, where the true gradient has vanished and
            // the factor would only amplify the rounding noise of G (the original kernel gives an exact zero there too)
#pragma unroll
            for (int e = 0; e < 8; ++e) fw[e] = fw[e] < -30.0f ? 0.f : fw[e];
            st8(&S.f[st][sj], fw);
        }
    }
    if constexpr (PASS == P_GK && !F32) {
        *reinterpret_cast<float4*>(&S.rdr[st][sj]) = p.rdr0;
        *reinterpret_cast<float4*>(&S.rdr[st][sj + 4]) = p.rdr1;
    }
    float d = 0.f;
    if constexpr (PASS == P_FWD || PASS == P_GV) {
#pragma unroll
        for (int e = 0; e < 8; ++e) d = fmaf(fr[e] * S.u[sj + e], fk[e], d);   // sum_j u r k
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) d = fmaf(fv[e], fg[e], d);                 // sum_i v gy
    }
    d = group_sum<8>(d);
    if ((threadIdx.x & 7) == 0) S.dot[st] = d;
    if constexpr (TWO) {
        // the bonus (u[j] + u2[i]) splits into the one-sided term above and a second scalar per step
        float d2 = 0.f;
        if constexpr (PASS == P_FWD || PASS == P_GV) {
#pragma unroll
            for (int e = 0; e < 8; ++e) d2 = fmaf(fr[e], fk[e], d2);                   // sum_j r k
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) d2 = fmaf(fv[e] * S.u2[sj + e], fg[e], d2);    // sum_i u2 v gy
        }
        d2 = group_sum<8>(d2);
        if ((threadIdx.x & 7) == 0) S.dot2[st] = d2;
        if constexpr (PASS == P_GR) {
            float d3 = 0.f, g2[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                d3 = fmaf(fr[e], fk[e], d3);                                           // sum_j r k, for gu2
                g2[e] = fg[e] * S.w2[sj + e];                                          // w2[i] gy[i], for gw
            }
            d3 = group_sum<8>(d3);
            if ((threadIdx.x & 7) == 0) S.dot3[st] = d3;
            st8(&S.w[st][sj], g2);                         // the per-token decay rows are free in this mode
        }
    }
}

template <int PASS, int WMODE, bool F32 = false, bool TWO = false>
__global__ __launch_bounds__(NT) void wkv_sweep(const Args a) {
    static_assert(!F32 || WMODE == W_HEAD, "fp32 I/O exists for wkv5 only");
    static_assert(!TWO || F32, "the two-sided op is fp32 only, as in the reference (wkv5a_cuda_v1a2.cu:5)");
    constexpr bool REV = (PASS == P_GK || PASS == P_GV);
    constexpr bool SHAPE_F = (PASS == P_FWD || PASS == P_GV);
    __shared__ Smem<PASS> S;

    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int st = tid >> 3, sj = (tid & 7) * 8;            // staging / epilogue coordinates
    const int rowslot = q * JW + (lane & (JW - 1));         // element of a broadcast vector held by this lane
    const size_t base = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const bool stateful = a.s0 != nullptr;

    if (tid < N) S.u[tid] = load1<F32>(a.u, h * N + tid);
    if constexpr (TWO) {
        if (tid < N) {
            S.u2[tid] = load1<F32>(a.u2, h * N + tid);
            S.w2[tid] = a.w2[h * N + tid];
        }
    }

    // ---- state registers
    float St[JW];
#pragma unroll
    for (int e = 0; e < JW; ++e) St[e] = 0.f;
    if (stateful) {
        if constexpr (PASS == P_FWD) {
            const uint16_t* s = a.s0 + (bh * N + lane) * N + q * JW;        // row i = lane, JW consecutive j
            static_assert(JW == 8, "one 16-byte load per lane");
            float lo[8];
            unpack8(*reinterpret_cast<const uint4*>(s), lo);
#pragma unroll
            for (int e = 0; e < 8; ++e) St[e] = lo[e];
        } else if constexpr (PASS == P_GR) {
#pragma unroll
            for (int e = 0; e < JW; ++e) St[e] = bf2f(a.s0[(bh * N + q * JW + e) * N + lane]);
        }
    }
    // time-constant decay (wkv5)
    float w_const = 1.f;
    if constexpr (WMODE == W_HEAD) {
        const float* eew = static_cast<const float*>(a.w) + h * N;
        w_const = SHAPE_F ? eew[rowslot] : eew[lane];
    }
#pragma unroll
    for (int e = 0; e < JW; ++e) asm volatile("" : "+v"(St[e]));
    // Values loaded here are first used inside the step loop.  Left alone, the compiler waits for them there, with a
    // vmcnt(0) in every chunk that also waits for the next chunk's prefetch (issued just before the steps) and so
    // serialises load latency with compute.  Pinning them to a register now puts the wait up here, once.
    asm volatile("" : "+v"(w_const));
    // time-constant decays that vary along the in-register axis live in registers (a plain multiply instead of a
    // row-broadcast one): w[j] in shape F, and every element's w[j] * w2[i] of the two-sided op
    constexpr bool REGW = TWO || (WMODE == W_HEAD && SHAPE_F);
    float wreg[REGW ? JW : 1];
    if constexpr (TWO) {
        const float* w1 = static_cast<const float*>(a.w) + h * N;
        const float* w2 = a.w2 + h * N;
#pragma unroll
        for (int e = 0; e < JW; ++e) wreg[e] = SHAPE_F ? w1[q * JW + e] * w2[lane] : w1[lane] * w2[q * JW + e];
    } else if constexpr (REGW) {
        const float* eew = static_cast<const float*>(a.w) + h * N;
#pragma unroll
        for (int e = 0; e < JW; ++e) wreg[e] = eew[q * JW + e];
    }
    if constexpr (REGW) {
#pragma unroll
        for (int e = 0; e < JW; ++e) asm volatile("" : "+v"(wreg[e]));
    }

    float gu_acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) gu_acc[e] = 0.f;
    float P = 0.f, gw_acc = 0.f;                            // GK scan state (threads < 64)
    // fp32 I/O: the P recurrence above loses a digit per decade of T to cancellation, which bf16 outputs hide and
    // fp32 outputs do not.  GR carries Q = dS/dw instead (Q_{t+1} = S_t + w Q_t, the reference's second recurrence,
    // wkv5/run.py:249-252) and sums gw[j] = sum_t r_t[j] sum_i gy_t[i] Q_t[i,j] per lane; GK then makes gk only.
    constexpr bool DIRECT_GW = F32 && PASS == P_GR;
    constexpr bool SCAN_GW = !F32 && PASS == P_GK;
    float Q[DIRECT_GW ? JW : 1];
#pragma unroll
    for (int e = 0; e < (DIRECT_GW ? JW : 1); ++e) Q[e] = 0.f;
    // two-sided: with gW[i,j] = sum_t gy_t[i] r_t[j] Q_t[i,j], gw1[j] = sum_i w2[i] gW[i,j] stays a per-lane sum
    // (the broadcast operand becomes w2[i] gy[i]); gw2[i] = sum_j w1[j] gW[i,j] is kept per state element in A and
    // summed over the lanes once, at the end.
    constexpr bool GW2 = TWO && PASS == P_GR;
    float A[GW2 ? JW : 1], gu2_acc[8];
#pragma unroll
    for (int e = 0; e < (GW2 ? JW : 1); ++e) A[e] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) gu2_acc[e] = 0.f;

    const int nchunks = (a.T + TC - 1) / TC;
    const bool stager = tid < NSTAGE;                       // whole waves
    Staged<F32> pre;
    if (stager) prefetch<PASS, WMODE, F32>(pre, a, base, (REV ? nchunks - 1 : 0) * TC, st, sj);
    __syncthreads();                                        // S.u (u2, w2) visible

    for (int ci = 0; ci < nchunks; ++ci) {
        const int c0 = (REV ? nchunks - 1 - ci : ci) * TC;
        __syncthreads();                                    // previous epilogue is done with LDS
        if (stager) commit<PASS, WMODE, F32, TWO>(S, pre, a, c0, st, sj);
        __syncthreads();
        if (stager && ci + 1 < nchunks) prefetch<PASS, WMODE, F32>(pre, a, base, (REV ? nchunks - 2 - ci : ci + 1) * TC, st, sj);

        // ---- TC sequential steps
#pragma unroll 4
        for (int tt = 0; tt < TC; ++tt) {
            const int t = REV ? TC - 1 - tt : tt;
            float acc = 0.f;
            if constexpr (SHAPE_F) {
                const float av = (PASS == P_FWD) ? S.r[t][rowslot] : S.k[t][rowslot];
                const float bv = (PASS == P_FWD) ? S.k[t][rowslot] : S.r[t][rowslot];
                const float wv = (WMODE == W_HEAD) ? w_const : S.w[t][rowslot];
                const float x = (PASS == P_FWD) ? S.v[t][lane] : S.g[t][lane];
                static_for<JW>([&](auto J) {
                    fmac_bc<decltype(J)::value>(acc, av, St[decltype(J)::value]);
                    if constexpr (REGW) St[decltype(J)::value] *= wreg[decltype(J)::value];
                    else mul_bc<decltype(J)::value>(St[decltype(J)::value], wv);
                    fmac_bc<decltype(J)::value>(St[decltype(J)::value], bv, x);
                });
            } else {
                const float av = (PASS == P_GR) ? S.g[t][rowslot] : S.v[t][rowslot];
                const float xv = (PASS == P_GR) ? S.v[t][rowslot] : S.g[t][rowslot];
                const float bl = (PASS == P_GR) ? S.k[t][lane] : S.r[t][lane];
                const float wl = (WMODE == W_HEAD) ? w_const : S.w[t][lane];
                float acc2 = 0.f, g2 = 0.f, w1r = 0.f;
                if constexpr (GW2) {
                    g2 = S.w[t][rowslot];                       // w2[i] gy[i]
                    w1r = w_const * S.r[t][lane];               // w1[j] r[j]
                }
                static_for<JW>([&](auto I) {
                    constexpr int i = decltype(I)::value;
                    const float dec = TWO ? wreg[TWO ? i : 0] : wl;
                    fmac_bc<i>(acc, av, St[i]);
                    if constexpr (DIRECT_GW) {
                        fmac_bc<i>(acc2, GW2 ? g2 : av, Q[i]);
                        if constexpr (GW2) fmac_bc<i>(A[i], av, Q[i] * w1r);
                        Q[i] = fmaf(Q[i], dec, St[i]);
                    }
                    St[i] *= dec;
                    fmac_bc<i>(St[i], xv, bl);
                });
                if constexpr (DIRECT_GW) gw_acc = fmaf(S.r[t][lane], acc2, gw_acc);
            }
            S.part[q][t][lane] = acc;
        }
        __syncthreads();

        // ---- chunk epilogue: thread (st, sj..sj+7) of the staging waves
        const bool ok = stager && (c0 + st) < a.T;
        const int es = stager ? st : 0;                       // the other waves only keep the barriers company
        const size_t off = base + static_cast<size_t>(c0 + es) * a.C + sj;
        float sum[8];
        ld8f(&S.part[0][es][sj], sum);
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            float p1[8];
            ld8f(&S.part[w][es][sj], p1);
#pragma unroll
            for (int e = 0; e < 8; ++e) sum[e] += p1[e];
        }
        const float dot = S.dot[es];
        float out[8];
        if constexpr (PASS == P_FWD) {
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] = fmaf(S.v[es][sj + e], TWO ? fmaf(S.u2[sj + e], S.dot2[es], dot) : dot, sum[e]);
            if (ok) store8<F32>(a.y, off, out);
        } else if constexpr (PASS == P_GV) {
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] = fmaf(S.g[es][sj + e], TWO ? fmaf(S.u2[sj + e], S.dot2[es], dot) : dot, sum[e]);
            if (ok) store8<F32>(a.gv, off, out);
        } else if constexpr (PASS == P_GR) {
            float rdr[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float rr = S.r[es][sj + e], kk = S.k[es][sj + e];
                out[e] = TWO ? fmaf(kk, fmaf(S.u[sj + e], dot, S.dot2[es]), sum[e]) : fmaf(S.u[sj + e] * kk, dot, sum[e]);
                rdr[e] = rr * sum[e];
                gu_acc[e] = fmaf(rr * kk, dot, gu_acc[e]);
                if constexpr (TWO) gu2_acc[e] = fmaf(S.v[es][sj + e] * S.g[es][sj + e], S.dot3[es], gu2_acc[e]);
            }
            if (ok) {
                store8<F32>(a.gr, off, out);
                if constexpr (!F32) {
                    *reinterpret_cast<float4*>(a.rdr + off) = make_float4(rdr[0], rdr[1], rdr[2], rdr[3]);
                    *reinterpret_cast<float4*>(a.rdr + off + 4) = make_float4(rdr[4], rdr[5], rdr[6], rdr[7]);
                }
            }
        } else {  // P_GK
            float kdk[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                out[e] = TWO ? fmaf(S.r[es][sj + e], fmaf(S.u[sj + e], dot, S.dot2[es]), sum[e])
                             : fmaf(S.u[sj + e] * S.r[es][sj + e], dot, sum[e]);
                kdk[e] = S.k[es][sj + e] * sum[e];
            }
            if (ok) store8<F32>(a.gk, off, out);
            if constexpr (SCAN_GW) {
                if (stager) st8(&S.k[st][sj], kdk);              // k is no longer needed: keep k*dk' there
                __syncthreads();
                if (tid < N) {                                   // per-channel scan over the chunk, t descending
                    for (int t = TC - 1; t >= 0; --t) {
                        float G = P - S.k[t][tid];
                        if (!stateful && (c0 + t) == 0) G = 0.f; // S_0 = 0: exact zero, as the reference leaves it
                        P = G + S.rdr[t][tid];
                        if constexpr (WMODE == W_HEAD) gw_acc += G;
                        else S.part[0][t][tid] = S.f[t][tid] * G;
                    }
                }
                if constexpr (WMODE != W_HEAD) {
                    __syncthreads();
                    ld8f(&S.part[0][es][sj], out);
                    if (ok) store8<F32>(a.gw, off, out);
                }
            }
        }
    }

    // ---- tails
    if constexpr (PASS == P_GR) {
        __syncthreads();
        if (stager) st8(&S.part[0][st][sj], gu_acc);
        __syncthreads();
        if (tid < N) {
            float s = 0.f;
#pragma unroll 8
            for (int t = 0; t < TC; ++t) s += S.part[0][t][tid];
            store1<F32>(a.gu, static_cast<size_t>(b) * a.C + h * N + tid, s);
        }
        if constexpr (DIRECT_GW) {
            __syncthreads();
            S.part[q][0][lane] = gw_acc;
            __syncthreads();
            if (tid < N) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) s += S.part[w][0][tid];
                const float eew = static_cast<const float*>(a.w)[h * N + tid];   // d eew / d w_raw = eew * ew
                store1<F32>(a.gw, static_cast<size_t>(b) * a.C + h * N + tid, a.ew_head[h * N + tid] * eew * s);
            }
        }
        if constexpr (TWO) {
            __syncthreads();
            if (stager) st8(&S.part[0][st][sj], gu2_acc);
            __syncthreads();
            if (tid < N) {
                float s = 0.f;
#pragma unroll 8
                for (int t = 0; t < TC; ++t) s += S.part[0][t][tid];
                store1<F32>(a.gu2, static_cast<size_t>(b) * a.C + h * N + tid, s);
            }
            __syncthreads();
#pragma unroll
            for (int e = 0; e < JW; ++e) S.part[q][e][lane] = A[GW2 ? e : 0];     // [wave][i within the wave][j]
            __syncthreads();
            if (tid < N) {                                                        // tid = i
                float s = 0.f;
                for (int j = 0; j < N; ++j) s += S.part[tid / JW][tid % JW][(j + tid) & (N - 1)];
                store1<F32>(a.gw2, static_cast<size_t>(b) * a.C + h * N + tid, a.ew2_head[h * N + tid] * a.w2[h * N + tid] * s);
            }
        }
    }
    if constexpr (PASS == P_GK) {
        if constexpr (WMODE == W_HEAD && SCAN_GW) {
            if (tid < N) {
                const float f = a.ew_head[h * N + tid];
                store1<F32>(a.gw, static_cast<size_t>(b) * a.C + h * N + tid, (f < -30.0f ? 0.f : f) * gw_acc);
            }
        }
        if (a.gs != nullptr) {
#pragma unroll
            for (int e = 0; e < JW; ++e) a.gs[(bh * N + q * JW + e) * N + lane] = f2bf(St[e]);
        }
    }
}

// ----------------------------------------------------------------------------------------------------------------------
// Head sizes other than 64 (the reference builds its kernels with -D_N_=HEAD_SIZE: wkv5_bf16/run.py:21 ships 128, the
// self-checks of wkv5/run.py, wkv6/run.py and wkv6_state/run.py use 2, 4 and 8).  One workgroup per (batch, head).  A row
// of the state (S[i][.] in FWD and GV, S[.][j] in GR and GK) is kept in the registers of PARTS adjacent lanes, EL elements
// each, so every sum of the recurrence is a private loop over LDS-broadcast vectors plus one or two cross-lane adds.
// Same passes, formulas, rounding points and workspace as the sweeps above; hn (the head size, 1..NP) is a run-time
// value, NP the padded size the registers are unrolled for.
constexpr int GTC = 16;          // time steps per staged chunk

// The step loops below are unrolled over a thread's part of a state row.  Left alone, the compiler issues all of the LDS
// reads first and the arithmetic afterwards, which keeps three more copies of the row alive in registers.  Passing the
// running sum and the eight state elements just updated through an empty asm statement with a memory clobber ends the
// live ranges of a block's operands before the next block's reads are issued.
DEVINL void row_fence(float& acc, float* s8) {
    asm volatile("" : "+v"(acc), "+v"(s8[0]), "+v"(s8[1]), "+v"(s8[2]), "+v"(s8[3]), "+v"(s8[4]), "+v"(s8[5]), "+v"(s8[6]), "+v"(s8[7]) : : "memory");
}

template <int NP, int PARTS> struct RowGeom {
    static constexpr int EL = NP / PARTS;                    // state elements per thread
    static constexpr int SLOT = EL + (PARTS > 1 ? 4 : 0);    // a part's slice of a staged vector; the 16-byte skew keeps the
    static constexpr int LEN = PARTS * SLOT;                 // PARTS broadcast reads of a wave on different banks
    static constexpr int NTHREADS = NP * PARTS < 64 ? 64 : NP * PARTS;
    static_assert(EL % 8 == 0, "row_fence takes blocks of eight");
    static __device__ __forceinline__ int at(int n) { return (n / EL) * SLOT + n % EL; }   // where channel n of a vector sits
};

// staged vectors of one chunk; the ones a pass does not use shrink to one row
template <int NP, int PARTS, int PASS, bool F32, bool TWO> struct SmemRows {
    static constexpr int LEN = RowGeom<NP, PARTS>::LEN;
    static constexpr bool kF = (PASS == P_GK && !F32) || (TWO && PASS == P_GR);     // gw factor, or w2[i] gy[i]
    alignas(16) float r[GTC][LEN], k[GTC][LEN], w[GTC][LEN];
    alignas(16) float v[PASS != P_GV ? GTC : 1][LEN], g[PASS != P_FWD ? GTC : 1][LEN];
    alignas(16) float f[kF ? GTC : 1][LEN], rdr[(PASS == P_GK && !F32) ? GTC : 1][LEN];
    float dot[GTC], dot2[TWO ? GTC : 1], dot3[TWO ? GTC : 1];
    alignas(16) float u[LEN], u2[TWO ? LEN : 4], w2[TWO ? LEN : 4];
};

// sum over the PARTS adjacent lanes that share a row; every one of them gets the total
template <int PARTS> DEVINL float parts_sum(float x) {
    if constexpr (PARTS >= 2) x += __shfl_xor(x, 1, 64);
    if constexpr (PARTS >= 4) x += __shfl_xor(x, 2, 64);
    if constexpr (PARTS >= 8) x += __shfl_xor(x, 4, 64);
    static_assert(PARTS == 1 || PARTS == 2 || PARTS == 4 || PARTS == 8, "adjacent lanes");
    return x;
}

template <int NP, int PARTS, int PASS, int WMODE, bool F32, bool TWO = false>
__global__ __launch_bounds__((RowGeom<NP, PARTS>::NTHREADS)) void wkv_rows(const Args a, const int hn) {
    static_assert(!F32 || WMODE == W_HEAD, "fp32 I/O exists for wkv5 only");
    static_assert(!TWO || F32, "the two-sided op is fp32 only");
    using G = RowGeom<NP, PARTS>;
    constexpr int EL = G::EL, SLOT = G::SLOT;
    constexpr bool REV = (PASS == P_GK || PASS == P_GV);
    constexpr bool ROW_I = (PASS == P_FWD || PASS == P_GV);     // row = value channel, registers = key channels
    constexpr bool DIRECT_GW = F32 && PASS == P_GR;             // as in wkv_sweep: the fp32 op carries Q = dS/dw
    constexpr bool SCAN_GW = !F32 && PASS == P_GK;
    __shared__ SmemRows<NP, PARTS, PASS, F32, TWO> S;

    const int tid = threadIdx.x;
    const int row = tid / PARTS, part = tid % PARTS;            // threads beyond NP * PARTS (NP * PARTS < 64) only idle
    const bool in_rows = row < NP;
    const int rrow = in_rows ? row : 0;                         // a valid row to read for idle threads
    const bool live = in_rows && row < hn;                      // this thread's row is a channel of the head
    const bool writer = live && part == 0;
    const int own = G::at(rrow);                                // where this row's element of a staged vector sits
    const int sl = part * SLOT;                                 // where this thread's slice of a staged vector starts
    const int o0 = part * EL;                                   // first in-register channel of this thread
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const size_t base = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(h) * hn;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const bool stateful = a.s0 != nullptr;
    // the staging role: thread (channel cn, group sg) moves SPT steps of channel cn in every chunk
    constexpr int SG = G::NTHREADS / NP, SPT = GTC / SG;
    static_assert(SG * NP == G::NTHREADS && SPT * SG == GTC && SPT >= 1, "the workgroup tiles a chunk");
    const int cn = tid % NP, t_first = (tid / NP) * SPT;
    const bool chan = cn < hn;
    const int cat = G::at(cn);

    if (tid < NP) {
        S.u[cat] = chan ? load1<F32>(a.u, h * hn + cn) : 0.f;
        if constexpr (TWO) {
            S.u2[cat] = chan ? load1<F32>(a.u2, h * hn + cn) : 0.f;
            S.w2[cat] = chan ? a.w2[h * hn + cn] : 1.f;
        }
    }
    const float w_chan = (WMODE == W_HEAD && chan) ? static_cast<const float*>(a.w)[h * hn + cn] : 1.f;     // stager's channel
    const float w_row = (WMODE == W_HEAD && live) ? static_cast<const float*>(a.w)[h * hn + row] : 1.f;     // this row's channel
    float St[EL], Q[DIRECT_GW ? EL : 1];
#pragma unroll
    for (int e = 0; e < EL; ++e) St[e] = 0.f;
#pragma unroll
    for (int e = 0; e < (DIRECT_GW ? EL : 1); ++e) Q[e] = 0.f;
    // two-sided: state element [i][j] decays by w1[j] w2[i]; A collects gw2 per state element
    constexpr bool GW2 = TWO && PASS == P_GR;
    float A[GW2 ? EL : 1];
    float u2_row = 0.f, w2_row = 1.f, gu2_acc = 0.f;
    if constexpr (TWO) {
        u2_row = live ? load1<F32>(a.u2, h * hn + row) : 0.f;
        w2_row = live ? a.w2[h * hn + row] : 1.f;
#pragma unroll
        for (int e = 0; e < (GW2 ? EL : 1); ++e) A[e] = 0.f;
    }
    if (stateful && live) {
        if constexpr (PASS == P_FWD) {
#pragma unroll
            for (int e = 0; e < EL; ++e) if (o0 + e < hn) St[e] = bf2f(a.s0[(bh * hn + row) * hn + o0 + e]);
        } else if constexpr (PASS == P_GR) {
#pragma unroll
            for (int e = 0; e < EL; ++e) if (o0 + e < hn) St[e] = bf2f(a.s0[(bh * hn + o0 + e) * hn + row]);
        }
    }
    float gu_acc = 0.f, gw_acc = 0.f, P = 0.f;

    const int nchunks = (a.T + GTC - 1) / GTC;
    // Inputs of a chunk are fetched into registers, unconverted, while the steps of the chunk before run, and go to LDS at
    // the top of their own chunk: the first use, and with it the compiler's wait, comes after the step loop.
    using Elem = typename std::conditional<F32, float, uint16_t>::type;
    Elem pre_r[SPT], pre_k[SPT], pre_v[SPT], pre_g[SPT];
    uint32_t pre_w[SPT];
    float pre_d[SPT];
    auto widen = [](Elem x) __attribute__((always_inline)) -> float {
        if constexpr (F32) return x; else return bf2f(x);
    };
    auto prefetch = [&](const int c0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < SPT; ++i) {
            const int tg = c0 + t_first + i;
            const bool ok = chan && tg < a.T;
            const size_t off = base + static_cast<size_t>(ok ? tg : 0) * a.C + (chan ? cn : 0);   // an address that exists
            pre_r[i] = reinterpret_cast<const Elem*>(a.r)[off];
            pre_k[i] = reinterpret_cast<const Elem*>(a.k)[off];
            if constexpr (PASS != P_GV) pre_v[i] = reinterpret_cast<const Elem*>(a.v)[off];
            if constexpr (PASS != P_FWD) pre_g[i] = reinterpret_cast<const Elem*>(a.gy)[off];
            if constexpr (WMODE == W_RAW) pre_w[i] = static_cast<const uint16_t*>(a.w)[off];
            if constexpr (WMODE == W_EW) pre_w[i] = static_cast<const uint32_t*>(a.w)[off];
            if constexpr (SCAN_GW) pre_d[i] = a.rdr[off];
        }
    };
    prefetch((REV ? nchunks - 1 : 0) * GTC);
    for (int ci = 0; ci < nchunks; ++ci) {
        const int c0 = (REV ? nchunks - 1 - ci : ci) * GTC;
        __syncthreads();                                        // the previous chunk is done with LDS
#pragma unroll
        for (int i = 0; i < SPT; ++i) {                         // registers (fetched during the previous chunk's steps) -> LDS
            const int t = t_first + i;
            const bool ok = chan && (c0 + t) < a.T;             // rows past T and padded channels: no input, no decay
            S.r[t][cat] = ok ? widen(pre_r[i]) : 0.f;
            S.k[t][cat] = ok ? widen(pre_k[i]) : 0.f;
            if constexpr (PASS != P_GV) S.v[t][cat] = ok ? widen(pre_v[i]) : 0.f;
            if constexpr (PASS != P_FWD) S.g[t][cat] = ok ? widen(pre_g[i]) : 0.f;
            if constexpr (WMODE != W_HEAD) {
                float ew = 0.f;
                if (ok) ew = (WMODE == W_RAW) ? -__expf(bf2f(static_cast<uint16_t>(pre_w[i]))) : __uint_as_float(pre_w[i]);
                S.w[t][cat] = ok ? __expf(ew) : 1.0f;
                if constexpr (PASS == P_GK) S.f[t][cat] = ew < -30.0f ? 0.f : ew;    // see wkv_sweep's commit()
            } else {
                S.w[t][cat] = ok ? w_chan : 1.0f;
            }
            if constexpr (SCAN_GW) S.rdr[t][cat] = ok ? pre_d[i] : 0.f;
            if constexpr (GW2) S.f[t][cat] = ok ? widen(pre_g[i]) * S.w2[cat] : 0.f;    // w2[i] gy[i]: the operand of gw1
        }
        __syncthreads();
        if (tid < GTC) {                                        // the scalar of each step: sum_j u r k, or sum_i v gy
            float d = 0.f, d2 = 0.f, d3 = 0.f;
            for (int n = 0; n < NP; ++n) {
                const int at = G::at(n);
                d = ROW_I ? fmaf(S.r[tid][at] * S.u[at], S.k[tid][at], d) : fmaf(S.v[tid][at], S.g[tid][at], d);
                if constexpr (TWO) {                            // the bonus u1[j] + u2[i] needs a second scalar, gu2 a third
                    d2 = ROW_I ? fmaf(S.r[tid][at], S.k[tid][at], d2) : fmaf(S.v[tid][at] * S.u2[at], S.g[tid][at], d2);
                    if constexpr (PASS == P_GR) d3 = fmaf(S.r[tid][at], S.k[tid][at], d3);
                }
            }
            S.dot[tid] = d;
            if constexpr (TWO) { S.dot2[tid] = d2; S.dot3[tid] = d3; }
        }
        __syncthreads();
        if constexpr (GW2) {                                    // gu2[i] = sum_t v_i gy_i sum_j r_j k_j, by the staging threads
#pragma unroll
            for (int i = 0; i < SPT; ++i) gu2_acc = fmaf(S.v[t_first + i][cat] * S.g[t_first + i][cat], S.dot3[t_first + i], gu2_acc);
        }
        if (ci + 1 < nchunks) prefetch((REV ? nchunks - 2 - ci : ci + 1) * GTC);

#pragma unroll 1
        for (int tt = 0; tt < GTC; ++tt) {
            const int t = REV ? GTC - 1 - tt : tt, tg = c0 + t;
            const bool ok = writer && tg < a.T;
            const size_t off = base + static_cast<size_t>(tg) * a.C + row;
            const float dot = S.dot[t];
            float acc = 0.f, acc2 = 0.f;
            if constexpr (ROW_I) {
                const float x = (PASS == P_FWD) ? S.v[t][own] : S.g[t][own];
#pragma unroll
                for (int e = 0; e < EL; ++e) {
                    const float av = (PASS == P_FWD) ? S.r[t][sl + e] : S.k[t][sl + e];
                    const float bv = (PASS == P_FWD) ? S.k[t][sl + e] : S.r[t][sl + e];
                    acc = fmaf(av, St[e], acc);
                    St[e] = fmaf(St[e], TWO ? S.w[t][sl + e] * w2_row : S.w[t][sl + e], bv * x);
                    if (e % 8 == 7) row_fence(acc, &St[e - 7]);
                }
                acc = parts_sum<PARTS>(acc);
                const float bonus = TWO ? fmaf(u2_row, S.dot2[t], dot) : dot;
                if (ok) store1<F32>(PASS == P_FWD ? a.y : a.gv, off, fmaf(x, bonus, acc));
            } else {
                const float bl = (PASS == P_GR) ? S.k[t][own] : S.r[t][own];
                const float wl = S.w[t][own];
                const float w1r = GW2 ? wl * S.r[t][own] : 0.f;                 // w1[j] r[j]
#pragma unroll
                for (int e = 0; e < EL; ++e) {
                    const float av = (PASS == P_GR) ? S.g[t][sl + e] : S.v[t][sl + e];
                    const float xv = (PASS == P_GR) ? S.v[t][sl + e] : S.g[t][sl + e];
                    const float de = TWO ? wl * S.w2[sl + e] : wl;
                    acc = fmaf(av, St[e], acc);
                    if constexpr (DIRECT_GW) {
                        acc2 = fmaf(GW2 ? S.f[t][sl + e] : av, Q[e], acc2);
                        if constexpr (GW2) A[e] = fmaf(av, Q[e] * w1r, A[e]);
                        Q[e] = fmaf(Q[e], de, St[e]);
                    }
                    St[e] = fmaf(St[e], de, xv * bl);
                    if (e % 8 == 7) {
                        row_fence(acc, &St[e - 7]);
                        if constexpr (DIRECT_GW) row_fence(acc2, &Q[e - 7]);
                        if constexpr (GW2) row_fence(acc, &A[e - 7]);
                    }
                }
                acc = parts_sum<PARTS>(acc);
                if constexpr (DIRECT_GW) acc2 = parts_sum<PARTS>(acc2);
                const float rr = S.r[t][own], kk = S.k[t][own], uu = S.u[own];
                if constexpr (PASS == P_GR) {
                    gu_acc = fmaf(rr * kk, dot, gu_acc);
                    if constexpr (DIRECT_GW) gw_acc = fmaf(rr, acc2, gw_acc);
                    if (ok) {
                        store1<F32>(a.gr, off, TWO ? fmaf(kk, fmaf(uu, dot, S.dot2[t]), acc) : fmaf(uu * kk, dot, acc));
                        if constexpr (!F32) a.rdr[off] = rr * acc;
                    }
                } else {
                    if (ok) store1<F32>(a.gk, off, TWO ? fmaf(rr, fmaf(uu, dot, S.dot2[t]), acc) : fmaf(uu * rr, dot, acc));
                    if constexpr (SCAN_GW) {
                        float Gt = P - kk * acc;
                        if (!stateful && tg == 0) Gt = 0.f;     // S_0 = 0: exact zero, as the reference leaves it
                        P = Gt + S.rdr[t][own];
                        if constexpr (WMODE == W_HEAD) gw_acc += Gt;
                        else if (ok) store1<F32>(a.gw, off, S.f[t][own] * Gt);
                    }
                }
            }
        }
    }

    const size_t pc = static_cast<size_t>(b) * a.C + static_cast<size_t>(h) * hn + row;
    if constexpr (PASS == P_GR) {
        if (writer) {
            store1<F32>(a.gu, pc, gu_acc);
            if constexpr (DIRECT_GW) store1<F32>(a.gw, pc, a.ew_head[h * hn + row] * w_row * gw_acc);     // d eew / d w_raw = eew * ew
        }
        if constexpr (GW2) {
            // gu2: the staging groups' partial sums, one row of LDS per group
            __syncthreads();
            S.r[tid / NP][cat] = gu2_acc;
            __syncthreads();
            if (tid < NP && chan) {
                float sum = 0.f;
                for (int q = 0; q < SG; ++q) sum += S.r[q][cat];
                store1<F32>(a.gu2, static_cast<size_t>(b) * a.C + static_cast<size_t>(h) * hn + cn, sum);
            }
            // gw2[i] = ew2[i] w2[i] sum_j A_j[i]: rows j pass through LDS sixteen at a time and are added in order
            float tot = 0.f;
            for (int r0 = 0; r0 < NP; r0 += GTC) {
                __syncthreads();
                if (in_rows && row >= r0 && row < r0 + GTC) {
#pragma unroll
                    for (int e = 0; e < EL; ++e) S.k[row - r0][sl + e] = A[GW2 ? e : 0];
                }
                __syncthreads();
                if (tid < NP)
                    for (int q = 0; q < (NP < GTC ? NP : GTC); ++q) tot += S.k[q][cat];
            }
            if (tid < NP && chan)
                store1<F32>(a.gw2, static_cast<size_t>(b) * a.C + static_cast<size_t>(h) * hn + cn, a.ew2_head[h * hn + cn] * a.w2[h * hn + cn] * tot);
        }
    }
    if constexpr (PASS == P_GK) {
        if constexpr (WMODE == W_HEAD && SCAN_GW) {
            if (writer) {
                const float f = a.ew_head[h * hn + row];
                store1<F32>(a.gw, pc, (f < -30.0f ? 0.f : f) * gw_acc);
            }
        }
        if (a.gs != nullptr && live) {
#pragma unroll
            for (int e = 0; e < EL; ++e) if (o0 + e < hn) a.gs[(bh * hn + o0 + e) * hn + row] = f2bf(St[e]);
        }
    }
}

constexpr int MAX_HEAD = 128;

template <int PASS, int WMODE, bool F32, bool TWO = false> void launch_rows(hipStream_t st, int B, const Args& a) {
    const int hn = a.C / a.H;
    const dim3 grid(B * a.H);
    if (hn <= 8) hipLaunchKernelGGL((wkv_rows<8, 1, PASS, WMODE, F32, TWO>), grid, dim3(RowGeom<8, 1>::NTHREADS), 0, st, a, hn);
    else if (hn <= 32) hipLaunchKernelGGL((wkv_rows<32, 2, PASS, WMODE, F32, TWO>), grid, dim3(RowGeom<32, 2>::NTHREADS), 0, st, a, hn);
    else if (hn <= 64) hipLaunchKernelGGL((wkv_rows<64, 4, PASS, WMODE, F32, TWO>), grid, dim3(RowGeom<64, 4>::NTHREADS), 0, st, a, hn);
    else if constexpr (TWO) hipLaunchKernelGGL((wkv_rows<128, 8, PASS, WMODE, F32, TWO>), grid, dim3(RowGeom<128, 8>::NTHREADS), 0, st, a, hn);
    else hipLaunchKernelGGL((wkv_rows<128, 4, PASS, WMODE, F32, TWO>), grid, dim3(RowGeom<128, 4>::NTHREADS), 0, st, a, hn);
}

// The chunked matrix-core kernels serve all three decay conventions; the sequential sweeps remain as the second algorithm.
// They address one batch row with 32-bit byte offsets (up to 4 bytes per element), so rows of 2^30 elements or more
// take the sweeps.
bool use_chunked(const Args& a, unsigned flags) { return !(flags & RWKV_FLAG_SWEEPS) && static_cast<long long>(a.T) * a.C < (1LL << 30); }

// pass mask of a flags word: no bit set means every pass
unsigned passes_of(unsigned flags) { return (flags & RWKV_PASS_ALL) ? (flags & RWKV_PASS_ALL) : RWKV_PASS_ALL; }

template <int WMODE> int launch_fwd(hipStream_t st, int B, const Args& a, unsigned flags) {
    if (a.C != a.H * N) {                              // another head size: the row-per-thread kernels
        launch_rows<P_FWD, WMODE, false>(st, B, a);
        return launch_status();
    }
    if (use_chunked(a, flags))
        return launch_wkv6_fwd_chunk(st, WMODE, B, a.T, a.C, a.H, a.r, a.k, a.v, a.w, a.u, a.s0, a.y);
    hipLaunchKernelGGL((wkv_sweep<P_FWD, WMODE>), dim3(B * a.H), dim3(NT), 0, st, a);
    return launch_status();
}

// GR and GV are independent; GK consumes GR's workspace.  All three run on `st` in order.
// `passes` is a bit mask (RWKV_PASS_*) so that a profiler can time one kernel at a time.
template <int WMODE> int launch_bwd(hipStream_t st, int B, const Args& a, unsigned flags) {
    const unsigned passes = passes_of(flags);
    if (a.C != a.H * N) {                              // another head size: GR and GV are independent, GK reads GR's workspace
        if (passes & RWKV_PASS_GR) launch_rows<P_GR, WMODE, false>(st, B, a);
        if (passes & RWKV_PASS_GV) launch_rows<P_GV, WMODE, false>(st, B, a);
        if (passes & RWKV_PASS_GK) launch_rows<P_GK, WMODE, false>(st, B, a);
        return launch_status();
    }
    const bool chunked = use_chunked(a, flags);
    const void* w = (WMODE == W_HEAD) ? static_cast<const void*>(a.ew_head) : a.w;   // wkv5: the log decay
    if ((passes & RWKV_PASS_GR) && chunked) {
        if (int e = launch_wkv6_bwd_a_chunk(st, WMODE, B, a.T, a.C, a.H, a.r, a.k, a.v, w, a.u, a.s0, a.gy, a.gr, a.gu, a.rdr)) return e;
    } else if (passes & RWKV_PASS_GR) hipLaunchKernelGGL((wkv_sweep<P_GR, WMODE>), dim3(B * a.H), dim3(NT), 0, st, a);
    if (chunked) {
        // the chunked second sweep produces gk, gv, gw (and gs) together: it runs for GK, and GV alone is a no-op
        if (passes & RWKV_PASS_GK)
            if (int e = launch_wkv6_bwd_b_chunk(st, WMODE, B, a.T, a.C, a.H, a.r, a.k, a.v, w, a.u, a.s0, a.gy, a.gk, a.gv, a.gw, a.gs, a.rdr)) return e;
        return launch_status();
    }
    if (passes & RWKV_PASS_GV) hipLaunchKernelGGL((wkv_sweep<P_GV, WMODE>), dim3(B * a.H), dim3(NT), 0, st, a);
    if (passes & RWKV_PASS_GK) hipLaunchKernelGGL((wkv_sweep<P_GK, WMODE>), dim3(B * a.H), dim3(NT), 0, st, a);
    return launch_status();
}

// head size 64 takes the kernels this file and wkv6_*.hip are written for, any other size up to 128 the row kernels (wkv_rows)
int check_dims(int B, int T, int C, int H) {
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0) return RWKV_ERR_SHAPE;
    if (C % H != 0 || C / H > MAX_HEAD) return RWKV_ERR_SHAPE;
    if (static_cast<long long>(B) * H > 0x7fffffffLL) return RWKV_ERR_SHAPE;
    return RWKV_OK;
}

// r * dr' in fp32 [B,T,C], then the forward states that the first chunked sweep hands to the second every PCK chunks
// (wkv6_chunk.h): [B*H][ceil(chunks / 4)][64*64] fp32
size_t ws_bytes(int B, int T, int C, int H) {
    if (check_dims(B, T, C, H) != RWKV_OK) return 0;
    const size_t nchunks = (static_cast<size_t>(T) + 31) / 32, npck = (nchunks + 3) / 4;
    return static_cast<size_t>(B) * T * C * sizeof(float) + static_cast<size_t>(B) * H * npck * 64 * 64 * sizeof(float);
}

// ---- wrapper-side steps of WKV_5 / WKV_6 (wkv5_bf16/run.py:63-64,86-87; wkv6/run.py:169) as two small kernels
// ew = -exp(w_raw), eew = exp(ew) in fp32 from the raw bf16 decay parameter [H*N]; decay = [eew | ew]
__global__ __launch_bounds__(256) void wkv5_decay_transform(int C, const uint16_t* __restrict__ w_raw, float* __restrict__ decay) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const float ew = -expf(bf2f(w_raw[c]));
    decay[c] = expf(ew);
    decay[C + c] = ew;
}
// out[c] = bf16(sum_b float(part[b][c])) for one or two [B,C] bf16 arrays: torch.sum(x, 0) of the per-batch partials
__global__ __launch_bounds__(256) void bf16_batch_sum(int B, int C, const uint16_t* __restrict__ p0, uint16_t* __restrict__ o0,
                                                      const uint16_t* __restrict__ p1, uint16_t* __restrict__ o1) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    float a = 0.f, b2 = 0.f;
    for (int b = 0; b < B; ++b) {
        a += bf2f(p0[static_cast<size_t>(b) * C + c]);
        if (p1 != nullptr) b2 += bf2f(p1[static_cast<size_t>(b) * C + c]);
    }
    o0[c] = f2bf(a);
    if (p1 != nullptr) o1[c] = f2bf(b2);
}

size_t round16(size_t x) { return (x + 15) & ~static_cast<size_t>(15); }
// a fill kernel rather than hipMemsetAsync, which a caller's graph capture replays unreliably
__global__ void zero_words_kernel(int* p, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}
void zero_words(hipStream_t st, int* p, size_t n) {
    hipLaunchKernelGGL(zero_words_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, p, n);
}

// ---- wkv5 with heads of 128 channels on the matrix-core kernels: every head as four heads of 64, two launches per kernel,
//      each leaving one fp32 term of every output element (see ArgsB in wkv6_chunk.h); the terms are added here
constexpr int N_SPLIT = 2 * N;
bool use_split(int T, int C, int H, unsigned flags) {
    return C == H * N_SPLIT && !(flags & RWKV_FLAG_SWEEPS) && static_cast<long long>(T) * C < (1LL << 30);
}
// out[i] = bf16(p0[i] + p1[i]), four elements per thread (n is a multiple of 64)
__global__ __launch_bounds__(256) void split_sum(size_t n4, const float4* __restrict__ p0, const float4* __restrict__ p1, uint2* __restrict__ out) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 a = p0[i], b = p1[i];
    out[i] = make_uint2(static_cast<uint32_t>(f2bf(a.x + b.x)) | (static_cast<uint32_t>(f2bf(a.y + b.y)) << 16),
                        static_cast<uint32_t>(f2bf(a.z + b.z)) | (static_cast<uint32_t>(f2bf(a.w + b.w)) << 16));
}
void launch_split_sum(hipStream_t st, size_t n, const float* p0, const float* p1, uint16_t* out) {
    const size_t n4 = n / 4;
    hipLaunchKernelGGL(split_sum, dim3(static_cast<unsigned>((n4 + 255) / 256)), dim3(256), 0, st, n4,
                       reinterpret_cast<const float4*>(p0), reinterpret_cast<const float4*>(p1), reinterpret_cast<uint2*>(out));
}
// forward: the first launch's term of y
size_t fwd_split_bytes(int B, int T, int C) { return static_cast<size_t>(B) * T * C * sizeof(float); }
// backward: r dr' [B,T,C], the stored states of 2 H heads of 64, then fp32 terms: the first launch's gr [B,T,C], both
// launches' gk and gv, the first launch's gu [B,C], both launches' gw
size_t bwd_split_floats_before_terms(int B, int T, int C, int H) {
    const size_t nchunks = (static_cast<size_t>(T) + 31) / 32, npck = (nchunks + 3) / 4;
    return static_cast<size_t>(B) * T * C + static_cast<size_t>(B) * 2 * H * npck * 64 * 64;
}
size_t bwd_split_bytes(int B, int T, int C, int H) {
    return (bwd_split_floats_before_terms(B, T, C, H) + 5 * static_cast<size_t>(B) * T * C + 3 * static_cast<size_t>(B) * C) * sizeof(float);
}
int launch_fwd_split(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                     const float* eew, const uint16_t* u, uint16_t* y, float* ws) {
    for (int cross = 0; cross < 2; ++cross)
        if (int e = launch_wkv5_fwd_split(st, cross, B, T, C, H, r, k, v, eew, u, ws, y)) return e;
    return launch_status();
}
int launch_bwd_split(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                     const float* ew, const uint16_t* u, const uint16_t* gy, uint16_t* gr, uint16_t* gk, uint16_t* gv,
                     uint16_t* gw, uint16_t* gu, float* ws, unsigned flags) {
    const unsigned passes = passes_of(flags);
    const size_t n = static_cast<size_t>(B) * T * C, m = static_cast<size_t>(B) * C;
    float* rdr = ws;
    float* gr32 = ws + bwd_split_floats_before_terms(B, T, C, H);
    float* gk32 = gr32 + n;
    float* gv32 = gk32 + 2 * n;
    float* gu32 = gv32 + 2 * n;
    float* gw32 = gu32 + m;
    // the second sweep of a launch reads the r dr' its own first sweep has left: first, second, first, second
    for (int cross = 0; cross < 2; ++cross) {
        if (passes & RWKV_PASS_GR)
            if (int e = launch_wkv5_bwd_a_split(st, cross, B, T, C, H, r, k, v, ew, u, gy, gr32, gu32, gr, gu, rdr)) return e;
        if (passes & RWKV_PASS_GK)
            if (int e = launch_wkv5_bwd_b_split(st, cross, B, T, C, H, r, k, v, ew, u, gy, gk32 + cross * n, gv32 + cross * n, gw32 + cross * m, rdr)) return e;
    }
    if (passes & RWKV_PASS_GK) {
        launch_split_sum(st, n, gk32, gk32 + n, gk);
        launch_split_sum(st, n, gv32, gv32 + n, gv);
        launch_split_sum(st, m, gw32, gw32 + m, gw);
    }
    return launch_status();
}

}  // namespace
}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_wkv5_forward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                      const rwkv_bf16* v, const float* eew, const rwkv_bf16* u, rwkv_bf16* y, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, eew, u, y}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = eew; a.u = u; a.y = y;
    return launch_fwd<W_HEAD>(static_cast<hipStream_t>(stream), B, a, flags);
}

size_t rwkv_wkv5_forward_workspace_bytes(int B, int T, int C, int H) {
    if (check_dims(B, T, C, H) != RWKV_OK) return 0;
    return use_split(T, C, H, 0u) ? fwd_split_bytes(B, T, C) : 0;
}

int rwkv_wkv5_forward_ws(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                         const float* eew, const rwkv_bf16* u, rwkv_bf16* y, void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (!use_split(T, C, H, flags)) return rwkv_wkv5_forward_ex(stream, B, T, C, H, r, k, v, eew, u, y, flags);
    if (int e = check_ptrs({r, k, v, eew, u, y})) return e;
    if (workspace == nullptr || workspace_bytes < fwd_split_bytes(B, T, C) || !aligned16(workspace)) return RWKV_ERR_WORKSPACE;
    return launch_fwd_split(static_cast<hipStream_t>(stream), B, T, C, H, r, k, v, eew, u, y, static_cast<float*>(workspace));
}

size_t rwkv_wkv5_backward_workspace_bytes(int B, int T, int C, int H) {
    if (check_dims(B, T, C, H) != RWKV_OK) return 0;
    return use_split(T, C, H, 0u) ? bwd_split_bytes(B, T, C, H) : ws_bytes(B, T, C, H);
}

int rwkv_wkv5_backward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                       const rwkv_bf16* v, const float* eew, const float* ew, const rwkv_bf16* u,
                       const rwkv_bf16* gy, rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw,
                       rwkv_bf16* gu, void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu}, C == H * N || C == H * N_SPLIT)) return e;
    if (workspace == nullptr || workspace_bytes < rwkv_wkv5_backward_workspace_bytes(B, T, C, H) || !aligned16(workspace))
        return RWKV_ERR_WORKSPACE;
    if (use_split(T, C, H, flags))
        return launch_bwd_split(static_cast<hipStream_t>(stream), B, T, C, H, r, k, v, ew, u, gy, gr, gk, gv, gw, gu,
                                static_cast<float*>(workspace), flags);
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = eew; a.ew_head = ew; a.u = u; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.rdr = static_cast<float*>(workspace);
    return launch_bwd<W_HEAD>(static_cast<hipStream_t>(stream), B, a, flags);
}

// ---- wkv5, fp32 I/O: the sequential fp32 sweeps only (the chunked kernels work to bf16-I/O accuracy)
namespace {
const uint16_t* as_elems(const float* p) { return reinterpret_cast<const uint16_t*>(p); }
uint16_t* out_elems(float* p) { return reinterpret_cast<uint16_t*>(p); }
}  // namespace

int rwkv_wkv5f32_forward(void* stream, int B, int T, int C, int H, const float* r, const float* k, const float* v,
                         const float* eew, const float* u, float* y) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, eew, u, y}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = as_elems(r); a.k = as_elems(k); a.v = as_elems(v); a.w = eew; a.u = as_elems(u);
    a.y = out_elems(y);
    if (C != H * N) launch_rows<P_FWD, W_HEAD, true>(static_cast<hipStream_t>(stream), B, a);
    else hipLaunchKernelGGL((wkv_sweep<P_FWD, W_HEAD, true>), dim3(B * H), dim3(NT), 0, static_cast<hipStream_t>(stream), a);
    return launch_status();
}

int rwkv_wkv5f32_backward_ex(void* stream, int B, int T, int C, int H, const float* r, const float* k, const float* v,
                          const float* eew, const float* ew, const float* u, const float* gy, float* gr, float* gk,
                          float* gv, float* gw, float* gu, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = as_elems(r); a.k = as_elems(k); a.v = as_elems(v); a.w = eew; a.ew_head = ew;
    a.u = as_elems(u); a.gy = as_elems(gy); a.gr = out_elems(gr); a.gk = out_elems(gk); a.gv = out_elems(gv);
    a.gw = out_elems(gw); a.gu = out_elems(gu);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (C != H * N) {
        if (passes_of(flags) & RWKV_PASS_GR) launch_rows<P_GR, W_HEAD, true>(st, B, a);
        if (passes_of(flags) & RWKV_PASS_GV) launch_rows<P_GV, W_HEAD, true>(st, B, a);
        if (passes_of(flags) & RWKV_PASS_GK) launch_rows<P_GK, W_HEAD, true>(st, B, a);
        return launch_status();
    }
    // three independent sweeps: gr + gu + gw, gv, gk
    if (passes_of(flags) & RWKV_PASS_GR) hipLaunchKernelGGL((wkv_sweep<P_GR, W_HEAD, true>), dim3(B * H), dim3(NT), 0, st, a);
    if (passes_of(flags) & RWKV_PASS_GV) hipLaunchKernelGGL((wkv_sweep<P_GV, W_HEAD, true>), dim3(B * H), dim3(NT), 0, st, a);
    if (passes_of(flags) & RWKV_PASS_GK) hipLaunchKernelGGL((wkv_sweep<P_GK, W_HEAD, true>), dim3(B * H), dim3(NT), 0, st, a);
    return launch_status();
}

// ---- wkv5a: two-sided decay and bonus, fp32, on the same sweeps
int rwkv_wkv5a_forward(void* stream, int B, int T, int C, int H, const float* r, const float* k, const float* v,
                       const float* eew1, const float* u1, const float* eew2, const float* u2, float* y) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, eew1, u1, eew2, u2, y}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = as_elems(r); a.k = as_elems(k); a.v = as_elems(v); a.w = eew1; a.u = as_elems(u1);
    a.w2 = eew2; a.u2 = as_elems(u2); a.y = out_elems(y);
    if (C != H * N) {
        launch_rows<P_FWD, W_HEAD, true, true>(static_cast<hipStream_t>(stream), B, a);
        return launch_status();
    }
    hipLaunchKernelGGL((wkv_sweep<P_FWD, W_HEAD, true, true>), dim3(B * H), dim3(NT), 0, static_cast<hipStream_t>(stream), a);
    return launch_status();
}

int rwkv_wkv5a_backward_ex(void* stream, int B, int T, int C, int H, const float* r, const float* k, const float* v,
                        const float* eew1, const float* ew1, const float* u1, const float* eew2, const float* ew2,
                        const float* u2, const float* gy, float* gr, float* gk, float* gv, float* gw1, float* gu1,
                        float* gw2, float* gu2, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, eew1, ew1, u1, eew2, ew2, u2, gy, gr, gk, gv, gw1, gu1, gw2, gu2}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = as_elems(r); a.k = as_elems(k); a.v = as_elems(v); a.w = eew1; a.ew_head = ew1;
    a.u = as_elems(u1); a.w2 = eew2; a.ew2_head = ew2; a.u2 = as_elems(u2); a.gy = as_elems(gy);
    a.gr = out_elems(gr); a.gk = out_elems(gk); a.gv = out_elems(gv);
    a.gw = out_elems(gw1); a.gu = out_elems(gu1); a.gw2 = out_elems(gw2); a.gu2 = out_elems(gu2);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (C != H * N) {
        if (passes_of(flags) & RWKV_PASS_GR) launch_rows<P_GR, W_HEAD, true, true>(st, B, a);
        if (passes_of(flags) & RWKV_PASS_GV) launch_rows<P_GV, W_HEAD, true, true>(st, B, a);
        if (passes_of(flags) & RWKV_PASS_GK) launch_rows<P_GK, W_HEAD, true, true>(st, B, a);
        return launch_status();
    }
    // three independent sweeps: gr + gu1 + gu2 + gw1 + gw2, gv, gk
    if (passes_of(flags) & RWKV_PASS_GR) hipLaunchKernelGGL((wkv_sweep<P_GR, W_HEAD, true, true>), dim3(B * H), dim3(NT), 0, st, a);
    if (passes_of(flags) & RWKV_PASS_GV) hipLaunchKernelGGL((wkv_sweep<P_GV, W_HEAD, true, true>), dim3(B * H), dim3(NT), 0, st, a);
    if (passes_of(flags) & RWKV_PASS_GK) hipLaunchKernelGGL((wkv_sweep<P_GK, W_HEAD, true, true>), dim3(B * H), dim3(NT), 0, st, a);
    return launch_status();
}

int rwkv_wkv6_forward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                      const rwkv_bf16* v, const float* ew, const rwkv_bf16* u, rwkv_bf16* y, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, ew, u, y}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = ew; a.u = u; a.y = y;
    return launch_fwd<W_EW>(static_cast<hipStream_t>(stream), B, a, flags);
}

size_t rwkv_wkv6_backward_workspace_bytes(int B, int T, int C, int H) { return ws_bytes(B, T, C, H); }

int rwkv_wkv6_backward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                       const rwkv_bf16* v, const float* ew, const rwkv_bf16* u, const rwkv_bf16* gy,
                       rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                       void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, ew, u, gy, gr, gk, gv, gw, gu}, C == H * N)) return e;
    if (workspace == nullptr || workspace_bytes < ws_bytes(B, T, C, H) || !aligned16(workspace)) return RWKV_ERR_WORKSPACE;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = ew; a.u = u; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.rdr = static_cast<float*>(workspace);
    return launch_bwd<W_EW>(static_cast<hipStream_t>(stream), B, a, flags);
}

int rwkv_wkv6raw_forward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                         const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, rwkv_bf16* y, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w, u, y}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.y = y;
    return launch_fwd<W_RAW>(static_cast<hipStream_t>(stream), B, a, flags);
}

int rwkv_wkv6raw_backward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                          const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* gy,
                          rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                          void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w, u, gy, gr, gk, gv, gw, gu}, C == H * N)) return e;
    if (workspace == nullptr || workspace_bytes < ws_bytes(B, T, C, H) || !aligned16(workspace)) return RWKV_ERR_WORKSPACE;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.rdr = static_cast<float*>(workspace);
    return launch_bwd<W_RAW>(static_cast<hipStream_t>(stream), B, a, flags);
}

int rwkv_wkv6state_forward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                           const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s,
                           rwkv_bf16* y, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w, u, s, y}, C == H * N)) return e;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s; a.y = y;
    return launch_fwd<W_RAW>(static_cast<hipStream_t>(stream), B, a, flags);
}

size_t rwkv_wkv6state_backward_workspace_bytes(int B, int T, int C, int H) { return ws_bytes(B, T, C, H); }

int rwkv_wkv6state_backward_ex(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                            const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s,
                            const rwkv_bf16* gy, rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw,
                            rwkv_bf16* gu, rwkv_bf16* gs, void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w, u, s, gy, gr, gk, gv, gw, gu, gs}, C == H * N)) return e;
    if (workspace == nullptr || workspace_bytes < ws_bytes(B, T, C, H) || !aligned16(workspace)) return RWKV_ERR_WORKSPACE;
    Args a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.gs = gs; a.rdr = static_cast<float*>(workspace);
    return launch_bwd<W_RAW>(static_cast<hipStream_t>(stream), B, a, flags);
}

// ---- the whole of WKV_5 / WKV_6 / WKV_6STATE forward and backward behind the C ABI: raw decay parameter in, parameter
//      gradients summed over the batch out (no torch kernel is left in the autograd step)
int rwkv_wkv5raw_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                         const rwkv_bf16* w_raw, const rwkv_bf16* u, rwkv_bf16* y, float* decay, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w_raw, u, y, decay}, C == H * N)) return e;
    hipLaunchKernelGGL(wkv5_decay_transform, dim3((C + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), C, w_raw, decay);
    return rwkv_wkv5_forward_ex(stream, B, T, C, H, r, k, v, decay, u, y, flags);
}

int rwkv_wkv5raw_forward_ws(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                            const rwkv_bf16* w_raw, const rwkv_bf16* u, rwkv_bf16* y, float* decay, void* workspace,
                            size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w_raw, u, y, decay}, C == H * N || C == H * N_SPLIT)) return e;
    hipLaunchKernelGGL(wkv5_decay_transform, dim3((C + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), C, w_raw, decay);
    return rwkv_wkv5_forward_ws(stream, B, T, C, H, r, k, v, decay, u, y, workspace, workspace_bytes, flags);
}

size_t rwkv_wkv5raw_backward_workspace_bytes(int B, int T, int C, int H) {
    const size_t n = rwkv_wkv5_backward_workspace_bytes(B, T, C, H);
    return n == 0 ? 0 : round16(n) + round16(2 * static_cast<size_t>(B) * C * sizeof(uint16_t));
}

int rwkv_wkv5raw_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                          const float* decay, const rwkv_bf16* u, const rwkv_bf16* gy, rwkv_bf16* gr, rwkv_bf16* gk,
                          rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu, void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({decay, gw, gu}, C == H * N)) return e;
    if (workspace == nullptr || workspace_bytes < rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H) || !aligned16(workspace))
        return RWKV_ERR_WORKSPACE;
    const size_t n = round16(rwkv_wkv5_backward_workspace_bytes(B, T, C, H));
    uint16_t* pw = reinterpret_cast<uint16_t*>(static_cast<char*>(workspace) + n);      // per-batch gw, then per-batch gu
    uint16_t* pu = pw + static_cast<size_t>(B) * C;
    if (int e = rwkv_wkv5_backward_ex(stream, B, T, C, H, r, k, v, decay, decay + C, u, gy, gr, gk, gv, pw, pu, workspace, n, flags)) return e;
    hipLaunchKernelGGL(bf16_batch_sum, dim3((C + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), B, C, pw, gw, pu, gu);
    return launch_status();
}

size_t rwkv_wkv6f_backward_workspace_bytes(int B, int T, int C, int H) {
    const size_t n = ws_bytes(B, T, C, H);
    return n == 0 ? 0 : round16(n) + round16(static_cast<size_t>(B) * C * sizeof(uint16_t));
}

int rwkv_wkv6f_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                        const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, const rwkv_bf16* gy, rwkv_bf16* gr,
                        rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu, rwkv_bf16* gs, void* workspace,
                        size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({gu}, C == H * N)) return e;
    if ((s == nullptr) != (gs == nullptr)) return RWKV_ERR_NULL;           // state and its gradient come together
    if (workspace == nullptr || workspace_bytes < rwkv_wkv6f_backward_workspace_bytes(B, T, C, H) || !aligned16(workspace))
        return RWKV_ERR_WORKSPACE;
    const size_t n = round16(ws_bytes(B, T, C, H));
    uint16_t* pu = reinterpret_cast<uint16_t*>(static_cast<char*>(workspace) + n);      // per-batch gu
    const int e = s != nullptr
        ? rwkv_wkv6state_backward_ex(stream, B, T, C, H, r, k, v, w, u, s, gy, gr, gk, gv, gw, pu, gs, workspace, n, flags)
        : rwkv_wkv6raw_backward_ex(stream, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, pu, workspace, n, flags);
    if (e) return e;
    hipLaunchKernelGGL(bf16_batch_sum, dim3((C + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), B, C, pu, gu,
                       static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(nullptr));
    return launch_status();
}

// ---- WKV_6 / WKV_6STATE with states handed from the forward to the backward: the forward keeps the state entering
//      every second chunk, and the backward is one reverse sweep (wkv6_bwd_f.hip).  Head size 64 and the chunked
//      kernels only; otherwise `saved` has no bytes and both calls are the ones above.
bool fused_ok(int T, int C, int H, unsigned flags) {
    return C == H * N && !(flags & (RWKV_FLAG_SWEEPS | RWKV_PASS_ALL)) && static_cast<long long>(T) * C < (1LL << 30);
}

// Fewer (batch, head) pairs than the chip has CUs: the sequences are cut into blocks of whole 64-token segments, as many
// as it takes to give every CU a workgroup (and at least 128 tokens each, the pipeline needs a few chunks to fill).
constexpr int NUM_CU = 256;
int scan_blocks(int B, int T, int H, int* TB, unsigned flags = 0u) {
    const long long bh = static_cast<long long>(B) * H;
    const int seg = (T + 63) / 64;
    long long want = NUM_CU / bh;
    *TB = T;
    if (want < 2 || seg < 4 || (flags & RWKV_FLAG_WHOLE)) return 1;
    if (want > seg / 2) want = seg / 2;
    const int per = static_cast<int>((seg + want - 1) / want);
    *TB = per * 64;
    return (T + *TB - 1) / *TB;
}
size_t saved_states_bytes(int B, int T, int H) {
    const size_t nchunks = (static_cast<size_t>(T) + 31) / 32, nseg = (nchunks + 1) / 2;
    return static_cast<size_t>(B) * H * nseg * 64 * 64 * 3;          // 24 bits per value (SAVED_STATE_B, wkv6_chunk.h)
}
size_t scan_scratch_bytes(int B, int T, int H) {           // local results and scanned states (fp32 [64][64]) and log decays per block
    int TB;
    const int NB = scan_blocks(B, T, H, &TB);
    return NB <= 1 ? 0 : static_cast<size_t>(B) * H * NB * (2 * 64 * 64 + 64) * sizeof(float);
}

size_t rwkv_wkv6f_saved_bytes(int B, int T, int C, int H) {
    if (check_dims(B, T, C, H) != RWKV_OK || C != H * N || static_cast<long long>(T) * C >= (1LL << 30)) return 0;
    return saved_states_bytes(B, T, H) + round16(static_cast<size_t>(B) * H * 8 * sizeof(int)) + scan_scratch_bytes(B, T, H);
}

int rwkv_wkv6f_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, rwkv_bf16* y, void* saved, size_t saved_bytes,
                       unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w, u, y}, C == H * N)) return e;
    if (s != nullptr && C == H * N && !aligned16(s)) return RWKV_ERR_ALIGN;
    if (!fused_ok(T, C, H, flags) || saved == nullptr) {
        Args a{};
        a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s; a.y = y;
        return launch_fwd<W_RAW>(static_cast<hipStream_t>(stream), B, a, flags);
    }
    if (saved_bytes < rwkv_wkv6f_saved_bytes(B, T, C, H) || !aligned16(saved)) return RWKV_ERR_WORKSPACE;
    // the states, then a word per prep wave of every (batch, head): set where a decay is too strong for the mid-point
    // factors; those pairs are redone (y and states) by the kernel that has a step-by-step path, all others return at once
    const hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t nflag = round16(static_cast<size_t>(B) * H * 8 * sizeof(int));
    char* sb = static_cast<char*>(saved);
    int* flg = reinterpret_cast<int*>(sb + saved_states_bytes(B, T, H));
    int TB;
    const int NB = scan_blocks(B, T, H, &TB, flags);
    if (NB > 1) {
        const size_t nq = static_cast<size_t>(B) * H * NB;
        float* local = reinterpret_cast<float*>(sb + saved_states_bytes(B, T, H) + nflag);
        float* s32 = local + nq * 64 * 64;
        float* logdec = s32 + nq * 64 * 64;
        zero_words(st, flg, static_cast<size_t>(B) * H * 8);
        if (int e = launch_wkv6_fwd_fused(st, B, T, C, H, r, k, v, w, u, s, y, static_cast<char*>(saved), flg, NB, TB, local, logdec, s32)) return e;
    } else if (int e = launch_wkv6_fwd_fused(st, B, T, C, H, r, k, v, w, u, s, y, static_cast<char*>(saved), flg)) return e;
    return launch_wkv6_fwd_chunk(st, W_RAW, B, T, C, H, r, k, v, w, u, s, y, static_cast<char*>(saved), flg);
}

size_t rwkv_wkv6f_backward_saved_workspace_bytes(int B, int T, int C, int H) {
    const size_t n = rwkv_wkv6f_backward_workspace_bytes(B, T, C, H);
    if (n == 0) return 0;
    int TB;
    const int NB = C == H * N ? scan_blocks(B, T, H, &TB) : 1;
    // several blocks per sequence: the scan's scratch and gu per block and batch row in fp32
    const size_t scan = NB <= 1 ? 0 : scan_scratch_bytes(B, T, H) + static_cast<size_t>(NB) * B * C * sizeof(float);
    return round16(n) + round16(static_cast<size_t>(B) * H * 8 * sizeof(int)) + scan;
}

int rwkv_wkv6f_backward_saved(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                              const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, const rwkv_bf16* gy, rwkv_bf16* gr,
                              rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu, rwkv_bf16* gs, const void* saved,
                              size_t saved_bytes, void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (workspace == nullptr || workspace_bytes < rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H) || !aligned16(workspace))
        return RWKV_ERR_WORKSPACE;
    if (!fused_ok(T, C, H, flags) || saved == nullptr)
        return rwkv_wkv6f_backward(stream, B, T, C, H, r, k, v, w, u, s, gy, gr, gk, gv, gw, gu, gs, workspace, workspace_bytes, flags);
    if (int e = check_ptrs({r, k, v, w, u, gy, gr, gk, gv, gw, gu})) return e;
    if ((s == nullptr) != (gs == nullptr)) return RWKV_ERR_NULL;
    if (s != nullptr && (!aligned16(s) || !aligned16(gs))) return RWKV_ERR_ALIGN;
    if (saved_bytes < rwkv_wkv6f_saved_bytes(B, T, C, H) || !aligned16(saved)) return RWKV_ERR_WORKSPACE;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t n = round16(ws_bytes(B, T, C, H));
    char* wsb = static_cast<char*>(workspace);
    float* rdr = static_cast<float*>(workspace);
    uint16_t* pu = reinterpret_cast<uint16_t*>(wsb + n);                                  // per-batch gu
    int* flg = reinterpret_cast<int*>(wsb + round16(rwkv_wkv6f_backward_workspace_bytes(B, T, C, H)));
    int TB;
    const int NB = scan_blocks(B, T, H, &TB, flags);
    if (NB > 1) {
        const size_t nq = static_cast<size_t>(B) * H * NB;
        float* local = reinterpret_cast<float*>(reinterpret_cast<char*>(flg) + round16(static_cast<size_t>(B) * H * 8 * sizeof(int)));
        float* ds32 = local + nq * 64 * 64;
        float* logdec = ds32 + nq * 64 * 64;
        float* gu32 = logdec + nq * 64;
        zero_words(st, flg, static_cast<size_t>(B) * H * 8);
        if (int e = launch_wkv6_bwd_fused(st, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, pu, gs, static_cast<const char*>(saved), flg,
                                          NB, TB, local, logdec, ds32, gu32)) return e;
    } else if (int e = launch_wkv6_bwd_fused(st, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, pu, gs, static_cast<const char*>(saved), flg)) return e;
    // (batch, head) pairs with a decay the mid-point factors cannot carry: the two sweeps redo them, all others return at once
    if (int e = launch_wkv6_bwd_a_chunk(st, W_RAW, B, T, C, H, r, k, v, w, u, s, gy, gr, pu, rdr, flg)) return e;
    // (the second sweep's workgroups of batch row 0 first add the per-batch gu rows up: they are complete by then, and a
    //  launch of its own for that costs as much as any other, about 5 us)
    return launch_wkv6_bwd_b_chunk(st, W_RAW, B, T, C, H, r, k, v, w, u, s, gy, gk, gv, gw, gs, rdr, flg, pu, gu);
}

// ---- wkv5 (head size 64) on the one-sweep pair: the raw decay of a channel stands in for every token's, its gradient is
//      summed over the tokens inside the kernel.  `decay` = [eew | ew] is made for the kernels that redo flagged heads.
size_t rwkv_wkv5s_saved_bytes(int B, int T, int C, int H) { return rwkv_wkv6f_saved_bytes(B, T, C, H); }

int rwkv_wkv5s_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const rwkv_bf16* w_raw, const rwkv_bf16* u, rwkv_bf16* y, float* decay, void* saved, size_t saved_bytes,
                       unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (int e = check_ptrs({r, k, v, w_raw, u, y, decay}, C == H * N)) return e;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    if (!fused_ok(T, C, H, flags) || saved == nullptr) {
        hipLaunchKernelGGL(wkv5_decay_transform, dim3((C + 255) / 256), dim3(256), 0, st, C, w_raw, decay);
        return rwkv_wkv5_forward_ex(stream, B, T, C, H, r, k, v, decay, u, y, flags);
    }
    // (the one-sweep kernel writes `decay` itself: its workgroups of batch row 0 hold every channel's raw value)
    if (saved_bytes < rwkv_wkv5s_saved_bytes(B, T, C, H) || !aligned16(saved)) return RWKV_ERR_WORKSPACE;
    const size_t nflag = round16(static_cast<size_t>(B) * H * 8 * sizeof(int));
    char* sb = static_cast<char*>(saved);
    int* flg = reinterpret_cast<int*>(sb + saved_states_bytes(B, T, H));
    int TB;
    const int NB = scan_blocks(B, T, H, &TB, flags);
    if (NB > 1) {
        const size_t nq = static_cast<size_t>(B) * H * NB;
        float* local = reinterpret_cast<float*>(sb + saved_states_bytes(B, T, H) + nflag);
        float* s32 = local + nq * 64 * 64;
        float* logdec = s32 + nq * 64 * 64;
        zero_words(st, flg, static_cast<size_t>(B) * H * 8);
        if (int e = launch_wkv6_fwd_fused(st, B, T, C, H, r, k, v, w_raw, u, nullptr, y, static_cast<char*>(saved), flg, NB, TB, local, logdec, s32, decay)) return e;
    } else if (int e = launch_wkv6_fwd_fused(st, B, T, C, H, r, k, v, w_raw, u, nullptr, y, static_cast<char*>(saved), flg, 1, 0, nullptr, nullptr, nullptr, decay)) return e;
    return launch_wkv6_fwd_chunk(st, W_HEAD, B, T, C, H, r, k, v, decay, u, nullptr, y, static_cast<char*>(saved), flg);
}

size_t rwkv_wkv5s_backward_workspace_bytes(int B, int T, int C, int H) {
    const size_t n = rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H);
    if (n == 0) return 0;
    int TB;
    const int NB = C == H * N ? scan_blocks(B, T, H, &TB) : 1;
    // several blocks per sequence: the scan's scratch and gw, gu per block and batch row in fp32
    const size_t scan = NB <= 1 ? 0 : scan_scratch_bytes(B, T, H) + 2 * static_cast<size_t>(NB) * B * C * sizeof(float);
    return round16(n) + round16(static_cast<size_t>(B) * H * 8 * sizeof(int)) + scan;
}

int rwkv_wkv5s_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                        const rwkv_bf16* w_raw, const float* decay, const rwkv_bf16* u, const rwkv_bf16* gy, rwkv_bf16* gr,
                        rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu, const void* saved, size_t saved_bytes,
                        void* workspace, size_t workspace_bytes, unsigned flags) {
    if (int e = check_dims(B, T, C, H)) return e;
    if (workspace == nullptr || workspace_bytes < rwkv_wkv5s_backward_workspace_bytes(B, T, C, H) || !aligned16(workspace))
        return RWKV_ERR_WORKSPACE;
    if (!fused_ok(T, C, H, flags) || saved == nullptr)
        return rwkv_wkv5raw_backward(stream, B, T, C, H, r, k, v, decay, u, gy, gr, gk, gv, gw, gu, workspace, workspace_bytes, flags);
    if (int e = check_ptrs({r, k, v, w_raw, decay, u, gy, gr, gk, gv, gw, gu})) return e;
    if (saved_bytes < rwkv_wkv5s_saved_bytes(B, T, C, H) || !aligned16(saved)) return RWKV_ERR_WORKSPACE;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    char* wsb = static_cast<char*>(workspace);
    const size_t n = round16(rwkv_wkv5_backward_workspace_bytes(B, T, C, H));
    float* rdr = static_cast<float*>(workspace);
    uint16_t* pw = reinterpret_cast<uint16_t*>(wsb + n);                                  // per-batch gw, then per-batch gu
    uint16_t* pu = pw + static_cast<size_t>(B) * C;
    int* flg = reinterpret_cast<int*>(wsb + round16(rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H)));
    int TB;
    const int NB = scan_blocks(B, T, H, &TB, flags);
    if (NB > 1) {
        const size_t nq = static_cast<size_t>(B) * H * NB;
        float* local = reinterpret_cast<float*>(reinterpret_cast<char*>(flg) + round16(static_cast<size_t>(B) * H * 8 * sizeof(int)));
        float* ds32 = local + nq * 64 * 64;
        float* logdec = ds32 + nq * 64 * 64;
        float* gu32 = logdec + nq * 64;
        float* gw32 = gu32 + static_cast<size_t>(NB) * B * C;
        zero_words(st, flg, static_cast<size_t>(B) * H * 8);
        if (int e = launch_wkv6_bwd_fused(st, B, T, C, H, r, k, v, w_raw, u, gy, gr, gk, gv, nullptr, pu, nullptr, static_cast<const char*>(saved), flg,
                                          NB, TB, local, logdec, ds32, gu32, pw, gw32)) return e;
    } else if (int e = launch_wkv6_bwd_fused(st, B, T, C, H, r, k, v, w_raw, u, gy, gr, gk, gv, nullptr, pu, nullptr, static_cast<const char*>(saved), flg,
                                             1, 0, nullptr, nullptr, nullptr, nullptr, pw, nullptr)) return e;
    // heads whose decay the mid-point factors cannot carry: the two sweeps redo them (their per-batch gw, gu rows included)
    const float* ew = decay + C;
    if (int e = launch_wkv6_bwd_a_chunk(st, W_HEAD, B, T, C, H, r, k, v, ew, u, nullptr, gy, gr, pu, rdr, flg)) return e;
    if (int e = launch_wkv6_bwd_b_chunk(st, W_HEAD, B, T, C, H, r, k, v, ew, u, nullptr, gy, gk, gv, pw, nullptr, rdr, flg)) return e;
    hipLaunchKernelGGL(bf16_batch_sum, dim3((C + 255) / 256), dim3(256), 0, st, B, C, pw, gw, pu, gu);
    return launch_status();
}

// ---- the reference-signature entry points: default kernels, every pass
int rwkv_wkv5_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                      const rwkv_bf16* v, const float* eew, const rwkv_bf16* u, rwkv_bf16* y) {
    return rwkv_wkv5_forward_ex(stream, B, T, C, H, r, k, v, eew, u, y, 0u);
}

int rwkv_wkv5_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                       const rwkv_bf16* v, const float* eew, const float* ew, const rwkv_bf16* u,
                       const rwkv_bf16* gy, rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw,
                       rwkv_bf16* gu, void* workspace, size_t workspace_bytes) {
    return rwkv_wkv5_backward_ex(stream, B, T, C, H, r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu, workspace, workspace_bytes, 0u);
}

int rwkv_wkv5f32_backward(void* stream, int B, int T, int C, int H, const float* r, const float* k, const float* v,
                          const float* eew, const float* ew, const float* u, const float* gy, float* gr, float* gk,
                          float* gv, float* gw, float* gu) {
    return rwkv_wkv5f32_backward_ex(stream, B, T, C, H, r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu, 0u);
}

int rwkv_wkv5a_backward(void* stream, int B, int T, int C, int H, const float* r, const float* k, const float* v,
                        const float* eew1, const float* ew1, const float* u1, const float* eew2, const float* ew2,
                        const float* u2, const float* gy, float* gr, float* gk, float* gv, float* gw1, float* gu1,
                        float* gw2, float* gu2) {
    return rwkv_wkv5a_backward_ex(stream, B, T, C, H, r, k, v, eew1, ew1, u1, eew2, ew2, u2, gy, gr, gk, gv, gw1, gu1, gw2, gu2, 0u);
}

int rwkv_wkv6_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                      const rwkv_bf16* v, const float* ew, const rwkv_bf16* u, rwkv_bf16* y) {
    return rwkv_wkv6_forward_ex(stream, B, T, C, H, r, k, v, ew, u, y, 0u);
}

int rwkv_wkv6_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                       const rwkv_bf16* v, const float* ew, const rwkv_bf16* u, const rwkv_bf16* gy,
                       rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                       void* workspace, size_t workspace_bytes) {
    return rwkv_wkv6_backward_ex(stream, B, T, C, H, r, k, v, ew, u, gy, gr, gk, gv, gw, gu, workspace, workspace_bytes, 0u);
}

int rwkv_wkv6raw_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                         const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, rwkv_bf16* y) {
    return rwkv_wkv6raw_forward_ex(stream, B, T, C, H, r, k, v, w, u, y, 0u);
}

int rwkv_wkv6raw_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                          const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* gy,
                          rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                          void* workspace, size_t workspace_bytes) {
    return rwkv_wkv6raw_backward_ex(stream, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, workspace, workspace_bytes, 0u);
}

int rwkv_wkv6state_forward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                           const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s,
                           rwkv_bf16* y) {
    return rwkv_wkv6state_forward_ex(stream, B, T, C, H, r, k, v, w, u, s, y, 0u);
}

int rwkv_wkv6state_backward(void* stream, int B, int T, int C, int H, const rwkv_bf16* r, const rwkv_bf16* k,
                            const rwkv_bf16* v, const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s,
                            const rwkv_bf16* gy, rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw,
                            rwkv_bf16* gu, rwkv_bf16* gs, void* workspace, size_t workspace_bytes) {
    return rwkv_wkv6state_backward_ex(stream, B, T, C, H, r, k, v, w, u, s, gy, gr, gk, gv, gw, gu, gs, workspace, workspace_bytes, 0u);
}

}  // extern "C"
