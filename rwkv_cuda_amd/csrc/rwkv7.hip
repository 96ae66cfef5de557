// RWKV-7 "clamp-w" generalised delta rule with state passing, gfx950.
//
//   w_t = exp(-e^{-0.5} sigmoid(w_raw_t));  sa_t = S_t a_t;
//   S_{t+1} = S_t diag(w_t) + sa_t b_t^T + v_t k_t^T;  y_t = S_{t+1} r_t;  sT = S_T        S[i][j]: i value, j key
//
// One workgroup of four waves per (batch, head); each wave owns 16 of the 64 state rows
// (forward) so that every reduction the recurrence feeds back on stays inside a wave:
//   layout H   wave q, lane l: row i = 16q + (l&15), columns j = 16(l>>4) + J,  J = 0..15 in VGPRs
//   layout HT  wave q, lane l: column j = 16q + (l&15), rows i = 16(l>>4) + I,  I = 0..15 in VGPRs
// A vector indexed by the in-register axis sits one element per lane (lane l holds element l) and
// enters the FMAs through DPP row_newbcast; sums over the in-register axis are finished across the
// four 16-lane rows with two register swaps (allreduce_rows).  Forward uses H only and needs no
// barrier inside a chunk.  Backward keeps S and dS in HT (column sums dr, dw, dk, db, da) and a
// second copy of dS in H (row sums dv and dSb = dS b); dSb is the only value that crosses waves,
// once per step through LDS.
//
// Like the reference (rwkv7_statepassing_clampw.cu) the forward keeps sa_t and a state checkpoint
// every 16 steps, and the backward recovers S_t inside a chunk by inverting the step.
#include "common.h"

namespace rwkv {
namespace {

constexpr int N = 64;
constexpr int CL = RWKV7_CHUNK_LEN;   // 16: checkpoint interval = staging chunk
constexpr int NW = 4;
constexpr int NT = NW * 64;
constexpr int JW = 16;
constexpr float W_SCALE = -0.6065306597f;   // -exp(-0.5)

// Element pointers are typed for the bf16 mode; the fp32 mode (the reference's -D_FP32_ build) stores float pointers in
// the same fields and its kernels (F32 = true) read them back as such through ldg4 / stg4.
struct Args7 {
    int T, H;
    const uint16_t *r, *w, *k, *v, *a, *b, *dy;
    const float *s0, *dsT;
    uint16_t *y, *dr, *dw, *dk, *dv, *da, *db;
    float *sT, *ds0;
    float* s;     // checkpoints [B,H,T/CL][j][i]
    float* sa;    // [B,T,H,N]
};

DEVINL void unpack4(const uint2& q, float (&f)[4]) {
    f[0] = bf_lo(q.x); f[1] = bf_hi(q.x); f[2] = bf_lo(q.y); f[3] = bf_hi(q.y);
}
DEVINL uint2 pack4(const float (&f)[4]) {
    uint2 q;
    q.x = pack_bf2(f[0], f[1]); q.y = pack_bf2(f[2], f[3]);
    return q;
}
DEVINL void st4(float* dst, const float (&f)[4]) { *reinterpret_cast<float4*>(dst) = make_float4(f[0], f[1], f[2], f[3]); }
// four consecutive elements as they come from memory
template <bool F32> struct Raw4;
template <> struct Raw4<false> { uint2 q; };
template <> struct Raw4<true> { float4 q; };
template <bool F32> DEVINL Raw4<F32> ldg4(const uint16_t* p, size_t o) {
    Raw4<F32> x;
    if constexpr (F32) x.q = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + o);
    else x.q = *reinterpret_cast<const uint2*>(p + o);
    return x;
}
template <bool F32> DEVINL void widen4(const Raw4<F32>& x, float (&f)[4]) {
    if constexpr (F32) { f[0] = x.q.x; f[1] = x.q.y; f[2] = x.q.z; f[3] = x.q.w; }
    else unpack4(x.q, f);
}
template <bool F32> DEVINL void stg4(uint16_t* p, size_t o, const float (&f)[4]) {
    if constexpr (F32) *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + o) = make_float4(f[0], f[1], f[2], f[3]);
    else *reinterpret_cast<uint2*>(p + o) = pack4(f);
}
DEVINL void ld16(float (&f)[16], const float* src) {          // 16 consecutive floats, 16-byte aligned (LDS)
#pragma unroll
    for (int e = 0; e < 16; e += 4) {
        const float4 x = *reinterpret_cast<const float4*>(src + e);
        f[e] = x.x; f[e + 1] = x.y; f[e + 2] = x.z; f[e + 3] = x.w;
    }
}

// ------------------------------------------------------------------------------------ forward
struct SmemF {
    float r[CL][N], w[CL][N], k[CL][N], v[CL][N], a[CL][N], b[CL][N];
    float y[CL][N], sa[CL][N];
};

template <bool F32>
__global__ __launch_bounds__(NT) void rwkv7_fwd(const Args7 p) {
    __shared__ SmemF S;
    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6, lo = lane & 15, hi = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y, H = p.H, T = p.T;
    const size_t bh = static_cast<size_t>(b) * H + h;
    const int st = tid >> 4, sj = (tid & 15) * 4;
    const int row = q * JW + lo;                                  // this lane's state row i
    auto off = [&](int t) { return ((static_cast<size_t>(b) * T + t) * H + h) * N + sj; };

    float St[JW];
#pragma unroll
    for (int e = 0; e < JW; ++e) St[e] = 0.f;
    if (p.s0 != nullptr) {                         // the entry points without an initial state start from zero
        const float* s0 = p.s0 + (bh * N + row) * N + hi * JW;
#pragma unroll
        for (int e = 0; e < JW; e += 4) {
            const float4 x = *reinterpret_cast<const float4*>(s0 + e);
            St[e] = x.x; St[e + 1] = x.y; St[e + 2] = x.z; St[e + 3] = x.w;
        }
    }

    const int nchunks = T / CL;
    Raw4<F32> gr, gw, gk, gv, ga, gb;
    auto prefetch = [&](int c) {
        const size_t o = off(c * CL + st);
        gr = ldg4<F32>(p.r, o); gw = ldg4<F32>(p.w, o); gk = ldg4<F32>(p.k, o);
        gv = ldg4<F32>(p.v, o); ga = ldg4<F32>(p.a, o); gb = ldg4<F32>(p.b, o);
    };
    prefetch(0);

    for (int c = 0; c < nchunks; ++c) {
        __syncthreads();
        {
            float f[4];
            widen4<F32>(gr, f); st4(&S.r[st][sj], f);
            widen4<F32>(gk, f); st4(&S.k[st][sj], f);
            widen4<F32>(gv, f); st4(&S.v[st][sj], f);
            widen4<F32>(ga, f); st4(&S.a[st][sj], f);
            widen4<F32>(gb, f); st4(&S.b[st][sj], f);
            widen4<F32>(gw, f);
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] = __expf(W_SCALE / (1.0f + __expf(-f[e])));
            st4(&S.w[st][sj], f);
        }
        __syncthreads();
        if (c + 1 < nchunks) prefetch(c + 1);

#pragma unroll 2
        for (int t = 0; t < CL; ++t) {
            // The vectors indexed by the in-register axis (this lane's 16 columns) come as 16-byte LDS reads whose address
            // is the same in all 16 lanes of a row (about 1 clock per operand on the otherwise idle LDS pipe) and enter
            // plain FMAs; the DPP row-broadcast form of the same step measured 7 % slower.
            float av[JW], bv[JW], kv[JW], rv[JW], wv[JW];
            ld16(av, &S.a[t][hi * JW]);
            const float vi = S.v[t][row];
            float sa = 0.f;
#pragma unroll
            for (int j = 0; j < JW; ++j) sa = fmaf(av[j], St[j], sa);
            ld16(wv, &S.w[t][hi * JW]); ld16(bv, &S.b[t][hi * JW]); ld16(kv, &S.k[t][hi * JW]); ld16(rv, &S.r[t][hi * JW]);
            sa = allreduce_rows(sa);
            float y = 0.f;
#pragma unroll
            for (int j = 0; j < JW; ++j) {
                St[j] = fmaf(St[j], wv[j], fmaf(bv[j], sa, kv[j] * vi));
                y = fmaf(rv[j], St[j], y);
            }
            y = allreduce_rows(y);
            if (hi == 0) { S.sa[t][row] = sa; S.y[t][row] = y; }
        }
        // checkpoint S_{(c+1) CL}, stored [j][i] so that the backward reads 16 consecutive rows per lane
        {
            float* chk = p.s + (bh * nchunks + c) * (N * N);
#pragma unroll
            for (int e = 0; e < JW; ++e) chk[(hi * JW + e) * N + row] = St[e];
        }
        __syncthreads();
        {
            const size_t o = off(c * CL + st);
            float f[4] = {S.y[st][sj], S.y[st][sj + 1], S.y[st][sj + 2], S.y[st][sj + 3]};
            stg4<F32>(p.y, o, f);
            *reinterpret_cast<float4*>(p.sa + o) = *reinterpret_cast<const float4*>(&S.sa[st][sj]);
        }
    }
    if (p.sT != nullptr) {
        float* sT = p.sT + (bh * N + row) * N + hi * JW;
#pragma unroll
        for (int e = 0; e < JW; e += 4)
            *reinterpret_cast<float4*>(sT + e) = make_float4(St[e], St[e + 1], St[e + 2], St[e + 3]);
    }
}

// ------------------------------------------------------------------------------------ backward
struct SmemB {
    float r[CL][N], w[CL][N], k[CL][N], v[CL][N], a[CL][N], b[CL][N], dy[CL][N], sa[CL][N];
    float wf[CL][N];                       // d w / d w_raw = W_SCALE * w * sig * (1 - sig)
    float dr[CL][N], dw[CL][N], dk[CL][N], db[CL][N];      // in this order: row h of a wave's four-way reduction goes to array h
    float dv[CL][N];
    float da[CL][4][N];                    // one partial per lane row, summed when the chunk is stored: no reduction in the step
    float dSb[2][N];
};

template <bool F32>
__global__ __launch_bounds__(NT) void rwkv7_bwd(const Args7 p) {
    __shared__ SmemB S;
    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6, lo = lane & 15, hi = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y, H = p.H, T = p.T;
    const size_t bh = static_cast<size_t>(b) * H + h;
    const int st = tid >> 4, sj = (tid & 15) * 4;
    const int own = q * JW + lo;           // HT: this lane's column j;  H: this lane's row i
    auto off = [&](int t) { return ((static_cast<size_t>(b) * T + t) * H + h) * N + sj; };

    float ST[JW], dST[JW], dSH[JW];
#pragma unroll
    for (int e = 0; e < JW; ++e) { ST[e] = 0.f; dST[e] = 0.f; dSH[e] = 0.f; }
    if (p.dsT != nullptr) {                        // no gradient arrives through a final state that is not an output
        const float* g = p.dsT + bh * N * N;
#pragma unroll
        for (int e = 0; e < JW; ++e) {
            dST[e] = g[(hi * JW + e) * N + own];          // dS[i = 16hi+e][j = own]
            ST[e] = 0.f;
        }
        const float* gh = g + own * N + hi * JW;           // dS[i = own][j = 16hi+e]
#pragma unroll
        for (int e = 0; e < JW; e += 4) {
            const float4 x = *reinterpret_cast<const float4*>(gh + e);
            dSH[e] = x.x; dSH[e + 1] = x.y; dSH[e + 2] = x.z; dSH[e + 3] = x.w;
        }
    }

    const int nchunks = T / CL;
    Raw4<F32> gr, gw, gk, gv, ga, gb, gdy;
    float4 gsa;
    auto prefetch = [&](int c) {
        const size_t o = off(c * CL + st);
        gr = ldg4<F32>(p.r, o); gw = ldg4<F32>(p.w, o); gk = ldg4<F32>(p.k, o); gv = ldg4<F32>(p.v, o);
        ga = ldg4<F32>(p.a, o); gb = ldg4<F32>(p.b, o); gdy = ldg4<F32>(p.dy, o);
        gsa = *reinterpret_cast<const float4*>(p.sa + o);
    };
    prefetch(nchunks - 1);

    for (int c = nchunks - 1; c >= 0; --c) {
        __syncthreads();
        {
            float f[4], g[4];
            widen4<F32>(gr, f); st4(&S.r[st][sj], f);
            widen4<F32>(gk, f); st4(&S.k[st][sj], f);
            widen4<F32>(gv, f); st4(&S.v[st][sj], f);
            widen4<F32>(ga, f); st4(&S.a[st][sj], f);
            widen4<F32>(gb, f); st4(&S.b[st][sj], f);
            widen4<F32>(gdy, f); st4(&S.dy[st][sj], f);
            *reinterpret_cast<float4*>(&S.sa[st][sj]) = gsa;
            widen4<F32>(gw, f);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float sig = 1.0f / (1.0f + __expf(-f[e]));
                const float w = __expf(W_SCALE * sig);
                f[e] = w;
                g[e] = W_SCALE * w * sig * (1.0f - sig);
            }
            st4(&S.w[st][sj], f);
            st4(&S.wf[st][sj], g);
        }
        // S_{(c+1) CL} from the checkpoint, [j][i]: 16 consecutive rows of column `own`
        {
            const float* chk = p.s + (bh * nchunks + c) * (N * N) + own * N + hi * JW;
#pragma unroll
            for (int e = 0; e < JW; e += 4) {
                const float4 x = *reinterpret_cast<const float4*>(chk + e);
                ST[e] = x.x; ST[e + 1] = x.y; ST[e + 2] = x.z; ST[e + 3] = x.w;
            }
        }
        __syncthreads();
        if (c > 0) prefetch(c - 1);

        for (int t = CL - 1; t >= 0; --t) {
            const int par = t & 1;
            // vectors, one element per lane
            const float dyv = S.dy[t][lane], vv = S.v[t][lane], sav = S.sa[t][lane];
            const float rv = S.r[t][lane], kv = S.k[t][lane], bv = S.b[t][lane], wv = S.w[t][lane], av = S.a[t][lane];
            // scalars of this lane's own column (HT) / row (H)
            const float rj = S.r[t][own], kj = S.k[t][own], bj = S.b[t][own], wj = S.w[t][own], aj = S.a[t][own];
            const float dyi = S.dy[t][own];
            const float nk = -kj, nb = -bj, iw = 1.0f / wj;

            float drp = 0.f, dwp = 0.f, dkp = 0.f, dbp = 0.f, dvp = 0.f, dSbp = 0.f;
            static_for<JW>([&](auto E) {
                constexpr int e = decltype(E)::value;
                // HT: column sums over i and the inverse step
                fmac_bc<e>(drp, dyv, ST[e]);              // dr_j += dy_i S_{t+1}[i][j]
                fmac_bc<e>(ST[e], vv, nk);                // S_t = (S_{t+1} - v_i k_j - sa_i b_j) / w_j
                fmac_bc<e>(ST[e], sav, nb);
                ST[e] *= iw;
                fmac_bc<e>(dST[e], dyv, rj);              // dS += dy_i r_j
                dwp = fmaf(dST[e], ST[e], dwp);
                fmac_bc<e>(dkp, vv, dST[e]);
                fmac_bc<e>(dbp, sav, dST[e]);
                // H: row sums over j
                fmac_bc<e>(dSH[e], rv, dyi);              // dS += dy_i r_j
                fmac_bc<e>(dvp, kv, dSH[e]);
                fmac_bc<e>(dSbp, bv, dSH[e]);
            });
            float dSb = dSbp, dv = dvp;
            allreduce2_rows(dSb, dv);
            static_for<JW>([&](auto E) {
                constexpr int e = decltype(E)::value;
                mul_bc<e>(dSH[e], wv);                    // dS <- dS w_j + dSb_i a_j
                fmac_bc<e>(dSH[e], av, dSb);
            });
            // dr, dw, dk, db: the four column sums reduced together, lane row h ends up with the h-th of them
            (&S.dr[0][0])[(hi * CL + t) * N + own] = reduce4_rows(drp, dwp * S.wf[t][own], dkp, dbp);
            if (hi == 0) {
                S.dSb[par][own] = dSb;
                S.dv[t][own] = dv;
            }
            __syncthreads();
            const float dSbv = S.dSb[par][lane];
            float dap = 0.f;
            static_for<JW>([&](auto E) {
                constexpr int e = decltype(E)::value;
                fmac_bc<e>(dap, dSbv, ST[e]);             // da_j += S_t[i][j] dSb_i
                dST[e] *= wj;                             // dS <- dS w_j + dSb_i a_j
                fmac_bc<e>(dST[e], dSbv, aj);
            });
            S.da[t][hi][own] = dap;
        }
        __syncthreads();
        {
            const size_t o = off(c * CL + st);
            auto put = [&](uint16_t* dst, const float (*src)[N]) {
                float f[4] = {src[st][sj], src[st][sj + 1], src[st][sj + 2], src[st][sj + 3]};
                stg4<F32>(dst, o, f);
            };
            put(p.dr, S.dr); put(p.dw, S.dw); put(p.dk, S.dk);
            put(p.dv, S.dv); put(p.db, S.db);
            float f[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] = (S.da[st][0][sj + e] + S.da[st][1][sj + e]) + (S.da[st][2][sj + e] + S.da[st][3][sj + e]);
            stg4<F32>(p.da, o, f);
        }
    }
    if (p.ds0 != nullptr) {
        float* d = p.ds0 + (bh * N + own) * N + hi * JW;
#pragma unroll
        for (int e = 0; e < JW; e += 4)
            *reinterpret_cast<float4*>(d + e) = make_float4(dSH[e], dSH[e + 1], dSH[e + 2], dSH[e + 3]);
    }
}

int check7(int B, int T, int H) {
    if (B <= 0 || T <= 0 || H <= 0) return RWKV_ERR_SHAPE;
    if (T % CL != 0) return RWKV_ERR_SHAPE;
    if (B > 65535) return RWKV_ERR_SHAPE;
    return RWKV_OK;
}

const uint16_t* el(const void* p) { return static_cast<const uint16_t*>(p); }
uint16_t* el(void* p) { return static_cast<uint16_t*>(p); }

// r..b, y (and dy, dr..db below) are bf16 or, with f32, float
int launch7_fwd(void* stream, bool f32, int B, int T, int H, const float* s0, const void* r, const void* w,
                const void* k, const void* v, const void* a, const void* b, void* y,
                float* sT, float* s, float* sa) {
    Args7 p{};
    p.T = T; p.H = H; p.s0 = s0; p.r = el(r); p.w = el(w); p.k = el(k); p.v = el(v); p.a = el(a); p.b = el(b);
    p.y = el(y); p.sT = sT; p.s = s; p.sa = sa;
    if (f32) hipLaunchKernelGGL(rwkv7_fwd<true>, dim3(H, B), dim3(NT), 0, static_cast<hipStream_t>(stream), p);
    else hipLaunchKernelGGL(rwkv7_fwd<false>, dim3(H, B), dim3(NT), 0, static_cast<hipStream_t>(stream), p);
    return launch_status();
}

int launch7_bwd(void* stream, bool f32, int B, int T, int H, const void* r, const void* w, const void* k,
                const void* v, const void* a, const void* b, const void* dy, const float* dsT,
                const float* s, const float* sa, float* ds0, void* dr, void* dw, void* dk,
                void* dv, void* da, void* db) {
    Args7 p{};
    p.T = T; p.H = H; p.r = el(r); p.w = el(w); p.k = el(k); p.v = el(v); p.a = el(a); p.b = el(b); p.dy = el(dy);
    p.dsT = dsT; p.s = const_cast<float*>(s); p.sa = const_cast<float*>(sa);
    p.ds0 = ds0; p.dr = el(dr); p.dw = el(dw); p.dk = el(dk); p.dv = el(dv); p.da = el(da); p.db = el(db);
    if (f32) hipLaunchKernelGGL(rwkv7_bwd<true>, dim3(H, B), dim3(NT), 0, static_cast<hipStream_t>(stream), p);
    else hipLaunchKernelGGL(rwkv7_bwd<false>, dim3(H, B), dim3(NT), 0, static_cast<hipStream_t>(stream), p);
    return launch_status();
}


// bf16 mode: the chunked matrix-core kernels (rwkv7_chunk.hip) unless RWKV_FLAG_SWEEPS asks for the step kernels above.
// The two families lay out the scratch tensor `s` differently, so a backward must get the flags of its forward.
constexpr unsigned DEFAULT7 = 0u;                   // what the entry points without a flags argument run: the chunked kernels
int bf16_fwd(void* stream, unsigned flags, int B, int T, int H, const float* s0, const rwkv_bf16* r, const rwkv_bf16* w,
             const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b, rwkv_bf16* y, float* sT,
             float* s, float* sa) {
    if (flags & RWKV_FLAG_SWEEPS) return launch7_fwd(stream, false, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa);
    return launch7c_fwd(static_cast<hipStream_t>(stream), B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa);
}
int bf16_bwd(void* stream, unsigned flags, int B, int T, int H, const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k,
             const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b, const rwkv_bf16* dy, const float* dsT,
             const float* s, const float* sa, float* ds0, rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
             rwkv_bf16* da, rwkv_bf16* db) {
    if (flags & RWKV_FLAG_SWEEPS) return launch7_bwd(stream, false, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db);
    return launch7c_bwd(static_cast<hipStream_t>(stream), B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db);
}

}  // namespace
}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv7_statepassing_forward(void* stream, int B, int T, int H, const float* s0, const rwkv_bf16* r,
                               const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a,
                               const rwkv_bf16* b, rwkv_bf16* y, float* sT, float* s, float* sa) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({s0, r, w, k, v, a, b, y, sT, s, sa})) return e;
    return bf16_fwd(stream, DEFAULT7, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa);
}

int rwkv7_statepassing_backward(void* stream, int B, int T, int H, const rwkv_bf16* r, const rwkv_bf16* w,
                                const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                                const rwkv_bf16* dy, const float* dsT, const float* s, const float* sa,
                                float* ds0, rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
                                rwkv_bf16* da, rwkv_bf16* db) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db})) return e;
    return bf16_bwd(stream, DEFAULT7, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db);
}

// Initial state with its gradient, no final state: the same kernels without the sT store and with dsT = 0.
int rwkv7_state_forward(void* stream, int B, int T, int H, const float* s0, const rwkv_bf16* r, const rwkv_bf16* w,
                        const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                        rwkv_bf16* y, float* s, float* sa) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({s0, r, w, k, v, a, b, y, s, sa})) return e;
    return bf16_fwd(stream, DEFAULT7, B, T, H, s0, r, w, k, v, a, b, y, nullptr, s, sa);
}

int rwkv7_state_backward(void* stream, int B, int T, int H, const rwkv_bf16* r, const rwkv_bf16* w,
                         const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                         const rwkv_bf16* dy, const float* s, const float* sa, float* ds0, rwkv_bf16* dr,
                         rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv, rwkv_bf16* da, rwkv_bf16* db) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, s, sa, ds0, dr, dw, dk, dv, da, db})) return e;
    return bf16_bwd(stream, DEFAULT7, B, T, H, r, w, k, v, a, b, dy, nullptr, s, sa, ds0, dr, dw, dk, dv, da, db);
}

// No state on either side: zero initial state, no final state, no state gradients.
int rwkv7_forward(void* stream, int B, int T, int H, const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k,
                  const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b, rwkv_bf16* y, float* s, float* sa) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, y, s, sa})) return e;
    return bf16_fwd(stream, DEFAULT7, B, T, H, nullptr, r, w, k, v, a, b, y, nullptr, s, sa);
}

int rwkv7_backward(void* stream, int B, int T, int H, const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k,
                   const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b, const rwkv_bf16* dy, const float* s,
                   const float* sa, rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv, rwkv_bf16* da,
                   rwkv_bf16* db) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, s, sa, dr, dw, dk, dv, da, db})) return e;
    return bf16_bwd(stream, DEFAULT7, B, T, H, r, w, k, v, a, b, dy, nullptr, s, sa, nullptr, dr, dw, dk, dv, da, db);
}

// The state-passing op with per-call flags; s0, sT (forward) and dsT, ds0 (backward) may be NULL, which makes these two
// entry points cover the state-only and the stateless siblings as well.
int rwkv7_statepassing_forward_ex(void* stream, int B, int T, int H, const float* s0, const rwkv_bf16* r,
                                  const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a,
                                  const rwkv_bf16* b, rwkv_bf16* y, float* sT, float* s, float* sa, unsigned flags) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, y, s, sa})) return e;
    if (!aligned16(s0) || !aligned16(sT)) return RWKV_ERR_ALIGN;
    return bf16_fwd(stream, flags, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa);
}

int rwkv7_statepassing_backward_ex(void* stream, int B, int T, int H, const rwkv_bf16* r, const rwkv_bf16* w,
                                   const rwkv_bf16* k, const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                                   const rwkv_bf16* dy, const float* dsT, const float* s, const float* sa,
                                   float* ds0, rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
                                   rwkv_bf16* da, rwkv_bf16* db, unsigned flags) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, s, sa, dr, dw, dk, dv, da, db})) return e;
    if (!aligned16(dsT) || !aligned16(ds0)) return RWKV_ERR_ALIGN;
    return bf16_bwd(stream, flags, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db);
}

// ---- fp32 I/O: what the reference builds from the same sources with -D_FP32_ (rwkv7_cuda_benchmark.py:102-126 and the
// same lines of its _state and _state_passing siblings).  Same kernels, same fp32 arithmetic; only loads and stores differ.
int rwkv7_statepassing_forward_f32(void* stream, int B, int T, int H, const float* s0, const float* r, const float* w,
                                   const float* k, const float* v, const float* a, const float* b, float* y,
                                   float* sT, float* s, float* sa) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({s0, r, w, k, v, a, b, y, sT, s, sa})) return e;
    return launch7_fwd(stream, true, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa);
}

int rwkv7_statepassing_backward_f32(void* stream, int B, int T, int H, const float* r, const float* w, const float* k,
                                    const float* v, const float* a, const float* b, const float* dy, const float* dsT,
                                    const float* s, const float* sa, float* ds0, float* dr, float* dw, float* dk,
                                    float* dv, float* da, float* db) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db})) return e;
    return launch7_bwd(stream, true, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db);
}

int rwkv7_state_forward_f32(void* stream, int B, int T, int H, const float* s0, const float* r, const float* w,
                            const float* k, const float* v, const float* a, const float* b, float* y, float* s,
                            float* sa) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({s0, r, w, k, v, a, b, y, s, sa})) return e;
    return launch7_fwd(stream, true, B, T, H, s0, r, w, k, v, a, b, y, nullptr, s, sa);
}

int rwkv7_state_backward_f32(void* stream, int B, int T, int H, const float* r, const float* w, const float* k,
                             const float* v, const float* a, const float* b, const float* dy, const float* s,
                             const float* sa, float* ds0, float* dr, float* dw, float* dk, float* dv, float* da,
                             float* db) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, s, sa, ds0, dr, dw, dk, dv, da, db})) return e;
    return launch7_bwd(stream, true, B, T, H, r, w, k, v, a, b, dy, nullptr, s, sa, ds0, dr, dw, dk, dv, da, db);
}

int rwkv7_forward_f32(void* stream, int B, int T, int H, const float* r, const float* w, const float* k,
                      const float* v, const float* a, const float* b, float* y, float* s, float* sa) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, y, s, sa})) return e;
    return launch7_fwd(stream, true, B, T, H, nullptr, r, w, k, v, a, b, y, nullptr, s, sa);
}

int rwkv7_backward_f32(void* stream, int B, int T, int H, const float* r, const float* w, const float* k,
                       const float* v, const float* a, const float* b, const float* dy, const float* s,
                       const float* sa, float* dr, float* dw, float* dk, float* dv, float* da, float* db) {
    if (int e = check7(B, T, H)) return e;
    if (int e = check_ptrs({r, w, k, v, a, b, dy, s, sa, dr, dw, dk, dv, da, db})) return e;
    return launch7_bwd(stream, true, B, T, H, r, w, k, v, a, b, dy, nullptr, s, sa, nullptr, dr, dw, dk, dv, da, db);
}

}  // extern "C"
