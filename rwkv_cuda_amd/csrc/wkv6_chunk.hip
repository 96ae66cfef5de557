// wkv6 / wkv6_state, chunked formulation on the matrix cores (gfx950, v_mfma_f32_16x16x32_bf16).
//
// Time is cut into chunks of L = 32 steps.  With lam_t[j] = log w_t[j] <= 0 and the in-chunk
// cumulative sums c_t = sum_{z<t} lam_z (c_0 = 0), everything is referred to the chunk's MIDDLE
// (m = 16) so that neither factor of a product can run away unless 16 consecutive decays shrink a
// channel by more than e^-60 (then the chunk is redone step by step, see `exact`):
//     R'_t = r_t e^{c_t - c_m}        K'_s = k_s e^{c_m - c_{s+1}}
//     Rs_t = r_t e^{c_t}     = R'_t e^{c_m}            (reads the state that entered the chunk)
//     Ke_s = k_s e^{c_L - c_{s+1}} = K'_s e^{c_L - c_m} (carries token s to the end of the chunk)
//     A[t,s] = sum_j R'_t[j] K'_s[j]  (s < t),   A[t,t] = sum_j r_t[j] u[j] k_t[j]
//     Y   = Rs S0^T + A V                               S[i][j]: i value channel, j key channel
//     S_L = S0 diag(e^{c_L}) + V^T Ke
// Every product runs on bf16 MFMA with fp32 accumulation; an fp32 operand x is split into
// hi = bf16(x), lo = bf16(x - hi) (v, gy are exact in bf16 and need no split), which keeps ~16
// mantissa bits per operand -- far below the bf16 rounding of the outputs, which is the error
// the original fp32 kernels have.
//
// The state never leaves the accumulator registers: the accumulator layout of a 16x16 tile
// (lane = column, lane group g and register v = row 4g+v) is used AS IS as the B operand of the
// next chunk's Rs S0^T product, because the K slots of an MFMA may be assigned to channels in any
// order as long as the A operand uses the same order; no transpose is ever needed.
#include "wkv6_chunk.h"

namespace rwkv {
namespace {

// ======================================================================================================================
// Backward, first sweep (time ascending): gr, gu and the workspace r * dr' that the decay gradient needs.
//     dr'_t[j] = sum_i gy_t[i] S_t[i][j] = Ea_t[j] ( e^{c_m}[j] (GY S0)[t][j] + (Bm K')[t][j] ),   Ea_t = e^{c_t - c_m},
//     Bm[t][s] = gy_t . v_s (s < t),   gr = dr' + u k_t (gy_t . v_t),   S_L = S0 diag(e^{c_L}) + diag(e^{c_L - c_m}) V^T K'.
// Wave (q = wid & 3, ih = wid >> 2) owns key channels [16q, 16q+16) and the value-channel half [32ih, 32ih+32) of the
// state S[i][j]: D[m][v] <-> i = 32ih + 16m + 4g + v, lane <-> j, so every decay factor is a per-lane scalar.
// ======================================================================================================================
constexpr int PS = 36;            // row stride (dwords) of plain bf16 [token][channel] arrays: 144 B

struct alignas(16) SmemA {
    uint32_t KpT[N][TS];           // k e^{c_m - c_{s+1}}  hi/lo cells along tokens [j][s]   (exact path: decay as float [t][j])
    uint32_t Bm[L][TS];            // gy_t . v_s (s < t)   hi/lo cells along s      [t][s]
    uint32_t Vt[N][VS];            // v  plain bf16 [i][s]
    uint32_t GY[L][PS];            // gy plain bf16 [t][i]
    uint32_t V[L][PS];             // v  plain bf16 [s][i]
    uint32_t Rr[L][PS], Kr[L][PS]; // r, k plain bf16 [t][j]
    float Ea[L][N];                // e^{c_t - c_m}       (exact path: 1)
    float d1[N], d2[N], dec[N];    // e^{c_m}, e^{c_L - c_m}, e^{c_L}
    float u[N];
    float vgy[2][L];               // gy_t . v_t  (two partial sums)
    float part[8][N];
    uint32_t flag[8];
    float P[2][2][L][RS];          // staging, double buffered: partial dr' of the two value-channel halves
};

template <int WMODE>
__global__ __launch_bounds__(NT) void wkv6_bwd_a_chunk(const ArgsB a) {
    __shared__ SmemA S;
    const int tid = threadIdx.x, lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, g = lane >> 4;
    const int q = wid & 3, ih = wid >> 2;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int T = a.T, C = a.C;
    const size_t base = static_cast<size_t>(b) * T * C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb_ = a.v + base;
    const uint16_t* __restrict__ gb = a.gy + base;
    const int jp = lane & 31, th = lane >> 5, pt0 = 4 * wid + 2 * th;

    if (tid < N) S.u[tid] = bf2f(a.u[h * N + tid]);
    f32x4 D[2];
    D[0] = D[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.s0 != nullptr) {
        const uint16_t* s = a.s0 + bh * N * N + 16 * q + l16;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) D[m][v] = bf2f(s[(32 * ih + 16 * m + 4 * g + v) * N]);
    }
    for (int i = tid; i < L * TS; i += NT) (&S.Bm[0][0])[i] = 0;     // tile (t < 16 <= s) stays zero

    const int nchunks = (T + L - 1) / L;
    struct Raw { uint32_t r[2], k[2], v[2], g[2], w[2][2]; };
    Raw ring[STAGES];
    // Loads are asm so that the wait before their first use can leave the younger batches in flight (the compiler would
    // wait for every outstanding load); each call issues the same ten loads (chunk index clamped), so that count is fixed.
    const uint32_t* __restrict__ wb32 = reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + base);
    const float* __restrict__ wbf = static_cast<const float*>(a.w) + base;
    auto prefetch = [&](int c, Raw& x) __attribute__((always_inline)) {
        c = c < nchunks ? c : nchunks - 1;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = c * L + pt0 + e;
            const uint32_t o = (static_cast<uint32_t>(t < T ? t : T - 1) * C + 2 * jp) * 2;    // byte offset
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.r[e]) : "v"(o), "s"(rb));
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.k[e]) : "v"(o), "s"(kb));
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.v[e]) : "v"(o), "s"(vb_));
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.g[e]) : "v"(o), "s"(gb));
            if constexpr (WMODE == W_RAW) {
                asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.w[e][0]) : "v"(o), "s"(wb32));
            } else {
                uint2 y;
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(y) : "v"(2 * o), "s"(wbf));
                x.w[e][0] = y.x; x.w[e][1] = y.y;
            }
        }
    };
    // the batches of the next STAGES - 1 chunks (ten loads each) may stay in flight
    auto arrived = [&](Raw& x) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%12)" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                     "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.w[0][0]), "+v"(x.w[0][1]), "+v"(x.w[1][0]), "+v"(x.w[1][1]) : "n"(10 * (STAGES - 1)));
    };
    static_for<STAGES>([&](auto Z) { prefetch(decltype(Z)::value, ring[decltype(Z)::value]); });

    float gu_acc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) gu_acc[e] = 0.f;

    auto process = [&](const int c, Raw& x) __attribute__((always_inline)) {
        const int c0 = c * L, buf = c & 1;
        arrived(x);
        float pk[2][2], plam[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const bool ok = (c0 + pt0 + e) < T;
            if (!ok) { x.r[e] = 0; x.k[e] = 0; x.v[e] = 0; x.g[e] = 0; }
            pk[e][0] = bf_lo(x.k[e]); pk[e][1] = bf_hi(x.k[e]);
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                float lam;
                if constexpr (WMODE == W_RAW) lam = -exp2_fast(LOG2E * (z ? bf_hi(x.w[e][0]) : bf_lo(x.w[e][0])));
                else lam = __uint_as_float(x.w[e][z]);
                plam[e][z] = ok ? lam * LOG2E : 0.f;
            }
        }
        float s2[2], s4[2], other[2];
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            s2[z] = plam[0][z] + plam[1][z];
            other[z] = __shfl_xor(s2[z], 32, 64);
            s4[z] = s2[z] + other[z];
        }
        if (th == 0) *reinterpret_cast<float2*>(&S.part[wid][2 * jp]) = make_float2(s4[0], s4[1]);
        {
            const unsigned long long any = __ballot((-s4[0] > 0.25f * RANGE_LIMIT * LOG2E) || (-s4[1] > 0.25f * RANGE_LIMIT * LOG2E));
            if (lane == 0) S.flag[wid] = any != 0ull;
        }
        __syncthreads();
        const uint4 fl0 = *reinterpret_cast<const uint4*>(&S.flag[0]), fl1 = *reinterpret_cast<const uint4*>(&S.flag[4]);
        const bool exact = (fl0.x | fl0.y | fl0.z | fl0.w | fl1.x | fl1.y | fl1.z | fl1.w) != 0;
        float pre[2] = {0.f, 0.f}, cm[2] = {0.f, 0.f}, cl[2] = {0.f, 0.f};
#pragma unroll
        for (int w8 = 0; w8 < 8; ++w8) {
            const float2 y = *reinterpret_cast<const float2*>(&S.part[w8][2 * jp]);
            if (w8 < wid) { pre[0] += y.x; pre[1] += y.y; }
            if (w8 < 4) { cm[0] += y.x; cm[1] += y.y; }
            cl[0] += y.x; cl[1] += y.y;
        }
        if (th) { pre[0] += other[0]; pre[1] += other[1]; }
        if (wid == 0 && th == 0) {
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                S.d1[2 * jp + z] = exp2_fast(cm[z]);
                S.d2[2 * jp + z] = exp2_fast(cl[z] - cm[z]);
                S.dec[2 * jp + z] = exp2_fast(cl[z]);
            }
        }
        if (!exact) {
            float kp[2][2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const float ct0 = pre[z], ct1 = ct0 + plam[0][z], ct2 = ct1 + plam[1][z];
                kp[0][z] = pk[0][z] * exp2_fast(cm[z] - ct1);
                kp[1][z] = pk[1][z] * exp2_fast(cm[z] - ct2);
                S.Ea[pt0][2 * jp + z] = exp2_fast(ct0 - cm[z]);
                S.Ea[pt0 + 1][2 * jp + z] = exp2_fast(ct1 - cm[z]);
                const HL y = hilo2(kp[0][z], kp[1][z]);
                S.KpT[2 * jp + z][4 * wid + th] = y.h;
                S.KpT[2 * jp + z][4 * wid + 2 + th] = y.l;
            }
        } else {
            float* W = reinterpret_cast<float*>(&S.KpT[0][0]);       // decay [t][j]
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<float2*>(&W[(pt0 + e) * N + 2 * jp]) = make_float2(exp2_fast(plam[e][0]), exp2_fast(plam[e][1]));
                *reinterpret_cast<float2*>(&S.Ea[pt0 + e][2 * jp]) = make_float2(1.f, 1.f);
            }
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            S.Rr[pt0 + e][jp] = x.r[e];
            S.Kr[pt0 + e][jp] = x.k[e];
            S.GY[pt0 + e][jp] = x.g[e];
            S.V[pt0 + e][jp] = x.v[e];
        }
        {
            uint16_t* vt = reinterpret_cast<uint16_t*>(&S.Vt[0][0]);
            *reinterpret_cast<uint32_t*>(vt + (2 * jp) * (2 * VS) + pt0) = (x.v[0] & 0xffffu) | (x.v[1] << 16);
            *reinterpret_cast<uint32_t*>(vt + (2 * jp + 1) * (2 * VS) + pt0) = (x.v[0] >> 16) | (x.v[1] & 0xffff0000u);
        }
        __syncthreads();
        prefetch(c + STAGES, x);

        const float d1j = S.d1[16 * q + l16], d2j = S.d2[16 * q + l16], decj = S.dec[16 * q + l16];
        if (!exact) {
            // ---------------------------------------------------------- Bm^T tiles: waves 0,1,2 -> (0,0) (1,0) (1,1)
            if (wid < 3) {
                const int ta = (wid == 0) ? 0 : 1, tb = (wid == 2) ? 1 : 0;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};     // acc[v]: s = 16 tb + 4g + v (rows, from V), t = 16 ta + l16 (from GY)
#pragma unroll
                for (int kk = 0; kk < 2; ++kk)
                    acc = mfma(lds_op(&S.V[16 * tb + l16][16 * kk + 4 * g]), lds_op(&S.GY[16 * ta + l16][16 * kk + 4 * g]), acc);
                if (ta == tb) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int sl = 4 * g + v;
                        if (sl == l16) { S.vgy[0][16 * ta + l16] = acc[v]; S.vgy[1][16 * ta + l16] = 0.f; }
                        acc[v] = (sl < l16) ? acc[v] : 0.f;
                    }
                }
                const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
                *reinterpret_cast<uint4*>(&S.Bm[16 * ta + l16][16 * tb + 4 * g]) = make_uint4(x0.h, x1.h, x0.l, x1.l);
            }
            // ---------------------------------------------------------- (GY S0) over this half of the value channels
            f32x4 A1[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const HL x0 = hilo2(D[m][0], D[m][1]), x1 = hilo2(D[m][2], D[m][3]);
                const bf16x8 sb = as_op(x0.h, x1.h, x0.l, x1.l);
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
                    A1[mt] = mfma(lds_dup(&S.GY[16 * mt + l16][(32 * ih + 16 * m + 4 * g) >> 1]), sb, A1[mt]);
            }
            __syncthreads();                           // Bm is in LDS
            // ---------------------------------------------------------- (Bm K') over the tokens of half ih
            f32x4 A2[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
            const bf16x8 kb0 = lds_op(&S.KpT[16 * q + l16][4 * g]);
            const bf16x8 kb1 = lds_op(&S.KpT[16 * q + l16][16 + 4 * g]);
            if (ih == 0) {
                A2[0] = mfma_full(lds_op(&S.Bm[l16][4 * g]), kb0, A2[0]);
                A2[1] = mfma_full(lds_op(&S.Bm[16 + l16][4 * g]), kb0, A2[1]);
            } else {
                A2[1] = mfma_full(lds_op(&S.Bm[16 + l16][16 + 4 * g]), kb1, A2[1]);
            }
            // ---------------------------------------------------------- S = S diag(dec) + diag(d2) V^T K'
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                f32x4 U = {0.f, 0.f, 0.f, 0.f};
                U = mfma(lds_dup(&S.Vt[32 * ih + 16 * m + l16][2 * g]), kb0, U);
                U = mfma(lds_dup(&S.Vt[32 * ih + 16 * m + l16][8 + 2 * g]), kb1, U);
#pragma unroll
                for (int v = 0; v < 4; ++v) D[m][v] = fmaf(D[m][v], decj, d2j * U[v]);
            }
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) S.P[buf][ih][16 * mt + 4 * g + v][16 * q + l16] = fmaf(d1j, A1[mt][v], A2[mt][v]);
        } else {
            // ---------------------------------------------------------- exact path: 32 sequential steps
            __syncthreads();
            const float* W = reinterpret_cast<const float*>(&S.KpT[0][0]);
            const uint16_t* kr = reinterpret_cast<const uint16_t*>(&S.Kr[0][0]);
            for (int t = 0; t < L; ++t) {
                const float wj = W[t * N + 16 * q + l16], kj = bf2f(kr[t * (2 * PS) + 16 * q + l16]);
                float drp = 0.f, vg = 0.f;
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const int i2 = (32 * ih + 16 * m + 4 * g) >> 1;
                    const uint2 gg = *reinterpret_cast<const uint2*>(&S.GY[t][i2]);
                    const uint2 vv = *reinterpret_cast<const uint2*>(&S.V[t][i2]);
                    const float gyi[4] = {bf_lo(gg.x), bf_hi(gg.x), bf_lo(gg.y), bf_hi(gg.y)};
                    const float vi[4] = {bf_lo(vv.x), bf_hi(vv.x), bf_lo(vv.y), bf_hi(vv.y)};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        drp = fmaf(gyi[v], D[m][v], drp);
                        vg = fmaf(gyi[v], vi[v], vg);
                        D[m][v] = fmaf(D[m][v], wj, kj * vi[v]);
                    }
                }
                drp = allreduce_rows(drp);
                vg = allreduce_rows(vg);
                if (g == 0) S.P[buf][ih][t][16 * q + l16] = drp;
                if (q == 0 && lane == 0) S.vgy[ih][t] = vg;
            }
        }
        __syncthreads();
        {
            const int t = tid >> 4, j0 = (tid & 15) * 4;
            const float4 x0 = *reinterpret_cast<const float4*>(&S.P[buf][0][t][j0]);
            const float4 x1 = *reinterpret_cast<const float4*>(&S.P[buf][1][t][j0]);
            const float4 ea = *reinterpret_cast<const float4*>(&S.Ea[t][j0]);
            const float drp[4] = {(x0.x + x1.x) * ea.x, (x0.y + x1.y) * ea.y, (x0.z + x1.z) * ea.z, (x0.w + x1.w) * ea.w};
            const uint2 rq = *reinterpret_cast<const uint2*>(&S.Rr[t][j0 >> 1]);
            const uint2 kq = *reinterpret_cast<const uint2*>(&S.Kr[t][j0 >> 1]);
            const float rr[4] = {bf_lo(rq.x), bf_hi(rq.x), bf_lo(rq.y), bf_hi(rq.y)};
            const float kk[4] = {bf_lo(kq.x), bf_hi(kq.x), bf_lo(kq.y), bf_hi(kq.y)};
            const float4 uu = *reinterpret_cast<const float4*>(&S.u[j0]);
            const float ue[4] = {uu.x, uu.y, uu.z, uu.w};
            const float vgy = S.vgy[0][t] + S.vgy[1][t];
            float out[4], rdr[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                out[e] = fmaf(ue[e] * kk[e], vgy, drp[e]);
                rdr[e] = rr[e] * drp[e];
                gu_acc[e] = fmaf(rr[e] * kk[e], vgy, gu_acc[e]);
            }
            if (c0 + t < T) {
                const size_t off = base + static_cast<size_t>(c0 + t) * C + j0;
                *reinterpret_cast<uint2*>(a.gr + off) = make_uint2(pack_bf2(out[0], out[1]), pack_bf2(out[2], out[3]));
                *reinterpret_cast<float4*>(a.rdr + off) = make_float4(rdr[0], rdr[1], rdr[2], rdr[3]);
            }
        }
    };

    for (int cb = 0; cb < nchunks; cb += STAGES)
        static_for<STAGES>([&](auto Z) { if (cb + decltype(Z)::value < nchunks) process(cb + decltype(Z)::value, ring[decltype(Z)::value]); });

    // gu[j] = sum over the 32 staging rows of the per-thread accumulators
    __syncthreads();
    {
        float* G = &S.P[0][0][0][0];
#pragma unroll
        for (int e = 0; e < 4; ++e) G[(tid >> 4) * RS + (tid & 15) * 4 + e] = gu_acc[e];
    }
    __syncthreads();
    if (tid < N) {
        const float* G = &S.P[0][0][0][0];
        float s = 0.f;
        for (int t = 0; t < L; ++t) s += G[t * RS + tid];
        a.gu[static_cast<size_t>(b) * C + h * N + tid] = f2bf(s);
    }
}


// ======================================================================================================================
// Backward, second sweep (time descending): gk, gv, gw, gs.  With dS the gradient of the state at the END of the chunk,
//     dk'_s[j] = Eb_s[j] ( e^{c_L - c_m}[j] (V dS)[s][j] + (Bm^T R')[s][j] ),        Eb_s = e^{c_m - c_{s+1}},
//     gv_s[i]  = (K' (diag(e^{c_L - c_m}) dS^T))[s][i] + (A^T GY)[s][i],             A as in the forward, diagonal included,
//     dS_0     = dS diag(e^{c_L}) + diag(e^{c_m}) GY^T R',        gk = dk' + u r_s (gy_s . v_s),
//     G_t = P_{t+1} - k_t dk'_t,  P_t = G_t + (r dr')_t  (P_T = 0),   gw_t = lam_t G_t        (lam = -exp(w_raw)).
// dS is kept twice: D = dS[i][j] sliced by key channel (column sums over i: dk') and E = dS^T[j][i] sliced by value
// channel (row sums over j: gv).  Wave (q = wid & 3, hf = wid >> 2): D[m][v] <-> i = 32hf + 16m + 4g + v, lane <-> j = 16q + l16;
// E[m][v] <-> j = 32hf + 16m + 4g + v, lane <-> i = 16q + l16.  G is a suffix sum over time of (r dr' - k dk'), taken in
// the accumulator layout of dk' (lane = channel, registers and lane groups = time); every term is linear in the two
// halves' partial sums, so each wave scans its own part and only the chunk totals cross waves.
// ======================================================================================================================
constexpr float LN2 = 0.69314718055994530942f;
constexpr int STAGES_B = 2;       // the second sweep carries two copies of the state: fewer input stages fit the registers

struct alignas(16) SmemB {
    uint32_t Rp[L][RS];            // r e^{c_t - c_m}      cells along j  [t][j]   A of A^T tiles
    uint32_t Kp[L][RS];            // k e^{c_m - c_{s+1}}  cells along j  [s][j]   B of A^T tiles, A of K' dS^T  (exact path: decay floats)
    uint32_t RpT[N][TS];           // r e^{c_t - c_m}      cells along t  [j][t]   B of Bm^T R', operand of the dS updates
    uint32_t AmT[L][TS];           // A[tau][s]            cells along tau [s][tau]
    uint32_t BmT[L][TS];           // gy_tau . v_s (s<tau) cells along tau [s][tau]
    uint32_t GYt[N][VS];           // gy plain bf16 [i][t]
    uint32_t GY[L][PS];            // gy plain bf16 [t][i]
    uint32_t V[L][PS];             // v  plain bf16 [s][i]
    uint32_t Rr[L][PS], Kr[L][PS]; // r, k plain bf16 [t][j]
    float Eb[L][N];                // e^{c_m - c_{s+1}}   (exact path: 1)
    float rdr[L][N];               // r dr' from the first sweep
    float lam[L][N];               // -exp(w_raw)
    float X[L][N];                 // r u k
    float d1[N], d2[N], dec[N], u[N];
    float vgy[2][L];
    float ruk[2][L];               // exact path: sum_j r u k (two partial sums)
    float part[8][N];
    uint32_t flag[8];
    float Ptot[2][N];              // chunk totals of (r dr' - k dk'), two partial sums
    float Pk[2][L][RS], Pv[2][L][RS], Pw[2][L][RS];   // staging: partial dk', gv, G of the two halves
};

template <int WMODE>
__global__ __launch_bounds__(NT) void wkv6_bwd_b_chunk(const ArgsB a) {
    __shared__ SmemB S;
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, l16 = lane & 15, g = lane >> 4;
    const int q = wid & 3, hf = wid >> 2;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int T = a.T, C = a.C;
    const size_t base = static_cast<size_t>(b) * T * C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb_ = a.v + base;
    const uint16_t* __restrict__ gb = a.gy + base;
    const float* __restrict__ db = a.rdr + base;
    const int jp = lane & 31, th = lane >> 5, pt0 = 4 * wid + 2 * th;
    const bool stateful = a.s0 != nullptr;
    float uj[2];
    {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.u + h * N + 2 * jp);
        uj[0] = bf_lo(x); uj[1] = bf_hi(x);
    }
    if (tid < N) { S.u[tid] = bf2f(a.u[h * N + tid]); S.Ptot[0][tid] = 0.f; S.Ptot[1][tid] = 0.f; }
    for (int i = tid; i < L * TS; i += NT) { (&S.AmT[0][0])[i] = 0; (&S.BmT[0][0])[i] = 0; }   // tile (s >= 16 > tau) stays zero

    f32x4 D[2], E[2];
    D[0] = D[1] = E[0] = E[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    float Pend = 0.f;                                  // P at the end of the current chunk, channel j = 16q + l16

    const int nchunks = (T + L - 1) / L;
    struct Raw { uint32_t r[2], k[2], v[2], g[2], w[2][2]; float2 d[2]; };
    Raw ring[STAGES_B];
    // asm loads with an explicit wait, as in the first sweep; twelve loads per call
    const uint32_t* __restrict__ wb32 = reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + base);
    const float* __restrict__ wbf = static_cast<const float*>(a.w) + base;
    auto prefetch = [&](int c, Raw& x) __attribute__((always_inline)) {
        c = c > 0 ? c : 0;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = c * L + pt0 + e;
            const uint32_t o = (static_cast<uint32_t>(t < T ? t : T - 1) * C + 2 * jp) * 2;    // byte offset
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.r[e]) : "v"(o), "s"(rb));
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.k[e]) : "v"(o), "s"(kb));
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.v[e]) : "v"(o), "s"(vb_));
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.g[e]) : "v"(o), "s"(gb));
            asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(x.d[e]) : "v"(2 * o), "s"(db));
            if constexpr (WMODE == W_RAW) {
                asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.w[e][0]) : "v"(o), "s"(wb32));
            } else {
                uint2 y;
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(y) : "v"(2 * o), "s"(wbf));
                x.w[e][0] = y.x; x.w[e][1] = y.y;
            }
        }
    };
    auto arrived = [&](Raw& x) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%14)" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                     "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.w[0][0]), "+v"(x.w[0][1]), "+v"(x.w[1][0]), "+v"(x.w[1][1]),
                     "+v"(x.d[0]), "+v"(x.d[1]) : "n"(12 * (STAGES_B - 1)));
    };
    // chunks are visited last to first; ci counts visits
    static_for<STAGES_B>([&](auto Z) { prefetch(nchunks - 1 - decltype(Z)::value, ring[decltype(Z)::value]); });

    auto process = [&](const int ci, Raw& x) __attribute__((always_inline)) {
        const int c = nchunks - 1 - ci, c0 = c * L;
        arrived(x);
        float pr[2][2], pk[2][2], plam[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const bool ok = (c0 + pt0 + e) < T;
            if (!ok) { x.r[e] = 0; x.k[e] = 0; x.v[e] = 0; x.g[e] = 0; x.d[e] = make_float2(0.f, 0.f); }
            pr[e][0] = bf_lo(x.r[e]); pr[e][1] = bf_hi(x.r[e]);
            pk[e][0] = bf_lo(x.k[e]); pk[e][1] = bf_hi(x.k[e]);
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                float lam;
                if constexpr (WMODE == W_RAW) lam = -exp2_fast(LOG2E * (z ? bf_hi(x.w[e][0]) : bf_lo(x.w[e][0])));
                else lam = __uint_as_float(x.w[e][z]);
                plam[e][z] = ok ? lam * LOG2E : 0.f;
            }
        }
        float s2[2], s4[2], other[2];
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            s2[z] = plam[0][z] + plam[1][z];
            other[z] = __shfl_xor(s2[z], 32, 64);
            s4[z] = s2[z] + other[z];
        }
        if (th == 0) *reinterpret_cast<float2*>(&S.part[wid][2 * jp]) = make_float2(s4[0], s4[1]);
        {
            const unsigned long long any = __ballot((-s4[0] > 0.25f * RANGE_LIMIT * LOG2E) || (-s4[1] > 0.25f * RANGE_LIMIT * LOG2E));
            if (lane == 0) S.flag[wid] = any != 0ull;
        }
        __syncthreads();
        const uint4 fl0 = *reinterpret_cast<const uint4*>(&S.flag[0]), fl1 = *reinterpret_cast<const uint4*>(&S.flag[4]);
        const bool exact = (fl0.x | fl0.y | fl0.z | fl0.w | fl1.x | fl1.y | fl1.z | fl1.w) != 0;
        // totals of the chunk processed before this one (later in time) are complete now
        Pend += S.Ptot[0][16 * q + l16] + S.Ptot[1][16 * q + l16];
        float pre[2] = {0.f, 0.f}, cm[2] = {0.f, 0.f}, cl[2] = {0.f, 0.f};
#pragma unroll
        for (int w8 = 0; w8 < 8; ++w8) {
            const float2 y = *reinterpret_cast<const float2*>(&S.part[w8][2 * jp]);
            if (w8 < wid) { pre[0] += y.x; pre[1] += y.y; }
            if (w8 < 4) { cm[0] += y.x; cm[1] += y.y; }
            cl[0] += y.x; cl[1] += y.y;
        }
        if (th) { pre[0] += other[0]; pre[1] += other[1]; }
        if (wid == 0 && th == 0) {
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                S.d1[2 * jp + z] = exp2_fast(cm[z]);
                S.d2[2 * jp + z] = exp2_fast(cl[z] - cm[z]);
                S.dec[2 * jp + z] = exp2_fast(cl[z]);
            }
        }
        if (!exact) {
            float rp[2][2], kp[2][2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const float ct0 = pre[z], ct1 = ct0 + plam[0][z], ct2 = ct1 + plam[1][z];
                const float eb0 = exp2_fast(cm[z] - ct1), eb1 = exp2_fast(cm[z] - ct2);
                rp[0][z] = pr[0][z] * exp2_fast(ct0 - cm[z]);
                rp[1][z] = pr[1][z] * exp2_fast(ct1 - cm[z]);
                kp[0][z] = pk[0][z] * eb0;
                kp[1][z] = pk[1][z] * eb1;
                S.Eb[pt0][2 * jp + z] = eb0;
                S.Eb[pt0 + 1][2 * jp + z] = eb1;
                const HL y = hilo2(rp[0][z], rp[1][z]);
                S.RpT[2 * jp + z][4 * wid + th] = y.h;
                S.RpT[2 * jp + z][4 * wid + 2 + th] = y.l;
            }
            const int ph = hpos(jp);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                HL y = hilo2(rp[e][0], rp[e][1]); S.Rp[pt0 + e][ph] = y.h; S.Rp[pt0 + e][ph + 2] = y.l;
                y = hilo2(kp[e][0], kp[e][1]);    S.Kp[pt0 + e][ph] = y.h; S.Kp[pt0 + e][ph + 2] = y.l;
            }
        } else {
            float* W = reinterpret_cast<float*>(&S.Kp[0][0]);        // decay [t][j]
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<float2*>(&W[(pt0 + e) * N + 2 * jp]) = make_float2(exp2_fast(plam[e][0]), exp2_fast(plam[e][1]));
                *reinterpret_cast<float2*>(&S.Eb[pt0 + e][2 * jp]) = make_float2(1.f, 1.f);
            }
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = pt0 + e;
            S.Rr[t][jp] = x.r[e];
            S.Kr[t][jp] = x.k[e];
            S.GY[t][jp] = x.g[e];
            S.V[t][jp] = x.v[e];
            *reinterpret_cast<float2*>(&S.rdr[t][2 * jp]) = x.d[e];
            *reinterpret_cast<float2*>(&S.lam[t][2 * jp]) = make_float2(plam[e][0] * LN2, plam[e][1] * LN2);
            *reinterpret_cast<float2*>(&S.X[t][2 * jp]) = make_float2(pr[e][0] * uj[0] * pk[e][0], pr[e][1] * uj[1] * pk[e][1]);
        }
        {
            uint16_t* gt = reinterpret_cast<uint16_t*>(&S.GYt[0][0]);
            *reinterpret_cast<uint32_t*>(gt + (2 * jp) * (2 * VS) + pt0) = (x.g[0] & 0xffffu) | (x.g[1] << 16);
            *reinterpret_cast<uint32_t*>(gt + (2 * jp + 1) * (2 * VS) + pt0) = (x.g[0] >> 16) | (x.g[1] & 0xffff0000u);
        }
        __syncthreads();
        prefetch(nchunks - 1 - (ci + STAGES_B), x);

        const int jl = 16 * q + l16;                   // D: this lane's key channel;  E: this lane's value channel
        const float d1j = S.d1[jl], d2j = S.d2[jl], decj = S.dec[jl];
        if (!exact) {
            // ---------------------------------------------------------- tiles: waves 0..2 A^T, waves 3..5 Bm^T
            if (wid < 3) {
                const int ta = (wid == 0) ? 0 : 1, tb = (wid == 2) ? 1 : 0;      // tau tile, s tile
                f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int js = 0; js < 4; js += 2) {     // rows: tau (from R'), columns: s (from K')
                    acc0 = mfma_full(lds_op(&S.Rp[16 * ta + l16][16 * js + 4 * g]), lds_op(&S.Kp[16 * tb + l16][16 * js + 4 * g]), acc0);
                    acc1 = mfma_full(lds_op(&S.Rp[16 * ta + l16][16 * js + 16 + 4 * g]), lds_op(&S.Kp[16 * tb + l16][16 * js + 16 + 4 * g]), acc1);
                }
                f32x4 acc = acc0 + acc1;                // acc[v]: tau = 4g + v, s = l16
                if (ta == tb) {
                    float d = 0.f;                      // sum_j r u k of row s = 16 tb + l16
#pragma unroll
                    for (int z = 0; z < 4; ++z) {
                        const float4 y = *reinterpret_cast<const float4*>(&S.X[16 * tb + l16][16 * g + 4 * z]);
                        d += (y.x + y.y) + (y.z + y.w);
                    }
                    d = allreduce_rows(d);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int tl = 4 * g + v;
                        acc[v] = (l16 < tl) ? acc[v] : (l16 == tl ? d : 0.f);
                    }
                }
                const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
                *reinterpret_cast<uint4*>(&S.AmT[16 * tb + l16][16 * ta + 4 * g]) = make_uint4(x0.h, x1.h, x0.l, x1.l);
            } else if (wid < 6) {
                const int w3 = wid - 3;
                const int ta = (w3 == 0) ? 0 : 1, tb = (w3 == 2) ? 1 : 0;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};     // acc[v]: tau = 16 ta + 4g + v (rows, from GY), s = 16 tb + l16 (from V)
#pragma unroll
                for (int kk = 0; kk < 2; ++kk)
                    acc = mfma(lds_op(&S.GY[16 * ta + l16][16 * kk + 4 * g]), lds_op(&S.V[16 * tb + l16][16 * kk + 4 * g]), acc);
                if (ta == tb) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int tl = 4 * g + v;
                        if (tl == l16) { S.vgy[0][16 * ta + l16] = acc[v]; S.vgy[1][16 * ta + l16] = 0.f; }
                        acc[v] = (l16 < tl) ? acc[v] : 0.f;
                    }
                }
                const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
                *reinterpret_cast<uint4*>(&S.BmT[16 * tb + l16][16 * ta + 4 * g]) = make_uint4(x0.h, x1.h, x0.l, x1.l);
            }
            // ---------------------------------------------------------- state products of this half
            f32x4 K1[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};   // (V dS)[s][j], i in this half
            f32x4 V3[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};   // (K' diag(d2) dS^T)[s][i], j in this half
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                {
                    const HL x0 = hilo2(D[m][0], D[m][1]), x1 = hilo2(D[m][2], D[m][3]);
                    const bf16x8 sb = as_op(x0.h, x1.h, x0.l, x1.l);
#pragma unroll
                    for (int st = 0; st < 2; ++st)
                        K1[st] = mfma(lds_dup(&S.V[16 * st + l16][(32 * hf + 16 * m + 4 * g) >> 1]), sb, K1[st]);
                }
                {
                    const int j0 = 32 * hf + 16 * m + 4 * g;
                    const float4 dd = *reinterpret_cast<const float4*>(&S.d2[j0]);
                    const HL x0 = hilo2(E[m][0] * dd.x, E[m][1] * dd.y), x1 = hilo2(E[m][2] * dd.z, E[m][3] * dd.w);
                    const bf16x8 sb = as_op(x0.h, x1.h, x0.l, x1.l);
#pragma unroll
                    for (int st = 0; st < 2; ++st)
                        V3[st] = mfma_full(lds_op(&S.Kp[16 * st + l16][32 * hf + 16 * m + 4 * g]), sb, V3[st]);
                }
            }
            // ---------------------------------------------------------- state updates (do not need the tiles)
            const bf16x8 rb0 = lds_op(&S.RpT[jl][4 * g]), rb1 = lds_op(&S.RpT[jl][16 + 4 * g]);          // B: j = jl, tokens
            const bf16x8 gd0 = lds_dup(&S.GYt[jl][2 * g]), gd1 = lds_dup(&S.GYt[jl][8 + 2 * g]);          // B: i = jl, tokens
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                // D[i][j] = D dec_j + d1_j sum_t gy_t[i] R'_t[j]
                const int i0 = 32 * hf + 16 * m + l16;
                f32x4 U = {0.f, 0.f, 0.f, 0.f};
                U = mfma(lds_dup(&S.GYt[i0][2 * g]), rb0, U);
                U = mfma(lds_dup(&S.GYt[i0][8 + 2 * g]), rb1, U);
#pragma unroll
                for (int v = 0; v < 4; ++v) D[m][v] = fmaf(D[m][v], decj, d1j * U[v]);
                // E[j][i] = E dec_j + d1_j sum_t R'_t[j] gy_t[i]      (j runs over the registers)
                const int j0 = 32 * hf + 16 * m;
                f32x4 W2 = {0.f, 0.f, 0.f, 0.f};
                W2 = mfma(lds_op(&S.RpT[j0 + l16][4 * g]), gd0, W2);
                W2 = mfma(lds_op(&S.RpT[j0 + l16][16 + 4 * g]), gd1, W2);
                const float4 de = *reinterpret_cast<const float4*>(&S.dec[j0 + 4 * g]);
                const float4 d1 = *reinterpret_cast<const float4*>(&S.d1[j0 + 4 * g]);
                E[m][0] = fmaf(E[m][0], de.x, d1.x * W2[0]); E[m][1] = fmaf(E[m][1], de.y, d1.y * W2[1]);
                E[m][2] = fmaf(E[m][2], de.z, d1.z * W2[2]); E[m][3] = fmaf(E[m][3], de.w, d1.w * W2[3]);
            }
            __syncthreads();                           // tiles are in LDS
            // ---------------------------------------------------------- tile products over the tokens tau of half hf
            f32x4 K2[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};   // (Bm^T R')[s][j]
            if (hf == 0) {
                K2[0] = mfma_full(lds_op(&S.BmT[l16][4 * g]), rb0, K2[0]);
                V3[0] = mfma(lds_op(&S.AmT[l16][4 * g]), gd0, V3[0]);
            } else {
                K2[0] = mfma_full(lds_op(&S.BmT[l16][16 + 4 * g]), rb1, K2[0]);
                K2[1] = mfma_full(lds_op(&S.BmT[16 + l16][16 + 4 * g]), rb1, K2[1]);
                V3[0] = mfma(lds_op(&S.AmT[l16][16 + 4 * g]), gd1, V3[0]);
                V3[1] = mfma(lds_op(&S.AmT[16 + l16][16 + 4 * g]), gd1, V3[1]);
            }
            // ---------------------------------------------------------- decay gradient: suffix sum in the layout of dk'
            // this lane: channel j = jl, tokens s = 16 st + 4 g + v
            const uint16_t* kr = reinterpret_cast<const uint16_t*>(&S.Kr[0][0]);
            float dlt[2][4], zz[2][4];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int s_ = 16 * st + 4 * g + v;
                    const float dkp = fmaf(d2j, K1[st][v], K2[st][v]);
                    K1[st][v] = dkp;                                          // partial dk' before the Eb factor
                    zz[st][v] = dkp * S.Eb[s_][jl] * bf2f(kr[s_ * (2 * PS) + jl]);   // partial k dk'
                    dlt[st][v] = (hf == 0 ? S.rdr[s_][jl] : 0.f) - zz[st][v];
                }
            float sfx[2][4], tot[2];                   // sfx: sum of dlt over the later tokens of this lane's 4
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                sfx[st][3] = 0.f;
                sfx[st][2] = dlt[st][3];
                sfx[st][1] = dlt[st][2] + sfx[st][2];
                sfx[st][0] = dlt[st][1] + sfx[st][1];
                tot[st] = dlt[st][0] + sfx[st][0];
            }
            float later[2];                            // sum over the lane groups holding later tokens of the same tile
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const float a1 = __shfl_down(tot[st], 16, 64), a2 = __shfl_down(tot[st], 32, 64), a3 = __shfl_down(tot[st], 48, 64);
                later[st] = (g < 3 ? a1 : 0.f) + (g < 2 ? a2 : 0.f) + (g < 1 ? a3 : 0.f);
            }
            const float all1 = allreduce_rows(tot[1]), all0 = allreduce_rows(tot[0]);
            if (g == 0) S.Ptot[hf][jl] = all0 + all1;
            const float p0 = (hf == 0) ? Pend : 0.f;
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int s_ = 16 * st + 4 * g + v;
                    const float Gp = p0 + sfx[st][v] + later[st] + (st == 0 ? all1 : 0.f) - zz[st][v];
                    S.Pw[hf][s_][jl] = Gp;
                    S.Pk[hf][s_][jl] = K1[st][v];
                    S.Pv[hf][s_][jl] = V3[st][v];
                }
        } else {
            // ---------------------------------------------------------- exact path: 32 sequential steps, time descending
            __syncthreads();
            const float* W = reinterpret_cast<const float*>(&S.Kp[0][0]);
            const uint16_t* kr = reinterpret_cast<const uint16_t*>(&S.Kr[0][0]);
            const uint16_t* rr = reinterpret_cast<const uint16_t*>(&S.Rr[0][0]);
            const uint16_t* gyr = reinterpret_cast<const uint16_t*>(&S.GY[0][0]);
            const uint16_t* vr = reinterpret_cast<const uint16_t*>(&S.V[0][0]);
            float Pp = (hf == 0) ? Pend : 0.f;
            for (int t = L - 1; t >= 0; --t) {
                // D side: lane = key channel jl, registers = value channels of this half
                const float wj = W[t * N + jl], kj = bf2f(kr[t * (2 * PS) + jl]), rj = bf2f(rr[t * (2 * PS) + jl]);
                // E side: lane = value channel jl, registers = key channels of this half
                const float gyi = bf2f(gyr[t * (2 * PS) + jl]);
                float dkp = 0.f, dvp = 0.f, vg = 0.f, ruk = 0.f;
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const int c4 = 32 * hf + 16 * m + 4 * g;
                    const uint2 gg = *reinterpret_cast<const uint2*>(gyr + t * (2 * PS) + c4);
                    const uint2 vv = *reinterpret_cast<const uint2*>(vr + t * (2 * PS) + c4);
                    const uint2 k2 = *reinterpret_cast<const uint2*>(kr + t * (2 * PS) + c4);
                    const uint2 r2 = *reinterpret_cast<const uint2*>(rr + t * (2 * PS) + c4);
                    const float4 w4 = *reinterpret_cast<const float4*>(&W[t * N + c4]);
                    const float4 u4 = *reinterpret_cast<const float4*>(&S.u[c4]);
                    const float gy4[4] = {bf_lo(gg.x), bf_hi(gg.x), bf_lo(gg.y), bf_hi(gg.y)};
                    const float v4[4] = {bf_lo(vv.x), bf_hi(vv.x), bf_lo(vv.y), bf_hi(vv.y)};
                    const float k4[4] = {bf_lo(k2.x), bf_hi(k2.x), bf_lo(k2.y), bf_hi(k2.y)};
                    const float r4[4] = {bf_lo(r2.x), bf_hi(r2.x), bf_lo(r2.y), bf_hi(r2.y)};
                    const float ww[4] = {w4.x, w4.y, w4.z, w4.w}, uu[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        dkp = fmaf(v4[v], D[m][v], dkp);              // sum_i v_i dS[i][j]
                        vg = fmaf(v4[v], gy4[v], vg);
                        D[m][v] = fmaf(D[m][v], wj, gy4[v] * rj);
                        dvp = fmaf(k4[v], E[m][v], dvp);              // sum_j k_j dS[i][j]
                        ruk = fmaf(r4[v] * uu[v], k4[v], ruk);
                        E[m][v] = fmaf(E[m][v], ww[v], r4[v] * gyi);
                    }
                }
                dkp = allreduce_rows(dkp); dvp = allreduce_rows(dvp); vg = allreduce_rows(vg); ruk = allreduce_rows(ruk);
                const float z = kj * dkp;
                const float Gp = Pp - z;
                Pp = Gp + (hf == 0 ? S.rdr[t][jl] : 0.f);
                if (g == 0) { S.Pk[hf][t][jl] = dkp; S.Pv[hf][t][jl] = dvp; S.Pw[hf][t][jl] = Gp; }
                if (q == 0 && lane == 0) { S.vgy[hf][t] = vg; S.ruk[hf][t] = ruk; }
            }
            if (g == 0) S.Ptot[hf][jl] = Pp - ((hf == 0) ? Pend : 0.f);
        }
        __syncthreads();
        {
            const int t = tid >> 4, j0 = (tid & 15) * 4;
            const float4 k0 = *reinterpret_cast<const float4*>(&S.Pk[0][t][j0]);
            const float4 k1 = *reinterpret_cast<const float4*>(&S.Pk[1][t][j0]);
            const float4 eb = *reinterpret_cast<const float4*>(&S.Eb[t][j0]);
            float dk[4] = {(k0.x + k1.x) * eb.x, (k0.y + k1.y) * eb.y, (k0.z + k1.z) * eb.z, (k0.w + k1.w) * eb.w};
            const float4 v0 = *reinterpret_cast<const float4*>(&S.Pv[0][t][j0]);
            const float4 v1 = *reinterpret_cast<const float4*>(&S.Pv[1][t][j0]);
            float dv[4] = {v0.x + v1.x, v0.y + v1.y, v0.z + v1.z, v0.w + v1.w};
            const float4 w0 = *reinterpret_cast<const float4*>(&S.Pw[0][t][j0]);
            const float4 w1 = *reinterpret_cast<const float4*>(&S.Pw[1][t][j0]);
            const float4 lm = *reinterpret_cast<const float4*>(&S.lam[t][j0]);
            float gw[4] = {(w0.x + w1.x) * lm.x, (w0.y + w1.y) * lm.y, (w0.z + w1.z) * lm.z, (w0.w + w1.w) * lm.w};
            const uint2 rq = *reinterpret_cast<const uint2*>(&S.Rr[t][j0 >> 1]);
            const float rr[4] = {bf_lo(rq.x), bf_hi(rq.x), bf_lo(rq.y), bf_hi(rq.y)};
            const float4 uu = *reinterpret_cast<const float4*>(&S.u[j0]);
            const float ue[4] = {uu.x, uu.y, uu.z, uu.w};
            const float vgy = S.vgy[0][t] + S.vgy[1][t];
            if (exact) {                               // the bonus term of gv is not inside a tile here
                const uint2 gq = *reinterpret_cast<const uint2*>(&S.GY[t][j0 >> 1]);
                const float gg[4] = {bf_lo(gq.x), bf_hi(gq.x), bf_lo(gq.y), bf_hi(gq.y)};
                const float ruk = S.ruk[0][t] + S.ruk[1][t];
#pragma unroll
                for (int e = 0; e < 4; ++e) dv[e] = fmaf(gg[e], ruk, dv[e]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) dk[e] = fmaf(ue[e] * rr[e], vgy, dk[e]);
            if (!stateful && c0 + t == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) gw[e] = 0.f;              // S_0 = 0: exact zero, as the reference leaves it
            }
            if (c0 + t < T) {
                const size_t off = base + static_cast<size_t>(c0 + t) * C + j0;
                *reinterpret_cast<uint2*>(a.gk + off) = make_uint2(pack_bf2(dk[0], dk[1]), pack_bf2(dk[2], dk[3]));
                *reinterpret_cast<uint2*>(a.gv + off) = make_uint2(pack_bf2(dv[0], dv[1]), pack_bf2(dv[2], dv[3]));
                *reinterpret_cast<uint2*>(a.gw + off) = make_uint2(pack_bf2(gw[0], gw[1]), pack_bf2(gw[2], gw[3]));
            }
        }
    };

    for (int cb = 0; cb < nchunks; cb += STAGES_B)
        static_for<STAGES_B>([&](auto Z) { if (cb + decltype(Z)::value < nchunks) process(cb + decltype(Z)::value, ring[decltype(Z)::value]); });

    if (a.gs != nullptr) {
        uint16_t* s = a.gs + bh * N * N + 16 * q + l16;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) s[(32 * hf + 16 * m + 4 * g + v) * N] = f2bf(D[m][v]);
    }
}

}  // namespace

// Launchers used by wkv56.hip's entry points.
int launch_wkv6_bwd_a_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                            const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                            const uint16_t* s0, const uint16_t* gy, uint16_t* gr, uint16_t* gu, float* rdr) {
    ArgsB a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.gy = gy;
    a.gr = gr; a.gu = gu; a.rdr = rdr;
    if (wmode == W_RAW) hipLaunchKernelGGL(wkv6_bwd_a_chunk<W_RAW>, dim3(B * H), dim3(NT), 0, st, a);
    else hipLaunchKernelGGL(wkv6_bwd_a_chunk<W_EW>, dim3(B * H), dim3(NT), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
