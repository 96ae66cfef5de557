// wkv6 / wkv6_state backward, second sweep (time descending): gk, gv, gw, gs.  Wave-specialised workgroup (gfx950).
//
// With dS the gradient of the state at the END of a chunk (formulas and symbols as in wkv6_chunk.h):
//     dk'_s[j] = Eb_s[j] ( d2[j] (V dS)[s][j] + sum_{tau>s} Bm[tau][s] R'_tau[j] ),    Bm[tau][s] = gy_tau . v_s,  Eb_s = e^{c_m - c_{s+1}}
//     gv_s[i]  = sum_j K'_s[j] d2[j] dS[i][j] + sum_{tau>=s} A[tau][s] gy_tau[i],      A as in the forward, diagonal included
//     dS_0     = dS diag(dec) + diag(d1) GY^T R',                                       gk = dk' + u r_s (gy_s . v_s)
//     G_t = P_{t+1} - k_t dk'_t,   P_t = G_t + (r dr')_t  (P_T = 0),   gw_t = lam_t G_t   (lam = -exp(w_raw); r dr' from the first sweep)
// One workgroup of 16 waves per (batch, head):
//   waves 0..7   ("prep")  load the inputs ahead of time, take the decay sums and write R', K' (hi / lo bf16 planes), r, k, v, gy,
//                          Eb and lam into LDS in natural [token][channel] layout; waves 0..5 form the two causal tiles.
//   waves 8..11  ("D")     wave q keeps dS[i][j] for key channels j in [16q, 16q+16) (lane = j, registers = all 64 i):
//                          dk' with a lane per TOKEN and four consecutive key channels per lane, the time scan of G across
//                          lanes, gk and gw stored from registers.
//   waves 12..15 ("E")     wave q keeps dS^T[j][i] for value channels i in [16q, 16q+16): gv the same way.
// Operands whose contraction runs over tokens (gy and R' in the state update and in the tile products) are transposed on
// the matrix cores by a one-hot selection matrix, exactly as in the forward kernel; the K-slot conventions are the same:
//   state tile m, row 4g+v  <->  channel 32 (m>>1) + 8g + 4 (m&1) + v;   token slot (g, e) <-> token 16 (e>>2) + 4g + (e&3);
//   the tiles are stored as [s][position of tau], position = 8 ((tau&15)>>2) + 4 (tau>>4) + (tau&3).
// Two barriers per chunk:  [tiles(i) | first half of operands(i+1) | state products, update]  B  [scan(i+2), second half of
// operands(i+1) | tile products, epilogue, stores]  B.   i counts visits; chunk c = nchunks - 1 - i.
#include "wkv6_chunk.h"

namespace rwkv {
namespace {

constexpr int NPREP = 8;
constexpr int NTB = 1024;
constexpr int STB = 3;            // visits of input kept in flight

struct alignas(16) SetB {
    uint32_t RpH[L][OS], RpL[L][OS];   // r e^{c_t - c_m}      hi, lo   (exact path: r as fp32 [t][N] over both planes)
    uint32_t KpH[L][OS], KpL[L][OS];   // k e^{c_m - c_{s+1}}  hi, lo   (exact path: k as fp32)
    uint32_t Rr[L][OS];                // r
    uint32_t V[L][OS], GY[L][OS];      // v, gy
    float Eb[L][FS];                   // e^{c_m - c_{s+1}}             (exact path: decay of each step)
    float lam[L][FS];                  // -exp(w_raw)
    float rdr[L][FS];                  // r dr' from the first sweep
    float d1[N], d2[N], dec[N];        // e^{c_m}, e^{c_L - c_m}, e^{c_L}
    float diag[L];                     // sum_j r u k
    uint32_t exact, pad[3];
};

struct alignas(16) SmemB2 {
    SetB set[2];
    uint32_t AmH[L][AS], AmL[L][AS];   // A[tau][s]  as [s][position of tau], hi and lo
    uint32_t BmH[L][AS], BmL[L][AS];   // Bm[tau][s] (s < tau) likewise
    uint4 sel[2][64];                  // selection operands per lane, tile parity 0 and 1
    uint4 TR[4][2][64];                // R'^T tile m (hi, lo): lane = row r of the tile, K slots = tokens; written by D wave m
    uint4 TG[4][64];                   // gy^T tile m likewise; written by E wave m
    float vgy[L];                      // gy_s . v_s
    float u[N];
    float pc[N];                       // P per channel, when it changes layout around an exact chunk
    float part[2][NPREP][N];
};

// ---------------------------------------------------------------------------------------------------- prep waves
// base, h: where r, k, w, u and r dr' of this workgroup sit; vbase: where v, gy sit (the same place unless the head is split)
template <int WMODE>
DEVINL void bwd_prep(SmemB2& S, const ArgsB& a, const int tid, const size_t base, const size_t vbase, const int h, const int nchunks) {
    const int lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb = a.v + vbase;
    const uint16_t* __restrict__ gb = a.gy + vbase;
    // channel pair (2 jp, 2 jp + 1), tokens 4 wid + 2 th + {0, 1}
    const int jp = lane & 31, th = lane >> 5, pt0 = 4 * wid + 2 * th;
    const bool second = wid >= 4;
    float uj[2];
    {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.u + h * N + 2 * jp);
        uj[0] = bf_lo(x); uj[1] = bf_hi(x);
    }
    struct Raw { uint32_t r[2], k[2], v[2], g[2], w[2]; uint2 wq[2]; float2 d[2]; float lam[2][2], other[2], kp[2][2]; };
    Raw ring[STB];
    // The inputs are read once and never again by this kernel: the loads carry the non-temporal hint (measured -3.5 %).
    // Loads are asm so that the wait before their first use can leave the younger batches in flight; every call issues the
    // same twelve loads (visit index clamped), which keeps the count fixed.  Visit ci reads chunk nchunks - 1 - ci.
    const uint32_t* __restrict__ wb32 = reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + base);
    const float* __restrict__ wbf = static_cast<const float*>(a.w) + base;
    const float* __restrict__ db = a.rdr + base;
    auto prefetch = [&](int ci, Raw& x) __attribute__((always_inline)) {
        const int c = ci < nchunks ? nchunks - 1 - ci : 0;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = c * L + pt0 + e;
            const uint32_t o = (static_cast<uint32_t>(t < T ? t : T - 1) * C + 2 * jp) * 2;    // byte offset of the channel pair
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.r[e]) : "v"(o), "s"(rb) : "memory");
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.k[e]) : "v"(o), "s"(kb) : "memory");
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.v[e]) : "v"(o), "s"(vb) : "memory");
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.g[e]) : "v"(o), "s"(gb) : "memory");
            asm volatile("global_load_dwordx2 %0, %1, %2 nt" : "=&v"(x.d[e]) : "v"(2 * o), "s"(db) : "memory");
            if constexpr (WMODE == W_RAW) {
                asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.w[e]) : "v"(o), "s"(wb32) : "memory");
            } else if constexpr (WMODE == W_EW) {
                // straight into the ring: a copy here would read the register before the load has landed
                asm volatile("global_load_dwordx2 %0, %1, %2 nt" : "=&v"(x.wq[e]) : "v"(2 * o), "s"(wbf) : "memory");
            }
        }
    };
    constexpr int NLOADS = WMODE == W_HEAD ? 10 : 12;  // loads per prefetch call
    auto arrived = [&](Raw& x, auto younger) __attribute__((always_inline)) {
        if constexpr (WMODE == W_RAW)
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.w[0]), "+v"(x.w[1]), "+v"(x.d[0]), "+v"(x.d[1])
                         : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
        else if constexpr (WMODE == W_EW)
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.wq[0]), "+v"(x.wq[1]), "+v"(x.d[0]), "+v"(x.d[1])
                         : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.d[0]), "+v"(x.d[1]) : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
    };
    // wkv5: one decay per channel for the whole sequence, given as ew = -exp(w_raw) = log of the decay
    float lamc[2] = {0.f, 0.f};
    if constexpr (WMODE == W_HEAD) {
        const float2 e2 = *reinterpret_cast<const float2*>(static_cast<const float*>(a.w) + h * N + 2 * jp);
        lamc[0] = LOG2E * e2.x; lamc[1] = LOG2E * e2.y;
    }
    static_for<STB>([&](auto Z) { prefetch(decltype(Z)::value, ring[decltype(Z)::value]); });

    // ---- scan of visit ci: lam (log2 units) of this thread's four elements, sums over each eighth of the chunk
    auto scan = [&](const int ci, Raw& x) __attribute__((always_inline)) {
        const int c0 = (nchunks - 1 - ci) * L, pb = ci & 1;
        if (c0 + L > T) {                              // last, partial chunk: rows past T carry no input and no decay
#pragma unroll
            for (int e = 0; e < 2; ++e)
                if (c0 + pt0 + e >= T) {
                    x.r[e] = 0; x.k[e] = 0; x.v[e] = 0; x.g[e] = 0; x.d[e] = make_float2(0.f, 0.f);
                    if constexpr (WMODE == W_RAW) x.w[e] = 0xff80ff80u;   // w = -inf  ->  lam = -exp(w) = 0
                    if constexpr (WMODE == W_EW) x.wq[e] = make_uint2(0u, 0u);
                }
        }
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                if constexpr (WMODE == W_RAW) x.lam[e][z] = -LOG2E * exp2_fast(LOG2E * (z ? bf_hi(x.w[e]) : bf_lo(x.w[e])));
                else if constexpr (WMODE == W_EW) x.lam[e][z] = LOG2E * __uint_as_float(z ? x.wq[e].y : x.wq[e].x);
                else x.lam[e][z] = (c0 + pt0 + e < T) ? lamc[z] : 0.f;
            }
        float s2[2];
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            s2[z] = x.lam[0][z] + x.lam[1][z];
            x.other[z] = __shfl_xor(s2[z], 32, 64);    // the other two tokens of this wave's four
        }
        const float s4a = s2[0] + x.other[0], s4b = s2[1] + x.other[1];
        *reinterpret_cast<float2*>(&S.part[pb][wid][2 * jp]) = make_float2(s4a, s4b);   // both half-waves hold the same sums
    };

    // ---- operands of visit ci into set ci & 1, first part: R' planes, Eb, plain r (K' values stay in registers)
    auto operands_a = [&](const int ci, Raw& x) __attribute__((always_inline)) -> bool {
        SetB& O = S.set[ci & 1];
        const int pb = ci & 1;
        float2 pe[4], po[4];
#pragma unroll
        for (int w4 = 0; w4 < 4; ++w4) {
            pe[w4] = *reinterpret_cast<const float2*>(&S.part[pb][4 * second + w4][2 * jp]);
            po[w4] = *reinterpret_cast<const float2*>(&S.part[pb][4 * !second + w4][2 * jp]);
        }
        const bool exact = chunk_needs_exact_path(pe, po);                       // the same in every wave: a scalar
        if (tid == 0) O.exact = exact;
        float near[2];
        near[0] = second ? (th ? x.other[0] : 0.f) : (th ? 0.f : x.other[0]);
        near[1] = second ? (th ? x.other[1] : 0.f) : (th ? 0.f : x.other[1]);
        {   // eighths between this wave's and the middle: first half w_own+1..3, second half 0..w_own-1 (scalar branches)
            const int w_own = wid & 3;
            const int lo = second ? 0 : w_own + 1, hi = second ? w_own : 4;
            if (lo <= 0 && 0 < hi) { near[0] += pe[0].x; near[1] += pe[0].y; }
            if (lo <= 1 && 1 < hi) { near[0] += pe[1].x; near[1] += pe[1].y; }
            if (lo <= 2 && 2 < hi) { near[0] += pe[2].x; near[1] += pe[2].y; }
            if (lo <= 3 && 3 < hi) { near[0] += pe[3].x; near[1] += pe[3].y; }
        }
        float pr[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) { pr[e][0] = bf_lo(x.r[e]); pr[e][1] = bf_hi(x.r[e]); }
        if (!exact) {
            float rp[2][2], eb[2][2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const Scale sc = chunk_scale(second, near[z], x.lam[0][z], x.lam[1][z]);
                rp[0][z] = pr[0][z] * sc.ea[0]; rp[1][z] = pr[1][z] * sc.ea[1];
                eb[0][z] = sc.eb[0]; eb[1][z] = sc.eb[1];
                x.kp[0][z] = (z ? bf_hi(x.k[0]) : bf_lo(x.k[0])) * sc.eb[0];
                x.kp[1][z] = (z ? bf_hi(x.k[1]) : bf_lo(x.k[1])) * sc.eb[1];
            }
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const HL y = hilo2(rp[e][0], rp[e][1]);
                O.RpH[pt0 + e][jp] = y.h; O.RpL[pt0 + e][jp] = y.l;
                *reinterpret_cast<float2*>(&O.Eb[pt0 + e][2 * jp]) = make_float2(eb[e][0], eb[e][1]);
            }
        } else {
            float* R = reinterpret_cast<float*>(&O.RpH[0][0]);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<float2*>(&R[(pt0 + e) * N + 2 * jp]) = make_float2(pr[e][0], pr[e][1]);
                *reinterpret_cast<float2*>(&O.Eb[pt0 + e][2 * jp]) = make_float2(exp2_fast(x.lam[e][0]), exp2_fast(x.lam[e][1]));
            }
        }
        O.Rr[pt0][jp] = x.r[0];
        O.Rr[pt0 + 1][jp] = x.r[1];
        return exact;
    };
    // ---- second part: K' planes, k, v, gy, lam, the diagonal of A; wave 3 adds the per-channel factors of the chunk
    auto operands_b = [&](const int ci, Raw& x, const bool exact) __attribute__((always_inline)) {
        SetB& O = S.set[ci & 1];
        const int pb = ci & 1;
        float pk[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) { pk[e][0] = bf_lo(x.k[e]); pk[e][1] = bf_hi(x.k[e]); }
        if (!exact) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const HL y = hilo2(x.kp[e][0], x.kp[e][1]);
                O.KpH[pt0 + e][jp] = y.h; O.KpL[pt0 + e][jp] = y.l;
                const float d = half_wave_sum(fmaf(bf_lo(x.r[e]) * uj[0], pk[e][0], bf_hi(x.r[e]) * uj[1] * pk[e][1]));
                if (jp == 31) O.diag[pt0 + e] = d;
            }
        } else {
            float* K = reinterpret_cast<float*>(&O.KpH[0][0]);
#pragma unroll
            for (int e = 0; e < 2; ++e) *reinterpret_cast<float2*>(&K[(pt0 + e) * N + 2 * jp]) = make_float2(pk[e][0], pk[e][1]);
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            *reinterpret_cast<float2*>(&O.rdr[pt0 + e][2 * jp]) = x.d[e];
            O.V[pt0 + e][jp] = x.v[e];
            O.GY[pt0 + e][jp] = x.g[e];
            *reinterpret_cast<float2*>(&O.lam[pt0 + e][2 * jp]) = make_float2(gw_factor(x.lam[e][0] * LN2), gw_factor(x.lam[e][1] * LN2));
        }
        if (wid == 3 && th == 0) {
            float cm[2] = {0.f, 0.f}, ch[2] = {0.f, 0.f};
#pragma unroll
            for (int w8 = 0; w8 < 4; ++w8) {
                const float2 y0 = *reinterpret_cast<const float2*>(&S.part[pb][w8][2 * jp]);
                const float2 y1 = *reinterpret_cast<const float2*>(&S.part[pb][4 + w8][2 * jp]);
                cm[0] += y0.x; cm[1] += y0.y; ch[0] += y1.x; ch[1] += y1.y;
            }
            *reinterpret_cast<float2*>(&O.d1[2 * jp]) = make_float2(exp2_fast(cm[0]), exp2_fast(cm[1]));
            *reinterpret_cast<float2*>(&O.d2[2 * jp]) = make_float2(exp2_fast(ch[0]), exp2_fast(ch[1]));
            *reinterpret_cast<float2*>(&O.dec[2 * jp]) = make_float2(exp2_fast(cm[0] + ch[0]), exp2_fast(cm[1] + ch[1]));
        }
    };

    // ---- causal tiles of visit ci: waves 0..2 A, waves 3..5 Bm; quadrants (tau tile, s tile) = (0,0) (1,0) (1,1).
    //      Accumulator rows are tau, lanes are s; stored as [s][position of tau].
    auto tiles = [&](const int ci) __attribute__((always_inline)) {
        const SetB& O = S.set[ci & 1];
        const int w3 = wid < 3 ? wid : wid - 3;
        const int ta = (w3 == 0) ? 0 : 1, tb = (w3 == 2) ? 1 : 0;          // tau tile, s tile
        f32x4 acc;
        if (wid < 3) {
            f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const bf16x8 rh = lds_op(&O.RpH[16 * ta + l16][16 * ks + 4 * g]), rl = lds_op(&O.RpL[16 * ta + l16][16 * ks + 4 * g]);
                const bf16x8 kh = lds_op(&O.KpH[16 * tb + l16][16 * ks + 4 * g]), kl = lds_op(&O.KpL[16 * tb + l16][16 * ks + 4 * g]);
                acc0 = mfma(rh, kh, acc0);
                acc1 = mfma(rh, kl, acc1);
                acc1 = mfma(rl, kh, acc1);
            }
            acc = acc0 + acc1;                          // acc[v]: tau = 16 ta + 4g + v, s = 16 tb + l16
            if (ta == tb) {
                const float d = O.diag[16 * tb + l16];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int tl = 4 * g + v;
                    acc[v] = (l16 < tl) ? acc[v] : (l16 == tl ? d : 0.f);
                }
            }
        } else {
            acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
                acc = mfma(lds_op(&O.GY[16 * ta + l16][16 * ks + 4 * g]), lds_op(&O.V[16 * tb + l16][16 * ks + 4 * g]), acc);
            if (ta == tb) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int tl = 4 * g + v;
                    if (tl == l16) S.vgy[16 * tb + l16] = acc[v];
                    acc[v] = (l16 < tl) ? acc[v] : 0.f;
                }
            }
        }
        const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
        uint32_t* H = wid < 3 ? &S.AmH[0][0] : &S.BmH[0][0];
        uint32_t* Lo = wid < 3 ? &S.AmL[0][0] : &S.BmL[0][0];
        *reinterpret_cast<uint2*>(&H[(16 * tb + l16) * AS + 4 * g + 2 * ta]) = make_uint2(x0.h, x1.h);
        *reinterpret_cast<uint2*>(&Lo[(16 * tb + l16) * AS + 4 * g + 2 * ta]) = make_uint2(x0.l, x1.l);
    };

    static_for<STB>([&](auto Z) { arrived(ring[decltype(Z)::value], std::integral_constant<int, 0>{}); });
    scan(0, ring[0]);
    if (nchunks > 1) scan(1, ring[1]);
    __syncthreads();
    bool exact_cur = operands_a(0, ring[0]);
    operands_b(0, ring[0], exact_cur);
    prefetch(STB, ring[0]);
    __syncthreads();
    for (int ib = 0; ib < nchunks; ib += STB)
        static_for<STB>([&](auto Z) {
            constexpr int z = decltype(Z)::value;
            const int i = ib + z;
            if (i < nchunks) {
                if (wid < 6 && !exact_cur) tiles(i);
                bool exact_next = false;
                if (i + 1 < nchunks) exact_next = operands_a(i + 1, ring[(z + 1) % STB]);
                __syncthreads();
                // younger than the loads of visit i+2: those of visit i+3
                arrived(ring[(z + 2) % STB], std::integral_constant<int, STB - 2>{});
                if (i + 2 < nchunks) scan(i + 2, ring[(z + 2) % STB]);
                if (i + 1 < nchunks) operands_b(i + 1, ring[(z + 1) % STB], exact_next);
                prefetch(i + 1 + STB, ring[(z + 1) % STB]);
                __syncthreads();
                exact_cur = exact_next;
            }
        });
}

// ---------------------------------------------------------------------------------------------------- D waves: gk, gw, gs
// bh: this workgroup (stored states, s0, gs); bhk: the (batch, head) its key channels belong to (w, gw)
template <int WMODE, bool SPLIT>
DEVINL void bwd_state_d(SmemB2& S, const ArgsB& a, const int tid, const size_t base, const size_t bh, const size_t bhk, const int nchunks) {
    const int lane = tid & 63, q = (__builtin_amdgcn_readfirstlane(tid >> 6) - NPREP) & 3, l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    const bool stateful = a.s0 != nullptr;
    // this wave owns the key channels of state tile q:  column / operand row r = l16  <->  j_own
    const int j_own = 32 * (q >> 1) + 8 * (l16 >> 2) + 4 * (q & 1) + (l16 & 3);
    const int j4 = 32 * (q >> 1) + 8 * g + 4 * (q & 1);      // output rows 4g + v of this lane: key channels j4 .. j4+3
    int i0[4];                                         // first value channel of this lane's four rows in state tile m
#pragma unroll
    for (int m = 0; m < 4; ++m) i0[m] = 32 * (m >> 1) + 8 * g + 4 * (m & 1);

    f32x4 D[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) D[m] = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    float gw_acc[4] = {0.f, 0.f, 0.f, 0.f};            // wkv5: sum over tokens of G (chunked path: this lane's tokens)
    float gw_lane = 0.f;                               //       exact path: channel j_own
    float Pend[4] = {0.f, 0.f, 0.f, 0.f};              // P at the end of the current chunk for channels j4 + v (same in all 16 lanes of a row)

    __syncthreads();
    __syncthreads();
    for (int i = 0; i < nchunks; ++i) {
        const int c0 = (nchunks - 1 - i) * L;
        const SetB& O = S.set[i & 1];
        const bool exact = __builtin_amdgcn_readfirstlane(O.exact) != 0;
        {
            constexpr int pck = WMODE == W_HEAD ? PCK : 4 * PCK;      // as in the first sweep
            const int cn = nchunks - i;                // the chunk after this one; D is dS at its first token
            if (cn < nchunks && cn % pck == 0) {       // P at that boundary from the stored S (see PCK), replacing the carried value
                const int npck = (nchunks + PCK - 1) / PCK;
                const float* slot = a.rdr + static_cast<size_t>(gridDim.x / a.H) * T * C + (bh * npck + cn / PCK) * PCK_FLOATS;
                // D[m][v] <-> sweep A's state wave (q, ih = m >> 1), register 4 (m & 1) + v.  Loaded with a scalar base and one
                // 32-bit lane offset (per-lane 64-bit addresses kept across the loop cost this wave registers it does not have).
                uint32_t voff = lane;
                asm volatile("" : "+v"(voff));         // keeps the shift below inside this block instead of a register held across the loop
                voff <<= 5;
                slot += q * 64 * 8;
                const float* slot1 = slot + 4 * 64 * 8;
                f32x4 s0, s1, s2, s3;
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(s0) : "v"(voff), "s"(slot));
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=&v"(s1) : "v"(voff), "s"(slot));
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(s2) : "v"(voff), "s"(slot1));
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=&v"(s3) : "v"(voff), "s"(slot1));
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(s0), "+v"(s1), "+v"(s2), "+v"(s3));
                float p = 0.f;
                const f32x4 sv[4] = {s0, s1, s2, s3};
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    p = fmaf(D[m][0], sv[m][0], p); p = fmaf(D[m][1], sv[m][1], p);
                    p = fmaf(D[m][2], sv[m][2], p); p = fmaf(D[m][3], sv[m][3], p);
                }
                p = allreduce_rows(p);                 // over the four lanes that share key channel j_own
                if (g == 0) S.pc[j_own] = p;
                const float4 p4 = *reinterpret_cast<const float4*>(&S.pc[j4]);
                Pend[0] = p4.x; Pend[1] = p4.y; Pend[2] = p4.z; Pend[3] = p4.w;
            }
        }
        f32x4 dkin[2];                                 // (V dS)^T: rows j4 + v, lane = token 16 st + l16
        bf16x8 rtH, rtL;                               // R'^T of this wave's key channels: lane = j_own, K slots = tokens
        if (!exact) {
            // ------------------------------------------------------------ (V dS)^T, contraction over value channels
            dkin[0] = zero4; dkin[1] = zero4;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const HL x0 = hilo2(D[2 * ks][0], D[2 * ks][1]), x1 = hilo2(D[2 * ks][2], D[2 * ks][3]);
                const HL x2 = hilo2(D[2 * ks + 1][0], D[2 * ks + 1][1]), x3 = hilo2(D[2 * ks + 1][2], D[2 * ks + 1][3]);
                const bf16x8 sh = as_op(x0.h, x1.h, x2.h, x3.h), sl = as_op(x0.l, x1.l, x2.l, x3.l);
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    const bf16x8 vb = lds_op(&O.V[16 * st + l16][16 * ks + 4 * g]);
                    dkin[st] = mfma(sh, vb, dkin[st]);
                    dkin[st] = mfma(sl, vb, dkin[st]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ R'^T of the own key channels
            {
                const bf16x8 selOwn = op4(S.sel[q & 1][lane]);
                const f32x4 zh0 = mfma(lds_op(&O.RpH[l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                const f32x4 zh1 = mfma(lds_op(&O.RpH[16 + l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                const f32x4 zl0 = mfma(lds_op(&O.RpL[l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                const f32x4 zl1 = mfma(lds_op(&O.RpL[16 + l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                rtH = pack_tokens(zh0, zh1); rtL = pack_tokens(zl0, zl1);
                S.TR[q][0][lane] = __builtin_bit_cast(uint4, rtH);          // the E waves use it as a row operand of their update
                S.TR[q][1][lane] = __builtin_bit_cast(uint4, rtL);
            }
        } else {
            // ------------------------------------------------------------ exact path: 32 sequential steps, time descending
            // P changes layout: rows (j4 + v) -> lane (j_own)
            if (l16 == 0) *reinterpret_cast<float4*>(&S.pc[j4]) = make_float4(Pend[0], Pend[1], Pend[2], Pend[3]);
            float P = S.pc[j_own];
            const float* R = reinterpret_cast<const float*>(&O.RpH[0][0]);
            const float* K = reinterpret_cast<const float*>(&O.KpH[0][0]);
            const float uj = S.u[j_own];
            for (int t = L - 1; t >= 0; --t) {
                float vv[4][4], gg[4][4];
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    unpack4(*reinterpret_cast<const uint2*>(&O.V[t][i0[m] >> 1]), vv[m]);
                    unpack4(*reinterpret_cast<const uint2*>(&O.GY[t][i0[m] >> 1]), gg[m]);
                }
                const float rj = R[t * N + j_own], kj = K[t * N + j_own], wj = O.Eb[t][j_own], lmj = O.lam[t][j_own];
                const int tg = c0 + t;
                const float rdrj = O.rdr[t][j_own];
                float dkp = 0.f, vg = 0.f;
#pragma unroll
                for (int m = 0; m < 4; ++m)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        dkp = fmaf(vv[m][v], D[m][v], dkp);
                        vg = fmaf(vv[m][v], gg[m][v], vg);
                        D[m][v] = fmaf(D[m][v], wj, gg[m][v] * rj);
                    }
                allreduce2_rows(dkp, vg);
                const float Gt = P - kj * dkp;
                P = Gt + rdrj;
                if (g == 0 && tg < T) {
                    if constexpr (SPLIT) a.gk32[base + static_cast<size_t>(tg) * C + j_own] = fmaf(uj * rj, vg, dkp);
                    else a.gk[base + static_cast<size_t>(tg) * C + j_own] = f2bf(fmaf(uj * rj, vg, dkp));
                    if constexpr (WMODE != W_HEAD) a.gw[base + static_cast<size_t>(tg) * C + j_own] = f2bf((!stateful && tg == 0) ? 0.f : lmj * Gt);
                }
                if constexpr (WMODE == W_HEAD) gw_lane += (tg == 0 || tg >= T) ? 0.f : Gt;
            }
            if (g == 0) S.pc[j_own] = P;
            const float4 p4 = *reinterpret_cast<const float4*>(&S.pc[j4]);
            Pend[0] = p4.x; Pend[1] = p4.y; Pend[2] = p4.z; Pend[3] = p4.w;
        }
        __syncthreads();
        if (!exact) {
            float d2v[4], u4[4];
            {
                const float4 y = *reinterpret_cast<const float4*>(&O.d2[j4]);
                d2v[0] = y.x; d2v[1] = y.y; d2v[2] = y.z; d2v[3] = y.w;
                const float4 z = *reinterpret_cast<const float4*>(&S.u[j4]);
                u4[0] = z.x; u4[1] = z.y; u4[2] = z.z; u4[3] = z.w;
            }
            float tot1[4] = {0.f, 0.f, 0.f, 0.f};
            [[maybe_unused]] f32x4 out_k32[2];
            uint2 out_k[2], out_w[2];                   // stored after both tiles: a store in between would make every later
                                                        // register reload from scratch wait for its acknowledgement
#pragma unroll
            for (int st = 1; st >= 0; --st) {           // later tokens first: their total enters the earlier tile's suffix
                const int s = 16 * st + l16, tg = c0 + s;
                // ---------------------------------------------------- sum_{tau > s} Bm[tau][s] R'_tau[j]
                const bf16x8 bh_ = lds_op(&S.BmH[s][4 * g]);
                f32x4 dq = mfma(rtH, bh_, zero4);
                dq = mfma(rtH, lds_op(&S.BmL[s][4 * g]), dq);
                dq = mfma(rtL, bh_, dq);
                const float4 eb4 = *reinterpret_cast<const float4*>(&O.Eb[s][j4]);
                const float4 lm4 = *reinterpret_cast<const float4*>(&O.lam[s][j4]);
                const float4 rd4 = *reinterpret_cast<const float4*>(&O.rdr[s][j4]);
                float rr[4], kh[4], kl[4];
                unpack4(*reinterpret_cast<const uint2*>(&O.Rr[s][j4 >> 1]), rr);
                unpack4(*reinterpret_cast<const uint2*>(&O.KpH[s][j4 >> 1]), kh);      // k Eb = K' = hi + lo
                unpack4(*reinterpret_cast<const uint2*>(&O.KpL[s][j4 >> 1]), kl);
                const float vgy = S.vgy[s];
                const float eb[4] = {eb4.x, eb4.y, eb4.z, eb4.w}, lm[4] = {lm4.x, lm4.y, lm4.z, lm4.w}, rd[4] = {rd4.x, rd4.y, rd4.z, rd4.w};
                float gk[4], gw[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float dkq = fmaf(d2v[v], dkin[st][v], dq[v]);
                    gk[v] = fmaf(u4[v] * rr[v], vgy, dkq * eb[v]);
                    const float kd = (kh[v] + kl[v]) * dkq;                    // k times dk_prime
                    const float dl = rd[v] - kd;
                    const float suf = row_suffix_sum(dl);                      // sum over the tokens s' >= s of this tile
                    const float tot = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, suf), 0x150, 0xf, 0xf, true));
                    const float Gt = (suf - dl) + (st == 0 ? tot1[v] : 0.f) + Pend[v] - kd;
                    gw[v] = (!stateful && tg == 0) ? 0.f : lm[v] * Gt;
                    if constexpr (WMODE == W_HEAD) gw_acc[v] += (tg == 0 || tg >= T) ? 0.f : Gt;
                    if (st == 1) tot1[v] = tot; else Pend[v] += tot + tot1[v];
                }
                if constexpr (SPLIT) out_k32[st] = f32x4{gk[0], gk[1], gk[2], gk[3]};
                else out_k[st] = make_uint2(pack_bf2(gk[0], gk[1]), pack_bf2(gk[2], gk[3]));
                out_w[st] = make_uint2(pack_bf2(gw[0], gw[1]), pack_bf2(gw[2], gw[3]));
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const int tg = c0 + 16 * st + l16;
                if (tg < T) {
                    const uint32_t off = (static_cast<uint32_t>(tg) * C + j4) * 2;
                    if constexpr (SPLIT) store16(a.gk32 + base, 2 * off, out_k32[st]);
                    else store8(a.gk + base, off, out_k[st]);
                    if constexpr (WMODE != W_HEAD) store8(a.gw + base, off, out_w[st]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ dS = dS diag(dec) + diag(d1) GY^T R'
            const float decj = O.dec[j_own], d1j = O.d1[j_own];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const bf16x8 gt = op4(S.TG[m][lane]);   // gy^T of state tile m: lane = value-channel row, slots = tokens
                f32x4 U = mfma(gt, rtH, zero4);
                U = mfma(gt, rtL, U);
#pragma unroll
                for (int v = 0; v < 4; ++v) D[m][v] = fmaf(D[m][v], decj, d1j * U[v]);
            }
        }
        __syncthreads();
    }
    if constexpr (WMODE == W_HEAD) {                   // gw[b][h][j] = ew_j sum_t G_t[j]
        if (g == 0) S.pc[j_own] = gw_lane;
        const float4 px = *reinterpret_cast<const float4*>(&S.pc[j4]);
        const float4 e4 = *reinterpret_cast<const float4*>(static_cast<const float*>(a.w) + (bhk % a.H) * N + j4);
        const float pxv[4] = {px.x, px.y, px.z, px.w}, ev[4] = {e4.x, e4.y, e4.z, e4.w};
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float s = row_sum_to_last(gw_acc[v]) + pxv[v];
            if (l16 == 15) {
                if constexpr (SPLIT) a.gw32[bhk * N + j4 + v] = gw_factor(ev[v]) * s;
                else a.gw[bhk * N + j4 + v] = f2bf(gw_factor(ev[v]) * s);
            }
        }
    }
    if (a.gs != nullptr) {
        uint16_t* s = a.gs + bh * N * N + j_own;
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) s[(i0[m] + v) * N] = f2bf(D[m][v]);
    }
}

// ---------------------------------------------------------------------------------------------------- E waves: gv
template <int WMODE, bool SPLIT>
DEVINL void bwd_state_e(SmemB2& S, const ArgsB& a, const int tid, const size_t base, const int nchunks) {
    const int lane = tid & 63, q = (__builtin_amdgcn_readfirstlane(tid >> 6) - NPREP) & 3, l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    // this wave owns the value channels of state tile q:  column / operand row r = l16  <->  i_own
    const int i_own = 32 * (q >> 1) + 8 * (l16 >> 2) + 4 * (q & 1) + (l16 & 3);
    const int i4 = 32 * (q >> 1) + 8 * g + 4 * (q & 1);      // output rows 4g + v: value channels i4 .. i4+3
    int j0[4];                                         // first key channel of this lane's four rows in state tile m
#pragma unroll
    for (int m = 0; m < 4; ++m) j0[m] = 32 * (m >> 1) + 8 * g + 4 * (m & 1);

    f32x4 E[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) E[m] = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

    __syncthreads();
    __syncthreads();
    for (int i = 0; i < nchunks; ++i) {
        const int c0 = (nchunks - 1 - i) * L;
        const SetB& O = S.set[i & 1];
        const bool exact = __builtin_amdgcn_readfirstlane(O.exact) != 0;
        f32x4 dvin[2];                                 // (K' diag(d2) dS^T)^T: rows i4 + v, lane = token 16 st + l16
        bf16x8 gto;                                    // gy^T of this wave's value channels: lane = i_own, K slots = tokens
        if (!exact) {
            dvin[0] = zero4; dvin[1] = zero4;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const float4 da = *reinterpret_cast<const float4*>(&O.d2[j0[2 * ks]]);
                const float4 db = *reinterpret_cast<const float4*>(&O.d2[j0[2 * ks + 1]]);
                const HL x0 = hilo2(E[2 * ks][0] * da.x, E[2 * ks][1] * da.y), x1 = hilo2(E[2 * ks][2] * da.z, E[2 * ks][3] * da.w);
                const HL x2 = hilo2(E[2 * ks + 1][0] * db.x, E[2 * ks + 1][1] * db.y), x3 = hilo2(E[2 * ks + 1][2] * db.z, E[2 * ks + 1][3] * db.w);
                const bf16x8 sh = as_op(x0.h, x1.h, x2.h, x3.h), sl = as_op(x0.l, x1.l, x2.l, x3.l);
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    const bf16x8 kh = lds_op(&O.KpH[16 * st + l16][16 * ks + 4 * g]), kl = lds_op(&O.KpL[16 * st + l16][16 * ks + 4 * g]);
                    dvin[st] = mfma(sh, kh, dvin[st]);
                    dvin[st] = mfma(sh, kl, dvin[st]);
                    dvin[st] = mfma(sl, kh, dvin[st]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                const bf16x8 selOwn = op4(S.sel[q & 1][lane]);
                gto = pack_tokens(mfma(lds_op(&O.GY[l16][16 * (q >> 1) + 4 * g]), selOwn, zero4),
                                  mfma(lds_op(&O.GY[16 + l16][16 * (q >> 1) + 4 * g]), selOwn, zero4));
                S.TG[q][lane] = __builtin_bit_cast(uint4, gto);             // the D waves use it as a row operand of their update
            }
        } else {
            // ------------------------------------------------------------ exact path: 32 sequential steps, time descending
            const float* R = reinterpret_cast<const float*>(&O.RpH[0][0]);
            const float* K = reinterpret_cast<const float*>(&O.KpH[0][0]);
            float uv[4][4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float4 y = *reinterpret_cast<const float4*>(&S.u[j0[m]]);
                uv[m][0] = y.x; uv[m][1] = y.y; uv[m][2] = y.z; uv[m][3] = y.w;
            }
            for (int t = L - 1; t >= 0; --t) {
                const uint32_t gq = O.GY[t][i_own >> 1];
                const float gi = (l16 & 1) ? bf_hi(gq) : bf_lo(gq);
                float gvp = 0.f;
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const float4 r4 = *reinterpret_cast<const float4*>(&R[t * N + j0[m]]);
                    const float4 k4 = *reinterpret_cast<const float4*>(&K[t * N + j0[m]]);
                    const float4 w4 = *reinterpret_cast<const float4*>(&O.Eb[t][j0[m]]);
                    const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float rg = rr[v] * gi;
                        gvp = fmaf(kk[v], fmaf(uv[m][v], rg, E[m][v]), gvp);
                        E[m][v] = fmaf(E[m][v], ww[v], rg);
                    }
                }
                gvp = allreduce_rows(gvp);
                const int tg = c0 + t;
                if (g == 0 && tg < T) {
                    if constexpr (SPLIT) a.gv32[base + static_cast<size_t>(tg) * C + i_own] = gvp;
                    else a.gv[base + static_cast<size_t>(tg) * C + i_own] = f2bf(gvp);
                }
            }
        }
        __syncthreads();
        if (!exact) {
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const int s = 16 * st + l16, tg = c0 + s;
                f32x4 y = mfma(gto, lds_op(&S.AmH[s][4 * g]), dvin[st]);
                y = mfma(gto, lds_op(&S.AmL[s][4 * g]), y);
                if (tg < T) {
                    if constexpr (SPLIT) store16(a.gv32 + base, (static_cast<uint32_t>(tg) * C + i4) * 4, y);
                    else store8(a.gv + base, (static_cast<uint32_t>(tg) * C + i4) * 2, make_uint2(pack_bf2(y[0], y[1]), pack_bf2(y[2], y[3])));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ dS^T = diag(dec) dS^T + diag(d1) R'^T GY
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                f32x4 U = mfma(op4(S.TR[m][0][lane]), gto, zero4);   // R'^T of state tile m: lane = key-channel row, slots = tokens
                U = mfma(op4(S.TR[m][1][lane]), gto, U);
                const float4 de = *reinterpret_cast<const float4*>(&O.dec[j0[m]]);
                const float4 d1 = *reinterpret_cast<const float4*>(&O.d1[j0[m]]);
                E[m][0] = fmaf(E[m][0], de.x, d1.x * U[0]); E[m][1] = fmaf(E[m][1], de.y, d1.y * U[1]);
                E[m][2] = fmaf(E[m][2], de.z, d1.z * U[2]); E[m][3] = fmaf(E[m][3], de.w, d1.w * U[3]);
            }
        }
        __syncthreads();
    }
}

template <int WMODE, bool SPLIT = false>
__global__ __launch_bounds__(NTB) void wkv6_bwd_b_ws(const ArgsB a) {
    __shared__ SmemB2 S;
    if (a.sum_out != nullptr && blockIdx.x < static_cast<unsigned>(a.H) && threadIdx.x < N) {
        const int c = blockIdx.x * N + threadIdx.x;
        float x = 0.f;
        for (int b = 0; b < a.sum_B; ++b) x += bf2f(a.sum_in[static_cast<size_t>(b) * a.C + c]);
        a.sum_out[c] = f2bf(x);
    }
    if (skip_unflagged(a.only_flagged, blockIdx.x)) return;
    const int tid = threadIdx.x;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int hk = SPLIT ? h ^ a.cross : h;            // the block of 64 channels that r, k, w, u come from and gk, gw go to
    const size_t vbase = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(h) * N;
    const size_t base = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(hk) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h, bhk = static_cast<size_t>(b) * a.H + hk;
    const int nchunks = (a.T + L - 1) / L;
    // positions of the tiles that are never written (s >= 16 > tau) must read as zero
    for (int i = tid; i < 4 * L * AS; i += NTB) (&S.AmH[0][0])[i] = 0;
    if (tid < N) S.u[tid] = bf2f(a.u[hk * N + tid]);
    if (tid < 128) {
        // One-hot B operand of the transposing products, per lane (column r = l16, K-slot group g), for tile parity p:
        // column r <-> channel 8 (r>>2) + 4 p + (r&3) of a 32-channel half.
        const int p = tid >> 6, ln = tid & 63, c16 = ln & 15, gg = ln >> 4;
        S.sel[p][ln] = one_hot(gg == (c16 >> 2), 4 * p + (c16 & 3));
    }
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (wid < NPREP) bwd_prep<WMODE>(S, a, tid, base, vbase, hk, nchunks);
    else if (wid < NPREP + 4) bwd_state_d<WMODE, SPLIT>(S, a, tid, base, bh, bhk, nchunks);
    else bwd_state_e<WMODE, SPLIT>(S, a, tid, vbase, nchunks);
}

}  // namespace

int launch_wkv6_bwd_b_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                            const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                            const uint16_t* s0, const uint16_t* gy, uint16_t* gk, uint16_t* gv, uint16_t* gw,
                            uint16_t* gs, const float* rdr, const int* only_flagged, const uint16_t* sum_in, uint16_t* sum_out) {
    ArgsB a{};
    a.sum_in = sum_in; a.sum_out = sum_out; a.sum_B = B;
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.gy = gy;
    a.gk = gk; a.gv = gv; a.gw = gw; a.gs = gs; a.rdr = const_cast<float*>(rdr); a.only_flagged = only_flagged;
    if (wmode == W_RAW) hipLaunchKernelGGL(wkv6_bwd_b_ws<W_RAW>, dim3(B * H), dim3(NTB), 0, st, a);
    else if (wmode == W_EW) hipLaunchKernelGGL(wkv6_bwd_b_ws<W_EW>, dim3(B * H), dim3(NTB), 0, st, a);
    else hipLaunchKernelGGL(wkv6_bwd_b_ws<W_HEAD>, dim3(B * H), dim3(NTB), 0, st, a);
    return launch_status();
}

// wkv5 with heads of 128 channels: the second sweep of one of the two launches described at ArgsB (H counts the heads of 128)
int launch_wkv5_bwd_b_split(hipStream_t st, int cross, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k,
                            const uint16_t* v, const float* ew, const uint16_t* u, const uint16_t* gy, float* gk32, float* gv32,
                            float* gw32, const float* rdr) {
    ArgsB a{};
    a.T = T; a.C = C; a.H = 2 * H; a.r = r; a.k = k; a.v = v; a.w = ew; a.u = u; a.s0 = nullptr; a.gy = gy;
    a.gs = nullptr; a.rdr = const_cast<float*>(rdr); a.cross = cross; a.gk32 = gk32; a.gv32 = gv32; a.gw32 = gw32;
    hipLaunchKernelGGL((wkv6_bwd_b_ws<W_HEAD, true>), dim3(B * 2 * H), dim3(NTB), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
