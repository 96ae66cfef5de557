// wkv6 / wkv6_state backward, first sweep (time ascending): gr, gu and the workspace r * dr' that the decay gradient needs.
// Wave-specialised workgroup (gfx950); formulas and symbols as in wkv6_chunk.h, S the state at the START of a chunk:
//     dr'_t[j] = Ea_t[j] ( d1[j] (GY S)[t][j] + sum_{s<t} Bm[t][s] K'_s[j] ),    Bm[t][s] = gy_t . v_s,   Ea_t = e^{c_t - c_m}
//     gr = dr' + u k_t (gy_t . v_t),     gu[j] = sum_t r_t[j] k_t[j] (gy_t . v_t),     S_L = S diag(dec) + diag(d2) V^T K'
// One workgroup of 16 waves per (batch, head):
//   waves 0..7  ("prep")   load r, k, v, w, gy ahead of time, take the decay sums, write K' (hi / lo bf16 planes), r, k, v, gy and
//                          Ea into LDS in natural [token][channel] layout; waves 0..2 form the causal tile Bm.
//   waves 8..15 ("state")  wave (q, ih) keeps S[i][j] for the key channels of state tile q and the value-channel half ih
//                          (lane = j, registers = 32 values of i).  dr' comes out with a lane per TOKEN and four consecutive key
//                          channels per lane; the two waves of a q exchange one partial tile and each finishes 16 tokens:
//                          gr and r dr' are stored from registers.
// K-slot conventions, selection-matrix transposes and tile storage are those of the forward kernel (wkv6_fwd.hip).
// Two barriers per chunk:  [tile(i) | first half of operands(i+1) | GY S, K'^T, V^T, state update]  B
//                          [scan(i+2), second half of operands(i+1) | Bm K', epilogue, stores]  B.
#include "wkv6_chunk.h"

namespace rwkv {
namespace {

constexpr int NPREP = 8;
constexpr int NSTATE = 8;
constexpr int NTA = (NPREP + NSTATE) * 64;
constexpr int STA = 3;            // chunks of input kept in flight

struct alignas(16) SetA {
    uint32_t KpH[L][OS], KpL[L][OS];   // k e^{c_m - c_{s+1}}  hi, lo
    uint32_t Rr[L][OS], Kr[L][OS];     // r, k
    uint32_t V[L][OS], GY[L][OS];      // v, gy
    float Ea[L][FS];                   // e^{c_t - c_m}                 (exact path: decay of each step)
    float d1[N], d2[N], dec[N];        // e^{c_m}, e^{c_L - c_m}, e^{c_L}
    uint32_t exact, pad[3];
};

struct alignas(16) SmemA2 {
    SetA set[2];
    uint32_t BmH[L][AS], BmL[L][AS];   // Bm[t][s] (s < t) as [t][position of s], hi and lo
    uint4 sel[2][64];                  // selection operands per lane, tile parity 0 and 1
    float4 Xch[NSTATE][64];            // partial (GY S)^T tile handed to the partner wave
    float outR[2][L][N + 4];              // r dr' and gr of the chunk just finished, [token][channel]: stored one phase later as
    uint32_t outG[2][L][N / 2 + 2];       // whole rows (a lane of the state waves holds one token and four channels)
    float Yx[2][L][N];                 // exact path: partial dr' of the two value-channel halves;  at the end: gu partial sums
    float Vx[2][L];                    // exact path: partial gy . v
    float vgy[L];                      // gy_t . v_t
    float gfast[2][N];                 // gu of the chunked path, two token halves
    float u[N];
    float part[2][NPREP][N];
};

// ---------------------------------------------------------------------------------------------------- prep waves
// base, h: where r, k, w, u (and gu) of this workgroup sit; vbase: where v, gy sit (the same place unless the head is split)
// SPLIT: 0 = whole heads; 1 = first launch of a split head (gr, gu leave as fp32 terms); 2 = second launch (the first
// launch's terms are added and gr, gu leave in bf16)
template <int WMODE, int SPLIT>
DEVINL void bwa_prep(SmemA2& S, const ArgsB& a, const int tid, const size_t base, const size_t vbase, const int h, const int nchunks) {
    const int lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb = a.v + vbase;
    const uint16_t* __restrict__ gb = a.gy + vbase;
    // channel pair (2 jp, 2 jp + 1), tokens 4 wid + 2 th + {0, 1}
    const int jp = lane & 31, th = lane >> 5, pt0 = 4 * wid + 2 * th;
    const bool second = wid >= 4;
    struct Raw { uint32_t r[2], k[2], v[2], g[2], w[2]; uint2 wq[2]; float lam[2][2], other[2], kp[2][2]; };
    Raw ring[STA];
    // Loads are asm so that the wait before their first use can leave the younger batches in flight; every call issues the
    // same ten loads (chunk index clamped), which keeps the count fixed.
    const uint32_t* __restrict__ wb32 = reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + base);
    const float* __restrict__ wbf = static_cast<const float*>(a.w) + base;
    // The inputs are read once and never again by this kernel: the loads carry the non-temporal hint (measured -2.4 % here,
    // -3.5 % in the second sweep, nothing in the forward).
    auto prefetch = [&](int c, Raw& x) __attribute__((always_inline)) {
        c = c < nchunks ? c : nchunks - 1;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = c * L + pt0 + e;
            const uint32_t o = (static_cast<uint32_t>(t < T ? t : T - 1) * C + 2 * jp) * 2;    // byte offset of the channel pair
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.r[e]) : "v"(o), "s"(rb) : "memory");
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.k[e]) : "v"(o), "s"(kb) : "memory");
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.v[e]) : "v"(o), "s"(vb) : "memory");
            asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.g[e]) : "v"(o), "s"(gb) : "memory");
            if constexpr (WMODE == W_RAW) {
                asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(x.w[e]) : "v"(o), "s"(wb32) : "memory");
            } else if constexpr (WMODE == W_EW) {
                // straight into the ring: a copy here would read the register before the load has landed
                asm volatile("global_load_dwordx2 %0, %1, %2 nt" : "=&v"(x.wq[e]) : "v"(2 * o), "s"(wbf) : "memory");
            }
        }
    };
    constexpr int NLOADS = WMODE == W_HEAD ? 8 : 10;   // loads per prefetch call
    auto arrived = [&](Raw& x, auto younger) __attribute__((always_inline)) {
        if constexpr (WMODE == W_RAW)
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.w[0]), "+v"(x.w[1]) : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
        else if constexpr (WMODE == W_EW)
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.g[0]), "+v"(x.g[1]), "+v"(x.wq[0]), "+v"(x.wq[1])
                         : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.g[0]), "+v"(x.g[1]) : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
    };
    // wkv5: one decay per channel for the whole sequence, given as ew = -exp(w_raw) = log of the decay
    float lamc[2] = {0.f, 0.f};
    if constexpr (WMODE == W_HEAD) {
        const float2 e2 = *reinterpret_cast<const float2*>(static_cast<const float*>(a.w) + h * N + 2 * jp);
        lamc[0] = LOG2E * e2.x; lamc[1] = LOG2E * e2.y;
    }
    static_for<STA>([&](auto Z) { prefetch(decltype(Z)::value, ring[decltype(Z)::value]); });

    // ---- scan of chunk c: lam (log2 units) of this thread's four elements, sums over each eighth of the chunk
    auto scan = [&](const int c, Raw& x) __attribute__((always_inline)) {
        const int c0 = c * L, pb = c & 1;
        if (c0 + L > T) {                              // last, partial chunk: rows past T carry no input and no decay
#pragma unroll
            for (int e = 0; e < 2; ++e)
                if (c0 + pt0 + e >= T) {
                    x.r[e] = 0; x.k[e] = 0; x.v[e] = 0; x.g[e] = 0;
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

    // ---- operands of chunk c into set c & 1, first part: Ea, plain r (K' values stay in registers)
    auto operands_a = [&](const int c, Raw& x) __attribute__((always_inline)) -> bool {
        SetA& O = S.set[c & 1];
        const int pb = c & 1;
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
        if (!exact) {
            float ea[2][2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const Scale sc = chunk_scale(second, near[z], x.lam[0][z], x.lam[1][z]);
                ea[0][z] = sc.ea[0]; ea[1][z] = sc.ea[1];
                x.kp[0][z] = (z ? bf_hi(x.k[0]) : bf_lo(x.k[0])) * sc.eb[0];
                x.kp[1][z] = (z ? bf_hi(x.k[1]) : bf_lo(x.k[1])) * sc.eb[1];
            }
#pragma unroll
            for (int e = 0; e < 2; ++e) *reinterpret_cast<float2*>(&O.Ea[pt0 + e][2 * jp]) = make_float2(ea[e][0], ea[e][1]);
        } else {
#pragma unroll
            for (int e = 0; e < 2; ++e)
                *reinterpret_cast<float2*>(&O.Ea[pt0 + e][2 * jp]) = make_float2(exp2_fast(x.lam[e][0]), exp2_fast(x.lam[e][1]));
        }
        O.Rr[pt0][jp] = x.r[0];
        O.Rr[pt0 + 1][jp] = x.r[1];
        return exact;
    };
    // ---- second part: K' planes, k, v, gy; wave 3 adds the per-channel factors of the chunk
    auto operands_b = [&](const int c, Raw& x, const bool exact) __attribute__((always_inline)) {
        SetA& O = S.set[c & 1];
        const int pb = c & 1;
        if (!exact) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const HL y = hilo2(x.kp[e][0], x.kp[e][1]);
                O.KpH[pt0 + e][jp] = y.h; O.KpL[pt0 + e][jp] = y.l;
            }
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            O.Kr[pt0 + e][jp] = x.k[e];
            O.V[pt0 + e][jp] = x.v[e];
            O.GY[pt0 + e][jp] = x.g[e];
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

    // ---- causal tile of chunk c: waves 0..2, quadrants (t tile, s tile) = (0,0) (1,0) (1,1).  Accumulator rows are s,
    //      lanes are t; stored as [t][position of s].  The diagonal gy_t . v_t goes to vgy.
    auto tile = [&](const int c) __attribute__((always_inline)) {
        const SetA& O = S.set[c & 1];
        const int ta = (wid == 0) ? 0 : 1, tb = (wid == 2) ? 1 : 0;          // t tile, s tile
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
            acc = mfma(lds_op(&O.V[16 * tb + l16][16 * ks + 4 * g]), lds_op(&O.GY[16 * ta + l16][16 * ks + 4 * g]), acc);
        if (ta == tb) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int sl = 4 * g + v;
                if (sl == l16) S.vgy[16 * ta + l16] = acc[v];
                acc[v] = (sl < l16) ? acc[v] : 0.f;
            }
        }
        const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
        *reinterpret_cast<uint2*>(&S.BmH[16 * ta + l16][4 * g + 2 * tb]) = make_uint2(x0.h, x1.h);
        *reinterpret_cast<uint2*>(&S.BmL[16 * ta + l16][4 * g + 2 * tb]) = make_uint2(x0.l, x1.l);
    };

    static_for<STA>([&](auto Z) { arrived(ring[decltype(Z)::value], std::integral_constant<int, 0>{}); });
    scan(0, ring[0]);
    if (nchunks > 1) scan(1, ring[1]);
    __syncthreads();
    bool exact_cur = operands_a(0, ring[0]);
    operands_b(0, ring[0], exact_cur);
    prefetch(STA, ring[0]);
    __syncthreads();
    for (int ib = 0; ib < nchunks; ib += STA)
        static_for<STA>([&](auto Z) {
            constexpr int z = decltype(Z)::value;
            const int i = ib + z;
            if (i < nchunks) {
                if (wid < 3 && !exact_cur) tile(i);
                bool exact_next = false;
                if (i + 1 < nchunks) exact_next = operands_a(i + 1, ring[(z + 1) % STA]);
                __syncthreads();
                // younger than the loads of chunk i+2: those of chunk i+3
                arrived(ring[(z + 2) % STA], std::integral_constant<int, STA - 2>{});
                if (i + 2 < nchunks) scan(i + 2, ring[(z + 2) % STA]);
                if (i + 1 < nchunks) operands_b(i + 1, ring[(z + 1) % STA], exact_next);
                prefetch(i + 1 + STA, ring[(z + 1) % STA]);
                __syncthreads();
                exact_cur = exact_next;
            }
        });
    __syncthreads();                                   // the state waves publish their gu sums
    if (tid < N) {
        float s = S.gfast[0][tid] + S.gfast[1][tid];
        for (int t = 0; t < L; ++t) s += S.Yx[0][t][tid];
        const size_t at = static_cast<size_t>(blockIdx.x / a.H) * C + h * N + tid;
        if constexpr (SPLIT == 1) a.gu32[at] = s;
        else if constexpr (SPLIT == 2) a.gu[at] = f2bf(s + a.gu32[at]);
        else a.gu[at] = f2bf(s);
    }
}

// ---------------------------------------------------------------------------------------------------- state waves
template <int WMODE, int SPLIT>
DEVINL void bwa_state(SmemA2& S, const ArgsB& a, const int tid, const size_t base, const size_t bh, const int nchunks) {
    const int lane = tid & 63, sw = __builtin_amdgcn_readfirstlane(tid >> 6) - NPREP, q = sw & 3, ih = sw >> 2, l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    // this wave owns the key channels of state tile q:  column / operand row r = l16  <->  j_own
    const int j_own = 32 * (q >> 1) + 8 * (l16 >> 2) + 4 * (q & 1) + (l16 & 3);
    const int j4 = 32 * (q >> 1) + 8 * g + 4 * (q & 1);      // output rows 4g + v of this lane: key channels j4 .. j4+3
    const int i0[2] = {32 * ih + 8 * g, 32 * ih + 8 * g + 4};   // first value channel of this lane's four rows in tile mm
    const int idx = tid - NPREP * 64, xt = idx >> 4, xj = (idx & 15) * 4;   // exact path: (token, channels) this thread finishes

    f32x4 D[2];
    D[0] = D[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.s0 != nullptr) {
        const uint16_t* s = a.s0 + bh * N * N + j_own;
#pragma unroll
        for (int mm = 0; mm < 2; ++mm)
#pragma unroll
            for (int v = 0; v < 4; ++v) D[mm][v] = bf2f(s[(i0[mm] + v) * N]);
    }
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    float gu_acc[4] = {0.f, 0.f, 0.f, 0.f};            // chunked path: lane = token of tile ih, rows j4 + v
    float gu_x[4] = {0.f, 0.f, 0.f, 0.f};              // exact path: token xt, channels xj + e

    // The outputs of a chunk leave one phase after they were formed, read back from LDS as whole rows: wave sw takes tokens
    // 4 sw .. 4 sw + 3, 16 lanes per token (128 B of gr, 256 B of r dr' per row).  Stored straight from the accumulator
    // layout they would be 8- and 16-byte pieces of sixteen different rows per instruction, which measured 8 % slower.
    bool staged = false;
    auto flush = [&](const int c0p, const int pb) __attribute__((always_inline)) {
        const int row = 4 * sw + g, tg = c0p + row;
        const uint2 y = *reinterpret_cast<const uint2*>(&S.outG[pb][row][2 * l16]);
        const float4 x = *reinterpret_cast<const float4*>(&S.outR[pb][row][4 * l16]);
        if (tg < T) {
            const uint32_t o = static_cast<uint32_t>(tg) * C + 4 * l16;
            if constexpr (SPLIT != 1) store8(a.gr + base, o * 2, y);  // first launch of a split head: gr has left as an fp32 term
            store16(a.rdr + base, o * 4, f32x4{x.x, x.y, x.z, x.w});
        }
    };

    __syncthreads();
    __syncthreads();
    for (int i = 0; i < nchunks; ++i) {
        const int c0 = i * L;
        const SetA& O = S.set[i & 1];
        const bool exact = __builtin_amdgcn_readfirstlane(O.exact) != 0;
        bool staged_now = false;
        {
            constexpr int pck = WMODE == W_HEAD ? PCK : 4 * PCK;      // wkv5 sums G over time and needs the shorter walk
            if (i > 0 && i % pck == 0) {               // S at the start of chunk i, for the second sweep's P (see PCK)
                const int npck = (nchunks + PCK - 1) / PCK;
                const float* slot = a.rdr + static_cast<size_t>(gridDim.x / a.H) * T * C + (bh * npck + i / PCK) * PCK_FLOATS;
                store16(slot, (sw * 64 + lane) * 32, D[0]);
                store16(slot, (sw * 64 + lane) * 32 + 16, D[1]);
            }
        }
        [[maybe_unused]] f32x4 term = zero4;           // SPLIT == 2: the first launch's term of this lane's gr
        if constexpr (SPLIT == 2) {
            const int tg = c0 + 16 * ih + l16;
            term = *reinterpret_cast<const f32x4*>(a.gr32 + base + static_cast<size_t>(tg < T ? tg : T - 1) * C + j4);
        }
        f32x4 own;                                     // (GY S)^T of this half of i: rows j4 + v, token 16 ih + l16
        bf16x8 ktH, ktL;                               // K'^T of the own key channels: lane = j_own, K slots = tokens
        if (!exact) {
            const float d1j = O.d1[j_own];
            const HL x0 = hilo2(D[0][0] * d1j, D[0][1] * d1j), x1 = hilo2(D[0][2] * d1j, D[0][3] * d1j);
            const HL x2 = hilo2(D[1][0] * d1j, D[1][1] * d1j), x3 = hilo2(D[1][2] * d1j, D[1][3] * d1j);
            const bf16x8 sh = as_op(x0.h, x1.h, x2.h, x3.h), sl = as_op(x0.l, x1.l, x2.l, x3.l);
            const bf16x8 g0 = lds_op(&O.GY[l16][16 * ih + 4 * g]), g1 = lds_op(&O.GY[16 + l16][16 * ih + 4 * g]);
            f32x4 Y0 = mfma(sh, g0, zero4), Y1 = mfma(sh, g1, zero4);
            Y0 = mfma(sl, g0, Y0); Y1 = mfma(sl, g1, Y1);
            S.Xch[sw][lane] = ih ? make_float4(Y0[0], Y0[1], Y0[2], Y0[3]) : make_float4(Y1[0], Y1[1], Y1[2], Y1[3]);
            own = ih ? Y1 : Y0;
            __builtin_amdgcn_sched_barrier(0);
            // ------------------------------------------------------------ K'^T of the own key channels
            {
                const bf16x8 selOwn = op4(S.sel[q & 1][lane]);
                const f32x4 zh0 = mfma(lds_op(&O.KpH[l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                const f32x4 zh1 = mfma(lds_op(&O.KpH[16 + l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                const f32x4 zl0 = mfma(lds_op(&O.KpL[l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                const f32x4 zl1 = mfma(lds_op(&O.KpL[16 + l16][16 * (q >> 1) + 4 * g]), selOwn, zero4);
                ktH = pack_tokens(zh0, zh1); ktL = pack_tokens(zl0, zl1);
            }
            // ------------------------------------------------------------ S = S diag(dec) + diag(d2) V^T K'
            const float decj = O.dec[j_own], d2j = O.d2[j_own];
            const bf16x8 v0 = lds_op(&O.V[l16][16 * ih + 4 * g]), v1 = lds_op(&O.V[16 + l16][16 * ih + 4 * g]);
#pragma unroll
            for (int mm = 0; mm < 2; ++mm) {
                const bf16x8 sel = op4(S.sel[mm][lane]);
                const bf16x8 vt = pack_tokens(mfma(v0, sel, zero4), mfma(v1, sel, zero4));   // lane = value-channel row, slots = tokens
                f32x4 U = mfma(vt, ktH, zero4);
                U = mfma(vt, ktL, U);
#pragma unroll
                for (int v = 0; v < 4; ++v) D[mm][v] = fmaf(D[mm][v], decj, d2j * U[v]);
            }
        } else {
            // ------------------------------------------------------------ exact path: 32 sequential steps
            for (int t4 = 0; t4 < L; t4 += 4) {
                float dr[4], vg[4];                     // four steps, then their sums over the lane rows in one go
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int t = t4 + s;
                    float vv[2][4], gg[2][4];
#pragma unroll
                    for (int mm = 0; mm < 2; ++mm) {
                        unpack4(*reinterpret_cast<const uint2*>(&O.V[t][i0[mm] >> 1]), vv[mm]);
                        unpack4(*reinterpret_cast<const uint2*>(&O.GY[t][i0[mm] >> 1]), gg[mm]);
                    }
                    const uint32_t kq = O.Kr[t][j_own >> 1];
                    const float kj = (j_own & 1) ? bf_hi(kq) : bf_lo(kq), wj = O.Ea[t][j_own];
                    dr[s] = 0.f; vg[s] = 0.f;
#pragma unroll
                    for (int mm = 0; mm < 2; ++mm)
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            dr[s] = fmaf(gg[mm][v], D[mm][v], dr[s]);
                            vg[s] = fmaf(gg[mm][v], vv[mm][v], vg[s]);
                            D[mm][v] = fmaf(D[mm][v], wj, vv[mm][v] * kj);
                        }
                }
                S.Yx[ih][t4 + g][j_own] = reduce4_rows(dr[0], dr[1], dr[2], dr[3]);     // lane row g holds step t4 + g
                const float vgs = reduce4_rows(vg[0], vg[1], vg[2], vg[3]);
                if (q == 0 && l16 == 0) S.Vx[ih][t4 + g] = vgs;
            }
        }
        __syncthreads();
        if (!exact) {
            const int t = 16 * ih + l16;
            const float4 p = S.Xch[sw ^ 4][lane];
            const bf16x8 bh_ = lds_op(&S.BmH[t][4 * g]);
            f32x4 dr = own + f32x4{p.x, p.y, p.z, p.w};
            dr = mfma(ktH, bh_, dr);
            dr = mfma(ktH, lds_op(&S.BmL[t][4 * g]), dr);
            dr = mfma(ktL, bh_, dr);
            const float4 ea4 = *reinterpret_cast<const float4*>(&O.Ea[t][j4]);
            const float4 u4 = *reinterpret_cast<const float4*>(&S.u[j4]);
            float rr[4], kk[4];
            unpack4(*reinterpret_cast<const uint2*>(&O.Rr[t][j4 >> 1]), rr);
            unpack4(*reinterpret_cast<const uint2*>(&O.Kr[t][j4 >> 1]), kk);
            const float vgy = S.vgy[t];
            const float ea[4] = {ea4.x, ea4.y, ea4.z, ea4.w}, uu[4] = {u4.x, u4.y, u4.z, u4.w};
            float gr[4], rd[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float drp = dr[v] * ea[v];
                const float kv = kk[v] * vgy;
                gr[v] = fmaf(uu[v], kv, drp);
                rd[v] = rr[v] * drp;
                gu_acc[v] = fmaf(rr[v], kv, gu_acc[v]);
            }
            if constexpr (SPLIT == 1) {
                if (c0 + t < T) store16(a.gr32 + base, (static_cast<uint32_t>(c0 + t) * C + j4) * 4, f32x4{gr[0], gr[1], gr[2], gr[3]});
            } else {
                if constexpr (SPLIT == 2) { gr[0] += term[0]; gr[1] += term[1]; gr[2] += term[2]; gr[3] += term[3]; }
                *reinterpret_cast<uint2*>(&S.outG[i & 1][t][j4 >> 1]) = make_uint2(pack_bf2(gr[0], gr[1]), pack_bf2(gr[2], gr[3]));
            }
            *reinterpret_cast<float4*>(&S.outR[i & 1][t][j4]) = make_float4(rd[0], rd[1], rd[2], rd[3]);
            staged_now = true;
        } else {
            // exact path: add the two halves; token xt, key channels xj .. xj+3
            const float4 p0 = *reinterpret_cast<const float4*>(&S.Yx[0][xt][xj]);
            const float4 p1 = *reinterpret_cast<const float4*>(&S.Yx[1][xt][xj]);
            const float4 u4 = *reinterpret_cast<const float4*>(&S.u[xj]);
            const float vg = S.Vx[0][xt] + S.Vx[1][xt];
            float rr[4], kk[4];
            unpack4(*reinterpret_cast<const uint2*>(&O.Rr[xt][xj >> 1]), rr);
            unpack4(*reinterpret_cast<const uint2*>(&O.Kr[xt][xj >> 1]), kk);
            const float dr[4] = {p0.x + p1.x, p0.y + p1.y, p0.z + p1.z, p0.w + p1.w}, uu[4] = {u4.x, u4.y, u4.z, u4.w};
            float gr[4], rd[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float kv = kk[e] * vg;
                gr[e] = fmaf(uu[e], kv, dr[e]);
                rd[e] = rr[e] * dr[e];
                gu_x[e] = fmaf(rr[e], kv, gu_x[e]);
            }
            if (c0 + xt < T) {
                const uint32_t o = static_cast<uint32_t>(c0 + xt) * C + xj;
                if constexpr (SPLIT == 2) {            // rare path: read the first launch's term here
                    const f32x4 f = *reinterpret_cast<const f32x4*>(a.gr32 + base + o);
                    gr[0] += f[0]; gr[1] += f[1]; gr[2] += f[2]; gr[3] += f[3];
                }
                if constexpr (SPLIT == 1) store16(a.gr32 + base, o * 4, f32x4{gr[0], gr[1], gr[2], gr[3]});
                else store8(a.gr + base, o * 2, make_uint2(pack_bf2(gr[0], gr[1]), pack_bf2(gr[2], gr[3])));
                store16(a.rdr + base, o * 4, f32x4{rd[0], rd[1], rd[2], rd[3]});
            }
        }
        if (staged) flush(c0 - L, (i & 1) ^ 1);             // the chunk before: its rows were complete at the last barrier
        staged = staged_now;
        __syncthreads();
    }
    if (staged) flush((nchunks - 1) * L, (nchunks - 1) & 1);
    // gu: the chunked path sums over the 16 tokens of a row of lanes; the exact path's sums go by (token, channel) rows
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const float s = row_sum_to_last(gu_acc[v]);
        if (l16 == 15) S.gfast[ih][j4 + v] = s;
    }
    *reinterpret_cast<float4*>(&S.Yx[0][xt][xj]) = make_float4(gu_x[0], gu_x[1], gu_x[2], gu_x[3]);
    __syncthreads();
}

template <int WMODE, int SPLIT = 0>
__global__ __launch_bounds__(NTA) void wkv6_bwd_a_ws(const ArgsB a) {
    __shared__ SmemA2 S;
    if (skip_unflagged(a.only_flagged, blockIdx.x)) return;
    const int tid = threadIdx.x;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int hk = SPLIT != 0 ? h ^ a.cross : h;       // the block of 64 channels that r, k, w, u come from and gr, gu go to
    const size_t vbase = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(h) * N;
    const size_t base = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(hk) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const int nchunks = (a.T + L - 1) / L;
    // positions of the tile that are never written (t < 16 <= s) must read as zero
    for (int i = tid; i < 2 * L * AS; i += NTA) (&S.BmH[0][0])[i] = 0;
    if (tid < N) S.u[tid] = bf2f(a.u[hk * N + tid]);
    if (tid < 128) {
        // One-hot B operand of the transposing products, per lane (column r = l16, K-slot group g), for tile parity p:
        // column r <-> channel 8 (r>>2) + 4 p + (r&3) of a 32-channel half.
        const int p = tid >> 6, ln = tid & 63, c16 = ln & 15, gg = ln >> 4;
        S.sel[p][ln] = one_hot(gg == (c16 >> 2), 4 * p + (c16 & 3));
    }
    if (__builtin_amdgcn_readfirstlane(tid >> 6) < NPREP) bwa_prep<WMODE, SPLIT>(S, a, tid, base, vbase, hk, nchunks);
    // The state waves carry the chunk-to-chunk dependence; the prep waves work ahead and have slack.  Issue priority goes
    // to the state waves (the hardware otherwise favours the oldest waves of a SIMD, which are the prep waves).
    else { __builtin_amdgcn_s_setprio(2); bwa_state<WMODE, SPLIT>(S, a, tid, base, bh, nchunks); }
}

}  // namespace

int launch_wkv6_bwd_a_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                            const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                            const uint16_t* s0, const uint16_t* gy, uint16_t* gr, uint16_t* gu, float* rdr,
                            const int* only_flagged) {
    ArgsB a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.gy = gy;
    a.gr = gr; a.gu = gu; a.rdr = rdr; a.only_flagged = only_flagged;
    if (wmode == W_RAW) hipLaunchKernelGGL(wkv6_bwd_a_ws<W_RAW>, dim3(B * H), dim3(NTA), 0, st, a);
    else if (wmode == W_EW) hipLaunchKernelGGL(wkv6_bwd_a_ws<W_EW>, dim3(B * H), dim3(NTA), 0, st, a);
    else hipLaunchKernelGGL(wkv6_bwd_a_ws<W_HEAD>, dim3(B * H), dim3(NTA), 0, st, a);
    return launch_status();
}

// wkv5 with heads of 128 channels: the first sweep of one of the two launches described at ArgsB (H counts the heads of 128)
int launch_wkv5_bwd_a_split(hipStream_t st, int cross, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k,
                            const uint16_t* v, const float* ew, const uint16_t* u, const uint16_t* gy, float* gr32, float* gu32,
                            uint16_t* gr, uint16_t* gu, float* rdr) {
    ArgsB a{};
    a.T = T; a.C = C; a.H = 2 * H; a.r = r; a.k = k; a.v = v; a.w = ew; a.u = u; a.s0 = nullptr; a.gy = gy;
    a.rdr = rdr; a.cross = cross; a.gr32 = gr32; a.gu32 = gu32; a.gr = gr; a.gu = gu;
    // the first launch leaves its terms in gr32, gu32; the second adds them to its own and writes gr, gu
    if (cross == 0) hipLaunchKernelGGL((wkv6_bwd_a_ws<W_HEAD, 1>), dim3(B * 2 * H), dim3(NTA), 0, st, a);
    else hipLaunchKernelGGL((wkv6_bwd_a_ws<W_HEAD, 2>), dim3(B * 2 * H), dim3(NTA), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
