// wkv6 / wkv6_state forward: chunked formulation, wave-specialised workgroup (gfx950).
//
// One workgroup of 16 waves per (batch, head) walks the sequence in chunks of L = 32 tokens (formulas in wkv6_chunk.h).
//   waves 0..7  ("prep")  load r, k, v, w ahead of time, take the in-chunk decay sums, and write the bf16 hi / lo planes of
//                         R', K' and plain v into LDS in their natural [token][channel] layout; waves 0..2 also form the
//                         causal tile A from those planes.
//   waves 8..15 ("state") wave (q, jh) owns value channels [16q, 16q+16) x key channels [32jh, 32jh+32) of the state:
//                         S^T[j][i] in two 16x16 accumulator tiles.  The two waves of a q exchange one partial y tile
//                         (a 16-byte LDS write and read per lane) and each stores 16 tokens of y straight from registers.
// The two kinds of wave meet at two barriers per chunk and otherwise run different chunks: while the state waves consume
// chunk i, the prep waves write the operands of chunk i+1 (other buffer) and scan chunk i+2.
//
// Every operand whose contraction runs over tokens (v and K' in the state update, v in A V) is needed "transposed", i.e.
// with a lane per channel and the tokens along the K slots.  Instead of writing transposed copies to LDS (narrow, bank
// conflicting stores) the state waves multiply the natural planes by a one-hot selection matrix on the matrix cores:
// the accumulator of  X[token][channel] * Sel  has a lane per selected channel and tokens down the registers, which after
// packing to bf16 (exact: the inputs are bf16) IS the operand layout.  K slots may be assigned to channels or tokens in any
// order as long as both operands agree, so accumulator layouts are used directly everywhere:
//   state tile m, row 4g+v  <->  key channel 32 (m>>1) + 8g + 4 (m&1) + v     (so lane group g reads 8 consecutive channels)
//   token slot (g, e)       <->  token 16 (e>>2) + 4g + (e&3);  A is stored with token s at position 8 ((s&15)>>2) + 4 (s>>4) + (s&3).
#include "wkv6_chunk.h"

namespace rwkv {
namespace {

constexpr int NPREP = 8;
constexpr int NSTATE = 8;
constexpr int NTF = (NPREP + NSTATE) * 64;

struct alignas(16) OperandSet {
    uint32_t RpH[L][OS], RpL[L][OS];   // r e^{c_t - c_m}      hi, lo   (exact path: r as fp32 [t][j] over both planes)
    uint32_t KpH[L][OS], KpL[L][OS];   // k e^{c_m - c_{s+1}}  hi, lo   (exact path: k as fp32)
    uint32_t V[L][OS];                 // v
    float Wx[L][N];                    // exact path: decay of every step
    float d1[N], d2[N], dec[N];        // e^{c_m}, e^{c_L - c_m}, e^{c_L}
    float diag[L];                     // sum_j r u k
    uint32_t exact, pad[3];
};

struct alignas(16) SmemF {
    OperandSet set[2];
    uint32_t AmH[2][L][OS], AmL[2][L][OS];   // A[t][position of s], hi and lo, double buffered
    float4 Xch[2][NSTATE][64];         // partial y tile handed to the partner wave, double buffered
    float Yx[2][2][L][N];              // exact path: partial y of the two key-channel halves, double buffered
    float u[N];
    float part[2][NPREP][N];           // sums of lam over each eighth of a chunk
};

// ---------------------------------------------------------------------------------------------------- prep waves
// base, h: where r, k, w, u of this workgroup sit; vbase: where v sits (the same place unless the head is split)
template <int WMODE>
DEVINL void fwd_prep(SmemF& S, const ArgsC& a, const int tid, const size_t base, const size_t vbase, const int h, const int nchunks) {
    const int lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb = a.v + vbase;
    // channel pair (2 jp, 2 jp + 1), tokens 4 wid + 2 th + {0, 1}
    const int jp = lane & 31, th = lane >> 5, pt0 = 4 * wid + 2 * th;
    const bool second = wid >= 4;
    float uj[2];
    {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.u + h * N + 2 * jp);
        uj[0] = bf_lo(x); uj[1] = bf_hi(x);
    }
    struct Raw { uint32_t r[2], k[2], v[2], w[2]; uint2 wq[2]; float lam[2][2], other[2], kp[2][2]; };
    // fp32 decays take two more registers per token: one stage less keeps the ring in registers
    constexpr int NST = WMODE == W_EW ? STAGES - 1 : STAGES;
    Raw ring[NST];
    // The loads of a chunk are issued NST chunks before they are used.  They are written as asm so that the wait before
    // the first use can name the number of younger loads that may still be in flight (the compiler would wait for all of
    // them); every call issues the same eight loads (chunk index clamped), which keeps that number fixed.
    const uint32_t* __restrict__ wb32 = reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + base);
    const float* __restrict__ wbf = static_cast<const float*>(a.w) + base;
    auto prefetch = [&](int c, Raw& x) __attribute__((always_inline)) {
        c = c < nchunks ? c : nchunks - 1;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = c * L + pt0 + e;
            const uint32_t o = (static_cast<uint32_t>(t < T ? t : T - 1) * C + 2 * jp) * 2;    // byte offset of the channel pair
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.r[e]) : "v"(o), "s"(rb) : "memory");
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.k[e]) : "v"(o), "s"(kb) : "memory");
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.v[e]) : "v"(o), "s"(vb) : "memory");
            if constexpr (WMODE == W_RAW) {
                asm volatile("global_load_dword %0, %1, %2" : "=&v"(x.w[e]) : "v"(o), "s"(wb32) : "memory");
            } else if constexpr (WMODE == W_EW) {
                // straight into the ring: a copy here would read the register before the load has landed
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(x.wq[e]) : "v"(2 * o), "s"(wbf) : "memory");
            }
        }
    };
    // wait until at most `younger` loads issued after those of x are outstanding
    constexpr int NLOADS = WMODE == W_HEAD ? 6 : 8;    // loads per prefetch call
    auto arrived = [&](Raw& x, auto younger) __attribute__((always_inline)) {
        if constexpr (WMODE == W_EW)
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.wq[0]), "+v"(x.wq[1]) : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
        else if constexpr (WMODE == W_RAW)
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1]),
                         "+v"(x.w[0]), "+v"(x.w[1]) : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(x.r[0]), "+v"(x.r[1]), "+v"(x.k[0]), "+v"(x.k[1]), "+v"(x.v[0]), "+v"(x.v[1])
                         : [n] "n"(decltype(younger)::value * NLOADS) : "memory");
    };
    // wkv5: one decay per channel for the whole sequence, given as eew = exp(-exp(w_raw)); lam = log2(eew)
    float lamc[2] = {0.f, 0.f};
    if constexpr (WMODE == W_HEAD) {
        const float2 e2 = *reinterpret_cast<const float2*>(static_cast<const float*>(a.w) + h * N + 2 * jp);
        lamc[0] = __builtin_amdgcn_logf(e2.x); lamc[1] = __builtin_amdgcn_logf(e2.y);
    }
    // wkv5: every full chunk has the same factors, computed here once; a last, partial chunk takes the general route.
    // Tokens between this thread's pair and the middle of the chunk: 14 - pt0 in the first half, pt0 - 16 in the second.
    Scale sc_head[2] = {};
    bool exact_head = false;
    if constexpr (WMODE == W_HEAD) {
        const float between = static_cast<float>(second ? pt0 - 16 : 14 - pt0);
        sc_head[0] = chunk_scale(second, between * lamc[0], lamc[0], lamc[0]);
        sc_head[1] = chunk_scale(second, between * lamc[1], lamc[1], lamc[1]);
        const bool fast_decay = (-4.f * lamc[0] > 0.25f * RANGE_LIMIT * LOG2E) || (-4.f * lamc[1] > 0.25f * RANGE_LIMIT * LOG2E);
        exact_head = __ballot(fast_decay) != 0ull;
        if (wid == 3 && th == 0)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
                *reinterpret_cast<float2*>(&S.set[pb].d1[2 * jp]) = make_float2(exp2_fast(16.f * lamc[0]), exp2_fast(16.f * lamc[1]));
                *reinterpret_cast<float2*>(&S.set[pb].d2[2 * jp]) = make_float2(exp2_fast(16.f * lamc[0]), exp2_fast(16.f * lamc[1]));
                *reinterpret_cast<float2*>(&S.set[pb].dec[2 * jp]) = make_float2(exp2_fast(32.f * lamc[0]), exp2_fast(32.f * lamc[1]));
            }
    }
    auto head_full = [&](const int c) __attribute__((always_inline)) { return WMODE == W_HEAD && c * L + L <= T; };
    static_for<NST>([&](auto Z) { prefetch(decltype(Z)::value, ring[decltype(Z)::value]); });

    // ---- scan of chunk c: lam (log2 units) of this thread's four elements, sums over each eighth of the chunk
    auto scan = [&](const int c, Raw& x) __attribute__((always_inline)) {
        const int c0 = c * L, pb = c & 1;
        if (head_full(c)) {
#pragma unroll
            for (int e = 0; e < 2; ++e) { x.lam[e][0] = lamc[0]; x.lam[e][1] = lamc[1]; }
            return;
        }
        if (c0 + L > T) {                              // last, partial chunk: rows past T carry no input and no decay
#pragma unroll
            for (int e = 0; e < 2; ++e)
                if (c0 + pt0 + e >= T) {
                    x.r[e] = 0; x.k[e] = 0; x.v[e] = 0;
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

    // ---- operands of chunk c into set c & 1, first part: R' planes (and the K' values kept in registers for the second
    //      part); returns whether the chunk takes the exact path
    auto operands_a = [&](const int c, Raw& x) __attribute__((always_inline)) -> bool {
        OperandSet& O = S.set[c & 1];
        const int pb = c & 1;
        const bool hf = head_full(c);
        bool exact = exact_head;
        float near[2] = {0.f, 0.f};
        if (!hf) {
            // sums of lam over the eighths of this thread's half-chunk; those between this wave's eighth and the middle count
            float2 pe[4], po[4];
#pragma unroll
            for (int w4 = 0; w4 < 4; ++w4) {
                pe[w4] = *reinterpret_cast<const float2*>(&S.part[pb][4 * second + w4][2 * jp]);
                po[w4] = *reinterpret_cast<const float2*>(&S.part[pb][4 * !second + w4][2 * jp]);
            }
            exact = chunk_needs_exact_path(pe, po);                              // the same in every wave: a scalar
            near[0] = second ? (th ? x.other[0] : 0.f) : (th ? 0.f : x.other[0]);
            near[1] = second ? (th ? x.other[1] : 0.f) : (th ? 0.f : x.other[1]);
            // eighths between this wave's and the middle: first half w_own+1..3, second half 0..w_own-1 (scalar branches)
            const int w_own = wid & 3;
            const int lo = second ? 0 : w_own + 1, hi = second ? w_own : 4;
            if (lo <= 0 && 0 < hi) { near[0] += pe[0].x; near[1] += pe[0].y; }
            if (lo <= 1 && 1 < hi) { near[0] += pe[1].x; near[1] += pe[1].y; }
            if (lo <= 2 && 2 < hi) { near[0] += pe[2].x; near[1] += pe[2].y; }
            if (lo <= 3 && 3 < hi) { near[0] += pe[3].x; near[1] += pe[3].y; }
        }
        if (tid == 0) O.exact = exact;
        float pr[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) { pr[e][0] = bf_lo(x.r[e]); pr[e][1] = bf_hi(x.r[e]); }
        if (!exact) {
            float rp[2][2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const Scale sc = hf ? sc_head[z] : chunk_scale(second, near[z], x.lam[0][z], x.lam[1][z]);
                rp[0][z] = pr[0][z] * sc.ea[0]; rp[1][z] = pr[1][z] * sc.ea[1];
                x.kp[0][z] = (z ? bf_hi(x.k[0]) : bf_lo(x.k[0])) * sc.eb[0];
                x.kp[1][z] = (z ? bf_hi(x.k[1]) : bf_lo(x.k[1])) * sc.eb[1];
            }
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const HL y = hilo2(rp[e][0], rp[e][1]);
                O.RpH[pt0 + e][jp] = y.h; O.RpL[pt0 + e][jp] = y.l;
            }
        } else {
            float* R = reinterpret_cast<float*>(&O.RpH[0][0]);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<float2*>(&R[(pt0 + e) * N + 2 * jp]) = make_float2(pr[e][0], pr[e][1]);
                *reinterpret_cast<float2*>(&O.Wx[pt0 + e][2 * jp]) = make_float2(exp2_fast(x.lam[e][0]), exp2_fast(x.lam[e][1]));
            }
        }
        return exact;
    };
    // ---- second part: K' planes, v, the diagonal of A; wave 3 adds the per-channel factors of the whole chunk
    auto operands_b = [&](const int c, Raw& x, const bool exact) __attribute__((always_inline)) {
        OperandSet& O = S.set[c & 1];
        const int pb = c & 1;
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
        O.V[pt0][jp] = x.v[0];
        O.V[pt0 + 1][jp] = x.v[1];
        if (wid == 3 && th == 0 && !head_full(c)) {
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

    // ---- causal tile of chunk c (waves 0, 1, 2 -> quadrants (t,s) = (0,0) (1,0) (1,1)); rows of the accumulator are s
    auto tile = [&](const int c) __attribute__((always_inline)) {
        const OperandSet& O = S.set[c & 1];
        const int ta = (wid == 0) ? 0 : 1, tb = (wid == 2) ? 1 : 0;
        f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bf16x8 kh = lds_op(&O.KpH[16 * tb + l16][16 * ks + 4 * g]), kl = lds_op(&O.KpL[16 * tb + l16][16 * ks + 4 * g]);
            const bf16x8 rh = lds_op(&O.RpH[16 * ta + l16][16 * ks + 4 * g]), rl = lds_op(&O.RpL[16 * ta + l16][16 * ks + 4 * g]);
            acc0 = mfma(kh, rh, acc0);
            acc1 = mfma(kh, rl, acc1);
            acc1 = mfma(kl, rh, acc1);
        }
        f32x4 acc = acc0 + acc1;                        // acc[v]: s = 16 tb + 4g + v, t = 16 ta + l16
        if (ta == tb) {
            const float d = O.diag[16 * ta + l16];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int sl = 4 * g + v;
                acc[v] = (sl < l16) ? acc[v] : (sl == l16 ? d : 0.f);
            }
        }
        const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
        *reinterpret_cast<uint2*>(&S.AmH[c & 1][16 * ta + l16][4 * g + 2 * tb]) = make_uint2(x0.h, x1.h);
        *reinterpret_cast<uint2*>(&S.AmL[c & 1][16 * ta + l16][4 * g + 2 * tb]) = make_uint2(x0.l, x1.l);
    };

    static_for<NST>([&](auto Z) { arrived(ring[decltype(Z)::value], std::integral_constant<int, 0>{}); });
    scan(0, ring[0]);
    if (nchunks > 1) scan(1, ring[1]);
    __syncthreads();
    bool exact_cur = operands_a(0, ring[0]);
    operands_b(0, ring[0], exact_cur);
    prefetch(NST, ring[0]);
    __syncthreads();
    // iteration i: scan(i+2), tile(i), operands(i+1); one barrier
    for (int ib = 0; ib < nchunks; ib += NST)
        static_for<NST>([&](auto Z) {
            constexpr int z = decltype(Z)::value;
            const int i = ib + z;
            if (i < nchunks) {
                // younger than the loads of chunk i+2: those of chunks i+3 and i+4
                arrived(ring[(z + 2) % NST], std::integral_constant<int, NST - 2>{});
                if (i + 2 < nchunks) scan(i + 2, ring[(z + 2) % NST]);
                if (wid < 3 && !exact_cur) tile(i);
                bool exact_next = false;
                if (i + 1 < nchunks) {
                    exact_next = operands_a(i + 1, ring[(z + 1) % NST]);
                    operands_b(i + 1, ring[(z + 1) % NST], exact_next);
                }
                prefetch(i + 1 + NST, ring[(z + 1) % NST]);
                __syncthreads();
                exact_cur = exact_next;
            }
        });
    __syncthreads();
}

// ---------------------------------------------------------------------------------------------------- state waves
// SPLIT: 0 = whole heads; 1 = first launch of a split head (y leaves as an fp32 term); 2 = second launch (the first
// launch's term is added and y leaves in bf16)
template <int WMODE, int SPLIT>
DEVINL void fwd_state(SmemF& S, const ArgsC& a, const int tid, const size_t base, const size_t bh, const int nchunks) {
    const int lane = tid & 63, sw = __builtin_amdgcn_readfirstlane(tid >> 6) - NPREP, q = sw & 3, jh = sw >> 2, l16 = lane & 15, g = lane >> 4;
    const int T = a.T, C = a.C;
    const int i_own = 16 * q + l16;                    // this lane's value channel as a column of the state tiles
    const int j0[2] = {32 * jh + 8 * g, 32 * jh + 8 * g + 4};   // first key channel of this lane's four rows in tile mm

    f32x4 D[2];
    D[0] = D[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.s0 != nullptr) {
        const uint4 x = *reinterpret_cast<const uint4*>(a.s0 + (bh * N + i_own) * N + j0[0]);
        D[0] = f32x4{bf_lo(x.x), bf_hi(x.x), bf_lo(x.y), bf_hi(x.y)};
        D[1] = f32x4{bf_lo(x.z), bf_hi(x.z), bf_lo(x.w), bf_hi(x.w)};
    }
    // selection matrices (B operands).  v: column n <-> channel 16q + n of the 32-channel half q>>1;
    // K', parity p: column n = row r of a state tile <-> channel 8 (r>>2) + 4p + (r&3) of the half jh.
    const bf16x8 selV = op4(one_hot(g == 2 * (q & 1) + (l16 >> 3), l16 & 7));
    const bf16x8 selK0 = op4(one_hot(g == (l16 >> 2), l16 & 3));
    const bf16x8 selK1 = op4(one_hot(g == (l16 >> 2), 4 + (l16 & 3)));
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

    bf16x8 Vop = op4(make_uint4(0, 0, 0, 0));          // v of the chunk in flight: lane = value channel, K slots = tokens
    f32x4 Yk = zero4;                                  // y^T rows 16q + 4g + v, tokens 16 jh + l16: this half of the key channels
    [[maybe_unused]] float4 term = make_float4(0.f, 0.f, 0.f, 0.f);   // SPLIT == 2: the first launch's term of the tile in flight
    auto fetch_term = [&](const int c) __attribute__((always_inline)) {
        if constexpr (SPLIT == 2) {
            const int t = c * L + 16 * jh + l16;
            term = *reinterpret_cast<const float4*>(a.y32 + base + static_cast<size_t>(t < T ? t : T - 1) * C + 16 * q + 4 * g);
        }
    };

    // y of chunk c (tokens 16 jh + l16): own half + partner's half + A V
    auto finish = [&](const int c, const bool was_exact) __attribute__((always_inline)) {
        if (!was_exact) {
            const float4 p = S.Xch[c & 1][sw ^ 4][lane];
            f32x4 Y = Yk + f32x4{p.x, p.y, p.z, p.w};
            Y = mfma(Vop, lds_op(&S.AmH[c & 1][16 * jh + l16][4 * g]), Y);
            Y = mfma(Vop, lds_op(&S.AmL[c & 1][16 * jh + l16][4 * g]), Y);
            const int t = c * L + 16 * jh + l16;
            if constexpr (SPLIT == 2) { Y[0] += term.x; Y[1] += term.y; Y[2] += term.z; Y[3] += term.w; }
            if (t < T) {
                if constexpr (SPLIT == 1)
                    *reinterpret_cast<float4*>(a.y32 + base + static_cast<size_t>(t) * C + 16 * q + 4 * g) = make_float4(Y[0], Y[1], Y[2], Y[3]);
                else
                    *reinterpret_cast<uint2*>(a.y + base + static_cast<size_t>(t) * C + 16 * q + 4 * g) =
                        make_uint2(pack_bf2(Y[0], Y[1]), pack_bf2(Y[2], Y[3]));
            }
        } else {                                       // exact path: add the two halves and store
            const int idx = tid - NPREP * 64, t = idx >> 4, i4 = (idx & 15) * 4;
            const float4 p0 = *reinterpret_cast<const float4*>(&S.Yx[c & 1][0][t][i4]);
            const float4 p1 = *reinterpret_cast<const float4*>(&S.Yx[c & 1][1][t][i4]);
            if (c * L + t < T) {
                float4 s4 = make_float4(p0.x + p1.x, p0.y + p1.y, p0.z + p1.z, p0.w + p1.w);
                if constexpr (SPLIT == 2) {            // this thread's elements are not those of `term`: read here (rare path)
                    const float4 f = *reinterpret_cast<const float4*>(a.y32 + base + static_cast<size_t>(c * L + t) * C + i4);
                    s4 = make_float4(s4.x + f.x, s4.y + f.y, s4.z + f.z, s4.w + f.w);
                }
                if constexpr (SPLIT == 1)
                    *reinterpret_cast<float4*>(a.y32 + base + static_cast<size_t>(c * L + t) * C + i4) = s4;
                else
                    *reinterpret_cast<uint2*>(a.y + base + static_cast<size_t>(c * L + t) * C + i4) =
                        make_uint2(pack_bf2(s4.x, s4.y), pack_bf2(s4.z, s4.w));
            }
        }
    };

    __syncthreads();
    __syncthreads();
    bool exact_prev = false;
    for (int i = 0; i < nchunks; ++i) {
        const OperandSet& O = S.set[i & 1];
        const bool exact = __builtin_amdgcn_readfirstlane(O.exact) != 0;
        if (i > 0) finish(i - 1, exact_prev);
        fetch_term(i);                                 // used by finish(i), one iteration from here
        if constexpr (SPLIT == 0) {
            if (a.saved != nullptr && !(i & 1)) {      // the state entering every even chunk, for the one-sweep backward
                char* dst = a.saved + (bh * ((nchunks + 1) / 2) + (i >> 1)) * SAVED_STATE_B;
                saved_put4(dst, i_own, j0[0], D[0]);
                saved_put4(dst, i_own, j0[1], D[1]);
            }
        }
        if (!exact) {
            // ------------------------------------------------------------ y^T = (d1 S) R'^T over this wave's key channels
            const float4 da = *reinterpret_cast<const float4*>(&O.d1[j0[0]]);
            const float4 db = *reinterpret_cast<const float4*>(&O.d1[j0[1]]);
            const bf16x8 rh0 = lds_op(&O.RpH[l16][16 * jh + 4 * g]), rl0 = lds_op(&O.RpL[l16][16 * jh + 4 * g]);
            const bf16x8 rh1 = lds_op(&O.RpH[16 + l16][16 * jh + 4 * g]), rl1 = lds_op(&O.RpL[16 + l16][16 * jh + 4 * g]);
            const bf16x8 va0 = lds_op(&O.V[l16][16 * (q >> 1) + 4 * g]), va1 = lds_op(&O.V[16 + l16][16 * (q >> 1) + 4 * g]);
            const HL x0 = hilo2(D[0][0] * da.x, D[0][1] * da.y), x1 = hilo2(D[0][2] * da.z, D[0][3] * da.w);
            const HL x2 = hilo2(D[1][0] * db.x, D[1][1] * db.y), x3 = hilo2(D[1][2] * db.z, D[1][3] * db.w);
            const bf16x8 sh = as_op(x0.h, x1.h, x2.h, x3.h), sl = as_op(x0.l, x1.l, x2.l, x3.l);
            f32x4 Y0 = mfma(sh, rh0, zero4), Y1 = mfma(sh, rh1, zero4);
            Y0 = mfma(sh, rl0, Y0); Y1 = mfma(sh, rl1, Y1);
            Y0 = mfma(sl, rh0, Y0); Y1 = mfma(sl, rh1, Y1);
            // the partner wave (other key-channel half) finishes the other 16 tokens
            S.Xch[i & 1][sw][lane] = jh ? make_float4(Y0[0], Y0[1], Y0[2], Y0[3]) : make_float4(Y1[0], Y1[1], Y1[2], Y1[3]);
            Yk = jh ? Y1 : Y0;
            // ------------------------------------------------------------ v with a lane per value channel
            const f32x4 z0 = mfma(va0, selV, zero4), z1 = mfma(va1, selV, zero4);
            Vop = as_op(cvt2(z0[0], z0[1]), cvt2(z0[2], z0[3]), cvt2(z1[0], z1[1]), cvt2(z1[2], z1[3]));
            // ------------------------------------------------------------ S^T = diag(dec) S^T + diag(d2) K'^T V
            const bf16x8 ah0 = lds_op(&O.KpH[l16][16 * jh + 4 * g]), ah1 = lds_op(&O.KpH[16 + l16][16 * jh + 4 * g]);
            const bf16x8 al0 = lds_op(&O.KpL[l16][16 * jh + 4 * g]), al1 = lds_op(&O.KpL[16 + l16][16 * jh + 4 * g]);
#pragma unroll
            for (int par = 0; par < 2; ++par) {
                const bf16x8 sel = par ? selK1 : selK0;
                const f32x4 zh0 = mfma(ah0, sel, zero4), zh1 = mfma(ah1, sel, zero4);
                const f32x4 zl0 = mfma(al0, sel, zero4), zl1 = mfma(al1, sel, zero4);
                const bf16x8 kh = as_op(cvt2(zh0[0], zh0[1]), cvt2(zh0[2], zh0[3]), cvt2(zh1[0], zh1[1]), cvt2(zh1[2], zh1[3]));
                const bf16x8 kl = as_op(cvt2(zl0[0], zl0[1]), cvt2(zl0[2], zl0[3]), cvt2(zl1[0], zl1[1]), cvt2(zl1[2], zl1[3]));
                f32x4 U = mfma(kh, Vop, zero4);
                U = mfma(kl, Vop, U);
                const float4 de = *reinterpret_cast<const float4*>(&O.dec[j0[par]]);
                const float4 d2 = *reinterpret_cast<const float4*>(&O.d2[j0[par]]);
                D[par][0] = fmaf(D[par][0], de.x, d2.x * U[0]); D[par][1] = fmaf(D[par][1], de.y, d2.y * U[1]);
                D[par][2] = fmaf(D[par][2], de.z, d2.z * U[2]); D[par][3] = fmaf(D[par][3], de.w, d2.w * U[3]);
            }
        } else {
            // ------------------------------------------------------------ exact path: 32 sequential steps
            const float* R = reinterpret_cast<const float*>(&O.RpH[0][0]);
            const float* K = reinterpret_cast<const float*>(&O.KpH[0][0]);
            float uv[2][4];
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const float4 y = *reinterpret_cast<const float4*>(&S.u[j0[m]]);
                uv[m][0] = y.x; uv[m][1] = y.y; uv[m][2] = y.z; uv[m][3] = y.w;
            }
            for (int t4 = 0; t4 < L; t4 += 4) {
                float yp[4];                            // four steps, then their sums over the lane rows in one go
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int t = t4 + s;
                    const uint32_t vv = O.V[t][i_own >> 1];
                    const float vi = (l16 & 1) ? bf_hi(vv) : bf_lo(vv);
                    yp[s] = 0.f;
#pragma unroll
                    for (int m = 0; m < 2; ++m) {
                        const float4 r4 = *reinterpret_cast<const float4*>(&R[t * N + j0[m]]);
                        const float4 k4 = *reinterpret_cast<const float4*>(&K[t * N + j0[m]]);
                        const float4 w4 = *reinterpret_cast<const float4*>(&O.Wx[t][j0[m]]);
                        const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const float kv = kk[v] * vi;
                            yp[s] = fmaf(rr[v], fmaf(uv[m][v], kv, D[m][v]), yp[s]);
                            D[m][v] = fmaf(D[m][v], ww[v], kv);
                        }
                    }
                }
                S.Yx[i & 1][jh][t4 + g][i_own] = reduce4_rows(yp[0], yp[1], yp[2], yp[3]);   // lane row g holds step t4 + g
            }
        }
        __syncthreads();
        exact_prev = exact;
    }
    __syncthreads();
    finish(nchunks - 1, exact_prev);
}

template <int WMODE, int SPLIT = 0>
__global__ __launch_bounds__(NTF) void wkv6_fwd_ws(const ArgsC a) {
    __shared__ SmemF S;
    const int tid = threadIdx.x;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const size_t base = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const int nchunks = (a.T + L - 1) / L;
    if (skip_unflagged(a.only_flagged, blockIdx.x)) return;
    // positions of A that no tile ever writes (t < 16 <= s) must read as zero
    for (int i = tid; i < 2 * L * OS; i += NTF) { (&S.AmH[0][0][0])[i] = 0; (&S.AmL[0][0][0])[i] = 0; }
    if constexpr (SPLIT != 0) {
        const int hk = h ^ a.cross;                    // the block of 64 channels that r, k, w, u come from
        const size_t kbase = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(hk) * N;
        if (tid < N) S.u[tid] = bf2f(a.u[hk * N + tid]);
        if (__builtin_amdgcn_readfirstlane(tid >> 6) < NPREP) fwd_prep<WMODE>(S, a, tid, kbase, base, hk, nchunks);
        else fwd_state<WMODE, SPLIT>(S, a, tid, base, bh, nchunks);
    } else {
        if (tid < N) S.u[tid] = bf2f(a.u[h * N + tid]);
        if (__builtin_amdgcn_readfirstlane(tid >> 6) < NPREP) fwd_prep<WMODE>(S, a, tid, base, base, h, nchunks);
        else fwd_state<WMODE, 0>(S, a, tid, base, bh, nchunks);
    }
}

}  // namespace

int launch_wkv6_fwd_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                          const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                          const uint16_t* s0, uint16_t* y, char* saved, const int* only_flagged) {
    ArgsC a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.y = y; a.saved = saved;
    a.only_flagged = only_flagged;
    if (wmode == W_RAW) hipLaunchKernelGGL(wkv6_fwd_ws<W_RAW>, dim3(B * H), dim3(NTF), 0, st, a);
    else if (wmode == W_EW) hipLaunchKernelGGL(wkv6_fwd_ws<W_EW>, dim3(B * H), dim3(NTF), 0, st, a);
    else hipLaunchKernelGGL(wkv6_fwd_ws<W_HEAD>, dim3(B * H), dim3(NTF), 0, st, a);
    return launch_status();
}

// wkv5 with heads of 128 channels: one of the two launches described at ArgsB (H counts the heads of 128)
int launch_wkv5_fwd_split(hipStream_t st, int cross, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k,
                          const uint16_t* v, const float* eew, const uint16_t* u, float* y32, uint16_t* y) {
    ArgsC a{};
    a.T = T; a.C = C; a.H = 2 * H; a.r = r; a.k = k; a.v = v; a.w = eew; a.u = u; a.s0 = nullptr; a.y = y;
    a.cross = cross; a.y32 = y32;
    // the first launch leaves its term in y32, the second adds it to its own and writes y
    if (cross == 0) hipLaunchKernelGGL((wkv6_fwd_ws<W_HEAD, 1>), dim3(B * 2 * H), dim3(NTF), 0, st, a);
    else hipLaunchKernelGGL((wkv6_fwd_ws<W_HEAD, 2>), dim3(B * 2 * H), dim3(NTF), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
