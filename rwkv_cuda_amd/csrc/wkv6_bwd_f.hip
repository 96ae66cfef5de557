// wkv6 / wkv6_state backward in ONE reverse sweep (gfx950), from the chunk states that the forward kernel saved.
//
// Formulas (wkv6_chunk.h for R', K', d1, d2, dec; chunk of L = 32 tokens, factors referred to its middle m = 16):
//     Bm[t][s] = gy_t . v_s (s < t)              A[t][s] = R'_t . K'_s (s < t),  A[t][t] = sum_j r u k
//     X_t = GY_t (S0 d1) + sum_{s<t} Bm[t][s] K'_s            dr'_t = ea_t X_t      gr = dr' + u k_t (v_t . gy_t)
//     Z_s = V_s (dS d2) + sum_{t>s} Bm[t][s] R'_t             dk'_s = eb_s Z_s      gk = dk' + u r_s (v_s . gy_s)
//     gv_s = (dS d2) K'_s + sum_{t>=s} A[t][s] gy_t
//     dS <- dS dec + d1 GY^T R'                               (gradient of the state that enters the chunk)
//     gw_t = lam_t G_t,  G_t = P_{t+1} - k_t dk'_t,  P_t = P_{t+1} + r_t dr'_t - k_t dk'_t,  P = sum_i dS S exactly where a saved state is at hand
// S0 = the forward state entering the chunk: the forward kernel stores it for every second chunk (fp32, [value][key]);
// the state of the odd chunk in between is rebuilt here with one update, S <- S dec + d2 V^T K'.
//
// One workgroup of 12 waves per (batch, head), three roles of four waves each; wave w of a role owns 16 channels:
//   P  (prep)   channels 16w..16w+15 of r, k, w, v, gy for all 32 tokens of a chunk: lane = 16 * (channel quad) + token,
//               so the time scans of a half-chunk are four DPP adds inside a 16-lane row and no prep wave ever needs
//               another one's sums.  Writes the bf16 hi / lo planes of R', K', plain v, gy; keeps r, k and the exponents
//               cc_t = log2 ea_t of the chunks in flight in registers and, three iterations later, turns the X and Z of
//               that chunk into gr, gk, gw (and gu) and stores them: all elementwise work sits where the inputs are.
//   SD (states) forward state S[i][j] and gradient state dS[i][j], key channels j = 16w..: lane = j, registers = i.
//               X, Z, gs, the dS update, P at the anchors.
//   E  (dstate^T) dS[i][j], value channels i = 16w..: lane = i, registers = j.  gv, dS update, and the causal tiles A, Bm of
//               the next chunk.
// A state is the accumulator of its update product and, as it stands, the A operand of the products that read it
// (K slots <-> channels in accumulator order).  Operands with the tokens along K come from the natural [token][channel]
// planes through ds_read_b64_tr_b16: 16 lanes read a 4 x 16 block and each ends up with one column of it.
// The accumulators of X, Z, gv have lane = token and four consecutive channels in registers -- the layout of the prep
// waves: X and Z cross to prep wave w through LDS lane for lane, gv is stored from registers.
//
// Pipeline (one barrier per chunk): in iteration `it` the P waves prepare chunk n-1-it, the EW waves make the tiles of
// chunk n-it, the SD and E waves do the products of chunk n+1-it, and the P waves finish chunk n+2-it.
//
// A chunk in which some channel decays by more than e^-60 over either half cannot use the mid-point factors.  Such a
// (batch, head) is flagged in `flags` and the caller reruns it with the two-sweep kernels, which have a step-by-step path.
#include "wkv6_chunk.h"

namespace rwkv {
namespace {

constexpr int NTG = 12 * 64;           // 3 waves per SIMD: 168 registers per lane
constexpr int CS = 72;             // row stride (dwords) of an fp32 [token][channel] array

struct alignas(16) SlotG {
    uint32_t RpH[L][OS], RpL[L][OS], KpH[L][OS], KpL[L][OS], V[L][OS], GY[L][OS];
    float d1[N], d2[N], dec[N], l2[N];     // 2^{c_m}, 2^{c_L - c_m}, 2^{c_L}, cc_32 = c_L - c_m
    float ruk[4][L];                        // sum of r u k over the 16 channels of each prep wave
};
struct alignas(16) TilesG {
    uint32_t AH[L][AS], AL[L][AS], BH[L][AS], BL[L][AS];   // [t][s] bf16 hi / lo
};
struct alignas(16) SmemG {
    SlotG slot[3];
    TilesG tile[2];
    float xz[2][2][L][CS];                  // [chunk parity][X, Z][token][key channel]: from SD wave w to P wave w
    float vg[4][L];                         // v_t . gy_t of the chunks in flight
    float pex[2][N];                        // P = sum_i dS S at the last two anchors
};
static_assert(sizeof(SmemG) <= 160 * 1024, "LDS");

typedef short v4s __attribute__((ext_vector_type(4)));
typedef v4s __attribute__((address_space(3))) * lds_v4s_ptr;

// Operand with the rows of an LDS matrix along K: slot (g, e) <-> row row0 + e (e = 0..7), lane l16 <-> column col + l16.
// p points at element [row0][col] of a matrix of bf16 with `stride` dwords per row; row0 = 8 g for a 32-row contraction.
DEVINL bf16x8 tr_pair(const uint32_t* p, const int stride, const int l16) {
    const uint32_t* q = p + (l16 >> 2) * stride + 2 * (l16 & 3);
    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(q));
    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(q + 4 * stride));
    const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return as_op(a.x, a.y, b.x, b.y);
}
// Operand with channels along K in accumulator order: slot (g, e) <-> channel 32 ks + 16 (e >> 2) + 4 g + (e & 3).
// row points at the first dword of a [token] row of a bf16 plane.
DEVINL bf16x8 acc_order_op(const uint32_t* row, const int ks, const int g) {
    const uint2 a = *reinterpret_cast<const uint2*>(row + 16 * ks + 2 * g);
    const uint2 b = *reinterpret_cast<const uint2*>(row + 16 * ks + 8 + 2 * g);
    return as_op(a.x, a.y, b.x, b.y);
}
// inclusive prefix sum over the 16 lanes of a row: lane l gets the sum of lanes 0..l
DEVINL float row_prefix_sum(float x) {
    x = dpp_add<0x111, 0xf>(x);       // row_shr:1
    x = dpp_add<0x112, 0xf>(x);
    x = dpp_add<0x114, 0xf>(x);
    x = dpp_add<0x118, 0xf>(x);
    return x;
}
// value of the next lane of the row (lane 15 gets 0)
DEVINL float row_next(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x101, 0xf, 0xf, true));
}
DEVINL void split16(const f32x4 (&x)[4], const float s, bf16x8 (&h)[2], bf16x8 (&l)[2]) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const HL a = hilo2(x[2 * ks][0] * s, x[2 * ks][1] * s), b = hilo2(x[2 * ks][2] * s, x[2 * ks][3] * s);
        const HL c = hilo2(x[2 * ks + 1][0] * s, x[2 * ks + 1][1] * s), d = hilo2(x[2 * ks + 1][2] * s, x[2 * ks + 1][3] * s);
        h[ks] = as_op(a.h, b.h, c.h, d.h);
        l[ks] = as_op(a.l, b.l, c.l, d.l);
    }
}

struct ArgsG {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *gy;
    const void* w;
    uint16_t *gr, *gk, *gv, *gw, *gu, *gs;
    const float* saved;            // [B*H][ceil(n/2)][64][64]: the forward state entering every even chunk
    int* flags;                    // [B*H][4]
};

// state entering even chunk e of this (batch, head), in the layout of the SD waves: lane <-> key channel 16w + l16,
// x[tile][v] <-> value channel 16 tile + 4g + v
DEVINL void load_state(const float* __restrict__ p, f32x4 (&x)[4], const int g) {
#pragma unroll
    for (int tl = 0; tl < 4; ++tl)
#pragma unroll
        for (int v = 0; v < 4; ++v) x[tl][v] = p[(16 * tl + 4 * g + v) * N];
}

// ---------------------------------------------------------------------------------------------------- P waves
template <int WMODE>
DEVINL void role_prep(SmemG& S, const ArgsG& a, const int lane, const int w, const size_t base, const int h, const size_t bh, const int n) {
    const int jq = lane >> 4, tp = lane & 15, ch = 16 * w + 4 * jq;
    const int T = a.T, C = a.C;
    // wave-uniform bases plus one 32-bit per-lane offset: the addresses stay out of the vector registers
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb = a.v + base;
    const uint16_t* __restrict__ gb = a.gy + base;
    const uint16_t* __restrict__ wb = static_cast<const uint16_t*>(a.w) + base;
    float uj[4];
    {
        const uint2 x = *reinterpret_cast<const uint2*>(a.u + h * N + ch);
        uj[0] = bf_lo(x.x); uj[1] = bf_hi(x.x); uj[2] = bf_lo(x.y); uj[3] = bf_hi(x.y);
    }
    // r, k, w are needed by the arithmetic of a preparation and are fetched two chunks ahead; v, gy are only copied
    // into their planes at its end and are fetched one chunk ahead
    struct Raw { uint2 r[2], k[2], w[2]; };
    struct RawVG { uint2 v[2], g[2]; };
    Raw ring[2];
    RawVG vgn;
    auto row_of = [&](const int c, const int e) __attribute__((always_inline)) {
        const int t = c * L + tp + 16 * e;
        return static_cast<uint32_t>(t < T ? t : T - 1) * C + ch;
    };
    auto fetch = [&](const int c, Raw& x) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t o = row_of(c, e);
            x.r[e] = *reinterpret_cast<const uint2*>(rb + o);
            x.k[e] = *reinterpret_cast<const uint2*>(kb + o);
            x.w[e] = *reinterpret_cast<const uint2*>(wb + o);
        }
    };
    auto fetch_vg = [&](const int c, RawVG& x) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t o = row_of(c, e);
            x.v[e] = *reinterpret_cast<const uint2*>(vb + o);
            x.g[e] = *reinterpret_cast<const uint2*>(gb + o);
        }
    };
    // what the finishing of a chunk needs from its preparation, three iterations earlier
    struct Held { uint2 r[2], k[2]; float cc[2][4]; };
    Held hq[3] = {};
    bool any_exact = false;
    float carry[4] = {0.f, 0.f, 0.f, 0.f}, gu_acc[4] = {0.f, 0.f, 0.f, 0.f};

    auto prep = [&](const int c, Raw& x, Held& hd) __attribute__((always_inline)) {
        SlotG& O = S.slot[c % 3];
        float lam[2][4], rf[2][4], kf[2][4];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const bool live = c * L + tp + 16 * e < T;
            if (!live) { x.r[e] = make_uint2(0, 0); x.k[e] = make_uint2(0, 0); }
            float wf[4];
            unpack4(x.w[e], wf); unpack4(x.r[e], rf[e]); unpack4(x.k[e], kf[e]);
#pragma unroll
            for (int z = 0; z < 4; ++z) lam[e][z] = live ? -LOG2E * exp2_fast(LOG2E * wf[z]) : 0.f;
            hd.r[e] = x.r[e]; hd.k[e] = x.k[e];
        }
        float l1[4], l2[4];
#pragma unroll
        for (int z = 0; z < 4; ++z) {
            const float s0 = row_suffix_sum(lam[0][z]);        // sum over tokens tp..15
            const float p1 = row_prefix_sum(lam[1][z]);        // sum over tokens 16..16+tp
            hd.cc[0][z] = -s0;
            hd.cc[1][z] = p1 - lam[1][z];
            l1[z] = bc<0>(s0);
            l2[z] = bc<15>(p1);
        }
        {
            bool bad = false;
#pragma unroll
            for (int z = 0; z < 4; ++z) bad = bad || (-l1[z] > RANGE_LIMIT * LOG2E) || (-l2[z] > RANGE_LIMIT * LOG2E);
            any_exact = any_exact || (__ballot(bad) != 0ull);
        }
        if (tp == 0) {
            *reinterpret_cast<float4*>(&O.d1[ch]) = make_float4(exp2_fast(l1[0]), exp2_fast(l1[1]), exp2_fast(l1[2]), exp2_fast(l1[3]));
            *reinterpret_cast<float4*>(&O.d2[ch]) = make_float4(exp2_fast(l2[0]), exp2_fast(l2[1]), exp2_fast(l2[2]), exp2_fast(l2[3]));
            *reinterpret_cast<float4*>(&O.dec[ch]) = make_float4(exp2_fast(l1[0] + l2[0]), exp2_fast(l1[1] + l2[1]), exp2_fast(l1[2] + l2[2]), exp2_fast(l1[3] + l2[3]));
            *reinterpret_cast<float4*>(&O.l2[ch]) = make_float4(l2[0], l2[1], l2[2], l2[3]);
        }
        float ruk[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = tp + 16 * e;
            float rp[4], kp[4];
            ruk[e] = 0.f;
#pragma unroll
            for (int z = 0; z < 4; ++z) {
                rp[z] = rf[e][z] * exp2_fast(hd.cc[e][z]);
                kp[z] = kf[e][z] * exp2_fast(-(hd.cc[e][z] + lam[e][z]));
                ruk[e] = fmaf(rf[e][z] * uj[z], kf[e][z], ruk[e]);
            }
            const HL r0 = hilo2(rp[0], rp[1]), r1 = hilo2(rp[2], rp[3]), k0 = hilo2(kp[0], kp[1]), k1 = hilo2(kp[2], kp[3]);
            *reinterpret_cast<uint2*>(&O.RpH[t][8 * w + 2 * jq]) = make_uint2(r0.h, r1.h);
            *reinterpret_cast<uint2*>(&O.RpL[t][8 * w + 2 * jq]) = make_uint2(r0.l, r1.l);
            *reinterpret_cast<uint2*>(&O.KpH[t][8 * w + 2 * jq]) = make_uint2(k0.h, k1.h);
            *reinterpret_cast<uint2*>(&O.KpL[t][8 * w + 2 * jq]) = make_uint2(k0.l, k1.l);
        }
        allreduce2_rows(ruk[0], ruk[1]);                       // sums over the four channel quads of this wave
        if (jq == 0) { O.ruk[w][tp] = ruk[0]; O.ruk[w][tp + 16] = ruk[1]; }
    };
    // v, gy of chunk c into their planes.  This comes first in an iteration: the loads it waits for are then older than
    // everything else in flight except the r, k, w of the next chunk, which the wait can count.
    auto copy_vg = [&](const int c, const RawVG& y) __attribute__((always_inline)) {
        SlotG& O = S.slot[c % 3];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const bool live = c * L + tp + 16 * e < T;
            *reinterpret_cast<uint2*>(&O.V[tp + 16 * e][8 * w + 2 * jq]) = live ? y.v[e] : make_uint2(0, 0);
            *reinterpret_cast<uint2*>(&O.GY[tp + 16 * e][8 * w + 2 * jq]) = live ? y.g[e] : make_uint2(0, 0);
        }
    };

    // gr, gk, gw of chunk c from X, Z (left by SD wave w in the last iteration) and what prep kept
    auto finish = [&](const int c, const Held& hd) __attribute__((always_inline)) {
        const float4 e4 = *reinterpret_cast<const float4*>(&S.slot[c % 3].l2[ch]);
        const float l2v[4] = {e4.x, e4.y, e4.z, e4.w};
        float q[2][4], kdk[2][4], lam[2][4];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = tp + 16 * e, tg = c * L + t;
            const float4 x4 = *reinterpret_cast<const float4*>(&S.xz[c & 1][0][t][ch]);
            const float4 z4 = *reinterpret_cast<const float4*>(&S.xz[c & 1][1][t][ch]);
            const float X[4] = {x4.x, x4.y, x4.z, x4.w}, Z[4] = {z4.x, z4.y, z4.z, z4.w};
            const float vg = S.vg[c & 3][t];
            float rf[4], kf[4], gr[4], gk[4];
            unpack4(hd.r[e], rf); unpack4(hd.k[e], kf);
#pragma unroll
            for (int z = 0; z < 4; ++z) {
                const float cc = hd.cc[e][z];
                const float nx = row_next(cc);
                const float ccn = tp == 15 ? (e ? l2v[z] : 0.f) : nx;
                const float drp = exp2_fast(cc) * X[z], dkp = exp2_fast(-ccn) * Z[z];
                const float uvg = uj[z] * vg;
                gr[z] = fmaf(uvg, kf[z], drp);
                gk[z] = fmaf(uvg, rf[z], dkp);
                kdk[e][z] = kf[z] * dkp;
                q[e][z] = fmaf(rf[z], drp, -kdk[e][z]);
                gu_acc[z] = fmaf(rf[z] * kf[z], vg, gu_acc[z]);
                lam[e][z] = gw_factor((ccn - cc) * LN2);
            }
            if (tg < T) {
                const uint32_t o = static_cast<uint32_t>(tg) * C + ch;
                *reinterpret_cast<uint2*>(a.gr + base + o) = make_uint2(pack_bf2(gr[0], gr[1]), pack_bf2(gr[2], gr[3]));
                *reinterpret_cast<uint2*>(a.gk + base + o) = make_uint2(pack_bf2(gk[0], gk[1]), pack_bf2(gk[2], gk[3]));
            }
        }
        float gw[2][4];
#pragma unroll
        for (int z = 0; z < 4; ++z) {
            const float s1 = row_suffix_sum(q[1][z]) + carry[z];           // P_t of the second half
            const float s0 = row_suffix_sum(q[0][z]) + bc<0>(s1);
            gw[1][z] = lam[1][z] * ((s1 - q[1][z]) - kdk[1][z]);          // lam (P_{t+1} - k dk')
            gw[0][z] = lam[0][z] * ((s0 - q[0][z]) - kdk[0][z]);
            carry[z] = bc<0>(s0);
        }
        if (!(c & 1)) {
            // the chunk began at an anchor: from here on P counts from its exact value there
            const float4 p4 = *reinterpret_cast<const float4*>(&S.pex[(c >> 1) & 1][ch]);
            carry[0] = p4.x; carry[1] = p4.y; carry[2] = p4.z; carry[3] = p4.w;
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int tg = c * L + tp + 16 * e;
            if (tg < T)
                *reinterpret_cast<uint2*>(a.gw + base + (static_cast<uint32_t>(tg) * C + ch)) =
                    make_uint2(pack_bf2(gw[e][0], gw[e][1]), pack_bf2(gw[e][2], gw[e][3]));
        }
    };

    fetch_vg(n - 1, vgn);
    fetch(n - 1, ring[0]);
    fetch(n >= 2 ? n - 2 : 0, ring[1]);
    for (int it0 = 0; it0 <= n + 2; it0 += 2)
        static_for<2>([&](auto Z) {
            constexpr int z = decltype(Z)::value;
            const int it = it0 + z;
            if (it <= n + 2) {
                const int cp = n - 1 - it;
                // The same loads in every iteration (chunk index clamped): the wait for a chunk's registers is then the
                // count of loads issued after them on every path, and never has to cover the newest ones.
                if (cp >= 0) copy_vg(cp, vgn);
                fetch_vg(cp >= 1 ? cp - 1 : 0, vgn);
                __builtin_amdgcn_sched_barrier(0);
                if (it >= 3) finish(cp + 3, hq[2]);
                __builtin_amdgcn_sched_barrier(0);
                hq[2] = hq[1]; hq[1] = hq[0];
                if (cp >= 0) prep(cp, ring[z], hq[0]);
                __builtin_amdgcn_sched_barrier(0);
                fetch(cp >= 2 ? cp - 2 : 0, ring[z]);
                __syncthreads();
            }
        });
    if (lane == 0) a.flags[bh * 4 + w] = any_exact ? 1 : 0;
    // gu of this batch row: sum over the tokens (lanes of a row)
#pragma unroll
    for (int z = 0; z < 4; ++z) gu_acc[z] = row_sum_to_last(gu_acc[z]);
    if (tp == 15)
        *reinterpret_cast<uint2*>(a.gu + bh * N + ch) = make_uint2(pack_bf2(gu_acc[0], gu_acc[1]), pack_bf2(gu_acc[2], gu_acc[3]));
}

// ---------------------------------------------------------------------------------------------------- SD waves
template <int WMODE>
DEVINL void role_sd(SmemG& S, const ArgsG& a, const int lane, const int w, const size_t bh, const int n) {
    const int g = lane >> 4, l16 = lane & 15, j = 16 * w + l16;
    const int nseg = (n + 1) / 2;
    const float* __restrict__ sv = a.saved + bh * nseg * (N * N) + j;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 D[4] = {zero4, zero4, zero4, zero4};
    // one chunk: X and Z of chunk c, the update of dS, and P at an anchor; Sa = the saved state of the chunk's segment
    auto chunk = [&](const int c, const f32x4 (&Sa)[4]) __attribute__((always_inline)) {
        const SlotG& O = S.slot[c % 3];
        const TilesG& Tl = S.tile[c & 1];
        const float d1 = O.d1[j], d2 = O.d2[j], dec = O.dec[j];
        {
            f32x4 Sc[4];
            if (c & 1) {
                // state entering the odd chunk: one update of the saved state with the chunk below
                const SlotG& Q = S.slot[(c - 1) % 3];
                const float qdec = Q.dec[j], qd2 = Q.d2[j];
                const bf16x8 kh = tr_pair(&Q.KpH[8 * g][8 * w], OS, l16), kl = tr_pair(&Q.KpL[8 * g][8 * w], OS, l16);
#pragma unroll
                for (int tl = 0; tl < 4; ++tl) {
                    const bf16x8 vop = tr_pair(&Q.V[8 * g][8 * tl], OS, l16);
                    f32x4 U = mfma(vop, kh, zero4);
                    U = mfma(vop, kl, U);
#pragma unroll
                    for (int v = 0; v < 4; ++v) Sc[tl][v] = fmaf(Sa[tl][v], qdec, qd2 * U[v]);
                }
            } else {
#pragma unroll
                for (int tl = 0; tl < 4; ++tl) Sc[tl] = Sa[tl];
            }
            // -------------------------------------------------------- X^T[j][t] = (S d1)^T GY^T + K'^T Bm^T
            bf16x8 sh[2], sl[2];
            split16(Sc, d1, sh, sl);
            f32x4 X[2] = {zero4, zero4};
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const bf16x8 gop = acc_order_op(&O.GY[16 * tt + l16][0], ks, g);
                    X[tt] = mfma(sh[ks], gop, X[tt]);
                    X[tt] = mfma(sl[ks], gop, X[tt]);
                }
            const bf16x8 kh = tr_pair(&O.KpH[8 * g][8 * w], OS, l16), kl = tr_pair(&O.KpL[8 * g][8 * w], OS, l16);
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const bf16x8 bh_ = lds_op(&Tl.BH[16 * tt + l16][4 * g]), bl_ = lds_op(&Tl.BL[16 * tt + l16][4 * g]);
                X[tt] = mfma(kh, bh_, X[tt]);
                X[tt] = mfma(kh, bl_, X[tt]);
                X[tt] = mfma(kl, bh_, X[tt]);
                *reinterpret_cast<float4*>(&S.xz[c & 1][0][16 * tt + l16][16 * w + 4 * g]) = make_float4(X[tt][0], X[tt][1], X[tt][2], X[tt][3]);
            }
        }
        // ------------------------------------------------------------ Z^T[j][s] = (dS d2)^T V^T + R'^T Bm
        bf16x8 dh[2], dl[2];
        split16(D, d2, dh, dl);
        f32x4 Z[2] = {zero4, zero4};
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const bf16x8 vop = acc_order_op(&O.V[16 * tt + l16][0], ks, g);
                Z[tt] = mfma(dh[ks], vop, Z[tt]);
                Z[tt] = mfma(dl[ks], vop, Z[tt]);
            }
        const bf16x8 rh = tr_pair(&O.RpH[8 * g][8 * w], OS, l16), rl = tr_pair(&O.RpL[8 * g][8 * w], OS, l16);
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            const bf16x8 bh_ = tr_pair(&Tl.BH[8 * g][8 * tt], AS, l16), bl_ = tr_pair(&Tl.BL[8 * g][8 * tt], AS, l16);
            Z[tt] = mfma(rh, bh_, Z[tt]);
            Z[tt] = mfma(rh, bl_, Z[tt]);
            Z[tt] = mfma(rl, bh_, Z[tt]);
            *reinterpret_cast<float4*>(&S.xz[c & 1][1][16 * tt + l16][16 * w + 4 * g]) = make_float4(Z[tt][0], Z[tt][1], Z[tt][2], Z[tt][3]);
        }
        // ------------------------------------------------------------ dS <- dS dec + d1 GY^T R'
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            const bf16x8 gop = tr_pair(&O.GY[8 * g][8 * tl], OS, l16);
            f32x4 U = mfma(gop, rh, zero4);
            U = mfma(gop, rl, U);
#pragma unroll
            for (int v = 0; v < 4; ++v) D[tl][v] = fmaf(D[tl][v], dec, d1 * U[v]);
        }
        if (!(c & 1)) {
            // anchor: P = sum_i dS S with the saved state entering this chunk
            float p = 0.f;
#pragma unroll
            for (int tl = 0; tl < 4; ++tl)
#pragma unroll
                for (int v = 0; v < 4; ++v) p = fmaf(D[tl][v], Sa[tl][v], p);
            p = allreduce_rows(p);
            if (g == 0) S.pex[(c >> 1) & 1][j] = p;
        }
    };
    // a segment = an even chunk and the odd chunk above it, taken in reverse; one barrier per chunk
    auto segment = [&](const int sg, const f32x4 (&Sa)[4]) __attribute__((always_inline)) {
        if (2 * sg + 1 < n) { chunk(2 * sg + 1, Sa); __syncthreads(); }
        chunk(2 * sg, Sa);
        __syncthreads();
    };
    // The saved states alternate between two register sets with fixed roles, each refilled as soon as its segment is
    // done, two chunks before it is read again: no value that is still in flight is ever copied.
    f32x4 SA[4], SB[4];
    const int top = nseg - 1;
    // (every refill is issued on every path, with the segment index clamped, so that the waits can count them)
    load_state(sv + static_cast<size_t>(top) * (N * N), SA, g);
    load_state(sv + static_cast<size_t>(top >= 1 ? top - 1 : 0) * (N * N), SB, g);
    __syncthreads();                       // iterations 0 and 1: nothing prepared yet
    __syncthreads();
    for (int sg = top; sg >= 0; sg -= 2) {
        segment(sg, SA);
        load_state(sv + static_cast<size_t>(sg >= 2 ? sg - 2 : 0) * (N * N), SA, g);
        if (sg >= 1) segment(sg - 1, SB);
        load_state(sv + static_cast<size_t>(sg >= 3 ? sg - 3 : 0) * (N * N), SB, g);
    }
    __syncthreads();                       // iteration n + 2: the P waves finish chunk 0
    if (a.gs != nullptr) {
#pragma unroll
        for (int tl = 0; tl < 4; ++tl)
#pragma unroll
            for (int v = 0; v < 4; ++v) a.gs[(bh * N + 16 * tl + 4 * g + v) * N + j] = f2bf(D[tl][v]);
    }
}

// ---------------------------------------------------------------------------------------------------- EW waves
template <int WMODE>
DEVINL void role_e(SmemG& S, const ArgsG& a, const int lane, const int w, const size_t base, const int n) {
    const int g = lane >> 4, l16 = lane & 15;
    const int T = a.T, C = a.C;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 E[4] = {zero4, zero4, zero4, zero4};     // dS[i = 16w + l16][j = 16 tile + 4g + v]

    // causal tiles of chunk c (waves 0, 1, 2 -> quadrants (t, s) = (0,0) (1,0) (1,1)); accumulator rows are s, lanes t
    auto tiles = [&](const int c) __attribute__((always_inline)) {
        const SlotG& O = S.slot[c % 3];
        TilesG& Tl = S.tile[c & 1];
        const int ta = (w == 0) ? 0 : 1, tb = (w == 2) ? 1 : 0;
        f32x4 a0 = zero4, a1 = zero4, bm = zero4;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bf16x8 kh = lds_op(&O.KpH[16 * tb + l16][16 * ks + 4 * g]), kl = lds_op(&O.KpL[16 * tb + l16][16 * ks + 4 * g]);
            const bf16x8 rh = lds_op(&O.RpH[16 * ta + l16][16 * ks + 4 * g]), rl = lds_op(&O.RpL[16 * ta + l16][16 * ks + 4 * g]);
            const bf16x8 vo = lds_op(&O.V[16 * tb + l16][16 * ks + 4 * g]), go = lds_op(&O.GY[16 * ta + l16][16 * ks + 4 * g]);
            a0 = mfma(kh, rh, a0);
            a1 = mfma(kh, rl, a1);
            a1 = mfma(kl, rh, a1);
            bm = mfma(vo, go, bm);
        }
        f32x4 am = a0 + a1;                                    // [v]: s = 16 tb + 4g + v, t = 16 ta + l16
        if (ta == tb) {
            const int t = 16 * ta + l16;
            const float d = (O.ruk[0][t] + O.ruk[1][t]) + (O.ruk[2][t] + O.ruk[3][t]);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int sl = 4 * g + v;
                if (sl == l16) S.vg[c & 3][t] = bm[v];
                am[v] = (sl < l16) ? am[v] : (sl == l16 ? d : 0.f);
                bm[v] = (sl < l16) ? bm[v] : 0.f;
            }
        }
        const HL x0 = hilo2(am[0], am[1]), x1 = hilo2(am[2], am[3]), y0 = hilo2(bm[0], bm[1]), y1 = hilo2(bm[2], bm[3]);
        *reinterpret_cast<uint2*>(&Tl.AH[16 * ta + l16][8 * tb + 2 * g]) = make_uint2(x0.h, x1.h);
        *reinterpret_cast<uint2*>(&Tl.AL[16 * ta + l16][8 * tb + 2 * g]) = make_uint2(x0.l, x1.l);
        *reinterpret_cast<uint2*>(&Tl.BH[16 * ta + l16][8 * tb + 2 * g]) = make_uint2(y0.h, y1.h);
        *reinterpret_cast<uint2*>(&Tl.BL[16 * ta + l16][8 * tb + 2 * g]) = make_uint2(y0.l, y1.l);
    };

    for (int it = 0; it <= n + 2; ++it) {
        const int c = n + 1 - it;
        if (it >= 2 && c >= 0) {
            const SlotG& O = S.slot[c % 3];
            const TilesG& Tl = S.tile[c & 1];
            // ------------------------------------------------------------ gv^T[i][s] = (dS d2) K'^T + GY^T A
            bf16x8 dh[2], dl[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const float4 p = *reinterpret_cast<const float4*>(&O.d2[32 * ks + 4 * g]);
                const float4 q = *reinterpret_cast<const float4*>(&O.d2[32 * ks + 16 + 4 * g]);
                const HL x0 = hilo2(E[2 * ks][0] * p.x, E[2 * ks][1] * p.y), x1 = hilo2(E[2 * ks][2] * p.z, E[2 * ks][3] * p.w);
                const HL x2 = hilo2(E[2 * ks + 1][0] * q.x, E[2 * ks + 1][1] * q.y), x3 = hilo2(E[2 * ks + 1][2] * q.z, E[2 * ks + 1][3] * q.w);
                dh[ks] = as_op(x0.h, x1.h, x2.h, x3.h);
                dl[ks] = as_op(x0.l, x1.l, x2.l, x3.l);
            }
            f32x4 G[2] = {zero4, zero4};
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const bf16x8 kh = acc_order_op(&O.KpH[16 * tt + l16][0], ks, g), kl = acc_order_op(&O.KpL[16 * tt + l16][0], ks, g);
                    G[tt] = mfma(dh[ks], kh, G[tt]);
                    G[tt] = mfma(dh[ks], kl, G[tt]);
                    G[tt] = mfma(dl[ks], kh, G[tt]);
                }
            const bf16x8 gyo = tr_pair(&O.GY[8 * g][8 * w], OS, l16);       // lane = value channel 16w + l16, K = tokens
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const bf16x8 ah = tr_pair(&Tl.AH[8 * g][8 * tt], AS, l16), al = tr_pair(&Tl.AL[8 * g][8 * tt], AS, l16);
                G[tt] = mfma(gyo, ah, G[tt]);
                G[tt] = mfma(gyo, al, G[tt]);
                const int tg = c * L + 16 * tt + l16;
                if (tg < T)
                    *reinterpret_cast<uint2*>(a.gv + base + static_cast<size_t>(tg) * C + 16 * w + 4 * g) =
                        make_uint2(pack_bf2(G[tt][0], G[tt][1]), pack_bf2(G[tt][2], G[tt][3]));
            }
            // ------------------------------------------------------------ dS^T <- dS^T dec + d1 R'^T GY
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                const bf16x8 rh = tr_pair(&O.RpH[8 * g][8 * tl], OS, l16), rl = tr_pair(&O.RpL[8 * g][8 * tl], OS, l16);
                f32x4 U = mfma(rh, gyo, zero4);
                U = mfma(rl, gyo, U);
                const float4 de = *reinterpret_cast<const float4*>(&O.dec[16 * tl + 4 * g]);
                const float4 d1 = *reinterpret_cast<const float4*>(&O.d1[16 * tl + 4 * g]);
                E[tl][0] = fmaf(E[tl][0], de.x, d1.x * U[0]); E[tl][1] = fmaf(E[tl][1], de.y, d1.y * U[1]);
                E[tl][2] = fmaf(E[tl][2], de.z, d1.z * U[2]); E[tl][3] = fmaf(E[tl][3], de.w, d1.w * U[3]);
            }
        }
        if (it >= 1 && c - 1 >= 0 && w < 3) tiles(c - 1);
        __syncthreads();
    }
}

template <int WMODE>
__global__ __launch_bounds__(NTG) void wkv6_bwd_fused(const ArgsG a) {
    __shared__ SmemG S;
    const int tid = threadIdx.x;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const size_t base = static_cast<size_t>(b) * a.T * a.C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const int n = (a.T + L - 1) / L;
    // the quadrant t < 16 <= s of the tiles is never written and must read as zero
    for (int i = tid; i < static_cast<int>(sizeof(S.tile) / 4); i += NTG) reinterpret_cast<uint32_t*>(&S.tile[0])[i] = 0;
    __syncthreads();
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, w = wid & 3;
    if (wid < 4) role_prep<WMODE>(S, a, lane, w, base, h, bh, n);
    else if (wid < 8) role_sd<WMODE>(S, a, lane, w, bh, n);
    else role_e<WMODE>(S, a, lane, w, base, n);
}

}  // namespace

int launch_wkv6_bwd_fused(hipStream_t st, int B, int T, int C, int H, const uint16_t* r, const uint16_t* k, const uint16_t* v,
                          const uint16_t* w, const uint16_t* u, const uint16_t* gy, uint16_t* gr, uint16_t* gk, uint16_t* gv,
                          uint16_t* gw, uint16_t* gu, uint16_t* gs, const float* saved, int* flags) {
    ArgsG a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.gy = gy;
    a.gr = gr; a.gk = gk; a.gv = gv; a.gw = gw; a.gu = gu; a.gs = gs; a.saved = saved; a.flags = flags;
    hipLaunchKernelGGL(wkv6_bwd_fused<W_RAW>, dim3(B * H), dim3(NTG), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
