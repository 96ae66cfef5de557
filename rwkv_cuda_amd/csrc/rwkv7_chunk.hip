// RWKV-7 "clamp-w" generalised delta rule in CHUNKED form on the matrix cores (gfx950, v_mfma_f32_16x16x4_f32).
//
// Step form (rwkv7_fast_fused/cuda/rwkv7_statepassing_clampw.cu:20-187), one head, S[i][j] (i value, j key):
//     sa_t = S_t a_t;   S_{t+1} = S_t diag(w_t) + sa_t b_t^T + v_t k_t^T;   y_t = S_{t+1} r_t;   w_t = exp(W_SCALE sigmoid(w_raw_t))
// A chunk of L = 16 steps (the reference's CHUNK_LEN), local t = 0..15, S0 the state entering it.  With lam_t = log w_t,
// c_t = sum_{z<t} lam_z and the chunk's middle m = 8 as the reference point (the clamp bounds |c_t - c_m| by 0.607 * 8, so
// no factor exceeds e^4.9 and nothing needs a fallback):
//     A'_t = a_t e^{c_t - c_m}    R'_t = r_t e^{c_{t+1} - c_m}    B'_s = b_s e^{c_m - c_{s+1}}    K'_s = k_s e^{c_m - c_{s+1}}
//     d1 = e^{c_m}   d2 = e^{c_L - c_m}   dec = e^{c_L}
//     AB = tril_-(A' B'^T)  AK = tril_-(A' K'^T)  RB = tril(R' B'^T)  RK = tril(R' K'^T)                 [16 x 16]
//     U  = (I - AB)^{-1} ((A' d1) S0^T + AK V)         rows of U are sa_t (the tensor `sa` of the interface)
//     Y  = (R' d1) S0^T + RB U + RK V
//     S_L = S0 diag(dec) + U^T (B' d2) + V^T (K' d2)
// (the state update takes B' d2 = b e^{c_L - c_{s+1}} and K' d2 from one exponential each: a factor's relative error is the
// absolute error of its exponent, and referred to the chunk's end the newest, largest contributions have the smallest
// exponents; through the middle every term would carry two factors of e^{+-4.9} -- 3e-7 on the fp32 state instead of 5e-8.)
// Backward of a chunk from dY and dS_L (the gradient w.r.t. S_L through everything after the chunk):
//     dU  = RB^T dY + (B' d2) dS_L^T          dW = (I - AB)^{-T} dU
//     dAB = tril_-(dW U^T)  dAK = tril_-(dW V^T)  dRB = tril(dY U^T)  dRK = tril(dY V^T)
//     dV  = AK^T dW + RK^T dY + (K' d2) dS_L^T
//     dS0 = dS_L diag(dec) + d1 (dY^T R' + dW^T A')
//     dA' = dAB B' + dAK K' + d1 (dW S0)      dR' = dRB B' + dRK K' + d1 (dY S0)
//     dB' = dAB^T A' + dRB^T R' + d2 (U dS_L)  dK' = dAK^T A' + dRK^T R' + d2 (V dS_L)
//     da = dA' e^{c_t - c_m}, dr = dR' e^{c_{t+1} - c_m}, db = dB' e^{c_m - c_{t+1}}, dk likewise
//     decay: with P_t = sum_i dS_t o S_t per key channel,  G_t = P_{t+1} + r dr - b db - k dk,  P_t = G_t + a da,
//            dw_raw = G W_SCALE sig (1 - sig);  P at the end of the call = sum_i dsT o S_T.
// Every product is an fp32 matrix instruction (no operand is rounded below fp32), so the fp32 outputs sT, ds0 and the
// saved sa keep the accuracy class of the reference's fp32 recurrence; the bf16 outputs are rounded once at the store.
//
// One workgroup of four waves per (batch, head).  A 16x16x4 fp32 matrix instruction takes A[row = lane & 15][k = lane >> 4],
// B[k = lane >> 4][col = lane & 15] and leaves D[row = 4 (lane >> 4) + v][col = lane & 15] in register v.  The state is
// kept TRANSPOSED in accumulator registers, S^T tile jt of wave q: register v of lane (l16, g) = S[i = 16 q + l16][j = 16 jt + 4 g + v].
// K slots may be assigned to channels (or tokens) in any order as long as both operands agree, so with slot g <-> channel
// 16 jt + 4 g + v in step (jt, v) an accumulator register IS the B operand of that step, and an accumulator tile whose rows
// are tokens (U, W, dU, dW) is the B operand of a contraction over tokens with slot g <-> token 4 g + v.  Nothing is ever
// transposed through LDS except the gradient state for the two products that contract over the value channel.
//
// Private layout of the interface's scratch tensors: `s` slot c holds the state ENTERING chunk c as [i][j] fp32 (the
// reference stores the state leaving it; the backward here needs the entering one and never inverts a step), `sa` is U.
#include "common.h"

namespace rwkv {
namespace {

constexpr int N = 64;
constexpr int CL = RWKV7_CHUNK_LEN;
constexpr int NT = 256;
constexpr int PS = 68;            // row stride (floats) of a [token][channel] plane
constexpr int TS = 20;            // row stride (floats) of a 16 x 16 tile
constexpr float W_SCALE = -0.6065306597f;   // -exp(-0.5), rwkv7_statepassing_clampw.cu:16

typedef float f32x4 __attribute__((ext_vector_type(4)));
DEVINL f32x4 mm(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
DEVINL f32x4 ld4(const float* p) { const float4 x = *reinterpret_cast<const float4*>(p); return f32x4{x.x, x.y, x.z, x.w}; }
DEVINL void st4(float* p, const f32x4& x) { *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]); }
constexpr f32x4 ZERO4 = {0.f, 0.f, 0.f, 0.f};

struct Args7c {
    int T, H;
    const uint16_t *r, *w, *k, *v, *a, *b, *dy;
    const float *s0, *dsT;
    uint16_t *y, *dr, *dw, *dk, *dv, *da, *db;
    float *sT, *ds0;
    float* s;     // [B,H,T/16][i][j]: state entering each chunk
    float* sa;    // [B,T,H,N]: U
};

// the value a lane group g takes from four candidates (register index that depends on the lane group)
DEVINL float by_group(int g, float x0, float x1, float x2, float x3) { return g == 0 ? x0 : (g == 1 ? x1 : (g == 2 ? x2 : x3)); }

// Rows of M = (I - AB)^{-1}: lane (l16 = r) gets m[s] = M[r][s] from the column recurrence M[r][s] = [r == s] + sum_{t>s} M[r][t] AB[t][s].
// ABt[s][t] = AB[t][s] is read with wave-uniform addresses (LDS broadcast).
DEVINL void inverse_rows(const float (*ABt)[TS], int r, float (&m)[CL]) {
    m[CL - 1] = r == CL - 1 ? 1.f : 0.f;
#pragma unroll
    for (int s = CL - 2; s >= 0; --s) {
        float acc = r == s ? 1.f : 0.f;
#pragma unroll
        for (int t4 = (s + 1) / 4 * 4; t4 < CL; t4 += 4) {
            const f32x4 x = ld4(&ABt[s][t4]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (t4 + e > s) acc = fmaf(m[t4 + e], x[e], acc);
        }
        m[s] = acc;
    }
}
// Columns of the same M: lane (l16 = c) gets m[t] = M[t][c] from the row recurrence M[t][c] = [t == c] + sum_{s<t} AB[t][s] M[s][c].
DEVINL void inverse_cols(const float (*AB)[TS], int c, float (&m)[CL]) {
    m[0] = c == 0 ? 1.f : 0.f;
#pragma unroll
    for (int t = 1; t < CL; ++t) {
        float acc = c == t ? 1.f : 0.f;
#pragma unroll
        for (int s4 = 0; s4 < t; s4 += 4) {
            const f32x4 x = ld4(&AB[t][s4]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (s4 + e < t) acc = fmaf(x[e], m[s4 + e], acc);
        }
        m[t] = acc;
    }
}

// e^x to fp32 accuracy for |x| of a few units: the hardware exponential takes x log2(e), whose rounding alone costs |x| 6e-8;
// the product is carried as a rounded part plus its error, and the error enters to first order.
DEVINL float exp_acc(float x) {
    constexpr float L2E_HI = 1.44269502162933349609f, L2E_LO = 1.92596299112661746e-8f, LN2 = 0.69314718055994530942f;
    const float t = x * L2E_HI;
    const float e = fmaf(x, L2E_HI, -t) + x * L2E_LO;
    const float y = __builtin_amdgcn_exp2f(t);
    return fmaf(y, e * LN2, y);
}

// In-chunk factors of the four tokens (4 q + e) of channel j held by a thread, from lam and the per-wave sums in part[][].
// Every exponent is formed as a direct sum of the lam between the token and its reference point (never as a difference of
// two long cumulative sums), so its absolute error -- the factor's relative error -- scales with the exponent itself.
struct Factors { float ea[4], er[4], eb[4], es[4], ee[4]; };   // e^{c_t - c_m}, e^{c_{t+1} - c_m}, e^{c_m - c_{t+1}}, e^{c_t}, e^{c_L - c_{t+1}}
template <int E0 = 0, int E1 = 4>
DEVINL Factors chunk_factors(const float (&lam)[4], const float (*part)[N], int q, int j, float& cm_out, float& cl_out) {
    const float p0 = part[0][j], p1 = part[1][j], p2 = part[2][j], p3 = part[3][j];
    const float cm = p0 + p1, cl = (p0 + p1) + (p2 + p3);
    const float before = q == 0 ? 0.f : (q == 1 ? p0 : (q == 2 ? cm : cm + p2));        // c_t of the wave's first token
    const float after = q == 3 ? 0.f : (q == 2 ? p3 : (q == 1 ? p2 + p3 : p1 + (p2 + p3)));   // c_L - c of the token after the wave's last
    // lam between the wave's tokens and the middle: first half, the tokens after the wave up to the middle; second half, those from the middle up to the wave
    const float gap = q == 0 ? p1 : (q == 3 ? p2 : 0.f);
    float pre[5], suf[5];                      // pre[e] = sum of lam[0..e-1], suf[e] = sum of lam[e..3]
    pre[0] = 0.f; suf[4] = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) pre[e + 1] = pre[e] + lam[e];
#pragma unroll
    for (int e = 3; e >= 0; --e) suf[e] = suf[e + 1] + lam[e];
    Factors f = {};
#pragma unroll
    for (int e = E0; e < E1; ++e) {                // (the exponentials of the tokens asked for; the sums above are cheap)
        // c_t - c_m and c_{t+1} - c_m
        const float xt = q < 2 ? -(suf[e] + gap) : gap + pre[e];
        const float xn = q < 2 ? -(suf[e + 1] + gap) : gap + pre[e + 1];
        // the middle-referenced factors always come in pairs whose exponents cancel only partly, so the extra digits of
        // exp_acc would be lost anyway; the start- and end-referenced ones carry the fp32 states and keep them
        f.ea[e] = __expf(xt);
        f.er[e] = __expf(xn);
        f.eb[e] = __expf(-xn);
        f.es[e] = exp_acc(before + pre[e]);
        f.ee[e] = exp_acc(suf[e + 1] + after);
    }
    cm_out = cm; cl_out = cl;
    return f;
}

DEVINL float sigmoid_fast(float x) { return __frcp_rn(1.f + __expf(-x)); }

// ---------------------------------------------------------------------------------------------------- forward
struct SmemCF {
    float Ap[CL][PS], Rp[CL][PS], Bp[CL][PS], Kp[CL][PS], V[CL][PS];
    float Be[CL][PS], Ke[CL][PS];      // b, k carried to the end of the chunk: e^{c_L - c_{s+1}}
    float As[CL][PS];                  // a referred to the start of the chunk: e^{c_t}
    float Yo[CL][PS], Uo[CL][PS];
    float ABt[CL][TS], AK[CL][TS], RB[CL][TS], RK[CL][TS];
    float M[CL][TS];                   // (I - AB)^{-1}, rows by the wave that made AB
    float part[4][N];
    float d1[N], dec[N];
};

__global__ __launch_bounds__(NT, 2) void rwkv7c_fwd(const Args7c p) {
    __shared__ SmemCF S;
    const int tid = threadIdx.x, lane = tid & 63, q = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, g = lane >> 4;
    const int h = blockIdx.x, b = blockIdx.y, H = p.H, T = p.T;
    const int nch = T / CL;
    const size_t bh = static_cast<size_t>(b) * H + h;
    const size_t tok0 = static_cast<size_t>(b) * T;                       // first token row of this batch
    const int i_own = 16 * q + l16;

    // state, transposed tiles: St[jt][v] = S[i_own][16 jt + 4 g + v]
    f32x4 St[4];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
        St[jt] = p.s0 != nullptr ? ld4(p.s0 + bh * N * N + static_cast<size_t>(i_own) * N + 16 * jt + 4 * g) : ZERO4;

    // prep role: channel j = lane, tokens 4 q + e
    uint32_t nx[6][4];
    auto fetch = [&](int c) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const size_t o = ((tok0 + static_cast<size_t>(c) * CL + 4 * q + e) * H + h) * N + lane;
            nx[0][e] = p.w[o]; nx[1][e] = p.r[o]; nx[2][e] = p.k[o]; nx[3][e] = p.v[o]; nx[4][e] = p.a[o]; nx[5][e] = p.b[o];
        }
    };
    fetch(0);

    for (int c = 0; c < nch; ++c) {
        // ---------------------------------------------------------------- prep: decay sums, scaled operand planes
        float lam[4], rr[4], kk[4], vv[4], aa[4], bb[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lam[e] = W_SCALE * sigmoid_fast(bf2f(nx[0][e]));
            rr[e] = bf2f(nx[1][e]); kk[e] = bf2f(nx[2][e]); vv[e] = bf2f(nx[3][e]); aa[e] = bf2f(nx[4][e]); bb[e] = bf2f(nx[5][e]);
        }
        S.part[q][lane] = (lam[0] + lam[1]) + (lam[2] + lam[3]);
        if (c + 1 < nch) fetch(c + 1);
        __syncthreads();
        float cm, cl;
        const Factors f = chunk_factors(lam, S.part, q, lane, cm, cl);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int t = 4 * q + e;
            S.Ap[t][lane] = aa[e] * f.ea[e];
            S.Rp[t][lane] = rr[e] * f.er[e];
            S.Bp[t][lane] = bb[e] * f.eb[e];
            S.Kp[t][lane] = kk[e] * f.eb[e];
            S.As[t][lane] = aa[e] * f.es[e];
            S.Be[t][lane] = bb[e] * f.ee[e];
            S.Ke[t][lane] = kk[e] * f.ee[e];
            S.V[t][lane] = vv[e];
        }
        if (q == 0) { S.d1[lane] = exp_acc(cm); S.dec[lane] = exp_acc(cl); }
        // the state entering the chunk, for the backward
        {
            float* slot = p.s + (bh * nch + c) * N * N + static_cast<size_t>(i_own) * N + 4 * g;
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) st4(slot + 16 * jt, St[jt]);
        }
        __syncthreads();
        // ---------------------------------------------------------------- one causal tile per wave
        {
            const float (*X)[PS] = q < 2 ? S.Ap : S.Rp;
            const float (*Y)[PS] = (q & 1) ? S.Kp : S.Bp;
            f32x4 acc = ZERO4;
#pragma unroll
            for (int jb = 0; jb < 4; ++jb) {
                const f32x4 xa = ld4(&X[l16][16 * jb + 4 * g]), yb = ld4(&Y[l16][16 * jb + 4 * g]);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc = mm(xa[v], yb[v], acc);
            }
            // acc[v] = tile[t = 4 g + v][s = l16]
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int t = 4 * g + v;
                acc[v] = (q < 2 ? l16 < t : l16 <= t) ? acc[v] : 0.f;
            }
            if (q == 0) {
                st4(&S.ABt[l16][4 * g], acc);
                // this wave wrote AB itself (LDS keeps a wave's accesses in order): the inverse once, for all four waves
                float m[CL];
                inverse_rows(S.ABt, l16, m);
                if (g == 0)
#pragma unroll
                    for (int s4 = 0; s4 < CL; s4 += 4) st4(&S.M[l16][s4], f32x4{m[s4], m[s4 + 1], m[s4 + 2], m[s4 + 3]});
            } else {
                float (*Tl)[TS] = q == 1 ? S.AK : (q == 2 ? S.RB : S.RK);
#pragma unroll
                for (int v = 0; v < 4; ++v) Tl[4 * g + v][l16] = acc[v];
            }
        }
        __syncthreads();
        // ---------------------------------------------------------------- W = (a e^{c_t}) S0^T + AK V, value channels of this wave
        f32x4 vop;                                   // V[s = 4 g + v][i_own]
#pragma unroll
        for (int v = 0; v < 4; ++v) vop[v] = S.V[4 * g + v][i_own];
        f32x4 W = ZERO4;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            const f32x4 xa = ld4(&S.As[l16][16 * jt + 4 * g]);
#pragma unroll
            for (int v = 0; v < 4; ++v) W = mm(xa[v], St[jt][v], W);
        }
        {
            const f32x4 ak = ld4(&S.AK[l16][4 * g]);
#pragma unroll
            for (int v = 0; v < 4; ++v) W = mm(ak[v], vop[v], W);
        }
        // ---------------------------------------------------------------- U = (I - AB)^{-1} W
        f32x4 U = ZERO4;
        {
            const f32x4 mr = ld4(&S.M[l16][4 * g]);   // M[t = l16][s = 4 g + v]
#pragma unroll
            for (int v = 0; v < 4; ++v) U = mm(mr[v], W[v], U);
        }
        // ---------------------------------------------------------------- Y = R' (d1 S0^T) + RB U + RK V
        f32x4 Sd[4];
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) Sd[jt] = St[jt] * ld4(&S.d1[16 * jt + 4 * g]);
        f32x4 Y = ZERO4;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            const f32x4 xa = ld4(&S.Rp[l16][16 * jt + 4 * g]);
#pragma unroll
            for (int v = 0; v < 4; ++v) Y = mm(xa[v], Sd[jt][v], Y);
        }
        {
            const f32x4 rb = ld4(&S.RB[l16][4 * g]), rk = ld4(&S.RK[l16][4 * g]);
#pragma unroll
            for (int v = 0; v < 4; ++v) Y = mm(rb[v], U[v], Y);
#pragma unroll
            for (int v = 0; v < 4; ++v) Y = mm(rk[v], vop[v], Y);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) { S.Yo[4 * g + v][i_own] = Y[v]; S.Uo[4 * g + v][i_own] = U[v]; }
        // ---------------------------------------------------------------- S^T = diag(dec) S^T + (B' d2)^T U + (K' d2)^T V
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            f32x4 acc = ZERO4;
#pragma unroll
            for (int v = 0; v < 4; ++v) acc = mm(S.Be[4 * g + v][16 * jt + l16], U[v], acc);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc = mm(S.Ke[4 * g + v][16 * jt + l16], vop[v], acc);
            St[jt] = St[jt] * ld4(&S.dec[16 * jt + 4 * g]) + acc;
        }
        __syncthreads();
        // ---------------------------------------------------------------- y (bf16) and sa = U (fp32) as whole rows
        {
            const int t = tid >> 4, i4 = (tid & 15) * 4;
            const size_t o = ((tok0 + static_cast<size_t>(c) * CL + t) * H + h) * N + i4;
            const f32x4 y = ld4(&S.Yo[t][i4]);
            *reinterpret_cast<uint2*>(p.y + o) = make_uint2(pack_bf2(y[0], y[1]), pack_bf2(y[2], y[3]));
            st4(p.sa + o, ld4(&S.Uo[t][i4]));
        }
    }
    if (p.sT != nullptr) {
        float* dst = p.sT + bh * N * N + static_cast<size_t>(i_own) * N + 4 * g;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) st4(dst + 16 * jt, St[jt]);
    }
}

// ---------------------------------------------------------------------------------------------------- backward
// One workgroup of twelve waves per (batch, head), three roles with their own loops; wave w: q = w & 3.
//   waves 0..3 ("A", value-channel tile q): dSa[jt][v] = dS[i = 16 q + l16][j = 16 jt + 4 g + v]   (rows j, columns i): the B operand
//                of the contractions over the key channel, (B' d2) dS^T and (K' d2) dS^T; they make the causal tiles, dU, the
//                triangular solve, dW, dV and ds0.
//   waves 4..7 ("B", key-channel tile q):   dSb[ib][v] = dS[i = 16 ib + 4 g + v][j = 16 q + l16]   (rows i, columns j): the B operand
//                of the contractions over the value channel, U dS and V dS, next to S0 of the chunk loaded from `s` in the same
//                layout (dW S0, dY S0); they make dA', dR', dB', dK' (register v <-> token 4 g + v, lane <-> key channel), scale
//                them, scan the decay gradient and park the results; they run one phase behind the A waves.
//   waves 8..11 ("P"): fetch the seven input rows and `sa` two chunks ahead, convert them and build the operand planes
//                (double-buffered).  The finished gradient rows leave LDS-staged, as whole rows, through A waves 2 and 3.
// The gradient state is therefore kept twice (both copies get the same update); nothing is transposed through LDS.
constexpr int NTB = 12 * 64;       // waves 0..3 role A, 4..7 role B, 8..11 role P

// Everything that is a function of one chunk's inputs alone; two copies: the P waves fill one while the A and B waves work on the other.
struct PlanesB {
    float Ap[CL][PS], Rp[CL][PS], Bp[CL][PS], Kp[CL][PS];   // referred to the middle of the chunk (tiles, dA' .. dK')
    float As[CL][PS], Rs[CL][PS];                            // a e^{c_t}, r e^{c_{t+1}}: the state-gradient update
    float Bd[CL][PS], Kd[CL][PS];                            // b, k times e^{c_L - c_{s+1}}: dU, dV, S_T
    float V[CL][PS], dY[CL][PS], U[CL][PS];
    float EA[CL][PS], ER[CL][PS], DWF[CL][PS];               // e^{c_t - c_m}, e^{c_{t+1} - c_m}, W_SCALE sig (1 - sig)
    float part[4][N];
    float d1[N], d2[N], dec[N];
};
constexpr int PK = 72;            // row stride (bf16 elements) of a parked output
struct SmemCB {
    PlanesB pl[2];
    float dW[CL][PS];
    float M[CL][TS];                                         // (I - AB)^{-1}
    float AB[CL][TS], AK[CL][TS], RB[CL][TS], RK[CL][TS];
    float dAB[CL][TS], dAK[CL][TS], dRB[CL][TS], dRK[CL][TS];
    uint16_t park[5][CL][PK];                                // da, dr, db, dk, dw of the chunk whose phase 4 ran last, [token][channel]
    uint16_t parkv[2][CL][PK];                               // dv, which is ready one visit earlier than the other five
};

// tile[t][s] = sum_c X[t][c] Y[s][c] over 64 channels, masked to s < t (strict) or s <= t, stored as [t][s]
DEVINL void causal_tile(const float (*X)[PS], const float (*Y)[PS], float (*Tl)[TS], bool strict, int l16, int g) {
    f32x4 part[2] = {ZERO4, ZERO4};               // two independent chains
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
        const f32x4 xa = ld4(&X[l16][16 * cb + 4 * g]), yb = ld4(&Y[l16][16 * cb + 4 * g]);
#pragma unroll
        for (int v = 0; v < 4; ++v) part[cb & 1] = mm(xa[v], yb[v], part[cb & 1]);
    }
    const f32x4 acc = part[0] + part[1];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int t = 4 * g + v;
        Tl[t][l16] = (strict ? l16 < t : l16 <= t) ? acc[v] : 0.f;
    }
}

// Per visit i (chunks in descending order) every wave passes three barriers; role B trails role A by one phase, so that
// both always have matrix work in the same phase:
//          phase 1                          | phase 2                                   | phase 3
//   A:     tile, M, tile-free parts of (i)   | dU, dW, dV, state update of (i)           | dAB, dAK of (i)
//   B:     tile parts + epilogue of (i - 1)  | dY S0, U dS, V dS, dRB, dRK of (i)        | dW S0, state update of (i)
//   P:     raw inputs -> decay sums (i + 1)  | factors, planes (i + 1)                   | -
// (the rows of visit i - 1 leave in phase 3, through the two A waves that have no tile there)

// ---- role P: elementwise preparation (lane = channel, tokens 4 wp + e) one visit ahead, and the row-wise output stores
struct Prep7 { uint32_t nx[7][4]; float nsa[4]; };
struct Conv7 { float sg[4], uu[4]; uint32_t pk[6][2]; };      // sigmoid(w), sa, and r k v a b dy as bf16 pairs (tokens 2 z, 2 z + 1)
DEVINL void bwd_fetch(const Args7c& p, Prep7& x, size_t row0, int wp, int lane, int H, int h) {
    // wave-uniform base (scalar registers) plus a 32-bit lane offset: no 64-bit address per tensor and token in vector registers
    // (the lane part is hidden from the optimiser: it would otherwise turn every tensor-and-token address into a 64-bit
    // induction variable of the chunk loop, 64 vector registers)
    const size_t base = (row0 * H + h) * N;
    uint32_t lo = lane;
    asm volatile("" : "+v"(lo));
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t o = static_cast<uint32_t>((4 * wp + e) * H) * N + lo;
        x.nx[0][e] = (p.w + base)[o]; x.nx[1][e] = (p.r + base)[o]; x.nx[2][e] = (p.k + base)[o]; x.nx[3][e] = (p.v + base)[o];
        x.nx[4][e] = (p.a + base)[o]; x.nx[5][e] = (p.b + base)[o]; x.nx[6][e] = (p.dy + base)[o];
        x.nsa[e] = (p.sa + base)[o];
    }
}
// first half of the preparation: the decay of each token, this wave's decay sum; the other inputs are kept packed so that the
// registers of x are free for the next fetch
DEVINL void bwd_convert(PlanesB& O, const Prep7& x, Conv7& y, int wp, int lane) {
#pragma unroll
    for (int e = 0; e < 4; ++e) { y.sg[e] = sigmoid_fast(bf2f(x.nx[0][e])); y.uu[e] = x.nsa[e]; }
#pragma unroll
    for (int k = 0; k < 6; ++k)
#pragma unroll
        for (int z = 0; z < 2; ++z) y.pk[k][z] = x.nx[k + 1][2 * z] | (x.nx[k + 1][2 * z + 1] << 16);
    O.part[wp][lane] = W_SCALE * ((y.sg[0] + y.sg[1]) + (y.sg[2] + y.sg[3]));
}
// second half (after a barrier): the in-chunk factors and every plane
template <int E0 = 0, int E1 = 4>
DEVINL void bwd_planes(PlanesB& O, const Conv7& y, int wp, int lane) {
    float cm, cl;
    const float lam[4] = {W_SCALE * y.sg[0], W_SCALE * y.sg[1], W_SCALE * y.sg[2], W_SCALE * y.sg[3]};
    const Factors f = chunk_factors<E0, E1>(lam, O.part, wp, lane, cm, cl);
#pragma unroll
    for (int e = E0; e < E1; ++e) {
        const int t = 4 * wp + e;
        auto in = [&](int k) __attribute__((always_inline)) { return (e & 1) ? bf_hi(y.pk[k][e >> 1]) : bf_lo(y.pk[k][e >> 1]); };
        const float rr = in(0), kk = in(1), vv = in(2), aa = in(3), bb = in(4), gg = in(5);
        O.Ap[t][lane] = aa * f.ea[e];
        O.Rp[t][lane] = rr * f.er[e];
        O.Bp[t][lane] = bb * f.eb[e];
        O.Kp[t][lane] = kk * f.eb[e];
        O.As[t][lane] = aa * f.es[e];
        O.Rs[t][lane] = rr * (f.es[e] * __expf(lam[e]));
        O.Bd[t][lane] = bb * f.ee[e];
        O.Kd[t][lane] = kk * f.ee[e];
        O.V[t][lane] = vv;
        O.dY[t][lane] = gg;
        O.U[t][lane] = y.uu[e];
        O.EA[t][lane] = f.ea[e];
        O.ER[t][lane] = f.er[e];
        O.DWF[t][lane] = W_SCALE * y.sg[e] * (1.f - y.sg[e]);
    }
    if (E0 == 0 && wp == 0) { O.d1[lane] = exp_acc(cm); O.d2[lane] = exp_acc(cl - cm); O.dec[lane] = exp_acc(cl); }
}
// da dr db dk dw (and dv) of one chunk leave their parking places as whole rows (256 threads, four channels each)
DEVINL void bwd_store_rows(const SmemCB& S, int vbuf, const Args7c& p, size_t row0, int tp, int H, int h) {
    const int t = tp >> 4, c4 = (tp & 15) * 4;
    const size_t base = (row0 * H + h) * N;
    uint32_t o = static_cast<uint32_t>(t * H) * N + c4;
    asm volatile("" : "+v"(o));
    auto put = [&](uint16_t* dst, const uint16_t* src) __attribute__((always_inline)) {
        *reinterpret_cast<uint2*>(dst + base + o) = *reinterpret_cast<const uint2*>(src);
    };
    put(p.da, &S.park[0][t][c4]); put(p.dr, &S.park[1][t][c4]); put(p.db, &S.park[2][t][c4]); put(p.dk, &S.park[3][t][c4]);
    put(p.dw, &S.park[4][t][c4]); put(p.dv, &S.parkv[vbuf][t][c4]);
}
DEVINL void bwd_role_p(SmemCB& S, const Args7c& p, int tid, int w, size_t tok0, int nch, int H, int h) {
    const int lane = tid & 63, wp = w - 8, tp = tid - 8 * 64;
    // Raw rows are asked for two visits before they are converted (one visit, of which only two phases lie between the
    // request and the use, is less than the memory system takes under load: the A and B waves then waited for the P waves
    // at two of the three barriers of every visit).  Two register sets take turns; the chunk index is clamped instead of
    // the request being skipped, so that every visit issues the same loads and the waits count the same.
    Prep7 x[2];
    Conv7 y;
    auto row_of = [&](int visit) { const int c = nch - 1 - visit; return tok0 + static_cast<size_t>(c > 0 ? c : 0) * CL; };
    bwd_fetch(p, x[0], row_of(0), wp, lane, H, h);
    bwd_fetch(p, x[1], row_of(1), wp, lane, H, h);
    bwd_convert(S.pl[0], x[0], y, wp, lane);          // visit 0, before the loop
    bwd_fetch(p, x[0], row_of(2), wp, lane, H, h);
    __syncthreads();
    bwd_planes(S.pl[0], y, wp, lane);
    __syncthreads();
    auto visit = [&](const int i, auto Z) __attribute__((always_inline)) {     // visit i is chunk nch - 1 - i
        constexpr int z = decltype(Z)::value;        // the set that holds visit i + 1
        const bool next = i + 1 < nch;
        if (next) bwd_convert(S.pl[(i + 1) & 1], x[z], y, wp, lane);
        bwd_fetch(p, x[z], row_of(i + 3), wp, lane, H, h);
        __syncthreads();
        // the planes of two of this wave's four tokens in phase 2, the other two in phase 3, in which these waves used to idle
        // while everybody waited for them in phase 2 (nothing reads these planes before the next visit)
        if (next) bwd_planes<0, 2>(S.pl[(i + 1) & 1], y, wp, lane);
        __syncthreads();
        if (next) bwd_planes<2, 4>(S.pl[(i + 1) & 1], y, wp, lane);
        __syncthreads();
    };
    for (int i = 0; i < nch; i += 2) {
        visit(i, std::integral_constant<int, 1>{});
        if (i + 1 < nch) visit(i + 1, std::integral_constant<int, 0>{});
    }
    __syncthreads();                                 // role B finishes the last chunk
    bwd_store_rows(S, (nch - 1) & 1, p, tok0, tp, H, h);
}

DEVINL void bwd_role_a(SmemCB& S, const Args7c& p, int tid, int w, size_t bh, int nch, size_t tok0, int H, int h) {
    const int lane = tid & 63, q = w & 3, l16 = lane & 15, g = lane >> 4;
    const int own = 16 * q + l16;                    // value channel i of this lane's column
    f32x4 dS[4];                                     // dS[i = own][j = 16 jt + 4 g + v]
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
        dS[jt] = p.dsT != nullptr ? ld4(p.dsT + bh * N * N + static_cast<size_t>(own) * N + 16 * jt + 4 * g) : ZERO4;
    __syncthreads();
    __syncthreads();
    for (int i = 0; i < nch; ++i) {
        const PlanesB& O = S.pl[i & 1];
        // ---------------------------------------------------------------- phase 1: the parts of dU, dV, dS that need no tile; a causal tile; M
        // (a chain of dependent matrix instructions runs slower than independent ones: two partial sums each)
        f32x4 dyop, dUp[2] = {ZERO4, ZERO4}, dVp[2] = {ZERO4, ZERO4}, accA[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) dyop[v] = O.dY[4 * g + v][own];           // dY[tau = 4 g + v][i]
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            const f32x4 xb = ld4(&O.Bd[l16][16 * jt + 4 * g]), xk = ld4(&O.Kd[l16][16 * jt + 4 * g]);
            f32x4 acc = ZERO4;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                dUp[jt & 1] = mm(xb[v], dS[jt][v], dUp[jt & 1]);
                dVp[jt & 1] = mm(xk[v], dS[jt][v], dVp[jt & 1]);
                acc = mm(O.Rs[4 * g + v][16 * jt + l16], dyop[v], acc);
            }
            accA[jt] = acc;
        }
        causal_tile(q < 2 ? O.Ap : O.Rp, (q & 1) ? O.Kp : O.Bp, q == 0 ? S.AB : (q == 1 ? S.AK : (q == 2 ? S.RB : S.RK)), q < 2, l16, g);
        if (q == 0) {                                // this wave wrote AB itself: LDS keeps a wave's accesses in order
            float m[CL];
            inverse_cols(S.AB, l16, m);
            if (g == 0)
#pragma unroll
                for (int t = 0; t < CL; ++t) S.M[t][l16] = m[t];
        }
        f32x4 dU = dUp[0] + dUp[1], dV = dVp[0] + dVp[1];
        __syncthreads();
        // ---------------------------------------------------------------- phase 2: dU, dW = M^T dU, dV, the gradient state
        {
#pragma unroll
            for (int v = 0; v < 4; ++v) dU = mm(S.RB[4 * g + v][l16], dyop[v], dU);
            f32x4 dW = ZERO4;
#pragma unroll
            for (int v = 0; v < 4; ++v) dW = mm(S.M[4 * g + v][l16], dU[v], dW);
#pragma unroll
            for (int v = 0; v < 4; ++v) S.dW[4 * g + v][own] = dW[v];
#pragma unroll
            for (int v = 0; v < 4; ++v) dV = mm(S.AK[4 * g + v][l16], dW[v], dV);
#pragma unroll
            for (int v = 0; v < 4; ++v) dV = mm(S.RK[4 * g + v][l16], dyop[v], dV);
#pragma unroll
            for (int v = 0; v < 4; ++v) S.parkv[i & 1][4 * g + v][own] = f2bf(dV[v]);
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                f32x4 acc = accA[jt];
#pragma unroll
                for (int v = 0; v < 4; ++v) acc = mm(O.As[4 * g + v][16 * jt + l16], dW[v], acc);
                dS[jt] = dS[jt] * ld4(&O.dec[16 * jt + 4 * g]) + acc;
            }
        }
        __syncthreads();
        // ---------------------------------------------------------------- phase 3: dAB, dAK (they need dW)
        if (q < 2) causal_tile(S.dW, q == 0 ? O.U : O.V, q == 0 ? S.dAB : S.dAK, true, l16, g);
        else if (i > 0) {
            // The two waves without a tile here carry the finished rows of the visit before to global memory (parked by the
            // B waves in phase 1, dv by this role one visit earlier; both stay as they are until the next visit): the P
            // waves, for which this was a third of a phase that everybody waits for, keep to loads.
            const int tp = tid - 2 * 64;
            bwd_store_rows(S, (i - 1) & 1, p, tok0 + static_cast<size_t>(nch - i) * CL, tp, H, h);
            bwd_store_rows(S, (i - 1) & 1, p, tok0 + static_cast<size_t>(nch - i) * CL, tp + 128, H, h);
        }
        __syncthreads();
    }
    __syncthreads();
    if (p.ds0 != nullptr) {
        float* dst = p.ds0 + bh * N * N + static_cast<size_t>(own) * N + 4 * g;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) st4(dst + 16 * jt, dS[jt]);
    }
}

DEVINL void bwd_role_b(SmemCB& S, const Args7c& p, int tid, int w, size_t bh, int nch) {
    const int lane = tid & 63, q = w & 3, l16 = lane & 15, g = lane >> 4;
    const int own = 16 * q + l16;                    // key channel j of this lane's column
    f32x4 dS[4], S0b[4];                             // dS, S0 at [i = 16 ib + 4 g + v][j = own]
#pragma unroll
    for (int ib = 0; ib < 4; ++ib)
#pragma unroll
        for (int v = 0; v < 4; ++v)
            dS[ib][v] = p.dsT != nullptr ? p.dsT[bh * N * N + static_cast<size_t>(16 * ib + 4 * g + v) * N + own] : 0.f;
    auto fetch_state = [&](int c) __attribute__((always_inline)) {
        const float* slot = p.s + (bh * nch + c) * N * N;
        uint32_t o = static_cast<uint32_t>(4 * g) * N + own;
        asm volatile("" : "+v"(o));
#pragma unroll
        for (int ib = 0; ib < 4; ++ib)
#pragma unroll
            for (int v = 0; v < 4; ++v) S0b[ib][v] = slot[o + (16 * ib + v) * N];
    };
    float Pj = 0.f;                                  // P at the end of the chunk whose phase 4 comes next
    f32x4 xA = ZERO4, xR = ZERO4, xB = ZERO4, xK = ZERO4;     // state parts of dA', dR', dB', dK', carried into the next visit's phase 1
    // tile parts, scaling, decay gradient of the chunk whose planes are O; results parked as bf16
    auto finish = [&](const PlanesB& O) __attribute__((always_inline)) {
        const float d1j = O.d1[own], d2j = O.d2[own];
        f32x4 bp, kp, ap, rp;                        // planes at [s or t = 4 g + v][j]
#pragma unroll
        for (int v = 0; v < 4; ++v) { bp[v] = O.Bp[4 * g + v][own]; kp[v] = O.Kp[4 * g + v][own]; ap[v] = O.Ap[4 * g + v][own]; rp[v] = O.Rp[4 * g + v][own]; }
        f32x4 tA = ZERO4, tR = ZERO4, tB = ZERO4, tK = ZERO4;
        const f32x4 dab = ld4(&S.dAB[l16][4 * g]), dak = ld4(&S.dAK[l16][4 * g]), drb = ld4(&S.dRB[l16][4 * g]), drk = ld4(&S.dRK[l16][4 * g]);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            tA = mm(dab[v], bp[v], tA); tR = mm(drb[v], bp[v], tR);
            tB = mm(S.dAB[4 * g + v][l16], ap[v], tB); tK = mm(S.dAK[4 * g + v][l16], ap[v], tK);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            tA = mm(dak[v], kp[v], tA); tR = mm(drk[v], kp[v], tR);
            tB = mm(S.dRB[4 * g + v][l16], rp[v], tB); tK = mm(S.dRK[4 * g + v][l16], rp[v], tK);
        }
        float del[4], ada[4], dwf[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int t = 4 * g + v;
            const float dAp = fmaf(d1j, xA[v], tA[v]), dRp = fmaf(d1j, xR[v], tR[v]);
            const float dBp = fmaf(d2j, xB[v], tB[v]), dKp = fmaf(d2j, xK[v], tK[v]);
            const float ea = O.EA[t][own], er = O.ER[t][own];
            const float eb = __frcp_rn(er);
            S.park[0][t][own] = f2bf(dAp * ea);
            S.park[1][t][own] = f2bf(dRp * er);
            S.park[2][t][own] = f2bf(dBp * eb);
            S.park[3][t][own] = f2bf(dKp * eb);
            ada[v] = ap[v] * dAp;
            del[v] = fmaf(rp[v], dRp, -fmaf(bp[v], dBp, kp[v] * dKp));      // r dr - b db - k dk
            dwf[v] = O.DWF[t][own];
        }
        // G_t = P_{t+1} + del_t,  P_t = G_t + a da:  suffix sums over t = 4 g + v, later lane groups first
        const float tot = (del[0] + ada[0]) + (del[1] + ada[1]) + (del[2] + ada[2]) + (del[3] + ada[3]);
        const float t1 = __shfl_down(tot, 16, 64), t2 = __shfl_down(tot, 32, 64), t3 = __shfl_down(tot, 48, 64);
        float Pn = Pj + (g < 3 ? t1 : 0.f) + (g < 2 ? t2 : 0.f) + (g < 1 ? t3 : 0.f);     // P after this lane's last token
#pragma unroll
        for (int v = 3; v >= 0; --v) {
            const float G = Pn + del[v];
            Pn = G + ada[v];
            S.park[4][4 * g + v][own] = f2bf(G * dwf[v]);
        }
        Pj = __shfl(Pn, l16, 64);                    // lane group 0 holds P at the start of the chunk
    };
    fetch_state(nch - 1);
    __syncthreads();
    __syncthreads();
    for (int i = 0; i < nch; ++i) {
        const int c = nch - 1 - i;
        const PlanesB& O = S.pl[i & 1];
        // ---------------------------------------------------------------- phase 1: finish the previous visit's chunk
        if (i > 0) finish(S.pl[(i - 1) & 1]);
        __syncthreads();
        // ---------------------------------------------------------------- phase 2: dY S0, U dS, V dS; dRB, dRK
        if (i == 0 && p.dsT != nullptr) {
            // P at the end of the call: sum_i dsT o S_T with S_T = S0 dec + U^T (B' d2) + V^T (K' d2) of the last chunk
            const float decj = O.dec[own];
            float pp = 0.f;
#pragma unroll
            for (int ib = 0; ib < 4; ++ib) {
                f32x4 acc = ZERO4;
#pragma unroll
                for (int v = 0; v < 4; ++v) acc = mm(O.U[4 * g + v][16 * ib + l16], O.Bd[4 * g + v][own], acc);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc = mm(O.V[4 * g + v][16 * ib + l16], O.Kd[4 * g + v][own], acc);
#pragma unroll
                for (int v = 0; v < 4; ++v) pp = fmaf(dS[ib][v], fmaf(S0b[ib][v], decj, acc[v]), pp);
            }
            pp += __shfl_xor(pp, 16, 64);
            pp += __shfl_xor(pp, 32, 64);
            Pj = pp;
        }
        {
            f32x4 pr[2] = {ZERO4, ZERO4}, pb[2] = {ZERO4, ZERO4}, pk[2] = {ZERO4, ZERO4};   // two partial sums each: independent chains
#pragma unroll
            for (int ib = 0; ib < 4; ++ib) {
                const f32x4 ya = ld4(&O.dY[l16][16 * ib + 4 * g]), ua = ld4(&O.U[l16][16 * ib + 4 * g]), va = ld4(&O.V[l16][16 * ib + 4 * g]);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    pr[ib & 1] = mm(ya[v], S0b[ib][v], pr[ib & 1]);
                    pb[ib & 1] = mm(ua[v], dS[ib][v], pb[ib & 1]);
                    pk[ib & 1] = mm(va[v], dS[ib][v], pk[ib & 1]);
                }
            }
            xR = pr[0] + pr[1]; xB = pb[0] + pb[1]; xK = pk[0] + pk[1];
        }
        if (q >= 2) causal_tile(O.dY, q == 2 ? O.U : O.V, q == 2 ? S.dRB : S.dRK, false, l16, g);
        __syncthreads();
        // ---------------------------------------------------------------- phase 3: dW S0; the gradient state
        {
            const float decj = O.dec[own];
            f32x4 rs, as;
#pragma unroll
            for (int v = 0; v < 4; ++v) { rs[v] = O.Rs[4 * g + v][own]; as[v] = O.As[4 * g + v][own]; }
            f32x4 pa[2] = {ZERO4, ZERO4};
#pragma unroll
            for (int ib = 0; ib < 4; ++ib) {
                const f32x4 wa = ld4(&S.dW[l16][16 * ib + 4 * g]);
#pragma unroll
                for (int v = 0; v < 4; ++v) pa[ib & 1] = mm(wa[v], S0b[ib][v], pa[ib & 1]);
                f32x4 acc = ZERO4;
#pragma unroll
                for (int v = 0; v < 4; ++v) acc = mm(O.dY[4 * g + v][16 * ib + l16], rs[v], acc);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc = mm(S.dW[4 * g + v][16 * ib + l16], as[v], acc);
                dS[ib] = dS[ib] * decj + acc;
            }
            xA = pa[0] + pa[1];
            if (c > 0) fetch_state(c - 1);
        }
        __syncthreads();
    }
    finish(S.pl[(nch - 1) & 1]);
    __syncthreads();
}

__global__ __launch_bounds__(NTB, 3) void rwkv7c_bwd(const Args7c p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    SmemCB& S = *reinterpret_cast<SmemCB*>(smem_raw);
    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x, b = blockIdx.y;
    const size_t bh = static_cast<size_t>(b) * p.H + h;
    const size_t tok0 = static_cast<size_t>(b) * p.T;
    const int nch = p.T / CL;
    if (w < 4) bwd_role_a(S, p, tid, w, bh, nch, tok0, p.H, h);
    else if (w < 8) bwd_role_b(S, p, tid, w, bh, nch);
    else bwd_role_p(S, p, tid, w, tok0, nch, p.H, h);
}

}  // namespace


int launch7c_fwd(hipStream_t st, int B, int T, int H, const float* s0, const uint16_t* r, const uint16_t* w, const uint16_t* k,
                 const uint16_t* v, const uint16_t* a, const uint16_t* b, uint16_t* y, float* sT, float* s, float* sa) {
    Args7c p{};
    p.T = T; p.H = H; p.s0 = s0; p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b; p.y = y; p.sT = sT; p.s = s; p.sa = sa;
    hipLaunchKernelGGL(rwkv7c_fwd, dim3(H, B), dim3(NT), 0, st, p);
    return launch_status();
}

int launch7c_bwd(hipStream_t st, int B, int T, int H, const uint16_t* r, const uint16_t* w, const uint16_t* k, const uint16_t* v,
                 const uint16_t* a, const uint16_t* b, const uint16_t* dy, const float* dsT, const float* s, const float* sa,
                 float* ds0, uint16_t* dr, uint16_t* dw, uint16_t* dk, uint16_t* dv, uint16_t* da, uint16_t* db) {
    Args7c p{};
    p.T = T; p.H = H; p.r = r; p.w = w; p.k = k; p.v = v; p.a = a; p.b = b; p.dy = dy; p.dsT = dsT;
    p.s = const_cast<float*>(s); p.sa = const_cast<float*>(sa); p.ds0 = ds0;
    p.dr = dr; p.dw = dw; p.dk = dk; p.dv = dv; p.da = da; p.db = db;
    static_assert(sizeof(SmemCB) <= 160 * 1024, "the backward's LDS must fit one CU");
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rwkv7c_bwd), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       static_cast<int>(sizeof(SmemCB)));
    if (attr != hipSuccess) { g_last_hip_error = static_cast<int>(attr); return RWKV_ERR_LAUNCH; }
    hipLaunchKernelGGL(rwkv7c_bwd, dim3(H, B), dim3(NTB), sizeof(SmemCB), st, p);
    return launch_status();
}

}  // namespace rwkv
