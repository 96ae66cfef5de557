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
#include "common.h"

namespace rwkv {
namespace {

constexpr int N = 64;
constexpr int L = 32;             // chunk length
constexpr int NW = 8;             // waves per workgroup: two per SIMD (a single wave per SIMD issues VALU ~3x slower)
constexpr int NT = NW * 64;
constexpr int RS = 68;            // row stride (dwords) of [token][channel] operand arrays: 272 B
constexpr int TS = 36;            // row stride (dwords) of [channel][token] hi/lo operand arrays: 144 B
constexpr int VS = 20;            // row stride (dwords) of the bf16 [channel][token] array: 80 B
constexpr int STAGES = 4;         // chunks of input kept in flight
constexpr float RANGE_LIMIT = 60.0f;
constexpr float LOG2E = 1.44269504088896340736f;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

enum { W_EW = 1, W_RAW = 2 };     // wkv6: fp32 ew = -exp(w_raw) [B,T,C];  wkv6_state: raw bf16 w

struct ArgsC {
    int T, C, H;
    const uint16_t *r, *k, *v, *u, *s0;
    const void* w;
    uint16_t* y;
};

// Operand format.  An fp32 value x is used as hi = bf16(x), lo = bf16(x - hi).  Along the K axis of an MFMA a lane holds
// 8 slots = 4 consecutive elements e0..e3 as  P = [h0 h1 h2 h3 | l0 l1 l2 l3]  (dwords H01, H23, L01, L23).  With the
// halves exchanged, P~ = [l0 l1 l2 l3 | h0 h1 h2 h3] (a register renaming, no instruction), and Q in the same format,
//     mfma(P, Q) + mfma(P~, Q) = sum_e (h + l)_P (h + l)_Q
// i.e. the full product at ~16 mantissa bits per operand.  An operand that is exact in bf16 (v) is used as
// [v0 v1 v2 v3 | v0 v1 v2 v3], which makes a single mfma(P, .) = sum_e (h + l)_P v.
struct HL { uint32_t h, l; };     // two elements: bf16 pair of the hi parts, bf16 pair of the lo parts
DEVINL uint32_t cvt2(float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 p = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, p);
}
DEVINL HL hilo2(float a, float b) {
    HL r;
    r.h = cvt2(a, b);
    r.l = cvt2(a - __uint_as_float(r.h << 16), b - __uint_as_float(r.h & 0xffff0000u));
    return r;
}
DEVINL bf16x8 as_op(uint32_t a, uint32_t b, uint32_t c, uint32_t d) { return __builtin_bit_cast(bf16x8, make_uint4(a, b, c, d)); }
DEVINL bf16x8 lds_op(const uint32_t* p) { return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p)); }
DEVINL bf16x8 lds_dup(const uint32_t* p) {          // 4 exact bf16 -> [v0..v3 | v0..v3]
    const uint2 x = *reinterpret_cast<const uint2*>(p);
    return as_op(x.x, x.y, x.x, x.y);
}
DEVINL bf16x8 swapped(const bf16x8& a) {
    const uint4 x = __builtin_bit_cast(uint4, a);
    return as_op(x.z, x.w, x.x, x.y);
}
DEVINL f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
DEVINL f32x4 mfma_full(bf16x8 a, bf16x8 b, f32x4 c) { return mfma(swapped(a), b, mfma(a, b, c)); }
DEVINL float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// dword position, inside a stored row, of the (H, L) pair of elements (2p, 2p+1): groups of 4 elements are H01 H23 L01 L23
DEVINL int hpos(int p) { return 4 * (p >> 1) + (p & 1); }

struct alignas(16) SmemFwd {
    uint32_t Rs[L][RS];            // r e^{c_t}             [t][j]   A operand of  Rs S0^T
    uint32_t Rp[L][RS];            // r e^{c_t - c_m}       [t][j]   B operand of  A^T = K' R'^T
    uint32_t Kp[L][RS];            // k e^{c_m - c_{t+1}}   [s][j]   A operand of  A^T
    uint32_t Ke[N][TS];            // k e^{c_L - c_{s+1}}   [j][s]   A operand of  S^T += Ke^T V
    uint32_t Am[L][TS];            // A                     [t][s]   A operand of  A V
    uint32_t Vt[N][VS];            // v, plain bf16         [i][s]   B operand
    float X[L][N];                 // r u k [t][j], summed over j into the diagonal of A;  exact path: r
    float raw[2][L][N];            // exact path only: k, decay as fp32 [t][j]
    float dec[N];                  // e^{c_L}[j]   (exact path: u)
    float part[8][N];              // sum of lam (in log2 units) over each eighth of the chunk
    float Y[2][2][L][RS];          // output staging, double buffered: partial sums of the two key-channel halves
};

// One workgroup of 8 waves per (batch, head).  Wave (q = wid & 3, jh = wid >> 2) owns value channels [16q, 16q+16) and the
// key-channel half [32jh, 32jh+32) of the state: S^T[j][i] in two accumulator tiles,  D[m][v] <-> j = 32jh + 16m + 4g + v.
// The accumulator layout is used as is as the B operand of Rs S0^T (lane group g holds channels 4g..4g+3 of each tile).
template <int WMODE>
__global__ __launch_bounds__(NT) void wkv6_fwd_chunk(const ArgsC a) {
    __shared__ SmemFwd S;
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, l16 = lane & 15, g = lane >> 4;
    const int q = wid & 3, jh = wid >> 2;
    const int b = blockIdx.x / a.H, h = blockIdx.x % a.H;
    const int T = a.T, C = a.C;
    const size_t base = static_cast<size_t>(b) * T * C + static_cast<size_t>(h) * N;
    const size_t bh = static_cast<size_t>(b) * a.H + h;
    const uint16_t* __restrict__ rb = a.r + base;
    const uint16_t* __restrict__ kb = a.k + base;
    const uint16_t* __restrict__ vb_ = a.v + base;
    // prep coordinates: channel pair (2 jp, 2 jp + 1), tokens 4 wid + 2 th + {0, 1}
    const int jp = lane & 31, th = lane >> 5, pt0 = 4 * wid + 2 * th;
    float uj[2];
    {
        const uint32_t x = *reinterpret_cast<const uint32_t*>(a.u + h * N + 2 * jp);
        uj[0] = bf_lo(x); uj[1] = bf_hi(x);
    }

    f32x4 D[2];
    D[0] = D[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (a.s0 != nullptr) {
        const uint16_t* s = a.s0 + (bh * N + q * 16 + l16) * N + 32 * jh;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const uint2 x = *reinterpret_cast<const uint2*>(s + 16 * m + 4 * g);
            D[m] = f32x4{bf_lo(x.x), bf_hi(x.x), bf_lo(x.y), bf_hi(x.y)};
        }
    }
    // the upper-right 16x16 tile of A (t < 16 <= s) is never written: keep it zero
    for (int i = tid; i < L * TS; i += NT) (&S.Am[0][0])[i] = 0;

    const int nchunks = (T + L - 1) / L;
    // Raw bits of the chunks to come (two channels per load), converted only when a chunk is prepared.  HBM latency is
    // a few microseconds and a chunk is ~1 us of work, so STAGES chunks are kept in flight (one register set each; the
    // chunk loop is unrolled by STAGES to keep the set index static).
    struct Raw { uint32_t r[2], k[2], v[2], w[2][2]; };
    Raw ring[STAGES];
    auto prefetch = [&](int c, Raw& x) __attribute__((always_inline)) {
        uint32_t (&qr)[2] = x.r; uint32_t (&qk)[2] = x.k; uint32_t (&qv)[2] = x.v; uint32_t (&qw)[2][2] = x.w;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = c * L + pt0 + e;
            const uint32_t o = static_cast<uint32_t>(t < T ? t : T - 1) * C + 2 * jp;
            qr[e] = *reinterpret_cast<const uint32_t*>(rb + o);
            qk[e] = *reinterpret_cast<const uint32_t*>(kb + o);
            qv[e] = *reinterpret_cast<const uint32_t*>(vb_ + o);
            if constexpr (WMODE == W_RAW) {
                qw[e][0] = *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(a.w) + base + o);
            } else {
                const uint2 x = *reinterpret_cast<const uint2*>(static_cast<const float*>(a.w) + base + o);
                qw[e][0] = x.x; qw[e][1] = x.y;
            }
        }
    };
    static_for<STAGES>([&](auto Z) { if (decltype(Z)::value < nchunks) prefetch(decltype(Z)::value, ring[decltype(Z)::value]); });

    auto process = [&](const int c, Raw& x) __attribute__((always_inline)) {
        uint32_t (&qr)[2] = x.r; uint32_t (&qk)[2] = x.k; uint32_t (&qv)[2] = x.v; uint32_t (&qw)[2][2] = x.w;
        const int c0 = c * L, buf = c & 1;
        // ------------------------------------------------------------------ prep
        // element [e][z]: token pt0 + e, channel 2 jp + z.  lam is kept in log2 units.
        float pr[2][2], pk[2][2], plam[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const bool ok = (c0 + pt0 + e) < T;            // rows past T: no input, no decay
            if (!ok) { qr[e] = 0; qk[e] = 0; qv[e] = 0; }
            pr[e][0] = bf_lo(qr[e]); pr[e][1] = bf_hi(qr[e]);
            pk[e][0] = bf_lo(qk[e]); pk[e][1] = bf_hi(qk[e]);
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                float lam;
                if constexpr (WMODE == W_RAW) lam = -exp2_fast(LOG2E * (z ? bf_hi(qw[e][0]) : bf_lo(qw[e][0])));
                else lam = __uint_as_float(qw[e][z]);
                plam[e][z] = ok ? lam * LOG2E : 0.f;
            }
        }
        // sums over this wave's 4 tokens: lanes 0..31 hold tokens 0,1, lanes 32..63 tokens 2,3 of the same channels
        float s2[2], s4[2], other[2];
#pragma unroll
        for (int z = 0; z < 2; ++z) {
            s2[z] = plam[0][z] + plam[1][z];
            other[z] = __shfl_xor(s2[z], 32, 64);
            s4[z] = s2[z] + other[z];
        }
        if (th == 0) *reinterpret_cast<float2*>(&S.part[wid][2 * jp]) = make_float2(s4[0], s4[1]);
        // a chunk whose decays could overflow the mid-point factors is redone exactly; any half-chunk sum beyond
        // the limit implies an eighth beyond limit/4, so this local test is sufficient (and conservative)
        const bool exact = __syncthreads_or((-s4[0] > 0.25f * RANGE_LIMIT * LOG2E) || (-s4[1] > 0.25f * RANGE_LIMIT * LOG2E)) != 0;
        float pre[2] = {0.f, 0.f}, cm[2] = {0.f, 0.f}, cl[2] = {0.f, 0.f};   // before this wave's tokens / middle / whole
#pragma unroll
        for (int w8 = 0; w8 < 8; ++w8) {
            const float2 x = *reinterpret_cast<const float2*>(&S.part[w8][2 * jp]);
            if (w8 < wid) { pre[0] += x.x; pre[1] += x.y; }
            if (w8 < 4) { cm[0] += x.x; cm[1] += x.y; }
            cl[0] += x.x; cl[1] += x.y;
        }
        if (th) { pre[0] += other[0]; pre[1] += other[1]; }
        if (!exact) {
            float rp[2][2], rs[2][2], kp[2][2], ke[2][2];
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const float d1 = exp2_fast(cm[z]), d2 = exp2_fast(cl[z] - cm[z]);
                if (wid == 0 && th == 0) S.dec[2 * jp + z] = exp2_fast(cl[z]);
                const float ct0 = pre[z], ct1 = ct0 + plam[0][z], ct2 = ct1 + plam[1][z];
                rp[0][z] = pr[0][z] * exp2_fast(ct0 - cm[z]);
                rp[1][z] = pr[1][z] * exp2_fast(ct1 - cm[z]);
                kp[0][z] = pk[0][z] * exp2_fast(cm[z] - ct1);
                kp[1][z] = pk[1][z] * exp2_fast(cm[z] - ct2);
#pragma unroll
                for (int e = 0; e < 2; ++e) { rs[e][z] = rp[e][z] * d1; ke[e][z] = kp[e][z] * d2; }
            }
            const int ph = hpos(jp);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int t = pt0 + e;
                HL x = hilo2(rp[e][0], rp[e][1]); S.Rp[t][ph] = x.h; S.Rp[t][ph + 2] = x.l;
                x = hilo2(rs[e][0], rs[e][1]);    S.Rs[t][ph] = x.h; S.Rs[t][ph + 2] = x.l;
                x = hilo2(kp[e][0], kp[e][1]);    S.Kp[t][ph] = x.h; S.Kp[t][ph + 2] = x.l;
                *reinterpret_cast<float2*>(&S.X[t][2 * jp]) = make_float2(pr[e][0] * uj[0] * pk[e][0], pr[e][1] * uj[1] * pk[e][1]);
            }
#pragma unroll
            for (int z = 0; z < 2; ++z) {                  // Ke^T: pair along the two tokens
                const HL x = hilo2(ke[0][z], ke[1][z]);
                S.Ke[2 * jp + z][4 * wid + th] = x.h;
                S.Ke[2 * jp + z][4 * wid + 2 + th] = x.l;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int t = pt0 + e;
                *reinterpret_cast<float2*>(&S.X[t][2 * jp]) = make_float2(pr[e][0], pr[e][1]);
                *reinterpret_cast<float2*>(&S.raw[0][t][2 * jp]) = make_float2(pk[e][0], pk[e][1]);
                *reinterpret_cast<float2*>(&S.raw[1][t][2 * jp]) = make_float2(exp2_fast(plam[e][0]), exp2_fast(plam[e][1]));
            }
            if (wid == 0 && th == 0) *reinterpret_cast<float2*>(&S.dec[2 * jp]) = make_float2(uj[0], uj[1]);
        }
        // V^T[i][s]: the two tokens of channel 2jp+z are one dword
        {
            uint16_t* vt = reinterpret_cast<uint16_t*>(&S.Vt[0][0]);
            *reinterpret_cast<uint32_t*>(vt + (2 * jp) * (2 * VS) + pt0) = (qv[0] & 0xffffu) | (qv[1] << 16);
            *reinterpret_cast<uint32_t*>(vt + (2 * jp + 1) * (2 * VS) + pt0) = (qv[0] >> 16) | (qv[1] & 0xffff0000u);
        }
        __syncthreads();
        if (c + STAGES < nchunks) prefetch(c + STAGES, x);   // this register set is free again

        if (!exact) {
            // -------------------------------------------------------------- A^T tiles: waves 0,1,2 -> A(0,0) A(1,0) A(1,1)
            if (wid < 3) {
                const int ta = (wid == 0) ? 0 : 1, tb = (wid == 2) ? 1 : 0;
                f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int js = 0; js < 4; js += 2) {     // rows of the result: s (from K'), columns: t (from R')
                    acc0 = mfma_full(lds_op(&S.Kp[16 * tb + l16][16 * js + 4 * g]), lds_op(&S.Rp[16 * ta + l16][16 * js + 4 * g]), acc0);
                    acc1 = mfma_full(lds_op(&S.Kp[16 * tb + l16][16 * js + 16 + 4 * g]), lds_op(&S.Rp[16 * ta + l16][16 * js + 16 + 4 * g]), acc1);
                }
                f32x4 acc = acc0 + acc1;                // acc[v]: s = 4g + v, t = l16
                if (ta == tb) {
                    // diagonal: sum_j r u k of row t = 16 ta + l16 (this lane sums 16 channels, the 4 groups the rest)
                    float d = 0.f;
#pragma unroll
                    for (int z = 0; z < 4; ++z) {
                        const float4 x = *reinterpret_cast<const float4*>(&S.X[16 * ta + l16][16 * g + 4 * z]);
                        d += (x.x + x.y) + (x.z + x.w);
                    }
                    d = allreduce_rows(d);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int sl = 4 * g + v;
                        acc[v] = (sl < l16) ? acc[v] : (sl == l16 ? d : 0.f);
                    }
                }
                const HL x0 = hilo2(acc[0], acc[1]), x1 = hilo2(acc[2], acc[3]);
                *reinterpret_cast<uint4*>(&S.Am[16 * ta + l16][16 * tb + 4 * g]) = make_uint4(x0.h, x1.h, x0.l, x1.l);
            }
            // -------------------------------------------------------------- Y (this half of j) = Rs S0^T
            f32x4 Y[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const HL x0 = hilo2(D[m][0], D[m][1]), x1 = hilo2(D[m][2], D[m][3]);
                const bf16x8 sb = as_op(x0.h, x1.h, x0.l, x1.l);
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
                    Y[mt] = mfma_full(lds_op(&S.Rs[16 * mt + l16][32 * jh + 16 * m + 4 * g]), sb, Y[mt]);
            }
            __syncthreads();                           // A is in LDS
            // -------------------------------------------------------------- Y += A V (tokens of half jh);  S^T = S^T diag(dec) + Ke^T V
            const bf16x8 vb0 = lds_dup(&S.Vt[16 * q + l16][2 * g]);        // tokens  4g..4g+3
            const bf16x8 vb1 = lds_dup(&S.Vt[16 * q + l16][8 + 2 * g]);    // tokens 16+4g..
            if (jh == 0) {
                Y[0] = mfma(lds_op(&S.Am[l16][4 * g]), vb0, Y[0]);
                Y[1] = mfma(lds_op(&S.Am[16 + l16][4 * g]), vb0, Y[1]);
            } else {
                Y[1] = mfma(lds_op(&S.Am[16 + l16][16 + 4 * g]), vb1, Y[1]);
            }
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const int j0 = 32 * jh + 16 * m;
                const float4 dj = *reinterpret_cast<const float4*>(&S.dec[j0 + 4 * g]);
                f32x4 x = {D[m][0] * dj.x, D[m][1] * dj.y, D[m][2] * dj.z, D[m][3] * dj.w};
                x = mfma(lds_op(&S.Ke[j0 + l16][4 * g]), vb0, x);
                D[m] = mfma(lds_op(&S.Ke[j0 + l16][16 + 4 * g]), vb1, x);
            }
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) S.Y[buf][jh][16 * mt + 4 * g + v][16 * q + l16] = Y[mt][v];
        } else {
            // -------------------------------------------------------------- exact path: 32 sequential steps
            // lane (i = 16q + l16, group g) holds S[i][j] for j = 32 jh + 16 m + 4 g + v
            __syncthreads();                           // keeps the barrier count equal on both paths
            float uv[2][4];
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const float4 x = *reinterpret_cast<const float4*>(&S.dec[32 * jh + 16 * m + 4 * g]);
                uv[m][0] = x.x; uv[m][1] = x.y; uv[m][2] = x.z; uv[m][3] = x.w;
            }
            const uint16_t* vt = reinterpret_cast<const uint16_t*>(&S.Vt[16 * q + l16][0]);
            for (int t = 0; t < L; ++t) {
                const float vi = bf2f(vt[t]);
                float yp = 0.f;
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const int j0 = 32 * jh + 16 * m + 4 * g;
                    const float4 r4 = *reinterpret_cast<const float4*>(&S.X[t][j0]);
                    const float4 k4 = *reinterpret_cast<const float4*>(&S.raw[0][t][j0]);
                    const float4 w4 = *reinterpret_cast<const float4*>(&S.raw[1][t][j0]);
                    const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float kv = kk[v] * vi;
                        yp = fmaf(rr[v], fmaf(uv[m][v], kv, D[m][v]), yp);
                        D[m][v] = fmaf(D[m][v], ww[v], kv);
                    }
                }
                const float y = allreduce_rows(yp);
                if (g == 0) S.Y[buf][jh][t][16 * q + l16] = y;
            }
        }
        __syncthreads();
        if (tid < 256) {
            const int t = tid >> 3, i0 = (tid & 7) * 8;
            if (c0 + t < T) {
                float f[8];
#pragma unroll
                for (int z = 0; z < 2; ++z) {
                    const float4 x0 = *reinterpret_cast<const float4*>(&S.Y[buf][0][t][i0 + 4 * z]);
                    const float4 x1 = *reinterpret_cast<const float4*>(&S.Y[buf][1][t][i0 + 4 * z]);
                    f[4 * z] = x0.x + x1.x; f[4 * z + 1] = x0.y + x1.y; f[4 * z + 2] = x0.z + x1.z; f[4 * z + 3] = x0.w + x1.w;
                }
                *reinterpret_cast<uint4*>(a.y + base + static_cast<size_t>(c0 + t) * C + i0) = pack8(f);
            }
        }
    };

    for (int cb = 0; cb < nchunks; cb += STAGES)
        static_for<STAGES>([&](auto Z) { if (cb + decltype(Z)::value < nchunks) process(cb + decltype(Z)::value, ring[decltype(Z)::value]); });
}

}  // namespace

// Launchers used by wkv56.hip's entry points.
int launch_wkv6_fwd_chunk(hipStream_t st, int wmode, int B, int T, int C, int H, const uint16_t* r,
                          const uint16_t* k, const uint16_t* v, const void* w, const uint16_t* u,
                          const uint16_t* s0, uint16_t* y) {
    ArgsC a{};
    a.T = T; a.C = C; a.H = H; a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.s0 = s0; a.y = y;
    if (wmode == W_RAW) hipLaunchKernelGGL(wkv6_fwd_chunk<W_RAW>, dim3(B * H), dim3(NT), 0, st, a);
    else hipLaunchKernelGGL(wkv6_fwd_chunk<W_EW>, dim3(B * H), dim3(NT), 0, st, a);
    return launch_status();
}

}  // namespace rwkv
